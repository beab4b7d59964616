// SAPA-D kernels that gather from an LDS-resident window instead of global
// memory: deform_qk, deform_av and the fused deform_qk -> softmax -> deform_av.
//
// A workgroup owns a TPW x TPH tile of low-res parent cells of one (image,
// group) pair; a thread owns one high-res query pixel of it.  The sampled
// tensor's window -- the tile plus HR = 4 cells on every side, one more on the
// high side for the +1 bilinear corners -- is staged in LDS CH channels at a
// time, zero-filled outside the image, so a sample whose floor() corner lies
// in the window reads its four corners from LDS and needs no border masks
// (a zero there is exactly the reference's per-corner zero padding,
// deformsapa/deformsapa/src/cuda/deform_qk_cuda_kernel.cu:39-62).  A sample
// that leaves the window -- offsets beyond +-4 cells -- takes the same taps
// from global memory, so any offset is handled.  The P logits / weights of a
// pixel live in LDS as well ([P][thread], conflict-free), which keeps the
// loop over sample points a run-time loop: any P, no register arrays.
//
// Arithmetic is the reference kernels' own (fp32 for 16-bit tensors):
// coordinates parent + offset, floor, strict guard, weights hh*hw.., the
// value w1*v1 + w2*v2 + w3*v3 + w4*v4 left to right, one FMA per channel in
// channel order for a logit (deform_qk_cuda_kernel.cu:180-193), one FMA per
// sample point in point order for an output (deform_av_cuda_kernel.cu:178-192).
#include "deform_tap.hpp"
#include "kernels.hpp"

namespace sapa {

enum DeformMode { DEFORM_QK = 0, DEFORM_AV = 1, DEFORM_FUSED = 2, DEFORM_OFFGRAD = 3 };

// TS: the type of the per-point scalar tensors [B, G, P, sH, sW] -- the logits
// (out of DEFORM_QK) and attn_in -- which the backward pass keeps in fp32 next to
// 16-bit features.  accumulate (DEFORM_OFFGRAD): add to what out -- or partial,
// if given -- holds.
template <typename T, typename TS, int S, int TPW, int TPH, int CH, int MODE>
__global__ void __launch_bounds__(TPW *TPH *S *S)
deform_lds_kernel(const T *__restrict__ q, const T *__restrict__ key,
                  const TS *__restrict__ attn_in, const T *__restrict__ value,
                  const T *__restrict__ offset, T *__restrict__ out, int Cq, int C, int H, int W,
                  int P, int G, int olayout, int tiles_x, int tiles_y, int nblocks, int per_xcd,
                  int accumulate, float *__restrict__ partial) {
    typedef float A;
    typedef float F4 __attribute__((ext_vector_type(4)));
    constexpr int HR = 4;                           // window reach in low-res cells
    constexpr int NT = TPW * TPH * S * S;
    constexpr int WW = TPW + 2 * HR + 1, WH = TPH + 2 * HR + 1;
    constexpr int WIN = WH * WW;
    // LDS window: [cell][CH channels], cells CST floats apart.  A thread reads the
    // CH channels of a corner as 16-byte vectors; with CST = 4 mod 16 the cells
    // that the lanes of a wave pick -- anywhere in the window -- spread over all
    // 16 four-bank groups instead of colliding on the one bank that a
    // [channel][cell] layout gives each channel.
    constexpr int CST = CH + 4;
    constexpr int RS = WW * CST;                    // floats between window rows
    static_assert(CH % 4 == 0, "channels are read four at a time");
    constexpr int TXP = TPW * S;                    // tile width in pixels
    constexpr bool DO_QK = MODE == DEFORM_QK || MODE == DEFORM_FUSED;
    constexpr bool DO_AV = MODE == DEFORM_AV || MODE == DEFORM_FUSED;

    extern __shared__ __attribute__((aligned(16))) float smem[];
    A *win = smem;                                  // [WH][WW][CST]
    A *lg = smem + WIN * CST;                       // [P][NT]

    const int logical = (int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8);
    if (logical >= nblocks) return;
    const int tx = logical % tiles_x;
    const int ty = (logical / tiles_x) % tiles_y;
    const int g = (logical / (tiles_x * tiles_y)) % G;
    const int b = logical / (tiles_x * tiles_y * G);

    const int tid = threadIdx.x;
    const int hH = H * S, hW = W * S, GP = G * P, d = Cq / G, cg = C / G;
    const long lplane = (long)H * W, hplane = (long)hH * hW;
    const int qw = tx * TXP + tid % TXP, qh = ty * TPH * S + tid / TXP;
    const bool active = qw < hW && qh < hH;
    // idle threads of a partial tile read through clamped coordinates
    const long pix = (long)(qh < hH ? qh : hH - 1) * hW + (qw < hW ? qw : hW - 1);
    const A ph = (A)((qh < hH ? qh : hH - 1) / S), pw = (A)((qw < hW ? qw : hW - 1) / S);
    const int wx0 = tx * TPW - HR, wy0 = ty * TPH - HR;
    const OffsetRef<T> op = offset_ref(offset, olayout, (long)b * GP + (long)g * P,
                                       qh < hH ? qh : hH - 1, qw < hW ? qw : hW - 1, S, H, W);
    A *lgt = lg + tid;

    // window of `nvalid` channels starting at plane `src` -> LDS, zero-filled
    // outside the image and past the last channel
    auto stage = [&](const T *src, int nvalid) {
        for (int idx = tid; idx < CH * WIN; idx += NT) {
            const int ch = idx / WIN, pos = idx % WIN;
            const int row = pos / WW, col = pos % WW;
            const int gy = wy0 + row, gx = wx0 + col;
            A v = 0;
            if (ch < nvalid && gy >= 0 && gy < H && gx >= 0 && gx < W)
                v = (A)src[(long)ch * lplane + (long)gy * W + gx];
            win[row * RS + col * CST + ch] = v;
        }
    };

    if (MODE == DEFORM_OFFGRAD) {
        // Gradient with respect to the offsets of either sampled operator
        // (deform_qk_cuda_kernel.cu:98-133): q = the per-channel high-res
        // tensor (query, or grad of the output), key = the sampled tensor,
        // attn_in = the per-point scalar (grad of the logits, or the
        // attention weights), out = grad_offset [B,2GP,sH,sW].  Per point the
        // two running sums live in LDS next to each other ([2P][thread]).
        const long ch0 = (long)b * Cq + (long)g * d;
        const TS *sp = attn_in + ((long)b * GP + (long)g * P) * hplane + pix;
        for (int c0 = 0; c0 < d; c0 += CH) {
            const int nvalid = d - c0 < CH ? d - c0 : CH;
            A qv[CH];
#pragma unroll
            for (int ch = 0; ch < CH; ++ch)
                qv[ch] = (active && ch < nvalid) ? (A)q[(ch0 + c0 + ch) * hplane + pix] : (A)0;
            __syncthreads();
            stage(key + (ch0 + c0) * lplane, nvalid);
            __syncthreads();
            // the next point's offsets are fetched while this point is evaluated
            A ow = (A)op.base[0], oh = (A)op.base[op.stride];
            for (int p = 0; p < P; ++p) {
                const A kw = pw + ow, kh = ph + oh;
                {
                    const int pn = p + 1 < P ? p + 1 : p;
                    ow = (A)op.base[(long)(2 * pn) * op.stride];
                    oh = (A)op.base[(long)(2 * pn + 1) * op.stride];
                }
                const A scv = (A)sp[(long)p * hplane];
                A gw = c0 == 0 ? (A)0 : lgt[(2 * p) * NT];
                A gh = c0 == 0 ? (A)0 : lgt[(2 * p + 1) * NT];
                Tap<A> tap;
                if (tap_setup(kh, kw, H, W, tap)) {
                    const int hl = (int)floor_(kh) - wy0, wl = (int)floor_(kw) - wx0;
                    if (hl >= 0 && hl <= WH - 2 && wl >= 0 && wl <= WW - 2) {
                        const A *wp = win + hl * RS + wl * CST;
#pragma unroll
                        for (int c4 = 0; c4 < CH; c4 += 4) {
                            const F4 a1 = *(const F4 *)(wp + c4), a2 = *(const F4 *)(wp + CST + c4);
                            const F4 a3 = *(const F4 *)(wp + RS + c4), a4 = *(const F4 *)(wp + RS + CST + c4);
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                const A tv = qv[c4 + e] * scv;
                                const A v1 = a1[e], v2 = a2[e], v3 = a3[e], v4 = a4[e];
                                const A ghc = -tap.hw * v1 - tap.lw * v2 + tap.hw * v3 + tap.lw * v4;
                                const A gwc = -tap.hh * v1 + tap.hh * v2 - tap.lh * v3 + tap.lh * v4;
                                gh = fma_(ghc, tv, gh);
                                gw = fma_(gwc, tv, gw);
                            }
                        }
                    } else {
                        const T *kp = key + (ch0 + c0) * lplane;
                        for (int ch = 0; ch < nvalid; ++ch) {
                            const T *plane = kp + (long)ch * lplane;
                            const A tv = qv[ch] * scv;
                            const A v1 = tap.m1 ? ld(plane + tap.i1) : (A)0;
                            const A v2 = tap.m2 ? ld(plane + tap.i2) : (A)0;
                            const A v3 = tap.m3 ? ld(plane + tap.i3) : (A)0;
                            const A v4 = tap.m4 ? ld(plane + tap.i4) : (A)0;
                            const A ghc = -tap.hw * v1 - tap.lw * v2 + tap.hw * v3 + tap.lw * v4;
                            const A gwc = -tap.hh * v1 + tap.hh * v2 - tap.lh * v3 + tap.lh * v4;
                            gh = fma_(ghc, tv, gh);
                            gw = fma_(gwc, tv, gw);
                        }
                    }
                }
                lgt[(2 * p) * NT] = gw;
                lgt[(2 * p + 1) * NT] = gh;
            }
        }
        if (active) {
            T *o = out + ((((long)b * GP + (long)g * P)) << 1) * hplane + pix;
            // `partial` (same shape as out, fp32): the first of two contributions is
            // parked there instead of out, the second adds it and rounds once
            float *po = partial ? partial + ((((long)b * GP + (long)g * P)) << 1) * hplane + pix : nullptr;
            for (int p = 0; p < 2 * P; ++p) {
                const A prev = !accumulate ? (A)0 : po ? (A)po[(long)p * hplane] : (A)o[(long)p * hplane];
                if (po && !accumulate) po[(long)p * hplane] = lgt[p * NT];
                else o[(long)p * hplane] = (T)(lgt[p * NT] + prev);
            }
        }
        return;
    }

    // `fn(wp)` with wp = LDS address of the tap's low corner if the tap is
    // inside the window; otherwise `fg()` (global-memory taps)
    if (DO_QK) {
        const long ch0 = (long)b * Cq + (long)g * d;
        for (int c0 = 0; c0 < d; c0 += CH) {
            const int nvalid = d - c0 < CH ? d - c0 : CH;
            A qv[CH];
#pragma unroll
            for (int ch = 0; ch < CH; ++ch)
                qv[ch] = (active && ch < nvalid) ? (A)q[(ch0 + c0 + ch) * hplane + pix] : (A)0;
            __syncthreads();                       // the previous chunk's readers are done
            stage(key + (ch0 + c0) * lplane, nvalid);
            __syncthreads();
            // the next point's offsets are fetched while this point is evaluated
            A ow = (A)op.base[0], oh = (A)op.base[op.stride];
            for (int p = 0; p < P; ++p) {
                const A kw = pw + ow, kh = ph + oh;
                {
                    const int pn = p + 1 < P ? p + 1 : p;
                    ow = (A)op.base[(long)(2 * pn) * op.stride];
                    oh = (A)op.base[(long)(2 * pn + 1) * op.stride];
                }
                A acc = c0 == 0 ? (A)0 : lgt[p * NT];
                Tap<A> tap;
                if (tap_setup(kh, kw, H, W, tap)) {
                    const int hl = (int)floor_(kh) - wy0, wl = (int)floor_(kw) - wx0;
                    if (hl >= 0 && hl <= WH - 2 && wl >= 0 && wl <= WW - 2) {
                        const A *wp = win + hl * RS + wl * CST;
#pragma unroll
                        for (int c4 = 0; c4 < CH; c4 += 4) {
                            const F4 a1 = *(const F4 *)(wp + c4), a2 = *(const F4 *)(wp + CST + c4);
                            const F4 a3 = *(const F4 *)(wp + RS + c4), a4 = *(const F4 *)(wp + RS + CST + c4);
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                A val = tap.w1 * a1[e];
                                val = fma_(tap.w2, a2[e], val);
                                val = fma_(tap.w3, a3[e], val);
                                val = fma_(tap.w4, a4[e], val);
                                acc = fma_(val, qv[c4 + e], acc);
                            }
                        }
                    } else {
                        const T *kp = key + (ch0 + c0) * lplane;
                        for (int ch = 0; ch < nvalid; ++ch)
                            acc = fma_(tap_sample(kp + (long)ch * lplane, tap), qv[ch], acc);
                    }
                }
                lgt[p * NT] = acc;
            }
        }
        if (MODE == DEFORM_FUSED) {
            // softmax over the P points of this pixel (guard failures keep
            // logit 0 and take part, as in softmax(deform_qk(...), dim=2))
            A m = lgt[0];
            for (int p = 1; p < P; ++p) m = max_(m, lgt[p * NT]);
            A sum = 0;
            for (int p = 0; p < P; ++p) {
                const A e = exp_(lgt[p * NT] - m);
                lgt[p * NT] = e;
                sum += e;
            }
            const A inv = (A)1 / sum;
            for (int p = 0; p < P; ++p) lgt[p * NT] *= inv;
        } else if (active) {
            TS *o = (TS *)out + ((long)b * GP + (long)g * P) * hplane + pix;
            for (int p = 0; p < P; ++p) o[(long)p * hplane] = (TS)lgt[p * NT];
        }
    } else {
        const TS *ap = attn_in + ((long)b * GP + (long)g * P) * hplane + pix;
        for (int p = 0; p < P; ++p) lgt[p * NT] = (A)ap[(long)p * hplane];
    }

    if (DO_AV) {
        const long ch0 = (long)b * C + (long)g * cg;
        for (int c0 = 0; c0 < cg; c0 += CH) {
            const int nvalid = cg - c0 < CH ? cg - c0 : CH;
            __syncthreads();
            stage(value + (ch0 + c0) * lplane, nvalid);
            __syncthreads();
            A o[CH];
#pragma unroll
            for (int ch = 0; ch < CH; ++ch) o[ch] = 0;
            // the next point's offsets are fetched while this point is evaluated
            A ow = (A)op.base[0], oh = (A)op.base[op.stride];
            for (int p = 0; p < P; ++p) {
                const A kw = pw + ow, kh = ph + oh;
                {
                    const int pn = p + 1 < P ? p + 1 : p;
                    ow = (A)op.base[(long)(2 * pn) * op.stride];
                    oh = (A)op.base[(long)(2 * pn + 1) * op.stride];
                }
                const A wa = lgt[p * NT];
                // Straight-line path for the common case (tap inside the
                // window): same expressions as tap_setup, results kept only
                // where the guard holds, so that consecutive points can be
                // interleaved by the scheduler.
                const WinTap<A> wt = win_tap(kh, kw, H, W, wy0, wx0, WH, WW);
                const A *wp = win + (wt.inwin ? wt.hl * RS + wt.wl * CST : 0);
#pragma unroll
                for (int c4 = 0; c4 < CH; c4 += 4) {
                    const F4 a1 = *(const F4 *)(wp + c4), a2 = *(const F4 *)(wp + CST + c4);
                    const F4 a3 = *(const F4 *)(wp + RS + c4), a4 = *(const F4 *)(wp + RS + CST + c4);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        A val = wt.w1 * a1[e];
                        val = fma_(wt.w2, a2[e], val);
                        val = fma_(wt.w3, a3[e], val);
                        val = fma_(wt.w4, a4[e], val);
                        const A on = fma_(val, wa, o[c4 + e]);
                        o[c4 + e] = wt.inwin ? on : o[c4 + e];
                    }
                }
                if (wt.guard && !wt.inwin) {       // rare: the tap left the window
                    Tap<A> tap;
                    tap_setup(kh, kw, H, W, tap);
                    const T *vp = value + (ch0 + c0) * lplane;
#pragma unroll
                    for (int ch = 0; ch < CH; ++ch)
                        if (ch < nvalid)
                            o[ch] = fma_(tap_sample(vp + (long)ch * lplane, tap), wa, o[ch]);
                }
            }
            if (active) {
                T *dst = out + (ch0 + c0) * hplane + pix;
#pragma unroll
                for (int ch = 0; ch < CH; ++ch)
                    if (ch < nvalid) dst[(long)ch * hplane] = (T)o[ch];
            }
        }
    }
}

// ------------------------------------------------------------------ launcher
template <typename T, typename TS, int S, int TPW, int TPH, int CH>
static hipError_t launch_geom(int mode, const void *q, const void *key, const void *attn_in,
                              const void *value, const void *offset, void *out, int B, int Cq,
                              int C, int H, int W, int P, int G, int olayout, hipStream_t st,
                              int accumulate, float *partial) {
    constexpr int HR = 4, NT = TPW * TPH * S * S;
    constexpr int WW = TPW + 2 * HR + 1, WH = TPH + 2 * HR + 1, CST = CH + 4;
    const size_t smem =
        ((size_t)WH * WW * CST + (size_t)(mode == DEFORM_OFFGRAD ? 2 : 1) * P * NT) * sizeof(float);
    if (smem > 160 * 1024) return hipErrorNotSupported;  // LDS of one CU
    const bool big = smem > 64 * 1024;                   // beyond the default dynamic-LDS limit
    const int tiles_x = (W + TPW - 1) / TPW, tiles_y = (H + TPH - 1) / TPH;
    const long nb = (long)tiles_x * tiles_y * G * B;
    if (nb > (1L << 30)) return hipErrorNotSupported;
    const int per_xcd = (int)((nb + 7) / 8);
    const dim3 grid(per_xcd * 8), block(NT);
#define SAPA_DL_CASE(M)                                                                       \
    case M:                                                                                   \
        if (big && hipFuncSetAttribute(                                                       \
                       reinterpret_cast<const void *>(&deform_lds_kernel<T, TS, S, TPW, TPH, CH, M>), \
                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess) { \
            (void)hipGetLastError();                                                          \
            return hipErrorNotSupported;                                                      \
        }                                                                                     \
        hipLaunchKernelGGL((deform_lds_kernel<T, TS, S, TPW, TPH, CH, M>), grid, block, smem, st, \
                           (const T *)q, (const T *)key, (const TS *)attn_in,                 \
                           (const T *)value, (const T *)offset, (T *)out, Cq, C, H, W, P, G,  \
                           olayout, tiles_x, tiles_y, (int)nb, per_xcd, accumulate, partial); \
        break;
    switch (mode) {
        SAPA_DL_CASE(DEFORM_QK) SAPA_DL_CASE(DEFORM_AV) SAPA_DL_CASE(DEFORM_FUSED)
        SAPA_DL_CASE(DEFORM_OFFGRAD)
        default: return hipErrorInvalidValue;
    }
#undef SAPA_DL_CASE
    return hipGetLastError();
}

template <typename T, typename TS>
static hipError_t launch_t(int mode, const void *q, const void *key, const void *attn_in,
                           const void *value, const void *offset, void *out, int B, int Cq, int C,
                           int H, int W, int P, int s, int G, int olayout, hipStream_t st,
                           int accumulate, float *partial) {
#ifdef SAPA_DLDS_TUNE
    if (s == 2) return launch_geom<T, TS, 2, SAPA_DLDS_TUNE>(mode, q, key, attn_in, value, offset, out, B, Cq, C, H, W, P, G, olayout, st, accumulate, partial);
    return hipErrorNotSupported;
#else
    switch (s) {
        case 1: return launch_geom<T, TS, 1, 16, 16, 8>(mode, q, key, attn_in, value, offset, out, B, Cq, C, H, W, P, G, olayout, st, accumulate, partial);
        case 2:
            // few points leave LDS room for a 16 x 8-parent tile (512 threads): a
            // smaller share of halo cells per staged window (measured at P = 9: 12 % faster;
            // at P = 25 the [P][thread] logits of 512 threads cost a workgroup per CU)
            if (P <= 12 && W > 8)
                return launch_geom<T, TS, 2, 16, 8, 16>(mode, q, key, attn_in, value, offset, out, B, Cq, C, H, W, P, G, olayout, st, accumulate, partial);
            return launch_geom<T, TS, 2, 8, 8, 16>(mode, q, key, attn_in, value, offset, out, B, Cq, C, H, W, P, G, olayout, st, accumulate, partial);
        case 4: return launch_geom<T, TS, 4, 4, 4, 16>(mode, q, key, attn_in, value, offset, out, B, Cq, C, H, W, P, G, olayout, st, accumulate, partial);
        default: return hipErrorNotSupported;
    }
#endif
}

// mode: 0 = deform_qk (out = logits), 1 = deform_av (attn_in given),
// 2 = fused, 3 = gradient of the offsets (q = per-channel high-res tensor,
// key = sampled tensor, attn_in = per-point scalar, out = grad_offset).  hipErrorNotSupported: no instance for (s, dtype) or P too large
// for the LDS budget; the caller then takes the global-memory kernels.  wide:
// the per-point tensors (attn_in, the logits) are fp32 next to 16-bit features;
// accumulate: mode 3 adds to grad_offset; partial (fp32, grad_offset's shape):
// the first contribution is kept there unrounded until the second adds it.
hipError_t deform_lds_launch(int mode, const void *q, const void *key, const void *attn_in,
                             const void *value, const void *offset, void *out, int B, int Cq, int C,
                             int H, int W, int P, int s, int G, int olayout, int dtype,
                             hipStream_t st, bool wide, bool accumulate, float *partial) {
    // the fused mode has no per-point tensor in memory
    if (wide && mode == DEFORM_FUSED) return hipErrorNotSupported;
    const int acc = accumulate ? 1 : 0;
    switch (dtype) {
        case 0: return launch_t<float, float>(mode, q, key, attn_in, value, offset, out, B, Cq, C, H, W, P, s, G, olayout, st, acc, partial);
#ifndef SAPA_DLDS_TUNE
        case 2:
            return wide ? launch_t<f16_t, float>(mode, q, key, attn_in, value, offset, out, B, Cq, C, H, W, P, s, G, olayout, st, acc, partial)
                        : launch_t<f16_t, f16_t>(mode, q, key, attn_in, value, offset, out, B, Cq, C, H, W, P, s, G, olayout, st, acc, partial);
        case 3:
            return wide ? launch_t<bf16_t, float>(mode, q, key, attn_in, value, offset, out, B, Cq, C, H, W, P, s, G, olayout, st, acc, partial)
                        : launch_t<bf16_t, bf16_t>(mode, q, key, attn_in, value, offset, out, B, Cq, C, H, W, P, s, G, olayout, st, acc, partial);
#endif
        default: return hipErrorNotSupported;
    }
}

}  // namespace sapa
