// SAPA-B kernels for 16-bit tensors (f16, bf16) built on the two-term dot
// product instructions v_dot2c_f32_f16 / v_dot2c_f32_bf16: qk, qk+softmax and
// the fused qk -> softmax -> av forward.
//
// With 16-bit operands one dot2 instruction does two multiply-adds into an fp32
// accumulator; the logits run on it over a PAIR OF CHANNELS
//   a[j][k] += key[c][k]*q[c][j] + key[c+1][k]*q[c+1][j]
// i.e. 50 instructions per channel and parent instead of the 100 fp32 FMAs of
// sapa_b_tiled.hip, and half the LDS words.  On gfx950 a dot2 issues at half
// the rate of an fp32 FMA (measured: 4 against 2 cycles per wave and SIMD with
// enough waves), so the multiplier time of the logits halves.  The aggregation
// keeps the softmax weights in fp32: each 16-bit value is widened (one byte
// permute) and multiplied with fp32 FMAs, 25 + 100 instructions per channel
// and parent at full rate -- the same issue time as 60 half-rate dot2 on
// weight pairs rounded to 16 bits, without that rounding.  Products of a
// 16-bit value and an fp32 weight and all sums are fp32; only the inputs and
// the result are 16-bit.
//
// Work decomposition as in sapa_b_tiled.hip: a thread owns one low-res parent
// with its 2 x 2 children, a wave 32 x 2 parents, a workgroup NWX x NWY waves.
// LDS holds raw 16-bit data, one chunk at a time, double-buffered:
//   key chunk:   CHK = 16 channels as 8 planes of channel PAIRS, one 32-bit
//                word = (key[c], key[c+1]) at one window position;
//   value chunk: CHV = 16 channels, each window row as it lies in memory, one
//                word = (v[2i], v[2i+1]).  A parent whose first tap falls on an
//                even window column reads the words (t0,t1) (t2,t3) (t4,-);
//                one on an odd column reads (-,t0) (t1,t2) (t3,t4); a per-lane
//                byte selector picks the taps, so neither needs a shifted copy.
// Window positions outside the image and channels past the last one are
// fetched through a buffer descriptor sized to the remaining channels of the
// chunk: the hardware returns zeros for them, which is the zero padding the
// operators define, without masks or clamped addresses.
#include "kernels.hpp"

namespace sapa {

namespace dot2 {

typedef unsigned u32;
typedef u32 u32x2 __attribute__((ext_vector_type(2)));
typedef u32 u32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

template <typename T> struct Dot;
template <> struct Dot<f16_t> {
    static __device__ __forceinline__ float run(u32 a, u32 b, float c) {
        union { u32 u; f16x2 v; } x, y;
        x.u = a;
        y.u = b;
        return __builtin_amdgcn_fdot2(x.v, y.v, c, false);
    }
};
template <> struct Dot<bf16_t> {
    static __device__ __forceinline__ float run(u32 a, u32 b, float c) {
        union { u32 u; bf16x2 v; } x, y;
        x.u = a;
        y.u = b;
        return __builtin_amdgcn_fdot2_f32_bf16(x.v, y.v, c, false);
    }
};

// (lo, hi) 16-bit halves of two words -> one word
__device__ __forceinline__ u32 pack_lo(u32 a, u32 b) { return __builtin_amdgcn_perm(b, a, 0x05040100u); }
__device__ __forceinline__ u32 pack_hi(u32 a, u32 b) { return __builtin_amdgcn_perm(b, a, 0x07060302u); }

template <typename T>
__device__ __forceinline__ u32 pack2(float lo, float hi) {
    union { T t[2]; u32 u; } x;
    x.t[0] = (T)lo;
    x.t[1] = (T)hi;
    return x.u;
}
template <typename T>
__device__ __forceinline__ float lo_f(u32 w) {
    union { T t[2]; u32 u; } x;
    x.u = w;
    return (float)x.t[0];
}
template <typename T>
__device__ __forceinline__ float hi_f(u32 w) {
    union { T t[2]; u32 u; } x;
    x.u = w;
    return (float)x.t[1];
}

// WIDE: the K*K-channel tensors of the call (the result of qk+softmax; attn_in
// and the result of TILED_QK_SOFTMAX_BWD) are fp32 next to the 16-bit features
template <typename T, int K, int NWX, int NWY, int MODE, bool WIDE = false>
__global__ void __launch_bounds__(64 * NWX *NWY) __attribute__((amdgpu_waves_per_eu(3, 3)))
sapa_b_dot2_kernel(const T *__restrict__ q, const T *__restrict__ key,
                   const T *__restrict__ attn_in, const T *__restrict__ value,
                   T *__restrict__ out, int d, int C, int H, int W, int tiles_x, int tiles_y,
                   int nblocks, int per_xcd, int cgroups, int cper) {
    constexpr int S = 2, NJ = 4, WLX = 32, WLY = 2;
    constexpr int KK = K * K, R = (K - 1) / 2, KP = (K + 1) / 2, NPK = K * KP;
    constexpr int TW = WLX * NWX, TH = WLY * NWY, NT = 64 * NWX * NWY;
    constexpr int VEC = 4;                                   // elements per staging load
    constexpr int HL = (R + VEC - 1) / VEC * VEC;            // left halo, staged
    constexpr int WW = (HL + TW + R + VEC - 1) / VEC * VEC;  // staged window width
    constexpr int WH = TH + K - 1;
    constexpr int RSK = WW;                                  // key pair plane: words per row
    constexpr int RSV = WW / 2;                              // value plane: words per row
    constexpr int PLK = WH * RSK, PLV = WH * RSV;            // words per key pair / value channel
    constexpr int CHK = 16, CHV = 16;                        // channels per chunk
    constexpr int BUF = (CHK / 2) * PLK;
    constexpr int NVR = WW / VEC, NVP = WH * NVR;            // staging vectors per row / plane
    constexpr int PPI = NT / NVP;                            // planes staged per pass of the workgroup
    constexpr int NIK = CHK / 2 / PPI, NIV = CHV / PPI;      // passes per key / value chunk
    constexpr bool DO_QK = MODE != TILED_AV;
    constexpr bool DO_SOFTMAX = MODE == TILED_QK_SOFTMAX || MODE == TILED_FUSED;
    constexpr bool DO_AV = MODE == TILED_AV || MODE == TILED_FUSED;
    static_assert(PPI >= 1 && (CHK / 2) % PPI == 0 && CHV % PPI == 0, "staging passes");
    static_assert(CHV * PLV <= BUF, "a value chunk fits a buffer");
    static_assert(HL == VEC && WW % 4 == 0 && HL % 2 == 0 && HL - R + TW - 1 + K <= WW, "window layout");
    static_assert(sizeof(T) == 2, "16-bit tensors only");

    __shared__ __attribute__((aligned(16))) u32 lds[2 * BUF];

    const int logical = (int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8);
    if (logical >= nblocks) return;
    const int tx = logical % tiles_x;
    const int ty = (logical / tiles_x) % tiles_y;
    const int cg = (logical / (tiles_x * tiles_y)) % cgroups;
    const int n = logical / (tiles_x * tiles_y * cgroups);
    const int cbeg = cg * cper;
    const int cend = cbeg + cper < C ? cbeg + cper : C;
    if (DO_AV && cbeg >= C) return;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int lx = (wave % NWX) * WLX + (lane % WLX), ly = (wave / NWX) * WLY + (lane / WLX);
    const int x0 = tx * TW, y0 = ty * TH;
    const int px = x0 + lx, py = y0 + ly;
    const bool active = px < W && py < H;
    const int hH = H * S, hW = W * S;
    const long lplane = (long)H * W, hplane = (long)hH * hW;
    const long hpix = (long)(py * S) * hW + (long)px * S;
    const long hpix_ld = (long)((py < H ? py : H - 1) * S) * hW + (long)(px < W ? px : W - 1) * S;

    const int nKc = DO_QK ? (d + CHK - 1) / CHK : 0;
    const int nVc = DO_AV ? (cend - cbeg + CHV - 1) / CHV : 0;
    const int ntot = nKc + nVc;

    // ---- staging: in every pass thread t moves one 4-element vector of plane
    // (pass * PPI + t / NVP) at window position t % NVP; threads past PPI * NVP
    // have no part in it.  Byte offsets; an offset of 2^31 or more is outside
    // every descriptor (the launcher checks that the tensors are smaller).
    const u32 pb = (u32)lplane * 2u;                         // bytes per low-res plane
    const int sp = tid / NVP, sv = tid % NVP;
    const int srow = sv / NVR, svec = sv % NVR;
    const bool stager = sp < PPI;
    u32 goff;                                                // position inside a plane
    {
        const int gy = y0 - R + srow, gx = x0 - HL + svec * VEC;
        // W and gx are multiples of 4: a vector is all inside or all outside
        const bool ok = stager && gy >= 0 && gy < H && gx >= 0 && gx + VEC <= W;
        goff = ok ? (u32)(gy * W + gx) * 2u : 0x80000000u;
    }
    const u32 koff = goff + (u32)sp * 2u * pb, voff = goff + (u32)sp * pb;
    const int lk = sp * PLK + srow * RSK + svec * VEC, lv = sp * PLV + srow * RSV + svec * (VEC / 2);
    constexpr int NST = NIK * 4 > NIV * 2 ? NIK * 4 : NIV * 2;
    u32 st[NST];
    // descriptor over the `rem` planes that start at `base` (none if rem <= 0)
    auto planes_rsrc = [&](const T *base, int rem) {
        return __builtin_amdgcn_make_buffer_rsrc((void *)base, 0, rem > 0 ? rem * (int)pb : 0, 0x00020000);
    };
    auto stage_load = [&](int j) {
        if (j < nKc) {
            const int c0 = j * CHK;
#pragma unroll
            for (int i = 0; i < NIK; ++i) {
                const int c = c0 + 2 * PPI * i;              // first channel of this pass
                const __amdgpu_buffer_rsrc_t r = planes_rsrc(key + ((long)n * d + c) * lplane, d - c);
                const u32x2 ka = __builtin_amdgcn_raw_buffer_load_b64(r, koff, 0, 0);
                const u32x2 kb = __builtin_amdgcn_raw_buffer_load_b64(r, koff + pb, 0, 0);
                st[4 * i] = ka[0];
                st[4 * i + 1] = ka[1];
                st[4 * i + 2] = kb[0];
                st[4 * i + 3] = kb[1];
            }
        } else {
            const int c0 = cbeg + (j - nKc) * CHV;
#pragma unroll
            for (int i = 0; i < NIV; ++i) {
                const int c = c0 + PPI * i;
                const __amdgpu_buffer_rsrc_t r = planes_rsrc(value + ((long)n * C + c) * lplane, C - c);
                const u32x2 vv = __builtin_amdgcn_raw_buffer_load_b64(r, voff, 0, 0);
                st[2 * i] = vv[0];
                st[2 * i + 1] = vv[1];
            }
        }
    };
    auto stage_store = [&](int j) {
        if (!stager) return;
        u32 *dst = lds + (j & 1) * BUF;
        if (j < nKc) {
#pragma unroll
            for (int i = 0; i < NIK; ++i) {
                u32x4 o;
                o[0] = pack_lo(st[4 * i], st[4 * i + 2]);
                o[1] = pack_hi(st[4 * i], st[4 * i + 2]);
                o[2] = pack_lo(st[4 * i + 1], st[4 * i + 3]);
                o[3] = pack_hi(st[4 * i + 1], st[4 * i + 3]);
                *(u32x4 *)(dst + lk + i * PPI * PLK) = o;
            }
        } else {
#pragma unroll
            for (int i = 0; i < NIV; ++i) {
                u32x2 o;
                o[0] = st[2 * i];
                o[1] = st[2 * i + 1];
                *(u32x2 *)(dst + lv + i * PPI * PLV) = o;
            }
        }
    };

    // logits / weights of the four children, fp32
    float a[NJ][KK];
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
        for (int k = 0; k < KK; ++k) a[j][k] = 0;

    stage_load(0);
    if (MODE == TILED_AV && active) {
        const T *ap = attn_in + (long)n * KK * hplane + hpix;
#pragma unroll
        for (int k = 0; k < KK; ++k)
#pragma unroll
            for (int cy = 0; cy < S; ++cy) {
                const u32 w2 = *(const u32 *)(ap + (long)k * hplane + (long)cy * hW);
                a[cy * S][k] = lo_f<T>(w2);
                a[cy * S + 1][k] = hi_f<T>(w2);
            }
    }
    stage_store(0);
    __syncthreads();

    const int wcol = lx + HL - R;                  // window column of this parent's first tap

    if (DO_QK) {
        const u32 *kbase = lds + ly * RSK + wcol;
        const T *qp = q + (long)n * d * hplane + hpix_ld;
        // q of channel c, both child rows: one word (child x = 0, 1) per row
        auto load_q = [&](int c, u32 (&dst)[2]) {
            const int cc = c < d ? c : d - 1;
#pragma unroll
            for (int cy = 0; cy < S; ++cy)
                dst[cy] = __builtin_nontemporal_load((const u32 *)(qp + (long)cc * hplane + (long)cy * hW));
        };
        constexpr int PF = 2;                      // channel pairs in flight
        u32 qa[PF][2], qb[PF][2];
#pragma unroll
        for (int u = 0; u < PF; ++u) {
            load_q(2 * u, qa[u]);
            load_q(2 * u + 1, qb[u]);
        }
        for (int j = 0; j < nKc; ++j) {
            if (j + 1 < ntot) stage_load(j + 1);
            const int c0 = j * CHK;
            const u32 *wb = kbase + (j & 1) * BUF;
#pragma unroll 1
            for (int p0 = 0; p0 < CHK / 2; p0 += PF) {
#pragma unroll
                for (int u = 0; u < PF; ++u) {
                    const int c = c0 + 2 * (p0 + u);
                    // (q[c][child], q[c+1][child]) per child; channels past d are zero
                    const u32 ma = (active && c < d) ? 0xffffffffu : 0u;
                    const u32 mb = (active && c + 1 < d) ? 0xffffffffu : 0u;
                    u32 qv[NJ];
#pragma unroll
                    for (int cy = 0; cy < S; ++cy) {
                        const u32 x = qa[u][cy] & ma, y = qb[u][cy] & mb;
                        qv[cy * S] = pack_lo(x, y);
                        qv[cy * S + 1] = pack_hi(x, y);
                    }
                    load_q(c + 2 * PF, qa[u]);
                    load_q(c + 2 * PF + 1, qb[u]);
                    const u32 *wc = wb + (p0 + u) * PLK;
#pragma unroll
                    for (int ky = 0; ky < K; ++ky)
#pragma unroll
                        for (int kx = 0; kx < K; ++kx) {
                            const u32 kk = wc[ky * RSK + kx];
#pragma unroll
                            for (int jj = 0; jj < NJ; ++jj)
                                a[jj][ky * K + kx] = Dot<T>::run(kk, qv[jj], a[jj][ky * K + kx]);
                        }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            if (j + 1 < ntot) stage_store(j + 1);
            __syncthreads();
        }
        if (DO_SOFTMAX) {
#pragma unroll
            for (int jj = 0; jj < NJ; ++jj) softmax_inplace<float, KK>(a[jj]);
        }
        typedef float f32x2 __attribute__((ext_vector_type(2)));
        if (MODE == TILED_QK_SOFTMAX_BWD && active) {
            // a[][] holds g = d(loss)/d(attn); with the fp32 weights in attn_in it
            // becomes d(loss)/d(logits) = attn * (g - sum_k g * attn).  The weights
            // are read twice (the second time from cache) rather than kept.
            static_assert(MODE != TILED_QK_SOFTMAX_BWD || WIDE, "the weights of this mode are fp32");
            const float *ap = reinterpret_cast<const float *>(attn_in) + (long)n * KK * hplane + hpix;
            float dot[NJ];
#pragma unroll
            for (int jj = 0; jj < NJ; ++jj) dot[jj] = 0;
#pragma unroll
            for (int k = 0; k < KK; ++k)
#pragma unroll
                for (int cy = 0; cy < S; ++cy) {
                    const f32x2 v = *(const f32x2 *)(ap + (long)k * hplane + (long)cy * hW);
#pragma unroll
                    for (int cx = 0; cx < S; ++cx)
                        dot[cy * S + cx] = fma_(a[cy * S + cx][k], v[cx], dot[cy * S + cx]);
                }
            // (through an opaque copy of the pointer: the compiler would otherwise keep
            // the first pass's K*K loads for this one and spill them)
            const float *ap2 = ap;
            asm volatile("" : "+v"(ap2));
#pragma unroll
            for (int k = 0; k < KK; ++k)
#pragma unroll
                for (int cy = 0; cy < S; ++cy) {
                    const f32x2 v = *(const f32x2 *)(ap2 + (long)k * hplane + (long)cy * hW);
#pragma unroll
                    for (int cx = 0; cx < S; ++cx)
                        a[cy * S + cx][k] = v[cx] * (a[cy * S + cx][k] - dot[cy * S + cx]);
                }
        }
        if (!DO_AV && active) {
            if (WIDE) {
                float *op = reinterpret_cast<float *>(out) + (long)n * KK * hplane + hpix;
#pragma unroll
                for (int k = 0; k < KK; ++k)
#pragma unroll
                    for (int cy = 0; cy < S; ++cy)
                        *(f32x2 *)(op + (long)k * hplane + (long)cy * hW) = f32x2{a[cy * S][k], a[cy * S + 1][k]};
            } else {
                T *op = out + (long)n * KK * hplane + hpix;
#pragma unroll
                for (int k = 0; k < KK; ++k)
#pragma unroll
                    for (int cy = 0; cy < S; ++cy)
                        *(u32 *)(op + (long)k * hplane + (long)cy * hW) =
                            pack2<T>(a[cy * S][k], a[cy * S + 1][k]);
            }
        }
    }

    if (DO_AV) {
        // The weights stay fp32 (only the tensors are 16-bit): every tap's value is
        // widened to fp32 and multiplied with plain FMAs.  The words this parent
        // reads hold its row of taps as (t0,t1) (t2,t3) (t4,-) when its first tap
        // falls on an even window column and as (-,t0) (t1,t2) (t3,t4) on an odd
        // one; one byte permute with a per-lane selector picks tap k out of the
        // word pair (k / 2, (k + 1) / 2) either way and, for bf16, already is the
        // widening (the 16 bits land in the upper half of a zero word).
        const bool odd = wcol & 1;
        constexpr bool BF = sizeof(T) == 2 && !__is_same(T, f16_t);
        // bytes 0-3 = first word, 4-7 = second word, 0x0c = zero
        constexpr u32 LO1 = BF ? 0x01000c0cu : 0x0c0c0100u, HI1 = BF ? 0x03020c0cu : 0x0c0c0302u,
                      LO2 = BF ? 0x05040c0cu : 0x0c0c0504u;
        const u32 sel_even = odd ? HI1 : LO1;      // taps 0, 2, 4: one word, either half
        const u32 sel_odd = odd ? LO2 : HI1;       // taps 1, 3: end of one word or start of the next
        auto tap_value = [&](u32 w_first, u32 w_second, u32 sel) {
            const u32 r = __builtin_amdgcn_perm(w_second, w_first, sel);
            if (BF) return __builtin_bit_cast(float, r);
            return (float)__builtin_bit_cast(_Float16, (unsigned short)r);
        };
        const u32 *vbase = lds + ly * RSV + wcol / 2;
        // The results leave through buffer stores whose descriptor covers exactly the
        // channels of the chunk that exist: idle lanes (offset 2^31) and channels past
        // the slice fall outside it and the hardware drops them.  No branch around a
        // store, so the channel loop unrolls with a known number of stores behind the
        // next chunk's staging loads, and the wait for those loads leaves this chunk's
        // stores in flight.
        const u32 ooff = active ? (u32)(hpix * 2) : 0x80000000u;
        const u32 plane_bytes = (u32)(hplane * 2);
        __amdgpu_buffer_rsrc_t orsrc;
        auto load_v = [&](const u32 *wc, u32 (&dst)[NPK]) {
#pragma unroll
            for (int ky = 0; ky < K; ++ky)
#pragma unroll
                for (int p = 0; p < KP; ++p) dst[ky * KP + p] = wc[ky * RSV + p];
        };
        auto channel = [&](int ch, const u32 (&vv)[NPK]) {
            float o[NJ];
#pragma unroll
            for (int jj = 0; jj < NJ; ++jj) o[jj] = 0;
#pragma unroll
            for (int ky = 0; ky < K; ++ky)
#pragma unroll
                for (int kx = 0; kx < K; ++kx) {
                    const float v = tap_value(vv[ky * KP + kx / 2], vv[ky * KP + (kx + 1) / 2],
                                              kx % 2 ? sel_odd : sel_even);
#pragma unroll
                    for (int jj = 0; jj < NJ; ++jj) o[jj] = fma_(v, a[jj][ky * K + kx], o[jj]);
                }
#pragma unroll
            for (int cy = 0; cy < S; ++cy)
                __builtin_amdgcn_raw_buffer_store_b32(pack2<T>(o[cy * S], o[cy * S + 1]), orsrc,
                                                      ooff + (u32)ch * plane_bytes + (u32)(cy * hW) * 2u, 0,
                                                      2 /* non-temporal */);
        };
        for (int j = nKc; j < ntot; ++j) {
            if (j + 1 < ntot) stage_load(j + 1);
            const int c0 = cbeg + (j - nKc) * CHV;
            const u32 *wb = vbase + (j & 1) * BUF;
            const int nleft = cend - c0 < CHV ? cend - c0 : CHV;
            orsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(out + ((long)n * C + c0) * hplane), 0,
                                                      (int)((u32)nleft * plane_bytes), 0x00020000);
            // two channels per trip: the next channel's words are read from
            // LDS while the current one is multiplied
            u32 va[NPK], vb[NPK];
            load_v(wb, va);
#pragma unroll 1
            for (int ch = 0; ch < CHV; ch += 2) {
                load_v(wb + (ch + 1) * PLV, vb);
                channel(ch, va);
                __builtin_amdgcn_sched_barrier(0);
                load_v(wb + (ch + 2 < CHV ? ch + 2 : ch) * PLV, va);
                channel(ch + 1, vb);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (j + 1 < ntot) stage_store(j + 1);
            __syncthreads();
        }
    }
}

template <typename T, int K, int NWX, int NWY>
static hipError_t launch_mode(int mode, bool wide, const void *q, const void *key, const void *attn_in,
                              const void *value, void *out, int B, int d, int C, int H, int W,
                              hipStream_t st) {
    constexpr int TW = 32 * NWX, TH = 2 * NWY, NT = 64 * NWX * NWY, CHV = 16;
    const int tiles_x = (W + TW - 1) / TW, tiles_y = (H + TH - 1) / TH;
    int cgroups = 1;
    if (mode == TILED_FUSED || mode == TILED_AV) {
        const long tiles = (long)tiles_x * tiles_y * B;
        const int max_groups = C / (4 * CHV) > 0 ? C / (4 * CHV) : 1;
        while (cgroups * 2 <= max_groups && tiles * cgroups * 2 <= 1024) cgroups *= 2;
    }
    const int cper = ((C + cgroups - 1) / cgroups + CHV - 1) / CHV * CHV;
    const long nb = (long)tiles_x * tiles_y * B * cgroups;
    if (nb > (1L << 30)) return hipErrorNotSupported;
    const int per_xcd = (int)((nb + 7) / 8);
    const dim3 grid(per_xcd * 8), block(NT);
#define SAPA_D2_LAUNCH(M, WD)                                                                  \
    hipLaunchKernelGGL((sapa_b_dot2_kernel<T, K, NWX, NWY, M, WD>), grid, block, 0, st,        \
                       (const T *)q, (const T *)key, (const T *)attn_in, (const T *)value,     \
                       (T *)out, d, C, H, W, tiles_x, tiles_y, (int)nb, per_xcd, cgroups, cper)
#define SAPA_D2_CASE(M)                                                                        \
    case M:                                                                                    \
        SAPA_D2_LAUNCH(M, false);                                                              \
        break;
    if (wide) {
        switch (mode) {
            case TILED_QK_SOFTMAX: SAPA_D2_LAUNCH(TILED_QK_SOFTMAX, true); break;
            case TILED_QK_SOFTMAX_BWD: SAPA_D2_LAUNCH(TILED_QK_SOFTMAX_BWD, true); break;
            default: return hipErrorNotSupported;
        }
        return hipGetLastError();
    }
    switch (mode) {
        SAPA_D2_CASE(TILED_QK) SAPA_D2_CASE(TILED_QK_SOFTMAX) SAPA_D2_CASE(TILED_FUSED)
        default: return hipErrorNotSupported;
    }
#undef SAPA_D2_CASE
#undef SAPA_D2_LAUNCH
    return hipGetLastError();
}

}  // namespace dot2

// f16 / bf16, K = 5, s = 2, W a multiple of 4, key / value 8-byte aligned and
// the high-res tensors 4-byte aligned; hipErrorNotSupported otherwise (the
// caller then takes the fp32-arithmetic kernels).  av() alone is left to those
// as well: a dot2 instruction issues at half the rate of an fp32 FMA, so
// pairing 5 row neighbours as 3 words costs more multiplier time than 5 FMAs,
// while the channel pairs of the logits have no such padding.
hipError_t sapa_b_dot2_launch(int mode, const void *q, const void *key, const void *attn_in,
                              const void *value, void *out, int B, int d, int C, int H, int W,
                              int K, int s, int dtype, hipStream_t st, bool wide) {
    if (mode == TILED_AV || K != 5 || s != 2 || W % 4 != 0 || W < 32) return hipErrorNotSupported;
    if (mode == TILED_QK_SOFTMAX_BWD && !wide) return hipErrorNotSupported;
    // staging offsets are 32-bit byte offsets below 2^31 inside one image
    const long plane_bytes = (long)H * W * 2;
    if ((long)(d > C ? d : C) * plane_bytes >= (1L << 30)) return hipErrorNotSupported;
    const void *lo_ptrs[2] = {key, value}, *hi_ptrs[3] = {q, attn_in, out};
    for (const void *p : lo_ptrs)
        if (p && (uintptr_t)p % 8 != 0) return hipErrorNotSupported;
    for (const void *p : hi_ptrs)
        if (p && (uintptr_t)p % 4 != 0) return hipErrorNotSupported;
    // fp32 K*K tensors are accessed as pairs of floats
    if (wide && (((uintptr_t)attn_in | (uintptr_t)out) % 8 != 0)) return hipErrorNotSupported;
    switch (dtype) {
        case 2: return dot2::launch_mode<f16_t, 5, 1, 4>(mode, wide, q, key, attn_in, value, out, B, d, C, H, W, st);
        case 3: return dot2::launch_mode<bf16_t, 5, 1, 4>(mode, wide, q, key, attn_in, value, out, B, d, C, H, W, st);
        default: return hipErrorNotSupported;
    }
}

}  // namespace sapa
