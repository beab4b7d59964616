// Gradient of the SAPA-D operators with respect to the sampled low-res tensor
// (grad_key of deform_qk, grad_value of deform_av) as a matrix product:
//
//   grad_low[b, g*cg + c, cell] += sum over (pixel, point, corner j that lands on
//                                  cell) of w_j * sc[b, g, p, pixel] * hi[b, g*cg + c, pixel]
//
// (hi = query and sc = grad of the logits for deform_qk; hi = grad of the output
// and sc = attention weights for deform_av; the reference issues one global
// atomicAdd per term, deformsapa/deformsapa/src/cuda/deform_qk_cuda_kernel.cu:107-122).
// With the corner weights of a pixel written as a row over the window cells
// of its region -- Wm[pixel][cell] = sum of sc * w_j over the samples that land
// there, the same matrix as in the forward kernels of sapa_d_nhwc.hip -- this is
//
//   grad_low[cell][c] += sum_pixels Wm[pixel][cell] * hi[pixel][c]        (Wm^T . hi)
//
// A workgroup owns a region of RG x RG hi-res pixels of one (image, group,
// 64-channel chunk) and walks over it 16 pixels at a time: the rows of Wm for
// those pixels are built in LDS (integer adds of per-row-scaled values: exact in
// any order, and several times the rate of LDS float atomics), their hi values
// are staged next to them, and v_mfma_f32_16x16x4f32 accumulates
// [cells of the region's window] x [64 channels] in registers over all 256
// pixels.  One global float atomic per window cell and channel at the end adds
// the region's sums to grad_low (the caller zero-fills it), as the LDS-window
// kernel of sapa_d_lowgrad.hip does -- which needs four 64-bit LDS atomics per
// sample AND channel where this kernel needs four 32-bit ones per sample.
//
// Samples that leave the region's window (offsets beyond +-4 cells), and all
// samples of a pixel whose scalars or hi values are not finite (an inf / NaN
// must reach exactly the cells it reaches in the reference, which 0 * inf in a
// dense product would not respect), add their terms straight to grad_low.
#include <utility>

#include "deform_tap.hpp"
#include "kernels.hpp"

namespace sapa {

namespace dscat {

typedef unsigned u32;
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int RCH = 4;          // window reach around the region's parents, in low-res cells
constexpr int NT = 256;
constexpr int CHK = 64;         // channels per workgroup
constexpr int SPX = 16;         // pixels per step
constexpr int GS = CHK + 16;    // floats per pixel of the staged hi tile: 16 mod 64, so that the
                                // 4 pixels a matrix operand read touches fall on disjoint banks

template <typename T, typename TS, int S, int RG>
__global__ void __launch_bounds__(NT) __attribute__((amdgpu_waves_per_eu(2, 2)))
deform_scatter_mat_kernel(const T *__restrict__ hi, const TS *__restrict__ sc,
                          const T *__restrict__ offset, float *__restrict__ grad_low, int Cx, int H,
                          int W, int P, int G, int regions_x, int regions_y, int nchunks, int nblocks,
                          int per_xcd) {
    constexpr int RP = RG / S;                               // parents of a region per axis
    constexpr int WWR = RP + 2 * RCH + 1, NPOS = WWR * WWR;  // window cells
    constexpr int NCB = (NPOS + 15) / 16, KPC = NCB * 16;    // blocks of 16 cells
    constexpr int WSR = KPC;        // dwords per row of Wm: 48 mod 64 (304, 176), the 4 rows of an operand read on disjoint banks
    constexpr int CBI = (NCB + 3) / 4;                       // cell blocks per wave
    constexpr int NSTEP = RG * RG / SPX;
    static_assert(RG % S == 0 && (RG * RG) % SPX == 0 && SPX % RG == 0 || RG % SPX == 0, "whole steps");
    static_assert(WSR % 64 == 48, "bank layout of the weight rows");

    constexpr int TS_ = 65;         // floats per channel row of the epilogue's transposition buffer
    constexpr int WLN = SPX * WSR > CHK * TS_ ? SPX * WSR : CHK * TS_;
    __shared__ __attribute__((aligned(16))) int Wl[WLN];            // Wm rows of the step, scaled integers
    __shared__ __attribute__((aligned(16))) float Gl[SPX * GS];     // hi of the step's pixels [pixel][channel]
    __shared__ float invl[SPX];                                     // 1 / scale of each row
    __shared__ u32 badmask;                                         // pixels of the step that go the direct way

    const int logical = (int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8);
    if (logical >= nblocks) return;
    const int rx = logical % regions_x;
    const int ry = (logical / regions_x) % regions_y;
    int rest = logical / (regions_x * regions_y);
    const int chunk = rest % nchunks;
    rest /= nchunks;
    const int g = rest % G, n = rest / G;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int mi = lane & 15, mk = lane >> 4;
    const int hH = H * S, hW = W * S, cg = Cx / G;
    const long lpix = (long)H * W, hpl = (long)hH * hW;
    const int y0 = ry * RG, x0 = rx * RG;                    // region origin, hi-res
    const int wy0 = y0 / S - RCH, wx0 = x0 / S - RCH;        // window origin, low-res cell
    const int c0 = chunk * CHK;                              // first channel of the chunk within the group
    const int cvalid = cg - c0 < CHK ? cg - c0 : CHK;
    const long ch0 = (long)n * Cx + (long)g * cg + c0;       // its plane index
    const long k0 = ((long)n * G + g) * P;                   // the group's first point

    // pixel t of step `step`: row / column within the region
    auto step_pixel = [&](int step, int t, int &qh, int &qw) __attribute__((always_inline)) {
        const int lin = step * SPX + t;
        qh = y0 + lin / RG;
        qw = x0 + lin % RG;
    };

    // ---- hi tile of a step: thread t brings channel t % 64, pixels 4 (t / 64) .. + 3
    const int gch = tid & 63, gq = tid >> 6;
    const bool vec4 = hW % 4 == 0 && (uintptr_t)hi % (4 * sizeof(T)) == 0;
    float greg[4];
    auto load_hi = [&](int step) __attribute__((always_inline)) {
        int qh, qw;
        step_pixel(step, 4 * gq, qh, qw);
#pragma unroll
        for (int e = 0; e < 4; ++e) greg[e] = 0.f;
        if (gch < cvalid && qh < hH) {
            const T *hp = hi + (ch0 + gch) * hpl + (long)qh * hW + qw;
            if (vec4 && qw + 3 < hW) {
                struct alignas(4 * sizeof(T)) V4 { T v[4]; };
                const V4 x = *(const V4 *)hp;
#pragma unroll
                for (int e = 0; e < 4; ++e) greg[e] = (float)x.v[e];
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (qw + e < hW) greg[e] = (float)hp[e];
            }
        }
    };
    // into LDS; a value that is not finite is replaced by 0 there and its pixel marked
    auto store_hi = [&]() __attribute__((always_inline)) {
        u32 bad = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const bool fin = __builtin_fabsf(greg[e]) < __builtin_huge_valf();
            bad |= fin ? 0u : 1u << (4 * gq + e);
            Gl[(4 * gq + e) * GS + gch] = fin ? greg[e] : 0.f;
        }
        if (bad) atomicOr(&badmask, bad);
    };

    // ---- per-sample view: P <= 16 -> 16 lanes per pixel, one pass per step; else 32, two
    const bool narrow = P <= 16;
    const int pt = narrow ? (tid & 15) : (tid & 31);
    const int prow = narrow ? (tid >> 4) : (tid >> 5);
    const int npass = narrow ? 1 : 2, ppp = narrow ? 16 : 8;
    // the scalar and the offsets of this lane's point, per pass, fetched a step ahead
    float scr[2], oxr[2], oyr[2];
    auto load_samples = [&](int step) __attribute__((always_inline)) {
#pragma unroll
        for (int ps = 0; ps < 2; ++ps) {
            scr[ps] = oxr[ps] = oyr[ps] = 0.f;
            if (ps < npass && pt < P) {
                int qh, qw;
                step_pixel(step, ps * ppp + prow, qh, qw);
                if (qh < hH && qw < hW) {
                    const long pp = (long)qh * hW + qw;
                    scr[ps] = (float)sc[(k0 + pt) * hpl + pp];
                    const T *op = offset + ((k0 + pt) << 1) * hpl + pp;
                    oxr[ps] = (float)op[0];
                    oyr[ps] = (float)op[hpl];
                }
            }
        }
    };

    f32x4 D[CBI][CHK / 16];
#pragma unroll
    for (int cbi = 0; cbi < CBI; ++cbi)
#pragma unroll
        for (int nb = 0; nb < CHK / 16; ++nb) D[cbi][nb] = f32x4{0.f, 0.f, 0.f, 0.f};

    if (tid == 0) badmask = 0;
    load_hi(0);
    load_samples(0);
    __syncthreads();

    for (int step = 0; step < NSTEP; ++step) {
        // ---- (a) empty weight rows, the step's hi tile
        for (int i = tid; i < SPX * WSR / 4; i += NT) ((int __attribute__((ext_vector_type(4))) *)Wl)[i] = {0, 0, 0, 0};
        store_hi();
        __syncthreads();

        // ---- (b) per (pixel, point): the corners' shares of sc into the pixel's row
        const u32 bad = badmask;
        auto sample = [&](auto nl, int ps) __attribute__((always_inline)) {
            constexpr int NL = decltype(nl)::value;
            const int t = ps * (NT / NL) + tid / NL;
            int qh, qw;
            step_pixel(step, t, qh, qw);
            const bool live = qh < hH && qw < hW && pt < P;
            const float scv = scr[ps];
            // the row's scale: |sum of any subset of its entries| <= L1 < 2^ex
            const float l1 = reduce_lanes<false, NL>(live ? __builtin_fabsf(scv) : 0.f);
            const bool finite = l1 < __builtin_huge_valf();
            int ex = 0;
            (void)__builtin_frexpf(l1, &ex);
            const float scale = __builtin_ldexpf(1.f, 30 - ex);
            if (pt == 0) invl[t] = (finite && l1 > 0.f) ? __builtin_ldexpf(1.f, ex - 30) : 0.f;
            if (!live || (scv == 0.f && !(bad >> t & 1))) return;
            const float kw = (float)(qw / S) + oxr[ps], kh = (float)(qh / S) + oyr[ps];
            const WinTap<float> wt = win_tap<float>(kh, kw, H, W, wy0, wx0, WWR, WWR);
            if (!wt.guard) return;
            if (wt.inwin && finite && !(bad >> t & 1)) {
                int *wp = Wl + t * WSR + wt.hl * WWR + wt.wl;
                const float sv = scv * scale;
                __hip_atomic_fetch_add(wp, (int)__builtin_rintf(sv * wt.w1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                __hip_atomic_fetch_add(wp + 1, (int)__builtin_rintf(sv * wt.w2), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                __hip_atomic_fetch_add(wp + WWR, (int)__builtin_rintf(sv * wt.w3), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                __hip_atomic_fetch_add(wp + WWR + 1, (int)__builtin_rintf(sv * wt.w4), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            } else {
                // the reference's own way: one float atomic per term (rare)
                Tap<float> tp = {};
                tap_setup(kh, kw, H, W, tp);
                const T *hp = hi + ch0 * hpl + (long)qh * hW + qw;
                for (int c = 0; c < cvalid; ++c) {
                    float *gp = grad_low + (ch0 + c) * lpix;
                    const float tv = (float)hp[c * hpl] * scv;
                    if (tp.m1) unsafeAtomicAdd(gp + tp.i1, tp.w1 * tv);
                    if (tp.m2) unsafeAtomicAdd(gp + tp.i2, tp.w2 * tv);
                    if (tp.m3) unsafeAtomicAdd(gp + tp.i3, tp.w3 * tv);
                    if (tp.m4) unsafeAtomicAdd(gp + tp.i4, tp.w4 * tv);
                }
            }
        };
        if (narrow) {
            sample(std::integral_constant<int, 16>{}, 0);
        } else {
            sample(std::integral_constant<int, 32>{}, 0);
            sample(std::integral_constant<int, 32>{}, 1);
        }
        __syncthreads();

        // ---- (c) D[cell][channel] += Wm^T . hi over the step's 16 pixels; the next
        // step's loads travel meanwhile
        if (tid == 0) badmask = 0;
        if (step + 1 < NSTEP) {
            load_hi(step + 1);
            load_samples(step + 1);
        }
#pragma unroll
        for (int ks = 0; ks < SPX / 4; ++ks) {
            const float inv = invl[4 * ks + mk];
            float b[CHK / 16];
#pragma unroll
            for (int nb = 0; nb < CHK / 16; ++nb) b[nb] = Gl[(4 * ks + mk) * GS + 16 * nb + mi];
#pragma unroll
            for (int cbi = 0; cbi < CBI; ++cbi) {
                const int cb = wave + 4 * cbi;
                if (cb < NCB) {
                    const float a = (float)Wl[(4 * ks + mk) * WSR + 16 * cb + mi] * inv;
#pragma unroll
                    for (int nb = 0; nb < CHK / 16; ++nb)
                        if (16 * nb < cvalid)       // (uniform) a short chunk skips its empty channel blocks
                            D[cbi][nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b[nb], D[cbi][nb], 0, 0, 0);
                }
            }
        }
        __syncthreads();
    }

    // ---- the region's sums into grad_low.  D[cbi][nb][r] = cell 16 cb + 4 mk + r,
    // channel 16 nb + mi: as it stands a wave's 64 lanes would hit 64 channel planes,
    // one atomic per cache line.  Through LDS ([channel][64 cells], the 4 waves'
    // blocks of a round side by side) the lanes of an instruction run along the
    // cells of one channel instead -- runs of up to WWR consecutive floats.
    float *const Tl = (float *)Wl;
#pragma unroll
    for (int cbi = 0; cbi < CBI; ++cbi) {
#pragma unroll
        for (int nb = 0; nb < CHK / 16; ++nb)
#pragma unroll
            for (int r = 0; r < 4; ++r) Tl[(16 * nb + mi) * TS_ + 16 * wave + 4 * mk + r] = D[cbi][nb][r];
        __syncthreads();
        // lane <-> cell 64 cbi + lane; this wave: channels 16 wave .. + 15
        const int cell = 64 * cbi + lane;
        const int gy = wy0 + cell / WWR, gx = wx0 + cell % WWR;
        const bool ok = cell < NPOS && gy >= 0 && gy < H && gx >= 0 && gx < W;
        float *gp = grad_low + (ch0 + 16 * wave) * lpix + (long)gy * W + gx;
#pragma unroll 4
        for (int c = 0; c < 16; ++c) {
            const float v = Tl[(16 * wave + c) * TS_ + lane];
            if (ok && 16 * wave + c < cvalid && v != 0.f) unsafeAtomicAdd(gp + c * lpix, v);
        }
        __syncthreads();
    }
}

template <typename T, typename TS, int S, int RG>
static hipError_t launch_geom(const void *hi, const void *sc, const void *offset, void *grad_low, int B,
                              int Cx, int H, int W, int P, int G, hipStream_t st) {
    const int regions_x = (W * S + RG - 1) / RG, regions_y = (H * S + RG - 1) / RG;
    const int nchunks = (Cx / G + CHK - 1) / CHK;
    const long nb = (long)regions_x * regions_y * nchunks * G * B;
    if (nb > (1L << 30)) return hipErrorNotSupported;
    const int per_xcd = (int)((nb + 7) / 8);
    hipLaunchKernelGGL((deform_scatter_mat_kernel<T, TS, S, RG>), dim3(per_xcd * 8), dim3(NT), 0, st,
                       (const T *)hi, (const TS *)sc, (const T *)offset, (float *)grad_low, Cx, H, W, P, G,
                       regions_x, regions_y, nchunks, (int)nb, per_xcd);
    return hipGetLastError();
}

template <typename T, typename TS>
static hipError_t launch_t(const void *hi, const void *sc, const void *offset, void *grad_low, int B, int Cx,
                           int H, int W, int P, int s, int G, hipStream_t st) {
    switch (s) {
        case 1: return launch_geom<T, TS, 1, 8>(hi, sc, offset, grad_low, B, Cx, H, W, P, G, st);
        case 2: return launch_geom<T, TS, 2, 16>(hi, sc, offset, grad_low, B, Cx, H, W, P, G, st);
        case 4: return launch_geom<T, TS, 4, 16>(hi, sc, offset, grad_low, B, Cx, H, W, P, G, st);
        default: return hipErrorNotSupported;
    }
}

}  // namespace dscat

// fp32 tensors, or (wide) f16 / bf16 features and offsets with fp32 per-point
// scalars; s in {1, 2, 4}, P <= 32; grad_low is fp32 and is accumulated into.
// hipErrorNotSupported otherwise.
hipError_t deform_scatter_mat_launch(const void *hi, const void *sc, const void *offset, void *grad_low,
                                     int B, int Cx, int H, int W, int P, int s, int G, int dtype,
                                     hipStream_t st, bool wide) {
    if (P > 32 || (long)H * s * W * s >= (1L << 31)) return hipErrorNotSupported;
    // The two products over the region's whole window are a fixed cost; the LDS-window
    // scatter's cost grows with points x channels.  Measured at B=8, G=4, 64 channels per
    // group, 64x64 -> 128x128 (us, this kernel / that one): P = 2 342 / 227, P = 5 349 / 452,
    // P = 9 352 / 770, P = 25 400 / 2052.
    const int cg = Cx / G;
    if ((long)P * (cg < 64 ? cg : 64) < 256) return hipErrorNotSupported;
    if (dtype == 0) return dscat::launch_t<float, float>(hi, sc, offset, grad_low, B, Cx, H, W, P, s, G, st);
    if (wide && dtype == 2) return dscat::launch_t<f16_t, float>(hi, sc, offset, grad_low, B, Cx, H, W, P, s, G, st);
    if (wide && dtype == 3) return dscat::launch_t<bf16_t, float>(hi, sc, offset, grad_low, B, Cx, H, W, P, s, G, st);
    return hipErrorNotSupported;
}

}  // namespace sapa
