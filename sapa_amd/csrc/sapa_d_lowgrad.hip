// Gradient of the SAPA-D operators with respect to the sampled low-res tensor
// (grad_key of deform_qk, grad_value of deform_av):
//
//   grad_low[b, g*cg + c, corner_j(pixel, p)] += w_j * hi[b, g*cg + c, pixel] * sc[b, g, p, pixel]
//
// over the four bilinear corners j of every (pixel, point) pair that passes
// the guard (hi = query and sc = grad of the logits for deform_qk; hi = grad
// of the output and sc = attention weights for deform_av).  The reference
// issues one global atomicAdd per term
// (deformsapa/deformsapa/src/cuda/deform_qk_cuda_kernel.cu:107-122), which on
// this GPU is bound by the rate of scattered float atomics in memory.
//
// Here a workgroup owns a tile of parent cells of one (image, group) pair, a
// thread one high-res pixel, and the terms are first summed in an LDS window
// (tile + 4 cells of halo, CH channels at a time).  LDS float atomics are very
// slow on gfx950 (about 1/40 of the integer rate), so the window holds 64-bit
// fixed-point sums updated with integer atomics: every term is scaled by a
// power of two chosen per (workgroup, chunk) from the largest |hi| * |sc| in
// it, so that no sum can overflow 2^50, and rounded to an integer once.  The
// rounding error per term is below 2^-40 of that largest magnitude -- far
// under fp32 resolution -- and integer addition is order-independent.  After
// the chunk each touched window cell is converted back and added to grad_low
// with ONE global float atomic (the caller zero-fills grad_low, as for the
// reference).  Taps that leave the window (offsets beyond +-4 cells) add
// their four terms straight to grad_low.
#include "deform_tap.hpp"
#include "kernels.hpp"

namespace sapa {

// T: the features' and the offsets' type, TS: the per-point scalars' (fp32 next
// to 16-bit features in the fused backward pass); grad_low is fp32 either way.
template <typename T, typename TS, int S, int TPW, int TPH, int CH>
__global__ void __launch_bounds__(TPW *TPH *S *S)
deform_lowgrad_lds_kernel(const T *__restrict__ hi, const TS *__restrict__ sc,
                          const T *__restrict__ offset, float *__restrict__ grad_low, int Cx,
                          int H, int W, int P, int G, int tiles_x, int tiles_y, int nblocks,
                          int per_xcd) {
    constexpr int HR = 4;                           // window reach in low-res cells
    constexpr int NT = TPW * TPH * S * S;
    constexpr int WW = TPW + 2 * HR + 1, WH = TPH + 2 * HR + 1;
    constexpr int WIN = WH * WW;
    constexpr int TXP = TPW * S;
    constexpr double MAGIC = 6755399441055744.0;    // 1.5 * 2^52: adding it leaves round(x) in
                                                    // the low mantissa bits for |x| < 2^51
    __shared__ long long acc[CH * WIN];
    __shared__ unsigned smax;
    __shared__ int sbad;

    const int logical = (int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8);
    if (logical >= nblocks) return;
    const int tx = logical % tiles_x;
    const int ty = (logical / tiles_x) % tiles_y;
    const int g = (logical / (tiles_x * tiles_y)) % G;
    const int b = logical / (tiles_x * tiles_y * G);

    const int tid = threadIdx.x;
    const int hH = H * S, hW = W * S, GP = G * P, cg = Cx / G;
    const long lplane = (long)H * W, hplane = (long)hH * hW;
    const int qw = tx * TXP + tid % TXP, qh = ty * TPH * S + tid / TXP;
    const bool active = qw < hW && qh < hH;
    const int cqh = qh < hH ? qh : hH - 1, cqw = qw < hW ? qw : hW - 1;   // clamped for loads
    const long pix = (long)cqh * hW + cqw;
    const float ph = (float)(cqh / S), pw = (float)(cqw / S);
    const int wx0 = tx * TPW - HR, wy0 = ty * TPH - HR;
    const long k0 = (long)b * GP + (long)g * P;
    const T *op = offset + (k0 << 1) * hplane + pix;
    const TS *sp = sc + k0 * hplane + pix;
    const long ch0 = (long)b * Cx + (long)g * cg;

    for (int i = tid; i < CH * WIN; i += NT) acc[i] = 0;
    if (tid == 0) { smax = 0; sbad = 0; }
    __syncthreads();

    // the largest |sc| of this pixel: half of the magnitude bound; inf / NaN
    // scalars are noted apart (the maximum drops NaNs)
    float scmax = 0.f;
    bool scbad = false;
    if (active)
        for (int p = 0; p < P; ++p) {
            const float a = fabsf((float)sp[(long)p * hplane]);
            scbad |= !(a < __builtin_huge_valf());
            scmax = fmaxf(scmax, a);
        }
    // a window cell receives at most one term per (pixel, point)
    int lg_terms = 0;
    while ((1L << lg_terms) < (long)NT * P) ++lg_terms;

    for (int c0 = 0; c0 < cg; c0 += CH) {
        const int nvalid = cg - c0 < CH ? cg - c0 : CH;
        float hv[CH];
        float hmax = 0.f;
        bool bad = scbad;
#pragma unroll
        for (int ch = 0; ch < CH; ++ch) {
            hv[ch] = (active && ch < nvalid) ? (float)hi[(ch0 + c0 + ch) * hplane + pix] : 0.f;
            const float a = fabsf(hv[ch]);
            bad |= !(a < __builtin_huge_valf());
            hmax = fmaxf(hmax, a);
        }
        // workgroup-wide bound on |term| (non-negative floats order like their bits)
        const float mine = hmax * scmax;
        bad |= !(mine < __builtin_huge_valf());
        if (bad)
            sbad = 1;       // an inf / NaN term: the fixed-point sums cannot carry it
        else if (mine > 0.f)
            atomicMax(&smax, __float_as_uint(mine));
        __syncthreads();                            // also: the window is zero, smax complete
        // a chunk with a non-finite term goes through the float atomics as a
        // whole, so that inf / NaN reach grad_low as they do in the reference
        const bool direct = sbad != 0;
        const float bound = __uint_as_float(smax);
        int ex = 0;
        (void)frexpf(bound, &ex);                   // bound < 2^ex
        const int shift = 50 - ex - lg_terms;
        const double scale = ldexp(1.0, shift), unscale = ldexp(1.0, -shift);
        double hs[CH];
#pragma unroll
        for (int ch = 0; ch < CH; ++ch) hs[ch] = (double)hv[ch] * scale;

        if (active) {
            // the next point's offsets and scalar are fetched while this one is scattered
            float ow = (float)op[0], oh = (float)op[hplane], sn = (float)sp[0];
            for (int p = 0; p < P; ++p) {
                const float kw = pw + ow, kh = ph + oh, scv = sn;
                {
                    const int pn = p + 1 < P ? p + 1 : p;
                    ow = (float)op[(long)(2 * pn) * hplane];
                    oh = (float)op[(long)(2 * pn + 1) * hplane];
                    sn = (float)sp[(long)pn * hplane];
                }
                Tap<float> tap;
                if (!tap_setup(kh, kw, H, W, tap)) continue;
                const int hl = (int)floor_(kh) - wy0, wl = (int)floor_(kw) - wx0;
                if (!direct && hl >= 0 && hl <= WH - 2 && wl >= 0 && wl <= WW - 2) {
                    // corners outside the image fall on window cells that are
                    // never written back: no masks needed
                    unsigned long long *cell = (unsigned long long *)acc + hl * WW + wl;
                    const double w1 = tap.w1, w2 = tap.w2, w3 = tap.w3, w4 = tap.w4, sd = scv;
#pragma unroll
                    for (int ch = 0; ch < CH; ++ch) {
                        const double t = hs[ch] * sd;
                        const long long mbits = __double_as_longlong(MAGIC);
                        const long long a1 = __double_as_longlong(fma(w1, t, MAGIC)) - mbits;
                        const long long a2 = __double_as_longlong(fma(w2, t, MAGIC)) - mbits;
                        const long long a3 = __double_as_longlong(fma(w3, t, MAGIC)) - mbits;
                        const long long a4 = __double_as_longlong(fma(w4, t, MAGIC)) - mbits;
                        __hip_atomic_fetch_add(cell + ch * WIN, (unsigned long long)a1,
                                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                        __hip_atomic_fetch_add(cell + ch * WIN + 1, (unsigned long long)a2,
                                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                        __hip_atomic_fetch_add(cell + ch * WIN + WW, (unsigned long long)a3,
                                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                        __hip_atomic_fetch_add(cell + ch * WIN + WW + 1, (unsigned long long)a4,
                                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                    }
                } else {
                    for (int ch = 0; ch < nvalid; ++ch) {
                        float *gp = grad_low + (ch0 + c0 + ch) * lplane;
                        const float tv = hv[ch] * scv;
                        if (tap.m1) unsafeAtomicAdd(gp + tap.i1, tap.w1 * tv);
                        if (tap.m2) unsafeAtomicAdd(gp + tap.i2, tap.w2 * tv);
                        if (tap.m3) unsafeAtomicAdd(gp + tap.i3, tap.w3 * tv);
                        if (tap.m4) unsafeAtomicAdd(gp + tap.i4, tap.w4 * tv);
                    }
                }
            }
        }
        __syncthreads();
        // write the touched cells back and clear the window for the next chunk
        for (int idx = tid; idx < CH * WIN; idx += NT) {
            const long long a = acc[idx];
            if (a == 0) continue;
            acc[idx] = 0;
            const int ch = idx / WIN, pos = idx % WIN;
            const int gy = wy0 + pos / WW, gx = wx0 + pos % WW;
            if (ch < nvalid && gy >= 0 && gy < H && gx >= 0 && gx < W)
                unsafeAtomicAdd(grad_low + (ch0 + c0 + ch) * lplane + (long)gy * W + gx,
                                (float)((double)a * unscale));
        }
        if (tid == 0) { smax = 0; sbad = 0; }
        // the next chunk's barrier (after its atomicMax) orders these writes
        // before any scatter; its atomicMax must not race the reset above
        __syncthreads();
    }
}

template <typename T, typename TS, int S, int TPW, int TPH, int CH>
static hipError_t deform_lowgrad_launch_geom(const void *hi, const void *sc, const void *offset, void *grad_low, int B,
                       int Cx, int H, int W, int P, int G, hipStream_t st) {
    constexpr int NT = TPW * TPH * S * S;
    const int tiles_x = (W + TPW - 1) / TPW, tiles_y = (H + TPH - 1) / TPH;
    const long nb = (long)tiles_x * tiles_y * G * B;
    if (nb > (1L << 30)) return hipErrorNotSupported;
    const int per_xcd = (int)((nb + 7) / 8);
    hipLaunchKernelGGL((deform_lowgrad_lds_kernel<T, TS, S, TPW, TPH, CH>), dim3(per_xcd * 8), dim3(NT),
                       0, st, (const T *)hi, (const TS *)sc, (const T *)offset,
                       (float *)grad_low, Cx, H, W, P, G, tiles_x, tiles_y, (int)nb, per_xcd);
    return hipGetLastError();
}

template <typename T, typename TS>
static hipError_t deform_lowgrad_lds_t(const void *hi, const void *sc, const void *offset, void *grad_low,
                                       int B, int Cx, int H, int W, int P, int s, int G, hipStream_t st) {
    switch (s) {
        case 1: return deform_lowgrad_launch_geom<T, TS, 1, 16, 16, 4>(hi, sc, offset, grad_low, B, Cx, H, W, P, G, st);
        case 2: return deform_lowgrad_launch_geom<T, TS, 2, 8, 8, 8>(hi, sc, offset, grad_low, B, Cx, H, W, P, G, st);
        case 4: return deform_lowgrad_launch_geom<T, TS, 4, 4, 4, 8>(hi, sc, offset, grad_low, B, Cx, H, W, P, G, st);
        default: return hipErrorNotSupported;
    }
}

// fp32 tensors, or (wide) f16 / bf16 features and offsets with fp32 per-point
// scalars; s in {1, 2, 4}; hipErrorNotSupported otherwise (the caller then takes
// the per-term atomic kernel).  grad_low is fp32 and is accumulated into.
hipError_t deform_lowgrad_lds_launch(const void *hi, const void *sc, const void *offset,
                                     void *grad_low, int B, int Cx, int H, int W, int P, int s,
                                     int G, int dtype, hipStream_t st, bool wide) {
    if (dtype == 0) return deform_lowgrad_lds_t<float, float>(hi, sc, offset, grad_low, B, Cx, H, W, P, s, G, st);
    if (wide && dtype == 2) return deform_lowgrad_lds_t<f16_t, float>(hi, sc, offset, grad_low, B, Cx, H, W, P, s, G, st);
    if (wide && dtype == 3) return deform_lowgrad_lds_t<bf16_t, float>(hi, sc, offset, grad_low, B, Cx, H, W, P, s, G, st);
    return hipErrorNotSupported;
}

}  // namespace sapa
