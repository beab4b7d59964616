// SAPA-D kernels: similarity and aggregation over P bilinear samples taken
// at parent + learned offset.  Index math, the strict in-range guard and the
// per-corner zero padding follow
//   deformsapa/deformsapa/src/cuda/deform_qk_cuda_kernel.cu:23-68,151-196
//   deformsapa/deformsapa/src/cuda/deform_av_cuda_kernel.cu:151-194
// Coordinates, floor and weights are evaluated in the tensor's arithmetic
// type (fp32 for 16-bit tensors), so the corner indices are the reference's.
#include "kernels.hpp"
#include "deform_tap.hpp"

namespace sapa {

static inline int grid_for(long total, int block) {
    long g = (total + block - 1) / block;
    const long cap = 256L * 64;
    return (int)(g < cap ? (g > 0 ? g : 1) : cap);
}

// out[b,g,p,qh,qw] = sum_{c<d} q[b,g*d+c,qh,qw] * bilinear(key[b,g*d+c])
template <typename T>
__global__ void __launch_bounds__(256)
deform_qk_forward_kernel(const T *__restrict__ q, const T *__restrict__ key,
                         const T *__restrict__ offset, T *__restrict__ out, int B, int Cq, int H,
                         int W, int P, int s, int G, int olayout) {
    typedef typename Acc<T>::type A;
    const int hH = H * s, hW = W * s, GP = G * P, d = Cq / G;
    const long lplane = (long)H * W, hplane = (long)hH * hW;
    const long total = (long)B * GP * hplane;
    for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
         idx += (long)gridDim.x * blockDim.x) {
        const int qw = (int)(idx % hW);
        long t = idx / hW;
        const int qh = (int)(t % hH);
        t /= hH;
        const int k = (int)(t % GP);
        const int b = (int)(t / GP);
        const int g = k / P;
        const long pix = (long)qh * hW + qw;
        const OffsetRef<T> op = offset_ref(offset, olayout, (long)b * GP + k, qh, qw, s, H, W);
        const A off_w = ld(op.base), off_h = ld(op.base + op.stride);
        const A kh = (A)(qh / s) + off_h, kw = (A)(qw / s) + off_w;
        Tap<A> tap;
        A acc = 0;
        if (tap_setup(kh, kw, H, W, tap)) {
            const long ch0 = (long)b * Cq + (long)g * d;
            const T *qp = q + ch0 * hplane + pix;
            const T *kp = key + ch0 * lplane;
            for (int c = 0; c < d; ++c)
                acc = fma_(tap_sample(kp + c * lplane, tap), ld(qp + c * hplane), acc);
        }
        out[idx] = (T)acc;
    }
}

// out[b,c,qh,qw] = sum_p attn[b,g(c),p,qh,qw] * bilinear(value[b,c])
template <typename T>
__global__ void __launch_bounds__(256)
deform_av_forward_kernel(const T *__restrict__ attn, const T *__restrict__ value,
                         const T *__restrict__ offset, T *__restrict__ out, int B, int C, int H,
                         int W, int P, int s, int G, int olayout) {
    typedef typename Acc<T>::type A;
    const int hH = H * s, hW = W * s, GP = G * P, cg = C / G;
    const long lplane = (long)H * W, hplane = (long)hH * hW;
    const long total = (long)B * C * hplane;
    for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
         idx += (long)gridDim.x * blockDim.x) {
        const int qw = (int)(idx % hW);
        long t = idx / hW;
        const int qh = (int)(t % hH);
        t /= hH;
        const int c = (int)(t % C);
        const int b = (int)(t / C);
        const int g = c / cg;
        const long pix = (long)qh * hW + qw;
        const long k0 = (long)b * GP + (long)g * P;
        const T *ap = attn + k0 * hplane + pix;
        const OffsetRef<T> op = offset_ref(offset, olayout, k0, qh, qw, s, H, W);
        const T *plane = value + ((long)b * C + c) * lplane;
        const A ph = (A)(qh / s), pw = (A)(qw / s);
        A acc = 0;
        for (int ip = 0; ip < P; ++ip) {
            const A off_w = ld(op.base + (2 * ip) * op.stride);
            const A off_h = ld(op.base + (2 * ip + 1) * op.stride);
            const A wa = ld(ap + ip * hplane);
            Tap<A> tap;
            if (tap_setup(ph + off_h, pw + off_w, H, W, tap))
                acc = fma_(tap_sample(plane, tap), wa, acc);
        }
        out[idx] = (T)acc;
    }
}

// Fused deform_qk -> softmax over P -> deform_av; one thread per
// (b, g, qh, qw).  The P sample positions and logits stay in registers
// (PMAX >= P compile-time bound); taps are rebuilt from the positions where
// they are needed, which costs a few ALU ops against the channel loop.
template <typename T, int PMAX>
__global__ void __launch_bounds__(256)
deform_fused_forward_kernel(const T *__restrict__ q, const T *__restrict__ key,
                            const T *__restrict__ value, const T *__restrict__ offset,
                            T *__restrict__ out, int B, int Cq, int C, int H, int W, int P, int s,
                            int G, int olayout) {
    typedef typename Acc<T>::type A;
    constexpr int CC = 8;  // value channels accumulated together
    const int hH = H * s, hW = W * s, GP = G * P, d = Cq / G, cg = C / G;
    const long lplane = (long)H * W, hplane = (long)hH * hW;
    const long total = (long)B * G * hplane;
    for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
         idx += (long)gridDim.x * blockDim.x) {
        const int qw = (int)(idx % hW);
        long t = idx / hW;
        const int qh = (int)(t % hH);
        t /= hH;
        const int g = (int)(t % G);
        const int b = (int)(t / G);
        const long pix = (long)qh * hW + qw;
        const long k0 = (long)b * GP + (long)g * P;
        const OffsetRef<T> op = offset_ref(offset, olayout, k0, qh, qw, s, H, W);
        const A ph = (A)(qh / s), pw = (A)(qw / s);
        const T *qp = q + ((long)b * Cq + (long)g * d) * hplane + pix;
        const T *kp = key + ((long)b * Cq + (long)g * d) * lplane;

        A kh[PMAX], kw[PMAX], a[PMAX];
#pragma unroll
        for (int ip = 0; ip < PMAX; ++ip) {
            if (ip < P) {
                kw[ip] = pw + ld(op.base + (2 * ip) * op.stride);
                kh[ip] = ph + ld(op.base + (2 * ip + 1) * op.stride);
                Tap<A> tap;
                A acc = 0;
                if (tap_setup(kh[ip], kw[ip], H, W, tap))
                    for (int c = 0; c < d; ++c)
                        acc = fma_(tap_sample(kp + c * lplane, tap), ld(qp + c * hplane), acc);
                a[ip] = acc;
            }
        }
        // softmax over the P live entries (guard failures keep logit 0 and
        // take part, as in softmax(deform_qk(...), dim=2))
        A m = a[0];
#pragma unroll
        for (int ip = 1; ip < PMAX; ++ip)
            if (ip < P) m = max_(m, a[ip]);
        A sum = 0;
#pragma unroll
        for (int ip = 0; ip < PMAX; ++ip)
            if (ip < P) {
                a[ip] = exp_(a[ip] - m);
                sum += a[ip];
            }
        const A inv = (A)1 / sum;
#pragma unroll
        for (int ip = 0; ip < PMAX; ++ip)
            if (ip < P) a[ip] *= inv;

        const T *vp = value + ((long)b * C + (long)g * cg) * lplane;
        T *outp = out + ((long)b * C + (long)g * cg) * hplane + pix;
        for (int c0 = 0; c0 < cg; c0 += CC) {
            A acc[CC];
#pragma unroll
            for (int cc = 0; cc < CC; ++cc) acc[cc] = 0;
#pragma unroll
            for (int ip = 0; ip < PMAX; ++ip) {
                if (ip < P) {
                    Tap<A> tap;
                    if (tap_setup(kh[ip], kw[ip], H, W, tap)) {
#pragma unroll
                        for (int cc = 0; cc < CC; ++cc)
                            if (c0 + cc < cg)
                                acc[cc] = fma_(tap_sample(vp + (c0 + cc) * lplane, tap), a[ip],
                                               acc[cc]);
                    }
                }
            }
#pragma unroll
            for (int cc = 0; cc < CC; ++cc)
                if (c0 + cc < cg) outp[(c0 + cc) * hplane] = (T)acc[cc];
        }
    }
}

// Backward of either sampled op with respect to the sampled low-res tensor
// (scatter, atomics) and the offsets (owned by this thread, plain store).
// One thread per (b, g, p, qh, qw); per channel c of the group
//   tv = hi[b,g*cg+c,qh,qw] * sc[b,g,p,qh,qw]
// is the reference's top_grad * weight (deform_qk_cuda_kernel.cu:93):
//   qk backward: hi = query, sc = grad_out;  av backward: hi = grad_out, sc = attn.
template <typename T>
__global__ void __launch_bounds__(256)
deform_lowgrad_kernel(const T *__restrict__ hi, const T *__restrict__ sc,
                      const T *__restrict__ low, const T *__restrict__ offset,
                      T *__restrict__ grad_low, T *__restrict__ grad_offset, int B, int Cx, int H,
                      int W, int P, int s, int G) {
    typedef typename Acc<T>::type A;
    const int hH = H * s, hW = W * s, GP = G * P, cg = Cx / G;
    const long lplane = (long)H * W, hplane = (long)hH * hW;
    const long total = (long)B * GP * hplane;
    for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
         idx += (long)gridDim.x * blockDim.x) {
        const int qw = (int)(idx % hW);
        long t = idx / hW;
        const int qh = (int)(t % hH);
        t /= hH;
        const int k = (int)(t % GP);
        const int b = (int)(t / GP);
        const int g = k / P;
        const long pix = (long)qh * hW + qw;
        const long oi = (((long)b * GP + k) << 1) * hplane + pix;
        const A kw = (A)(qw / s) + ld(offset + oi);
        const A kh = (A)(qh / s) + ld(offset + oi + hplane);
        const A scv = ld(sc + idx);
        A gw = 0, gh = 0;
        Tap<A> tap;
        if (tap_setup(kh, kw, H, W, tap)) {
            const long ch0 = (long)b * Cx + (long)g * cg;
            const T *hp = hi + ch0 * hplane + pix;
            for (int c = 0; c < cg; ++c) {
                const T *plane = low + (ch0 + c) * lplane;
                const A tv = ld(hp + c * hplane) * scv;
                const A v1 = tap.m1 ? ld(plane + tap.i1) : (A)0;
                const A v2 = tap.m2 ? ld(plane + tap.i2) : (A)0;
                const A v3 = tap.m3 ? ld(plane + tap.i3) : (A)0;
                const A v4 = tap.m4 ? ld(plane + tap.i4) : (A)0;
                const A ghc = -tap.hw * v1 - tap.lw * v2 + tap.hw * v3 + tap.lw * v4;
                const A gwc = -tap.hh * v1 + tap.hh * v2 - tap.lh * v3 + tap.lh * v4;
                gh = fma_(ghc, tv, gh);
                gw = fma_(gwc, tv, gw);
                if (grad_low) {
                    T *gp = grad_low + (ch0 + c) * lplane;
                    if (tap.m1) unsafeAtomicAdd(gp + tap.i1, (T)(tap.w1 * tv));
                    if (tap.m2) unsafeAtomicAdd(gp + tap.i2, (T)(tap.w2 * tv));
                    if (tap.m3) unsafeAtomicAdd(gp + tap.i3, (T)(tap.w3 * tv));
                    if (tap.m4) unsafeAtomicAdd(gp + tap.i4, (T)(tap.w4 * tv));
                }
            }
        }
        if (grad_offset) {
            grad_offset[oi] = (T)gw;
            grad_offset[oi + hplane] = (T)gh;
        }
    }
}

// ------------------------------------------------------------------ launchers
#define SAPA_DISPATCH_DTYPE(dtype, ...)                                        \
    switch (dtype) {                                                           \
        case 0: { typedef float T; __VA_ARGS__; break; }                       \
        case 1: { typedef double T; __VA_ARGS__; break; }                      \
        case 2: { typedef f16_t T; __VA_ARGS__; break; }                       \
        case 3: { typedef bf16_t T; __VA_ARGS__; break; }                      \
        default: return hipErrorInvalidValue;                                  \
    }

hipError_t deform_qk_forward_launch(const void *q, const void *key, const void *offset, void *out,
                                    int B, int Cq, int H, int W, int P, int s, int G, int olayout,
                                    int dtype, hipStream_t st) {
    const long total = (long)B * G * P * H * s * W * s;
    SAPA_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL(deform_qk_forward_kernel<T>,
        dim3(grid_for(total, 256)), dim3(256), 0, st, (const T *)q, (const T *)key,
        (const T *)offset, (T *)out, B, Cq, H, W, P, s, G, olayout));
    return hipGetLastError();
}

hipError_t deform_av_forward_launch(const void *attn, const void *value, const void *offset,
                                    void *out, int B, int C, int H, int W, int P, int s, int G,
                                    int olayout, int dtype, hipStream_t st) {
    const long total = (long)B * C * H * s * W * s;
    SAPA_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL(deform_av_forward_kernel<T>,
        dim3(grid_for(total, 256)), dim3(256), 0, st, (const T *)attn, (const T *)value,
        (const T *)offset, (T *)out, B, C, H, W, P, s, G, olayout));
    return hipGetLastError();
}

template <typename T>
static hipError_t deform_fused_t(const void *q, const void *key, const void *value,
                                 const void *offset, void *out, int B, int Cq, int C, int H, int W,
                                 int P, int s, int G, int olayout, hipStream_t st) {
    const long total = (long)B * G * H * s * W * s;
    const dim3 grid(grid_for(total, 256)), block(256);
#define SAPA_DF_CASE(PM)                                                                       \
    hipLaunchKernelGGL((deform_fused_forward_kernel<T, PM>), grid, block, 0, st, (const T *)q, \
                       (const T *)key, (const T *)value, (const T *)offset, (T *)out, B, Cq,   \
                       C, H, W, P, s, G, olayout)
    if (P <= 8) SAPA_DF_CASE(8);
    else if (P <= 16) SAPA_DF_CASE(16);
    else if (P <= 32) SAPA_DF_CASE(32);
    else if (P <= 64) SAPA_DF_CASE(64);
    else return hipErrorNotSupported;
#undef SAPA_DF_CASE
    return hipGetLastError();
}

hipError_t deform_fused_forward_launch(const void *q, const void *key, const void *value,
                                       const void *offset, void *out, int B, int Cq, int C, int H,
                                       int W, int P, int s, int G, int olayout, int dtype,
                                       hipStream_t st) {
    SAPA_DISPATCH_DTYPE(dtype, return (deform_fused_t<T>(q, key, value, offset, out, B, Cq, C, H,
                                                         W, P, s, G, olayout, st)));
    return hipSuccess;
}

hipError_t deform_lowgrad_launch(const void *hi, const void *sc, const void *low,
                                 const void *offset, void *grad_low, void *grad_offset, int B,
                                 int Cx, int H, int W, int P, int s, int G, int dtype,
                                 hipStream_t st) {
    const long total = (long)B * G * P * H * s * W * s;
    const dim3 grid(grid_for(total, 256)), block(256);
    if (dtype == 0)
        hipLaunchKernelGGL(deform_lowgrad_kernel<float>, grid, block, 0, st, (const float *)hi,
                           (const float *)sc, (const float *)low, (const float *)offset,
                           (float *)grad_low, (float *)grad_offset, B, Cx, H, W, P, s, G);
    else if (dtype == 1)
        hipLaunchKernelGGL(deform_lowgrad_kernel<double>, grid, block, 0, st, (const double *)hi,
                           (const double *)sc, (const double *)low, (const double *)offset,
                           (double *)grad_low, (double *)grad_offset, B, Cx, H, W, P, s, G);
    else
        return hipErrorNotSupported;
    return hipGetLastError();
}

}  // namespace sapa
