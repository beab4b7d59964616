// SAPA-B kernels that work for every (K, s, dtype): one thread per output
// element (or per pixel for the fused form).  They are the correctness path
// for shapes the LDS-tiled kernels in sapa_b_tiled.hip do not cover, and
// the building blocks of the backward pass.
//
// Arithmetic mirrors the reference kernels term by term (one FMA per term,
// same order), so fp32 results are bit-identical to theirs:
//   qk: sapa/sapa/src/cuda/qk_cuda_kernel.cu:39-67
//   av: sapa/sapa/src/cuda/av_cuda_kernel.cu:37-74
#include "kernels.hpp"

namespace sapa {

static inline int grid_for(long total, int block) {
    long g = (total + block - 1) / block;
    const long cap = 256L * 64;  // grid-stride beyond 64 blocks per CU
    return (int)(g < cap ? (g > 0 ? g : 1) : cap);
}

// out[n,k,ph,pw] = sum_c key[n,c,ph/s-r+ky,pw/s-r+kx] * q[n,c,ph,pw]
template <typename T>
__global__ void __launch_bounds__(256)
qk_forward_generic(const T *__restrict__ q, const T *__restrict__ key, T *__restrict__ out,
                   int B, int d, int H, int W, int K, int s) {
    typedef typename Acc<T>::type A;
    const int hH = H * s, hW = W * s, KK = K * K, r = (K - 1) / 2;
    const long lplane = (long)H * W, hplane = (long)hH * hW;
    const long total = (long)B * KK * hplane;
    for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
         idx += (long)gridDim.x * blockDim.x) {
        const int pw = (int)(idx % hW);
        long t = idx / hW;
        const int ph = (int)(t % hH);
        t /= hH;
        const int k = (int)(t % KK);
        const int n = (int)(t / KK);
        const int dh = ph / s - r + k / K;
        const int dw = pw / s - r + k % K;
        A acc = 0;
        if (dh >= 0 && dh < H && dw >= 0 && dw < W) {
            const T *kp = key + (long)n * d * lplane + (long)dh * W + dw;
            const T *qp = q + (long)n * d * hplane + (long)ph * hW + pw;
            for (int c = 0; c < d; ++c) acc = fma_(ld(kp + c * lplane), ld(qp + c * hplane), acc);
        }
        out[idx] = (T)acc;
    }
}

// out[n,c,ph,pw] = sum_{ky,kx} value[n,c,ph/s-r+ky,pw/s-r+kx] * attn[n,ky*K+kx,ph,pw]
template <typename T>
__global__ void __launch_bounds__(256)
av_forward_generic(const T *__restrict__ attn, const T *__restrict__ value, T *__restrict__ out,
                   int B, int C, int H, int W, int K, int s) {
    typedef typename Acc<T>::type A;
    const int hH = H * s, hW = W * s, KK = K * K, r = (K - 1) / 2;
    const long lplane = (long)H * W, hplane = (long)hH * hW;
    const long total = (long)B * C * hplane;
    for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
         idx += (long)gridDim.x * blockDim.x) {
        const int pw = (int)(idx % hW);
        long t = idx / hW;
        const int ph = (int)(t % hH);
        t /= hH;
        const int c = (int)(t % C);
        const int n = (int)(t / C);
        const int y0 = ph / s - r, x0 = pw / s - r;
        const T *vp = value + ((long)n * C + c) * lplane;
        const T *ap = attn + (long)n * KK * hplane + (long)ph * hW + pw;
        A acc = 0;
        for (int ky = 0; ky < K; ++ky) {
            const int iy = y0 + ky;
            if (iy < 0 || iy >= H) continue;
            for (int kx = 0; kx < K; ++kx) {
                const int ix = x0 + kx;
                if (ix < 0 || ix >= W) continue;
                acc = fma_(ld(vp + (long)iy * W + ix), ld(ap + (ky * K + kx) * hplane), acc);
            }
        }
        out[idx] = (T)acc;
    }
}

// Low-res gradient shared by both backward passes:
//   out[n,c,y,x] = sum_k sum_{children (ph,pw) of parent (y+r-ky, x+r-kx)}
//                  hi[n,c,ph,pw] * w[n,k,ph,pw]
// qk backward: hi = query, w = grad_out      -> grad_key
// av backward: hi = grad_out, w = attn       -> grad_value
// It is the gather form of the scatter in qk_cuda_kernel.cu:124-135 /
// av_cuda_kernel.cu:130-145: each low-res element sums its s*s*K*K
// contributions itself, so no atomics and a fixed summation order.
template <typename T>
__global__ void __launch_bounds__(256)
lowres_grad_generic(const T *__restrict__ hi, const T *__restrict__ w, T *__restrict__ out,
                    int B, int C, int H, int W, int K, int s) {
    typedef typename Acc<T>::type A;
    const int hH = H * s, hW = W * s, KK = K * K, r = (K - 1) / 2;
    const long hplane = (long)hH * hW;
    const long total = (long)B * C * H * W;
    for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
         idx += (long)gridDim.x * blockDim.x) {
        const int x = (int)(idx % W);
        long t = idx / W;
        const int y = (int)(t % H);
        t /= H;
        const int c = (int)(t % C);
        const int n = (int)(t / C);
        const T *hp = hi + ((long)n * C + c) * hplane;
        const T *wp = w + (long)n * KK * hplane;
        A acc = 0;
        for (int ky = 0; ky < K; ++ky) {
            const int py = y + r - ky;
            if (py < 0 || py >= H) continue;
            for (int kx = 0; kx < K; ++kx) {
                const int px = x + r - kx;
                if (px < 0 || px >= W) continue;
                const T *wk = wp + (ky * K + kx) * hplane;
                for (int cy = 0; cy < s; ++cy) {
                    const long row = (long)(py * s + cy) * hW + px * s;
                    for (int cx = 0; cx < s; ++cx)
                        acc = fma_(ld(hp + row + cx), ld(wk + row + cx), acc);
                }
            }
        }
        out[idx] = (T)acc;
    }
}

// Softmax over the middle axis of [N,R,M]; one thread per (n, m).
template <typename T>
__global__ void __launch_bounds__(256)
softmax_generic(const T *x, T *y, long N, int R, long M) {
    typedef typename Acc<T>::type A;
    const long total = N * M;
    for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
         idx += (long)gridDim.x * blockDim.x) {
        const long n = idx / M, m = idx % M;
        const T *xp = x + n * R * M + m;
        T *yp = y + n * R * M + m;
        A mx = ld(xp);
        for (int j = 1; j < R; ++j) mx = max_(mx, ld(xp + j * M));
        A sum = 0;
        for (int j = 0; j < R; ++j) sum += exp_(ld(xp + j * M) - mx);
        const A inv = (A)1 / sum;
        for (int j = 0; j < R; ++j) yp[j * M] = (T)(exp_(ld(xp + j * M) - mx) * inv);
    }
}

// Fused qk -> softmax (-> av), one thread per high-res pixel, K compile-time
// so that the K*K logits live in registers.  ATTN_ONLY: stop after the
// softmax and write the weights.
template <typename T, int K, bool ATTN_ONLY>
__global__ void __launch_bounds__(256)
fused_pixel(const T *__restrict__ q, const T *__restrict__ key, const T *__restrict__ value,
            T *__restrict__ out, int B, int d, int C, int H, int W, int s) {
    typedef typename Acc<T>::type A;
    constexpr int KK = K * K, r = (K - 1) / 2;
    const int hH = H * s, hW = W * s;
    const long lplane = (long)H * W, hplane = (long)hH * hW;
    const long total = (long)B * hplane;
    for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
         idx += (long)gridDim.x * blockDim.x) {
        const int pw = (int)(idx % hW);
        const long t = idx / hW;
        const int ph = (int)(t % hH);
        const int n = (int)(t / hH);
        const int y0 = ph / s - r, x0 = pw / s - r;
        const long pix = (long)ph * hW + pw;
        unsigned rowok = 0, colok = 0;
#pragma unroll
        for (int i = 0; i < K; ++i) {
            rowok |= (unsigned)(y0 + i >= 0 && y0 + i < H) << i;
            colok |= (unsigned)(x0 + i >= 0 && x0 + i < W) << i;
        }
        A a[KK];
#pragma unroll
        for (int k = 0; k < KK; ++k) a[k] = 0;
        const T *qp = q + (long)n * d * hplane + pix;
        const T *kp = key + (long)n * d * lplane + (long)y0 * W + x0;
        for (int c = 0; c < d; ++c) {
            const A qv = ld(qp + c * hplane);
            const T *kc = kp + c * lplane;
#pragma unroll
            for (int ky = 0; ky < K; ++ky)
#pragma unroll
                for (int kx = 0; kx < K; ++kx)
                    if ((rowok >> ky & 1u) && (colok >> kx & 1u))
                        a[ky * K + kx] = fma_(ld(kc + ky * W + kx), qv, a[ky * K + kx]);
        }
        softmax_inplace<A, KK>(a);
        if (ATTN_ONLY) {
            T *op = out + (long)n * KK * hplane + pix;
#pragma unroll
            for (int k = 0; k < KK; ++k) op[k * hplane] = (T)a[k];
        } else {
            const T *vp = value + (long)n * C * lplane + (long)y0 * W + x0;
            T *op = out + (long)n * C * hplane + pix;
            for (int c = 0; c < C; ++c) {
                const T *vc = vp + c * lplane;
                A acc = 0;
#pragma unroll
                for (int ky = 0; ky < K; ++ky)
#pragma unroll
                    for (int kx = 0; kx < K; ++kx)
                        if ((rowok >> ky & 1u) && (colok >> kx & 1u))
                            acc = fma_(ld(vc + ky * W + kx), a[ky * K + kx], acc);
                op[c * hplane] = (T)acc;
            }
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

hipError_t qk_forward_generic_launch(const void *q, const void *key, void *out, int B, int d,
                                     int H, int W, int K, int s, int dtype, hipStream_t st) {
    const long total = (long)B * K * K * H * s * W * s;
    SAPA_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL(qk_forward_generic<T>, dim3(grid_for(total, 256)),
        dim3(256), 0, st, (const T *)q, (const T *)key, (T *)out, B, d, H, W, K, s));
    return hipGetLastError();
}

hipError_t av_forward_generic_launch(const void *attn, const void *value, void *out, int B, int C,
                                     int H, int W, int K, int s, int dtype, hipStream_t st) {
    const long total = (long)B * C * H * s * W * s;
    SAPA_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL(av_forward_generic<T>, dim3(grid_for(total, 256)),
        dim3(256), 0, st, (const T *)attn, (const T *)value, (T *)out, B, C, H, W, K, s));
    return hipGetLastError();
}

hipError_t lowres_grad_generic_launch(const void *hi, const void *w, void *out, int B, int C,
                                      int H, int W, int K, int s, int dtype, hipStream_t st) {
    const long total = (long)B * C * H * W;
    SAPA_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL(lowres_grad_generic<T>, dim3(grid_for(total, 256)),
        dim3(256), 0, st, (const T *)hi, (const T *)w, (T *)out, B, C, H, W, K, s));
    return hipGetLastError();
}

hipError_t softmax_generic_launch(const void *x, void *y, long N, int R, long M, int dtype,
                                  hipStream_t st) {
    SAPA_DISPATCH_DTYPE(dtype, hipLaunchKernelGGL(softmax_generic<T>, dim3(grid_for(N * M, 256)),
        dim3(256), 0, st, (const T *)x, (T *)y, N, R, M));
    return hipGetLastError();
}

template <typename T, bool ATTN_ONLY>
static hipError_t fused_pixel_k(const void *q, const void *key, const void *value, void *out,
                                int B, int d, int C, int H, int W, int K, int s, hipStream_t st) {
    const long total = (long)B * H * s * W * s;
    const dim3 grid(grid_for(total, 256)), block(256);
#define SAPA_FP_CASE(KV)                                                                  \
    case KV:                                                                              \
        hipLaunchKernelGGL((fused_pixel<T, KV, ATTN_ONLY>), grid, block, 0, st,           \
                           (const T *)q, (const T *)key, (const T *)value, (T *)out, B,   \
                           d, C, H, W, s);                                                \
        break;
    switch (K) {
        SAPA_FP_CASE(1) SAPA_FP_CASE(3) SAPA_FP_CASE(5) SAPA_FP_CASE(7) SAPA_FP_CASE(9)
        SAPA_FP_CASE(11)
        default: return hipErrorNotSupported;
    }
#undef SAPA_FP_CASE
    return hipGetLastError();
}

hipError_t fused_pixel_launch(const void *q, const void *key, const void *value, void *out,
                              int B, int d, int C, int H, int W, int K, int s, int attn_only,
                              int dtype, hipStream_t st) {
    if (attn_only) {
        SAPA_DISPATCH_DTYPE(dtype, return (fused_pixel_k<T, true>(q, key, value, out, B, d, C, H,
                                                                    W, K, s, st)));
    } else {
        SAPA_DISPATCH_DTYPE(dtype, return (fused_pixel_k<T, false>(q, key, value, out, B, d, C, H,
                                                                     W, K, s, st)));
    }
    return hipSuccess;
}

}  // namespace sapa
