// Per (image, channel) mean and biased variance of a feature map in one pass
// over it: the statistics that GroupNorm needs (sapa_base.py:17-19,27-31 feed
// norm_y(y) and norm_x(x) to the q / k projections), from which the host folds
// the normalisation into the projection weights.  HBM-bound: every element is
// read once, 16 bytes per lane.
//
// Two kernels, no atomics (results do not depend on scheduling):
//   1. partial sums of (x - shift) and (x - shift)^2 in fp32 over a chunk of an
//      image's pixels, shift = the channel's first element (keeps the squares
//      small when |mean| >> spread);
//        contiguous [B, C, HW]:     one block per (image, channel, chunk), the
//                                   lanes along the pixels;
//        channels-last [B, HW, C]:  one block per (image, chunk), a lane owns 4
//                                   channels and every 256 / (C / 4)-th pixel,
//                                   the pixel lanes are summed through LDS;
//   2. one thread per (image, channel) adds the chunks in order and writes
//      mean = shift + S1 / HW, var = S2 / HW - (S1 / HW)^2.
#include "kernels.hpp"

#include <mutex>

namespace sapa {

namespace moments {

typedef unsigned u32;
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef u32 u32x2 __attribute__((ext_vector_type(2)));
typedef u32 u32x4 __attribute__((ext_vector_type(4)));

// N consecutive elements -> floats
template <typename T, int N> struct Pack;
template <> struct Pack<float, 4> {
    static __device__ __forceinline__ void load(const float *p, float (&v)[4]) {
        const f32x4 r = __builtin_nontemporal_load((const f32x4 *)p);
        v[0] = r[0], v[1] = r[1], v[2] = r[2], v[3] = r[3];
    }
};
template <typename H> struct Pack<H, 8> {
    static __device__ __forceinline__ void load(const H *p, float (&v)[8]) {
        union { u32x4 u; H h[8]; } x;
        x.u = __builtin_nontemporal_load((const u32x4 *)p);
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = (float)x.h[i];
    }
};
template <typename H> struct Pack<H, 4> {
    static __device__ __forceinline__ void load(const H *p, float (&v)[4]) {
        union { u32x2 u; H h[4]; } x;
        x.u = __builtin_nontemporal_load((const u32x2 *)p);
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = (float)x.h[i];
    }
};

// sum over the 256 threads of a block; the result is valid in thread 0
__device__ __forceinline__ void block_sum2(float &a, float &b, float (*red)[2]) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        a += __shfl_xor(a, o);
        b += __shfl_xor(b, o);
    }
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) red[wave][0] = a, red[wave][1] = b;
    __syncthreads();
    if (threadIdx.x == 0) {
        a = red[0][0] + red[1][0] + red[2][0] + red[3][0];
        b = red[0][1] + red[1][1] + red[2][1] + red[3][1];
    }
}

// contiguous layout: block = (chunk, image * C + channel); VEC elements per load
// (1: any alignment)
template <typename T, int VEC>
__global__ void __launch_bounds__(256)
partial_nchw_kernel(const T *__restrict__ x, float *__restrict__ part, long HW, long seg, int chunks) {
    __shared__ float red[4][2];
    const long bc = blockIdx.y;
    const int chunk = blockIdx.x;
    const T *xc = x + bc * HW;
    const float shift = (float)xc[0];
    const long lo = chunk * seg, hi = lo + seg < HW ? lo + seg : HW;
    float s1 = 0.f, s2 = 0.f;
    if constexpr (VEC == 1) {
        for (long i = lo + threadIdx.x; i < hi; i += 256) {
            const float v = (float)xc[i] - shift;
            s1 += v;
            s2 = fma_(v, v, s2);
        }
    } else {
        for (long i = lo + (long)threadIdx.x * VEC; i < hi; i += 256 * VEC) {
            float v[VEC];
            Pack<T, VEC>::load(xc + i, v);
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const float t = v[e] - shift;
                s1 += t;
                s2 = fma_(t, t, s2);
            }
        }
    }
    block_sum2(s1, s2, red);
    if (threadIdx.x == 0) {
        part[(bc * chunks + chunk) * 2] = s1;
        part[(bc * chunks + chunk) * 2 + 1] = s2;
    }
}

#ifndef SAPA_MOMENTS_UNROLL
#define SAPA_MOMENTS_UNROLL 8
#endif
// channels-last layout: block = (chunk, image); thread = (pixel lane, group of
// CPT channels); SAPA_MOMENTS_UNROLL pixels per thread are in flight at a time
template <typename T, int CPT>
__global__ void __launch_bounds__(256)
partial_nhwc_kernel(const T *__restrict__ x, float *__restrict__ part, int C, long HW, long seg,
                    int chunks) {
    __shared__ float red[256][2 * CPT];
    const int b = blockIdx.y, chunk = blockIdx.x;
    const int nq = C / CPT, npl = 256 / nq;            // channel groups, pixel lanes
    const int quad = threadIdx.x % nq, pl = threadIdx.x / nq;
    const T *xb = x + (long)b * HW * C + CPT * quad;
    float shift[CPT], s1[CPT], s2[CPT];
    Pack<T, CPT>::load(xb, shift);
#pragma unroll
    for (int e = 0; e < CPT; ++e) s1[e] = 0.f, s2[e] = 0.f;
    const long lo = chunk * seg, hi = lo + seg < HW ? lo + seg : HW;
    if (pl < npl) {
        long p = lo + pl;
        constexpr int U = SAPA_MOMENTS_UNROLL;
        for (; p + (U - 1) * npl < hi; p += U * npl) {
            float v[U][CPT];
#pragma unroll
            for (int u = 0; u < U; ++u) Pack<T, CPT>::load(xb + (p + u * npl) * C, v[u]);
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int e = 0; e < CPT; ++e) {
                    const float t = v[u][e] - shift[e];
                    s1[e] += t;
                    s2[e] = fma_(t, t, s2[e]);
                }
        }
        for (; p < hi; p += npl) {
            float v[CPT];
            Pack<T, CPT>::load(xb + p * C, v);
#pragma unroll
            for (int e = 0; e < CPT; ++e) {
                const float t = v[e] - shift[e];
                s1[e] += t;
                s2[e] = fma_(t, t, s2[e]);
            }
        }
    }
#pragma unroll
    for (int e = 0; e < CPT; ++e) red[threadIdx.x][e] = s1[e], red[threadIdx.x][CPT + e] = s2[e];
    __syncthreads();
    if (pl == 0) {
        float *out = part + (((long)b * chunks + chunk) * C + CPT * quad) * 2;
#pragma unroll
        for (int e = 0; e < CPT; ++e) {
            float a = 0.f, q = 0.f;
            for (int l = 0; l < npl; ++l) a += red[l * nq + quad][e], q += red[l * nq + quad][CPT + e];
            out[2 * e] = a;
            out[2 * e + 1] = q;
        }
    }
}

// thread = (image, channel): the chunks in order
template <typename T, bool CL>
__global__ void __launch_bounds__(256)
finish_kernel(const T *__restrict__ x, const float *__restrict__ part, float *__restrict__ mean_var,
              int B, int C, long HW, int chunks) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= (long)B * C) return;
    const int b = (int)(i / C), c = (int)(i % C);
    float s1 = 0.f, s2 = 0.f;
    auto at = [&](int k) { return CL ? part + (((long)b * chunks + k) * C + c) * 2 : part + (i * chunks + k) * 2; };
    // (eight chunks' loads in flight at a time; the additions in the chunks' order)
    int k = 0;
    for (; k + 8 <= chunks; k += 8) {
        float a[8], q[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) a[u] = at(k + u)[0], q[u] = at(k + u)[1];
#pragma unroll
        for (int u = 0; u < 8; ++u) s1 += a[u], s2 += q[u];
    }
    for (; k < chunks; ++k) {
        s1 += at(k)[0];
        s2 += at(k)[1];
    }
    const float shift = (float)(CL ? x[(long)b * HW * C + c] : x[i * HW]);
    const float m = s1 / (float)HW;
    mean_var[2 * i] = shift + m;
    mean_var[2 * i + 1] = __builtin_fmaxf(s2 / (float)HW - m * m, 0.f);
}

// pixels per chunk and number of chunks: about `target` blocks in all, at least
// `min_px` pixels per chunk
static void chunking(long HW, long blocks_per_chunk_set, long target, long min_px, long &seg,
                     int &chunks) {
    long want = (target + blocks_per_chunk_set - 1) / blocks_per_chunk_set;
    long most = (HW + min_px - 1) / min_px;
    long n = want < most ? want : most;
    if (n < 1) n = 1;
    if (n > 4096) n = 4096;
    seg = (HW + n - 1) / n;
    seg = (seg + 7) / 8 * 8;                       // whole 16-byte loads in every chunk
    chunks = (int)((HW + seg - 1) / seg);
}
#ifndef SAPA_MOMENTS_CL_TUNE
#define SAPA_MOMENTS_CL_TUNE 2048, 1024
#endif
static void chunking_for(long HW, int B, int C, bool cl, long &seg, int &chunks) {
    if (cl) chunking(HW, B, SAPA_MOMENTS_CL_TUNE, seg, chunks);
    else chunking(HW, (long)B * C, 4096, 512, seg, chunks);
}

template <typename T>
static hipError_t launch_t(const T *x, float *ws, float *mean_var, int B, int C, long HW, bool cl,
                           hipStream_t st) {
    long seg;
    int chunks;
    if (cl) {
        chunking_for(HW, B, C, true, seg, chunks);
        // 16 bytes per lane where the channel count and the alignment allow it
        constexpr int WIDE = 16 / (int)sizeof(T);
        if (WIDE == 8 && C % 8 == 0 && (uintptr_t)x % 16 == 0)
            hipLaunchKernelGGL((partial_nhwc_kernel<T, WIDE>), dim3(chunks, B), dim3(256), 0, st, x, ws, C,
                               HW, seg, chunks);
        else
            hipLaunchKernelGGL((partial_nhwc_kernel<T, 4>), dim3(chunks, B), dim3(256), 0, st, x, ws, C,
                               HW, seg, chunks);
        hipLaunchKernelGGL((finish_kernel<T, true>), dim3(((long)B * C + 255) / 256), dim3(256), 0, st, x,
                           ws, mean_var, B, C, HW, chunks);
    } else {
        chunking_for(HW, B, C, false, seg, chunks);
        constexpr int VEC = 16 / (int)sizeof(T);
        const dim3 grid(chunks, B * C);
        if (HW % VEC == 0 && (uintptr_t)x % 16 == 0)
            hipLaunchKernelGGL((partial_nchw_kernel<T, VEC>), grid, dim3(256), 0, st, x, ws, HW, seg, chunks);
        else
            hipLaunchKernelGGL((partial_nchw_kernel<T, 1>), grid, dim3(256), 0, st, x, ws, HW, seg, chunks);
        hipLaunchKernelGGL((finish_kernel<T, false>), dim3(((long)B * C + 255) / 256), dim3(256), 0, st, x,
                           ws, mean_var, B, C, HW, chunks);
    }
    return hipGetLastError();
}

// GroupNorm folded into a 1x1 projection, per image: from the (image, channel)
// moments, gamma / beta and the projection's weight W [O, C] and bias,
//   rstd_g   = 1 / sqrt(var_g + eps),  group moments from the channel moments
//   W'[b,o,c] = W[o,c] * gamma[c] * rstd_g(c)
//   b'[b,o]   = bias[o] + sum_c W[o,c] * (beta[c] - mean_g(c) * gamma[c] * rstd_g(c))
// so that  conv(groupnorm(x))[b] = W'[b] x[b] + b'[b].  Block = (image, 4 output
// rows): scale and shift of every channel go through LDS (recomputed per block:
// a few hundred operations), then one wave per output row.
template <typename T>
__global__ void __launch_bounds__(256)
fold_kernel(const float *__restrict__ mean_var, const T *__restrict__ gamma,
            const T *__restrict__ beta, const T *__restrict__ w, const T *__restrict__ bias,
            T *__restrict__ w_out, T *__restrict__ b_out, int C, int O, int G, float eps) {
    extern __shared__ float sh[];                  // scale[C], shift[C]
    float *scale = sh, *shift = sh + C;
    const int b = blockIdx.x, per = C / G;
    const float *mv = mean_var + (long)b * C * 2;
    for (int g = threadIdx.x; g < G; g += 256) {
        float m = 0.f;
        for (int c = g * per; c < (g + 1) * per; ++c) m += mv[2 * c];
        m /= (float)per;
        float v = 0.f;
        for (int c = g * per; c < (g + 1) * per; ++c) {
            const float dm = mv[2 * c] - m;
            v += mv[2 * c + 1] + dm * dm;
        }
        const float rstd = 1.f / __builtin_sqrtf(v / (float)per + eps);
        for (int c = g * per; c < (g + 1) * per; ++c) {
            const float ga = gamma ? (float)gamma[c] : 1.f, be = beta ? (float)beta[c] : 0.f;
            scale[c] = ga * rstd;
            shift[c] = be - m * ga * rstd;
        }
    }
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int o = blockIdx.y * 4 + wave; o < O; o += 4 * gridDim.y) {
        const T *wr = w + (long)o * C;
        T *wo = w_out + ((long)b * O + o) * C;
        float acc = 0.f;
        for (int c = lane; c < C; c += 64) {
            const float x = (float)wr[c];
            wo[c] = (T)(x * scale[c]);
            acc = fma_(x, shift[c], acc);
        }
#pragma unroll
        for (int d = 32; d > 0; d >>= 1) acc += __shfl_xor(acc, d);
        if (lane == 0) b_out[(long)b * O + o] = (T)(acc + (bias ? (float)bias[o] : 0.f));
    }
}

template <typename T>
static hipError_t fold_t(const float *mean_var, const void *gamma, const void *beta, const void *w,
                         const void *bias, void *w_out, void *b_out, int B, int C, int O, int G,
                         float eps, hipStream_t st) {
    hipLaunchKernelGGL((fold_kernel<T>), dim3(B, (O + 3) / 4), dim3(256), 2 * C * sizeof(float), st, mean_var,
                       (const T *)gamma, (const T *)beta, (const T *)w, (const T *)bias, (T *)w_out,
                       (T *)b_out, C, O, G, eps);
    return hipGetLastError();
}

}  // namespace moments

// bytes of workspace channel_moments_launch needs for these extents
long channel_moments_workspace(int B, int C, long HW, bool channels_last) {
    long seg;
    int chunks;
    moments::chunking_for(HW, B, C, channels_last, seg, chunks);
    return (long)B * C * chunks * 2 * (long)sizeof(float);
}

// x: [B, C, HW] contiguous or [B, HW, C] (channels_last), f32 / f16 / bf16;
// mean_var: [B, C, 2] fp32.  Channels-last needs C % 4 == 0, C <= 1024 and x
// aligned to 4 elements; the contiguous layout B * C <= 65535.
// hipErrorNotSupported otherwise.
hipError_t channel_moments_launch(const void *x, void *workspace, float *mean_var, int B, int C,
                                  long HW, bool channels_last, int dtype, hipStream_t st) {
    if (channels_last) {
        const int esize = dtype == 0 ? 4 : 2;
        if (C % 4 != 0 || C > 1024 || (uintptr_t)x % (4 * esize) != 0 || B > 65535)
            return hipErrorNotSupported;
    } else if ((long)B * C > 65535) {
        return hipErrorNotSupported;
    }
    float *ws = (float *)workspace;
    switch (dtype) {
        case 0: return moments::launch_t((const float *)x, ws, mean_var, B, C, HW, channels_last, st);
        case 2: return moments::launch_t((const f16_t *)x, ws, mean_var, B, C, HW, channels_last, st);
        case 3: return moments::launch_t((const bf16_t *)x, ws, mean_var, B, C, HW, channels_last, st);
        default: return hipErrorNotSupported;
    }
}

// ---- the same statistics for callers that cannot bring a workspace ----
//
// The partial sums go to a fixed array in device memory that is part of the
// library's code object: no allocation on any path, so the call can be made
// under stream capture or from a loop that must not touch the allocator.
// Every device holds its own copy of the array at its own address; host code
// only ever uses the address hipGetSymbolAddress reports for the current
// device (the array's name is not a device address on the host side).
}  // namespace sapa

constexpr long kStaticScratchBytes = 8L << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices] = {};

// address of `scratch` on the current device; looked up once per device
hipError_t scratch_address(void **out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        if (!p) return hipErrorInvalidSymbol;
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return hipSuccess;
}
}  // namespace

namespace sapa {

long channel_moments_static_capacity() { return kStaticScratchBytes; }

// channel_moments_launch with the partial sums in the library's own fixed
// array.  The caller has checked that channel_moments_workspace(...) fits
// channel_moments_static_capacity().  Every partial sum that the second kernel
// reads is written by the first one of the same call, so nothing has to be
// cleared between calls; two calls in flight on one device share the array and
// must not overlap.
hipError_t channel_moments_static_launch(const void *x, float *mean_var, int B, int C, long HW,
                                         bool channels_last, int dtype, hipStream_t st) {
    if (channel_moments_workspace(B, C, HW, channels_last) > kStaticScratchBytes)
        return hipErrorInvalidValue;
    void *ws = nullptr;
    const hipError_t e = scratch_address(&ws);
    if (e != hipSuccess) return e;
    return channel_moments_launch(x, ws, mean_var, B, C, HW, channels_last, dtype, st);
}

// mean_var [B, C, 2] fp32 (channel_moments_launch); gamma, beta [C] or null, w
// [O, C], bias [O] or null, all of type `dtype` (f32 / f16 / bf16); w_out
// [B, O, C] and b_out [B, O] of the same type.  C % G == 0, C <= 8192.
hipError_t groupnorm_fold_launch(const float *mean_var, const void *gamma, const void *beta,
                                 const void *w, const void *bias, void *w_out, void *b_out, int B,
                                 int C, int O, int G, float eps, int dtype, hipStream_t st) {
    if (G < 1 || C % G != 0 || C > 8192) return hipErrorNotSupported;
    switch (dtype) {
        case 0: return moments::fold_t<float>(mean_var, gamma, beta, w, bias, w_out, b_out, B, C, O, G, eps, st);
        case 2: return moments::fold_t<f16_t>(mean_var, gamma, beta, w, bias, w_out, b_out, B, C, O, G, eps, st);
        case 3: return moments::fold_t<bf16_t>(mean_var, gamma, beta, w, bias, w_out, b_out, B, C, O, G, eps, st);
        default: return hipErrorNotSupported;
    }
}

}  // namespace sapa
