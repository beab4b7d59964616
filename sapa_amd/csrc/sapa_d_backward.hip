// Backward pass of the fused SAPA-D operator
//   out = deform_av(softmax(deform_qk(q, key, offset), dim = points), value, offset)
// (SAPADeform.attention, sapa_deform.py:51-53) in one call: the chain of the two
// reference backward functions (deform_qk.cpp:50-70 -> DeformQKBackward,
// deform_av.cpp:50-70 -> DeformAVBackward) with the softmax between them.
//
// The attention weights and the gradient of the logits, [B, G, P, sH, sW], live
// in the caller's workspace as fp32 whatever the tensors' type is; f16 / bf16
// features, offsets and gradients are read and written as they are (no fp32
// copies of them), and the low-res gradients, which are sums of many terms, are
// accumulated in fp32 and rounded once.
//
//   attn        = softmax(deform_qk(q, key))                    sampled similarity
//   grad_attn   = deform_qk(grad_out, value)                    (the same kernel)
//   grad_logits = attn * (grad_attn - sum_p attn * grad_attn)
//   grad_value  = scatter(grad_out, attn);   grad_offset  = d/d offset of the aggregation
//   grad_query  = deform_av(grad_logits, key)                   sampled aggregation
//   grad_key    = scatter(q, grad_logits);   grad_offset += d/d offset of the similarity
#include "kernels.hpp"

namespace sapa {

namespace dbwd {

// grad_logits = attn * (grad_attn - sum_r attn * grad_attn) over the middle axis
// of [N, R, M], in place on g; one thread per (n, m)
__global__ void __launch_bounds__(256)
softmax_backward_kernel(const float *__restrict__ attn, float *__restrict__ g, long N, int R, long M) {
    const long total = N * M;
    for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
         idx += (long)gridDim.x * blockDim.x) {
        const long n = idx / M, m = idx % M;
        const float *ap = attn + n * R * M + m;
        float *gp = g + n * R * M + m;
        float dot = 0.f;
        for (int j = 0; j < R; ++j) dot = fma_(ap[j * M], gp[j * M], dot);
        for (int j = 0; j < R; ++j) gp[j * M] = ap[j * M] * (gp[j * M] - dot);
    }
}

__global__ void __launch_bounds__(256) zero_kernel(float *__restrict__ x, long n) {
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x)
        x[i] = 0.f;
}

template <typename T>
__global__ void __launch_bounds__(256) narrow_kernel(const float *__restrict__ x, T *__restrict__ y, long n) {
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x)
        y[i] = (T)x[i];
}

static unsigned blocks_for(long n) {
    const long b = (n + 255) / 256;
    return (unsigned)(b < 1 ? 1 : (b > 65536 ? 65536 : b));
}

static long align256(long x) { return (x + 255) / 256 * 256; }

// One low-res gradient (grad_key from q and the gradient of the logits, grad_value
// from grad_out and the attention weights), a sum of many terms: accumulated in
// fp32 in `acc` and rounded once.  The matrix-product scatter, where it applies,
// accumulates in channels-last order (a cell's channels in one piece: its final
// atomics then fall on two cache lines per instruction instead of one per window
// row and channel) and a transposing pass writes the tensor; else the LDS-window
// scatter accumulates in the tensor's own order.
static bool low_gradient_channels_last(int B, int Cx, int H, int W, int P, int s, int G, int dtype) {
#ifdef SAPA_SCATTER_MAT_OFF
    return false;
#else
    return deform_scatter_mat_serves(B, Cx, H, W, P, s, G, dtype);
#endif
}

// (cleared: `acc` was cleared by an earlier launch already -- channels-last accumulation only)
static hipError_t low_gradient(const void *hi, const void *sc, const void *offset, float *acc, void *grad_low,
                               int B, int Cx, int H, int W, int P, int s, int G, int dtype, hipStream_t st,
                               bool cleared) {
    const bool wide = dtype != 0;
    const long n = (long)B * Cx * H * W;
    const bool mat = low_gradient_channels_last(B, Cx, H, W, P, s, G, dtype);
    float *const target = (mat || wide) ? acc : (float *)grad_low;
    hipError_t e = hipSuccess;
    if (!(mat && cleared)) {
        hipLaunchKernelGGL(zero_kernel, dim3(blocks_for(n)), dim3(256), 0, st, target, n);
        e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    if (mat) {
        e = deform_scatter_mat_launch(hi, sc, offset, acc, B, Cx, H, W, P, s, G, dtype, st, wide, true);
        if (e != hipSuccess) return e;
        return nhwc_f32_to_nchw_launch(acc, grad_low, Cx, B, (long)H * W, dtype, st);
    }
    e = deform_lowgrad_lds_launch(hi, sc, offset, target, B, Cx, H, W, P, s, G, dtype, st, wide);
    if (e != hipSuccess || !wide) return e;
    if (dtype == 2) hipLaunchKernelGGL(narrow_kernel<f16_t>, dim3(blocks_for(n)), dim3(256), 0, st, acc, (f16_t *)grad_low, n);
    else hipLaunchKernelGGL(narrow_kernel<bf16_t>, dim3(blocks_for(n)), dim3(256), 0, st, acc, (bf16_t *)grad_low, n);
    return hipGetLastError();
}

// The per-pixel part of the chain (attention weights, gradient of the logits,
// grad_offset, grad_query) in one matrix-form kernel instead of five launches
// of per-pixel gathers.  (B=8, C=256, G=4, d=32, 64x64 -> 128x128, fp32: the
// whole backward call with / without it, us: P = 25 ... ; P = 9 ...; P = 5 ...)
static bool matrix_stage(int B, int Cq, int C, int H, int W, int P, int s, int G, int dtype) {
#ifdef SAPA_BWD_MAT_OFF
    return false;
#else
    return deform_bwd_wmat_serves(B, Cq, C, H, W, P, s, G, dtype);
#endif
}



template <typename T>
__global__ void __launch_bounds__(256) widen_kernel(const T *__restrict__ x, float *__restrict__ y, long n) {
    for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x)
        y[i] = (float)x[i];
}

static hipError_t widen(const void *x, float *y, long n, int dtype, hipStream_t st) {
    if (dtype == 2) hipLaunchKernelGGL(widen_kernel<f16_t>, dim3(blocks_for(n)), dim3(256), 0, st, (const f16_t *)x, y, n);
    else hipLaunchKernelGGL(widen_kernel<bf16_t>, dim3(blocks_for(n)), dim3(256), 0, st, (const bf16_t *)x, y, n);
    return hipGetLastError();
}

}  // namespace dbwd

// ---- the separate sampled operators' backward passes on f16 / bf16 tensors, read and
// written as they are (the reference dispatches DeformQKBackward / DeformAVBackward on
// half directly, deform_qk_cuda_kernel.cu:298-337, deform_av_cuda_kernel.cu:294-333).
// The per-pixel gradients come from the forward kernels with swapped roles on the 16-bit
// tensors; the low-res gradient, a sum of many terms, is accumulated in fp32 in the
// workspace (next to an fp32 copy of the per-point tensor, which the scatter kernels
// take) and rounded once.
long deform_separate_backward_workspace(int B, int Cx, int H, int W, int P, int s, int G, int dtype) {
    using dbwd::align256;
    if (dtype != 2 && dtype != 3) return 0;
    if (s != 1 && s != 2 && s != 4) return 0;
    if (P > 48) return 0;
    return align256((long)B * G * P * H * s * W * s * 4) + align256((long)B * Cx * H * W * 4);
}

// which = 0: gradients of deform_qk -- a = query, low = key, pp = grad_out [B,G,P,sH,sW];
//            grad_a = grad_query, grad_low = grad_key;
// which = 1: gradients of deform_av -- a = grad_out [B,C,sH,sW], low = value, pp = attn;
//            grad_pp = grad_attn, grad_low = grad_value.
// Any gradient may be NULL.
hipError_t deform_separate_backward_launch(int which, const void *a, const void *low, const void *pp,
                                           const void *offset, void *workspace, void *grad_a_or_pp,
                                           void *grad_low, void *grad_offset, int B, int Cx, int H, int W,
                                           int P, int s, int G, int dtype, hipStream_t st) {
    using namespace dbwd;
    if (deform_separate_backward_workspace(B, Cx, H, W, P, s, G, dtype) == 0) return hipErrorNotSupported;
    if (!workspace || (uintptr_t)workspace % 256 != 0) return hipErrorNotSupported;
    const long n_pp = (long)B * G * P * H * s * W * s;
    float *pp32 = (float *)workspace;
    float *acc = (float *)((char *)workspace + align256(n_pp * 4));
    const int HIRES = 0;
    hipError_t e;
#define SAPA_STEP(call)                  \
    do {                                 \
        e = (call);                      \
        if (e != hipSuccess) return e;   \
    } while (0)
    if (grad_a_or_pp) {
        if (which == 0)   // grad_query: the sampled aggregation of key with grad_out as the weights
            SAPA_STEP(deform_lds_launch(1, nullptr, nullptr, pp, low, offset, grad_a_or_pp, B, Cx, Cx, H, W, P, s, G,
                                        HIRES, dtype, st));
        else              // grad_attn: the sampled similarity of grad_out and value
            SAPA_STEP(deform_lds_launch(0, a, low, nullptr, nullptr, offset, grad_a_or_pp, B, Cx, Cx, H, W, P, s, G,
                                        HIRES, dtype, st));
    }
    if (grad_offset)
        SAPA_STEP(deform_lds_launch(3, a, low, pp, nullptr, offset, grad_offset, B, Cx, Cx, H, W, P, s, G, HIRES,
                                    dtype, st));
    if (grad_low) {
        SAPA_STEP(widen(pp, pp32, n_pp, dtype, st));
        SAPA_STEP(low_gradient(a, pp32, offset, acc, grad_low, B, Cx, H, W, P, s, G, dtype, st, false));
    }
#undef SAPA_STEP
    return hipSuccess;
}

// Bytes of workspace, or 0 for configurations this call does not serve (the
// caller then chains the separate backward entry points): f32 / f16 / bf16,
// s in {1, 2, 4}, P small enough for the LDS kernels.
long deform_fused_backward_workspace(int B, int Cq, int C, int H, int W, int P, int s, int G, int dtype) {
    using dbwd::align256;
    if (dtype != 0 && dtype != 2 && dtype != 3) return 0;
    if (s != 1 && s != 2 && s != 4) return 0;
    if (P > 48) return 0;       // [2P][thread] sums of the offset gradient next to the window in LDS
    const long per_point = (long)B * G * P * H * s * W * s * (long)sizeof(float);
    long n = 2 * align256(per_point);
    // fp32 accumulators of the low-res gradients
    n += align256((long)B * Cq * H * W * 4) + align256((long)B * C * H * W * 4);
    if (dbwd::matrix_stage(B, Cq, C, H, W, P, s, G, dtype)) {
        // channels-last copies of key and value for the matrix-form kernel
        const long esize = dtype == 0 ? 4 : 2;
        n += align256((long)B * Cq * H * W * esize) + align256((long)B * C * H * W * esize);
    } else if (dtype != 0) {
        // the first half of grad_offset in fp32
        n += align256(2 * per_point);
    }
    return n;
}

// Any of the four gradients may be NULL.  hipErrorNotSupported before anything
// is written when the configuration is not served.
hipError_t deform_fused_backward_launch(const void *grad_out, const void *q, const void *key,
                                        const void *value, const void *offset, void *workspace,
                                        void *grad_q, void *grad_key, void *grad_value,
                                        void *grad_offset, int B, int Cq, int C, int H, int W, int P,
                                        int s, int G, int dtype, hipStream_t st) {
    using namespace dbwd;
    if (deform_fused_backward_workspace(B, Cq, C, H, W, P, s, G, dtype) == 0) return hipErrorNotSupported;
    if (!workspace || (uintptr_t)workspace % 256 != 0) return hipErrorNotSupported;
    const bool wide = dtype != 0;
    const long hpix = (long)H * s * W * s, lpix = (long)H * W;
    const long n_pp = (long)B * G * P * hpix;
    char *w = (char *)workspace;
    float *attn = (float *)w;
    float *gl = (float *)(w + align256(n_pp * 4));
    float *gk32 = (float *)(w + 2 * align256(n_pp * 4));
    float *gv32 = (float *)((char *)gk32 + align256((long)B * Cq * lpix * 4));
    char *rest = (char *)gv32 + align256((long)B * C * lpix * 4);
    const bool mat = matrix_stage(B, Cq, C, H, W, P, s, G, dtype);
    float *goff32 = wide && !mat ? (float *)rest : nullptr;
    const int HIRES = 0;
    bool cleared = false;
    hipError_t e;
#define SAPA_STEP(call)                  \
    do {                                 \
        e = (call);                      \
        if (e != hipSuccess) return e;   \
    } while (0)

    if (mat) {
        const long esize = wide ? 2 : 4;
        char *key_cl = rest, *value_cl = rest + align256((long)B * Cq * lpix * esize);
        // (the accumulators of grad_key / grad_value have the copies' extents and, where
        // they are channels-last, their order: cleared by the same launch)
        SAPA_STEP(nchw_to_nhwc_launch(key, key_cl, Cq, value, value_cl, C, B, lpix, (int)esize, st,
                                      grad_key && low_gradient_channels_last(B, Cq, H, W, P, s, G, dtype) ? gk32 : nullptr,
                                      grad_value && low_gradient_channels_last(B, C, H, W, P, s, G, dtype) ? gv32 : nullptr,
                                      &cleared));
        SAPA_STEP(deform_bwd_wmat_launch(grad_out, q, key_cl, value_cl, offset, attn, gl, grad_q, grad_offset, B,
                                         Cq, C, H, W, P, s, G, dtype, st));
    } else {
        // attention weights: sampled similarity (mode 0), softmax over the points
        SAPA_STEP(deform_lds_launch(0, q, key, nullptr, nullptr, offset, attn, B, Cq, Cq, H, W, P, s, G, HIRES,
                                    dtype, st, wide));
        SAPA_STEP(softmax_generic_launch(attn, attn, (long)B * G, P, hpix, 0, st));
        // gradient of the weights: the similarity of grad_out and value
        SAPA_STEP(deform_lds_launch(0, grad_out, value, nullptr, nullptr, offset, gl, B, C, C, H, W, P, s, G,
                                    HIRES, dtype, st, wide));
        hipLaunchKernelGGL(softmax_backward_kernel, dim3(blocks_for((long)B * G * hpix)), dim3(256), 0, st, attn,
                           gl, (long)B * G, P, hpix);
        SAPA_STEP(hipGetLastError());
        // grad_offset: the aggregation's share, then the similarity's
        if (grad_offset) {
            SAPA_STEP(deform_lds_launch(3, grad_out, value, attn, nullptr, offset, grad_offset, B, C, C, H, W, P, s,
                                        G, HIRES, dtype, st, wide, false, goff32));
            SAPA_STEP(deform_lds_launch(3, q, key, gl, nullptr, offset, grad_offset, B, Cq, Cq, H, W, P, s, G, HIRES,
                                        dtype, st, wide, true, goff32));
        }
        // grad_query: aggregation of key with the gradient of the logits
        if (grad_q)
            SAPA_STEP(deform_lds_launch(1, nullptr, nullptr, gl, key, offset, grad_q, B, Cq, Cq, H, W, P, s, G, HIRES,
                                        dtype, st, wide));
    }
    // the low-res gradients: grad_value (attention weights x grad_out) and
    // grad_key (gradient of the logits x query), scattered
    if (grad_value) SAPA_STEP(low_gradient(grad_out, attn, offset, gv32, grad_value, B, C, H, W, P, s, G, dtype, st, cleared));
    if (grad_key) SAPA_STEP(low_gradient(q, gl, offset, gk32, grad_key, B, Cq, H, W, P, s, G, dtype, st, cleared));
#undef SAPA_STEP
    return hipSuccess;
}

}  // namespace sapa
