// extern "C" entry points of libsapa_hip.so (declared in include/sapa_hip.h):
// argument validation, kernel selection, error mapping.  No allocation, no
// global state apart from a thread-local copy of the last HIP error text.
#include "../../include/sapa_hip.h"

#include <string.h>

#include "kernels.hpp"

using namespace sapa;

namespace {

thread_local char g_hip_error[256] = "";
// kernel that took the calling thread's last forward request (sapa_hip_last_kernel)
thread_local const char *g_last_kernel = "";

// runs one candidate launcher; when it takes the request (anything but
// hipErrorNotSupported) its kernel's name is recorded
hipError_t took(const char *kernel, hipError_t e) {
    if (e != hipErrorNotSupported) g_last_kernel = kernel;
    return e;
}

int fail_hip(hipError_t e) {
    strncpy(g_hip_error, hipGetErrorString(e), sizeof(g_hip_error) - 1);
    g_hip_error[sizeof(g_hip_error) - 1] = 0;
    return SAPA_ERR_LAUNCH;
}

int finish(hipError_t e) { return e == hipSuccess ? SAPA_OK : fail_hip(e); }

bool dtype_ok(int dt) { return dt >= SAPA_F32 && dt <= SAPA_BF16; }

// element counts stay below 2^40 and extents below 2^24 so that the kernels'
// 64-bit flat indices and 32-bit in-plane indices cannot overflow
const long long kMaxElems = 1LL << 40;

// fused K = 5, s = 2 problems of at most this many low-res cells go to the matrix-pipe kernel
const long kSmallFusedCells = 12288;

// LDS-tiled SAPA-B kernel for `mode`: the VALU kernel where it has an
// instance (K = 5, s = 2, where it is the faster one), else the matrix-pipe
// kernel; hipErrorNotSupported when neither covers the request.
hipError_t tiled_launch(int mode, const void *q, const void *key, const void *attn_in,
                        const void *value, void *out, int B, int d, int C, int H, int W, int K,
                        int s, int dtype, hipStream_t st) {
    // 16-bit fused problems of the common window first: both products on the 16-bit matrix
    // instructions, whatever the size (B=8, d=32, C=256, bf16: 32x32 21 -> 16 us, 64x64 48 -> 20 us)
    hipError_t e = hipErrorNotSupported;
#ifndef SAPA_WMAT16_OFF
    e = took("sapa_b_wmat16_kernel", sapa_b_wmat16_launch(mode, q, key, value, out, B, d, C, H, W, K, s, dtype, st));
#endif
    // small fused problems next: the matrix-pipe kernel's lane-per-child decomposition fills the
    // chip where the thread-per-parent kernels leave it latency-bound
    // (B=8, d=32, C=256, fp32: 16x16 32 -> 12 us, 32x32 32 -> 23 us)
    if (e == hipErrorNotSupported && K == 5 && s == 2 && dtype != SAPA_F64 && mode == TILED_FUSED &&
        (long)B * H * W <= kSmallFusedCells)
        e = took("sapa_b_mfma_kernel",
                 sapa_b_mfma_launch(mode, q, key, attn_in, value, out, B, d, C, H, W, K, s, dtype, st));
    if (e == hipErrorNotSupported)
        e = took("sapa_b_dot2_kernel", sapa_b_dot2_launch(mode, q, key, attn_in, value, out, B,
                                                          d, C, H, W, K, s, dtype, st));
    if (e == hipErrorNotSupported)
        e = took("sapa_b_tiled_kernel",
                 sapa_b_tiled_launch(mode, q, key, attn_in, value, out, B, d, C, H, W, K, s, dtype, st));
    if (e == hipErrorNotSupported)
        e = took("sapa_b_mfma_kernel",
                 sapa_b_mfma_launch(mode, q, key, attn_in, value, out, B, d, C, H, W, K, s, dtype, st));
    return e;
}

// grad_low / grad_offset of a sampled op (hi = per-channel high-res tensor,
// sc = per-point scalar tensor, low = sampled tensor): the LDS kernels where
// they apply, the per-term kernel for whatever they leave.
hipError_t deform_lowgrad_any(const void *hi, const void *sc, const void *low, const void *offset,
                              void *grad_low, void *grad_offset, int B, int Cx, int H, int W,
                              int P, int s, int G, int dtype, hipStream_t st) {
    if (grad_offset) {
        const hipError_t e = deform_lds_launch(3, hi, low, sc, nullptr, offset, grad_offset, B, Cx,
                                               Cx, H, W, P, s, G, SAPA_OFFSET_HIRES, dtype, st);
        if (e == hipSuccess) grad_offset = nullptr;
        else if (e != hipErrorNotSupported) return e;
    }
    if (grad_low) {
        // the matrix-product form first (SAPA_SCATTER_MAT_OFF: a tuning build without it),
        // then the LDS-window scatter
#ifdef SAPA_SCATTER_MAT_OFF
        hipError_t e = hipErrorNotSupported;
#else
        hipError_t e = deform_scatter_mat_launch(hi, sc, offset, grad_low, B, Cx, H, W, P, s, G, dtype, st);
#endif
        if (e == hipErrorNotSupported)
            e = deform_lowgrad_lds_launch(hi, sc, offset, grad_low, B, Cx, H, W, P, s, G, dtype, st);
        if (e == hipSuccess) grad_low = nullptr;
        else if (e != hipErrorNotSupported) return e;
    }
    if (!grad_low && !grad_offset) return hipSuccess;
    return deform_lowgrad_launch(hi, sc, low, offset, grad_low, grad_offset, B, Cx, H, W, P, s, G,
                                 dtype, st);
}

// Low-res gradient of qk / av: tiled scatter where it applies, else the
// gather kernel.
hipError_t lowres_grad_any(const void *hi, const void *w, void *out, int B, int C, int H, int W,
                           int K, int s, int dtype, hipStream_t st) {
    hipError_t e = lowres_grad_tiled_launch(hi, w, out, B, C, H, W, K, s, dtype, st);
    if (e == hipErrorNotSupported)
        e = lowres_grad_generic_launch(hi, w, out, B, C, H, W, K, s, dtype, st);
    return e;
}

// The sampled forward ops: LDS-windowed kernel where it applies, else the
// global-memory kernel.
hipError_t deform_qk_any(const void *q, const void *key, const void *offset, void *out, int B,
                         int Cq, int H, int W, int P, int s, int G, int olayout, int dtype,
                         hipStream_t st) {
    hipError_t e = took("deform_lds_kernel", deform_lds_launch(0, q, key, nullptr, nullptr, offset, out, B,
                                                                Cq, Cq, H, W, P, s, G, olayout, dtype, st));
    if (e == hipErrorNotSupported)
        e = took("deform_qk_forward_kernel",
                 deform_qk_forward_launch(q, key, offset, out, B, Cq, H, W, P, s, G, olayout, dtype, st));
    return e;
}

hipError_t deform_av_any(const void *attn, const void *value, const void *offset, void *out, int B,
                         int C, int H, int W, int P, int s, int G, int olayout, int dtype,
                         hipStream_t st) {
    hipError_t e = took("deform_lds_kernel", deform_lds_launch(1, nullptr, nullptr, attn, value, offset, out,
                                                                B, C, C, H, W, P, s, G, olayout, dtype, st));
    if (e == hipErrorNotSupported)
        e = took("deform_av_forward_kernel",
                 deform_av_forward_launch(attn, value, offset, out, B, C, H, W, P, s, G, olayout, dtype, st));
    return e;
}

hipError_t deform_fused_any(const void *q, const void *key, const void *value, const void *offset,
                            void *out, int B, int Cq, int C, int H, int W, int P, int s, int G,
                            int olayout, int dtype, hipStream_t st) {
    hipError_t e = took("deform_lds_kernel", deform_lds_launch(2, q, key, nullptr, value, offset, out, B, Cq,
                                                                C, H, W, P, s, G, olayout, dtype, st));
    if (e == hipErrorNotSupported)
        e = took("deform_fused_forward_kernel",
                 deform_fused_forward_launch(q, key, value, offset, out, B, Cq, C, H, W, P, s, G, olayout,
                                             dtype, st));
    return e;
}

int check_window_args(int B, int c1, int c2, int H, int W, int K, int s, int dtype) {
    if (!dtype_ok(dtype)) return SAPA_ERR_INVALID_ARGUMENT;
    if (B < 0 || c1 <= 0 || c2 <= 0 || H <= 0 || W <= 0 || s < 1 || K < 1 || (K - 1) % 2 != 0)
        return SAPA_ERR_INVALID_ARGUMENT;
    if (K > 255 || (long long)H * s >= (1 << 24) || (long long)W * s >= (1 << 24) ||
        (long long)H * s * W * s >= (1LL << 31))
        return SAPA_ERR_TOO_LARGE;
    const long long hi = (long long)B * H * s * W * s;
    const int cmax = c1 > c2 ? c1 : c2;
    if (hi * cmax >= kMaxElems || hi * K * K >= kMaxElems) return SAPA_ERR_TOO_LARGE;
    return SAPA_OK;
}

int check_deform_args(int B, int Cq, int C, int H, int W, int P, int s, int G, int dtype) {
    if (!dtype_ok(dtype)) return SAPA_ERR_INVALID_ARGUMENT;
    if (B < 0 || Cq <= 0 || C <= 0 || H <= 0 || W <= 0 || s < 1 || P < 1 || G < 1 ||
        Cq % G != 0 || C % G != 0)
        return SAPA_ERR_INVALID_ARGUMENT;
    if ((long long)H * s >= (1 << 24) || (long long)W * s >= (1 << 24) ||
        (long long)H * s * W * s >= (1LL << 31))
        return SAPA_ERR_TOO_LARGE;
    const long long hi = (long long)B * H * s * W * s;
    const int cmax = Cq > C ? Cq : C;
    if (hi * cmax >= kMaxElems || hi * 2 * G * P >= kMaxElems) return SAPA_ERR_TOO_LARGE;
    return SAPA_OK;
}

}  // namespace

extern "C" {

int sapa_hip_abi_version(void) { return 1; }

const char *sapa_hip_status_string(int status) {
    switch (status) {
        case SAPA_OK: return "ok";
        case SAPA_ERR_INVALID_ARGUMENT: return "invalid argument";
        case SAPA_ERR_UNSUPPORTED: return "unsupported configuration";
        case SAPA_ERR_TOO_LARGE: return "tensor too large for the kernels' index range";
        case SAPA_ERR_LAUNCH: return "HIP launch error";
        default: return "unknown status";
    }
}

const char *sapa_hip_last_hip_error(void) { return g_hip_error; }

const char *sapa_hip_last_kernel(void) { return g_last_kernel; }

int sapa_qk_forward(const void *query, const void *key, void *out, int B, int d, int H, int W,
                    int K, int s, int dtype, void *stream) {
    const int rc = check_window_args(B, d, d, H, W, K, s, dtype);
    if (rc != SAPA_OK) return rc;
    if (B == 0) return SAPA_OK;
    if (!query || !key || !out) return SAPA_ERR_INVALID_ARGUMENT;
    hipStream_t st = (hipStream_t)stream;
    hipError_t e = tiled_launch(TILED_QK, query, key, nullptr, nullptr, out, B, d, 0, H, W,
                                       K, s, dtype, st);
    if (e == hipErrorNotSupported)
        e = took("qk_forward_generic_kernel",
                 qk_forward_generic_launch(query, key, out, B, d, H, W, K, s, dtype, st));
    return finish(e);
}

int sapa_av_forward(const void *attn, const void *value, void *out, int B, int C, int H, int W,
                    int K, int s, int dtype, void *stream) {
    const int rc = check_window_args(B, C, C, H, W, K, s, dtype);
    if (rc != SAPA_OK) return rc;
    if (B == 0) return SAPA_OK;
    if (!attn || !value || !out) return SAPA_ERR_INVALID_ARGUMENT;
    hipStream_t st = (hipStream_t)stream;
    hipError_t e = tiled_launch(TILED_AV, nullptr, nullptr, attn, value, out, B, 0, C, H, W,
                                       K, s, dtype, st);
    if (e == hipErrorNotSupported)
        e = took("av_forward_generic_kernel",
                 av_forward_generic_launch(attn, value, out, B, C, H, W, K, s, dtype, st));
    return finish(e);
}

int sapa_qk_backward(const void *grad_out, const void *query, const void *key, void *grad_query,
                     void *grad_key, int B, int d, int H, int W, int K, int s, int dtype,
                     void *stream) {
    const int rc = check_window_args(B, d, d, H, W, K, s, dtype);
    if (rc != SAPA_OK) return rc;
    if (B == 0) return SAPA_OK;
    if (!grad_out || !query || !key) return SAPA_ERR_INVALID_ARGUMENT;
    hipStream_t st = (hipStream_t)stream;
    // grad_query[n,c,ph,pw] = sum_k key[n,c,nbr_k] * grad_out[n,k,ph,pw]: the
    // aggregation with key in the value's place.
    if (grad_query) {
        const int r2 = sapa_av_forward(grad_out, key, grad_query, B, d, H, W, K, s, dtype, stream);
        if (r2 != SAPA_OK) return r2;
    }
    if (grad_key) {
        const hipError_t e =
            lowres_grad_any(query, grad_out, grad_key, B, d, H, W, K, s, dtype, st);
        if (e != hipSuccess) return fail_hip(e);
    }
    return SAPA_OK;
}

int sapa_av_backward(const void *grad_out, const void *attn, const void *value, void *grad_attn,
                     void *grad_value, int B, int C, int H, int W, int K, int s, int dtype,
                     void *stream) {
    const int rc = check_window_args(B, C, C, H, W, K, s, dtype);
    if (rc != SAPA_OK) return rc;
    if (B == 0) return SAPA_OK;
    if (!grad_out || !attn || !value) return SAPA_ERR_INVALID_ARGUMENT;
    hipStream_t st = (hipStream_t)stream;
    // grad_attn[n,k,ph,pw] = sum_c value[n,c,nbr_k] * grad_out[n,c,ph,pw]: the
    // similarity with grad_out as the query and value as the key.
    if (grad_attn) {
        const int r2 = sapa_qk_forward(grad_out, value, grad_attn, B, C, H, W, K, s, dtype, stream);
        if (r2 != SAPA_OK) return r2;
    }
    if (grad_value) {
        const hipError_t e =
            lowres_grad_any(grad_out, attn, grad_value, B, C, H, W, K, s, dtype, st);
        if (e != hipSuccess) return fail_hip(e);
    }
    return SAPA_OK;
}

int sapa_av_backward_logits(const void *grad_out, const void *attn, const void *value,
                            void *grad_logits, int B, int C, int H, int W, int K, int s, int dtype,
                            void *stream) {
    const int rc = check_window_args(B, C, C, H, W, K, s, dtype);
    if (rc != SAPA_OK) return rc;
    if (B == 0) return SAPA_OK;
    if (!grad_out || !attn || !value || !grad_logits) return SAPA_ERR_INVALID_ARGUMENT;
    // only the register-tiled kernel has this epilogue
    const hipError_t e =
        sapa_b_tiled_launch(TILED_QK_SOFTMAX_BWD, grad_out, value, attn, nullptr, grad_logits, B, C,
                            0, H, W, K, s, dtype, (hipStream_t)stream);
    if (e == hipErrorNotSupported) return SAPA_ERR_UNSUPPORTED;
    return finish(e);
}

long long sapa_fused_backward_workspace(int B, int H, int W, int K, int s) {
    if (B < 0 || H <= 0 || W <= 0 || K < 1 || s < 1) return 0;
    return 2LL * B * K * K * H * s * W * s * (long long)sizeof(float);
}

// The chain behind sapa_fused_backward / sapa_fused_backward_attn: `attn_given` = the
// fp32 weights kept by sapa_fused_forward_attn, or NULL to recompute them into the
// first half of the workspace.
static int fused_backward_impl(const void *grad_out, const void *query, const void *key, const void *value,
                               const float *attn_given, void *workspace, void *grad_query, void *grad_key,
                               void *grad_value, int B, int d, int C, int H, int W, int K, int s, int dtype,
                               void *stream) {
    const int rc = check_window_args(B, d, C, H, W, K, s, dtype);
    if (rc != SAPA_OK) return rc;
    if (dtype == SAPA_F64 || K != 5 || s != 2) return SAPA_ERR_UNSUPPORTED;
    if (B == 0) return SAPA_OK;
    if (!grad_out || !query || !key || !value || !workspace) return SAPA_ERR_INVALID_ARGUMENT;
    hipStream_t st = (hipStream_t)stream;
    float *grad_logits = (float *)workspace + (attn_given ? 0LL : (long long)B * K * K * H * s * W * s);
    const float *attn = attn_given ? attn_given : (const float *)workspace;
    // every stage on the LDS-tiled kernels with fp32 K*K tensors; a stage they do
    // not cover ends the call before anything the caller keeps has been written
    // by a later stage (the caller recomputes everything on its own path)
#define SAPA_STAGE(call)                                                       \
    do {                                                                       \
        const hipError_t e_ = (call);                                          \
        if (e_ == hipErrorNotSupported) return SAPA_ERR_UNSUPPORTED;           \
        if (e_ != hipSuccess) return fail_hip(e_);                             \
    } while (0)
    // the similarity stages: the dot-product kernel where it applies (16-bit
    // tensors), else the fp32-arithmetic one
    auto similarity = [&](int mode, const void *qq, const void *kk, const void *attn_in, void *res, int ch) {
        hipError_t e = sapa_b_dot2_launch(mode, qq, kk, attn_in, nullptr, res, B, ch, 0, H, W, K, s, dtype, st,
                                          true);
        if (e == hipErrorNotSupported)
            e = sapa_b_tiled_launch(mode, qq, kk, attn_in, nullptr, res, B, ch, 0, H, W, K, s, dtype, st, true);
        return e;
    };
    if (!attn_given) SAPA_STAGE(similarity(TILED_QK_SOFTMAX, query, key, nullptr, workspace, d));
    if (grad_value)
        SAPA_STAGE(lowres_grad_tiled_launch(grad_out, attn, grad_value, B, C, H, W, K, s, dtype, st, true));
    if (grad_query || grad_key) {
        SAPA_STAGE(similarity(TILED_QK_SOFTMAX_BWD, grad_out, value, attn, grad_logits, C));
        if (grad_query)
            SAPA_STAGE(sapa_b_tiled_launch(TILED_AV, nullptr, nullptr, grad_logits, key, grad_query, B, 0,
                                           d, H, W, K, s, dtype, st, true));
        if (grad_key)
            SAPA_STAGE(lowres_grad_tiled_launch(query, grad_logits, grad_key, B, d, H, W, K, s, dtype, st,
                                                true));
    }
    return SAPA_OK;
}

int sapa_fused_backward(const void *grad_out, const void *query, const void *key, const void *value,
                        void *workspace, void *grad_query, void *grad_key, void *grad_value, int B,
                        int d, int C, int H, int W, int K, int s, int dtype, void *stream) {
    return fused_backward_impl(grad_out, query, key, value, nullptr, workspace, grad_query, grad_key,
                               grad_value, B, d, C, H, W, K, s, dtype, stream);
}

int sapa_fused_forward_attn(const void *query, const void *key, const void *value, void *attn,
                            void *out, int B, int d, int C, int H, int W, int K, int s, int dtype,
                            void *stream) {
    const int rc = check_window_args(B, d, C, H, W, K, s, dtype);
    if (rc != SAPA_OK) return rc;
    if (dtype == SAPA_F64 || K != 5 || s != 2) return SAPA_ERR_UNSUPPORTED;
    if (B == 0) return SAPA_OK;
    if (!query || !key || !value || !attn || !out) return SAPA_ERR_INVALID_ARGUMENT;
    hipStream_t st = (hipStream_t)stream;
    // the weights once, in fp32, then the aggregation with them: the two launches of
    // the separate operators, without a 16-bit rounding between them
    hipError_t e = sapa_b_dot2_launch(TILED_QK_SOFTMAX, query, key, nullptr, nullptr, attn, B, d, 0, H, W, K, s,
                                      dtype, st, true);
    if (e == hipErrorNotSupported)
        e = sapa_b_tiled_launch(TILED_QK_SOFTMAX, query, key, nullptr, nullptr, attn, B, d, 0, H, W, K, s, dtype,
                                st, true);
    SAPA_STAGE(e);
    // the output of 16-bit tensors from the one-launch forward where it runs on the matrix
    // instructions (its weights are the same fp32 softmax of the same fp32 sums): 208 us against
    // 285 for the aggregation with the fp32 weights at B=16, C=256, 100x168
    e = hipErrorNotSupported;
#ifndef SAPA_WMAT16_OFF
    e = sapa_b_wmat16_launch(TILED_FUSED, query, key, value, out, B, d, C, H, W, K, s, dtype, st);
#endif
    if (e == hipErrorNotSupported)
        e = sapa_b_tiled_launch(TILED_AV, nullptr, nullptr, attn, value, out, B, 0, C, H, W, K, s, dtype, st, true);
    SAPA_STAGE(e);
    return SAPA_OK;
}

long long sapa_fused_backward_attn_workspace(int B, int H, int W, int K, int s) {
    return sapa_fused_backward_workspace(B, H, W, K, s) / 2;
}

int sapa_fused_backward_attn(const void *grad_out, const void *query, const void *key, const void *value,
                             const void *attn, void *workspace, void *grad_query, void *grad_key,
                             void *grad_value, int B, int d, int C, int H, int W, int K, int s, int dtype,
                             void *stream) {
    if (!attn) return SAPA_ERR_INVALID_ARGUMENT;
    return fused_backward_impl(grad_out, query, key, value, (const float *)attn, workspace, grad_query,
                               grad_key, grad_value, B, d, C, H, W, K, s, dtype, stream);
}
#undef SAPA_STAGE

int sapa_softmax_forward(const void *x, void *y, long long N, int R, long long M, int dtype,
                         void *stream) {
    if (!dtype_ok(dtype) || N < 0 || R < 1 || M < 0) return SAPA_ERR_INVALID_ARGUMENT;
    if (N == 0 || M == 0) return SAPA_OK;
    if (!x || !y) return SAPA_ERR_INVALID_ARGUMENT;
    if (N * M >= kMaxElems / R) return SAPA_ERR_TOO_LARGE;
    return finish(softmax_generic_launch(x, y, (long)N, R, (long)M, dtype, (hipStream_t)stream));
}

static int fused_common(int attn_only, const void *query, const void *key, const void *value,
                        void *out, int B, int d, int C, int H, int W, int K, int s, int dtype,
                        void *stream) {
    const int rc = check_window_args(B, d, C, H, W, K, s, dtype);
    if (rc != SAPA_OK) return rc;
    if (K * K > 121) return SAPA_ERR_UNSUPPORTED;
    if (B == 0) return SAPA_OK;
    if (!query || !key || !out || (!attn_only && !value)) return SAPA_ERR_INVALID_ARGUMENT;
    hipStream_t st = (hipStream_t)stream;
    hipError_t e = tiled_launch(attn_only ? TILED_QK_SOFTMAX : TILED_FUSED, query, key,
                                       nullptr, value, out, B, d, attn_only ? 0 : C, H, W, K, s,
                                       dtype, st);
    if (e == hipErrorNotSupported)
        e = took("fused_pixel_kernel",
                 fused_pixel_launch(query, key, value, out, B, d, C, H, W, K, s, attn_only, dtype, st));
    if (e == hipErrorNotSupported) return SAPA_ERR_UNSUPPORTED;
    return finish(e);
}

int sapa_fused_forward(const void *query, const void *key, const void *value, void *out, int B,
                       int d, int C, int H, int W, int K, int s, int dtype, void *stream) {
    return fused_common(0, query, key, value, out, B, d, C, H, W, K, s, dtype, stream);
}

int sapa_qk_softmax_forward(const void *query, const void *key, void *attn, int B, int d, int H,
                            int W, int K, int s, int dtype, void *stream) {
    return fused_common(1, query, key, nullptr, attn, B, d, d, H, W, K, s, dtype, stream);
}

// Channels-last memory order: only the kernel of sapa_b_nhwc.hip serves it.
static int nhwc_common(int mode, const void *query, const void *key, const void *attn,
                       const void *value, void *out, int B, int d, int C, int H, int W, int K,
                       int s, int dtype, void *stream, const void *q_bias = nullptr) {
    const int rc = check_window_args(B, d, C, H, W, K, s, dtype);
    if (rc != SAPA_OK) return rc;
    if (B == 0) return SAPA_OK;
    const bool need_qk = mode != TILED_AV, need_av = mode == TILED_AV || mode == TILED_FUSED;
    if (!out || (need_qk && (!query || !key)) || (need_av && !value) || (mode == TILED_AV && !attn))
        return SAPA_ERR_INVALID_ARGUMENT;
    // 16-bit tensors: the kernel on the 16-bit matrix instructions first
    // (SAPA_NHWC16_OFF: a tuning build without it, for comparisons)
    hipError_t e = hipErrorNotSupported;
#ifndef SAPA_NHWC_WM16_OFF
    // the fused forward: dense window products (sapa_b_nhwc_wm16.hip;
    // SAPA_NHWC_WM16_OFF: a tuning build without it, for comparisons)
    e = took("sapa_b_nhwc_wm16_kernel", sapa_b_nhwc_wm16_launch(mode, query, key, value, q_bias, out, B, d, C, H, W,
                                                                K, s, dtype, (hipStream_t)stream));
#endif
#ifndef SAPA_NHWC16_OFF
    if (e == hipErrorNotSupported)
        e = took("sapa_b_nhwc16_kernel",
                        sapa_b_nhwc16_launch(mode, query, key, attn, value, q_bias, out, B, d, C, H, W, K, s,
                                             dtype, (hipStream_t)stream));
#endif
    if (e == hipErrorNotSupported)
        e = took(sapa_b_nhwc_kernel_name(K, s, dtype), sapa_b_nhwc_launch(mode, query, key, attn, value, q_bias, out, B, d, C,
                                                          H, W, K, s, dtype, (hipStream_t)stream));
    if (e == hipErrorNotSupported) return SAPA_ERR_UNSUPPORTED;
    return finish(e);
}

int sapa_qk_forward_nhwc(const void *query, const void *key, void *out, int B, int d, int H, int W,
                         int K, int s, int dtype, void *stream) {
    return nhwc_common(TILED_QK, query, key, nullptr, nullptr, out, B, d, d, H, W, K, s, dtype, stream);
}

int sapa_qk_softmax_forward_nhwc(const void *query, const void *key, void *attn, int B, int d,
                                 int H, int W, int K, int s, int dtype, void *stream) {
    return nhwc_common(TILED_QK_SOFTMAX, query, key, nullptr, nullptr, attn, B, d, d, H, W, K, s,
                       dtype, stream);
}

int sapa_av_forward_nhwc(const void *attn, const void *value, void *out, int B, int C, int H,
                         int W, int K, int s, int dtype, void *stream) {
    return nhwc_common(TILED_AV, nullptr, nullptr, attn, value, out, B, C, C, H, W, K, s, dtype, stream);
}

int sapa_fused_forward_nhwc(const void *query, const void *key, const void *value, void *out,
                            int B, int d, int C, int H, int W, int K, int s, int dtype,
                            void *stream) {
    return nhwc_common(TILED_FUSED, query, key, nullptr, value, out, B, d, C, H, W, K, s, dtype, stream);
}

int sapa_fused_forward_nhwc_qbias(const void *query, const void *key, const void *value,
                                  const void *q_bias, void *out, int B, int d, int C, int H, int W,
                                  int K, int s, int dtype, void *stream) {
    return nhwc_common(TILED_FUSED, query, key, nullptr, value, out, B, d, C, H, W, K, s, dtype, stream,
                       q_bias);
}

int sapa_deform_qk_forward_from(const void *query, const void *key, const void *offset,
                                void *out, int B, int Cq, int H, int W, int P, int s, int G,
                                int offset_layout, int dtype, void *stream) {
    const int rc = check_deform_args(B, Cq, Cq, H, W, P, s, G, dtype);
    if (rc != SAPA_OK) return rc;
    if (offset_layout < 0 || offset_layout > 2) return SAPA_ERR_INVALID_ARGUMENT;
    if (B == 0) return SAPA_OK;
    if (!query || !key || !offset || !out) return SAPA_ERR_INVALID_ARGUMENT;
    return finish(deform_qk_any(query, key, offset, out, B, Cq, H, W, P, s, G, offset_layout,
                                dtype, (hipStream_t)stream));
}

int sapa_deform_qk_forward(const void *query, const void *key, const void *offset, void *out,
                           int B, int Cq, int H, int W, int P, int s, int G, int dtype,
                           void *stream) {
    return sapa_deform_qk_forward_from(query, key, offset, out, B, Cq, H, W, P, s, G,
                                       SAPA_OFFSET_HIRES, dtype, stream);
}

int sapa_deform_av_forward_from(const void *attn, const void *value, const void *offset,
                                void *out, int B, int C, int H, int W, int P, int s, int G,
                                int offset_layout, int dtype, void *stream) {
    const int rc = check_deform_args(B, C, C, H, W, P, s, G, dtype);
    if (rc != SAPA_OK) return rc;
    if (offset_layout < 0 || offset_layout > 2) return SAPA_ERR_INVALID_ARGUMENT;
    if (B == 0) return SAPA_OK;
    if (!attn || !value || !offset || !out) return SAPA_ERR_INVALID_ARGUMENT;
    return finish(deform_av_any(attn, value, offset, out, B, C, H, W, P, s, G, offset_layout,
                                dtype, (hipStream_t)stream));
}

int sapa_deform_av_forward(const void *attn, const void *value, const void *offset, void *out,
                           int B, int C, int H, int W, int P, int s, int G, int dtype,
                           void *stream) {
    return sapa_deform_av_forward_from(attn, value, offset, out, B, C, H, W, P, s, G,
                                       SAPA_OFFSET_HIRES, dtype, stream);
}

int sapa_deform_fused_forward_from(const void *query, const void *key, const void *value,
                                   const void *offset, void *out, int B, int Cq, int C, int H,
                                   int W, int P, int s, int G, int offset_layout, int dtype,
                                   void *stream) {
    const int rc = check_deform_args(B, Cq, C, H, W, P, s, G, dtype);
    if (rc != SAPA_OK) return rc;
    if (offset_layout < 0 || offset_layout > 2) return SAPA_ERR_INVALID_ARGUMENT;
    if (P > 64) return SAPA_ERR_UNSUPPORTED;
    if (B == 0) return SAPA_OK;
    if (!query || !key || !value || !offset || !out) return SAPA_ERR_INVALID_ARGUMENT;
    return finish(deform_fused_any(query, key, value, offset, out, B, Cq, C, H, W, P, s, G,
                                   offset_layout, dtype, (hipStream_t)stream));
}

int sapa_deform_fused_forward(const void *query, const void *key, const void *value,
                              const void *offset, void *out, int B, int Cq, int C, int H, int W,
                              int P, int s, int G, int dtype, void *stream) {
    return sapa_deform_fused_forward_from(query, key, value, offset, out, B, Cq, C, H, W, P, s, G,
                                          SAPA_OFFSET_HIRES, dtype, stream);
}

int sapa_deform_fused_forward_nhwc(const void *query, const void *key, const void *value,
                                   const void *offset, void *out, int B, int Cq, int C, int H,
                                   int W, int P, int s, int G, int dtype, void *stream) {
    const int rc = check_deform_args(B, Cq, C, H, W, P, s, G, dtype);
    if (rc != SAPA_OK) return rc;
    if (B == 0) return SAPA_OK;
    if (!query || !key || !value || !offset || !out) return SAPA_ERR_INVALID_ARGUMENT;
    const char *name = "";
    const hipError_t e0 = deform_fused_nhwc_launch(query, key, value, offset, out, B, Cq, C, H, W, P,
                                                   s, G, dtype, (hipStream_t)stream, &name);
    const hipError_t e = took(name, e0);
    if (e == hipErrorNotSupported) return SAPA_ERR_UNSUPPORTED;
    return finish(e);
}

long long sapa_deform_fused_forward_workspace(int B, int Cq, int C, int H, int W, int P, int s,
                                              int G, int dtype) {
    if (check_deform_args(B, Cq, C, H, W, P, s, G, dtype) != SAPA_OK) return 0;
    return deform_fused_nchw_workspace(B, Cq, C, H, W, P, s, G, dtype);
}

int sapa_deform_fused_forward_ws(const void *query, const void *key, const void *value,
                                 const void *offset, void *out, void *workspace, int B, int Cq,
                                 int C, int H, int W, int P, int s, int G, int offset_layout,
                                 int dtype, void *stream) {
    const int rc = check_deform_args(B, Cq, C, H, W, P, s, G, dtype);
    if (rc != SAPA_OK) return rc;
    if (offset_layout < SAPA_OFFSET_HIRES || offset_layout > SAPA_OFFSET_NEAREST)
        return SAPA_ERR_INVALID_ARGUMENT;
    if (B == 0) return SAPA_OK;
    if (!query || !key || !value || !offset || !out) return SAPA_ERR_INVALID_ARGUMENT;
    const char *name = "";
    const hipError_t e0 = deform_fused_nchw_ws_launch(query, key, value, offset, out, workspace, B, Cq, C,
                                                      H, W, P, s, G, offset_layout, dtype,
                                                      (hipStream_t)stream, &name);
    const hipError_t e = took(name, e0);
    if (e == hipErrorNotSupported) return SAPA_ERR_UNSUPPORTED;
    return finish(e);
}

int sapa_deform_qk_backward(const void *grad_out, const void *query, const void *key,
                            const void *offset, void *grad_query, void *grad_key,
                            void *grad_offset, int B, int Cq, int H, int W, int P, int s, int G,
                            int dtype, void *stream) {
    const int rc = check_deform_args(B, Cq, Cq, H, W, P, s, G, dtype);
    if (rc != SAPA_OK) return rc;
    if (dtype != SAPA_F32 && dtype != SAPA_F64) return SAPA_ERR_UNSUPPORTED;
    if (B == 0) return SAPA_OK;
    if (!grad_out || !query || !key || !offset) return SAPA_ERR_INVALID_ARGUMENT;
    hipStream_t st = (hipStream_t)stream;
    // grad_query[b,g*d+c] = sum_p grad_out[b,g,p] * bilinear(key[b,g*d+c]): the
    // sampled aggregation with key in the value's place.
    if (grad_query) {
        const hipError_t e =
            deform_av_any(grad_out, key, offset, grad_query, B, Cq, H, W, P, s, G, SAPA_OFFSET_HIRES,
                          dtype, st);
        if (e != hipSuccess) return fail_hip(e);
    }
    if (grad_key || grad_offset) {
        const hipError_t e = deform_lowgrad_any(query, grad_out, key, offset, grad_key,
                                                   grad_offset, B, Cq, H, W, P, s, G, dtype, st);
        if (e != hipSuccess) return fail_hip(e);
    }
    return SAPA_OK;
}

int sapa_deform_av_backward(const void *grad_out, const void *attn, const void *value,
                            const void *offset, void *grad_attn, void *grad_value,
                            void *grad_offset, int B, int C, int H, int W, int P, int s, int G,
                            int dtype, void *stream) {
    const int rc = check_deform_args(B, C, C, H, W, P, s, G, dtype);
    if (rc != SAPA_OK) return rc;
    if (dtype != SAPA_F32 && dtype != SAPA_F64) return SAPA_ERR_UNSUPPORTED;
    if (B == 0) return SAPA_OK;
    if (!grad_out || !attn || !value || !offset) return SAPA_ERR_INVALID_ARGUMENT;
    hipStream_t st = (hipStream_t)stream;
    // grad_attn[b,g,p] = sum_{c in g} grad_out[b,c] * bilinear(value[b,c]): the
    // sampled similarity with grad_out as the query and value as the key.
    if (grad_attn) {
        const hipError_t e =
            deform_qk_any(grad_out, value, offset, grad_attn, B, C, H, W, P, s, G, SAPA_OFFSET_HIRES,
                          dtype, st);
        if (e != hipSuccess) return fail_hip(e);
    }
    if (grad_value || grad_offset) {
        const hipError_t e = deform_lowgrad_any(grad_out, attn, value, offset, grad_value,
                                                   grad_offset, B, C, H, W, P, s, G, dtype, st);
        if (e != hipSuccess) return fail_hip(e);
    }
    return SAPA_OK;
}

long long sapa_deform_backward_workspace(int B, int Cx, int H, int W, int P, int s, int G, int dtype) {
    if (check_deform_args(B, Cx, Cx, H, W, P, s, G, dtype) != SAPA_OK) return 0;
    return deform_separate_backward_workspace(B, Cx, H, W, P, s, G, dtype);
}

int sapa_deform_qk_backward_ws(const void *grad_out, const void *query, const void *key,
                               const void *offset, void *workspace, void *grad_query, void *grad_key,
                               void *grad_offset, int B, int Cq, int H, int W, int P, int s, int G,
                               int dtype, void *stream) {
    const int rc = check_deform_args(B, Cq, Cq, H, W, P, s, G, dtype);
    if (rc != SAPA_OK) return rc;
    if (B == 0) return SAPA_OK;
    if (!grad_out || !query || !key || !offset) return SAPA_ERR_INVALID_ARGUMENT;
    const hipError_t e = deform_separate_backward_launch(0, query, key, grad_out, offset, workspace, grad_query,
                                                         grad_key, grad_offset, B, Cq, H, W, P, s, G, dtype,
                                                         (hipStream_t)stream);
    if (e == hipErrorNotSupported) return SAPA_ERR_UNSUPPORTED;
    return finish(e);
}

int sapa_deform_av_backward_ws(const void *grad_out, const void *attn, const void *value,
                               const void *offset, void *workspace, void *grad_attn, void *grad_value,
                               void *grad_offset, int B, int C, int H, int W, int P, int s, int G,
                               int dtype, void *stream) {
    const int rc = check_deform_args(B, C, C, H, W, P, s, G, dtype);
    if (rc != SAPA_OK) return rc;
    if (B == 0) return SAPA_OK;
    if (!grad_out || !attn || !value || !offset) return SAPA_ERR_INVALID_ARGUMENT;
    const hipError_t e = deform_separate_backward_launch(1, grad_out, value, attn, offset, workspace, grad_attn,
                                                         grad_value, grad_offset, B, C, H, W, P, s, G, dtype,
                                                         (hipStream_t)stream);
    if (e == hipErrorNotSupported) return SAPA_ERR_UNSUPPORTED;
    return finish(e);
}

long long sapa_deform_fused_backward_workspace(int B, int Cq, int C, int H, int W, int P, int s,
                                               int G, int dtype) {
    if (check_deform_args(B, Cq, C, H, W, P, s, G, dtype) != SAPA_OK) return 0;
    return deform_fused_backward_workspace(B, Cq, C, H, W, P, s, G, dtype);
}

int sapa_deform_fused_backward(const void *grad_out, const void *query, const void *key,
                               const void *value, const void *offset, void *workspace,
                               void *grad_query, void *grad_key, void *grad_value,
                               void *grad_offset, int B, int Cq, int C, int H, int W, int P, int s,
                               int G, int dtype, void *stream) {
    const int rc = check_deform_args(B, Cq, C, H, W, P, s, G, dtype);
    if (rc != SAPA_OK) return rc;
    if (B == 0) return SAPA_OK;
    if (!grad_out || !query || !key || !value || !offset) return SAPA_ERR_INVALID_ARGUMENT;
    const hipError_t e = deform_fused_backward_launch(grad_out, query, key, value, offset, workspace,
                                                      grad_query, grad_key, grad_value, grad_offset, B, Cq,
                                                      C, H, W, P, s, G, dtype, (hipStream_t)stream);
    if (e == hipErrorNotSupported) return SAPA_ERR_UNSUPPORTED;
    return finish(e);
}

long long sapa_channel_moments_workspace(int B, int C, long long HW, int channels_last) {
    if (B <= 0 || C <= 0 || HW <= 0) return 0;
    return channel_moments_workspace(B, C, (long)HW, channels_last != 0);
}

int sapa_channel_moments(const void *x, void *workspace, float *mean_var, int B, int C,
                         long long HW, int channels_last, int dtype, void *stream) {
    if (!dtype_ok(dtype) || B < 0 || C <= 0 || HW <= 0) return SAPA_ERR_INVALID_ARGUMENT;
    if (dtype == SAPA_F64) return SAPA_ERR_UNSUPPORTED;
    if ((long long)B * C * HW >= kMaxElems) return SAPA_ERR_TOO_LARGE;
    if (B == 0) return SAPA_OK;
    if (!x || !workspace || !mean_var) return SAPA_ERR_INVALID_ARGUMENT;
    const hipError_t e = channel_moments_launch(x, workspace, mean_var, B, C, (long)HW,
                                                channels_last != 0, dtype, (hipStream_t)stream);
    if (e == hipErrorNotSupported) return SAPA_ERR_UNSUPPORTED;
    return finish(e);
}

long long sapa_channel_moments_static_capacity(void) { return channel_moments_static_capacity(); }

int sapa_channel_moments_static(const void *x, float *mean_var, int B, int C, long long HW,
                                int channels_last, int dtype, void *stream) {
    if (!dtype_ok(dtype) || B < 0 || C <= 0 || HW <= 0) return SAPA_ERR_INVALID_ARGUMENT;
    if (dtype == SAPA_F64) return SAPA_ERR_UNSUPPORTED;
    if ((long long)B * C * HW >= kMaxElems) return SAPA_ERR_TOO_LARGE;
    if (B == 0) return SAPA_OK;
    if (!x || !mean_var) return SAPA_ERR_INVALID_ARGUMENT;
    // partial sums beyond the library's fixed array: the workspace form serves those extents
    if (channel_moments_workspace(B, C, (long)HW, channels_last != 0) > channel_moments_static_capacity())
        return SAPA_ERR_TOO_LARGE;
    const hipError_t e = channel_moments_static_launch(x, mean_var, B, C, (long)HW, channels_last != 0,
                                                       dtype, (hipStream_t)stream);
    if (e == hipErrorNotSupported) return SAPA_ERR_UNSUPPORTED;
    return finish(e);
}

int sapa_groupnorm_fold(const float *mean_var, const void *gamma, const void *beta, const void *weight,
                        const void *bias, void *weight_out, void *bias_out, int B, int C, int O,
                        int groups, float eps, int dtype, void *stream) {
    if (!dtype_ok(dtype) || B < 0 || C <= 0 || O <= 0 || groups < 1 || C % groups != 0 || !(eps >= 0.f))
        return SAPA_ERR_INVALID_ARGUMENT;
    if (dtype == SAPA_F64) return SAPA_ERR_UNSUPPORTED;
    if (B == 0) return SAPA_OK;
    if (!mean_var || !weight || !weight_out || !bias_out) return SAPA_ERR_INVALID_ARGUMENT;
    const hipError_t e = groupnorm_fold_launch(mean_var, gamma, beta, weight, bias, weight_out, bias_out,
                                               B, C, O, groups, eps, dtype, (hipStream_t)stream);
    if (e == hipErrorNotSupported) return SAPA_ERR_UNSUPPORTED;
    return finish(e);
}

int sapa_project_nhwc(const void *x, const void *weight, const void *bias, void *out, int B, int C,
                      int O, long long HW, int dtype, void *stream) {
    if (!dtype_ok(dtype) || B < 0 || C <= 0 || O <= 0 || HW <= 0) return SAPA_ERR_INVALID_ARGUMENT;
    if ((long long)B * HW * (C > O ? C : O) >= kMaxElems) return SAPA_ERR_TOO_LARGE;
    if (B == 0) return SAPA_OK;
    if (!x || !weight || !out) return SAPA_ERR_INVALID_ARGUMENT;
    const hipError_t e = project_nhwc_launch(x, weight, bias, out, B, C, O, (long)HW, dtype,
                                             (hipStream_t)stream);
    if (e == hipErrorNotSupported) return SAPA_ERR_UNSUPPORTED;
    return finish(e);
}

int sapa_project_nchw(const void *x, const void *weight, const void *bias, void *out, int B, int C,
                      int O, long long HW, int out_channels_last, int dtype, void *stream) {
    if (!dtype_ok(dtype) || B < 0 || C <= 0 || O <= 0 || HW <= 0) return SAPA_ERR_INVALID_ARGUMENT;
    if ((long long)B * HW * (C > O ? C : O) >= kMaxElems) return SAPA_ERR_TOO_LARGE;
    if (B == 0) return SAPA_OK;
    if (!x || !weight || !out) return SAPA_ERR_INVALID_ARGUMENT;
    const hipError_t e = project_nchw_launch(x, weight, bias, out, B, C, O, (long)HW, out_channels_last,
                                             dtype, (hipStream_t)stream);
    if (e == hipErrorNotSupported) return SAPA_ERR_UNSUPPORTED;
    return finish(e);
}

namespace {
long long round256(long long n) { return (n + 255) / 256 * 256; }
long long esize_of(int dtype) { return dtype == SAPA_F32 ? 4 : dtype == SAPA_F64 ? 8 : 2; }
}  // namespace

long long sapa_norm_project_scratch(int B, int C, int O, long long HW, int x_channels_last, int dtype) {
    if (B <= 0 || C <= 0 || O <= 0 || HW <= 0 || !dtype_ok(dtype)) return 0;
    return round256(channel_moments_workspace(B, C, (long)HW, x_channels_last != 0)) + round256((long long)B * C * 8) +
           round256((long long)B * O * C * esize_of(dtype)) + round256((long long)B * O * esize_of(dtype));
}

int sapa_norm_project(const void *x, const void *gamma, const void *beta, const void *weight, const void *bias,
                      void *scratch, void *out, void *bias_out, int B, int C, int O, long long HW, int groups,
                      float eps, int x_channels_last, int out_channels_last, int dtype, void *stream) {
    if (!dtype_ok(dtype) || B < 0 || C <= 0 || O <= 0 || HW <= 0 || groups <= 0) return SAPA_ERR_INVALID_ARGUMENT;
    if ((long long)B * HW * (C > O ? C : O) >= kMaxElems) return SAPA_ERR_TOO_LARGE;
    if (B == 0) return SAPA_OK;
    if (!x || !weight || !scratch || !out) return SAPA_ERR_INVALID_ARGUMENT;
    // nothing is launched unless every step has a kernel for the configuration
    if (dtype == SAPA_F64 || C % groups != 0 || C > 8192 ||
        !project_supported(C, O, (long)HW, x_channels_last != 0, out_channels_last != 0, dtype) ||
        ((uintptr_t)x | (uintptr_t)out | (uintptr_t)scratch) % 16 != 0)
        return SAPA_ERR_UNSUPPORTED;
    char *p = (char *)scratch;
    void *ws = p;
    p += round256(channel_moments_workspace(B, C, (long)HW, x_channels_last != 0));
    float *mean_var = (float *)p;
    p += round256((long long)B * C * 8);
    void *w_b = p;
    p += round256((long long)B * O * C * esize_of(dtype));
    void *b_b = bias_out ? bias_out : (void *)p;
    hipStream_t st = (hipStream_t)stream;
    hipError_t e = channel_moments_launch(x, ws, mean_var, B, C, (long)HW, x_channels_last != 0, dtype, st);
    if (e == hipSuccess)
        e = groupnorm_fold_launch(mean_var, gamma, beta, weight, bias, w_b, b_b, B, C, O, groups, eps, dtype, st);
    if (e == hipSuccess)
        e = x_channels_last ? project_nhwc_launch(x, w_b, bias_out ? nullptr : b_b, out, B, C, O, (long)HW, dtype, st)
                            : project_nchw_launch(x, w_b, bias_out ? nullptr : b_b, out, B, C, O, (long)HW,
                                                  out_channels_last, dtype, st);
    if (e == hipErrorNotSupported) return SAPA_ERR_UNSUPPORTED;
    return finish(e);
}

int sapa_layout_copy(const void *src, void *dst, int B, int C, long long HW, int to_channels_last,
                     int esize, void *stream) {
    if (B < 0 || C < 0 || HW < 0 || (esize != 2 && esize != 4)) return SAPA_ERR_INVALID_ARGUMENT;
    if ((long long)B * C * HW >= kMaxElems) return SAPA_ERR_TOO_LARGE;
    if (B == 0 || C == 0 || HW == 0) return SAPA_OK;
    if (!src || !dst || ((uintptr_t)src | (uintptr_t)dst) % (uintptr_t)esize != 0) return SAPA_ERR_INVALID_ARGUMENT;
    // [B, rows, cols] -> [B, cols, rows]: the way back is the same transposition with the
    // roles of C and HW exchanged
    if (!to_channels_last && HW > 0x7fffffffLL) return SAPA_ERR_UNSUPPORTED;
    const hipError_t e = to_channels_last
        ? nchw_to_nhwc_launch(src, dst, C, nullptr, nullptr, 0, B, (long)HW, esize, (hipStream_t)stream)
        : nchw_to_nhwc_launch(src, dst, (int)HW, nullptr, nullptr, 0, B, (long)C, esize, (hipStream_t)stream);
    if (e == hipErrorNotSupported) return SAPA_ERR_UNSUPPORTED;
    return finish(e);
}

int sapa_stream_mix(const void *src, void *dst, long long units, int reads, int writes, int reps,
                    int nontemporal, void *stream) {
    if (units < 0 || reads < 0 || writes < 0 || reps < 1 || (reads == 0 && writes == 0) || nontemporal < 0 || nontemporal > 7)
        return SAPA_ERR_INVALID_ARGUMENT;
    if (units > (1LL << 30)) return SAPA_ERR_TOO_LARGE;
    if (units == 0) return SAPA_OK;
    if ((reads > 0 && !src) || !dst) return SAPA_ERR_INVALID_ARGUMENT;
    if (((uintptr_t)src | (uintptr_t)dst) % 16 != 0) return SAPA_ERR_INVALID_ARGUMENT;
    // bit 2: readers and writers in different workgroups (`units` = groups of 9 + 16)
    const hipError_t e = (nontemporal & 4)
        ? (reads == 9 && writes == 16 ? stream_split_launch(src, dst, (long)units, reps, nontemporal & 3, (hipStream_t)stream)
                                      : hipErrorNotSupported)
        : stream_mix_launch(src, dst, (long)units, reads, writes, reps, nontemporal, (hipStream_t)stream);
    if (e == hipErrorNotSupported) return SAPA_ERR_UNSUPPORTED;
    return finish(e);
}

}  // extern "C"
