// Internal launch interface between the C ABI (capi.hip) and the kernel files.
// Every launcher enqueues on `st` and returns the HIP status of the launch;
// arguments are validated by the caller.  `dtype` is the sapa_dtype value.
#pragma once
#include "common.hpp"

namespace sapa {

// sapa_b_generic.hip: any K, s, dtype
hipError_t qk_forward_generic_launch(const void *q, const void *key, void *out, int B, int d,
                                     int H, int W, int K, int s, int dtype, hipStream_t st);
hipError_t av_forward_generic_launch(const void *attn, const void *value, void *out, int B, int C,
                                     int H, int W, int K, int s, int dtype, hipStream_t st);
hipError_t lowres_grad_generic_launch(const void *hi, const void *w, void *out, int B, int C,
                                      int H, int W, int K, int s, int dtype, hipStream_t st);
hipError_t softmax_generic_launch(const void *x, void *y, long N, int R, long M, int dtype,
                                  hipStream_t st);
// K in {1,3,5,7,9,11}; hipErrorNotSupported otherwise
hipError_t fused_pixel_launch(const void *q, const void *key, const void *value, void *out,
                              int B, int d, int C, int H, int W, int K, int s, int attn_only,
                              int dtype, hipStream_t st);

// sapa_b_tiled.hip: LDS-tiled kernels.  `mode` selects the stages:
// TILED_QK_SOFTMAX_BWD: the similarity g = qk(q, key) followed by the softmax
// backward against the weights in attn_in: out[k] = attn[k] * (g[k] - sum_k' g[k'] * attn[k']).
enum TiledMode { TILED_QK = 0, TILED_QK_SOFTMAX = 1, TILED_AV = 2, TILED_FUSED = 3,
                 TILED_QK_SOFTMAX_BWD = 4 };
// Returns hipErrorNotSupported when no tiled kernel covers (K, s, dtype, shape);
// the caller then takes the generic path.  wide: the K*K-channel tensors of the
// call (attn_in; the result of the modes without aggregation) are fp32 whatever
// dtype is (modes TILED_QK_SOFTMAX, TILED_AV, TILED_QK_SOFTMAX_BWD only).
hipError_t sapa_b_tiled_launch(int mode, const void *q, const void *key, const void *attn_in,
                               const void *value, void *out, int B, int d, int C, int H, int W,
                               int K, int s, int dtype, hipStream_t st, bool wide = false);

// sapa_b_nhwc.hip: the four forward modes for tensors in channels-last memory
// order ([B, H, W, channels]); f32 / f16 / bf16, (K, s) in {(3,2), (5,2), (7,2), (5,4), (7,4)}, channel
// counts multiples of 4.  hipErrorNotSupported otherwise.
hipError_t sapa_b_nhwc_launch(int mode, const void *q, const void *key, const void *attn_in,
                              const void *value, const void *qbias, void *out, int B, int d, int C,
                              int H, int W, int K, int s, int dtype, hipStream_t st);
// the kernel template sapa_b_nhwc_launch sends (K, s, dtype) to
const char *sapa_b_nhwc_kernel_name(int K, int s, int dtype);

// sapa_b_nhwc16.hip: the same four modes for f16 / bf16 channels-last tensors
// on the 16-bit matrix instructions (hipErrorNotSupported for anything else)
hipError_t sapa_b_nhwc16_launch(int mode, const void *q, const void *key, const void *attn_in,
                                const void *value, const void *qbias, void *out, int B, int d,
                                int C, int H, int W, int K, int s, int dtype, hipStream_t st);
// sapa_b_nhwc_wm16.hip: the fused forward of channels-last f16 / bf16 tensors (K = 5, s = 2, optional query
// bias) as dense window products on the 16-bit matrix instructions; hipErrorNotSupported otherwise.
hipError_t sapa_b_nhwc_wm16_launch(int mode, const void *q, const void *key, const void *value, const void *qbias,
                                   void *out, int B, int d, int C, int H, int W, int K, int s, int dtype,
                                   hipStream_t st);


// sapa_moments.hip: per (image, channel) mean and variance of a feature map
long channel_moments_workspace(int B, int C, long HW, bool channels_last);
hipError_t channel_moments_launch(const void *x, void *workspace, float *mean_var, int B, int C,
                                  long HW, bool channels_last, int dtype, hipStream_t st);
// the same with the partial sums in a fixed array inside the library (no workspace argument);
// hipErrorInvalidValue when they would not fit channel_moments_static_capacity() bytes
long channel_moments_static_capacity();
hipError_t channel_moments_static_launch(const void *x, float *mean_var, int B, int C, long HW,
                                         bool channels_last, int dtype, hipStream_t st);
hipError_t groupnorm_fold_launch(const float *mean_var, const void *gamma, const void *beta,
                                 const void *w, const void *bias, void *w_out, void *b_out, int B,
                                 int C, int O, int G, float eps, int dtype, hipStream_t st);

// sapa_stream.hip: a kernel that only moves bytes, `units` units that each read one
// contiguous run of reads * 4 KiB and write one of writes * 4 KiB, `reps` consecutive units per
// workgroup (calibration of measured rates); (reads, writes) in {(9,16), (8,8), (0,16), (16,0)},
// hipErrorNotSupported otherwise; nt: bit 0 = streaming loads, bit 1 = streaming stores
hipError_t stream_mix_launch(const void *src, void *dst, long units, int reads, int writes, int reps,
                             int nt, hipStream_t st);
// the 9 : 16 mix with readers and writers in different workgroups: `groups` groups of 9 reading
// and 16 writing workgroups, each with one contiguous run of reps * 64 KiB
hipError_t stream_split_launch(const void *src, void *dst, long groups, int reps, int nt, hipStream_t st);

// sapa_project.hip: 1x1 projection of a channels-last 16-bit feature with per-image weights
hipError_t project_nhwc_launch(const void *x, const void *w, const void *bias, void *out, int B,
                               int C, int O, long HW, int dtype, hipStream_t st);
// ... of a contiguous feature [B, C, HW] into [B, HW, O] (out_channels_last) or [B, O, HW]; fp32
hipError_t project_nchw_launch(const void *x, const void *w, const void *bias, void *out, int B,
                               int C, int O, long HW, int out_channels_last, int dtype, hipStream_t st);
// whether one of the two has a kernel for the configuration (pointer alignment aside)
bool project_supported(int C, int O, long HW, bool x_channels_last, bool out_channels_last, int dtype);

// sapa_d_nhwc.hip: fused SAPA-D forward for tensors in channels-last memory
// order (offsets [B, sH, sW, 2GP]); f32 / f16 / bf16, s in {1, 2, 4}, P <= 32,
// channels per group multiples of 4, at most 64 query / key channels per group.
// hipErrorNotSupported otherwise.
// *kernel (if given): the name of the kernel the call went to.
hipError_t deform_fused_nhwc_launch(const void *q, const void *key, const void *value,
                                    const void *offset, void *out, int B, int Cq, int C, int H,
                                    int W, int P, int s, int G, int dtype, hipStream_t st,
                                    const char **kernel = nullptr);

// sapa_d_scatter.hip: the same gradient (grad_key / grad_value of the sampled
// operators) as a matrix product per region; fp32 tensors, or (wide) f16 / bf16
// features with fp32 per-point scalars; s in {1, 2, 4}, P <= 32; grad_low fp32,
// accumulated into.  hipErrorNotSupported otherwise.
// channels_last_out: grad_low is a [B, H, W, Cx] fp32 buffer instead of the contiguous tensor.
bool deform_scatter_mat_serves(int B, int Cx, int H, int W, int P, int s, int G, int dtype);
hipError_t deform_scatter_mat_launch(const void *hi, const void *sc, const void *offset, void *grad_low,
                                     int B, int Cx, int H, int W, int P, int s, int G, int dtype,
                                     hipStream_t st, bool wide = false, bool channels_last_out = false);

// The per-pixel part of the fused SAPA-D backward in the matrix form of the
// forward kernel (sapa_d_bwdmat.hip): attention weights and gradient of the
// logits (fp32 [B, G, P, sH, sW], for the scatter kernels), grad_offset and
// grad_query (either may be NULL).  key_cl, value_cl: channels-last copies.
bool deform_bwd_wmat_serves(int B, int Cq, int C, int H, int W, int P, int s, int G, int dtype);
hipError_t deform_bwd_wmat_launch(const void *grad_out, const void *q, const void *key_cl,
                                  const void *value_cl, const void *offset, float *attn_ws,
                                  float *gl_ws, void *grad_q, void *grad_offset, int B, int Cq, int C,
                                  int H, int W, int P, int s, int G, int dtype, hipStream_t st);

// sapa_d_backward.hip: the backward pass of the fused SAPA-D operator in one call;
// attention weights and logit gradients as fp32 in `workspace` (256-byte aligned,
// deform_fused_backward_workspace() bytes; 0 = not served), f16 / bf16 tensors read
// and written as they are.  Any gradient may be NULL.  hipErrorNotSupported otherwise.
long deform_fused_backward_workspace(int B, int Cq, int C, int H, int W, int P, int s, int G, int dtype);
hipError_t deform_fused_backward_launch(const void *grad_out, const void *q, const void *key,
                                        const void *value, const void *offset, void *workspace,
                                        void *grad_q, void *grad_key, void *grad_value,
                                        void *grad_offset, int B, int Cq, int C, int H, int W, int P,
                                        int s, int G, int dtype, hipStream_t st);

// sapa_d_backward.hip: backward of deform_qk (which = 0: a = query, low = key, pp = grad_out,
// grad_a_or_pp = grad_query) or deform_av (which = 1: a = grad_out, low = value, pp = attn,
// grad_a_or_pp = grad_attn) on f16 / bf16 tensors as they are; `workspace` (256-byte aligned,
// deform_separate_backward_workspace() bytes; 0 = not served) holds fp32 intermediates.
long deform_separate_backward_workspace(int B, int Cx, int H, int W, int P, int s, int G, int dtype);
hipError_t deform_separate_backward_launch(int which, const void *a, const void *low, const void *pp,
                                           const void *offset, void *workspace, void *grad_a_or_pp,
                                           void *grad_low, void *grad_offset, int B, int Cx, int H, int W,
                                           int P, int s, int G, int dtype, hipStream_t st);

// sapa_d_nhwc.hip: contiguous (NCHW) tensors through the matrix-form kernels:
// key and value are copied into channels-last order in `workspace` (256-byte
// aligned, deform_fused_nchw_workspace() bytes; 0 = this path does not serve the
// case), q / offset / out are used in place; olayout: where the offsets are read
// from (deform_tap.hpp: OffsetLayout).  hipErrorNotSupported otherwise.
long deform_fused_nchw_workspace(int B, int Cq, int C, int H, int W, int P, int s, int G, int dtype);
hipError_t deform_fused_nchw_ws_launch(const void *q, const void *key, const void *value,
                                       const void *offset, void *out, void *workspace, int B, int Cq,
                                       int C, int H, int W, int P, int s, int G, int olayout,
                                       int dtype, hipStream_t st, const char **kernel = nullptr);

// sapa_layout.hip: contiguous [B, C, HW] -> channels-last [B, HW, C] for two tensors
// of the same B and HW in one launch (C1 = 0: one); esize 2 or 4 bytes
// zero0 / zero1: optional fp32 buffers of the same extents, cleared by the same launch when the
// vector form of the kernel applies (*zeroed tells)
hipError_t nchw_to_nhwc_launch(const void *src0, void *dst0, int C0, const void *src1, void *dst1,
                               int C1, int B, long HW, int esize, hipStream_t st, float *zero0 = nullptr,
                               float *zero1 = nullptr, bool *zeroed = nullptr);
// channels-last fp32 [B, HW, C] -> contiguous [B, C, HW] of dtype f32 / f16 / bf16 (0 / 2 / 3)
hipError_t nhwc_f32_to_nchw_launch(const float *src, void *dst, int C, int B, long HW, int dtype, hipStream_t st);

// sapa_d_wmat16.hip: the same operator for f16 / bf16 on the 16-bit matrix
// instructions; channels per group multiples of 8, key / value channels-last and
// aligned to 16 bytes, P <= 32.  nchw: query, offset and out are contiguous
// [B, channels, sH, sW] tensors instead of channels-last ones.
// hipErrorNotSupported otherwise.
hipError_t deform_fused_wmat16_launch(const void *q, const void *key, const void *value,
                                      const void *offset, void *out, int B, int Cq, int C, int H,
                                      int W, int P, int s, int G, int dtype, hipStream_t st,
                                      bool nchw = false, int olayout = 0);

// sapa_b_dot2.hip: qk, qk+softmax and fused for f16 / bf16 tensors on the
// two-term dot-product instructions (K = 5, s = 2); hipErrorNotSupported
// otherwise.  wide: fp32 K*K-channel tensors next to the 16-bit features
// (TILED_QK_SOFTMAX, and TILED_QK_SOFTMAX_BWD, which exists in this form only).
hipError_t sapa_b_dot2_launch(int mode, const void *q, const void *key, const void *attn_in,
                              const void *value, void *out, int B, int d, int C, int H, int W,
                              int K, int s, int dtype, hipStream_t st, bool wide = false);

// sapa_b_wmat16.hip: the fused forward for contiguous f16 / bf16 tensors (K = 5, s = 2) as two
// dense products over the 8 x 8 window of each 4 x 4 block of parents, on the 16-bit matrix
// instructions; hipErrorNotSupported otherwise.
hipError_t sapa_b_wmat16_launch(int mode, const void *q, const void *key, const void *value, void *out, int B,
                                int d, int C, int H, int W, int K, int s, int dtype, hipStream_t st);

// sapa_b_mfma.hip: the same four modes on the matrix pipe (4x4x1 MFMA, one
// block per parent); hipErrorNotSupported when (K, s, dtype) has no instance.
hipError_t sapa_b_mfma_launch(int mode, const void *q, const void *key, const void *attn_in,
                              const void *value, void *out, int B, int d, int C, int H, int W,
                              int K, int s, int dtype, hipStream_t st);

// sapa_b_lowgrad.hip: grad_key / grad_value as an LDS-tiled gather (no
// atomics, `out` fully overwritten).  hipErrorNotSupported unless f32 / f16 /
// bf16, s = 2, K in {3, 5}.  wide: the weight tensor w is fp32 whatever dtype is.
hipError_t lowres_grad_tiled_launch(const void *hi, const void *w, void *out, int B, int C, int H,
                                    int W, int K, int s, int dtype, hipStream_t st,
                                    bool wide = false);

// sapa_d_lds.hip: the SAPA-D forward ops gathering from an LDS-resident
// window; mode 0 = deform_qk (out = logits), 1 = deform_av (attn_in given),
// 2 = fused.  hipErrorNotSupported when (s, dtype, P) has no instance / does
// not fit LDS; the caller then takes the global-memory kernels below.
hipError_t deform_lds_launch(int mode, const void *q, const void *key, const void *attn_in,
                             const void *value, const void *offset, void *out, int B, int Cq, int C,
                             int H, int W, int P, int s, int G, int olayout, int dtype,
                             hipStream_t st, bool wide = false, bool accumulate = false,
                             float *partial = nullptr);

// sapa_d.hip.  olayout (OffsetLayout in deform_tap.hpp) says whether `offset`
// is the hi-res tensor or the low-res tensor it is produced from.
hipError_t deform_qk_forward_launch(const void *q, const void *key, const void *offset, void *out,
                                    int B, int Cq, int H, int W, int P, int s, int G, int olayout,
                                    int dtype, hipStream_t st);
hipError_t deform_av_forward_launch(const void *attn, const void *value, const void *offset,
                                    void *out, int B, int C, int H, int W, int P, int s, int G,
                                    int olayout, int dtype, hipStream_t st);
// P <= 64; hipErrorNotSupported otherwise
hipError_t deform_fused_forward_launch(const void *q, const void *key, const void *value,
                                       const void *offset, void *out, int B, int Cq, int C, int H,
                                       int W, int P, int s, int G, int olayout, int dtype,
                                       hipStream_t st);
// sapa_d_lowgrad.hip: grad_low of either sampled op (hi, sc as below) summed
// in LDS windows first (64-bit fixed point, integer atomics), one global float
// atomic per touched window cell.  fp32, s in {1, 2, 4}; hipErrorNotSupported
// otherwise.  Accumulates into grad_low.
hipError_t deform_lowgrad_lds_launch(const void *hi, const void *sc, const void *offset,
                                     void *grad_low, int B, int Cx, int H, int W, int P, int s,
                                     int G, int dtype, hipStream_t st, bool wide = false);

// grad_low (atomic accumulate, may be null) and grad_offset (store, may be
// null) of either sampled op: hi = per-channel high-res tensor [B,Cx,sH,sW],
// sc = per-point tensor [B,G,P,sH,sW], low = sampled tensor [B,Cx,H,W].
// dtype f32 / f64 only.
hipError_t deform_lowgrad_launch(const void *hi, const void *sc, const void *low,
                                 const void *offset, void *grad_low, void *grad_offset, int B,
                                 int Cx, int H, int W, int P, int s, int G, int dtype,
                                 hipStream_t st);

}  // namespace sapa
