/* C ABI of libsapa_hip.so: SAPA's upsampling operators as hand-written HIP
 * kernels for gfx950 (MI355X).
 *
 * This is the native boundary that the reference's four pybind11 extension
 * modules (qk_ext, av_ext, dqk, dav) occupy; each entry point below names the
 * reference function it stands in for.  Plain pointers and sizes only.
 *
 * Conventions, shared by every entry point:
 *   - every tensor is a DEVICE pointer to an NCHW-contiguous array of `dtype`
 *     elements (the reference's CHECK_CONTIGUOUS contract,
 *     sapa/sapa/src/cuda/qk_cuda.cpp:34-39);
 *   - H, W are the LOW-RES extents (key / value); the high-res extents are
 *     s*H, s*W (sapa/sapa/sapa_func.py:15-16);
 *   - buffers are borrowed for the duration of the asynchronous launch on
 *     `stream` (a hipStream_t; NULL = the default stream) and are never
 *     allocated, freed or retained by the library;
 *   - forward outputs are fully overwritten; gradient buffers are
 *     overwritten too, EXCEPT the low-res gradients of the sampled (deform)
 *     operators, which are accumulated with atomics and must arrive
 *     zero-filled, as the reference's callers provide them
 *     (deformsapa/deformsapa/deform_func.py:49-51);
 *   - the return value is SAPA_OK or a negative sapa_status; nothing here
 *     calls exit() or throws (the reference exits on a launch failure,
 *     qk_cuda_kernel.cu:92-96);
 *   - the library keeps no global state between calls: entry points are
 *     re-entrant and may be called from several host threads.
 *   - the device that is current on the calling thread must be the one that
 *     owns the buffers and `stream`.
 */
#ifndef SAPA_HIP_H
#define SAPA_HIP_H

#ifdef __cplusplus
extern "C" {
#endif

typedef enum sapa_dtype {
    SAPA_F32 = 0,
    SAPA_F64 = 1,
    SAPA_F16 = 2,
    SAPA_BF16 = 3
} sapa_dtype;

/* Where the sampled operators read the offsets from (the *_from entry points).
 * SAPADeform builds the hi-res offset tensor from a low-res 1x1-conv output,
 * by pixel_shuffle or by nearest interpolation (sapa_deform.py:44-47); the
 * last two values read that conv output in place instead. */
typedef enum sapa_offset_layout {
    SAPA_OFFSET_HIRES = 0,         /* [B, 2*G*P, sH, sW], as the reference's extensions take it */
    SAPA_OFFSET_PIXEL_SHUFFLE = 1, /* [B, 2*G*P*s*s, H, W]: hi[c][qh][qw] = lo[c*s*s + (qh%s)*s + qw%s][qh/s][qw/s] */
    SAPA_OFFSET_NEAREST = 2        /* [B, 2*G*P, H, W]: hi[c][qh][qw] = lo[c][qh/s][qw/s] */
} sapa_offset_layout;

typedef enum sapa_status {
    SAPA_OK = 0,
    SAPA_ERR_INVALID_ARGUMENT = -1, /* null pointer, non-positive extent, even K, ... */
    SAPA_ERR_UNSUPPORTED = -2,      /* valid request this build has no kernel for */
    SAPA_ERR_TOO_LARGE = -3,        /* an extent or element count exceeds the kernels' index range */
    SAPA_ERR_LAUNCH = -4            /* HIP reported a launch error; see sapa_hip_last_hip_error() */
} sapa_status;

/* Version of this ABI (bumped on any signature change). */
int sapa_hip_abi_version(void);
/* Static, human-readable text for a sapa_status. */
const char *sapa_hip_status_string(int status);
/* Text of the HIP error behind the calling thread's most recent
 * SAPA_ERR_LAUNCH ("" if none). */
const char *sapa_hip_last_hip_error(void);
/* Name of the kernel that served the calling thread's most recent forward
 * entry-point call ("" before the first): several kernels stand behind one
 * entry point and the choice depends on dtype, extents and alignment, so a
 * profile or a benchmark line can say which one it measured. */
const char *sapa_hip_last_kernel(void);

/* ------------------------------------------------------------------ SAPA-B */

/* Local query-key similarity.
 *   out[n, ky*K+kx, ph, pw] = sum_{c<d} key[n,c,ph/s-r+ky,pw/s-r+kx] * query[n,c,ph,pw],
 *   r = (K-1)/2; the whole sum is 0 where the neighbour is out of range.
 * query [B,d,sH,sW], key [B,d,H,W] -> out [B,K*K,sH,sW].
 * Replaces qk_ext.forward = qk_forward (sapa/sapa/src/qk_ext.cpp:22-34) ->
 * qk_forward_cuda (src/cuda/qk_cuda.cpp:41-60) -> QKForward
 * (src/cuda/qk_cuda_kernel.cu:30-68).  fp32 results are bit-identical to that
 * kernel's arithmetic (one FMA per channel, channels in order). */
int sapa_qk_forward(const void *query, const void *key, void *out,
                    int B, int d, int H, int W, int K, int s,
                    int dtype, void *stream);

/* Gradients of sapa_qk_forward.  grad_out [B,K*K,sH,sW] -> grad_query
 * [B,d,sH,sW], grad_key [B,d,H,W], both overwritten; either may be NULL to
 * skip it.  Gather formulation: deterministic, no atomics.
 * Replaces qk_ext.backward = qk_backward (qk_ext.cpp:36-50) -> QKBackward
 * (qk_cuda_kernel.cu:101-137). */
int sapa_qk_backward(const void *grad_out, const void *query, const void *key,
                     void *grad_query, void *grad_key,
                     int B, int d, int H, int W, int K, int s,
                     int dtype, void *stream);

/* Attention-value aggregation.
 *   out[n,c,ph,pw] = sum_{ky,kx} value[n,c,ph/s-r+ky,pw/s-r+kx] * attn[n,ky*K+kx,ph,pw],
 *   out-of-range neighbours skipped.
 * attn [B,K*K,sH,sW], value [B,C,H,W] -> out [B,C,sH,sW].
 * Replaces av_ext.forward = av_forward (sapa/sapa/src/av_ext.cpp:18-30) ->
 * av_forward_cuda (src/cuda/av_cuda.cpp:28-47) -> AVForward
 * (src/cuda/av_cuda_kernel.cu:30-75).  fp32 results are bit-identical to that
 * kernel's arithmetic (one FMA per neighbour, ky-major order). */
int sapa_av_forward(const void *attn, const void *value, void *out,
                    int B, int C, int H, int W, int K, int s,
                    int dtype, void *stream);

/* Gradients of sapa_av_forward.  grad_out [B,C,sH,sW] -> grad_attn
 * [B,K*K,sH,sW], grad_value [B,C,H,W], both overwritten; either may be NULL.
 * Replaces av_ext.backward = av_backward (av_ext.cpp:32-46) -> AVBackward
 * (av_cuda_kernel.cu:103-148). */
int sapa_av_backward(const void *grad_out, const void *attn, const void *value,
                     void *grad_attn, void *grad_value,
                     int B, int C, int H, int W, int K, int s,
                     int dtype, void *stream);

/* Gradient of the logits through the aggregation and the softmax in one
 * launch:  g = d(loss)/d(attn) = sum_c value[n,c,nbr_k] * grad_out[n,c,ph,pw]  (the
 * grad_attn of sapa_av_backward), then
 *   grad_logits[n,k,ph,pw] = attn[n,k,ph,pw] * (g[k] - sum_k' g[k'] * attn[n,k',ph,pw]),
 * the backward of F.softmax(., dim=1) in SAPA.attention (sapa_base.py:39-40).
 * grad_out [B,C,sH,sW], attn [B,K*K,sH,sW], value [B,C,H,W] -> grad_logits
 * [B,K*K,sH,sW].  SAPA_ERR_UNSUPPORTED when no register-tiled kernel covers
 * (K, s): use sapa_av_backward and a separate softmax backward then. */
int sapa_av_backward_logits(const void *grad_out, const void *attn, const void *value,
                            void *grad_logits, int B, int C, int H, int W,
                            int K, int s, int dtype, void *stream);

/* Backward of sapa_fused_forward in one call: the attention weights are
 * recomputed (they are not kept by the forward pass), then
 *   grad_value  = the aggregation's gradient for its low-res operand,
 *   grad_logits = softmax backward of the aggregation's gradient for the weights,
 *   grad_query, grad_key = the similarity's gradients for grad_logits,
 * i.e. what autograd derives from SAPA.attention (sapa_base.py:38-40) through
 * AVFunction.backward and QKFunction.backward (sapa/sapa/sapa_func.py:34-48,
 * 79-93).  The two [B,K*K,sH,sW] intermediates live in `workspace` as fp32
 * whatever `dtype` is (sapa_fused_backward_workspace bytes), so 16-bit tensors
 * are read and written as they are while nothing between them is rounded to 16
 * bits.  grad_query / grad_key / grad_value may each be NULL (not wanted); the
 * others are fully overwritten.  SAPA_ERR_UNSUPPORTED when the LDS-tiled
 * kernels do not cover the call (K other than 5, s other than 2, f64, unaligned
 * tensors): compose the gradient from sapa_av_backward / sapa_qk_backward then. */
long long sapa_fused_backward_workspace(int B, int H, int W, int K, int s);
int sapa_fused_backward(const void *grad_out, const void *query, const void *key,
                        const void *value, void *workspace, void *grad_query,
                        void *grad_key, void *grad_value, int B, int d, int C,
                        int H, int W, int K, int s, int dtype, void *stream);

/* The same pair for a training step that keeps the attention weights between its
 * two passes, as the reference does (QKFunction / AVFunction save their operands,
 * sapa/sapa/sapa_func.py:28,73, and autograd keeps the softmax output):
 * sapa_fused_forward_attn writes attn [B,K*K,sH,sW] -- fp32 whatever `dtype` is --
 * next to out (two launches: the weights, then the aggregation with them -- for
 * 16-bit tensors the one-launch forward, which forms the same fp32 weights itself;
 * nothing between the two products is rounded to 16 bits either way), and sapa_fused_backward_attn takes that
 * tensor instead of recomputing it; its workspace holds grad_logits only
 * (sapa_fused_backward_attn_workspace bytes, half of the other's).  Same results
 * as sapa_fused_backward on the same operands, one launch less per step and a
 * faster one in the forward pass of 16-bit tensors; the price is the attn tensor
 * kept alive.  Same SAPA_ERR_UNSUPPORTED cases. */
int sapa_fused_forward_attn(const void *query, const void *key, const void *value,
                            void *attn, void *out, int B, int d, int C, int H, int W,
                            int K, int s, int dtype, void *stream);
long long sapa_fused_backward_attn_workspace(int B, int H, int W, int K, int s);
int sapa_fused_backward_attn(const void *grad_out, const void *query, const void *key,
                             const void *value, const void *attn, void *workspace,
                             void *grad_query, void *grad_key, void *grad_value, int B,
                             int d, int C, int H, int W, int K, int s, int dtype,
                             void *stream);

/* Softmax over the middle axis of x [N,R,M] -> y [N,R,M] (max-subtracted,
 * fp32 arithmetic for 16-bit types).  Covers the reference's
 * F.softmax(logits, dim=1) on [B,K*K,sH,sW] (sapa_base.py:39: N=B, R=K*K,
 * M=sH*sW) and F.softmax(logits, dim=2) on [B,G,P,sH,sW]
 * (sapa_deform.py:52: N=B*G, R=P, M=sH*sW).  x == y (in place) is allowed. */
int sapa_softmax_forward(const void *x, void *y, long long N, int R, long long M,
                         int dtype, void *stream);

/* Fused sapa_qk_forward -> softmax over K*K -> sapa_av_forward in one launch:
 * the [B,K*K,sH,sW] logits/weights never touch HBM.  Out-of-range
 * neighbours have logit 0 and DO take part in the softmax denominator, as in
 * the three-launch composition SAPA.attention (sapa_base.py:38-40).
 * query [B,d,sH,sW], key [B,d,H,W], value [B,C,H,W] -> out [B,C,sH,sW].
 * Logits and weights are kept in fp32 (fp64 for SAPA_F64) whatever `dtype`.
 * K*K must not exceed 121 (SAPA_ERR_UNSUPPORTED otherwise). */
int sapa_fused_forward(const void *query, const void *key, const void *value,
                       void *out, int B, int d, int C, int H, int W,
                       int K, int s, int dtype, void *stream);

/* sapa_qk_forward -> softmax in one launch, writing the attention weights
 * attn [B,K*K,sH,sW] (what a training step keeps for the backward pass). */
int sapa_qk_softmax_forward(const void *query, const void *key, void *attn,
                            int B, int d, int H, int W, int K, int s,
                            int dtype, void *stream);

/* The same four forward operators for tensors in channels-last memory order
 * (torch.channels_last: a logical [B,C,H,W] tensor stored as [B,H,W,C]):
 * query [B,sH,sW,d], key [B,H,W,d], value [B,H,W,C], attn [B,sH,sW,K*K],
 * out [B,sH,sW,C] (qk: [B,sH,sW,K*K]).  The reference requires contiguous
 * NCHW tensors (CHECK_CONTIGUOUS, sapa/sapa/src/qk_cuda.cpp:35-39); these let
 * a channels-last model call the operators without a layout copy.  Covered:
 * SAPA_F32 / F16 / BF16, (K, s) in {(3,2), (5,2), (7,2), (5,4), (7,4)}, channel counts that are multiples
 * of 4, tensors aligned to 4 elements; SAPA_ERR_UNSUPPORTED otherwise.  The
 * channel sums run in tree order: results agree with sapa_*_forward to
 * rounding (1e-5 relative in fp32), not bit for bit.  16-bit tensors whose d
 * is a multiple of 8 run on the 16-bit matrix instructions: fp32 accumulation,
 * and in the fused operator the softmax weights are rounded to the tensor type
 * before the aggregation, as they are when qk, softmax and av are called one
 * after the other on 16-bit tensors. */
int sapa_qk_forward_nhwc(const void *query, const void *key, void *out,
                         int B, int d, int H, int W, int K, int s,
                         int dtype, void *stream);
int sapa_qk_softmax_forward_nhwc(const void *query, const void *key, void *attn,
                                 int B, int d, int H, int W, int K, int s,
                                 int dtype, void *stream);
int sapa_av_forward_nhwc(const void *attn, const void *value, void *out,
                         int B, int C, int H, int W, int K, int s,
                         int dtype, void *stream);
int sapa_fused_forward_nhwc(const void *query, const void *key, const void *value,
                            void *out, int B, int d, int C, int H, int W,
                            int K, int s, int dtype, void *stream);

/* sapa_fused_forward_nhwc on query + q_bias: q_bias [B,d] (may be NULL) is the
 * per-image bias of the query projection, added to every query vector inside
 * the kernel.  With the GroupNorm-folded projections of the module front end
 * (below) this replaces the bias pass over the hi-res query tensor that the
 * reference's Conv2d does as part of self.q (sapa/sapa/sapa_base.py:32).
 * q_bias aligned like the tensors (16 bytes for 16-bit tensors). */
int sapa_fused_forward_nhwc_qbias(const void *query, const void *key, const void *value,
                                  const void *q_bias, void *out, int B, int d, int C,
                                  int H, int W, int K, int s, int dtype, void *stream);

/* ------------------------------------------------------------------ SAPA-D */

/* Offset-sampled query-key similarity.
 *   out[b,g,p,qh,qw] = sum_{c<d} query[b,g*d+c,qh,qw] * bilinear(key[b,g*d+c]; kh, kw),
 *   kh = qh/s + offset[b,2*(g*P+p)+1,qh,qw], kw = qw/s + offset[b,2*(g*P+p),qh,qw]
 *   (offsets in low-res pixels, added to the integer parent coordinate);
 *   0 unless kh > -1 && kh < H && kw > -1 && kw < W; each of the four corners
 *   is zero-padded on its own.  d = Cq / G.
 * query [B,Cq,sH,sW], key [B,Cq,H,W], offset [B,2*G*P,sH,sW] -> out [B,G,P,sH,sW].
 * Replaces dqk.forward = deform_qk_forward
 * (deformsapa/deformsapa/src/deform_qk.cpp:32-48) -> deform_qk_forward_cuda
 * (src/cuda/deform_qk_cuda.cpp:45-68) -> DeformQKForward
 * (src/cuda/deform_qk_cuda_kernel.cu:139-197, bilinear :23-68).  Coordinates,
 * floor and the guard are evaluated in `dtype`'s arithmetic (fp32 for 16-bit
 * types), so fp32 corner indices are bit-exact with the reference's. */
int sapa_deform_qk_forward(const void *query, const void *key, const void *offset,
                           void *out, int B, int Cq, int H, int W,
                           int P, int s, int G, int dtype, void *stream);

/* Gradients of sapa_deform_qk_forward.  grad_query and grad_offset are
 * overwritten; grad_key is ACCUMULATED with atomics and must be zero-filled
 * by the caller.  Any of the three may be NULL.  SAPA_F32 / SAPA_F64 only.
 * Replaces dqk.backward = deform_qk_backward (deform_qk.cpp:50-70) ->
 * DeformQKBackward (deform_qk_cuda_kernel.cu:233-296, col2im :70-137). */
int sapa_deform_qk_backward(const void *grad_out, const void *query,
                            const void *key, const void *offset,
                            void *grad_query, void *grad_key, void *grad_offset,
                            int B, int Cq, int H, int W, int P, int s, int G,
                            int dtype, void *stream);

/* Offset-sampled attention-value aggregation.
 *   out[b,c,qh,qw] = sum_{p<P} attn[b,g(c),p,qh,qw] * bilinear(value[b,c]; kh, kw),
 *   g(c) = c / (C/G), same coordinates and guard as above.
 * attn [B,G,P,sH,sW], value [B,C,H,W], offset [B,2*G*P,sH,sW] -> out [B,C,sH,sW].
 * Replaces dav.forward = deform_av_forward
 * (deformsapa/deformsapa/src/deform_av.cpp:32-48) -> DeformAVForward
 * (src/cuda/deform_av_cuda_kernel.cu:139-195). */
int sapa_deform_av_forward(const void *attn, const void *value, const void *offset,
                           void *out, int B, int C, int H, int W,
                           int P, int s, int G, int dtype, void *stream);

/* Gradients of sapa_deform_av_forward.  grad_attn and grad_offset are
 * overwritten; grad_value is ACCUMULATED with atomics and must be
 * zero-filled by the caller.  Any may be NULL.  SAPA_F32 / SAPA_F64 only.
 * Replaces dav.backward = deform_av_backward (deform_av.cpp:50-70) ->
 * DeformAVBackward (deform_av_cuda_kernel.cu:230-292). */
int sapa_deform_av_backward(const void *grad_out, const void *attn,
                            const void *value, const void *offset,
                            void *grad_attn, void *grad_value, void *grad_offset,
                            int B, int C, int H, int W, int P, int s, int G,
                            int dtype, void *stream);

/* sapa_deform_qk_backward / sapa_deform_av_backward for SAPA_F16 / SAPA_BF16
 * tensors, read and written as they are: the half dispatch of the reference's
 * backward kernels (DeformQKBackwardLauncher, deform_qk_cuda_kernel.cu:298-337;
 * DeformAVBackwardLauncher, deform_av_cuda_kernel.cu:294-333).  The per-pixel
 * gradients are computed in fp32 from the 16-bit operands and rounded once; the
 * low-res gradient (grad_key / grad_value), a sum of many terms, is accumulated
 * in fp32 in `workspace` and rounded once -- so, unlike the fp32 entry points,
 * grad_key / grad_value are OVERWRITTEN here and need no zero fill.
 * sapa_deform_backward_workspace: bytes of device memory either call needs for
 * Cx = Cq (deform_qk) or C (deform_av) channels; 0 when this path does not serve
 * the case (s not in {1, 2, 4}, P > 48, other dtypes).  workspace: at least that
 * many bytes, aligned to 256, contents undefined before and after.
 * SAPA_ERR_UNSUPPORTED when the size is 0, workspace is NULL, or a kernel's window
 * does not fit the configuration (nothing the caller relies on is then written:
 * run the fp32 entry points on widened copies instead).  Any gradient may be NULL. */
long long sapa_deform_backward_workspace(int B, int Cx, int H, int W,
                                         int P, int s, int G, int dtype);
int sapa_deform_qk_backward_ws(const void *grad_out, const void *query,
                               const void *key, const void *offset, void *workspace,
                               void *grad_query, void *grad_key, void *grad_offset,
                               int B, int Cq, int H, int W, int P, int s, int G,
                               int dtype, void *stream);
int sapa_deform_av_backward_ws(const void *grad_out, const void *attn,
                               const void *value, const void *offset, void *workspace,
                               void *grad_attn, void *grad_value, void *grad_offset,
                               int B, int C, int H, int W, int P, int s, int G,
                               int dtype, void *stream);


/* Fused sapa_deform_qk_forward -> softmax over P -> sapa_deform_av_forward in
 * one launch (SAPADeform.attention, sapa_deform.py:51-53).  Sample positions
 * and bilinear weights are computed once per (pixel, group, point) and shared
 * by the similarity and the aggregation.  P must not exceed 64.
 * query [B,Cq,sH,sW], key [B,Cq,H,W], value [B,C,H,W],
 * offset [B,2*G*P,sH,sW] -> out [B,C,sH,sW]. */
int sapa_deform_fused_forward(const void *query, const void *key,
                              const void *value, const void *offset, void *out,
                              int B, int Cq, int C, int H, int W,
                              int P, int s, int G, int dtype, void *stream);

/* sapa_deform_fused_forward for tensors in channels-last memory order:
 * query [B,sH,sW,Cq], key [B,H,W,Cq], value [B,H,W,C], offset [B,sH,sW,2*G*P]
 * (channel 2(gP+p) = dx, +1 = dy), out [B,sH,sW,C].  No counterpart in the
 * reference, which requires contiguous NCHW tensors
 * (deformsapa/deformsapa/src/deform_qk.cpp, CHECK_CONTIGUOUS); this lets a
 * channels-last model call SAPADeform.attention (sapa_deform.py:51-53) without
 * layout copies.  Covered: SAPA_F32 / F16 / BF16, s in {1, 2, 4}, P <= 32,
 * Cq / G (at most 64) and C / G multiples of 4, tensors aligned to 4 elements;
 * SAPA_ERR_UNSUPPORTED otherwise.  The logits' channel sums run in tree order
 * (rounding-level differences from sapa_deform_fused_forward). */
int sapa_deform_fused_forward_nhwc(const void *query, const void *key,
                                   const void *value, const void *offset, void *out,
                                   int B, int Cq, int C, int H, int W,
                                   int P, int s, int G, int dtype, void *stream);

/* sapa_deform_fused_forward (same contiguous tensors, same result up to the
 * order of the sums) through the matrix-form kernels that serve the
 * channels-last entry point: the low-res key and value are first copied into
 * channels-last order in `workspace`, query / offset / out are used in place.
 * At B=8, C=256, G=4, d=32, P=25, 64x64 -> 128x128 this is 1.5x (fp32) to 2.5x
 * (bf16) faster than sapa_deform_fused_forward.  It replaces the same reference
 * calls (dqk.forward -> softmax -> dav.forward, sapa_deform.py:51-53).
 * sapa_deform_fused_forward_workspace: bytes of device memory the call needs,
 * 0 when this path does not serve the case (use sapa_deform_fused_forward).
 * workspace: at least that many bytes, aligned to 256; contents undefined
 * before and after.  SAPA_ERR_UNSUPPORTED when the size is 0 or workspace NULL.
 * offset_layout as in sapa_deform_fused_forward_from below: the offsets are
 * read from the hi-res tensor or in place from the low-res convolution output.
 * Served: s in {1, 2, 4}, Cq / G (at most 64) and C / G multiples of 4, and
 * enough points for it to pay: 4 <= P <= 32 for SAPA_F16 / BF16 with Cq / G and
 * C / G multiples of 8, 13 <= P <= 32 otherwise (SAPA_F32 included).  The sums
 * run per window cell instead of per point: fp32 results differ from
 * sapa_deform_fused_forward at rounding level (no further from the
 * double-precision result than it). */
long long sapa_deform_fused_forward_workspace(int B, int Cq, int C, int H, int W,
                                              int P, int s, int G, int dtype);
int sapa_deform_fused_forward_ws(const void *query, const void *key,
                                 const void *value, const void *offset, void *out,
                                 void *workspace, int B, int Cq, int C, int H, int W,
                                 int P, int s, int G, int offset_layout, int dtype,
                                 void *stream);

/* Backward pass of sapa_deform_fused_forward in one call: gradients of
 *   deform_av(softmax(deform_qk(query, key, offset), dim = points), value, offset)
 * with respect to query, key, value and offset (hi-res layout).  It replaces the
 * chain dav.backward (deform_av.cpp:50-70) -> softmax backward (ATen) ->
 * dqk.backward (deform_qk.cpp:50-70) that autograd runs for
 * SAPADeform.attention (sapa_deform.py:51-53), with the weights recomputed from
 * query / key.  The attention weights and the gradient of the logits
 * [B,G,P,sH,sW] are fp32 in `workspace` whatever `dtype` is; SAPA_F16 / BF16
 * tensors are read and written as they are; the low-res gradients and the two
 * contributions to grad_offset are summed in fp32 and rounded once.  All four gradients are overwritten; any may be NULL.
 * sapa_deform_fused_backward_workspace: bytes needed (256-byte aligned), 0 when
 * the configuration is not served -- SAPA_F64, s outside {1, 2, 4}, P > 48 --
 * and the caller chains sapa_deform_av_backward / sapa_deform_qk_backward;
 * SAPA_ERR_UNSUPPORTED then, before anything is written. */
long long sapa_deform_fused_backward_workspace(int B, int Cq, int C, int H, int W,
                                               int P, int s, int G, int dtype);
int sapa_deform_fused_backward(const void *grad_out, const void *query, const void *key,
                               const void *value, const void *offset, void *workspace,
                               void *grad_query, void *grad_key, void *grad_value,
                               void *grad_offset, int B, int Cq, int C, int H, int W,
                               int P, int s, int G, int dtype, void *stream);

/* The three sampled forward operators reading the offsets in the layout
 * `offset_layout` (sapa_offset_layout) names; with SAPA_OFFSET_HIRES they are
 * the functions above.  They replace
 *   F.pixel_shuffle(self.offset(x_), s)  /  F.interpolate(self.offset(x_), scale_factor=s)
 * followed by dqk.forward / dav.forward (sapa_deform.py:44-53): the hi-res
 * offset tensor is never written.  Results are bit-identical to materialising
 * it first. */
int sapa_deform_qk_forward_from(const void *query, const void *key, const void *offset,
                                void *out, int B, int Cq, int H, int W, int P, int s, int G,
                                int offset_layout, int dtype, void *stream);
int sapa_deform_av_forward_from(const void *attn, const void *value, const void *offset,
                                void *out, int B, int C, int H, int W, int P, int s, int G,
                                int offset_layout, int dtype, void *stream);
int sapa_deform_fused_forward_from(const void *query, const void *key, const void *value,
                                   const void *offset, void *out, int B, int Cq, int C,
                                   int H, int W, int P, int s, int G, int offset_layout,
                                   int dtype, void *stream);

/* ------------------------------------------------------- module front end */

/* Mean and biased variance of every (image, channel) of a feature map, one
 * pass over it: x [B,C,HW] contiguous (channels_last = 0) or [B,HW,C]
 * (channels_last = 1) -> mean_var [B,C,2] fp32.  These are the statistics
 * behind the reference's GroupNorm(32) on y and x ahead of the q / k
 * projections (sapa/sapa/sapa_base.py:17-19,27-31, an ATen call there); the
 * caller combines them per group and folds the normalisation into the 1x1
 * projection weights.  workspace: sapa_channel_moments_workspace(...) bytes of
 * device memory, contents undefined before and after.  SAPA_F32 / F16 / BF16;
 * channels_last needs C % 4 == 0, C <= 1024 and x aligned to 4 elements, the
 * contiguous layout B * C <= 65535; SAPA_ERR_UNSUPPORTED otherwise.  No
 * atomics: the result does not depend on scheduling. */
long long sapa_channel_moments_workspace(int B, int C, long long HW, int channels_last);
int sapa_channel_moments(const void *x, void *workspace, float *mean_var,
                         int B, int C, long long HW, int channels_last,
                         int dtype, void *stream);

/* sapa_channel_moments without a workspace argument, for callers that cannot
 * allocate device memory: code under HIP graph capture, serving loops and
 * harnesses that forbid allocator calls.  No counterpart in the reference.
 * The partial sums go to a fixed array of sapa_channel_moments_static_capacity()
 * bytes (8 MiB) that is part of the library's code object on every device it
 * runs on; the call allocates and frees nothing.  Same arguments, coverage and
 * results (bit for bit) as sapa_channel_moments; SAPA_ERR_TOO_LARGE when
 * sapa_channel_moments_workspace(B, C, HW, channels_last) exceeds the capacity.
 * All calls on one device share that array: calls that overlap in time on the
 * same device (different streams or host threads) race and must be serialised
 * by the caller.  The first call on each device looks the array's address up
 * (hipGetSymbolAddress): make that call outside a stream capture; later calls
 * only launch kernels and may be captured. */
long long sapa_channel_moments_static_capacity(void);
int sapa_channel_moments_static(const void *x, float *mean_var,
                                int B, int C, long long HW, int channels_last,
                                int dtype, void *stream);

/* GroupNorm folded into a 1x1 projection, per image: from mean_var (above),
 * the norm's gamma / beta [C] (NULL: 1 / 0), `groups` and eps, and the
 * projection's weight [O,C] and bias [O] (NULL: none), all of type `dtype`:
 *   weight_out[b,o,c] = weight[o,c] * gamma[c] * rstd[b,g(c)]
 *   bias_out[b,o]     = bias[o] + sum_c weight[o,c] * (beta[c] - mean[b,g(c)] * gamma[c] * rstd[b,g(c)])
 * so that conv(groupnorm(x))[b] = weight_out[b] x[b] + bias_out[b]: the
 * reference's norm_y -> q and norm_x -> k (sapa/sapa/sapa_base.py:26-36) become
 * one GEMM each on the un-normalised feature.  SAPA_F32 / F16 / BF16,
 * C <= 8192. */
int sapa_groupnorm_fold(const float *mean_var, const void *gamma, const void *beta,
                        const void *weight, const void *bias, void *weight_out, void *bias_out,
                        int B, int C, int O, int groups, float eps, int dtype, void *stream);

/* 1x1 projection with per-image weights on a channels-last feature:
 *   out[b,p,o] = sum_c x[b,p,c] * weight[b,o,c] (+ bias[b,o]),
 * x [B,HW,C], weight [B,O,C] (sapa_groupnorm_fold's output), bias [B,O] or NULL,
 * out [B,HW,O] -- self.q(norm_y(y)) / self.k(norm_x(x)) of the reference
 * (sapa/sapa/sapa_base.py:32-35; Conv2d and GroupNorm, ATen calls there) as one
 * stream over the feature.  SAPA_F16 / SAPA_BF16 / SAPA_F32, C in {64,128,256,512},
 * O in {32,64,128} (not every pair; SAPA_F32: the pairs with 6 * C * O bytes of
 * weights within the LDS, e.g. (256,64), (512,32)), pointers aligned to 16 bytes;
 * SAPA_ERR_UNSUPPORTED otherwise.  SAPA_F32 multiplies on the bf16 matrix
 * instruction, each product as six products of bf16 pieces with fp32 sums: the
 * result of an fp32 dot product to rounding, in another order of summation than a
 * library GEMM's. */
int sapa_project_nhwc(const void *x, const void *weight, const void *bias, void *out,
                      int B, int C, int O, long long HW, int dtype, void *stream);

/* The same projection of a contiguous feature x [B,C,HW] (the reference's layout:
 * self.q(norm_y(y)) on an NCHW tensor, sapa/sapa/sapa_base.py:32-35): out [B,O,HW],
 * or [B,HW,O] (channels-last, what the channels-last operator takes) when
 * out_channels_last is non-zero.  SAPA_F32 / SAPA_F16 / SAPA_BF16, the (C,O) pairs of
 * sapa_project_nhwc's SAPA_F32 form; SAPA_F32: HW a multiple of 4 for a [B,O,HW]
 * result; 16-bit: HW a multiple of 8; x and out aligned to 16 bytes;
 * SAPA_ERR_UNSUPPORTED otherwise (the caller uses a library GEMM). */
int sapa_project_nchw(const void *x, const void *weight, const void *bias, void *out,
                      int B, int C, int O, long long HW, int out_channels_last, int dtype,
                      void *stream);

/* self.q(self.norm_y(y)) / self.k(self.norm_x(x)) (sapa/sapa/sapa_base.py:27-35; GroupNorm and a
 * 1x1 Conv2d, ATen calls there) in one call: sapa_channel_moments, sapa_groupnorm_fold and
 * sapa_project_nhwc (x_channels_last != 0; the result is channels-last) or sapa_project_nchw
 * (result [B,O,HW], or [B,HW,O] when out_channels_last != 0) on one stream -- four launches,
 * the normalised feature never written.  gamma / beta [C] (NULL: 1 / 0), weight [O,C], bias
 * [O] or NULL, all of type `dtype`.  scratch: sapa_norm_project_scratch(...) bytes, aligned
 * to 16 (intermediates; nothing to keep).  bias_out, if not NULL, receives the folded
 * per-image bias [B,O] and the projection is written WITHOUT it (for
 * sapa_fused_forward_nhwc_qbias); if NULL the bias is added.  Nothing is launched and
 * SAPA_ERR_UNSUPPORTED returned unless every step has a kernel for the configuration
 * (SAPA_F32 / F16 / BF16, C a multiple of groups and <= 8192, the (C,O) pairs and extents
 * of the projection entry points, x and out aligned to 16 bytes). */
long long sapa_norm_project_scratch(int B, int C, int O, long long HW, int x_channels_last,
                                    int dtype);
int sapa_norm_project(const void *x, const void *gamma, const void *beta, const void *weight,
                      const void *bias, void *scratch, void *out, void *bias_out, int B, int C,
                      int O, long long HW, int groups, float eps, int x_channels_last,
                      int out_channels_last, int dtype, void *stream);

/* ------------------------------------------------------------ calibration */

/* Layout copy between the two memory orders the library serves: a dense
 * [B, C, HW] tensor (contiguous, the reference's order) into channels-last
 * order [B, HW, C] (to_channels_last = 1) or the other way (0), elements of
 * esize = 2 or 4 bytes moved as they are.  No counterpart in the reference
 * (which has no channels-last tensors); it is for the callers of the *_nhwc
 * entry points whose backward pass runs on the contiguous kernels: one
 * transposing launch (64 x 64-element tiles through LDS, 16-byte accesses on
 * both sides where C, HW and the pointers allow) in place of a generic
 * strided copy.  src and dst must not overlap.  SAPA_ERR_UNSUPPORTED for more
 * than 65535 images or 4194240 rows of the side that is split into tiles
 * (C for to_channels_last = 1, HW for 0). */
int sapa_layout_copy(const void *src, void *dst, int B, int C, long long HW, int to_channels_last,
                     int esize, void *stream);

/* A kernel that only moves bytes, for putting the operators' measured rates
 * beside what the memory system gives a plain stream of the same read : write
 * mix.  No counterpart in the reference (which has no measurement code).
 * Unit u reads the contiguous run src[u * reads * 4096 ... + reads * 4096) and
 * writes the contiguous run dst[u * writes * 4096 ... + writes * 4096) (bytes),
 * the written words being a function of the words read; a workgroup takes
 * `reps` consecutive units (runs `reps` times as long), the next unit's loads
 * issued before the current unit's stores.  writes = 0: src is only read (dst
 * needs 4096 bytes per workgroup and is left untouched unless a 16-byte group
 * of src is ff..fe in every word).  nontemporal: bit 0 = streaming
 * (non-temporal) loads, bit 1 = streaming stores; bit 2 ((9,16) only): readers
 * and writers are different workgroups -- `units` groups of 9 workgroups that
 * each read one run of reps * 65536 bytes of src and 16 that each write one of
 * dst, nothing written depending on anything read (src needs units * 9 * reps
 * * 65536 bytes, dst units * 16 * reps * 65536).  (reads, writes) in {(9,16): a fused SAPA-B forward at up_factor 2
 * with C = 4 d, (8,8), (0,16), (16,0)}; SAPA_ERR_UNSUPPORTED otherwise.
 * Pointers aligned to 16 bytes. */
int sapa_stream_mix(const void *src, void *dst, long long units, int reads, int writes, int reps,
                    int nontemporal, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* SAPA_HIP_H */
