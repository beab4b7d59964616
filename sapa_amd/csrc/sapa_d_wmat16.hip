// Fused SAPA-D forward for f16 / bf16 tensors in channels-last memory order,
// as two matrix products per (tile, group) on the 16-bit matrix instructions
// (v_mfma_f32_16x16x32).  Tensors as in sapa_d_nhwc.hip: query [B, sH, sW, G*d],
// key [B, H, W, G*d], value [B, H, W, C], offset [B, sH, sW, 2*G*P], out
// [B, sH, sW, C].
//
// Every sample of a pixel lies within RCH cells of the pixel's parent (the few
// that do not are handled apart), so the 4 P bilinear corners of a pixel fall on
// the window cells of its tile, and both sampled products become dense ones
// whose big operand -- the window -- is shared by all pixels of the tile:
//
//   similarity  Sim[pixel][cell] = q[pixel] . key[cell]                 (NPX x KP x d)
//   logits      l[pixel][p]      = sum_corners w_c * Sim[pixel][cell_c]      (gather)
//   softmax over the P points of the pixel
//   weights     Wm[pixel][cell] += att_p * w_c                              (scatter)
//   output      out[pixel][ch]   = sum_cells Wm[pixel][cell] * value[cell][ch]
//                                                                       (NPX x KP x 64)
//
// The windows stay 16-bit in LDS, in the tensors' own [cell][channel] order:
//   * Sim contracts over channels, which both operands hold contiguously;
//   * the output contracts over cells: its B operand -- 8 cells of one channel
//     per lane -- comes from ds_read_b64_tr_b16, which hands each lane of a
//     16-lane block one 16-bit column of the 4 x 16 elements the block addresses;
//   * Wm is built as 2^30-scaled integers with LDS integer adds (exact in any
//     order, so the result does not depend on scheduling, and several times
//     faster than float atomics), then split in place into a 16-bit high part and
//     a 16-bit remainder, each an A operand: the softmax weights enter the
//     product with ~16 significant bits, fp32 accumulation.
// q . key products of 16-bit inputs are exact in fp32, so the logits differ
// from an fp32 evaluation of the reference's expression
// (deformsapa/deformsapa/src/cuda/deform_qk_cuda_kernel.cu:23-68,187) only by
// summation order.  Index math, the strict guard and the zero padding are those
// of deform_tap.hpp; window cells outside the image hold zeros.
#include <utility>

#include "deform_tap.hpp"
#include "kernels.hpp"

namespace sapa {

namespace dwm16 {

typedef unsigned u32;
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef u32 u32x2 __attribute__((ext_vector_type(2)));
typedef u32 u32x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));

constexpr int RCH = 4;          // window reach around the tile's parents, in low-res cells
constexpr int NT = 256;
constexpr float WSCALE = 1073741824.f;      // 2^30: fixed-point scale of Wm

template <typename T> struct Half;
template <> struct Half<f16_t> {
    typedef _Float16 v8 __attribute__((ext_vector_type(8)));
    static __device__ __forceinline__ f32x4 mma(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8, a), __builtin_bit_cast(v8, b), c, 0, 0, 0);
    }
    // Wm entries reach the A operand times 2^10 (2^30 would overflow the format)
    static constexpr float IN_SCALE = 1.f / 1048576.f, OUT_SCALE = 1.f / 1024.f;
};
template <> struct Half<bf16_t> {
    typedef __bf16 v8 __attribute__((ext_vector_type(8)));
    static __device__ __forceinline__ f32x4 mma(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8, a), __builtin_bit_cast(v8, b), c, 0, 0, 0);
    }
    static constexpr float IN_SCALE = 1.f, OUT_SCALE = 1.f / WSCALE;
};

// 8 fixed-point weights -> 8 high parts and 8 remainders
template <typename T>
__device__ __forceinline__ void split8(u32x4 a, u32x4 b, u32x4 &hi, u32x4 &lo);
template <>
__device__ __forceinline__ void split8<f16_t>(u32x4 a, u32x4 b, u32x4 &hi, u32x4 &lo) {
    union { f16_t h[8]; u32x4 u; } xh, xl;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const float f = (float)(e < 4 ? a[e] : b[e - 4]) * Half<f16_t>::IN_SCALE;
        const f16_t h = (f16_t)f;
        xh.h[e] = h;
        xl.h[e] = (f16_t)(f - (float)h);
    }
    hi = xh.u;
    lo = xl.u;
}
// bf16 = the upper half of an fp32: the high part is the value truncated to
// it, the remainder (exact in fp32) is truncated likewise -- what is dropped is
// below 2^-14 of the weight
template <>
__device__ __forceinline__ void split8<bf16_t>(u32x4 a, u32x4 b, u32x4 &hi, u32x4 &lo) {
    u32 fb[8], rb[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const float f = (float)(e < 4 ? a[e] : b[e - 4]);
        fb[e] = __builtin_bit_cast(u32, f);
        rb[e] = __builtin_bit_cast(u32, f - __builtin_bit_cast(float, fb[e] & 0xffff0000u));
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        hi[e] = __builtin_amdgcn_perm(fb[2 * e + 1], fb[2 * e], 0x07060302);    // upper halves of the two
        lo[e] = __builtin_amdgcn_perm(rb[2 * e + 1], rb[2 * e], 0x07060302);
    }
}

// two consecutive 16-bit elements held as loaded -> floats
template <typename T>
__device__ __forceinline__ f32x2 widen_pair(u32 raw) {
    union { u32 u; T h[2]; } x;
    x.u = raw;
    f32x2 f = {(float)x.h[0], (float)x.h[1]};
    return f;
}

template <typename T>
__device__ __forceinline__ u32x4 narrow8(f32x4 a, f32x4 b) {
    union { T h[8]; u32x4 u; } x;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        x.h[e] = (T)a[e];
        x.h[4 + e] = (T)b[e];
    }
    return x.u;
}

// TH x TW hi-res pixels per workgroup, DP = the group's query / key channels
// rounded up to 32.  Thread views of the 256 threads: 8 lanes per window cell
// or output pixel (lane = 8 channels) for staging and stores; the matrix
// instruction's (lane % 16, lane / 16) operand layout; 16 or 32 lanes per
// pixel, one lane per point, for the per-sample work.
#ifndef SAPA_WM16_WPE
#define SAPA_WM16_WPE 4
#endif
#ifndef SAPA_WM16_VPAD
#define SAPA_WM16_VPAD 8
#endif
// NCHW: query, offset and out are contiguous [B, channels, sH, sW] tensors (the
// reference's layout); key and value are channels-last either way (the launcher
// hands copies in that order to this kernel).
template <typename T, int S, int TH, int TW, int DP, bool NCHW>
__global__ void __launch_bounds__(NT) __attribute__((amdgpu_waves_per_eu(SAPA_WM16_WPE, SAPA_WM16_WPE)))
deform_fused_wmat16_kernel(const T *__restrict__ q, const T *__restrict__ key,
                           const T *__restrict__ value, const T *__restrict__ offset,
                           T *__restrict__ out, int Cq, int C, int H, int W, int P, int G,
                           int tiles_x, int tiles_y, int nblocks, int per_xcd, int olayout) {
    constexpr int NPX = TH * TW, NMB = NPX / 16;             // pixels, blocks of 16 matrix rows
    constexpr int WWY = (TH + S - 1) / S + 2 * RCH + 1;      // window cells per axis
    constexpr int WWX = (TW + S - 1) / S + 2 * RCH + 1;
    constexpr int NPOS = WWY * WWX;
    constexpr int KP = (NPOS + 31) / 32 * 32;                // cells padded to whole contraction steps
    constexpr int NCB = (NPOS + 15) / 16, NKS = KP / 32;     // blocks of 16 cells that hold any; steps of 32
    constexpr int CHK = 64;                                  // value channels per chunk
    // Row strides.  Key rows: DP + 8 elements = 20 or 36 dwords, so that the 16
    // rows a 16-byte operand read touches start in 16 different banks of 4.  Value
    // rows: 80 elements = 40 dwords, so that the 8 rows of 32 bytes a transposing
    // read touches per half cover the 64 banks once.
    constexpr int KSB = DP + 8, VSB = CHK + SAPA_WM16_VPAD;
    constexpr int XSZ = KP * (KSB > VSB ? KSB : VSB);
    constexpr int WS = KP + 4;      // dwords per row of Sim / Wm: 4 mod 32
    constexpr int OS = CHK + 4;     // floats per row of the output tile
    static_assert(NPX % 16 == 0 && DP % 32 == 0 && DP <= 64, "whole blocks of matrix rows, whole contraction steps");
    static_assert(TH % S == 0 || S % TH == 0, "tile rows start at a parent's first row");

    __shared__ __attribute__((aligned(16))) T Xl[XSZ];              // key window, then value window
    __shared__ __attribute__((aligned(16))) u32 SWl[NPX * WS];      // Sim (fp32), then Wm, then its 16-bit split
    __shared__ __attribute__((aligned(16))) float Ol[NPX * OS];     // output tile
    constexpr int QSB = DP + 8;     // elements per pixel of the q tile (contiguous-layout callers)
    __shared__ __attribute__((aligned(16))) T Ql[NCHW ? NPX * QSB : 8];
    float *const Sl = (float *)SWl;

    const int logical = (int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8);
    if (logical >= nblocks) return;
    const int tx = logical % tiles_x;
    const int ty = (logical / tiles_x) % tiles_y;
    const int n = logical / (tiles_x * tiles_y);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int hH = H * S, hW = W * S;
    const int y0 = ty * TH, x0 = tx * TW;                            // tile origin, hi-res
    const int wy0 = y0 / S - RCH, wx0 = x0 / S - RCH;                // window origin, low-res cell
    const long lpix = (long)H * W;
    const int d = Cq / G, cg = C / G;
    const int nVc = (cg + CHK - 1) / CHK;

    // pixel i of the tile (row-major): inside the image?  its flat hi-res index,
    // clamped for loads, and its parent
    struct Pix { bool active; long hp; int pp, ph, pw; };
    const long hpl = (long)hH * hW;                                  // a hi-res channel plane (NCHW)
    auto pixel = [&](int i) __attribute__((always_inline)) {
        const int qh = y0 + i / TW, qw = x0 + i % TW;
        Pix r;
        r.active = qh < hH && qw < hW;
        const int ch = qh < hH ? qh : hH - 1, cw = qw < hW ? qw : hW - 1;
        r.pp = ch * hW + cw;
        r.hp = (long)n * hH * hW + r.pp;
        r.ph = ch / S;
        r.pw = cw / S;
        return r;
    };
    const int mi = lane & 15, mk = lane >> 4;        // matrix operand view
    const int c8 = tid & 7;                          // staging / store view: 8 channels per lane

    // ---- window staging.  Key: DP / 8 lanes per cell; value: 8 lanes per cell, 32
    // cells per pass.  Per-thread byte offsets into the image's key and value
    // tensor, fixed for the whole kernel; 2^31 = beyond every descriptor, i.e.
    // zero fill: cells outside the image, the padding cells NPOS .. KP, channels
    // past the group's.  A chunk's first channel travels as the instruction's
    // scalar offset.
    constexpr int TK = DP / 8, CPK = NT / TK, NPK = (KP + CPK - 1) / CPK, NPV = KP / 32;
    constexpr int NST = NPK > NPV ? NPK : NPV;
    const int kc8 = tid % TK;
    const int cv0 = cg < CHK ? cg : CHK;                             // channels of a full value chunk
    u32 koff[NPK], voff[NPV];
    auto cell_pix = [&](int pos, bool &ok) __attribute__((always_inline)) {
        const int gy = wy0 + pos / WWX, gx = wx0 + pos % WWX;
        ok = pos < NPOS && gy >= 0 && gy < H && gx >= 0 && gx < W;
        return gy * W + gx;
    };
#pragma unroll
    for (int p = 0; p < NPK; ++p) {
        bool ok;
        const int pix = cell_pix(p * CPK + tid / TK, ok);
        koff[p] = (ok && 8 * kc8 < d) ? (u32)(pix * Cq + 8 * kc8) * 2u : 0x80000000u;
    }
#pragma unroll
    for (int p = 0; p < NPV; ++p) {
        bool ok;
        const int pix = cell_pix(p * 32 + tid / 8, ok);
        voff[p] = (ok && 8 * c8 < cv0) ? (u32)(pix * C + 8 * c8) * 2u : 0x80000000u;
    }
    const __amdgpu_buffer_rsrc_t krsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(key + (long)n * lpix * Cq), 0, (int)(lpix * Cq * 2L), 0x00020000);
    const __amdgpu_buffer_rsrc_t vrsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(value + (long)n * lpix * C), 0, (int)(lpix * C * 2L), 0x00020000);
    u32x4 st[NST];
    auto stage_load_key = [&](int cbase) __attribute__((always_inline)) {
#pragma unroll
        for (int p = 0; p < NPK; ++p) st[p] = __builtin_amdgcn_raw_buffer_load_b128(krsrc, koff[p], (u32)cbase * 2u, 0);
    };
    auto stage_load_value = [&](int cbase, int cvalid) __attribute__((always_inline)) {
        const bool whole = cvalid == cv0 || 8 * c8 < cvalid;        // else: past the ragged last chunk
#pragma unroll
        for (int p = 0; p < NPV; ++p)
            st[p] = __builtin_amdgcn_raw_buffer_load_b128(vrsrc, whole ? voff[p] : 0x80000000u, (u32)cbase * 2u, 0);
    };
    auto stage_store_key = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int p = 0; p < NPK; ++p) {
            const int pos = p * CPK + tid / TK;
            if (KP % CPK == 0 || pos < KP) *(u32x4 *)(Xl + pos * KSB + 8 * kc8) = st[p];
        }
    };
    auto stage_store_value = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int p = 0; p < NPV; ++p) *(u32x4 *)(Xl + (p * 32 + tid / 8) * VSB + 8 * c8) = st[p];
    };
    // q of pixel 16 mb + mi as the A operand: channels 32 ks + 8 mk .. + 7 of the group.
    // Channels-last: 16 contiguous bytes of global memory per lane.  Contiguous
    // layout: the tile's q (NPX pixels x d channel planes) comes in once per
    // workgroup, a thread fetching pairs of x-neighbours of one plane, and goes
    // through LDS as [pixel][channel], from where every wave reads its operands.
    u32x4 qa[NCHW ? 1 : NMB][DP / 32];
    constexpr int QN = NCHW ? NPX * DP / 2 / NT : 1;     // pixel pairs per thread
    static_assert(!NCHW || (NPX * DP / 2) % NT == 0, "the q tile divides over the threads");
    u32 qraw[QN];
    const bool q32 = hW % 2 == 0 && (uintptr_t)q % 4 == 0;           // pairs are aligned dwords
    auto load_q = [&](int g) __attribute__((always_inline)) {
        if (NCHW) {
#pragma unroll
            for (int i = 0; i < QN; ++i) {
                const int item = i * NT + tid;
                const int ch = item / (NPX / 2), pr = item % (NPX / 2);
                const int qh = y0 + pr / (TW / 2), qw = x0 + 2 * (pr % (TW / 2));
                qraw[i] = 0u;
                if (ch < d && qh < hH && qw < hW) {
                    const T *qp = q + ((long)n * Cq + g * d + ch) * hpl + (long)qh * hW + qw;
                    if (q32) {
                        qraw[i] = *(const u32 *)qp;
                    } else {
                        union { T h[2]; u32 u; } x;
                        x.u = 0u;
                        x.h[0] = qp[0];
                        if (qw + 1 < hW) x.h[1] = qp[1];
                        qraw[i] = x.u;
                    }
                }
            }
        } else {
#pragma unroll
            for (int mb = 0; mb < NMB; ++mb) {
                const Pix px = pixel(16 * mb + mi);
#pragma unroll
                for (int ks = 0; ks < DP / 32; ++ks) {
                    qa[mb][ks] = u32x4{0u, 0u, 0u, 0u};
                    if (px.active && 32 * ks + 8 * mk < d)
                        qa[mb][ks] = *(const u32x4 *)(q + px.hp * Cq + g * d + 32 * ks + 8 * mk);
                }
            }
        }
    };
    // (contiguous layout) the fetched pairs into the q tile; channels d .. DP hold zeros
    auto stage_store_q = [&]() __attribute__((always_inline)) {
        if (!NCHW) return;
#pragma unroll
        for (int i = 0; i < QN; ++i) {
            const int item = i * NT + tid;
            const int ch = item / (NPX / 2), pr = item % (NPX / 2);
            const int pi = (pr / (TW / 2)) * TW + 2 * (pr % (TW / 2));
            union { u32 u; T h[2]; } x;
            x.u = qraw[i];
            Ql[pi * QSB + ch] = x.h[0];
            Ql[(pi + 1) * QSB + ch] = x.h[1];
        }
    };

    // per-sample passes over the tile: P <= 16 -> 16 lanes per pixel, else 32
    const bool narrow = P <= 16;
    constexpr int NSP = NPX / 8;                     // passes of the 32-lane mapping
    const int nsp = narrow ? NPX / 16 : NPX / 8;
    const int pt = narrow ? (tid & 15) : (tid & 31); // this lane's point
    const int prow = narrow ? (tid >> 4) : (tid >> 5);
    const int ppp = narrow ? 16 : 8;                 // pixels per pass

    // a group's offsets (dx, dy of this lane's point, per pass) are fetched while the
    // group before it is aggregated, and stay as loaded until their use: nothing
    // waits for them where they are issued
    u32 offraw[NSP], offnext[NSP];
    // Contiguous hi-res offsets whose tile rows are whole aligned vectors come in as
    // such: thread t fetches the 4 x-neighbours of tile row (t / 2) % 4 in the dx
    // (t even) or dy plane of point t / 8 -- one 8-byte load per thread instead of
    // four 2-byte ones, and a quarter of the memory requests -- through a buffer
    // descriptor (out-of-range offset = no access), and they reach the lanes that
    // use them through LDS, as the (dx, dy) pairs the other paths load directly.
    __shared__ __attribute__((aligned(16))) T Ost[NCHW ? 32 * NPX * 2 : 8];
    const bool ovec = NCHW && olayout == OFFSET_HIRES && hW % TW == 0 && TW == 4 && TH == 4 &&
                      (uintptr_t)offset % 8 == 0 && 2L * G * P * hpl * (long)sizeof(T) < (1L << 31);
    const __amdgpu_buffer_rsrc_t orsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(offset + (long)n * 2 * G * P * hpl), 0, ovec ? (int)(2L * G * P * hpl * (long)sizeof(T)) : 0, 0x00020000);
    static_assert(NSP >= 2 || !NCHW, "the vector form keeps its 8 bytes in the two offnext registers");
    auto load_offsets = [&](int g) __attribute__((always_inline)) {
        if (ovec) {
            // this thread's piece within a group's planes (worked out here each time,
            // from an opaque copy of the thread index: kept across the kernel it would
            // cost a register the kernel does not have); the group's first plane
            // travels as the load's scalar offset
            int t = tid;
            asm volatile("" : "+v"(t));
            const int xy = t & 1, row = (t >> 1) & 3, opt = t >> 3;
            const u32 ovoff = (opt < P && y0 + row < hH)
                                  ? (u32)(((2L * opt + xy) * hpl + (long)(y0 + row) * hW + x0) * (long)sizeof(T))
                                  : 0x80000000u;
            const u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(orsrc, ovoff, (u32)(2L * g * P * hpl * (long)sizeof(T)), 0);
            offnext[0] = v[0];
            offnext[NSP > 1 ? 1 : 0] = v[1];
            return;
        }
        // (the addresses are worked out from an opaque copy of the lane's pixel row:
        // hoisted out of the loop over the groups they would be spilled)
        int prow_o = prow;
        asm volatile("" : "+v"(prow_o));
#pragma unroll
        for (int ps = 0; ps < NSP; ++ps) {
            offnext[ps] = 0u;
            if (ps < nsp) {
                const Pix px = pixel(ps * ppp + prow_o);
                if (px.active && pt < P) {
                    if (NCHW) {
                        // channel cx = dx, cx + 1 = dy of the point, from the hi-res tensor
                        // or from the low-res one it is a pixel shuffle / a nearest
                        // interpolation of (deform_tap.hpp: OffsetLayout)
                        const long cx = (long)n * 2 * G * P + 2L * ((long)g * P + pt);
                        const T *op;
                        long dy;
                        if (olayout == OFFSET_PIXEL_SHUFFLE) {
                            const int qh = px.pp / hW, qw = px.pp % hW;
                            op = offset + (cx * (S * S) + (qh % S) * S + qw % S) * lpix + (long)px.ph * W + px.pw;
                            dy = (long)(S * S) * lpix;
                        } else if (olayout == OFFSET_NEAREST) {
                            op = offset + cx * lpix + (long)px.ph * W + px.pw;
                            dy = lpix;
                        } else {
                            op = offset + cx * hpl + px.pp;
                            dy = hpl;
                        }
                        union { T h[2]; u32 u; } x;
                        x.h[0] = op[0];
                        x.h[1] = op[dy];
                        offnext[ps] = x.u;
                    } else {
                        offnext[ps] = *(const u32 *)(offset + px.hp * (2L * G * P) + 2L * ((long)g * P + pt));
                    }
                }
            }
        }
    };
    __shared__ int fb_flag;         // some point of the tile left the window (this group)

    stage_load_key(0);
    load_q(0);
    load_offsets(0);
    for (int g = 0; g < G; ++g) {
        // ---- (a) key window
        stage_store_key();
        stage_store_q();
        if (ovec) {
            // Ost[point][pixel][dx, dy]
            const int xy = tid & 1, row = (tid >> 1) & 3, opt = tid >> 3;
            union { u32x2 u; T h[4]; } x;
            x.u = u32x2{offnext[0], offnext[NSP > 1 ? 1 : 0]};
#pragma unroll
            for (int e = 0; e < 4; ++e) Ost[((opt * NPX) + row * 4 + e) * 2 + xy] = x.h[e];
        }
        if (tid == 0) fb_flag = 0;
        __syncthreads();
        // the group's first value chunk travels during the similarity and the sampling
        stage_load_value(g * cg, cv0);
        f32x2 off2[NSP];
#pragma unroll
        for (int ps = 0; ps < NSP; ++ps) {
            offraw[ps] = offnext[ps];
            if (ovec) offraw[ps] = ps < nsp ? ((const u32 *)Ost)[pt * NPX + ps * ppp + prow] : 0u;
            off2[ps] = widen_pair<T>(offraw[ps]);
        }

        // ---- (b) Sim = q . key over the window: this wave's blocks of 16 cells
        for (int nb = wave; nb < NCB; nb += 4) {
            u32x4 b[DP / 32];
#pragma unroll
            for (int ks = 0; ks < DP / 32; ++ks)
                b[ks] = *(const u32x4 *)(Xl + (16 * nb + mi) * KSB + 32 * ks + 8 * mk);
#pragma unroll
            for (int mb = 0; mb < NMB; ++mb) {
                f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < DP / 32; ++ks) {
                    const u32x4 a = NCHW ? *(const u32x4 *)(Ql + (16 * mb + mi) * QSB + 32 * ks + 8 * mk) : qa[NCHW ? 0 : mb][ks];
                    acc = Half<T>::mma(a, b[ks], acc);
                }
#pragma unroll
                for (int r = 0; r < 4; ++r) Sl[(16 * mb + 4 * mk + r) * WS + 16 * nb + mi] = acc[r];
            }
        }
        __syncthreads();

        // ---- (c) per (pixel, point): logit from Sim, softmax over the points,
        // attention-weighted corner weights into Wm.  A pixel's row of Sim / Wm is
        // touched by the lanes of that pixel only, all in one wave, whose LDS
        // operations run in program order: gathers, then the row is cleared,
        // then the adds, then the split -- no barrier in between.
        u32 fbmask = 0;             // pass ps: the point passes the guard but leaves the window
        float fatt[NSP];
        auto sample = [&](auto nl, int ps) __attribute__((always_inline)) {
            constexpr int NL = decltype(nl)::value;
            const int pi = ps * (NT / NL) + tid / NL;
            const Pix px = pixel(pi);
            const bool live = px.active && pt < P;
            const float kw = (float)px.pw + off2[ps][0], kh = (float)px.ph + off2[ps][1];
            const WinTap<float> t = win_tap<float>(kh, kw, H, W, wy0, wx0, WWY, WWX);
            const bool in = live && t.inwin;
            const bool fb = live && t.guard && !t.inwin;
            fbmask |= fb ? 1u << ps : 0u;
            const int cell = in ? t.hl * WWX + t.wl : 0;
            float *const srow = Sl + pi * WS;
            float lg = 0.f;
            if (in) {
                const float *sp = srow + cell;
                lg = t.w1 * sp[0];
                lg = fma_(t.w2, sp[1], lg);
                lg = fma_(t.w3, sp[WWX], lg);
                lg = fma_(t.w4, sp[WWX + 1], lg);
            }
            if (fb) {
                // sampled straight from global memory (rare)
                Tap<float> tp = {};
                tap_setup(kh, kw, H, W, tp);
                const T *kp = key + (long)n * lpix * Cq + g * d;
                const T *qp = NCHW ? q + ((long)n * Cq + g * d) * hpl + px.pp : q + px.hp * Cq + g * d;
                const long qcs = NCHW ? hpl : 1;        // from one channel of the pixel to the next
                for (int c = 0; c < d; ++c) {
                    const float v1 = tp.m1 ? (float)kp[(long)tp.i1 * Cq + c] : 0.f;
                    const float v2 = tp.m2 ? (float)kp[(long)tp.i2 * Cq + c] : 0.f;
                    const float v3 = tp.m3 ? (float)kp[(long)tp.i3 * Cq + c] : 0.f;
                    const float v4 = tp.m4 ? (float)kp[(long)tp.i4 * Cq + c] : 0.f;
                    float v = tp.w1 * v1;
                    v = fma_(tp.w2, v2, v);
                    v = fma_(tp.w3, v3, v);
                    v = fma_(tp.w4, v4, v);
                    lg = fma_(v, (float)qp[c * qcs], lg);
                }
            }
            // softmax over the pixel's points = the lanes pt < P of its group of NL lanes
            const float mx = reduce_lanes<true, NL>(pt < P ? lg : -__builtin_huge_valf());
            const float e = pt < P ? exp_(lg - mx) : 0.f;
            const float att = e * __builtin_amdgcn_rcpf(reduce_lanes<false, NL>(e));
            fatt[ps] = att;
            // a non-finite logit makes every weight of the pixel NaN, which the integer
            // entries of Wm cannot carry: such a point takes the per-sample path, where its
            // weight multiplies the sample in floating point like the reference's attn * val
            const bool nonfinite = live && t.guard && att != att;
            fbmask |= nonfinite ? 1u << ps : 0u;
            // the row becomes Wm: cleared, then the corners' shares as 2^30-scaled
            // integers (every entry and every row sum is at most 1; the rounding of
            // a contribution, 2^-31, is below that of an fp32 weight near 1)
            u32 *const wrow = SWl + pi * WS;
#pragma unroll
            for (int i4 = 0; i4 < (KP / 4 + NL - 1) / NL; ++i4)
                if (i4 * NL + pt < KP / 4) *(u32x4 *)(wrow + 4 * (i4 * NL + pt)) = u32x4{0u, 0u, 0u, 0u};
            if (in && !nonfinite) {
                u32 *wp = wrow + cell;
                const float sc = att * WSCALE;
                __hip_atomic_fetch_add(wp, (u32)fma_(sc, t.w1, 0.5f), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                __hip_atomic_fetch_add(wp + 1, (u32)fma_(sc, t.w2, 0.5f), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                __hip_atomic_fetch_add(wp + WWX, (u32)fma_(sc, t.w3, 0.5f), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                __hip_atomic_fetch_add(wp + WWX + 1, (u32)fma_(sc, t.w4, 0.5f), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            }
            // 8 entries (32 bytes) -> their 8 high parts, then their 8 remainders
#pragma unroll
            for (int i8 = 0; i8 < (KP / 8 + NL - 1) / NL; ++i8)
                if (i8 * NL + pt < KP / 8) {
                    u32x4 *blk = (u32x4 *)(wrow + 8 * (i8 * NL + pt));
                    u32x4 hi, lo;
                    split8<T>(blk[0], blk[1], hi, lo);
                    blk[0] = hi;
                    blk[1] = lo;
                }
        };
#pragma unroll
        for (int ps = 0; ps < NSP; ++ps) {
            if (narrow) {
                if (ps < NPX / 16) sample(std::integral_constant<int, 16>{}, ps);
            } else {
                sample(std::integral_constant<int, 32>{}, ps);
            }
        }

        // ---- (d) value chunks: out tile = Wm . value window (the key window is done with)
        stage_store_value();
        if (fbmask != 0) fb_flag = 1;
        if (g + 1 < G) load_offsets(g + 1);
        __syncthreads();
        const bool any_fb = fb_flag != 0;
        for (int vc = 0; vc < nVc; ++vc) {
            const int cbase = g * cg + vc * CHK;
            const int cvalid = cg - vc * CHK < CHK ? cg - vc * CHK : CHK;
            // next in line: the group's next value chunk, or the next group's key and q
            if (vc + 1 < nVc) {
                const int left = cg - (vc + 1) * CHK;
                stage_load_value(cbase + CHK, left < CHK ? left : CHK);
            } else if (g + 1 < G) {
                stage_load_key((g + 1) * d);
                load_q(g + 1);
            }
            if (16 * wave < cvalid) {
                // this wave: channels 16 wave .. + 15 of the chunk, all pixels
                f32x4 acch[NMB], accl[NMB];
#pragma unroll
                for (int mb = 0; mb < NMB; ++mb) acch[mb] = accl[mb] = f32x4{0.f, 0.f, 0.f, 0.f};
                // a transposing read: lane m of a 16-lane block addresses channels
                // 4 (m % 4) .. + 3 of cell m / 4 and receives channel m of those 4 cells
                const T *vt = Xl + (8 * mk + (mi >> 2)) * VSB + 16 * wave + 4 * (mi & 3);
#pragma unroll
                for (int ks = 0; ks < NKS; ++ks) {
                    union { s16x4 h[2]; u32x4 u; } b;
                    b.h[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (s16x4 __attribute__((address_space(3))) *)(vt + (32 * ks) * VSB));
                    b.h[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (s16x4 __attribute__((address_space(3))) *)(vt + (32 * ks + 4) * VSB));
#pragma unroll
                    for (int mb = 0; mb < NMB; ++mb) {
                        const u32x4 *ap = (const u32x4 *)(SWl + (16 * mb + mi) * WS + 32 * ks + 8 * mk);
                        acch[mb] = Half<T>::mma(ap[0], b.u, acch[mb]);
                        accl[mb] = Half<T>::mma(ap[1], b.u, accl[mb]);
                    }
                }
#pragma unroll
                for (int mb = 0; mb < NMB; ++mb)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        Ol[(16 * mb + 4 * mk + r) * OS + 16 * wave + mi] = (acch[mb][r] + accl[mb][r]) * Half<T>::OUT_SCALE;
            }
            __syncthreads();
            if (any_fb) {
                // points outside the window add their sample to the tile (rare)
#pragma unroll
                for (int ps = 0; ps < NSP; ++ps) {
                    if (!(fbmask >> ps & 1)) continue;
                    const int pi = ps * ppp + prow;
                    const Pix px = pixel(pi);
                    // (opaque to the compiler, which would otherwise set these taps up
                    // ahead of the branch, for every tile)
                    u32 raw = offraw[ps];
                    asm volatile("" : "+v"(raw));
                    const f32x2 o2 = widen_pair<T>(raw);
                    Tap<float> tp = {};
                    tap_setup((float)px.ph + o2[1], (float)px.pw + o2[0], H, W, tp);
                    const T *vp = value + (long)n * lpix * C + cbase;
                    for (int c = 0; c < cvalid; ++c) {
                        const float v1 = tp.m1 ? (float)vp[(long)tp.i1 * C + c] : 0.f;
                        const float v2 = tp.m2 ? (float)vp[(long)tp.i2 * C + c] : 0.f;
                        const float v3 = tp.m3 ? (float)vp[(long)tp.i3 * C + c] : 0.f;
                        const float v4 = tp.m4 ? (float)vp[(long)tp.i4 * C + c] : 0.f;
                        float v = tp.w1 * v1;
                        v = fma_(tp.w2, v2, v);
                        v = fma_(tp.w3, v3, v);
                        v = fma_(tp.w4, v4, v);
                        __hip_atomic_fetch_add(Ol + pi * OS + c, fatt[ps] * v, __ATOMIC_RELAXED,
                                               __HIP_MEMORY_SCOPE_WORKGROUP);
                    }
                }
                __syncthreads();
            }
            if (NCHW) {
                // a thread stores one row of the tile in one channel plane: TW
                // contiguous pixels.  Plain stores: the rest of each line comes from
                // the neighbouring tiles, and the L2 puts the pieces together.
                static_assert(TW == 4 || TW == 8, "a tile row is one 8- or 16-byte store");
                typedef u32 RowVec __attribute__((ext_vector_type(TW / 2)));
                const bool ovec = hW % TW == 0 && (uintptr_t)out % (TW * sizeof(T)) == 0;
#pragma unroll
                for (int it = 0; it < (CHK * TH + NT - 1) / NT; ++it) {
                    const int item = it * NT + tid;
                    const int ch = item / TH, row = item % TH;
                    if ((CHK * TH) % NT != 0 && item >= CHK * TH) break;
                    const int qh = y0 + row;
                    if (ch < cvalid && qh < hH) {
                        union { T h[TW]; RowVec v; } x;
#pragma unroll
                        for (int e = 0; e < TW; ++e) x.h[e] = (T)Ol[(row * TW + e) * OS + ch];
                        T *op = out + ((long)n * C + cbase + ch) * hpl + (long)qh * hW + x0;
                        if (ovec && x0 + TW <= hW) {
                            *(RowVec *)op = x.v;
                        } else {
#pragma unroll
                            for (int e = 0; e < TW; ++e)
                                if (x0 + e < hW) op[e] = x.h[e];
                        }
                    }
                }
            } else {
                // 8 lanes store a pixel's 64 channels: 128 contiguous bytes
#pragma unroll
                for (int sp = 0; sp < (NPX + 31) / 32; ++sp) {
                    const int pi = sp * 32 + tid / 8;
                    if (NPX % 32 != 0 && pi >= NPX) break;
                    const Pix px = pixel(pi);
                    if (px.active && 8 * c8 < cvalid) {
                        const f32x4 *op = (const f32x4 *)(Ol + pi * OS + 8 * c8);
                        __builtin_nontemporal_store(narrow8<T>(op[0], op[1]), (u32x4 *)(out + px.hp * C + cbase + 8 * c8));
                    }
                }
            }
            if (vc + 1 < nVc) {
                __syncthreads();        // everyone is done with this chunk's window and tile
                stage_store_value();
                __syncthreads();
            }
        }
    }
}

template <typename T, int S, int TH, int TW, int DP, bool NCHW>
static hipError_t launch_tile(const void *q, const void *key, const void *value, const void *offset,
                              void *out, int B, int Cq, int C, int H, int W, int P, int G,
                              hipStream_t st, int olayout) {
    const int tiles_x = (W * S + TW - 1) / TW, tiles_y = (H * S + TH - 1) / TH;
    const long nb = (long)tiles_x * tiles_y * B;
    if (nb > (1L << 30)) return hipErrorNotSupported;
    const int per_xcd = (int)((nb + 7) / 8);
    hipLaunchKernelGGL((deform_fused_wmat16_kernel<T, S, TH, TW, DP, NCHW>), dim3(per_xcd * 8), dim3(NT), 0, st,
                       (const T *)q, (const T *)key, (const T *)value, (const T *)offset, (T *)out,
                       Cq, C, H, W, P, G, tiles_x, tiles_y, (int)nb, per_xcd, olayout);
    return hipGetLastError();
}

#ifndef SAPA_WM16_TILE
#define SAPA_WM16_TILE 4, 4
#endif

template <typename T, bool NCHW>
static hipError_t launch_t(const void *q, const void *key, const void *value, const void *offset,
                           void *out, int B, int Cq, int C, int H, int W, int P, int s, int G,
                           hipStream_t st, int olayout) {
    const int d = Cq / G;
#define SAPA_WM16(SV)                                                                                  \
    case SV:                                                                                           \
        return d <= 32 ? launch_tile<T, SV, SAPA_WM16_TILE, 32, NCHW>(q, key, value, offset, out, B, Cq, C, H, W, P, G, st, olayout) \
                       : launch_tile<T, SV, SAPA_WM16_TILE, 64, NCHW>(q, key, value, offset, out, B, Cq, C, H, W, P, G, st, olayout);
    switch (s) {
        SAPA_WM16(1) SAPA_WM16(2) SAPA_WM16(4)
        default: return hipErrorNotSupported;
    }
#undef SAPA_WM16
}

}  // namespace dwm16

// f16 / bf16 tensors, s in {1, 2, 4}, P <= 32, channels per group (Cq / G and
// C / G) multiples of 8, Cq / G <= 64, one image's key / value tensor below 2^31
// bytes.  key and value in channels-last order, aligned to 16 bytes; query, offset
// and out either channels-last too (query and out aligned to 16 bytes, offset to
// 4) or, nchw = true, contiguous [B, channels, sH, sW] with one plane below 2^31
// elements, the offsets in the layout olayout names (deform_tap.hpp).
// hipErrorNotSupported otherwise.
hipError_t deform_fused_wmat16_launch(const void *q, const void *key, const void *value,
                                      const void *offset, void *out, int B, int Cq, int C, int H,
                                      int W, int P, int s, int G, int dtype, hipStream_t st, bool nchw, int olayout) {
    if (dtype != 2 && dtype != 3) return hipErrorNotSupported;
    if (P > 32 || (Cq / G) % 8 != 0 || Cq / G > 64 || (C / G) % 8 != 0) return hipErrorNotSupported;
    const long plane = (long)H * W * 2;
    if (plane * Cq >= (1L << 31) || plane * C >= (1L << 31)) return hipErrorNotSupported;
    if ((uintptr_t)key % 16 != 0 || (uintptr_t)value % 16 != 0) return hipErrorNotSupported;
    if (nchw) {
        // the pixel index within a plane and the row stores use 32-bit arithmetic
        if ((long)H * s * W * s >= (1L << 31)) return hipErrorNotSupported;
        return dtype == 2 ? dwm16::launch_t<f16_t, true>(q, key, value, offset, out, B, Cq, C, H, W, P, s, G, st, olayout)
                          : dwm16::launch_t<bf16_t, true>(q, key, value, offset, out, B, Cq, C, H, W, P, s, G, st, olayout);
    }
    if ((uintptr_t)q % 16 != 0 || (uintptr_t)out % 16 != 0 || (uintptr_t)offset % 4 != 0) return hipErrorNotSupported;
    return dtype == 2 ? dwm16::launch_t<f16_t, false>(q, key, value, offset, out, B, Cq, C, H, W, P, s, G, st, OFFSET_HIRES)
                      : dwm16::launch_t<bf16_t, false>(q, key, value, offset, out, B, Cq, C, H, W, P, s, G, st, OFFSET_HIRES);
}

}  // namespace sapa
