// Backward of the fused SAPA-D operator, everything that is per high-res pixel,
// in one kernel and in the matrix form of the forward kernel (sapa_d_nhwc.hip):
//
//   attention weights   att = softmax_p( sampled key . q )            (recomputed)
//   grad of the weights gat[p] = grad_out . sampled value
//   grad of the logits  gl[p]  = att[p] * (gat[p] - sum_p' att[p'] gat[p'])
//   grad_offset[p]      = att[p] * d(gat[p]) / d(position) + gl[p] * d(logit[p]) / d(position)
//   grad_query          = sum_p gl[p] * sampled key
//
// which the separate kernels compute in five launches of per-pixel gathers
// (deform_qk / deform_av forward and backward with swapped roles,
// deformsapa/deformsapa/src/cuda/deform_qk_cuda_kernel.cu:70-137 and
// deform_av_cuda_kernel.cu:70-137; autograd's softmax backward between them).
// Per 4 x 4-pixel tile and group, with the window of the tile's parents +- RCH
// cells (+ the high corners' cell) in LDS:
//
//   G'  [pixel][cell] = grad_out[pixel] . value[cell]      (16 x KP x cg, matrix pipe)
//   Sim [pixel][cell] = q[pixel] . key[cell]               (16 x KP x d,  matrix pipe)
//   per (pixel, point): the four corners' entries of Sim and G' give the logit,
//     gat and both position derivatives (the bilinear weights' derivatives times
//     the same four entries); softmax and its backward run across the lanes
//   Wg  [pixel][cell] += gl[p] * corner weight              (integer LDS adds)
//   grad_query tile   = Wg . key window                     (16 x KP x d,  matrix pipe)
//
// att and gl go to a workspace as fp32 [B, G, P, sH, sW] tensors: the low-res
// gradients (grad_value from att and grad_out, grad_key from gl and q) are the
// scatter kernels' work.  Sums run per window cell instead of per point and
// channel: results agree with the reference's order to fp32 rounding.
// Points that pass the guard but leave the window take their eight corner
// products from global memory.  q, grad_out, offset, grad_query, grad_offset are
// contiguous [B, channels, sH, sW]; key and value are channels-last copies.
#include "deform_quad.hpp"
#include "deform_tap.hpp"
#include "kernels.hpp"

namespace sapa {

namespace dbm {

using dnhwc::f32x2;
using dnhwc::f32x4;
using dnhwc::Quad;
using dnhwc::u32;
using dnhwc::u32x4;

constexpr int RCH = 4;          // window reach around the tile's parents, in low-res cells
constexpr int TPW = 4;          // tile edge, hi-res pixels

template <typename T, int S, int DP>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3, 3)))
deform_bwd_wmat_kernel(const T *__restrict__ grad_out, const T *__restrict__ q,
                       const T *__restrict__ key, const T *__restrict__ value,
                       const T *__restrict__ offset, float *__restrict__ attn_ws,
                       float *__restrict__ gl_ws, T *__restrict__ grad_q, T *__restrict__ grad_offset,
                       int Cq, int C, int H, int W, int P, int G, int tiles_x, int tiles_y,
                       int nblocks, int per_xcd) {
    constexpr int TPL = (TPW + S - 1) / S;                   // parents of a tile per axis
    constexpr int WW = TPL + 2 * RCH + 1, NPOS = WW * WW;    // window cells
    constexpr int KP = (NPOS + 15) / 16 * 16, NKB = KP / 16; // cells padded to blocks of 16
    constexpr int CHK = 64;                                  // value channels per chunk
    constexpr int VS = CHK + 4;     // row strides in floats: 4 mod 16, so that the four
    constexpr int KS = DP + 4;      // k-quarters of a matrix operand read disjoint banks
    constexpr int WS = KP + 4;
    constexpr int QS = DP + 4;                               // floats per pixel of the q / grad_query tile
    constexpr int NPX = TPW * TPW;                           // pixels of a tile
    constexpr int NT = 256, NPASS = (NPOS * 16 + NT - 1) / NT;
    constexpr int NBW = (NKB + 3) / 4;                       // cell blocks per wave (block nb: wave nb % 4)
    constexpr int NCB = DP / 16, KSPL = 4 / NCB;             // grad_query: channel blocks, shares of the cells
    constexpr int KPER = (NKB + KSPL - 1) / KSPL;            // cell blocks per share
    constexpr float WSCALE = 1073741824.f;                   // 2^30: fixed-point scale of Wg
    static_assert(NPX == 16 && WS >= VS && KS <= VS, "one block of 16 matrix rows; shared buffers");
    static_assert(NPASS * (NT / 16) == KP, "the staging passes cover the padded window exactly");
    static_assert(KSPL * NPX * QS <= NPX * WS, "grad_query partial tiles fit");
    typedef Quad<T> Q4;
    typedef typename Q4::raw Raw;

    // the value window [cell][VS] (G'), then the key window [cell][KS] (Sim, grad_query)
    __shared__ __attribute__((aligned(16))) float Xl[KP * VS];
    // the grad_out tile [pixel][VS]; the q tile [pixel][QS]; Sim [pixel][cell]; the grad_query tile(s)
    __shared__ __attribute__((aligned(16))) float Sl[NPX * WS];
    // G' [pixel][cell]; then Wg [pixel][cell], integers scaled per pixel
    __shared__ __attribute__((aligned(16))) float Gl[NPX * WS];
    __shared__ float invl[NPX];     // Wg row -> floats
    __shared__ int fb_flag;         // some point of the tile left the window (this group)

    const int logical = (int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8);
    if (logical >= nblocks) return;
    const int tx = logical % tiles_x;
    const int ty = (logical / tiles_x) % tiles_y;
    const int n = logical / (tiles_x * tiles_y);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int hH = H * S, hW = W * S;
    const int y0 = ty * TPW, x0 = tx * TPW;                          // tile origin, hi-res
    const int wy0 = y0 / S - RCH, wx0 = x0 / S - RCH;                // window origin, low-res cell
    const long lpix = (long)H * W, hpl = (long)hH * hW;
    const int d = Cq / G, cg = C / G;
    const int nVc = (cg + CHK - 1) / CHK;

    struct Pix { bool active; int pp, ph, pw; };
    auto pixel = [&](int i) __attribute__((always_inline)) {
        const int qh = y0 + i / TPW, qw = x0 + i % TPW;
        Pix r;
        r.active = qh < hH && qw < hW;
        const int ch = qh < hH ? qh : hH - 1, cw = qw < hW ? qw : hW - 1;
        r.pp = ch * hW + cw;
        r.ph = ch / S;
        r.pw = cw / S;
        return r;
    };
    // view 1: a row of 16 lanes per pixel (window staging; a lane per point for P <= 16)
    const int srow = tid >> 4, sq = tid & 15;
    const Pix spx = pixel(srow);
    // view 2: matrix operands
    const int mi = lane & 15, mk = lane >> 4;
    // view 3: half a wave per pixel (two passes over the tile), a lane per point
    const int half = tid >> 5, pl = tid & 31;
    const Pix bpx[2] = {pixel(half), pixel(8 + half)};
    // view 4: a thread per (channel, tile row): 4 contiguous pixels of a channel plane
    const int tch = tid / TPW, trow = tid % TPW;
    // tile rows are whole aligned vectors
    const bool hvec = hW % TPW == 0 &&
                      ((uintptr_t)grad_out | (uintptr_t)q | (uintptr_t)grad_q) % sizeof(typename Quad<T>::raw) == 0;

    // ---- window staging (as the forward kernel): pass p, thread t moves channel
    // quad t % 16 of window cell p * 16 + t / 16; 2^31 = zero fill
    const int cv0 = cg < CHK ? cg : CHK;
    // (the cell's pixel index, negative outside the image and for the padding
    // cells; the byte offsets are put together at the loads: fewer registers)
    int cpix[NPASS];
#pragma unroll
    for (int p = 0; p < NPASS; ++p) {
        const int pos = p * (NT / 16) + tid / 16;
        const int gy = wy0 + pos / WW, gx = wx0 + pos % WW;
        const bool ok = pos < NPOS && gy >= 0 && gy < H && gx >= 0 && gx < W;
        cpix[p] = ok ? gy * W + gx : -1;
    }
    const __amdgpu_buffer_rsrc_t krsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(key + (long)n * lpix * Cq), 0, (int)(lpix * Cq * (long)sizeof(T)), 0x00020000);
    const __amdgpu_buffer_rsrc_t vrsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(value + (long)n * lpix * C), 0, (int)(lpix * C * (long)sizeof(T)), 0x00020000);
    Raw st[NPASS];
    // channels cbase .. cbase + cvalid of the key (is_key) or value window
    auto stage_load = [&](bool is_key, int cbase, int cvalid) __attribute__((always_inline)) {
        const u32 soff = (u32)cbase * (u32)sizeof(T);
        const int nch = is_key ? Cq : C;
        // bit 31 = past the descriptor: the quad lies beyond the chunk's channels
        const u32 qbad = (u32)(cvalid - 1 - 4 * sq) & 0x80000000u;
#pragma unroll
        for (int p = 0; p < NPASS; ++p) {
            int cp = cpix[p];
            asm volatile("" : "+v"(cp));    // (or the offsets of both tensors are kept in registers throughout)
            const u32 off = ((u32)(cp * nch + 4 * sq) * (u32)sizeof(T)) | ((u32)cp & 0x80000000u) | qbad;
            st[p] = is_key ? Q4::buffer_load(krsrc, off, soff) : Q4::buffer_load(vrsrc, off, soff);
        }
    };
    float *const xrow = Xl + 4 * sq;
    auto stage_store = [&](int stride, int nquads) __attribute__((always_inline)) {
        if (sq < nquads) {
            float *dst = xrow + (tid / 16) * stride;
#pragma unroll
            for (int p = 0; p < NPASS; ++p) *(f32x4 *)(dst + p * (NT / 16) * stride) = Q4::widen(st[p]);
        }
    };
    // ---- hi-res tiles: 16 pixels x up to 64 channel planes of q or grad_out, a
    // thread fetching one tile row (4 x-neighbours) of one plane; zeros for
    // channels past nch and rows / columns past the image
    // (addresses are worked out at each use from opaque copies of the thread's
    // indices: hoisted out of the loops as 64-bit pointers they are spilled, and
    // the spill stores of every workgroup are memory traffic)
    auto load_tile_row = [&](const T *base, int nch) __attribute__((always_inline)) {
        Raw r = Raw{};
        int tch_o = tch, trow_o = trow;
        asm volatile("" : "+v"(tch_o), "+v"(trow_o));
        const int qh = y0 + trow_o;
        if (tch_o < nch && qh < hH) {
            const T *p = base + (long)tch_o * hpl + (long)qh * hW + x0;
            if (hvec) {
                r = *(const Raw *)p;
            } else {
                union { T h[4]; Raw r; } x;
                x.r = Raw{};
#pragma unroll
                for (int e = 0; e < TPW; ++e)
                    if (x0 + e < hW) x.h[e] = p[e];
                r = x.r;
            }
        }
        return r;
    };
    // into LDS as [pixel][stride], channels tch < nrows
    auto store_tile_row = [&](Raw r, int stride, int nrows) __attribute__((always_inline)) {
        if (tch < nrows) {
            const f32x4 v = Q4::widen(r);
#pragma unroll
            for (int e = 0; e < TPW; ++e) Sl[(trow * TPW + e) * stride + tch] = v[e];
        }
    };
    const T *const go_n = grad_out + (long)n * C * hpl;
    const T *const q_n = q + (long)n * Cq * hpl;
    const T *const off_n = offset + (long)n * 2 * G * P * hpl;

    Raw gorow, qrow = Raw{};
    stage_load(false, 0, cv0);
    gorow = load_tile_row(go_n, cv0);
    for (int g = 0; g < G; ++g) {
        // ---- (a) G' = grad_out . value over the window, chunk by chunk
        f32x4 gacc[NBW];
#pragma unroll
        for (int i = 0; i < NBW; ++i) gacc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
        for (int vc = 0; vc < nVc; ++vc) {
            stage_store(VS, 16);
            store_tile_row(gorow, VS, CHK);
            __syncthreads();
            // next in line: the group's next value chunk, or its key window and q
            if (vc + 1 < nVc) {
                const int left = cg - (vc + 1) * CHK;
                stage_load(false, g * cg + (vc + 1) * CHK, left < CHK ? left : CHK);
                gorow = load_tile_row(go_n + (long)(g * cg + (vc + 1) * CHK) * hpl, left < CHK ? left : CHK);
            } else {
                stage_load(true, g * d, d);
                qrow = load_tile_row(q_n + (long)(g * d) * hpl, d);
            }
#pragma unroll
            for (int s16 = 0; s16 < CHK / 16; ++s16) {
                const f32x4 a4 = *(const f32x4 *)(Sl + mi * VS + 16 * s16 + 4 * mk);
#pragma unroll
                for (int i = 0; i < NBW; ++i) {
                    if (NKB % 4 != 0 && wave + 4 * i >= NKB) continue;
                    const f32x4 b4 = *(const f32x4 *)(Xl + (16 * (wave + 4 * i) + mi) * VS + 16 * s16 + 4 * mk);
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        gacc[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[r], b4[r], gacc[i], 0, 0, 0);
                }
            }
            __syncthreads();
        }
#pragma unroll
        for (int i = 0; i < NBW; ++i) {
            if (NKB % 4 != 0 && wave + 4 * i >= NKB) continue;
#pragma unroll
            for (int r = 0; r < 4; ++r) Gl[(4 * mk + r) * WS + 16 * (wave + 4 * i) + mi] = gacc[i][r];
        }

        // ---- (b) Sim = q . key over the window
        stage_store(KS, DP / 4);
        store_tile_row(qrow, QS, DP);
        if (tid == 0) fb_flag = 0;
        __syncthreads();
        // the offsets travel meanwhile
        const bool narrow = P <= 16;
        f32x2 off2[2] = {f32x2{0.f, 0.f}, f32x2{0.f, 0.f}};
        auto load_offset = [&](const Pix &px, int pt) __attribute__((always_inline)) {
            int pp = px.pp;
            asm volatile("" : "+v"(pp));
            const T *op = off_n + 2L * ((long)g * P + pt) * hpl + pp;
            return f32x2{(float)op[0], (float)op[hpl]};
        };
        if (narrow) {
            if (spx.active && sq < P) off2[0] = load_offset(spx, sq);
        } else {
#pragma unroll
            for (int ps = 0; ps < 2; ++ps)
                if (bpx[ps].active && pl < P) off2[ps] = load_offset(bpx[ps], pl);
        }
        {
            f32x4 a4[DP / 16];
#pragma unroll
            for (int s16 = 0; s16 < DP / 16; ++s16) a4[s16] = *(const f32x4 *)(Sl + mi * QS + 16 * s16 + 4 * mk);
            __syncthreads();        // every wave has its operands: the buffer takes Sim
#pragma unroll
            for (int i = 0; i < NBW; ++i) {
                const int nb = wave + 4 * i;
                if (NKB % 4 != 0 && nb >= NKB) continue;
                f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int s16 = 0; s16 < DP / 16; ++s16) {
                    const f32x4 b4 = *(const f32x4 *)(Xl + (16 * nb + mi) * KS + 16 * s16 + 4 * mk);
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[s16][r], b4[r], acc, 0, 0, 0);
                }
#pragma unroll
                for (int r = 0; r < 4; ++r) Sl[(4 * mk + r) * WS + 16 * nb + mi] = acc[r];
            }
        }
        __syncthreads();

        // ---- (c) per (pixel, point)
        struct Smp {
            float gl, w1, w2, w3, w4, kh, kw;
            int cell;
            bool in, fb;
        };
        Smp sm[2] = {};
        float l1[2] = {0.f, 0.f};
        auto sample = [&](auto nl, int ps, int pi, const Pix &px, int pt) __attribute__((always_inline)) {
            constexpr int NL = decltype(nl)::value;
            asm volatile("" : "+v"(pi));        // (its LDS rows' addresses: not kept across the groups)
            const bool live = px.active && pt < P;
            const float kw = (float)px.pw + off2[ps][0], kh = (float)px.ph + off2[ps][1];
            const bool guard = kh > -1.f && kh < (float)H && kw > -1.f && kw < (float)W;
            const float fh = floor_(kh), fw = floor_(kw);
            const int hl = (int)fh - wy0, wl = (int)fw - wx0;
            const bool inwin = guard && hl >= 0 && hl <= WW - 2 && wl >= 0 && wl <= WW - 2;
            const float lh = kh - fh, lw = kw - fw, hh = 1.f - lh, hw = 1.f - lw;
            Smp &m = sm[ps];
            m.in = live && inwin;
            m.fb = live && guard && !inwin;
            m.kh = kh;
            m.kw = kw;
            m.cell = m.in ? hl * WW + wl : 0;
            const bool use = m.in || m.fb;
            m.w1 = use ? hh * hw : 0.f;
            m.w2 = use ? hh * lw : 0.f;
            m.w3 = use ? lh * hw : 0.f;
            m.w4 = use ? lh * lw : 0.f;
            // the four corners' entries of Sim (s) and of G' (v)
            float s1 = 0.f, s2 = 0.f, s3 = 0.f, s4 = 0.f, v1 = 0.f, v2 = 0.f, v3 = 0.f, v4 = 0.f;
            if (m.in) {
                const float *sp = Sl + pi * WS + m.cell, *gp = Gl + pi * WS + m.cell;
                s1 = sp[0], s2 = sp[1], s3 = sp[WW], s4 = sp[WW + 1];
                v1 = gp[0], v2 = gp[1], v3 = gp[WW], v4 = gp[WW + 1];
            }
            if (m.fb) {
                // the same eight products straight from global memory (rare; the
                // position is made opaque, so that its taps are set up in this branch only)
                float fkh = kh, fkw = kw;
                asm volatile("" : "+v"(fkh), "+v"(fkw));
                Tap<float> tp = {};
                tap_setup(fkh, fkw, H, W, tp);
                const T *kp = key + (long)n * lpix * Cq + g * d;
                const T *qp = q_n + (long)(g * d) * hpl + px.pp;
                for (int c = 0; c < d; ++c) {
                    const float x = (float)qp[c * hpl];
                    s1 = fma_(tp.m1 ? (float)kp[(long)tp.i1 * Cq + c] : 0.f, x, s1);
                    s2 = fma_(tp.m2 ? (float)kp[(long)tp.i2 * Cq + c] : 0.f, x, s2);
                    s3 = fma_(tp.m3 ? (float)kp[(long)tp.i3 * Cq + c] : 0.f, x, s3);
                    s4 = fma_(tp.m4 ? (float)kp[(long)tp.i4 * Cq + c] : 0.f, x, s4);
                }
                const T *vp = value + (long)n * lpix * C + g * cg;
                const T *gp = go_n + (long)(g * cg) * hpl + px.pp;
                for (int c = 0; c < cg; ++c) {
                    const float x = (float)gp[c * hpl];
                    v1 = fma_(tp.m1 ? (float)vp[(long)tp.i1 * C + c] : 0.f, x, v1);
                    v2 = fma_(tp.m2 ? (float)vp[(long)tp.i2 * C + c] : 0.f, x, v2);
                    v3 = fma_(tp.m3 ? (float)vp[(long)tp.i3 * C + c] : 0.f, x, v3);
                    v4 = fma_(tp.m4 ? (float)vp[(long)tp.i4 * C + c] : 0.f, x, v4);
                }
            }
            float lg = m.w1 * s1;
            lg = fma_(m.w2, s2, lg);
            lg = fma_(m.w3, s3, lg);
            lg = fma_(m.w4, s4, lg);
            // softmax over the pixel's points = the lanes pt < P of its group of NL lanes
            const float mx = reduce_lanes<true, NL>(pt < P ? lg : -__builtin_huge_valf());
            const float e = pt < P ? exp_(lg - mx) : 0.f;
            const float sum = reduce_lanes<false, NL>(e);
            float rs = __builtin_amdgcn_rcpf(sum);
            rs = fma_(fma_(-sum, rs, 1.f), rs, rs);
            const float att = e * rs;
            // its backward: gat = grad of the weight, gl = grad of the logit
            float gat = m.w1 * v1;
            gat = fma_(m.w2, v2, gat);
            gat = fma_(m.w3, v3, gat);
            gat = fma_(m.w4, v4, gat);
            const float dot = reduce_lanes<false, NL>(pt < P ? att * gat : 0.f);
            const float gl = att * (gat - dot);
            m.gl = pt < P ? gl : 0.f;
            l1[ps] = reduce_lanes<false, NL>(m.in ? __builtin_fabsf(gl) : 0.f);
            if (live) {
                int pp = px.pp;
                asm volatile("" : "+v"(pp));
                const long pidx = (((long)n * G + g) * P + pt) * hpl + pp;
                attn_ws[pidx] = att;
                gl_ws[pidx] = gl;
                if (grad_offset) {
                    // d / d(kw) and d / d(kh) of w1 x1 + w2 x2 + w3 x3 + w4 x4
                    // (deform_qk_cuda_kernel.cu:98-133), of the aggregation with the
                    // weight and of the logit with its gradient
                    float gw = 0.f, gh = 0.f;
                    if (use) {
                        const float dvw = -hh * v1 + hh * v2 - lh * v3 + lh * v4;
                        const float dvh = -hw * v1 - lw * v2 + hw * v3 + lw * v4;
                        const float dsw = -hh * s1 + hh * s2 - lh * s3 + lh * s4;
                        const float dsh = -hw * s1 - lw * s2 + hw * s3 + lw * s4;
                        gw = fma_(gl, dsw, att * dvw);
                        gh = fma_(gl, dsh, att * dvh);
                    }
                    T *op = grad_offset + ((long)n * 2 * G * P + 2L * ((long)g * P + pt)) * hpl + pp;
                    op[0] = (T)gw;
                    op[hpl] = (T)gh;
                }
            }
            if (grad_q) {
                // ---- (d) Wg[pixel][cell] += gl * corner weight, as integers scaled by
                // 2^30 / sum_p |gl| of the pixel: every partial sum stays within 2^30, the
                // adds are exact in any order and run at the rate of plain LDS writes.
                // Wg takes the place of G': the rows of this pass's pixels (NPP of them,
                // read and written by this wave only, whose LDS operations execute in
                // order) are emptied here, after the reads above.
                constexpr int NPP = 64 / NL;
                f32x4 *rows = (f32x4 *)(Gl + (pi - (lane / NL)) * WS);
                for (int i = lane; i < NPP * WS / 4; i += 64) rows[i] = f32x4{0.f, 0.f, 0.f, 0.f};
                const float sc = l1[ps] > 0.f ? WSCALE / l1[ps] : 0.f;
                // (a sum that is not finite reaches the result through this factor)
                if (pt == 0) invl[pi] = l1[ps] * (1.f / WSCALE);
                if (m.in) {
                    u32 *wp = (u32 *)Gl + pi * WS + m.cell;
                    const float x = gl * sc;
                    __hip_atomic_fetch_add(wp, (u32)(int)__builtin_rintf(x * m.w1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                    __hip_atomic_fetch_add(wp + 1, (u32)(int)__builtin_rintf(x * m.w2), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                    __hip_atomic_fetch_add(wp + WW, (u32)(int)__builtin_rintf(x * m.w3), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                    __hip_atomic_fetch_add(wp + WW + 1, (u32)(int)__builtin_rintf(x * m.w4), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                }
            }
        };
        if (narrow) {
            sample(std::integral_constant<int, 16>{}, 0, srow, spx, sq);
        } else {
            sample(std::integral_constant<int, 32>{}, 0, half, bpx[0], pl);
            sample(std::integral_constant<int, 32>{}, 1, 8 + half, bpx[1], pl);
        }
        if (sm[0].fb || (!narrow && sm[1].fb)) fb_flag = 1;
        // the next group's first value chunk travels during the rest
        if (g + 1 < G) {
            stage_load(false, (g + 1) * cg, cv0);
            gorow = load_tile_row(go_n + (long)((g + 1) * cg) * hpl, cv0);
        }
        if (grad_q) {
            __syncthreads();        // the rows of Wg are complete; Sim is done with
            // ---- (e) grad_query tile = Wg . key window: wave = (channel block, share of the cells)
            {
                const int cb = wave % NCB, ks = wave / NCB;
                const float inv = invl[mi];
                f32x4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int j = 0; j < KPER; ++j) {
                    const int s16 = ks * KPER + j;
                    if (NKB % KSPL != 0 && s16 >= NKB) continue;
                    const u32x4 ai = *(const u32x4 *)(Gl + mi * WS + 16 * s16 + 4 * mk);
                    const f32x4 a4 = {(float)(int)ai[0] * inv, (float)(int)ai[1] * inv,
                                      (float)(int)ai[2] * inv, (float)(int)ai[3] * inv};
                    const float *kp = Xl + (16 * s16 + 4 * mk) * KS + 16 * cb + mi;
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        if (r % 2 == 0) acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[r], kp[r * KS], acc0, 0, 0, 0);
                        else acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[r], kp[r * KS], acc1, 0, 0, 0);
                    }
                }
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    Sl[ks * NPX * QS + (4 * mk + r) * QS + 16 * cb + mi] = acc0[r] + acc1[r];
            }
            __syncthreads();
            if (fb_flag != 0) {
                // points outside the window add their share to the tile (rare)
#pragma unroll
                for (int ps = 0; ps < 2; ++ps) {
                    if (!sm[ps].fb) continue;
                    const int pi = narrow ? srow : ps * 8 + half;
                    // (opaque to the compiler, which would otherwise set these taps up
                    // ahead of the branch, for every tile)
                    float kh = sm[ps].kh, kw = sm[ps].kw;
                    asm volatile("" : "+v"(kh), "+v"(kw));
                    Tap<float> tp = {};
                    tap_setup(kh, kw, H, W, tp);
                    const T *kp = key + (long)n * lpix * Cq + g * d;
                    for (int c = 0; c < d; ++c) {
                        const float k1 = tp.m1 ? (float)kp[(long)tp.i1 * Cq + c] : 0.f;
                        const float k2 = tp.m2 ? (float)kp[(long)tp.i2 * Cq + c] : 0.f;
                        const float k3 = tp.m3 ? (float)kp[(long)tp.i3 * Cq + c] : 0.f;
                        const float k4 = tp.m4 ? (float)kp[(long)tp.i4 * Cq + c] : 0.f;
                        float v = tp.w1 * k1;
                        v = fma_(tp.w2, k2, v);
                        v = fma_(tp.w3, k3, v);
                        v = fma_(tp.w4, k4, v);
                        __hip_atomic_fetch_add(Sl + pi * QS + c, sm[ps].gl * v, __ATOMIC_RELAXED,
                                               __HIP_MEMORY_SCOPE_WORKGROUP);
                    }
                }
                __syncthreads();
            }
            // a thread stores one row of the tile in one channel plane
            const int qh = y0 + trow;
            if (tch < d && qh < hH) {
                f32x4 v;
#pragma unroll
                for (int e = 0; e < TPW; ++e) {
                    float x = Sl[(trow * TPW + e) * QS + tch];
#pragma unroll
                    for (int k = 1; k < KSPL; ++k) x += Sl[k * NPX * QS + (trow * TPW + e) * QS + tch];
                    v[e] = x;
                }
                union { T h[4]; Raw r; } x;
                x.r = Q4::narrow(v);
                T *op = grad_q + ((long)n * Cq + g * d + tch) * hpl + (long)qh * hW + x0;
                if (hvec) {
                    *(Raw *)op = x.r;
                } else {
#pragma unroll
                    for (int e = 0; e < TPW; ++e)
                        if (x0 + e < hW) op[e] = x.h[e];
                }
            }
        }
        __syncthreads();            // the buffers go back to the next group
    }
}

template <typename T, int S, int DP>
static hipError_t launch(const void *grad_out, const void *q, const void *key, const void *value,
                         const void *offset, float *attn_ws, float *gl_ws, void *grad_q,
                         void *grad_offset, int B, int Cq, int C, int H, int W, int P, int G,
                         hipStream_t st) {
    const int tiles_x = (W * S + TPW - 1) / TPW, tiles_y = (H * S + TPW - 1) / TPW;
    const long nb = (long)tiles_x * tiles_y * B;
    if (nb > (1L << 30)) return hipErrorNotSupported;
    const int per_xcd = (int)((nb + 7) / 8);
    hipLaunchKernelGGL((deform_bwd_wmat_kernel<T, S, DP>), dim3(per_xcd * 8), dim3(256), 0, st,
                       (const T *)grad_out, (const T *)q, (const T *)key, (const T *)value,
                       (const T *)offset, attn_ws, gl_ws, (T *)grad_q, (T *)grad_offset, Cq, C, H, W, P, G,
                       tiles_x, tiles_y, (int)nb, per_xcd);
    return hipGetLastError();
}

template <typename T>
static hipError_t launch_t(const void *grad_out, const void *q, const void *key, const void *value,
                           const void *offset, float *attn_ws, float *gl_ws, void *grad_q,
                           void *grad_offset, int B, int Cq, int C, int H, int W, int P, int s, int G,
                           hipStream_t st) {
    const int d = Cq / G;
#define SAPA_BWM(SV)                                                                                   \
    case SV:                                                                                           \
        return d <= 32 ? launch<T, SV, 32>(grad_out, q, key, value, offset, attn_ws, gl_ws, grad_q,    \
                                           grad_offset, B, Cq, C, H, W, P, G, st)                      \
                       : launch<T, SV, 64>(grad_out, q, key, value, offset, attn_ws, gl_ws, grad_q,    \
                                           grad_offset, B, Cq, C, H, W, P, G, st);
    switch (s) {
        SAPA_BWM(1)
        SAPA_BWM(2)
        SAPA_BWM(4)
        default: return hipErrorNotSupported;
    }
#undef SAPA_BWM
}

}  // namespace dbm

// Configurations the kernel serves: f32 / f16 / bf16, s in {1, 2, 4}, up to 32
// points, groups of whole channel quads with at most 64 query / key channels.
bool deform_bwd_wmat_serves(int B, int Cq, int C, int H, int W, int P, int s, int G, int dtype) {
    if (dtype != 0 && dtype != 2 && dtype != 3) return false;
    if (s != 1 && s != 2 && s != 4) return false;
    if (G <= 0 || Cq % G != 0 || C % G != 0 || P < 1 || P > 32) return false;
    const int d = Cq / G, cg = C / G;
    if (d % 4 != 0 || d > 64 || cg % 4 != 0) return false;
    const long plane = (long)H * W * (dtype == 0 ? 4 : 2);
    if (plane * Cq >= (1L << 31) || plane * C >= (1L << 31)) return false;
    if ((long)H * s * W * s >= (1L << 31)) return false;
    return true;
}

// key_cl, value_cl: channels-last copies [B, H, W, channels]; attn_ws, gl_ws: fp32
// [B, G, P, sH, sW]; grad_q and / or grad_offset may be NULL.
hipError_t deform_bwd_wmat_launch(const void *grad_out, const void *q, const void *key_cl,
                                  const void *value_cl, const void *offset, float *attn_ws,
                                  float *gl_ws, void *grad_q, void *grad_offset, int B, int Cq, int C,
                                  int H, int W, int P, int s, int G, int dtype, hipStream_t st) {
    if (!deform_bwd_wmat_serves(B, Cq, C, H, W, P, s, G, dtype)) return hipErrorNotSupported;
    switch (dtype) {
        case 0: return dbm::launch_t<float>(grad_out, q, key_cl, value_cl, offset, attn_ws, gl_ws, grad_q, grad_offset, B, Cq, C, H, W, P, s, G, st);
        case 2: return dbm::launch_t<f16_t>(grad_out, q, key_cl, value_cl, offset, attn_ws, gl_ws, grad_q, grad_offset, B, Cq, C, H, W, P, s, G, st);
        case 3: return dbm::launch_t<bf16_t>(grad_out, q, key_cl, value_cl, offset, attn_ws, gl_ws, grad_q, grad_offset, B, Cq, C, H, W, P, s, G, st);
        default: return hipErrorNotSupported;
    }
}

}  // namespace sapa
