// Fused SAPA-D forward (deform_qk -> softmax over the P points -> deform_av)
// for tensors in channels-last memory order: query [B, sH, sW, G*d], key
// [B, H, W, G*d], value [B, H, W, C], offset [B, sH, sW, 2*G*P] (channel
// 2(gP+p) = dx, +1 = dy), out [B, sH, sW, C].
//
// The contiguous-layout kernels (sapa_d_lds.hip) gather bilinear corners from
// an LDS window with one lane per pixel: 64 lanes read 64 unrelated addresses
// and the LDS bank conflicts of those gathers bound them.  Here the lanes run
// along the CHANNELS: a row of 16 lanes owns one (pixel, group) pair, lane i
// holds 4 channels, and a corner is read by the row as 256 contiguous bytes --
// no bank conflicts whatever the offsets are.
//
//   * a wave works on 4 hi-res pixels that are neighbours in x (a quad), a
//     workgroup of 4 waves on a 4 x 4-pixel tile (larger tiles: one wave takes
//     several quads in turn), one group at a time: the key window of
//     the group (the tile's parents + 4 cells of halo and the high corners'
//     extra cell, [position][64 channels] fp32) goes through LDS, then the value
//     window(s) of the group; the next chunk's global loads are in flight while
//     the current one is consumed;
//   * the sample positions are set up once per point, spread over the lanes:
//     lane l of a row computes the guard, the four bilinear weights and the
//     window address of points l and l + 16 of its pixel; the loops over the
//     points fetch them from that lane with DPP row broadcasts;
//   * logits: every lane accumulates its 4 channels' part of a point's
//     sampled-key . query product; 16 points at a time are then summed over the
//     16 lanes with a butterfly that leaves point 16 m + l in lane l -- the same
//     lane that holds its setup -- and the softmax runs across the row;
//   * aggregation: per point one broadcast of the weight, the usual
//     w1*v1 + w2*v2 + w3*v3 + w4*v4 in the reference's order, one FMA per
//     channel into 4 accumulators; a row stores 256 contiguous bytes.
//
// Index math, the strict guard (a point outside it has logit 0, takes part in
// the softmax and contributes nothing) and the per-corner zero padding follow
// deformsapa/deformsapa/src/cuda/deform_qk_cuda_kernel.cu:23-68,187: window
// cells outside the image hold zeros, a point whose guard fails reads a
// block of zeros with zero weights.  Points that pass the guard but leave the
// window (offsets beyond +-4 cells) are sampled from global memory.  The
// channel sums of the logits run in tree order (rounding-level differences
// from the reference's sequential sums); the aggregation keeps its order.
#include <utility>

#include "deform_quad.hpp"
#include "deform_tap.hpp"
#include "kernels.hpp"

namespace sapa {

namespace dnhwc {

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>)
template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// value of lane (l ^ D) of the same row of 16 lanes
template <int D>
__device__ __forceinline__ float row_xor(float v, int lane) {
    union { float f; int i; } x, y;
    x.f = v;
    if (D == 1) y.i = __builtin_amdgcn_mov_dpp(x.i, 0xB1, 0xf, 0xf, true);        // quad_perm [1,0,3,2]
    else if (D == 2) y.i = __builtin_amdgcn_mov_dpp(x.i, 0x4E, 0xf, 0xf, true);   // quad_perm [2,3,0,1]
    else y.i = __builtin_amdgcn_ds_bpermute((lane ^ D) << 2, x.i);
    return y.f;
}
// value of lane SRC of the own row of 16 lanes
template <int SRC>
__device__ __forceinline__ float row_bcast(float v) {
    union { float f; int i; } x, y;
    x.f = v;
    y.i = __builtin_amdgcn_mov_dpp(x.i, 0x150 + SRC, 0xf, 0xf, true);   // row_newbcast
    return y.f;
}
template <int SRC>
__device__ __forceinline__ int row_bcast(int v) {
    return __builtin_amdgcn_mov_dpp(v, 0x150 + SRC, 0xf, 0xf, true);
}

// One butterfly step over lane distance D: n values per lane -> n / 2; the
// lane whose bit D is clear keeps the even-indexed sums, its partner the odd
// (distances 4 and 8: two DPP additions per result, pair_sum_dpp -- the inputs
// here are always results of ordinary vector instructions).
template <int D, int N>
__device__ __forceinline__ void halve(const float (&in)[N], float (&out)[N / 2], int lane) {
    const bool hi = lane & D;
    (void)hi;
#pragma unroll
    for (int m = 0; m < N / 2; ++m) {
        const float a = in[2 * m], b = in[2 * m + 1];
        if constexpr (SAPA_NHWC_DPP_HALVE && (D == 4 || D == 8)) {
            out[m] = pair_sum_dpp<D>(a, b);
        } else {
            const float keep = hi ? b : a, send = hi ? a : b;
            out[m] = keep + row_xor<D>(send, lane);
        }
    }
}

constexpr int RCH = 4;          // window reach around the tile's parents, in low-res cells
constexpr int MAXSETS = 2;      // points are handled 16 at a time: P <= 32
constexpr u32 FALLBACK = 1u << 30;   // the point passes the guard but leaves the window

template <typename T, int S, int NQX, int NQY>
__global__ void __launch_bounds__(256)
deform_fused_nhwc_kernel(const T *__restrict__ q, const T *__restrict__ key,
                         const T *__restrict__ value, const T *__restrict__ offset,
                         T *__restrict__ out, int Cq, int C, int H, int W, int P, int G,
                         int tiles_x, int tiles_y, int nblocks, int per_xcd) {
    // tile: TPX x TPY hi-res pixels; a wave owns NQY pixel rows of NQX quads
    // (4 pixels in x) each and works through them one quad at a time
    constexpr int TPX = 4 * NQX, TPY = 4 * NQY, NQ = NQX * NQY;
    static_assert(TPX == TPY, "square tiles: one window extent");
    constexpr int TPL = (TPX + S - 1) / S;       // parents of a tile per axis
    constexpr int WW = TPL + 2 * RCH + 1, NPOS = WW * WW;   // window cells
    constexpr int CHK = 64;                      // channels per chunk: 16 lanes x 4
    constexpr int BUF = NPOS * CHK;              // floats of the window
    constexpr int ZERO = BUF;                    // then (WW + 2) cells of zeros
    constexpr int NT = 256, NPASS = (NPOS * 16 + NT - 1) / NT;
    typedef Quad<T> Q4;
    typedef typename Q4::raw Raw;

    __shared__ __attribute__((aligned(16))) float lds[BUF + (WW + 2) * CHK];

    const int logical = (int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8);
    if (logical >= nblocks) return;
    const int tx = logical % tiles_x;
    const int ty = (logical / tiles_x) % tiles_y;
    const int n = logical / (tiles_x * tiles_y);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int row = lane >> 4, li = lane & 15;
    const int hH = H * S, hW = W * S;
    // the pixel of this row of lanes in the wave's current quad (set_quad)
    bool active;
    int ph, pw;
    long hpixel;
    auto set_quad = [&](int qi) __attribute__((always_inline)) {
        const int qh = ty * TPY + wave * NQY + qi / NQX, qw = tx * TPX + 4 * (qi % NQX) + row;
        active = qh < hH && qw < hW;
        const int ch = qh < hH ? qh : hH - 1, cw = qw < hW ? qw : hW - 1;   // clamped for loads
        ph = ch / S;
        pw = cw / S;
        hpixel = (long)n * hH * hW + (long)ch * hW + cw;
    };
    const int wy0 = (ty * TPY) / S - RCH, wx0 = (tx * TPX) / S - RCH;   // window origin (low-res cell)
    const long lpix = (long)H * W;
    const int d = Cq / G, cg = C / G;
    const int nVc = (cg + CHK - 1) / CHK, nPer = 1 + nVc, ntot = G * nPer;
    const int nsets = (P + 15) / 16;

    for (int i = tid; i < (WW + 2) * CHK; i += NT) lds[ZERO + i] = 0.f;

    // ---- staging: pass p, thread t moves channel quad t % 16 of window cell
    // p * 16 + t / 16; -1 marks a cell outside the image (zero fill)
    int spix[NPASS];
#pragma unroll
    for (int p = 0; p < NPASS; ++p) {
        const int pos = p * (NT / 16) + tid / 16;
        const int gy = wy0 + pos / WW, gx = wx0 + pos % WW;
        spix[p] = (pos < NPOS && gy >= 0 && gy < H && gx >= 0 && gx < W) ? gy * W + gx : -1;
    }
    const int sq = tid & 15;
    // chunk j: group j / nPer; its key channels (j % nPer == 0) or value chunk j % nPer - 1
    auto chunk_of = [&](int j, bool &is_key, int &cbase, int &cvalid, int &nch) __attribute__((always_inline)) {
        const int g = j / nPer, r = j % nPer;
        is_key = r == 0;
        nch = is_key ? Cq : C;
        cbase = is_key ? g * d : g * cg + (r - 1) * CHK;     // first channel of the chunk
        const int left = is_key ? d : cg - (r - 1) * CHK;
        cvalid = left < CHK ? left : CHK;                    // channels of the chunk that exist
    };
    Raw st[NPASS];
    auto stage_load = [&](int j) __attribute__((always_inline)) {
        bool is_key;
        int cbase, cvalid, nch;
        chunk_of(j, is_key, cbase, cvalid, nch);
        const T *base = (is_key ? key : value) + (long)n * lpix * nch;
        const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(
            (void *)base, 0, (int)(lpix * nch * (long)sizeof(T)), 0x00020000);
        const bool c_ok = 4 * sq < cvalid;
#pragma unroll
        for (int p = 0; p < NPASS; ++p) {
            const u32 off = (c_ok && spix[p] >= 0)
                                ? (u32)(spix[p] * nch + cbase + 4 * sq) * (u32)sizeof(T)
                                : 0x80000000u;
            st[p] = Q4::buffer_load(r, off);
        }
    };
    auto stage_store = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int p = 0; p < NPASS; ++p) {
            const int pos = p * (NT / 16) + tid / 16;
            if (NPOS % (NT / 16) == 0 || pos < NPOS) *(f32x4 *)(lds + pos * CHK + 4 * sq) = Q4::widen(st[p]);
        }
    };

    // per point set m (points 16 m + li of this row's pixel): bilinear weights,
    // the LDS offset of the low corner (or of the zeros) with the FALLBACK
    // flag, the sample position for the fallback, the logit / attention weight
    float tw1[MAXSETS], tw2[MAXSETS], tw3[MAXSETS], tw4[MAXSETS], tkh[MAXSETS], tkw[MAXSETS];
    int tpk[MAXSETS];
    // the attention weights of the wave's quads wait in LDS between the key
    // chunk and the value chunks of a group (per thread: no synchronisation)
    __shared__ float att_keep[NQ][MAXSETS][NT];

    auto setup_points = [&](int g) __attribute__((always_inline)) {
        const T *op = offset + hpixel * (2L * G * P) + 2L * g * P;
#pragma unroll
        for (int m = 0; m < MAXSETS; ++m) {
            const int p = 16 * m + li;
            f32x2 o2 = {0.f, 0.f};
            if (m < nsets && p < P) o2 = Q4::load_pair(op + 2 * p);
            const float kw = (float)pw + o2[0], kh = (float)ph + o2[1];
            const WinTap<float> t = win_tap<float>(kh, kw, H, W, wy0, wx0, WW, WW);
            const bool live = m < nsets && p < P;
            const bool in = live && t.inwin;
            tw1[m] = in ? t.w1 : 0.f;
            tw2[m] = in ? t.w2 : 0.f;
            tw3[m] = in ? t.w3 : 0.f;
            tw4[m] = in ? t.w4 : 0.f;
            tkh[m] = kh;
            tkw[m] = kw;
            tpk[m] = (in ? (t.hl * WW + t.wl) * CHK : ZERO) |
                     ((live && t.guard && !t.inwin) ? (int)FALLBACK : 0);
        }
    };

    // w1*v1 + w2*v2 + w3*v3 + w4*v4 of this lane's 4 channels, left to right with FMAs
    auto sample_lds = [&](int pk, float w1, float w2, float w3, float w4,
                          float (&val)[4]) __attribute__((always_inline)) {
        const float *p0 = lds + (pk & 0xffffff) + 4 * li;
        const f32x4 v1 = *(const f32x4 *)p0, v2 = *(const f32x4 *)(p0 + CHK);
        const f32x4 v3 = *(const f32x4 *)(p0 + WW * CHK), v4 = *(const f32x4 *)(p0 + (WW + 1) * CHK);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            float v = w1 * v1[e];
            v = fma_(w2, v2[e], v);
            v = fma_(w3, v3[e], v);
            val[e] = fma_(w4, v4[e], v);
        }
    };
    // the same sample straight from global memory (the point left the window)
    auto sample_global = [&](const T *src, int nch, int cbase, int cvalid, float kh, float kw,
                             float (&val)[4]) __attribute__((always_inline)) {
        Tap<float> t = {};
        const bool ok = tap_setup(kh, kw, H, W, t) && 4 * li < cvalid;
        f32x4 v[4];
        const int idx[4] = {t.i1, t.i2, t.i3, t.i4};
        const bool msk[4] = {t.m1, t.m2, t.m3, t.m4};
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            Raw raw = Raw{};
            if (ok && msk[c])
                raw = *(const Raw *)(src + ((long)n * lpix + idx[c]) * nch + cbase + 4 * li);
            v[c] = Q4::widen(raw);
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            float x = t.w1 * v[0][e];
            x = fma_(t.w2, v[1][e], x);
            x = fma_(t.w3, v[2][e], x);
            val[e] = ok ? fma_(t.w4, v[3][e], x) : 0.f;
        }
    };

    // logits of the group's points from the key window in LDS
    auto qk_group = [&](int cbase, int cvalid, float (&att)[MAXSETS]) __attribute__((always_inline)) {
        f32x4 qv = {0.f, 0.f, 0.f, 0.f};
        if (active && 4 * li < cvalid)
            qv = Q4::widen(__builtin_nontemporal_load((const Raw *)(q + hpixel * Cq + cbase + 4 * li)));
#pragma unroll
        for (int m = 0; m < MAXSETS; ++m) {
            if (m >= nsets) {
                att[m] = 0.f;
                continue;
            }
            float part[16];
            static_for<16>([&](auto il) {
                constexpr int l = decltype(il)::value;
                part[l] = 0.f;
                if (16 * m + l < P) {
                    const int pk = row_bcast<l>(tpk[m]);
                    float val[4];
                    sample_lds(pk, row_bcast<l>(tw1[m]), row_bcast<l>(tw2[m]), row_bcast<l>(tw3[m]),
                               row_bcast<l>(tw4[m]), val);
                    if (pk & FALLBACK)
                        sample_global(key, Cq, cbase, cvalid, row_bcast<l>(tkh[m]),
                                      row_bcast<l>(tkw[m]), val);
                    float a = val[0] * qv[0];
#pragma unroll
                    for (int e = 1; e < 4; ++e) a = fma_(val[e], qv[e], a);
                    part[l] = a;
                }
            });
            float p1[8], p2[4], p3[2], p4[1];
            halve<1, 16>(part, p1, lane);
            halve<2, 8>(p1, p2, lane);
            halve<4, 4>(p2, p3, lane);
            halve<8, 2>(p3, p4, lane);
            att[m] = p4[0];                       // logit of point 16 m + li
        }
        // softmax over the P points of the pixel: across the row's lanes and sets
        bool okp[MAXSETS];
#pragma unroll
        for (int m = 0; m < MAXSETS; ++m) okp[m] = m < nsets && 16 * m + li < P;
        float mx = okp[0] ? att[0] : -__builtin_huge_valf();
#pragma unroll
        for (int m = 1; m < MAXSETS; ++m)
            if (okp[m]) mx = max_(mx, att[m]);
        mx = reduce_lanes<true, 16>(mx);      // (DPP steps: no exchange through LDS)
        float sum = 0.f;
#pragma unroll
        for (int m = 0; m < MAXSETS; ++m) {
            att[m] = okp[m] ? exp_(att[m] - mx) : 0.f;
            sum += att[m];
        }
        sum = reduce_lanes<false, 16>(sum);
        const float inv = 1.f / sum;
#pragma unroll
        for (int m = 0; m < MAXSETS; ++m) att[m] *= inv;
    };

    // one value chunk of the group: 64 output channels of this row's pixel
    auto av_chunk = [&](int cbase, int cvalid,
                        const float (&att)[MAXSETS]) __attribute__((always_inline)) {
        float o[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int m = 0; m < MAXSETS; ++m) {
            if (m >= nsets) continue;
            static_for<16>([&](auto il) {
                constexpr int l = decltype(il)::value;
                if (16 * m + l < P) {
                    const int pk = row_bcast<l>(tpk[m]);
                    const float wa = row_bcast<l>(att[m]);
                    float val[4];
                    sample_lds(pk, row_bcast<l>(tw1[m]), row_bcast<l>(tw2[m]), row_bcast<l>(tw3[m]),
                               row_bcast<l>(tw4[m]), val);
                    if (pk & FALLBACK)
                        sample_global(value, C, cbase, cvalid, row_bcast<l>(tkh[m]),
                                      row_bcast<l>(tkw[m]), val);
#pragma unroll
                    for (int e = 0; e < 4; ++e) o[e] = fma_(val[e], wa, o[e]);
                }
            });
        }
        if (active && 4 * li < cvalid)
            __builtin_nontemporal_store(Q4::narrow(f32x4{o[0], o[1], o[2], o[3]}),
                                        (Raw *)(out + hpixel * C + cbase + 4 * li));
    };

    stage_load(0);
    for (int j = 0; j < ntot; ++j) {
        stage_store();
        __syncthreads();
        if (j + 1 < ntot) stage_load(j + 1);
        bool is_key;
        int cbase, cvalid, nch;
        chunk_of(j, is_key, cbase, cvalid, nch);
        // the sample positions are set up again for every chunk (two points per
        // lane: cheap) rather than kept for all the wave's quads
#pragma unroll 1
        for (int qi = 0; qi < NQ; ++qi) {
            set_quad(qi);
            setup_points(j / nPer);
            float att[MAXSETS];
            if (is_key) {
                qk_group(cbase, cvalid, att);
#pragma unroll
                for (int m = 0; m < MAXSETS; ++m) att_keep[qi][m][tid] = att[m];
            } else {
#pragma unroll
                for (int m = 0; m < MAXSETS; ++m) att[m] = att_keep[qi][m][tid];
                av_chunk(cbase, cvalid, att);
            }
        }
        __syncthreads();
    }
}

// quads per tile row / pixel rows per wave: 1, 1 = 4 x 4-pixel tiles.  8 x 8
// tiles (2, 2) stage 2.9 x fewer window cells per pixel but leave room for two
// workgroups per CU instead of three and measured 25 % slower.
#ifndef SAPA_DNHWC_TILE
#define SAPA_DNHWC_TILE 1, 1
#endif
template <typename T, int S, int NQX, int NQY>
static hipError_t launch_geom(const void *q, const void *key, const void *value, const void *offset,
                           void *out, int B, int Cq, int C, int H, int W, int P, int G,
                           hipStream_t st) {
    const int tiles_x = (W * S + 4 * NQX - 1) / (4 * NQX), tiles_y = (H * S + 4 * NQY - 1) / (4 * NQY);
    const long nb = (long)tiles_x * tiles_y * B;
    if (nb > (1L << 30)) return hipErrorNotSupported;
    const int per_xcd = (int)((nb + 7) / 8);
    hipLaunchKernelGGL((deform_fused_nhwc_kernel<T, S, NQX, NQY>), dim3(per_xcd * 8), dim3(256), 0, st,
                       (const T *)q, (const T *)key, (const T *)value, (const T *)offset, (T *)out,
                       Cq, C, H, W, P, G, tiles_x, tiles_y, (int)nb, per_xcd);
    return hipGetLastError();
}

template <typename T>
static hipError_t launch_t(const void *q, const void *key, const void *value, const void *offset,
                           void *out, int B, int Cq, int C, int H, int W, int P, int s, int G,
                           hipStream_t st) {
    switch (s) {
        case 1: return launch_geom<T, 1, SAPA_DNHWC_TILE>(q, key, value, offset, out, B, Cq, C, H, W, P, G, st);
        case 2: return launch_geom<T, 2, SAPA_DNHWC_TILE>(q, key, value, offset, out, B, Cq, C, H, W, P, G, st);
        case 4: return launch_geom<T, 4, SAPA_DNHWC_TILE>(q, key, value, offset, out, B, Cq, C, H, W, P, G, st);
        default: return hipErrorNotSupported;
    }
}


// ---------------------------------------------------------------------------
// The same operator as two small matrix products per (tile, group).
//
// Every sample of a pixel lies within RCH cells of the pixel's parent (the
// few that do not are handled apart), so all 4 P corners of a pixel fall on the
// WW x WW window cells of its tile.  Writing the bilinear corner weights of a
// pixel as a row over those cells turns both sampled products into dense ones
// whose big operand -- the window -- is shared by all 16 pixels of the tile:
//
//   similarity  Sim[pixel][cell] = q[pixel] . key[cell]              (16 x KP x d)
//   logits      l[pixel][p]      = sum_corners w_c * Sim[pixel][cell_c]   (gather)
//   softmax over the P points of the pixel
//   weights     Wm[pixel][cell] += att_p * w_c                            (scatter)
//   output      out[pixel][ch]   = sum_cells Wm[pixel][cell] * value[cell][ch]
//                                                                    (16 x KP x 64)
//
// Both products run on v_mfma_f32_16x16x4f32.  A window cell is read from LDS
// once per 16-channel block and tile instead of once per sample and pixel,
// which takes the LDS traffic of the gather formulation above -- what bounds
// it -- down by more than an order of magnitude.  The sums run in another
// order than the reference's (per cell instead of per point): results agree to
// fp32 rounding.  All contributions to a row of Wm come from one wave, in
// program order, so the result does not depend on scheduling.
//
// Thread views of the 256 threads: a row of 16 lanes per pixel for staging q
// and storing the output (lane = 4 channels); the matrix instruction's
// (lane % 16, lane / 16) operand layout; half a wave per pixel, one lane per
// point, for the per-sample work.
constexpr int TPW = 4;          // tile edge, hi-res pixels
#ifndef SAPA_DNHWC_GATHER_MAXP
#define SAPA_DNHWC_GATHER_MAXP 7
#endif

// NCHW: query, offset and out are contiguous [B, channels, sH, sW] tensors (the
// reference's layout); key and value are channels-last either way (the launcher
// hands copies in that order to this kernel).
template <typename T, int S, int DP, bool NCHW>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3, 3)))
deform_fused_wmat_kernel(const T *__restrict__ q, const T *__restrict__ key,
                         const T *__restrict__ value, const T *__restrict__ offset,
                         T *__restrict__ out, int Cq, int C, int H, int W, int P, int G,
                         int tiles_x, int tiles_y, int nblocks, int per_xcd, int olayout) {
    constexpr int TPL = (TPW + S - 1) / S;                   // parents of a tile per axis
    constexpr int WW = TPL + 2 * RCH + 1, NPOS = WW * WW;    // window cells
    constexpr int KP = (NPOS + 15) / 16 * 16, NKB = KP / 16; // cells padded to blocks of 16
    constexpr int CHK = 64;                                  // value channels per chunk
    constexpr int VS = CHK + 4;     // row strides in floats: 4 mod 16, so that the four
    constexpr int KS = DP + 4;      // k-quarters of a matrix operand read disjoint banks
    constexpr int WS = KP + 4;
    constexpr int NPX = TPW * TPW;                           // pixels of a tile
    constexpr int NT = 256, NPASS = (NPOS * 16 + NT - 1) / NT;
    constexpr float WSCALE = 1073741824.f;                   // 2^30: fixed-point scale of Wm
    static_assert(NPX == 16 && WS >= VS && KS <= VS, "one block of 16 matrix rows; shared buffers");
    typedef Quad<T> Q4;
    typedef typename Q4::raw Raw;

    // the key window [cell][KS] (similarity), then the value window [cell][VS]
    __shared__ __attribute__((aligned(16))) float Xl[KP * VS];
    __shared__ __attribute__((aligned(16))) float Sl[NPX * WS];    // Sim [pixel][cell]; later the output tile [pixel][VS]
    __shared__ __attribute__((aligned(16))) float Wl[NPX * WS];    // Wm [pixel][cell], 2^30-scaled integers

    const int logical = (int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8);
    if (logical >= nblocks) return;
    const int tx = logical % tiles_x;
    const int ty = (logical / tiles_x) % tiles_y;
    const int n = logical / (tiles_x * tiles_y);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int hH = H * S, hW = W * S;
    const int y0 = ty * TPW, x0 = tx * TPW;                          // tile origin, hi-res
    const int wy0 = y0 / S - RCH, wx0 = x0 / S - RCH;                // window origin, low-res cell
    const long lpix = (long)H * W;
    const int d = Cq / G, cg = C / G;
    const int nVc = (cg + CHK - 1) / CHK;

    // pixel i of the tile (row-major 4 x 4): inside the image?  its flat hi-res
    // index, clamped for loads, and its parent
    struct Pix { bool active; long hp; int pp, ph, pw; };
    const long hpl = (long)hH * hW;                                  // a hi-res channel plane (NCHW)
    auto pixel = [&](int i) __attribute__((always_inline)) {
        const int qh = y0 + i / TPW, qw = x0 + i % TPW;
        Pix r;
        r.active = qh < hH && qw < hW;
        const int ch = qh < hH ? qh : hH - 1, cw = qw < hW ? qw : hW - 1;
        r.pp = ch * hW + cw;
        r.hp = (long)n * hH * hW + r.pp;
        r.ph = ch / S;
        r.pw = cw / S;
        return r;
    };
    // view 1: a row of 16 lanes per pixel (output stores, window staging)
    const int srow = tid >> 4, sq = tid & 15;
    const Pix spx = pixel(srow);
    // view 2: matrix operands
    const int mi = lane & 15, mk = lane >> 4;
    const Pix mpx = pixel(mi);
    // view 3: half a wave per pixel (two passes over the tile), a lane per point
    const int half = tid >> 5, pl = tid & 31;
    const Pix bpx[2] = {pixel(half), pixel(8 + half)};

    // ---- window staging: pass p, thread t moves channel quad t % 16 of window
    // cell p * 16 + t / 16.  Per-thread byte offsets of the key and the value
    // tensor, fixed for the whole kernel; 2^31 = beyond every descriptor, i.e.
    // zero fill: cells outside the image, the padding cells NPOS .. KP, channel
    // quads past the group's channels.  A chunk's first channel travels as the
    // instruction's scalar offset, so a load costs no address arithmetic.
    static_assert(NPASS * (NT / 16) == KP, "the staging passes cover the padded window exactly");
    const int cv0 = cg < CHK ? cg : CHK;                             // channels of a full value chunk
    u32 koff[NPASS], voff[NPASS];
#pragma unroll
    for (int p = 0; p < NPASS; ++p) {
        const int pos = p * (NT / 16) + tid / 16;
        const int gy = wy0 + pos / WW, gx = wx0 + pos % WW;
        const bool ok = pos < NPOS && gy >= 0 && gy < H && gx >= 0 && gx < W;
        const int pix = gy * W + gx;
        koff[p] = (ok && 4 * sq < d) ? (u32)(pix * Cq + 4 * sq) * (u32)sizeof(T) : 0x80000000u;
        voff[p] = (ok && 4 * sq < cv0) ? (u32)(pix * C + 4 * sq) * (u32)sizeof(T) : 0x80000000u;
    }
    const __amdgpu_buffer_rsrc_t krsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(key + (long)n * lpix * Cq), 0, (int)(lpix * Cq * (long)sizeof(T)), 0x00020000);
    const __amdgpu_buffer_rsrc_t vrsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(value + (long)n * lpix * C), 0, (int)(lpix * C * (long)sizeof(T)), 0x00020000);
    Raw st[NPASS];
    auto stage_load = [&](bool is_key, int cbase, int cvalid) __attribute__((always_inline)) {
        const u32 soff = (u32)cbase * (u32)sizeof(T);
        if (is_key) {
#pragma unroll
            for (int p = 0; p < NPASS; ++p) st[p] = Q4::buffer_load(krsrc, koff[p], soff);
        } else if (cvalid == cv0) {
#pragma unroll
            for (int p = 0; p < NPASS; ++p) st[p] = Q4::buffer_load(vrsrc, voff[p], soff);
        } else {
            // the ragged last chunk of a group
#pragma unroll
            for (int p = 0; p < NPASS; ++p)
                st[p] = Q4::buffer_load(vrsrc, 4 * sq < cvalid ? voff[p] : 0x80000000u, soff);
        }
    };
    // rows of `stride` floats; quads past `nquads` have no place in them
    float *const xrow = Xl + 4 * sq;
    auto stage_store = [&](int stride, int nquads) __attribute__((always_inline)) {
        if (sq < nquads) {
            float *dst = xrow + (tid / 16) * stride;
#pragma unroll
            for (int p = 0; p < NPASS; ++p) *(f32x4 *)(dst + p * (NT / 16) * stride) = Q4::widen(st[p]);
        }
    };
    // q of pixel mi as the A operand: channels 16 s + 4 mk .. + 3 of the group, s < DP / 16
    // Channels-last: 4 contiguous elements of global memory per lane.  Contiguous
    // layout: the tile's q (16 pixels x d channel planes) comes in once per workgroup,
    // a thread fetching one tile row (4 x-neighbours) of one plane, and goes through
    // LDS as [pixel][channel], from where every wave reads its operands.
    Raw qa[DP / 16];
    constexpr int QS = DP + 4;                                       // floats per pixel of the q tile
    static_assert(NPX * QS <= NPX * WS, "the q tile fits the weight matrix's buffer");
    float *const Ql = Wl;           // (contiguous layout) the q tile, until the similarity has its operands
    constexpr int QN = NCHW ? (TPW * DP + NT - 1) / NT : 1;          // tile rows per thread
    Raw qrow[QN];
    const bool qvec = hW % TPW == 0 && (uintptr_t)q % sizeof(Raw) == 0;
    auto load_q = [&](int g) __attribute__((always_inline)) {
        if (NCHW) {
#pragma unroll
            for (int i = 0; i < QN; ++i) {
                const int item = i * NT + tid, ch = item / TPW, qh = y0 + item % TPW;
                qrow[i] = Raw{};
                if (ch < d && qh < hH) {        // (ch < d <= DP: also the bound of the items)
                    const T *qp = q + ((long)n * Cq + g * d + ch) * hpl + (long)qh * hW + x0;
                    if (qvec) {
                        qrow[i] = *(const Raw *)qp;
                    } else {
                        union { T h[4]; Raw r; } x;
                        x.r = Raw{};
#pragma unroll
                        for (int e = 0; e < TPW; ++e)
                            if (x0 + e < hW) x.h[e] = qp[e];
                        qrow[i] = x.r;
                    }
                }
            }
        } else {
#pragma unroll
            for (int s16 = 0; s16 < DP / 16; ++s16) {
                qa[s16] = Raw{};
                if (mpx.active && 16 * s16 + 4 * mk < d)
                    qa[s16] = *(const Raw *)(q + mpx.hp * Cq + g * d + 16 * s16 + 4 * mk);
            }
        }
    };
    // (contiguous layout) the fetched rows into the q tile; channels d .. DP hold zeros
    auto stage_store_q = [&]() __attribute__((always_inline)) {
        if (!NCHW) return;
#pragma unroll
        for (int i = 0; i < QN; ++i) {
            const int item = i * NT + tid, ch = item / TPW, row = item % TPW;
            if (TPW * DP % NT != 0 && ch >= DP) break;
            const f32x4 v = Q4::widen(qrow[i]);
#pragma unroll
            for (int e = 0; e < TPW; ++e) Ql[(row * TPW + e) * QS + ch] = v[e];
        }
    };

    __shared__ int fb_flag;         // some point of the tile left the window (this group)
    stage_load(true, 0, d);
    load_q(0);
    for (int g = 0; g < G; ++g) {
        // ---- (a) key window and an empty weight matrix
        stage_store(KS, DP / 4);
        stage_store_q();
        if (tid == 0) fb_flag = 0;
        if (!NCHW)
            for (int i = tid; i < NPX * WS / 4; i += NT) ((f32x4 *)Wl)[i] = f32x4{0.f, 0.f, 0.f, 0.f};
        __syncthreads();
        // the group's first value chunk and the offsets travel during the similarity
        stage_load(false, g * cg, cg < CHK ? cg : CHK);
        // per-sample work: P <= 16 -> a row of 16 lanes per pixel, one pass over
        // the tile; else half a wave per pixel, two passes
        const bool narrow = P <= 16;
        f32x2 off2[2] = {f32x2{0.f, 0.f}, f32x2{0.f, 0.f}};
        // (dx, dy) of point pt of pixel px
        auto load_offset = [&](const Pix &pxc, int pt) __attribute__((always_inline)) {
            if (NCHW) {
                // (opaque copies: the addresses below, hoisted out of the loop over the
                // groups as 64-bit pointers, would be spilled -- and the spill stores of
                // every workgroup are memory traffic)
                Pix px = pxc;
                asm volatile("" : "+v"(px.pp), "+v"(px.ph), "+v"(px.pw));
                // channel cx = dx, cx + 1 = dy of the point, from the hi-res tensor or
                // from the low-res one it is a pixel shuffle / a nearest interpolation
                // of (deform_tap.hpp: OffsetLayout)
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
                return f32x2{(float)op[0], (float)op[dy]};
            }
            return Q4::load_pair(offset + pxc.hp * (2L * G * P) + 2L * ((long)g * P + pt));
        };
        if (narrow) {
            if (spx.active && sq < P) off2[0] = load_offset(spx, sq);
        } else {
#pragma unroll
            for (int ps = 0; ps < 2; ++ps)
                if (bpx[ps].active && pl < P) off2[ps] = load_offset(bpx[ps], pl);
        }

        // ---- (b) Sim = q . key over the window: this wave's blocks of 16 cells
        {
            f32x4 a4[DP / 16];
#pragma unroll
            for (int s16 = 0; s16 < DP / 16; ++s16)
                a4[s16] = NCHW ? *(const f32x4 *)(Ql + mi * QS + 16 * s16 + 4 * mk) : Q4::widen(qa[s16]);
            if (NCHW) {
                // every wave has its operands: the buffer becomes the empty weight matrix
                __syncthreads();
                for (int i = tid; i < NPX * WS / 4; i += NT) ((f32x4 *)Wl)[i] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
            for (int nb = wave; nb < NKB; nb += 4) {
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

        // ---- (c) per (pixel, point): logit from Sim, softmax over the points,
        // attention-weighted corner weights into Wm
        bool fb[2] = {false, false};        // the point passes the guard but leaves the window
        float fatt[2], fkh[2], fkw[2];
        // sample `pt` of pixel `pi` of the tile (its Pix record px); NL lanes per pixel
        auto sample = [&](auto nl, int ps, int pi, const Pix &px, int pt) __attribute__((always_inline)) {
            constexpr int NL = decltype(nl)::value;
            const bool live = px.active && pt < P;
            const float kw = (float)px.pw + off2[ps][0], kh = (float)px.ph + off2[ps][1];
            const WinTap<float> t = win_tap<float>(kh, kw, H, W, wy0, wx0, WW, WW);
            const bool in = live && t.inwin;
            fb[ps] = live && t.guard && !t.inwin;
            fkh[ps] = kh;
            fkw[ps] = kw;
            const int cell = in ? t.hl * WW + t.wl : 0;
            float lg = 0.f;
            if (in) {
                const float *sp = Sl + pi * WS + cell;
                lg = t.w1 * sp[0];
                lg = fma_(t.w2, sp[1], lg);
                lg = fma_(t.w3, sp[WW], lg);
                lg = fma_(t.w4, sp[WW + 1], lg);
            }
            if (fb[ps]) {
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
            // 1 / sum: the hardware reciprocal (1 ulp) and one Newton step
            const float sum = reduce_lanes<false, NL>(e);
            float rs = __builtin_amdgcn_rcpf(sum);
            rs = fma_(fma_(-sum, rs, 1.f), rs, rs);
            const float att = e * rs;
            fatt[ps] = att;
            // A non-finite logit anywhere in the pixel makes every weight of the pixel NaN
            // (exp(inf - inf), NaN sums), which the integer entries of Wm cannot carry: such
            // a point takes the per-sample path below, where its weight multiplies the sample
            // in floating point, as the reference's attn * val does
            // (deform_av_cuda_kernel.cu:185-190)
            const bool nonfinite = live && t.guard && att != att;
            if (nonfinite) fb[ps] = true;
            if (in && !nonfinite) {
                // Wm holds 2^30-scaled integers: every entry and every row sum is at
                // most 1, integer adds are exact in any order (the result does not
                // depend on which lane the LDS serves first) and run at the rate of
                // plain LDS writes, which float atomics do not; the rounding of a
                // contribution, 2^-31, is below that of an fp32 weight near 1
                u32 *wp = (u32 *)Wl + pi * WS + cell;
                const float sc = att * WSCALE;
                __hip_atomic_fetch_add(wp, (u32)fma_(sc, t.w1, 0.5f), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                __hip_atomic_fetch_add(wp + 1, (u32)fma_(sc, t.w2, 0.5f), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                __hip_atomic_fetch_add(wp + WW, (u32)fma_(sc, t.w3, 0.5f), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                __hip_atomic_fetch_add(wp + WW + 1, (u32)fma_(sc, t.w4, 0.5f), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            }
        };
        if (narrow) {
            sample(std::integral_constant<int, 16>{}, 0, srow, spx, sq);
        } else {
            sample(std::integral_constant<int, 32>{}, 0, half, bpx[0], pl);
            sample(std::integral_constant<int, 32>{}, 1, 8 + half, bpx[1], pl);
        }
        // ---- (d) value chunks: out tile = Wm . value window (the key window is done with)
        stage_store(VS, 16);
        if (fb[0] || fb[1]) fb_flag = 1;
        __syncthreads();
        const bool any_fb = fb_flag != 0;
        for (int vc = 0; vc < nVc; ++vc) {
            const int cbase = g * cg + vc * CHK;
            const int cvalid = cg - vc * CHK < CHK ? cg - vc * CHK : CHK;
            // next in line: the group's next value chunk, or the next group's key and q
            if (vc + 1 < nVc) {
                const int left = cg - (vc + 1) * CHK;
                stage_load(false, cbase + CHK, left < CHK ? left : CHK);
            } else if (g + 1 < G) {
                stage_load(true, (g + 1) * d, d);
                load_q(g + 1);
            }
            if (16 * wave < cvalid) {
                // two accumulators: consecutive instructions do not wait for each other
                f32x4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int s16 = 0; s16 < NKB; ++s16) {
                    const u32x4 ai = *(const u32x4 *)(Wl + mi * WS + 16 * s16 + 4 * mk);
                    const f32x4 a4 = {(float)ai[0] * (1.f / WSCALE), (float)ai[1] * (1.f / WSCALE),
                                      (float)ai[2] * (1.f / WSCALE), (float)ai[3] * (1.f / WSCALE)};
                    const float *vp = Xl + (16 * s16 + 4 * mk) * VS + 16 * wave + mi;
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        if (r % 2 == 0) acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[r], vp[r * VS], acc0, 0, 0, 0);
                        else acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[r], vp[r * VS], acc1, 0, 0, 0);
                    }
                }
#pragma unroll
                for (int r = 0; r < 4; ++r) Sl[(4 * mk + r) * VS + 16 * wave + mi] = acc0[r] + acc1[r];
            }
            __syncthreads();
            if (any_fb) {
                // points outside the window add their sample to the tile (rare)
#pragma unroll
                for (int ps = 0; ps < 2; ++ps) {
                    if (!fb[ps]) continue;
                    const int pi = narrow ? srow : ps * 8 + half;
                    // (opaque to the compiler, which would otherwise set these taps up
                    // ahead of the branch, for every tile)
                    float kh = fkh[ps], kw = fkw[ps];
                    asm volatile("" : "+v"(kh), "+v"(kw));
                    Tap<float> tp = {};
                    tap_setup(kh, kw, H, W, tp);
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
                        __hip_atomic_fetch_add(Sl + pi * VS + c, fatt[ps] * v, __ATOMIC_RELAXED,
                                               __HIP_MEMORY_SCOPE_WORKGROUP);
                    }
                }
                __syncthreads();
            }
            if (NCHW) {
                // a thread stores one row of the tile in one channel plane: 4
                // contiguous pixels.  Plain stores: the rest of each line comes from
                // the neighbouring tiles, and the L2 puts the pieces together.
                const int ch = tid / TPW, row = tid % TPW, qh = y0 + row;
                if (ch < cvalid && qh < hH) {
                    const f32x4 v = {Sl[(row * TPW + 0) * VS + ch], Sl[(row * TPW + 1) * VS + ch],
                                     Sl[(row * TPW + 2) * VS + ch], Sl[(row * TPW + 3) * VS + ch]};
                    union { T h[4]; Raw r; } x;
                    x.r = Q4::narrow(v);
                    T *op = out + ((long)n * C + cbase + ch) * hpl + (long)qh * hW + x0;
                    if (hW % TPW == 0 && (uintptr_t)out % sizeof(Raw) == 0) {
                        *(Raw *)op = x.r;
                    } else {
#pragma unroll
                        for (int e = 0; e < TPW; ++e)
                            if (x0 + e < hW) op[e] = x.h[e];
                    }
                }
            } else if (spx.active && 4 * sq < cvalid) {
                // a row of 16 lanes stores its pixel's 64 channels: 256 contiguous bytes
                __builtin_nontemporal_store(Q4::narrow(*(const f32x4 *)(Sl + srow * VS + 4 * sq)),
                                            (Raw *)(out + spx.hp * C + cbase + 4 * sq));
            }
            if (vc + 1 < nVc) {
                __syncthreads();        // everyone is done with this chunk's window and tile
                stage_store(VS, 16);
                __syncthreads();
            }
        }
    }
}

template <typename T, int S, int DP, bool NCHW>
static hipError_t launch_wmat(const void *q, const void *key, const void *value, const void *offset,
                              void *out, int B, int Cq, int C, int H, int W, int P, int G,
                              hipStream_t st, int olayout) {
    const int tiles_x = (W * S + TPW - 1) / TPW, tiles_y = (H * S + TPW - 1) / TPW;
    const long nb = (long)tiles_x * tiles_y * B;
    if (nb > (1L << 30)) return hipErrorNotSupported;
    const int per_xcd = (int)((nb + 7) / 8);
    hipLaunchKernelGGL((deform_fused_wmat_kernel<T, S, DP, NCHW>), dim3(per_xcd * 8), dim3(256), 0, st,
                       (const T *)q, (const T *)key, (const T *)value, (const T *)offset, (T *)out,
                       Cq, C, H, W, P, G, tiles_x, tiles_y, (int)nb, per_xcd, olayout);
    return hipGetLastError();
}

template <typename T, bool NCHW = false>
static hipError_t launch_wmat_t(const void *q, const void *key, const void *value, const void *offset,
                                void *out, int B, int Cq, int C, int H, int W, int P, int s, int G,
                                hipStream_t st, int olayout = OFFSET_HIRES) {
    const int d = Cq / G;
#define SAPA_WMAT(SV)                                                                               \
    case SV:                                                                                        \
        return d <= 32 ? launch_wmat<T, SV, 32, NCHW>(q, key, value, offset, out, B, Cq, C, H, W, P, G, st, olayout) \
                       : launch_wmat<T, SV, 64, NCHW>(q, key, value, offset, out, B, Cq, C, H, W, P, G, st, olayout);
    switch (s) {
        SAPA_WMAT(1) SAPA_WMAT(2) SAPA_WMAT(4)
        default: return hipErrorNotSupported;
    }
#undef SAPA_WMAT
}

}  // namespace dnhwc

// Channels-last tensors, f32 / f16 / bf16, s in {1, 2, 4}, P <= 32, channels per
// group (Cq / G and C / G) multiples of 4, Cq / G <= 64, tensors aligned to 4
// elements, one image's key / value tensor below 2^31 bytes.
// hipErrorNotSupported otherwise.
hipError_t deform_fused_nhwc_launch(const void *q, const void *key, const void *value,
                                    const void *offset, void *out, int B, int Cq, int C, int H,
                                    int W, int P, int s, int G, int dtype, hipStream_t st,
                                    const char **kernel) {
    const char *unused;
    if (!kernel) kernel = &unused;
    // the query / key channels of a group are one LDS chunk
    if (P > 16 * dnhwc::MAXSETS || (Cq / G) % 4 != 0 || Cq / G > 64 || (C / G) % 4 != 0)
        return hipErrorNotSupported;
    const int esize = dtype == 0 ? 4 : 2;
    const long plane = (long)H * W * esize;
    if (plane * Cq >= (1L << 31) || plane * C >= (1L << 31)) return hipErrorNotSupported;
    const void *ptrs[4] = {q, key, value, out};
    for (const void *p : ptrs)
        if ((uintptr_t)p % (4 * esize) != 0) return hipErrorNotSupported;
    if ((uintptr_t)offset % (2 * esize) != 0) return hipErrorNotSupported;
#ifndef SAPA_DNHWC_GATHER
    // 16-bit tensors whose groups are whole 16-byte pieces: the 16-bit matrix
    // instructions, for any number of points
    if (dtype != 0) {
        *kernel = "deform_fused_wmat16_kernel";
        const hipError_t e = deform_fused_wmat16_launch(q, key, value, offset, out, B, Cq, C, H, W, P, s, G, dtype, st);
        if (e != hipErrorNotSupported) return e;
    }
    // Few points: the fp32 matrix formulation's fixed work per tile (two products over
    // the whole window whatever P is) outweighs the gathers it saves; measured at
    // B=8, C=256, G=4, d=32, 64x64 -> 128x128, fp32: P = 5 236 against 211 us, P = 9
    // 237 against 249 us, P = 12 238 against 277 us, P = 25 268 against 450 us.
    // (SAPA_DNHWC_GATHER: a tuning build with the gather formulation throughout.)
    if (P > SAPA_DNHWC_GATHER_MAXP) {
        *kernel = "deform_fused_wmat_kernel";
        switch (dtype) {
            case 0: return dnhwc::launch_wmat_t<float>(q, key, value, offset, out, B, Cq, C, H, W, P, s, G, st);
            case 2: return dnhwc::launch_wmat_t<f16_t>(q, key, value, offset, out, B, Cq, C, H, W, P, s, G, st);
            case 3: return dnhwc::launch_wmat_t<bf16_t>(q, key, value, offset, out, B, Cq, C, H, W, P, s, G, st);
            default: return hipErrorNotSupported;
        }
    }
#endif
    *kernel = "deform_fused_nhwc_kernel";
    switch (dtype) {
        case 0: return dnhwc::launch_t<float>(q, key, value, offset, out, B, Cq, C, H, W, P, s, G, st);
        case 2: return dnhwc::launch_t<f16_t>(q, key, value, offset, out, B, Cq, C, H, W, P, s, G, st);
        case 3: return dnhwc::launch_t<bf16_t>(q, key, value, offset, out, B, Cq, C, H, W, P, s, G, st);
        default: return hipErrorNotSupported;
    }
}

// ---- contiguous (NCHW) callers through the matrix-form kernels -------------
// The kernels above read q and the offsets and write the output in place in
// the contiguous layout (NCHW = true); only the low-res key and value are
// copied into channels-last order first, into a workspace of the caller.

static long align256(long x) { return (x + 255) / 256 * 256; }

// Bytes of workspace, or 0 when the contiguous-layout kernels serve the case
// (shapes the matrix form does not cover, or too few points for it to pay).
long deform_fused_nchw_workspace(int B, int Cq, int C, int H, int W, int P, int s, int G, int dtype) {
    if (dtype != 0 && dtype != 2 && dtype != 3) return 0;
    if (s != 1 && s != 2 && s != 4) return 0;
    if (G <= 0 || Cq % G != 0 || C % G != 0) return 0;
    const int d = Cq / G, cg = C / G;
    if (P > 32 || d % 4 != 0 || d > 64 || cg % 4 != 0) return 0;
    const int esize = dtype == 0 ? 4 : 2;
    const long plane = (long)H * W * esize;
    if (plane * Cq >= (1L << 31) || plane * C >= (1L << 31)) return 0;
    if ((long)H * s * W * s >= (1L << 31)) return 0;
    // Where this path is the faster one (B=8, C=256, G=4, d=32, 64x64 -> 128x128, us,
    // the copy included, against the contiguous-layout kernels): fp32 P = 25 317 / 491,
    // P = 14 289 / 304, P = 12 282 / 247 (that kernel's wider tile up to 12 points), P = 8
    // 278 / 197; bf16 on the 16-bit kernel P = 25 194 / 470, P = 9 141 / 199, P = 5 145 / 159,
    // P = 4 138 / 142, P = 3 137 / 130.
    const bool wm16 = dtype != 0 && d % 8 == 0 && cg % 8 == 0;
#ifndef SAPA_DNCHW_MINP16
#define SAPA_DNCHW_MINP16 4
#endif
#ifndef SAPA_DNCHW_MINP32
#define SAPA_DNCHW_MINP32 13
#endif
    if (P < (wm16 ? SAPA_DNCHW_MINP16 : SAPA_DNCHW_MINP32)) return 0;
    return align256((long)B * plane * Cq) + align256((long)B * plane * C);
}

hipError_t deform_fused_nchw_ws_launch(const void *q, const void *key, const void *value,
                                       const void *offset, void *out, void *workspace, int B, int Cq,
                                       int C, int H, int W, int P, int s, int G, int olayout,
                                       int dtype, hipStream_t st, const char **kernel) {
    const char *unused;
    if (!kernel) kernel = &unused;
    if (olayout != OFFSET_HIRES && olayout != OFFSET_PIXEL_SHUFFLE && olayout != OFFSET_NEAREST)
        return hipErrorNotSupported;
    if (!workspace || (uintptr_t)workspace % 256 != 0) return hipErrorNotSupported;
    if (deform_fused_nchw_workspace(B, Cq, C, H, W, P, s, G, dtype) == 0) return hipErrorNotSupported;
    const int esize = dtype == 0 ? 4 : 2;
    const long lpix = (long)H * W;
    char *key_cl = (char *)workspace;
    char *value_cl = key_cl + align256((long)B * lpix * Cq * esize);
    hipError_t e = nchw_to_nhwc_launch(key, key_cl, Cq, value, value_cl, C, B, lpix, esize, st);
    if (e != hipSuccess) return e;
    if (dtype != 0) {
        *kernel = "deform_fused_wmat16_kernel";
        e = deform_fused_wmat16_launch(q, key_cl, value_cl, offset, out, B, Cq, C, H, W, P, s, G, dtype, st, true, olayout);
        if (e != hipErrorNotSupported) return e;
    }
    *kernel = "deform_fused_wmat_kernel";
    switch (dtype) {
        case 0: return dnhwc::launch_wmat_t<float, true>(q, key_cl, value_cl, offset, out, B, Cq, C, H, W, P, s, G, st, olayout);
        case 2: return dnhwc::launch_wmat_t<f16_t, true>(q, key_cl, value_cl, offset, out, B, Cq, C, H, W, P, s, G, st, olayout);
        case 3: return dnhwc::launch_wmat_t<bf16_t, true>(q, key_cl, value_cl, offset, out, B, Cq, C, H, W, P, s, G, st, olayout);
        default: return hipErrorNotSupported;
    }
}

}  // namespace sapa
