// SAPA-B kernels on the gfx950 matrix pipe: qk, qk+softmax, av and the fused
// qk -> softmax -> av forward built from v_mfma_f32_4x4x1_16b_f32, i.e.
// sixteen independent 4x4 outer-product accumulations per instruction.
//
// Why this instruction: SAPA's aggregation is, per low-res parent cell, a
// tiny GEMM  out[C x s*s] = V_window[C x K*K] * attn[K*K x s*s]  whose right
// operand differs from parent to parent, so there is no shared large GEMM to
// feed a 16x16 or 32x32 tile without padding the band structure with zeros.
// The 16-block 4x4x1 form maps one block to one parent: no padding, and one
// step D = A*B + C on fp32 data rounds exactly like fmaf(a, b, c) (verified
// on the hardware), so accumulating term by term in the reference kernels'
// order keeps fp32 results bit-identical to theirs
// (sapa/sapa/src/cuda/qk_cuda_kernel.cu:55-66, av_cuda_kernel.cu:57-72).
// What it buys over plain VALU FMAs is registers: a lane holds the K*K
// weights of ONE child instead of s*s children, which is what makes large
// windows and scale factors fit at all (K = 7, s = 4 would need 784
// accumulators per parent in the VALU kernel's scheme).
//
// Operand layout of the instruction (lane = 4*b + r, block b = 0..15):
//   A: lane 4b+i holds A_b[i];  B: lane 4b+j holds B_b[j];
//   D: lane 4b+j, register i holds D_b[i][j] = A_b[i] * B_b[j] + C_b[i][j].
// Work decomposition: a wave owns 16 consecutive parents of one low-res row
// (block b = parent) and 4 of the s*s children of each (lane 4b+j = child j
// of the group); a workgroup owns a (16*NWX) x NR tile of parents.
//   logits:  A_b[i] = key[c, neighbour 4g+i of parent b],  B_b[j] = q[c, child j]
//            -> lane (b,j) accumulates logit(child j, neighbour 4g+i) in
//            register i of accumulator g, channel after channel;
//   softmax: per lane, over its own K*K registers;
//   output:  A_b[i] = value[c0+i, neighbour k of parent b], B_b[j] = weight(child j, k)
//            -> lane (b,j), register i = out[c0+i, child j], neighbour after
//            neighbour in ky-major order.
// The low-res windows are staged through LDS exactly as in the VALU kernel
// (chunks of CH channels, double-buffered, next chunk's loads in flight
// during the current chunk's math); layout [channel][row][column] with a
// channel stride that is 8 mod 32 floats, so the A-operand reads of the
// output phase (16 parents x 4 channels per instruction) are conflict-free.
// Out-of-range neighbours are zeros in LDS: logit exactly 0 (it takes part
// in the softmax), contribution exactly 0, as the reference's `continue`.
#include "kernels.hpp"

namespace sapa {

typedef float f32x4 __attribute__((ext_vector_type(4)));

template <int NB> struct StreamBits;
template <> struct StreamBits<2> { typedef unsigned short type; };
template <> struct StreamBits<4> { typedef unsigned type; };
template <> struct StreamBits<8> { typedef unsigned long long type; };

// The high-res tensors are touched exactly once: stream them past the caches.
template <typename T>
__device__ __forceinline__ float load_stream1(const T *p) {
    typedef typename StreamBits<sizeof(T)>::type B;
    union { B b; T v; } u;
    u.b = __builtin_nontemporal_load((const B *)p);
    return (float)u.v;
}
template <typename T>
__device__ __forceinline__ void store_stream1(T *p, float x) {
    typedef typename StreamBits<sizeof(T)>::type B;
    union { B b; T v; } u;
    u.v = (T)x;
    __builtin_nontemporal_store(u.b, (B *)p);
}

#ifndef SAPA_MFMA_WPE
#define SAPA_MFMA_WPE 4
#endif

template <typename T, int K, int S, int NWX, int NR, int CH, int WPE, int MODE>
__global__ void __launch_bounds__(64 * NWX * NR * (S * S / 4))
    __attribute__((amdgpu_waves_per_eu(WPE, WPE)))
sapa_b_mfma_kernel(const T *__restrict__ q, const T *__restrict__ key,
                   const T *__restrict__ attn_in, const T *__restrict__ value,
                   T *__restrict__ out, int d, int C, int H, int W, int tiles_x, int tiles_y,
                   int nblocks, int per_xcd, int cgroups, int cper) {
    typedef float A;
    constexpr int KK = K * K, R = (K - 1) / 2;
    constexpr int NG = S * S / 4;            // child groups (waves) per 16 parents
    constexpr int NGK = (KK + 3) / 4;        // neighbour groups of 4
    constexpr int NT = 64 * NWX * NR * NG;   // threads per workgroup
    constexpr int TW = 16 * NWX, TH = NR;    // parents per workgroup
    constexpr int WW = TW + K - 1, WH = TH + K - 1;
    constexpr int RS = WW + 1;               // row stride, one padding column
    constexpr int CS = ((WH * RS - 8 + 31) / 32) * 32 + 8;   // channel stride, 8 mod 32
    constexpr int WIN = WH * WW;
    constexpr int NPOS = (WIN + NT - 1) / NT;
    constexpr int NSTAGE = CH * NPOS;
    constexpr int BUF = CH * CS;
    constexpr bool DO_QK = MODE != TILED_AV;
    constexpr bool DO_SOFTMAX = MODE == TILED_QK_SOFTMAX || MODE == TILED_FUSED;
    constexpr bool DO_AV = MODE == TILED_AV || MODE == TILED_FUSED;
    static_assert(S * S % 4 == 0, "children come in groups of 4");
    static_assert(CH % 4 == 0, "the output phase takes 4 channels per MFMA");
    static_assert(CS % 32 == 8 && CS >= WH * RS, "LDS channel stride");

    __shared__ A lds[2 * BUF];

    const int logical = (int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8);
    if (logical >= nblocks) return;
    const int tx = logical % tiles_x;
    const int ty = (logical / tiles_x) % tiles_y;
    const int cg = (logical / (tiles_x * tiles_y)) % cgroups;
    const int n = logical / (tiles_x * tiles_y * cgroups);
    const int cbeg = cg * cper;
    const int cend = cbeg + cper < C ? cbeg + cper : C;
    if (DO_AV && cbeg >= C) return;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int gi = wave % NG, wxr = wave / NG;
    const int wx = wxr % NWX, wr = wxr / NWX;
    const int b = lane >> 2, r4 = lane & 3;      // r4 is j for B/D, i for A
    const int x0 = tx * TW, y0 = ty * TH;
    const int px = x0 + wx * 16 + b, py = y0 + wr;
    const bool active = px < W && py < H;
    const int cj = gi * 4 + r4, cy = cj / S, cx = cj % S;   // this lane's child
    const int hH = H * S, hW = W * S;
    const long lplane = (long)H * W, hplane = (long)hH * hW;
    const long hpix = (long)(py * S + cy) * hW + (long)px * S + cx;
    const long hpix_ld = (long)((py < H ? py : H - 1) * S + cy) * hW +
                         (long)(px < W ? px : W - 1) * S + cx;

    const int nKc = DO_QK ? (d + CH - 1) / CH : 0;
    const int nVc = DO_AV ? (cend - cbeg + CH - 1) / CH : 0;
    const int ntot = nKc + nVc;

    // ---- staging of the low-res windows (same scheme as the VALU kernel)
    int g_off[NPOS], l_off[NPOS];
    unsigned g_mask[NPOS];
#pragma unroll
    for (int i = 0; i < NPOS; ++i) {
        const int pos = tid + i * NT;
        const int row = pos / WW, col = pos % WW;
        const int gy = y0 - R + row, gx = x0 - R + col;
        const bool l_ok = WIN % NT == 0 || pos < WIN;
        const bool g_ok = l_ok && gy >= 0 && gy < H && gx >= 0 && gx < W;
        const int yy = gy < 0 ? 0 : (gy < H ? gy : H - 1);
        const int xx = gx < 0 ? 0 : (gx < W ? gx : W - 1);
        g_off[i] = yy * W + xx;              // clamped: always a legal address
        g_mask[i] = g_ok ? 0xffffffffu : 0u;
        l_off[i] = l_ok ? row * RS + col : WW;   // surplus -> padding column of row 0
    }
    A st[NSTAGE];
    auto stage_load = [&](int j) {
        const bool is_key = j < nKc;
        const T *src = is_key ? key : value;
        const int nch = is_key ? d : C;
        const int c0 = is_key ? j * CH : cbeg + (j - nKc) * CH;
        const T *base = src + (long)n * nch * lplane;
#pragma unroll
        for (int ch = 0; ch < CH; ++ch) {
            const int c = c0 + ch;
            const T *plane = base + (long)(c < nch ? c : nch - 1) * lplane;
#pragma unroll
            for (int i = 0; i < NPOS; ++i) st[ch * NPOS + i] = (A)plane[g_off[i]];
        }
    };
    auto stage_store = [&](int j) {
        const bool is_key = j < nKc;
        const int nch = is_key ? d : C;
        const int c0 = is_key ? j * CH : cbeg + (j - nKc) * CH;
        A *dst = lds + (j & 1) * BUF;
#pragma unroll
        for (int ch = 0; ch < CH; ++ch)
#pragma unroll
            for (int i = 0; i < NPOS; ++i)
                dst[ch * CS + l_off[i]] = __uint_as_float(
                    __float_as_uint(st[ch * NPOS + i]) & (c0 + ch < nch ? g_mask[i] : 0u));
    };

    // logits / weights of this lane's child: w[g][i] belongs to neighbour 4g+i
    f32x4 w[NGK];
#pragma unroll
    for (int g = 0; g < NGK; ++g) w[g] = (f32x4){0.f, 0.f, 0.f, 0.f};

    stage_load(0);
    if (MODE == TILED_AV && active) {
        const T *ap = attn_in + (long)n * KK * hplane + hpix;
#pragma unroll
        for (int k = 0; k < KK; ++k) w[k / 4][k % 4] = load_stream1(ap + (long)k * hplane);
    }
    stage_store(0);
    __syncthreads();

    const int lbase = wr * RS + wx * 16 + b;   // window origin of this lane's parent

    if (DO_QK) {
        // A-operand offsets: lane with r4 = i fetches neighbour 4g+i
        int koff[NGK];
#pragma unroll
        for (int g = 0; g < NGK; ++g) {
            const int k = 4 * g + r4;
            koff[g] = k < KK ? lbase + (k / K) * RS + (k % K) : lbase;
        }
        const T *qp = q + (long)n * d * hplane + hpix_ld;
        const unsigned qmask = active ? 0xffffffffu : 0u;
        constexpr int PF = 4;   // q is fetched PF channels ahead of its use
        A qr[PF];
#pragma unroll
        for (int u = 0; u < PF; ++u) qr[u] = load_stream1(qp + (long)(u < d ? u : d - 1) * hplane);
        for (int j = 0; j < nKc; ++j) {
            if (j + 1 < ntot) stage_load(j + 1);
            const int c0 = j * CH;
            const A *wb = lds + (j & 1) * BUF;
#pragma unroll 1
            for (int ch0 = 0; ch0 < CH; ch0 += PF) {
#pragma unroll
                for (int u = 0; u < PF; ++u) {
                    const int c = c0 + ch0 + u;
                    const A qv = __uint_as_float(__float_as_uint(qr[u]) & (c < d ? qmask : 0u));
                    const int cn = c + PF;
                    qr[u] = load_stream1(qp + (long)(cn < d ? cn : d - 1) * hplane);
                    const A *wc = wb + (ch0 + u) * CS;
#pragma unroll
                    for (int g = 0; g < NGK; ++g)
                        w[g] = __builtin_amdgcn_mfma_f32_4x4x1f32(wc[koff[g]], qv, w[g], 0, 0, 0);
                }
            }
            if (j + 1 < ntot) stage_store(j + 1);
            __syncthreads();
        }
        if (DO_SOFTMAX) {
            A v[KK];
#pragma unroll
            for (int k = 0; k < KK; ++k) v[k] = w[k / 4][k % 4];
            softmax_inplace<A, KK>(v);
#pragma unroll
            for (int k = 0; k < KK; ++k) w[k / 4][k % 4] = v[k];
        }
        if (!DO_AV && active) {
            T *op = out + (long)n * KK * hplane + hpix;
#pragma unroll
            for (int k = 0; k < KK; ++k) store_stream1(op + (long)k * hplane, w[k / 4][k % 4]);
        }
    }

    if (DO_AV) {
        // A = the weights (lane 4b+i: child i of parent b, tap k), B = the window values (lane
        // 4b+j: channel c0+j at tap k of parent b), so lane 4b+j ends up with the 4 children's
        // results for ITS channel: PXR x-neighbours of 4 / PXR rows, stored as whole vectors.
        // The stores are buffer stores without a branch: the descriptor covers the channels of
        // the chunk that exist, idle lanes carry an offset beyond it and the hardware drops them.
        const int vbase = lbase + r4 * CS;   // lane with r4 = j fetches channel c0+j
        constexpr int PXR = S >= 4 ? 4 : 2, NROW = 4 / PXR;
        const int cy0 = (gi * 4) / S, cx0 = (gi * 4) % S;     // first child of the lane's group
        const long hpg = (long)(py * S + cy0) * hW + (long)px * S + cx0;
        const unsigned ooff = active ? (unsigned)(hpg * (long)sizeof(T)) : 0x80000000u;
        const unsigned plane_bytes = (unsigned)(hplane * (long)sizeof(T));
        for (int j = nKc; j < ntot; ++j) {
            if (j + 1 < ntot) stage_load(j + 1);
            const int c0 = cbeg + (j - nKc) * CH;
            const A *wb = lds + (j & 1) * BUF + vbase;
            const int nleft = cend - c0 < CH ? cend - c0 : CH;
            const __amdgpu_buffer_rsrc_t orsrc = __builtin_amdgcn_make_buffer_rsrc(
                (void *)(out + ((long)n * C + c0) * hplane), 0, (int)((unsigned)nleft * plane_bytes), 0x00020000);
#pragma unroll
            for (int cq = 0; cq < CH / 4; ++cq) {
                const A *wc = wb + cq * 4 * CS;
                f32x4 o = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ky = 0; ky < K; ++ky)
#pragma unroll
                    for (int kx = 0; kx < K; ++kx) {
                        const int k = ky * K + kx;
                        o = __builtin_amdgcn_mfma_f32_4x4x1f32(w[k / 4][k % 4], wc[ky * RS + kx], o,
                                                              0, 0, 0);
                    }
#pragma unroll
                for (int r = 0; r < NROW; ++r) {
                    Vec<T, PXR> v;
#pragma unroll
                    for (int e = 0; e < PXR; ++e) v.v[e] = (T)o[r * PXR + e];
                    store_buffer<T, PXR>(orsrc, ooff + (unsigned)(cq * 4 + r4) * plane_bytes +
                                                    (unsigned)(r * hW) * (unsigned)sizeof(T), v);
                }
            }
            if (j + 1 < ntot) stage_store(j + 1);
            __syncthreads();
        }
    }
}

// ------------------------------------------------------------------ launcher
template <typename T, int K, int S, int NWX, int NR, int CH, int WPE>
static hipError_t launch_mode(int mode, const void *q, const void *key, const void *attn_in,
                              const void *value, void *out, int B, int d, int C, int H, int W,
                              hipStream_t st) {
    constexpr int TW = 16 * NWX, TH = NR, NT = 64 * NWX * NR * (S * S / 4);
    const int tiles_x = (W + TW - 1) / TW, tiles_y = (H + TH - 1) / TH;
    int cgroups = 1;
    if (mode == TILED_FUSED || mode == TILED_AV) {
        const long tiles = (long)tiles_x * tiles_y * B;
        const int max_groups = C / (4 * CH) > 0 ? C / (4 * CH) : 1;
        while (cgroups * 2 <= max_groups && tiles * cgroups * 2 <= 512) cgroups *= 2;
    }
    const int cper = ((C + cgroups - 1) / cgroups + CH - 1) / CH * CH;
    const long nb = (long)tiles_x * tiles_y * B * cgroups;
    if (nb > (1L << 30)) return hipErrorNotSupported;
    if (mode == TILED_FUSED || mode == TILED_AV) {
        // the results leave as vectors of 2 (s = 2) or 4 x-neighbours through 32-bit byte
        // offsets inside one chunk of CH planes
        const uintptr_t va = (uintptr_t)(sizeof(T) * (S >= 4 ? 4 : 2));
        if ((uintptr_t)out % va != 0) return hipErrorNotSupported;
        if ((long)CH * H * S * W * S * (long)sizeof(T) > (1L << 31)) return hipErrorNotSupported;
    }
    const int per_xcd = (int)((nb + 7) / 8);
    const dim3 grid(per_xcd * 8), block(NT);
#define SAPA_MM_CASE(M)                                                                        \
    case M:                                                                                    \
        hipLaunchKernelGGL((sapa_b_mfma_kernel<T, K, S, NWX, NR, CH, WPE, M>), grid, block, 0, \
                           st, (const T *)q, (const T *)key, (const T *)attn_in,               \
                           (const T *)value, (T *)out, d, C, H, W, tiles_x, tiles_y, (int)nb,  \
                           per_xcd, cgroups, cper);                                            \
        break;
    switch (mode) {
        SAPA_MM_CASE(TILED_QK) SAPA_MM_CASE(TILED_QK_SOFTMAX) SAPA_MM_CASE(TILED_AV)
        SAPA_MM_CASE(TILED_FUSED)
        default: return hipErrorInvalidValue;
    }
#undef SAPA_MM_CASE
    return hipGetLastError();
}

template <typename T>
static hipError_t launch_t(int mode, const void *q, const void *key, const void *attn_in,
                           const void *value, void *out, int B, int d, int C, int H, int W, int K,
                           int s, hipStream_t st) {
#ifdef SAPA_MFMA_TUNE
    if (K == 5 && s == 2)
        return launch_mode<T, 5, 2, SAPA_MFMA_TUNE>(mode, q, key, attn_in, value, out, B, d, C, H, W, st);
#else
    // s = 2: 32x4-parent tiles, 8 waves; s = 4: 16x2-parent tiles, 8 waves (4
    // child groups per parent row) and 16-channel chunks: with s*s = 16
    // children per parent the low-res halo is cheap, and two workgroups per CU
    // overlap each other's barriers (a 16-wave workgroup owns the CU alone).  K = 5, s = 2 is left to the VALU
    // kernel, which is the faster one except on small problems (below).
#define SAPA_MM_INST(KV, SV, ...)                                                              \
    if (K == KV && s == SV)                                                                    \
        return launch_mode<T, KV, SV, __VA_ARGS__>(mode, q, key, attn_in, value, out, B, d, C, \
                                                   H, W, st);
    // K = 5, s = 2 (the callers send only small problems here: with a lane per child
    // a launch has four times the waves of the VALU kernel, and a wave alone issues these
    // instructions back to back): 16x4-parent tiles, 16-channel chunks from 4096 cells up
    if (K == 5 && s == 2 && (long)B * H * W <= 4096)
        return launch_mode<T, 5, 2, 1, 4, 8, 4>(mode, q, key, attn_in, value, out, B, d, C, H, W, st);
    SAPA_MM_INST(5, 2, 1, 4, 16, 4)
    SAPA_MM_INST(3, 2, 2, 4, 8, 5)
    SAPA_MM_INST(7, 2, 2, 4, 8, 4)
    SAPA_MM_INST(3, 4, 1, 2, 16, 5)
    SAPA_MM_INST(5, 4, 1, 2, 16, 4)
#ifdef SAPA_MFMA_TUNE_74
    SAPA_MM_INST(7, 4, SAPA_MFMA_TUNE_74)
#else
    SAPA_MM_INST(7, 4, 1, 2, 16, 4)
#endif
#undef SAPA_MM_INST
#endif
    return hipErrorNotSupported;
}

hipError_t sapa_b_mfma_launch(int mode, const void *q, const void *key, const void *attn_in,
                              const void *value, void *out, int B, int d, int C, int H, int W,
                              int K, int s, int dtype, hipStream_t st) {
    switch (dtype) {
        case 0: return launch_t<float>(mode, q, key, attn_in, value, out, B, d, C, H, W, K, s, st);
#ifndef SAPA_MFMA_TUNE
        case 2: return launch_t<f16_t>(mode, q, key, attn_in, value, out, B, d, C, H, W, K, s, st);
        case 3: return launch_t<bf16_t>(mode, q, key, attn_in, value, out, B, d, C, H, W, K, s, st);
#endif
        default: return hipErrorNotSupported;
    }
}

}  // namespace sapa
