// Fused SAPA-B forward (qk -> softmax -> av) for channels-last f16 / bf16 tensors as two dense
// products per 4 x 4 block of parents over the block's 8 x 8 window, on the 16-bit matrix
// instructions; K = 5, s = 2.  q [B,2H,2W,d], key [B,H,W,d], value [B,H,W,C], out [B,2H,2W,C].
//
//   Sim[cell][child]   = sum_c key[cell][c] * q[child][c]             64 x 64 x d
//   P[child][cell]     = softmax over the child's 5 x 5 cells of Sim, 0 on the window's other cells
//   out^T[ch][child]   = sum_cell value[cell][ch] * P[child][cell]     C x 64 x 64
//
// (reference: sapa/sapa/src/cuda/qk_cuda_kernel.cu:55-66, av_cuda_kernel.cu:52-66, the softmax
// between them in sapa_base.py:38-40; a cell outside the image holds zeros, the reference's zero
// padding.)  The decomposition is that of sapa_b_wmat16.hip; what the layout changes:
//   * both operands of the logits hold the reduction index (channels) contiguously: the key
//     window is read from LDS 16 bytes at a time, q goes from global memory straight into the
//     B-operand registers (16 bytes = 8 channels of one child per lane; it is used once);
//   * the aggregation reduces over cells, which lie a whole channel vector apart:
//     ds_read_tr16_b64 hands each lane one channel of 4 cells; the softmax result is used in
//     place as the other operand (the accumulator layout of the first product is an operand
//     layout of the second);
//   * with channels as the M index a lane ends up with 4 consecutive channels of a child: 8-byte
//     writes into a wave-private LDS slot [16 children][64 channels], read back 16 bytes per
//     lane, so that every global store covers whole 128-byte lines (a child's 64 channels);
//   * a window cell is a whole unit of memory: positions outside the image are loads with an
//     out-of-range offset (zeros), no edge cases in registers.
// A workgroup is 4 waves = 4 blocks side by side; key / value windows go through two LDS
// buffers of 64 channels, loaded straight from global memory (buffer loads with the LDS
// modifier) with the 16-byte pieces of a cell XOR-swizzled by the cell's index against bank
// conflicts.  The weights enter the aggregation as a 16-bit value plus a 16-bit remainder, sums
// are fp32: the result is within half a 16-bit spacing of the exact one.  A masked cell still
// enters both products (logit plus -inf, weight 0 times value): a non-finite key or value
// reaches every child of the 4 x 4 block whose window holds it.
#include "kernels.hpp"

namespace sapa {

namespace cwm16 {

typedef unsigned u32;
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef u32 u32x2 __attribute__((ext_vector_type(2)));
typedef u32 u32x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));

constexpr int CHK = 64;            // channels per staged chunk = 8 pieces of 16 bytes per cell
constexpr int WROWS = 8;           // window rows
constexpr int CELL = CHK / 2;      // dwords per cell
constexpr u32 OUTSIDE = 0x80000000u;

template <typename T> struct Mma;
template <> struct Mma<f16_t> {
    typedef _Float16 v8 __attribute__((ext_vector_type(8)));
    static __device__ __forceinline__ f32x4 k32(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8, a), __builtin_bit_cast(v8, b), c, 0, 0, 0);
    }
};
template <> struct Mma<bf16_t> {
    typedef __bf16 v8 __attribute__((ext_vector_type(8)));
    static __device__ __forceinline__ f32x4 k32(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8, a), __builtin_bit_cast(v8, b), c, 0, 0, 0);
    }
};

template <typename T>
__device__ __forceinline__ u32 pack2(float a, float b) {
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    typedef T tx2 __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(u32, __builtin_convertvector(f32x2{a, b}, tx2));
}

// 4 cells x 4 channels out of LDS, transposed: each lane of a 16-lane block addresses 4
// consecutive channels of one cell and receives one channel of the 4 cells
__device__ __forceinline__ u32x2 read_tr(const u32 *p) {
    return __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                                         (s16x4 __attribute__((address_space(3))) *)p));
}

// dword offset of the 16-byte piece `piece` (0..7) of cell / child `idx` in a [idx][64 channels] array
__device__ __forceinline__ int piece_at(int idx, int piece) { return idx * CELL + ((piece ^ (idx & 7)) << 2); }

// QB: a per-image bias [B, d] of the query projection: key . (q + b) = key . q + key . b, the second
// product with the bias as the operand of every child (nothing is rounded in between)
template <typename T, int NSW, bool STREAM, bool QB>
__global__ __launch_bounds__(64 * NSW) void
sapa_b_nhwc_wm16_kernel(const T *__restrict__ q, const T *__restrict__ key, const T *__restrict__ value,
                        const T *__restrict__ qbias, T *__restrict__ out, int d, int C, int H, int W, int tiles_x, int tiles_y, int ns,
                        int nblocks, int per_xcd) {
    constexpr int NT = 64 * NSW;
    constexpr int WC = 4 * NSW + 4;                          // window cells per row of the tile
    constexpr int NCELL = WROWS * WC;
    constexpr int LOWBUF = NCELL * CELL;                     // dwords per window buffer
    constexpr int NLP = NCELL * 8;                           // 16-byte pieces per window buffer
    constexpr int NLI = (NLP + NT - 1) / NT;                 // direct loads per thread and window, at most
    constexpr int OSLOT = 16 * CELL;                         // dwords of a wave's output slot: 16 children x 64 channels
    static_assert(NLP % 64 == 0, "whole direct loads");
    constexpr int STREAM_AUX = STREAM ? 2 : 0;

    __shared__ __attribute__((aligned(16))) u32 lds[2 * LOWBUF + NSW * OSLOT];
    u32 *const lowbuf = lds;

    const int logical = (int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8);
    if (logical >= nblocks) return;
    const int tx = logical % tiles_x, ty = (logical / tiles_x) % tiles_y, n = logical / (tiles_x * tiles_y);
    const int X0 = tx * 4 * ns, Y0 = ty * 4;                 // first parent of the tile
    const int nsx = (W + 3) / 4;
    const int ns_here = nsx - tx * ns < ns ? nsx - tx * ns : ns;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = lane >> 4, i16 = lane & 15;
    const long lpix = (long)H * W;
    const bool active = wave < ns_here;
    const int t = wave;                                       // this wave's block of the tile

    // window loads: piece `slot % 8` of cell `slot / 8` (row cell / WC, column cell % WC of the
    // window, which starts 2 cells left of and above the tile); byte offset inside the image
    // without the channel part, and the piece's first channel inside the chunk
    u32 off_low[NLI];
    int ch_low[NLI];
#pragma unroll
    for (int i = 0; i < NLI; ++i) {
        const int slot = i * NT + tid, cell = slot >> 3;
        const int piece = (slot & 7) ^ (cell & 7);            // the piece this slot of the cell holds
        const int y = Y0 - 2 + cell / WC, x = X0 - 2 + cell % WC;
        const bool ok = slot < NLP && cell % WC < 4 * ns_here + 4 && y >= 0 && y < H && x >= 0 && x < W;
        off_low[i] = ok ? (u32)(y * W + x) : OUTSIDE;         // cell index; times the channel count below
        ch_low[i] = 8 * piece;
    }
    const __amdgpu_buffer_rsrc_t rq = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(q + (long)n * d * 4 * lpix), 0, (int)(d * 4 * lpix * (long)sizeof(T)), 0x00020000);
    const __amdgpu_buffer_rsrc_t rk = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(key + (long)n * d * lpix), 0, (int)(d * lpix * (long)sizeof(T)), 0x00020000);
    const __amdgpu_buffer_rsrc_t rv = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(value + (long)n * C * lpix), 0, (int)(C * lpix * (long)sizeof(T)), 0x00020000);
    const __amdgpu_buffer_rsrc_t ro = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(out + (long)n * C * 4 * lpix), 0, (int)(C * 4 * lpix * (long)sizeof(T)), 0x00020000);
    (void)rk, (void)rv;

    const int nKc = (d + CHK - 1) / CHK, nVc = (C + CHK - 1) / CHK, ntot = nKc + nVc;
    // chunk j: key channels 64 j .. for j < nKc, value channels 64 (j - nKc) .. after; buffer j % 2,
    // requested two chunks ahead.  A piece past the tensor's last channel would be the next
    // cell's: out of range instead (zeros).
    auto stage = [&](int j) __attribute__((always_inline)) {
#if defined(__HIP_DEVICE_COMPILE__)
        if (j >= ntot) return;
        const bool is_key = j < nKc;
        const int cx = is_key ? d : C, c0 = (is_key ? j : j - nKc) * CHK;
        const __amdgpu_buffer_rsrc_t r = is_key ? rk : rv;
        u32 *lb = lowbuf + (j & 1) * LOWBUF + wave * 256;
#pragma unroll
        for (int i = 0; i < NLI; ++i)
            if ((i + 1) * NT <= NLP || i * NT + wave * 64 < NLP) {
                const u32 off = c0 + ch_low[i] < cx && off_low[i] != OUTSIDE
                                    ? (off_low[i] * (u32)cx + (u32)(c0 + ch_low[i])) * (u32)sizeof(T)
                                    : OUTSIDE;
                __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (__attribute__((address_space(3))) void *)(lb + i * NT * 4), 16,
                                                         off, 0, 0, 0);
            }
#endif
    };
    // (waits are counted by hand: the compiler does not track a direct load's LDS write; the
    // counter of vector-memory operations retires in issue order)
    auto barrier = [&]() __attribute__((always_inline)) {
#if defined(__HIP_DEVICE_COMPILE__)
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
#endif
    };

    stage(0);
    stage(1);
    // One barrier per chunk: a wave computes on chunk j, waits until chunk j + 1 has landed in its own
    // slots, meets the others (chunk j + 1 complete, buffer j % 2 free) and requests chunk j + 2.
    auto landed_barrier = [&](bool stores_after) __attribute__((always_inline)) {
#if defined(__HIP_DEVICE_COMPILE__)
        // (the 8 stores a wave issues per chunk of the aggregation come after the loads waited for)
        if (stores_after) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#endif
        barrier();
    };
    landed_barrier(false);

    // this lane's child of block nb: row 2 nb + i16 / 8, column i16 % 8 of the block's 8 x 8 children
    // (pixel offset of nb = 0; nb adds two rows)
    const int cy0 = 2 * Y0 + (i16 >> 3), cx0 = 2 * X0 + 8 * t + (i16 & 7);
    const int hW = 2 * W, hH = 2 * H;

    // ---- logits: Sim[cell][child], 4 x 4 accumulator blocks of 16 x 16 ----
    // block (mb, nb), lane (g, i16), element v: cell (row 2 mb + g / 2, column 4 (g % 2) + v) of the
    // window, child (row 2 nb + i16 / 8, column i16 % 8)
    f32x4 sim[4][4];
#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) sim[mb][nb] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int j = 0; j < nKc; ++j) {
        // q of this chunk: B operand of reduction step s = channels 32 s + 8 g .. + 7 of the child
        u32x4 qb[4][2], bb[2];
        if (active) {
            if constexpr (QB) {
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    const int c = j * CHK + 32 * s + 8 * g;
                    bb[s] = c < d ? *(const u32x4 *)(qbias + (long)n * d + c) : u32x4{0u, 0u, 0u, 0u};
                }
            }
#pragma unroll
            for (int nb = 0; nb < 4; ++nb)
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    const int cy = cy0 + 2 * nb, c = j * CHK + 32 * s + 8 * g;
                    const u32 off = cy < hH && cx0 < hW && c < d
                                        ? (u32)(((long)cy * hW + cx0) * d + c) * (u32)sizeof(T)
                                        : OUTSIDE;
                    qb[nb][s] = __builtin_amdgcn_raw_buffer_load_b128(rq, off, 0, STREAM_AUX);
                }
        }
        if (active) {
            const u32 *kb = lowbuf + (j & 1) * LOWBUF;
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                u32x4 a[4];
#pragma unroll
                for (int mb = 0; mb < 4; ++mb) {
                    const int cell = (2 * mb + (i16 >> 3)) * WC + 4 * t + (i16 & 7);
                    a[mb] = *(const u32x4 *)(kb + piece_at(cell, 4 * s + g));
                }
#pragma unroll
                for (int mb = 0; mb < 4; ++mb)
#pragma unroll
                    for (int nb = 0; nb < 4; ++nb) sim[mb][nb] = Mma<T>::k32(a[mb], qb[nb][s], sim[mb][nb]);
                if constexpr (QB) {
                    // key . b is the same for every child: one product per block of cells, added to all four
#pragma unroll
                    for (int mb = 0; mb < 4; ++mb) {
                        const f32x4 kb4 = Mma<T>::k32(a[mb], bb[s], f32x4{0.f, 0.f, 0.f, 0.f});
#pragma unroll
                        for (int nb = 0; nb < 4; ++nb) sim[mb][nb] += kb4;
                    }
                }
            }
        }
        landed_barrier(false);
        stage(j + 2);
    }

    // ---- softmax over each child's 5 x 5 cells; the weights as operands of the aggregation ----
    u32x4 whi[4][2], wlo[4][2];
    if (active) {
        // a child of parent column px takes window columns px .. px + 4: -inf added to the others
        const int px = (i16 & 7) >> 1;
        const float NEG_INF = -__builtin_inff(), LOG2E = 1.4426950408889634f;
        float col_bias[4];
#pragma unroll
        for (int v = 0; v < 4; ++v) col_bias[v] = (u32)(4 * (g & 1) + v - px) <= 4u ? 0.f : NEG_INF;
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) {
            // child row 2 nb + i16 / 8 -> parent row nb: window rows nb .. nb + 4.  Block mb holds
            // rows 2 mb (lanes g < 2) and 2 mb + 1: all, some or none of its lanes take part
            float x[4][4], m = NEG_INF;
#pragma unroll
            for (int mb = 0; mb < 4; ++mb) {
                const bool lo_in = 2 * mb >= nb && 2 * mb <= nb + 4, hi_in = 2 * mb + 1 >= nb && 2 * mb + 1 <= nb + 4;
                if (!lo_in && !hi_in) continue;
                const float row_bias = lo_in && hi_in ? 0.f : ((g >> 1) ? hi_in : lo_in) ? 0.f : NEG_INF;
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    x[mb][v] = sim[mb][nb][v] + (lo_in && hi_in ? col_bias[v] : col_bias[v] + row_bias);
                    m = fmaxf(m, x[mb][v]);
                }
            }
            m = fmaxf(m, __shfl_xor(m, 16));
            m = fmaxf(m, __shfl_xor(m, 32));
            // exp(x - m) as 2^(x log2 e - m log2 e); a masked cell gives 2^-inf = 0
            const float mneg = -m * LOG2E;
            float e[4][4], sum = 0.f;
#pragma unroll
            for (int mb = 0; mb < 4; ++mb) {
                const bool lo_in = 2 * mb >= nb && 2 * mb <= nb + 4, hi_in = 2 * mb + 1 >= nb && 2 * mb + 1 <= nb + 4;
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    e[mb][v] = lo_in || hi_in ? __builtin_amdgcn_exp2f(__builtin_fmaf(x[mb][v], LOG2E, mneg)) : 0.f;
                    if (lo_in || hi_in) sum += e[mb][v];
                }
            }
            sum += __shfl_xor(sum, 16);
            sum += __shfl_xor(sum, 32);
            const float inv = 1.f / sum;
            // reduction step s of the aggregation covers the cells of blocks mb = 2 s, 2 s + 1
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                float p[8];
#pragma unroll
                for (int k = 0; k < 8; ++k) p[k] = e[2 * s + k / 4][k % 4] * inv;
                typedef T tx8 __attribute__((ext_vector_type(8)));
                whi[nb][s] = u32x4{pack2<T>(p[0], p[1]), pack2<T>(p[2], p[3]), pack2<T>(p[4], p[5]), pack2<T>(p[6], p[7])};
                const tx8 hi = __builtin_bit_cast(tx8, whi[nb][s]);
#pragma unroll
                for (int k = 0; k < 8; ++k) p[k] -= (float)hi[k];
                wlo[nb][s] = u32x4{pack2<T>(p[0], p[1]), pack2<T>(p[2], p[3]), pack2<T>(p[4], p[5]), pack2<T>(p[6], p[7])};
            }
        }
    }

    // ---- aggregation: out^T[channel][child], per chunk of 64 channels ----
    // output rows of block nb leave through this wave's slot: lane l reads pieces l and l + 64 of
    // the slot's 16 children x 8 pieces
    u32 *oslot = lds + 2 * LOWBUF + wave * OSLOT;
    u32 off_out[2];
    int ch_out[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int p = lane + 64 * i, child = p >> 3;
        const int cy = 2 * Y0 + (child >> 3), cx = 2 * X0 + 8 * t + (child & 7);
        off_out[i] = cy < hH && cx < hW ? (u32)(cy * hW + cx) : OUTSIDE;      // pixel index of nb = 0
        ch_out[i] = 8 * (p & 7);
    }
    for (int j = nKc; j < ntot; ++j) {
        const int c0 = (j - nKc) * CHK;
        if (active) {
            const u32 *vb = lowbuf + (j & 1) * LOWBUF;
            // A operand of (channel block mk, step s): lane (g, channel i16) holds the cells of rows
            // 4 s + g / 2 and 4 s + 2 + g / 2, columns 4 (g % 2) .. + 3 -- the order the weights are
            // held in.  Transposing read: lane L of a 16-lane block addresses cell L / 4 of the 4,
            // channels 16 mk + 4 (L % 4) .. + 3.
            u32x4 va[4][2];
#pragma unroll
            for (int mk = 0; mk < 4; ++mk)
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    const int cell = (4 * s + (g >> 1)) * WC + 4 * t + 4 * (g & 1) + (i16 >> 2);
                    const int piece = 2 * mk + ((i16 & 3) >> 1);
                    const u32x2 lo = read_tr(vb + piece_at(cell, piece) + 2 * (i16 & 1));
                    const u32x2 hi = read_tr(vb + piece_at(cell + 2 * WC, piece) + 2 * (i16 & 1));
                    va[mk][s] = u32x4{lo[0], lo[1], hi[0], hi[1]};
                }
#pragma unroll
            for (int nb = 0; nb < 4; ++nb) {
#pragma unroll
                for (int mk = 0; mk < 4; ++mk) {
                    f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int s = 0; s < 2; ++s) {
                        acc = Mma<T>::k32(va[mk][s], whi[nb][s], acc);
                        acc = Mma<T>::k32(va[mk][s], wlo[nb][s], acc);
                    }
                    // element v: channel c0 + 16 mk + 4 g + v of child i16: 8 bytes, half (g % 2) of
                    // piece 2 mk + g / 2
                    *(u32x2 *)(oslot + piece_at(i16, 2 * mk + (g >> 1)) + 2 * (g & 1)) =
                        u32x2{pack2<T>(acc[0], acc[1]), pack2<T>(acc[2], acc[3])};
                }
                // (LDS operations of a wave complete in order: no wait between the writes above and
                // these reads beyond the one the compiler places for the data)
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    const int p = lane + 64 * i;
                    const u32x4 o = *(const u32x4 *)(oslot + piece_at(p >> 3, p & 7));
                    const u32 off = off_out[i] != OUTSIDE && c0 + ch_out[i] < C
                                        ? ((off_out[i] + (u32)(2 * nb * hW)) * (u32)C + (u32)(c0 + ch_out[i])) * (u32)sizeof(T)
                                        : OUTSIDE;
                    const bool row_ok = 2 * Y0 + 2 * nb + (p >> 6) < hH;
                    __builtin_amdgcn_raw_buffer_store_b128(o, ro, row_ok ? off : OUTSIDE, 0, STREAM_AUX);
                }
            }
        }
        landed_barrier(active);
        stage(j + 2);
    }
}

template <typename T, int NSW, bool STREAM>
static hipError_t launch_geom(const void *q, const void *key, const void *value, const void *qbias, void *out, int B, int d,
                              int C, int H, int W, hipStream_t st) {
    const int nsx = (W + 3) / 4;
    const int tiles_x = (nsx + NSW - 1) / NSW, tiles_y = (H + 3) / 4;
    const int ns = (nsx + tiles_x - 1) / tiles_x;             // blocks per tile, balanced over the row
    const long nb = (long)tiles_x * tiles_y * B;
    if (nb > (1L << 30)) return hipErrorNotSupported;
    const int per_xcd = (int)((nb + 7) / 8);
    if (qbias)
        hipLaunchKernelGGL((sapa_b_nhwc_wm16_kernel<T, NSW, STREAM, true>), dim3(per_xcd * 8), dim3(64 * NSW), 0, st,
                           (const T *)q, (const T *)key, (const T *)value, (const T *)qbias, (T *)out, d, C, H, W,
                           tiles_x, tiles_y, ns, (int)nb, per_xcd);
    else
        hipLaunchKernelGGL((sapa_b_nhwc_wm16_kernel<T, NSW, STREAM, false>), dim3(per_xcd * 8), dim3(64 * NSW), 0, st,
                           (const T *)q, (const T *)key, (const T *)value, (const T *)nullptr, (T *)out, d, C, H, W,
                           tiles_x, tiles_y, ns, (int)nb, per_xcd);
    return hipGetLastError();
}

}  // namespace cwm16

// Fused forward only (qbias: optional [B, d], aligned to 16 bytes); f16 / bf16, K = 5, s = 2, d and C multiples of 8, tensors
// aligned to 16 bytes, every image of every tensor below 2 GiB; hipErrorNotSupported otherwise.
hipError_t sapa_b_nhwc_wm16_launch(int mode, const void *q, const void *key, const void *value, const void *qbias,
                                   void *out, int B, int d, int C, int H, int W, int K, int s, int dtype,
                                   hipStream_t st) {
    if (mode != TILED_FUSED || K != 5 || s != 2 || d % 8 != 0 || C % 8 != 0) return hipErrorNotSupported;
    // small images: the kernel with a workgroup per 4 x 4 parents has four times the workgroups and a
    // shorter chain per workgroup (B=8, 32x32: 9 against 12 us; B=16, 25x42: 15 against 17 us; from
    // 64x64 on this one wins: 19 against 25 us).  By image size, not batch size: a batch and its images
    // one by one take the same kernel.
    if ((long)H * W < 2048) return hipErrorNotSupported;
    if (dtype != 2 && dtype != 3) return hipErrorNotSupported;
    if ((long)(d > C ? d : C) * H * W * 8 >= (1L << 31)) return hipErrorNotSupported;
    if (((uintptr_t)q | (uintptr_t)key | (uintptr_t)value | (uintptr_t)out | (uintptr_t)qbias) % 16 != 0)
        return hipErrorNotSupported;
    const bool stream = 2L * ((long)B * H * W * (5L * d + 5L * C)) > (256L << 20);
    if (dtype == 2)
        return stream ? cwm16::launch_geom<f16_t, 4, true>(q, key, value, qbias, out, B, d, C, H, W, st)
                      : cwm16::launch_geom<f16_t, 4, false>(q, key, value, qbias, out, B, d, C, H, W, st);
    return stream ? cwm16::launch_geom<bf16_t, 4, true>(q, key, value, qbias, out, B, d, C, H, W, st)
                  : cwm16::launch_geom<bf16_t, 4, false>(q, key, value, qbias, out, B, d, C, H, W, st);
}

}  // namespace sapa
