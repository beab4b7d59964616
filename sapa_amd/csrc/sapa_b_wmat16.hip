// Fused SAPA-B forward (qk -> softmax -> av) for contiguous (NCHW) f16 / bf16 tensors on the
// 16-bit matrix instructions, K = 5, s = 2.
//
// The 16 parents of a 4 x 4 block share one 8 x 8 window of low-res cells (block + halo of 2),
// and their 64 children need, each, 25 of those 64 cells.  Written over the whole window the two
// products are dense and small enough for the matrix pipe to do them many times over:
//
//   Sim[cell][child]  = sum_c key[c][cell] * q[c][child]            64 x 64 x d
//   P[child][cell]    = softmax over the child's 5 x 5 cells of Sim, 0 on the window's other cells
//   out[child][ch]    = sum_cell P[child][cell] * value[ch][cell]    64 x C x 64
//
// (reference: sapa/sapa/src/cuda/qk_cuda_kernel.cu:55-66, av_cuda_kernel.cu:52-66 and the
// softmax between them in sapa_base.py:38-40; the zero padding of the reference is the zero a
// cell outside the image holds here).  A wave owns one block; a workgroup of NSW waves owns up to
// NSW blocks side by side, so that the rows it writes are up to 8 * NSW children long.
//
// Layouts follow the tensors: NCHW planes are contiguous along x, which is the M / N index of
// every operand here, while the matrix instructions want the reduction index contiguous in a
// lane.  For the logits both operands reduce over channels: ds_read_tr16_b64 transposes 4
// channels x 16 positions on the way out of LDS.  For the aggregation the reduction runs over
// cells, which the value window holds contiguously (two 8-byte reads per operand), and the
// softmax result is already one lane per child with its cells in registers -- the accumulator
// layout of the first product is the A-operand layout of the second, so the weights never leave
// the registers.  They enter the product as a 16-bit value plus a 16-bit remainder (two
// instructions), the sums are fp32: the result is within half a 16-bit spacing of the exact one.
// The 4 x 4 output blocks go back through LDS so that global stores are 16 bytes per lane along
// whole tile rows.
//
// All global -> LDS traffic is direct (buffer loads with the LDS modifier, 16 bytes per lane); an
// offset of 2^31 is outside every descriptor and reads as zero, which is the zero padding above
// and below the image.  A window row starts 2 cells left of its block, so its 16-byte pieces are
// only 4-byte aligned in memory and the first / last of a row run over the row's ends: what they
// bring from the neighbouring row is put right in the registers (logit 0, weight 0 for a cell left
// of x = 0 or right of x = W - 1).  The q / output tile is stored with its 16-byte pieces
// XOR-swizzled so that transposing reads, accumulator writes and the linear store pass are all
// free of 4-way bank conflicts without padding.
//
// Masked cells still enter both products (a logit plus -inf, a weight of 0 times a value): a
// non-finite key or value spreads to every child of the 4 x 4 block whose window holds it rather
// than to the 25-cell neighbourhoods only.
#include "kernels.hpp"

namespace sapa {

namespace wm16 {

typedef unsigned u32;
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef u32 u32x2 __attribute__((ext_vector_type(2)));
typedef u32 u32x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));

constexpr int CHK = 16;            // channels per staged chunk
constexpr int WROWS = 8;           // window rows = child rows of a block row
constexpr u32 OUTSIDE = 0x80000000u;


template <typename T> struct Mma;
template <> struct Mma<f16_t> {
    typedef _Float16 v4 __attribute__((ext_vector_type(4)));
    typedef _Float16 v8 __attribute__((ext_vector_type(8)));
    static __device__ __forceinline__ f32x4 k16(u32x2 a, u32x2 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(v4, a), __builtin_bit_cast(v4, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4 k32(u32x4 a, u32x4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8, a), __builtin_bit_cast(v8, b), c, 0, 0, 0);
    }
};
template <> struct Mma<bf16_t> {
    typedef __bf16 v8 __attribute__((ext_vector_type(8)));
    static __device__ __forceinline__ f32x4 k16(u32x2 a, u32x2 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, a), __builtin_bit_cast(s16x4, b), c, 0, 0, 0);
    }
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

// 4 positions x 4 channels out of LDS, transposed: each lane of a 16-lane block addresses 4
// consecutive positions of one channel and receives one position's 4 channels
__device__ __forceinline__ u32x2 read_tr(const u32 *p) {
    return __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                                         (s16x4 __attribute__((address_space(3))) *)p));
}

// position of the 16-byte piece `pc` of row r, channel ch in the swizzled q / output tile
__device__ __forceinline__ int swz(int ch, int r) { return ((ch & 7) << 1) | ((r + (ch >> 3)) & 1); }

// STREAM: q loads and output stores are non-temporal -- each byte passes once and must not push the
// low-res windows, which neighbouring tiles re-read, out of the caches (fused FPN-large bf16, 860 MB:
// 271 -> 213 us; at a quarter of the size, where everything fits the memory-side cache, 50 -> 58 us:
// the launcher decides by size)
template <typename T, int NSW, bool STREAM>
__global__ __launch_bounds__(64 * NSW) void
sapa_b_wmat16_kernel(const T *__restrict__ q, const T *__restrict__ key, const T *__restrict__ value,
                     T *__restrict__ out, int d, int C, int H, int W, int tiles_x, int tiles_y, int ns,
                     int nblocks, int per_xcd) {
    constexpr int NT = 64 * NSW;
    constexpr int LROW = (4 * NSW + 4 + 7) / 8 * 4;          // dwords per staged window row: whole pieces of 8 cells
    constexpr int LOWBUF = WROWS * CHK * LROW;               // dwords per low-res buffer
    constexpr int NLP = LOWBUF / 4;                          // 16-byte pieces per low-res buffer
    constexpr int NLI = (NLP + NT - 1) / NT;                 // 16-byte direct loads per thread and window, at most
    constexpr int HIROW = 8 * NSW / 2;                       // dwords per q / output tile row
    constexpr int HICH = WROWS * HIROW;                      // dwords per channel of the tile
    constexpr int HIBUF = CHK * HICH;                        // dwords per q / output buffer
    constexpr int NHI = HIBUF / 4 / NT;                      // 16-byte pieces per thread and tile
    static_assert(HIBUF % (4 * NT) == 0 && NLP % 64 == 0, "whole direct loads");
    static_assert(4 * NSW + 4 <= 2 * LROW, "window row");
    static_assert(NSW == 16 || NSW == 8, "piece swizzle");
    constexpr int NPC = 2 * NSW / 2;                         // 16-byte pieces per tile row = NSW

    // two buffers of each kind (three, i.e. requests two chunks ahead, measured slower: 208 against
    // 199 us at FPN-large)
    __shared__ __attribute__((aligned(16))) u32 lds[2 * (LOWBUF + HIBUF)];
    u32 *const lowbuf = lds, *const hibuf = lds + 2 * LOWBUF;

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
    const u32 lplane = (u32)(lpix * sizeof(T)), hplane = 4 * lplane;

    // direct-load offsets inside one image, without the chunk's first channel.  A low-res piece is
    // 8 cells from x = X0 - 2 + 8 pc on: 4-byte aligned, and where it runs over an end of its row it
    // brings the neighbouring row's cells (zeros past the tensor's end) -- the cells left of x = 0
    // and right of x = W - 1 are put right in the registers below (cell_outside).  Only the piece
    // that starts 2 cells before the image's first has no address: it reads as zeros and its 6
    // cells are fetched apart (patch_low).
    u32 off_low[NLI], off_hi[NHI];
    bool half_piece[NHI];      // W % 4 == 2: a row's last 16-byte piece holds 4 of its children and 4 of the next row's
    int patch_slot = -1;
#pragma unroll
    for (int i = 0; i < NLI; ++i) {
        const int slot = i * NT + tid, rc = slot / (LROW / 4), pc = slot % (LROW / 4);
        const int r = rc / CHK, ch = rc % CHK;
        const int y = Y0 - 2 + r, x = X0 - 2 + 8 * pc;
        const bool ok = slot < NLP && 8 * pc < 4 * ns_here + 4 && y >= 0 && y < H && x < W;
        off_low[i] = ok ? (u32)(ch * lpix + (long)y * W + x) * (u32)sizeof(T) : OUTSIDE;
        if (ok && x < 0 && y == 0 && ch == 0) patch_slot = slot;
    }
#pragma unroll
    for (int i = 0; i < NHI; ++i) {
        const int slot = i * NT + tid, ch = slot / (WROWS * NPC), r = (slot / NPC) % WROWS;
        const int pc = (slot % NPC) ^ (swz(ch, r) & (NPC - 1));
        const int cy = 2 * Y0 + r, cx = 2 * X0 + 8 * pc;
        const bool ok = pc < ns_here && cy < 2 * H && cx < 2 * W;
        off_hi[i] = ok ? (u32)(ch * 4 * lpix + (long)cy * 2 * W + cx) * (u32)sizeof(T) : OUTSIDE;
        half_piece[i] = ok && cx + 8 > 2 * W;
    }

    const int nKc = (d + CHK - 1) / CHK, nVc = (C + CHK - 1) / CHK, ntot = nKc + nVc;
    const __amdgpu_buffer_rsrc_t rq = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(q + (long)n * d * 4 * lpix), 0, (int)(d * hplane), 0x00020000);
    const __amdgpu_buffer_rsrc_t rk = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(key + (long)n * d * lpix), 0, (int)(d * lplane), 0x00020000);
    const __amdgpu_buffer_rsrc_t rv = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(value + (long)n * C * lpix), 0, (int)(C * lplane), 0x00020000);
    const __amdgpu_buffer_rsrc_t ro = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(out + (long)n * C * 4 * lpix), 0, (int)(C * hplane), 0x00020000);

    (void)rq, (void)rk, (void)rv;
    // Chunk j is the key + q channels 16 j .. for j < nKc and the value channels 16 (j - nKc) ..
    // after; it lives in buffer j % 2 and is requested two chunks ahead, as soon as every wave is
    // done with that buffer.  A channel past the tensor's last lies past the descriptor: zeros.
    auto stage_low = [&](__amdgpu_buffer_rsrc_t r, u32 c0, int buf) __attribute__((always_inline)) {
#if defined(__HIP_DEVICE_COMPILE__)
        u32 *lb = lowbuf + buf * LOWBUF + wave * 256;
#pragma unroll
        for (int i = 0; i < NLI; ++i)
            if ((i + 1) * NT <= NLP || i * NT + wave * 64 < NLP)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (__attribute__((address_space(3))) void *)(lb + i * NT * 4), 16,
                                                         off_low[i] + c0 * lplane, 0, 0, 0);
#endif
    };
    auto stage_q = [&](u32 c0, int buf) __attribute__((always_inline)) {
#if defined(__HIP_DEVICE_COMPILE__)
        u32 *hb = hibuf + buf * HIBUF + wave * 256;
#pragma unroll
        for (int i = 0; i < NHI; ++i)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rq, (__attribute__((address_space(3))) void *)(hb + i * NT * 4), 16,
                                                     off_hi[i] + c0 * hplane, 0, 0, STREAM ? 2 : 0);
#endif
    };
    auto stage = [&](int j) __attribute__((always_inline)) {
        if (j < nKc) {
            stage_low(rk, (u32)(j * CHK), j & 1);
            stage_q((u32)(j * CHK), j & 1);
        } else if (j < ntot) {
            stage_low(rv, (u32)((j - nKc) * CHK), j & 1);
        }
    };
    // Waits are counted: the counter of vector-memory operations retires in issue order, so
    // "at most N outstanding" means that everything but the last N issued is complete.  Written out
    // because the compiler does not track a direct load's LDS write.
    auto wait_all_but = [&](int after) __attribute__((always_inline)) {
#if defined(__HIP_DEVICE_COMPILE__)
#define SAPA_WM16_WAIT(N) case N: asm volatile("s_waitcnt vmcnt(" #N ")" ::: "memory"); break;
        switch (after) {
            SAPA_WM16_WAIT(1) SAPA_WM16_WAIT(2) SAPA_WM16_WAIT(3) SAPA_WM16_WAIT(4)
            default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
        }
#undef SAPA_WM16_WAIT
#endif
    };
    // chunk jn (the first of the keys or of the values) has landed in this wave's slots: the 6
    // cells of the piece that has no address (first row of the image's first channel, tile at the
    // left edge)
    auto patch_low = [&](int jn) __attribute__((always_inline)) {
        if (tx == 0 && ty == 0 && patch_slot >= 0) {
            const __amdgpu_buffer_rsrc_t r = jn < nKc ? rk : rv;
            u32 *dst = lowbuf + (jn & 1) * LOWBUF + patch_slot * 4;
#pragma unroll
            for (int k = 1; k < 4; ++k) dst[k] = __builtin_amdgcn_raw_buffer_load_b32(r, 4 * (k - 1), 0, 0);
        }
    };
    // this wave's LDS writes are done; then every wave's (and every wave's landed loads)
    auto barrier = [&]() __attribute__((always_inline)) {
#if defined(__HIP_DEVICE_COMPILE__)
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
#endif
    };

    const bool row_tail = (W & 3) != 0 && X0 + 4 * ns_here > W;      // wave-uniform
    const bool active = wave < ns_here;
    const int t = wave;                                       // this wave's block of the tile

    stage(0);
    stage(1);
    // chunk 0: all but chunk 1's loads
    wait_all_but(ntot < 2 ? 0 : (NLP - wave * 64 + NT - 1) / NT + (1 < nKc ? NHI : 0));
    patch_low(0);
    barrier();

    // ---- logits: Sim[cell][child], 4 x 4 accumulator blocks of 16 x 16 ----
    // block (mb, nb), lane (g, i16), element v: cell (row 2 mb + g / 2, column 4 (g % 2) + v) of the
    // window, child (row 2 nb + i16 / 8, column i16 % 8) of the block's 8 x 8 children
    f32x4 sim[4][4];
#pragma unroll
    for (int mb = 0; mb < 4; ++mb)
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) sim[mb][nb] = f32x4{0.f, 0.f, 0.f, 0.f};
    // transposing reads: lane (g, L = i16) addresses channel 4 g + L / 4, the 4 positions of group
    // L % 4 of the 16 (row (L % 4) / 2 of the pair, columns 4 (L % 2) ..)
    const int tch = 4 * g + (i16 >> 2), trow = (i16 & 3) >> 1, tcol = i16 & 1;
    for (int j = 0; j < nKc; ++j) {
        if (active) {
            const u32 *kb = lowbuf + (j & 1) * LOWBUF, *qb = hibuf + (j & 1) * HIBUF;
            u32x2 a[4], b[4];
#pragma unroll
            for (int mb = 0; mb < 4; ++mb)
                a[mb] = read_tr(kb + ((2 * mb + trow) * CHK + tch) * LROW + 2 * t + 2 * tcol);
#pragma unroll
            for (int nb = 0; nb < 4; ++nb) {
                const int r = 2 * nb + trow;
                b[nb] = read_tr(qb + tch * HICH + r * HIROW + ((t ^ (swz(tch, r) & (NPC - 1))) << 2) + 2 * tcol);
            }
#pragma unroll
            for (int mb = 0; mb < 4; ++mb)
#pragma unroll
                for (int nb = 0; nb < 4; ++nb) sim[mb][nb] = Mma<T>::k16(a[mb], b[nb], sim[mb][nb]);
        }
        // chunk j + 1: nothing was issued after its loads
        wait_all_but(0);
        if (j + 1 == nKc) patch_low(nKc);
        barrier();
        stage(j + 2);
    }

    // ---- softmax over each child's 5 x 5 cells; the weights as A operands of the aggregation ----
    // reduction step s of the aggregation covers the cells of blocks mb = 2 s, 2 s + 1; lane
    // (g, child) holds 4 + 4 of its 32
    u32x4 whi[4][2], wlo[4][2];
    if (active) {
        // element v of every block is window column 4 (g % 2) + v.  Outside the image the key is zero
        // (logit 0) and so is the value (the weight may as well be 0): only the waves at a row's
        // ends have such columns.
        bool cell_outside[4];
#pragma unroll
        for (int v = 0; v < 4; ++v) cell_outside[v] = (u32)(X0 + 4 * t - 2 + 4 * (g & 1) + v) >= (u32)W;
        const bool at_row_end = X0 + 4 * t - 2 < 0 || X0 + 4 * t + 5 >= W;      // wave-uniform
        if (at_row_end) {
#pragma unroll
            for (int mb = 0; mb < 4; ++mb)
#pragma unroll
                for (int nb = 0; nb < 4; ++nb)
#pragma unroll
                    for (int v = 0; v < 4; ++v)
                        if (cell_outside[v]) sim[mb][nb][v] = 0.f;
        }
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
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                float p[8];
#pragma unroll
                for (int k = 0; k < 8; ++k) p[k] = e[2 * s + k / 4][k % 4] * inv;
                if (at_row_end) {
#pragma unroll
                    for (int k = 0; k < 8; ++k)
                        if (cell_outside[k % 4]) p[k] = 0.f;
                }
                typedef T tx8 __attribute__((ext_vector_type(8)));
                whi[nb][s] = u32x4{pack2<T>(p[0], p[1]), pack2<T>(p[2], p[3]), pack2<T>(p[4], p[5]), pack2<T>(p[6], p[7])};
                const tx8 hi = __builtin_bit_cast(tx8, whi[nb][s]);
#pragma unroll
                for (int k = 0; k < 8; ++k) p[k] -= (float)hi[k];
                wlo[nb][s] = u32x4{pack2<T>(p[0], p[1]), pack2<T>(p[2], p[3]), pack2<T>(p[4], p[5]), pack2<T>(p[6], p[7])};
            }
        }
    }

    // ---- aggregation: out[child][channel], per chunk of 16 channels ----
    for (int j = nKc; j < ntot; ++j) {
        const u32 c0 = (u32)((j - nKc) * CHK);
        u32 *ob = hibuf + (j & 1) * HIBUF;                      // no loads into this ring any more
        if (active) {
            const u32 *vb = lowbuf + (j & 1) * LOWBUF;
            // B operand of step s: lane (g, channel i16) holds the cells of rows 4 s + g / 2 and
            // 4 s + 2 + g / 2, columns 4 (g % 2) .. + 3 -- the order the weights are held in
            u32x4 b[2];
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                const u32 *p = vb + ((4 * s + (g >> 1)) * CHK + i16) * LROW + 2 * t + 2 * (g & 1);
                const u32x2 lo = *(const u32x2 *)p, hi = *(const u32x2 *)(p + 2 * CHK * LROW);
                b[s] = u32x4{lo[0], lo[1], hi[0], hi[1]};
            }
#pragma unroll
            for (int nb = 0; nb < 4; ++nb) {
                f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    acc = Mma<T>::k32(whi[nb][s], b[s], acc);
                    acc = Mma<T>::k32(wlo[nb][s], b[s], acc);
                }
                // element v: child (row 2 nb + g / 2, column 4 (g % 2) + v), channel c0 + i16
                const int r = 2 * nb + (g >> 1);
                *(u32x2 *)(ob + i16 * HICH + r * HIROW + ((t ^ (swz(i16, r) & (NPC - 1))) << 2) + 2 * (g & 1)) =
                    u32x2{pack2<T>(acc[0], acc[1]), pack2<T>(acc[2], acc[3])};
            }
        }
        // chunk j + 1: its loads were the last operations issued
#if defined(__HIP_DEVICE_COMPILE__)
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#endif
        barrier();
        // the tile's 16 channels x 8 rows, 16 bytes per lane, right after the barrier that completes
        // them (sending them behind the next chunk's matrix instructions measured slower); a piece
        // outside the tensor (ragged tile, channel past the last) lies outside the descriptor and
        // is dropped
#pragma unroll
        for (int i = 0; i < NHI; ++i) {
            const u32x4 o = *(const u32x4 *)(ob + (i * NT + tid) * 4);
            u32 off = off_hi[i] + c0 * hplane;
            if (row_tail && half_piece[i]) {
                __builtin_amdgcn_raw_buffer_store_b64(u32x2{o[0], o[1]}, ro, off, 0, 0);
                off = OUTSIDE;
            }
            if constexpr (STREAM) __builtin_amdgcn_raw_buffer_store_b128(o, ro, off, 0, 2);
            else __builtin_amdgcn_raw_buffer_store_b128(o, ro, off, 0, 0);
        }
        // (the next request behind the stores: 208 us at FPN-large against 216 with the loads first)
        if (j + 2 < ntot) stage_low(rv, (u32)((j + 2 - nKc) * CHK), j & 1);
    }
}

template <typename T, int NSW, bool STREAM>
static hipError_t launch_geom(const void *q, const void *key, const void *value, void *out, int B, int d,
                              int C, int H, int W, hipStream_t st) {
    const int nsx = (W + 3) / 4;
    const int tiles_x = (nsx + NSW - 1) / NSW, tiles_y = (H + 3) / 4;
    const int ns = (nsx + tiles_x - 1) / tiles_x;             // blocks per tile, balanced over the row
    const long nb = (long)tiles_x * tiles_y * B;
    if (nb > (1L << 30)) return hipErrorNotSupported;
    const int per_xcd = (int)((nb + 7) / 8);
    hipLaunchKernelGGL((sapa_b_wmat16_kernel<T, NSW, STREAM>), dim3(per_xcd * 8), dim3(64 * NSW), 0, st, (const T *)q,
                       (const T *)key, (const T *)value, (T *)out, d, C, H, W, tiles_x, tiles_y, ns, (int)nb,
                       per_xcd);
    return hipGetLastError();
}

}  // namespace wm16

// Fused forward only; f16 / bf16, K = 5, s = 2, W even (rows of whole dwords), low-res tensors 4-byte and
// high-res tensors 16-byte aligned, every image of every tensor below 2 GiB (32-bit offsets
// inside an image); hipErrorNotSupported otherwise.
hipError_t sapa_b_wmat16_launch(int mode, const void *q, const void *key, const void *value, void *out, int B,
                                int d, int C, int H, int W, int K, int s, int dtype, hipStream_t st) {
    if (mode != TILED_FUSED || K != 5 || s != 2 || W % 2 != 0 || W < 16) return hipErrorNotSupported;
    if (dtype != 2 && dtype != 3) return hipErrorNotSupported;
    const long hplane = (long)H * W * 8;
    if ((long)(d > C ? d : C) * hplane >= (1L << 31)) return hipErrorNotSupported;
    if (((uintptr_t)key | (uintptr_t)value) % 4 != 0 || ((uintptr_t)q | (uintptr_t)out) % 16 != 0)
        return hipErrorNotSupported;
    // bytes read and written once; beyond the 256 MB memory-side cache they are streamed, in tiles of
    // up to 16 blocks (longer rows per store); what fits the cache takes tiles of 8 blocks, two
    // workgroups per CU (FPN 25x42 at B=16: 24 -> 19 us, SegFormer 64x64 at B=8: 25 -> 20 us).  The
    // arithmetic of a child does not depend on the tiling: results are the same bit for bit.
    const bool stream = 2L * ((long)B * H * W * (5L * d + 5L * C)) > (256L << 20);
    if (dtype == 2)
        return stream ? wm16::launch_geom<f16_t, 16, true>(q, key, value, out, B, d, C, H, W, st)
                      : wm16::launch_geom<f16_t, 8, false>(q, key, value, out, B, d, C, H, W, st);
    return stream ? wm16::launch_geom<bf16_t, 16, true>(q, key, value, out, B, d, C, H, W, st)
                  : wm16::launch_geom<bf16_t, 8, false>(q, key, value, out, B, d, C, H, W, st);
}

}  // namespace sapa
