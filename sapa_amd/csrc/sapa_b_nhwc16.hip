// SAPA-B for fp16 / bf16 tensors in channels-last memory order on the 16-bit
// matrix instructions: qk, qk+softmax, av and the fused qk -> softmax -> av
// forward, (K, s) in {(3,2), (5,2), (7,2), (5,4), (7,4)}.
//
// Same decomposition as the fp32-in-LDS kernel of sapa_b_nhwc.hip -- a row of
// 16 lanes owns one low-res parent with its s x s children, a wave 4 parents
// that are neighbours in x, a workgroup of 4 waves a tile of 4 x 4 parents;
// key and value windows go through LDS one 64-channel chunk at a time,
// double-buffered -- but the windows stay 16-bit in LDS and both products run
// as v_mfma_f32_4x4x4 (16 independent blocks of 4 lanes, each D(4x4) +=
// A(4x4) B(4x4) with 4 x 16-bit operands per lane, fp32 accumulation):
//
//   * logits: A = key, B = q, the reduction index = 4 channels.  Lane (b, i)
//     of a row (b = lane quad 0..3, i = lane in the quad) supplies, as A, the
//     key of tap 4 tau + i and, as B, the q of child i, both for the 16
//     channels of quad b (4 instructions per tap group tau); lane (b, j) then
//     holds [tap 4 tau + i][child j] for i = 0..3, summed over those 16
//     channels.  Two butterfly steps over the 4 quads of the row (halving the
//     live values at each step) finish the sum and leave tap 4 tau + b of child
//     j in lane (b, j): K*K logits per child in ceil(K*K / 4) registers;
//   * softmax per child over its registers and the 4 quads of the row;
//   * aggregation: A = the weights, rounded to the tensors' 16-bit type, of 4
//     taps (4 consecutive registers of a lane, packed), B = the value of those
//     4 taps for one channel of the lane, the reduction index = the 4 taps.  The
//     weights of taps 4 m + b live in quad b only; the instruction's A
//     broadcast (cbsz = 2: one quad feeds the row of 16 lanes, abid = b picks
//     it) hands them to the whole row.  A lane reads its 4 channels of the 4 taps
//     (8 bytes each) and transposes the 4 x 4 block with 8 byte permutes into
//     the 4 B operands (one per channel).
//
// LDS: [position][64 channels] of 16-bit values, positions 192 bytes apart:
// the logits' 16-byte reads (a quad's lanes read 4 consecutive taps, the 4
// quads 4 channel blocks) then fall on disjoint banks.
//
// Numerics: products of 16-bit values are exact in fp32; the sums run in the
// matrix pipe's order.  In the fused mode the softmax weights enter the
// aggregation as hi + lo pairs of 16-bit numbers (two instructions per B
// operand), i.e. with fp32-like precision: only the inputs and the result are
// 16-bit.  av() on its own takes the 16-bit weights it is given.
#include <utility>

#include "kernels.hpp"

namespace sapa {

namespace nhwc16 {

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>)
template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

typedef unsigned u32;
typedef u32 u32x2 __attribute__((ext_vector_type(2)));
typedef u32 u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// c += a * b over 16 blocks of 4 lanes; a, b: 4 x 16-bit per lane.  CBSZ / ABID:
// the A operand of block ABID of every group of 2^CBSZ blocks serves the group.
template <typename T> struct Mma;
template <> struct Mma<f16_t> {
    typedef _Float16 v4 __attribute__((ext_vector_type(4)));
    template <int CBSZ, int ABID>
    static __device__ __forceinline__ f32x4 run(u32x2 a, u32x2 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(v4, a), __builtin_bit_cast(v4, b),
                                                  c, CBSZ, ABID, 0);
    }
};
template <> struct Mma<bf16_t> {
    typedef short v4 __attribute__((ext_vector_type(4)));
    template <int CBSZ, int ABID>
    static __device__ __forceinline__ f32x4 run(u32x2 a, u32x2 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(v4, a),
                                                      __builtin_bit_cast(v4, b), c, CBSZ, ABID, 0);
    }
};

// two floats -> two T (round to nearest even) in one dword
template <typename T>
__device__ __forceinline__ u32 pack2(float a, float b) {
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    typedef T tx2 __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(u32, __builtin_convertvector(f32x2{a, b}, tx2));
}

// value of lane (l ^ D) of the same row of 16 lanes, D = 4 or 8
template <int D>
__device__ __forceinline__ float row_xor(float v, int lane) {
    union { float f; int i; } x, y;
    x.f = v;
    y.i = __builtin_amdgcn_ds_bpermute((lane ^ D) << 2, x.i);
    return y.f;
}
// One butterfly step over lane distance D: n values per lane -> n / 2.  The lane
// whose bit D is clear keeps the even-indexed sums, its partner the odd-indexed
// ones; each adds what the other held of them.  FROM_VALU: the inputs were written by
// ordinary vector instructions -- then two DPP additions per result do it
// (pair_sum_dpp, whose wait states cover those, not a matrix instruction's result).
template <int D, int N, bool FROM_VALU>
__device__ __forceinline__ void halve(const float (&in)[N], float (&out)[N / 2], int lane) {
    const bool hi = lane & D;
    (void)hi;
#pragma unroll
    for (int m = 0; m < N / 2; ++m) {
        const float a = in[2 * m], b = in[2 * m + 1];
        if constexpr (SAPA_NHWC_DPP_HALVE && FROM_VALU) {
            out[m] = pair_sum_dpp<D>(a, b);
        } else {
            const float keep = hi ? b : a, send = hi ? a : b;
            out[m] = keep + row_xor<D>(send, lane);
        }
    }
}

// QB: the query bias is given (its own instantiation: the bias costs 8 registers)
template <typename T, int K, int S, int QX, int TY, int MODE, bool QB>
__global__ void __launch_bounds__(64 * QX * TY)
sapa_b_nhwc16_kernel(const T *__restrict__ q, const T *__restrict__ key,
                     const T *__restrict__ attn_in, const T *__restrict__ value,
                     const T *__restrict__ qbias, T *__restrict__ out, int d, int C, int H, int W,
                     int tiles_x, int tiles_y, int nblocks, int per_xcd) {
    static_assert(S == 2 || S == 4, "children are handled in groups of 4");
    // children j = cy * S + cx of a parent, in NG groups of 4 (s = 2: all four;
    // s = 4: one child row per group)
    constexpr int NJ = S * S, NG = NJ / 4, KK = K * K, R = (K - 1) / 2;
    constexpr int TX = 4 * QX;                    // tile: TX x TY parents, QX waves per row
    constexpr int WW = TX + K - 1, WH = TY + K - 1, NPOS = WW * WH;   // window positions
    constexpr int CHK = 64;                       // channels per chunk
    constexpr int PSW = 48;                       // dwords between positions in LDS (32 of data)
    constexpr int BUF = NPOS * PSW;               // dwords per LDS buffer
    constexpr int NT = 64 * QX * TY, NPASS = (NPOS * 16 + NT - 1) / NT;   // staging passes (16 quads per position)
    constexpr int NTAU = (KK + 3) / 4;            // taps in groups of 4: weight registers per child
    constexpr int NGRP = (NTAU + 3) / 4;          // those registers in packs of 4
    constexpr int NR = NG * NTAU;
    constexpr bool DO_QK = MODE != TILED_AV;
    constexpr bool DO_SOFTMAX = MODE == TILED_QK_SOFTMAX || MODE == TILED_FUSED;
    constexpr bool DO_AV = MODE == TILED_AV || MODE == TILED_FUSED;
    typedef Mma<T> M;

    // The windows go from global memory straight into LDS (buffer loads with the LDS modifier:
    // lane l of a wave's load fills the 16-byte slot l of 64 consecutive ones, 12 slots per
    // position of which 8 hold its 64 channels): no staging registers, no LDS write
    // instructions.  A buffer is a whole number of 64-slot blocks.
#ifndef SAPA_NHWC16_DMA
#define SAPA_NHWC16_DMA 1
#endif
    constexpr bool DMA = SAPA_NHWC16_DMA;
    constexpr int SPP = PSW / 4;                                  // 16-byte slots per position
    constexpr int BUFA = DMA ? (BUF + 255) / 256 * 256 : BUF;     // dwords per buffer
    constexpr int NPD = (NPOS * SPP + NT - 1) / NT;               // direct loads per thread and chunk
    static_assert(PSW % 4 == 0 && CHK == 64, "slot layout");
    __shared__ __attribute__((aligned(16))) u32 lds[2 * BUFA];

    const int logical = (int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8);
    if (logical >= nblocks) return;
    const int tx = logical % tiles_x;
    const int ty = (logical / tiles_x) % tiles_y;
    const int n = logical / (tiles_x * tiles_y);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int row = lane >> 4, li = lane & 15;    // parent within the wave, lane in the row
    const int jl = li & 3, bq = li >> 2;          // lane in its quad, quad in the row
    const int x0 = tx * TX, y0 = ty * TY;
    const int wx = wave % QX, wy = wave / QX;     // this wave's 4 parents in the tile
    const int px = x0 + 4 * wx + row, py = y0 + wy;
    const bool active = px < W && py < H;
    const int hW = W * S;
    const long lpix = (long)H * W, hpix = lpix * S * S;

    const int nKc = DO_QK ? (d + CHK - 1) / CHK : 0;
    const int nVc = DO_AV ? (C + CHK - 1) / CHK : 0;
    const int ntot = nKc + nVc;

    // ---- staging: pass p, thread t moves channel quad t % 16 of window position
    // p * 16 + t / 16 (8 bytes).  Offset 2^31 marks a position outside the image
    // (beyond every descriptor: zero fill).
    int spix[NPASS];
#pragma unroll
    for (int p = 0; p < NPASS; ++p) {
        const int pos = p * (NT / 16) + tid / 16;
        const int gy = y0 - R + pos / WW, gx = x0 - R + pos % WW;
        spix[p] = (pos < NPOS && gy >= 0 && gy < H && gx >= 0 && gx < W) ? gy * W + gx : -1;
    }
    const int sq = tid & 15;
    // direct loads: pass p, thread t fills slot p * NT + t = 8 channels (slot % SPP < 8) of
    // position slot / SPP; dpix: the position's pixel, -1 outside the image / for a spare
    // slot / past the window
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    (void)wave_u;
    int dpix[NPD], dq8[NPD];
#pragma unroll
    for (int p = 0; p < NPD; ++p) {
        const int slot = p * NT + tid, pos = slot / SPP;
        dq8[p] = slot % SPP;
        const int gy = y0 - R + pos / WW, gx = x0 - R + pos % WW;
        dpix[p] = (pos < NPOS && dq8[p] < 8 && gy >= 0 && gy < H && gx >= 0 && gx < W) ? gy * W + gx : -1;
    }
    // one chunk's loads from per-thread offsets `off`; (device pass only: the host pass, which
    // sees this body for the launch stub, does not know the builtin)
    auto direct_loads = [&](__amdgpu_buffer_rsrc_t r, int j, const u32 (&off)[NPD]) __attribute__((always_inline)) {
#if defined(__HIP_DEVICE_COMPILE__)
#pragma unroll
        for (int p = 0; p < NPD; ++p) {
            const int slot0 = p * NT + wave_u * 64;
            if ((p + 1) * NT <= NPOS * SPP || slot0 < NPOS * SPP)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(
                    r, (__attribute__((address_space(3))) void *)(lds + (j & 1) * BUFA + slot0 * 4), 16, off[p], 0, 0, 0);
        }
#endif
    };
    u32x2 st[NPASS];
    auto stage_load = [&](int j) __attribute__((always_inline)) {
        const bool is_key = j < nKc;
        const int nch = is_key ? d : C;
        const int c0 = (is_key ? j : j - nKc) * CHK;
        const T *base = (is_key ? key : value) + (long)n * lpix * nch;
        const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(
            (void *)base, 0, (int)(lpix * nch * (long)sizeof(T)), 0x00020000);
        if constexpr (DMA) {
            u32 off[NPD];
#pragma unroll
            for (int p = 0; p < NPD; ++p) {
                const u32 c_bad = (u32)(nch - 1 - (c0 + 8 * dq8[p]));
                off[p] = ((u32)(dpix[p] * nch + c0 + 8 * dq8[p]) * (u32)sizeof(T)) |
                         ((c_bad | (u32)dpix[p]) & 0x80000000u);
            }
            direct_loads(r, j, off);
            return;
        }
        // bit 31 set = past the descriptor; pure arithmetic (sign bits of "channel
        // within the tensor" and "position within the image") instead of selects
        const u32 c_bad = (u32)(nch - 1 - (c0 + 4 * sq));
#pragma unroll
        for (int p = 0; p < NPASS; ++p) {
            const u32 off = ((u32)(spix[p] * nch + c0 + 4 * sq) * (u32)sizeof(T)) |
                            ((c_bad | (u32)spix[p]) & 0x80000000u);
            st[p] = __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, 0);
        }
    };
    // the same for value chunk jv from offsets prepared once (voff0, set up before
    // the aggregation): two instructions per load instead of the full address
    u32 voff0[DMA ? NPD : NPASS];
    auto stage_load_value = [&](int jv) __attribute__((always_inline)) {
        const T *base = value + (long)n * lpix * C;
        const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(
            (void *)base, 0, (int)(lpix * C * (long)sizeof(T)), 0x00020000);
        if constexpr (DMA) {
            u32 off[NPD];
#pragma unroll
            for (int p = 0; p < NPD; ++p)
                off[p] = (voff0[p] + (u32)(jv * CHK) * (u32)sizeof(T)) |
                         ((u32)(C - 1 - (jv * CHK + 8 * dq8[p])) & 0x80000000u);
            direct_loads(r, nKc + jv, off);
            return;
        }
        const u32 c_bad = (u32)(C - 1 - (jv * CHK + 4 * sq)) & 0x80000000u;
#pragma unroll
        for (int p = 0; p < NPASS; ++p)
            st[p] = __builtin_amdgcn_raw_buffer_load_b64(
                r, (voff0[p] + (u32)(jv * CHK) * (u32)sizeof(T)) | c_bad, 0, 0);
    };
    // registers -> LDS; direct loads: wait for them (the counter retires in issue order, so
    // that is a wait for everything issued before them as well)
    auto stage_store = [&](int j) __attribute__((always_inline)) {
        if constexpr (DMA) {
#if defined(__HIP_DEVICE_COMPILE__)
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#endif
            return;
        }
        u32 *dst = lds + (j & 1) * BUFA;
#pragma unroll
        for (int p = 0; p < NPASS; ++p) {
            const int pos = p * (NT / 16) + tid / 16;
            if (NPOS % (NT / 16) == 0 || pos < NPOS) *(u32x2 *)(dst + pos * PSW + 2 * sq) = st[p];
        }
    };

    // every wave is done with the current window and the next one is in LDS (direct loads:
    // the bare barrier instruction -- the loads were waited for in stage_store, and a fence
    // here would drain the output stores issued since)
    auto chunk_barrier = [&]() __attribute__((always_inline)) {
        if constexpr (DMA) {
#if defined(__HIP_DEVICE_COMPILE__)
            asm volatile("s_barrier" ::: "memory");
#endif
        } else {
            __syncthreads();
        }
    };
    // this row's window origin: tap (ky, kx) of its parent sits at position
    // (wy + ky) * WW + 4 wx + row + kx.  Aggregation: lane li reads channels
    // 4 li .. 4 li + 3 (dwords 2 li, 2 li + 1 of the position); logits: lane
    // (bq, jl) reads channels 8 bq .. +7 and 32 + 8 bq .. +7 (dwords 4 bq .. +3 and
    // 16 + 4 bq .. +3) of tap 4 tau + jl
    const u32 *win = lds + ((wy * WW + 4 * wx + row) * PSW + 2 * li);
    const u32 *kwin = lds + ((wy * WW + 4 * wx + row) * PSW + 4 * bq);
    int kofs[NTAU];
#pragma unroll
    for (int tau = 0; tau < NTAU; ++tau) {
        const int t = min(4 * tau + jl, KK - 1);
        kofs[tau] = ((t / K) * WW + t % K) * PSW;
    }

    // logits, then weights: w[g * NTAU + m] of lane (bq, jl) belongs to child jl
    // of group g and tap 4 m + bq; ok[m]: that tap exists
    float w[NR];
    bool ok[NTAU];
#pragma unroll
    for (int m = 0; m < NTAU; ++m) ok[m] = 4 * m + bq < KK;
    // child j of this row's parent: its pixel in a [B, sH, sW, n_ch] tensor
    auto child_pixel = [&](int j) __attribute__((always_inline)) {
        return (long)n * hpix + (long)(py * S + j / S) * hW + (long)px * S + j % S;
    };
    // q of child jl of group g: channels 8 bq .. +7 and 32 + 8 bq .. +7 of key chunk j
    // (zeros past d and for idle rows; d is a multiple of 8)
    u32x4 qraw[2];
    auto load_q = [&](int j, int g) __attribute__((always_inline)) {
        const int c0 = j * CHK + 8 * bq;
        const T *qp = q + child_pixel(g * 4 + jl) * d + c0;
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            qraw[e] = u32x4{0u, 0u, 0u, 0u};
            if (active && c0 + 32 * e < d) qraw[e] = __builtin_nontemporal_load((const u32x4 *)(qp + 32 * e));
        }
    };
    if (DO_QK) load_q(0, 0);
    stage_load(0);
    stage_store(0);
    chunk_barrier();

    if (DO_QK) {
#pragma unroll
        for (int i = 0; i < NR; ++i) w[i] = 0.f;
        for (int j = 0; j < nKc; ++j) {
            if (j + 1 < ntot) stage_load(j + 1);
            const u32 *kb = kwin + (j & 1) * BUFA;
            // optional per-image bias of the query projection [B, d]: key . (q + b) =
            // key . q + key . b, the second product as four more instructions per tap
            // group with the bias as the B operand (same for the four children)
            u32x4 qb0 = {0u, 0u, 0u, 0u}, qb1 = {0u, 0u, 0u, 0u};
            if (QB) {
                const T *bp = qbias + (long)n * d + j * CHK + 8 * bq;
                if (j * CHK + 8 * bq < d) qb0 = *(const u32x4 *)bp;
                if (j * CHK + 8 * bq + 32 < d) qb1 = *(const u32x4 *)(bp + 32);
            }
#pragma unroll
            for (int g = 0; g < NG; ++g) {
                const u32x4 q0 = qraw[0], q1 = qraw[1];
                // the next group's (or chunk's) q while this one is used
                if (g + 1 < NG) load_q(j, g + 1);
                else if (j + 1 < nKc) load_q(j + 1, 0);
                static_for<NTAU>([&](auto itau) __attribute__((always_inline)) {
                    constexpr int tau = decltype(itau)::value;
                    const u32 *kp = kb + kofs[tau];
                    const u32x4 k0 = *(const u32x4 *)kp, k1 = *(const u32x4 *)(kp + 16);
                    f32x4 a = f32x4{0.f, 0.f, 0.f, 0.f};
                    a = M::template run<0, 0>(u32x2{k0[0], k0[1]}, u32x2{q0[0], q0[1]}, a);
                    a = M::template run<0, 0>(u32x2{k0[2], k0[3]}, u32x2{q0[2], q0[3]}, a);
                    a = M::template run<0, 0>(u32x2{k1[0], k1[1]}, u32x2{q1[0], q1[1]}, a);
                    a = M::template run<0, 0>(u32x2{k1[2], k1[3]}, u32x2{q1[2], q1[3]}, a);
                    if (QB) {
                        a = M::template run<0, 0>(u32x2{k0[0], k0[1]}, u32x2{qb0[0], qb0[1]}, a);
                        a = M::template run<0, 0>(u32x2{k0[2], k0[3]}, u32x2{qb0[2], qb0[3]}, a);
                        a = M::template run<0, 0>(u32x2{k1[0], k1[1]}, u32x2{qb1[0], qb1[1]}, a);
                        a = M::template run<0, 0>(u32x2{k1[2], k1[3]}, u32x2{qb1[2], qb1[3]}, a);
                    }
                    // a[i]: tap 4 tau + i times child jl over the 16 channels of quad bq;
                    // summed over the 4 quads, tap 4 tau + bq stays in this lane
                    const float flat[4] = {a[0], a[1], a[2], a[3]};
                    float h1[2], h2[1];
                    halve<4, 4, false>(flat, h1, lane);    // (inputs: a matrix instruction's result)
                    halve<8, 2, true>(h1, h2, lane);
                    w[g * NTAU + tau] += h2[0];
                    // keeps the reads of at most two tap groups in flight (registers)
                    if (tau % 2 == 1) __builtin_amdgcn_sched_barrier(0);
                });
            }
            if (j + 1 < ntot) stage_store(j + 1);
            chunk_barrier();
        }
        if (DO_SOFTMAX) {
            // a child's taps lie in this lane's registers of its group and in the
            // lanes at distance 4, 8, 12
#pragma unroll
            for (int g = 0; g < NG; ++g) {
                float mx = w[g * NTAU];            // tap bq < K * K always
#pragma unroll
                for (int m = 0; m < NTAU; ++m)
                    if (ok[m]) mx = max_(mx, w[g * NTAU + m]);
                if constexpr (SAPA_NHWC_DPP_HALVE) {
                    mx = xor_max_dpp<4>(mx);
                    mx = xor_max_dpp<8>(mx);
                } else {
                    mx = max_(mx, row_xor<4>(mx, lane));
                    mx = max_(mx, row_xor<8>(mx, lane));
                }
                float sum = 0.f;
#pragma unroll
                for (int m = 0; m < NTAU; ++m) {
                    float &x = w[g * NTAU + m];
                    x = ok[m] ? exp_(x - mx) : 0.f;
                    sum += x;
                }
                if constexpr (SAPA_NHWC_DPP_HALVE) {
                    sum = pair_sum_dpp<4>(sum, sum);
                    sum = pair_sum_dpp<8>(sum, sum);
                } else {
                    sum += row_xor<4>(sum, lane);
                    sum += row_xor<8>(sum, lane);
                }
                const float inv = 1.f / sum;
#pragma unroll
                for (int m = 0; m < NTAU; ++m) w[g * NTAU + m] *= inv;
            }
        }
        if (!DO_AV && active) {
            // attn[pixel of this lane's child][tap]: lanes at distance 4 write consecutive taps
#pragma unroll
            for (int g = 0; g < NG; ++g) {
                T *ap = out + child_pixel(g * 4 + jl) * KK;
#pragma unroll
                for (int m = 0; m < NTAU; ++m)
                    if (ok[m]) ap[4 * m + bq] = (T)w[g * NTAU + m];
            }
        }
    } else {
        // av(): the weights come from memory, in the same lane layout
#pragma unroll
        for (int g = 0; g < NG; ++g) {
            const T *ap = attn_in + child_pixel(g * 4 + jl) * KK;
#pragma unroll
            for (int m = 0; m < NTAU; ++m)
                w[g * NTAU + m] = (active && ok[m]) ? (float)ap[4 * m + bq] : 0.f;
        }
    }

    if (DO_AV) {
        // the weights of taps 4 (4 gi + k) + bq, k = 0..3, as one A operand.  Fused
        // mode: the fp32 softmax weights go in as a sum of two 16-bit numbers,
        // w = hi + lo with hi = T(w), lo = T(w - hi) (relative error 2^-16 for
        // bf16, 2^-22 for fp16), each with its own matrix instruction on the same
        // B operand, so the aggregation sees weights of fp32 quality.
        constexpr bool SPLIT = MODE == TILED_FUSED;
        u32x2 wpk[NG][NGRP], wlo[SPLIT ? NG : 1][SPLIT ? NGRP : 1];
#pragma unroll
        for (int g = 0; g < NG; ++g)
#pragma unroll
            for (int gi = 0; gi < NGRP; ++gi) {
                float x[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) x[k] = 4 * gi + k < NTAU ? w[g * NTAU + 4 * gi + k] : 0.f;
                wpk[g][gi] = u32x2{pack2<T>(x[0], x[1]), pack2<T>(x[2], x[3])};
                if constexpr (SPLIT) {
                    typedef T tx4 __attribute__((ext_vector_type(4)));
                    const tx4 hi = __builtin_bit_cast(tx4, wpk[g][gi]);
#pragma unroll
                    for (int k = 0; k < 4; ++k) x[k] -= (float)hi[k];
                    wlo[g][gi] = u32x2{pack2<T>(x[0], x[1]), pack2<T>(x[2], x[3])};
                }
            }
        if constexpr (DMA) {
#pragma unroll
            for (int p = 0; p < NPD; ++p)
                voff0[p] = ((u32)(dpix[p] * C + 8 * dq8[p]) * (u32)sizeof(T)) | ((u32)dpix[p] & 0x80000000u);
        } else {
#pragma unroll
            for (int p = 0; p < NPASS; ++p)
                voff0[p] = ((u32)(spix[p] * C + 4 * sq) * (u32)sizeof(T)) | ((u32)spix[p] & 0x80000000u);
        }
        for (int j = nKc; j < ntot; ++j) {
            if (j + 1 < ntot) stage_load_value(j + 1 - nKc);
            const int c0 = (j - nKc) * CHK;
            const u32 *wb = win + (j & 1) * BUFA;
            // acc[g][u][i]: child 4g + i, channel c0 + 4 li + u
            f32x4 acc[NG][4];
#pragma unroll
            for (int g = 0; g < NG; ++g)
#pragma unroll
                for (int u = 0; u < 4; ++u) acc[g][u] = f32x4{0.f, 0.f, 0.f, 0.f};
            static_for<4 * NGRP>([&](auto ib) __attribute__((always_inline)) {
                // pack gi of quad bsel: taps 4 (4 gi + k) + bsel; a tap past the window
                // has weight 0 and reads the window's last tap
                constexpr int bsel = decltype(ib)::value % 4, gi = decltype(ib)::value / 4;
                if (4 * (4 * gi) + bsel < KK) {
                    u32x2 r[4];
                    static_for<4>([&](auto ik) __attribute__((always_inline)) {
                        constexpr int k = decltype(ik)::value;
                        constexpr int t = 4 * (4 * gi + k) + bsel < KK ? 4 * (4 * gi + k) + bsel : KK - 1;
                        r[k] = *(const u32x2 *)(wb + ((t / K) * WW + t % K) * PSW);
                    });
                    // [tap][channel] -> [channel][tap]
                    u32x2 bop[4];
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        const u32 sel = u % 2 ? 0x07060302u : 0x05040100u;
                        bop[u] = u32x2{__builtin_amdgcn_perm(r[1][u / 2], r[0][u / 2], sel),
                                       __builtin_amdgcn_perm(r[3][u / 2], r[2][u / 2], sel)};
                    }
#pragma unroll
                    for (int g = 0; g < NG; ++g)
#pragma unroll
                        for (int u = 0; u < 4; ++u) {
                            acc[g][u] = M::template run<2, bsel>(wpk[g][gi], bop[u], acc[g][u]);
                            if constexpr (SPLIT)
                                acc[g][u] = M::template run<2, bsel>(wlo[g][gi], bop[u], acc[g][u]);
                        }
                }
            });
            // The next chunk goes to LDS BEFORE the results are stored: a wait for
            // a load while stores are in flight is a wait for those stores too
            // (one counter, no order between the two kinds), so the stores are
            // issued right after the wait and have a whole chunk to complete.
            if (j + 1 < ntot) stage_store(j + 1);
            if (active && c0 + 4 * li < C) {
#pragma unroll
                for (int jj = 0; jj < NJ; ++jj) {
                    const u32x2 o = {pack2<T>(acc[jj / 4][0][jj % 4], acc[jj / 4][1][jj % 4]),
                                     pack2<T>(acc[jj / 4][2][jj % 4], acc[jj / 4][3][jj % 4])};
                    __builtin_nontemporal_store(o, (u32x2 *)(out + child_pixel(jj) * C + c0 + 4 * li));
                }
            }
            chunk_barrier();
        }
    }
}

template <typename T, int K, int S, int QX, int TY>
static hipError_t launch_geom(int mode, const void *q, const void *key, const void *attn_in,
                              const void *value, const void *qbias, void *out, int B, int d, int C,
                              int H, int W, hipStream_t st) {
    const int tiles_x = (W + 4 * QX - 1) / (4 * QX), tiles_y = (H + TY - 1) / TY;
    const long nb = (long)tiles_x * tiles_y * B;
    if (nb > (1L << 30)) return hipErrorNotSupported;
    const int per_xcd = (int)((nb + 7) / 8);
    const dim3 grid(per_xcd * 8), block(64 * QX * TY);
#define SAPA_NHWC16_LAUNCH(M, QB)                                                               \
    hipLaunchKernelGGL((sapa_b_nhwc16_kernel<T, K, S, QX, TY, M, QB>), grid, block, 0, st,      \
                       (const T *)q, (const T *)key, (const T *)attn_in, (const T *)value,      \
                       (const T *)qbias, (T *)out, d, C, H, W, tiles_x, tiles_y, (int)nb, per_xcd)
#define SAPA_NHWC16_CASE(M)                                                                     \
    case M:                                                                                     \
        SAPA_NHWC16_LAUNCH(M, false);                                                           \
        break;
    if (qbias) {
        // the bias is carried by the fused mode only
        if (mode != TILED_FUSED) return hipErrorNotSupported;
        SAPA_NHWC16_LAUNCH(TILED_FUSED, true);
        return hipGetLastError();
    }
    switch (mode) {
        SAPA_NHWC16_CASE(TILED_QK) SAPA_NHWC16_CASE(TILED_QK_SOFTMAX) SAPA_NHWC16_CASE(TILED_AV)
        SAPA_NHWC16_CASE(TILED_FUSED)
        default: return hipErrorNotSupported;
    }
#undef SAPA_NHWC16_CASE
#undef SAPA_NHWC16_LAUNCH
    return hipGetLastError();
}

#ifndef SAPA_NHWC16_TILE
#define SAPA_NHWC16_TILE 1, 4
#endif
template <typename T>
static hipError_t launch_t(int mode, const void *q, const void *key, const void *attn_in,
                           const void *value, const void *qbias, void *out, int B, int d, int C,
                           int H, int W, int K, int s, hipStream_t st) {
#define SAPA_NHWC16_KS(KV, SV)                                                                  \
    if (K == KV && s == SV)                                                                     \
        return launch_geom<T, KV, SV, SAPA_NHWC16_TILE>(mode, q, key, attn_in, value, qbias, out, \
                                                        B, d, C, H, W, st);
    SAPA_NHWC16_KS(3, 2) SAPA_NHWC16_KS(5, 2) SAPA_NHWC16_KS(7, 2) SAPA_NHWC16_KS(5, 4)
    SAPA_NHWC16_KS(7, 4)
#undef SAPA_NHWC16_KS
    return hipErrorNotSupported;
}

}  // namespace nhwc16

// Channels-last f16 / bf16 tensors (layouts as for sapa_b_nhwc_launch), (K, s) in
// {(3,2), (5,2), (7,2), (5,4), (7,4)}, d a multiple of 8, C of 4, q aligned to 16
// bytes and key / value / out to 8; one image's key / value tensor below 2^31
// bytes; qbias: optional [B, d] added to every query vector, aligned to 16 bytes.
// hipErrorNotSupported otherwise (fp32 tensors included).
hipError_t sapa_b_nhwc16_launch(int mode, const void *q, const void *key, const void *attn_in,
                                const void *value, const void *qbias, void *out, int B, int d,
                                int C, int H, int W, int K, int s, int dtype, hipStream_t st) {
    if (dtype != 2 && dtype != 3) return hipErrorNotSupported;
    if (!((s == 2 && (K == 3 || K == 5 || K == 7)) || (s == 4 && (K == 5 || K == 7))))
        return hipErrorNotSupported;
    const bool need_qk = mode != TILED_AV, need_av = mode == TILED_AV || mode == TILED_FUSED;
    if ((need_qk && d % 8 != 0) || (need_av && C % 4 != 0)) return hipErrorNotSupported;
    const long plane = (long)H * W * 2;
    if ((need_qk && plane * d >= (1L << 31)) || (need_av && plane * C >= (1L << 31)))
        return hipErrorNotSupported;
    if (need_qk && ((uintptr_t)q % 16 != 0 || (uintptr_t)key % 8 != 0 || (uintptr_t)qbias % 16 != 0))
        return hipErrorNotSupported;
    if (need_av && ((uintptr_t)value % 8 != 0 || (uintptr_t)out % 8 != 0)) return hipErrorNotSupported;
    if (dtype == 2)
        return nhwc16::launch_t<f16_t>(mode, q, key, attn_in, value, qbias, out, B, d, C, H, W, K, s, st);
    return nhwc16::launch_t<bf16_t>(mode, q, key, attn_in, value, qbias, out, B, d, C, H, W, K, s, st);
}

}  // namespace sapa
