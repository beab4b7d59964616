// SAPA-B for fp32 tensors in channels-last memory order with BOTH products on the
// matrix pipe: qk, qk+softmax, av and the fused qk -> softmax -> av forward, (K, s) in
// {(3,2), (5,2), (7,2), (5,4), (7,4)}.
//
// Decomposition, LDS staging (global memory straight into LDS) and the aggregation are
// those of sapa_b_nhwc.hip: a row of 16 lanes owns one low-res parent with its s x s
// children, a wave 4 parents that are neighbours in x, a workgroup of 4 waves a tile of
// 4 x 4 parents; windows go through LDS as [position][64 channels], double-buffered; the
// aggregation is one v_mfma_f32_4x4x1 (16 independent blocks of 4 lanes, D(4x4) +=
// A(4x1) B(1x4)) per tap and channel of a lane.  The logits differ:
//
//   * logits: lane (b, i) of a row (b = lane quad 0..3, i = lane in the quad) supplies, as
//     A, the key of tap 4 tau + i and, as B, the q of child i, both for one of the 16
//     channels of quad b per instruction; lane (b, j) then holds [tap 4 tau + i][child j],
//     i = 0..3, summed over those 16 channels in channel order.  Two butterfly steps over
//     the 4 quads of the row (halving the live values at each step) finish the sum and
//     leave tap 4 tau + b of child j in lane (b, j): K*K logits per child in
//     ceil(K*K / 4) registers.  That is 16 matrix instructions and 12 vector instructions
//     per 4 taps x 4 children x 64 channels, against 64 multiply-adds and 52 exchange
//     instructions of the all-lanes butterfly in sapa_b_nhwc.hip;
//   * softmax per child over its registers and the 4 quads of the row;
//   * the aggregation's A operand is register t / 4 of quad t % 4 for tap t (the
//     instruction's A broadcast, cbsz = 2, hands it to the row).
//
// Positions are 68 floats apart in LDS (64 of data): the 4 lanes of a quad read 4
// consecutive positions and the 4 quads 4 blocks of 16 bytes, which then fall on
// disjoint banks.  Measured against sapa_b_nhwc.hip on MI355X: faster where the
// arithmetic shows (K = 7, s = 4: 234 -> 194-206 us at B=4, C=512, 64x64), 3-6 % slower at
// (5, 2) -- the launcher of sapa_b_nhwc.hip sends K = 7 and s = 4 here (SAPA_NHWC_MM_ALL
// in a tuning build: everything).
//
// The channel sums run in the order above, not in the reference kernels' sequential
// order: results agree with them to rounding (1e-5 relative), not bit for bit.
#include "nhwc_common.hpp"

namespace sapa {

namespace nhwc {

template <typename T, int K, int S, int QX, int TY, int MODE>
__global__ void __launch_bounds__(64 * QX * TY)
sapa_b_nhwc_mm_kernel(const T *__restrict__ q, const T *__restrict__ key,
                   const T *__restrict__ attn_in, const T *__restrict__ value,
                   const T *__restrict__ qbias, T *__restrict__ out, int d, int C, int H, int W,
                   int tiles_x, int tiles_y, int nblocks, int per_xcd) {
    static_assert(S == 2 || S == 4, "children are handled in groups of 4");
    // children j = cy * S + cx of a parent, in NG groups of 4 (s = 2: all four;
    // s = 4: one child row per group)
    constexpr int NJ = S * S, NG = NJ / 4, KK = K * K, R = (K - 1) / 2;
    constexpr int TX = 4 * QX;                    // tile: TX x TY parents, QX waves per row
    constexpr int WW = TX + K - 1, WH = TY + K - 1, NPOS = WW * WH;   // window positions
    constexpr int CHK = 64;                       // channels per chunk: 16 lanes x 4
    // floats between positions in LDS: 64 of data and 4 spare, so that the logits' reads
    // (the 4 lanes of a quad read 4 consecutive positions, the 4 quads of a row 4 blocks
    // of 16 channels) fall on disjoint banks
    constexpr int PS = CHK + 4, SPP = PS / 4;     // ... and 16-byte slots per position
    constexpr int BUF = NPOS * PS;                // floats per LDS buffer
    constexpr int NT = 64 * QX * TY;
    constexpr int NTAU = (KK + 3) / 4;            // taps in groups of 4: weight registers per child
    constexpr int NR = NG * NTAU;
    constexpr bool DO_QK = MODE != TILED_AV;
    constexpr bool DO_SOFTMAX = MODE == TILED_QK_SOFTMAX || MODE == TILED_FUSED;
    constexpr bool DO_AV = MODE == TILED_AV || MODE == TILED_FUSED;
    typedef Quad<T> Q4;
    typedef typename Q4::raw Raw;

    // fp32 windows go from global memory straight into LDS (buffer loads with the LDS
    // modifier; thread t of pass p fills the 16-byte slot p * NT + t of a buffer): no
    // staging registers and no LDS write instructions.  A wave's load fills 64 consecutive
    // slots, so a buffer is a whole number of those.  16-bit tensors are widened on the
    // way through registers (their threads skip the spare slots).
#ifndef SAPA_NHWC_DMA
#define SAPA_NHWC_DMA 1
#endif
    constexpr bool DMA = SAPA_NHWC_DMA && std::is_same<T, float>::value;
    constexpr int BUFA = DMA ? (BUF + 255) / 256 * 256 : BUF;
    constexpr int SPT = DMA ? SPP : 16;           // slots a position takes in the staging order
    constexpr int NPASS = (NPOS * SPT + NT - 1) / NT;
    __shared__ __attribute__((aligned(16))) float lds[2 * BUFA];

    const int logical = (int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8);
    if (logical >= nblocks) return;
    const int tx = logical % tiles_x;
    const int ty = (logical / tiles_x) % tiles_y;
    const int n = logical / (tiles_x * tiles_y);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int row = lane >> 4, li = lane & 15;    // parent within the wave, lane in the row
    const int jl = li & 3, bq = li >> 2;          // lane in its quad, quad in the row
    const int x0 = tx * TX, y0 = ty * TY;
    const int wx = wave % QX, wy = wave / QX;     // this wave's quad of parents in the tile
    const int px = x0 + 4 * wx + row, py = y0 + wy;
    const bool active = px < W && py < H;
    const int hW = W * S;
    const long lpix = (long)H * W, hpix = lpix * S * S;

    const int nKc = DO_QK ? (d + CHK - 1) / CHK : 0;
    const int nVc = DO_AV ? (C + CHK - 1) / CHK : 0;
    const int ntot = nKc + nVc;

    // ---- staging: pass p, thread t moves slot p * NT + t: channel quad (slot % SPT) of
    // window position slot / SPT.  spix: the position's pixel in the image, -1 for a
    // position outside it, a spare slot or a slot past the window (offset 2^31 then:
    // beyond every descriptor, zero fill).
    int spix[NPASS], squad[NPASS];
#pragma unroll
    for (int p = 0; p < NPASS; ++p) {
        const int slot = p * NT + tid;
        const int pos = slot / SPT;
        // slot 4 b + e of a position holds channels 16 e + 4 b .. +3 (see the logits below)
        const int qd = slot % SPT;
        squad[p] = (qd & 3) * 4 + (qd >> 2);
        const int gy = y0 - R + pos / WW, gx = x0 - R + pos % WW;
        spix[p] = (pos < NPOS && qd < 16 && gy >= 0 && gy < H && gx >= 0 && gx < W) ? gy * W + gx : -1;
    }
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    (void)wave_u;
    Raw st[NPASS];
    auto stage_load = [&](int j) {
        const bool is_key = j < nKc;
        const int nch = is_key ? d : C;
        const int c0 = (is_key ? j : j - nKc) * CHK;
        const T *base = (is_key ? key : value) + (long)n * lpix * nch;
        const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(
            (void *)base, 0, (int)(lpix * nch * (long)sizeof(T)), 0x00020000);
#pragma unroll
        for (int p = 0; p < NPASS; ++p) {
            const u32 off = (c0 + 4 * squad[p] < nch && spix[p] >= 0)
                                ? (u32)(spix[p] * nch + c0 + 4 * squad[p]) * (u32)sizeof(T)
                                : 0x80000000u;
            if constexpr (DMA) {
                // (device pass only: the host pass, which sees this body for the launch
                // stub, does not know the builtin)
#if defined(__HIP_DEVICE_COMPILE__)
                const int slot0 = p * NT + wave_u * 64;      // first slot of this wave's load
                if ((p + 1) * NT <= NPOS * SPT || slot0 < NPOS * SPT)
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(
                        r, (__attribute__((address_space(3))) void *)(lds + (j & 1) * BUFA + slot0 * 4), 16,
                        off, 0, 0, 0);
#endif
            } else {
                st[p] = Q4::buffer_load(r, off);
            }
        }
    };
    // registers -> LDS; direct-to-LDS: wait for the loads (the counter retires in issue
    // order, so that is a wait for everything issued before them as well)
    auto stage_store = [&](int j) {
        if constexpr (DMA) {
#if defined(__HIP_DEVICE_COMPILE__)
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#endif
            return;
        }
        float *dst = lds + (j & 1) * BUFA;
#pragma unroll
        for (int p = 0; p < NPASS; ++p) {
            const int pos = (p * NT + tid) / 16;
            if (NPOS % (NT / 16) == 0 || pos < NPOS) *(f32x4 *)(dst + pos * PS + 4 * (tid & 15)) = Q4::widen(st[p]);
        }
    };
    // every wave is done with the current window and the next one is in LDS (direct-to-LDS:
    // the bare barrier instruction -- the loads were waited for above, and a fence here
    // would drain the output stores issued since)
    auto chunk_barrier = [&]() {
        if constexpr (DMA) {
#if defined(__HIP_DEVICE_COMPILE__)
            asm volatile("s_barrier" ::: "memory");
#endif
        } else {
            __syncthreads();
        }
    };

    // this row's window origin: tap (ky, kx) of its parent sits at position
    // (wy + ky) * WW + 4 wx + row + kx.  Inside a position the 16 channel quads are stored
    // transposed: slot 4 b + e holds channels 16 e + 4 b .. +3.  Aggregation: lane li reads
    // its channels 4 li .. +3 (slot 4 (li % 4) + li / 4); logits: lane (bq, jl) reads slots
    // 4 bq .. 4 bq + 3 of tap 4 tau + jl (64 contiguous bytes), i.e. channels 16 e + 4 bq .. +3,
    // e = 0..3 -- the channels whose q the 4 lanes bq = 0..3 of a child fetch as 64 contiguous
    // bytes per load.
    const float *win = lds + ((wy * WW + 4 * wx + row) * PS + 4 * (4 * jl + bq));
    const float *kwin = lds + ((wy * WW + 4 * wx + row) * PS + 16 * bq);
    int kofs[NTAU];
#pragma unroll
    for (int tau = 0; tau < NTAU; ++tau) {
        const int t = min(4 * tau + jl, KK - 1);
        kofs[tau] = ((t / K) * WW + t % K) * PS;
    }

    // logits, then weights: w[g * NTAU + m] of lane (bq, jl) belongs to child jl of group g
    // and tap 4 m + bq; ok[m]: that tap exists
    float w[NR];
    bool ok[NTAU];
#pragma unroll
    for (int m = 0; m < NTAU; ++m) ok[m] = 4 * m + bq < KK;
    // child j of this row's parent: its pixel in a [B, sH, sW, n_ch] tensor
    auto child_pixel = [&](int j) {
        return (long)n * hpix + (long)(py * S + j / S) * hW + (long)px * S + j % S;
    };
    // q of child jl of group g: channels 16 e + 4 bq .. +3, e = 0..3, of key chunk j (zeros
    // past d and for idle rows; d is a multiple of 4)
    Raw qraw[4];
    auto load_q = [&](int j, int g) {
        const int c0 = j * CHK + 4 * bq;
        const T *qp = q + child_pixel(g * 4 + jl) * d + c0;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            qraw[e] = Raw{};
            if (active && c0 + 16 * e < d) qraw[e] = __builtin_nontemporal_load((const Raw *)(qp + 16 * e));
        }
    };
    // the first q is fetched before anything else so that it arrives while the
    // first window is staged
    if (DO_QK) load_q(0, 0);
    stage_load(0);
    stage_store(0);
    chunk_barrier();

    if (DO_QK) {
#pragma unroll
        for (int i = 0; i < NR; ++i) w[i] = 0.f;
        for (int j = 0; j < nKc; ++j) {
            if (j + 1 < ntot) stage_load(j + 1);
            const float *kb = kwin + (j & 1) * BUFA;
#pragma unroll
            for (int g = 0; g < NG; ++g) {
                f32x4 qv[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) qv[e] = Q4::widen(qraw[e]);
                // optional per-image bias of the query projection [B, d], added here
                // instead of in a pass of its own over the query tensor
                if (qbias) {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (j * CHK + 4 * bq + 16 * e < d)
                            qv[e] += Q4::widen(*(const Raw *)(qbias + (long)n * d + j * CHK + 4 * bq + 16 * e));
                }
                // the next group's (or chunk's) q while this one is used
                if (g + 1 < NG) load_q(j, g + 1);
                else if (j + 1 < nKc) load_q(j + 1, 0);
                // On the matrix pipe: block (row, bq) of 4 lanes takes one channel per
                // instruction; lane jl supplies the key of tap 4 tau + jl as A and the q of
                // child jl as B, so lane (bq, jl) accumulates [tap 4 tau + i][child jl],
                // i = 0..3, over its 16 channels (in channel order).
                static_for<NTAU>([&](auto itau) {
                    constexpr int tau = decltype(itau)::value;
                    const float *kp = kb + kofs[tau];
                    f32x4 kv[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) kv[e] = *(const f32x4 *)(kp + 4 * e);
                    f32x4 a = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int e = 0; e < 4; ++e)
#pragma unroll
                        for (int c = 0; c < 4; ++c)
                            a = __builtin_amdgcn_mfma_f32_4x4x1f32(kv[e][c], qv[e][c], a, 0, 0, 0);
                    // summed over the 4 quads of the row, tap 4 tau + bq stays in this lane
                    const float flat[4] = {a[0], a[1], a[2], a[3]};
                    float h1[2], h2[1];
                    halve<4, 4, false>(flat, h1, lane);    // (inputs: a matrix instruction's result)
                    halve<8, 2>(h1, h2, lane);
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
        for (int j = nKc; j < ntot; ++j) {
            if (j + 1 < ntot) stage_load(j + 1);
            const int c0 = (j - nKc) * CHK;
            const float *wb = win + (j & 1) * BUFA;
            // acc[g][u][i]: child 4g + i, channel c0 + 4 li + u
            f32x4 acc[NG][4];
#pragma unroll
            for (int g = 0; g < NG; ++g)
#pragma unroll
                for (int u = 0; u < 4; ++u) acc[g][u] = f32x4{0.f, 0.f, 0.f, 0.f};
            // the window values travel through a ring of AHEAD + 1 registers of
            // 4 channels: tap t + AHEAD is read while tap t is multiplied
            constexpr int AHEAD = S == 2 ? 3 : 1;
            f32x4 ring[AHEAD + 1];
            static_for<AHEAD>([&](auto it) {
                constexpr int t = decltype(it)::value;
                ring[t] = *(const f32x4 *)(wb + ((t / K) * WW + t % K) * PS);
            });
            static_for<KK>([&](auto it) {
                constexpr int t = decltype(it)::value, tn = t + AHEAD;
                if (tn < KK)
                    ring[tn % (AHEAD + 1)] = *(const f32x4 *)(wb + ((tn / K) * WW + tn % K) * PS);
                const f32x4 vv = ring[t % (AHEAD + 1)];
                static_for<NG>([&](auto ig) {
                    // the 4 children's weights of tap t sit in quad t % 4 of the row, register
                    // t / 4; the instruction's A broadcast (cbsz = 2: one block feeds its group
                    // of 4 blocks, i.e. the row; abid picks it) hands them to all 16 lanes
                    constexpr int g = decltype(ig)::value;
                    const float wr = w[g * NTAU + t / 4];
                    static_for<4>([&](auto iu) {
                        constexpr int u = decltype(iu)::value;
                        acc[g][u] = __builtin_amdgcn_mfma_f32_4x4x1f32(wr, vv[u], acc[g][u], 2, t % 4, 0);
                    });
                });
            });
            // The next chunk goes to LDS BEFORE the results are stored: a wait for
            // a load while stores are in flight is a wait for those stores too
            // (one counter, no order between the two kinds), so the stores are
            // issued right after the wait and have a whole chunk to complete.
            if (j + 1 < ntot) stage_store(j + 1);
            if (active && c0 + 4 * li < C) {
#pragma unroll
                for (int jj = 0; jj < NJ; ++jj)
                    __builtin_nontemporal_store(
                        Q4::narrow(f32x4{acc[jj / 4][0][jj % 4], acc[jj / 4][1][jj % 4],
                                         acc[jj / 4][2][jj % 4], acc[jj / 4][3][jj % 4]}),
                        (Raw *)(out + child_pixel(jj) * C + c0 + 4 * li));
            }
            chunk_barrier();
        }
    }
}

template <int K, int S, int QX, int TY>
static hipError_t launch_mm_geom(int mode, const void *q, const void *key, const void *attn_in,
                                 const void *value, const void *qbias, void *out, int B, int d, int C,
                                 int H, int W, hipStream_t st) {
    typedef float T;
    const int tiles_x = (W + 4 * QX - 1) / (4 * QX), tiles_y = (H + TY - 1) / TY;
    const long nb = (long)tiles_x * tiles_y * B;
    if (nb > (1L << 30)) return hipErrorNotSupported;
    const int per_xcd = (int)((nb + 7) / 8);
    const dim3 grid(per_xcd * 8), block(64 * QX * TY);
#define SAPA_NHWC_CASE(M)                                                                      \
    case M:                                                                                    \
        hipLaunchKernelGGL((sapa_b_nhwc_mm_kernel<T, K, S, QX, TY, M>), grid, block, 0, st,    \
                           (const T *)q, (const T *)key, (const T *)attn_in, (const T *)value, \
                           (const T *)qbias, (T *)out, d, C, H, W, tiles_x, tiles_y, (int)nb,  \
                           per_xcd);                                                           \
        break;
    switch (mode) {
        SAPA_NHWC_CASE(TILED_QK) SAPA_NHWC_CASE(TILED_QK_SOFTMAX) SAPA_NHWC_CASE(TILED_AV)
        SAPA_NHWC_CASE(TILED_FUSED)
        default: return hipErrorNotSupported;
    }
#undef SAPA_NHWC_CASE
    return hipGetLastError();
}

// fp32 channels-last tensors; the caller (sapa_b_nhwc_launch) has checked shapes and alignment
hipError_t launch_mm(int mode, const void *q, const void *key, const void *attn_in, const void *value,
                     const void *qbias, void *out, int B, int d, int C, int H, int W, int K, int s,
                     hipStream_t st) {
#define SAPA_NHWC_KS(KV, SV)                                                                   \
    if (K == KV && s == SV)                                                                    \
        return launch_mm_geom<KV, SV, 1, 4>(mode, q, key, attn_in, value, qbias, out, B, d, C, H, W, st);
    SAPA_NHWC_KS(3, 2) SAPA_NHWC_KS(5, 2) SAPA_NHWC_KS(7, 2) SAPA_NHWC_KS(5, 4) SAPA_NHWC_KS(7, 4)
#undef SAPA_NHWC_KS
    return hipErrorNotSupported;
}

}  // namespace nhwc

}  // namespace sapa
