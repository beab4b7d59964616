// SAPA-B for tensors in channels-last memory order (torch.channels_last: the
// logical [B, C, H, W] tensor stored as [B, H, W, C]): qk, qk+softmax, av and
// the fused qk -> softmax -> av forward, (K, s) in {(3,2), (5,2), (7,2), (5,4),
// (7,4)}.
//
// With the channels innermost every access of the operation is a long
// contiguous run -- a pixel's q is one record of d elements, an output pixel
// one record of C elements -- so the lanes of a wave run along the CHANNELS:
//
//   * a row of 16 lanes owns one low-res parent with its s x s children; lane i
//     of the row holds channels 4i .. 4i+3 of the current 64-channel chunk.  A
//     wave works on 4 parents that are neighbours in x, a workgroup of 4 waves
//     on a tile of 4 x 4 parents;
//   * key and value windows (tile + K-1 halo positions) go through LDS as
//     [position][64 channels], one chunk at a time, double-buffered; a row of
//     lanes reads one position as 256 contiguous bytes (no bank conflicts);
//   * logits, one window row and one group of 4 children (s = 2: all of them,
//     s = 4: one child row) at a time, K taps x 4 children = 20 values for
//     K = 5: every lane accumulates its 4 channels' part of the products; the 16
//     lanes of a row are then summed with a 4-step butterfly that halves the
//     number of live values at every step (the lane keeps the sums whose index
//     bit matches its lane bit and hands the others to its partner: DPP quad
//     permutes for lane distances 1 and 2, a cross-lane permute for 4 and 8).
//     Afterwards lane l holds, for window row ky, the logits with in-row index
//     16 m + l (index = 4 * kx + child): 100 values in 10 registers per lane;
//   * softmax per child across the 4 lanes x 10 registers that hold its taps;
//   * aggregation on the matrix pipe: for one tap, out[child][channel] +=
//     weight[child] * value[channel] is a 4 x 4 outer product per lane quad,
//     which is what v_mfma_f32_4x4x1 computes for 16 independent blocks of 4
//     lanes (one FMA per element, so the tap order and the rounding are those
//     of the scalar loop).  Lanes 4b .. 4b+3 (block b) supply 4 value channels
//     as B; the weights stay where the butterfly left them -- the 4 children's
//     weights of tap kx sit in lanes 4 (kx % 4) .. +3 of the row -- and the
//     instruction's A-broadcast (cbsz = 2: one block feeds its group of 4
//     blocks, i.e. the row of 16 lanes; abid = kx % 4 picks it) hands them to
//     the whole row.  One 16-byte LDS read feeds 4 such instructions (one per
//     channel of the lane), 4 s^2 accumulators per lane, no copy of the weights.
//
// The channel sums run in tree order, not in the reference kernels' sequential
// order: results agree with them to rounding (1e-5 relative in fp32), not bit
// for bit.  Out-of-range window positions are zeros in LDS: logit exactly 0
// (and part of the softmax), contribution exactly 0.
#include "nhwc_common.hpp"

namespace sapa {

namespace nhwc {

#ifdef SAPA_NHWC_WPE
#define SAPA_NHWC_OCC __attribute__((amdgpu_waves_per_eu(SAPA_NHWC_WPE, SAPA_NHWC_WPE)))
#else
#define SAPA_NHWC_OCC
#endif
template <typename T, int K, int S, int QX, int TY, int MODE>
__global__ void __launch_bounds__(64 * QX * TY) SAPA_NHWC_OCC
sapa_b_nhwc_kernel(const T *__restrict__ q, const T *__restrict__ key,
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
    constexpr int BUF = NPOS * CHK;               // floats per LDS buffer
    constexpr int NT = 64 * QX * TY, NPASS = (NPOS * 16 + NT - 1) / NT;   // staging passes (16 quads per position)
    constexpr int NV = K * 4;                     // logits of one window row and child group, index = 4 * kx + child in group
    constexpr int N1 = (NV + 1) / 2, N2 = (N1 + 1) / 2, N3 = (N2 + 1) / 2;
    constexpr int RPR = (N3 + 1) / 2, NR = K * NG * RPR;   // registers per (row, group) / in all
    constexpr bool DO_QK = MODE != TILED_AV;
    constexpr bool DO_SOFTMAX = MODE == TILED_QK_SOFTMAX || MODE == TILED_FUSED;
    constexpr bool DO_AV = MODE == TILED_AV || MODE == TILED_FUSED;
    typedef Quad<T> Q4;
    typedef typename Q4::raw Raw;

    // fp32 windows go from global memory straight into LDS (buffer loads with the LDS
    // modifier; thread t of pass p fills the 16-byte slot p * NT + t, which is the layout
    // below): no staging registers and no LDS write instructions.  A wave's load fills 64
    // consecutive slots, so a buffer is a whole number of those.
#ifndef SAPA_NHWC_DMA
#define SAPA_NHWC_DMA 1
#endif
    constexpr bool DMA = SAPA_NHWC_DMA && std::is_same<T, float>::value;
    constexpr int BUFA = DMA ? (BUF + 255) / 256 * 256 : BUF;
    __shared__ __attribute__((aligned(16))) float lds[2 * BUFA];

    const int logical = (int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8);
    if (logical >= nblocks) return;
    const int tx = logical % tiles_x;
    const int ty = (logical / tiles_x) % tiles_y;
    const int n = logical / (tiles_x * tiles_y);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int row = lane >> 4, li = lane & 15;    // parent within the wave, channel quad
    const int x0 = tx * TX, y0 = ty * TY;
    const int wx = wave % QX, wy = wave / QX;     // this wave's quad of parents in the tile
    const int px = x0 + 4 * wx + row, py = y0 + wy;
    const bool active = px < W && py < H;
    const int hW = W * S;
    const long lpix = (long)H * W, hpix = lpix * S * S;

    const int nKc = DO_QK ? (d + CHK - 1) / CHK : 0;
    const int nVc = DO_AV ? (C + CHK - 1) / CHK : 0;
    const int ntot = nKc + nVc;

    // ---- staging: pass p, thread t moves channel quad t % 16 of window position
    // p * 16 + t / 16.  Byte offsets into the image's tensor; 2^31 marks a
    // position outside the image (beyond every descriptor: zero fill).
    int spix[NPASS];
#pragma unroll
    for (int p = 0; p < NPASS; ++p) {
        const int pos = p * (NT / 16) + tid / 16;
        const int gy = y0 - R + pos / WW, gx = x0 - R + pos % WW;
        spix[p] = (pos < NPOS && gy >= 0 && gy < H && gx >= 0 && gx < W) ? gy * W + gx : -1;
    }
    const int sq = tid & 15;                      // channel quad staged by this thread
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
        const bool c_ok = c0 + 4 * sq < nch;
#pragma unroll
        for (int p = 0; p < NPASS; ++p) {
            const u32 off = (c_ok && spix[p] >= 0)
                                ? (u32)(spix[p] * nch + c0 + 4 * sq) * (u32)sizeof(T)
                                : 0x80000000u;
            if constexpr (DMA) {
                // (device pass only: the host pass, which sees this body for the launch
                // stub, does not know the builtin)
#if defined(__HIP_DEVICE_COMPILE__)
                const int slot0 = p * NT + wave_u * 64;      // first slot of this wave's load
                if ((p + 1) * NT <= NPOS * 16 || slot0 < NPOS * 16)
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
            const int pos = p * (NT / 16) + tid / 16;
            if (NPOS % (NT / 16) == 0 || pos < NPOS) *(f32x4 *)(dst + pos * CHK + 4 * sq) = Q4::widen(st[p]);
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
    // (wy + ky) * WW + 4 wx + row + kx
    const float *win = lds + ((wy * WW + 4 * wx + row) * CHK + 4 * li);

    // logits, then weights: w[(ky * NG + g) * RPR + m] of lane li is in-row index
    // 16 m + li of window row ky and child group g, i.e. child jl = li & 3 of the
    // group and kx = 4 m + (li >> 2); ok[m]: that index exists
    float w[NR];
    bool ok[RPR];
#pragma unroll
    for (int m = 0; m < RPR; ++m) ok[m] = 16 * m + li < NV;
    const int jl = li & 3, kxl = li >> 2;          // this lane's child in a group and first kx
    // this lane's child of group g: its pixel in a [B, sH, sW, n_ch] tensor
    auto child_pixel = [&](int j) {
        return (long)n * hpix + (long)(py * S + j / S) * hW + (long)px * S + j % S;
    };
    // q of the 4 children of group g, this lane's 4 channels of key chunk j
    // (zeros past d and for idle rows)
    Raw qraw[4];
    auto load_q = [&](int j, int g) {
        const int c0 = j * CHK;
        const bool q_ok = active && c0 + 4 * li < d;
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
            qraw[jj] = Raw{};
            if (q_ok)
                qraw[jj] = __builtin_nontemporal_load(
                    (const Raw *)(q + child_pixel(g * 4 + jj) * d + c0 + 4 * li));
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
            const float *wb = win + (j & 1) * BUFA;
#pragma unroll
            for (int g = 0; g < NG; ++g) {
                f32x4 qv[4];
#pragma unroll
                for (int jj = 0; jj < 4; ++jj) qv[jj] = Q4::widen(qraw[jj]);
                // optional per-image bias of the query projection [B, d], added here
                // instead of in a pass of its own over the query tensor
                if (qbias && j * CHK + 4 * li < d) {
                    const f32x4 qb = Q4::widen(*(const Raw *)(qbias + (long)n * d + j * CHK + 4 * li));
#pragma unroll
                    for (int jj = 0; jj < 4; ++jj) qv[jj] += qb;
                }
                // the next group's (or chunk's) q while this one is used
                if (g + 1 < NG) load_q(j, g + 1);
                else if (j + 1 < nKc) load_q(j + 1, 0);
#pragma unroll
                for (int ky = 0; ky < K; ++ky) {
                    float part[NV];
#pragma unroll
                    for (int kx = 0; kx < K; ++kx) {
                        const f32x4 kv = *(const f32x4 *)(wb + (ky * WW + kx) * CHK);
#pragma unroll
                        for (int jj = 0; jj < 4; ++jj) {
                            float a = kv[0] * qv[jj][0];
#pragma unroll
                            for (int e = 1; e < 4; ++e) a = fma_(kv[e], qv[jj][e], a);
                            part[kx * 4 + jj] = a;
                        }
                    }
                    // sum over the 16 lanes of the row
                    float p1[N1], p2[N2], p3[N3], p4[RPR];
                    halve<1, NV>(part, p1, lane);
                    halve<2, N1>(p1, p2, lane);
                    halve<4, N2>(p2, p3, lane);
                    halve<8, N3>(p3, p4, lane);
#pragma unroll
                    for (int m = 0; m < RPR; ++m) w[(ky * NG + g) * RPR + m] += p4[m];
                }
            }
            if (j + 1 < ntot) stage_store(j + 1);
            chunk_barrier();
        }
        if (DO_SOFTMAX) {
            // a child's taps lie in this lane's registers of its group and in the
            // lanes at distance 4, 8, 12
#pragma unroll
            for (int g = 0; g < NG; ++g) {
                float mx = w[g * RPR];             // ky = 0, in-row index li < NV always
#pragma unroll
                for (int ky = 0; ky < K; ++ky)
#pragma unroll
                    for (int m = 0; m < RPR; ++m)
                        if (ok[m]) mx = max_(mx, w[(ky * NG + g) * RPR + m]);
                if constexpr (SAPA_NHWC_DPP_HALVE) {
                    mx = xor_max_dpp<4>(mx);
                    mx = xor_max_dpp<8>(mx);
                } else {
                    mx = max_(mx, row_xor<4>(mx, lane));
                    mx = max_(mx, row_xor<8>(mx, lane));
                }
                float sum = 0.f;
#pragma unroll
                for (int ky = 0; ky < K; ++ky)
#pragma unroll
                    for (int m = 0; m < RPR; ++m) {
                        float &x = w[(ky * NG + g) * RPR + m];
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
                for (int ky = 0; ky < K; ++ky)
#pragma unroll
                    for (int m = 0; m < RPR; ++m) w[(ky * NG + g) * RPR + m] *= inv;
            }
        }
        if (!DO_AV && active) {
            // attn[pixel of this lane's child][tap]: 4 lanes write 4 consecutive taps
#pragma unroll
            for (int g = 0; g < NG; ++g) {
                T *ap = out + child_pixel(g * 4 + jl) * KK;
#pragma unroll
                for (int ky = 0; ky < K; ++ky)
#pragma unroll
                    for (int m = 0; m < RPR; ++m)
                        if (ok[m]) ap[ky * K + 4 * m + kxl] = (T)w[(ky * NG + g) * RPR + m];
            }
        }
    } else {
        // av(): the weights come from memory, in the same lane layout
#pragma unroll
        for (int g = 0; g < NG; ++g) {
            const T *ap = attn_in + child_pixel(g * 4 + jl) * KK;
#pragma unroll
            for (int ky = 0; ky < K; ++ky)
#pragma unroll
                for (int m = 0; m < RPR; ++m)
                    w[(ky * NG + g) * RPR + m] =
                        (active && ok[m]) ? (float)ap[ky * K + 4 * m + kxl] : 0.f;
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
                ring[t] = *(const f32x4 *)(wb + ((t / K) * WW + t % K) * CHK);
            });
            static_for<KK>([&](auto it) {
                constexpr int t = decltype(it)::value, ky = t / K, kx = t % K, tn = t + AHEAD;
                if (tn < KK)
                    ring[tn % (AHEAD + 1)] = *(const f32x4 *)(wb + ((tn / K) * WW + tn % K) * CHK);
                const f32x4 vv = ring[t % (AHEAD + 1)];
                static_for<NG>([&](auto ig) {
                    // in-row index 4 kx + child: register kx / 4 of (ky, g), lanes 4 (kx % 4) .. +3
                    constexpr int g = decltype(ig)::value;
                    const float wr = w[(ky * NG + g) * RPR + kx / 4];
                    static_for<4>([&](auto iu) {
                        constexpr int u = decltype(iu)::value;
                        acc[g][u] = __builtin_amdgcn_mfma_f32_4x4x1f32(wr, vv[u], acc[g][u], 2, kx % 4, 0);
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

#ifndef SAPA_NHWC_TILE
#define SAPA_NHWC_TILE 1, 4
#endif
template <typename T, int K, int S, int QX, int TY>
static hipError_t launch_geom(int mode, const void *q, const void *key, const void *attn_in,
                              const void *value, const void *qbias, void *out, int B, int d, int C,
                              int H, int W, hipStream_t st) {
    const int tiles_x = (W + 4 * QX - 1) / (4 * QX), tiles_y = (H + TY - 1) / TY;
    const long nb = (long)tiles_x * tiles_y * B;
    if (nb > (1L << 30)) return hipErrorNotSupported;
    const int per_xcd = (int)((nb + 7) / 8);
    const dim3 grid(per_xcd * 8), block(64 * QX * TY);
#define SAPA_NHWC_CASE(M)                                                                      \
    case M:                                                                                    \
        hipLaunchKernelGGL((sapa_b_nhwc_kernel<T, K, S, QX, TY, M>), grid, block, 0, st, (const T *)q, \
                           (const T *)key, (const T *)attn_in, (const T *)value,               \
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

// fp32 cases of the kernel with the logits on the matrix pipe (SAPA_NHWC_MM_ALL in a tuning
// build: all of them)
static bool takes_mm(int K, int s) {
#ifdef SAPA_NHWC_MM_ALL
    return true;
#else
    return K == 7 || s == 4;
#endif
}

template <typename T>
static hipError_t launch_t(int mode, const void *q, const void *key, const void *attn_in,
                           const void *value, const void *qbias, void *out, int B, int d, int C,
                           int H, int W, int K, int s, hipStream_t st) {
    // fp32: the variant with the logits on the matrix pipe (sapa_b_nhwc_mm.hip) for the
    // large windows / up-factors, whose arithmetic shows: measured faster there (K = 7, s = 4
    // at B=4, C=512, 64x64: 234 -> 194-206 us), 3-6 % slower at (5, 2).  The choice depends on
    // (K, s) alone so that a batch and its images one by one take the same kernel
    // (bit-identical results).
    if constexpr (std::is_same<T, float>::value)
        if (takes_mm(K, s))
            return launch_mm(mode, q, key, attn_in, value, qbias, out, B, d, C, H, W, K, s, st);
#define SAPA_NHWC_KS(KV, SV)                                                                  \
    if (K == KV && s == SV)                                                                   \
        return launch_geom<T, KV, SV, SAPA_NHWC_TILE>(mode, q, key, attn_in, value, qbias, out, B, \
                                                      d, C, H, W, st);
    SAPA_NHWC_KS(3, 2) SAPA_NHWC_KS(5, 2) SAPA_NHWC_KS(7, 2) SAPA_NHWC_KS(5, 4) SAPA_NHWC_KS(7, 4)
#undef SAPA_NHWC_KS
    return hipErrorNotSupported;
}

}  // namespace nhwc

const char *sapa_b_nhwc_kernel_name(int K, int s, int dtype) {
    return dtype == 0 && nhwc::takes_mm(K, s) ? "sapa_b_nhwc_mm_kernel" : "sapa_b_nhwc_kernel";
}

// Channels-last tensors (q [B, sH, sW, d], key [B, H, W, d], value [B, H, W, C],
// attn [B, sH, sW, K*K], out like q with C or K*K channels), f32 / f16 / bf16,
// (K, s) in {(3,2), (5,2), (7,2), (5,4), (7,4)}, channel counts multiples of 4 and every tensor aligned to
// 4 elements; one image's key / value tensor below 2^31 bytes.  qbias: optional
// [B, d] added to every query vector (the modes that read the query).
// hipErrorNotSupported otherwise.
hipError_t sapa_b_nhwc_launch(int mode, const void *q, const void *key, const void *attn_in,
                              const void *value, const void *qbias, void *out, int B, int d, int C,
                              int H, int W, int K, int s, int dtype, hipStream_t st) {
    if (!((s == 2 && (K == 3 || K == 5 || K == 7)) || (s == 4 && (K == 5 || K == 7))))
        return hipErrorNotSupported;
    const bool need_qk = mode != TILED_AV, need_av = mode == TILED_AV || mode == TILED_FUSED;
    if ((need_qk && d % 4 != 0) || (need_av && C % 4 != 0)) return hipErrorNotSupported;
    const int esize = dtype == 0 ? 4 : 2;
    const long plane = (long)H * W * esize;
    if ((need_qk && plane * d >= (1L << 31)) || (need_av && plane * C >= (1L << 31)))
        return hipErrorNotSupported;
    const void *vec_ptrs[5] = {need_qk ? q : nullptr, need_qk ? key : nullptr,
                               need_av ? value : nullptr, need_av ? out : nullptr,
                               need_qk ? qbias : nullptr};
    for (const void *p : vec_ptrs)
        if (p && (uintptr_t)p % (4 * esize) != 0) return hipErrorNotSupported;
    switch (dtype) {
        case 0: return nhwc::launch_t<float>(mode, q, key, attn_in, value, qbias, out, B, d, C, H, W, K, s, st);
        case 2: return nhwc::launch_t<f16_t>(mode, q, key, attn_in, value, qbias, out, B, d, C, H, W, K, s, st);
        case 3: return nhwc::launch_t<bf16_t>(mode, q, key, attn_in, value, qbias, out, B, d, C, H, W, K, s, st);
        default: return hipErrorNotSupported;
    }
}

}  // namespace sapa
