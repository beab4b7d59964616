// Gradient of the SAPA-B operators with respect to their low-res operand
// (grad_key of qk, grad_value of av): an LDS-tiled gather, and further down the
// same sums with the products owned by the parents (lanes exchange partial sums):
//
//   out[n,c,y,x] = sum over window entries k = (ky,kx), i.e. over the parents
//                  (py,px) = (y + r - ky, x + r - kx) that see cell (y,x) as
//                  their entry k, and over their S*S children j, of
//                  w[n, k, child j] * hi[n, c, child j]
//
// (w = grad of the logits and hi = query for grad_key; w = attention weights
// and hi = grad of the output for grad_value).  The reference scatters the
// same products with one global atomicAdd each
// (sapa/sapa/src/cuda/qk_cuda_kernel.cu:120-135, av_cuda_kernel.cu:128-145);
// here every output element is owned by one thread, so there are no atomics,
// the output needs no zero-fill and the result is the same on every run.
// (Scattering into LDS was measured too: LDS float atomics run at a small
// fraction of the plain LDS rate on this part, and tile-level global atomics
// alone cost more than this whole kernel.)
//
// A workgroup owns a tile of TW x TH = (16*NWX) x (4*NWY) low-res cells of one
// image; a thread owns one cell and keeps the K*K x S*S weights that multiply
// into it in registers for the whole launch (they do not depend on the
// channel).  The high-res window of `hi` that the tile's cells draw from --
// the children of the tile's parents plus r parents on every side -- is staged
// through LDS CH channels at a time, double-buffered, with the next chunk's
// global loads in flight during the current chunk's FMAs; a thread reads the
// S children of a parent row with one S-wide LDS access.  Each child row has
// its own running sum over k in ascending order, one FMA per term; the row
// sums are added at the end.
#include <type_traits>
#include <utility>

#include "kernels.hpp"

namespace sapa {

template <int N> struct FVec;
template <> struct FVec<2> { typedef float type __attribute__((ext_vector_type(2))); };
template <> struct FVec<4> { typedef float type __attribute__((ext_vector_type(4))); };

// N consecutive tensor elements as one load, widened to floats
template <typename T, int N>
__device__ __forceinline__ typename FVec<N>::type load_wide(const T *p) {
    typedef T tvec __attribute__((ext_vector_type(N)));
    const tvec v = *(const tvec *)p;
    typename FVec<N>::type f;
#pragma unroll
    for (int i = 0; i < N; ++i) f[i] = (float)v[i];
    return f;
}

// T = float, f16_t or bf16_t: the type of hi and out; WT: that of the weight
// tensor (T, or float next to 16-bit features); the window in LDS, the weights
// in registers and the sums are fp32 whatever they are
template <typename T, typename WT, int K, int S, int NWX, int NWY, int CH, int VEC>
__global__ void __launch_bounds__(64 * NWX *NWY) __attribute__((amdgpu_waves_per_eu(3, 3)))
lowgrad_gather_kernel(const T *__restrict__ hi, const WT *__restrict__ w,
                      T *__restrict__ out, int C, int H, int W, int tiles_x, int tiles_y,
                      int nblocks, int per_xcd, int cgroups, int cper) {
    static_assert(S == 2, "children are read as 2-wide vectors");
    constexpr int TW = 16 * NWX, TH = 4 * NWY, NT = 64 * NWX * NWY;
    constexpr int KK = K * K, R = (K - 1) / 2, NJ = S * S;
    constexpr int WPW = TW + 2 * R, WPH = TH + 2 * R;   // window in parents
    constexpr int WW = WPW * S, WH = WPH * S;            // window in high-res pixels
    constexpr int RS = WW;                               // LDS row stride (floats)
    constexpr int PS = WH * RS;                          // one channel's plane
    constexpr int NV = WH * (WW / VEC);                  // vector loads per channel
    constexpr int NLD = (CH * NV + NT - 1) / NT;         // per thread and chunk
    static_assert(WW % VEC == 0 && (R * S) % VEC == 0, "window rows must be whole aligned vectors");
    static_assert(NLD <= 32, "validity mask is 32 bits");
    typedef typename FVec<VEC>::type V;
    typedef typename FVec<S>::type V2;
    // 16-bit tensors stay 16-bit in LDS (a dword = the two children of a parent in a
    // row): the kernel is bound by the bytes it reads from LDS, and widening at the
    // use -- a shift and a mask for bf16, two conversions for f16 -- costs less than
    // those bytes
    constexpr bool PACK = sizeof(T) == 2;
    constexpr int LW = PACK ? 2 : 1;                     // pixels per LDS dword
    static_assert(!PACK || (S == 2 && VEC % 2 == 0), "a dword holds the two children of a parent row");
    typedef unsigned RawV __attribute__((ext_vector_type(VEC / 2 > 0 ? VEC / 2 : 1)));   // VEC 16-bit elements

    __shared__ __attribute__((aligned(16))) float win[2 * CH * PS / LW];

    const int logical = (int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8);
    if (logical >= nblocks) return;
    const int tx = logical % tiles_x;
    const int ty = (logical / tiles_x) % tiles_y;
    const int cg = (logical / (tiles_x * tiles_y)) % cgroups;
    const int n = logical / (tiles_x * tiles_y * cgroups);
    const int cbeg = cg * cper, cend = cbeg + cper < C ? cbeg + cper : C;

    const int tid = threadIdx.x, lane = tid % 64, wv = tid / 64;
    const int lx = (wv % NWX) * 16 + lane % 16, ly = (wv / NWX) * 4 + lane / 16;
    const int x = tx * TW + lx, y = ty * TH + ly;
    const int hW = W * S, hH = H * S;
    const long hplane = (long)hH * hW;

    // weights of the terms that flow into cell (y, x); parents outside the
    // image contribute nothing
    float wr[KK][NJ];
    {
        const WT *wp = w + (long)n * KK * hplane;
#pragma unroll
        for (int k = 0; k < KK; ++k) {
            const int py = y + R - k / K, px = x + R - k % K;
            const bool ok = py >= 0 && py < H && px >= 0 && px < W;
            const long base = (long)k * hplane + (long)((ok ? py : 0) * S) * hW + (ok ? px : 0) * S;
#pragma unroll
            for (int cy = 0; cy < S; ++cy) {
                const V2 v = load_wide<WT, S>(wp + base + (long)cy * hW);
#pragma unroll
                for (int cx = 0; cx < S; ++cx) wr[k][cy * S + cx] = ok ? v[cx] : 0.f;
            }
        }
    }

    // staging: element e of a chunk = (channel, window row, vector in the row)
    const int wy0 = (ty * TH - R) * S, wx0 = (tx * TW - R) * S;   // window origin, high-res
    const T *hp = hi + (long)n * C * hplane;
    typedef typename std::conditional<PACK, RawV, V>::type StageV;
    StageV stage[NLD];
    unsigned okmask = 0;
    auto issue = [&](int c0) {
        okmask = 0;
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int e = tid + i * NT;
            const int ch = e / NV, rem = e % NV;
            const int row = rem / (WW / VEC), col = rem % (WW / VEC) * VEC;
            const int gy = wy0 + row, gx = wx0 + col;
            // a vector is either all inside or all outside the image: gx and
            // the image width are both multiples of VEC
            const bool ok =
                e < CH * NV && c0 + ch < cend && gy >= 0 && gy < hH && gx >= 0 && gx < hW;
            const long off = ok ? (long)(c0 + ch) * hplane + (long)gy * hW + gx : 0;
            if constexpr (PACK) stage[i] = *(const RawV *)(hp + off);
            else stage[i] = load_wide<T, VEC>(hp + off);
            okmask |= (unsigned)ok << i;
        }
    };
    auto commit = [&](float *buf) {
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int e = tid + i * NT;
            if (e < CH * NV) {
                const int ch = e / NV, rem = e % NV;
                const int row = rem / (WW / VEC), col = rem % (WW / VEC) * VEC;
                StageV v = stage[i];
                if (!((okmask >> i) & 1)) v = StageV{};
                *(StageV *)(buf + (ch * PS + row * RS + col) / LW) = v;
            }
        }
    };

    issue(cbeg);
    commit(win);
    __syncthreads();

    // the children of window parent (ly + 2r - ky, lx + 2r - kx) feed entry k
    const float *base = win + ((ly + 2 * R) * S * RS + (lx + 2 * R) * S) / LW;
    const bool live = x < W && y < H;
    const long lplane = (long)H * W;
    T *op = out + (long)n * C * lplane + (long)(y < H ? y : 0) * W + (x < W ? x : 0);
    int parity = 0;
    for (int c0 = cbeg; c0 < cend; c0 += CH, parity ^= 1) {
        const bool more = c0 + CH < cend;
        if (more) issue(c0 + CH);
        const float *buf = base + parity * (CH * PS / LW);
#pragma unroll 1
        for (int ch = 0; ch < CH; ++ch) {
            float acc[S];   // one running sum per child row: two shorter FMA chains
#pragma unroll
            for (int cy = 0; cy < S; ++cy) acc[cy] = 0.f;
#pragma unroll
            for (int k = 0; k < KK; ++k)
#pragma unroll
                for (int cy = 0; cy < S; ++cy) {
                    V2 h;
                    if constexpr (PACK) {
                        const unsigned u = *(const unsigned *)(buf + (ch * PS + (cy - (k / K) * S) * RS - (k % K) * S) / LW);
                        if constexpr (std::is_same<T, bf16_t>::value) {
                            h[0] = __builtin_bit_cast(float, u << 16);
                            h[1] = __builtin_bit_cast(float, u & 0xffff0000u);
                        } else {
                            union { unsigned u; T t[2]; } x;
                            x.u = u;
                            h[0] = (float)x.t[0];
                            h[1] = (float)x.t[1];
                        }
                    } else {
                        h = *(const V2 *)(buf + ch * PS + (cy - (k / K) * S) * RS - (k % K) * S);
                    }
                    acc[cy] = __builtin_fmaf(wr[k][cy * S], h[0], acc[cy]);
                    acc[cy] = __builtin_fmaf(wr[k][cy * S + 1], h[1], acc[cy]);
                }
            if (live && c0 + ch < cend) op[(long)(c0 + ch) * lplane] = (T)(acc[0] + acc[1]);
        }
        if (more) commit(win + (parity ^ 1) * (CH * PS / LW));
        __syncthreads();
    }
}

// ---------------------------------------------------------------------------
// The same sums with the products owned by the PARENTS.  A lane is one parent
// (py, px) and keeps its own K*K x S*S weights; per channel it reads its four
// children of `hi` straight from global memory (every element of `hi` belongs to
// exactly one parent: no staging, no reuse to organise) and forms
//
//   t[ky][kx] = sum over children j of w[(ky,kx)][j] * hi[j]      (K*K*S*S FMAs)
//
// which is what this parent adds to cell (py - r + ky, px - r + kx).  The sum over
// kx is an exchange between x-neighbours: a row of RW lanes holds RW consecutive
// parents, and DPP shifts hand t[ky][kx] of lane L + r - kx to lane L (K - 1 shifted
// adds per ky: row shifts inside rows of 16 lanes, a running sum on wave shifts in
// wider rows).  The sum over ky crosses lane rows and waves and goes through LDS:
// K floats written and K read per lane and channel, against the K*K*S*S floats the
// gather above reads per output element, which are what bounds the gather.  The
// price is a halo: the r outermost parents on every side of a tile of RW x TH lanes
// do not complete their cells (they lack neighbours), so a tile delivers
// (RW - 2r) x (TH - 2r) cells and neighbouring tiles overlap.  Deterministic: fixed
// order, no atomics.
template <typename F, int... I>
__device__ __forceinline__ void lg_static_for_impl(F &&f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
    lg_static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// lane L receives v of lane L + 1 of the wave (0 for the last lane)
__device__ __forceinline__ float wave_shift_left(float v) {
    union { float f; int i; } x, y;
    x.f = v;
    y.i = __builtin_amdgcn_mov_dpp(x.i, 0x130, 0xf, 0xf, true);   // wave_shl:1
    return y.f;
}

template <int SH>   // lane L receives v of lane L + SH of its row of 16 lanes (0 where there is none)
__device__ __forceinline__ float row_shift(float v) {
    union { float f; int i; } x, y;
    x.f = v;
    y.i = __builtin_amdgcn_mov_dpp(x.i, SH > 0 ? 0x100 + SH : 0x110 - SH, 0xf, 0xf, true);   // row_shl / row_shr
    return y.f;
}

// NW waves of RW x (64 / RW) lanes stacked in y (RW = 16: sums over kx by row shifts;
// RW = 32: by wave shifts, see below), CH channels per chunk (one barrier per chunk),
// register budget for WPE waves per SIMD
template <typename T, typename WT, int K, int NW, int CH, int WPE, int RW>
__global__ void __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu(WPE, WPE)))
lowgrad_shift_kernel(const T *__restrict__ hi, const WT *__restrict__ w, T *__restrict__ out, int C,
                     int H, int W, int tiles_x, int tiles_y, int nblocks, int per_xcd, int cgroups,
                     int cper) {
    constexpr int S = 2, KK = K * K, R = (K - 1) / 2, NJ = S * S;
    constexpr int TH = 64 / RW * NW;                 // lane rows of a tile
    constexpr int VX = RW - 2 * R, VY = TH - 2 * R;  // cells a tile completes
    constexpr int ROWS = TH + 2 * R;                 // exchange rows incl. an unwritten halo, so that
    constexpr int PL = ROWS * RW + 2 * R;            // every lane reads at constant distances
    static_assert(RW == 16 || RW == 32 || RW == 64, "a wave is whole rows of lanes");
    constexpr bool PACK = sizeof(T) == 2;
    typedef typename std::conditional<PACK, unsigned, typename FVec<2>::type>::type Raw;   // one child row
    typedef typename FVec<2>::type V2;

    __shared__ float xbuf[2 * CH * K * PL];

    const int logical = (int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8);
    if (logical >= nblocks) return;
    const int tx = logical % tiles_x;
    const int ty = (logical / tiles_x) % tiles_y;
    const int cg = (logical / (tiles_x * tiles_y)) % cgroups;
    const int n = logical / (tiles_x * tiles_y * cgroups);
    const int cbeg = cg * cper, cend = cbeg + cper < C ? cbeg + cper : C;

    const int tid = threadIdx.x, lx = tid % RW, ly = tid / RW;
    const int x = tx * VX - R + lx, y = ty * VY - R + ly;    // this lane's parent, and its cell
    const bool inside = x >= 0 && x < W && y >= 0 && y < H;
    const int hW = W * S;
    const long hplane = (long)H * S * hW;

    // the parent's weights; a parent outside the image has none
    float wr[KK][NJ];
    {
        const WT *wp = w + (long)n * KK * hplane + (inside ? (long)(y * S) * hW + x * S : 0);
#pragma unroll
        for (int k = 0; k < KK; ++k)
#pragma unroll
            for (int cy = 0; cy < S; ++cy) {
                const V2 v = load_wide<WT, S>(wp + (long)k * hplane + (long)cy * hW);
#pragma unroll
                for (int cx = 0; cx < S; ++cx) wr[k][cy * S + cx] = inside ? v[cx] : 0.f;
            }
    }

    // the children: two rows of S elements per channel, through a descriptor over the
    // image (offset 2^31 = outside: the hardware returns zeros); the channel travels as
    // the scalar offset
    const __amdgpu_buffer_rsrc_t hrsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(hi + (long)n * C * hplane), 0, (int)((long)C * hplane * (long)sizeof(T)), 0x00020000);
    const unsigned off0 = inside ? (unsigned)((y * S) * hW + x * S) * (unsigned)sizeof(T) : 0x80000000u;
    const unsigned rowb = (unsigned)hW * (unsigned)sizeof(T);    // (outside + a row is still outside)
    const unsigned planeb = (unsigned)hplane * (unsigned)sizeof(T);
#ifndef SAPA_LOWGRAD_SHIFT_PF
#define SAPA_LOWGRAD_SHIFT_PF 1
#endif
    constexpr int PF = SAPA_LOWGRAD_SHIFT_PF;     // chunks in flight ahead of the one in work
    auto issue = [&](Raw (&nxt)[CH][S], int c0) __attribute__((always_inline)) {
#pragma unroll
        for (int ch = 0; ch < CH; ++ch) {
            const bool ok = c0 + ch < cend;
            const unsigned soff = (unsigned)(ok ? c0 + ch : 0) * planeb;
            const unsigned o0 = ok ? off0 : 0x80000000u, o1 = o0 + rowb;
            if constexpr (PACK) {
                nxt[ch][0] = __builtin_amdgcn_raw_buffer_load_b32(hrsrc, o0, soff, 0);
                nxt[ch][1] = __builtin_amdgcn_raw_buffer_load_b32(hrsrc, o1, soff, 0);
            } else {
                union { unsigned u __attribute__((ext_vector_type(2))); V2 f; } a, b;
                a.u = __builtin_amdgcn_raw_buffer_load_b64(hrsrc, o0, soff, 0);
                b.u = __builtin_amdgcn_raw_buffer_load_b64(hrsrc, o1, soff, 0);
                nxt[ch][0] = a.f;
                nxt[ch][1] = b.f;
            }
        }
    };
    auto widen = [&](Raw r) __attribute__((always_inline)) {
        if constexpr (PACK) {
            V2 h;
            if constexpr (std::is_same<T, bf16_t>::value) {
                h[0] = __builtin_bit_cast(float, r << 16);
                h[1] = __builtin_bit_cast(float, r & 0xffff0000u);
            } else {
                union { unsigned u; T t[2]; } v;
                v.u = r;
                h[0] = (float)v.t[0];
                h[1] = (float)v.t[1];
            }
            return h;
        } else {
            return r;
        }
    };

    const bool live = lx >= R && lx < RW - R && ly >= R && ly < TH - R && x < W && y < H;
    const long lplane = (long)H * W;
    // results leave through a descriptor over the image's output planes: a lane without a
    // cell of its own carries an offset outside it and the hardware drops its store
    const __amdgpu_buffer_rsrc_t orsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(out + (long)n * C * lplane), 0, (int)((long)C * lplane * (long)sizeof(T)), 0x00020000);
    const unsigned ooff = live ? (unsigned)(y * W + x) * (unsigned)sizeof(T) : 0x80000000u;
    const unsigned lplaneb = (unsigned)lplane * (unsigned)sizeof(T);
    // where this lane writes (with wave shifts its sum belongs to the cell r lanes to its right)
    float *const wrow = xbuf + (ly + R) * RW + lx + (RW == 16 ? 0 : R);
    const float *const rrow = xbuf + (ly + 2 * R) * RW + lx;   // row ly + 2r - ky holds what cell row ly gets for ky

    // PF + 1 register sets take turns (the loop is unrolled by as many chunks, so that no
    // load result is ever copied: a copy would wait for its load)
    auto work = [&](const Raw (&cur)[CH][S], int c0, int parity) __attribute__((always_inline)) {
        float *const wb = wrow + parity * (CH * K * PL);
#pragma unroll
        for (int ch = 0; ch < CH; ++ch) {
            const V2 ha = widen(cur[ch][0]), hb = widen(cur[ch][1]);
#pragma unroll
            for (int ky = 0; ky < K; ++ky) {
                float t[K];
#pragma unroll
                for (int kx = 0; kx < K; ++kx) {
                    const int k = ky * K + kx;
                    float v = wr[k][0] * ha[0];
                    v = __builtin_fmaf(wr[k][1], ha[1], v);
                    v = __builtin_fmaf(wr[k][2], hb[0], v);
                    t[kx] = __builtin_fmaf(wr[k][3], hb[1], v);
                }
                // cell column L collects t[kx] of the parent R - kx lanes to its right
                float sum;
                if constexpr (RW == 16) {
                    sum = t[R];
                    static_for<R>([&](auto i) {
                        constexpr int D = decltype(i)::value + 1;
                        sum += row_shift<D>(t[R - D]);
                        sum += row_shift<-D>(t[R + D]);
                    });
                } else {
                    // rows wider than a DPP row: the running sum moves one lane to the left
                    // through the whole wave per step, sum[L] = t[0][L + K - 1] + ... +
                    // t[K - 1][L], which is what cell L + r gets; the last 2r lanes of a row
                    // pick up the next row's first ones and belong to the halo anyway
                    sum = t[0];
#pragma unroll
                    for (int kx = 1; kx < K; ++kx) sum = wave_shift_left(sum) + t[kx];
                }
                wb[(ch * K + ky) * PL] = sum;
            }
        }
        __syncthreads();
        const float *const rb = rrow + parity * (CH * K * PL);
#pragma unroll
        for (int ch = 0; ch < CH; ++ch) {
            float acc = rb[(ch * K) * PL];
#pragma unroll
            for (int ky = 1; ky < K; ++ky) acc += rb[(ch * K + ky) * PL - ky * RW];
            if (c0 + ch < cend) {
                const unsigned soff = (unsigned)(c0 + ch) * lplaneb;
                if constexpr (PACK) {
                    const T r = (T)acc;
                    __builtin_amdgcn_raw_buffer_store_b16(__builtin_bit_cast(unsigned short, r), orsrc, ooff, soff, 0);
                } else {
                    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, acc), orsrc, ooff, soff, 0);
                }
            }
        }
    };
    Raw sets[PF + 1][CH][S];
    static_for<PF>([&](auto p) { issue(sets[decltype(p)::value], cbeg + decltype(p)::value * CH); });
    int parity = 0;
    for (int c0 = cbeg; c0 < cend; c0 += (PF + 1) * CH) {
        static_for<PF + 1>([&](auto ui) {
            constexpr int u = decltype(ui)::value;
            // (past the last channel: offsets outside the descriptor, no branch around the loads)
            issue(sets[(u + PF) % (PF + 1)], c0 + (u + PF) * CH);
            if (c0 + u * CH < cend) {
                work(sets[u], c0 + u * CH, parity);
                parity ^= 1;
            }
        });
    }
}

template <typename T, typename WT, int K, int NW, int CH, int WPE, int RW>
static hipError_t lowgrad_shift_launch(const void *hi, const void *w, void *out, int B, int C, int H, int W,
                                       hipStream_t st) {
    constexpr int R = (K - 1) / 2, VX = RW - 2 * R, VY = 64 / RW * NW - 2 * R;
    const int tiles_x = (W + VX - 1) / VX, tiles_y = (H + VY - 1) / VY;
    const long tiles = (long)tiles_x * tiles_y * B;
    // the channels of a tile over several workgroups until the grid fills the chip a
    // few times over (each re-reads the tile's weights)
#ifndef SAPA_LOWGRAD_SHIFT_MINWG
#define SAPA_LOWGRAD_SHIFT_MINWG 2048
#endif
    int cgroups = 1;
    const int max_groups = C / (4 * CH) > 0 ? C / (4 * CH) : 1;
    while (cgroups * 2 <= max_groups && tiles * cgroups < SAPA_LOWGRAD_SHIFT_MINWG) cgroups *= 2;
    const int cper = ((C + cgroups - 1) / cgroups + CH - 1) / CH * CH;
    const long nb = tiles * cgroups;
    if (nb > (1L << 30)) return hipErrorNotSupported;
    const int per_xcd = (int)((nb + 7) / 8);
    hipLaunchKernelGGL((lowgrad_shift_kernel<T, WT, K, NW, CH, WPE, RW>), dim3(per_xcd * 8), dim3(64 * NW), 0, st,
                       (const T *)hi, (const WT *)w, (T *)out, C, H, W, tiles_x, tiles_y, (int)nb,
                       per_xcd, cgroups, cper);
    return hipGetLastError();
}

template <typename T, typename WT, int K, int S, int NWX, int NWY, int CH, int VEC>
static hipError_t lowgrad_launch_geom(const void *hi, const void *w, void *out, int B, int C, int H, int W,
                       hipStream_t st) {
    constexpr int TW = 16 * NWX, TH = 4 * NWY, NT = 64 * NWX * NWY;
    const int tiles_x = (W + TW - 1) / TW, tiles_y = (H + TH - 1) / TH;
    const long tiles = (long)tiles_x * tiles_y * B;
    // few tiles: slice the channels over several workgroups per tile (each
    // re-reads the tile's weights, which is small against C channels of hi)
    int cgroups = 1;
    const int max_groups = C / (4 * CH) > 0 ? C / (4 * CH) : 1;
    while (cgroups * 2 <= max_groups && tiles * cgroups * 2 <= 1024) cgroups *= 2;
    const int cper = ((C + cgroups - 1) / cgroups + CH - 1) / CH * CH;
    const long nb = tiles * cgroups;
    if (nb > (1L << 30)) return hipErrorNotSupported;
    const int per_xcd = (int)((nb + 7) / 8);
    hipLaunchKernelGGL((lowgrad_gather_kernel<T, WT, K, S, NWX, NWY, CH, VEC>), dim3(per_xcd * 8),
                       dim3(NT), 0, st, (const T *)hi, (const WT *)w, (T *)out, C, H, W,
                       tiles_x, tiles_y, (int)nb, per_xcd, cgroups, cper);
    return hipGetLastError();
}

template <typename T, typename WT, int K, int VEC>
static hipError_t lowgrad_launch_k(const void *hi, const void *w, void *out, int B, int C, int H, int W,
                    hipStream_t st) {
    const bool wide = (W + 31) / 32 * 32 * 0.9 <= (W + 15) / 16 * 16;
    // channels per chunk (a barrier per chunk): 16-bit tensors take half the LDS per channel
#ifndef SAPA_LOWGRAD_CH16
#define SAPA_LOWGRAD_CH16 4
#endif
#ifndef SAPA_LOWGRAD_CH32
#define SAPA_LOWGRAD_CH32 2
#endif
    // (with 2-element staging loads 4 channels per chunk do not fit the registers)
    constexpr int CHN = sizeof(T) == 2 ? (VEC == 4 ? SAPA_LOWGRAD_CH16 : 2) : SAPA_LOWGRAD_CH32;
    return wide ? lowgrad_launch_geom<T, WT, K, 2, 2, 2, CHN, VEC>(hi, w, out, B, C, H, W, st)
                : lowgrad_launch_geom<T, WT, K, 2, 1, 2, sizeof(T) == 2 ? 2 : CHN, VEC>(hi, w, out, B, C, H, W, st);
}

template <typename T, typename WT>
static hipError_t lowgrad_launch_t(const void *hi, const void *w, void *out, int B, int C, int H, int W,
                                   int K, hipStream_t st) {
    // vector loads of s = 2 elements
    if ((uintptr_t)hi % (2 * sizeof(T)) || (uintptr_t)w % (2 * sizeof(WT))) return hipErrorNotSupported;
#ifndef SAPA_LOWGRAD_SHIFT_OFF
#ifndef SAPA_LOWGRAD_SHIFT_GAIN
#define SAPA_LOWGRAD_SHIFT_GAIN 0.47
#endif
    {
        // The lane-exchange form costs about half of the gather per lane and channel
        // (measured), but its tiles deliver (RW - 2r) x (TH - 2r) cells for RW x TH
        // lanes: it is taken where that still leaves it ahead.  It reads `hi` through
        // a 32-bit buffer descriptor per image.  Tiles of 8 waves with chunks of 2
        // channels keep it within 128 registers (four waves per SIMD, two workgroups per
        // CU), as 32 x 16 lanes (rows of whole cache lines) unless 16 x 32 wastes
        // clearly fewer lanes on the shape.
        constexpr int NW = 8, CH = 2, WPE = 4;
        const int R = (K - 1) / 2;
        auto lanes = [&](int rw) {
            const int vx = rw - 2 * R, vy = 64 / rw * NW - 2 * R;
            return (double)((W + vx - 1) / vx) * ((H + vy - 1) / vy) * (64 * NW);
        };
        const bool rows32 = lanes(32) <= 1.1 * lanes(16);
        const double lanes_shift = rows32 ? lanes(32) : lanes(16);
        const bool wide = (W + 31) / 32 * 32 * 0.9 <= (W + 15) / 16 * 16;    // (the gather's choice of tile)
        const int tw = wide ? 32 : 16;
        const double lanes_gather = (double)((W + tw - 1) / tw) * ((H + 7) / 8) * (tw * 8);
        if ((long)C * H * 2 * W * 2 * (long)sizeof(T) < (1L << 31) &&
            lanes_gather >= SAPA_LOWGRAD_SHIFT_GAIN * lanes_shift) {
            if (rows32)
                return K == 3 ? lowgrad_shift_launch<T, WT, 3, NW, CH, WPE, 32>(hi, w, out, B, C, H, W, st)
                              : lowgrad_shift_launch<T, WT, 5, NW, CH, WPE, 32>(hi, w, out, B, C, H, W, st);
            return K == 3 ? lowgrad_shift_launch<T, WT, 3, NW, CH, WPE, 16>(hi, w, out, B, C, H, W, st)
                          : lowgrad_shift_launch<T, WT, 5, NW, CH, WPE, 16>(hi, w, out, B, C, H, W, st);
        }
    }
#endif
    if (K == 3) return lowgrad_launch_k<T, WT, 3, 2>(hi, w, out, B, C, H, W, st);
    // 4-element staging loads when the rows of hi allow it (the window starts
    // r * s = 4 pixels left of a tile, which keeps them aligned)
    const bool v4 = (uintptr_t)hi % (4 * sizeof(T)) == 0 && W % 2 == 0;
    return v4 ? lowgrad_launch_k<T, WT, 5, 4>(hi, w, out, B, C, H, W, st)
              : lowgrad_launch_k<T, WT, 5, 2>(hi, w, out, B, C, H, W, st);
}

// f32 / f16 / bf16, (K, s) in {(3, 2), (5, 2)}, hi / w aligned to s elements;
// hipErrorNotSupported otherwise (the caller then takes the generic kernel).
// `out` is fully overwritten.
hipError_t lowres_grad_tiled_launch(const void *hi, const void *w, void *out, int B, int C, int H,
                                    int W, int K, int s, int dtype, hipStream_t st, bool wide) {
    if (s != 2 || (K != 3 && K != 5)) return hipErrorNotSupported;
    switch (dtype) {
        case 0: return lowgrad_launch_t<float, float>(hi, w, out, B, C, H, W, K, st);
        case 2:
            return wide ? lowgrad_launch_t<f16_t, float>(hi, w, out, B, C, H, W, K, st)
                        : lowgrad_launch_t<f16_t, f16_t>(hi, w, out, B, C, H, W, K, st);
        case 3:
            return wide ? lowgrad_launch_t<bf16_t, float>(hi, w, out, B, C, H, W, K, st)
                        : lowgrad_launch_t<bf16_t, bf16_t>(hi, w, out, B, C, H, W, K, st);
        default: return hipErrorNotSupported;
    }
}

}  // namespace sapa
