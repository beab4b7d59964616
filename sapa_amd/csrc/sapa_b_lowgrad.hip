// Gradient of the SAPA-B operators with respect to their low-res operand
// (grad_key of qk, grad_value of av) as an LDS-tiled gather:
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
