// 1x1 projection of a channels-last 16-bit feature map with per-image weights:
//   out[b, p, o] = sum_c x[b, p, c] * w[b, o, c] (+ bias[b, o]),   x [B, HW, C],
//   w [B, O, C], out [B, HW, O], fp16 / bf16, fp32 accumulation
// -- the q / k projections of the SAPA modules (sapa_base.py:32-35) after
// GroupNorm has been folded into per-image weights.  O is small (32 .. 128), so
// the operation is a stream over x: 2 C bytes read and 2 O written per pixel.
//
//   * a workgroup of 4 waves serves one image; its weights (O x C, up to 64 KB)
//     sit in LDS, rows padded by 16 bytes so that the matrix instruction's B
//     operand reads (16 rows x 4 column groups) fall on disjoint banks;
//   * a wave takes tiles of 16 consecutive pixels: 16 C-byte records, one
//     contiguous run of memory, fetched as 16 bytes per lane with the next
//     tile's loads in flight during the current tile's arithmetic, and passed
//     through a wave-private LDS tile (rows padded the same way) into the A
//     operand layout of v_mfma_f32_16x16x16 (row = pixel);
//   * the 16 x 16 results per output tile go back through LDS, so that a lane
//     stores 16 contiguous bytes and the wave one contiguous run of 32 O bytes.
#include "kernels.hpp"

namespace sapa {

namespace project {

typedef unsigned u32;
typedef u32 u32x2 __attribute__((ext_vector_type(2)));
typedef u32 u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

template <typename T> struct Mma;
template <> struct Mma<f16_t> {
    typedef _Float16 v4 __attribute__((ext_vector_type(4)));
    static __device__ __forceinline__ f32x4 run(u32x2 a, u32x2 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(v4, a), __builtin_bit_cast(v4, b),
                                                     c, 0, 0, 0);
    }
};
template <> struct Mma<bf16_t> {
    typedef short v4 __attribute__((ext_vector_type(4)));
    static __device__ __forceinline__ f32x4 run(u32x2 a, u32x2 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(v4, a),
                                                         __builtin_bit_cast(v4, b), c, 0, 0, 0);
    }
};

template <typename T>
__device__ __forceinline__ u32 pack2(float a, float b) {
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    typedef T tx2 __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(u32, __builtin_convertvector(f32x2{a, b}, tx2));
}

// C input channels, O outputs (both multiples of 16); tiles of 16 pixels
template <typename T, int C, int O>
__global__ void __launch_bounds__(256)
project_kernel(const T *__restrict__ x, const T *__restrict__ w, const T *__restrict__ bias,
               T *__restrict__ out, long HW, int tiles_per_block) {
    constexpr int RW = C / 2 + 4;                 // dwords per padded row of C 16-bit values
    constexpr int NL = C / 32;                    // 16-byte loads per lane and tile (16 rows of 2 C bytes)
    constexpr int NT = O / 16;                    // output tiles of 16 columns
    constexpr int OW = O / 2 + 4;                 // dwords per padded row of the result tile
    constexpr int XT = 16 * RW > 16 * OW ? 16 * RW : 16 * OW;   // dwords of a wave's tile (x, then results)
    extern __shared__ __attribute__((aligned(16))) u32 sh[];
    u32 *wl = sh;                                 // weights: O rows of RW dwords
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    u32 *xt = sh + O * RW + wave * XT;            // this wave's tile
    const int b = blockIdx.y;
    const T *xb = x + (long)b * HW * C;
    T *ob = out + (long)b * HW * O;

    // the image's weights -> LDS (16 bytes per thread and step)
    {
        const u32x4 *src = (const u32x4 *)(w + (long)b * O * C);
        for (int i = threadIdx.x; i < O * C / 8; i += 256) {
            const int row = i / (C / 8), col = i % (C / 8);
            *(u32x4 *)(wl + row * RW + 4 * col) = src[i];
        }
    }
    __syncthreads();

    const long ntiles = (HW + 15) / 16;
    const long t0 = ((long)blockIdx.x * 4 + wave) * tiles_per_block;
    const long t1 = t0 + tiles_per_block < ntiles ? t0 + tiles_per_block : ntiles;
    const int r16 = lane & 15, kg = lane >> 4;    // row / column of a 16 x 16 tile, k group
    float bv[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) bv[nt] = bias ? (float)bias[(long)b * O + 16 * nt + r16] : 0.f;

    // a tile's 16 records are one run of 32 C bytes: lane l takes 16-byte piece
    // j * 64 + l (pieces past the image: zeros)
    u32x4 st[NL];
    auto load_tile = [&](long t) __attribute__((always_inline)) {
        const long base = t * 16 * (C / 8), limit = HW * (C / 8);   // in 16-byte pieces
        const u32x4 *src = (const u32x4 *)xb;
#pragma unroll
        for (int j = 0; j < NL; ++j) {
            const long i = base + j * 64 + lane;
            st[j] = u32x4{0u, 0u, 0u, 0u};
            if (i < limit) st[j] = __builtin_nontemporal_load(src + i);
        }
    };
    if (t0 < t1) load_tile(t0);
    for (long t = t0; t < t1; ++t) {
        // registers -> the wave's LDS tile (row = pixel)
#pragma unroll
        for (int j = 0; j < NL; ++j) {
            const int i = j * 64 + lane, row = i / (C / 8), col = i % (C / 8);
            *(u32x4 *)(xt + row * RW + 4 * col) = st[j];
        }
        if (t + 1 < t1) load_tile(t + 1);
        f32x4 acc[NT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[nt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < C / 16; ++ks) {
            // A: pixel r16, channels 16 ks + 4 kg .. +3; B: output 16 nt + r16, same channels
            const u32x2 a = *(const u32x2 *)(xt + r16 * RW + 8 * ks + 2 * kg);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const u32x2 bm = *(const u32x2 *)(wl + (16 * nt + r16) * RW + 8 * ks + 2 * kg);
                acc[nt] = Mma<T>::run(a, bm, acc[nt]);
            }
        }
        // acc[nt][i]: pixel 4 kg + i, output 16 nt + r16 -> the tile again, as 16-bit
        // rows of O values (the x tile has been consumed by this wave's own reads)
        unsigned short *rt = (unsigned short *)xt;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const u32 h = pack2<T>(acc[nt][i] + bv[nt], 0.f);
                rt[(4 * kg + i) * (2 * OW) + 16 * nt + r16] = (unsigned short)h;
            }
        // 16 rows of 2 O bytes -> one contiguous run of 32 O bytes
        const long obase = t * 16 * (O / 8), olimit = HW * (O / 8);
#pragma unroll
        for (int j = 0; j < (16 * O / 8 + 63) / 64; ++j) {
            const int i = j * 64 + lane, row = i / (O / 8), col = i % (O / 8);
            if (i < 16 * O / 8 && obase + i < olimit)
                __builtin_nontemporal_store(*(const u32x4 *)(xt + row * OW + 4 * col),
                                            (u32x4 *)ob + obase + i);
        }
    }
}

template <typename T, int C, int O>
static hipError_t launch_co(const void *x, const void *w, const void *bias, void *out, int B, long HW,
                            hipStream_t st) {
    constexpr int RW = C / 2 + 4, OW = O / 2 + 4;
    constexpr int XT = 16 * RW > 16 * OW ? 16 * RW : 16 * OW;
    constexpr size_t lds = (size_t)(O * RW + 4 * XT) * 4;
    static_assert(lds <= 160 * 1024, "weights and tiles must fit LDS");
    const long ntiles = (HW + 15) / 16;
    // about 8 workgroups per CU over the whole launch, at least 8 tiles per wave
    long per = (ntiles * B + 4L * 2048 - 1) / (4L * 2048);
    if (per < 8) per = 8;
    const long blocks = (ntiles + 4 * per - 1) / (4 * per);
    if (blocks > 65535 * 32L || B > 65535) return hipErrorNotSupported;
    auto kern = project_kernel<T, C, O>;
    if (lds > 64 * 1024) {
        // more than the default 64 KB per workgroup: ask for it; a device that
        // cannot give it is not served by this kernel
        int dev = 0, most = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&most, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) != hipSuccess ||
            (size_t)most < lds ||
            hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)lds) != hipSuccess) {
            (void)hipGetLastError();
            return hipErrorNotSupported;
        }
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks, B), dim3(256), lds, st, (const T *)x, (const T *)w,
                       (const T *)bias, (T *)out, HW, (int)per);
    return hipGetLastError();
}

template <typename T>
static hipError_t launch_t(const void *x, const void *w, const void *bias, void *out, int B, int C,
                           int O, long HW, hipStream_t st) {
#define SAPA_PROJECT_CASE(CV, OV) \
    if (C == CV && O == OV) return launch_co<T, CV, OV>(x, w, bias, out, B, HW, st);
    SAPA_PROJECT_CASE(64, 32) SAPA_PROJECT_CASE(64, 64)
    SAPA_PROJECT_CASE(128, 32) SAPA_PROJECT_CASE(128, 64) SAPA_PROJECT_CASE(128, 128)
    SAPA_PROJECT_CASE(256, 32) SAPA_PROJECT_CASE(256, 64) SAPA_PROJECT_CASE(256, 128)
    SAPA_PROJECT_CASE(512, 32) SAPA_PROJECT_CASE(512, 64)
#undef SAPA_PROJECT_CASE
    return hipErrorNotSupported;
}

}  // namespace project

// x [B, HW, C], w [B, O, C], bias [B, O] or null, out [B, HW, O]; f16 / bf16;
// (C, O) among the instantiated pairs (C in {64, 128, 256, 512}, O in {32, 64, 128});
// every pointer aligned to 16 bytes.  hipErrorNotSupported otherwise.
hipError_t project_nhwc_launch(const void *x, const void *w, const void *bias, void *out, int B,
                               int C, int O, long HW, int dtype, hipStream_t st) {
    const void *ptrs[3] = {x, w, out};
    for (const void *p : ptrs)
        if ((uintptr_t)p % 16 != 0) return hipErrorNotSupported;
    if (dtype == 2) return project::launch_t<f16_t>(x, w, bias, out, B, C, O, HW, st);
    if (dtype == 3) return project::launch_t<bf16_t>(x, w, bias, out, B, C, O, HW, st);
    return hipErrorNotSupported;
}

}  // namespace sapa
