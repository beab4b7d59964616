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
//
// fp32 features (project32_kernel) take the same stream through the bf16 matrix
// instruction: every fp32 number is the exact sum of three bf16 numbers (8 + 8 + 8
// significant bits), a product of two bf16 numbers is exact in fp32, and of the nine
// piece products of x * w the six largest are kept (the other three are below 2^-23 of
// the product): six v_mfma_f32_16x16x32_bf16 per fp32 matrix step, fp32 sums -- an
// fp32 dot product to fp32 rounding at 32 / 6 times the rate of the fp32 matrix
// instruction, which leaves the kernel waiting for memory, not arithmetic.  The image's
// weights are taken apart once per workgroup into three bf16 planes in LDS; x goes
// from global memory straight into the A-operand registers (a lane reads two 16-byte
// pieces of its pixel's record per step of 32 channels) and is taken apart there.
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

template <typename T> struct Mma32;
template <> struct Mma32<f16_t> {
    static __device__ __forceinline__ f32x4 run(u32x4 a, u32x4 b, f32x4 c) {
        typedef _Float16 v8 __attribute__((ext_vector_type(8)));
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8, a), __builtin_bit_cast(v8, b), c, 0, 0, 0);
    }
};
template <> struct Mma32<bf16_t> {
    static __device__ __forceinline__ f32x4 run(u32x4 a, u32x4 b, f32x4 c) {
        typedef __bf16 v8 __attribute__((ext_vector_type(8)));
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8, a), __builtin_bit_cast(v8, b), c, 0, 0, 0);
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
    // two workgroups are resident per CU (LDS) and the part has 256 CUs: one round of at most 512
    // workgroups, at least 2 tiles per wave (16 images of 100 x 168 pixels, 256 -> 64: 37 us against
    // 46 with a fixed 8 tiles per wave; 200 x 336 pixels: 141 against 146)
    long per = (ntiles * B + 4L * 512 - 1) / (4L * 512);
    if (per < 2) per = 2;
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

// ---- 16-bit, contiguous feature (planes) ----
// x [B, C, HW]: a lane fetches 8 neighbouring pixels of one channel (a wave: 8 channels x 128
// bytes per load); a reduction step's 32 channels x 64 pixels pass through a wave-private LDS
// tile [channel][pixel] from which ds_read_tr16_b64 hands every lane its pixel's 4 channels (rows
// of 160 bytes: the four rows of a transposing read lie on disjoint banks).  Same order of the
// channels inside a step as in the fp32 kernel below; weights [O][C] in that order in LDS.
// Tiles of 64 pixels (four blocks of 16 matrix rows).  OUT_CL: out [B, HW, O], else [B, O, HW].
// HW a multiple of 8 (16-byte pieces never run from one plane into the next).
template <typename T, int C, int O, bool OUT_CL>
__global__ void __launch_bounds__(256)
project16p_kernel(const T *__restrict__ x, const T *__restrict__ w, const T *__restrict__ bias,
                  T *__restrict__ out, long HW, int tiles_per_wave) {
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    constexpr int NW = 4;
    constexpr int RW = C / 2 + 4;                 // dwords per padded row of C 16-bit values
    constexpr int NT = O / 16;                    // output tiles of 16 columns
    constexpr int OW = O / 2 + 4;                 // dwords per padded row of the result tile (channels-last)
    constexpr int PW = 64 / 2 + 4;                // ... of a block of 16 outputs x 64 pixels (planes)
    constexpr int XS = 64 / 2 + 8;                // dwords per row of the x tile: 160 bytes
    constexpr int KS = C / 32;                    // reduction steps
    constexpr int RING = KS < 4 ? KS : 4;         // steps of x in flight
    constexpr int RT = OUT_CL ? 16 * OW : 16 * PW;
    constexpr int WF = RT > 32 * XS ? RT : 32 * XS;
    static_assert(KS % RING == 0, "the ring of x registers is indexed by the step");
    extern __shared__ __attribute__((aligned(16))) u32 sh[];
    u32 *wl = sh;                                 // weights: O rows of RW dwords
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    u32 *xt = sh + O * RW + wave * WF;            // this wave's x tile / result tile
    const int b = blockIdx.y;

    // the image's weights -> LDS, 8 channels per thread and step: two groups of 4, which lie 8
    // places apart in the step's order
    {
        const u32x4 *src = (const u32x4 *)(w + (long)b * O * C);
        for (int i = threadIdx.x; i < O * C / 8; i += 64 * NW) {
            const int o = i / (C / 8), c = 8 * (i % (C / 8)), cs = c % 32;
            const int pos = 32 * (c / 32) + 8 * ((cs % 16) / 4) + 4 * (cs / 16);
            const u32x4 v = src[i];
            u32 *dst = wl + o * RW + pos / 2;
            *(u32x2 *)dst = u32x2{v[0], v[1]};
            *(u32x2 *)(dst + 4) = u32x2{v[2], v[3]};
        }
    }
    __syncthreads();

    const long ntiles = (HW + 63) / 64;
    const long t0 = ((long)blockIdx.x * NW + wave) * tiles_per_wave;
    const long t1 = t0 + tiles_per_wave < ntiles ? t0 + tiles_per_wave : ntiles;
    if (t0 >= t1) return;
    const int r16 = lane & 15, kg = lane >> 4;
    float bv[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) bv[nt] = bias ? (float)bias[(long)b * O + 16 * nt + r16] : 0.f;

    const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(x + (long)b * HW * C), 0, (int)(HW * C * 2), 0x00020000);
    const __amdgpu_buffer_rsrc_t ro = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(out + (long)b * HW * O), 0, (int)(HW * O * 2), 0x00020000);
    // step (t, ks) of x: piece j = pixels 8 (lane % 8) .. + 7 of channel 8 j + lane / 8 of the step
    const u32 xoff = (u32)((lane >> 3) * HW + 8 * (lane & 7)) * 2u, xstride = (u32)(8 * HW * 2);
    u32x4 raw[RING][4];
    auto load_step = [&](int slot, long t, int ks) __attribute__((always_inline)) {
        const u32 so = (u32)((32L * ks * HW + t * 64) * 2);
#pragma unroll
        for (int j = 0; j < 4; ++j)
            raw[slot][j] = __builtin_amdgcn_raw_buffer_load_b128(rx, xoff + (u32)j * xstride, so, 0);
    };
    u32 *const xw = xt + (lane >> 3) * XS + 4 * (lane & 7);
    // transposing reads: lane L of a 16-lane block addresses row L / 4, pixels 4 (L % 4) .. + 3 of
    // the block's 16 and receives pixel L's value of the 4 rows; block kg takes channels 4 kg ..
    // (and 16 + 4 kg ..) of the step
    const u32 *const xr = xt + (4 * kg + (r16 >> 2)) * XS + 2 * (r16 & 3);
#pragma unroll
    for (int k = 0; k < RING; ++k) load_step(k, t0, k);
    for (long t = t0; t < t1; ++t) {
        f32x4 acc[4][NT];
#pragma unroll
        for (int mb = 0; mb < 4; ++mb)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) acc[mb][nt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
            for (int j = 0; j < 4; ++j) *(u32x4 *)(xw + 8 * j * XS) = raw[ks % RING][j];
            if (ks + RING < KS) load_step(ks % RING, t, ks + RING);
            else if (t + 1 < t1) load_step(ks % RING, t + 1, ks + RING - KS);
            u32x4 a[4];
#pragma unroll
            for (int mb = 0; mb < 4; ++mb) {
                const u32x2 lo = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                                     (s16x4 __attribute__((address_space(3))) *)(xr + 8 * mb)));
                const u32x2 hi = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                                     (s16x4 __attribute__((address_space(3))) *)(xr + 16 * XS + 8 * mb)));
                a[mb] = u32x4{lo[0], lo[1], hi[0], hi[1]};
            }
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const u32x4 bm = *(const u32x4 *)(wl + (16 * nt + r16) * RW + 16 * ks + 4 * kg);
#pragma unroll
                for (int mb = 0; mb < 4; ++mb) acc[mb][nt] = Mma32<T>::run(a[mb], bm, acc[mb][nt]);
            }
        }
        // acc[mb][nt][i]: pixel 16 mb + 4 kg + i, output 16 nt + r16
        if (OUT_CL) {
            // 16 rows of 2 O bytes per block -> one contiguous run of 32 O bytes
            unsigned short *rt = (unsigned short *)xt;
#pragma unroll
            for (int mb = 0; mb < 4; ++mb) {
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                        rt[(4 * kg + i) * (2 * OW) + 16 * nt + r16] = (unsigned short)pack2<T>(acc[mb][nt][i] + bv[nt], 0.f);
                const u32 obase = (u32)((t * 64 + 16 * mb) * O * 2);
#pragma unroll
                for (int j = 0; j < (16 * O / 8 + 63) / 64; ++j) {
                    const int i = j * 64 + lane, row = i / (O / 8), col = i % (O / 8);
                    if (16 * O / 8 % 64 == 0 || i < 16 * O / 8)
                        __builtin_amdgcn_raw_buffer_store_b128(*(const u32x4 *)(xt + row * OW + 4 * col), ro, (u32)(i * 16), obase, 2);
                }
            }
        } else {
            // a block of 16 outputs x 64 pixels (a lane holds 4 neighbouring pixels), then 16 rows of
            // 128 bytes; pieces past the plane's end are dropped
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
                for (int mb = 0; mb < 4; ++mb)
                    *(u32x2 *)(xt + r16 * PW + 8 * mb + 2 * kg) =
                        u32x2{pack2<T>(acc[mb][nt][0] + bv[nt], acc[mb][nt][1] + bv[nt]),
                              pack2<T>(acc[mb][nt][2] + bv[nt], acc[mb][nt][3] + bv[nt])};
                const u32 obase = (u32)((16L * nt * HW + t * 64) * 2);
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const int row = 8 * j + (lane >> 3), col = lane & 7;
                    const u32 off = t * 64 + 8 * col < HW ? (u32)(row * HW + 8 * col) * 2u : 0x80000000u;
                    __builtin_amdgcn_raw_buffer_store_b128(*(const u32x4 *)(xt + row * PW + 4 * col), ro, off, obase, 2);
                }
            }
        }
    }
}

template <typename T, int C, int O, bool OUT_CL>
static hipError_t launch16p_co(const void *x, const void *w, const void *bias, void *out, int B, long HW,
                               hipStream_t st) {
    constexpr int RT = OUT_CL ? 16 * (O / 2 + 4) : 16 * 36, XT = 32 * 40;
    constexpr size_t lds = (size_t)(O * (C / 2 + 4) + 4 * (RT > XT ? RT : XT)) * 4;
    static_assert(lds <= 64 * 1024, "weights and tiles within the default LDS of a workgroup");
    if (HW % 8 != 0 || HW * (long)(C > O ? C : O) * 2 >= (1L << 31)) return hipErrorNotSupported;
    const long ntiles = (HW + 63) / 64;
    // two workgroups are resident per CU (their registers) and the part has 256 CUs: one round of
    // at most 512 workgroups, at least 2 tiles per wave (q projection at 16 x 200 x 336 pixels:
    // 140 us against 152 with 704 workgroups)
    long per = (ntiles * B + 4L * 512 - 1) / (4L * 512);
    if (per < 2) per = 2;
    const long blocks = (ntiles + 4 * per - 1) / (4 * per);
    if (blocks > 65535 * 32L || B > 65535) return hipErrorNotSupported;
    hipLaunchKernelGGL((project16p_kernel<T, C, O, OUT_CL>), dim3((unsigned)blocks, B), dim3(256), lds, st,
                       (const T *)x, (const T *)w, (const T *)bias, (T *)out, HW, (int)per);
    return hipGetLastError();
}

template <typename T, bool OUT_CL>
static hipError_t launch16p(const void *x, const void *w, const void *bias, void *out, int B, int C, int O,
                            long HW, hipStream_t st) {
#define SAPA_PROJECT_CASE(CV, OV) \
    if (C == CV && O == OV) return launch16p_co<T, CV, OV, OUT_CL>(x, w, bias, out, B, HW, st);
    SAPA_PROJECT_CASE(64, 32) SAPA_PROJECT_CASE(64, 64)
    SAPA_PROJECT_CASE(128, 32) SAPA_PROJECT_CASE(128, 64)
    SAPA_PROJECT_CASE(256, 32) SAPA_PROJECT_CASE(256, 64)
    SAPA_PROJECT_CASE(512, 32)
#undef SAPA_PROJECT_CASE
    return hipErrorNotSupported;
}

// ---- fp32 ----
// the three bf16 pieces of two fp32 numbers, each pair packed in a dword (x0 in the low half)
struct Pieces {
    u32 hi, mid, lo;
};
__device__ __forceinline__ Pieces split2(float x0, float x1) {
    const u32 TOP = 0xffff0000u, SEL = 0x07060302u;        // SEL: the upper halves of two dwords
    const u32 u0 = __builtin_bit_cast(u32, x0), u1 = __builtin_bit_cast(u32, x1);
    const float r0 = x0 - __builtin_bit_cast(float, u0 & TOP), r1 = x1 - __builtin_bit_cast(float, u1 & TOP);
    const u32 v0 = __builtin_bit_cast(u32, r0), v1 = __builtin_bit_cast(u32, r1);
    const float l0 = r0 - __builtin_bit_cast(float, v0 & TOP), l1 = r1 - __builtin_bit_cast(float, v1 & TOP);
    Pieces p;
    p.hi = __builtin_amdgcn_perm(u1, u0, SEL);
    p.mid = __builtin_amdgcn_perm(v1, v0, SEL);
    p.lo = __builtin_amdgcn_perm(__builtin_bit_cast(u32, l1), __builtin_bit_cast(u32, l0), SEL);
    return p;
}
__device__ __forceinline__ f32x4 mma32(u32x4 a, u32x4 b, f32x4 c) {
    typedef __bf16 v8 __attribute__((ext_vector_type(8)));
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8, a), __builtin_bit_cast(v8, b), c, 0, 0, 0);
}

// C input channels (a multiple of 32), O outputs (a multiple of 16); 8 waves, tiles of 32
// pixels (two blocks of 16 matrix rows share every weight operand read from LDS).
// Reduction step ks takes channels 32 ks ..; inside it lane group kg holds channels
// 4 kg .. + 3 and 16 + 4 kg .. + 3 (two 16-byte pieces of memory; the 16 lanes of a piece
// read 64 contiguous bytes per pixel) -- the weight planes are stored in that order.
//
// IN_CL = false: x is [B, C, HW] (contiguous planes).  A lane fetches 4 neighbouring pixels of
// one channel (a wave: 8 channels x 128 bytes per load), four such loads per step, and the step's
// 32 channels x 32 pixels pass through a wave-private LDS tile from which the A operands are read
// as single dwords (the 16-pixel halves of a row swapped for every other group of 4 channels, so
// that the two channel groups of a half-wave read disjoint banks).  OUT_CL = false: out is
// [B, O, HW]; a block of 16 outputs x 32 pixels goes back through LDS and leaves as 128-byte rows
// (HW a multiple of 4: a 16-byte piece never runs from one plane into the next).
template <int C, int O, bool IN_CL, bool OUT_CL>
__global__ void __launch_bounds__(512)
project32_kernel(const float *__restrict__ x, const float *__restrict__ w, const float *__restrict__ bias,
                 float *__restrict__ out, long HW, int tiles_per_wave) {
    static_assert(IN_CL ? OUT_CL : true, "channels-last features give channels-last projections");
    constexpr int NW = 8;
    constexpr int RW = C / 2 + 4;                 // dwords per padded row of C bf16 values
    constexpr int PLANE = O * RW;                 // dwords per piece plane
    constexpr int NT = O / 16;                    // output tiles of 16 columns
    constexpr int OS = O + 4;                     // floats per padded row of the result tile (channels-last)
    constexpr int PS = 32 + 4;                    // ... of a block of 16 outputs x 32 pixels (planes)
    constexpr int XB = IN_CL ? 0 : 32 * 32;       // floats of the wave's x tile
    constexpr int RT = OUT_CL ? 16 * OS : 16 * PS;
    constexpr int WF = RT > XB ? RT : XB;         // floats of a wave's LDS (x tile, then results)
    constexpr int KS = C / 32;                    // reduction steps
    constexpr int RING = KS < 4 ? KS : 4;         // steps of x in flight
    static_assert(KS % RING == 0, "the ring of x registers is indexed by the step");
    extern __shared__ __attribute__((aligned(16))) u32 sh[];
    u32 *wl = sh;                                 // weights: 3 planes of O rows of RW dwords
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    float *rt = (float *)(sh + 3 * PLANE) + wave * WF;          // this wave's x tile / result tile
    const int b = blockIdx.y;

    // the image's weights, taken apart, -> LDS (two neighbouring channels per thread and step)
    {
        typedef float f32x2 __attribute__((ext_vector_type(2)));
        const f32x2 *src = (const f32x2 *)(w + (long)b * O * C);
        for (int i = threadIdx.x; i < O * C / 2; i += 64 * NW) {
            const int o = i / (C / 2), c = 2 * (i % (C / 2)), cs = c % 32;
            const int pos = 32 * (c / 32) + 8 * ((cs % 16) / 4) + 4 * (cs / 16) + cs % 4;
            const f32x2 v = src[i];
            const Pieces pc = split2(v[0], v[1]);
            u32 *dst = wl + o * RW + pos / 2;
            dst[0] = pc.hi;
            dst[PLANE] = pc.mid;
            dst[2 * PLANE] = pc.lo;
        }
    }
    __syncthreads();

    const long ntiles = (HW + 31) / 32;
    const long t0 = ((long)blockIdx.x * NW + wave) * tiles_per_wave;
    const long t1 = t0 + tiles_per_wave < ntiles ? t0 + tiles_per_wave : ntiles;
    if (t0 >= t1) return;
    const int r16 = lane & 15, kg = lane >> 4;    // row / column of a 16 x 16 tile, k group
    float bv[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) bv[nt] = bias ? bias[(long)b * O + 16 * nt + r16] : 0.f;

    // byte offsets inside the image: out of range = past the last pixel = zeros / dropped
    const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(x + (long)b * HW * C), 0, (int)(HW * C * 4), 0x00020000);
    const __amdgpu_buffer_rsrc_t ro = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(out + (long)b * HW * O), 0, (int)(HW * O * 4), 0x00020000);
    // step (t, ks) of x, 4 pieces of 16 bytes per lane.  Channels-last: blocks mb = 0, 1 x pieces
    // h = 0, 1 of pixel r16's record.  Planes: piece j = pixels 4 (lane % 8) .. + 3 of channel
    // 8 j + lane / 8 of the step
    const u32 xoff = IN_CL ? (u32)(r16 * C + 4 * kg) * 4u : (u32)((lane >> 3) * HW + 4 * (lane & 7)) * 4u;
    const u32 xstride = IN_CL ? 0u : (u32)(8 * HW * 4);
    u32x4 raw[RING][2][2];
    auto load_step = [&](int slot, long t, int ks) __attribute__((always_inline)) {
        const u32 so = IN_CL ? (u32)((t * 32 * C + 32 * ks) * 4) : (u32)((32L * ks * HW + t * 32) * 4);
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
#pragma unroll
            for (int h = 0; h < 2; ++h)
                raw[slot][mb][h] = __builtin_amdgcn_raw_buffer_load_b128(
                    rx, IN_CL ? xoff + (u32)((mb * 16 * C + 16 * h) * 4) : xoff + (u32)(2 * mb + h) * xstride, so, 0);
    };
    // (planes) the x tile [32 channels][32 pixels]: where this lane writes its pieces, and where it
    // reads channel 4 kg (+ 16) of pixel r16 (+ 16)
    float *const xw = rt + (lane >> 3) * 32 + (((lane & 7) ^ ((lane >> 5) << 2)) << 2);
    const float *const xr = rt + 4 * kg * 32 + ((((r16 >> 2)) ^ ((kg & 1) << 2)) << 2) + (r16 & 3);
#pragma unroll
    for (int k = 0; k < RING; ++k) load_step(k, t0, k);
    for (long t = t0; t < t1; ++t) {
        f32x4 acc[2][NT];
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) acc[mb][nt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            u32x4 ahi[2], amid[2], alo[2];
            if (!IN_CL) {
#pragma unroll
                for (int j = 0; j < 4; ++j) *(u32x4 *)(xw + 8 * j * 32) = raw[ks % RING][j >> 1][j & 1];
            }
#pragma unroll
            for (int mb = 0; mb < 2; ++mb) {
                f32x4 p0, p1;
                if (IN_CL) {
                    p0 = __builtin_bit_cast(f32x4, raw[ks % RING][mb][0]);
                    p1 = __builtin_bit_cast(f32x4, raw[ks % RING][mb][1]);
                } else {
                    // (block mb: the other 16-pixel half of the row, i.e. piece index bit 2 flipped)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        p0[e] = xr[e * 32 + (mb ? 16 - 32 * (kg & 1) : 0)];
                        p1[e] = xr[(16 + e) * 32 + (mb ? 16 - 32 * (kg & 1) : 0)];
                    }
                }
                const Pieces s0 = split2(p0[0], p0[1]), s1 = split2(p0[2], p0[3]);
                const Pieces s2 = split2(p1[0], p1[1]), s3 = split2(p1[2], p1[3]);
                ahi[mb] = u32x4{s0.hi, s1.hi, s2.hi, s3.hi};
                amid[mb] = u32x4{s0.mid, s1.mid, s2.mid, s3.mid};
                alo[mb] = u32x4{s0.lo, s1.lo, s2.lo, s3.lo};
            }
            // the ring slot is free: the step RING further on (of this tile or of the next)
            if (ks + RING < KS) load_step(ks % RING, t, ks + RING);
            else if (t + 1 < t1) load_step(ks % RING, t + 1, ks + RING - KS);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const u32 *wp = wl + (16 * nt + r16) * RW + 16 * ks + 4 * kg;
                const u32x4 bhi = *(const u32x4 *)wp, bmid = *(const u32x4 *)(wp + PLANE), blo = *(const u32x4 *)(wp + 2 * PLANE);
#pragma unroll
                for (int mb = 0; mb < 2; ++mb) {
                    // smallest terms first
                    f32x4 a = mma32(ahi[mb], blo, acc[mb][nt]);
                    a = mma32(alo[mb], bhi, a);
                    a = mma32(amid[mb], bmid, a);
                    a = mma32(ahi[mb], bmid, a);
                    a = mma32(amid[mb], bhi, a);
                    acc[mb][nt] = mma32(ahi[mb], bhi, a);
                }
            }
        }
        // acc[mb][nt][i]: pixel 16 mb + 4 kg + i, output 16 nt + r16
        if (!OUT_CL) {
            // planes: a block of 16 outputs x 32 pixels -> the wave's tile (a lane holds 4
            // neighbouring pixels), then 16 rows of 128 bytes; pieces past the plane's end are dropped
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
                for (int mb = 0; mb < 2; ++mb) {
                    const f32x4 v = {acc[mb][nt][0] + bv[nt], acc[mb][nt][1] + bv[nt], acc[mb][nt][2] + bv[nt],
                                     acc[mb][nt][3] + bv[nt]};
                    *(f32x4 *)(rt + r16 * PS + 16 * mb + 4 * kg) = v;
                }
                const u32 obase = (u32)((16L * nt * HW + t * 32) * 4);
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const int row = 8 * j + (lane >> 3), col = lane & 7;
                    const u32 off = t * 32 + 4 * col < HW ? (u32)(row * HW + 4 * col) * 4u : 0x80000000u;
                    __builtin_amdgcn_raw_buffer_store_b128(*(const u32x4 *)(rt + row * PS + 4 * col), ro, off, obase, 2);
                }
            }
            continue;
        }
        // channels-last: the wave's tile, then 16 rows of 4 O bytes -> one contiguous run of 64 O
        // bytes per block
#pragma unroll
        for (int mb = 0; mb < 2; ++mb) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int i = 0; i < 4; ++i) rt[(4 * kg + i) * OS + 16 * nt + r16] = acc[mb][nt][i] + bv[nt];
            const u32 obase = (u32)((t * 32 + 16 * mb) * O * 4);
#pragma unroll
            for (int j = 0; j < (16 * O / 4 + 63) / 64; ++j) {
                const int i = j * 64 + lane, row = i / (O / 4), col = i % (O / 4);
                if (16 * O / 4 % 64 == 0 || i < 16 * O / 4)
                    __builtin_amdgcn_raw_buffer_store_b128(*(const u32x4 *)(rt + row * OS + 4 * col), ro, (u32)(i * 16), obase, 2);
            }
        }
    }
}

template <int C, int O, bool IN_CL, bool OUT_CL>
static hipError_t launch32_co(const void *x, const void *w, const void *bias, void *out, int B, long HW,
                              hipStream_t st) {
    constexpr int RT = OUT_CL ? 16 * (O + 4) : 16 * 36, XB = IN_CL ? 0 : 32 * 32;
    constexpr size_t lds = (size_t)(3 * O * (C / 2 + 4) + 8 * (RT > XB ? RT : XB)) * 4;
    if (!OUT_CL && HW % 4 != 0) return hipErrorNotSupported;
    static_assert(lds <= 160 * 1024, "weights and tiles must fit LDS");
    // 32-bit byte offsets inside an image
    if (HW * (long)(C > O ? C : O) * 4 >= (1L << 31)) return hipErrorNotSupported;
    const long ntiles = (HW + 31) / 32;
    // One workgroup is resident per CU (its weight planes fill most of the LDS) and the part has
    // 256 CUs: two full rounds of workgroups where that leaves a wave 8 tiles or more, else one
    // (16 images: 200x336 pixels 301 us in two rounds against 315 in one; 100x168 pixels 71 us in
    // one round against 98 in 272 workgroups)
    const long slots = 256;
    long blocks = 2 * slots / B > 1 ? 2 * slots / B : 1;
    long per = (ntiles + 8 * blocks - 1) / (8 * blocks);
    if (per < 8) {
        blocks = slots / B > 1 ? slots / B : 1;
        per = (ntiles + 8 * blocks - 1) / (8 * blocks);
    }
    blocks = (ntiles + 8 * per - 1) / (8 * per);
    if (blocks > 65535 * 32L || B > 65535) return hipErrorNotSupported;
    auto kern = project32_kernel<C, O, IN_CL, OUT_CL>;
    if (lds > 64 * 1024) {
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
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks, B), dim3(512), lds, st, (const float *)x, (const float *)w,
                       (const float *)bias, (float *)out, HW, (int)per);
    return hipGetLastError();
}

template <bool IN_CL, bool OUT_CL>
static hipError_t launch32(const void *x, const void *w, const void *bias, void *out, int B, int C, int O,
                           long HW, hipStream_t st) {
#define SAPA_PROJECT_CASE(CV, OV) \
    if (C == CV && O == OV) return launch32_co<CV, OV, IN_CL, OUT_CL>(x, w, bias, out, B, HW, st);
    SAPA_PROJECT_CASE(64, 32) SAPA_PROJECT_CASE(64, 64)
    SAPA_PROJECT_CASE(128, 32) SAPA_PROJECT_CASE(128, 64)
    SAPA_PROJECT_CASE(256, 32) SAPA_PROJECT_CASE(256, 64)
    SAPA_PROJECT_CASE(512, 32)
#undef SAPA_PROJECT_CASE
    return hipErrorNotSupported;
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

// x [B, HW, C], w [B, O, C], bias [B, O] or null, out [B, HW, O]; f16 / bf16 / fp32;
// (C, O) among the instantiated pairs (C in {64, 128, 256, 512}, O in {32, 64, 128}; fp32:
// those whose three weight planes fit LDS); every pointer aligned to 16 bytes.
// hipErrorNotSupported otherwise.
hipError_t project_nhwc_launch(const void *x, const void *w, const void *bias, void *out, int B,
                               int C, int O, long HW, int dtype, hipStream_t st) {
    const void *ptrs[3] = {x, w, out};
    for (const void *p : ptrs)
        if ((uintptr_t)p % 16 != 0) return hipErrorNotSupported;
    if (dtype == 0) return project::launch32<true, true>(x, w, bias, out, B, C, O, HW, st);
    if (dtype == 2) return project::launch_t<f16_t>(x, w, bias, out, B, C, O, HW, st);
    if (dtype == 3) return project::launch_t<bf16_t>(x, w, bias, out, B, C, O, HW, st);
    return hipErrorNotSupported;
}

// The same projection of a contiguous feature x [B, C, HW] (planes): out [B, HW, O]
// (out_channels_last) or [B, O, HW]; the (C, O) pairs of the fp32 kernel above; fp32: HW a
// multiple of 4 for a planar result; f16 / bf16: HW a multiple of 8; x and out aligned to 16
// bytes.  hipErrorNotSupported otherwise.
hipError_t project_nchw_launch(const void *x, const void *w, const void *bias, void *out, int B, int C,
                               int O, long HW, int out_channels_last, int dtype, hipStream_t st) {
    const void *ptrs[3] = {x, w, out};
    for (const void *p : ptrs)
        if ((uintptr_t)p % 16 != 0) return hipErrorNotSupported;
    if (dtype == 2)
        return out_channels_last ? project::launch16p<f16_t, true>(x, w, bias, out, B, C, O, HW, st)
                                 : project::launch16p<f16_t, false>(x, w, bias, out, B, C, O, HW, st);
    if (dtype == 3)
        return out_channels_last ? project::launch16p<bf16_t, true>(x, w, bias, out, B, C, O, HW, st)
                                 : project::launch16p<bf16_t, false>(x, w, bias, out, B, C, O, HW, st);
    if (dtype != 0) return hipErrorNotSupported;
    return out_channels_last ? project::launch32<false, true>(x, w, bias, out, B, C, O, HW, st)
                             : project::launch32<false, false>(x, w, bias, out, B, C, O, HW, st);
}

// Whether project_nhwc_launch (x_channels_last; the result is channels-last then) / project_nchw_launch
// has a kernel for the configuration, pointer alignment aside.
bool project_supported(int C, int O, long HW, bool x_channels_last, bool out_channels_last, int dtype) {
    const bool small_pair = (C == 64 && (O == 32 || O == 64)) || (C == 128 && (O == 32 || O == 64)) ||
                            (C == 256 && (O == 32 || O == 64)) || (C == 512 && O == 32);
    if (dtype == 2 || dtype == 3) {
        if (x_channels_last)
            return out_channels_last && (small_pair || (C == 128 && O == 128) || (C == 256 && O == 128) || (C == 512 && O == 64));
        return small_pair && HW % 8 == 0 && HW * (long)(C > O ? C : O) * 2 < (1L << 31);
    }
    if (dtype != 0 || !small_pair || HW * (long)(C > O ? C : O) * 4 >= (1L << 31)) return false;
    if (x_channels_last) return out_channels_last;
    return out_channels_last || HW % 4 == 0;
}

}  // namespace sapa
