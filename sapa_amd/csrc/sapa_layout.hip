// Layout helpers: a contiguous [B, C, H*W] tensor copied into channels-last
// order [B, H*W, C].  The matrix-form SAPA-D kernels read their low-res key and
// value windows in channels-last order (a window cell's channels are one
// contiguous piece); for callers with the reference's contiguous tensors
// (deformsapa/deformsapa/src/cuda/deform_qk_cuda.cpp:37-43: CHECK_CONTIGUOUS)
// these two small tensors are copied into a caller-provided workspace first,
// while the large hi-res tensors are read and written in place.
#include "kernels.hpp"

namespace sapa {

namespace layout {

// 64 pixels x 64 channels per workgroup through LDS: reads run along the
// pixels of a channel plane, writes along the channels of a pixel.  Two tensors
// of the same extent [B, C*, HW] in one launch: blockIdx.y < yblocks0 works on
// the first.
template <typename U>
__global__ void __launch_bounds__(256)
nchw_to_nhwc_kernel(const U *__restrict__ src0, U *__restrict__ dst0, int C0, int yblocks0,
                    const U *__restrict__ src1, U *__restrict__ dst1, int C1, long HW) {
    __shared__ U tile[64][65];
    const bool first = (int)blockIdx.y < yblocks0;
    const U *src = first ? src0 : src1;
    U *dst = first ? dst0 : dst1;
    const int C = first ? C0 : C1;
    const long p0 = (long)blockIdx.x * 64;
    const int c0 = ((int)blockIdx.y - (first ? 0 : yblocks0)) * 64;
    const long n = blockIdx.z;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    for (int c = ty; c < 64; c += 4)
        tile[c][tx] = (c0 + c < C && p0 + tx < HW) ? src[(n * C + c0 + c) * HW + p0 + tx] : (U)0;
    __syncthreads();
    for (int p = ty; p < 64; p += 4)
        if (c0 + tx < C && p0 + p < HW) dst[(n * HW + p0 + p) * C + c0 + tx] = tile[tx][p];
}

// The same with 4-element vectors on both sides (pixel counts and channel counts
// that are multiples of 4, aligned pointers): a thread reads 4 x-neighbours of a
// channel plane and writes 4 channels of a pixel -- a quarter of the memory
// instructions of the kernel above, which is bound by their number.
template <typename U>
__global__ void __launch_bounds__(256)
nchw_to_nhwc_vec_kernel(const U *__restrict__ src0, U *__restrict__ dst0, int C0, int yblocks0,
                        const U *__restrict__ src1, U *__restrict__ dst1, int C1, long HW,
                        float *__restrict__ zero0, float *__restrict__ zero1) {
    struct alignas(4 * sizeof(U)) V4 { U v[4]; };
    __shared__ U tile[64][65];
    const bool first = (int)blockIdx.y < yblocks0;
    const U *src = first ? src0 : src1;
    U *dst = first ? dst0 : dst1;
    float *zero = first ? zero0 : zero1;
    const int C = first ? C0 : C1;
    const long p0 = (long)blockIdx.x * 64;
    const int c0 = ((int)blockIdx.y - (first ? 0 : yblocks0)) * 64;
    const long n = blockIdx.z;
#pragma unroll
    for (int it = 0; it < 4; ++it) {
        const int i = it * 256 + (int)threadIdx.x, c = i / 16, pq = i % 16;
        V4 x = {};
        if (c0 + c < C && p0 + 4 * pq < HW) x = *(const V4 *)(src + (n * C + c0 + c) * HW + p0 + 4 * pq);
#pragma unroll
        for (int e = 0; e < 4; ++e) tile[c][4 * pq + e] = x.v[e];
    }
    __syncthreads();
#pragma unroll
    for (int it = 0; it < 4; ++it) {
        const int i = it * 256 + (int)threadIdx.x, p = i / 16, cq = i % 16;
        if (c0 + 4 * cq < C && p0 + p < HW) {
            V4 x;
#pragma unroll
            for (int e = 0; e < 4; ++e) x.v[e] = tile[4 * cq + e][p];
            *(V4 *)(dst + (n * HW + p0 + p) * C + c0 + 4 * cq) = x;
            // an fp32 buffer of the same extent cleared on the way (the accumulator of
            // the tensor's gradient: one launch less)
            if (zero) {
                struct alignas(16) F4 { float v[4]; };
                *(F4 *)(zero + (n * HW + p0 + p) * C + c0 + 4 * cq) = F4{};
            }
        }
    }
}

// The way back for an fp32 accumulation buffer: channels-last [B, HW, C] floats
// into a contiguous [B, C, HW] tensor of type T (rounded once).
template <typename T>
__global__ void __launch_bounds__(256)
nhwc_f32_to_nchw_kernel(const float *__restrict__ src, T *__restrict__ dst, int C, long HW) {
    __shared__ float tile[64][65];
    const long p0 = (long)blockIdx.x * 64;
    const int c0 = (int)blockIdx.y * 64;
    const long n = blockIdx.z;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    for (int p = ty; p < 64; p += 4)
        tile[p][tx] = (c0 + tx < C && p0 + p < HW) ? src[(n * HW + p0 + p) * C + c0 + tx] : 0.f;
    __syncthreads();
    for (int c = ty; c < 64; c += 4)
        if (c0 + c < C && p0 + tx < HW) dst[(n * C + c0 + c) * HW + p0 + tx] = (T)tile[tx][c];
}

// (with 4-element vectors on both sides, as above)
template <typename T>
__global__ void __launch_bounds__(256)
nhwc_f32_to_nchw_vec_kernel(const float *__restrict__ src, T *__restrict__ dst, int C, long HW) {
    struct alignas(16) F4 { float v[4]; };
    struct alignas(4 * sizeof(T)) V4 { T v[4]; };
    __shared__ float tile[64][65];      // [pixel][channel]
    const long p0 = (long)blockIdx.x * 64;
    const int c0 = (int)blockIdx.y * 64;
    const long n = blockIdx.z;
#pragma unroll
    for (int it = 0; it < 4; ++it) {
        const int i = it * 256 + (int)threadIdx.x, p = i / 16, cq = i % 16;
        F4 x = {};
        if (c0 + 4 * cq < C && p0 + p < HW) x = *(const F4 *)(src + (n * HW + p0 + p) * C + c0 + 4 * cq);
#pragma unroll
        for (int e = 0; e < 4; ++e) tile[p][4 * cq + e] = x.v[e];
    }
    __syncthreads();
#pragma unroll
    for (int it = 0; it < 4; ++it) {
        const int i = it * 256 + (int)threadIdx.x, c = i / 16, pq = i % 16;
        if (c0 + c < C && p0 + 4 * pq < HW) {
            V4 x;
#pragma unroll
            for (int e = 0; e < 4; ++e) x.v[e] = (T)tile[4 * pq + e][c];
            *(V4 *)(dst + (n * C + c0 + c) * HW + p0 + 4 * pq) = x;
        }
    }
}

}  // namespace layout

// Two tensors [B, C0, HW] and [B, C1, HW] (C1 = 0: one) in one launch.  esize:
// bytes per element, 2 or 4.  zero0 / zero1 (may be NULL): fp32 buffers of the two
// tensors' extents that the vector form of the kernel clears on the way; *zeroed
// says whether it did.  hipErrorNotSupported otherwise, or for more than
// 65535 images or 64-channel blocks.
hipError_t nchw_to_nhwc_launch(const void *src0, void *dst0, int C0, const void *src1, void *dst1,
                               int C1, int B, long HW, int esize, hipStream_t st, float *zero0, float *zero1,
                               bool *zeroed) {
    if (zeroed) *zeroed = false;
    if (B <= 0 || C0 <= 0 || HW <= 0) return hipSuccess;
    const long gx = (HW + 63) / 64;
    const int gy0 = (C0 + 63) / 64, gy1 = (C1 + 63) / 64;
    if (gx > 0x7fffffffL || gy0 + gy1 > 65535 || B > 65535) return hipErrorNotSupported;
    const dim3 grid((unsigned)gx, (unsigned)(gy0 + gy1), (unsigned)B);
    const uintptr_t ptrs = (uintptr_t)src0 | (uintptr_t)dst0 | (uintptr_t)src1 | (uintptr_t)dst1;
    if (HW % 4 == 0 && C0 % 4 == 0 && C1 % 4 == 0 && ptrs % (4 * (uintptr_t)esize) == 0 && (esize == 2 || esize == 4) &&
        ((uintptr_t)zero0 | (uintptr_t)zero1) % 16 == 0) {
        if (esize == 2)
            hipLaunchKernelGGL(layout::nchw_to_nhwc_vec_kernel<unsigned short>, grid, dim3(256), 0, st,
                               (const unsigned short *)src0, (unsigned short *)dst0, C0, gy0,
                               (const unsigned short *)src1, (unsigned short *)dst1, C1, HW, zero0, zero1);
        else
            hipLaunchKernelGGL(layout::nchw_to_nhwc_vec_kernel<unsigned>, grid, dim3(256), 0, st, (const unsigned *)src0,
                               (unsigned *)dst0, C0, gy0, (const unsigned *)src1, (unsigned *)dst1, C1, HW, zero0, zero1);
        if (zeroed) *zeroed = true;
        return hipGetLastError();
    }
    if (esize == 2)
        hipLaunchKernelGGL(layout::nchw_to_nhwc_kernel<unsigned short>, grid, dim3(256), 0, st,
                           (const unsigned short *)src0, (unsigned short *)dst0, C0, gy0,
                           (const unsigned short *)src1, (unsigned short *)dst1, C1, HW);
    else if (esize == 4)
        hipLaunchKernelGGL(layout::nchw_to_nhwc_kernel<unsigned>, grid, dim3(256), 0, st, (const unsigned *)src0,
                           (unsigned *)dst0, C0, gy0, (const unsigned *)src1, (unsigned *)dst1, C1, HW);
    else
        return hipErrorNotSupported;
    return hipGetLastError();
}

hipError_t nhwc_f32_to_nchw_launch(const float *src, void *dst, int C, int B, long HW, int dtype, hipStream_t st) {
    if (B <= 0 || C <= 0 || HW <= 0) return hipSuccess;
    const long gx = (HW + 63) / 64;
    const int gy = (C + 63) / 64;
    if (gx > 0x7fffffffL || gy > 65535 || B > 65535) return hipErrorNotSupported;
    const dim3 grid((unsigned)gx, (unsigned)gy, (unsigned)B);
    const int esize = dtype == 0 ? 4 : 2;
    if (HW % 4 == 0 && C % 4 == 0 && (uintptr_t)src % 16 == 0 && (uintptr_t)dst % (4 * (uintptr_t)esize) == 0 &&
        (dtype == 0 || dtype == 2 || dtype == 3)) {
        if (dtype == 0) hipLaunchKernelGGL(layout::nhwc_f32_to_nchw_vec_kernel<float>, grid, dim3(256), 0, st, src, (float *)dst, C, HW);
        else if (dtype == 2) hipLaunchKernelGGL(layout::nhwc_f32_to_nchw_vec_kernel<f16_t>, grid, dim3(256), 0, st, src, (f16_t *)dst, C, HW);
        else hipLaunchKernelGGL(layout::nhwc_f32_to_nchw_vec_kernel<bf16_t>, grid, dim3(256), 0, st, src, (bf16_t *)dst, C, HW);
        return hipGetLastError();
    }
    if (dtype == 0) hipLaunchKernelGGL(layout::nhwc_f32_to_nchw_kernel<float>, grid, dim3(256), 0, st, src, (float *)dst, C, HW);
    else if (dtype == 2) hipLaunchKernelGGL(layout::nhwc_f32_to_nchw_kernel<f16_t>, grid, dim3(256), 0, st, src, (f16_t *)dst, C, HW);
    else if (dtype == 3) hipLaunchKernelGGL(layout::nhwc_f32_to_nchw_kernel<bf16_t>, grid, dim3(256), 0, st, src, (bf16_t *)dst, C, HW);
    else return hipErrorNotSupported;
    return hipGetLastError();
}

}  // namespace sapa
