// Helpers shared by the channels-last SAPA-B kernels that keep fp32 windows in LDS
// (sapa_b_nhwc.hip, sapa_b_nhwc_mm.hip).
#pragma once
#include <type_traits>
#include <utility>

#include "kernels.hpp"

namespace sapa {

namespace nhwc {

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>): a loop whose
// index is a compile-time constant in the body (DPP controls are immediates)
template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

typedef unsigned u32;
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef u32 u32x2 __attribute__((ext_vector_type(2)));
typedef u32 u32x4 __attribute__((ext_vector_type(4)));

// 4 consecutive elements <-> 4 floats
template <typename T> struct Quad;
template <> struct Quad<float> {
    typedef f32x4 raw;
    static __device__ __forceinline__ raw buffer_load(__amdgpu_buffer_rsrc_t r, u32 off) {
        union { u32x4 u; f32x4 f; } x;
        x.u = __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0);
        return x.f;
    }
    static __device__ __forceinline__ f32x4 widen(raw v) { return v; }
    static __device__ __forceinline__ raw narrow(f32x4 v) { return v; }
};
template <typename H> struct Quad16 {
    typedef u32x2 raw;
    static __device__ __forceinline__ raw buffer_load(__amdgpu_buffer_rsrc_t r, u32 off) {
        return __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, 0);
    }
    static __device__ __forceinline__ f32x4 widen(raw v) {
        union { u32x2 u; H h[4]; } x;
        x.u = v;
        f32x4 f = {(float)x.h[0], (float)x.h[1], (float)x.h[2], (float)x.h[3]};
        return f;
    }
    static __device__ __forceinline__ raw narrow(f32x4 v) {
        union { u32x2 u; H h[4]; } x;
        x.h[0] = (H)v[0];
        x.h[1] = (H)v[1];
        x.h[2] = (H)v[2];
        x.h[3] = (H)v[3];
        return x.u;
    }
};
template <> struct Quad<f16_t> : Quad16<f16_t> {};
template <> struct Quad<bf16_t> : Quad16<bf16_t> {};

// value of lane (l ^ D) of the same row of 16 lanes
template <int D>
__device__ __forceinline__ float row_xor(float v, int lane) {
    union { float f; int i; } x, y;
    x.f = v;
    if (D == 1) y.i = __builtin_amdgcn_mov_dpp(x.i, 0xB1, 0xf, 0xf, true);        // quad_perm [1,0,3,2]
    else if (D == 2) y.i = __builtin_amdgcn_mov_dpp(x.i, 0x4E, 0xf, 0xf, true);   // quad_perm [2,3,0,1]
    else y.i = __builtin_amdgcn_ds_bpermute((lane ^ D) << 2, x.i);
    return y.f;
}
// One butterfly step over lane distance D: n values per lane -> (n + 1) / 2.
// The lane whose bit D is clear keeps the even-indexed sums, its partner the
// odd-indexed ones; each adds what the other held of them.
// Distances 4 and 8 take two DPP additions per result and no select (pair_sum_dpp) when
// FROM_VALU says that the inputs were written by ordinary vector instructions: the wait
// states inside pair_sum_dpp cover those, not a matrix instruction's result (the compiler
// cannot see into the instruction text to add the longer wait itself).
template <int D, int N, bool FROM_VALU = true>
__device__ __forceinline__ void halve(const float (&in)[N], float (&out)[(N + 1) / 2], int lane) {
    const bool hi = lane & D;
    (void)hi;
#pragma unroll
    for (int m = 0; m < (N + 1) / 2; ++m) {
        const float a = in[2 * m], b = 2 * m + 1 < N ? in[2 * m + 1] : 0.f;
        if constexpr (SAPA_NHWC_DPP_HALVE && FROM_VALU && (D == 4 || D == 8)) {
            out[m] = pair_sum_dpp<D>(a, b);
        } else {
            const float keep = hi ? b : a, send = hi ? a : b;
            out[m] = keep + row_xor<D>(send, lane);
        }
    }
}

// sapa_b_nhwc_mm.hip: the same four modes with the logits on the matrix pipe (fp32 tensors)
hipError_t launch_mm(int mode, const void *q, const void *key, const void *attn_in, const void *value,
                     const void *qbias, void *out, int B, int d, int C, int H, int W, int K, int s,
                     hipStream_t st);

}  // namespace nhwc

}  // namespace sapa
