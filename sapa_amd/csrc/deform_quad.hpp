// Types shared by the matrix-form SAPA-D kernels: four consecutive tensor
// elements as one register group, widened to floats and back.
#pragma once
#include "common.hpp"

namespace sapa {

namespace dnhwc {

typedef unsigned u32;
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef u32 u32x2 __attribute__((ext_vector_type(2)));
typedef u32 u32x4 __attribute__((ext_vector_type(4)));

// 4 consecutive elements <-> 4 floats, 2 consecutive elements -> 2 floats
template <typename T> struct Quad;
template <> struct Quad<float> {
    typedef f32x4 raw;
    static __device__ __forceinline__ raw buffer_load(__amdgpu_buffer_rsrc_t r, u32 off, u32 soff = 0) {
        union { u32x4 u; f32x4 f; } x;
        x.u = __builtin_amdgcn_raw_buffer_load_b128(r, off, soff, 0);
        return x.f;
    }
    static __device__ __forceinline__ f32x4 widen(raw v) { return v; }
    static __device__ __forceinline__ raw narrow(f32x4 v) { return v; }
    static __device__ __forceinline__ f32x2 load_pair(const float *p) { return *(const f32x2 *)p; }
};
template <typename H> struct Quad16 {
    typedef u32x2 raw;
    static __device__ __forceinline__ raw buffer_load(__amdgpu_buffer_rsrc_t r, u32 off, u32 soff = 0) {
        return __builtin_amdgcn_raw_buffer_load_b64(r, off, soff, 0);
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
    static __device__ __forceinline__ f32x2 load_pair(const H *p) {
        union { u32 u; H h[2]; } x;
        x.u = *(const u32 *)p;
        f32x2 f = {(float)x.h[0], (float)x.h[1]};
        return f;
    }
};
template <> struct Quad<f16_t> : Quad16<f16_t> {};
template <> struct Quad<bf16_t> : Quad16<bf16_t> {};

}  // namespace dnhwc

}  // namespace sapa
