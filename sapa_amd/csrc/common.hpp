// Shared device helpers for the SAPA HIP kernels (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace sapa {

typedef _Float16 f16_t;
typedef __bf16 bf16_t;

// Arithmetic type for a storage type: 16-bit tensors compute in fp32.
template <typename T> struct Acc { typedef float type; };
template <> struct Acc<double> { typedef double type; };

__device__ __forceinline__ float fma_(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
__device__ __forceinline__ double fma_(double a, double b, double c) { return __builtin_fma(a, b, c); }
__device__ __forceinline__ float floor_(float a) { return __builtin_floorf(a); }
__device__ __forceinline__ double floor_(double a) { return __builtin_floor(a); }

template <typename T>
__device__ __forceinline__ typename Acc<T>::type ld(const T *p) {
    return (typename Acc<T>::type)(*p);
}

// exp(x) for x <= 0 in fp32 to ~1 ulp: hardware exp2 on the high part of
// x*log2(e), first-order correction for the part the product rounds away.
__device__ __forceinline__ float exp_(float x) {
    const float l2e_hi = 1.44269502162933349609375f;    // fl(log2 e)
    const float l2e_lo = 1.925963033500011e-8f;         // log2 e - l2e_hi
    const float t = x * l2e_hi;
    float e = __builtin_fmaf(x, l2e_hi, -t);
    e = __builtin_fmaf(x, l2e_lo, e);
    // x = -inf: t = -inf and the correction term is inf - inf = NaN; the maximum
    // returns its other operand for a NaN, so exp(-inf) comes out as r = 0 as in
    // torch.softmax, and a finite x (|e| < 1e-6) is untouched
    e = __builtin_fmaxf(e, -1.0f);
    const float r = __builtin_amdgcn_exp2f(t);
    return __builtin_fmaf(r, e * 0.693147182464599609375f, r);
}
__device__ __forceinline__ double exp_(double x) { return exp(x); }

__device__ __forceinline__ float max_(float a, float b) { return __builtin_fmaxf(a, b); }
__device__ __forceinline__ double max_(double a, double b) { return __builtin_fmax(a, b); }

// In-register softmax of v[0..N): max-subtracted, sum in index order,
// one correctly rounded reciprocal, then a multiply per element.
template <typename A, int N>
__device__ __forceinline__ void softmax_inplace(A (&v)[N]) {
    A m = v[0];
#pragma unroll
    for (int i = 1; i < N; ++i) m = max_(m, v[i]);
    A sum = 0;
#pragma unroll
    for (int i = 0; i < N; ++i) {
        v[i] = exp_(v[i] - m);
        sum += v[i];
    }
    const A inv = (A)1 / sum;
#pragma unroll
    for (int i = 0; i < N; ++i) v[i] *= inv;
}

// max / sum of a value over the aligned group of N = 8, 16 or 32 lanes a lane is in.
// The maximum is written as one DPP instruction per step: from the builtin the
// compiler makes three (a move and two canonicalising maxima).  The s_nop covers
// the two wait states a DPP read needs after the VALU write of its source.
#define SAPA_MAX_DPP(x, ctrl) \
    asm volatile("s_nop 1\n\tv_max_f32_dpp %0, %1, %1 " ctrl " row_mask:0xf bank_mask:0xf bound_ctrl:1" : "=v"(x) : "v"(x))
template <bool MAX, int N>
__device__ __forceinline__ float reduce_lanes(float v) {
    union { float f; int i; } x, y;
    x.f = v;
    if (MAX) {
        SAPA_MAX_DPP(x.f, "quad_perm:[1,0,3,2]");      // lane ^ 1
        SAPA_MAX_DPP(x.f, "quad_perm:[2,3,0,1]");      // lane ^ 2
        SAPA_MAX_DPP(x.f, "row_half_mirror");          // the other quad of 8
        if (N >= 16) SAPA_MAX_DPP(x.f, "row_mirror");  // the other 8 of the row
        if (N == 32) {
            y.i = __builtin_amdgcn_ds_swizzle(x.i, 0x401F);    // lane ^ 16
            asm volatile("v_max_f32 %0, %1, %2" : "=v"(x.f) : "v"(x.f), "v"(y.f));
        }
        return x.f;
    }
    auto step = [&](int other) __attribute__((always_inline)) {
        y.i = other;
        x.f = x.f + y.f;
    };
    step(__builtin_amdgcn_mov_dpp(x.i, 0xB1, 0xf, 0xf, true));     // lane ^ 1 (quad_perm [1,0,3,2])
    step(__builtin_amdgcn_mov_dpp(x.i, 0x4E, 0xf, 0xf, true));     // lane ^ 2 (quad_perm [2,3,0,1])
    step(__builtin_amdgcn_mov_dpp(x.i, 0x141, 0xf, 0xf, true));    // the other quad of 8 (row_half_mirror)
    if (N >= 16) step(__builtin_amdgcn_mov_dpp(x.i, 0x140, 0xf, 0xf, true));   // the other 8 of the row (row_mirror)
    if (N == 32) step(__builtin_amdgcn_ds_swizzle(x.i, 0x401F));   // lane ^ 16
    return x.f;
}

// ---- vector accesses to the high-res tensors (read or written exactly once: streaming)
template <typename T, int N>
struct alignas(sizeof(T) * N) Vec {
    T v[N];
};

// Unsigned integer of NB bytes, as the carrier of a streaming access.
template <int NB> struct Bits;
template <> struct Bits<2> { typedef unsigned short type; };
template <> struct Bits<4> { typedef unsigned type; };
template <> struct Bits<8> { typedef unsigned type __attribute__((ext_vector_type(2))); };
template <> struct Bits<16> { typedef unsigned type __attribute__((ext_vector_type(4))); };

// The high-res tensors are touched exactly once (q read, output written), so
// both go around the caches as non-temporal accesses: that leaves L2 to the
// low-res windows, which neighbouring tiles re-read, and lets partial-line
// output writes drain without allocating.
#ifndef SAPA_STREAM_LOADS
#define SAPA_STREAM_LOADS 1
#endif
template <typename T, int N>
__device__ __forceinline__ Vec<T, N> load_stream(const T *p) {
    typedef typename Bits<sizeof(T) * N>::type B;
    union { B b; Vec<T, N> v; } u;
#if SAPA_STREAM_LOADS
    u.b = __builtin_nontemporal_load((const B *)p);
#else
    u.b = *(const B *)p;
#endif
    return u.v;
}
template <typename T, int N>
__device__ __forceinline__ void store_stream(T *p, const Vec<T, N> &v) {
    typedef typename Bits<sizeof(T) * N>::type B;
    union { B b; Vec<T, N> v; } u;
    u.v = v;
    __builtin_nontemporal_store(u.b, (B *)p);
}

// The same streaming store through a buffer descriptor: byte offset `off`
// from the descriptor's base, dropped by the hardware when off + size exceeds
// the descriptor's extent.
template <typename T, int N>
__device__ __forceinline__ void store_buffer(__amdgpu_buffer_rsrc_t r, unsigned off, const Vec<T, N> &v) {
    typedef typename Bits<sizeof(T) * N>::type B;
    union { B b; Vec<T, N> v; } u;
    u.v = v;
    constexpr int NT_HINT = 2;      // non-temporal
    if constexpr (sizeof(B) == 2) __builtin_amdgcn_raw_buffer_store_b16(u.b, r, off, 0, NT_HINT);
    else if constexpr (sizeof(B) == 4) __builtin_amdgcn_raw_buffer_store_b32(u.b, r, off, 0, NT_HINT);
    else if constexpr (sizeof(B) == 8) __builtin_amdgcn_raw_buffer_store_b64(u.b, r, off, 0, NT_HINT);
    else __builtin_amdgcn_raw_buffer_store_b128(u.b, r, off, 0, NT_HINT);
}

// ---- butterfly step over lane distance 4 or 8 inside rows of 16 lanes (channels-last kernels)
// For a pair of per-lane values (a, b): the lanes whose bit D is clear get a + (a of lane ^ D),
// the others b + (b of lane ^ D) -- each lane keeps one of the two sums and adds what its
// partner held of it.  Two DPP additions and no select: the lanes with the bit clear are
// whole banks of 4 lanes (banks 0, 2 for distance 4; 0, 1 for distance 8), which the
// instruction's bank mask can pick, and their partners are a row rotation away (by 12 / 4
// lanes for distance 4, by 8 for distance 8).  Lanes outside the mask keep what the other
// instruction wrote.  (s_nop 1: the two wait states a DPP read needs after the vector
// instruction that wrote its source.)
#ifndef SAPA_NHWC_DPP_HALVE
#define SAPA_NHWC_DPP_HALVE 1
#endif
// (the same exchange as an all-to-partner maximum / sum of one value: every lane gets
// max / sum of its own v and that of lane ^ D)
template <int D>
__device__ __forceinline__ float xor_max_dpp(float v) {
    static_assert(D == 4 || D == 8, "lane distance");
    float r;
#if defined(__HIP_DEVICE_COMPILE__)
    if constexpr (D == 4)
        asm volatile("s_nop 1\n\t"
                     "v_max_f32_dpp %0, %1, %1 row_ror:12 row_mask:0xf bank_mask:0x5\n\t"
                     "v_max_f32_dpp %0, %1, %1 row_ror:4 row_mask:0xf bank_mask:0xa"
                     : "=&v"(r) : "v"(v));
    else
        asm volatile("s_nop 1\n\t"
                     "v_max_f32_dpp %0, %1, %1 row_ror:8 row_mask:0xf bank_mask:0xf"
                     : "=&v"(r) : "v"(v));
#else
    r = v;
#endif
    return r;
}
template <int D>
__device__ __forceinline__ float pair_sum_dpp(float a, float b) {
    static_assert(D == 4 || D == 8, "lane distance");
    float r;
#if defined(__HIP_DEVICE_COMPILE__)
    if constexpr (D == 4)
        asm volatile("s_nop 1\n\t"
                     "v_add_f32_dpp %0, %1, %1 row_ror:12 row_mask:0xf bank_mask:0x5\n\t"
                     "v_add_f32_dpp %0, %2, %2 row_ror:4 row_mask:0xf bank_mask:0xa"
                     : "=&v"(r) : "v"(a), "v"(b));
    else
        asm volatile("s_nop 1\n\t"
                     "v_add_f32_dpp %0, %1, %1 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
                     "v_add_f32_dpp %0, %2, %2 row_ror:8 row_mask:0xf bank_mask:0xc"
                     : "=&v"(r) : "v"(a), "v"(b));
#else
    r = a + b;
#endif
    return r;
}

}  // namespace sapa
