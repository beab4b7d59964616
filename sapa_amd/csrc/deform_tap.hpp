// Bilinear sample ("tap") helpers shared by the SAPA-D kernels.  Index math,
// the strict in-range guard and the per-corner zero padding follow
// deformsapa/deformsapa/src/cuda/deform_qk_cuda_kernel.cu:23-68,187.
#pragma once
#include "common.hpp"

namespace sapa {

// Where the kernels read a pixel's sampling offsets from.  The module that
// owns these operators produces the hi-res offset tensor [B, 2GP, sH, sW]
// from a low-res 1x1-conv output, either by pixel_shuffle of [B, 2GP*s*s, H, W]
// or by nearest interpolation of [B, 2GP, H, W] (sapa_deform.py:44-47); the
// last two layouts read that low-res tensor in place, which saves writing and
// re-reading the hi-res copy.
enum OffsetLayout { OFFSET_HIRES = 0, OFFSET_PIXEL_SHUFFLE = 1, OFFSET_NEAREST = 2 };

// Channel j (0 = x of the first point, 1 = y, 2 = x of the next point ...)
// of one pixel's offsets is base[j * stride].
template <typename T>
struct OffsetRef {
    const T *base;
    long stride;
};

// k0 = b * G * P + g * P + p: the first sample point wanted.
// pixel_shuffle: hi[b, c, qh, qw] = lo[b, c*s*s + (qh%s)*s + qw%s, qh/s, qw/s].
template <typename T>
__device__ __forceinline__ OffsetRef<T> offset_ref(const T *offset, int layout, long k0, int qh,
                                                   int qw, int s, int H, int W) {
    const long lplane = (long)H * W;
    OffsetRef<T> r;
    if (layout == OFFSET_HIRES) {
        r.stride = lplane * s * s;
        r.base = offset + (k0 << 1) * r.stride + (long)qh * (W * s) + qw;
    } else if (layout == OFFSET_PIXEL_SHUFFLE) {
        r.stride = lplane * s * s;
        r.base = offset + (k0 << 1) * r.stride + (long)((qh % s) * s + qw % s) * lplane +
                 (long)(qh / s) * W + qw / s;
    } else {
        r.stride = lplane;
        r.base = offset + (k0 << 1) * lplane + (long)(qh / s) * W + qw / s;
    }
    return r;
}

// One bilinear sample position: four weights, four plane offsets, four
// per-corner validity flags (deform_qk_cuda_kernel.cu:30-64).
template <typename A>
struct Tap {
    A w1, w2, w3, w4;
    A lh, lw, hh, hw;
    int i1, i2, i3, i4;
    bool m1, m2, m3, m4;
};

// False when the position fails the guard kh > -1 && kh < H && kw > -1 &&
// kw < W (deform_qk_cuda_kernel.cu:187): the sample then contributes nothing.
template <typename A>
__device__ __forceinline__ bool tap_setup(A kh, A kw, int H, int W, Tap<A> &t) {
    if (!(kh > (A)-1 && kh < (A)H && kw > (A)-1 && kw < (A)W)) return false;
    const int h_low = (int)floor_(kh), w_low = (int)floor_(kw);
    const int h_high = h_low + 1, w_high = w_low + 1;
    t.lh = kh - (A)h_low;
    t.lw = kw - (A)w_low;
    t.hh = (A)1 - t.lh;
    t.hw = (A)1 - t.lw;
    t.m1 = h_low >= 0 && w_low >= 0;
    t.m2 = h_low >= 0 && w_high <= W - 1;
    t.m3 = h_high <= H - 1 && w_low >= 0;
    t.m4 = h_high <= H - 1 && w_high <= W - 1;
    t.i1 = t.m1 ? h_low * W + w_low : 0;
    t.i2 = t.m2 ? h_low * W + w_high : 0;
    t.i3 = t.m3 ? h_high * W + w_low : 0;
    t.i4 = t.m4 ? h_high * W + w_high : 0;
    t.w1 = t.hh * t.hw;
    t.w2 = t.hh * t.lw;
    t.w3 = t.lh * t.hw;
    t.w4 = t.lh * t.lw;
    return true;
}

// The same sample position for a kernel that gathers from an LDS window whose
// origin is the low-res cell (wy0, wx0) and which is WH x WW cells large:
// everything is computed unconditionally (no early exit), `guard` is the
// reference's range test and `inwin` says that all four corners lie in the
// window, where out-of-image cells hold zeros.  Weights are the expressions of
// tap_setup, bit for bit.
template <typename A>
struct WinTap {
    A w1, w2, w3, w4;
    int hl, wl;          // window-relative low corner
    bool guard, inwin;
};

template <typename A>
__device__ __forceinline__ WinTap<A> win_tap(A kh, A kw, int H, int W, int wy0, int wx0, int WH,
                                             int WW) {
    WinTap<A> t;
    t.guard = kh > (A)-1 && kh < (A)H && kw > (A)-1 && kw < (A)W;
    const A fh = floor_(kh), fw = floor_(kw);
    t.hl = (int)fh - wy0;
    t.wl = (int)fw - wx0;
    t.inwin = t.guard && t.hl >= 0 && t.hl <= WH - 2 && t.wl >= 0 && t.wl <= WW - 2;
    const A lh = kh - fh, lw = kw - fw;
    const A hh = (A)1 - lh, hw = (A)1 - lw;
    t.w1 = hh * hw;
    t.w2 = hh * lw;
    t.w3 = lh * hw;
    t.w4 = lh * lw;
    return t;
}

// w1*v1 + w2*v2 + w3*v3 + w4*v4, evaluated left to right with FMAs.
template <typename T, typename A>
__device__ __forceinline__ A tap_sample(const T *plane, const Tap<A> &t) {
    const A v1 = t.m1 ? ld(plane + t.i1) : (A)0;
    const A v2 = t.m2 ? ld(plane + t.i2) : (A)0;
    const A v3 = t.m3 ? ld(plane + t.i3) : (A)0;
    const A v4 = t.m4 ? ld(plane + t.i4) : (A)0;
    A val = t.w1 * v1;
    val = fma_(t.w2, v2, val);
    val = fma_(t.w3, v3, val);
    val = fma_(t.w4, v4, val);
    return val;
}

}  // namespace sapa
