// Gradient of the SAPA-D operators with respect to the sampled low-res tensor
// (grad_key of deform_qk, grad_value of deform_av) as a matrix product:
//
//   grad_low[b, g*cg + c, cell] += sum over (pixel, point, corner j that lands on
//                                  cell) of w_j * sc[b, g, p, pixel] * hi[b, g*cg + c, pixel]
//
// (hi = query and sc = grad of the logits for deform_qk; hi = grad of the output
// and sc = attention weights for deform_av; the reference issues one global
// atomicAdd per term, deformsapa/deformsapa/src/cuda/deform_qk_cuda_kernel.cu:107-122).
// With the corner weights of a pixel written as a row over the window cells
// of its region -- Wm[pixel][cell] = sum of sc * w_j over the samples that land
// there, the same matrix as in the forward kernels of sapa_d_nhwc.hip -- this is
//
//   grad_low[cell][c] += sum_pixels Wm[pixel][cell] * hi[pixel][c]        (Wm^T . hi)
//
// A workgroup owns a region of RG x RG hi-res pixels of one (image, group,
// 64-channel chunk) and walks over it 16 pixels (a step) at a time: the rows of
// Wm for those pixels are built in LDS (integer adds of per-row-scaled values:
// exact in any order, and several times the rate of LDS float atomics), their hi
// values are staged next to them, and v_mfma_f32_16x16x4f32 accumulates
// [cells of the region's window] x [64 channels] in registers over all 256
// pixels.  Half of the workgroup's 8 waves build the operands of step s while the
// other half multiplies those of step s - 1 (two sets of LDS buffers, one barrier
// per step), so that the vector and the matrix pipe work at the same time.  One
// global float atomic per window cell and channel at the end adds the region's
// sums to grad_low (the caller zero-fills it), as the LDS-window kernel of
// sapa_d_lowgrad.hip does -- which needs four 64-bit LDS atomics per sample AND
// channel where this kernel needs four 32-bit ones per sample.
//
// Samples that leave the region's window (offsets beyond +-4 cells), and all
// samples of a pixel whose scalars or hi values are not finite (an inf / NaN
// must reach exactly the cells it reaches in the reference, which 0 * inf in a
// dense product would not respect), add their terms straight to grad_low.
#include <utility>

#include "deform_tap.hpp"
#include "kernels.hpp"

namespace sapa {

namespace dscat {

typedef unsigned u32;
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int RCH = 4;          // window reach around the region's parents, in low-res cells

// Tensor elements through a buffer descriptor, widened to float: an offset with
// bit 31 set lies beyond every descriptor and returns 0 without touching memory,
// so a load needs no branch around it (and the compiler can count the loads in
// flight: with loads in branches it waits for all of them at every use).
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
constexpr unsigned OOB = 0x80000000u;
template <typename T> struct Ld;
template <> struct Ld<float> {
    static __device__ __forceinline__ float one(__amdgpu_buffer_rsrc_t r, unsigned off) {
        return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, off, 0, 0));
    }
    static __device__ __forceinline__ void four(__amdgpu_buffer_rsrc_t r, unsigned off, float (&v)[4]) {
        union { u32x4 u; float f[4]; } x;
        x.u = __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0);
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = x.f[e];
    }
};
template <typename H> struct Ld16 {
    static __device__ __forceinline__ float one(__amdgpu_buffer_rsrc_t r, unsigned off) {
        return (float)__builtin_bit_cast(H, (unsigned short)__builtin_amdgcn_raw_buffer_load_b16(r, off, 0, 0));
    }
    static __device__ __forceinline__ void four(__amdgpu_buffer_rsrc_t r, unsigned off, float (&v)[4]) {
        union { u32x2 u; H h[4]; } x;
        x.u = __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, 0);
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = (float)x.h[e];
    }
};
template <> struct Ld<f16_t> : Ld16<f16_t> {};
template <> struct Ld<bf16_t> : Ld16<bf16_t> {};
constexpr int NT = 512;         // 4 waves that accumulate the products + 4 waves that build their operands
constexpr int NTP = 256;        // threads of either kind
constexpr int CHK = 64;         // channels per workgroup
constexpr int SPX = 16;         // pixels per step
constexpr int GS = CHK + 16;    // floats per pixel of the staged hi tile: 16 mod 64, so that the
                                // 4 pixels a matrix operand read touches fall on disjoint banks

// CLO: grad_low is a channels-last fp32 buffer [B, H, W, Cx] (a cell's channels in
// one piece: the final atomics of a wave then fall on two cache lines instead of
// one per window row and channel); else the contiguous [B, Cx, H, W] tensor.
template <typename T, typename TS, int S, int RG, bool CLO>
__global__ void __launch_bounds__(NT) __attribute__((amdgpu_waves_per_eu(4, 4)))
deform_scatter_mat_kernel(const T *__restrict__ hi, const TS *__restrict__ sc,
                          const T *__restrict__ offset, float *__restrict__ grad_low, int Cx, int H,
                          int W, int P, int G, int regions_x, int regions_y, int nchunks, int nblocks,
                          int per_xcd) {
    constexpr int RP = RG / S;                               // parents of a region per axis
    constexpr int WWR = RP + 2 * RCH + 1, NPOS = WWR * WWR;  // window cells
    constexpr int NCB = (NPOS + 15) / 16, KPC = NCB * 16;    // blocks of 16 cells
    constexpr int WSR = KPC;        // dwords per row of Wm: 48 mod 64 (304, 176), the 4 rows of an operand read on disjoint banks
    constexpr int CBI = (NCB + 3) / 4;                       // cell blocks per wave
    constexpr int NSTEP = RG * RG / SPX;
    static_assert(RG % S == 0 && (RG * RG) % SPX == 0 && SPX % RG == 0 || RG % SPX == 0, "whole steps");
    static_assert(WSR % 64 == 48, "bank layout of the weight rows");
    static_assert(NSTEP % 2 == 0, "the steps take the two buffers in turn");

    constexpr int TS_ = 65;         // floats per channel row of the epilogue's transposition buffer
    static_assert(2 * SPX * WSR >= CHK * TS_, "the transposition buffer fits the weight rows' buffers");
    // two sets of buffers: the producer waves fill one for step s while the consumer
    // waves multiply the other (step s - 1)
    __shared__ __attribute__((aligned(16))) int Wl2[2 * SPX * WSR];     // Wm rows of a step, scaled integers
    __shared__ __attribute__((aligned(16))) float Gl2[2 * SPX * GS];    // hi of a step's pixels [pixel][channel]
    __shared__ float invl2[2 * SPX];                                    // 1 / scale of each row

    const int logical = (int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8);
    if (logical >= nblocks) return;
    const int rx = logical % regions_x;
    const int ry = (logical / regions_x) % regions_y;
    int rest = logical / (regions_x * regions_y);
    const int chunk = rest % nchunks;
    rest /= nchunks;
    const int g = rest % G, n = rest / G;

    const bool producer = threadIdx.x >= NTP;
    const int tid = threadIdx.x & (NTP - 1), lane = tid & 63, wave = tid >> 6;   // within the 4 waves of a kind
    const int mi = lane & 15, mk = lane >> 4;
    const int hH = H * S, hW = W * S, cg = Cx / G;
    const long lpix = (long)H * W, hpl = (long)hH * hW;
    const int y0 = ry * RG, x0 = rx * RG;                    // region origin, hi-res
    const int wy0 = y0 / S - RCH, wx0 = x0 / S - RCH;        // window origin, low-res cell
    const int c0 = chunk * CHK;                              // first channel of the chunk within the group
    const int cvalid = cg - c0 < CHK ? cg - c0 : CHK;
    const long ch0 = (long)n * Cx + (long)g * cg + c0;       // its plane index
    const long k0 = ((long)n * G + g) * P;                   // the group's first point

    // pixel t of step `step`: row / column within the region
    auto step_pixel = [&](int step, int t, int &qh, int &qw) __attribute__((always_inline)) {
        const int lin = step * SPX + t;
        qh = y0 + lin / RG;
        qw = x0 + lin % RG;
    };
    // The step's pixels belong to one or two rows of parents, and a sample within
    // RCH cells of its parent lands on the window rows b0 .. b1 (the band), i.e. on
    // the cell blocks cb0 .. cb1: only those take part in the step's product.  A
    // sample that lands elsewhere in the window goes the direct way.
    auto band = [&](int step, int &b0, int &b1, int &cb0, int &cb1) __attribute__((always_inline)) {
        b0 = (step * SPX / RG) / S;
        b1 = ((step * SPX + SPX - 1) / RG) / S + 2 * RCH + 1;
        cb0 = b0 * WWR / 16;
        cb1 = ((b1 + 1) * WWR - 1) / 16;
    };

    // ===== producer waves: wave w owns pixels 4 w .. 4 w + 3 of every step -- their hi
    // values (lane = channel), their rows of Wm (zeroed, then filled by the wave's
    // own lanes: LDS operations of one wave execute in order, so no barrier sits
    // between the two) and their scales
    const bool vec4 = hW % 4 == 0 && (uintptr_t)hi % (4 * sizeof(T)) == 0;
    // the chunk's planes of hi, the group's scalars and offsets (byte offsets below 2^31: the launcher checks)
    const __amdgpu_buffer_rsrc_t hrsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(hi + ch0 * hpl), 0, (int)(cvalid * hpl * (long)sizeof(T)), 0x00020000);
    const __amdgpu_buffer_rsrc_t srsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(sc + k0 * hpl), 0, (int)(P * hpl * (long)sizeof(TS)), 0x00020000);
    const __amdgpu_buffer_rsrc_t orsrc = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(offset + (k0 << 1) * hpl), 0, (int)(2 * P * hpl * (long)sizeof(T)), 0x00020000);
    // what a step needs from global memory, fetched two steps ahead (two sets in turn)
    struct Pre { float greg[4], scr[2], oxr[2], oyr[2]; };
    auto load_hi = [&](int step, Pre &pre) __attribute__((always_inline)) {
        int qh, qw;
        step_pixel(step, 4 * wave, qh, qw);
        const bool row_ok = lane < cvalid && qh < hH;
        const unsigned off = (unsigned)(((long)lane * hpl + (long)qh * hW + qw) * (long)sizeof(T));
        if (vec4) {     // (uniform) whole aligned vectors: inside the image or outside as a whole
            Ld<T>::four(hrsrc, row_ok && qw < hW ? off : OOB, pre.greg);
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                pre.greg[e] = Ld<T>::one(hrsrc, row_ok && qw + e < hW ? off + e * (unsigned)sizeof(T) : OOB);
        }
    };
    // per-sample view: P <= 16 -> 16 lanes per pixel, one pass over the wave's 4
    // pixels; else 32 lanes per pixel, two passes
    const bool narrow = P <= 16;
    const int pt = narrow ? (lane & 15) : (lane & 31);
    const int npass = narrow ? 1 : 2;
    // this lane's pixel of the step in pass ps
    auto sample_pixel = [&](int ps) __attribute__((always_inline)) {
        return 4 * wave + (narrow ? lane >> 4 : 2 * ps + (lane >> 5));
    };
    auto load_samples = [&](int step, Pre &pre) __attribute__((always_inline)) {
#pragma unroll
        for (int ps = 0; ps < 2; ++ps) {
            int qh, qw;
            step_pixel(step, sample_pixel(ps), qh, qw);
            const bool ok = ps < npass && pt < P && qh < hH && qw < hW;
            const long pp = (long)pt * hpl + (long)qh * hW + qw;        // the point's plane of sc
            const long po = pp + (long)pt * hpl;                        // its dx plane of the offsets
            pre.scr[ps] = Ld<TS>::one(srsrc, ok ? (unsigned)(pp * (long)sizeof(TS)) : OOB);
            pre.oxr[ps] = Ld<T>::one(orsrc, ok ? (unsigned)(po * (long)sizeof(T)) : OOB);
            pre.oyr[ps] = Ld<T>::one(orsrc, ok ? (unsigned)((po + hpl) * (long)sizeof(T)) : OOB);
        }
    };
    auto produce = [&](int step, Pre &pre) __attribute__((always_inline)) {
        const float (&scr)[2] = pre.scr, (&oxr)[2] = pre.oxr, (&oyr)[2] = pre.oyr;
        int *const Wl = Wl2 + (step & 1) * SPX * WSR;
        float *const Gl = Gl2 + (step & 1) * SPX * GS;
        float *const invl = invl2 + (step & 1) * SPX;
        int b0, b1, cb0, cb1;
        band(step, b0, b1, cb0, cb1);
        // ---- empty weight rows; the hi values, a value that is not finite replaced
        // by 0 and its pixel marked (bit e of bad: pixel 4 w + e)
        {
            int __attribute__((ext_vector_type(4))) *rows = (int __attribute__((ext_vector_type(4))) *)(Wl + 4 * wave * WSR);
            for (int i = lane; i < 4 * WSR / 4; i += 64) rows[i] = {0, 0, 0, 0};
        }
        u32 bad = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const bool fin = __builtin_fabsf(pre.greg[e]) < __builtin_huge_valf();
            bad |= __builtin_amdgcn_ballot_w64(!fin) != 0 ? 1u << e : 0u;
            Gl[(4 * wave + e) * GS + lane] = fin ? pre.greg[e] : 0.f;
        }
        // ---- per (pixel, point): the corners' shares of sc into the pixel's row
        auto sample = [&](auto nl, int ps) __attribute__((always_inline)) {
            constexpr int NL = decltype(nl)::value;
            const int t = sample_pixel(ps);
            const bool isbad = bad >> (t & 3) & 1;
            int qh, qw;
            step_pixel(step, t, qh, qw);
            const bool live = qh < hH && qw < hW && pt < P;
            const float scv = scr[ps];
            // the row's scale: |sum of any subset of its entries| <= L1 < 2^ex
            const float l1 = reduce_lanes<false, NL>(live ? __builtin_fabsf(scv) : 0.f);
            const bool finite = l1 < __builtin_huge_valf();
            int ex = 0;
            (void)__builtin_frexpf(l1, &ex);
            const float scale = __builtin_ldexpf(1.f, 30 - ex);
            if (pt == 0) invl[t] = (finite && l1 > 0.f) ? __builtin_ldexpf(1.f, ex - 30) : 0.f;
            if (!live || (scv == 0.f && !isbad)) return;
            const float kw = (float)(qw / S) + oxr[ps], kh = (float)(qh / S) + oyr[ps];
            const WinTap<float> wt = win_tap<float>(kh, kw, H, W, wy0, wx0, WWR, WWR);
            if (!wt.guard) return;
            if (wt.inwin && wt.hl >= b0 && wt.hl < b1 && finite && !isbad) {
                int *wp = Wl + t * WSR + wt.hl * WWR + wt.wl;
                const float sv = scv * scale;
                __hip_atomic_fetch_add(wp, (int)__builtin_rintf(sv * wt.w1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                __hip_atomic_fetch_add(wp + 1, (int)__builtin_rintf(sv * wt.w2), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                __hip_atomic_fetch_add(wp + WWR, (int)__builtin_rintf(sv * wt.w3), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                __hip_atomic_fetch_add(wp + WWR + 1, (int)__builtin_rintf(sv * wt.w4), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            } else {
                // the reference's own way: one float atomic per term (rare).  (The
                // position is made opaque: its taps are set up in this branch only.)
                float fkh = kh, fkw = kw;
                asm volatile("" : "+v"(fkh), "+v"(fkw));
                Tap<float> tp = {};
                tap_setup(fkh, fkw, H, W, tp);
                const T *hp = hi + ch0 * hpl + (long)qh * hW + qw;
                // element (cell i, channel c of the chunk) of grad_low
                const long cstep = CLO ? Cx : 1, chstep = CLO ? 1 : lpix;
                float *const g0 = grad_low + (CLO ? (long)n * lpix * Cx + (long)g * cg + c0 : ch0 * lpix);
                for (int c = 0; c < cvalid; ++c) {
                    float *gp = g0 + c * chstep;
                    const float tv = (float)hp[c * hpl] * scv;
                    if (tp.m1) unsafeAtomicAdd(gp + tp.i1 * cstep, tp.w1 * tv);
                    if (tp.m2) unsafeAtomicAdd(gp + tp.i2 * cstep, tp.w2 * tv);
                    if (tp.m3) unsafeAtomicAdd(gp + tp.i3 * cstep, tp.w3 * tv);
                    if (tp.m4) unsafeAtomicAdd(gp + tp.i4 * cstep, tp.w4 * tv);
                }
            }
        };
        if (narrow) {
            sample(std::integral_constant<int, 16>{}, 0);
        } else {
            sample(std::integral_constant<int, 32>{}, 0);
            sample(std::integral_constant<int, 32>{}, 1);
        }
        // the loads of the step after the next go out (into the set this step has used up)
        if (step + 2 < NSTEP) {
            load_hi(step + 2, pre);
            load_samples(step + 2, pre);
        }
    };

    // ---- the region's sums into grad_low.  D[cbi][nb][r] = cell 16 cb + 4 mk + r,
    // channel 16 nb + mi: as it stands a wave's 64 lanes would hit 64 channel planes,
    // one atomic per cache line.  The 64 cells x 64 channels of a round (the 4
    // consumer waves' blocks side by side) go through LDS, after which all 8 waves
    // issue the atomics with their lanes along what is contiguous in grad_low:
    // the cells of one channel (contiguous layout: runs of up to WWR floats), or the
    // channels of one cell (channels-last buffer: 256 bytes).
    float *const Tl = (float *)Wl2;
    constexpr int TSC = 68;         // floats per cell row of the channels-last form: 4 x 68 = 16 mod 64
    static_assert(2 * SPX * WSR >= 64 * TSC, "the transposition buffer fits the weight rows' buffers");
    auto stash = [&](int cbi, const f32x4 (&Dc)[CHK / 16]) __attribute__((always_inline)) {
#pragma unroll
        for (int nb = 0; nb < CHK / 16; ++nb)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                if (CLO) Tl[(16 * wave + 4 * mk + r) * TSC + 16 * nb + mi] = Dc[nb][r];
                else Tl[(16 * nb + mi) * TS_ + 16 * wave + 4 * mk + r] = Dc[nb][r];
            }
    };
    auto flush = [&](int cbi) __attribute__((always_inline)) {
        const int w8 = (int)(threadIdx.x >> 6);
        if (CLO) {
            // this wave: cells 8 w8 .. + 7 of the round; lane <-> channel
            float *const g0 = grad_low + (long)n * lpix * Cx + (long)g * cg + c0 + lane;
#pragma unroll 4
            for (int c = 0; c < 8; ++c) {
                const int cell = 64 * cbi + 8 * w8 + c;
                const int gy = wy0 + cell / WWR, gx = wx0 + cell % WWR;
                const bool ok = cell < NPOS && gy >= 0 && gy < H && gx >= 0 && gx < W;
                const float v = Tl[(8 * w8 + c) * TSC + lane];
                if (ok && lane < cvalid && v != 0.f) unsafeAtomicAdd(g0 + ((long)gy * W + gx) * Cx, v);
            }
        } else {
            // lane <-> cell 64 cbi + lane; this wave: channels 8 w8 .. + 7
            const int cell = 64 * cbi + lane;
            const int gy = wy0 + cell / WWR, gx = wx0 + cell % WWR;
            const bool ok = cell < NPOS && gy >= 0 && gy < H && gx >= 0 && gx < W;
            float *gp = grad_low + (ch0 + 8 * w8) * lpix + (long)gy * W + gx;
#pragma unroll 4
            for (int c = 0; c < 8; ++c) {
                const float v = Tl[(8 * w8 + c) * TS_ + lane];
                if (ok && 8 * w8 + c < cvalid && v != 0.f) unsafeAtomicAdd(gp + c * lpix, v);
            }
        }
    };

    // The two kinds of waves run their own code from here on and meet at the
    // barriers (the same number on both paths): in iteration i step i is produced
    // while step i - 1 is consumed.  (One loop with both roles in it would keep the
    // consumers' accumulators alive in the producers' registers.)
    if (producer) {
        Pre pre0, pre1;
        load_hi(0, pre0);
        load_samples(0, pre0);
        load_hi(1, pre1);
        load_samples(1, pre1);
        for (int i = 0; i <= NSTEP; i += 2) {
            if (i < NSTEP) produce(i, pre0);
            __syncthreads();
            if (i + 1 < NSTEP) produce(i + 1, pre1);
            __syncthreads();
        }
        for (int cbi = 0; cbi < CBI; ++cbi) {
            __syncthreads();
            flush(cbi);
            __syncthreads();
        }
    } else {
        // ===== consumer waves: D[cell][channel] += Wm^T . hi over a step's 16 pixels
        f32x4 D[CBI][CHK / 16];
#pragma unroll
        for (int cbi = 0; cbi < CBI; ++cbi)
#pragma unroll
            for (int nb = 0; nb < CHK / 16; ++nb) D[cbi][nb] = f32x4{0.f, 0.f, 0.f, 0.f};
        auto consume = [&](int step) __attribute__((always_inline)) {
            const int *const Wl = Wl2 + (step & 1) * SPX * WSR;
            const float *const Gl = Gl2 + (step & 1) * SPX * GS;
            const float *const invl = invl2 + (step & 1) * SPX;
            int b0, b1, cb0, cb1;
            band(step, b0, b1, cb0, cb1);
#pragma unroll
            for (int ks = 0; ks < SPX / 4; ++ks) {
                const float inv = invl[4 * ks + mk];
                float b[CHK / 16];
#pragma unroll
                for (int nb = 0; nb < CHK / 16; ++nb) b[nb] = Gl[(4 * ks + mk) * GS + 16 * nb + mi];
#pragma unroll
                for (int cbi = 0; cbi < CBI; ++cbi) {
                    const int cb = wave + 4 * cbi;
                    if (cb >= cb0 && cb <= cb1) {
                        const float a = (float)Wl[(4 * ks + mk) * WSR + 16 * cb + mi] * inv;
#pragma unroll
                        for (int nb = 0; nb < CHK / 16; ++nb)
                            if (16 * nb < cvalid)       // (uniform) a short chunk skips its empty channel blocks
                                D[cbi][nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b[nb], D[cbi][nb], 0, 0, 0);
                    }
                }
            }
        };
        for (int i = 0; i <= NSTEP; i += 2) {
            if (i > 0) consume(i - 1);
            __syncthreads();
            if (i < NSTEP) consume(i);
            __syncthreads();
        }
#pragma unroll
        for (int cbi = 0; cbi < CBI; ++cbi) {
            stash(cbi, D[cbi]);
            __syncthreads();
            flush(cbi);
            __syncthreads();
        }
    }
}

template <typename T, typename TS, int S, int RG, bool CLO>
static hipError_t launch_geom(const void *hi, const void *sc, const void *offset, void *grad_low, int B,
                              int Cx, int H, int W, int P, int G, hipStream_t st) {
    const int regions_x = (W * S + RG - 1) / RG, regions_y = (H * S + RG - 1) / RG;
    const int nchunks = (Cx / G + CHK - 1) / CHK;
    const long nb = (long)regions_x * regions_y * nchunks * G * B;
    if (nb > (1L << 30)) return hipErrorNotSupported;
    const int per_xcd = (int)((nb + 7) / 8);
    hipLaunchKernelGGL((deform_scatter_mat_kernel<T, TS, S, RG, CLO>), dim3(per_xcd * 8), dim3(NT), 0, st,
                       (const T *)hi, (const TS *)sc, (const T *)offset, (float *)grad_low, Cx, H, W, P, G,
                       regions_x, regions_y, nchunks, (int)nb, per_xcd);
    return hipGetLastError();
}

template <typename T, typename TS>
static hipError_t launch_t(const void *hi, const void *sc, const void *offset, void *grad_low, int B, int Cx,
                           int H, int W, int P, int s, int G, hipStream_t st, bool clo) {
#define SAPA_SCAT(SV, RGV)                                                                                     \
    case SV:                                                                                                   \
        return clo ? launch_geom<T, TS, SV, RGV, true>(hi, sc, offset, grad_low, B, Cx, H, W, P, G, st)        \
                   : launch_geom<T, TS, SV, RGV, false>(hi, sc, offset, grad_low, B, Cx, H, W, P, G, st);
    switch (s) {
        SAPA_SCAT(1, 8)
        SAPA_SCAT(2, 16)
        SAPA_SCAT(4, 16)
        default: return hipErrorNotSupported;
    }
#undef SAPA_SCAT
}

}  // namespace dscat

// Whether deform_scatter_mat_launch serves the configuration (dtype as the C ABI
// numbers them; 16-bit features go with fp32 scalars).
bool deform_scatter_mat_serves(int B, int Cx, int H, int W, int P, int s, int G, int dtype) {
    if (dtype != 0 && dtype != 2 && dtype != 3) return false;
    if (s != 1 && s != 2 && s != 4) return false;
    if (P < 1 || P > 32 || G <= 0 || Cx % G != 0 || (long)H * s * W * s >= (1L << 31)) return false;
    // byte offsets within a group's planes of the scalars, the offsets and a chunk of hi stay below 2^31
    if (2L * P * H * s * W * s * 4 >= (1L << 31) || 64L * H * s * W * s * 4 >= (1L << 31)) return false;
    // The two products over the region's whole window are a fixed cost; the LDS-window
    // scatter's cost grows with points x channels.  Measured at B=8, G=4, 64 channels per
    // group, 64x64 -> 128x128 (us, this kernel / that one): P = 2 342 / 227, P = 5 349 / 452,
    // P = 9 352 / 770, P = 25 400 / 2052.
    const int cg = Cx / G;
    return (long)P * (cg < 64 ? cg : 64) >= 256;
}

// fp32 tensors, or (wide) f16 / bf16 features and offsets with fp32 per-point
// scalars; s in {1, 2, 4}, P <= 32; grad_low is fp32 and is accumulated into: the
// contiguous [B, Cx, H, W] tensor, or (channels_last_out) a [B, H, W, Cx] buffer.
// hipErrorNotSupported otherwise.
hipError_t deform_scatter_mat_launch(const void *hi, const void *sc, const void *offset, void *grad_low,
                                     int B, int Cx, int H, int W, int P, int s, int G, int dtype,
                                     hipStream_t st, bool wide, bool channels_last_out) {
    if (!deform_scatter_mat_serves(B, Cx, H, W, P, s, G, dtype)) return hipErrorNotSupported;
    const bool clo = channels_last_out;
    if (dtype == 0) return dscat::launch_t<float, float>(hi, sc, offset, grad_low, B, Cx, H, W, P, s, G, st, clo);
    if (wide && dtype == 2) return dscat::launch_t<f16_t, float>(hi, sc, offset, grad_low, B, Cx, H, W, P, s, G, st, clo);
    if (wide && dtype == 3) return dscat::launch_t<bf16_t, float>(hi, sc, offset, grad_low, B, Cx, H, W, P, s, G, st, clo);
    return hipErrorNotSupported;
}

}  // namespace sapa
