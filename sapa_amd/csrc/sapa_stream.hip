// Streaming calibration kernel: what this GPU's memory system gives a kernel
// that does nothing but move a stated mix of bytes in and out, each workgroup
// in long contiguous runs.  It is the yardstick the operators' measured rates
// are put beside (the published HBM peak is not reachable by any kernel): a
// fused SAPA-B forward at up_factor 2 reads 9 bytes for every 16 it writes
// (q and the low-res key / value in, the C-channel high-res result out, with
// C = 4 d), a copy reads 1 for 1, a fill reads nothing.
//
// A unit = 256 threads, 16 bytes per thread and row: R rows read (one
// contiguous run of R * 4 KiB) and WR rows written (one contiguous run of
// WR * 4 KiB); what is written depends on what was read, so no access can be
// dropped.  A workgroup takes `reps` consecutive units -- runs `reps` times as
// long -- with the next unit's loads issued before the current unit's stores.
#include "kernels.hpp"

namespace sapa {

typedef unsigned u4 __attribute__((ext_vector_type(4)));

template <int R, int WR, bool NTL, bool NTS>
__global__ void __launch_bounds__(256) stream_mix_kernel(const u4 *__restrict__ src, u4 *__restrict__ dst,
                                                         long units, int reps) {
    const int t = threadIdx.x;
    const long u0 = (long)blockIdx.x * reps;
    auto load = [&](long u, u4 (&v)[R > 0 ? R : 1]) {
        if constexpr (R > 0) {
            const u4 *s = src + u * (long)(R * 256) + t;
#pragma unroll
            for (int i = 0; i < R; ++i) v[i] = NTL ? __builtin_nontemporal_load(s + i * 256) : s[i * 256];
        } else {
            v[0] = u4{(unsigned)u, (unsigned)t, 0u, 0u};
        }
    };
    u4 v[R > 0 ? R : 1], vn[R > 0 ? R : 1];
    if (u0 >= units) return;
    load(u0, v);
    u4 a = {0u, 0u, 0u, 0u};
    for (int r = 0; r < reps; ++r) {
        const long u = u0 + r;
        if (u >= units) break;
        // the next unit's loads go out before this unit's stores
        const bool more = r + 1 < reps && u + 1 < units;
        if (more) load(u + 1, vn);
        if constexpr (WR > 0) {
            u4 *d = dst + u * (long)(WR * 256) + t;
#pragma unroll
            for (int j = 0; j < WR; ++j) {
                u4 o = v[R > 0 ? j % R : 0];
                o.x += (unsigned)j;
                if (NTS) __builtin_nontemporal_store(o, d + j * 256);
                else d[j * 256] = o;
            }
        } else {
#pragma unroll
            for (int i = 0; i < R; ++i) a ^= v[i];
        }
        if (more) {
#pragma unroll
            for (int i = 0; i < (R > 0 ? R : 1); ++i) v[i] = vn[i];
        }
    }
    if constexpr (WR == 0) {
        // never true for the data the caller fills src with; keeps the loads
        if ((a.x & a.y & a.z & a.w) == 0xfffffffeu) dst[u0 * 256 + t] = a;
    }
}

// The same byte mix with readers and writers apart: of every 25 consecutive
// workgroups 9 only read and 16 only write, each one contiguous run of
// reps * 64 KiB -- nothing written depends on anything read, so this measures
// what the memory system gives the mix when neither stream waits for the other.
template <bool NTL, bool NTS>
__global__ void __launch_bounds__(256) stream_split_kernel(const u4 *__restrict__ src, u4 *__restrict__ dst,
                                                           long groups, int reps) {
    const int t = threadIdx.x;
    const long grp = blockIdx.x / 25;
    const int slot = blockIdx.x % 25;
    if (grp >= groups) return;
    if (slot < 9) {
        const u4 *s = src + (grp * 9 + slot) * (long)reps * 4096 + t;
        u4 a = {0u, 0u, 0u, 0u};
        for (int r = 0; r < reps; ++r) {
            u4 v[16];
#pragma unroll
            for (int i = 0; i < 16; ++i)
                v[i] = NTL ? __builtin_nontemporal_load(s + (r * 16 + i) * 256) : s[(r * 16 + i) * 256];
#pragma unroll
            for (int i = 0; i < 16; ++i) a ^= v[i];
        }
        if ((a.x & a.y & a.z & a.w) == 0xfffffffeu) dst[(grp * 16) * (long)reps * 4096 + t] = a;
    } else {
        u4 *d = dst + (grp * 16 + slot - 9) * (long)reps * 4096 + t;
        u4 o = {(unsigned)blockIdx.x, (unsigned)t, 0u, 0u};
        for (int r = 0; r < reps; ++r) {
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                o.x += 1u;
                if (NTS) __builtin_nontemporal_store(o, d + (r * 16 + j) * 256);
                else d[(r * 16 + j) * 256] = o;
            }
        }
    }
}

hipError_t stream_split_launch(const void *src, void *dst, long groups, int reps, int nt, hipStream_t st) {
    if (groups * 25 > (1L << 30)) return hipErrorInvalidValue;
    const dim3 grid((unsigned)(groups * 25)), block(256);
#define SAPA_NT(L, S) \
    hipLaunchKernelGGL((stream_split_kernel<L, S>), grid, block, 0, st, (const u4 *)src, (u4 *)dst, groups, reps)
    switch (nt & 3) {
        case 0: SAPA_NT(false, false); break;
        case 1: SAPA_NT(true, false); break;
        case 2: SAPA_NT(false, true); break;
        default: SAPA_NT(true, true); break;
    }
#undef SAPA_NT
    return hipGetLastError();
}

template <int R, int WR>
static hipError_t launch_rw(const void *src, void *dst, long units, int reps, int nt, hipStream_t st) {
    const long blocks = (units + reps - 1) / reps;
    if (blocks > (1L << 30)) return hipErrorInvalidValue;
    const dim3 grid((unsigned)blocks), block(256);
#define SAPA_NT(L, S)                                                                                  \
    hipLaunchKernelGGL((stream_mix_kernel<R, WR, L, S>), grid, block, 0, st, (const u4 *)src, (u4 *)dst, \
                       units, reps)
    switch (nt & 3) {
        case 0: SAPA_NT(false, false); break;
        case 1: SAPA_NT(true, false); break;
        case 2: SAPA_NT(false, true); break;
        default: SAPA_NT(true, true); break;
    }
#undef SAPA_NT
    return hipGetLastError();
}

hipError_t stream_mix_launch(const void *src, void *dst, long units, int reads, int writes, int reps,
                             int nt, hipStream_t st) {
#define SAPA_MIX(R, WR) \
    if (reads == R && writes == WR) return launch_rw<R, WR>(src, dst, units, reps, nt, st)
    SAPA_MIX(9, 16);   // fused SAPA-B forward at up_factor 2 with C = 4 d
    SAPA_MIX(8, 8);    // copy
    SAPA_MIX(0, 16);   // fill
    SAPA_MIX(16, 0);   // read
#undef SAPA_MIX
    return hipErrorNotSupported;
}

}  // namespace sapa
