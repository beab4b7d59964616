// Streaming calibration kernel: what this GPU's memory system gives a kernel
// that does nothing but move a stated mix of bytes in and out, each workgroup
// in long contiguous runs.  It is the yardstick the operators' measured rates
// are put beside (the published HBM peak is not reachable by any kernel): a
// fused SAPA-B forward at up_factor 2 reads 9 bytes for every 16 it writes
// (q and the low-res key / value in, the C-channel high-res result out, with
// C = 4 d), a copy reads 1 for 1, a fill reads nothing.
//
// A unit = one workgroup of 256 threads, 16 bytes per thread and row: it
// reads R rows (one contiguous run of R * 4 KiB) and writes WR rows (one
// contiguous run of WR * 4 KiB); what it writes depends on what it read, so
// no access can be dropped.  Loads of a unit are all issued before its first
// store; overlap of loads and stores comes from the workgroups that share a CU.
#include "kernels.hpp"

namespace sapa {

typedef unsigned u4 __attribute__((ext_vector_type(4)));

template <int R, int WR, bool NT>
__global__ void __launch_bounds__(256) stream_mix_kernel(const u4 *__restrict__ src, u4 *__restrict__ dst,
                                                         long units) {
    const long u = blockIdx.x;
    if (u >= units) return;
    const int t = threadIdx.x;
    u4 v[R > 0 ? R : 1];
    if constexpr (R > 0) {
        const u4 *s = src + u * (long)(R * 256) + t;
#pragma unroll
        for (int i = 0; i < R; ++i) v[i] = NT ? __builtin_nontemporal_load(s + i * 256) : s[i * 256];
    } else {
        v[0] = u4{(unsigned)u, (unsigned)t, 0u, 0u};
    }
    if constexpr (WR > 0) {
        u4 *d = dst + u * (long)(WR * 256) + t;
#pragma unroll
        for (int j = 0; j < WR; ++j) {
            u4 o = v[R > 0 ? j % R : 0];
            o.x += (unsigned)j;
            if (NT) __builtin_nontemporal_store(o, d + j * 256);
            else d[j * 256] = o;
        }
    } else {
        u4 a = v[0];
#pragma unroll
        for (int i = 1; i < R; ++i) a ^= v[i];
        // never true for the data the caller fills src with; keeps the loads
        if ((a.x & a.y & a.z & a.w) == 0xfffffffeu) dst[u * 256 + t] = a;
    }
}

template <int R, int WR>
static hipError_t launch_rw(const void *src, void *dst, long units, bool nt, hipStream_t st) {
    if (units > (1L << 30)) return hipErrorInvalidValue;
    const dim3 grid((unsigned)units), block(256);
    if (nt) hipLaunchKernelGGL((stream_mix_kernel<R, WR, true>), grid, block, 0, st, (const u4 *)src, (u4 *)dst, units);
    else hipLaunchKernelGGL((stream_mix_kernel<R, WR, false>), grid, block, 0, st, (const u4 *)src, (u4 *)dst, units);
    return hipGetLastError();
}

hipError_t stream_mix_launch(const void *src, void *dst, long units, int reads, int writes, bool nt,
                             hipStream_t st) {
#define SAPA_MIX(R, WR) \
    if (reads == R && writes == WR) return launch_rw<R, WR>(src, dst, units, nt, st)
    SAPA_MIX(9, 16);   // fused SAPA-B forward at up_factor 2 with C = 4 d
    SAPA_MIX(18, 32);  // the same mix in runs twice as long
    SAPA_MIX(8, 8);    // copy
    SAPA_MIX(0, 16);   // fill
    SAPA_MIX(16, 0);   // read
#undef SAPA_MIX
    return hipErrorNotSupported;
}

}  // namespace sapa
