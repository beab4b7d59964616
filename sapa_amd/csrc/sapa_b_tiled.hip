// LDS-tiled SAPA-B kernels for gfx950: qk, qk+softmax, av and the fused
// qk -> softmax -> av forward, all from one template.
//
// Work decomposition (NCHW tensors, so the contiguous axis is W):
//   * a wave owns WLX x (64/WLX) low-res parent cells of one image (16 x 4 or
//     32 x 2), lane = (lx 0..WLX-1, ly 0..64/WLX-1); a workgroup owns a tile
//     of NWX x NWY waves, TW x TH = (WLX*NWX) x ((64/WLX)*NWY) parents;
//   * a thread owns CY x S of the S x S high-res children of its parent
//     (CY = S: all of them; CY < S: S/CY waves share the parent rows), and
//     keeps their K*K logits / weights in registers (CY*S*K*K values);
//   * the low-res key (then value) window of the tile, tile + (K-1) halo, is
//     staged through LDS in chunks of CH channels, double-buffered, with the
//     next chunk's global loads in flight during the current chunk's FMAs.
//     Every staged value is reused by the CY*S children in registers and by
//     up to K*K parents through LDS;
//   * q is read and the output written exactly once, as S-wide vectors that
//     are contiguous across the WLX lanes of a row (S*WLX elements per row:
//     the longer these row segments, the fewer partial cache lines).
// LDS layout: two channels side by side in one LDS row, each in HALF >= WW+1
// floats with HALF = 8 mod 16, so the row stride 2*HALF is 16 mod 32 (48 for
// a 16-wide tile).  That puts the four 16-lane rows of a wave on disjoint
// banks, so the window reads (row ly+ky, column lx+kx) are conflict-free.
// What bounds the kernel on MI355X is the number of 64-byte requests between
// a CU's vector L1 and L2, not HBM bytes: a window row that starts 2 floats
// left of a 64-byte boundary costs a whole extra line per side, which is why
// wider tiles (NWX = 2) win even though they idle more lanes on ragged widths.
//
// Arithmetic is the reference kernels' own, term by term: one FMA per
// channel in channel order for the logits (qk_cuda_kernel.cu:55-66), one FMA
// per neighbour in ky-major order for the aggregation
// (av_cuda_kernel.cu:57-72).  Out-of-range neighbours are zeros in LDS: they
// leave a logit at exactly 0 (and that 0 takes part in the softmax) and add
// exactly 0 to the aggregation, which is what the reference's `continue`
// does.  16-bit tensors are widened to fp32 on the way into LDS/registers.
#include <type_traits>

#include "kernels.hpp"

namespace sapa {

#ifndef SAPA_TILED_WPE
#define SAPA_TILED_WPE 3
#endif
// fused fp32 problems of at most this many low-res cells take the two-waves-per-band geometry
#ifndef SAPA_TILED_SMALL_PARENTS
#define SAPA_TILED_SMALL_PARENTS 24576
#endif
// WIDE: the K*K-channel tensors of the call (attn_in; the result of the modes
// without aggregation) are fp32 while the feature tensors are T -- the form the
// backward pass of 16-bit tensors keeps its intermediates in
// (a thread with fewer than S x S children needs fewer registers: four waves per SIMD)
template <typename T, int K, int S, int CY, int NWX, int NWY, int CH, int VEC, int WLX, int MODE, bool WIDE = false>
__global__ void __launch_bounds__(64 * NWX * NWY * (S / CY))
    __attribute__((amdgpu_waves_per_eu(CY < S ? SAPA_TILED_WPE + 1 : SAPA_TILED_WPE, CY < S ? SAPA_TILED_WPE + 1 : SAPA_TILED_WPE)))
sapa_b_tiled_kernel(const T *__restrict__ q, const T *__restrict__ key,
                    const T *__restrict__ attn_in, const T *__restrict__ value,
                    T *__restrict__ out, int d, int C, int H, int W, int tiles_x, int tiles_y,
                    int nblocks, int per_xcd, int cgroups, int cper) {
    typedef float A;
    constexpr int KK = K * K, R = (K - 1) / 2;
    constexpr int NSUB = S / CY;           // waves sharing one band of parent rows
    constexpr int NT = 64 * NWX * NWY * NSUB;    // threads per workgroup
    constexpr int WLY = 64 / WLX;                  // a wave owns WLX x WLY parents
    static_assert(WLX == 16 || WLX == 32 || WLX == 64, "wave shape");
    constexpr int TW = WLX * NWX, TH = WLY * NWY;   // parents per workgroup
    // The window is staged as VEC-wide vectors (VEC = 1, 2 or 4 elements):
    // its left edge is moved out to a multiple of VEC and its width rounded up.
    constexpr int HL = (R + VEC - 1) / VEC * VEC;                 // left halo, staged
    constexpr int WW = (HL + TW + R + VEC - 1) / VEC * VEC;       // staged window width
    constexpr int WH = TH + K - 1;
    // LDS row: two channels side by side, each HALF > WW floats wide (spare
    // columns absorb surplus staging lanes) with HALF = 8 mod 16, so the row
    // stride is 16 mod 32
#ifndef SAPA_TILED_OPAQUE_BASE
#define SAPA_TILED_OPAQUE_BASE 1
#endif
#ifndef SAPA_TILED_PLAIN_ROWS
#define SAPA_TILED_PLAIN_ROWS 1
#endif
    constexpr bool PAIRED = WLX == 16 || !SAPA_TILED_PLAIN_ROWS;
    constexpr int HALF = PAIRED ? ((WW + VEC - 8 + 15) / 16) * 16 + 8 : (WW + VEC + 3) / 4 * 4;
    constexpr int STRIDE = PAIRED ? 2 * HALF : HALF;
    // float offset of channel ch of a chunk inside a buffer
    auto ch_off = [](int ch) { return PAIRED ? (ch >> 1) * WH * STRIDE + (ch & 1) * HALF : ch * WH * STRIDE; };
    constexpr int NVR = WW / VEC, NVP = WH * NVR;   // vectors per row / per channel
    // staging threads are split into NSL slices that take every NSL-th channel
    constexpr int NSL = (CH % 4 == 0 && NT >= 4 * NVP && NT % 256 == 0) ? 4
                        : (NT >= 2 * NVP && NT % 128 == 0) ? 2 : 1;
    constexpr int TPC = NT / NSL;                   // threads per slice (whole waves)
    constexpr int NPOS = (NVP + TPC - 1) / TPC;     // vectors per thread and channel
    constexpr int CPT = CH / NSL;                   // channels per thread
    constexpr int NSTAGE = CPT * NPOS * VEC;
    constexpr int BUF = (PAIRED ? CH / 2 : CH) * WH * STRIDE;
    constexpr int NJ = CY * S;             // children per thread
    constexpr bool DO_QK = MODE != TILED_AV;
    constexpr bool DO_SOFTMAX = MODE == TILED_QK_SOFTMAX || MODE == TILED_FUSED;
    constexpr bool DO_AV = MODE == TILED_AV || MODE == TILED_FUSED;
    static_assert(WW + VEC <= HALF && (!PAIRED || STRIDE % 32 == 16), "LDS row layout");
    static_assert(TPC % 64 == 0 && CH % NSL == 0, "staging slices are whole waves");
    typedef Vec<T, VEC> VecV;
    static_assert(CH % 2 == 0, "channels are staged in pairs");
    static_assert(S % CY == 0, "CY must divide S");
    typedef Vec<T, S> VecS;
    static_assert(!WIDE || MODE == TILED_AV || MODE == TILED_QK_SOFTMAX || MODE == TILED_QK_SOFTMAX_BWD,
                  "fp32 K*K tensors: the modes the backward pass uses");
    typedef typename std::conditional<WIDE, float, T>::type TA;   // type of the K*K-channel tensors
    typedef Vec<TA, S> VecA;
    const TA *attn_w = reinterpret_cast<const TA *>(attn_in);

    // fp32 windows staged as 16-byte vectors go from global memory straight into LDS
    // (buffer loads with the LDS modifier): no staging registers, no LDS write instructions,
    // and the hardware's zero for an out-of-range offset is the window's zero padding.
#ifndef SAPA_TILED_DMA
#define SAPA_TILED_DMA 1
#endif
    constexpr bool DMA = SAPA_TILED_DMA && std::is_same<T, float>::value && VEC == 4;
    // a wave's load fills 64 consecutive 16-byte slots: buffers are whole numbers of those
    constexpr int BUFA = DMA ? (BUF + 255) / 256 * 256 : BUF;
    constexpr int NW = NT / 64, NBLK = BUFA / 256;   // waves; 64-slot blocks per buffer
    constexpr int NLD = DMA ? (NBLK + NW - 1) / NW : 1;       // loads per wave and chunk
    // vector memory operations a wave issues per chunk after its staging loads (q loads in
    // the logits phase, output stores in the aggregation): the staging loads have landed
    // when no more than these are outstanding
    constexpr int NAFTER = CH * CY;
    static_assert(STRIDE % 4 == 0 && HALF % 4 == 0 && NAFTER < 64, "direct-to-LDS staging");
    __shared__ __attribute__((aligned(16))) A lds[2 * BUFA];

    // Workgroups are handed to the 8 XCDs round-robin; give each XCD a
    // contiguous run of tiles so that neighbouring tiles (which share halo
    // rows) meet in the same L2.
    const int logical = (int)(blockIdx.x % 8) * per_xcd + (int)(blockIdx.x / 8);
    if (logical >= nblocks) return;
    // logical = ((n * cgroups + cg) * tiles_y + ty) * tiles_x + tx; a small
    // problem is split over `cgroups` slices of `cper` value channels each
    // (every slice recomputes the logits) so that the chip is still filled
    const int tx = logical % tiles_x;
    const int ty = (logical / tiles_x) % tiles_y;
    const int cg = (logical / (tiles_x * tiles_y)) % cgroups;
    const int n = logical / (tiles_x * tiles_y * cgroups);
    const int cbeg = cg * cper;                      // first value channel of this slice
    const int cend = cbeg + cper < C ? cbeg + cper : C;
    if (DO_AV && cbeg >= C) return;                  // rounding left this slice empty

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int sub = wave % NSUB, wxy = wave / NSUB;
    const int lx = (wxy % NWX) * WLX + (lane % WLX), ly = (wxy / NWX) * WLY + (lane / WLX);
    const int x0 = tx * TW, y0 = ty * TH;          // tile origin (parents)
    const int px = x0 + lx, py = y0 + ly;
    const bool active = px < W && py < H;
    const int hH = H * S, hW = W * S;
    const long lplane = (long)H * W, hplane = (long)hH * hW;
    // first child of this thread; idle threads of a partial tile read (never
    // write) through the clamped copy, so their loads need no branch
    const long hpix = (long)(py * S + sub * CY) * hW + (long)px * S;
    const long hpix_ld =
        (long)((py < H ? py : H - 1) * S + sub * CY) * hW + (long)(px < W ? px : W - 1) * S;

    const int nKc = DO_QK ? (d + CH - 1) / CH : 0;
    const int nVc = DO_AV ? (cend - cbeg + CH - 1) / CH : 0;
    const int ntot = nKc + nVc;

    // Staging map: thread t of slice sl carries vectors t, t+TPC, ... of the
    // window of channels sl, sl+NSL, ... of a chunk, so the per-thread part
    // of each address (in-plane offset, LDS offset, inside-the-image mask) is
    // fixed for the whole kernel and the channel part is wave-uniform.
    // (a slice is whole waves: its number is wave-uniform, and so is every channel address)
    const int sl = __builtin_amdgcn_readfirstlane(tid / TPC), vt = tid % TPC;
    unsigned g_off[NPOS];   // byte offset inside a channel plane
    int l_off[NPOS];
    unsigned g_mask[NPOS];
#pragma unroll
    for (int i = 0; i < NPOS; ++i) {
        const int v = vt + i * TPC;
        const int row = v / NVR, col = (v % NVR) * VEC;
        const int gy = y0 - R + row, gx = x0 - HL + col;
        const bool l_ok = NVP % TPC == 0 || v < NVP;
        // W is a multiple of VEC and gx too: a vector is all inside or all outside
        const bool g_ok = l_ok && gy >= 0 && gy < H && gx >= 0 && gx + VEC <= W;
        const int yy = gy < 0 ? 0 : (gy < H ? gy : H - 1);
        const int xx = gx < 0 ? 0 : (gx + VEC <= W ? gx : W - VEC);
        g_off[i] = (unsigned)(yy * W + xx) * (unsigned)sizeof(T);   // clamped: always a legal address
        g_mask[i] = g_ok ? 0xffffffffu : 0u;
        // surplus vectors land in the unread spare columns of row 0
        l_off[i] = l_ok ? row * STRIDE + col : WW;
    }
    // Direct-to-LDS map: load i of wave w fills slots ((i * NW + w) * 64 + lane) of a buffer;
    // the slot's place in the LDS layout gives the channel of the chunk and the window
    // position it holds, i.e. a byte offset from the chunk's first plane -- or 2^31 (out of
    // any range: the hardware writes zeros) for padding columns, positions outside the
    // image and the tail of the last block.  Channels past the last one fall outside the
    // descriptor the same way.
    const int wave_u = __builtin_amdgcn_readfirstlane(tid >> 6);
    unsigned d_off[NLD];
    if constexpr (DMA) {
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int f = (((i * NW + wave_u) * 64) + (tid & 63)) * 4;   // float index in the buffer
            const int prow = f / STRIDE, cf = f % STRIDE;
            const int half = PAIRED && cf >= HALF ? 1 : 0;
            const int col = cf - half * HALF;
            const int ch = PAIRED ? (prow / WH) * 2 + half : prow / WH;
            const int gy = y0 - R + prow % WH, gx = x0 - HL + col;
            const bool ok = f < BUF && col < WW && gy >= 0 && gy < H && gx >= 0 && gx + VEC <= W;
            d_off[i] = ok ? (unsigned)ch * (unsigned)(lplane * (long)sizeof(T)) +
                                (unsigned)(gy * W + gx) * (unsigned)sizeof(T)
                          : 0x80000000u;
        }
    }
    A st[NSTAGE];
    // global -> registers (or straight into LDS buffer j&1) for staged chunk j (key chunks
    // first, then value)
    auto stage_load = [&](int j) {
        const bool is_key = j < nKc;
        const T *src = is_key ? key : value;
        const int nch = is_key ? d : C;
        const int c0 = is_key ? j * CH : cbeg + (j - nKc) * CH;
        if constexpr (DMA) {
            // (device pass only: the host pass, which sees this body for the launch stub,
            // knows neither the builtin nor the instructions of the chunk barrier)
#if defined(__HIP_DEVICE_COMPILE__)
            const int nleft = nch - c0 < CH ? nch - c0 : CH;
            const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
                (void *)(src + ((long)n * nch + c0) * lplane), 0,
                (int)((unsigned)nleft * (unsigned)(lplane * (long)sizeof(T))), 0x00020000);
            A *dst = lds + (j & 1) * BUFA;
#pragma unroll
            for (int i = 0; i < NLD; ++i) {
                const int blk = i * NW + wave_u;
                if ((i + 1) * NW <= NBLK || blk < NBLK)
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(
                        rsrc, (__attribute__((address_space(3))) void *)(dst + blk * 256), 16, d_off[i], 0, 0, 0);
            }
            // everything below is issued after these loads (the wait at the end of the
            // chunk counts on it)
            asm volatile("" ::: "memory");
            __builtin_amdgcn_sched_barrier(0);
#endif
            return;
        }
        const T *base = src + (long)n * nch * lplane;
#pragma unroll
        for (int ci = 0; ci < CPT; ++ci) {
            const int c = c0 + sl + ci * NSL;
            const char *plane = (const char *)(base + (long)(c < nch ? c : nch - 1) * lplane);
#pragma unroll
            for (int i = 0; i < NPOS; ++i) {
                // unconditional load from the clamped address; the value is
                // masked when it is stored to LDS, so that the load stays in
                // flight across the FMAs of the current chunk
                unsigned o = g_off[i];
                asm volatile("" : "+v"(o));
                const VecV v = *(const VecV *)(plane + o);
#pragma unroll
                for (int e = 0; e < VEC; ++e) st[(ci * NPOS + i) * VEC + e] = (A)v.v[e];
            }
        }
    };
    // registers -> LDS buffer j&1, zeroing what lies outside the image or
    // past the last channel
    auto stage_store = [&](int j) {
        if constexpr (DMA) return;
        const bool is_key = j < nKc;
        const int nch = is_key ? d : C;
        const int c0 = is_key ? j * CH : cbeg + (j - nKc) * CH;
        A *dst = lds + (j & 1) * BUFA;
#pragma unroll
        for (int ci = 0; ci < CPT; ++ci) {
            const int ch = sl + ci * NSL;
            A *dc = dst + ch_off(ch);
#pragma unroll
            for (int i = 0; i < NPOS; ++i) {
                const unsigned m = c0 + ch < nch ? g_mask[i] : 0u;
                Vec<A, VEC> o;
#pragma unroll
                for (int e = 0; e < VEC; ++e)
                    o.v[e] = __uint_as_float(__float_as_uint(st[(ci * NPOS + i) * VEC + e]) & m);
                *(Vec<A, VEC> *)(dc + l_off[i]) = o;
            }
        }
    };

    A a[NJ][KK];
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
        for (int k = 0; k < KK; ++k) a[j][k] = 0;

    stage_load(0);
    if (MODE == TILED_AV && active) {
        const TA *ap = attn_w + (long)n * KK * hplane + hpix;
#pragma unroll
        for (int k = 0; k < KK; ++k)
#pragma unroll
            for (int cy = 0; cy < CY; ++cy) {
                const VecA v = *(const VecA *)(ap + (long)k * hplane + (long)cy * hW);
#pragma unroll
                for (int cx = 0; cx < S; ++cx) a[cy * S + cx][k] = (A)v.v[cx];
            }
    }
    stage_store(0);
    // End of a chunk: the next chunk's window is in LDS and every wave is done with this one.
    // (Direct-to-LDS: wait until only the operations issued after the staging loads are
    // outstanding -- the counter retires in issue order -- so output stores stay in flight.)
    auto chunk_barrier = [&](bool staged, bool first) {
        if constexpr (DMA) {
#if defined(__HIP_DEVICE_COMPILE__)
            if (first) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            else if (staged) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NAFTER) : "memory");
            asm volatile("s_barrier" ::: "memory");
#endif
        } else {
            __syncthreads();
        }
    };
    chunk_barrier(true, true);

    // this thread's window origin in buffer 0 (its neighbour kx = 0 column)
    const A *win = lds + ly * STRIDE + lx + (HL - R);   // (buffer 1 is BUFA floats further)

    if (DO_QK) {
        // (wave-uniform plane address + a 32-bit per-lane byte offset: no per-lane address arithmetic)
        const char *qp = (const char *)(q + (long)n * d * hplane);
        unsigned qoff[CY];
#pragma unroll
        for (int cy = 0; cy < CY; ++cy) qoff[cy] = (unsigned)((hpix_ld + (long)cy * hW) * (long)sizeof(T));
        const unsigned qmask = active ? 0xffffffffu : 0u;
        // q is fetched PF channels ahead of its use (a ring of PF x NJ
        // registers), so HBM latency hides behind the FMAs of PF channels.
#ifndef SAPA_TILED_PF
#define SAPA_TILED_PF 4
#endif
        // (twice as far ahead when a thread has half the children: a channel is then over
        // in half the time)
        constexpr int PFW = CY < S ? 2 * SAPA_TILED_PF : SAPA_TILED_PF;
        constexpr int PF = CH < PFW ? CH : PFW;
        static_assert(CH % PF == 0, "prefetch ring must divide the chunk");
        A qr[PF][NJ];
        auto load_q = [&](int c, A (&dst)[NJ]) {
#pragma unroll
            for (int cy = 0; cy < CY; ++cy) {
                const char *plane = qp + (long)(c < d ? c : d - 1) * hplane * (long)sizeof(T);
                // (the offset is widened next to its use, or the compiler keeps a 64-bit copy
                // of it and adds the plane address per lane)
                unsigned o = qoff[cy];
                asm volatile("" : "+v"(o));
                const VecS v = load_stream<T, S>((const T *)(plane + o));
#pragma unroll
                for (int cx = 0; cx < S; ++cx) dst[cy * S + cx] = (A)v.v[cx];
            }
        };
#pragma unroll
        for (int u = 0; u < PF; ++u) load_q(u, qr[u]);
        for (int j = 0; j < nKc; ++j) {
            if (j + 1 < ntot) stage_load(j + 1);
            const int c0 = j * CH;
            const A *wb = win + (j & 1) * BUFA;
#pragma unroll 1
            for (int ch0 = 0; ch0 < CH; ch0 += PF) {
#pragma unroll
                for (int u = 0; u < PF; ++u) {
                    const int ch = ch0 + u;
                    // ring values are raw loads from clamped addresses: zero
                    // them for idle threads and past the last channel here
                    const unsigned m = c0 + ch < d ? qmask : 0u;
                    A qv[NJ];
#pragma unroll
                    for (int jj = 0; jj < NJ; ++jj)
                        qv[jj] = __uint_as_float(__float_as_uint(qr[u][jj]) & m);
                    load_q(c0 + ch + PF, qr[u]);
                    int co = ch_off(ch);
#if SAPA_TILED_OPAQUE_BASE
                    asm volatile("" : "+v"(co));
#endif
                    const A *wc = wb + co;
#pragma unroll
                    for (int ky = 0; ky < K; ++ky)
#pragma unroll
                        for (int kx = 0; kx < K; ++kx) {
                            const A kv = wc[ky * STRIDE + kx];
#pragma unroll
                            for (int jj = 0; jj < NJ; ++jj)
                                a[jj][ky * K + kx] = fma_(kv, qv[jj], a[jj][ky * K + kx]);
                        }
                    // keep the next channel's window reads from being hoisted
                    // over this channel's FMAs (register pressure)
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            if (j + 1 < ntot) stage_store(j + 1);
            chunk_barrier(j + 1 < ntot, false);
        }
        if (DO_SOFTMAX) {
#pragma unroll
            for (int jj = 0; jj < NJ; ++jj) softmax_inplace<A, KK>(a[jj]);
        }
        if (MODE == TILED_QK_SOFTMAX_BWD && active) {
            // a[][] holds g = d(loss)/d(attn); turn it into d(loss)/d(logits).
            // The weights are read twice (the second time from cache) rather
            // than kept in another K*K registers per child.
            const TA *ap = attn_w + (long)n * KK * hplane + hpix;
            A dot[NJ];
#pragma unroll
            for (int jj = 0; jj < NJ; ++jj) dot[jj] = 0;
#pragma unroll
            for (int k = 0; k < KK; ++k)
#pragma unroll
                for (int cy = 0; cy < CY; ++cy) {
                    const VecA v = *(const VecA *)(ap + (long)k * hplane + (long)cy * hW);
#pragma unroll
                    for (int cx = 0; cx < S; ++cx)
                        dot[cy * S + cx] = fma_(a[cy * S + cx][k], (A)v.v[cx], dot[cy * S + cx]);
                }
            // (through an opaque copy of the pointer: the compiler would otherwise keep
            // the first pass's K*K loads for this one and spill them)
            const TA *ap2 = ap;
            asm volatile("" : "+v"(ap2));
#pragma unroll
            for (int k = 0; k < KK; ++k)
#pragma unroll
                for (int cy = 0; cy < CY; ++cy) {
                    const VecA v = *(const VecA *)(ap2 + (long)k * hplane + (long)cy * hW);
#pragma unroll
                    for (int cx = 0; cx < S; ++cx)
                        a[cy * S + cx][k] = (A)v.v[cx] * (a[cy * S + cx][k] - dot[cy * S + cx]);
                }
        }
        if (!DO_AV && active) {
            TA *op = reinterpret_cast<TA *>(out) + (long)n * KK * hplane + hpix;
#pragma unroll
            for (int k = 0; k < KK; ++k)
#pragma unroll
                for (int cy = 0; cy < CY; ++cy) {
                    VecA v;
#pragma unroll
                    for (int cx = 0; cx < S; ++cx) v.v[cx] = (TA)a[cy * S + cx][k];
                    *(VecA *)(op + (long)k * hplane + (long)cy * hW) = v;
                }
        }
    }

    if (DO_AV) {
        // The results leave through buffer stores whose descriptor covers exactly
        // the channels of the chunk that exist: idle lanes (offset 2^31) and
        // channels past the slice fall outside it and the hardware drops them.
        // That keeps the channel loop free of branches, so it can be unrolled with
        // a known number of stores behind the next chunk's staging loads: the wait
        // for those loads then leaves this chunk's stores in flight (the counter
        // retires in issue order) instead of draining them at every chunk.
        const unsigned ooff = active ? (unsigned)(hpix * (long)sizeof(T)) : 0x80000000u;
        const unsigned plane_bytes = (unsigned)(hplane * (long)sizeof(T));
        for (int j = nKc; j < ntot; ++j) {
            if (j + 1 < ntot) stage_load(j + 1);
            const int c0 = cbeg + (j - nKc) * CH;
            const A *wb = win + (j & 1) * BUFA;
            const int nleft = cend - c0 < CH ? cend - c0 : CH;
            const __amdgpu_buffer_rsrc_t orsrc = __builtin_amdgcn_make_buffer_rsrc(
                (void *)(out + ((long)n * C + c0) * hplane), 0, (int)((unsigned)nleft * plane_bytes), 0x00020000);
#pragma unroll
            for (int ch = 0; ch < CH; ++ch) {
                int co = ch_off(ch);
#if SAPA_TILED_OPAQUE_BASE
                    asm volatile("" : "+v"(co));
#endif
                    const A *wc = wb + co;
                A o[NJ];
#pragma unroll
                for (int jj = 0; jj < NJ; ++jj) o[jj] = 0;
#pragma unroll
                for (int ky = 0; ky < K; ++ky)
#pragma unroll
                    for (int kx = 0; kx < K; ++kx) {
                        const A vv = wc[ky * STRIDE + kx];
#pragma unroll
                        for (int jj = 0; jj < NJ; ++jj)
                            o[jj] = fma_(vv, a[jj][ky * K + kx], o[jj]);
                    }
#pragma unroll
                for (int cy = 0; cy < CY; ++cy) {
                    VecS v;
#pragma unroll
                    for (int cx = 0; cx < S; ++cx) v.v[cx] = (T)o[cy * S + cx];
                    store_buffer<T, S>(orsrc, ooff + (unsigned)ch * plane_bytes +
                                                  (unsigned)(cy * hW) * (unsigned)sizeof(T), v);
                }
                // one channel at a time: keeps the next channel's window reads from
                // being hoisted over this channel's FMAs (register pressure)
                __builtin_amdgcn_sched_barrier(0);
            }
            if (j + 1 < ntot) stage_store(j + 1);
            chunk_barrier(j + 1 < ntot, false);
        }
    }
}

// ------------------------------------------------------------------ launcher
template <typename T, int K, int S, int CY, int NWX, int NWY, int CH, int VEC, int WLX>
static hipError_t launch_mode(int mode, bool wide, const void *q, const void *key, const void *attn_in,
                              const void *value, void *out, int B, int d, int C, int H, int W,
                              hipStream_t st) {
    constexpr int TW = WLX * NWX, TH = (64 / WLX) * NWY, NT = 64 * NWX * NWY * (S / CY);
    const int tiles_x = (W + TW - 1) / TW, tiles_y = (H + TH - 1) / TH;
    // Few tiles: slice the value channels over several workgroups per tile,
    // up to two workgroups per CU (256 CUs) -- beyond that the recomputed
    // logits cost more than the added parallelism gains (measured).  A slice
    // is a multiple of CH channels and at least 4 chunks long.
    int cgroups = 1;
    if (mode == TILED_FUSED || mode == TILED_AV) {
        const long tiles = (long)tiles_x * tiles_y * B;
        const int max_groups = C / (4 * CH) > 0 ? C / (4 * CH) : 1;
        // (16-bit tensors: up to four per CU -- their recomputed logits cost
        // relatively less -- measured on the FPN levels)
        const long limit = sizeof(T) == 2 ? 1024 : 512;
        while (cgroups * 2 <= max_groups && tiles * cgroups * 2 <= limit) cgroups *= 2;
#ifdef SAPA_TUNE_CGROUPS
        cgroups = SAPA_TUNE_CGROUPS;
#endif
    }
    const int cper = ((C + cgroups - 1) / cgroups + CH - 1) / CH * CH;
    const long nb = (long)tiles_x * tiles_y * B * cgroups;
    if (nb > (1L << 30)) return hipErrorNotSupported;
    // the output leaves through 32-bit byte offsets inside one chunk of CH planes
    if ((long)CH * H * S * W * S * (long)sizeof(T) > (1L << 31)) return hipErrorNotSupported;
    const int per_xcd = (int)((nb + 7) / 8);
    const dim3 grid(per_xcd * 8), block(NT);
#define SAPA_TM_LAUNCH(M, WD)                                                                 \
    hipLaunchKernelGGL((sapa_b_tiled_kernel<T, K, S, CY, NWX, NWY, CH, VEC, WLX, M, WD>), grid, block, 0, st, \
                       (const T *)q, (const T *)key, (const T *)attn_in, (const T *)value,    \
                       (T *)out, d, C, H, W, tiles_x, tiles_y, (int)nb, per_xcd, cgroups, cper)
#define SAPA_TM_CASE(M)                                                                       \
    case M:                                                                                   \
        SAPA_TM_LAUNCH(M, false);                                                             \
        break;
    if (wide) {
        // fp32 K*K tensors next to 16-bit features (for fp32 features that is the plain form)
        if constexpr (sizeof(T) == 2) {
            switch (mode) {
                case TILED_QK_SOFTMAX: SAPA_TM_LAUNCH(TILED_QK_SOFTMAX, true); break;
                case TILED_AV: SAPA_TM_LAUNCH(TILED_AV, true); break;
                case TILED_QK_SOFTMAX_BWD: SAPA_TM_LAUNCH(TILED_QK_SOFTMAX_BWD, true); break;
                default: return hipErrorNotSupported;
            }
            return hipGetLastError();
        }
    }
    switch (mode) {
        SAPA_TM_CASE(TILED_QK) SAPA_TM_CASE(TILED_QK_SOFTMAX) SAPA_TM_CASE(TILED_AV)
        SAPA_TM_CASE(TILED_FUSED) SAPA_TM_CASE(TILED_QK_SOFTMAX_BWD)
        default: return hipErrorInvalidValue;
    }
#undef SAPA_TM_LAUNCH
#undef SAPA_TM_CASE
    return hipGetLastError();
}

template <typename T>
static hipError_t launch_t(int mode, bool wide, const void *q, const void *key, const void *attn_in,
                           const void *value, void *out, int B, int d, int C, int H, int W, int K,
                           int s, hipStream_t st) {
    // vector accesses of s elements on the high-res tensors
    const uintptr_t align = (uintptr_t)(sizeof(T) * s), walign = wide ? (uintptr_t)(4 * s) : align;
    const bool out_is_kk = mode != TILED_AV && mode != TILED_FUSED;
    const void *hi_ptrs[3] = {q, attn_in, out};
    const uintptr_t hi_align[3] = {align, walign, out_is_kk ? walign : align};
    for (int i = 0; i < 3; ++i)
        if (hi_ptrs[i] && ((uintptr_t)hi_ptrs[i] % hi_align[i]) != 0) return hipErrorNotSupported;
    if (K == 5 && s == 2) {
#ifdef SAPA_TUNE_GEOM
        return launch_mode<T, 5, 2, SAPA_TUNE_GEOM>(mode, wide, q, key, attn_in, value, out, B, d, C, H, W, st);
#else
        // Tile geometry: padded parent count times the relative cost per
        // parent measured at the FPN shapes on MI355X (wider tiles fetch
        // fewer partial cache lines per window row, taller ones fewer halo
        // rows; both idle more lanes on ragged extents).
        auto padded = [&](int tw, int th) {
            return (double)((W + tw - 1) / tw * tw) * (double)((H + th - 1) / th * th);
        };
        // 32 x 8 tiles are built from 32 x 2-parent waves: their hi-res row
        // segments are twice as long as those of 16 x 4-parent waves.
        const double c12 = padded(16, 8), c14 = 0.96 * padded(16, 16), c22 = 0.81 * padded(32, 8);
        // The low-res windows are staged with 4- or 2-element vector loads
        // when rows and base pointers allow it (scalar loads otherwise).
        auto aligned = [&](int vec) {
            const uintptr_t a = (uintptr_t)(sizeof(T) * vec);
            return W % vec == 0 && (!key || (uintptr_t)key % a == 0) &&
                   (!value || (uintptr_t)value % a == 0);
        };
        // Small problems (a few waves per SIMD at most, so a wave's own instruction latencies
        // show): two waves per band of parent rows, each thread with the two children of one
        // hi-res row (half the accumulators, twice the waves), 16-channel chunks (half the
        // barriers).  Measured at B=16, 25x42, d=64, C=256, fp32: 80 -> 59 us.
        // (fp32 windows of 16-wide tiles are also staged as 4-element vectors where the rows
        // allow it, 4 columns wider: those go straight into LDS.  25x42-class shapes measured
        // 59 -> 57 us, the 16 x 8 tiles 85 -> 73 us, the 16 x 16 tiles 66 -> 60 us.)
        constexpr bool F32 = std::is_same<T, float>::value;
        if (mode == TILED_FUSED && !wide && (long)B * H * W <= SAPA_TILED_SMALL_PARENTS) {
            if constexpr (F32)
                if (aligned(4))
                    return launch_mode<T, 5, 2, 1, 1, 2, 16, 4, 16>(mode, wide, q, key, attn_in, value, out, B, d, C, H, W, st);
            return aligned(2)
                       ? launch_mode<T, 5, 2, 1, 1, 2, 16, 2, 16>(mode, wide, q, key, attn_in, value, out, B, d, C, H, W, st)
                       : launch_mode<T, 5, 2, 1, 1, 2, 16, 1, 16>(mode, wide, q, key, attn_in, value, out, B, d, C, H, W, st);
        }
#define SAPA_GEOM(NWX, NWY, VEC, WLX)                                                            \
    launch_mode<T, 5, 2, 2, NWX, NWY, 8, VEC, WLX>(mode, wide, q, key, attn_in, value, out, B, d, C, H, \
                                                   W, st)
        if (c22 <= c12 && c22 <= c14)
            return aligned(4) ? SAPA_GEOM(1, 4, 4, 32) : SAPA_GEOM(1, 4, 1, 32);
        if (c14 <= c12) {
            if constexpr (F32)
                if (aligned(4)) return SAPA_GEOM(1, 4, 4, 16);
            return aligned(2) ? SAPA_GEOM(1, 4, 2, 16) : SAPA_GEOM(1, 4, 1, 16);
        }
        if constexpr (F32)
            if (aligned(4)) return SAPA_GEOM(1, 2, 4, 16);
        return aligned(2) ? SAPA_GEOM(1, 2, 2, 16) : SAPA_GEOM(1, 2, 1, 16);
#undef SAPA_GEOM
#endif
    }
    return hipErrorNotSupported;
}

hipError_t sapa_b_tiled_launch(int mode, const void *q, const void *key, const void *attn_in,
                               const void *value, void *out, int B, int d, int C, int H, int W,
                               int K, int s, int dtype, hipStream_t st, bool wide) {
    switch (dtype) {
        case 0: return launch_t<float>(mode, wide, q, key, attn_in, value, out, B, d, C, H, W, K, s, st);
#if (!defined(SAPA_TUNE_GEOM) || defined(SAPA_TUNE_ALLTYPES)) && !defined(SAPA_TUNE_ONLY_F32)
        case 2: return launch_t<f16_t>(mode, wide, q, key, attn_in, value, out, B, d, C, H, W, K, s, st);
        case 3: return launch_t<bf16_t>(mode, wide, q, key, attn_in, value, out, B, d, C, H, W, K, s, st);
#endif
        default: return hipErrorNotSupported;
    }
}

}  // namespace sapa
