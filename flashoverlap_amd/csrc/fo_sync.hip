// Counter side of the overlap protocol: the wait (counting) kernel, the
// persistent wait+consume kernel, the consumer copy and the slot->group table.
//
// The GEMM epilogue bumps MM[g] once a tile of group g is visible device-wide:
// by default its tile stores are agent-scope write-through stores whose
// acknowledgement every wavefront waits for, then the workgroup meets at a
// barrier and a relaxed agent-scope atomic moves the counter (the
// release-ordered atomic is a tuning knob of the GEMM, not what runs by
// default).  The kernels here run on a second stream while the GEMM is still
// executing.  MI355X has one L2 per XCD and they
// are not coherent with each other, so a reader on another XCD must not hit a
// stale line.  An acquire would do that by invalidating its caches - including
// the A/B panels that the GEMM workgroups of that XCD are sharing through the
// same L2, once per poll.  So the counters are polled with relaxed agent-scope
// loads (which bypass the non-coherent caches and invalidate nothing), and the
// persistent consumer then reads the released tiles with agent-scope coherent
// loads as well; nothing is invalidated while the GEMM runs.  Every wait is
// bounded in wall-clock time so that a wrong cSeg can delay a stream but never
// hang the device.
#include <hip/hip_runtime.h>

#include <atomic>

#include "fo_internal.h"
#include "fo_knobs.h"

namespace fo {

// Expired waits are counted in the word the caller passes (`expired`, one that it owns: the count
// of its own calls) or, if it passes none, in this per-device word (fo_wait_timeouts).
__device__ int g_wait_timeouts = 0;

__device__ __forceinline__ void count_expired(int* expired) { atomicAdd(expired ? expired : &g_wait_timeouts, 1); }

// Bounded poll of *addr until pred(value); returns false on expiry.
// long_naps: 127 x 64 clocks (about 3 us) between two looks instead of 8 x 64 (0.2 us).
template <typename Pred>
__device__ __forceinline__ bool bounded_poll(const int* addr, long long ticks, Pred pred, bool long_naps = false) {
    const long long t0 = wall_clock64();
    for (;;) {
        const int v = __hip_atomic_load(addr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (pred(v)) return true;
        if (wall_clock64() - t0 > ticks) return false;
        if (long_naps) __builtin_amdgcn_s_sleep(127);
        else __builtin_amdgcn_s_sleep(8);
    }
}

// Counterpart of the reference's kernel_wait_flag (src/wait.cuh:5-9): returns
// once *addr == that and leaves 0 there.  Nothing else writes *addr between
// the last tile's signal and the reset, so load-then-store equals the
// reference's compare-and-swap.  The kernel that follows on the stream sees
// the group's tiles through the cache invalidation at its own start.
__global__ void wait_kernel(int that, int* addr, long long ticks, int* expired) {
    if (threadIdx.x != 0) return;
    if (bounded_poll(addr, ticks, [that](int v) { return v == that; }))
        __hip_atomic_store(addr, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else
        count_expired(expired);
}

constexpr int kCopyThreads = 512;  // workgroup size of the per-group copy kernel
constexpr int kCopyUnroll = 8;     // 16-byte units in flight per thread
constexpr int kWavesPerBlock = 4;  // persistent consumer: one wavefront per SIMD
constexpr long long kUnitsPerMember = 8192;  // 128 KiB: what one workgroup takes of a group before another joins

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// Copies n 16-byte units as member `me` of a team of `team` members of WIDTH
// threads each (`t` is the thread's index inside its member), which interleave
// in chunks of WIDTH * kCopyUnroll units, every thread keeping kCopyUnroll
// loads in flight.  The loads are non-temporal: the source streams through once.
// STREAM: the stores are non-temporal too, which keeps the copy from displacing
// the operands of a GEMM running beside it from the 256 MB memory-side cache
// (with ordinary stores an overlapped 16384x8192x1024 GEMM ran 4 % longer);
// without it the destination may stay in that cache for the kernel that reads
// it next (reorder+RMSNorm right behind a copy took 25 us instead of 31).  A
// compile-time choice: as a run-time branch around the two kinds of store the
// compiler merges them into one ordinary store.
template <int WIDTH, bool STREAM>
__device__ __forceinline__ void team_copy(const uint4* __restrict__ s, uint4* __restrict__ d, long long n, int me,
                                          int team, int t) {
    const long long chunk = (long long)WIDTH * kCopyUnroll;
    for (long long base = (long long)me * chunk; base < n; base += (long long)team * chunk) {
        u32x4 v[kCopyUnroll];
#pragma unroll
        for (int u = 0; u < kCopyUnroll; ++u) {
            const long long i = base + u * WIDTH + t;
            if (i < n) v[u] = __builtin_nontemporal_load((const u32x4*)(s + i));
        }
#pragma unroll
        for (int u = 0; u < kCopyUnroll; ++u) {
            const long long i = base + u * WIDTH + t;
            if (i < n) {
                if constexpr (STREAM) __builtin_nontemporal_store(v[u], (u32x4*)(d + i));
                else *(u32x4*)(d + i) = v[u];
            }
        }
    }
}

// The same for the persistent consumer, which runs beside the GEMM and has to live in the 64
// registers that fit beside the GEMM's wavefront on a SIMD: the source is read with agent-scope
// loads that do not hit in the non-coherent caches (another XCD wrote it while this kernel runs),
// four units in flight per thread, source and destination addressed through buffer descriptors
// with 32-bit offsets (n * 16 < 4 GiB) instead of a 64-bit pointer per access.
constexpr int kCoherentUnroll = 4;
template <int WIDTH, bool STREAM>
__device__ __forceinline__ void team_copy_coherent(const uint4* __restrict__ s, uint4* __restrict__ d, unsigned n,
                                                   unsigned me, unsigned team, unsigned t) {
    constexpr unsigned chunk = WIDTH * kCoherentUnroll;
    const __amdgpu_buffer_rsrc_t src = __builtin_amdgcn_make_buffer_rsrc((void*)s, 0, (int)(n * 16u), 0x00020000);
    const __amdgpu_buffer_rsrc_t dst = __builtin_amdgcn_make_buffer_rsrc((void*)d, 0, (int)(n * 16u), 0x00020000);
    for (unsigned base = me * chunk; base < n; base += team * chunk) {
        u32x4 v[kCoherentUnroll];
        // a unit beyond n lies beyond the descriptors: it reads as zero and is not stored
#pragma unroll
        for (int u = 0; u < kCoherentUnroll; ++u)
            v[u] = __builtin_amdgcn_raw_buffer_load_b128(src, (int)((base + u * WIDTH + t) * 16u), 0, 16 | 2);   // sc1 nt
#pragma unroll
        for (int u = 0; u < kCoherentUnroll; ++u)
            __builtin_amdgcn_raw_buffer_store_b128(v[u], dst, (int)((base + u * WIDTH + t) * 16u), 0, STREAM ? 2 : 0);   // nt or not
    }
}

// Persistent form of the host loop in src/overlap_impl.cu:257-265 (and
// :312-323 for the ReduceScatter receive layout).  The members of the kernel
// are its workgroups (four wavefronts each); every member walks the groups in
// index order.  A group is handled by a team of members whose size grows with
// the group (one member per 128 KiB, at most all of them); the teams of
// consecutive groups are consecutive windows of the member list, so many small
// groups are spread over the members and one large group is copied by all of
// them.  A member waits for the group's count, bumps MM[g] once more (the
// member that brings it to cSeg[g] + team is the last to have seen the count
// and stores the 0) and copies its stripe of the range.  With every member on
// every group the groups are released strictly in index order; smaller teams
// release groups as they complete.  A group's range is cut into nslices equal
// parts; parts slice_first .. slice_first+slice_count-1 are copied, part k to
// dst + (k - slice_first)*stride + offset/nslices (the receive layout of a
// ReduceScatter; nslices = 1 is the plain copy).
//
// The kernel uses no LDS and few registers: the GEMM workgroup that runs on the
// same CU owns all of its LDS and most of its registers, and these wavefronts
// have to fit beside it.  Each wavefront finds the member's groups on its own
// (64 groups at a time, one per lane, with wavefront scans for the group
// offsets and the team windows), so the four wavefronts agree without
// exchanging anything.  Only the first wavefront of a member polls; the other
// three wait at a workgroup barrier (which needs no LDS), where they cost the
// SIMDs they share with the GEMM no issue slots and the memory system no
// polls.  Every wavefront polling its own groups, with short naps, cost the
// GEMM beside it 13 % on 4096 groups of 64 KiB; this form costs it 6-7 %.
// The poller naps long (3 us) between two looks at a counter, except on the
// groups at the end of the list, each member's last: there the time to notice
// is no longer hidden behind later groups and adds to the call.  The poller's
// result cannot be handed to the other wavefronts without LDS, so after an
// expired wait the workgroup goes on: it copies the incomplete group (as the
// copy behind an expired wait kernel does) and looks at every later counter
// just once.
// (At most 72 registers: the GEMM's wavefront on the same SIMD takes up to 440 of the 512.  A
// consumer that needs more would, once resident, keep the GEMM's workgroup from being placed on
// its CU, and then wait for that GEMM's signals until its waits expire.)
template <bool STREAM>
__global__ void __launch_bounds__(64 * kWavesPerBlock) __attribute__((amdgpu_waves_per_eu(7, 8))) wait_consume_kernel(
    const int* __restrict__ cseg, int G, int* MM, const uint4* __restrict__ src, uint4* __restrict__ dst,
    long long tile_units, int nslices, int slice_first, int slice_count, long long slice_stride_units,
    int* order_log, long long ticks, int* expired) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int self = (int)blockIdx.x;
    const int members = (int)gridDim.x;
    long long lo_base = 0;  // first 16-byte unit of the chunk's first group
    int start_base = 0;     // first member of that group's team
    for (int g0 = 0; g0 < G; g0 += 64) {
        const int g = g0 + lane;
        const int count = g < G ? cseg[g] : 0;
        const long long units = tile_units * count;
        int team = 0;
        if (g < G) {
            const long long want = (units + kUnitsPerMember - 1) / kUnitsPerMember;
            team = (int)(want < 1 ? 1 : (want > members ? members : want));
        }
        // inclusive scans of units and team sizes over the 64 groups of the chunk
        long long su = units;
        int st = team;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const long long u = __shfl_up(su, off, 64);
            const int t = __shfl_up(st, off, 64);
            if (lane >= off) {
                su += u;
                st += t;
            }
        }
        const long long lo = lo_base + su - units;
        const int start = (int)(((long long)start_base + st - team) % members);
        int me = self - start;   // the team is a window of the member list
        if (me < 0) me += members;
        unsigned long long mine = __ballot(g < G && me < team);
        while (mine) {   // uniform over the workgroup: the groups this member belongs to, in index order
            const int b = __builtin_ctzll(mine);
            mine &= mine - 1;
            const int gg = g0 + b;
            const int tm = __shfl(team, b, 64), mem = __shfl(me, b, 64), need = __shfl(count, b, 64);
            const long long glo = __shfl(lo, b, 64);
            if (wave == 0 && lane == 0) {
                const bool long_naps = gg + members < G;   // not among the last groups of the list
                if (!bounded_poll(MM + gg, ticks, [need](int v) { return v >= need; }, long_naps)) {
                    count_expired(expired);
                    ticks = -1;   // every later poll looks once and gives up
                } else {
                    // Every member has seen the full count once it has bumped it; the last one
                    // to do so puts the counter back.  The copies need not be finished for that:
                    // the next writer of the counter is ordered behind this kernel.
                    bool last = tm == 1;
                    if (!last)
                        last = __hip_atomic_fetch_add(MM + gg, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) ==
                               need + tm - 1;
                    if (last) {
                        __hip_atomic_store(MM + gg, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        if (order_log) order_log[gg] = gg;
                    }
                }
            }
            __builtin_amdgcn_s_barrier();   // the three other wavefronts slept here
            const long long part = tile_units * need / nslices;
            for (int k = 0; k < slice_count; ++k)
                team_copy_coherent<64 * kWavesPerBlock, STREAM>(src + glo + (slice_first + k) * part,
                                                                dst + k * slice_stride_units + glo / nslices,
                                                                (unsigned)part, (unsigned)mem, (unsigned)tm, threadIdx.x);
        }
        lo_base += __shfl(su, 63, 64);
        start_base = (int)(((long long)start_base + __shfl(st, 63, 64)) % members);
    }
}

// blockIdx.y is the slice: slice k of the source lies k * units behind the first, slice k of
// the destination k * dst_stride_units (the receive buffers of a ReduceScatter, side by side).
template <bool STREAM>
__global__ void __launch_bounds__(kCopyThreads) consume_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst,
                                                               long long units, long long dst_stride_units,
                                                               const unsigned short* src_tail, unsigned short* dst_tail,
                                                               int tail, int that, int* addr, int* expired) {
    // Settling a counter whose producer ran earlier on this stream takes no
    // waiting: it holds its final value.  The right value is cleared like
    // wait_kernel does; a wrong one is left and counted like an expired wait.
    if (addr && blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) {
        if (__hip_atomic_load(addr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == that)
            __hip_atomic_store(addr, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        else
            count_expired(expired);
    }
    team_copy<kCopyThreads, STREAM>(src + blockIdx.y * units, dst + blockIdx.y * dst_stride_units, units,
                                           blockIdx.x, gridDim.x, threadIdx.x);
    if (blockIdx.x == 0 && (int)threadIdx.x < tail) dst_tail[threadIdx.x] = src_tail[threadIdx.x];   // one slice only
}

// table[s] = number of inclusive prefix sums of cseg that are <= s, i.e. what
// the linear scan in src/overlap/gemm_with_signal.h:188-193 returns.  One
// workgroup: per-thread run sums, a block scan, then each thread fills the
// slots of its own run of groups.
__global__ void __launch_bounds__(1024) group_table_kernel(const int* __restrict__ cseg, int G, int T, int* table) {
    __shared__ int part[1024];
    const int tid = threadIdx.x;
    const int per = (G + 1023) / 1024;
    const int g0 = tid * per, g1 = min(G, g0 + per);
    int sum = 0;
    for (int g = g0; g < g1; ++g) sum += cseg[g];
    part[tid] = sum;
    __syncthreads();
    for (int off = 1; off < 1024; off <<= 1) {
        const int add = tid >= off ? part[tid - off] : 0;
        __syncthreads();
        part[tid] += add;
        __syncthreads();
    }
    int start = part[tid] - sum;  // exclusive prefix of this thread's run
    for (int g = g0; g < g1; ++g) {
        const int n = cseg[g];
        for (int s = start; s < start + n && s < T; ++s) table[s] = g;
        start += n;
    }
    // Slots beyond sum(cSeg) have no group in the reference (its scan runs off
    // the array); point them at the last group so a lookup stays in bounds.
    const int total = part[1023];
    for (int s = total + tid; s < T; s += 1024) table[s] = G - 1;
}

// Per-device facts the launchers need on every call, looked up once per device.
struct DeviceFacts {
    int wall_khz = 0;   // rate of wall_clock64()
    int cus = 0;
};
static int device_facts(const DeviceFacts** out) {
    static DeviceFacts facts[64];
    static std::atomic<unsigned long long> known{0};
    int dev = 0;
    FO_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= 64) return fail(FO_ERR_LIMIT, "device %d beyond 64", dev);
    const unsigned long long bit = 1ull << dev;
    if (!(known.load(std::memory_order_acquire) & bit)) {
        DeviceFacts f;
        FO_HIP(hipDeviceGetAttribute(&f.wall_khz, hipDeviceAttributeWallClockRate, dev));
        if (f.wall_khz <= 0) f.wall_khz = 100000;  // the constant 100 MHz counter of gfx9
        FO_HIP(hipDeviceGetAttribute(&f.cus, hipDeviceAttributeMultiprocessorCount, dev));
        facts[dev] = f;   // racing threads write the same values
        known.fetch_or(bit, std::memory_order_release);
    }
    *out = &facts[dev];
    return FO_OK;
}

static int ticks_for_timeout(long long* ticks) {
    const DeviceFacts* f;
    if (int e = device_facts(&f)) return e;
    *ticks = (long long)knob(knobs().wait_timeout_ms) * f->wall_khz;
    return FO_OK;
}

int set_wait_timeout_ms(int ms) {
    if (!set_wait_timeout(ms)) return fail(FO_ERR_ARG, "fo_set_wait_timeout_ms: %d ms", ms);
    return FO_OK;
}

int wait_timeouts(int* count, int reset) {
    if (!count) return fail(FO_ERR_ARG, "fo_wait_timeouts: null count");
    FO_HIP(hipDeviceSynchronize());
    FO_HIP(hipMemcpyFromSymbol(count, HIP_SYMBOL(g_wait_timeouts), sizeof(int)));
    if (reset) {
        const int zero = 0;
        FO_HIP(hipMemcpyToSymbol(HIP_SYMBOL(g_wait_timeouts), &zero, sizeof(int)));
    }
    return FO_OK;
}

int launch_wait(int that, int* addr, int* expired, hipStream_t stream) {
    if (!addr) return fail(FO_ERR_ARG, "fo_wait: null counter address");
    long long ticks;
    if (int e = ticks_for_timeout(&ticks)) return e;
    hipLaunchKernelGGL(wait_kernel, dim3(1), dim3(64), 0, stream, that, addr, ticks, expired);
    FO_HIP(hipGetLastError());
    return FO_OK;
}

int launch_wait_consume(const int* cseg, int G, int* MM, const void* src, void* dst, long long tile_elems,
                        int nslices, int slice_first, int slice_count, long long slice_stride, int* order_log,
                        int nblocks, int* expired, hipStream_t stream) {
    if (!cseg || !MM || !src || !dst) return fail(FO_ERR_ARG, "fo_wait_consume: null argument");
    if (G <= 0 || nslices <= 0 || tile_elems <= 0) return fail(FO_ERR_ARG, "fo_wait_consume: G=%d nslices=%d tile_elems=%lld", G, nslices, tile_elems);
    if (nblocks <= 0) return fail(FO_ERR_LIMIT, "fo_wait_consume: nblocks=%d", nblocks);
    if (tile_elems % (8LL * nslices)) return fail(FO_ERR_SHAPE, "fo_wait_consume: a tile (%lld elements) must split into %d slices of whole 16-byte units", tile_elems, nslices);
    if (slice_first < 0 || slice_count <= 0 || slice_first + slice_count > nslices)
        return fail(FO_ERR_ARG, "fo_wait_consume: slices [%d, %d) outside 0..%d", slice_first, slice_first + slice_count, nslices);
    if (slice_count > 1 && slice_stride % 8) return fail(FO_ERR_SHAPE, "fo_wait_consume: slice_stride=%lld not a multiple of 8 elements", slice_stride);
    if (((uintptr_t)src | (uintptr_t)dst) & 15) return fail(FO_ERR_ARG, "fo_wait_consume: buffers must be 16-byte aligned");
    // The workgroups wait while GEMM workgroups still have to be placed: at most one per CU, so that
    // a consumer that is dispatched first can never keep a GEMM workgroup from fitting.
    const DeviceFacts* facts;
    if (int e = device_facts(&facts)) return e;
    if (nblocks > facts->cus)
        return fail(FO_ERR_LIMIT, "fo_wait_consume: nblocks=%d outside 1..%d (one workgroup per CU)", nblocks, facts->cus);
    long long ticks;
    if (int e = ticks_for_timeout(&ticks)) return e;
    auto kern = knob(knobs().copy_streaming_stores) ? wait_consume_kernel<true> : wait_consume_kernel<false>;   // it runs beside the GEMM
    hipLaunchKernelGGL(kern, dim3(nblocks), dim3(64 * kWavesPerBlock), 0, stream, cseg, G, MM, (const uint4*)src,
                       (uint4*)dst, tile_elems / 8, nslices, slice_first, slice_count, slice_stride / 8, order_log, ticks,
                       expired);
    FO_HIP(hipGetLastError());
    return FO_OK;
}

int launch_consume(const void* src, void* dst, size_t bytes, hipStream_t stream, int that, int* addr, int nslices,
                   size_t dst_stride_bytes, int policy, int* expired) {
    const char* who = nslices > 1 ? "fo_consume_slices" : "fo_consume";
    if (nslices <= 0 || nslices > 65535) return fail(FO_ERR_ARG, "%s: %d slices outside 1..65535", who, nslices);
    if (bytes == 0 && !addr) return FO_OK;
    if (!src || !dst) return fail(FO_ERR_ARG, "%s: null buffer", who);
    if (bytes & 1) return fail(FO_ERR_ARG, "%s: %zu bytes is not a whole number of 16-bit elements", who, bytes);
    if (((uintptr_t)src | (uintptr_t)dst) & 15) return fail(FO_ERR_ARG, "%s: buffers must be 16-byte aligned", who);
    if (nslices > 1 && ((bytes | dst_stride_bytes) & 15))
        return fail(FO_ERR_SHAPE, "%s: slices of %zu bytes, %zu apart, are not whole 16-byte units", who, bytes, dst_stride_bytes);
    const size_t units = bytes / 16;
    const int tail = (int)((bytes % 16) / 2);
    const size_t per_block = (size_t)kCopyThreads * kCopyUnroll;
    size_t blocks = (units + per_block - 1) / per_block;
    const size_t most = 1024 / (size_t)(nslices < 1024 ? nslices : 1024);   // about 1024 workgroups over all slices
    if (blocks > most) blocks = most;
    if (blocks == 0) blocks = 1;
    // Store policy.  What matters is how much is copied while a GEMM runs beside the copies: from some
    // tens of MB on, ordinary stores push that GEMM's operands out of the memory-side cache (c4, 201 MB
    // beside the GEMM: it ran 8 % longer; c5, 100 MB: 4 %), below that the reader of the destination
    // gains more from finding it still cached (c3, 33 MB: reorder+RMSNorm 23 us against 31).  A caller
    // that knows the whole call says which it wants; left to itself a launch goes by its own size, and
    // one that settles its own counter follows its GEMM and is read next, so it stores normally.
    if (policy < FO_COPY_AUTO || policy > FO_COPY_CACHED) return fail(FO_ERR_ARG, "%s: store policy %d", who, policy);
    constexpr size_t kStreamFrom = 48u << 20;
    bool stream_stores = policy == FO_COPY_STREAM ||
                         (policy == FO_COPY_AUTO && !addr && bytes * (size_t)nslices >= kStreamFrom);
    if (const int forced = knob(knobs().copy_streaming_stores); forced != 2) stream_stores = forced == 1;   // fo_tune
    auto kern = stream_stores ? consume_kernel<true> : consume_kernel<false>;
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks, (unsigned)nslices), dim3(kCopyThreads), 0, stream, (const uint4*)src,
                       (uint4*)dst, (long long)units, (long long)(dst_stride_bytes / 16),
                       (const unsigned short*)((const char*)src + units * 16),
                       (unsigned short*)((char*)dst + units * 16), tail, that, addr, expired);
    FO_HIP(hipGetLastError());
    return FO_OK;
}

int launch_group_table(const int* cseg, int G, int T, int* table, hipStream_t stream) {
    if (!cseg || !table) return fail(FO_ERR_ARG, "fo_build_group_table: null argument");
    if (G <= 0 || T <= 0) return fail(FO_ERR_ARG, "fo_build_group_table: G=%d T=%d", G, T);
    hipLaunchKernelGGL(group_table_kernel, dim3(1), dim3(1024), 0, stream, cseg, G, T, table);
    FO_HIP(hipGetLastError());
    return FO_OK;
}

}  // namespace fo
