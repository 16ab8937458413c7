// fo_gemm_signal_static: the signalling GEMM for callers that cannot allocate
// device memory (code under HIP graph capture, tight serving loops).  It is
// fo_gemm_signal with the slot->group table - the one workspace that entry
// point takes from its caller - kept in a file-scope device array instead.
//
// Each GPU the library runs on holds its own copy of the array, at its own
// address, until the process ends.  The array's name is only a host-side
// handle: the address a kernel can use is looked up once per device with
// hipGetSymbolAddress and every launch below passes that pointer.  Every call
// on a device rewrites slots [0, T) of that device's array before its GEMM
// reads them, on the caller's stream, so nothing has to be cleared between
// calls; two calls whose kernels can overlap on one device (different streams)
// race on the array and must not be issued.
#include <hip/hip_runtime.h>

#include <mutex>

#include "fo_internal.h"

namespace fo {

constexpr int kStaticSlots = FO_STATIC_MAX_TILES;  // 65536 tiles: 256 KiB per device

static __device__ __align__(256) int scratch[kStaticSlots];

constexpr int kMaxDevices = 64;
static int* g_scratch_ptr[kMaxDevices];   // device address of `scratch`, per device
static std::mutex g_scratch_mutex;

// Device address of this device's copy of the array (resolved on first use).
static int scratch_for_current_device(int** out) {
    int dev = 0;
    FO_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return fail(FO_ERR_LIMIT, "fo_gemm_signal_static: device %d beyond %d", dev, kMaxDevices);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        int* p = nullptr;
        FO_HIP(hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch)));
        if (!p) return fail(FO_ERR_HIP, "fo_gemm_signal_static: no device address for the static table");
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return FO_OK;
}

int gemm_signal_static(int dtype, int algo, int M, int N, int K, int rLDN, const int* cseg, int G, const void* A,
                       const void* B, void* D, int* MM, const int* RA, int monitor, hipStream_t stream) {
    // an event pair armed by fo_time_next_launch is this call's, also if the call is rejected below
    const LaunchTimer timer = t_launch_timer;
    t_launch_timer = LaunchTimer{};
    int BM, BN, BK;
    if (algo_tile(algo, &BM, &BN, &BK) != FO_OK) return fail(FO_ERR_ARG, "fo_gemm_signal_static: Algo %d out of range", algo);
    if (M <= 0 || N <= 0 || M % BM || N % BN)
        return fail(FO_ERR_SHAPE, "fo_gemm_signal_static: M=%d N=%d vs tile %dx%d", M, N, BM, BN);
    if (!cseg || G <= 0) return fail(FO_ERR_ARG, "fo_gemm_signal_static: null cSeg or G=%d", G);
    const long long T = (long long)(M / BM) * (N / BN);
    if (T > kStaticSlots)
        return fail(FO_ERR_LIMIT, "fo_gemm_signal_static: %lld tiles exceed the static table of %d; use fo_gemm_signal with a caller-owned table",
                    T, kStaticSlots);
    int* table = nullptr;
    if (int e = scratch_for_current_device(&table)) return e;
    if (int e = launch_group_table(cseg, G, (int)T, table, stream)) return e;
    t_launch_timer = timer;   // for the GEMM's own dispatch
    return launch_gemm(1, dtype, algo, M, N, K, rLDN, cseg, G, table, A, B, D, MM, RA, nullptr, monitor, stream);
}

}  // namespace fo
