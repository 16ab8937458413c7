// Internal declarations shared by the translation units of libfo_hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/flashoverlap_hip.h"

namespace fo {

// Records the message returned by fo_last_error() and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

#define FO_HIP(expr)                                                                        \
    do {                                                                                    \
        hipError_t fo_e_ = (expr);                                                          \
        if (fo_e_ != hipSuccess)                                                            \
            return ::fo::fail(FO_ERR_HIP, "%s failed: %s (%s:%d)", #expr, hipGetErrorString(fo_e_), \
                              __FILE__, __LINE__);                                          \
    } while (0)

int algo_tile(int algo, int* BM, int* BN, int* BK);

// fo_time_next_launch: a pair of events that the next GEMM or RMSNorm launch of this thread
// attaches to its own dispatch, so that the time between them is the kernel's, without the
// launch gaps an event pair recorded around the launch includes.  Taken by the launch that uses it.
struct LaunchTimer {
    hipEvent_t start = nullptr, stop = nullptr;
};
extern thread_local LaunchTimer t_launch_timer;

// fo_gemm.hip
int choose_macro_tile(int BM, int BN, int M, int N, bool any_shape);
int launch_gemm(int mode, int dtype, int algo, int M, int N, int K, int rLDN, const int* cseg, int G,
                const int* gtable, const void* A, const void* B, void* D, int* MM, const int* RA,
                const int* RE, int monitor, hipStream_t stream);
int raster_hint(int algo, int M, int N, int* hint);
int tune(const char* key, int value);

// fo_static.hip
int gemm_signal_static(int dtype, int algo, int M, int N, int K, int rLDN, const int* cseg, int G, const void* A,
                       const void* B, void* D, int* MM, const int* RA, int monitor, hipStream_t stream);

// fo_sync.hip
int launch_group_table(const int* cseg, int G, int T, int* table, hipStream_t stream);
int launch_wait(int that, int* addr, int* expired, hipStream_t stream);
int launch_wait_consume(const int* cseg, int G, int* MM, const void* src, void* dst, long long tile_elems,
                        int nslices, int slice_first, int slice_count, long long slice_stride, int* order_log,
                        int nblocks, int* expired, hipStream_t stream);
int launch_consume(const void* src, void* dst, size_t bytes, hipStream_t stream, int that = 0, int* addr = nullptr,
                   int nslices = 1, size_t dst_stride_bytes = 0, int policy = FO_COPY_AUTO, int* expired = nullptr);
int set_wait_timeout_ms(int ms);
int wait_timeouts(int* count, int reset);

// fo_rmsnorm.hip
int launch_rmsnorm(int dtype, const void* x, const void* gamma, void* out, int nbatch, int bs, int dim, int BM,
                   int BN, int rldn, const int* RA, float eps, hipStream_t stream);

}  // namespace fo
