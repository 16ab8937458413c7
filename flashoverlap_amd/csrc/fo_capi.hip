// extern "C" surface of libfo_hip.so (declared in include/flashoverlap_hip.h):
// argument marshalling only; the kernels and their launchers live in
// fo_gemm.hip, fo_sync.hip and fo_rmsnorm.hip.
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>

#include "fo_internal.h"

namespace fo {

static thread_local char t_error[512] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(t_error, sizeof t_error, fmt, ap);
    va_end(ap);
    return code;
}

// Layout tile selected by each Algo index, in the order of the reference's
// instance list (src/inc/signal_instances.inc:1-6).  The third number is the
// reference's k-tile; this library always stages 64 k-elements per LDS buffer,
// so entries that differ only in it select the same kernel.
static const int kAlgo[][3] = {
    {128, 128, 32}, {128, 128, 64}, {128, 256, 32}, {128, 256, 64}, {256, 128, 32}, {256, 128, 64},
};
constexpr int kAlgoCount = sizeof(kAlgo) / sizeof(kAlgo[0]);

thread_local LaunchTimer t_launch_timer;

int algo_tile(int algo, int* BM, int* BN, int* BK) {
    if (algo < 0 || algo >= kAlgoCount) return FO_ERR_ARG;
    *BM = kAlgo[algo][0];
    *BN = kAlgo[algo][1];
    *BK = kAlgo[algo][2];
    return FO_OK;
}

}  // namespace fo

using namespace fo;

extern "C" {

int fo_version(void) { return 100; }

const char* fo_last_error(void) { return t_error; }

int fo_algo_count(void) { return kAlgoCount; }

int fo_algo_tile(int algo, int* BM, int* BN, int* BK) {
    if (!BM || !BN || !BK) return fail(FO_ERR_ARG, "fo_algo_tile: null output");
    if (algo_tile(algo, BM, BN, BK) != FO_OK) return fail(FO_ERR_ARG, "fo_algo_tile: Algo %d out of range 0..%d", algo, kAlgoCount - 1);
    return FO_OK;
}

int fo_device_info(int* cu_count, int* clock_khz, int* xcd_count) {
    int dev = 0;
    FO_HIP(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    FO_HIP(hipGetDeviceProperties(&prop, dev));
    if (cu_count) *cu_count = prop.multiProcessorCount;
    if (clock_khz) *clock_khz = prop.clockRate;
    if (xcd_count) *xcd_count = 8;  // MI355X: 8 accelerator dies, 32 CUs each
    return FO_OK;
}

int fo_gemm(int dtype, int algo, int M, int N, int K, const void* A, const void* B, void* D, void* stream) {
    return launch_gemm(0, dtype, algo, M, N, K, 1, nullptr, 0, nullptr, A, B, D, nullptr, nullptr, nullptr, 0,
                       (hipStream_t)stream);
}

int fo_gemm_signal(int dtype, int algo, int M, int N, int K, int rLDN, const int* cseg_dev, int G,
                   const int* group_table, const void* A, const void* B, void* D, int* MM, const int* RA,
                   int monitor, void* stream) {
    return launch_gemm(1, dtype, algo, M, N, K, rLDN, cseg_dev, G, group_table, A, B, D, MM, RA, nullptr, monitor,
                       (hipStream_t)stream);
}

int fo_gemm_scatter(int dtype, int algo, int M, int N, int K, int rLDN, const int* cseg_dev, int G,
                    const int* group_table, const void* A, const void* B, void* D, int* MM, const int* RA,
                    const int* RE, int monitor, void* stream) {
    return launch_gemm(2, dtype, algo, M, N, K, rLDN, cseg_dev, G, group_table, A, B, D, MM, RA, RE, monitor,
                       (hipStream_t)stream);
}

int fo_gemm_signal_static(int dtype, int algo, int M, int N, int K, int rLDN, const int* cseg_dev, int G,
                          const void* A, const void* B, void* D, int* MM, const int* RA, int monitor, void* stream) {
    return gemm_signal_static(dtype, algo, M, N, K, rLDN, cseg_dev, G, A, B, D, MM, RA, monitor, (hipStream_t)stream);
}

int fo_build_group_table(const int* cseg_dev, int G, int T, int* group_table, void* stream) {
    return launch_group_table(cseg_dev, G, T, group_table, (hipStream_t)stream);
}

int fo_raster_hint(int algo, int M, int N, int* hint_host) { return raster_hint(algo, M, N, hint_host); }

int fo_tune(const char* key, int value) { return tune(key, value); }

int fo_wait(int that, int* addr, int* expired, void* stream) {
    return launch_wait(that, addr, expired, (hipStream_t)stream);
}

int fo_wait_consume(const int* cseg_dev, int G, int* MM, const void* src, void* dst, long long tile_elems,
                    int nslices, int slice_first, int slice_count, long long slice_stride, int* order_log,
                    int nblocks, int* expired, void* stream) {
    return launch_wait_consume(cseg_dev, G, MM, src, dst, tile_elems, nslices, slice_first, slice_count,
                               slice_stride, order_log, nblocks, expired, (hipStream_t)stream);
}

int fo_set_wait_timeout_ms(int ms) { return set_wait_timeout_ms(ms); }

int fo_wait_timeouts(int* count, int reset) { return wait_timeouts(count, reset); }

int fo_consume(const void* src, void* dst, size_t bytes, void* stream) {
    return launch_consume(src, dst, bytes, (hipStream_t)stream);
}

int fo_settle_consume(int that, int* addr, const void* src, void* dst, size_t bytes, int* expired, void* stream) {
    if (!addr) return fail(FO_ERR_ARG, "fo_settle_consume: null counter address");
    return launch_consume(src, dst, bytes, (hipStream_t)stream, that, addr, 1, 0, FO_COPY_AUTO, expired);
}

int fo_consume_slices(int that, int* addr, const void* src, void* dst, size_t slice_bytes, int nslices,
                      size_t dst_stride_bytes, int store_policy, int* expired, void* stream) {
    return launch_consume(src, dst, slice_bytes, (hipStream_t)stream, that, addr, nslices, dst_stride_bytes,
                          store_policy, expired);
}

int fo_reorder_rmsnorm(int dtype, const void* x, const void* gamma, void* out, int bs, int dim, int BM, int BN,
                       int rldn, const int* RA, float eps, void* stream) {
    if (!RA) return fail(FO_ERR_ARG, "fo_reorder_rmsnorm: null RA");
    return launch_rmsnorm(dtype, x, gamma, out, 1, bs, dim, BM, BN, rldn, RA, eps, (hipStream_t)stream);
}

int fo_reorder_rmsnorm_batched(int dtype, const void* x, const void* gamma, void* out, int nbatch, int bs, int dim,
                               int BM, int BN, int rldn, const int* RA, float eps, void* stream) {
    if (!RA) return fail(FO_ERR_ARG, "fo_reorder_rmsnorm_batched: null RA");
    return launch_rmsnorm(dtype, x, gamma, out, nbatch, bs, dim, BM, BN, rldn, RA, eps, (hipStream_t)stream);
}

int fo_rmsnorm(int dtype, const void* x, const void* gamma, void* out, int bs, int dim, float eps, void* stream) {
    return launch_rmsnorm(dtype, x, gamma, out, 1, bs, dim, 0, 0, 0, nullptr, eps, (hipStream_t)stream);
}

int fo_stream_create(void** stream) {
    if (!stream) return fail(FO_ERR_ARG, "fo_stream_create: null output");
    hipStream_t s;
    FO_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    *stream = (void*)s;
    return FO_OK;
}

int fo_stream_destroy(void* stream) {
    if (stream) FO_HIP(hipStreamDestroy((hipStream_t)stream));
    return FO_OK;
}

int fo_stream_sync(void* stream) {
    FO_HIP(hipStreamSynchronize((hipStream_t)stream));
    return FO_OK;
}

// Creating and destroying an event costs the host some 20 us a time, more than
// the rest of a join: every thread keeps a few events per device and takes
// them in turn.  A wait refers to the record that preceded it, so recording an
// event again later does not disturb waits already enqueued on it.
namespace {
constexpr int kMaxDevices = 16, kEventsPerDevice = 4;
struct JoinEvents {
    hipEvent_t ev[kMaxDevices][kEventsPerDevice] = {};
    unsigned next[kMaxDevices] = {};
    // never destroyed: a thread may end after the runtime has shut down
};
thread_local JoinEvents t_join_events;
}  // namespace

int fo_stream_join(void* signaller, void* waiter) {
    int dev = 0;
    FO_HIP(hipGetDevice(&dev));
    hipEvent_t ev;
    const bool pooled = dev >= 0 && dev < kMaxDevices;
    if (pooled) {
        hipEvent_t& slot = t_join_events.ev[dev][t_join_events.next[dev]++ % kEventsPerDevice];
        if (!slot) FO_HIP(hipEventCreateWithFlags(&slot, hipEventDisableTiming));
        ev = slot;
    } else {
        FO_HIP(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
    }
    hipError_t e = hipEventRecord(ev, (hipStream_t)signaller);
    if (e == hipSuccess) e = hipStreamWaitEvent((hipStream_t)waiter, ev, 0);
    if (!pooled) {
        hipError_t d = hipEventDestroy(ev);
        FO_HIP(e);
        FO_HIP(d);
        return FO_OK;
    }
    FO_HIP(e);
    return FO_OK;
}

int fo_time_next_launch(void* start_event, void* stop_event) {
    if (!start_event != !stop_event) return fail(FO_ERR_ARG, "fo_time_next_launch: pass both events or neither");
    t_launch_timer.start = (hipEvent_t)start_event;
    t_launch_timer.stop = (hipEvent_t)stop_event;
    return FO_OK;
}

int fo_stream_is_capturing(void* stream, int* capturing) {
    if (!capturing) return fail(FO_ERR_ARG, "fo_stream_is_capturing: null output");
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    FO_HIP(hipStreamIsCapturing((hipStream_t)stream, &status));
    *capturing = status == hipStreamCaptureStatusActive;
    return FO_OK;
}

int fo_event_create(void** ev) {
    if (!ev) return fail(FO_ERR_ARG, "fo_event_create: null output");
    hipEvent_t e;
    FO_HIP(hipEventCreate(&e));
    *ev = (void*)e;
    return FO_OK;
}

int fo_event_destroy(void* ev) {
    if (ev) FO_HIP(hipEventDestroy((hipEvent_t)ev));
    return FO_OK;
}

int fo_event_record(void* ev, void* stream) {
    FO_HIP(hipEventRecord((hipEvent_t)ev, (hipStream_t)stream));
    return FO_OK;
}

int fo_event_sync(void* ev) {
    FO_HIP(hipEventSynchronize((hipEvent_t)ev));
    return FO_OK;
}

int fo_event_elapsed_ms(void* start, void* stop, float* ms) {
    if (!ms) return fail(FO_ERR_ARG, "fo_event_elapsed_ms: null output");
    FO_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return FO_OK;
}

}  // extern "C"
