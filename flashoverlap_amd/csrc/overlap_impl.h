// OverlapImpl: host orchestration of the overlapped GEMM + per-group consumer,
// with the method set of the reference class (src/overlap_impl.h:9-40) so that
// torch.classes.flashoverlap_class.OverlapImpl is a drop-in on one MI355X.
//
// The device is reached only through the C ABI in flashoverlap_hip.h; torch is
// used for tensor plumbing (pointers, dtype, the caller's current stream) and
// for the two device buffers this object owns (the staging buffer that stands
// in for the collective's destination, and the slot->group table).
#pragma once

#include <ATen/ATen.h>
#include <torch/custom_class.h>

#include <cstdint>
#include <vector>

class OverlapImpl : public torch::CustomClassHolder {
  public:
    OverlapImpl();
    ~OverlapImpl() override;

    // src/overlap_impl.cu:38-40, 57-70, 146-148
    void MutlassInit();
    void McclInit(int64_t tp_rank, int64_t tp_size, std::vector<int64_t> tp_id);
    void OverlapInit();

    // src/overlap_impl.cu:42-55
    void Gemm(at::Tensor A, at::Tensor B, at::Tensor C, int64_t Algo);

    // src/overlap_impl.cu:221-271, 273-328
    void GemmAllReduceOverlap(at::Tensor A, at::Tensor B, at::Tensor C, at::Tensor MM, at::Tensor RA, int64_t rLDN,
                              at::Tensor cSEG_CPU, at::Tensor cSEG_GPU, int64_t Algo, bool if_monitor);
    void GemmReduceScatterOverlap(at::Tensor A, at::Tensor B, at::Tensor C, at::Tensor D, at::Tensor MM,
                                  at::Tensor RA, at::Tensor RE, int64_t rLDN, at::Tensor cSEG_CPU,
                                  at::Tensor cSEG_GPU, int64_t Algo, bool if_monitor);

    // src/overlap_impl.cu:72-144 (GEMM followed by one bulk collective, no overlap)
    void GemmAllReduce(at::Tensor A, at::Tensor B, at::Tensor C, int64_t Algo);
    void GemmReduceScatter(at::Tensor A, at::Tensor B, at::Tensor C, at::Tensor D, int64_t Algo);
    void GemmAll2All(at::Tensor A, at::Tensor B, at::Tensor C, at::Tensor D, int64_t Algo, at::Tensor mLen_CPU);

    // src/overlap_impl.cu:150-219
    void SegAllReduce(at::Tensor C, at::Tensor cSEG_CPU, int64_t SegNum);
    void McclAllReduce(at::Tensor C);
    void McclReduceScatter(at::Tensor C);
    void McclAll2All(at::Tensor C, at::Tensor D, at::Tensor mLen_CPU);

    // ---- additions (no counterpart in the reference) ----
    // Destination of the AllReduce stand-in: a flat buffer of the size of the
    // last C passed to an all-reduce style call.
    at::Tensor Staging() const;
    // Makes `buffer` (M*N elements of C's dtype) the destination of the next
    // all-reduce style calls instead of the internally allocated one, so that a
    // caller can own its result like it owns C in the reference.  A call whose C
    // does not match the buffer in size, dtype or device goes back to an internal one.
    void SetStaging(at::Tensor buffer);
    // 0 = automatic (per-group launches up to 32 groups, one persistent kernel
    // beyond), 1 = one (wait, consume) launch pair per group like the
    // reference's host loop, 2 = one persistent wait+consume kernel.
    void SetConsumerMode(int64_t mode);
    // Workgroups of the persistent consumer (default and maximum: one per CU).
    void SetConsumerBlocks(int64_t blocks);
    // The waits on the group counters are bounded (the reference's spin forever,
    // src/wait.cuh:6-8).  set_wait_timeout_ms sets the bound (process-wide, default
    // 10 s).  Expired waits are counted in a device word that this object owns, so
    // one object never sees, or is blamed for, another object's expiries:
    // wait_timeouts(reset) waits for this object's streams and returns how many of
    // its waits have expired; set_check_timeouts(true) makes every overlapped call
    // wait for its own completion and raise if one of its waits expired (debugging:
    // it serialises the caller, and it cannot be combined with graph capture, which
    // forbids that wait).  After an expiry MM must be zeroed before reuse.
    void SetWaitTimeoutMs(int64_t ms);
    int64_t WaitTimeouts(bool reset);
    void SetCheckTimeouts(bool on);

  private:
    void* gemm_stream_ = nullptr;
    void* comm_stream_ = nullptr;
    bool gemm_ready_ = false;
    int64_t my_rank_ = 0;
    int64_t my_size_ = 1;
    int64_t consumer_mode_ = 0;
    int64_t consumer_blocks_ = 0;   // 0: not chosen yet (one per CU at first use)
    bool check_timeouts_ = false;

    at::Tensor staging_;
    at::Tensor expired_;          // one int32 on the device: expired waits of this object's calls
    at::Tensor group_table_;
    std::vector<int> table_key_;  // cSeg contents + T the table was built for

    void require_gemm() const;
    void require_overlap() const;
    at::Tensor& staging_like(const at::Tensor& C);
    const int* group_table_for(const at::Tensor& cseg_cpu, const at::Tensor& cseg_gpu, int T);
    void fork_comm_stream(int G);
    void consume_groups(const at::Tensor& C, void* dst, int64_t tile_elems, const at::Tensor& cseg_cpu,
                        const at::Tensor& cseg_gpu, at::Tensor& MM, int nslices, int64_t slice_stride);
    void bulk_consume(const void* src, void* dst, size_t bytes);
    int* expired_word(const at::Tensor& like);
    void refuse_checked_capture(const char* who);
    void prepare_call(const at::Tensor& MM, const char* who);
    void raise_on_timeout(at::Tensor& MM, const char* who);
    int consumer_blocks();
};
