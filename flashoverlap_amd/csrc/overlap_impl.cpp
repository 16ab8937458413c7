// Host orchestration of the overlapped path on one MI355X.  Follows the call
// structure of the reference's src/overlap_impl.cu (GEMM on the caller's
// stream, a per-group wait -> collective loop on a second stream, an event
// join back), with the collective replaced by a consumer copy into a staging
// buffer and every failure reported through TORCH_CHECK instead of exit().
#include "overlap_impl.h"

#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>

#include "host_common.h"

// Copies made while the GEMM runs use non-temporal stores once a call makes this many bytes
// of them: c3 (33 MB) is 1.5 % faster with ordinary stores, c5 (100 MB) 2.5 % and c4 (201 MB)
// 4-8 % faster with non-temporal ones.
static constexpr size_t kStreamCopiesFrom = 64u << 20;

OverlapImpl::OverlapImpl() = default;

OverlapImpl::~OverlapImpl() {
    if (comm_stream_) fo_stream_destroy(comm_stream_);
}

void OverlapImpl::MutlassInit() {
    // Like the reference, the stream that is current now is used for every
    // later GEMM of this object (src/overlap_impl.cu:38-40).
    gemm_stream_ = (void*)c10::hip::getCurrentHIPStream().stream();
    gemm_ready_ = true;
}

void OverlapImpl::McclInit(int64_t tp_rank, int64_t tp_size, std::vector<int64_t> tp_id) {
    TORCH_CHECK(tp_size >= 1 && tp_rank >= 0 && tp_rank < tp_size, "mccl_init: rank ", tp_rank, " of ", tp_size);
    TORCH_CHECK(tp_id.size() == 16, "mccl_init: the id must have 16 entries, got ", tp_id.size());
    // One GPU: no communicator is created (the reference also skips it for
    // size 1, src/overlap_impl.cu:65-68).  A size above 1 only selects the
    // ReduceScatter slicing that a rank of that world would see.
    my_rank_ = tp_rank;
    my_size_ = tp_size;
}

void OverlapImpl::OverlapInit() {
    if (!comm_stream_) FO_CALL(fo_stream_create(&comm_stream_));
}

void OverlapImpl::SetConsumerMode(int64_t mode) {
    TORCH_CHECK(mode >= 0 && mode <= 2, "set_consumer_mode: 0 (auto), 1 (per group) or 2 (persistent), got ", mode);
    consumer_mode_ = mode;
}

void OverlapImpl::SetConsumerBlocks(int64_t blocks) {
    int cus = 0;
    FO_CALL(fo_device_info(&cus, nullptr, nullptr));
    // The persistent consumer's workgroups wait beside the GEMM's: at most one per CU.
    TORCH_CHECK(blocks >= 1 && blocks <= cus, "set_consumer_blocks: 1..", cus, " (one workgroup per CU), got ", blocks);
    consumer_blocks_ = blocks;
}

int OverlapImpl::consumer_blocks() {
    if (consumer_blocks_ == 0) {   // default: one workgroup per CU
        int cus = 0;
        FO_CALL(fo_device_info(&cus, nullptr, nullptr));
        consumer_blocks_ = cus;
    }
    return (int)consumer_blocks_;
}

void OverlapImpl::SetWaitTimeoutMs(int64_t ms) {
    TORCH_CHECK(ms >= 1 && ms <= 3600 * 1000, "set_wait_timeout_ms: 1..3600000, got ", ms);
    FO_CALL(fo_set_wait_timeout_ms((int)ms));
}

// The word this object's waits count their expiries in (one int32 on the device of `like`).
int* OverlapImpl::expired_word(const at::Tensor& like) {
    if (!expired_.defined() || expired_.device() != like.device()) {
        expired_ = at::zeros({1}, like.options().dtype(at::kInt));
        // once per object: the fill runs on torch's current stream, the waits on another one
        c10::hip::getCurrentHIPStream().synchronize();
    }
    return expired_.data_ptr<int>();
}

int64_t OverlapImpl::WaitTimeouts(bool reset) {
    if (!expired_.defined()) return 0;   // no overlapped call has run yet
    c10::DeviceGuard guard(expired_.device());
    if (comm_stream_) FO_CALL(fo_stream_sync(comm_stream_));
    if (gemm_ready_) FO_CALL(fo_stream_sync(gemm_stream_));
    const int64_t n = expired_.item<int>();
    if (reset && n) expired_.zero_();
    return n;
}

void OverlapImpl::SetCheckTimeouts(bool on) { check_timeouts_ = on; }

// Checked mode: wait for the call to finish and turn an expired wait into an
// error.  The counters then hold partial counts, which would make every later
// wait on them expire too (or pass at once), so they are cleared here.
void OverlapImpl::raise_on_timeout(at::Tensor& MM, const char* who) {
    if (!check_timeouts_) return;
    FO_CALL(fo_stream_sync(gemm_stream_));   // the call's join has ordered it behind the second stream
    const int n = expired_.item<int>();
    if (n == 0) return;
    expired_.zero_();
    MM.zero_();
    TORCH_CHECK(false, who, ": ", n, " bounded wait(s) expired before their group completed; the consumer's output "
                "is incomplete and MM has been zeroed (a cSeg that does not match the tiles, or a GEMM slower than the "
                "wait timeout)");
}

at::Tensor OverlapImpl::Staging() const {
    TORCH_CHECK(staging_.defined(), "staging: no all-reduce style call has run yet");
    return staging_;
}

void OverlapImpl::SetStaging(at::Tensor buffer) {
    TORCH_CHECK(buffer.defined() && buffer.is_cuda() && buffer.is_contiguous(),
                "set_staging: the buffer must be a contiguous GPU tensor");
    TORCH_CHECK(buffer.scalar_type() == at::kHalf || buffer.scalar_type() == at::kBFloat16,
                "set_staging: the buffer must be float16 or bfloat16, got ", buffer.scalar_type());
    staging_ = buffer.view({buffer.numel()});
}

void OverlapImpl::require_gemm() const {
    TORCH_CHECK(gemm_ready_, "OverlapImpl: call mutlass_init() first");
}

void OverlapImpl::require_overlap() const {
    require_gemm();
    TORCH_CHECK(comm_stream_ != nullptr, "OverlapImpl: call overlap_init() first");
}

at::Tensor& OverlapImpl::staging_like(const at::Tensor& C) {
    if (!staging_.defined() || staging_.numel() != C.numel() || staging_.scalar_type() != C.scalar_type() ||
        staging_.device() != C.device())
        staging_ = at::empty({C.numel()}, C.options());
    return staging_;
}

const int* OverlapImpl::group_table_for(const at::Tensor& cseg_cpu, const at::Tensor& cseg_gpu, int T) {
    const int G = (int)cseg_cpu.numel();
    const int* host = cseg_cpu.data_ptr<int>();
    std::vector<int> key(host, host + G);
    key.push_back(T);
    const bool same_device = group_table_.defined() && group_table_.device() == cseg_gpu.device();
    if (!same_device || key != table_key_) {
        group_table_ = at::empty({T}, cseg_gpu.options());
        FO_CALL(fo_build_group_table(cseg_gpu.data_ptr<int>(), G, T, group_table_.data_ptr<int>(), gemm_stream_));
        table_key_ = std::move(key);
    }
    return group_table_.data_ptr<int>();
}

void OverlapImpl::bulk_consume(const void* src, void* dst, size_t bytes) {
    FO_CALL(fo_consume(src, dst, bytes, gemm_stream_));
}

void OverlapImpl::Gemm(at::Tensor A, at::Tensor B, at::Tensor C, int64_t Algo) {
    require_gemm();
    const fo_host::GemmShape s = fo_host::check_gemm(A, B, C, "mutlass_gemm");
    c10::DeviceGuard guard(A.device());
    FO_CALL(fo_gemm(s.dtype, (int)Algo, s.M, s.N, s.K, A.data_ptr(), B.data_ptr(), C.data_ptr(), gemm_stream_));
}

// Called before the GEMM is enqueued.  While the caller's stream is being captured into a
// graph, the communication stream's part of the call is first ordered behind the caller's
// stream (not behind the GEMM, which comes later): the capture then follows the work onto the
// second stream, and with the join at the end the call is a closed fork/join pattern of
// kernels.  Outside a capture the fork is left out, as in the reference: the event it puts in
// front of the GEMM costs 5-9 us of every call.
// Ahead of the GEMM launch of an overlapped call: the word its waits count their expiries in
// exists (creating it waits for the stream once per object, which must not happen between the
// GEMM and its waiters), and checked mode is not combined with a capture.
void OverlapImpl::prepare_call(const at::Tensor& MM, const char* who) {
    refuse_checked_capture(who);
    expired_word(MM);
}

// Checked mode ends every call with a wait for the stream, which a capture forbids (it would
// invalidate the capture and leave the caller with an unrelated error).
void OverlapImpl::refuse_checked_capture(const char* who) {
    if (!check_timeouts_) return;
    int capturing = 0;
    FO_CALL(fo_stream_is_capturing(gemm_stream_, &capturing));
    TORCH_CHECK(!capturing, who, ": set_check_timeouts(true) makes the call wait for its own completion, which is not "
                "allowed while the stream is being captured into a graph; turn it off for captured calls and read "
                "wait_timeouts() after a replay instead");
}

void OverlapImpl::fork_comm_stream(int G) {
    const bool persistent = consumer_mode_ == 2 || (consumer_mode_ == 0 && G > 32);
    if (!persistent && G <= 1) return;   // the second stream is not used
    int capturing = 0;
    FO_CALL(fo_stream_is_capturing(gemm_stream_, &capturing));
    if (capturing) FO_CALL(fo_stream_join(gemm_stream_, comm_stream_));
}

// Per-group release: either the reference's host loop (one wait kernel and one
// consumer launch per group, src/overlap_impl.cu:257-265 / 312-323) or one
// persistent kernel that does the same walk on the device.  On return the GEMM
// stream is ordered behind every group's copy.
void OverlapImpl::consume_groups(const at::Tensor& C, void* dst, int64_t tile_elems, const at::Tensor& cseg_cpu,
                                 const at::Tensor& cseg_gpu, at::Tensor& MM, int nslices, int64_t slice_stride) {
    const int G = (int)cseg_cpu.numel();
    const int* cseg = cseg_cpu.data_ptr<int>();
    const int slice_first = slice_stride ? 0 : (int)my_rank_;      // stride 0: only this rank's slice
    const int slice_count = slice_stride ? nslices : 1;
    const bool persistent = consumer_mode_ == 2 || (consumer_mode_ == 0 && G > 32);
    int* expired = expired_.data_ptr<int>();   // this object's own count of expired waits (prepare_call)
    if (persistent) {
        FO_CALL(fo_wait_consume(cseg_gpu.data_ptr<int>(), G, MM.data_ptr<int>(), C.data_ptr(), dst, tile_elems,
                                nslices, slice_first, slice_count, slice_stride, nullptr, consumer_blocks(),
                                expired, comm_stream_));
        // The caller's stream continues only after the last group is consumed
        // (src/overlap_impl.cu:267-270).
        FO_CALL(fo_stream_join(comm_stream_, gemm_stream_));
        return;
    }
    const size_t esz = C.element_size();
    const char* src = (const char*)C.data_ptr();
    // The groups before the last are copied while the GEMM runs: if that is a lot of data,
    // with stores that leave the GEMM's operands in the memory-side cache.
    int64_t beside = 0;
    for (int g = 0; g + 1 < G; ++g) beside += tile_elems * cseg[g] / nslices * slice_count * (int64_t)esz;
    const int beside_policy = beside >= (int64_t)kStreamCopiesFrom ? FO_COPY_STREAM : FO_COPY_CACHED;
    int64_t acc = 0;
    for (int g = 0; g < G; ++g) {
        // The last group completes with the GEMM, so nothing is left for it to overlap with:
        // it is released on the GEMM's own stream, where stream order stands in for the wait
        // kernel (the counter is settled by the copy launch itself), and the groups before it,
        // finished long ago on the communication stream, are joined behind it.  A last group
        // on the communication stream would instead put a fresh cross-stream dependency
        // (10-20 us on this platform) between its copy and the caller's next kernel.
        const bool last = g == G - 1;
        void* stream = last ? gemm_stream_ : comm_stream_;
        const int64_t comm = tile_elems * cseg[g];
        if (!last) FO_CALL(fo_wait(cseg[g], MM.data_ptr<int>() + g, expired, stream));
        // One launch per group, like the one collective call per group of the reference: this
        // rank's slice of the group, or all ranks' slices into their receive buffers side by side.
        const int64_t part = comm / nslices;
        FO_CALL(fo_consume_slices(cseg[g], last ? MM.data_ptr<int>() + g : nullptr,
                                  src + (acc + slice_first * part) * esz, (char*)dst + (acc / nslices) * esz,
                                  part * esz, slice_count, slice_stride * esz,
                                  last ? FO_COPY_CACHED : beside_policy, expired, stream));
        acc += comm;
    }
    // The caller's stream continues only after every group is consumed (src/overlap_impl.cu:267-270).
    if (G > 1) FO_CALL(fo_stream_join(comm_stream_, gemm_stream_));
}

void OverlapImpl::GemmAllReduceOverlap(at::Tensor A, at::Tensor B, at::Tensor C, at::Tensor MM, at::Tensor RA,
                                       int64_t rLDN, at::Tensor cSEG_CPU, at::Tensor cSEG_GPU, int64_t Algo,
                                       bool if_monitor) {
    require_overlap();
    const fo_host::GemmShape s = fo_host::check_gemm(A, B, C, "gemm_allreduce_overlap");
    const fo_host::SignalShape g =
        fo_host::check_signal(s, MM, RA, at::Tensor(), rLDN, cSEG_CPU, cSEG_GPU, (int)Algo, if_monitor, 1,
                              "gemm_allreduce_overlap");
    c10::DeviceGuard guard(A.device());
    prepare_call(MM, "gemm_allreduce_overlap");
    at::Tensor& staging = staging_like(C);
    const int* table = group_table_for(cSEG_CPU, cSEG_GPU, g.T);
    fork_comm_stream(g.G);
    FO_CALL(fo_gemm_signal(s.dtype, (int)Algo, s.M, s.N, s.K, (int)rLDN, cSEG_GPU.data_ptr<int>(), g.G, table,
                           A.data_ptr(), B.data_ptr(), C.data_ptr(), MM.data_ptr<int>(), RA.data_ptr<int>(),
                           if_monitor ? 1 : 0, gemm_stream_));
    consume_groups(C, staging.data_ptr(), (int64_t)g.BM * g.BN, cSEG_CPU, cSEG_GPU, MM, 1, 0);
    raise_on_timeout(MM, "gemm_allreduce_overlap");
}

void OverlapImpl::GemmReduceScatterOverlap(at::Tensor A, at::Tensor B, at::Tensor C, at::Tensor D, at::Tensor MM,
                                           at::Tensor RA, at::Tensor RE, int64_t rLDN, at::Tensor cSEG_CPU,
                                           at::Tensor cSEG_GPU, int64_t Algo, bool if_monitor) {
    require_overlap();
    const fo_host::GemmShape s = fo_host::check_gemm(A, B, C, "gemm_reducescatter_overlap");
    const fo_host::SignalShape g =
        fo_host::check_signal(s, MM, RA, RE, rLDN, cSEG_CPU, cSEG_GPU, (int)Algo, if_monitor, (int)my_size_,
                              "gemm_reducescatter_overlap");
    const int64_t total = (int64_t)s.M * s.N;
    fo_host::check_buffer(D, C, "gemm_reducescatter_overlap", "D");
    // D is one rank's receive buffer [M/ws, N] as in the reference, or all ws
    // of them stacked [ws, M/ws, N].
    TORCH_CHECK(D.numel() == total / my_size_ || D.numel() == total,
                "gemm_reducescatter_overlap: D must hold M*N/world_size = ", total / my_size_, " or M*N = ", total,
                " elements, got ", D.numel());
    c10::DeviceGuard guard(A.device());
    prepare_call(MM, "gemm_reducescatter_overlap");
    const int* table = group_table_for(cSEG_CPU, cSEG_GPU, g.T);
    fork_comm_stream(g.G);
    FO_CALL(fo_gemm_scatter(s.dtype, (int)Algo, s.M, s.N, s.K, (int)rLDN, cSEG_GPU.data_ptr<int>(), g.G, table,
                            A.data_ptr(), B.data_ptr(), C.data_ptr(), MM.data_ptr<int>(), RA.data_ptr<int>(),
                            RE.data_ptr<int>(), if_monitor ? 1 : 0, gemm_stream_));
    const int64_t stride = (D.numel() == total && my_size_ > 1) ? total / my_size_ : 0;
    consume_groups(C, D.data_ptr(), (int64_t)g.BM * g.BN, cSEG_CPU, cSEG_GPU, MM, (int)my_size_, stride);
    raise_on_timeout(MM, "gemm_reducescatter_overlap");
}

void OverlapImpl::GemmAllReduce(at::Tensor A, at::Tensor B, at::Tensor C, int64_t Algo) {
    Gemm(A, B, C, Algo);
    McclAllReduce(C);
}

void OverlapImpl::GemmReduceScatter(at::Tensor A, at::Tensor B, at::Tensor C, at::Tensor D, int64_t Algo) {
    Gemm(A, B, C, Algo);
    fo_host::check_buffer(D, C, "gemm_reducescatter", "D");
    const int64_t recv = C.numel() / my_size_;
    TORCH_CHECK(D.numel() >= recv, "gemm_reducescatter: D holds ", D.numel(), " elements, needs ", recv);
    c10::DeviceGuard guard(C.device());
    // What this rank would receive (src/overlap_impl.cu:104-107), without the sum over ranks.
    bulk_consume((const char*)C.data_ptr() + my_rank_ * recv * C.element_size(), D.data_ptr(),
                 recv * C.element_size());
}

void OverlapImpl::GemmAll2All(at::Tensor A, at::Tensor B, at::Tensor C, at::Tensor D, int64_t Algo,
                              at::Tensor mLen_CPU) {
    TORCH_CHECK(my_size_ == 1, "gemm_all2all: exchanging rows with ", my_size_ - 1,
                " peers needs more than one GPU, which this build does not drive");
    Gemm(A, B, C, Algo);  // a world of one sends and receives nothing (src/overlap_impl.cu:132-143)
}

void OverlapImpl::McclAllReduce(at::Tensor C) {
    require_gemm();
    fo_host::check_buffer(C, C, "mccl_allreduce", "C");
    c10::DeviceGuard guard(C.device());
    at::Tensor& staging = staging_like(C);
    bulk_consume(C.data_ptr(), staging.data_ptr(), C.numel() * C.element_size());
}

void OverlapImpl::SegAllReduce(at::Tensor C, at::Tensor cSEG_CPU, int64_t SegNum) {
    require_gemm();
    fo_host::check_buffer(C, C, "seg_allreduce", "C");
    TORCH_CHECK(cSEG_CPU.device().is_cpu() && cSEG_CPU.scalar_type() == at::kInt && cSEG_CPU.is_contiguous(),
                "seg_allreduce: cSEG_CPU must be a contiguous int32 host tensor");
    TORCH_CHECK(SegNum > 0 && C.numel() % SegNum == 0, "seg_allreduce: SegNum=", SegNum, " must divide M*N");
    c10::DeviceGuard guard(C.device());
    at::Tensor& staging = staging_like(C);
    const int* cseg = cSEG_CPU.data_ptr<int>();
    const int64_t unit = C.numel() / SegNum;
    int64_t acc = 0;
    // src/overlap_impl.cu:160-173: cSEG_CPU[s] counts units of M*N/SegNum.
    for (int64_t sidx = 0; sidx < cSEG_CPU.numel() && acc < C.numel(); ++sidx) {
        const int64_t n = unit * cseg[sidx];
        TORCH_CHECK(n >= 0 && acc + n <= C.numel(), "seg_allreduce: segments exceed M*N");
        bulk_consume((const char*)C.data_ptr() + acc * C.element_size(),
                     (char*)staging.data_ptr() + acc * C.element_size(), n * C.element_size());
        acc += n;
    }
}

void OverlapImpl::McclReduceScatter(at::Tensor C) {
    require_gemm();
    fo_host::check_buffer(C, C, "mccl_reducescatter", "C");
    c10::DeviceGuard guard(C.device());
    // In place in the reference: the rank's part of C receives the sum
    // (src/overlap_impl.cu:183-186).  Stand-in: that part goes to staging.
    at::Tensor& staging = staging_like(C);
    const int64_t recv = C.numel() / my_size_;
    const size_t off = my_rank_ * recv * C.element_size();
    bulk_consume((const char*)C.data_ptr() + off, (char*)staging.data_ptr() + off, recv * C.element_size());
}

void OverlapImpl::McclAll2All(at::Tensor C, at::Tensor D, at::Tensor mLen_CPU) {
    TORCH_CHECK(my_size_ == 1, "mccl_all2all: exchanging rows with ", my_size_ - 1,
                " peers needs more than one GPU, which this build does not drive");
}
