// Non-overlapped baseline on one GPU: library GEMM, then one bulk consumer
// copy on the same stream (call structure of src/baseline_impl.cu:42-70,
// 84-115, 225-245).
#include "baseline_impl.h"

#include <ATen/ops/matmul.h>
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>

#include "host_common.h"

BaselineImpl::BaselineImpl() = default;
BaselineImpl::~BaselineImpl() = default;

void BaselineImpl::McclInit(int64_t tp_rank, int64_t tp_size, std::vector<int64_t> tp_id) {
    TORCH_CHECK(tp_size >= 1 && tp_rank >= 0 && tp_rank < tp_size, "mccl_init: rank ", tp_rank, " of ", tp_size);
    TORCH_CHECK(tp_id.size() == 16, "mccl_init: the id must have 16 entries, got ", tp_id.size());
    my_rank_ = tp_rank;
    my_size_ = tp_size;
}

void BaselineImpl::MublasInit() { ready_ = true; }

void* BaselineImpl::stream() const { return (void*)c10::hip::getCurrentHIPStream().stream(); }

at::Tensor& BaselineImpl::staging_like(const at::Tensor& C) {
    if (!staging_.defined() || staging_.numel() != C.numel() || staging_.scalar_type() != C.scalar_type() ||
        staging_.device() != C.device())
        staging_ = at::empty({C.numel()}, C.options());
    return staging_;
}

at::Tensor BaselineImpl::Staging() const {
    TORCH_CHECK(staging_.defined(), "staging: no all-reduce style call has run yet");
    return staging_;
}

void BaselineImpl::Gemm(at::Tensor A, at::Tensor B, at::Tensor C) {
    TORCH_CHECK(ready_, "BaselineImpl: call mublas_init() first");
    const fo_host::GemmShape s = fo_host::check_gemm(A, B, C, "mublas_gemm");
    c10::DeviceGuard guard(A.device());
    at::Tensor out = C.view({s.M, s.N});
    at::matmul_out(out, A, B.t());
}

void BaselineImpl::GemmAllReduce(at::Tensor A, at::Tensor B, at::Tensor C) {
    Gemm(A, B, C);
    McclAllReduce(C);
}

void BaselineImpl::GemmReduceScatter(at::Tensor A, at::Tensor B, at::Tensor C, at::Tensor D) {
    Gemm(A, B, C);
    fo_host::check_buffer(D, C, "gemm_reducescatter", "D");
    const int64_t recv = C.numel() / my_size_;
    TORCH_CHECK(D.numel() >= recv, "gemm_reducescatter: D holds ", D.numel(), " elements, needs ", recv);
    c10::DeviceGuard guard(C.device());
    FO_CALL(fo_consume((const char*)C.data_ptr() + my_rank_ * recv * C.element_size(), D.data_ptr(),
                       recv * C.element_size(), stream()));
}

void BaselineImpl::GemmAll2All(at::Tensor A, at::Tensor B, at::Tensor C, at::Tensor D, at::Tensor mLen_CPU) {
    TORCH_CHECK(my_size_ == 1, "gemm_all2all: exchanging rows with ", my_size_ - 1,
                " peers needs more than one GPU, which this build does not drive");
    Gemm(A, B, C);
}

void BaselineImpl::McclAllReduce(at::Tensor C) {
    fo_host::check_buffer(C, C, "mccl_allreduce", "C");
    c10::DeviceGuard guard(C.device());
    at::Tensor& staging = staging_like(C);
    FO_CALL(fo_consume(C.data_ptr(), staging.data_ptr(), C.numel() * C.element_size(), stream()));
}

void BaselineImpl::McclReduceScatter(at::Tensor C) {
    fo_host::check_buffer(C, C, "mccl_reducescatter", "C");
    c10::DeviceGuard guard(C.device());
    at::Tensor& staging = staging_like(C);
    const int64_t recv = C.numel() / my_size_;
    const size_t off = my_rank_ * recv * C.element_size();
    FO_CALL(fo_consume((const char*)C.data_ptr() + off, (char*)staging.data_ptr() + off, recv * C.element_size(),
                       stream()));
}

void BaselineImpl::McclAll2All(at::Tensor C, at::Tensor D, at::Tensor mLen_CPU) {
    TORCH_CHECK(my_size_ == 1, "mccl_all2all: exchanging rows with ", my_size_ - 1,
                " peers needs more than one GPU, which this build does not drive");
}
