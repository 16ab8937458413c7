// Registration of the torch-visible API: the class and op names of the
// reference (src/pybind.cpp:114-150), the spelling of its CUDA upstream
// (cutlass_* / nccl_* / cublas_*), and a few additions marked below.
#include <torch/custom_class.h>
#include <torch/library.h>

#include "baseline_impl.h"
#include "overlap_impl.h"
#include "rmsnorm_op.h"

TORCH_LIBRARY(flashoverlap_class, m) {
    m.class_<BaselineImpl>("BaselineImpl")
        .def(torch::init())
        .def("mccl_init", &BaselineImpl::McclInit)
        .def("mublas_init", &BaselineImpl::MublasInit)
        .def("gemm_allreduce", &BaselineImpl::GemmAllReduce)
        .def("gemm_reducescatter", &BaselineImpl::GemmReduceScatter)
        .def("gemm_all2all", &BaselineImpl::GemmAll2All)
        .def("mublas_gemm", &BaselineImpl::Gemm)
        .def("mccl_allreduce", &BaselineImpl::McclAllReduce)
        .def("mccl_reducescatter", &BaselineImpl::McclReduceScatter)
        .def("mccl_all2all", &BaselineImpl::McclAll2All)
        // CUDA-upstream spelling
        .def("nccl_init", &BaselineImpl::McclInit)
        .def("cublas_init", &BaselineImpl::MublasInit)
        .def("cublas_gemm", &BaselineImpl::Gemm)
        .def("nccl_allreduce", &BaselineImpl::McclAllReduce)
        .def("nccl_reducescatter", &BaselineImpl::McclReduceScatter)
        .def("nccl_all2all", &BaselineImpl::McclAll2All)
        // addition
        .def("staging", &BaselineImpl::Staging);

    m.class_<OverlapImpl>("OverlapImpl")
        .def(torch::init())
        .def("mutlass_init", &OverlapImpl::MutlassInit)
        .def("mutlass_gemm", &OverlapImpl::Gemm)
        .def("gemm_allreduce_overlap", &OverlapImpl::GemmAllReduceOverlap)
        .def("gemm_reducescatter_overlap", &OverlapImpl::GemmReduceScatterOverlap)
        .def("mccl_init", &OverlapImpl::McclInit)
        .def("gemm_allreduce", &OverlapImpl::GemmAllReduce)
        .def("gemm_reducescatter", &OverlapImpl::GemmReduceScatter)
        .def("gemm_all2all", &OverlapImpl::GemmAll2All)
        .def("overlap_init", &OverlapImpl::OverlapInit)
        .def("mccl_allreduce", &OverlapImpl::McclAllReduce)
        .def("mccl_reducescatter", &OverlapImpl::McclReduceScatter)
        .def("mccl_all2all", &OverlapImpl::McclAll2All)
        .def("seg_allreduce", &OverlapImpl::SegAllReduce)
        // CUDA-upstream spelling
        .def("cutlass_init", &OverlapImpl::MutlassInit)
        .def("cutlass_gemm", &OverlapImpl::Gemm)
        .def("nccl_init", &OverlapImpl::McclInit)
        .def("nccl_allreduce", &OverlapImpl::McclAllReduce)
        .def("nccl_reducescatter", &OverlapImpl::McclReduceScatter)
        .def("nccl_all2all", &OverlapImpl::McclAll2All)
        // additions
        .def("staging", &OverlapImpl::Staging)
        .def("set_consumer_mode", &OverlapImpl::SetConsumerMode)
        .def("set_staging", &OverlapImpl::SetStaging)
        .def("set_consumer_blocks", &OverlapImpl::SetConsumerBlocks)
        .def("set_wait_timeout_ms", &OverlapImpl::SetWaitTimeoutMs)
        .def("wait_timeouts", &OverlapImpl::WaitTimeouts)
        .def("set_check_timeouts", &OverlapImpl::SetCheckTimeouts);
}

TORCH_LIBRARY(flashoverlap_op, m) {
    m.def("generate_mccl_id", &generate_mccl_id);
    m.def("generate_nccl_id", &generate_mccl_id);
    m.def("reorder_rmsnorm", &reorder_rmsnorm);
    // additions
    m.def("rmsnorm", &rmsnorm);
    m.def("reorder_rmsnorm_eps", &reorder_rmsnorm_eps);
    m.def("rmsnorm_eps", &rmsnorm_eps);
}
