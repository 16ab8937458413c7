// BaselineImpl: the non-overlapped comparison path with the method set of the
// reference class (src/baseline_impl.h:10-34).  The reference pairs the vendor
// BLAS (mublasGemmEx, src/baseline_impl.cu:55-66) with one bulk collective on
// one stream; here the GEMM is torch's library matmul (hipBLASLt) and the
// collective is the same consumer copy the overlapped path uses.
#pragma once

#include <ATen/ATen.h>
#include <torch/custom_class.h>

#include <cstdint>
#include <vector>

class BaselineImpl : public torch::CustomClassHolder {
  public:
    BaselineImpl();
    ~BaselineImpl() override;

    void McclInit(int64_t tp_rank, int64_t tp_size, std::vector<int64_t> tp_id);
    void MublasInit();

    void Gemm(at::Tensor A, at::Tensor B, at::Tensor C);
    void GemmAllReduce(at::Tensor A, at::Tensor B, at::Tensor C);
    void GemmReduceScatter(at::Tensor A, at::Tensor B, at::Tensor C, at::Tensor D);
    void GemmAll2All(at::Tensor A, at::Tensor B, at::Tensor C, at::Tensor D, at::Tensor mLen_CPU);

    void McclAllReduce(at::Tensor C);
    void McclReduceScatter(at::Tensor C);
    void McclAll2All(at::Tensor C, at::Tensor D, at::Tensor mLen_CPU);

    at::Tensor Staging() const;

  private:
    bool ready_ = false;
    int64_t my_rank_ = 0;
    int64_t my_size_ = 1;
    at::Tensor staging_;

    void* stream() const;
    at::Tensor& staging_like(const at::Tensor& C);
};
