#pragma once
#include <ATen/ATen.h>

#include <cstdint>
#include <vector>

// src/rmsnorm/rmsnorm.h:6-8
void reorder_rmsnorm(at::Tensor X, at::Tensor RX, at::Tensor RW, int64_t BM, int64_t BN, int64_t rldn, at::Tensor RA);
void rmsnorm(at::Tensor X, at::Tensor O, at::Tensor RW);
// Same kernels with eps exposed (the reference fixes 1e-5, src/rmsnorm/rmsnorm.cuh:100).
void reorder_rmsnorm_eps(at::Tensor X, at::Tensor RX, at::Tensor RW, int64_t BM, int64_t BN, int64_t rldn,
                         at::Tensor RA, double eps);
void rmsnorm_eps(at::Tensor X, at::Tensor O, at::Tensor RW, double eps);
// src/mccl_utils.h:19
std::vector<int64_t> generate_mccl_id();
