// torch-facing wrappers of the RMSNorm kernels (src/rmsnorm/rmsnorm.cpp:10-36)
// and the communicator-id generator (src/mccl_utils.cpp:7-14).
#include "rmsnorm_op.h"

#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>
#include <unistd.h>

#include <atomic>
#include <chrono>

#include "host_common.h"

namespace {

void check_norm(const at::Tensor& X, const at::Tensor& O, const at::Tensor& W, const char* who) {
    TORCH_CHECK(X.defined() && X.dim() == 2, who, ": X must be [rows, dim]");
    fo_host::dtype_code(X, who);
    fo_host::check_buffer(X, X, who, "X");
    fo_host::check_buffer(O, X, who, "output");
    fo_host::check_buffer(W, X, who, "weight");
    TORCH_CHECK(O.numel() == X.numel(), who, ": output holds ", O.numel(), " elements, X has ", X.numel());
    TORCH_CHECK(W.numel() == X.size(1), who, ": weight has ", W.numel(), " entries, dim is ", X.size(1));
}

}  // namespace

void reorder_rmsnorm_eps(at::Tensor X, at::Tensor RX, at::Tensor RW, int64_t BM, int64_t BN, int64_t rldn,
                         at::Tensor RA, double eps) {
    check_norm(X, RX, RW, "reorder_rmsnorm");
    fo_host::check_index(RA, X, "reorder_rmsnorm", "RA");
    const int64_t bs = X.size(0), dim = X.size(1);
    TORCH_CHECK(BM > 0 && BN > 0 && bs % BM == 0 && dim % BN == 0, "reorder_rmsnorm: X [", bs, ",", dim,
                "] is not a whole number of ", BM, "x", BN, " tiles");
    TORCH_CHECK(RA.numel() == (bs / BM) * (dim / BN), "reorder_rmsnorm: RA has ", RA.numel(), " entries, expected ",
                (bs / BM) * (dim / BN));
    c10::DeviceGuard guard(X.device());
    FO_CALL(fo_reorder_rmsnorm(fo_host::dtype_code(X, "reorder_rmsnorm"), X.data_ptr(), RW.data_ptr(), RX.data_ptr(),
                               (int)bs, (int)dim, (int)BM, (int)BN, (int)rldn, RA.data_ptr<int>(), (float)eps,
                               (void*)c10::hip::getCurrentHIPStream().stream()));
}

void reorder_rmsnorm(at::Tensor X, at::Tensor RX, at::Tensor RW, int64_t BM, int64_t BN, int64_t rldn,
                     at::Tensor RA) {
    reorder_rmsnorm_eps(X, RX, RW, BM, BN, rldn, RA, 1e-5);
}

void rmsnorm_eps(at::Tensor X, at::Tensor O, at::Tensor RW, double eps) {
    check_norm(X, O, RW, "rmsnorm");
    c10::DeviceGuard guard(X.device());
    FO_CALL(fo_rmsnorm(fo_host::dtype_code(X, "rmsnorm"), X.data_ptr(), RW.data_ptr(), O.data_ptr(), (int)X.size(0),
                       (int)X.size(1), (float)eps, (void*)c10::hip::getCurrentHIPStream().stream()));
}

void rmsnorm(at::Tensor X, at::Tensor O, at::Tensor RW) { rmsnorm_eps(X, O, RW, 1e-5); }

std::vector<int64_t> generate_mccl_id() {
    // 128 opaque bytes as 16 int64, unique per call in this process.  No
    // communicator is built from it on one GPU.
    static std::atomic<int64_t> counter{0};
    std::vector<int64_t> id(16, 0);
    id[0] = 0x464f4d49333535LL;  // tag
    id[1] = (int64_t)getpid();
    id[2] = std::chrono::steady_clock::now().time_since_epoch().count();
    id[3] = counter.fetch_add(1);
    return id;
}
