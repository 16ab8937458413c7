// Argument validation shared by the torch-facing host classes.  The reference
// performs none (a wrong tensor makes it crash or hang); every check here
// raises a c10::Error that Python sees as RuntimeError.
#pragma once

#include <ATen/ATen.h>
#include <c10/util/Exception.h>

#include <numeric>

#include "../../include/flashoverlap_hip.h"

#define FO_CALL(expr)                                                        \
    do {                                                                     \
        const int fo_rc_ = (expr);                                           \
        TORCH_CHECK(fo_rc_ == FO_OK, "libfo_hip: ", fo_last_error(), " (status ", fo_rc_, ")"); \
    } while (0)

namespace fo_host {

struct GemmShape {
    int M, N, K, dtype;
};

struct SignalShape {
    int BM, BN, TM, TN, T, G;
};

inline int dtype_code(const at::Tensor& t, const char* who) {
    if (t.scalar_type() == at::kHalf) return FO_F16;
    if (t.scalar_type() == at::kBFloat16) return FO_BF16;
    TORCH_CHECK(false, who, ": tensors must be float16 or bfloat16, got ", t.scalar_type());
}

inline void check_buffer(const at::Tensor& t, const at::Tensor& like, const char* who, const char* name) {
    TORCH_CHECK(t.defined(), who, ": ", name, " is undefined");
    TORCH_CHECK(t.is_cuda(), who, ": ", name, " must be on the GPU");
    TORCH_CHECK(t.is_contiguous(), who, ": ", name, " must be contiguous");
    TORCH_CHECK(t.device() == like.device(), who, ": ", name, " is on ", t.device(), ", expected ", like.device());
    TORCH_CHECK(t.scalar_type() == like.scalar_type(), who, ": ", name, " has dtype ", t.scalar_type(),
                ", expected ", like.scalar_type());
}

inline void check_index(const at::Tensor& t, const at::Tensor& like, const char* who, const char* name) {
    TORCH_CHECK(t.defined() && t.is_cuda() && t.device() == like.device(), who, ": ", name,
                " must be on the same GPU as A");
    TORCH_CHECK(t.scalar_type() == at::kInt && t.is_contiguous(), who, ": ", name, " must be contiguous int32");
}

inline GemmShape check_gemm(const at::Tensor& A, const at::Tensor& B, const at::Tensor& C, const char* who) {
    TORCH_CHECK(A.defined() && A.dim() == 2 && B.defined() && B.dim() == 2, who, ": A [M,K] and B [N,K] must be 2-D");
    GemmShape s;
    s.dtype = dtype_code(A, who);
    check_buffer(A, A, who, "A");
    check_buffer(B, A, who, "B");
    check_buffer(C, A, who, "C");
    TORCH_CHECK(A.size(1) == B.size(1), who, ": A is [", A.size(0), ",", A.size(1), "] but B is [", B.size(0), ",",
                B.size(1), "]; both must have K columns");
    TORCH_CHECK(A.size(0) > 0 && B.size(0) > 0 && A.size(1) > 0, who, ": empty operand");
    TORCH_CHECK(A.size(0) * B.size(0) < (int64_t(1) << 31), who, ": M*N too large");
    s.M = (int)A.size(0);
    s.K = (int)A.size(1);
    s.N = (int)B.size(0);
    TORCH_CHECK(C.numel() == (int64_t)s.M * s.N, who, ": C must hold M*N = ", (int64_t)s.M * s.N, " elements, got ",
                C.numel());
    return s;
}

// Validates the tensors of a signalling call.  TM and TN are read from RA's
// shape like the reference does (src/overlap_impl.cu:238-239), and must agree
// with the tile that `Algo` selects.
inline SignalShape check_signal(const GemmShape& s, const at::Tensor& MM, const at::Tensor& RA, const at::Tensor& RE,
                                int64_t rLDN, const at::Tensor& cseg_cpu, const at::Tensor& cseg_gpu, int algo,
                                bool monitor, int world, const char* who) {
    SignalShape g;
    int bk;
    FO_CALL(fo_algo_tile(algo, &g.BM, &g.BN, &bk));
    TORCH_CHECK(RA.defined() && RA.dim() == 2, who, ": RA must be [TM,TN]");
    g.TM = (int)RA.size(0);
    g.TN = (int)RA.size(1);
    g.T = g.TM * g.TN;
    TORCH_CHECK(s.M % g.BM == 0 && s.N % g.BN == 0, who, ": M=", s.M, " N=", s.N, " must be multiples of the ", g.BM,
                "x", g.BN, " tile of Algo ", algo);
    TORCH_CHECK(g.TM == s.M / g.BM && g.TN == s.N / g.BN, who, ": RA is [", g.TM, ",", g.TN, "] but Algo ", algo,
                " tiles the output as [", s.M / g.BM, ",", s.N / g.BN, "]");
    TORCH_CHECK(cseg_cpu.defined() && cseg_cpu.device().is_cpu() && cseg_cpu.scalar_type() == at::kInt &&
                    cseg_cpu.is_contiguous() && cseg_cpu.dim() == 1,
                who, ": cSEG_CPU must be a 1-D contiguous int32 host tensor");
    g.G = (int)cseg_cpu.numel();
    TORCH_CHECK(g.G > 0, who, ": empty cSeg");
    TORCH_CHECK(cseg_gpu.defined() && cseg_gpu.numel() == g.G, who, ": cSEG_GPU must be the device copy of cSEG_CPU");
    check_index(RA, MM, who, "RA");
    check_index(cseg_gpu, RA, who, "cSEG_GPU");
    check_index(MM, RA, who, "MM");
    const int* c = cseg_cpu.data_ptr<int>();
    int64_t sum = 0;
    for (int i = 0; i < g.G; ++i) {
        TORCH_CHECK(c[i] >= 0, who, ": cSeg[", i, "] = ", c[i]);
        sum += c[i];
    }
    // A short or long cSeg makes the reference's waiter spin forever
    // (src/wait.cuh:6-8); refuse it up front.
    TORCH_CHECK(sum == g.T, who, ": sum(cSeg) = ", sum, " but the output has ", g.T, " tiles");
    TORCH_CHECK(rLDN >= 1 && g.T % rLDN == 0, who, ": rLDN=", rLDN, " must divide the tile count ", g.T);
    TORCH_CHECK(rLDN == 1, who, ": groups are contiguous ranges only for rLDN == 1 (got ", rLDN, ")");
    if (monitor) {
        // Monitor mode keeps its ticket counter in MM[TN-1] and the tickets in
        // MM[TN + slot] (src/overlap/gemm_with_signal.h:197-200).
        TORCH_CHECK(g.G <= g.TN - 1, who, ": monitor mode needs len(cSeg) <= TN-1 = ", g.TN - 1, ", got ", g.G);
        TORCH_CHECK(MM.numel() >= (int64_t)g.TN + g.T, who, ": monitor mode needs MM of at least (TM+1)*TN = ",
                    g.TN + g.T, " ints, got ", MM.numel());
    } else {
        TORCH_CHECK(MM.numel() >= g.G, who, ": MM holds ", MM.numel(), " counters but cSeg has ", g.G, " groups");
    }
    if (RE.defined()) {
        check_index(RE, RA, who, "RE");
        TORCH_CHECK(RE.numel() == (int64_t)s.M * s.N / g.BN, who, ": RE must have M*N/BN = ",
                    (int64_t)s.M * s.N / g.BN, " entries, got ", RE.numel());
        TORCH_CHECK(((int64_t)g.BM * g.BN) % (8 * world) == 0, who, ": a ", g.BM, "x", g.BN,
                    " tile does not split into ", world, " slices of whole 16-byte units");
    }
    return g;
}

}  // namespace fo_host
