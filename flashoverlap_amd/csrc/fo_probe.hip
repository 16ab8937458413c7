// fo_mfma_spin: a loop of nothing but the GEMM's MFMA instruction on operands held in registers.
//
// The GEMM of this library runs at the chip's power limit: its clock, and with it its rate,
// depends on how many bits the operands toggle in the matrix cores.  This probe measures what
// that limit leaves to a kernel that does no memory, LDS or address work at all: the same
// v_mfma_f32_16x16x32 instruction, 64 independent accumulators per wavefront, one wavefront per
// SIMD, the 16 operand fragments of a wavefront read once from the caller's buffer (`wide`: the
// 32x32x16 instruction on 4 + 4 fragments and 16 accumulators, the same flop per iteration).  Run on the
// GEMM's own operands it gives the ceiling the GEMM's rate can be read against; run on zeros it
// gives the instruction's issue rate at full clock.  No counterpart in the reference.
#include <type_traits>

#include "fo_internal.h"

namespace fo {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;

typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;

constexpr int kSpinMfmas = 64;   // 16x16x32 MFMAs per loop iteration and wavefront (32x32x16: half as many, same flop)

template <bool BF16, bool WIDE>
__global__ __launch_bounds__(256) void mfma_spin_kernel(const uint4* __restrict__ operands, unsigned n16, int iters,
                                                        float* sink) {
    using Frag = typename std::conditional<BF16, bf16x8_t, f16x8_t>::type;
    using Acc = typename std::conditional<WIDE, f32x16_t, f32x4_t>::type;
    constexpr int F = WIDE ? 4 : 8;                 // A and B fragments: F x F accumulators fill 256 registers
    constexpr int R = WIDE ? 16 : 4;                // registers per accumulator
    const unsigned lane = blockIdx.x * 256u + threadIdx.x;
    Frag a[F], b[F];
#pragma unroll
    for (int i = 0; i < F; ++i) {
        const uint4 va = operands[(lane * 16u + i) % n16];
        const uint4 vb = operands[(lane * 16u + 8 + i) % n16];
        a[i] = __builtin_bit_cast(Frag, va);
        b[i] = __builtin_bit_cast(Frag, vb);
    }
    Acc acc[F * F];
#pragma unroll
    for (int i = 0; i < F * F; ++i)
#pragma unroll
        for (int r = 0; r < R; ++r) acc[i][r] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int rep = 0; rep < (WIDE ? 2 : 1); ++rep)
#pragma unroll
            for (int i = 0; i < F; ++i)
#pragma unroll
                for (int j = 0; j < F; ++j) {
                    Acc& c = acc[i * F + j];
                    if constexpr (BF16 && WIDE) c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], c, 0, 0, 0);
                    else if constexpr (WIDE) c = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i], b[j], c, 0, 0, 0);
                    else if constexpr (BF16) c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b[j], c, 0, 0, 0);
                    else c = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[i], b[j], c, 0, 0, 0);
                }
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < F * F; ++i)
#pragma unroll
        for (int r = 0; r < R; ++r) s += acc[i][r];
    // keeps the loop alive; a sum of products of the operands never equals this value
    if (s == -1.2345e-30f) *sink = s;
}

}  // namespace fo

extern "C" int fo_mfma_spin(int dtype, int wide, const void* operands, size_t operand_bytes, int iters, void* sink,
                            long long* flop, void* stream) {
    using namespace fo;
    if (dtype != FO_F16 && dtype != FO_BF16) return fail(FO_ERR_ARG, "fo_mfma_spin: dtype=%d", dtype);
    if (!operands || !sink) return fail(FO_ERR_ARG, "fo_mfma_spin: null pointer");
    if (operand_bytes < 16 || operand_bytes / 16 > 0xffffffffull)
        return fail(FO_ERR_ARG, "fo_mfma_spin: operand_bytes=%zu outside 16..64 GiB", operand_bytes);
    if (iters < 1 || iters > (1 << 20)) return fail(FO_ERR_ARG, "fo_mfma_spin: iters=%d outside 1..2^20", iters);
    int cus = 0;
    if (int rc = fo_device_info(&cus, nullptr, nullptr)) return rc;
    const unsigned n16 = (unsigned)(operand_bytes / 16);
    auto kern = dtype == FO_BF16 ? (wide ? mfma_spin_kernel<true, true> : mfma_spin_kernel<true, false>)
                                 : (wide ? mfma_spin_kernel<false, true> : mfma_spin_kernel<false, false>);
    hipLaunchKernelGGL(kern, dim3(cus), dim3(256), 0, (hipStream_t)stream, (const uint4*)operands, n16, iters,
                       (float*)sink);
    FO_HIP(hipGetLastError());
    // one workgroup per CU, 4 wavefronts each, 64 MFMAs of 2*16*16*32 flop (or 32 of 2*32*32*16) per iteration
    if (flop) *flop = (long long)cus * 4 * iters * kSpinMfmas * (2ll * 16 * 16 * 32);
    return FO_OK;
}
