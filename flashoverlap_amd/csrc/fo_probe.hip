// fo_mfma_spin: a loop of nothing but the GEMM's MFMA instruction on operands held in registers.
//
// The GEMM of this library runs at the chip's power limit: its clock, and with it its rate,
// depends on how many bits the operands toggle in the matrix cores.  This probe measures what
// that limit leaves to a kernel that does no memory, LDS or address work at all: the same
// v_mfma_f32_16x16x32 instruction on the same 8 x 8 accumulators per wavefront, issued in the
// order of the GEMM's k-step (column by column, the two k halves of an accumulator back to back),
// one wavefront per SIMD, the 32 operand fragments of a wavefront read once from the caller's
// buffer.  Run on the GEMM's own operands it gives the ceiling the GEMM's rate can be read
// against; run on zeros it gives the instruction's issue rate at full clock.  `wide` runs the
// 32x32x16 instruction instead (4 x 4 accumulators, four k parts), which the same operands make
// draw more power per flop.  No counterpart in the reference.
#include <type_traits>

#include "fo_internal.h"

namespace fo {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;

constexpr int kSpinMfmas = 128;   // 16x16x32 MFMAs per loop iteration and wavefront (32x32x16: half as many, same flop)

// Issued from assembly, accumulator in the matrix core's own registers, like the GEMM's: the
// compiler then keeps the order written here.
template <bool BF16, bool WIDE, typename Acc, typename Frag>
__device__ __forceinline__ void spin_mfma(Acc& c, const Frag& x, const Frag& y) {
    if constexpr (BF16 && WIDE) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(x), "v"(y));
    else if constexpr (WIDE) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(c) : "v"(x), "v"(y));
    else if constexpr (BF16) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(x), "v"(y));
    else asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(x), "v"(y));
}

template <bool BF16, bool WIDE>
__global__ __launch_bounds__(256) void mfma_spin_kernel(const uint4* __restrict__ operands, unsigned n16, int iters,
                                                        float* sink) {
    using Frag = typename std::conditional<BF16, bf16x8_t, f16x8_t>::type;
    using Acc = typename std::conditional<WIDE, f32x16_t, f32x4_t>::type;
    constexpr int F = WIDE ? 4 : 8;                 // blocks per edge: F x F accumulators fill 256 registers
    constexpr int P = WIDE ? 4 : 2;                 // k parts of a 64-deep panel
    constexpr int R = WIDE ? 16 : 4;                // registers per accumulator
    const unsigned lane = blockIdx.x * 256u + threadIdx.x;
    Frag a[P][F], b[P][F];
#pragma unroll
    for (int h = 0; h < P; ++h)
#pragma unroll
        for (int i = 0; i < F; ++i) {
            const uint4 va = operands[(lane * 32u + h * 2 * F + i) % n16];
            const uint4 vb = operands[(lane * 32u + h * 2 * F + F + i) % n16];
            a[h][i] = __builtin_bit_cast(Frag, va);
            b[h][i] = __builtin_bit_cast(Frag, vb);
        }
    Acc acc[F][F];
#pragma unroll
    for (int i = 0; i < F; ++i)
#pragma unroll
        for (int j = 0; j < F; ++j)
#pragma unroll
            for (int r = 0; r < R; ++r) acc[i][j][r] = 0.f;
    asm volatile("s_nop 7" ::: "memory");           // the cleared accumulators have landed
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int hs = 0; hs < 2; ++hs)              // rows of blocks in two halves, as in the GEMM
#pragma unroll
            for (int j = 0; j < F; ++j)
#pragma unroll
                for (int rr = 0; rr < F / 2; ++rr) {
                    const int i = hs * (F / 2) + ((j & 1) ? F / 2 - 1 - rr : rr);
#pragma unroll
                    for (int h = 0; h < P; ++h) spin_mfma<BF16, WIDE>(acc[i][j], b[h][j], a[h][i]);
                }
    }
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");   // the last results are in the registers
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < F; ++i)
#pragma unroll
        for (int j = 0; j < F; ++j)
#pragma unroll
            for (int r = 0; r < R; ++r) s += acc[i][j][r];
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
    // one workgroup per CU, 4 wavefronts each, 128 MFMAs of 2*16*16*32 flop (or 64 of 2*32*32*16) per iteration
    if (flop) *flop = (long long)cus * 4 * iters * kSpinMfmas * (2ll * 16 * 16 * 32);
    return FO_OK;
}
