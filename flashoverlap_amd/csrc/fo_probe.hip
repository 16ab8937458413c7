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
// draw more power per flop.  `traffic` adds what a 256x256 GEMM tile moves per k-step beside the
// MFMAs, with nothing ever waiting for it: bit 0 the 32 fragment reads (LDS -> registers) of a
// wavefront, bit 1 its 16 one-KiB copies (L2 -> LDS, four workgroups per XCD reading the same
// stream, so three in four hit the L2 as in the GEMM).  The rate with both is what the power limit
// leaves to a kernel with this tile's operand traffic and a perfect schedule.
// No counterpart in the reference.  Built into libfo_bench.so, a library of its own that only the
// benchmark and its test load: nothing here is part of the product's C ABI.
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>

#include <type_traits>

#include "../../include/flashoverlap_bench.h"

namespace fo {

static thread_local char t_bench_error[256] = "";

static int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
static int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(t_bench_error, sizeof t_bench_error, fmt, ap);
    va_end(ap);
    return code;
}

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

typedef __attribute__((address_space(3))) void spin_lds_void;

template <bool BF16, bool WIDE, int TRAFFIC>
__global__ __launch_bounds__(256) void mfma_spin_kernel(const uint4* __restrict__ operands, unsigned n16, int iters,
                                                        unsigned window, float* sink) {
    using Frag = typename std::conditional<BF16, bf16x8_t, f16x8_t>::type;
    using Acc = typename std::conditional<WIDE, f32x16_t, f32x4_t>::type;
    constexpr int F = WIDE ? 4 : 8;                 // blocks per edge: F x F accumulators fill 256 registers
    constexpr int P = WIDE ? 4 : 2;                 // k parts of a 64-deep panel
    constexpr int R = WIDE ? 16 : 4;                // registers per accumulator
    static_assert(!WIDE || TRAFFIC == 0, "operand traffic is modelled for the GEMM's own instruction only");
    // 8 KiB that the fragment reads walk (16 rows of 128 bytes per wavefront and block row, swizzled
    // like the GEMM's panels) and 1 KiB per wavefront where the copies land
    __shared__ __attribute__((aligned(1024))) unsigned char lds[TRAFFIC ? 8192 + 4096 : 16];
    const unsigned lane = blockIdx.x * 256u + threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), l = threadIdx.x & 63;
    if constexpr ((TRAFFIC & 1) != 0) {
        for (int i = threadIdx.x; i < 512; i += 256) ((uint4*)lds)[i] = operands[(blockIdx.x * 512u + i) % n16];
        __syncthreads();
    }
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
    // Registers that the fragment reads land in.  They stay reserved for that until the end of the
    // kernel: a read still in flight must never find its destination handed to something else.
    [[maybe_unused]] Frag land[8];
    if constexpr ((TRAFFIC & 1) != 0) {
#pragma unroll
        for (int i = 0; i < 8; ++i) land[i] = a[0][i % F];
    }
    [[maybe_unused]] const unsigned rd =
        (unsigned)(__UINTPTR_TYPE__)((spin_lds_void*)lds) + (wave * 16 + (l & 15)) * 128 + (((((l >> 4) & 1) * 2 + (l >> 5)) ^ (l & 7)) * 16);
    [[maybe_unused]] __amdgpu_buffer_rsrc_t rsrc;
    [[maybe_unused]] unsigned goff = 0;
    if constexpr ((TRAFFIC & 2) != 0) {
        rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)operands, 0, 0xffffffff, 0x00020000);
        // workgroup i runs on XCD i % 8: workgroups i, i+8, i+16, i+24 of a group of 32 share one stream
        goff = __builtin_amdgcn_readfirstlane(((blockIdx.x / 32u) * 4u + wave) * 65536u);
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
                    const int sl = (hs * F + j) * (F / 2) + rr;        // 0..63 for the GEMM's instruction
                    if constexpr ((TRAFFIC & 1) != 0) {
                        if ((sl & 1) == 0) asm volatile("ds_read_b128 %0, %1" : "+v"(land[(sl >> 1) & 7]) : "v"(rd));
                    }
                    if constexpr ((TRAFFIC & 2) != 0) {
                        if ((sl & 3) == 1) {
                            // window is a power of two and at most half the buffer: the 1 KiB stays inside
                            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (spin_lds_void*)(lds + 8192 + wave * 1024), 16, l * 16,
                                                                     (int)(goff & (window - 1)), 0, 0);
                            goff += 1024;
                        }
                    }
#pragma unroll
                    for (int h = 0; h < P; ++h) spin_mfma<BF16, WIDE>(acc[i][j], b[h][j], a[h][i]);
                }
        if constexpr ((TRAFFIC & 1) != 0) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // this round's reads have landed
    }
    // nothing of this workgroup is in flight when it ends; the last MFMA results are in the registers
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_nop 15\n\ts_nop 15" ::: "memory");
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < F; ++i)
#pragma unroll
        for (int j = 0; j < F; ++j)
#pragma unroll
            for (int r = 0; r < R; ++r) s += acc[i][j][r];
    if constexpr ((TRAFFIC & 1) != 0) {
#pragma unroll
        for (int i = 0; i < 8; ++i) s += (float)land[i][0];
    }
    // keeps the loop alive; a sum of products of the operands never equals this value
    if (s == -1.2345e-30f) *sink = s;
}

}  // namespace fo

extern "C" const char* fo_bench_last_error(void) { return fo::t_bench_error; }

extern "C" int fo_mfma_spin(int dtype, int wide, int traffic, const void* operands, size_t operand_bytes, int iters,
                            void* sink, long long* flop, void* stream) {
    using namespace fo;
    if (dtype != FO_F16 && dtype != FO_BF16) return fail(FO_ERR_ARG, "fo_mfma_spin: dtype=%d", dtype);
    if (traffic < 0 || traffic > 3 || (wide && traffic))
        return fail(FO_ERR_ARG, "fo_mfma_spin: traffic=%d (0..3, and 0 with the wide instruction)", traffic);
    if (!operands || !sink) return fail(FO_ERR_ARG, "fo_mfma_spin: null pointer");
    if (operand_bytes < 16 || operand_bytes / 16 > 0xffffffffull)
        return fail(FO_ERR_ARG, "fo_mfma_spin: operand_bytes=%zu outside 16..64 GiB", operand_bytes);
    if ((traffic & 2) && (operand_bytes < (4u << 20) || operand_bytes > 0xffffffffull))
        return fail(FO_ERR_ARG, "fo_mfma_spin: copies need 4 MiB..4 GiB of operands, got %zu bytes", operand_bytes);
    if (iters < 1 || iters > (1 << 20)) return fail(FO_ERR_ARG, "fo_mfma_spin: iters=%d outside 1..2^20", iters);
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
        return fail(FO_ERR_HIP, "fo_mfma_spin: cannot read the CU count of the current device");
    const unsigned n16 = (unsigned)(operand_bytes / 16);
    // the copies walk a power-of-two window of at most half the buffer (and at most 64 MiB)
    unsigned window = 1u << 21;
    while (window < (64u << 20) && (size_t)window * 4 <= operand_bytes) window <<= 1;
    using Kernel = void (*)(const uint4*, unsigned, int, unsigned, float*);
    Kernel kern;
    if (wide) kern = dtype == FO_BF16 ? mfma_spin_kernel<true, true, 0> : mfma_spin_kernel<false, true, 0>;
    else if (dtype == FO_BF16) {
        static const Kernel k[4] = {mfma_spin_kernel<true, false, 0>, mfma_spin_kernel<true, false, 1>,
                                    mfma_spin_kernel<true, false, 2>, mfma_spin_kernel<true, false, 3>};
        kern = k[traffic];
    } else {
        static const Kernel k[4] = {mfma_spin_kernel<false, false, 0>, mfma_spin_kernel<false, false, 1>,
                                    mfma_spin_kernel<false, false, 2>, mfma_spin_kernel<false, false, 3>};
        kern = k[traffic];
    }
    hipLaunchKernelGGL(kern, dim3(cus), dim3(256), 0, (hipStream_t)stream, (const uint4*)operands, n16, iters, window,
                       (float*)sink);
    if (hipError_t e = hipGetLastError(); e != hipSuccess)
        return fail(FO_ERR_HIP, "fo_mfma_spin: launch failed: %s", hipGetErrorString(e));
    // one workgroup per CU, 4 wavefronts each, 128 MFMAs of 2*16*16*32 flop (or 64 of 2*32*32*16) per iteration
    if (flop) *flop = (long long)cus * 4 * iters * kSpinMfmas * (2ll * 16 * 16 * 32);
    return FO_OK;
}
