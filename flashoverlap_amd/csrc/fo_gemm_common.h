// Building blocks of the GEMM kernel in fo_gemm.hip: vector types, the MFMA wrappers, wait-count
// helpers, the LDS row swizzle, the launch parameters.
#pragma once

#include <hip/hip_runtime.h>

#include <type_traits>

#include "fo_internal.h"

namespace fo {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

template <typename T>
struct Mma;
template <>
struct Mma<_Float16> {
    using frag = f16x8;
    using out4 = f16x4;
    static __device__ __forceinline__ void run(frag a, frag b, f32x4& c) {
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
    }
    static __device__ __forceinline__ void clear(frag zeros, f32x4& c) {   // c = 0 x 0 + 0
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %1, 0" : "=a"(c) : "v"(zeros));
    }
};
template <>
struct Mma<__bf16> {
    using frag = bf16x8;
    using out4 = bf16x4;
    static __device__ __forceinline__ void run(frag a, frag b, f32x4& c) {
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
    }
    static __device__ __forceinline__ void clear(frag zeros, f32x4& c) {   // c = 0 x 0 + 0
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %1, 0" : "=a"(c) : "v"(zeros));
    }
};

// The MFMAs above are opaque to the compiler: it does not know that their
// results become readable only some cycles after issue, and it inserts no wait
// states between one of them and an instruction that reads its accumulator.  So
// the accumulators are kept in the matrix-core register file (constraint "a")
// from the first MFMA to the epilogue, where they are read by this statement
// behind an explicit settle() — the compiler is then never asked to move an
// accumulator on its own (a copy it places right behind an MFMA reads the value
// from before that MFMA).
static __device__ __forceinline__ float acc_read(const float& a) {
    float v;
    asm("v_accvgpr_read_b32 %0, %1" : "=v"(v) : "a"(a));   // not volatile: free to be scheduled within the epilogue
    return v;
}
// More wait states than the longest MFMA needs before its result can be read.
static __device__ __forceinline__ void settle_mfma() { asm volatile("s_nop 15\n\ts_nop 15" ::: "memory"); }

constexpr int kBK = 64;             // k-elements per LDS buffer
constexpr int kRowBytes = kBK * 2;  // one panel row in LDS: 128 bytes = 8 chunks of 16

enum { kPlain = 0, kSignal = 1, kScatter = 2 };

struct GemmParams {
    const void* A;
    const void* B;
    void* D;
    int M, N, K;
    int GM, GN;   // macro-tile grid
    unsigned gn_magic;   // raster_magic(GN)
    int BM, BN;   // layout tile
    int log_bm, log_bn;   // both edges are powers of two (128 or 256): shifts instead of divisions in the kernel
    int TN;       // N / BN
    int rLDN;
    const int* RA;
    const int* RE;
    const int* cseg;
    int G;
    const int* gtable;
    int* MM;
    int monitor;
};

typedef __attribute__((address_space(3))) void lds_void;

// s_waitcnt immediate of the gfx9 family: vmcnt in bits [3:0] and [15:14],
// expcnt [6:4], lgkmcnt [11:8]; 63 / 7 / 15 mean "do not wait".
constexpr int waitcnt_imm(int vm, int lgkm) {
    return (vm & 0xF) | ((vm >> 4) << 14) | (7 << 4) | ((lgkm & 0xF) << 8);
}
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(N, 15));
}
__device__ __forceinline__ void wait_lds_reads() { __builtin_amdgcn_s_waitcnt(waitcnt_imm(63, 0)); }

// The reference's linear scan over cSeg (src/overlap/gemm_with_signal.h:188-193).
__device__ __forceinline__ int scan_group(const int* cseg, int slot) {
    int bound = cseg[0];
    int g = 0;
    while (bound <= slot) {
        ++g;
        bound += cseg[g];
    }
    return g;
}

// Row swizzle shared by the copy and the fragment reads: LDS chunk (row, cc)
// holds k-chunk cc ^ swz(row).  Any 8 (or, two rows per 256 bytes, any 16)
// consecutive rows then hit distinct banks when they read the same k-chunk.
__device__ __forceinline__ int swz(int row) { return (row & 7) ^ ((row >> 3) & 1); }

template <int N>
using template_int = std::integral_constant<int, N>;

// f(integral_constant<0>) ... f(integral_constant<N-1>)
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (N > 0) {
        static_for<N - 1>(f);
        f(template_int<N - 1>{});
    }
}

}  // namespace fo
