// RMSNorm and reorder+RMSNorm for gfx950: one 64-lane wavefront per output row,
// the whole row held in registers between the sum of squares and the scaling,
// 128-bit coalesced HBM accesses, a wavefront butterfly for the reduction (no
// LDS in the reduction).  gamma is staged in LDS once per workgroup while the rows' loads
// are in flight and read from there chunk by chunk behind the reduction: held in registers
// beside the row it doubled the kernel's footprint (81 registers at dim 4096, 330 at 16384:
// a single wavefront per SIMD), and the registers decide how many rows a SIMD has in
// flight.  (Rows of more
// than 16384 elements take a second kernel: one workgroup per row, two passes.)  The reorder
// variant gathers the row from the tile-permuted GEMM output: 16 consecutive
// lanes read one 256-byte row segment of a 128-wide tile, so every access is
// made of whole cache lines.  In the common case (rldn == 1, power-of-two tile,
// at most 64 tiles per row) each lane fetches one RA entry and the lanes
// exchange them, so the gather costs one small load instead of one per chunk.
//
// Arithmetic follows src/rmsnorm/rmsnorm.cuh:62-115 of the reference: fp32 sum
// of squares, scale = rsqrt(sum/dim + eps), the scaled value rounded to the
// storage type and then multiplied by gamma in the storage type (the product
// of two 16-bit floats is exact in fp32, so rounding it once equals the
// reference's half-precision multiply).  eps is a parameter here.
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include "fo_internal.h"

namespace fo {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

template <typename T>
struct Vec8;
template <>
struct Vec8<_Float16> {
    using type = f16x8;
};
template <>
struct Vec8<__bf16> {
    using type = bf16x8;
};

constexpr int kRowsPerBlock = 4;  // one wavefront per row; neighbouring rows read neighbouring tile segments
constexpr int kWideThreads = 256;  // rows too long for one wavefront's registers: one workgroup per row

// Ordinary loads, streaming (non-temporal) stores: the result is not read again here, and it
// must not displace the GEMM operands held in the memory-side cache.  Measured on 8192 x 4096
// against this choice (inside a step / one buffer pair back to back, 21.8 / 21.7 us as it is):
// non-temporal loads 21.8 / 25.5, ordinary stores 23.9 / 22.2; the other cache-policy bits on the
// stores (sc1, sc0 sc1, with and without nt) equal or slower.
template <typename V>
__device__ __forceinline__ V load_row_chunk(const V* p) {
    return *p;
}
template <typename V>
__device__ __forceinline__ void store_row_chunk(V v, V* p) {
    __builtin_nontemporal_store(v, p);
}

enum { kNormPlain = 0, kNormGather = 1, kNormGatherFast = 2 };

struct NormParams {
    int bs, dim, BM, BN, rldn;
    int log_bm, log_bn;  // kNormGatherFast only
    float eps;
};

// CH = 16-byte chunks per lane (dim <= CH * 512).  GAMMA_IN_LDS: see the head of the file; measured per CH
// (reorder / plain, against gamma in registers, same box): CH 2 -3 % / -13 %, CH 4 -4 % / +3 %, CH 8 -1...-7 % /
// -8 %, CH 32 -37 % / -10 %, but CH 16 +2 % / +4 % on 16384 x 8192 (more rows in flight than that size likes),
// so CH 16 keeps gamma in registers.
template <int CH>
constexpr bool gamma_in_lds() { return CH != 16; }

template <typename T, int CH, int MODE>
__global__ void __launch_bounds__(64 * kRowsPerBlock) rmsnorm_kernel(const T* __restrict__ x0, const T* __restrict__ gamma,
                                                      T* __restrict__ out0, const int* __restrict__ RA,
                                                      const NormParams p) {
    using vec = typename Vec8<T>::type;
    constexpr bool GAMMA_IN_LDS = gamma_in_lds<CH>();
    extern __shared__ __attribute__((aligned(16))) unsigned char norm_smem[];   // dim * 2 bytes when gamma is staged
    vec* lds_gamma = (vec*)norm_smem;
    const int lane = threadIdx.x & 63;
    const int row_of_wave = blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6);
    const bool live = row_of_wave < p.bs;
    if (!GAMMA_IN_LDS && !live) return;
    const int row = live ? row_of_wave : p.bs - 1;   // a wavefront beyond the last row stays for the barrier, loading a row it never stores
    // blockIdx.y selects one of several independent [bs, dim] problems laid out back to back
    const T* __restrict__ x = x0 + (size_t)blockIdx.y * p.bs * p.dim;
    T* __restrict__ out = out0 + (size_t)blockIdx.y * p.bs * p.dim;

    const int dim = p.dim;
    const int nchunk = dim >> 3;
    vec xv[CH];
    [[maybe_unused]] vec gv[GAMMA_IN_LDS ? 1 : CH];
    if constexpr (MODE == kNormGatherFast) {
        // tiles of this row: RA[tile_row .. tile_row + ldn), ldn <= 64: one entry per lane
        const int ldn = dim >> p.log_bn;
        const int tile_row = (row >> p.log_bm) * ldn;
        const int in_row = row & (p.BM - 1);
        const int mine = RA[tile_row + (lane < ldn ? lane : 0)];
#pragma unroll
        for (int k = 0; k < CH; ++k) {
            const int c = k * 64 + lane;
            const int j = c << 3;
            const int s = __shfl(mine, (j >> p.log_bn) & 63, 64);  // all lanes take part in the exchange
            if (c < nchunk) {
                const size_t src = ((((size_t)s << p.log_bm) + in_row) << p.log_bn) + (j & (p.BN - 1));
                xv[k] = load_row_chunk((const vec*)(x + src));
            }
        }
    } else if constexpr (MODE == kNormGather) {
        const int ldn = dim / p.BN;
        const int tile_row = (row / p.BM) * ldn;
        const int in_row = row % p.BM;
        const int ld = p.rldn * p.BN;
#pragma unroll
        for (int k = 0; k < CH; ++k) {
            const int c = k * 64 + lane;
            if (c < nchunk) {
                const int j = c << 3;
                const int s = RA[tile_row + j / p.BN];
                const size_t src = (size_t)((s / p.rldn) * p.BM + in_row) * ld + (s % p.rldn) * p.BN + j % p.BN;
                xv[k] = load_row_chunk((const vec*)(x + src));
            }
        }
    } else {
        const T* xr = x + (size_t)row * dim;
#pragma unroll
        for (int k = 0; k < CH; ++k) {
            const int c = k * 64 + lane;
            if (c < nchunk) xv[k] = load_row_chunk((const vec*)(xr + (c << 3)));
        }
    }
    if constexpr (GAMMA_IN_LDS) {
        for (int c = threadIdx.x; c < nchunk; c += 64 * kRowsPerBlock) lds_gamma[c] = *(const vec*)(gamma + (c << 3));
        __syncthreads();
        if (!live) return;
    } else {
#pragma unroll
        for (int k = 0; k < CH; ++k) {
            const int c = k * 64 + lane;
            if (c < nchunk) gv[k] = *(const vec*)(gamma + (c << 3));
        }
    }

    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < CH; ++k) {
        if (k * 64 + lane < nchunk) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float f = (float)xv[k][e];
                ss += f * f;
            }
        }
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) ss += __shfl_xor(ss, off, 64);
    const float scale = rsqrtf(ss / (float)dim + p.eps);
    // The row stays packed in its 16-bit form across the reduction; without this
    // the fp32 copies made for the sum of squares are kept alive too, which
    // doubles the register footprint and halves the waves per SIMD.
#pragma unroll
    for (int k = 0; k < CH; ++k) asm volatile("" : "+v"(xv[k]));

    T* orow = out + (size_t)row * dim;
#pragma unroll
    for (int k = 0; k < CH; ++k) {
        const int c = k * 64 + lane;
        if (c < nchunk) {
            vec o, g;
            if constexpr (GAMMA_IN_LDS) g = lds_gamma[c];
            else g = gv[k];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const T y = (T)((float)xv[k][e] * scale);
                o[e] = (T)((float)y * (float)g[e]);
            }
            store_row_chunk(o, (vec*)(orow + (c << 3)));
        }
    }
}

// Rows longer than a wavefront keeps in registers (dim > 16384): one workgroup per row, two passes.
// The first pass sums the squares, the four wavefronts' partial sums meet in LDS (added in a fixed
// order), the second pass reads the row again (it is at most a few hundred KiB and still in the L2)
// and writes the result.  Same arithmetic per element as above; any dim that is a multiple of 8.
template <typename T, int MODE>
__global__ void __launch_bounds__(kWideThreads) rmsnorm_wide_kernel(const T* __restrict__ x0, const T* __restrict__ gamma,
                                                                  T* __restrict__ out0, const int* __restrict__ RA,
                                                                  const NormParams p) {
    static_assert(MODE == kNormPlain || MODE == kNormGather, "rows this long have more than 64 tiles");
    using vec = typename Vec8<T>::type;
    __shared__ float part[kWideThreads / 64];
    const int row = blockIdx.x;
    const T* __restrict__ x = x0 + (size_t)blockIdx.y * p.bs * p.dim;
    T* __restrict__ orow = out0 + (size_t)blockIdx.y * p.bs * p.dim + (size_t)row * p.dim;
    const int dim = p.dim, nchunk = dim >> 3;
    [[maybe_unused]] const int ldn = MODE == kNormGather ? dim / p.BN : 0;
    [[maybe_unused]] const int tile_row = MODE == kNormGather ? (row / p.BM) * ldn : 0;
    [[maybe_unused]] const int in_row = MODE == kNormGather ? row % p.BM : 0;
    auto chunk_at = [&](int c) -> const vec* {
        const int j = c << 3;
        if constexpr (MODE == kNormGather) {
            const int s = RA[tile_row + j / p.BN];
            return (const vec*)(x + (size_t)((s / p.rldn) * p.BM + in_row) * (p.rldn * p.BN) + (s % p.rldn) * p.BN + j % p.BN);
        } else {
            return (const vec*)(x + (size_t)row * dim + j);
        }
    };
    float ss = 0.f;
#pragma unroll 4
    for (int c = threadIdx.x; c < nchunk; c += kWideThreads) {
        const vec v = *chunk_at(c);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float f = (float)v[e];
            ss += f * f;
        }
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) ss += __shfl_xor(ss, off, 64);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
    __syncthreads();
    float total = part[0];
#pragma unroll
    for (int w = 1; w < kWideThreads / 64; ++w) total += part[w];
    const float scale = rsqrtf(total / (float)dim + p.eps);
#pragma unroll 4
    for (int c = threadIdx.x; c < nchunk; c += kWideThreads) {
        const vec v = *chunk_at(c);
        const vec g = *(const vec*)(gamma + (c << 3));
        vec o;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const T y = (T)((float)v[e] * scale);
            o[e] = (T)((float)y * (float)g[e]);
        }
        store_row_chunk(o, (vec*)(orow + (c << 3)));
    }
}

static int log2_exact(int v) {
    if (v <= 0 || (v & (v - 1))) return -1;
    int l = 0;
    while ((1 << l) < v) ++l;
    return l;
}

template <typename T, int MODE>
static int launch_wide(const void* x, const void* gamma, void* out, const int* RA, const NormParams& p, int nbatch,
                       const LaunchTimer& timer, hipStream_t stream) {
    const dim3 grid(p.bs, nbatch), block(kWideThreads);
    if (timer.start)
        hipExtLaunchKernelGGL((rmsnorm_wide_kernel<T, MODE>), grid, block, 0, stream, timer.start, timer.stop, 0,
                              (const T*)x, (const T*)gamma, (T*)out, RA, p);
    else
        hipLaunchKernelGGL((rmsnorm_wide_kernel<T, MODE>), grid, block, 0, stream, (const T*)x, (const T*)gamma, (T*)out,
                           RA, p);
    FO_HIP(hipGetLastError());
    return FO_OK;
}

template <typename T, int MODE>
static int launch_t(const void* x, const void* gamma, void* out, const int* RA, const NormParams& p, int nbatch,
                    const LaunchTimer& timer, hipStream_t stream) {
    const int ch = (p.dim / 8 + 63) / 64;
    if (ch > 32) {   // beyond what a wavefront keeps in registers
        if constexpr (MODE == kNormGatherFast) return fail(FO_ERR_SHAPE, "fo_reorder_rmsnorm: dim=%d", p.dim);   // not selected for such rows
        else return launch_wide<T, MODE>(x, gamma, out, RA, p, nbatch, timer, stream);
    }
    const dim3 grid((p.bs + kRowsPerBlock - 1) / kRowsPerBlock, nbatch), block(64 * kRowsPerBlock);
#define FO_RMS_CASE(CH)                                                                                           \
    do {                                                                                                          \
        const size_t smem = gamma_in_lds<CH>() ? (size_t)p.dim * sizeof(T) : 0;                                   \
        if (timer.start)                                                                                          \
            hipExtLaunchKernelGGL((rmsnorm_kernel<T, CH, MODE>), grid, block, smem, stream, timer.start,          \
                                  timer.stop, 0, (const T*)x, (const T*)gamma, (T*)out, RA, p);                   \
        else                                                                                                      \
            hipLaunchKernelGGL((rmsnorm_kernel<T, CH, MODE>), grid, block, smem, stream, (const T*)x,             \
                               (const T*)gamma, (T*)out, RA, p);                                                  \
    } while (0)
    if (ch <= 1) FO_RMS_CASE(1);
    else if (ch <= 2) FO_RMS_CASE(2);
    else if (ch <= 4) FO_RMS_CASE(4);
    else if (ch <= 8) FO_RMS_CASE(8);
    else if (ch <= 16) FO_RMS_CASE(16);
    else FO_RMS_CASE(32);
#undef FO_RMS_CASE
    FO_HIP(hipGetLastError());
    return FO_OK;
}

template <typename T>
static int launch_dtype(const void* x, const void* gamma, void* out, const int* RA, const NormParams& p, int nbatch,
                        const LaunchTimer& timer, hipStream_t stream) {
    if (!RA) return launch_t<T, kNormPlain>(x, gamma, out, RA, p, nbatch, timer, stream);
    if (p.log_bm >= 0) return launch_t<T, kNormGatherFast>(x, gamma, out, RA, p, nbatch, timer, stream);
    return launch_t<T, kNormGather>(x, gamma, out, RA, p, nbatch, timer, stream);
}

int launch_rmsnorm(int dtype, const void* x, const void* gamma, void* out, int nbatch, int bs, int dim, int BM,
                   int BN, int rldn, const int* RA, float eps, hipStream_t stream) {
    const bool reorder = RA != nullptr;
    const char* who = reorder ? "fo_reorder_rmsnorm" : "fo_rmsnorm";
    // an event pair armed by fo_time_next_launch is this call's, whether or not it gets as far as a launch
    const LaunchTimer timer = t_launch_timer;
    t_launch_timer = LaunchTimer{};
    if (dtype != FO_F16 && dtype != FO_BF16) return fail(FO_ERR_ARG, "%s: dtype %d not fp16/bf16", who, dtype);
    if (bs == 0 || nbatch == 0) return FO_OK;
    if (nbatch < 0 || nbatch > 65535) return fail(FO_ERR_LIMIT, "%s: %d batches outside 0..65535", who, nbatch);
    if (!x || !gamma || !out) return fail(FO_ERR_ARG, "%s: null buffer", who);
    if (bs < 0 || dim <= 0) return fail(FO_ERR_SHAPE, "%s: bs=%d dim=%d", who, bs, dim);
    if (dim % 8) return fail(FO_ERR_SHAPE, "%s: dim=%d not a multiple of 8", who, dim);
    if ((long long)bs * dim * nbatch >= (1LL << 40)) return fail(FO_ERR_LIMIT, "%s: %lld elements", who, (long long)bs * dim * nbatch);
    if (((uintptr_t)x | (uintptr_t)gamma | (uintptr_t)out) & 15) return fail(FO_ERR_ARG, "%s: buffers must be 16-byte aligned", who);
    NormParams p{bs, dim, BM, BN, rldn, -1, -1, eps};
    if (reorder) {
        if (BM <= 0 || BN <= 0 || rldn <= 0) return fail(FO_ERR_ARG, "%s: BM=%d BN=%d rldn=%d", who, BM, BN, rldn);
        if (BN % 8 || dim % BN) return fail(FO_ERR_SHAPE, "%s: BN=%d must be a multiple of 8 that divides dim=%d", who, BN, dim);
        if (bs % BM) return fail(FO_ERR_SHAPE, "%s: bs=%d not a multiple of BM=%d", who, bs, BM);
        if (((long long)(bs / BM) * (dim / BN)) % rldn) return fail(FO_ERR_SHAPE, "%s: rldn=%d must divide the tile count", who, rldn);
        if (rldn == 1 && dim / BN <= 64 && dim <= 32 * 512 && log2_exact(BM) >= 0 && log2_exact(BN) >= 0) {
            p.log_bm = log2_exact(BM);
            p.log_bn = log2_exact(BN);
        }
    }
    if (dtype == FO_F16) return launch_dtype<_Float16>(x, gamma, out, RA, p, nbatch, timer, stream);
    return launch_dtype<__bf16>(x, gamma, out, RA, p, nbatch, timer, stream);
}

}  // namespace fo
