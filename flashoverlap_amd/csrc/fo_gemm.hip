// Signalling GEMM for gfx950 (MI355X): D = A . B^T, A [M,K], B [N,K], both with
// K contiguous, 16-bit inputs (fp16 / bf16), fp32 accumulation on MFMA.
//
// One workgroup of 4 wavefronts computes one MT x MT macro tile (MT = 256, or
// 128 for small problems); each wavefront owns an (MT/2) x (MT/2) quadrant as
// (MT/64)^2 blocks of v_mfma_f32_32x32x16.  A and B panels of 64 k-elements
// are streamed HBM -> LDS with global_load_lds_dwordx4 (no register staging)
// into two LDS stages; the 16-byte chunks of a row are XOR-swizzled by row so
// that the ds_read_b128 fragment reads are bank-conflict free.
//
// The epilogue writes the quadrant either to the natural row-major D (plain
// GEMM) or to the slot RA[tile] of the tile-permuted layout, optionally with
// the row index mapped through RE (scatter), and then signals: after every
// wavefront's stores have been acknowledged and the workgroup has met at a
// barrier, one lane per layout tile bumps the tile's group counter with a
// release-ordered, agent-scope atomic.  The plain GEMM is the same kernel
// instantiated with the signalling code compiled out.
//
// Semantics follow the reference epilogues src/overlap/gemm_with_signal.h:145-201
// and src/overlap/gemm_with_scatter.h:146-196; the kernel itself shares nothing
// with the reference's MUTlass mainloop.
#include <hip/hip_runtime.h>

#include "fo_internal.h"
#include "fo_raster.h"

namespace fo {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

template <typename T>
struct Mma;
template <>
struct Mma<_Float16> {
    using frag = f16x8;
    using out4 = f16x4;
    static __device__ __forceinline__ f32x16 run(frag a, frag b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
};
template <>
struct Mma<__bf16> {
    using frag = bf16x8;
    using out4 = bf16x4;
    static __device__ __forceinline__ f32x16 run(frag a, frag b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
};

constexpr int kBK = 64;            // k-elements per LDS stage
constexpr int kRowBytes = kBK * 2; // one tile row in LDS: 128 bytes = 8 chunks of 16

enum { kPlain = 0, kSignal = 1, kScatter = 2 };

struct GemmParams {
    const void* A;
    const void* B;
    void* D;
    int M, N, K;
    int GM, GN;   // macro-tile grid
    int BM, BN;   // layout tile
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
typedef __attribute__((address_space(1))) const void gbl_void;

// One 1 KiB wave-wide copy HBM -> LDS: lane l's 16 bytes land at lds + 16*l.
__device__ __forceinline__ void async_copy16(const void* g, void* lds_wave_base) {
    __builtin_amdgcn_global_load_lds((gbl_void*)g, (lds_void*)lds_wave_base, 16, 0, 0);
}

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

template <typename T, int MT, int MODE>
__global__ void __launch_bounds__(256) gemm_kernel(const GemmParams p) {
    constexpr int WT = MT / 2;          // wave quadrant edge
    constexpr int NB = WT / 32;         // 32x32 MFMA blocks per quadrant edge
    constexpr int PANEL = MT * kRowBytes;   // bytes of one A (or B) panel per stage
    constexpr int STAGE = 2 * PANEL;
    constexpr int LOADS = MT / 32;      // wave-wide 1 KiB copies per wave per panel
    using frag = typename Mma<T>::frag;
    using out4 = typename Mma<T>::out4;

    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;

    const TileCoord mt = raster_map(blockIdx.x, p.GM, p.GN);
    const int K = p.K;

    // ---- where this wavefront's quadrant goes -------------------------------
    // row0/col0/ld describe the destination of quadrant element (0,0) in a
    // row-major view; rows are consecutive in that view (before RE).
    int row0, col0, ld;
    int sig_slot = 0, sig_group = 0;
    if constexpr (MODE == kPlain) {
        row0 = mt.m * MT + wm * WT;
        col0 = mt.n * MT + wn * WT;
        ld = p.N;
    } else {
        const int tiles_n = MT / p.BN;                // layout tiles per macro tile, N
        const int tiles_m = MT / p.BM;
        const int qm = wm * WT, qn = wn * WT;         // quadrant origin in the macro tile
        const int t = (mt.m * tiles_m + qm / p.BM) * p.TN + mt.n * tiles_n + qn / p.BN;
        const int s = __builtin_amdgcn_readfirstlane(p.RA[t]);
        row0 = (s / p.rLDN) * p.BM + qm % p.BM;
        col0 = (s % p.rLDN) * p.BN + qn % p.BN;
        ld = p.rLDN * p.BN;
        // The lanes that will signal look up their slot and group now, so the
        // two dependent loads are hidden behind the main loop.
        const int ntile = tiles_m * tiles_n;
        if (tid < ntile) {
            const int ts = (mt.m * tiles_m + tid / tiles_n) * p.TN + mt.n * tiles_n + tid % tiles_n;
            sig_slot = p.RA[ts];
            sig_group = p.gtable ? p.gtable[sig_slot] : scan_group(p.cseg, sig_slot);
        }
    }

    // ---- global -> LDS copy addressing ---------------------------------------
    // A wave-wide copy fills 64 consecutive 16-byte LDS chunks = 8 tile rows.
    // LDS chunk (row, cc) holds k-chunk cc ^ (row % 8) of that row.
    const int cp_row = lane >> 3;                      // row within the 8-row slab
    const int cp_kc = (lane & 7) ^ cp_row;             // k-chunk this lane fetches
    const T* gA = (const T*)p.A + (size_t)(mt.m * MT + wave * (LOADS * 8) + cp_row) * K + cp_kc * 8;
    const T* gB = (const T*)p.B + (size_t)(mt.n * MT + wave * (LOADS * 8) + cp_row) * K + cp_kc * 8;
    const size_t slab_stride = (size_t)8 * K;          // elements between consecutive slabs
    const int lds_cp = wave * (LOADS * 1024);          // this wave's first slab in a panel

    auto issue_loads = [&](int kt, int stage) {
        unsigned char* sA = smem + stage * STAGE + lds_cp;
        unsigned char* sB = sA + PANEL;
        const T* a = gA + (size_t)kt * kBK;
        const T* b = gB + (size_t)kt * kBK;
#pragma unroll
        for (int j = 0; j < LOADS; ++j) {
            async_copy16(a + j * slab_stride, sA + j * 1024);
            async_copy16(b + j * slab_stride, sB + j * 1024);
        }
    };

    // ---- LDS -> register fragment addressing ----------------------------------
    // MFMA 32x32x16 operand: lane l supplies row l%32, k = 8*(l/32) .. +7.
    const int fr_row = lane & 31, fr_h = lane >> 5, fr_x = lane & 7;
    const int a_lane = (wm * WT + fr_row) * kRowBytes;
    const int b_lane = PANEL + (wn * WT + fr_row) * kRowBytes;
    int ko[4];
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) ko[kk] = ((2 * kk + fr_h) ^ fr_x) * 16;

    f32x16 acc[NB][NB];
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    const int KT = K / kBK;
    issue_loads(0, 0);
    for (int kt = 0; kt < KT; ++kt) {
        // Tile kt has landed for every wave, and every wave is done reading the
        // stage that the next copies overwrite.
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        if (kt + 1 < KT) issue_loads(kt + 1, (kt + 1) & 1);
        const unsigned char* st = smem + (kt & 1) * STAGE;
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
            frag a[NB], b[NB];
#pragma unroll
            for (int i = 0; i < NB; ++i) a[i] = *(const frag*)(st + a_lane + i * (32 * kRowBytes) + ko[kk]);
#pragma unroll
            for (int j = 0; j < NB; ++j) b[j] = *(const frag*)(st + b_lane + j * (32 * kRowBytes) + ko[kk]);
            // Operands swapped (B rows as the MFMA "A" matrix) so that a lane
            // ends up with 4 consecutive n for one m: 8-byte stores.
#pragma unroll
            for (int i = 0; i < NB; ++i)
#pragma unroll
                for (int j = 0; j < NB; ++j) acc[i][j] = Mma<T>::run(b[j], a[i], acc[i][j]);
        }
    }

    // ---- epilogue: registers -> global -----------------------------------------
    // acc[i][j][4q+r] is element m = 32i + l%32, n = 32j + 8q + 4(l/32) + r.
    T* D = (T*)p.D;
#pragma unroll
    for (int i = 0; i < NB; ++i) {
        int row = row0 + 32 * i + fr_row;
        if constexpr (MODE == kScatter) row = p.RE[row];
        T* drow = D + (size_t)row * ld + col0 + 4 * fr_h;
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                out4 o;
#pragma unroll
                for (int r = 0; r < 4; ++r) o[r] = (T)acc[i][j][4 * q + r];
                *(out4*)(drow + 32 * j + 8 * q) = o;
            }
    }

    // ---- signal ---------------------------------------------------------------------
    if constexpr (MODE != kPlain) {
        // Every wave's tile stores are acknowledged by L2 before the barrier;
        // the release on the atomic then writes them back device-wide before
        // the counter moves.
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        const int ntile = (MT / p.BM) * (MT / p.BN);
        if (tid < ntile) {
            __hip_atomic_fetch_add(p.MM + sig_group, 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
            if (p.monitor) {
                const int order =
                    __hip_atomic_fetch_add(p.MM + p.TN - 1, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                p.MM[p.TN + sig_slot] = order;
            }
        }
    }
}

template <typename T, int MT, int MODE>
static int launch_one(const GemmParams& p, hipStream_t stream) {
    constexpr int smem_bytes = 2 * 2 * MT * kRowBytes;
    auto kern = gemm_kernel<T, MT, MODE>;
    static bool configured = false;  // attribute is per function, set once
    if (!configured) {
        FO_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, smem_bytes));
        configured = true;
    }
    hipLaunchKernelGGL(kern, dim3(p.GM * p.GN), dim3(256), smem_bytes, stream, p);
    FO_HIP(hipGetLastError());
    return FO_OK;
}

template <int MODE>
static int launch_mode(int dtype, int macro, const GemmParams& p, hipStream_t stream) {
    if (dtype == FO_F16)
        return macro == 256 ? launch_one<_Float16, 256, MODE>(p, stream) : launch_one<_Float16, 128, MODE>(p, stream);
    return macro == 256 ? launch_one<__bf16, 256, MODE>(p, stream) : launch_one<__bf16, 128, MODE>(p, stream);
}

int choose_macro_tile(int BM, int BN, int M, int N) {
    const bool ok256 = (M % 256 == 0) && (N % 256 == 0) && (256 % BM == 0) && (256 % BN == 0);
    const bool ok128 = (BM == 128 && BN == 128) && (M % 128 == 0) && (N % 128 == 0);
    if (ok256 && ok128) {
        // Small problems: prefer the tile that puts work on more CUs.
        const int wg256 = (M / 256) * (N / 256);
        return wg256 >= 128 ? 256 : 128;
    }
    if (ok256) return 256;
    if (ok128) return 128;
    return 0;
}

int launch_gemm(int mode, int dtype, int algo, int M, int N, int K, int rLDN, const int* cseg, int G,
                const int* gtable, const void* A, const void* B, void* D, int* MM, const int* RA,
                const int* RE, int monitor, hipStream_t stream) {
    int BM, BN, BK;
    if (algo_tile(algo, &BM, &BN, &BK) != FO_OK) return fail(FO_ERR_ARG, "fo_gemm: Algo %d out of range", algo);
    if (dtype != FO_F16 && dtype != FO_BF16) return fail(FO_ERR_ARG, "fo_gemm: dtype %d not fp16/bf16", dtype);
    if (!A || !B || !D) return fail(FO_ERR_ARG, "fo_gemm: null operand");
    if (M <= 0 || N <= 0 || K <= 0) return fail(FO_ERR_SHAPE, "fo_gemm: empty problem %dx%dx%d", M, N, K);
    if (M % BM || N % BN) return fail(FO_ERR_SHAPE, "fo_gemm: M=%d N=%d not multiples of the %dx%d tile", M, N, BM, BN);
    if (K % kBK) return fail(FO_ERR_SHAPE, "fo_gemm: K=%d not a multiple of %d", K, kBK);
    if ((long long)M * N >= (1LL << 31)) return fail(FO_ERR_LIMIT, "fo_gemm: M*N=%lld needs 64-bit tile offsets", (long long)M * N);
    if (((uintptr_t)A | (uintptr_t)B | (uintptr_t)D) & 15) return fail(FO_ERR_ARG, "fo_gemm: operands must be 16-byte aligned");
    const int macro = choose_macro_tile(BM, BN, M, N);
    if (!macro) return fail(FO_ERR_SHAPE, "fo_gemm: M=%d N=%d unsupported for tile %dx%d (need multiples of 256, or 128 with the 128x128 tile)", M, N, BM, BN);

    GemmParams p{};
    p.A = A; p.B = B; p.D = D;
    p.M = M; p.N = N; p.K = K;
    p.GM = M / macro; p.GN = N / macro;
    p.BM = BM; p.BN = BN; p.TN = N / BN;
    p.rLDN = rLDN;
    p.RA = RA; p.RE = RE; p.cseg = cseg; p.G = G; p.gtable = gtable; p.MM = MM; p.monitor = monitor;

    if (mode != kPlain) {
        if (!MM || !RA || !cseg) return fail(FO_ERR_ARG, "fo_gemm_signal: null MM/RA/cSeg");
        if (G <= 0) return fail(FO_ERR_ARG, "fo_gemm_signal: G=%d", G);
        const int T = (M / BM) * (N / BN);
        if (rLDN <= 0 || T % rLDN) return fail(FO_ERR_SHAPE, "fo_gemm_signal: rLDN=%d must divide the %d tiles", rLDN, T);
        if (mode == kScatter && !RE) return fail(FO_ERR_ARG, "fo_gemm_scatter: null RE");
    }
    switch (mode) {
        case kPlain: return launch_mode<kPlain>(dtype, macro, p, stream);
        case kSignal: return launch_mode<kSignal>(dtype, macro, p, stream);
        default: return launch_mode<kScatter>(dtype, macro, p, stream);
    }
}

int raster_hint(int algo, int M, int N, int* hint) {
    int BM, BN, BK;
    if (algo_tile(algo, &BM, &BN, &BK) != FO_OK) return fail(FO_ERR_ARG, "fo_raster_hint: Algo %d out of range", algo);
    if (!hint) return fail(FO_ERR_ARG, "fo_raster_hint: null hint");
    if (M <= 0 || N <= 0 || M % BM || N % BN) return fail(FO_ERR_SHAPE, "fo_raster_hint: M=%d N=%d vs tile %dx%d", M, N, BM, BN);
    const int macro = choose_macro_tile(BM, BN, M, N);
    if (!macro) return fail(FO_ERR_SHAPE, "fo_raster_hint: M=%d N=%d unsupported for tile %dx%d", M, N, BM, BN);
    const int GM = M / macro, GN = N / macro, TN = N / BN;
    const int tiles_m = macro / BM, tiles_n = macro / BN;
    int k = 0;
    for (int pid = 0; pid < GM * GN; ++pid) {
        const TileCoord c = raster_map(pid, GM, GN);
        for (int i = 0; i < tiles_m; ++i)
            for (int j = 0; j < tiles_n; ++j) hint[k++] = (c.m * tiles_m + i) * TN + c.n * tiles_n + j;
    }
    return FO_OK;
}

}  // namespace fo
