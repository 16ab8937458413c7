// Signalling GEMM for gfx950 (MI355X): D = A . B^T, A [M,K], B [N,K], both with
// K contiguous, 16-bit inputs (fp16 / bf16), fp32 accumulation on MFMA.
//
// One workgroup of 4 wavefronts computes one MT x MT macro tile (MT = 256, or
// 128 for small problems); each wavefront owns an (MT/2) x (MT/2) quadrant as
// (MT/32)^2 blocks of v_mfma_f32_16x16x32, accumulators in AGPRs.  The 16x16x32
// form reads and writes a quarter of the accumulator registers per flop of the
// 32x32x16 form (the k-reduction of 32 happens inside the instruction); the
// chip runs this kernel at its power limit, and the kernel measured 3-4 %
// faster with it.  The MFMAs are issued through inline assembly with the
// accumulators pinned to AGPRs: with the compiler builtin the register
// allocator moved 16x16 accumulators between the two register files inside
// the main loop.  The order of the main loop's instructions is therefore
// written out slot by slot in the source and fenced, not left to the scheduler.
//
// Main loop: A and B panels of 64 k-elements stream HBM -> LDS with
// buffer_load_dwordx4 ... lds (no register staging) into a ring of five panel
// slots (all of the 160 KiB of LDS at MT = 256): the A and B panels of the
// k-step being multiplied, those of the next one, and one free slot.  A panel
// row is 128 bytes, so every copy instruction fetches eight whole cache lines:
// the L2 serves one request per channel per clock whatever its size, and at
// this tile size the kernel sits at the edge of that request rate, so half-line
// requests cost a quarter of the throughput.  The 16-byte chunks of a row are
// XOR-swizzled by row so the ds_read_b128 fragment reads are bank-conflict
// free.  A k-step of 64 is two half steps of 64 MFMAs, each over half the rows
// of blocks and walked column by column, with the two MFMAs that an
// accumulator gets from the panel (k halves 0 and 1) issued back to back: the
// second then takes the running sum from inside the matrix core instead of
// from the register file, which lowers the power per flop and with it raises
// the clock the power limit allows.  All B fragments of the panel stay in
// registers for the whole k-step and are replaced, column by column, by those
// of the next panel during the second half step; the A fragments of the
// second half step are read during the first, so all reads of a panel are out
// by the middle of its k-step, where the workgroup barrier that releases the
// panel's two slots sits.  The free slot lets the copies of A(p+2) go out in
// the first half of k-step p and those of B(p+2) in the second half, one
// every few MFMAs, with more than a k-step to land, which is what the kernel
// needs when its operands come from HBM and not from the memory-side cache.
// There is one barrier per k-step.
//
// Epilogue: the quadrant goes through LDS in strips of 32 rows so that every
// global store instruction writes four whole 256-byte row segments, either to
// the natural row-major D (plain GEMM) or to slot RA[tile] of the
// tile-permuted layout, optionally with the row index mapped through RE
// (scatter).  Then the signal: after every wavefront's stores have been
// acknowledged and the workgroup has met at a barrier, one lane per layout
// tile bumps the tile's group counter with an agent-scope atomic.  The tile
// stores are agent-scope write-through stores (sc1), the instruction the
// compiler emits for an agent-scope atomic store: once s_waitcnt vmcnt(0)
// returns they have been performed at agent scope, so nothing dirty is left in
// this XCD's L2 for a release to write back, and the counter atomic can be a
// relaxed one.  (The release-ordered form, cached stores or not, is kept as a
// tuning knob: its buffer_wbl2 costs 3-10 % of a short-K GEMM.)  The plain
// GEMM is the same kernel with the signalling compiled out.
//
// Semantics follow the reference epilogues src/overlap/gemm_with_signal.h:145-201
// and src/overlap/gemm_with_scatter.h:146-196; the kernel itself shares nothing
// with the reference's MUTlass mainloop.
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <atomic>
#include <string_view>
#include <type_traits>

#include "fo_gemm_common.h"
#include "fo_internal.h"
#include "fo_knobs.h"
#include "fo_raster.h"

namespace fo {

// STORE: 0 cached, 1 write-through tile stores; REL: 0 release atomic, 1 relaxed atomic.
// EDGE (plain GEMM only): M and N are arbitrary; the rows and columns of a macro tile that lie
// outside the matrix are computed on zeros and not stored.
template <typename T, int MT, int MODE, int STORE, int REL, bool EDGE = false>
__global__ void __launch_bounds__(256) gemm_kernel(const GemmParams p) {
    static_assert(!EDGE || MODE == kPlain, "only the plain GEMM takes shapes that are not multiples of the layout tile");
    constexpr int WT = MT / 2;               // wave quadrant edge
    constexpr int NB = WT / 16;              // 16x16 MFMA blocks per quadrant edge
    constexpr int NH = NB / 2;               // rows of blocks per half step
    constexpr int PANEL = MT * kRowBytes;    // bytes of one A (or B) panel = one LDS slot
    constexpr int LOADS = MT / 32;           // wave-wide 1 KiB copies per wave per panel
    constexpr int LPT = 2 * LOADS;           // copies per wave per k-step
    constexpr int HALF = LPT / 2;
    constexpr int BLK = 16 * kRowBytes;      // LDS bytes between 16-row blocks
    using frag = typename Mma<T>::frag;
    using out4 = typename Mma<T>::out4;

    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;

    const TileCoord mt = raster_map(blockIdx.x, p.GM, p.GN, p.gn_magic);
    const int K = p.K;
    // M and N are multiples of the layout tile, not necessarily of the macro
    // tile: the last row or column of macro tiles may be half inside.  Such a
    // workgroup runs the full main loop (the waves of the outer half re-read the
    // panel rows of the inner half, so nothing outside the operands is touched)
    // and only the quadrants inside are stored and signalled.  EDGE: M and N are
    // arbitrary; the panel rows beyond the matrix are zero-filled by the
    // hardware (see the copy addressing below) and only the rows and columns
    // inside the matrix are stored.
    const int valid_m = min(MT, p.M - mt.m * MT), valid_n = min(MT, p.N - mt.n * MT);
    const bool live = wm * WT < valid_m && wn * WT < valid_n;                          // this wave's quadrant

    // ---- where this wavefront's quadrant goes -------------------------------
    // row0/col0/ld describe the destination of quadrant element (0,0) in a
    // row-major view; rows are consecutive in that view (before RE).  In the
    // signalling modes they follow from the slot of the quadrant's layout tile.
    // The slots (this wave's, and in the lanes that will signal that of "their"
    // layout tile) are fetched here, ahead of the first panel copies, but looked at
    // only behind the prologue's barrier, when they have long arrived: nothing may
    // stand between the start of the kernel and the issue of those copies.  What
    // depends on the slots (group, remapped rows) is fetched there too, under the
    // first k-steps.
    int row0 = mt.m * MT + wm * WT, col0 = mt.n * MT + wn * WT, ld = p.N;
    int sig_slot = 0, sig_group = -1;   // -1: a lane without a layout tile inside the matrix stays out of the signal
    [[maybe_unused]] int quad_slot = 0;
    [[maybe_unused]] bool sig_lane = false;
    if constexpr (MODE != kPlain) {
        const int tiles_n = MT >> p.log_bn;           // layout tiles per macro tile, N
        const int tiles_m = MT >> p.log_bm;
        const int qm = wm * WT, qn = wn * WT;         // quadrant origin in the macro tile
        if (live) quad_slot = p.RA[(mt.m * tiles_m + (qm >> p.log_bm)) * p.TN + mt.n * tiles_n + (qn >> p.log_bn)];
        const int sig_m = tiles_n == 2 ? tid >> 1 : tid, sig_n = tiles_n == 2 ? tid & 1 : 0;   // tiles_n is 1 or 2
        sig_lane = tid < tiles_m * tiles_n && (sig_m << p.log_bm) < valid_m && (sig_n << p.log_bn) < valid_n;
        if (sig_lane) sig_slot = p.RA[(mt.m * tiles_m + sig_m) * p.TN + mt.n * tiles_n + sig_n];
    }
    [[maybe_unused]] int re_lo = 0, re_hi = 0;   // scatter: the remapped destination rows of this quadrant
    auto resolve_destination = [&]() {
        if constexpr (MODE != kPlain) {
            const int s = __builtin_amdgcn_readfirstlane(quad_slot);
            row0 = (s / p.rLDN) * p.BM + ((wm * WT) & (p.BM - 1));
            col0 = (s % p.rLDN) * p.BN + ((wn * WT) & (p.BN - 1));
            ld = p.rLDN * p.BN;
            if (sig_lane) sig_group = p.gtable ? p.gtable[sig_slot] : scan_group(p.cseg, sig_slot);
        }
        // Scatter: one or two remapped rows per lane, handed round between the lanes in the epilogue.
        if constexpr (MODE == kScatter) {
            re_lo = p.RE[row0 + (lane < WT ? lane : 0)];
            if constexpr (WT > 64) re_hi = p.RE[row0 + 64 + lane];
        }
    };

    // ---- HBM -> LDS copy addressing ------------------------------------------
    // One copy instruction moves 1 KiB = 8 panel rows of 128 bytes: lane l's 16
    // bytes land at the LDS base + 16*l, i.e. row l/8, chunk l%8 of the slab, and
    // are fetched from k-chunk (l%8) ^ swz(row).  Buffer addressing: the operand
    // is the buffer, the wave-uniform part of the offset (panel row, slab, k)
    // lives in a scalar register and only the constant per-lane part in a vector
    // register, so a copy costs no vector ALU work.  Slabs alternate in bit 3 of
    // the row number, hence two per-lane offsets.
    const int cp_row = lane >> 3;
    const int cp_off0 = (cp_row * K + ((lane & 7) ^ swz(cp_row)) * 8) * 2;       // even slabs
    const int cp_off1 = (cp_row * K + ((lane & 7) ^ swz(cp_row + 8)) * 8) * 2;   // odd slabs
    // K need not be a multiple of the panel depth.  In the last, partial panel the
    // lanes whose k-chunk lies beyond K take a per-lane offset outside the buffer's
    // range instead: the hardware then fetches nothing for them and writes zeros to
    // their LDS bytes, so the panel is zero-padded and the main loop needs no k
    // mask.  The range (2 GiB, checked against the operand sizes on the host) only
    // has to separate that one offset from the real ones.
    const int k_rest = K % kBK;
    constexpr int kOutOfRange = (int)0x80000000u;
    int tail_off0 = cp_off0, tail_off1 = cp_off1;
    if (k_rest) {
        if (((lane & 7) ^ swz(cp_row)) * 8 >= k_rest) tail_off0 = kOutOfRange;
        if (((lane & 7) ^ swz(cp_row + 8)) * 8 >= k_rest) tail_off1 = kOutOfRange;
    }
    int vo0 = cp_off0, vo1 = cp_off1;   // the offsets in use: the tail pair for the last panel
    const int range = k_rest ? kOutOfRange : (int)0xffffffffu;
    // EDGE: the hardware checks only the per-lane part of an offset against the descriptor's range.
    // So the descriptor of an operand starts at the macro tile's first row and ends with the operand,
    // the row inside the tile goes into the per-lane part (one addition per copy) and only the k
    // position stays scalar: a lane whose row lies beyond the matrix is then out of range, fetches
    // nothing and gets zeros, whatever M and N are.
    const __amdgpu_buffer_rsrc_t rsrcA =
        EDGE ? __builtin_amdgcn_make_buffer_rsrc((char*)p.A + (size_t)mt.m * MT * K * 2, 0,
                                                 (int)((unsigned)(p.M - mt.m * MT) * (unsigned)K * 2u), 0x00020000)
             : __builtin_amdgcn_make_buffer_rsrc((void*)p.A, 0, range, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrcB =
        EDGE ? __builtin_amdgcn_make_buffer_rsrc((char*)p.B + (size_t)mt.n * MT * K * 2, 0,
                                                 (int)((unsigned)(p.N - mt.n * MT) * (unsigned)K * 2u), 0x00020000)
             : __builtin_amdgcn_make_buffer_rsrc((void*)p.B, 0, range, 0x00020000);
    const unsigned baseA = EDGE ? (unsigned)(wave * (LOADS * 8)) * (unsigned)K * 2u
                                : (unsigned)(mt.m * MT + ((wave * (LOADS * 8)) & (valid_m - 1))) * (unsigned)K * 2u;
    const unsigned baseB = EDGE ? (unsigned)(wave * (LOADS * 8)) * (unsigned)K * 2u
                                : (unsigned)(mt.n * MT + ((wave * (LOADS * 8)) & (valid_n - 1))) * (unsigned)K * 2u;
    const unsigned slab_bytes = 8u * (unsigned)K * 2u;    // bytes between consecutive slabs
    const int lds_cp = wave * (LOADS * 1024);             // this wave's first slab in a panel

    // The LDS is a ring of five panel slots.  Panel units alternate A(0) B(0)
    // A(1) B(1) ...; unit u lives in slot u % 5.  `slot` is the byte offset of
    // the receiving slot; the copies of a unit are issued in two halves.
    auto issue_unit = [&](int kt, int slot, auto isb_c, auto half_c) {
        constexpr bool ISB = decltype(isb_c)::value;
        constexpr int H = decltype(half_c)::value;
        unsigned char* dst = smem + slot + lds_cp;
        const unsigned koff = (unsigned)kt * (kBK * 2);
#pragma unroll
        for (int j = H * (LOADS / 2); j < (H + 1) * (LOADS / 2); ++j) {
            const int voff = (j & 1) ? vo1 : vo0;   // LOADS*8 is a multiple of 16: slab parity = j parity
            const unsigned rows = (ISB ? baseB : baseA) + j * slab_bytes;   // the slab's first row, in bytes
            if constexpr (ISB)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrcB, (lds_void*)(dst + j * 1024), 16, EDGE ? (int)((unsigned)voff + rows) : voff,
                                                         (int)(EDGE ? koff : rows + koff), 0, 0);
            else
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrcA, (lds_void*)(dst + j * 1024), 16, EDGE ? (int)((unsigned)voff + rows) : voff,
                                                         (int)(EDGE ? koff : rows + koff), 0, 0);
        }
    };
    std::false_type unit_a;
    std::true_type unit_b;

    // ---- LDS -> register fragment addressing ----------------------------------
    // MFMA 16x16x32 operand: lane l supplies row l%16 and the 8 k-values of lane
    // group l/16.  Which 8 of the k half's 32 a group takes is free as long as A
    // and B agree; groups 0..3 take the 16-byte chunks 0, 2, 1, 3.  The LDS
    // serves lanes l and l+32 in the same pass: this way the two read
    // neighbouring chunks of one row, which the row swizzle keeps on different
    // banks (chunks 0 and 2 of the same rows would collide two ways).
    const int fr_row = lane & 15, fr_g = lane >> 4;
    const int fr_kc = (fr_g & 1) * 2 + (fr_g >> 1);
    const int a_lane = (wm * WT + fr_row) * kRowBytes;
    const int b_lane = (wn * WT + fr_row) * kRowBytes;
    int ko[2];   // chunk offset of each k half (k 0..31, 32..63)
#pragma unroll
    for (int h = 0; h < 2; ++h) ko[h] = ((4 * h + fr_kc) ^ swz(fr_row)) * 16;

    f32x4 acc[NB][NB];   // cleared in the prologue, while the first panels are on their way

    // Fragments of the two k halves of a panel.  The B blocks of both halves stay in registers for
    // the whole k-step; the A blocks come in two sets, rows of blocks 0..NH-1 for the first half of
    // the k-step and NH..NB-1 for the second.
    frag fa[2][NB], fb[2][NB];   // [k half][block]

    const int NP = (K + kBK - 1) / kBK;   // panels, the last one possibly partial
    // One copy instruction (slab j of the A or B unit of panel kt) into slot `slot`.
    auto issue_one = [&](int kt, int slot, auto isb_c, auto j_c) {
        constexpr bool ISB = decltype(isb_c)::value;
        constexpr int j = decltype(j_c)::value;
        unsigned char* dst = smem + slot + lds_cp;
        const unsigned koff = (unsigned)kt * (kBK * 2);
        const int voff = (j & 1) ? vo1 : vo0;
        const unsigned rows = (ISB ? baseB : baseA) + j * slab_bytes;
        if constexpr (ISB)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrcB, (lds_void*)(dst + j * 1024), 16, EDGE ? (int)((unsigned)voff + rows) : voff,
                                                     (int)(EDGE ? koff : rows + koff), 0, 0);
        else
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrcA, (lds_void*)(dst + j * 1024), 16, EDGE ? (int)((unsigned)voff + rows) : voff,
                                                     (int)(EDGE ? koff : rows + koff), 0, 0);
    };
    // One fragment read.
    auto read_a = [&](int slot_a, int h, int i) { fa[h][i] = *(const frag*)(smem + slot_a + ko[h] + a_lane + i * BLK); };
    auto read_b = [&](int slot_b, int h, int j) { fb[h][j] = *(const frag*)(smem + slot_b + ko[h] + b_lane + j * BLK); };

    // One k-step on panel kt.  A(kt) sits in slot sa, the units of panel kt+1 in na and nb (landed
    // or landing), sp is the free slot; the B fragments of panel kt and the A fragments of its
    // first NH rows of blocks are in registers, or on their way there, on entry.
    //
    // The two MFMAs that an accumulator gets from a panel (k halves 0 and 1) are issued back to
    // back: the second then takes the running sum from inside the matrix core instead of from the
    // register file, and a loop of bare MFMAs in this order runs 5-7 % faster at the chip's power
    // limit than one that visits every accumulator once per k half.  The order is column by
    // column (B block j with the NH rows of the half step, both k halves each), which is what
    // lets the B fragments be replaced one column at a time:
    //   half step 0: rows 0..NH-1.  Reads the A fragments of rows NH..NB-1; copies A(kt+2) to the
    //     free slot.  All reads of panel kt are issued by its end, so sa and sb are handed over at
    //     the barrier in the middle of the k-step.
    //   half step 1: rows NH..NB-1.  Reads the first A fragments of panel kt+1 and, behind the last
    //     MFMA of column j, the B fragments j of panel kt+1 into the registers that column just
    //     left; copies B(kt+2) to slot sa.
    // LDS reads return in order.  Half step 0 therefore starts column j as soon as at most
    // 2(NB-1-j) reads younger than B fragments j are outstanding, plus its own reads issued so far.
    // NEXT: panel kt+1 exists.  C2: panel kt+2 exists.
    constexpr int COL = 2 * NH;          // MFMAs per column of a half step
    constexpr int NS = COL * NB;         // MFMAs per half step
    constexpr int CP_EVERY = NS / LOADS; // one copy every so many MFMAs
    auto half_step = [&](auto hs_c, int kt, int slot_reads_a, int slot_next_b, int slot_copy, auto next_c, auto c2_c) {
        constexpr int hs = decltype(hs_c)::value;
        constexpr bool NEXT = decltype(next_c)::value;
        constexpr bool C2 = decltype(c2_c)::value;
        constexpr int i0 = hs * NH;
        static_for<NS>([&](auto s_c) {
            constexpr int sl = decltype(s_c)::value;
            constexpr int j = sl / COL, w = sl % COL, h = w & 1;
            constexpr int r = (j & 1) ? NH - 1 - w / 2 : w / 2;   // rows down one column, up the next: the A pair stays over the turn
            if constexpr (hs == 0) {
                if constexpr (w == 0) {
                    constexpr int own = 2 * (j < NH ? j : NH);
                    __builtin_amdgcn_s_waitcnt(waitcnt_imm(63, 2 * (NB - 1 - j) + own));
                    __builtin_amdgcn_sched_barrier(0);
                }
                // its own reads: two per column in the first NH columns
                if constexpr (j < NH && w < 2) read_a(slot_reads_a, w, NH + j);
            } else if constexpr (NEXT) {
                if constexpr (sl < COL) read_a(slot_reads_a, sl & 1, sl / 2);
                if constexpr (w == 0 && j > 0) {
                    read_b(slot_next_b, 0, j - 1);
                    read_b(slot_next_b, 1, j - 1);
                }
            }
            if constexpr (C2 && sl % CP_EVERY == CP_EVERY / 2)
                issue_one(kt + 2, slot_copy, std::integral_constant<bool, hs == 1>{}, template_int<sl / CP_EVERY>{});
            __builtin_amdgcn_sched_barrier(0);   // nothing moves across an MFMA
            // operands swapped (B rows as the MFMA "A" matrix): a lane ends up with 4 consecutive n for one m
            Mma<T>::run(fb[h][j], fa[h][i0 + r], acc[i0 + r][j]);
            __builtin_amdgcn_sched_barrier(0);
        });
        if constexpr (hs == 1 && NEXT) {
            read_b(slot_next_b, 0, NB - 1);
            read_b(slot_next_b, 1, NB - 1);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    auto kstep = [&](int kt, int sa, int sb, int na, int nb, int sp, auto next_c, auto c2_c) {
        constexpr bool NEXT = decltype(next_c)::value;
        constexpr bool C2 = decltype(c2_c)::value;
        half_step(template_int<0>{}, kt, sa, 0, sp, next_c, c2_c);
        __builtin_amdgcn_sched_barrier(0);
        wait_lds_reads();                 // the A fragments of the second half step; panel kt has been read
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (NEXT) {
            // Panel kt+1 has landed for every wave (the copies of A(kt+2), the newest
            // LOADS of this wave, may still be in flight: copies complete in issue
            // order), and every wave has read panel kt for the last time.
            if constexpr (C2) wait_vmcnt<LOADS>(); else wait_vmcnt<0>();
            __builtin_amdgcn_s_barrier();
            __builtin_amdgcn_sched_barrier(0);
        }
        half_step(template_int<1>{}, kt, na, nb, sa, next_c, c2_c);
        (void)sb;
    };

    // Prologue: panels 0 and 1 go out; wait for panel 0.
    template_int<0> first_half;
    template_int<1> second_half;
    auto last_panel_next = [&](bool is_last) {   // called before the copies of a panel are issued
        if (is_last) {
            vo0 = tail_off0;
            vo1 = tail_off1;
        }
    };
    last_panel_next(NP == 1);
    issue_unit(0, 0 * PANEL, unit_a, first_half);
    issue_unit(0, 0 * PANEL, unit_a, second_half);
    issue_unit(0, 1 * PANEL, unit_b, first_half);
    issue_unit(0, 1 * PANEL, unit_b, second_half);
    if (NP > 1) {
        last_panel_next(NP == 2);
        issue_unit(1, 2 * PANEL, unit_a, first_half);
        issue_unit(1, 2 * PANEL, unit_a, second_half);
        issue_unit(1, 3 * PANEL, unit_b, first_half);
        issue_unit(1, 3 * PANEL, unit_b, second_half);
    }
    // The accumulators are cleared here, under the latency of those copies, by MFMAs on zero
    // operands (0 x 0 + 0).  Written as assignments of zero, the compiler places the 256 register
    // writes directly in front of the main loop, behind the wait for the first panel.
    {
        frag zeros;
        asm volatile("v_mov_b32 %0, 0\n\tv_mov_b32 %1, 0\n\tv_mov_b32 %2, 0\n\tv_mov_b32 %3, 0\n\ts_nop 7"
                     : "=v"(((float*)&zeros)[0]), "=v"(((float*)&zeros)[1]), "=v"(((float*)&zeros)[2]),
                       "=v"(((float*)&zeros)[3]));
#pragma unroll
        for (int i = 0; i < NB; ++i)
#pragma unroll
            for (int j = 0; j < NB; ++j) Mma<T>::clear(zeros, acc[i][j]);
    }
    if (NP > 1) wait_vmcnt<LPT>(); else wait_vmcnt<0>();
    __builtin_amdgcn_s_barrier();
    // fragments of the first half step, in the order the main loop leaves them for the next k-step
#pragma unroll
    for (int r = 0; r < 2 * NH; ++r) read_a(0, r & 1, r / 2);
#pragma unroll
    for (int j = 0; j < NB; ++j) {
        read_b(PANEL, 0, j);
        read_b(PANEL, 1, j);
    }
    __builtin_amdgcn_sched_barrier(0);
    resolve_destination();
    __builtin_amdgcn_sched_barrier(0);

    // The consumer's waves share SIMDs with these waves while a group is being
    // copied; the issue arbiter should always prefer the wave that feeds the MFMAs.
    __builtin_amdgcn_s_setprio(3);
    int kt = 0;
    int sa = 0, sb = PANEL, na = 2 * PANEL, nb = 3 * PANEL, sp = 4 * PANEL;
    auto rotate = [&]() {   // (sa, sb, na, nb, sp) <- (na, nb, sp, sa, sb)
        const int a0 = sa, b0 = sb;
        sa = na; sb = nb; na = sp; nb = a0; sp = b0;
    };
    for (; kt < NP - 2; ++kt) {
        last_panel_next(kt + 3 == NP);   // this k-step copies panel kt + 2
        kstep(kt, sa, sb, na, nb, sp, std::true_type{}, std::true_type{});
        rotate();
    }
    if (NP >= 2) {
        kstep(kt, sa, sb, na, nb, sp, std::true_type{}, std::false_type{});
        rotate();
        ++kt;
    }
    kstep(kt, sa, sb, na, nb, sp, std::false_type{}, std::false_type{});

    // ---- epilogue: registers -> LDS strip -> global -------------------------------
    // acc[i][j][r] is element m = 16i + l%16, n = 16j + 4(l/16) + r (fr_g = l/16).
    __builtin_amdgcn_s_setprio(0);
    settle_mfma();
    __builtin_amdgcn_sched_barrier(0);   // no accumulator read is scheduled ahead of the delay
    __syncthreads();  // every wave is done with the panel buffers
    constexpr int PITCH = WT * 2 + 16;                  // strip row pitch in bytes
    constexpr int ROWCH = WT / 8;                       // 16-byte chunks per strip row
    // Two strip buffers per wave, used in turn: the next strip is written while this one is being stored.
    unsigned char* ep0 = smem + wave * (32 * PITCH);
    unsigned char* ep1 = ep0 + 4 * 32 * PITCH;
    T* D = (T*)p.D;
    [[maybe_unused]] __amdgpu_buffer_rsrc_t drsrc;
    if constexpr (STORE == 1) drsrc = __builtin_amdgcn_make_buffer_rsrc(p.D, 0, 0xffffffff, 0x00020000);
#pragma unroll
    for (int i = 0; i < NB / 2; ++i) {   // strip i: rows 32i .. 32i+31 of the quadrant
        unsigned char* ep = (i & 1) ? ep1 : ep0;
#pragma unroll
        for (int ii = 0; ii < 2; ++ii)
#pragma unroll
            for (int j = 0; j < NB; ++j) {
                out4 o;
#pragma unroll
                for (int r = 0; r < 4; ++r) o[r] = (T)acc_read(acc[2 * i + ii][j][r]);
                *(out4*)(ep + (16 * ii + fr_row) * PITCH + (16 * j + 4 * fr_g) * 2) = o;
            }
#pragma unroll
        for (int it = 0; it < WT / 16; ++it) {
            const int c = it * 64 + lane;
            const int r = c / ROWCH, cc = c % ROWCH;
            const u32x4 v = *(const u32x4*)(ep + r * PITCH + cc * 16);
            int row = row0 + 32 * i + r;
            if constexpr (MODE == kScatter) {
                const int q_row = 32 * i + r;   // row within the quadrant: held by lane q_row % 64
                row = __shfl((WT > 64 && i >= 2) ? re_hi : re_lo, q_row & 63, 64);
            }
            const size_t off = (size_t)row * ld + col0 + cc * 8;
            if (!live) continue;   // a quadrant outside the matrix goes through the motions and stores nothing
            if constexpr (EDGE) {
                const int gcol = col0 + cc * 8;
                if (row >= p.M || gcol >= p.N) continue;
                if (p.N & 7) {     // rows of D are not 16-byte aligned: element by element
                    const T* e = (const T*)&v;
#pragma unroll
                    for (int k = 0; k < 8; ++k)
                        if (gcol + k < p.N) D[off + k] = e[k];
                    continue;
                }
            }
            if constexpr (STORE == 1)
                __builtin_amdgcn_raw_buffer_store_b128(v, drsrc, (int)(off * 2), 0, 16);  // sc1: write-through
            else
                *(u32x4*)(D + off) = v;
        }
    }

    // ---- signal ---------------------------------------------------------------------
    if constexpr (MODE != kPlain) {
        // Every wave's tile stores are acknowledged before the barrier: with
        // write-through stores they are then visible device-wide (REL = 1);
        // otherwise the release on the atomic writes this L2's dirty lines back
        // before the counter moves.
        wait_vmcnt<0>();
        __syncthreads();
        const int ntile = (MT >> p.log_bm) * (MT >> p.log_bn);
        // The tiles of a macro tile mostly fall into one group: the first lane of
        // every distinct group adds that group's tile count in one atomic (at most
        // four lanes take part, all in the first wavefront).  Monitor mode keeps
        // one atomic per tile, like the reference: the tickets are per tile.
        int same = 0, earlier = 0;
        if (wave == 0) {
#pragma unroll
            for (int o = 0; o < 4; ++o) {
                const int g = __shfl(sig_group, o, 64);
                if (o < ntile && g == sig_group && g >= 0) {
                    ++same;
                    if (o < tid) ++earlier;
                }
            }
        }
        if (tid < ntile && sig_group >= 0 && (p.monitor || earlier == 0)) {
            const int add = p.monitor ? 1 : same;
            if constexpr (REL == 1)  // the stores already went through to memory
                __hip_atomic_fetch_add(p.MM + sig_group, add, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            else
                __hip_atomic_fetch_add(p.MM + sig_group, add, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
            if (p.monitor) {
                const int order =
                    __hip_atomic_fetch_add(p.MM + p.TN - 1, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                p.MM[p.TN + sig_slot] = order;
            }
        }
    }
}

template <typename T, int MT, int MODE, int STORE, int REL, bool EDGE = false>
static int launch_one(const GemmParams& p, const LaunchTimer& timer, hipStream_t stream) {
    constexpr int smem_bytes = 5 * MT * kRowBytes;   // five panel slots: 160 KiB at MT = 256
    static_assert(2 * 4 * 32 * (MT + 16) <= smem_bytes, "epilogue strips must fit in the panel slots");
    auto kern = gemm_kernel<T, MT, MODE, STORE, REL, EDGE>;
    // The attribute belongs to the function on one device: set it once per device.
    static std::atomic<unsigned long long> configured{0};
    int dev = 0;
    FO_HIP(hipGetDevice(&dev));
    const unsigned long long bit = 1ull << (dev & 63);
    if (!(configured.load(std::memory_order_acquire) & bit)) {
        FO_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, smem_bytes));
        configured.fetch_or(bit, std::memory_order_release);
    }
    if (timer.start) {
        hipExtLaunchKernelGGL(kern, dim3(p.GM * p.GN), dim3(256), smem_bytes, stream, timer.start, timer.stop, 0, p);
    } else {
        hipLaunchKernelGGL(kern, dim3(p.GM * p.GN), dim3(256), smem_bytes, stream, p);
    }
    FO_HIP(hipGetLastError());
    return FO_OK;
}

template <typename T, int MT>
static int launch_mt(int mode, bool edge, const GemmParams& p, const LaunchTimer& timer, hipStream_t stream) {
    // fo_tune knobs (how the epilogue stores C and how it signals), each read once per launch
    const int store_mode = knob(knobs().store_mode), release_mode = knob(knobs().release_mode);
    const int store = mode == kPlain ? (store_mode ? 1 : 0) : (store_mode || release_mode ? 1 : 0);
    const int rel = (mode != kPlain && release_mode) ? 1 : 0;
    if (mode == kPlain && edge)
        return store ? launch_one<T, MT, kPlain, 1, 0, true>(p, timer, stream) : launch_one<T, MT, kPlain, 0, 0, true>(p, timer, stream);
    if (mode == kPlain)
        return store ? launch_one<T, MT, kPlain, 1, 0>(p, timer, stream) : launch_one<T, MT, kPlain, 0, 0>(p, timer, stream);
    if (mode == kSignal) {
        if (rel) return launch_one<T, MT, kSignal, 1, 1>(p, timer, stream);
        return store ? launch_one<T, MT, kSignal, 1, 0>(p, timer, stream) : launch_one<T, MT, kSignal, 0, 0>(p, timer, stream);
    }
    if (rel) return launch_one<T, MT, kScatter, 1, 1>(p, timer, stream);
    return store ? launch_one<T, MT, kScatter, 1, 0>(p, timer, stream) : launch_one<T, MT, kScatter, 0, 0>(p, timer, stream);
}

int choose_macro_tile(int BM, int BN, int M, int N, bool any_shape) {
    if (!any_shape && (M % BM || N % BN)) return 0;
    // Every layout tile (128 or 256 on a side) divides the 256x256 macro tile; a matrix edge
    // that is an odd multiple of 128 is covered by half a macro tile.  The plain GEMM has no
    // layout to respect: any M and N, either macro tile.
    const bool ok128 = any_shape || (BM == 128 && BN == 128);
    if (const int forced = knob(knobs().macro_tile); forced == 256 || (forced == 128 && ok128)) return forced;   // fo_tune
    if (ok128) {
        // Problems of up to half a round of 256x256 tiles: the 128x128 macro tile, of which a CU
        // holds two workgroups, keeps all CUs busy in one round (fp16, K = 4096: 2048x4096 64 us
        // against 80, level with the vendor library; from 160 macro tiles on the large tile wins).
        const int wg256 = ((M + 255) / 256) * ((N + 255) / 256);
        if (wg256 <= 128) return 128;
    }
    return 256;
}

int launch_gemm(int mode, int dtype, int algo, int M, int N, int K, int rLDN, const int* cseg, int G,
                const int* gtable, const void* A, const void* B, void* D, int* MM, const int* RA,
                const int* RE, int monitor, hipStream_t stream) {
    // An event pair armed by fo_time_next_launch belongs to this call whether or not it gets as far
    // as a launch: taken here, ahead of the validation, so that a rejected call cannot leave it
    // behind for some later, unrelated launch.
    const LaunchTimer timer = t_launch_timer;
    t_launch_timer = LaunchTimer{};
    if (timer.start) {   // a dispatch that carries events cannot be recorded into a graph
        hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
        FO_HIP(hipStreamIsCapturing(stream, &status));
        if (status != hipStreamCaptureStatusNone)
            return fail(FO_ERR_ARG, "fo_gemm: the event pair of fo_time_next_launch cannot be attached while the stream is being captured");
    }
    int BM, BN, BK;
    if (algo_tile(algo, &BM, &BN, &BK) != FO_OK) return fail(FO_ERR_ARG, "fo_gemm: Algo %d out of range", algo);
    if ((BM != 128 && BM != 256) || (BN != 128 && BN != 256))
        return fail(FO_ERR_ARG, "fo_gemm: layout tile %dx%d: the kernel takes edges of 128 or 256", BM, BN);
    if (dtype != FO_F16 && dtype != FO_BF16) return fail(FO_ERR_ARG, "fo_gemm: dtype %d not fp16/bf16", dtype);
    if (!A || !B || !D) return fail(FO_ERR_ARG, "fo_gemm: null operand");
    if (M <= 0 || N <= 0 || K <= 0) return fail(FO_ERR_SHAPE, "fo_gemm: empty problem %dx%dx%d", M, N, K);
    // The plain GEMM writes a natural row-major D and takes any M and N; the signalling modes place
    // whole layout tiles.
    const bool any_shape = mode == kPlain;
    if (!any_shape && (M % BM || N % BN))
        return fail(FO_ERR_SHAPE, "fo_gemm_signal: M=%d N=%d not multiples of the %dx%d tile", M, N, BM, BN);
    if (K % 8) return fail(FO_ERR_SHAPE, "fo_gemm: K=%d not a multiple of 8 (operand rows must be 16-byte aligned)", K);
    if ((long long)M * N >= (1LL << 31)) return fail(FO_ERR_LIMIT, "fo_gemm: M*N=%lld needs 64-bit tile offsets", (long long)M * N);
    // (the rows a macro tile may reach beyond an operand must still have 32-bit byte offsets)
    if (((long long)M + 256) * K >= (1LL << 31) || ((long long)N + 256) * K >= (1LL << 31))
        return fail(FO_ERR_LIMIT, "fo_gemm: an operand of %lld elements exceeds the 4 GiB a buffer descriptor addresses",
                    (long long)(M > N ? M : N) * K);
    if (K % kBK && ((long long)M * K >= (1LL << 30) || (long long)N * K >= (1LL << 30)))
        return fail(FO_ERR_LIMIT, "fo_gemm: K=%d is not a multiple of %d and an operand exceeds the 2 GiB this case addresses", K, kBK);
    if (((uintptr_t)A | (uintptr_t)B | (uintptr_t)D) & 15) return fail(FO_ERR_ARG, "fo_gemm: operands must be 16-byte aligned");
    const int macro = choose_macro_tile(BM, BN, M, N, any_shape);
    if (!macro) return fail(FO_ERR_SHAPE, "fo_gemm: M=%d N=%d not multiples of the %dx%d tile", M, N, BM, BN);
    // Shapes that are multiples of 128 keep the kernel without row and column predicates (an odd
    // multiple of 128 is half a macro tile, which that kernel handles by whole quadrants).
    const bool edge = any_shape && (M % 128 || N % 128);

    GemmParams p{};
    p.A = A; p.B = B; p.D = D;
    p.M = M; p.N = N; p.K = K;
    p.GM = (M + macro - 1) / macro; p.GN = (N + macro - 1) / macro;
    p.gn_magic = raster_magic(p.GN);
    p.BM = BM; p.BN = BN; p.TN = N / BN;
    p.log_bm = BM == 256 ? 8 : 7; p.log_bn = BN == 256 ? 8 : 7;
    p.rLDN = rLDN;
    p.RA = RA; p.RE = RE; p.cseg = cseg; p.G = G; p.gtable = gtable; p.MM = MM; p.monitor = monitor;

    if (mode != kPlain) {
        if (!MM || !RA || !cseg) return fail(FO_ERR_ARG, "fo_gemm_signal: null MM/RA/cSeg");
        if (G <= 0) return fail(FO_ERR_ARG, "fo_gemm_signal: G=%d", G);
        const int T = (M / BM) * (N / BN);
        if (rLDN <= 0 || T % rLDN) return fail(FO_ERR_SHAPE, "fo_gemm_signal: rLDN=%d must divide the %d tiles", rLDN, T);
        if (mode == kScatter && !RE) return fail(FO_ERR_ARG, "fo_gemm_scatter: null RE");
    }
    if (dtype == FO_F16)
        return macro == 256 ? launch_mt<_Float16, 256>(mode, edge, p, timer, stream)
                            : launch_mt<_Float16, 128>(mode, edge, p, timer, stream);
    return macro == 256 ? launch_mt<__bf16, 256>(mode, edge, p, timer, stream) : launch_mt<__bf16, 128>(mode, edge, p, timer, stream);
}

int raster_hint(int algo, int M, int N, int* hint) {
    int BM, BN, BK;
    if (algo_tile(algo, &BM, &BN, &BK) != FO_OK) return fail(FO_ERR_ARG, "fo_raster_hint: Algo %d out of range", algo);
    if (!hint) return fail(FO_ERR_ARG, "fo_raster_hint: null hint");
    if (M <= 0 || N <= 0 || M % BM || N % BN) return fail(FO_ERR_SHAPE, "fo_raster_hint: M=%d N=%d vs tile %dx%d", M, N, BM, BN);
    const int macro = choose_macro_tile(BM, BN, M, N, false);
    if (!macro) return fail(FO_ERR_SHAPE, "fo_raster_hint: M=%d N=%d unsupported for tile %dx%d", M, N, BM, BN);
    const int GM = (M + macro - 1) / macro, GN = (N + macro - 1) / macro, TM = M / BM, TN = N / BN;
    const int tiles_m = macro / BM, tiles_n = macro / BN;
    int k = 0;
    for (int pid = 0; pid < GM * GN; ++pid) {
        const TileCoord c = raster_map(pid, GM, GN, raster_magic(GN));
        for (int i = 0; i < tiles_m; ++i)
            for (int j = 0; j < tiles_n; ++j) {
                const int tm = c.m * tiles_m + i, tn = c.n * tiles_n + j;
                if (tm < TM && tn < TN) hint[k++] = tm * TN + tn;   // half macro tiles at the matrix edge
            }
    }
    return FO_OK;
}

int tune(const char* key, int value) {
    if (!key) return fail(FO_ERR_ARG, "fo_tune: null key");
    if (!set_knob(key, value)) return fail(FO_ERR_ARG, "fo_tune: unknown knob '%s' or value %d out of its range", key, value);
    return FO_OK;
}

}  // namespace fo
