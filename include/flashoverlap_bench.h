/*
 * flashoverlap_bench.h - C ABI of libfo_bench.so: measurement probes for the
 * benchmark of the FlashOverlap hot path on gfx950.  Not part of the product:
 * libfo_hip.so neither contains nor needs anything declared here, and nothing
 * here has a counterpart in the reference.  Status codes are those of
 * flashoverlap_hip.h; the message of the last failing call on the calling
 * thread is returned by fo_bench_last_error().
 */
#ifndef FLASHOVERLAP_BENCH_H
#define FLASHOVERLAP_BENCH_H

#include <stddef.h>

#include "flashoverlap_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

const char* fo_bench_last_error(void);

/* One launch of a kernel that does nothing but
 * the GEMM's MFMA instruction (v_mfma_f32_16x16x32 of `dtype`) on operands held in registers:
 * one workgroup of 4 wavefronts per CU, 8 x 8 accumulators per wavefront, `iters` rounds of 128
 * MFMAs each in the order of the GEMM's k-step (wide != 0: v_mfma_f32_32x32x16 instead, 4 x 4
 * accumulators, 64 MFMAs a round, the same flop).  Every lane reads its 32 operand fragments (16
 * bytes each) once from `operands` (any device buffer of operand_bytes >= 16 bytes, read modulo
 * its size): pass the GEMM's own A or B and the loop toggles the matrix cores like the GEMM does,
 * pass zeros and it toggles nothing.  The GEMM runs at the chip's power limit, so the rate of
 * this loop on the same operands, not the clock-times-width peak, is what the hardware leaves
 * for it to reach.  `traffic` adds, beside the MFMAs and with nothing waiting for it, what the
 * GEMM's 256x256 tile moves per k-step and wavefront: bit 0 its 32 fragment reads (LDS to
 * registers), bit 1 its 16 one-KiB copies (L2 to LDS; needs 4 MiB..4 GiB of operands, of which a
 * power-of-two window is walked, four workgroups per XCD sharing a stream like the GEMM's tiles
 * share panels); 3 is the GEMM's whole operand traffic under a perfect schedule; wide must then be
 * 0.  `sink` (>= 4 bytes of device memory) is never written in practice; *flop, if not null,
 * receives the floating-point operations of the launch. */
int fo_mfma_spin(int dtype, int wide, int traffic, const void* operands, size_t operand_bytes, int iters,
                 void* sink, long long* flop, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FLASHOVERLAP_BENCH_H */
