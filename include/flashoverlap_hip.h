/*
 * flashoverlap_hip.h - C ABI of libfo_hip.so, the gfx950 device library of the
 * FlashOverlap single-GPU hot path.
 *
 * Plain pointers, sizes and opaque stream handles only: no torch types cross
 * this boundary.  Every entry point returns 0 (FO_OK) or a positive FO_ERR_*
 * code and never calls exit(); fo_last_error() returns the message of the
 * last failing call on the calling thread.  All device pointers are on the
 * current HIP device; `stream` is a hipStream_t passed as void* (NULL = the
 * null stream).  Nothing here allocates device memory except where stated.
 *
 * Each declaration cites the reference interface it replaces (paths relative
 * to the reference checkout).
 *
 * Layout conventions (all row-major, 16-bit elements, K contiguous):
 *   A [M,K], B [N,K], D = A . B^T.  The "layout tile" is BM x BN as selected
 *   by `algo` (fo_algo_tile); TM = M/BM, TN = N/BN, T = TM*TN tiles, tile id
 *   t = m_tile*TN + n_tile, slot s = RA[t].  The permuted output is D viewed
 *   as [M*N/(rLDN*BN), rLDN*BN] with tile slot s at block-row s/rLDN,
 *   block-col s%rLDN.
 */
#ifndef FLASHOVERLAP_HIP_H
#define FLASHOVERLAP_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum fo_dtype { FO_F16 = 0, FO_BF16 = 1 };

enum fo_status {
    FO_OK = 0,
    FO_ERR_ARG = 1,     /* null pointer, bad enum, bad algo index */
    FO_ERR_SHAPE = 2,   /* shape not supported by the selected tile */
    FO_ERR_HIP = 3,     /* a HIP runtime call failed */
    FO_ERR_TIMEOUT = 4, /* a device-side bounded wait gave up */
    FO_ERR_LIMIT = 5    /* size beyond a documented maximum */
};

/* ---- library ---------------------------------------------------------- */

int fo_version(void);
const char* fo_last_error(void);

/* Number of `Algo` indices and the layout tile each one selects.  Replaces the
 * function-pointer tables indexed by Algo (src/tiling/gemm_tiling.cuh:3-10,
 * signal_tiling.cuh:3-10, scatter_tiling.cuh:3-10; instances in
 * src/inc/signal_instances.inc:1-6).  Index order matches the reference:
 * (128,128,32) (128,128,64) (128,256,32) (128,256,64) (256,128,32) (256,128,64). */
int fo_algo_count(void);
int fo_algo_tile(int algo, int* BM, int* BN, int* BK);

/* Device facts used for roofline reports: CU count and clock (kHz) as HIP
 * reports them.  xcd_count is not read from the device (HIP has no attribute
 * for it): it is the constant 8 that the workgroup rasterisation of the GEMM
 * is built for (MI355X: 8 accelerator dies of 32 CUs). */
int fo_device_info(int* cu_count, int* clock_khz, int* xcd_count);

/* ---- GEMM ------------------------------------------------------------- */

/* D[M,N] = A[M,K] . B[N,K]^T, fp32 accumulate, natural row-major D.
 * Replaces gemm_func_table[Algo] / mutlass_gemm<TM,TN,TK>
 * (src/tiling/gemm_dispatcher.h:16-20, src/gemm/gemm.cu:29-113).
 * Any M >= 1 and N >= 1 (the layout tile of `algo` places nothing here; rows
 * and columns of an edge tile that lie outside the matrix are computed on
 * zero-filled operand rows and not stored; an N that is not a multiple of 8
 * makes the rows of D unaligned and is stored element by element), K % 8 == 0
 * (a K that is not a multiple of 64 is zero-padded inside the kernel; the
 * operands must then be below 2 GiB each), 16-byte aligned pointers.  The
 * reference's kernels take only multiples of their tile (README.md:75; the
 * residue predicates of src/overlap/gemm_with_signal.h:176-181 are never
 * exercised by its callers). */
int fo_gemm(int dtype, int algo, int M, int N, int K,
            const void* A, const void* B, void* D, void* stream);

/* Signalling GEMM.  Tile t is stored at slot RA[t] of the permuted layout and,
 * after the tile's stores are visible device-wide, MM[group(slot)] is bumped.
 * By default (fo_tune "release_mode" 1) the tile stores are agent-scope
 * write-through stores; every wavefront waits until they are acknowledged,
 * the workgroup meets at a barrier, and then one lane per group adds the
 * group's tile count with a relaxed agent-scope atomic.  The release-ordered
 * form (the atomic itself a release at agent scope, which writes the L2's
 * dirty lines back first) is what "release_mode" 0 selects; counters, slots
 * and results are the same.  group(slot) is the index of the first
 * inclusive prefix sum of cseg_dev[0..G) that exceeds slot.  If `monitor` is
 * non-zero a ticket is also taken from MM[TN-1] and stored at MM[TN+slot].
 * Replaces signal_func_table[Algo] / mutlass_gemm_signal<TM,TN,TK>
 * (src/tiling/gemm_dispatcher.h:7-14, src/overlap/gemm_signal.cu:28-110,
 * epilogue src/overlap/gemm_with_signal.h:128-202).
 * group_table: optional device array of T ints, group_table[s] = group(s),
 * as written by fo_build_group_table; NULL makes every workgroup scan
 * cseg_dev linearly like the reference (fine for a few dozen groups).
 * MM must hold at least G ints (TN + T in monitor mode). */
int fo_gemm_signal(int dtype, int algo, int M, int N, int K, int rLDN,
                   const int* cseg_dev, int G, const int* group_table,
                   const void* A, const void* B, void* D,
                   int* MM, const int* RA, int monitor, void* stream);

/* As fo_gemm_signal, with the row index of the permuted view mapped through
 * RE (int32, M*N/BN entries) before the store.  Replaces
 * scatter_func_table[Algo] / mutlass_gemm_scatter<TM,TN,TK>
 * (src/tiling/gemm_dispatcher.h:22-28, src/overlap/gemm_scatter.cu,
 * epilogue src/overlap/gemm_with_scatter.h:128-197). */
int fo_gemm_scatter(int dtype, int algo, int M, int N, int K, int rLDN,
                    const int* cseg_dev, int G, const int* group_table,
                    const void* A, const void* B, void* D,
                    int* MM, const int* RA, const int* RE, int monitor, void* stream);

/* fo_gemm_signal for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).
 * It has no counterpart in the reference.  The slot->group table, which
 * fo_gemm_signal takes from its caller as `group_table`, is built by this call
 * (on `stream`, ahead of the GEMM) in a device array that is part of the
 * library image: FO_STATIC_MAX_TILES ints (256 KiB) per GPU, held until the
 * process ends.  The call allocates and frees nothing.  Shapes with more than
 * FO_STATIC_MAX_TILES layout tiles are rejected with FO_ERR_LIMIT.  All calls
 * on one GPU share that GPU's array: calls whose kernels may run concurrently
 * on one GPU (different streams) race on it; calls ordered on one stream, or
 * otherwise serialised, are safe and need no clearing in between.  Results are
 * identical to fo_gemm_signal with a table from fo_build_group_table. */
#define FO_STATIC_MAX_TILES 65536
int fo_gemm_signal_static(int dtype, int algo, int M, int N, int K, int rLDN,
                          const int* cseg_dev, int G,
                          const void* A, const void* B, void* D,
                          int* MM, const int* RA, int monitor, void* stream);

/* group_table[s] = group(s) for s in [0,T), computed on the device from
 * cseg_dev.  No counterpart in the reference, whose epilogue rescans cSeg for
 * every tile (src/overlap/gemm_with_signal.h:188-193); results are identical. */
int fo_build_group_table(const int* cseg_dev, int G, int T, int* group_table, void* stream);

/* The order in which the GEMM kernels issue layout tiles for this shape:
 * hint[i] = original tile id of the i-th tile issued (T entries, host memory).
 * Feeding it to reorder_indices makes slot order equal issue order.  Replaces
 * the sampled completion order of the reference tuner
 * (tune/search.py:164-263), which exists because its scheduler is opaque. */
int fo_raster_hint(int algo, int M, int N, int* hint_host);

/* Process-wide tuning knobs of the GEMM epilogue, for measurement; no
 * counterpart in the reference.  Results are identical for every setting.
 * The knobs are atomics: a thread may set one while others launch, and a
 * launch reads each knob once.
 *   "release_mode" 1 (default): the tile stores are agent-scope write-through
 *                  stores; every wave waits for their acknowledgement, the
 *                  workgroup meets at a barrier, then a relaxed agent-scope
 *                  atomic bumps the counter.  0: a release-ordered atomic
 *                  instead (L2 write-back first), with the tile stores as
 *                  "store_mode" says.
 *   "store_mode"   with release_mode 0 only.  1 (default): write-through tile
 *                  stores; 0: cached tile stores.
 *   "copy_streaming_stores"  how the consumer copies store.  2 (default):
 *                  chosen per launch: non-temporal stores in fo_wait_consume
 *                  and in fo_consume calls of 48 MiB or more (copies of that
 *                  size running beside a GEMM push its operands out of the
 *                  memory-side cache), ordinary stores in smaller ones and in
 *                  fo_settle_consume (their destination is then still cached
 *                  for the kernel that reads it next); 1: non-temporal
 *                  everywhere; 0: ordinary everywhere.
 *   "macro_tile"   the tile one workgroup computes.  0 (default): chosen per
 *                  shape (128x128 for outputs of up to 128 tiles of 256x256,
 *                  else 256x256); 128 or 256: forced, 128 only where the
 *                  layout tile is 128x128 or the GEMM is the plain one.  The
 *                  issue order fo_raster_hint reports follows the setting. */
int fo_tune(const char* key, int value);

/* ---- counting / wait -------------------------------------------------- */

/* Enqueue a one-wave kernel that returns once *addr == that and then stores 0
 * to *addr.  Replaces launch_kernel_wait_flag (src/wait_launch.h:5,
 * src/wait_launch.cu:5-7, kernel src/wait.cuh:5-9).  Unlike the reference the
 * wait is bounded (fo_set_wait_timeout_ms, default 10000 ms): on expiry the
 * kernel leaves *addr untouched, counts the expiry and returns; what follows
 * on the stream then works on an incomplete group, so a caller reads the count
 * at its next synchronisation point and zeroes MM after an expiry.
 * `expired` (here and in the other waiting calls): a device int that the
 * caller owns and that this call increments if its wait expires, so that a
 * caller sees the expiries of its own calls only; NULL counts them in a word
 * per device that fo_wait_timeouts reads. */
int fo_wait(int that, int* addr, int* expired, void* stream);

/* One persistent kernel in place of G (wait, collective) launch pairs: for
 * g = 0..G-1 in order, wait for MM[g] == cseg_dev[g], copy group g's
 * contiguous range of `src` (tile_elems * cseg[g] 16-bit elements starting at
 * tile_elems * sum(cseg[0..g))) to the consumer buffer, then reset MM[g].
 * The range is cut into nslices equal parts; parts slice_first ..
 * slice_first+slice_count-1 are copied, part k to
 * dst + (k - slice_first)*slice_stride + offset/nslices.  nslices == 1 copies
 * the range to the same offset of dst (the AllReduce stand-in,
 * src/overlap_impl.cu:257-265); nslices == world size with one slice is what a
 * rank receives from the per-group ReduceScatter (src/overlap_impl.cu:312-323),
 * with all slices it is every rank's receive buffer side by side.
 * The kernel runs nblocks workgroups of four wavefronts (1 <= nblocks <= CU
 * count; it uses no LDS and few registers, so a workgroup fits beside a GEMM
 * workgroup on a CU).  A team of workgroups, one per 128 KiB of the group (at
 * most all), handles a group: its first wavefronts poll the counter, the
 * others sleep at a barrier until it is full, then all copy.  Consecutive
 * groups go to consecutive teams.  Groups of nblocks x 128 KiB and more are therefore
 * released strictly in index order by the whole grid, smaller ones as they
 * complete.  order_log (optional, G ints) gets order_log[g] = g when group g
 * has been released and its counter reset.  If a wait expires the workgroup
 * counts it (in *expired, or for NULL in the word fo_wait_timeouts reads),
 * copies the incomplete group like the copy behind an expired fo_wait would,
 * and from then on looks at each of its later counters just once; MM then
 * holds partial counts and must be zeroed by the caller before it is used
 * again. */
int fo_wait_consume(const int* cseg_dev, int G, int* MM,
                    const void* src, void* dst, long long tile_elems,
                    int nslices, int slice_first, int slice_count, long long slice_stride,
                    int* order_log, int nblocks, int* expired, void* stream);

int fo_set_wait_timeout_ms(int ms);
/* Number of bounded waits that were given no `expired` word of their own and
 * expired on the current device since the last call with reset != 0
 * (synchronises the device). */
int fo_wait_timeouts(int* count, int reset);

/* Copy `bytes` bytes (multiple of 2) from src to dst with a device kernel: the
 * one-GPU stand-in for mcclAllReduce / mcclReduceScatter on one released
 * group (call sites src/overlap_impl.cu:263, 319-320). */
int fo_consume(const void* src, void* dst, size_t bytes, void* stream);

/* fo_wait + fo_consume in one launch, for a group whose producing GEMM was
 * enqueued earlier on the same `stream`: stream order has already made the
 * counter final, so there is nothing to poll.  *addr == that is cleared to 0 as
 * fo_wait does; any other value is left in place and counted as an expired wait
 * (`expired` as in fo_wait).  The copy is made either way, as it would be behind an
 * expired fo_wait.  Used for the last group of a call, which completes together
 * with the GEMM (the reference waits for it on the communication stream,
 * src/overlap_impl.cu:257-265, and then joins the streams). */
int fo_settle_consume(int that, int* addr, const void* src, void* dst, size_t bytes, int* expired, void* stream);

/* One launch for the `nslices` slices of a released group: slice k is the
 * `slice_bytes` bytes at src + k * slice_bytes and goes to dst + k *
 * dst_stride_bytes.  The one-GPU stand-in for one mcclReduceScatter call on a
 * group when all ranks' receive buffers are kept side by side
 * (src/overlap_impl.cu:319-320 makes one collective call per group, not one per
 * rank).  addr != NULL: also settle the group's counter like fo_settle_consume
 * (for the last group, on the GEMM's stream); addr == NULL: a plain copy.
 * store_policy: FO_COPY_STREAM = non-temporal stores (for copies that run
 * beside a GEMM when the call copies tens of MB that way: they then leave its
 * operands in the memory-side cache), FO_COPY_CACHED = ordinary stores (the
 * destination stays cached for its reader), FO_COPY_AUTO = by the size of this
 * launch alone, as fo_consume does.  fo_tune("copy_streaming_stores", 0 or 1)
 * overrides all three. */
#define FO_COPY_AUTO 0
#define FO_COPY_STREAM 1
#define FO_COPY_CACHED 2
int fo_consume_slices(int that, int* addr, const void* src, void* dst, size_t slice_bytes, int nslices,
                      size_t dst_stride_bytes, int store_policy, int* expired, void* stream);

/* ---- RMSNorm ---------------------------------------------------------- */

/* out[b,:] = rmsnorm(gather(x)[b,:]) * gamma, gather as in the layout header.
 * Replaces launch_reorder_rmsnorm_kernel (src/rmsnorm/rmsnorm_launch.h:7-8,
 * src/rmsnorm/rmsnorm_launch.cu:16-21, kernel src/rmsnorm/rmsnorm.cuh:62-115),
 * with eps a parameter (the reference fixes 1e-5) and an explicit stream (the
 * reference uses the null stream).  Requires dim % 8 == 0, BN % 8 == 0. */
int fo_reorder_rmsnorm(int dtype, const void* x, const void* gamma, void* out,
                       int bs, int dim, int BM, int BN, int rldn, const int* RA,
                       float eps, void* stream);

/* nbatch independent reorder+RMSNorm problems in one launch: x and out hold
 * nbatch consecutive [bs, dim] blocks that all use the same RA, BM, BN.  This is
 * the shape of the ReduceScatter receive buffers of all ranks side by side
 * (each a tile-permuted layout with tile height BM/world_size,
 * example/correctness_rs.py:107-108 builds one of them per rank); no counterpart
 * in the reference, where a process only ever holds its own rank's buffer. */
int fo_reorder_rmsnorm_batched(int dtype, const void* x, const void* gamma, void* out,
                               int nbatch, int bs, int dim, int BM, int BN, int rldn,
                               const int* RA, float eps, void* stream);

/* Plain row RMSNorm.  Replaces launch_rmsnorm_kernel
 * (src/rmsnorm/rmsnorm_launch.h:5, src/rmsnorm/rmsnorm.cuh:12-57). */
int fo_rmsnorm(int dtype, const void* x, const void* gamma, void* out,
               int bs, int dim, float eps, void* stream);

/* ---- streams and events ----------------------------------------------- */

/* Non-blocking stream at the default priority.  Replaces
 * musaStreamCreateWithPriority(.., NonBlocking, -5) (src/overlap_impl.cu:146-148). */
int fo_stream_create(void** stream);
int fo_stream_destroy(void* stream);
int fo_stream_sync(void* stream);
/* Make `waiter` wait for everything enqueued so far on `signaller`.  Replaces
 * the per-call event create/record/wait/destroy (src/overlap_impl.cu:267-270). */
int fo_stream_join(void* signaller, void* waiter);
/* Measurement aid, no counterpart in the reference: the next fo_gemm*, fo_rmsnorm* or
 * fo_reorder_rmsnorm* launch made by the calling thread attaches the two events (from
 * fo_event_create) to its own dispatch; fo_event_elapsed_ms between them is then the
 * kernel's duration, as a profiler reports it, without the launch gaps that an event
 * pair recorded around the call includes.  Passing two nulls cancels. */
int fo_time_next_launch(void* start_event, void* stop_event);
/* *capturing = 1 while `stream` is recording into a graph (stream capture), else 0.
 * No counterpart in the reference, whose overlapped call cannot be captured. */
int fo_stream_is_capturing(void* stream, int* capturing);

/* Timing helpers for harnesses that cannot use torch events on foreign
 * streams: opaque hipEvent_t handles. */
int fo_event_create(void** ev);
int fo_event_destroy(void* ev);
int fo_event_record(void* ev, void* stream);
int fo_event_sync(void* ev);
int fo_event_elapsed_ms(void* start, void* stop, float* ms);

#ifdef __cplusplus
}
#endif
#endif /* FLASHOVERLAP_HIP_H */
