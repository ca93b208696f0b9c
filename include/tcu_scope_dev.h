/*
 * tcu_scope_amd — development interface of libtcu_scope_amd.so: tuning switches, test hooks and measurement aids
 * used by this build's own benchmarks (bench.py, tcu_scope_amd/host) and tests.  None of them replaces anything in
 * the reference; a caller of the entry points in tcu_scope.h needs none of them.  Not covered by
 * TCU_SCOPE_ABI_VERSION: names and meanings may change with the kernels they steer.
 */
#ifndef TCU_SCOPE_DEV_H
#define TCU_SCOPE_DEV_H

#include "tcu_scope.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Tuning switches (process-wide: every later call of every thread sees them; not thread-safe against concurrent
 * launches, so set them before the threads that launch start):
 *   "nontemporal"     0/1, default 1: non-temporal loads and stores in the streaming kernels
 *   "scan_store_policy"  1/2, default 2: while "nontemporal" is on, the segmented scans (and mode 0 of
 *                     tcu_stream_probe) store all of their output non-temporally (2), or every other 1 KiB tile of
 *                     a wave through the cache (1).  With (1) a scan whose output stays in the 256 MiB memory-side
 *                     cache until it is overwritten or read again (one 512 MiB output buffer rewritten by every
 *                     launch: half of it is exactly that cache) runs 9 % faster, because those lines never have to
 *                     reach HBM; a scan whose output must reach HBM (outputs taken in turn, or 2 GiB of output) runs
 *                     1-3 % slower with it
 *   "scan_lds_pad"    KiB of LDS that a block of the segmented block scan (segments of 512 halves and more) asks for and
 *                     never touches, which caps the blocks a compute unit holds (160 KiB per unit: 39 = four blocks,
 *                     52 = three, 79 = two); -1 (default) = AUTO's table, which caps blocks of 16 KiB at three or four
 *                     per unit for segments of 4096 ... 16384 halves; 0 = never.  Requests beyond what a unit has left
 *                     beside the kernel's own LDS are clipped
 *   "static_order"    0/1, default 0: full scan takes partitions in block-index order instead of by ticket
 *   "offsets_scan_chain" 0/1, default 1: tcu_seg_scan_offsets_f16 with expected segments beyond 65536 halves in one pass (a
 *                     segment's slices meet through decoupled look-back) instead of slice sums followed by a second read
 *   "by_key_reduce_chain" 0/1, default 0: tcu_seg_reduce_by_key_f16 as one pass with a decoupled look-back (the form of the
 *                     scan by key; a wait that expires leaves ~0 in *d_num_runs and NaN in the sums that depended on it)
 *                     instead of the five launches that wait for nothing
 *   "by_key_waves"    waves per block of the two large launches of tcu_seg_reduce_by_key_f16 (1 .. 16; 0 = default 1)
 *   "by_key_key_tiles" KiB of keys a wave of its first launch has in flight: 4, 8 or 16 (0 = default 16)
 *   "scan_lds_tiles"  full scan AUTO parks 4 extra tiles per wave in LDS (partitions of 98304 halves): 1 always, 0 never,
 *                     -1 (default) where it measures faster, i.e. up to 2^27 elements
 *   "gemv_col_shape"  column-major GEMV: waves per block (4 or 8) * 10 + groups of 8 columns per wave and round (1 or 2); default 82
 *   "gemv_col_blocks" column-major GEMV: about this many blocks (slabs of 512 rows x stretches of K); default 1024
 *   "gemv_rows", "gemv_tiles", "gemv_waves"  0 = default: rows per block (1/2/4/8), tiles per wave and step
 *                     (1/2/4/8) and waves per block of the block GEMV kernel (rows of 8 KiB and more);
 *                     "gemv_waves" also sets the waves that split K in the strip kernels (TCU_VARIANT_MFMA_16N)
 *   "gemv_strip_lds"  0/1, default 1: TCU_VARIANT_MFMA_16N stages the 16-row strip through LDS where K is a
 *                     multiple of 512 (0: operands straight from global memory at every K)
 *   "gemm_big_tiles"  -1/0/1/192, default -1: 256 x 256 block tiles wherever M and N allow (1), never (0), or
 *                     where the output has at least 128 of them (-1; smaller outputs take 128 x 128 tiles, and outputs
 *                     that 192 x 192 tiles cut into fuller rounds of the chip take those, e.g. 3072 x 3072); 192 = 192 x 192
 *                     tiles wherever M and N are multiples of 192 and K of 64
 *   "gemm_direct_lds" -1/0/3/4/64/65/66, default -1: 3 or 4 = global -> LDS transfers, K step 32, that many LDS
 *                     buffers; 64 = K step 64, two buffers; 65 = K step 64, three buffers for A and two for B;
 *                     66 = as 65 on 16x16x32 instead of 32x32x16 MFMAs (C and D aligned to four outputs, else 65);
 *                     0 = register-staged kernel; -1 = 66 where K is a multiple of 64, else 4.  128 x 128 tiles:
 *                     -1 and 66 = the 16x16x32 loop of 66 (K a multiple of 64, C and D aligned to four outputs),
 *                     other values above 0 = 32x32x16 transfers with K step 64 (two buffers) or 32 (four)
 *   "gemm_split_tail" 0/1/2, default 1: the K steps of the tiles of a last, partly filled round of the big-tile GEMM
 *                     grid are spread over all compute units (fp32 shares in stream-ordered temporary memory, added
 *                     in a fixed order by a second kernel): never, where it pays (round at most a third full,
 *                     K >= 4096), or whenever there is such a round
 *   "compute_units"   blocks of the big-tile GEMM kernel the device runs at a time (set by tcu_init; for tests)
 *   "gemm_staged_epilogue" 0/1, default 1: the GEMM kernels on 16x16x32 MFMAs turn their outputs through LDS and
 *                     write (and read C in) whole rows of a wave's 128 or 64 columns, 16 bytes per lane, where C and D are
 *                     16-byte aligned; 0 = straight from the accumulator layout (64 / 32 bytes of 16 rows per store)
 *   "gemm_bk64"       0/1, default 0: K step 64 instead of 32 in the register-staged kernel
 *   "gemm_depth"      1..4, default 4: prefetch depth of the register-staged kernel
 *   "many_totals"     default 65536: TCU_FULL_MULTI_KERNEL adds (reduce) or scans (scan) the per-segment totals with one
 *                     block below this many segments, and with the two-launch partition sums / the single-pass scan
 *                     (whose own workspace then follows the totals) from there on
 *   "xcd_run"         -1/0/C, default -1: consecutive blocks of a launch run on different XCDs (block b on XCD
 *                     b % 8); with C > 0 the segmented kernels renumber their blocks inside groups of 8 * C so that
 *                     every XCD works on C consecutive pieces of the array (a piece = what one block takes) while
 *                     the launch still sweeps the array front to back; 0 = no renumbering; -1 = the value measured
 *                     best for the segment size and launch shape
 *   "lookback_poll_limit"  default 2^20 (negative restores it): how often a block of a single-pass full-array
 *                     kernel (and of the look-back path of tcu_seg_scan_f16 for segments of 2^21 halves and more)
 *                     looks again for a value another block has not published yet before it gives up.  Giving up
 *                     never yields a finite wrong number: the reduction's result, or the scan's outputs from the
 *                     waiting partition to the end of the array (or segment), become NaN
 *   "test_mute_partition"  default 0; p > 0: partition p - 1 of those kernels publishes nothing, so every wait
 *                     for it expires (for tests of the rule above; all kernels still run to their end)
 * Unknown names return TCU_ERR_INVALID_ARG. */
int tcu_set_option(const char *name, int value);

/* ---- measurement aids ---------------------------------------------------------------------------- */

/* Plain streaming kernels with the same access shape as the reductions/scans: mode 0
 * copies `bytes` from d_src to d_dst, mode 1 only reads d_src (one word per block is
 * written to d_dst), mode 2 only writes d_dst.  Used to calibrate hardware counters and
 * to report what fraction of peak a pure copy reaches.  bytes must be a multiple of 16. */
int tcu_stream_probe(void *d_dst, const void *d_src, size_t bytes, int mode, int tiles_per_wave, int waves_per_block, void *stream);
/* The next kernel that this host thread launches through the library carries the two events
 * (hipEvent_t created with timing enabled; either may be NULL): its dispatch stamps
 * start_event with the time the kernel begins and stop_event with the time it ends, so that
 * hipEventElapsedTime(start, stop) is the kernel's own duration, without the event packets a
 * hipEventRecord pair puts on the stream around it.  Meant for entry points that launch one
 * kernel; with several, only the first carries the events.  The reference brackets its
 * launches with cudaEventRecord (e.g. src/reduction/seg_wmma_16n.cu:57-73). */
int tcu_time_next_launch(void *start_event, void *stop_event);
/* How many times the library has taken temporary device memory (hipMallocFromPoolAsync) since the process began,
 * over all threads and devices: lets a test show that an entry point allocated nothing. */
unsigned long tcu_temporary_allocations(void);
/* Runs every cross-lane primitive the kernels rely on (MFMA 16x16x32 / 32x32x16 operand
 * layouts, DPP controls, lane swaps) on lane-indexed inputs and writes the raw results
 * to d_out (fp32 / u32 words; lane_probe_kernel in tcu_scope_amd/csrc/util_kernels.hpp has the record layout).
 * *out_words receives the number of 32-bit words (call with d_out == NULL to query). */
int tcu_lane_probe(void *d_out, size_t *out_words, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* TCU_SCOPE_DEV_H */
