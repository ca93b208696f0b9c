/*
 * tcu_scope_amd — C ABI of the MI355X (gfx950) implementation of the tcu_scope hot path:
 * fp16 segmented / full reduction and inclusive prefix sum (as contractions against
 * constant ones / triangular matrices on MFMA, and as DPP / LDS wave and block
 * collectives), and the fp16 GEMV / GEMM kernels.
 *
 * The reference (c3sr/tcu_scope) has no FFI layer; its boundary is the set of device
 * kernels its benchmark harnesses launch, all of the form
 *     kernel<<<grid, WARPS_PER_BLOCK*32>>>(const half *d_in, half *d_out, size_t num_segments)
 * with the segment size, tiles/segments per warp and warps per block as template
 * arguments.  Each entry point below replaces one such family; the template arguments
 * become run-time arguments.
 *
 * Conventions
 *   - every pointer named d_* is DEVICE memory owned by the caller; nothing here frees or
 *     retains it.  Reduction/scan inputs and outputs must be 16-byte aligned unless the
 *     variant is TCU_VARIANT_AUTO.
 *   - temporary device memory: the kernels of the common sizes need none.  A few paths take
 *     some in stream order from a memory pool the library keeps per device (it is given back
 *     to the pool when the enqueued work has run, and the pool keeps it for the next call):
 *     tcu_seg_reduce_f16 and tcu_seg_scan_f16 with TCU_VARIANT_AUTO where they cut segments into partitions: segments
 *     of 2^20 (reduction) / 2^21 (scan) halves and more, segments of 2^17 halves and more when there are fewer than 256
 *     of them, and segments of 2^19 halves and more from 2^30 elements on
 *     (reduction: 4 bytes per 4096 input halves, and a thousandth of that again for segments
 *     beyond 2^25; scan: 256 bytes per 65536 input halves), the *_offsets_f16 entry points with
 *     expected segment lengths beyond 65536 halves (reduction 4, scan up to 256 bytes per 65536 halves), and tcu_gemm_* when the
 *     last round of output tiles is sparsely filled (up to 128 MiB).  The full-array entry
 *     points work in the caller's workspace; tcu_seg_scan_f16_noalloc never allocates.
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).  Calls only
 *     enqueue work; they do not synchronise.
 *   - the return value is a tcu_status; on failure tcu_last_error() describes it (per
 *     host thread).  TCU_ERR_UNSUPPORTED is what the reference's harness turns into
 *     state.SkipWithError (e.g. "segment size must be 16").
 *   - thread-compatible: concurrent calls must use different streams and, where a
 *     workspace is taken, different workspaces.
 *   - this header holds what replaces a reference kernel or harness helper.  Tuning switches,
 *     the test hooks and the measurement aids of this build's own benchmarks and tests are
 *     declared in tcu_scope_dev.h; a caller of the entry points below needs none of them.
 *   - results: fp32 accumulation, one round-to-nearest-even conversion to fp16.
 */
#ifndef TCU_SCOPE_H
#define TCU_SCOPE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* 2: entry points over offsets and key arrays, tcu_seg_scan_f16_noalloc, the TCU_FULL_MFMA flag, block variants from 16
 * halves per segment, 256 bytes of workspace per partition of the full-array scan (a cached size from version 1 is too
 * small), tcu_init fails when the scratch symbol cannot be resolved; the tuning switches and measurement aids moved to
 * tcu_scope_dev.h.
 * 3: tcu_gemv_col_major_f16_f32 / _f16; the workspace of tcu_seg_reduce_by_key_f16 grew (ask again: about 0.63 n bytes). */
#define TCU_SCOPE_ABI_VERSION 3

typedef enum {
  TCU_OK = 0,
  TCU_ERR_INVALID_ARG = 1, /* null pointer, misalignment, bad enumerator, overflow */
  TCU_ERR_UNSUPPORTED = 2, /* (variant, size) pair this kernel family does not cover */
  TCU_ERR_RUNTIME = 3,     /* a HIP call failed; tcu_last_error() carries hipGetErrorString */
  TCU_ERR_WORKSPACE = 4    /* workspace missing or smaller than the size query reports */
} tcu_status;

/* Kernel families.  The MFMA_* values keep the reference's naming of its WMMA kernels
 * (one per benchmark family); WAVE_SHUFFLE and BLOCK_LDS are the counterparts of its
 * cub::Warp* and cub::Block* comparators. */
typedef enum {
  TCU_VARIANT_AUTO = 0,            /* fastest measured family for the size; any segment size >= 1 */
  TCU_VARIANT_MFMA_16 = 1,         /* segment size 16      (reference *_16)          */
  TCU_VARIANT_MFMA_16N = 2,        /* power of two >= 16   (reference *_16N, _16N_OPT) */
  TCU_VARIANT_MFMA_16N_BLOCK = 3,  /* power of two >= 16, 16 segments per block (reference *_16N_BLOCK) */
  TCU_VARIANT_MFMA_256 = 4,        /* segment size 256     (reference *_256)         */
  TCU_VARIANT_MFMA_256N = 5,       /* power of two >= 256  (reference *_256N)        */
  TCU_VARIANT_MFMA_256N_BLOCK = 6, /* power of two >= 256, block per segment (reference *_256N_BLOCK) */
  TCU_VARIANT_WAVE_SHUFFLE = 7,    /* DPP wavefront collectives (reference CUB_WARP_*) */
  TCU_VARIANT_BLOCK_LDS = 8        /* power of two >= 16, block collectives through LDS (reference CUB_BLOCK_*) */
} tcu_variant;
/* The three block families share a segment among the waves of a block from 512 halves (one 1 KiB tile) on.  A
 * shorter segment lies inside one wave's tile, so there the same launch shape (waves per block x tiles per wave)
 * runs the kernels whose waves take whole tiles: no wave of the block has anything to tell another. */

/* Strategies of the full-array entry points. */
typedef enum {
  TCU_FULL_AUTO = 0,
  TCU_FULL_SINGLE_PASS = 1, /* one kernel: published partials added by the grid's last blocks (reduce), decoupled look-back (scan);
                               replaces reference *_ATOMIC_W_BLOCK_SYNC / _ATOMIC_BALLOT / _CG */
  TCU_FULL_MULTI_KERNEL = 2, /* reference "2 kernels" (reduce) / "3 kernels" (scan) sequences; ask for the workspace size, it
                                is not a fixed number of bytes per segment */
  TCU_FULL_MFMA = 0x100     /* flag, OR-ed onto a strategy: the single-pass kernels add (reduce: D += A * ones) and scan
                               (U * X + carry) on the matrix unit, as the reference's *_CG / *_ATOMIC_* kernels do on
                               WMMA fragments; without it the DPP flavour runs.  AUTO | MFMA runs SINGLE_PASS | MFMA */
} tcu_full_strategy;

typedef enum {
  TCU_DIST_UNIFORM = 0, /* uniform [-1,1) */
  TCU_DIST_GRID = 1,    /* k/2048, exact in fp16 */
  TCU_DIST_NORMAL = 2,  /* N(0,1) */
  TCU_DIST_SMALLINT = 3 /* {0,1,2} */
} tcu_dist;

/* ---- library ------------------------------------------------------------------------ */

/* Selects the device and caches its properties.  Replaces reference init_cuda
 * (src/init/cuda.cpp:23-67): an out-of-range id falls back to device 0 as there. */
int tcu_init(int device_id);
const char *tcu_last_error(void);
int tcu_abi_version(void);
/* Compute units, wavefront size, LDS bytes per CU, 1 if the device is gfx950. */
int tcu_device_info(int *compute_units, int *wavefront_size, int *lds_bytes, int *is_gfx950);

/* ---- segmented reduction -------------------------------------------------------------- */

/* d_out[j] = fp16( sum of d_in[j*segment_size .. (j+1)*segment_size) ), j < num_segments.
 * Replaces compute_wmma_segmented_reduction_{16,16n,16n_opt,16n_block,256,256n,256n_block}
 * (reference src/reduction/kernel.cuh:33-559) and compute_cub_{warp,block}_segmented_reduction
 * (src/reduction/seg_cub_warp.cu:17-32, seg_cub_block.cu:13-29).
 * tiles_per_wave: 1 KiB tiles each wave keeps in flight (1,2,4,8; 0 = default) — the
 * reference's WMMA_TILES_PER_WARP / SEGMENTS_PER_WARP; waves_per_block: 1..16 (0 = default)
 * — the reference's WARPS_PER_BLOCK. */
int tcu_seg_reduce_f16(const void *d_in, void *d_out, size_t num_segments, size_t segment_size, int variant, int tiles_per_wave, int waves_per_block, void *stream);

/* Segments given by offsets: d_out[j] = fp16( sum of d_in[begin[j] .. end[j]) ), an empty
 * segment (end[j] <= begin[j]) gives 0.  Segments may start at any element, overlap or
 * leave gaps.  Replaces cub::DeviceSegmentedReduce::Sum(d_temp, bytes, d_in, d_out,
 * num_segments, d_offsets, d_offsets + 1) as the reference calls it
 * (src/reduction/seg_cub_device.cu:46-48, 61-63); no temporary storage is needed.
 * offset_bits: 32 or 64 (signed integers, device memory).  expected_segment_size: the
 * typical segment length, used to choose how many lanes share a segment (0 = unknown: a
 * whole wave per segment). */
int tcu_seg_reduce_offsets_f16(const void *d_in, void *d_out, size_t num_segments, const void *d_begin_offsets, const void *d_end_offsets, int offset_bits, size_t expected_segment_size, void *stream);

/* ---- segmented inclusive prefix sum ------------------------------------------------------ */

/* d_out[j*S + i] = fp16( d_in[j*S] + ... + d_in[j*S + i] ).  d_totals (may be NULL)
 * receives the fp16 total of every segment — the `_ps` kernels' partial_sums.
 * Replaces compute_wmma_segmented_prefixsum_{16,16n,16n_block,16n_opt,256,256_ps,256n,
 * 256n_ps,256n_block,256n_block_ps} (reference src/prefixsum/kernel.cuh:48-774) and
 * compute_cub_{warp,block}_segmented_prefixsum (src/prefixsum/seg_cub_warp.cu:17-27,
 * seg_cub_block.cu:13-51).  In-place (d_out == d_in) is allowed. */
int tcu_seg_scan_f16(const void *d_in, void *d_out, void *d_totals, size_t num_segments, size_t segment_size, int variant, int tiles_per_wave, int waves_per_block, void *stream);

/* tcu_seg_scan_f16 for callers that cannot allocate device memory (code under HIP graph
 * capture, serving loops, harnesses that forbid hipMalloc): same arguments, same kernels, same
 * results, but the partition descriptors of the look-back path (TCU_VARIANT_AUTO with segments of
 * 2^21 halves and more, of 2^17 and more when there are fewer than 256 of them, of 2^19 and more from 2^30
 * elements on: the only path of tcu_seg_scan_f16 that takes temporary memory) live in a
 * 1 MiB + 256 B array that is part of the library's device code, so this entry point never calls
 * an allocating routine.  Limit: num_segments * segment_size <= 2^33 halves on that path (131072
 * partitions of 65536 halves; larger calls return TCU_ERR_UNSUPPORTED).  Each GPU holds one such
 * array: calls of this entry point that overlap in time on one GPU (different streams or
 * threads) race on it and must be serialised by the caller; calls on the same stream are fine.
 * The descriptors are spaced 256 bytes apart while the call has at most 4096 partitions (2^28 halves) and
 * closer beyond that, which costs a few per cent of speed.  The array is cleared by a kernel at the start of
 * every call.  For segments of 4096 ... 16384 halves the block scan's launch asks for LDS it leaves unused
 * (it caps the blocks per compute unit); the first such launch of a kernel by a host thread on a device reads the
 * kernel's attributes and raises its limit of dynamic LDS once (hipFuncGetAttributes, hipFuncSetAttribute: host-side
 * calls that allocate nothing and put nothing on the stream).  No counterpart in the reference,
 * whose kernels take no temporary memory. */
int tcu_seg_scan_f16_noalloc(const void *d_in, void *d_out, void *d_totals, size_t num_segments, size_t segment_size, int variant, int tiles_per_wave, int waves_per_block, void *stream);

/* Segments given by offsets (conventions of tcu_seg_reduce_offsets_f16; segments must not
 * overlap): d_out[i] = fp16( d_in[begin[j]] + ... + d_in[i] ) for i in [begin[j], end[j]);
 * elements of d_out outside every segment are not written.  In-place is allowed.
 * Hand-written counterpart of the reference's key-based library scan
 * (thrust::inclusive_scan_by_key, src/prefixsum/seg_thrust.cu:46-47) for segments
 * described by an offsets array (src/reduction/seg_cub_device.cu:18-22). */
int tcu_seg_scan_offsets_f16(const void *d_in, void *d_out, size_t num_segments, const void *d_begin_offsets, const void *d_end_offsets, int offset_bits, size_t expected_segment_size, void *stream);

/* Segments given by a key array: a segment is a run of equal consecutive keys (d_keys: n signed integers of
 * key_bits = 32 or 64 bits in device memory; n < 2^32).  d_keys, d_in and the scan's d_out must be 16-byte
 * aligned.  Workspace: the two-phase protocol of the full-array entry points below (16-byte aligned; the scan:
 * 256 bytes per 32768 elements + 256; the reduction: n/8 bytes of run-start bits + one key per 8 elements + 12
 * bytes per 4096 elements, about 0.63 n bytes with 32-bit keys and 1.13 n with 64-bit keys).
 *
 * tcu_seg_scan_by_key_f16: d_out[i] = fp16( sum of d_in[j .. i] ), j = the first element of i's run.  In place
 * (d_out == d_in) is allowed.  Hand-written counterpart of thrust::inclusive_scan_by_key(keys, keys + n, in, out)
 * as the reference calls it (src/prefixsum/seg_thrust.cu:46-47).
 *
 * tcu_seg_reduce_by_key_f16: for the r-th run, d_out[r] = fp16(sum of the run) and, if d_keys_out is not NULL,
 * d_keys_out[r] = its key; *d_num_runs (a 64-bit unsigned in device memory, may be NULL) receives the number of
 * runs, which is what thrust::reduce_by_key(keys, keys + n, in, keys_out, out) returns as the end of its output
 * (src/reduction/seg_thrust.cu:50-51).  d_out and d_keys_out need room for as many entries as there are runs
 * (at most n) and must not overlap d_in or d_keys.  The scan is one pass over keys and values with a decoupled
 * look-back on (head flag, value) pairs.  The reduction is five launches none of which waits for another block: the
 * keys are read once (run-start bits and counts), the values once; sums are added in index order, so the same
 * input gives the same bits every time. */
int tcu_seg_scan_by_key_f16(const void *d_keys, const void *d_in, void *d_out, size_t n, int key_bits, void *d_workspace, size_t *workspace_bytes, void *stream);
int tcu_seg_reduce_by_key_f16(const void *d_keys, const void *d_in, void *d_keys_out, void *d_out, void *d_num_runs, size_t n, int key_bits, void *d_workspace, size_t *workspace_bytes, void *stream);

/* d_out[s*S + i] += d_partial_sums[s]  (one fp16 addition per element).
 * Replaces add_partial_sums (reference src/prefixsum/kernel.cuh:31-43). */
int tcu_add_partial_sums_f16(void *d_out, const void *d_partial_sums, size_t num_segments, size_t segment_size, void *stream);

/* ---- full-array reduction and prefix sum ---------------------------------------------------- */

/* Two-phase workspace protocol (as the reference uses cub's, src/reduction/wmma_2kers.cu:49-53):
 * call with d_workspace == NULL to receive the byte count in *workspace_bytes, then again
 * with a device buffer of at least that size (256-byte aligned).  The workspace needs no
 * initialisation; its contents are scratch.
 * segment_size is the tile each block/wave reduces before the cross-block step (the
 * reference's SEGMENT_SIZE template argument of the *_2KERS_* / *_3KERS / *_ATOMIC_*
 * benchmarks); 0 = default. */

/* d_out[0] = fp16(sum of all n elements).  Replaces compute_wmma_reduction_cg /
 * _atomic_w_syncthreads / _atomic_w_atomicballot (reference src/reduction/kernel.cuh:564-786)
 * and the segmented-kernel + cub::DeviceReduce sequence (src/reduction/wmma_2kers.cu:63-88). */
int tcu_full_reduce_f16(const void *d_in, void *d_out, size_t n, void *d_workspace, size_t *workspace_bytes, int strategy, size_t segment_size, int waves_per_block, void *stream);

/* d_out[i] = fp16(d_in[0] + ... + d_in[i]).  Replaces compute_wmma_prefixsum_cg /
 * _atomic_w_atomicballot (reference src/prefixsum/kernel.cuh:779-972) and the 3-kernel
 * sequence (src/prefixsum/wmma_3kers.cu:60-82).
 * The single-pass strategies are not bit-reproducible on general inputs: a partition's fp32 carry is the sum of the
 * aggregates of the predecessors it had to walk plus the first published prefix it met, and where that prefix is met
 * depends on timing, so the last bit of a carry (and of outputs that round differently because of it) can differ
 * between two runs.  Every run is within 2 ulp_fp16 + 1e-3 * sqrt(n) of the exact sum; inputs whose partial sums are
 * exact in fp32 give identical bits every time.  TCU_FULL_MULTI_KERNEL and the reductions add in a fixed order.
 * A wait for another partition that expires ("lookback_poll_limit" in tcu_scope_dev.h) is reported: the call still
 * returns TCU_OK (nothing is known when it returns), d_out then holds NaN from the waiting partition on, and word 1
 * of the workspace (a 32-bit unsigned, zeroed by every call) holds the number of partitions that gave up. */
int tcu_full_scan_f16(const void *d_in, void *d_out, size_t n, void *d_workspace, size_t *workspace_bytes, int strategy, size_t segment_size, int waves_per_block, void *stream);

/* ---- dense contractions -------------------------------------------------------------------- */

/* y = alpha * A x + beta * y.  A: M x K row-major fp16, x: K fp16, y: M fp32.
 * Replaces compute_wmma_gemv_naive / compute_wmma_gemv_sharedmem (reference
 * src/gemv/wmma_naive.cu:29-94, wmma_sharedmem.cu:43-137); note the reference stores A
 * column-major (tcu_gemv_col_major_* below take that layout) and returns y as column 0 of an M x 16 matrix.
 * variant: TCU_VARIANT_AUTO, TCU_VARIANT_WAVE_SHUFFLE (dot products + DPP),
 * TCU_VARIANT_MFMA_16N (16-row strips on MFMA with x as a replicated B operand, the
 * reference's formulation) or TCU_VARIANT_MFMA_256N (a 1 KiB tile of a row as the MFMA A
 * operand, the matching tile of x as the B operand, trace of the accumulated product: the
 * launch shapes and loads of the dot-product form with the arithmetic on the matrix unit). */
int tcu_gemv_f16_f32(const void *d_A, const void *d_x, void *d_y, size_t M, size_t K, float alpha, float beta, int variant, void *stream);

/* The same product with A column-major, element (m, k) at d_A[m + k * lda] (lda >= M, in elements): the layout in which
 * the reference's own kernels and its cuBLAS baseline take A (src/gemv/wmma_naive.cu:33-36, 61: lda = M_GLOBAL,
 * fragments loaded col_major), so a caller that holds the reference's buffers passes them as they are.  y: M values of
 * fp32 (_f32) or fp16 (_f16).  Columns are read 1 KiB at a time and scaled by x[k]; the sums of stretches of K meet in
 * M floats per stretch of stream-ordered temporary memory (about 1024 / (M / 512) stretches) and are added in a fixed order.  K a
 * multiple of 8, lda a multiple of 8 and 16-byte aligned A and x take the fast kernels, anything else a scalar one. */
int tcu_gemv_col_major_f16_f32(const void *d_A, size_t lda, const void *d_x, void *d_y, size_t M, size_t K, float alpha, float beta, void *stream);
int tcu_gemv_col_major_f16_f16(const void *d_A, size_t lda, const void *d_x, void *d_y, size_t M, size_t K, float alpha, float beta, void *stream);

/* D = alpha * A B + beta * C.  A: M x K row-major fp16; B: K x N column-major fp16
 * (element (k,n) at d_B[n*K + k]); C, D: M x N row-major fp32 (C may equal D, may be
 * NULL when beta == 0).  Operand layouts of reference compute_gemm (src/gemm/wmma.cu:15-18,
 * 171-365).  variant: TCU_VARIANT_AUTO / TCU_VARIANT_BLOCK_LDS = LDS-tiled MFMA kernel
 * (reference compute_gemm, compute_gemm_sharedmem); TCU_VARIANT_WAVE_SHUFFLE is not
 * defined here; TCU_VARIANT_MFMA_16N = one tile per wave straight from global memory
 * (reference compute_gemm_naive, src/gemm/wmma_naive.cu:33-88). */
int tcu_gemm_f16_f32(const void *d_A, const void *d_B, const void *d_C, void *d_D, size_t M, size_t N, size_t K, float alpha, float beta, int variant, void *stream);

/* The fp16-output twins: y (GEMV) and C, D (GEMM) hold fp16, alpha and beta are applied in
 * fp32 and the result is rounded once (to nearest even).  They replace
 * compute_wmma_hgemv_naive (reference src/gemv/wmma_naive.cu:96-160), compute_hgemm
 * (src/gemm/wmma.cu:367-560) and compute_hgemm_naive (src/gemm/wmma_naive.cu:90-145).  The
 * reference accumulates those in fp16 inside the WMMA unit; the MFMA unit accumulates in fp32
 * only, so products are summed in fp32 here as in the fp32-output entry points.  Layouts,
 * variants and the C == D allowance are the same; D and C must be 4-byte aligned for the
 * tiled GEMM kernels (any alignment falls back to the scalar kernel under AUTO). */
int tcu_gemv_f16_f16(const void *d_A, const void *d_x, void *d_y, size_t M, size_t K, float alpha, float beta, int variant, void *stream);
int tcu_gemm_f16_f16(const void *d_A, const void *d_B, const void *d_C, void *d_D, size_t M, size_t N, size_t K, float alpha, float beta, int variant, void *stream);

/* ---- fills, conversions, inputs ---------------------------------------------------------------- */

/* d[i] = (half) value.  Replaces cuda_memory_set / setFP16 (reference
 * src/utils/cuda_helpers.cuh:123-181). */
int tcu_fill_f16(void *d, float value, size_t n, void *stream);
/* d_out[i] = (half) d_in[i].  Replaces convertFp32ToFp16 (src/utils/cuda_helpers.cuh:116-121). */
int tcu_convert_f32_to_f16(void *d_out, const void *d_in, size_t n, void *stream);
/* Counter-based seeded inputs (element i depends on (seed, first + i) only).  Stands in
 * for the reference's cuRAND / rand() fills (src/gemm/wmma_naive.cu:177-181,
 * src/gemm/wmma.cu:110-127), which are not reproducible without cuRAND.  UNIFORM, GRID
 * and SMALLINT are bit-identical to the host generator used by the tests. */
int tcu_generate_f16(void *d, size_t n, uint64_t seed, int dist, size_t first, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* TCU_SCOPE_H */
