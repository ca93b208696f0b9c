/*
 * CPU oracle for the tcu_scope hot path (segmented / full reduction and inclusive
 * prefix sum over fp16 data, fp16 GEMV / GEMM).
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only the test-suite, the smoke
 * check and the CPU-baseline leg of the benchmark may link or call it; the GPU
 * library never does.
 *
 * Two families of functions live here:
 *   *_ref  : the reference's CPU verification loops restated (fp32 sequential running
 *            sum per segment, fp16 result).  In the reference these loops sit behind
 *            "#if 0" after every timed loop; each function cites the one it follows.
 *   *_f64  : the mathematical definition (sequential fp64 sum of the exact fp16 input
 *            values), which is what GPU results are checked against.
 *
 * Pinning status (what each function is checked against, in tests/test_oracle_*.py):
 *   fp16 <-> fp32 conversion : all 65536 half bit patterns and 2^20 random floats
 *                              against numpy's IEEE binary16 conversion; pinned.
 *   generator                : published SplitMix64 known-answer vector (seed 1234567)
 *                              and an independent numpy restatement; pinned.
 *   seg/full reduce+scan _ref: numpy float32 cumsum (sequential), the reference's
 *                              constant-0.001 fixture in closed form within the
 *                              reference's own tolerances, exact-grid inputs; pinned.
 *   *_f64                    : math.fsum / numpy float64 cumsum, one-hot and all-zero
 *                              inputs, scan-last == reduce; pinned.
 *   gemv/gemm _f64           : numpy float64 matmul and integer-exact inputs; pinned.
 *   The reference's GPU kernels accumulate in fp16 inside WMMA fragments; that
 *   rounding order is NOT reproduced anywhere here (parity unpinned for it, and not
 *   targeted: the build accumulates in fp32 and is judged against the fp64 sum).
 */
#ifndef TCU_ORACLE_H
#define TCU_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- fp16 conversion ---------------------------------------------------------- */
/* half -> float, bit recipe of reference src/utils/fp16_conversion.hpp:91-114. */
float tcu_oracle_f16_to_f32(uint16_t h);
/* float -> half, IEEE round-to-nearest-even (what a device `(half) float` cast does,
 * reference src/utils/cuda_helpers.cuh:116-132; NOT the truncating
 * approx_float_to_half of fp16_conversion.hpp:63-88). */
uint16_t tcu_oracle_f32_to_f16(float f);
/* double -> half, RNE in one rounding step. */
uint16_t tcu_oracle_f64_to_f16(double d);
/* Size of one unit in the last place of fp16 at the magnitude of v (2^-24 for
 * subnormals and zero, 32 at the top binade and beyond). */
double tcu_oracle_ulp_f16(double v);

/* ---- inputs --------------------------------------------------------------------- */
enum {
  TCU_ORACLE_DIST_UNIFORM = 0, /* uniform in [-1,1), 24-bit, RNE to fp16, never +1.0 */
  TCU_ORACLE_DIST_GRID    = 1, /* k/2048, k in [-2048,2047]: exact in fp16 */
  TCU_ORACLE_DIST_NORMAL  = 2, /* N(0,1) by Box-Muller, RNE to fp16 */
  TCU_ORACLE_DIST_SMALLINT = 3 /* {0,1,2}: the reference's rand()%3 GEMM fill */
};
/* i-th output of SplitMix64 started at `seed` (i counted from 0). */
uint64_t tcu_oracle_splitmix64(uint64_t seed, uint64_t i);
/* Counter-based generator: element i depends on (seed, i) only. */
void tcu_oracle_generate_f16(uint16_t *out, size_t n, uint64_t seed, int dist);
/* Same generator for elements [first, first+n). */
void tcu_oracle_generate_f16_range(uint16_t *out, size_t first, size_t n, uint64_t seed, int dist);
/* Constant fill with a float -> half cast: reference cuda_memory_set / setFP16,
 * src/utils/cuda_helpers.cuh:123-181. */
void tcu_oracle_fill_f16(uint16_t *out, float value, size_t n);
/* Element-wise float -> half cast (round to nearest even): reference convertFp32ToFp16,
 * src/utils/cuda_helpers.cuh:116-121. */
void tcu_oracle_convert_f32_to_f16(uint16_t *out, const float *in, size_t n);

/* ---- reference CPU path (fp32 sequential, fp16 out) ------------------------------- */
/* reference src/reduction/seg_wmma_16.cu:77-104, seg_wmma_256n.cu:85-121 */
void tcu_oracle_seg_reduce_ref(const uint16_t *in, uint16_t *out, size_t num_segments, size_t segment_size);
/* the same loop split over `nthreads` contiguous segment ranges (pthreads) */
void tcu_oracle_seg_reduce_ref_mt(const uint16_t *in, uint16_t *out, size_t num_segments, size_t segment_size, int nthreads);
/* reference src/prefixsum/seg_wmma_16.cu:79-107 */
void tcu_oracle_seg_scan_ref(const uint16_t *in, uint16_t *out, size_t num_segments, size_t segment_size);
void tcu_oracle_seg_scan_ref_mt(const uint16_t *in, uint16_t *out, size_t num_segments, size_t segment_size, int nthreads);
/* reference src/reduction/wmma_2kers.cu:106-129 */
void tcu_oracle_full_reduce_ref(const uint16_t *in, uint16_t *out, size_t n);
/* reference src/prefixsum/wmma_3kers.cu:92-116 */
void tcu_oracle_full_scan_ref(const uint16_t *in, uint16_t *out, size_t n);
/* reference src/prefixsum/kernel.cuh:31-43 (add_partial_sums): out[s*S+i] += ps[s],
 * one fp16 addition per element. */
void tcu_oracle_add_partial_sums_ref(uint16_t *out, const uint16_t *partial_sums, size_t num_segments, size_t segment_size);

/* Segments given by offsets: segment j covers in[begin[j], end[j]) and is empty when
 * end[j] <= begin[j]: the argument convention of cub::DeviceSegmentedReduce::Sum as the
 * reference calls it (src/reduction/seg_cub_device.cu:46-48: d_offsets, d_offsets + 1).
 * fp32 sequential sum, fp16 result, like the fixed-size loop above. */
void tcu_oracle_seg_reduce_offsets_ref(const uint16_t *in, uint16_t *out, size_t num_segments, const int64_t *begin, const int64_t *end);

/* Inclusive prefix sums inside every segment of an offsets array: out[i] for i in
 * [begin[j], end[j]) is the fp32 running sum of in[begin[j] .. i] rounded to fp16; elements
 * of `out` outside every segment are left as they are.  Offsets convention as above. */
void tcu_oracle_seg_scan_offsets_ref(const uint16_t *in, uint16_t *out, size_t num_segments, const int64_t *begin, const int64_t *end);

/* ---- definition (fp64) -------------------------------------------------------------- */
void tcu_oracle_seg_scan_offsets_f64(const uint16_t *in, double *out, size_t num_segments, const int64_t *begin, const int64_t *end);
void tcu_oracle_seg_reduce_offsets_f64(const uint16_t *in, double *out, size_t num_segments, const int64_t *begin, const int64_t *end);
void tcu_oracle_seg_reduce_f64(const uint16_t *in, double *out, size_t num_segments, size_t segment_size);
void tcu_oracle_seg_scan_f64(const uint16_t *in, double *out, size_t num_segments, size_t segment_size);
/* Segments as runs of equal consecutive keys: the semantics of thrust::inclusive_scan_by_key and
 * thrust::reduce_by_key as the reference calls them (src/prefixsum/seg_thrust.cu:46-47,
 * src/reduction/seg_thrust.cu:50-51).  _ref: fp32 running sum per run, fp16 results; _f64: the definition.
 * The reductions return the number of runs and fill keys_out / out with one entry per run. */
void tcu_oracle_seg_scan_by_key_ref(const int64_t *keys, const uint16_t *in, uint16_t *out, size_t n);
void tcu_oracle_seg_scan_by_key_f64(const int64_t *keys, const uint16_t *in, double *out, size_t n);
size_t tcu_oracle_seg_reduce_by_key_ref(const int64_t *keys, const uint16_t *in, int64_t *keys_out, uint16_t *out, size_t n);
size_t tcu_oracle_seg_reduce_by_key_f64(const int64_t *keys, const uint16_t *in, int64_t *keys_out, double *out, size_t n);

/* y = alpha*A*x + beta*y0; A is M x K row-major fp16, x fp16, y0 may be NULL when beta==0 */
void tcu_oracle_gemv_f64(const uint16_t *A, const uint16_t *x, const float *y0, double *y, size_t M, size_t K, double alpha, double beta);
/* D = alpha*A*B + beta*C; A M x K row-major, B K x N column-major (element (k,n) at
 * B[n*K+k]), C/D M x N row-major: operand layouts of reference src/gemm/wmma.cu:15-18.
 * Rows [row0,row0+rows) only. */
void tcu_oracle_gemm_f64(const uint16_t *A, const uint16_t *B, const float *C, double *D, size_t M, size_t N, size_t K, double alpha, double beta, size_t row0, size_t rows);

/* ---- tolerance rule ------------------------------------------------------------------ */
/* |got - ref| <= ulps*ulp_f16(ref) + abs_per_sqrt*sqrt(segment_size); an fp64 value
 * that rounds to +-inf in fp16 must be matched by the same infinity.  Returns the
 * number of violations; *worst receives the largest (err - allowance), *first_bad the
 * first offending index (or n). */
size_t tcu_oracle_check_f16(const uint16_t *got, const double *ref, size_t n, double ulps, double abs_per_sqrt, size_t segment_size, double *worst, size_t *first_bad);
/* fp32 results against fp64: |got-ref| <= rel*max(|ref|, scale). */
size_t tcu_oracle_check_f32_rel(const float *got, const double *ref, size_t n, double rel, double scale, double *worst, size_t *first_bad);

#ifdef __cplusplus
}
#endif
#endif
