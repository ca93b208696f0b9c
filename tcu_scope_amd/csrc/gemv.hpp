// y = alpha * A x + beta * y;  A: M x K row-major fp16, x: K fp16, y: M values of OUT = float
// or half_t (the reference's compute_wmma_hgemv_naive keeps y in fp16,
// src/gemv/wmma_naive.cu:96-160); products accumulate in fp32 either way.
//
// The operation streams A once (2*M*K bytes) and is bound by HBM bandwidth.
//   gemv_dot_kernel  : each wave owns ROWS consecutive rows; per step every lane loads one
//                      128-bit chunk of x and the matching chunk of each row (a wave reads
//                      1 KiB of a row contiguously), multiplies with packed fp16 dot
//                      products into fp32, and finishes with a DPP wave reduction.
//   gemv_block_kernel: rows of 8 KiB and more: a block of waves shares two rows (the access
//                      shape of the block-per-segment reduction), partials meet in LDS.
//   gemv_strip_lds_kernel, gemv_mfma_kernel : the reference's formulation (GEMV as a 16-wide GEMM,
//                      src/gemv/wmma_naive.cu:29-94): a block owns a 16-row strip, the strip
//                      is the A operand of v_mfma_f32_16x16x32_f16 and x, replicated over
//                      the 16 columns, the B operand; the block's waves split K (k order
//                      inside a step is permuted identically for A and x, which a
//                      contraction does not see).
//   Both of the first two also run with the matrix unit in place of the dot products
//   (GemvAcc<true>: a row tile times the x tile, trace of the product), which keeps their
//   access shape.
//   gemv_generic_kernel : any M, K (scalar loads).
#pragma once

#include "seg_reduce.hpp"

namespace tcu {

template <typename OUT>
TCU_DEVICE void gemv_update(OUT *p, float s, float alpha, float beta) {
  *p = (OUT)(beta == 0.0f ? alpha * s : alpha * s + beta * (float)*p);
}

TCU_DEVICE float dot8(half8_t a, half8_t x, float acc) {
  acc = fdot2(__builtin_shufflevector(a, a, 0, 1), __builtin_shufflevector(x, x, 0, 1), acc);
  acc = fdot2(__builtin_shufflevector(a, a, 2, 3), __builtin_shufflevector(x, x, 2, 3), acc);
  acc = fdot2(__builtin_shufflevector(a, a, 4, 5), __builtin_shufflevector(x, x, 4, 5), acc);
  acc = fdot2(__builtin_shufflevector(a, a, 6, 7), __builtin_shufflevector(x, x, 6, 7), acc);
  return acc;
}

// Accumulator of one row's dot product, one tile (64 chunks, lane l holding chunk l of the row
// and of x) at a time.  MFMA = false: packed fp16 dot products per lane.  MFMA = true: the row
// tile is the 16 x 32 A operand of v_mfma_f32_16x16x32_f16 and the x tile, loaded the same way,
// the 32 x 16 B operand.  Lane i + 16 b supplies A[i][8b .. 8b+7] and B[8b .. 8b+7][i], i.e. the
// same 8 positions of the row and of x, so the diagonal D[i][i] = sum_k A[i][k] B[k][i] is the
// dot product over the 32 positions of lanes i, i + 16, i + 32, i + 48, and the trace of the
// accumulated D is the dot product of the whole tiles: a GEMV on the matrix unit whose loads
// are as contiguous as those of the dot-product form (15 of 16 products are discarded, which
// a bandwidth-bound kernel does not notice).
template <bool MFMA>
struct GemvAcc {
  float v = 0.0f;
  TCU_DEVICE void add(half8_t a, half8_t x) { v = dot8(a, x, v); }
  TCU_DEVICE float lane_value(int) const { return v; }
};
template <>
struct GemvAcc<true> {
  float4_t v = {0.0f, 0.0f, 0.0f, 0.0f};
  TCU_DEVICE void add(half8_t a, half8_t x) { v = mfma_16x16x32(a, x, v); }
  // lane l holds D[4 * (l / 16) + j][l % 16], j = 0 .. 3: a diagonal element iff (l % 16) / 4 == l / 16, at j = l % 4
  TCU_DEVICE float lane_value(int lane) const {
    const int j = lane & 3;
    const float d = j == 0 ? v[0] : j == 1 ? v[1] : j == 2 ? v[2] : v[3];
    return ((lane & 15) >> 2) == (lane >> 4) ? d : 0.0f;
  }
};

// K must be a multiple of 8; rows are 16-byte aligned.
template <int ROWS, int UK, bool NT, typename OUT, bool MFMA = false>
__global__ __launch_bounds__(kMaxBlock) void gemv_dot_kernel(const half8_t *__restrict__ A, const half8_t *__restrict__ x, OUT *__restrict__ y, size_t M, size_t k_chunks, float alpha,
                                                              float beta) {
  const int lane = lane_id();
  const size_t row0 = ((size_t)blockIdx.x * (blockDim.x >> 6) + wave_in_block()) * ROWS;
  if (row0 >= M) return;
  GemvAcc<MFMA> acc[ROWS];
  const half8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
  for (size_t c0 = 0; c0 < k_chunks; c0 += (size_t)64 * UK) {
    half8_t xv[UK], av[UK][ROWS];
#pragma unroll
    for (int u = 0; u < UK; u++) {
      const size_t c = c0 + (size_t)u * 64 + lane;
      const bool ok = c < k_chunks;
      xv[u] = ok ? x[c] : zero;
#pragma unroll
      for (int r = 0; r < ROWS; r++) {
        const size_t row = row0 + r < M ? row0 + r : M - 1;  // clamp: duplicates are discarded below
        av[u][r] = ok ? load_chunk<NT>(A + row * k_chunks + c) : zero;
      }
    }
#pragma unroll
    for (int u = 0; u < UK; u++)
#pragma unroll
      for (int r = 0; r < ROWS; r++) acc[r].add(av[u][r], xv[u]);
  }
#pragma unroll
  for (int r = 0; r < ROWS; r++) {
    const float s = lane_group_sum<6>(acc[r].lane_value(lane));
    if (lane == 63 && row0 + r < M) gemv_update(y + row0 + r, s, alpha, beta);
  }
}

// Long rows: a block of WPB waves shares ROWS consecutive rows; wave w takes the tiles
// w*U .. w*U+U-1 of every step of WPB*U tiles (the x chunks it loads serve all ROWS rows),
// partial dot products meet in LDS.  Same access shape as the block-per-segment reduction,
// which is what moves long contiguous rows fastest.
template <int ROWS, int U, bool NT, typename OUT, bool MFMA = false>
__global__ __launch_bounds__(kMaxBlock) void gemv_block_kernel(const half8_t *__restrict__ A, const half8_t *__restrict__ x, OUT *__restrict__ y, size_t M, size_t k_chunks, float alpha,
                                                                float beta) {
  __shared__ float partial[ROWS][kMaxWaves];
  const int lane = lane_id(), wave = wave_in_block();
  const int WPB = (int)(blockDim.x >> 6);
  const size_t row0 = (size_t)blockIdx.x * ROWS;
  const half8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
  GemvAcc<MFMA> acc[ROWS];
  for (size_t c0 = (size_t)wave * U * 64; c0 < k_chunks; c0 += (size_t)WPB * U * 64) {
    half8_t xv[U], av[ROWS][U];
#pragma unroll
    for (int u = 0; u < U; u++) {
      const size_t c = c0 + (size_t)u * 64 + lane;
      const bool ok = c < k_chunks;
      xv[u] = ok ? x[c] : zero;
#pragma unroll
      for (int r = 0; r < ROWS; r++) {
        const size_t row = row0 + r < M ? row0 + r : M - 1;
        av[r][u] = ok ? load_chunk<NT>(A + row * k_chunks + c) : zero;
      }
    }
#pragma unroll
    for (int u = 0; u < U; u++)
#pragma unroll
      for (int r = 0; r < ROWS; r++) acc[r].add(av[r][u], xv[u]);
  }
#pragma unroll
  for (int r = 0; r < ROWS; r++) {
    const float s = lane_group_sum<6>(acc[r].lane_value(lane));
    if (lane == 63) partial[r][wave] = s;
  }
  __syncthreads();
  if (threadIdx.x < ROWS && row0 + threadIdx.x < M) {
    float s = 0.0f;
    for (int w = 0; w < WPB; w++) s += partial[threadIdx.x][w];
    gemv_update(y + row0 + threadIdx.x, s, alpha, beta);
  }
}

// K must be a multiple of 8.  A block per 16-row strip; its waves split K and meet in LDS (one wave per
// strip leaves a 16384-row matrix with 1024 waves, too few loads in flight: 171 us for 16384 x 16384 where
// the dot-product kernel needs 80).  Lane (r, b) reads chunks 4 s + b, s = 0 .. 3, of each half step, so that
// one load instruction reads 64 contiguous bytes of each of the 16 rows.
template <bool NT, typename OUT>
__global__ __launch_bounds__(kMaxBlock) void gemv_mfma_kernel(const half8_t *__restrict__ A, const half8_t *__restrict__ x, OUT *__restrict__ y, size_t M, size_t k_chunks, float alpha,
                                                               float beta) {
  __shared__ float partial[kMaxWaves][16];
  const int lane = lane_id(), wave = wave_in_block();
  const int WPB = (int)(blockDim.x >> 6);
  const int r = lane & 15, b = lane >> 4;
  const size_t row0 = (size_t)blockIdx.x * 16;
  const size_t row = row0 + r < M ? row0 + r : M - 1;
  const half8_t *arow = A + row * k_chunks;
  // this wave's share of K, in steps of 256 k = 32 chunks
  const size_t steps = (k_chunks + 31) / 32, per_wave = (steps + WPB - 1) / WPB;
  const size_t c_begin = (size_t)wave * per_wave * 32;
  const size_t c_end = c_begin + per_wave * 32 < k_chunks ? c_begin + per_wave * 32 : k_chunks;
  float4_t acc = {0, 0, 0, 0};
  constexpr int kSteps = 1;  // steps of 256 k whose loads are in flight together (two measured 181 us against 108 at 16384 x 16384)
  for (size_t c0 = c_begin; c0 < c_end; c0 += 32 * kSteps) {
    half8_t av[kSteps][2][4], xv[kSteps][2][4];
#pragma unroll
    for (int t = 0; t < kSteps; t++)
#pragma unroll
      for (int h = 0; h < 2; h++)
#pragma unroll
        for (int s = 0; s < 4; s++) {
          const size_t c = c0 + (size_t)t * 32 + (size_t)h * 16 + 4 * s + b;
          const bool ok = c < c_end;
          const half8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
          av[t][h][s] = ok ? load_chunk<NT>(arow + c) : zero;
          xv[t][h][s] = ok ? x[c] : zero;
        }
#pragma unroll
    for (int t = 0; t < kSteps; t++)
#pragma unroll
      for (int h = 0; h < 2; h++)
#pragma unroll
        for (int s = 0; s < 4; s++) acc = mfma_16x16x32(av[t][h][s], xv[t][h][s], acc);
  }
  // every column of D holds the strip's 16 partial results; column 0 hands them over
  if (r == 0) {
#pragma unroll
    for (int i = 0; i < 4; i++) partial[wave][4 * b + i] = acc[i];
  }
  __syncthreads();
  if (threadIdx.x < 16 && row0 + threadIdx.x < M) {
    float sum = 0.0f;
    for (int w = 0; w < WPB; w++) sum += partial[w][threadIdx.x];
    gemv_update(y + row0 + threadIdx.x, sum, alpha, beta);
  }
}

// The same formulation with the strip staged through LDS: K a multiple of 512.  A step takes 512 k: seventeen
// global -> LDS transfers move 1 KiB of each of the strip's rows and of x (whole cache lines, lane-contiguous, no
// registers), then sixteen products read the 16 x 32 operand blocks and the matching 32 values of x back from LDS
// (rows 16 bytes further apart than their length, so that the sixteen rows of one read fall into different
// banks).  The waves of a block split K and own their LDS, so there is no block barrier inside the loop (a
// second buffer per wave, with the next step's transfers in flight during the products, measured the same:
// 95.7 against 93.2 us at 16384 x 16384; the register form above 106).
constexpr int kGemvStripWaves = 4;
constexpr int kGemvStripRow = 512 + 8;  // halves per staged row
template <typename OUT>
__global__ __launch_bounds__(kGemvStripWaves * 64) void gemv_strip_lds_kernel(const half8_t *__restrict__ A, const half8_t *__restrict__ x, OUT *__restrict__ y, size_t M, size_t k_chunks, float alpha,
                                                                             float beta) {
  __shared__ __attribute__((aligned(16))) half_t staged[kGemvStripWaves][17 * kGemvStripRow];
  __shared__ float partial[kGemvStripWaves][16];
  const int lane = lane_id(), wave = wave_in_block();
  const int WPB = (int)(blockDim.x >> 6);
  const int r = lane & 15, b = lane >> 4;
  const size_t row0 = (size_t)blockIdx.x * 16;
  const size_t steps = k_chunks / 64, per_wave = (steps + WPB - 1) / WPB;
  const size_t s_begin = (size_t)wave * per_wave, s_end = s_begin + per_wave < steps ? s_begin + per_wave : steps;
  float4_t acc = {0, 0, 0, 0};
  half_t *mine = staged[wave];
  for (size_t s = s_begin; s < s_end; s++) {
    const size_t c0 = s * 64;
#pragma unroll
    for (int rr = 0; rr < 16; rr++) {
      const size_t row = row0 + rr < M ? row0 + rr : M - 1;
      load_chunk_to_lds(A + row * k_chunks + c0, (uint32_t)lane * 16u, lds_address_of(mine + rr * kGemvStripRow));
    }
    load_chunk_to_lds(x + c0, (uint32_t)lane * 16u, lds_address_of(mine + 16 * kGemvStripRow));
    wait_vector_loads<0>();
    wave_lds_fence();  // every lane's transfers have landed before any lane reads another lane's bytes
#pragma unroll
    for (int q = 0; q < 16; q++) {
      const half8_t a = *reinterpret_cast<const half8_t *>(mine + r * kGemvStripRow + q * 32 + b * 8);
      const half8_t xv = *reinterpret_cast<const half8_t *>(mine + 16 * kGemvStripRow + q * 32 + b * 8);
      acc = mfma_16x16x32(a, xv, acc);
    }
    wave_lds_fence();  // the reads above are done before the next step's transfers may land
  }
  if (r == 0) {
#pragma unroll
    for (int i = 0; i < 4; i++) partial[wave][4 * b + i] = acc[i];
  }
  __syncthreads();
  if (threadIdx.x < 16 && row0 + threadIdx.x < M) {
    float sum = 0.0f;
    for (int w = 0; w < WPB; w++) sum += partial[w][threadIdx.x];
    gemv_update(y + row0 + threadIdx.x, sum, alpha, beta);
  }
}

template <typename OUT>
__global__ __launch_bounds__(kMaxBlock) void gemv_generic_kernel(const uint16_t *__restrict__ A, const uint16_t *__restrict__ x, OUT *__restrict__ y, size_t M, size_t K, float alpha, float beta) {
  const int lane = lane_id();
  const size_t row = (size_t)blockIdx.x * (blockDim.x >> 6) + wave_in_block();
  if (row >= M) return;
  float acc = 0.0f;
  for (size_t k = lane; k < K; k += 64) acc += (float)__builtin_bit_cast(half_t, A[row * K + k]) * (float)__builtin_bit_cast(half_t, x[k]);
  acc = lane_group_sum<6>(acc);
  if (lane == 63) gemv_update(y + row, acc, alpha, beta);
}

// ---- A column-major ------------------------------------------------------------------------------------------
// y = alpha * A x + beta * y with element (m, k) of A at A[m + k * lda]: the layout of the reference's
// compute_wmma_gemv_naive (src/gemv/wmma_naive.cu:33-36, 61: lda = M_GLOBAL, fragments loaded col_major) and of the
// cuBLAS call beside it.  A column is contiguous, so the product is a sum of columns scaled by x[k]: a wave owns
// kColSlabRows consecutive rows (a lane 8 of them: one 16-byte load per column, the wave 1 KiB) and every WPB-th
// group of 8 columns of its block's stretch of K; the waves of a block add up in LDS and the block writes one fp32
// partial sum per row; gemv_col_finish_kernel adds the partials of a row in the order of the stretches and applies
// alpha, beta and y.  Every sum is taken in a fixed order.
constexpr int kColSlabRows = 512;

template <int WPB, int GROUPS, bool NT>
__global__ __launch_bounds__(WPB * 64) void gemv_col_partials_kernel(const uint16_t *__restrict__ A, size_t lda, const half8_t *__restrict__ x, float *__restrict__ partials, size_t M, size_t K,
                                                                     unsigned slabs, size_t cols_per_block) {
  __shared__ float sums[WPB][kColSlabRows];
  const int lane = lane_id(), wave = wave_in_block();
  const size_t slab = blockIdx.x % slabs, stretch = blockIdx.x / slabs;
  const size_t r0 = slab * kColSlabRows + (size_t)lane * 8;
  const int valid = r0 >= M ? 0 : (M - r0 >= 8 ? 8 : (int)(M - r0));
  const size_t k_lo = stretch * cols_per_block, k_hi = k_lo + cols_per_block < K ? k_lo + cols_per_block : K;
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; i++) acc[i] = 0.0f;
  // GROUPS groups of 8 columns per wave and round (8 * GROUPS loads in flight); K is a multiple of 8: whole groups
  for (size_t kb = k_lo + (size_t)wave * 8 * GROUPS; kb < k_hi; kb += (size_t)WPB * 8 * GROUPS) {
    half8_t xs[GROUPS], a[GROUPS][8];
#pragma unroll
    for (int g = 0; g < GROUPS; g++) {
      const size_t kg = kb + (size_t)g * 8;
      const bool there = kg < k_hi;  // wave-uniform
      xs[g] = there ? x[kg / 8] : half8_t{0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
      for (int j = 0; j < 8; j++) {
        const uint16_t *col = A + (kg + j) * lda + r0;
        a[g][j] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
        if (there && valid == 8) {
          a[g][j] = load_chunk<NT>(reinterpret_cast<const half8_t *>(col));
        } else if (there) {
#pragma unroll
          for (int i = 0; i < 8; i++)
            if (i < valid) a[g][j][i] = __builtin_bit_cast(half_t, col[i]);
        }
      }
    }
#pragma unroll
    for (int g = 0; g < GROUPS; g++) {
#pragma unroll
      for (int j = 0; j < 8; j++) {
        const float xk = (float)xs[g][j];
#pragma unroll
        for (int i = 0; i < 8; i++) acc[i] = __builtin_fmaf((float)a[g][j][i], xk, acc[i]);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < 8; i++) sums[wave][lane * 8 + i] = acc[i];
  __syncthreads();
  for (int r = (int)threadIdx.x; r < kColSlabRows; r += WPB * 64) {
    const size_t row = slab * kColSlabRows + r;
    if (row >= M) break;
    float s = 0.0f;
#pragma unroll
    for (int w = 0; w < WPB; w++) s += sums[w][r];
    partials[stretch * M + row] = s;
  }
}

template <typename OUT>
__global__ __launch_bounds__(256) void gemv_col_finish_kernel(const float *__restrict__ partials, OUT *__restrict__ y, size_t M, unsigned stretches, float alpha, float beta) {
  const size_t row = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (row >= M) return;
  float s = 0.0f;
  unsigned c = 0;
  for (; c + 8 <= stretches; c += 8) {  // eight loads in flight, added in the order of the stretches
    float p[8];
#pragma unroll
    for (int i = 0; i < 8; i++) p[i] = partials[(size_t)(c + i) * M + row];
#pragma unroll
    for (int i = 0; i < 8; i++) s += p[i];
  }
  for (; c < stretches; c++) s += partials[(size_t)c * M + row];
  gemv_update(y + row, s, alpha, beta);
}

// any M, K, lda, alignment: a thread per row, the threads of a wave read 128 contiguous bytes of a column
template <typename OUT>
__global__ __launch_bounds__(256) void gemv_col_generic_kernel(const uint16_t *__restrict__ A, size_t lda, const uint16_t *__restrict__ x, OUT *__restrict__ y, size_t M, size_t K, float alpha,
                                                               float beta) {
  const size_t row = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (row >= M) return;
  float s = 0.0f;
  for (size_t k = 0; k < K; k++) s = __builtin_fmaf((float)__builtin_bit_cast(half_t, A[k * lda + row]), (float)__builtin_bit_cast(half_t, x[k]), s);
  gemv_update(y + row, s, alpha, beta);
}

}  // namespace tcu
