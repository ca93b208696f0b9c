// Segmented inclusive prefix sum over fp16, fp32 accumulation, fp16 output of length N.
//
// Same HBM layout, chunk (8 halves) and tile (64 chunks, lane l <-> chunk l) as the
// reduction.  A tile is scanned in three steps:
//   1. chunk totals          T[c], c = 0..63
//   2. exclusive scan of the totals over each segment's chunks (+ the carry that enters
//      the tile when a segment spans several tiles)              E[c]
//   3. inclusive scan inside every chunk, started at E[c]        out[c][i]
// Flavour MFMA = false does 1 and 3 with packed fp16 dot products in the owning lane and
// 2 with DPP row shifts / broadcasts (the counterpart of the reference's cub::WarpScan /
// cub::BlockScan rows, src/prefixsum/seg_cub_warp.cu:17-27, seg_cub_block.cu:13-51).
// Flavour MFMA = true is the scan as a product with constant triangular matrices, the formulation of reference
// src/prefixsum/kernel.cuh:48-83 (seg 16: A * U), :303-363 (seg 256: L * A * O + A * U) and :442-506 (256n: the
// carry enters through the accumulator), on v_mfma_f32_16x16x32_f16.  The tile is read as 16 runs of 32 consecutive
// halves: lane (n, b) = (lane % 16, lane / 16) holds chunk 4 n + b, which makes the tile the 32 x 16 B operand
// X[k][n] = x[32 n + k] (and, in the same registers, its transpose as a 16 x 32 A operand).
//   3. D1 = A1 * X + C, D2 = A2 * X + C with A1[m][k] = [k <= m], A2[m][k] = [k <= 16 + m] (for 16-half segments
//      A2[m][k] = [16 <= k <= 16 + m]): D1[m][n], D2[m][n] are the inclusive prefixes at positions m and 16 + m of
//      run n -- U^T * X, the transpose of the reference's A * U;
//   1./2. for segments of more than one run, the carries C: Q = X^T * J (J all ones) gives every run's total (the
//      reference's "* O"), T * R with R[n'][n] = [n' < n, same segment] the sum of the runs in front of run n inside
//      its segment (the reference's strictly triangular "L *"), with what entered the tile as that product's own
//      accumulator input.  T holds the totals as operands: fp32 totals split into two fp16 parts (hi + lo, 22 bits)
//      that sit in different k slots, so that the product is formed from exact 0/1 weights and loses nothing that the
//      fp16 result could show.  No DPP, no LDS; four lane swaps put the 16-byte pieces of the result back into the
//      lanes that loaded them.
#pragma once

#include "seg_reduce.hpp"

namespace tcu {

// Exclusive scan of `t` over groups of 2^LOG2 adjacent lanes (lane order), LOG2 = 1..6.
template <int LOG2>
TCU_DEVICE float lane_group_exclusive_scan(float t, int lane) {
  constexpr int LPS = 1 << LOG2;
  float e = dpp<DPP_WAVE_SHR1>(0.0f, t);
  if ((lane & (LPS - 1)) == 0) e = 0.0f;
  if constexpr (LOG2 >= 2) {
    float s = dpp<DPP_ROW_SHR0 + 1>(0.0f, e);
    if (LPS < 16 && (lane & (LPS - 1)) < 1) s = 0.0f;
    e += s;
  }
  if constexpr (LOG2 >= 2) {
    float s = dpp<DPP_ROW_SHR0 + 2>(0.0f, e);
    if (LPS < 16 && (lane & (LPS - 1)) < 2) s = 0.0f;
    e += s;
  }
  if constexpr (LOG2 >= 3) {
    float s = dpp<DPP_ROW_SHR0 + 4>(0.0f, e);
    if (LPS < 16 && (lane & (LPS - 1)) < 4) s = 0.0f;
    e += s;
  }
  if constexpr (LOG2 >= 4) e += dpp<DPP_ROW_SHR0 + 8>(0.0f, e);
  if constexpr (LOG2 >= 5) e += dpp<DPP_ROW_BCAST15, 0xA, 0xF, false>(0.0f, e);
  if constexpr (LOG2 >= 6) e += dpp<DPP_ROW_BCAST31, 0xC, 0xF, false>(0.0f, e);
  return e;
}

// Exclusive scan of t over groups of 2^LOG2 lanes inside each 16-lane row, LOG2 = 1..4.
template <int LOG2>
TCU_DEVICE float row_group_exclusive_scan(float t, int n) {
  constexpr int LPS = 1 << LOG2;
  float e = dpp<DPP_ROW_SHR0 + 1>(0.0f, t);
  if ((n & (LPS - 1)) == 0) e = 0.0f;
  if constexpr (LOG2 >= 2) {
    float s = dpp<DPP_ROW_SHR0 + 1>(0.0f, e);
    if (LPS < 16 && (n & (LPS - 1)) < 1) s = 0.0f;
    e += s;
  }
  if constexpr (LOG2 >= 2) {
    float s = dpp<DPP_ROW_SHR0 + 2>(0.0f, e);
    if (LPS < 16 && (n & (LPS - 1)) < 2) s = 0.0f;
    e += s;
  }
  if constexpr (LOG2 >= 3) {
    float s = dpp<DPP_ROW_SHR0 + 4>(0.0f, e);
    if (LPS < 16 && (n & (LPS - 1)) < 4) s = 0.0f;
    e += s;
  }
  if constexpr (LOG2 >= 4) e += dpp<DPP_ROW_SHR0 + 8>(0.0f, e);
  return e;
}

// 8 inclusive prefixes of one chunk started at `e`, rounded to fp16 and packed.  The even
// positions are a plain addition, not a dot product with the weights (1, 0): 0 * inf and
// 0 * NaN would otherwise carry a non-finite value of position 2i + 1 back to position 2i.
TCU_DEVICE uint4_t chunk_scan_packed(half8_t v, float e) {
  const half2_t ones = {(half_t)1.0f, (half_t)1.0f};
  const half2_t h01 = __builtin_shufflevector(v, v, 0, 1), h23 = __builtin_shufflevector(v, v, 2, 3);
  const half2_t h45 = __builtin_shufflevector(v, v, 4, 5), h67 = __builtin_shufflevector(v, v, 6, 7);
  const float x0 = e + (float)v[0], x1 = fdot2(h01, ones, e);
  const float x2 = x1 + (float)v[2], x3 = fdot2(h23, ones, x1);
  const float x4 = x3 + (float)v[4], x5 = fdot2(h45, ones, x3);
  const float x6 = x5 + (float)v[6], x7 = fdot2(h67, ones, x5);
  uint4_t r = {pack_f16x2(x0, x1), pack_f16x2(x2, x3), pack_f16x2(x4, x5), pack_f16x2(x6, x7)};
  return r;
}

// The chunk of its tile that a lane holds in the matrix flavour (see the header comment); the DPP flavour and the
// reductions use chunk == lane.
TCU_DEVICE int matrix_chunk_of_lane(int lane) { return 4 * (lane & 15) + (lane >> 4); }

// Constant operands of the matrix flavour (see the header comment), built from the lane id.
struct ScanOperands {
  half8_t tri_lo;  // A1
  half8_t tri_hi;  // A2
  half8_t ones;    // J
  half8_t strict;  // R, rows in the order of the k slots of T: blocks 0 / 1 = hi / lo parts of totals 0..7, blocks 2 / 3 of totals 8..15
};
template <int LPS_LOG2>
TCU_DEVICE ScanOperands make_scan_operands(int lane) {
  const int m = lane & 15, b = lane >> 4;
  constexpr int RPS = LPS_LOG2 >= 3 ? (1 << (LPS_LOG2 - 2)) : 1;  // runs of 32 halves per segment (inside a tile)
  ScanOperands o;
  half8_t lo, hi, st;
#pragma unroll
  for (int e = 0; e < 8; e++) {
    const int k = 8 * b + e;
    lo[e] = (half_t)(k <= m ? 1.0f : 0.0f);
    hi[e] = (half_t)((k <= 16 + m && (LPS_LOG2 > 1 || k >= 16)) ? 1.0f : 0.0f);
    const int run = 8 * (b >> 1) + e;  // the run whose total sits in slot k of T; as a B operand this lane is column m
    st[e] = (half_t)((run < m && run / RPS == m / RPS) ? 1.0f : 0.0f);
  }
  o.tri_lo = lo;
  o.tri_hi = hi;
  o.ones = splat8(1.0f);
  o.strict = st;
  return o;
}

// One tile.  `carry` (wave-uniform) is what precedes the tile inside its segment; on
// return *tile_total is the sum of the whole tile (only meaningful for LPS_LOG2 == 6).
// Writes the scanned tile to out[chunk_base ..] (chunks >= n_chunks are skipped) and, when
// totals != nullptr and the tile holds whole segments (LPS_LOG2 < 6), their totals.
template <int LPS_LOG2, bool MFMA, bool NT>
TCU_DEVICE void scan_tile(half8_t v, float carry, const ScanOperands &ops, int lane, uint4_t *out, size_t chunk_base, size_t n_chunks, uint16_t *totals, size_t tile_seg0,
                          size_t num_segments, float *tile_total) {
  constexpr int LPS = 1 << LPS_LOG2;
  if constexpr (!MFMA) {
    const float t = sum8(v, 0.0f);
    const float e0 = lane_group_exclusive_scan<LPS_LOG2>(t, lane);
    const float e = e0 + carry;
    const uint4_t r = chunk_scan_packed(v, e);
    const size_t c = chunk_base + lane;
    if (c < n_chunks) store_chunk<NT>(out + c, r);
    const float incl = e + t;
    if constexpr (LPS_LOG2 == 6) {
      *tile_total = readlane(e0 + t, 63);
    } else {
      *tile_total = 0.0f;
      if (totals != nullptr && (lane & (LPS - 1)) == LPS - 1) {
        const size_t s = tile_seg0 + (size_t)(lane >> LPS_LOG2);
        if (s < num_segments) totals[s] = f16_bits(incl);
      }
    }
  } else {
    // lane (n, g): v = chunk 4 n + g of the tile (matrix_chunk_of_lane)
    const int n = lane & 15, g = lane >> 4;
    float4_t c = {0, 0, 0, 0};
    if constexpr (LPS_LOG2 >= 3) {
      // totals of the 16 runs: lane (*, g) gets those of runs 4 g .. 4 g + 3
      const float4_t q = mfma_16x16x32(v, ops.ones, c);
      // the same as an A operand: rows g = 0, 1 take the totals of runs 0..7, rows 2, 3 those of runs 8..15
      unsigned ta[4], tb[4];
#pragma unroll
      for (int i = 0; i < 4; i++) {
        ta[i] = tb[i] = __float_as_uint(q[i]);
        permlane16_swap(ta[i], tb[i]);  // ta = total of run 8 (g / 2) + i, tb = of run 8 (g / 2) + 4 + i
      }
      half8_t t;
#pragma unroll
      for (int i = 0; i < 8; i++) {
        const float x = __uint_as_float(i < 4 ? ta[i] : tb[i - 4]);
        const half_t hi = (half_t)x;
        const half_t lo = (half_t)(x - (float)hi);
        t[i] = (g & 1) ? lo : hi;
      }
      const float in = LPS_LOG2 == 6 ? carry : 0.0f;
      c = mfma_16x16x32(t, ops.strict, float4_t{in, in, in, in});  // every row: what precedes run n inside its segment
    }
    const float4_t d1 = mfma_16x16x32(ops.tri_lo, v, c);
    const float4_t d2 = mfma_16x16x32(ops.tri_hi, v, c);
    if constexpr (LPS_LOG2 == 6) {
      *tile_total = readlane(d2[3], 63) - carry;  // the last prefix of the tile is what enters the next one
    } else {
      *tile_total = 0.0f;
      if (totals != nullptr && g == 3) {  // lane (n, 3) holds the last prefix of both halves of run n
        if constexpr (LPS_LOG2 == 1) {
          const size_t s = tile_seg0 + 2 * (size_t)n;
          if (s < num_segments) totals[s] = f16_bits(d1[3]);
          if (s + 1 < num_segments) totals[s + 1] = f16_bits(d2[3]);
        } else {
          constexpr int RPS = LPS_LOG2 >= 3 ? (1 << (LPS_LOG2 - 2)) : 1;
          const size_t s = tile_seg0 + (size_t)(n / RPS);
          if ((n % RPS) == RPS - 1 && s < num_segments) totals[s] = f16_bits(d2[3]);
        }
      }
    }
    // lane (n, g) holds positions 4 g .. 4 g + 3 (d1) and 16 + 4 g .. (d2) of run n; it stores positions 8 g .. 8 g + 7
    unsigned a_lo = pack_f16x2(d1[0], d1[1]), a_hi = pack_f16x2(d1[2], d1[3]);
    unsigned b_lo = pack_f16x2(d2[0], d2[1]), b_hi = pack_f16x2(d2[2], d2[3]);
    permlane32_swap(a_lo, b_lo);
    permlane32_swap(a_hi, b_hi);
    permlane16_swap(a_lo, b_lo);
    permlane16_swap(a_hi, b_hi);
    const size_t cidx = chunk_base + (size_t)matrix_chunk_of_lane(lane);
    const uint4_t r = {a_lo, a_hi, b_lo, b_hi};
    if (cidx < n_chunks) store_chunk<NT>(out + cidx, r);
  }
}

// ---------------------------------------------------------------------------------------
// Wave-owned spans.  LPS_LOG2 = 1..5: S = 16..256, segments inside a tile.  LPS_LOG2 = 6:
// S = 512 << tiles_per_seg_log2, a wave walks its segment(s) carrying the running sum.
// Each wave owns iters*U consecutive tiles.
// ---------------------------------------------------------------------------------------
template <int LPS_LOG2, int U, bool MFMA, int NT>
__global__ __launch_bounds__(kMaxBlock) void seg_scan_wave_kernel(const half8_t *in, uint4_t *out, uint16_t *totals, size_t n_chunks, size_t num_segments, int tiles_per_seg_log2, unsigned iters,
                                                                   unsigned xcd_run) {
  const int lane = lane_id();
  const size_t gw = xcd_run_piece(blockIdx.x, gridDim.x, xcd_run) * (blockDim.x >> 6) + wave_in_block();
  const size_t tile0 = gw * (size_t)iters * U;
  if (tile0 * kTileChunks >= n_chunks) return;
  const size_t tmask = ((size_t)1 << tiles_per_seg_log2) - 1;
  ScanOperands ops;
  if constexpr (MFMA) ops = make_scan_operands<LPS_LOG2>(lane);
  const int chunk_lane = MFMA ? matrix_chunk_of_lane(lane) : lane;  // the chunk of a tile this lane loads
  constexpr int SEGS_PER_TILE = 64 >> LPS_LOG2;

  float carry = 0.0f;
  for (unsigned it = 0; it < iters; it++) {
    const size_t t_it = tile0 + (size_t)it * U;
    half8_t v[U];
    load_tiles<U, NT != 0>(v, in, t_it * kTileChunks, n_chunks, chunk_lane);
    static_for<U>([&](auto J) {
      constexpr int j = decltype(J)::value;
      const size_t t = t_it + j;
      if (LPS_LOG2 < 6 || (t & tmask) == 0) carry = 0.0f;
      float tile_total;
      scan_tile<LPS_LOG2, MFMA, kTileStoreNT<NT, j>>(v[j], carry, ops, lane, out, t * kTileChunks, n_chunks, totals, t * SEGS_PER_TILE, num_segments, &tile_total);
      if constexpr (LPS_LOG2 == 6) {
        carry += tile_total;
        if (totals != nullptr && ((t + 1) & tmask) == 0) {
          const size_t s = t >> tiles_per_seg_log2;
          if (lane == 0 && s < num_segments) totals[s] = f16_bits(carry);
        }
      }
    });
  }
}

// ---------------------------------------------------------------------------------------
// S >= 512: the waves of a block share segments.  A block owns segs_per_block consecutive
// segments; groups of waves_per_seg waves take one segment each, blockDim / 64 /
// waves_per_seg segments at a time (see seg_reduce_block_kernel).  Per step a group takes
// waves_per_seg * U tiles, its wave w the U consecutive tiles starting at w * U; wave totals
// meet in LDS.
// ---------------------------------------------------------------------------------------
template <int U, bool MFMA, int NT>
__global__ __launch_bounds__(kMaxBlock) void seg_scan_block_kernel(const half8_t *in, uint4_t *out, uint16_t *totals, size_t n_chunks, size_t num_segments, size_t tiles_per_seg,
                                                                    unsigned segs_per_block, unsigned waves_per_seg, unsigned xcd_run) {
  __shared__ float wave_total[2][kMaxWaves];
  const int lane = lane_id();
  const int wave = wave_in_block();
  const int WPB = (int)(blockDim.x >> 6);
  const int G = (int)waves_per_seg, Q = WPB / G;  // waves per segment, segments in flight
  const int q = wave / G, wg = wave % G;           // this wave's group, and its place in the group
  ScanOperands ops;
  if constexpr (MFMA) ops = make_scan_operands<6>(lane);
  const int chunk_lane = MFMA ? matrix_chunk_of_lane(lane) : lane;
  unsigned parity = 0;
  const size_t piece = xcd_run_piece(blockIdx.x, gridDim.x, xcd_run);
  for (unsigned sb = 0; sb < segs_per_block; sb += (unsigned)Q) {
    if (piece * segs_per_block + sb >= num_segments) break;  // block-uniform
    const size_t seg = piece * segs_per_block + sb + (unsigned)q;
    const bool live = sb + (unsigned)q < segs_per_block && seg < num_segments;  // uniform over the group
    const size_t tile_base = seg * tiles_per_seg;
    size_t lim = (tile_base + tiles_per_seg) * kTileChunks;
    if (lim > n_chunks) lim = n_chunks;
    if (!live) lim = 0;  // a group without a segment loads and stores nothing
    float block_carry = 0.0f;
    for (size_t step0 = 0; step0 < tiles_per_seg; step0 += (size_t)G * U) {
      const size_t t0 = step0 + (size_t)wg * U;  // first tile of this wave (may lie past the segment)
      half8_t v[U];
      load_tiles<U, NT != 0>(v, in, (tile_base + t0) * kTileChunks, t0 < tiles_per_seg ? lim : 0, chunk_lane);
      // pass 1: this wave's total
      float acc = 0.0f;
#pragma unroll
      for (int j = 0; j < U; j++) acc = sum8(v[j], acc);
      acc = lane_group_sum<6>(acc);
      float carry = block_carry, all = 0.0f;
      if (G == 1) {  // block-uniform: every wave has a segment of its own, nothing to exchange
        all = readlane(acc, 63);
      } else {
        if (lane == 63) wave_total[parity][wave] = acc;
        __syncthreads();
        for (int w = 0; w < G; w++) {
          const float x = wave_total[parity][q * G + w];
          if (w < wg) carry += x;
          all += x;
        }
        parity ^= 1u;
      }
      block_carry += all;
      // pass 2: scan the tiles held in registers
      static_for<U>([&](auto J) {
        constexpr int j = decltype(J)::value;
        float tile_total;
        scan_tile<6, MFMA, kTileStoreNT<NT, j>>(v[j], carry, ops, lane, out, (tile_base + t0 + j) * kTileChunks, t0 + j < tiles_per_seg ? lim : 0, nullptr, 0, 0, &tile_total);
        carry += tile_total;
      });
    }
    if (totals != nullptr && wg == 0 && lane == 0 && live) totals[seg] = f16_bits(block_carry);
  }
}

// ---------------------------------------------------------------------------------------
// any S >= 1: one wave per segment, 64 elements per step
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(kMaxBlock) void seg_scan_generic_kernel(const uint16_t *in, uint16_t *out, uint16_t *totals, size_t num_segments, size_t segment_size) {
  const int lane = lane_id();
  const size_t seg = (size_t)blockIdx.x * (blockDim.x >> 6) + wave_in_block();
  if (seg >= num_segments) return;
  const uint16_t *p = in + seg * segment_size;
  uint16_t *q = out + seg * segment_size;
  float carry = 0.0f;
  for (size_t base = 0; base < segment_size; base += 64) {
    const size_t i = base + lane;
    const float x = i < segment_size ? (float)__builtin_bit_cast(half_t, p[i]) : 0.0f;
    const float incl = lane_group_exclusive_scan<6>(x, lane) + x + carry;
    if (i < segment_size) q[i] = f16_bits(incl);
    carry = readlane(incl, 63);
  }
  if (totals != nullptr && lane == 0) totals[seg] = f16_bits(carry);
}

// out[s*S + i] += partial_sums[s], one fp16 addition per element (8 per lane per step).  With `shifted` the array
// holds inclusive sums and segment s takes partial_sums[s - 1] (segment 0 nothing): the exclusive sums without a
// pass that shifts them.
template <bool NT>
__global__ __launch_bounds__(256) void add_partial_sums_kernel(uint4_t *out, const uint16_t *partial_sums, size_t n_chunks, int seg_log2_chunks, int shifted) {
  const size_t c = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= n_chunks) return;
  const size_t seg = c >> seg_log2_chunks;
  if (shifted && seg == 0) return;
  const float ps = (float)__builtin_bit_cast(half_t, partial_sums[shifted ? seg - 1 : seg]);
  half8_t v = load_chunk<NT>(reinterpret_cast<const half8_t *>(out + c));
  uint4_t r = {pack_f16x2((float)v[0] + ps, (float)v[1] + ps), pack_f16x2((float)v[2] + ps, (float)v[3] + ps), pack_f16x2((float)v[4] + ps, (float)v[5] + ps),
               pack_f16x2((float)v[6] + ps, (float)v[7] + ps)};
  store_chunk<NT>(out + c, r);
}
__global__ __launch_bounds__(256) void add_partial_sums_generic_kernel(uint16_t *out, const uint16_t *partial_sums, size_t n, size_t segment_size, int shifted) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const size_t seg = i / segment_size;
  if (shifted && seg == 0) return;
  const float ps = (float)__builtin_bit_cast(half_t, partial_sums[shifted ? seg - 1 : seg]);
  out[i] = f16_bits((float)__builtin_bit_cast(half_t, out[i]) + ps);
}

// ---------------------------------------------------------------------------------------
// Segments given by offsets (segment j = [begin[j], end[j]) in halves, any start, any
// length, empty when end <= begin; segments must not overlap): inclusive prefix sums inside
// every segment, elements outside every segment are not written.  The counterpart of the
// reference's key-based library scan (thrust::inclusive_scan_by_key,
// src/prefixsum/seg_thrust.cu:46-47) for segments described the way its
// cub::DeviceSegmentedReduce baseline describes them (src/reduction/seg_cub_device.cu:18-22).
// G = 2^G_LOG2 (2..16) adjacent lanes share a segment and walk it in rounds of G aligned
// 8-half chunks: a chunk that lies wholly inside the segment is one 128-bit load and one
// 128-bit store, the ragged first / last chunk goes through 2-byte accesses; chunk totals
// are scanned across the G lanes with DPP and the round total is carried to the next round.
// With `vector` false (input or output not 16-byte aligned) every chunk takes the 2-byte path.
// ---------------------------------------------------------------------------------------
template <typename OFF, int G_LOG2, bool NT>
__global__ __launch_bounds__(256) void seg_scan_offsets_kernel(const uint16_t *in, uint16_t *out, size_t num_segments, const OFF *__restrict__ begin, const OFF *__restrict__ end, int vector) {
  constexpr int G = 1 << G_LOG2;
  static_assert(G_LOG2 >= 1 && G_LOG2 <= 4, "the round total must reach every lane of the group");
  const int lane = lane_id();
  const int sub = lane & (G - 1);
  const size_t seg = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) >> G_LOG2;
  size_t b = 0, e = 0;
  if (seg < num_segments) {
    const OFF ob = begin[seg], oe = end[seg];
    if (oe > ob) {
      b = (size_t)ob;
      e = (size_t)oe;
    }
  }
  const size_t c_first = b / 8, c_end = (e + 7) / 8;  // aligned chunks touched by the segment
  const size_t rounds = (c_end - c_first + G - 1) / G;
  float carry = 0.0f;
  const half8_t *in8 = reinterpret_cast<const half8_t *>(in);
  uint4_t *out8 = reinterpret_cast<uint4_t *>(out);
  // every lane of the wave runs as many rounds as the longest segment of the wave needs (the
  // DPP scans involve all lanes)
  for (size_t r = 0; ballot(r < rounds) != 0ull; r++) {
    const size_t c = c_first + r * G + sub;
    const size_t lo = c * 8, hi = lo + 8;
    const bool any = r < rounds && c < c_end;
    const bool full = any && vector && lo >= b && hi <= e;
    half8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
    if (full) {
      v = load_chunk<NT>(in8 + c);
    } else if (any) {
#pragma unroll
      for (int i = 0; i < 8; i++)
        if (lo + i >= b && lo + i < e) v[i] = __builtin_bit_cast(half_t, in[lo + i]);
    }
    const float t = sum8(v, 0.0f);
    const float start = lane_group_exclusive_scan<G_LOG2>(t, lane) + carry;
    carry += lane_group_sum<G_LOG2>(t);
    const uint4_t packed = chunk_scan_packed(v, start);
    if (full) {
      store_chunk<NT>(out8 + c, packed);
    } else if (any) {
#pragma unroll
      for (int i = 0; i < 8; i++)
        if (lo + i >= b && lo + i < e) out[lo + i] = (uint16_t)(packed[i / 2] >> (16 * (i & 1)));
    }
  }
}

// ---------------------------------------------------------------------------------------
// Long segments given by offsets: `slices` blocks share a segment.  The aligned 128-bit
// chunks a segment touches are split into `slices` equal runs; pass 1 writes the fp32 sum of
// every run, pass 2 turns the sums of a segment into exclusive prefixes (in place), pass 3
// scans every run with its prefix as the carry-in.  Six bytes of traffic per element where
// the short-segment kernel moves four, but every segment is spread over the whole chip.
// ---------------------------------------------------------------------------------------
struct OffsetsSlice {
  size_t b, e;        // the segment, in halves (b == e when empty)
  size_t c_lo, c_hi;  // the slice's aligned chunks
};
template <typename OFF>
TCU_DEVICE OffsetsSlice offsets_slice(const OFF *__restrict__ begin, const OFF *__restrict__ end, size_t seg, size_t p, unsigned slices) {
  OffsetsSlice s{0, 0, 0, 0};
  const OFF ob = begin[seg], oe = end[seg];
  if (oe > ob) {
    s.b = (size_t)ob;
    s.e = (size_t)oe;
    const size_t c_first = s.b / 8, c_end = (s.e + 7) / 8;
    const size_t per = (c_end - c_first + slices - 1) / slices;
    s.c_lo = c_first + p * per;
    s.c_hi = s.c_lo + per;
    if (s.c_lo > c_end) s.c_lo = c_end;
    if (s.c_hi > c_end) s.c_hi = c_end;
  }
  return s;
}
// the chunk's halves that lie inside [b, e), others zero
template <bool NT>
TCU_DEVICE half8_t offsets_masked_chunk(const uint16_t *in, size_t c, size_t b, size_t e, int vector, bool *full) {
  const size_t lo = c * 8;
  *full = vector && lo >= b && lo + 8 <= e;
  if (*full) return load_chunk<NT>(reinterpret_cast<const half8_t *>(in) + c);
  half8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
  for (int i = 0; i < 8; i++)
    if (lo + i >= b && lo + i < e) v[i] = __builtin_bit_cast(half_t, in[lo + i]);
  return v;
}

template <typename OFF, bool NT>
__global__ __launch_bounds__(kMaxBlock) void seg_scan_offsets_slice_sums_kernel(const uint16_t *__restrict__ in, float *__restrict__ sums, const OFF *__restrict__ begin, const OFF *__restrict__ end,
                                                                                unsigned slices, int vector) {
  __shared__ float wave_total[kMaxWaves];
  const int lane = lane_id(), wave = wave_in_block();
  const OffsetsSlice s = offsets_slice(begin, end, blockIdx.x / slices, blockIdx.x % slices, slices);
  float acc = 0.0f;
  for (size_t c = s.c_lo + threadIdx.x; c < s.c_hi; c += blockDim.x) {
    bool full;
    acc = sum8(offsets_masked_chunk<NT>(in, c, s.b, s.e, vector, &full), acc);
  }
  acc = lane_group_sum<6>(acc);
  if (lane == 63) wave_total[wave] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    float t = 0.0f;
    for (unsigned w = 0; w < (blockDim.x >> 6); w++) t += wave_total[w];
    sums[blockIdx.x] = t;
  }
}

// sums[j * slices + p] -> sum of slices 0 .. p-1 of segment j; one wave per segment
__global__ __launch_bounds__(64) void slice_prefix_kernel(float *sums, unsigned slices) {
  const int lane = lane_id();
  float *row = sums + (size_t)blockIdx.x * slices;
  float carry = 0.0f;
  for (unsigned base = 0; base < slices; base += 64) {
    const unsigned i = base + lane;
    const float x = i < slices ? row[i] : 0.0f;
    const float excl = lane_group_exclusive_scan<6>(x, lane) + carry;
    if (i < slices) row[i] = excl;
    carry = readlane(excl + x, 63);
  }
}

template <typename OFF, bool NT>
__global__ __launch_bounds__(kMaxBlock) void seg_scan_offsets_sliced_kernel(const uint16_t *in, uint16_t *out, const float *__restrict__ prefixes, const OFF *__restrict__ begin,
                                                                            const OFF *__restrict__ end, unsigned slices, int vector) {
  __shared__ float wave_total[2][kMaxWaves];
  const int lane = lane_id(), wave = wave_in_block();
  const int WPB = (int)(blockDim.x >> 6);
  const OffsetsSlice s = offsets_slice(begin, end, blockIdx.x / slices, blockIdx.x % slices, slices);
  float carry = prefixes ? prefixes[blockIdx.x] : 0.0f;  // no prefixes: one slice per segment
  unsigned parity = 0;
  // every thread of the block runs the same number of rounds (barriers inside)
  for (size_t c0 = s.c_lo; c0 < s.c_hi; c0 += blockDim.x) {
    const size_t c = c0 + threadIdx.x;
    const bool any = c < s.c_hi;
    bool full = false;
    half8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
    if (any) v = offsets_masked_chunk<NT>(in, c, s.b, s.e, vector, &full);
    const float t = sum8(v, 0.0f);
    const float excl = lane_group_exclusive_scan<6>(t, lane);
    const float wt = lane_group_sum<6>(t);
    if (lane == 63) wave_total[parity][wave] = wt;
    __syncthreads();
    float before = 0.0f, all = 0.0f;
    for (int w = 0; w < WPB; w++) {
      const float x = wave_total[parity][w];
      if (w < wave) before += x;
      all += x;
    }
    parity ^= 1u;
    const uint4_t packed = chunk_scan_packed(v, carry + before + excl);
    carry += all;
    if (full) {
      store_chunk<NT>(reinterpret_cast<uint4_t *>(out) + c, packed);
    } else if (any) {
      const size_t lo = c * 8;
#pragma unroll
      for (int i = 0; i < 8; i++)
        if (lo + i >= s.b && lo + i < s.e) out[lo + i] = (uint16_t)(packed[i / 2] >> (16 * (i & 1)));
    }
  }
}

}  // namespace tcu
