// Segmented sum reduction over fp16, fp32 accumulation, one fp16 result per segment.
//
// Data layout in HBM: `in` is N = num_segments * S contiguous halves, segment j at
// [j*S, (j+1)*S); `out` is num_segments halves.  The unit of access is a CHUNK
// (8 halves = one 128-bit load) and a TILE (64 chunks = 1 KiB = one load per lane of a
// wave, lane l taking chunk l so that a wave reads 1 KiB contiguously).
//
// Kernels (S is a power of two >= 16 in all of them):
//   seg_reduce_small_kernel : S = 16..512, a segment is 2..64 adjacent lanes of one tile.
//   seg_reduce_long_kernel  : S >= 1024, a segment is S/512 whole tiles; one wave walks
//                             its segments with U tiles in flight.
//   seg_reduce_block_kernel : S >= 512, a block of waves shares each segment; partials
//                             are combined through LDS.
// Each comes in two flavours selected by MFMA:
//   false: per-lane sums with packed fp16 dot products, then DPP butterflies
//          (the counterpart of the reference's cub::WarpReduce / cub::BlockReduce rows,
//          reference src/reduction/seg_cub_warp.cu:17-32, seg_cub_block.cu:13-29);
//   true : the tile is the A operand of v_mfma_f32_16x16x32_f16 against a constant 0/1
//          matrix (reduction == multiplication by ones), the formulation of reference
//          src/reduction/kernel.cuh:33-77 (seg 16), :81-125 (16n), :241-298 (256),
//          :302-356 (256n), :176-236 and :419-559 (block variants).
#pragma once

#include "wave_ops.hpp"

namespace tcu {

constexpr int kTileChunks = 64;   // chunks per tile
constexpr int kTileHalves = 512;  // halves per tile
constexpr int kMaxWaves = 16;     // waves per block, upper bound
constexpr int kMaxBlock = kMaxWaves * 64;

// U tiles of one wave, tile j of the wave starting at chunk0 + 64*j.  Chunks at or
// beyond n_chunks read as zero.
template <int U, bool NT>
TCU_DEVICE void load_tiles(half8_t (&v)[U], const half8_t *__restrict__ in, size_t chunk0, size_t n_chunks, int lane) {
  if (chunk0 + (size_t)U * kTileChunks <= n_chunks) {
#pragma unroll
    for (int j = 0; j < U; j++) v[j] = load_chunk<NT>(in + chunk0 + (size_t)j * kTileChunks + lane);
  } else {
#pragma unroll
    for (int j = 0; j < U; j++) {
      size_t c = chunk0 + (size_t)j * kTileChunks + lane;
      half8_t z = {0, 0, 0, 0, 0, 0, 0, 0};
      v[j] = c < n_chunks ? load_chunk<NT>(in + c) : z;
    }
  }
}

// Which piece of work the block with index b of a grid of `grid` blocks takes.  Consecutive
// blocks of a launch are dealt round-robin to the 8 XCDs (block b runs on XCD b % 8).  With
// run = 0 block b takes piece b, so neighbouring pieces of the array are worked on by different
// XCDs.  With run = C > 0 the blocks are renumbered inside groups of 8 * C so that every XCD
// takes C consecutive pieces (XCD x of a group: pieces x * C .. x * C + C - 1) while the
// launch as a whole still sweeps the array front to back; a last, incomplete group keeps its
// own numbering.  What this changes is the order in which the memory channels see the
// requests of one XCD; the best C per segment size is measured (dispatch.hpp).
TCU_DEVICE size_t xcd_run_piece(size_t b, size_t grid, unsigned run) {
  if (run == 0) return b;
  const size_t group = (size_t)8 * run;
  const size_t first = b / group * group;
  if (first + group > grid) return b;
  return first + (b & 7) * run + ((b - first) >> 3);
}

// Sum over groups of 2^LOG2 adjacent lanes.  For LOG2 <= 4 every lane of a group ends
// up with the group's sum; for LOG2 = 5 only lanes 16..31 / 48..63 do, for LOG2 = 6
// only lanes 48..63.
template <int LOG2>
TCU_DEVICE float lane_group_sum(float p) {
  if constexpr (LOG2 >= 1) p += dpp<DPP_QUAD_XOR1>(p, p);
  if constexpr (LOG2 >= 2) p += dpp<DPP_QUAD_XOR2>(p, p);
  if constexpr (LOG2 >= 3) p += dpp<DPP_ROW_HALF_MIRROR>(p, p);
  if constexpr (LOG2 >= 4) p += dpp<DPP_ROW_MIRROR>(p, p);
  if constexpr (LOG2 >= 5) p += dpp<DPP_ROW_BCAST15, 0xA, 0xF, false>(0.0f, p);
  if constexpr (LOG2 >= 6) p += dpp<DPP_ROW_BCAST31, 0xC, 0xF, false>(0.0f, p);
  return p;
}

// Constant B operand that routes the 8-half sum of lane (r, b) of the A operand into
// column 4*slot + b of D: B[k][n] = 1 iff k/8 == n - 4*slot.
TCU_DEVICE half8_t column_select_operand(int lane, int slot) { return splat8((lane & 15) == 4 * slot + (lane >> 4) ? 1.0f : 0.0f); }

// ---------------------------------------------------------------------------------------
// S = 16 .. 512
// ---------------------------------------------------------------------------------------
template <int LPS_LOG2, int U, bool MFMA, bool NT>
__global__ __launch_bounds__(kMaxBlock) void seg_reduce_small_kernel(const half8_t *__restrict__ in, uint16_t *__restrict__ out, size_t n_chunks, size_t num_segments, unsigned xcd_run) {
  constexpr int LPS = 1 << LPS_LOG2;  // lanes (chunks) per segment
  constexpr int R = 64 / LPS;         // segments per tile
  constexpr int RW = R * U;           // segments per wave
  const int lane = lane_id();
  const int wave = wave_in_block();
  const size_t gw = xcd_run_piece(blockIdx.x, gridDim.x, xcd_run) * (blockDim.x >> 6) + wave;
  const size_t chunk0 = gw * (size_t)(U * kTileChunks);
  if (chunk0 >= n_chunks) return;  // wave-uniform
  const size_t seg0 = gw * (size_t)RW;

  half8_t v[U];
  load_tiles<U, NT>(v, in, chunk0, n_chunks, lane);

  if constexpr (!MFMA) {
    __shared__ __attribute__((aligned(16))) uint16_t stage[kMaxWaves][RW < 8 ? 8 : RW];
    const bool holder = LPS <= 16 ? (lane & (LPS - 1)) == 0 : (lane & (LPS - 1)) == LPS - 1;
    const int q = lane >> LPS_LOG2;
#pragma unroll
    for (int j = 0; j < U; j++) {
      float p = lane_group_sum<LPS_LOG2>(sum8(v[j], 0.0f));
      if (holder) stage[wave][j * R + q] = f16_bits(p);
    }
    wave_lds_fence();
    if constexpr (RW >= 8) {
      if (lane < RW / 8) {
        const size_t s = seg0 + (size_t)lane * 8;
        if (s + 8 <= num_segments) {
          // 16 halves per segment write a sixteenth of what they read; non-temporal stores of those sums measure 3.5 %
          // faster (N = 2^28: 91.3 -> 88.2 us with events), from 32 halves per segment on 1-5 % slower
          store_chunk<NT && LPS_LOG2 == 1>(reinterpret_cast<uint4_t *>(out + s), *reinterpret_cast<const uint4_t *>(&stage[wave][lane * 8]));
        } else {
          for (int i = 0; i < 8; i++)
            if (s + i < num_segments) out[s + i] = stage[wave][lane * 8 + i];
        }
      }
    } else {
      if (lane < RW && seg0 + lane < num_segments) out[seg0 + lane] = stage[wave][lane];
    }
  } else {
    // Lane (n, g) = (lane % 16, lane / 16) of accumulator `grp` receives the sums of
    // chunks 16*(n%4) + 4*g + i, i = 0..3, of tile 4*grp + n/4.
    constexpr int G = (U + 3) / 4;
    half8_t bsel[U < 4 ? U : 4];
#pragma unroll
    for (int s = 0; s < (U < 4 ? U : 4); s++) bsel[s] = column_select_operand(lane, s);
    float4_t acc[G];
#pragma unroll
    for (int grp = 0; grp < G; grp++) acc[grp] = float4_t{0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < U; j++) acc[j / 4] = mfma_16x16x32(v[j], bsel[j % 4], acc[j / 4]);

    const int n = lane & 15, g = lane >> 4, cb = n & 3;
#pragma unroll
    for (int grp = 0; grp < G; grp++) {
      const int t = 4 * grp + (n >> 2);  // tile of this lane's column
      const float4_t a = acc[grp];
      if constexpr (LPS_LOG2 == 1) {
        const size_t s = seg0 + (size_t)(32 * t + 8 * cb + 2 * g);
        const unsigned pk = pack_f16x2(a[0] + a[1], a[2] + a[3]);
        if (t < U) {
          if (s + 2 <= num_segments) {
            *reinterpret_cast<unsigned *>(out + s) = pk;
          } else if (s < num_segments) {
            out[s] = (uint16_t)(pk & 0xffffu);
          }
        }
      } else {
        float s4 = (a[0] + a[1]) + (a[2] + a[3]);  // 4 chunks = 32 halves
        if constexpr (LPS_LOG2 >= 3) s4 = add_xor16(s4);
        if constexpr (LPS_LOG2 >= 4) s4 = add_xor32(s4);
        if constexpr (LPS_LOG2 >= 5) s4 += dpp<DPP_QUAD_XOR1>(s4, s4);
        if constexpr (LPS_LOG2 >= 6) s4 += dpp<DPP_QUAD_XOR2>(s4, s4);
        // position of this lane's 32-half group inside the wave's U tiles, in groups
        const int grp32 = 16 * t + 4 * cb + g;
        constexpr int GPS = LPS / 4;  // 32-half groups per segment
        const bool holder = (LPS_LOG2 == 2) || (LPS_LOG2 == 3 && (g & 1) == 0) || (LPS_LOG2 == 4 && g == 0) || (LPS_LOG2 == 5 && g == 0 && (cb & 1) == 0) ||
                            (LPS_LOG2 == 6 && g == 0 && cb == 0);
        const size_t s = seg0 + (size_t)(grp32 / GPS);
        if (t < U && holder && s < num_segments) out[s] = f16_bits(s4);
      }
    }
  }
}

// ---------------------------------------------------------------------------------------
// S >= 1024: whole tiles per segment, one wave walks consecutive segments
// ---------------------------------------------------------------------------------------
// tiles_per_seg_log2 = log2(S/512) >= 1.  Each wave owns `iters` steps of U tiles,
// i.e. iters*U/tiles_per_seg whole segments (the host picks iters so that this is >= 1).
template <int U, bool MFMA, bool NT>
__global__ __launch_bounds__(kMaxBlock) void seg_reduce_long_kernel(const half8_t *__restrict__ in, uint16_t *__restrict__ out, size_t n_chunks, size_t num_segments, int tiles_per_seg_log2,
                                                                     unsigned iters, unsigned xcd_run) {
  const int lane = lane_id();
  const size_t gw = xcd_run_piece(blockIdx.x, gridDim.x, xcd_run) * (blockDim.x >> 6) + wave_in_block();
  const size_t tile0 = gw * (size_t)iters * U;
  if (tile0 * kTileChunks >= n_chunks) return;
  const size_t tmask = ((size_t)1 << tiles_per_seg_log2) - 1;
  const half8_t ones = splat8(1.0f);

  float accs = 0.0f;
  float4_t accm = {0, 0, 0, 0};
  for (unsigned it = 0; it < iters; it++) {
    const size_t t_it = tile0 + (size_t)it * U;
    half8_t v[U];
    load_tiles<U, NT>(v, in, t_it * kTileChunks, n_chunks, lane);
#pragma unroll
    for (int j = 0; j < U; j++) {
      if constexpr (MFMA)
        accm = mfma_16x16x32(v[j], ones, accm);  // D[r][*] += sum_k A[r][k]
      else
        accs = sum8(v[j], accs);
      const size_t t = t_it + j;
      if (((t + 1) & tmask) == 0) {  // wave-uniform: last tile of a segment
        float total;
        if constexpr (MFMA) {
          // every column of D holds the 16 row sums; fold rows, then the 4 row groups
          total = add_xor32(add_xor16((accm[0] + accm[1]) + (accm[2] + accm[3])));
          accm = float4_t{0, 0, 0, 0};
        } else {
          total = lane_group_sum<6>(accs);
          accs = 0.0f;
        }
        const size_t s = t >> tiles_per_seg_log2;
        if (lane == 63 && s < num_segments) out[s] = f16_bits(total);
      }
    }
  }
}

// ---------------------------------------------------------------------------------------
// S >= 512: the waves of a block share segments.  A block owns segs_per_block consecutive
// segments; groups of waves_per_seg waves (a power of two that divides the block) take one
// segment each, blockDim / 64 / waves_per_seg segments at a time, so a block with more
// waves than a segment has tiles still keeps every wave busy.
// ---------------------------------------------------------------------------------------
template <int U, bool MFMA, bool NT>
__global__ __launch_bounds__(kMaxBlock) void seg_reduce_block_kernel(const half8_t *__restrict__ in, uint16_t *__restrict__ out, size_t n_chunks, size_t num_segments, size_t tiles_per_seg,
                                                                      unsigned segs_per_block, unsigned waves_per_seg, unsigned xcd_run) {
  __shared__ float partial[kMaxWaves];
  const int lane = lane_id();
  const int wave = wave_in_block();
  const int WPB = (int)(blockDim.x >> 6);
  const int G = (int)waves_per_seg, Q = WPB / G;  // waves per segment, segments in flight
  const int q = wave / G, wg = wave % G;           // this wave's group, and its place in the group
  const half8_t ones = splat8(1.0f);
  const size_t piece = xcd_run_piece(blockIdx.x, gridDim.x, xcd_run);
  for (unsigned sb = 0; sb < segs_per_block; sb += (unsigned)Q) {
    if (piece * segs_per_block + sb >= num_segments) break;  // block-uniform
    const size_t seg = piece * segs_per_block + sb + (unsigned)q;
    const bool live = sb + (unsigned)q < segs_per_block && seg < num_segments;  // uniform over the group
    const size_t tile_base = seg * tiles_per_seg;
    float accs = 0.0f;
    float4_t accm = {0, 0, 0, 0};
    if (live) {
      for (size_t t0 = (size_t)wg * U; t0 < tiles_per_seg; t0 += (size_t)G * U) {
        half8_t v[U];
        // tiles past the end of the segment must not be read: clamp the chunk limit
        size_t lim = (tile_base + tiles_per_seg) * kTileChunks;
        if (lim > n_chunks) lim = n_chunks;
        load_tiles<U, NT>(v, in, (tile_base + t0) * kTileChunks, lim, lane);
#pragma unroll
        for (int j = 0; j < U; j++) {
          if constexpr (MFMA)
            accm = mfma_16x16x32(v[j], ones, accm);
          else
            accs = sum8(v[j], accs);
        }
      }
    }
    float total;
    if constexpr (MFMA)
      total = add_xor32(add_xor16((accm[0] + accm[1]) + (accm[2] + accm[3])));
    else
      total = lane_group_sum<6>(accs);
    if (G == 1) {  // block-uniform: every wave has a segment of its own, nothing to exchange
      if (lane == 63 && live) out[seg] = f16_bits(total);
      continue;
    }
    if (lane == 63) partial[wave] = total;
    __syncthreads();
    if (wg == 0 && lane == 0 && live) {
      float s = 0.0f;
      for (int w = 0; w < G; w++) s += partial[q * G + w];
      out[seg] = f16_bits(s);
    }
    __syncthreads();
  }
}

// ---------------------------------------------------------------------------------------
// any S >= 1 (not a power of two, or below 16): one wave per segment, scalar loads
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(kMaxBlock) void seg_reduce_generic_kernel(const uint16_t *__restrict__ in, uint16_t *__restrict__ out, size_t num_segments, size_t segment_size) {
  const int lane = lane_id();
  const size_t seg = (size_t)blockIdx.x * (blockDim.x >> 6) + wave_in_block();
  if (seg >= num_segments) return;
  const uint16_t *p = in + seg * segment_size;
  float acc = 0.0f;
  for (size_t i = lane; i < segment_size; i += 64) acc += (float)__builtin_bit_cast(half_t, p[i]);
  acc = lane_group_sum<6>(acc);
  if (lane == 63) out[seg] = f16_bits(acc);
}

// Segments given by offsets: segment j = in[begin[j], end[j]) in halves, empty when
// end[j] <= begin[j]; segments may start anywhere, overlap or leave gaps (the interface of
// cub::DeviceSegmentedReduce::Sum as the reference calls it, src/reduction/seg_cub_device.cu:46-48).
// G = 2^G_LOG2 adjacent lanes share a segment: the aligned 16-byte chunks it touches are dealt
// out round-robin (lane `sub` takes the chunks sub, sub + G, ... counted from the segment's
// first chunk, four in flight); whole chunks are one 128-bit load, the ragged first and last
// chunk go through 2-byte loads, and a DPP butterfly adds the G partial sums.  With `vector`
// false (input not 16-byte aligned) every chunk takes the 2-byte path.
// this lane's share of the sum over in[b, e): lane `sub` of `g` lanes that split the range
// The sum is taken in two steps so that a caller with several ranges can have the first load of
// each in flight before it consumes any: range_begin issues the lane's first whole chunk,
// range_finish adds it and walks the rest.
struct RangeCursor {
  size_t b, e, c, c_full_end, c_end;
  half8_t first;
  float head;
  bool has_first;
};
TCU_DEVICE float range_partial_chunk(const uint16_t *__restrict__ in, size_t c, size_t b, size_t e) {  // the halves of chunk c inside [b, e), one by one
  float s = 0.0f;
  const size_t lo = c * 8;
#pragma unroll
  for (int i = 0; i < 8; i++)
    if (lo + i >= b && lo + i < e) s += (float)__builtin_bit_cast(half_t, in[lo + i]);
  return s;
}
template <bool NT>
TCU_DEVICE RangeCursor range_begin(const uint16_t *__restrict__ in, size_t b, size_t e, size_t sub, size_t g, int vector) {
  RangeCursor r;
  r.b = b;
  r.e = e;
  r.head = 0.0f;
  r.has_first = false;
  r.first = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
  if (b >= e) {
    r.c = r.c_full_end = r.c_end = 0;
    return r;
  }
  // the aligned chunks the range touches are dealt out round-robin: lane `sub` takes chunks
  // c_first + sub, + g, ...; only the first and the last chunk can be partial
  const size_t c_first = b >> 3;
  r.c_end = (e + 7) >> 3;
  r.c_full_end = e >> 3;
  r.c = c_first + sub;
  if (!vector) return r;
  if (r.c == c_first && (b & 7) != 0 && r.c < r.c_end) {
    r.head = range_partial_chunk(in, r.c, b, e);
    r.c += g;
  }
  if (r.c < r.c_full_end) {
    r.first = load_chunk<NT>(reinterpret_cast<const half8_t *>(in) + r.c);
    r.has_first = true;
    r.c += g;
  }
  return r;
}
template <bool NT>
TCU_DEVICE float range_finish(const uint16_t *__restrict__ in, const RangeCursor &r, size_t g, int vector) {
  const half8_t *chunks = reinterpret_cast<const half8_t *>(in);
  float acc = r.head, acc1 = 0.0f;
  size_t c = r.c;
  if (!vector) {
    for (; c < r.c_end; c += g) acc += range_partial_chunk(in, c, r.b, r.e);
    return acc;
  }
  if (r.has_first) acc = sum8(r.first, acc);
  for (; c + 3 * g < r.c_full_end; c += 4 * g) {
    const half8_t v0 = load_chunk<NT>(chunks + c), v1 = load_chunk<NT>(chunks + c + g), v2 = load_chunk<NT>(chunks + c + 2 * g), v3 = load_chunk<NT>(chunks + c + 3 * g);
    acc = sum8(v0, acc);
    acc1 = sum8(v1, acc1);
    acc = sum8(v2, acc);
    acc1 = sum8(v3, acc1);
  }
  for (; c < r.c_full_end; c += g) acc = sum8(load_chunk<NT>(chunks + c), acc);
  if (c == r.c_full_end && c < r.c_end) acc1 += range_partial_chunk(in, c, r.b, r.e);  // the ragged last chunk
  return acc + acc1;
}
template <bool NT>
TCU_DEVICE float offsets_range_sum(const uint16_t *__restrict__ in, size_t b, size_t e, size_t sub, size_t g, int vector) {
  return range_finish<NT>(in, range_begin<NT>(in, b, e, sub, g, vector), g, vector);
}

// A block takes PASSES * SEGS consecutive segments, SEGS = 256 / G at a time, and has the first
// load of every pass in flight before it consumes one: with a single 16-byte chunk per lane in
// flight the wave slots of a compute unit do not hold enough bytes to cover the memory latency
// (one pass: 120 us at N = 2^28 for segments up to 512 halves, two: 107-111 us, four: 131 us).
template <typename OFF, int G_LOG2, bool NT, int PASSES>
__global__ __launch_bounds__(256) void seg_reduce_offsets_kernel(const uint16_t *__restrict__ in, uint16_t *__restrict__ out, size_t num_segments, const OFF *__restrict__ begin,
                                                                 const OFF *__restrict__ end, int vector) {
  constexpr int G = 1 << G_LOG2;
  constexpr int SEGS = 256 >> G_LOG2;  // segments per block and pass
  constexpr int passes = PASSES;
  __shared__ __attribute__((aligned(16))) uint16_t stage[SEGS * PASSES];
  const int lane = lane_id();
  const int sub = lane & (G - 1);
  const bool holder = G_LOG2 <= 4 ? sub == 0 : sub == G - 1;
  const size_t seg0 = (size_t)blockIdx.x * SEGS * passes;
  RangeCursor cur[PASSES];
#pragma unroll
  for (int p = 0; p < PASSES; p++) {  // every pass's first load goes out before any is consumed
    const size_t seg = seg0 + (size_t)p * SEGS + (threadIdx.x >> G_LOG2);
    size_t b = 0, e = 0;
    if (seg < num_segments) {
      const OFF ob = begin[seg], oe = end[seg];
      if (oe > ob) {
        b = (size_t)ob;
        e = (size_t)oe;
      }
    }
    cur[p] = range_begin<NT>(in, b, e, (size_t)sub, (size_t)G, vector);
  }
#pragma unroll
  for (int p = 0; p < PASSES; p++) {
    const float total = lane_group_sum<G_LOG2>(range_finish<NT>(in, cur[p], (size_t)G, vector));
    if (holder) stage[p * SEGS + (threadIdx.x >> G_LOG2)] = f16_bits(total);
  }
  __syncthreads();
  // the block's results are consecutive in `out`: they leave as 128-bit stores where they can
  const int n_out = SEGS * passes;
  for (int i0 = (int)threadIdx.x * 8; i0 < n_out; i0 += 256 * 8) {
    const size_t s = seg0 + (size_t)i0;
    if (i0 + 8 <= n_out && s + 8 <= num_segments && (reinterpret_cast<uintptr_t>(out + s) & 15u) == 0) {
      *reinterpret_cast<uint4_t *>(out + s) = *reinterpret_cast<const uint4_t *>(&stage[i0]);
    } else {
      for (int i = 0; i < 8; i++)
        if (i0 + i < n_out && s + i < num_segments) out[s + i] = stage[i0 + i];
    }
  }
}

// Long segments: `slices` blocks share a segment.  Block (segment j, slice p) adds the p-th of
// `slices` equal parts of the segment (part length rounded up to whole 128-bit chunks) and
// writes an fp32 partial to partial[j * slices + p]; a second kernel adds the partials.
template <typename OFF, bool NT, bool DIRECT = false>
__global__ __launch_bounds__(kMaxBlock) void seg_reduce_offsets_sliced_kernel(const uint16_t *__restrict__ in, float *__restrict__ partial_out, const OFF *__restrict__ begin,
                                                                              const OFF *__restrict__ end, unsigned slices, int vector) {
  __shared__ float partial[kMaxWaves];
  const int lane = lane_id(), wave = wave_in_block();
  const size_t seg = blockIdx.x / slices, p = blockIdx.x % slices;
  size_t b = 0, e = 0;
  {
    const OFF ob = begin[seg], oe = end[seg];
    if (oe > ob) {
      b = (size_t)ob;
      e = (size_t)oe;
    }
  }
  const size_t part = (((e - b) + slices - 1) / slices + 7) & ~(size_t)7;
  size_t sb = b + p * part, se = sb + part;
  if (sb > e) sb = e;
  if (se > e) se = e;
  const float total = lane_group_sum<6>(offsets_range_sum<NT>(in, sb, se, (size_t)threadIdx.x, (size_t)blockDim.x, vector));
  if (lane == 63) partial[wave] = total;
  __syncthreads();
  if (threadIdx.x == 0) {
    float s = 0.0f;
    for (unsigned w = 0; w < (blockDim.x >> 6); w++) s += partial[w];
    if constexpr (DIRECT)  // one block per segment: partial_out is the fp16 result array
      reinterpret_cast<uint16_t *>(partial_out)[blockIdx.x] = f16_bits(s);
    else
      partial_out[blockIdx.x] = s;
  }
}

}  // namespace tcu
