// Full-array (unsegmented) sum and inclusive prefix sum over fp16, fp32 carries.
//
// Single-pass kernels:
//   full_reduce_kernel : one partition per block; every block publishes {1, fp32 partial} as
//     one 64-bit word; the last block of every group of 64 adds the group's words, the last
//     block of the grid adds the group sums (index order, so the result does not depend on
//     timing) and writes the fp16 result.  Replaces the reference's
//     atomic / cooperative-groups full reductions (src/reduction/kernel.cuh:564-786), whose
//     combine step is an atomicAdd on one half (or a serial loop in global thread 0).
//   full_scan_kernel, full_scan_lds_kernel : decoupled look-back.  Partitions are handed out
//     by an atomic ticket (so a partition's predecessors are always running or done); each
//     block publishes {flag, fp32 aggregate} as one 64-bit word, wave 0 looks back 64
//     descriptors at a time, then the block scans its tiles from registers (and, in the
//     second kernel, from LDS).  Replaces the reference's grid-sync / spin-barrier full scans
//     (src/prefixsum/kernel.cuh:779-972; both disabled upstream: the first needs more shared
//     memory than exists, the second deadlocks) and its 3-kernel sequence, which moves 8+
//     bytes per element.
// Two-launch reduction (the fastest; also what segments of 2^20 halves and more take):
//   partition_sums_kernel writes one fp32 partial per partition, segment_of_partials_kernel
//   adds the partials of every segment.
// Multi-kernel helpers (the reference's "2 kernels" / "3 kernels" sequences):
//   sum_f16_kernel, exclusive_scan_f16_kernel over the per-segment totals.
#pragma once

#include "seg_scan.hpp"

namespace tcu {

constexpr unsigned long long kFlagAggregate = 1ull << 32;
constexpr unsigned long long kFlagPrefix = 2ull << 32;

// words[0..n) = 0
__global__ __launch_bounds__(256) void zero_words_kernel(unsigned *words, size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) words[i] = 0u;
}

// Clears a look-back workspace: the ticket word and the first four words (two 64-bit descriptors) of
// every partition's slot; the rest of a slot is never read.
__global__ __launch_bounds__(256) void zero_look_back_kernel(unsigned *ws, size_t parts, unsigned desc_shift) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i == 0) {
    ws[0] = 0u;
    ws[1] = 0u;  // waits that gave up (WaitPolicy::expired)
  }
  if (i < parts) {
    unsigned *slot = ws + 64 + 2 * (i << desc_shift);
    slot[0] = 0u;
    slot[1] = 0u;
    if (desc_shift) {
      slot[2] = 0u;
      slot[3] = 0u;
    }
  }
}

// One partition (blockDim/64 * U tiles) per block, no loop: blocks dispatched in order sweep
// the array as one moving window, which is what HBM serves fastest (a persistent
// grid-stride version of this kernel measured 2-3x slower).
// Completion is detected without fences (an agent-scope release/acquire pair per block costs
// about 90 ns of L2 write-back/invalidate and made this kernel 20x slower than the data
// movement), without a hot counter (same-address device-scope atomics retire at about one
// per 11 ns) and without any atomic that returns a value (a block that waits for its ticket
// holds its compute unit 1-2 us longer: 352 against 314 us for the plain partition sums at
// 2^30): every block publishes {1, partial} as ONE 64-bit word and is done, like a block of
// partition_sums_kernel.  The last block BY INDEX of every group of 64 blocks goes on: its
// first wave reads the group's 64 words (polling the few that are still in flight: its
// predecessors were dispatched before it) and publishes the group sum the same way; the last
// block of the grid then adds the group sums and writes the result.  A block that adds never
// waits for a block that adds on the same level, and the blocks that only publish never wait
// at all, so the kernel finishes in whatever order the blocks are dispatched; every wait is
// bounded all the same, and a value that never shows up makes the result NaN.  All sums run
// in index order, so the result does not depend on timing.
// workspace words: [0 .. 64 + groups) unused (64 + groups rounded up to an even number),
// then u64 partial[blocks], u64 group_sum[groups]; zeroed before the launch.
constexpr unsigned kFullReduceGroup = 64;
constexpr unsigned long long kPublished = 1ull << 32;

// What bounds the waits of the single-pass kernels.  poll_limit: how often a wave looks again
// for a value that has not been published yet before it gives up; giving up makes the results
// that depend on the missing value NaN, never a finite wrong number.  mute_partition (tests
// only, 0 = none): partition mute_partition - 1 computes its own results but publishes
// nothing, which makes every wait for it expire while all kernels still run to their end.
// desc_shift: the look-back descriptors of consecutive partitions lie 8 << desc_shift bytes apart.  Packed
// descriptors (shift 0) put 16 partitions into one 128-byte line that hundreds of waiting waves poll while
// its owners keep storing into it; one descriptor per 256 bytes (shift 5) took the full-array scan of 2^28
// halves from 212 to 191 us.
// expired: device word (may be null) that counts the waits that gave up, so that a caller can tell without
// looking for NaN in the output; the workspace-taking entry points pass word 1 of the workspace.
struct WaitPolicy {
  unsigned poll_limit;
  unsigned mute_partition;
  unsigned desc_shift;
  unsigned *expired;
};
// called by every lane of the wave whose wait expired
TCU_DEVICE void note_expired_wait(const WaitPolicy &wait, int lane) {
  if (lane == 0 && wait.expired != nullptr) atomic_add_u32(wait.expired, 1u);
}
constexpr unsigned kDefaultPollLimit = 1u << 20;
constexpr unsigned kDescShift = 5;


// sum over lanes of the published values at p[lane], lane < count (count <= 64); false if a
// value never showed up
TCU_DEVICE bool gather_published(const unsigned long long *p, unsigned count, int lane, float *sum, const WaitPolicy &wait) {
  unsigned long long d = (unsigned)lane < count ? 0ull : kPublished;
  for (unsigned polls = 0;; polls++) {
    if ((d >> 32) != 1ull) d = atomic_load_u64(p + lane);  // only what has not shown up yet is read again
    if (ballot((d >> 32) == 1ull) == ~0ull) break;
    if (polls >= wait.poll_limit) {
      note_expired_wait(wait, lane);
      return false;
    }
    spin_pause();
  }
  const float v = (unsigned)lane < count ? __uint_as_float((unsigned)d) : 0.0f;
  *sum = readlane(lane_group_sum<6>(v), 63);
  return true;
}

template <int U, bool MFMA, bool NT>
__global__ __launch_bounds__(kMaxBlock) void full_reduce_kernel(const half8_t *__restrict__ in, uint16_t *__restrict__ out, size_t n_chunks, unsigned *ws, WaitPolicy wait) {
  __shared__ float partial[kMaxWaves];
  const int lane = lane_id();
  const int wave = wave_in_block();
  const int WPB = (int)(blockDim.x >> 6);
  const unsigned n_blocks = gridDim.x;
  const unsigned n_groups = (n_blocks + kFullReduceGroup - 1) / kFullReduceGroup;
  unsigned long long *partials = reinterpret_cast<unsigned long long *>(ws + 64 + ((n_groups + 1) & ~1u));
  unsigned long long *group_sum = partials + n_blocks;
  const half8_t ones = splat8(1.0f);

  half8_t v[U];
  load_tiles<U, NT>(v, in, ((size_t)blockIdx.x * WPB + wave) * U * kTileChunks, n_chunks, lane);
  float total;
  if constexpr (MFMA) {
    float4_t accm = {0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < U; j++) accm = mfma_16x16x32(v[j], ones, accm);
    total = add_xor32(add_xor16((accm[0] + accm[1]) + (accm[2] + accm[3])));
  } else {
    float accs[2] = {0.0f, 0.0f};
#pragma unroll
    for (int j = 0; j < U; j++) accs[j & 1] = sum8(v[j], accs[j & 1]);
    total = lane_group_sum<6>(accs[0] + accs[1]);
  }
  if (lane == 63) partial[wave] = total;
  __syncthreads();
  if (wave != 0) return;
  float s = 0.0f;
  for (int w = 0; w < WPB; w++) s += partial[w];
  const unsigned b = blockIdx.x;
  if (lane == 0 && b + 1 != wait.mute_partition) atomic_store_u64(partials + b, kPublished | __float_as_uint(s));
  const unsigned g = b / kFullReduceGroup;
  const unsigned first = g * kFullReduceGroup;
  const unsigned members = n_blocks - first < kFullReduceGroup ? n_blocks - first : kFullReduceGroup;
  if (b != first + members - 1) return;  // wave-uniform: only a group's last block goes on
  const float failed = __builtin_nanf("");  // a published value never became visible
  float gs;
  if (!gather_published(partials + first, members, lane, &gs, wait)) gs = failed;
  if (lane == 0) atomic_store_u64(group_sum + g, kPublished | __float_as_uint(gs));
  if (g != n_groups - 1) return;  // wave-uniform: only the last block of the grid goes on
  float t = 0.0f;
  for (unsigned base = 0; base < n_groups; base += 64) {
    const unsigned count = n_groups - base < 64 ? n_groups - base : 64;
    float part;
    if (!gather_published(group_sum + base, count, lane, &part, wait)) part = failed;
    t += part;
  }
  if (lane == 0) out[0] = t != t ? (uint16_t)0x7e00u : f16_bits(t);
}

// Decoupled look-back of partition `part` over the descriptors desc[floor .. part): wave 0 reads
// 64 descriptors per round (lane l takes desc[base - l]), adds the aggregates down to the
// nearest published inclusive prefix and returns the sum in every lane.  A descriptor that stays
// empty for more than wait.poll_limit polls ends the look-back with NaN: the partition's own
// results and, through the prefix it then publishes, those of every later partition of the scan
// become NaN instead of a plausible wrong number.  Every lane of the wave takes the same path.
TCU_DEVICE float look_back(const unsigned long long *desc, long long part, long long floor, int lane, WaitPolicy wait) {
  float prefix = 0.0f;
  long long base = part - 1;
  unsigned polls = 0;
  unsigned long long d = 0;
  bool reload = true;  // per lane: a poll repeats only the reads that found nothing and still matter
  while (true) {
    const long long idx = base - lane;
    if (reload) d = idx >= floor ? atomic_load_u64(desc + ((size_t)idx << wait.desc_shift)) : kFlagPrefix;
    const unsigned flag = (unsigned)(d >> 32);
    const unsigned long long is_prefix = ballot(flag == 2u);
    const unsigned long long is_empty = ballot(flag == 0u);
    const int first_prefix = is_prefix ? __builtin_ctzll(is_prefix) : 64;
    const unsigned long long needed = first_prefix >= 63 ? ~0ull : ((2ull << first_prefix) - 1ull);
    if (is_empty & needed) {
      if (polls++ >= wait.poll_limit) {  // never spin without bound
        note_expired_wait(wait, lane);
        return __builtin_nanf("");
      }
      // an aggregate that was read stays valid when its descriptor turns into a prefix (the look-back then
      // merely walks on to older descriptors), so only the empty ones in front of the nearest prefix are read again
      reload = flag == 0u && ((needed >> lane) & 1ull) != 0;
      spin_pause();
      continue;
    }
    float val = lane <= first_prefix ? __uint_as_float((unsigned)d) : 0.0f;
    val = lane_group_sum<6>(val);
    prefix += readlane(val, 63);
    if (first_prefix < 64) return prefix;
    base -= 64;
    reload = true;
  }
}

// One partition (blockDim/64 * U tiles) per block.  workspace: ticket counter at word 0,
// descriptors (64-bit: flag << 32 | float bits) from byte 256, 8 << wait.desc_shift bytes apart.
// parts_per_segment = 0: one scan over the whole array.  Otherwise the array is a sequence of
// segments of parts_per_segment whole partitions each, scanned independently (segments far
// larger than what one block can walk), and `totals`, if given, receives every segment's sum.
template <int U, bool MFMA, bool NT>
__global__ __launch_bounds__(kMaxBlock, 8) void full_scan_kernel(const half8_t *in, uint4_t *out, size_t n_chunks, unsigned *ws, int static_order, unsigned parts_per_segment, uint16_t *totals,
                                                               WaitPolicy wait) {
  __shared__ float wave_total[kMaxWaves];
  __shared__ unsigned s_part;
  __shared__ float s_prefix;
  const int lane = lane_id();
  const int wave = wave_in_block();
  const int WPB = (int)(blockDim.x >> 6);
  unsigned long long *desc = reinterpret_cast<unsigned long long *>(ws + 64);
  const int chunk_lane = MFMA ? matrix_chunk_of_lane(lane) : lane;

  if (!static_order) {
    if (threadIdx.x == 0) s_part = atomic_add_u32(ws, 1u);
    __syncthreads();
  }
  const unsigned part = static_order ? blockIdx.x : s_part;
  const size_t t0 = ((size_t)part * WPB + wave) * U;

  half8_t v[U];
  load_tiles<U, NT>(v, in, t0 * kTileChunks, n_chunks, chunk_lane);
  float acc = 0.0f;
#pragma unroll
  for (int j = 0; j < U; j++) acc = sum8(v[j], acc);
  acc = lane_group_sum<6>(acc);
  if (lane == 63) wave_total[wave] = acc;
  __syncthreads();

  if (wave == 0) {
    float aggregate = 0.0f;
    for (int w = 0; w < WPB; w++) aggregate += wave_total[w];
    float prefix = 0.0f;
    // the scan restarts at every segment: a segment's first partition has nothing to wait for,
    // and nobody looks back past it
    const unsigned in_segment = parts_per_segment ? part % parts_per_segment : part;
    const long long floor = (long long)part - in_segment;
    const bool muted = part + 1 == wait.mute_partition;
    unsigned long long *mine = desc + ((size_t)part << wait.desc_shift);
    if (in_segment == 0) {
      if (lane == 0 && !muted) atomic_store_u64(mine, kFlagPrefix | __float_as_uint(aggregate));
    } else {
      if (lane == 0 && !muted) atomic_store_u64(mine, kFlagAggregate | __float_as_uint(aggregate));
      prefix = look_back(desc, (long long)part, floor, lane, wait);
      if (lane == 0 && !muted) atomic_store_u64(mine, kFlagPrefix | __float_as_uint(prefix + aggregate));
    }
    if (totals && parts_per_segment && in_segment == parts_per_segment - 1 && lane == 0) totals[part / parts_per_segment] = f16_bits(prefix + aggregate);
    if (lane == 0) s_prefix = prefix;
  }
  __syncthreads();
  float carry = s_prefix;
  for (int w = 0; w < wave; w++) carry += wave_total[w];
  ScanOperands ops;  // built here, behind the wait: the tiles held in registers leave no room for constants before it
  if constexpr (MFMA) ops = make_scan_operands<6>(lane);
  static_for<U>([&](auto J) {
    constexpr int j = decltype(J)::value;
    float tile_total;
    scan_tile<6, MFMA, NT>(v[j], carry, ops, lane, out, (t0 + j) * kTileChunks, n_chunks, nullptr, 0, 0, &tile_total);
    carry += tile_total;
  });
}

// The look-back scan over segments given by offsets: slice p of segment j (offsets_slice: the segment's aligned chunks
// cut into `slices` equal stretches) is partition j * slices + p, and the look-back stops at the segment's first slice.
// A slice of up to U rounds of blockDim chunks stays in registers between its sum and its scan, so every element is
// read once; a longer one (the segment is far longer than the caller expected) is read twice by its block.
// Same workspace layout as full_scan_kernel.
template <typename OFF, int U, bool NT>
__global__ __launch_bounds__(kMaxBlock, 8) void seg_scan_offsets_chained_kernel(const uint16_t *in, uint16_t *out, const OFF *__restrict__ begin, const OFF *__restrict__ end, unsigned slices, int vector,
                                                                                unsigned *ws, int static_order, WaitPolicy wait) {
  static_assert(U >= 2, "the streaming path keeps two rows of wave totals");
  __shared__ float wave_total[U * kMaxWaves];  // [round][wave]; after the look-back: what precedes that wave's chunks of that round
  __shared__ unsigned s_part;
  __shared__ float s_prefix;
  const int lane = lane_id(), wave = wave_in_block();
  const int WPB = (int)(blockDim.x >> 6);
  unsigned long long *desc = reinterpret_cast<unsigned long long *>(ws + 64);
  if (!static_order) {
    if (threadIdx.x == 0) s_part = atomic_add_u32(ws, 1u);
    __syncthreads();
  }
  const unsigned part = static_order ? blockIdx.x : s_part;
  const unsigned p = part % slices;
  const OffsetsSlice s = offsets_slice(begin, end, part / slices, p, slices);
  const bool resident = s.c_hi - s.c_lo <= (size_t)U * blockDim.x;  // block-uniform

  half8_t v[U];
  if (resident) {
#pragma unroll
    for (int r = 0; r < U; r++) {
      const size_t c = s.c_lo + (size_t)r * blockDim.x + threadIdx.x;
      v[r] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
      bool whole;
      if (c < s.c_hi) v[r] = offsets_masked_chunk<NT>(in, c, s.b, s.e, vector, &whole);
    }
#pragma unroll
    for (int r = 0; r < U; r++) {
      const float wt = lane_group_sum<6>(sum8(v[r], 0.0f));
      if (lane == 63) wave_total[r * WPB + wave] = wt;
    }
  } else {
    float acc = 0.0f;
    for (size_t c = s.c_lo + threadIdx.x; c < s.c_hi; c += blockDim.x) {
      bool whole;
      acc = sum8(offsets_masked_chunk<false>(in, c, s.b, s.e, vector, &whole), acc);  // cached: read again below
    }
    acc = lane_group_sum<6>(acc);
    if (lane == 63) wave_total[wave] = acc;
  }
  __syncthreads();

  if (wave == 0) {
    // exclusive scan of the totals in (round, wave) order, 64 at a time; the slice's sum falls out at the end
    const int count = resident ? U * WPB : WPB;
    float before[(U * kMaxWaves + 63) / 64];
    float aggregate = 0.0f;
#pragma unroll
    for (int k = 0; k < (U * kMaxWaves + 63) / 64; k++) {
      const int i = k * 64 + lane;
      const float x = i < count ? wave_total[i] : 0.0f;
      before[k] = aggregate + lane_group_exclusive_scan<6>(x, lane);
      aggregate = readlane(before[k] + x, 63);
    }
    float prefix = 0.0f;
    const bool muted = part + 1 == wait.mute_partition;
    unsigned long long *mine = desc + ((size_t)part << wait.desc_shift);
    if (p == 0) {
      if (lane == 0 && !muted) atomic_store_u64(mine, kFlagPrefix | __float_as_uint(aggregate));
    } else {
      if (lane == 0 && !muted) atomic_store_u64(mine, kFlagAggregate | __float_as_uint(aggregate));
      prefix = look_back(desc, (long long)part, (long long)part - p, lane, wait);
      if (lane == 0 && !muted) atomic_store_u64(mine, kFlagPrefix | __float_as_uint(prefix + aggregate));
    }
    if (lane == 0) s_prefix = prefix;
    if (resident) {
#pragma unroll
      for (int k = 0; k < (U * kMaxWaves + 63) / 64; k++) {
        const int i = k * 64 + lane;
        if (i < count) wave_total[i] = prefix + before[k];
      }
    }
  }
  __syncthreads();

  if (resident) {
#pragma unroll
    for (int r = 0; r < U; r++) {
      const size_t c = s.c_lo + (size_t)r * blockDim.x + threadIdx.x;
      if (s.c_lo + (size_t)r * blockDim.x >= s.c_hi) break;  // block-uniform
      const float e = lane_group_exclusive_scan<6>(sum8(v[r], 0.0f), lane);
      const uint4_t packed = chunk_scan_packed(v[r], wave_total[r * WPB + wave] + e);
      const size_t lo = c * 8;
      if (c >= s.c_hi) continue;  // the round's last chunks lie beyond the slice
      if (vector && lo >= s.b && lo + 8 <= s.e) {
        store_chunk<NT>(reinterpret_cast<uint4_t *>(out) + c, packed);
      } else {
#pragma unroll
        for (int i = 0; i < 8; i++)
          if (lo + i >= s.b && lo + i < s.e) out[lo + i] = (uint16_t)(packed[i / 2] >> (16 * (i & 1)));
      }
    }
    return;
  }
  float carry = s_prefix;
  // the slice again, a round of blockDim chunks at a time (every thread runs the same number of rounds: barriers inside)
  unsigned parity = 0;
  for (size_t c0 = s.c_lo; c0 < s.c_hi; c0 += blockDim.x) {
    const size_t c = c0 + threadIdx.x;
    const bool any = c < s.c_hi;
    bool whole = false;
    half8_t x = {0, 0, 0, 0, 0, 0, 0, 0};
    if (any) x = offsets_masked_chunk<NT>(in, c, s.b, s.e, vector, &whole);
    const float t = sum8(x, 0.0f);
    const float e = lane_group_exclusive_scan<6>(t, lane);
    const float wt = lane_group_sum<6>(t);
    if (lane == 63) wave_total[parity * WPB + wave] = wt;
    __syncthreads();
    float before = 0.0f, all = 0.0f;
    for (int w = 0; w < WPB; w++) {
      const float y = wave_total[parity * WPB + w];
      if (w < wave) before += y;
      all += y;
    }
    parity ^= 1u;
    const uint4_t packed = chunk_scan_packed(x, carry + before + e);
    carry += all;
    if (whole) {
      store_chunk<NT>(reinterpret_cast<uint4_t *>(out) + c, packed);
    } else if (any) {
      const size_t lo = c * 8;
#pragma unroll
      for (int i = 0; i < 8; i++)
        if (lo + i >= s.b && lo + i < s.e) out[lo + i] = (uint16_t)(packed[i / 2] >> (16 * (i & 1)));
    }
  }
}

// The look-back scan with more bytes in flight per wave slot.  A block of full_scan_kernel
// waits about 30 % of its life for its predecessors' aggregates with its whole partition
// parked in registers and nothing in flight; wave slots (32 per CU), not registers, cap what a
// CU can hold.  Here every wave parks ULDS more tiles in LDS (global -> LDS transfers, no
// registers involved): 16 waves x (8 + 4) tiles = 98304 halves per partition, 64 KiB of LDS
// per block, still two blocks per CU.  Tiles U .. U+ULDS-1 of a wave follow its register
// tiles in memory and in scan order.  Same workspace and descriptors as full_scan_kernel.
template <int U, int ULDS, bool NT>
__global__ __launch_bounds__(kMaxBlock) void full_scan_lds_kernel(const half8_t *in, uint4_t *out, size_t n_chunks, unsigned *ws, int static_order, WaitPolicy wait) {
  __shared__ __attribute__((aligned(1024))) half_t held[kMaxWaves * ULDS * kTileHalves];
  __shared__ float wave_total[kMaxWaves];
  __shared__ unsigned s_part;
  __shared__ float s_prefix;
  const int lane = lane_id();
  const int wave = wave_in_block();
  const int WPB = (int)(blockDim.x >> 6);
  unsigned long long *desc = reinterpret_cast<unsigned long long *>(ws + 64);
  ScanOperands ops;

  if (!static_order) {
    if (threadIdx.x == 0) s_part = atomic_add_u32(ws, 1u);
    __syncthreads();
  }
  const unsigned part = static_order ? blockIdx.x : s_part;
  const size_t t0 = ((size_t)part * WPB + wave) * (U + ULDS);

  half8_t v[U];
  load_tiles<U, NT>(v, in, t0 * kTileChunks, n_chunks, lane);
  half_t *mine = held + (size_t)wave * ULDS * kTileHalves;
  const half8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
  for (int j = 0; j < ULDS; j++) {
    const size_t c0 = (t0 + U + j) * kTileChunks;
    if (c0 + lane < n_chunks)
      load_chunk_to_lds(in + c0, (uint32_t)lane * 16u, lds_address_of(mine + j * kTileHalves));
    else
      *reinterpret_cast<half8_t *>(mine + j * kTileHalves + lane * 8) = zero;
  }
  float acc = 0.0f;
#pragma unroll
  for (int j = 0; j < U; j++) acc = sum8(v[j], acc);
  wait_vector_loads<0>();
#pragma unroll
  for (int j = 0; j < ULDS; j++) acc = sum8(*reinterpret_cast<const half8_t *>(mine + j * kTileHalves + lane * 8), acc);
  acc = lane_group_sum<6>(acc);
  if (lane == 63) wave_total[wave] = acc;
  __syncthreads();

  if (wave == 0) {
    float aggregate = 0.0f;
    for (int w = 0; w < WPB; w++) aggregate += wave_total[w];
    float prefix = 0.0f;
    const bool muted = part + 1 == wait.mute_partition;
    unsigned long long *mine = desc + ((size_t)part << wait.desc_shift);
    if (part == 0) {
      if (lane == 0 && !muted) atomic_store_u64(mine, kFlagPrefix | __float_as_uint(aggregate));
    } else {
      if (lane == 0 && !muted) atomic_store_u64(mine, kFlagAggregate | __float_as_uint(aggregate));
      prefix = look_back(desc, (long long)part, 0, lane, wait);
      if (lane == 0 && !muted) atomic_store_u64(mine, kFlagPrefix | __float_as_uint(prefix + aggregate));
    }
    if (lane == 0) s_prefix = prefix;
  }
  __syncthreads();
  float carry = s_prefix;
  for (int w = 0; w < wave; w++) carry += wave_total[w];
  static_for<U>([&](auto J) {
    constexpr int j = decltype(J)::value;
    float tile_total;
    scan_tile<6, false, NT>(v[j], carry, ops, lane, out, (t0 + j) * kTileChunks, n_chunks, nullptr, 0, 0, &tile_total);
    carry += tile_total;
  });
  static_for<ULDS>([&](auto J) {
    constexpr int j = decltype(J)::value;
    float tile_total;
    const half8_t h = *reinterpret_cast<const half8_t *>(mine + j * kTileHalves + lane * 8);
    scan_tile<6, false, NT>(h, carry, ops, lane, out, (t0 + U + j) * kTileChunks, n_chunks, nullptr, 0, 0, &tile_total);
    carry += tile_total;
  });
}

// Segments far larger than one block's reach, first level: block b adds its partition
// (blockDim/64 * U tiles) and writes the fp32 partial to partial[b].
template <int U, bool NT>
__global__ __launch_bounds__(kMaxBlock) void partition_sums_kernel(const half8_t *__restrict__ in, float *__restrict__ partial_out, size_t n_chunks, unsigned xcd_run) {
  __shared__ float partial[kMaxWaves];
  const int lane = lane_id(), wave = wave_in_block();
  const int WPB = (int)(blockDim.x >> 6);
  const size_t part = xcd_run_piece(blockIdx.x, gridDim.x, xcd_run);
  half8_t v[U];
  load_tiles<U, NT>(v, in, (part * WPB + wave) * U * kTileChunks, n_chunks, lane);
  float accs[2] = {0.0f, 0.0f};
#pragma unroll
  for (int j = 0; j < U; j++) accs[j & 1] = sum8(v[j], accs[j & 1]);
  const float total = lane_group_sum<6>(accs[0] + accs[1]);
  if (lane == 63) partial[wave] = total;
  __syncthreads();
  if (threadIdx.x == 0) {
    float s = 0.0f;
    for (int w = 0; w < WPB; w++) s += partial[w];
    partial_out[part] = s;
  }
}
// second level: block j (1024 threads) adds the parts_per_segment partials of segment j (fewer for a last block
// that reaches total_parts) in a fixed order (four independent strided streams per thread, then lanes, then
// waves) and writes the result: fp16 (OUT = uint16_t), or fp32 for a further level (OUT = float)
template <typename OUT>
__global__ __launch_bounds__(1024) void segment_of_partials_kernel(const float *__restrict__ partial_in, OUT *__restrict__ out, size_t parts_per_segment, size_t total_parts) {
  __shared__ float partial[16];
  const int lane = lane_id(), wave = wave_in_block();
  const size_t first = (size_t)blockIdx.x * parts_per_segment;
  if (first + parts_per_segment > total_parts) parts_per_segment = total_parts > first ? total_parts - first : 0;
  const float *p = partial_in + first;
  float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f, a3 = 0.0f;
  size_t i = threadIdx.x;
  for (; i + 3 * 1024 < parts_per_segment; i += 4 * 1024) {
    a0 += p[i];
    a1 += p[i + 1024];
    a2 += p[i + 2048];
    a3 += p[i + 3072];
  }
  for (; i < parts_per_segment; i += 1024) a0 += p[i];
  const float acc = lane_group_sum<6>((a0 + a1) + (a2 + a3));
  if (lane == 63) partial[wave] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    float s = 0.0f;
    for (int w = 0; w < 16; w++) s += partial[w];
    if constexpr (sizeof(OUT) == 4)
      out[blockIdx.x] = s;
    else
      out[blockIdx.x] = f16_bits(s);
  }
}

// out[0] = fp16(sum of n halves), one block
__global__ __launch_bounds__(1024) void sum_f16_kernel(const uint16_t *__restrict__ in, uint16_t *__restrict__ out, size_t n) {
  __shared__ float partial[16];
  const int lane = lane_id(), wave = wave_in_block();
  float acc = 0.0f;
  for (size_t i = threadIdx.x; i < n; i += blockDim.x) acc += (float)__builtin_bit_cast(half_t, in[i]);
  acc = lane_group_sum<6>(acc);
  if (lane == 63) partial[wave] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    float s = 0.0f;
    for (unsigned w = 0; w < (blockDim.x >> 6); w++) s += partial[w];
    out[0] = f16_bits(s);
  }
}

// in-place exclusive prefix sum of n halves (fp32 running sum, fp16 storage), one block
__global__ __launch_bounds__(1024) void exclusive_scan_f16_kernel(uint16_t *data, size_t n) {
  __shared__ float wave_total[16];
  const int lane = lane_id(), wave = wave_in_block();
  const int waves = (int)(blockDim.x >> 6);
  float carry = 0.0f;
  for (size_t base = 0; base < n; base += blockDim.x) {
    const size_t i = base + threadIdx.x;
    const float x = i < n ? (float)__builtin_bit_cast(half_t, data[i]) : 0.0f;
    const float excl = lane_group_exclusive_scan<6>(x, lane);
    if (lane == 63) wave_total[wave] = excl + x;
    __syncthreads();
    float offset = carry, all = 0.0f;
    for (int w = 0; w < waves; w++) {
      const float wt = wave_total[w];
      if (w < wave) offset += wt;
      all += wt;
    }
    if (i < n) data[i] = f16_bits(excl + offset);
    carry += all;
    __syncthreads();
  }
}

}  // namespace tcu
