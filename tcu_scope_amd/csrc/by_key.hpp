// Segments given by a key array: a segment is a run of equal consecutive keys.  Inclusive prefix
// sums inside every run (the reference's thrust::inclusive_scan_by_key baseline,
// src/prefixsum/seg_thrust.cu:46-47) and one sum per run (thrust::reduce_by_key,
// src/reduction/seg_thrust.cu:50-51), fp16 values, fp32 accumulation, one rounding to fp16.
//
// One pass over keys and values.  The scan operator on pairs (head flag, value)
//     (f1, v1) (+) (f2, v2) = (f1 | f2, f2 ? v2 : v1 + v2)
// is associative, so the whole array is scanned like the full-array prefix sum: a lane scans
// its 8 elements serially, the 64 chunk summaries of a tile are scanned across the lanes with
// DPP, tiles are chained in the wave, waves meet in LDS, blocks (partitions of
// blockDim/64 * U tiles, handed out by a ticket) meet through decoupled look-back on 64-bit
// descriptors {status + 4 * flag, fp32 value}: a predecessor whose aggregate carries a head
// flag ends the look-back just as a published prefix does.  The reduction also counts the heads
// (a second, integer look-back) to know where a run's sum goes, and writes a run's sum at the
// head of the NEXT run (the value carried up to that head), so no element ever needs its
// successor's key; the last run is written by the lane that holds the last element.
//
// Every wait is bounded (WaitPolicy): a look-back that gives up yields NaN sums (and, for the
// reduction, counts of 0xffffffff that keep later partitions from writing anything).
#pragma once

#include "full_array.hpp"

namespace tcu {

constexpr unsigned kKeyStatusAggregate = 1u, kKeyStatusPrefix = 2u, kKeyFlagged = 4u;

// (fl, vl) (+) (f, v) -> (f, v)
TCU_DEVICE void seg_combine(unsigned fl, float vl, unsigned &f, float &v) {
  v = f ? v : vl + v;
  f |= fl;
}

// exclusive scan of (F, V) over the 64 lanes of a wave under the operator above
TCU_DEVICE void wave_exclusive_seg_scan(unsigned F, float V, unsigned &Fe, float &Ve) {
  unsigned f = dpp_u32<DPP_WAVE_SHR1>(0u, F);
  float v = dpp<DPP_WAVE_SHR1>(0.0f, V);
  seg_combine(dpp_u32<DPP_ROW_SHR0 + 1>(0u, f), dpp<DPP_ROW_SHR0 + 1>(0.0f, v), f, v);
  seg_combine(dpp_u32<DPP_ROW_SHR0 + 2>(0u, f), dpp<DPP_ROW_SHR0 + 2>(0.0f, v), f, v);
  seg_combine(dpp_u32<DPP_ROW_SHR0 + 4>(0u, f), dpp<DPP_ROW_SHR0 + 4>(0.0f, v), f, v);
  seg_combine(dpp_u32<DPP_ROW_SHR0 + 8>(0u, f), dpp<DPP_ROW_SHR0 + 8>(0.0f, v), f, v);
  seg_combine(dpp_u32<DPP_ROW_BCAST15, 0xA, 0xF, false>(0u, f), dpp<DPP_ROW_BCAST15, 0xA, 0xF, false>(0.0f, v), f, v);
  seg_combine(dpp_u32<DPP_ROW_BCAST31, 0xC, 0xF, false>(0u, f), dpp<DPP_ROW_BCAST31, 0xC, 0xF, false>(0.0f, v), f, v);
  Fe = f;
  Ve = v;
}
// exclusive prefix sum of an unsigned over the 64 lanes
TCU_DEVICE unsigned wave_exclusive_count(unsigned c) {
  unsigned e = dpp_u32<DPP_WAVE_SHR1>(0u, c);
  e += dpp_u32<DPP_ROW_SHR0 + 1>(0u, e);
  e += dpp_u32<DPP_ROW_SHR0 + 2>(0u, e);
  e += dpp_u32<DPP_ROW_SHR0 + 4>(0u, e);
  e += dpp_u32<DPP_ROW_SHR0 + 8>(0u, e);
  e += dpp_u32<DPP_ROW_BCAST15, 0xA, 0xF, false>(0u, e);
  e += dpp_u32<DPP_ROW_BCAST31, 0xC, 0xF, false>(0u, e);
  return e;
}

// Look-back over descriptors whose high word is status + 4 * flag: the walk ends at the nearest
// predecessor that has published its inclusive prefix or whose aggregate carries a head flag.
// Returns the value that precedes partition `part`; NaN when a wait expired.
TCU_DEVICE float look_back_flagged(const unsigned long long *desc, long long part, int lane, WaitPolicy wait) {
  float prefix = 0.0f;
  long long base = part - 1;
  unsigned polls = 0;
  while (true) {
    const long long idx = base - lane;
    const unsigned long long d = idx >= 0 ? atomic_load_u64(desc + ((size_t)idx << wait.desc_shift)) : (unsigned long long)kKeyStatusPrefix << 32;
    const unsigned hi = (unsigned)(d >> 32);
    const unsigned long long is_stop = ballot(hi >= kKeyStatusPrefix);
    const unsigned long long is_empty = ballot(hi == 0u);
    const int first_stop = is_stop ? __builtin_ctzll(is_stop) : 64;
    const unsigned long long needed = first_stop >= 63 ? ~0ull : ((2ull << first_stop) - 1ull);
    if (is_empty & needed) {
      if (polls++ >= wait.poll_limit) {
        note_expired_wait(wait, lane);
        return __builtin_nanf("");
      }
      spin_pause();
      continue;
    }
    float val = lane <= first_stop ? __uint_as_float((unsigned)d) : 0.0f;
    val = lane_group_sum<6>(val);
    prefix += readlane(val, 63);
    if (first_stop < 64) return prefix;
    base -= 64;
  }
}
// Both walks of the reduction in one loop, so that their polls travel together: the value walk as above, and
// the same walk over the {status, count} descriptors that follow the value descriptors in every slot (status
// 1 = aggregate, 2 = inclusive prefix; it ends at a published prefix only).  *count = 0xffffffff when a wait
// expired or a predecessor could not count either; the value is then NaN.
TCU_DEVICE void look_back_value_and_count(const unsigned long long *desc, long long part, int lane, WaitPolicy wait, float *value, unsigned *count) {
  float pv = 0.0f;
  unsigned pc = 0;
  long long base_v = part - 1, base_c = part - 1;
  bool v_done = false, c_done = false;
  unsigned polls = 0;
  const unsigned long long at_start = (unsigned long long)kKeyStatusPrefix << 32;
  while (!v_done || !c_done) {
    const long long iv = base_v - lane, ic = base_c - lane;
    unsigned long long dv = at_start, dc = at_start;
    if (!v_done && iv >= 0) dv = atomic_load_u64(desc + ((size_t)iv << wait.desc_shift));
    if (!c_done && ic >= 0) dc = atomic_load_u64(desc + ((size_t)ic << wait.desc_shift) + 1);
    bool waiting = false;
    if (!v_done) {
      const unsigned hi = (unsigned)(dv >> 32);
      const unsigned long long is_stop = ballot(hi >= kKeyStatusPrefix), is_empty = ballot(hi == 0u);
      const int first_stop = is_stop ? __builtin_ctzll(is_stop) : 64;
      const unsigned long long needed = first_stop >= 63 ? ~0ull : ((2ull << first_stop) - 1ull);
      if (is_empty & needed) {
        waiting = true;
      } else {
        float val = lane <= first_stop ? __uint_as_float((unsigned)dv) : 0.0f;
        val = lane_group_sum<6>(val);
        pv += readlane(val, 63);
        if (first_stop < 64) v_done = true;
        else base_v -= 64;
      }
    }
    if (!c_done) {
      const unsigned hi = (unsigned)(dc >> 32);
      const unsigned long long is_stop = ballot(hi == kKeyStatusPrefix), is_empty = ballot(hi == 0u);
      const int first_stop = is_stop ? __builtin_ctzll(is_stop) : 64;
      const unsigned long long needed = first_stop >= 63 ? ~0ull : ((2ull << first_stop) - 1ull);
      if (is_empty & needed) {
        waiting = true;
      } else {
        unsigned val = lane <= first_stop ? (unsigned)dc : 0u;
        if (ballot(val == 0xffffffffu) != 0ull) {  // a predecessor could not count
          pc = 0xffffffffu;
          c_done = true;
        } else {
          val += wave_exclusive_count(val);  // inclusive in lane 63
          pc += readlane_u32(val, 63);
          if (first_stop < 64) c_done = true;
          else base_c -= 64;
        }
      }
    }
    if (waiting) {
      if (polls++ >= wait.poll_limit) {
        note_expired_wait(wait, lane);
        *value = __builtin_nanf("");
        *count = 0xffffffffu;
        return;
      }
      spin_pause();
    }
  }
  *value = pv;
  *count = pc;
}

// the key in lane l - 1 (lane 0: undefined, the caller replaces it)
TCU_DEVICE int32_t key_of_previous_lane(int32_t k) { return (int32_t)dpp_u32<DPP_WAVE_SHR1>(0u, (unsigned)k); }
TCU_DEVICE int64_t key_of_previous_lane(int64_t k) {
  const unsigned lo = dpp_u32<DPP_WAVE_SHR1>(0u, (unsigned)(uint64_t)k), hi = dpp_u32<DPP_WAVE_SHR1>(0u, (unsigned)((uint64_t)k >> 32));
  return (int64_t)(((uint64_t)hi << 32) | lo);
}
TCU_DEVICE int32_t key_of_lane(int32_t k, int l) { return (int32_t)readlane_u32((unsigned)k, l); }
TCU_DEVICE int64_t key_of_lane(int64_t k, int l) {
  const unsigned lo = readlane_u32((unsigned)(uint64_t)k, l), hi = readlane_u32((unsigned)((uint64_t)k >> 32), l);
  return (int64_t)(((uint64_t)hi << 32) | lo);
}

// What a lane keeps of one chunk (8 elements) between the two passes: 7 registers, so that a wave can hold
// many tiles; the prefix sums inside the chunk are taken again from the raw values in the second pass.
struct KeyChunk {
  half8_t raw;    // the values (zero beyond the end of the array)
  unsigned heads; // bit i: element i starts a run
  unsigned fe;    // exclusive scan over the tile's lanes: a head lies between the tile start and this chunk
  float ve;       //   ... and the value carried from the tile start (or from that head) to this chunk
  unsigned he;    // heads between the tile start and this chunk (reduction only)
};

// workspace words: [0] ticket, [64 ...) per partition a u64 value descriptor followed by a u64 count descriptor
template <typename KEY, int U, bool REDUCE, bool NT>
__global__ __launch_bounds__(kMaxBlock) void by_key_kernel(const KEY *__restrict__ keys, const uint16_t *in, uint16_t *out, KEY *__restrict__ keys_out, unsigned long long *num_runs,
                                                           size_t n, unsigned *ws, int static_order, WaitPolicy wait) {
  __shared__ float wave_v[kMaxWaves];
  __shared__ unsigned wave_f[kMaxWaves], wave_h[kMaxWaves];
  __shared__ unsigned s_part, s_count;
  __shared__ float s_prefix;
  // The reduction writes a run's key where the run ends, after the look-back.  By then the partition's keys have
  // left the registers, and the 4 MiB of L2 of an XCD as well (32 partitions of 128 KiB in flight per XCD), so reading
  // them again from memory costs a second pass over the key array when runs are short (measured: 1.5x the
  // algorithmic bytes at 16 elements per run).  32-bit keys are therefore parked in LDS (128 KiB per partition).
  // 64-bit keys do not fit; for them every chunk parks one key, the one in front of the chunk's first run start (32 KiB),
  // which serves every run of 8 elements and more; only the further run starts of a chunk read their key again.
  constexpr bool STAGE_KEYS = REDUCE && sizeof(KEY) == 4 && U <= 4;
  constexpr bool STAGE_FIRST = REDUCE && !STAGE_KEYS;
  __shared__ __attribute__((aligned(16))) KEY staged_keys[STAGE_KEYS ? kMaxWaves * U * kTileChunks * 8 : 4];
  __shared__ KEY staged_first[STAGE_FIRST ? kMaxWaves * U * kTileChunks : 1];
  const int lane = lane_id(), wave = wave_in_block();
  const int WPB = (int)(blockDim.x >> 6);
  // a partition's two descriptors (value, head count) are neighbours; partitions are 8 << wait.desc_shift bytes apart
  unsigned long long *desc_v = reinterpret_cast<unsigned long long *>(ws + 64);
  unsigned long long *desc_c = desc_v + 1;

  if (!static_order) {
    if (threadIdx.x == 0) s_part = atomic_add_u32(ws, 1u);
    __syncthreads();
  }
  const unsigned part = static_order ? blockIdx.x : s_part;
  const size_t tile0 = ((size_t)part * WPB + wave) * U;

  // ---- pass 1: load, flags, chunk scans, tile scans --------------------------------------
  KeyChunk ch[U];
  KEY k7_prev_tile = 0;
  unsigned wf = 0, wh = 0;  // wave totals under the operator / head count
  float wv = 0.0f;
  unsigned tile_f[U], tile_h[U];
  float tile_v[U];
#pragma unroll
  for (int j = 0; j < U; j++) {
    const size_t e0 = ((tile0 + j) * kTileChunks + lane) * 8;  // first element of this lane's chunk
    const int valid = e0 >= n ? 0 : (n - e0 >= 8 ? 8 : (int)(n - e0));
    KEY k[8];
    half8_t v;
    if (valid == 8) {
      v = load_chunk<NT>(reinterpret_cast<const half8_t *>(in + e0));
      if constexpr (sizeof(KEY) == 4) {
        const uint4_t a = *reinterpret_cast<const uint4_t *>(keys + e0), b = *reinterpret_cast<const uint4_t *>(keys + e0 + 4);
#pragma unroll
        for (int i = 0; i < 4; i++) {
          k[i] = (KEY)a[i];
          k[4 + i] = (KEY)b[i];
        }
        if constexpr (STAGE_KEYS) {
          uint4_t *slot = reinterpret_cast<uint4_t *>(staged_keys + (((size_t)wave * U + j) * kTileChunks + lane) * 8);
          slot[0] = a;
          slot[1] = b;
        }
      } else {
#pragma unroll
        for (int q = 0; q < 4; q++) {
          const uint4_t a = *reinterpret_cast<const uint4_t *>(keys + e0 + 2 * q);
          k[2 * q] = (KEY)(((uint64_t)a[1] << 32) | a[0]);
          k[2 * q + 1] = (KEY)(((uint64_t)a[3] << 32) | a[2]);
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < 8; i++) {
        const bool ok = i < valid;
        v[i] = ok ? __builtin_bit_cast(half_t, in[e0 + i]) : (half_t)0.0f;
        k[i] = ok ? keys[e0 + i] : (KEY)0;
        if constexpr (STAGE_KEYS) staged_keys[(((size_t)wave * U + j) * kTileChunks + lane) * 8 + i] = k[i];
      }
    }
    // the key before the chunk: the previous lane's last key; lane 0 takes it from the wave's previous tile or from memory
    KEY pk = key_of_previous_lane(k[7]);
    if (lane == 0) {
      if (j > 0)
        pk = k7_prev_tile;
      else if (e0 > 0 && e0 < n)
        pk = keys[e0 - 1];
    }
    k7_prev_tile = key_of_lane(k[7], 63);
    unsigned heads = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const KEY before = i ? k[i - 1] : pk;
      if (i < valid && (k[i] != before || e0 + i == 0)) heads |= 1u << i;
    }
    if constexpr (STAGE_FIRST) {
      if (heads != 0u) {
        const int first = __builtin_ctz(heads);
        KEY kb = pk;
#pragma unroll
        for (int i = 1; i < 8; i++)
          if (first == i) kb = k[i - 1];
        staged_first[((size_t)wave * U + j) * kTileChunks + lane] = kb;
      }
    }
    float run = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; i++) run = ((heads >> i) & 1u) ? (float)v[i] : run + (float)v[i];
    ch[j].raw = v;
    ch[j].heads = heads;
    // chunk summary, its exclusive scan over the lanes, and the tile's summary (lane 63's inclusive value)
    const unsigned F = heads ? 1u : 0u;
    wave_exclusive_seg_scan(F, run, ch[j].fe, ch[j].ve);
    unsigned fi = F;
    float vi = run;
    seg_combine(ch[j].fe, ch[j].ve, fi, vi);
    unsigned tf = readlane_u32(fi, 63);
    float tv = readlane(vi, 63);
    unsigned th = 0;
    ch[j].he = 0;
    if constexpr (REDUCE) {
      const unsigned hc = (unsigned)__builtin_popcount(heads);
      ch[j].he = wave_exclusive_count(hc);
      th = readlane_u32(ch[j].he + hc, 63);
    }
    // what the wave's earlier tiles carry into this one, then the wave's running summary with this tile
    tile_f[j] = wf;
    tile_v[j] = wv;
    tile_h[j] = wh;
    seg_combine(wf, wv, tf, tv);
    wf = tf;
    wv = tv;
    wh += th;
  }
  if (lane == 0) {
    wave_f[wave] = wf;
    wave_v[wave] = wv;
    wave_h[wave] = wh;
  }
  __syncthreads();

  // ---- the block's aggregate, look-back, inclusive prefix ------------------------------------
  if (wave == 0) {
    unsigned af = 0, ah = 0;
    float av = 0.0f;
    for (int w = 0; w < WPB; w++) {
      unsigned f = wave_f[w];
      float v = wave_v[w];
      seg_combine(af, av, f, v);
      af = f;
      av = v;
      ah += wave_h[w];
    }
    const bool muted = part + 1 == wait.mute_partition;
    float prefix = 0.0f;
    unsigned count = 0;
    const size_t mine = (size_t)part << wait.desc_shift;
    if (part == 0) {
      if (lane == 0 && !muted) {
        atomic_store_u64(desc_v, ((unsigned long long)kKeyStatusPrefix << 32) | __float_as_uint(av));
        if constexpr (REDUCE) atomic_store_u64(desc_c, ((unsigned long long)kKeyStatusPrefix << 32) | ah);
      }
    } else {
      if (lane == 0 && !muted) {
        atomic_store_u64(desc_v + mine, ((unsigned long long)(kKeyStatusAggregate + (af ? kKeyFlagged : 0u)) << 32) | __float_as_uint(av));
        if constexpr (REDUCE) atomic_store_u64(desc_c + mine, ((unsigned long long)kKeyStatusAggregate << 32) | ah);
      }
      if constexpr (REDUCE)
        look_back_value_and_count(desc_v, (long long)part, lane, wait, &prefix, &count);
      else
        prefix = look_back_flagged(desc_v, (long long)part, lane, wait);
      if (lane == 0 && !muted) {
        atomic_store_u64(desc_v + mine, ((unsigned long long)kKeyStatusPrefix << 32) | __float_as_uint(af ? av : prefix + av));
        // a count that could not be had stays "unknown" for every later partition
        if constexpr (REDUCE) atomic_store_u64(desc_c + mine, ((unsigned long long)kKeyStatusPrefix << 32) | (count == 0xffffffffu ? count : count + ah));
      }
    }
    if (lane == 0) {
      s_prefix = prefix;
      s_count = count;
    }
  }
  __syncthreads();

  // ---- pass 2: carries in, results out -----------------------------------------------------------
  unsigned cf = 0;
  float cv = s_prefix;
  unsigned chd = s_count;
  const bool count_known = chd != 0xffffffffu;
  for (int w = 0; w < wave; w++) {
    unsigned f = wave_f[w];
    float v = wave_v[w];
    seg_combine(cf, cv, f, v);
    cf = f;
    cv = v;
    chd += wave_h[w];
  }
#pragma unroll
  for (int j = 0; j < U; j++) {
    // what precedes the tile: (block prefix, previous waves) (+) (this wave's tiles before j)
    unsigned tf = tile_f[j];
    float tv = tile_v[j];
    seg_combine(cf, cv, tf, tv);
    // what precedes this lane's chunk
    unsigned lf = ch[j].fe;
    float lv = ch[j].ve;
    seg_combine(tf, tv, lf, lv);
    const float carry = lv;
    const size_t e0 = ((tile0 + j) * kTileChunks + lane) * 8;
    const unsigned heads = ch[j].heads;
    const int valid = e0 >= n ? 0 : (n - e0 >= 8 ? 8 : (int)(n - e0));
    const bool last_lane = valid > 0 && e0 + (size_t)valid == n;  // holds the last element of the array
    float r[8];
    if (!REDUCE || heads != 0u || last_lane) {  // the reduction needs the sums only where a run ends
      float run = 0.0f;
#pragma unroll
      for (int i = 0; i < 8; i++) {
        run = ((heads >> i) & 1u) ? (float)ch[j].raw[i] : run + (float)ch[j].raw[i];
        r[i] = (heads & ((2u << i) - 1u)) ? run : carry + run;
      }
    }
    if constexpr (!REDUCE) {
      if (valid == 8) {
        const uint4_t packed = {pack_f16x2(r[0], r[1]), pack_f16x2(r[2], r[3]), pack_f16x2(r[4], r[5]), pack_f16x2(r[6], r[7])};
        store_chunk<NT>(reinterpret_cast<uint4_t *>(out + e0), packed);
      } else {
#pragma unroll
        for (int i = 0; i < 8; i++)
          if (i < valid) out[e0 + i] = f16_bits(r[i]);
      }
    } else {
      if (count_known) {
        const unsigned hb = chd + tile_h[j] + ch[j].he;  // runs started before this chunk
#pragma unroll
        for (int i = 0; i < 8; i++) {
          if ((heads >> i) & 1u) {
            const unsigned idx = hb + (unsigned)__builtin_popcount(heads & ((1u << i) - 1u));  // runs started before element i
            if (idx > 0) {  // the run that ends at element i - 1
              out[idx - 1] = f16_bits(i ? r[i - 1] : carry);
              if (keys_out) {  // idx > 0: element 0 is not meant, the read stays inside the array
                const size_t slot = ((size_t)wave * U + j) * kTileChunks + lane;  // this chunk's position in the partition
                const size_t local = slot * 8 + i;
                if constexpr (STAGE_KEYS)
                  keys_out[idx - 1] = local > 0 ? staged_keys[local - 1] : keys[e0 + i - 1];
                else
                  keys_out[idx - 1] = (heads & ((1u << i) - 1u)) == 0u ? staged_first[slot] : keys[e0 + i - 1];
              }
            }
          }
        }
        if (last_lane) {  // closes the last run
          const unsigned runs = hb + (unsigned)__builtin_popcount(heads);
          out[runs - 1] = f16_bits(r[valid - 1]);
          if (keys_out) keys_out[runs - 1] = keys[n - 1];
          if (num_runs) *num_runs = runs;
        }
      } else if (last_lane && num_runs) {
        *num_runs = ~0ull;  // a wait expired: the number of runs is unknown
      }
    }
  }
}


// ---- the reduction without a chain: four launches, no waits, sums added in index order ------------------------
//
// What makes the one-pass kernel above slow as a reduction is that a run's sum cannot be written before the
// number of runs in front of it is known, so every block holds its partition (keys parked in LDS, values in
// registers) while that count travels down the chain.  Here the count comes first:
//   1. key_heads_kernel    reads the keys once: a bit per element (1 = starts a run), the number of run starts per
//                          partition of kKeyPartElems elements, and the keys of the first kKeyListCap run starts
//                          of every partition, side by side in a list;
//   2. key_count_prefix_kernel  exclusive prefix of the counts (one block);
//   3. reduce_by_heads_kernel   reads the values and the bits: a run that starts after another run start of the same
//                          partition has its sum written where it belongs (prefix + position in the partition), the
//                          keys move from the list to keys_out; what precedes a partition's first run start
//                          ("lead") and what follows its last ("tail", the whole partition without a run start) go
//                          to two floats per partition;
//   4. close_boundary_runs_kernel  a segmented scan of the tails over the partitions (one block) gives every run
//                          that crosses a partition boundary its sum: tails back to the partition it started in +
//                          the lead of the partition it ends in.
// A partition is one wave's work in launches 1 and 3 (8 tiles), so both are grids of small blocks that depend on
// nothing.  The bits of a partition are kept lane-major: lane l owns 8 bytes, byte j = its chunk of tile j.

constexpr int kKeyPartTiles = 8;
constexpr size_t kKeyPartElems = (size_t)kKeyPartTiles * kTileChunks * 8;  // 4096
constexpr unsigned kKeyListCap = (unsigned)(kKeyPartElems / 8);           // run starts of a partition whose keys are parked

// workspace of the four launches, in 8-byte units: bits | list | counts (parts + 1, u32) | lead | tail (fp32)
struct KeyReduceLayout {
  size_t parts, bits_at, list_at, counts_at, lead_at, tail_at, total;  // offsets and total in bytes
};
inline KeyReduceLayout key_reduce_layout(size_t n, size_t key_bytes) {
  KeyReduceLayout l;
  l.parts = (n + kKeyPartElems - 1) / kKeyPartElems;
  auto up = [](size_t b) { return (b + 255) & ~(size_t)255; };
  l.bits_at = 0;
  l.list_at = up(l.parts * 64 * 8);
  l.counts_at = l.list_at + up(l.parts * kKeyListCap * key_bytes);
  l.lead_at = l.counts_at + up((l.parts + 1) * 4);
  l.tail_at = l.lead_at + up(l.parts * 4);
  l.total = l.tail_at + up(l.parts * 4);
  return l;
}

template <typename KEY, int G, bool NT>
__global__ __launch_bounds__(kMaxBlock) void key_heads_kernel(const KEY *__restrict__ keys, size_t n, size_t parts, unsigned long long *__restrict__ bits, unsigned *__restrict__ counts,
                                                              KEY *__restrict__ list, unsigned xcd_run) {
  static_assert(kKeyPartTiles % G == 0, "tiles are loaded in groups of G");
  const int lane = lane_id();
  const size_t p = xcd_run_piece(blockIdx.x, gridDim.x, xcd_run) * (blockDim.x >> 6) + wave_in_block();
  if (p >= parts) return;  // wave-uniform; the kernel has no barrier
  const size_t base = p * kKeyPartElems;
  unsigned long long mine = 0ull;
  unsigned seen = 0;  // run starts of the partition in the tiles before
  KEY last_of_tile = 0;
#pragma unroll
  for (int g = 0; g < kKeyPartTiles; g += G) {
    KEY k[G][8];
#pragma unroll
    for (int j = 0; j < G; j++) {
      const size_t e0 = base + ((size_t)(g + j) * kTileChunks + lane) * 8;
      if (e0 + 8 <= n) {
        constexpr int Q = (int)sizeof(KEY) / 2;  // 16-byte pieces per chunk of keys
#pragma unroll
        for (int q = 0; q < Q; q++) {
          const uint4_t a = __builtin_bit_cast(uint4_t, load_chunk<NT>(reinterpret_cast<const half8_t *>(keys + e0) + q));
          if constexpr (sizeof(KEY) == 4) {
#pragma unroll
            for (int i = 0; i < 4; i++) k[j][4 * q + i] = (KEY)a[i];
          } else {
            k[j][2 * q] = (KEY)(((uint64_t)a[1] << 32) | a[0]);
            k[j][2 * q + 1] = (KEY)(((uint64_t)a[3] << 32) | a[2]);
          }
        }
      } else {
#pragma unroll
        for (int i = 0; i < 8; i++) k[j][i] = e0 + i < n ? keys[e0 + i] : (KEY)0;
      }
    }
#pragma unroll
    for (int j = 0; j < G; j++) {
      const size_t e0 = base + ((size_t)(g + j) * kTileChunks + lane) * 8;
      const int valid = e0 >= n ? 0 : (n - e0 >= 8 ? 8 : (int)(n - e0));
      KEY pk = key_of_previous_lane(k[j][7]);
      if (lane == 0) {
        if (g + j > 0)
          pk = last_of_tile;
        else if (e0 > 0 && e0 < n)
          pk = keys[e0 - 1];
      }
      last_of_tile = key_of_lane(k[j][7], 63);
      unsigned heads = 0;
#pragma unroll
      for (int i = 0; i < 8; i++) {
        const KEY before = i ? k[j][i - 1] : pk;
        if (i < valid && (k[j][i] != before || e0 + i == 0)) heads |= 1u << i;
      }
      mine |= (unsigned long long)heads << (8 * (g + j));
      const unsigned hc = (unsigned)__builtin_popcount(heads);
      const unsigned he = wave_exclusive_count(hc);
      if (list != nullptr && heads != 0u && seen + he < kKeyListCap) {
        unsigned m = seen + he;
#pragma unroll
        for (int i = 0; i < 8; i++) {
          if (((heads >> i) & 1u) && m < kKeyListCap) list[p * kKeyListCap + m] = k[j][i];
          m += (heads >> i) & 1u;
        }
      }
      seen += readlane_u32(he + hc, 63);
    }
  }
  bits[p * 64 + lane] = mine;
  if (lane == 0) counts[p] = seen;
}

// counts[0 .. parts) -> their exclusive prefix, counts[parts] = the total.  One block of 16 waves; a wave takes a
// contiguous stretch, 64 entries at a time.
__global__ __launch_bounds__(1024) void key_count_prefix_kernel(unsigned *counts, size_t parts) {
  __shared__ unsigned wave_total[kMaxWaves];
  const int lane = lane_id(), wave = wave_in_block();
  const size_t steps = (parts + 1023) / 1024, first = (size_t)wave * steps * 64;
  unsigned total = 0;
  for (size_t s = 0; s < steps; s++) {
    const size_t i = first + s * 64 + lane;
    total += i < parts ? counts[i] : 0u;
  }
  total += wave_exclusive_count(total);  // inclusive: the wave's total in lane 63
  if (lane == 63) wave_total[wave] = total;
  __syncthreads();
  unsigned run = 0;
  for (int w = 0; w < wave; w++) run += wave_total[w];
  for (size_t s = 0; s < steps; s++) {
    const size_t i = first + s * 64 + lane;
    const unsigned c = i < parts ? counts[i] : 0u;
    const unsigned e = wave_exclusive_count(c);
    if (i < parts) counts[i] = run + e;
    run += readlane_u32(e + c, 63);
  }
  if (wave == kMaxWaves - 1 && lane == 0) counts[parts] = run;
}

template <typename KEY, bool NT>
__global__ __launch_bounds__(kMaxBlock) void reduce_by_heads_kernel(const uint16_t *__restrict__ in, const unsigned long long *__restrict__ bits, const unsigned *__restrict__ prefix,
                                                                    const KEY *__restrict__ keys, const KEY *__restrict__ list, uint16_t *__restrict__ out, KEY *__restrict__ keys_out,
                                                                    float *__restrict__ lead, float *__restrict__ tail, size_t n, size_t parts, unsigned xcd_run) {
  const int lane = lane_id();
  const size_t p = xcd_run_piece(blockIdx.x, gridDim.x, xcd_run) * (blockDim.x >> 6) + wave_in_block();
  if (p >= parts) return;  // wave-uniform; the kernel has no barrier
  const size_t base = p * kKeyPartElems;
  half8_t v[kKeyPartTiles];
#pragma unroll
  for (int j = 0; j < kKeyPartTiles; j++) {
    const size_t e0 = base + ((size_t)j * kTileChunks + lane) * 8;
    if (e0 + 8 <= n) {
      v[j] = load_chunk<NT>(reinterpret_cast<const half8_t *>(in + e0));
    } else {
#pragma unroll
      for (int i = 0; i < 8; i++) v[j][i] = e0 + i < n ? __builtin_bit_cast(half_t, in[e0 + i]) : (half_t)0.0f;
    }
  }
  const unsigned long long mine = bits[p * 64 + lane];
  const unsigned first_run = prefix[p], runs = prefix[p + 1] - first_run;
  // the keys of the runs that start here: from the list, as far as it goes
  if (keys_out) {
    const unsigned parked = runs < kKeyListCap ? runs : kKeyListCap;
    for (unsigned m = (unsigned)lane; m < parked; m += 64u) keys_out[(size_t)first_run + m] = list[p * kKeyListCap + m];
  }
  unsigned wf = 0, seen = 0;  // the partition so far: a run start seen / how many
  float wv = 0.0f;            //   ... and the sum since the last of them (or since the partition's start)
#pragma unroll
  for (int j = 0; j < kKeyPartTiles; j++) {
    const unsigned heads = (unsigned)(mine >> (8 * j)) & 0xffu;
    const size_t e0 = base + ((size_t)j * kTileChunks + lane) * 8;
    const unsigned hc = (unsigned)__builtin_popcount(heads);
    const unsigned hb = seen + wave_exclusive_count(hc);  // run starts of the partition before this chunk
    // the chunk, element by element: the second and further run starts of the chunk close a run that began in it
    float run = 0.0f, before_first = 0.0f;
    unsigned m = hb;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      if ((heads >> i) & 1u) {
        if (m == hb) {
          before_first = run;
        } else {
          out[(size_t)first_run + m - 1] = f16_bits(run);
        }
        if (keys_out && m >= kKeyListCap) keys_out[(size_t)first_run + m] = keys[e0 + i];
        m++;
        run = (float)v[j][i];
      } else {
        run += (float)v[j][i];
      }
    }
    const unsigned F = heads ? 1u : 0u;
    unsigned fe;
    float ve;
    wave_exclusive_seg_scan(F, run, fe, ve);
    // what precedes this lane's chunk inside the partition
    unsigned lf = fe;
    float lv = ve;
    seg_combine(wf, wv, lf, lv);
    if (heads != 0u) {  // the chunk's first run start closes the run that came in
      if (hb == 0u)
        lead[p] = lv + before_first;  // it came in from outside the partition: closed by the last launch
      else
        out[(size_t)first_run + hb - 1] = f16_bits(lv + before_first);
    }
    unsigned fi = F;
    float vi = run;
    seg_combine(fe, ve, fi, vi);
    unsigned tf = readlane_u32(fi, 63);
    float tv = readlane(vi, 63);
    seg_combine(wf, wv, tf, tv);
    wf = tf;
    wv = tv;
    seen = readlane_u32(hb + hc, 63);
  }
  if (lane == 0) tail[p] = wv;
}

// One block.  Over the partitions, under the operator of the top of this file with flag = "a run starts in the
// partition" and value = tail: the exclusive scan at partition p is what the run that comes into p has gathered
// before p.  That run ends at p's first run start (its sum goes to out[prefix[p] - 1], with p's lead) or runs on;
// the one that reaches the end of the array is the last run.
__global__ __launch_bounds__(1024) void close_boundary_runs_kernel(const unsigned *__restrict__ prefix, const float *__restrict__ lead, const float *__restrict__ tail,
                                                                   uint16_t *__restrict__ out, unsigned long long *num_runs, size_t parts) {
  __shared__ unsigned wave_f[kMaxWaves];
  __shared__ float wave_v[kMaxWaves];
  const int lane = lane_id(), wave = wave_in_block();
  const size_t steps = (parts + 1023) / 1024, first = (size_t)wave * steps * 64;
  unsigned wf = 0;
  float wv = 0.0f;
  for (size_t s = 0; s < steps; s++) {
    const size_t i = first + s * 64 + lane;
    const unsigned F = i < parts && prefix[i + 1] > prefix[i] ? 1u : 0u;
    const float V = i < parts ? tail[i] : 0.0f;
    unsigned fe;
    float ve;
    wave_exclusive_seg_scan(F, V, fe, ve);
    unsigned fi = F;
    float vi = V;
    seg_combine(fe, ve, fi, vi);
    unsigned tf = readlane_u32(fi, 63);
    float tv = readlane(vi, 63);
    seg_combine(wf, wv, tf, tv);
    wf = tf;
    wv = tv;
  }
  if (lane == 0) {
    wave_f[wave] = wf;
    wave_v[wave] = wv;
  }
  __syncthreads();
  unsigned cf = 0;
  float cv = 0.0f;
  for (int w = 0; w < wave; w++) {
    unsigned f = wave_f[w];
    float v = wave_v[w];
    seg_combine(cf, cv, f, v);
    cf = f;
    cv = v;
  }
  for (size_t s = 0; s < steps; s++) {
    const size_t i = first + s * 64 + lane;
    const unsigned before = i < parts ? prefix[i] : 0u;
    const unsigned F = i < parts && prefix[i + 1] > before ? 1u : 0u;
    const float V = i < parts ? tail[i] : 0.0f;
    unsigned fe;
    float ve;
    wave_exclusive_seg_scan(F, V, fe, ve);
    unsigned lf = fe;
    float lv = ve;
    seg_combine(cf, cv, lf, lv);
    if (F && before > 0u) out[(size_t)before - 1] = f16_bits(lv + lead[i]);
    unsigned fi = F;
    float vi = V;
    seg_combine(fe, ve, fi, vi);
    unsigned tf = readlane_u32(fi, 63);
    float tv = readlane(vi, 63);
    seg_combine(cf, cv, tf, tv);
    cf = tf;
    cv = tv;
  }
  if (wave == kMaxWaves - 1 && lane == 0) {  // the last wave's stretch reaches the end of the partitions (or is empty)
    const unsigned total = prefix[parts];
    if (total > 0u) out[(size_t)total - 1] = f16_bits(cv);
    if (num_runs) *num_runs = total;
  }
}

}  // namespace tcu
