// Segments given by a key array: a segment is a run of equal consecutive keys.  Inclusive prefix
// sums inside every run (the reference's thrust::inclusive_scan_by_key baseline,
// src/prefixsum/seg_thrust.cu:46-47) and one sum per run (thrust::reduce_by_key,
// src/reduction/seg_thrust.cu:50-51), fp16 values, fp32 accumulation, one rounding to fp16.
//
// by_key_kernel: one pass over keys and values.  The scan operator on pairs (head flag, value)
//     (f1, v1) (+) (f2, v2) = (f1 | f2, f2 ? v2 : v1 + v2)
// is associative, so the whole array is scanned like the full-array prefix sum: a lane scans
// its 8 elements serially, the 64 chunk summaries of a tile are scanned across the lanes with
// DPP, tiles are chained in the wave, waves meet in LDS, blocks (partitions of
// blockDim/64 * U tiles, handed out by a ticket) meet through decoupled look-back on 64-bit
// descriptors {status + 4 * flag, fp32 value}: a predecessor whose aggregate carries a head
// flag ends the look-back just as a published prefix does.  As a reduction it also counts the heads
// (a second, integer look-back) to know where a run's sum goes, and writes a run's sum at the
// head of the NEXT run (the value carried up to that head), so no element ever needs its
// successor's key; the last run is written by the lane that holds the last element.
// Every wait is bounded (WaitPolicy): a look-back that gives up yields NaN sums (and, for the
// reduction, counts of 0xffffffff that keep later partitions from writing anything).
//
// The reduction's default form is the sequence of launches in the second half of this file, which waits
// for nothing; by_key_kernel<..., REDUCE = true> stays selectable.
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
  unsigned long long d = 0;
  bool reload = true;  // per lane, as in look_back: a poll repeats only the reads that found nothing and still matter
  while (true) {
    const long long idx = base - lane;
    if (reload) d = idx >= 0 ? atomic_load_u64(desc + ((size_t)idx << wait.desc_shift)) : (unsigned long long)kKeyStatusPrefix << 32;
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
      reload = hi == 0u && ((needed >> lane) & 1ull) != 0;
      spin_pause();
      continue;
    }
    float val = lane <= first_stop ? __uint_as_float((unsigned)d) : 0.0f;
    val = lane_group_sum<6>(val);
    prefix += readlane(val, 63);
    if (first_stop < 64) return prefix;
    base -= 64;
    reload = true;
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


// ---- the reduction without a chain: five launches, no waits, sums added in index order ------------------------
//
// What makes the one-pass kernel above slow as a reduction is that a run's sum cannot be written before the
// number of runs in front of it is known, so every block holds its partition (keys parked in LDS, values in
// registers) while that count travels down the chain.  Here the count comes first:
//   1. key_heads_kernel    reads the keys once: a bit per element (1 = starts a run), the number of run starts per
//                          partition of kKeyPartElems elements, and the keys of the first kKeyListCap run starts
//                          of every partition, side by side in a list;
//   2. key_group_prefix_kernel  the run starts in front of every group of 64 partitions (one block);
//   3. reduce_by_heads_kernel   reads the values and the bits: a run that starts after another run start of the same
//                          partition has its sum written where it belongs (runs in front of the group + in front of
//                          the partition + in the partition), the keys move from the list to keys_out; what precedes
//                          a partition's first run start ("lead") and what follows its last ("tail", the whole
//                          partition without a run start) go to two floats per partition;
//   4. key_group_tails_kernel, 5. close_boundary_runs_kernel  a segmented scan of the tails over the partitions
//                          gives every run that crosses a partition boundary its sum: tails back to the partition it
//                          started in + the lead of the partition it ends in.
// A partition is one wave's work in launches 1 and 3 (8 tiles of values), so both are grids of small blocks that
// depend on nothing; launches 2, 4 and 5 touch a few bytes per partition.  The bits of a partition are kept
// lane-major for launch 3: lane l owns 8 bytes, byte j = its chunk of tile j.
// Measured (2^28 elements, 32-bit keys, runs of 16384 / 16 elements): launch 1 169 / 192 us (0.86 of the HBM peak as
// long as it writes nothing; the bits, 3 % of its bytes, cost 10 %), launch 3 83 / 122 us, the three small ones 21 us
// together; per call 265 / 334 us against 384 / 437 us for the one-pass kernel.

constexpr int kKeyPartTiles = 8;
constexpr size_t kKeyPartElems = (size_t)kKeyPartTiles * kTileChunks * 8;  // 4096
constexpr unsigned kKeyListCap = (unsigned)(kKeyPartElems / 8);           // run starts of a partition whose keys are parked

// workspace: bits | list | counts (u32) | lead | tail (fp32) per partition; prefix (groups + 1), flag, tail per group of 64 partitions
struct KeyReduceLayout {
  size_t parts, groups, bits_at, list_at, counts_at, lead_at, tail_at, gprefix_at, gflag_at, gtail_at, total;  // offsets and total in bytes
};
inline KeyReduceLayout key_reduce_layout(size_t n, size_t key_bytes) {
  KeyReduceLayout l;
  l.parts = (n + kKeyPartElems - 1) / kKeyPartElems;
  auto up = [](size_t b) { return (b + 255) & ~(size_t)255; };
  l.bits_at = 0;
  l.list_at = up(l.parts * 64 * 8);
  l.counts_at = l.list_at + up(l.parts * kKeyListCap * key_bytes);
  l.groups = (l.parts + 63) / 64;
  l.lead_at = l.counts_at + up(l.parts * 4);
  l.tail_at = l.lead_at + up(l.parts * 4);
  l.gprefix_at = l.tail_at + up(l.parts * 4);
  l.gflag_at = l.gprefix_at + up((l.groups + 1) * 4);
  l.gtail_at = l.gflag_at + up(l.groups * 4);
  l.total = l.gtail_at + up(l.groups * 4);
  return l;
}

// One partition's keys -> its bits, its number of run starts and its list.  WHOLE: the partition lies inside the array.
// The keys are read 16 bytes per lane with the lanes side by side (whole cache lines per instruction): a "key tile" is
// 1 KiB of keys, a lane holds KPL = 4 (32-bit) or 2 (64-bit) consecutive ones.  The bits are wanted by the byte, one
// byte per 8 consecutive elements: LPB = 8 / KPL neighbouring lanes put theirs together (quad permutes), and the first
// lane of each such set gathers the bytes of the value tile's lane it stands for (see reduce_partition_by_heads).
template <typename KEY, int G_ASKED, bool NT, bool WHOLE>
TCU_DEVICE void key_heads_of_partition(const KEY *__restrict__ keys, size_t n, size_t p, int lane, unsigned long long *__restrict__ bits, unsigned *__restrict__ counts, KEY *__restrict__ list) {
  constexpr int KPL = 16 / (int)sizeof(KEY);
  constexpr int KT_ELEMS = 64 * KPL;                        // elements per key tile
  constexpr int KTS = (int)(kKeyPartElems / KT_ELEMS);      // key tiles per partition: 16 or 32
  constexpr int KTPT = kTileChunks * 8 / KT_ELEMS;          // key tiles per tile of values: 2 or 4
  constexpr int LPB = 8 / KPL;
  constexpr int G = G_ASKED < KTS ? G_ASKED : KTS;  // key tiles in flight
  static_assert(KTS % G == 0, "key tiles are loaded in groups of G");
  const size_t base = p * kKeyPartElems;
  unsigned long long word[KTPT];
#pragma unroll
  for (int r = 0; r < KTPT; r++) word[r] = 0ull;
  unsigned seen = 0;  // run starts of the partition in the key tiles before
  KEY last_of_tile = 0;
#pragma unroll
  for (int g = 0; g < KTS; g += G) {
    KEY k[G][KPL];
#pragma unroll
    for (int j = 0; j < G; j++) {
      const size_t e0 = base + ((size_t)(g + j) * 64 + lane) * KPL;
      if (WHOLE || e0 + KPL <= n) {
        const uint4_t a = __builtin_bit_cast(uint4_t, load_chunk<NT>(reinterpret_cast<const half8_t *>(keys + e0)));
        if constexpr (sizeof(KEY) == 4) {
#pragma unroll
          for (int i = 0; i < 4; i++) k[j][i] = (KEY)a[i];
        } else {
          k[j][0] = (KEY)(((uint64_t)a[1] << 32) | a[0]);
          k[j][1] = (KEY)(((uint64_t)a[3] << 32) | a[2]);
        }
      } else {
#pragma unroll
        for (int i = 0; i < KPL; i++) k[j][i] = e0 + i < n ? keys[e0 + i] : (KEY)0;
      }
    }
#pragma unroll
    for (int j = 0; j < G; j++) {
      const int kt = g + j;
      const size_t e0 = base + ((size_t)kt * 64 + lane) * KPL;
      KEY pk = key_of_previous_lane(k[j][KPL - 1]);
      if (lane == 0) {
        if (kt > 0)
          pk = last_of_tile;
        else
          pk = e0 > 0 ? keys[e0 - 1] : (KEY)~k[j][0];  // the first element of the array starts a run
      }
      last_of_tile = key_of_lane(k[j][KPL - 1], 63);
      unsigned heads = 0;  // bit i = element i differs from the one before
#pragma unroll
      for (int i = KPL - 1; i >= 0; i--) heads = heads + heads + (k[j][i] != (i ? k[j][i - 1] : pk) ? 1u : 0u);
      if constexpr (!WHOLE) {
        const int valid = e0 >= n ? 0 : (n - e0 >= (size_t)KPL ? KPL : (int)(n - e0));
        heads &= (1u << valid) - 1u;
      }
      if (ballot(heads != 0u) == 0ull) continue;  // wave-uniform: most key tiles of long runs
      unsigned byte = heads;
      if constexpr (LPB == 2) {
        byte |= dpp_u32<0xF5>(0u, heads) << 4;  // quad_perm:[1,1,3,3]: the odd neighbour's bits
      } else {
        byte |= dpp_u32<0x55>(0u, heads) << 2;  // quad_perm:[1,1,1,1]
        byte |= dpp_u32<0xAA>(0u, heads) << 4;  // quad_perm:[2,2,2,2]
        byte |= dpp_u32<0xFF>(0u, heads) << 6;  // quad_perm:[3,3,3,3]
      }
      word[kt % KTPT] |= (unsigned long long)byte << (8 * (kt / KTPT));
      const unsigned hc = (unsigned)__builtin_popcount(heads);
      const unsigned he = wave_exclusive_count(hc);
      if (list != nullptr && heads != 0u && seen + he < kKeyListCap) {
        unsigned m = seen + he;
#pragma unroll
        for (int i = 0; i < KPL; i++) {
          if (((heads >> i) & 1u) && m < kKeyListCap) list[p * kKeyListCap + m] = k[j][i];
          m += (heads >> i) & 1u;
        }
      }
      seen += readlane_u32(he + hc, 63);
    }
  }
  // A partition without a run start writes no bits (nobody reads them: see reduce_partition_by_heads).  The bits are
  // 3 % of the bytes of this launch and cost 12 % of its time (writes among the reads; 10 % when non-temporal).
  if (seen != 0u && lane % LPB == 0) {
#pragma unroll
    for (int r = 0; r < KTPT; r++) {
      unsigned long long *at = bits + p * 64 + r * (64 / LPB) + lane / LPB;
      if constexpr (NT) __builtin_nontemporal_store(word[r], at);
      else *at = word[r];
    }
  }
  if (lane == 0) counts[p] = seen;
}

template <typename KEY, int G, bool NT>
__global__ __launch_bounds__(kMaxBlock) void key_heads_kernel(const KEY *__restrict__ keys, size_t n, size_t parts, unsigned long long *__restrict__ bits, unsigned *__restrict__ counts,
                                                              KEY *__restrict__ list, unsigned xcd_run) {
  const size_t p = xcd_run_piece(blockIdx.x, gridDim.x, xcd_run) * (blockDim.x >> 6) + wave_in_block();
  if (p >= parts) return;  // wave-uniform; the kernel has no barrier
  if ((p + 1) * kKeyPartElems <= n)
    key_heads_of_partition<KEY, G, NT, true>(keys, n, p, lane_id(), bits, counts, list);
  else
    key_heads_of_partition<KEY, G, NT, false>(keys, n, p, lane_id(), bits, counts, list);
}

// Scan over the 1024 threads of a block of what each of them has gathered: exclusive prefix of a count ...
TCU_DEVICE unsigned block_exclusive_count(unsigned mine, unsigned *wave_total, int lane, int wave) {
  const unsigned e = wave_exclusive_count(mine);
  if (lane == 63) wave_total[wave] = e + mine;
  __syncthreads();
  unsigned before = 0;
  for (int w = 0; w < wave; w++) before += wave_total[w];
  return before + e;
}
// ... and of a (flag, value) pair under the operator at the top of this file
TCU_DEVICE void block_exclusive_seg_scan(unsigned F, float V, unsigned *wave_f, float *wave_v, int lane, int wave, unsigned &Fe, float &Ve) {
  unsigned fe, fi = F;
  float ve, vi = V;
  wave_exclusive_seg_scan(F, V, fe, ve);
  seg_combine(fe, ve, fi, vi);
  if (lane == 63) {
    wave_f[wave] = fi;
    wave_v[wave] = vi;
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
  seg_combine(cf, cv, fe, ve);
  Fe = fe;
  Ve = ve;
}

// The partitions are taken in groups of 64: a wave reads a group's counts in one load.
// group_prefix[g] = the run starts in front of group g, g = 0 .. groups.
// One block of 16 waves; a wave takes a contiguous stretch of the groups, adds up each of them and keeps the sum of
// the stretch's i-th group in lane i % 64 of register i / 64 (at most kMaxGroupRows registers: 2^20 partitions).
constexpr int kMaxGroupRows = 16;
__global__ __launch_bounds__(1024) void key_group_prefix_kernel(const unsigned *__restrict__ counts, unsigned *__restrict__ group_prefix, size_t parts, size_t groups) {
  __shared__ unsigned wave_total[kMaxWaves];
  const int lane = lane_id(), wave = wave_in_block();
  const size_t per_wave = (groups + kMaxWaves - 1) / kMaxWaves, first = (size_t)wave * per_wave;
  const size_t mine = first >= groups ? 0 : (groups - first < per_wave ? groups - first : per_wave);  // groups of this wave
  unsigned row[kMaxGroupRows];
#pragma unroll
  for (int r = 0; r < kMaxGroupRows; r++) {
    row[r] = 0u;
    if ((size_t)r * 64 < mine) {
      for (int gl0 = 0; gl0 < 64; gl0 += 16) {  // 16 loads in flight, then their sums
        unsigned c[16];
#pragma unroll
        for (int b = 0; b < 16; b++) {
          const size_t i = (first + (size_t)r * 64 + gl0 + b) * 64 + lane;
          c[b] = (size_t)r * 64 + gl0 + b < mine && i < parts ? counts[i] : 0u;
        }
#pragma unroll
        for (int b = 0; b < 16; b++) {
          const unsigned sum = readlane_u32(c[b] + wave_exclusive_count(c[b]), 63);
          if (lane == gl0 + b) row[r] = sum;
        }
      }
    }
  }
  unsigned stretch = 0;
#pragma unroll
  for (int r = 0; r < kMaxGroupRows; r++) stretch += row[r];
  unsigned before = block_exclusive_count(stretch, wave_total, lane, wave);  // lanes of a wave: their sums of all rows, in lane order - not the order of the groups
  // so only the waves' totals are taken from it: what lies in front of this wave's stretch
  before = readlane_u32(before, 0);
#pragma unroll
  for (int r = 0; r < kMaxGroupRows; r++) {
    if ((size_t)r * 64 < mine) {
      const unsigned e = wave_exclusive_count(row[r]);
      const size_t gl = (size_t)r * 64 + lane;
      if (gl < mine) group_prefix[first + gl] = before + e;
      before += readlane_u32(e + row[r], 63);
    }
  }
  if (first + mine == groups && mine > 0 && lane == 0) group_prefix[groups] = before;  // the wave whose stretch ends the groups
  if (groups == 0 && threadIdx.x == 0) group_prefix[0] = 0u;
}
// run starts in front of partition p: those in front of its group + those of the group's partitions before it
TCU_DEVICE unsigned runs_before_partition(const unsigned *__restrict__ counts, const unsigned *__restrict__ group_prefix, size_t p, int lane, unsigned *own) {
  const size_t first = p & ~(size_t)63;
  const unsigned c = first + lane <= p ? counts[first + lane] : 0u;  // the partitions of p's group up to p: all exist
  const unsigned e = wave_exclusive_count(c);
  const int at = (int)(p - first);
  *own = readlane_u32(c, at);
  return group_prefix[p >> 6] + readlane_u32(e, at);
}

// One partition's values and bits -> the sums of the runs that start and end in it, the keys of the runs that
// start in it, its lead and its tail.
template <typename KEY, bool NT, bool WHOLE>
TCU_DEVICE void reduce_partition_by_heads(const uint16_t *__restrict__ in, const unsigned long long *__restrict__ bits, const unsigned *__restrict__ counts, const unsigned *__restrict__ group_prefix, const KEY *__restrict__ keys,
                                          const KEY *__restrict__ list, uint16_t *__restrict__ out, KEY *__restrict__ keys_out, float *__restrict__ lead, float *__restrict__ tail, size_t n, size_t p,
                                          int lane) {
  const size_t base = p * kKeyPartElems;
  half8_t v[kKeyPartTiles];
#pragma unroll
  for (int j = 0; j < kKeyPartTiles; j++) {
    const size_t e0 = base + ((size_t)j * kTileChunks + lane) * 8;
    if (WHOLE || e0 + 8 <= n) {
      v[j] = load_chunk<NT>(reinterpret_cast<const half8_t *>(in + e0));
    } else {
#pragma unroll
      for (int i = 0; i < 8; i++) v[j][i] = e0 + i < n ? __builtin_bit_cast(half_t, in[e0 + i]) : (half_t)0.0f;
    }
  }
  unsigned runs;
  const unsigned first_run = runs_before_partition(counts, group_prefix, p, lane, &runs);
  const unsigned long long mine = runs ? bits[p * 64 + lane] : 0ull;  // wave-uniform
  const bool keys_beyond_list = keys_out != nullptr && runs > kKeyListCap;  // wave-uniform
  if (keys_out) {  // the keys of the runs that start here: from the list, as far as it goes
    const unsigned parked = runs < kKeyListCap ? runs : kKeyListCap;
    for (unsigned m = (unsigned)lane; m < parked; m += 64u) keys_out[(size_t)first_run + m] = list[p * kKeyListCap + m];
  }
  unsigned wf = 0, seen = 0;  // the partition so far: a run start seen / how many
  float wv = 0.0f;            //   ... and the sum since the last of them (or since the partition's start)
#pragma unroll
  for (int j = 0; j < kKeyPartTiles; j++) {
    const unsigned heads = (unsigned)(mine >> (8 * j)) & 0xffu;
    if (ballot(heads != 0u) == 0ull) {  // wave-uniform: no run starts in this tile
      wv += readlane(lane_group_sum<6>(sum8(v[j], 0.0f)), 63);
      continue;
    }
    const size_t e0 = base + ((size_t)j * kTileChunks + lane) * 8;
    const unsigned hc = (unsigned)__builtin_popcount(heads);
    const unsigned hb = seen + wave_exclusive_count(hc);  // run starts of the partition before this chunk
    float run = 0.0f, before_first = 0.0f;
    if (ballot(hc > 1u) == 0ull) {  // wave-uniform: at most one run start per chunk, nothing to write from inside a chunk
#pragma unroll
      for (int i = 0; i < 8; i++) {
        const bool h = (heads >> i) & 1u;
        before_first = h ? run : before_first;
        run = (h ? 0.0f : run) + (float)v[j][i];
      }
      if (keys_beyond_list && heads != 0u && hb >= kKeyListCap) keys_out[(size_t)first_run + hb] = keys[e0 + __builtin_ctz(heads)];
    } else {  // the second and further run starts of a chunk close a run that began in it
      unsigned m = hb;
#pragma unroll
      for (int i = 0; i < 8; i++) {
        if ((heads >> i) & 1u) {
          if (m == hb)
            before_first = run;
          else
            out[(size_t)first_run + m - 1] = f16_bits(run);
          if (keys_beyond_list && m >= kKeyListCap) keys_out[(size_t)first_run + m] = keys[e0 + i];
          m++;
          run = 0.0f;
        }
        run += (float)v[j][i];
      }
    }
    const unsigned F = heads ? 1u : 0u;
    unsigned fe;
    float ve;
    wave_exclusive_seg_scan(F, run, fe, ve);
    unsigned lf = fe;  // what precedes this lane's chunk inside the partition
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

template <typename KEY, bool NT>
__global__ __launch_bounds__(kMaxBlock) void reduce_by_heads_kernel(const uint16_t *__restrict__ in, const unsigned long long *__restrict__ bits, const unsigned *__restrict__ counts, const unsigned *__restrict__ group_prefix,
                                                                    const KEY *__restrict__ keys, const KEY *__restrict__ list, uint16_t *__restrict__ out, KEY *__restrict__ keys_out,
                                                                    float *__restrict__ lead, float *__restrict__ tail, size_t n, size_t parts, unsigned xcd_run) {
  const size_t p = xcd_run_piece(blockIdx.x, gridDim.x, xcd_run) * (blockDim.x >> 6) + wave_in_block();
  if (p >= parts) return;  // wave-uniform; the kernel has no barrier
  if ((p + 1) * kKeyPartElems <= n)
    reduce_partition_by_heads<KEY, NT, true>(in, bits, counts, group_prefix, keys, list, out, keys_out, lead, tail, n, p, lane_id());
  else
    reduce_partition_by_heads<KEY, NT, false>(in, bits, counts, group_prefix, keys, list, out, keys_out, lead, tail, n, p, lane_id());
}

// The runs that cross a partition boundary.  Under the operator of the top of this file with flag = "a run starts in
// the partition" and value = tail, the exclusive scan at partition p is what the run that comes into p has gathered
// before p.  That run ends at p's first run start (its sum goes in front of p's first own run, with p's lead) or
// runs on; the one that reaches the end of the array is the last run.  Two small launches with one wave per group of
// 64 partitions: the groups' summaries; then every wave walks back over the summaries of the groups before its own to
// the nearest one in which a run starts - one step when runs are shorter than 2^18 elements - and scans its group.
__global__ __launch_bounds__(kMaxBlock) void key_group_tails_kernel(const unsigned *__restrict__ counts, const float *__restrict__ tail, unsigned *__restrict__ group_flag, float *__restrict__ group_tail,
                                                                    size_t parts, size_t groups) {
  const size_t g = (size_t)blockIdx.x * (blockDim.x >> 6) + wave_in_block();
  if (g >= groups) return;
  const int lane = lane_id();
  const size_t i = g * 64 + lane;
  unsigned F = i < parts && counts[i] > 0u ? 1u : 0u, fe;
  float V = i < parts ? tail[i] : 0.0f, ve;
  wave_exclusive_seg_scan(F, V, fe, ve);
  seg_combine(fe, ve, F, V);
  if (lane == 63) {
    group_flag[g] = F;
    group_tail[g] = V;
  }
}
__global__ __launch_bounds__(kMaxBlock) void close_boundary_runs_kernel(const unsigned *__restrict__ counts, const unsigned *__restrict__ group_prefix, const float *__restrict__ lead,
                                                                        const float *__restrict__ tail, const unsigned *__restrict__ group_flag, const float *__restrict__ group_tail,
                                                                        uint16_t *__restrict__ out, unsigned long long *num_runs, size_t parts, size_t groups) {
  const size_t g = (size_t)blockIdx.x * (blockDim.x >> 6) + wave_in_block();
  if (g >= groups) return;
  const int lane = lane_id();
  // what comes into the group: the groups before it, from the nearest back to the first one in which a run starts
  float carry = 0.0f;
  for (long long base = (long long)g - 1; base >= 0; base -= 64) {
    const long long at = base - lane;
    const unsigned f = at >= 0 ? group_flag[at] : 1u;
    const unsigned long long stops = ballot(f != 0u);
    const int first_stop = stops ? __builtin_ctzll(stops) : 64;
    float v = at >= 0 && lane <= first_stop ? group_tail[at] : 0.0f;
    carry += readlane(lane_group_sum<6>(v), 63);
    if (first_stop < 64) break;
  }
  const size_t i = g * 64 + lane;
  const unsigned c = i < parts ? counts[i] : 0u;
  unsigned F = c > 0u ? 1u : 0u, fe;
  float V = i < parts ? tail[i] : 0.0f, ve;
  wave_exclusive_seg_scan(F, V, fe, ve);
  seg_combine(0u, carry, fe, ve);  // ve: what the run that comes into this partition has gathered
  const unsigned before = group_prefix[g] + wave_exclusive_count(c);
  if (F && before > 0u) out[(size_t)before - 1] = f16_bits(ve + lead[i]);
  if (g + 1 == groups) {  // the run that reaches the end of the array
    seg_combine(fe, ve, F, V);
    const unsigned total = group_prefix[groups];
    if (lane == 63) {
      if (total > 0u) out[(size_t)total - 1] = f16_bits(V);
      if (num_runs) *num_runs = total;
    }
  }
}

}  // namespace tcu
