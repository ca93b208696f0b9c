// Host-side argument validation and kernel selection for the C entry points.
// Mirrors the preconditions of the reference's harnesses (segment-size checks ->
// "unsupported", num_elements % segment_size, grid limits: reference
// src/reduction/seg_wmma_16.cu:16-18, seg_wmma_16n.cu:17-22,44-49,
// src/reduction/wmma_2kers.cu:23-26).
#pragma once

#include <stddef.h>
#include <stdint.h>
#include <stdio.h>

#include <string>

#include "../../include/tcu_scope.h"
#include "../../include/tcu_scope_dev.h"
#include "launch.hpp"
#include "seg_reduce.hpp"
#include "seg_scan.hpp"
#include "full_array.hpp"
#include "by_key.hpp"
#include "gemv.hpp"
#include "gemm.hpp"
#include "util_kernels.hpp"

namespace tcu {

inline std::string &last_error_string() {
  static thread_local std::string s;
  return s;
}
inline int fail(int code, const std::string &msg) {
  last_error_string() = msg;
  return code;
}

struct Options {
  bool nontemporal = true;
  int scan_store_policy = kStoreStream;     // stores of the segmented scans and of the copy probe while `nontemporal` is on: kStoreAlternate or kStoreStream
  bool static_order = false;
  int gemm_big_tiles = -1;     // 256 x 256 block tiles: 1 wherever M and N allow, 0 never, -1 where there are at least 128 of them (and 192 x 192 tiles where they fill the chip better); 192: 192 x 192 tiles wherever M and N allow
  bool gemm_bk64 = false;      // K step 64 (prefetch depth <= 2) instead of 32
  bool gemm_staged_epilogue = true;   // 16x16x32 big-tile kernel: turn the outputs through LDS so that rows are written whole (C and D 16-byte aligned)
  int gemm_direct_lds = -1;    // 3 or 4: global -> LDS transfers, K step 32, that many LDS buffers; 64: K step 64, two buffers; 65: K step 64, three A and two B buffers; 66: as 65 on 16x16x32 MFMAs; 0: register-staged kernel; -1: by shape
  int scan_lds_tiles = -1;     // full scan AUTO: park 4 extra tiles per wave in LDS: 1 always, 0 never, -1 where it measures faster (up to 2^27 elements)
  int gemv_rows = 0, gemv_tiles = 0, gemv_waves = 0;  // block GEMV shape (rows per block, tiles per wave and step, waves); 0 = default
  int gemv_col_blocks = 1024;  // column-major GEMV: about this many blocks (slabs of 512 rows x stretches of K)
  int gemv_col_shape = 82;     // column-major GEMV: waves per block (4 or 8) * 10 + groups of 8 columns per wave and round (1 or 2)
  bool gemv_strip_lds = true;  // strip GEMV (TCU_VARIANT_MFMA_16N): stage the strip through LDS where K is a multiple of 512
  int gemm_depth = 4;          // global-load prefetch depth of the K-step-32 kernel (1..4)
  int scan_lds_pad = -1;       // KiB of LDS a block of the segmented block scan asks for and leaves unused (caps the blocks a compute unit holds); -1 = AUTO's table
  int compute_units = 256;     // blocks of the big-tile GEMM kernel the device runs at a time (one per compute unit; set by tcu_init)
  int gemm_split_tail = 1;     // spread the K steps of the tiles of a last, partly filled round of the GEMM grid over all compute units: 0 never, 1 where it pays, 2 always
  int many_totals = 65536;     // multi-kernel sequences: from this many per-segment totals on, the step over the totals is itself a multi-block launch
  int xcd_run = -1;            // consecutive pieces of work per XCD (xcd_run_piece): -1 = the measured value for the size, 0 = none, C > 0 = C
  unsigned lookback_poll_limit = kDefaultPollLimit;  // polls of an unpublished value before a single-pass kernel gives up (results become NaN)
  unsigned test_mute_partition = 0;                  // tests only: partition test_mute_partition - 1 of a single-pass kernel publishes nothing
  bool offsets_scan_chain = true;   // scan over offsets, expected segments beyond 65536 halves: one pass with look-back between a segment's slices instead of slice sums + a second read
  bool by_key_reduce_chain = false;  // reduction by key: the one-pass look-back kernel instead of the four launches that wait for nothing
  int by_key_waves = 0;              // waves per block of the two big launches of the reduction by key (0 = default)
  int by_key_key_tiles = 0;          // KiB of keys a wave of its first launch has in flight: 4, 8 or 16 (0 = default)
};
inline Options &options() {
  static Options o;
  return o;
}
inline int set_option(const char *name, int value) {
  if (!name) return fail(TCU_ERR_INVALID_ARG, "tcu_set_option: null name");
  const std::string n(name);
  Options &o = options();
  if (n == "nontemporal") o.nontemporal = value != 0;
  else if (n == "scan_store_policy") o.scan_store_policy = value == kStoreStream ? kStoreStream : kStoreAlternate;
  else if (n == "static_order") o.static_order = value != 0;
  else if (n == "gemm_big_tiles") o.gemm_big_tiles = value < 0 ? -1 : (value == 192 ? 192 : (value != 0));
  else if (n == "gemm_direct_lds") o.gemm_direct_lds = value;
  else if (n == "gemm_depth") o.gemm_depth = value;
  else if (n == "gemv_rows") o.gemv_rows = value;
  else if (n == "gemv_tiles") o.gemv_tiles = value;
  else if (n == "gemv_waves") o.gemv_waves = value;
  else if (n == "gemv_col_blocks") o.gemv_col_blocks = value < 1 ? 1 : value;
  else if (n == "gemv_col_shape") o.gemv_col_shape = value;
  else if (n == "gemv_strip_lds") o.gemv_strip_lds = value != 0;
  else if (n == "scan_lds_tiles") o.scan_lds_tiles = value < 0 ? -1 : (value != 0);
  else if (n == "gemm_bk64") o.gemm_bk64 = value != 0;
  else if (n == "offsets_scan_chain") o.offsets_scan_chain = value != 0;
  else if (n == "by_key_reduce_chain") o.by_key_reduce_chain = value != 0;
  else if (n == "by_key_key_tiles") o.by_key_key_tiles = value == 4 || value == 8 || value == 16 ? value : 0;
  else if (n == "by_key_waves") o.by_key_waves = value < 0 ? 0 : (value > kMaxWaves ? kMaxWaves : value);
  else if (n == "gemm_staged_epilogue") o.gemm_staged_epilogue = value != 0;
  else if (n == "gemm_split_tail") o.gemm_split_tail = value < 0 ? 0 : (value > 2 ? 2 : value);
  else if (n == "compute_units") o.compute_units = value < 1 ? 1 : value;
  else if (n == "scan_lds_pad") o.scan_lds_pad = value < 0 ? -1 : value;
  else if (n == "xcd_run") o.xcd_run = value < 0 ? -1 : value;
  else if (n == "many_totals") o.many_totals = value < 1 ? 65536 : value;
  else if (n == "lookback_poll_limit") o.lookback_poll_limit = value < 0 ? kDefaultPollLimit : (unsigned)value;
  else if (n == "test_mute_partition") o.test_mute_partition = value < 0 ? 0u : (unsigned)value;
  else return fail(TCU_ERR_INVALID_ARG, "tcu_set_option: unknown option " + n);
  return TCU_OK;
}

// the NT template argument of the scan kernels and of the copy probe (wave_ops.hpp: kTileStoreNT)
inline int scan_store_policy() { return options().nontemporal ? options().scan_store_policy : kStoreCached; }

// workspace: where the waits that give up are counted (word 1 of a look-back or single-pass reduction workspace)
inline WaitPolicy wait_policy(unsigned desc_shift, unsigned *workspace) { return WaitPolicy{options().lookback_poll_limit, options().test_mute_partition, desc_shift, workspace ? workspace + 1 : nullptr}; }
// 32-bit words of a look-back workspace: the ticket's line, then one slot of 8 << desc_shift bytes per partition
inline size_t look_back_words(size_t parts, unsigned desc_shift) { return 64 + 2 * ((parts ? parts : 1) << desc_shift); }
// 256 bytes per descriptor while that stays within 4 MiB, closer together for the (slow anyway) launches with more partitions
inline unsigned desc_shift_for(size_t parts) {
  unsigned shift = kDescShift;
  while (shift > 0 && (parts << shift) > ((size_t)1 << 19)) shift--;
  return shift;
}

inline bool is_pow2(size_t x) { return x && !(x & (x - 1)); }
inline int ilog2(size_t x) {
  int l = 0;
  while (x > 1) {
    x >>= 1;
    l++;
  }
  return l;
}
inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

constexpr size_t kMaxGrid = 0x7fffffffu;

struct SegArgs {
  size_t num_segments, segment_size;
  int variant, tiles_per_wave, waves_per_block;
  bool mfma;
};

// Common validation for the segmented entry points.  On success `a` holds defaults
// resolved and *generic says whether only the scalar kernel applies.
inline int validate_segmented(const char *what, const void *in, const void *out, SegArgs &a, bool *generic) {
  *generic = false;
  if (a.segment_size == 0) return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": segment_size must be positive");
  if (a.num_segments != 0 && (in == nullptr || out == nullptr)) return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": null device pointer");
  if (a.num_segments > ((size_t)1 << 62) / a.segment_size) return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": num_segments * segment_size overflows");
  if (a.variant < TCU_VARIANT_AUTO || a.variant > TCU_VARIANT_BLOCK_LDS) return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": unknown variant");
  const int u = a.tiles_per_wave, w = a.waves_per_block;
  if (!(u == 0 || u == 1 || u == 2 || u == 4 || u == 8)) return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": tiles_per_wave must be 0 (default), 1, 2, 4 or 8");
  if (!(w == 0 || w == 1 || w == 2 || w == 4 || w == 8 || w == 16)) return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": waves_per_block must be 0 (default), 1, 2, 4, 8 or 16");
  const size_t S = a.segment_size;
  const bool fast_ok = is_pow2(S) && S >= 16 && aligned16(in) && aligned16(out);
  switch (a.variant) {
    case TCU_VARIANT_AUTO:
      if (!fast_ok) *generic = true;
      break;
    case TCU_VARIANT_MFMA_16:
      if (S != 16) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": segment size must be 16");
      break;
    case TCU_VARIANT_MFMA_256:
      if (S != 256) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": segment size must be 256");
      break;
    case TCU_VARIANT_MFMA_256N:
    case TCU_VARIANT_MFMA_256N_BLOCK:  // the reference registers *_256N_BLOCK from 256 on (src/reduction/seg_wmma_256n_block.cu:242-248)
      if (!is_pow2(S) || S < 256) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": segment size must be a power-of-two multiple of 256");
      break;
    // MFMA_16N_BLOCK (reference *_16N_BLOCK, 16 ... 1024: src/reduction/seg_wmma_16n_block.cu:229-235) and BLOCK_LDS
    // (reference cub::Block*, THREADS * ITEMS from 32 on: src/reduction/seg_cub_block.cu:145-288) take every power
    // of two from 16 on, like the wave families
    default:
      if (!is_pow2(S) || S < 16) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": segment size must be a power of two >= 16");
  }
  if (a.variant != TCU_VARIANT_AUTO && !(aligned16(in) && aligned16(out))) return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": device pointers must be 16-byte aligned");
  a.mfma = a.variant >= TCU_VARIANT_MFMA_16 && a.variant <= TCU_VARIANT_MFMA_256N_BLOCK;
  return TCU_OK;
}

// Launch shapes measured on MI355X (timings in profiles/): for each segment size and element
// count the family and (tiles per wave, waves per block) that moved the most bytes per second.  MFMA and DPP flavours tie within run-to-run noise at every size (the kernels
// are bound by HBM, not by issue slots), so AUTO takes the DPP flavour.
struct Plan {
  bool block;  // block-per-segment kernel
  int u, w;
  unsigned c = 0;  // consecutive blocks per XCD (xcd_run_piece)
  unsigned pad = 0;  // KiB of LDS a block asks for and leaves unused, to cap the blocks per compute unit (block scan: 52 = three, 39 = four)
};
// the run length a launch uses: the option when set, else the plan's (only when the plan's shape is the one launched)
inline unsigned xcd_run_for(const Plan &plan, bool plan_shape) {
  if (options().xcd_run >= 0) return (unsigned)options().xcd_run;
  return plan_shape ? plan.c : 0u;
}
// N = num_segments * S.  The shapes were measured at N = 2^24, 2^26, 2^28 and 2^30 (randomised sweeps over family,
// tiles per wave, waves per block and XCD run length with the outputs of the launches taken in turn;
// profiles/seg_launch_shape_sweeps.md).  From 2^26 elements on one table serves every N but for the entries marked;
// below 2^25 a launch lasts 6-13 us and is bound by how fast blocks start, so fewer and larger blocks win.
// the unused LDS a block scan asks for, in bytes: the option when set, else the plan's (only with the plan's shape)
inline unsigned lds_pad_for(const Plan &plan, bool plan_shape) {
  if (options().scan_lds_pad >= 0) return (unsigned)options().scan_lds_pad * 1024u;
  return plan_shape ? plan.pad * 1024u : 0u;
}
inline Plan auto_plan_reduce(size_t S, size_t N) {
  if (N < ((size_t)1 << 25)) {
    if (S <= 1024) return {false, 2, 1, 128};
    if (S == 2048) return {false, 2, 1, 8};
    if (S == 4096) return {false, 4, 4, 0};
    if (S == 8192) return {false, 8, 1, 512};
    if (S == 16384) return {true, 4, 16, 0};
  }
  if (S <= 512) return {false, 2, 1, 512};
  if (S == 1024) return {true, 2, 1, 64};
  if (S == 2048) return {true, 2, 4, 128};
  if (S == 4096) return {true, 2, 4, 64};
  if (S == 8192) return {true, 2, 8, 0};
  if (S == 16384) return {true, 2, 8, 64};
  if (S == 65536 || S == 131072) return {true, 2, 16, 32};
  if (S == 262144) return {true, 4, 8, 0};
  if (S > 262144) return {true, 2, 8, 0};
  return {true, 1, 8, 0};
}
inline Plan auto_plan_scan(size_t S, size_t N) {
  if (N < ((size_t)1 << 25)) {
    if (S <= 512) return {false, 1, 1, 512};
    if (S == 1024) return {false, 8, 4, 512};
    if (S == 2048) return {false, 8, 8, 8};
    if (S == 4096) return {false, 8, 4, 32};
    if (S == 8192 || S == 16384) return {true, 8, 8, 32};
  }
  if (S <= 512) return {false, 2, 1, 512};
  if (S == 1024) return {true, 1, 1, 128};
  if (S == 2048) return {true, 2, 2, 256};
  // 4096 ... 16384: blocks of 16 KiB with three or four of them on a compute unit (48 - 64 KiB in flight per unit) run
  // 1.5 - 3 % faster than the same or larger blocks at full occupancy (2^28, identical launches back to back: 160.5 /
  // 159.3 / 162.9 us against 162.9 / 164.1 / 166.4; shuffled with other launches 157.3 / 159.1 / 162.7 against 162.9 /
  // 164.0 / 166.6).  Beyond 2^28 elements the two shorter sizes keep their uncapped shapes (2^29 back to back: level
  // or 2 % behind), the longest its capped one up to 2^29 (325.7 against 332.7 us).  At 2^30 the shapes with runs of 8
  // blocks per XCD alternate between 660 and 720 us from launch to launch inside a fixed sequence of launches (which of two
  // input and output buffers a launch gets), those with runs of 32 stay at 670 - 685: 2 tiles x 16 waves, as for 8192
  const size_t G = (size_t)1 << 30;
  if (S == 4096) return N > G / 4 ? Plan{true, 2, 4, 128} : (N <= G / 16 ? Plan{true, 4, 4, 32, 39} : Plan{true, 2, 8, 8, 52});
  if (S == 8192) return N >= G ? Plan{true, 2, 16, 32} : (N > G / 4 ? Plan{true, 2, 8, 32} : (N < G / 4 ? Plan{true, 4, 4, 32, 39} : Plan{true, 4, 4, 8, 39}));
  if (S == 16384) return N >= G ? Plan{true, 2, 16, 32} : Plan{true, 4, 4, 8, 52};
  if (S == 32768) return {true, 8, 8, 16};
  // 65536 and beyond: 8 tiles per wave, 0.72-0.74 against 0.68-0.71 for 4 (N = 2^28); the XCD runs by measurement per size
  if (S == 262144) return {true, 8, 16, 8};
  if (S == 524288) return {true, 8, 16, 0};
  return {true, 8, 16, 32};
}

inline bool is_block_variant(int v) { return v == TCU_VARIANT_MFMA_16N_BLOCK || v == TCU_VARIANT_MFMA_256N_BLOCK || v == TCU_VARIANT_BLOCK_LDS; }
// Default tiles per wave of a wave-kernel launch (segments shorter than a tile).  The reference's *_16N_BLOCK kernels
// give a block 16 segments (src/reduction/kernel.cuh:176-236): here the block's waves then cover at least 16
// segments, i.e. 16 * S / 512 tiles (rounded up to a whole tile per wave, at most 8).
inline int block_family_tiles(int variant, size_t S, int wpb, int otherwise) {
  if (variant != TCU_VARIANT_MFMA_16N_BLOCK) return otherwise;
  const size_t tiles = (16 * S + kTileHalves - 1) / kTileHalves;
  int u = 1;
  while (u < 8 && (size_t)u * wpb < tiles) u *= 2;
  return u;
}

// The launch of a block kernel (seg_*_block_kernel) whose block could hold more tiles than a segment has: a wave
// takes no more tiles than the segment has, the waves form groups of `group` that share a segment each (the
// smallest power of two whose waves cover the segment in one step, at most the block), and the block owns at
// least as many segments as it has groups.  All arguments are powers of two.
struct BlockShape {
  int u;
  unsigned group, spb;
};
inline BlockShape block_shape(size_t tiles_per_seg, int u, int wpb, unsigned spb) {
  while (u > 1 && (size_t)u > tiles_per_seg) u /= 2;
  unsigned group = 1;
  while (group < (unsigned)wpb && (size_t)group * u < tiles_per_seg) group *= 2;
  const unsigned in_flight = (unsigned)wpb / group;
  return {u, group, spb < in_flight ? in_flight : spb};
}

// ----- segmented reduction ----------------------------------------------------------------

template <int LPS_LOG2, int U, bool MFMA>
inline void launch_reduce_small(unsigned grid, unsigned block, void *stream, const half8_t *in, uint16_t *out, size_t n_chunks, size_t nseg, unsigned run) {
  if (options().nontemporal)
    launch(seg_reduce_small_kernel<LPS_LOG2, U, MFMA, true>, grid, block, stream, in, out, n_chunks, nseg, run);
  else
    launch(seg_reduce_small_kernel<LPS_LOG2, U, MFMA, false>, grid, block, stream, in, out, n_chunks, nseg, run);
}
template <int LPS_LOG2, bool MFMA>
inline void launch_reduce_small_u(int u, unsigned grid, unsigned block, void *stream, const half8_t *in, uint16_t *out, size_t n_chunks, size_t nseg, unsigned run) {
  switch (u) {
    case 1: return launch_reduce_small<LPS_LOG2, 1, MFMA>(grid, block, stream, in, out, n_chunks, nseg, run);
    case 2: return launch_reduce_small<LPS_LOG2, 2, MFMA>(grid, block, stream, in, out, n_chunks, nseg, run);
    case 4: return launch_reduce_small<LPS_LOG2, 4, MFMA>(grid, block, stream, in, out, n_chunks, nseg, run);
    default: return launch_reduce_small<LPS_LOG2, 8, MFMA>(grid, block, stream, in, out, n_chunks, nseg, run);
  }
}
template <bool MFMA>
inline void launch_reduce_small_s(int lps_log2, int u, unsigned grid, unsigned block, void *stream, const half8_t *in, uint16_t *out, size_t n_chunks, size_t nseg, unsigned run) {
  switch (lps_log2) {
    case 1: return launch_reduce_small_u<1, MFMA>(u, grid, block, stream, in, out, n_chunks, nseg, run);
    case 2: return launch_reduce_small_u<2, MFMA>(u, grid, block, stream, in, out, n_chunks, nseg, run);
    case 3: return launch_reduce_small_u<3, MFMA>(u, grid, block, stream, in, out, n_chunks, nseg, run);
    case 4: return launch_reduce_small_u<4, MFMA>(u, grid, block, stream, in, out, n_chunks, nseg, run);
    case 5: return launch_reduce_small_u<5, MFMA>(u, grid, block, stream, in, out, n_chunks, nseg, run);
    default: return launch_reduce_small_u<6, MFMA>(u, grid, block, stream, in, out, n_chunks, nseg, run);
  }
}

#define TCU_SWITCH_U_MFMA_NT(KERNEL, u, mfma, nt, ...)                    \
  do {                                                                     \
    const int _k = ((u) == 1 ? 0 : (u) == 2 ? 1 : (u) == 4 ? 2 : 3) * 4 + ((mfma) ? 2 : 0) + ((nt) ? 1 : 0); \
    switch (_k) {                                                          \
      case 0: launch(KERNEL<1, false, false>, __VA_ARGS__); break;         \
      case 1: launch(KERNEL<1, false, true>, __VA_ARGS__); break;          \
      case 2: launch(KERNEL<1, true, false>, __VA_ARGS__); break;          \
      case 3: launch(KERNEL<1, true, true>, __VA_ARGS__); break;           \
      case 4: launch(KERNEL<2, false, false>, __VA_ARGS__); break;         \
      case 5: launch(KERNEL<2, false, true>, __VA_ARGS__); break;          \
      case 6: launch(KERNEL<2, true, false>, __VA_ARGS__); break;          \
      case 7: launch(KERNEL<2, true, true>, __VA_ARGS__); break;           \
      case 8: launch(KERNEL<4, false, false>, __VA_ARGS__); break;         \
      case 9: launch(KERNEL<4, false, true>, __VA_ARGS__); break;          \
      case 10: launch(KERNEL<4, true, false>, __VA_ARGS__); break;         \
      case 11: launch(KERNEL<4, true, true>, __VA_ARGS__); break;          \
      case 12: launch(KERNEL<8, false, false>, __VA_ARGS__); break;        \
      case 13: launch(KERNEL<8, false, true>, __VA_ARGS__); break;         \
      case 14: launch(KERNEL<8, true, false>, __VA_ARGS__); break;         \
      default: launch(KERNEL<8, true, true>, __VA_ARGS__); break;          \
    }                                                                      \
  } while (0)

// the same choice for kernels whose last template argument is fixed by the caller (a store policy)
#define TCU_SWITCH_U_MFMA(KERNEL, u, mfma, LAST, ...)                      \
  do {                                                                     \
    const int _k = ((u) == 1 ? 0 : (u) == 2 ? 1 : (u) == 4 ? 2 : 3) * 2 + ((mfma) ? 1 : 0); \
    switch (_k) {                                                          \
      case 0: launch(KERNEL<1, false, LAST>, __VA_ARGS__); break;          \
      case 1: launch(KERNEL<1, true, LAST>, __VA_ARGS__); break;           \
      case 2: launch(KERNEL<2, false, LAST>, __VA_ARGS__); break;          \
      case 3: launch(KERNEL<2, true, LAST>, __VA_ARGS__); break;           \
      case 4: launch(KERNEL<4, false, LAST>, __VA_ARGS__); break;          \
      case 5: launch(KERNEL<4, true, LAST>, __VA_ARGS__); break;           \
      case 6: launch(KERNEL<8, false, LAST>, __VA_ARGS__); break;          \
      default: launch(KERNEL<8, true, LAST>, __VA_ARGS__); break;          \
    }                                                                      \
  } while (0)

// ----- segments far larger than one block's reach (AUTO only) ---------------------------------
// A block-per-segment kernel leaves the machine idle when there are fewer segments than
// compute units (measured at N = 2^28: reduce 148 us at S = 2^20, 31 ms at S = 2^28; scan
// 353 us at S = 2^21).  From these sizes on a segment is cut into partitions of 65536 halves:
// reduce = partition sums, then one small block per segment adds them in index order; scan =
// the single-pass look-back scan with the look-back stopped at segment starts.  Both need a
// few bytes per partition of temporary device memory, taken in stream order.
constexpr size_t kHugeReduceSegment = (size_t)1 << 20, kHugeScanSegment = (size_t)1 << 21, kHugePartHalves = 65536;
// Below those sizes a block walks a segment by itself, which also loses where the segments are too few to give every
// compute unit one (a block walks 1 MiB in about 40 us whatever the others do: N = 2^26 in segments of 2^19 halves
// reduces in 43.9 us walking and in 24.0 us cut into partitions, N = 2^26 in segments of 2^20 scans in 105 against 61 us),
// and, less, from 2^30 elements on in segments of 2^19 halves and more (reduce 317 against 298 - 307 us, scan 726 against
// 712 and 730 against 704); with 256 segments and more of up to 2^18 halves the walking block is level or ahead.
inline bool is_pow2_size(size_t x) { return x && !(x & (x - 1)); }
inline bool few_long_segments(size_t S, size_t num_segments) { return S >= ((size_t)1 << 17) && num_segments < 256; }
inline bool many_elements_long_segments(size_t S, size_t num_segments) { return S >= ((size_t)1 << 19) && num_segments * S >= ((size_t)1 << 30); }
inline bool reduce_cuts_segments(size_t S, size_t num_segments) { return S >= kHugeReduceSegment || (is_pow2_size(S) && (few_long_segments(S, num_segments) || many_elements_long_segments(S, num_segments))); }
inline bool scan_cuts_segments(size_t S, size_t num_segments) { return S >= kHugeScanSegment || (is_pow2_size(S) && (few_long_segments(S, num_segments) || many_elements_long_segments(S, num_segments))); }

// The partition sums (full-array reduction, segments of 2^20 halves and more) take the launch shape that the
// segmented reduction of 4096-half segments measures fastest: blocks of 4 waves x 2 tiles, every XCD on 128
// consecutive partitions (0.95-0.97 of 8 TB/s at 2^28 / 2^30 halves; blocks of 16 waves x 8 tiles in launch order,
// the shape of the look-back scan, gave 0.83-0.85).  One fp32 partial per 4096 halves.
constexpr int kSumTiles = 2, kSumWaves = 4;
constexpr size_t kSumPartHalves = (size_t)kSumTiles * kSumWaves * kTileHalves;
inline unsigned partition_sums_run() { return options().xcd_run >= 0 ? (unsigned)options().xcd_run : 128u; }
// out[j] = fp16(sum of the pps partials of segment j), j < num_segments.  A block adds up to kSumLevel partials;
// longer rows of partials are first cut into pieces of kSumLevel whose fp32 sums are written behind the partials
// (one block walking 262144 partials takes 21 us, two levels 8 us), so `partials` has room for
// sum_partials_floats(num_segments, pps) floats.
constexpr size_t kSumLevel = 4096;
inline size_t sum_partials_floats(size_t num_segments, size_t pps) {
  const size_t parts = num_segments * pps;
  return pps > 2 * kSumLevel ? parts + num_segments * ((pps + kSumLevel - 1) / kSumLevel) : parts;
}
inline void launch_sum_of_partials(void *stream, float *partials, uint16_t *out, size_t num_segments, size_t pps) {
  const size_t parts = num_segments * pps;
  if (pps > 2 * kSumLevel && pps % kSumLevel == 0) {  // whole pieces per segment: the pieces of all segments in one launch
    float *second = partials + parts;
    const size_t pieces = pps / kSumLevel;
    launch(segment_of_partials_kernel<float>, (unsigned)(num_segments * pieces), 1024u, stream, static_cast<const float *>(partials), second, kSumLevel, parts);
    launch(segment_of_partials_kernel<uint16_t>, (unsigned)num_segments, 1024u, stream, static_cast<const float *>(second), out, pieces, num_segments * pieces);
  } else if (pps > 2 * kSumLevel && num_segments == 1) {
    float *second = partials + parts;
    const size_t pieces = (pps + kSumLevel - 1) / kSumLevel;
    launch(segment_of_partials_kernel<float>, (unsigned)pieces, 1024u, stream, static_cast<const float *>(partials), second, kSumLevel, parts);
    launch(segment_of_partials_kernel<uint16_t>, 1u, 1024u, stream, static_cast<const float *>(second), out, pieces, pieces);
  } else {
    launch(segment_of_partials_kernel<uint16_t>, (unsigned)num_segments, 1024u, stream, static_cast<const float *>(partials), out, pps, parts);
  }
}
inline void launch_partition_sums(bool nt, size_t parts, void *stream, const half8_t *in, float *partials, size_t n_chunks) {
  if (nt)
    launch(partition_sums_kernel<kSumTiles, true>, (unsigned)parts, (unsigned)kSumWaves * 64u, stream, in, partials, n_chunks, partition_sums_run());
  else
    launch(partition_sums_kernel<kSumTiles, false>, (unsigned)parts, (unsigned)kSumWaves * 64u, stream, in, partials, n_chunks, partition_sums_run());
}

inline int seg_reduce_huge(const half8_t *in, uint16_t *out, size_t num_segments, size_t S, bool nt, void *stream) {
  const char *what = "tcu_seg_reduce_f16";
  const size_t pps = S / kSumPartHalves, parts = num_segments * pps;
  if (parts > kMaxGrid) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": grid exceeds the launch limit");
  float *partials = static_cast<float *>(stream_alloc(sum_partials_floats(num_segments, pps) * sizeof(float), stream));
  if (!partials) return fail(TCU_ERR_RUNTIME, std::string(what) + ": no temporary device memory for the partition sums");
  const size_t n_chunks = num_segments * S / 8;
  launch_partition_sums(nt, parts, stream, in, partials, n_chunks);
  launch_sum_of_partials(stream, partials, out, num_segments, pps);
  stream_free(partials, stream);
  return TCU_OK;
}

// Where the partition descriptors of seg_scan_huge live: in stream-ordered temporary memory
// (words == nullptr) or in a buffer the caller of the dispatcher brings (capacity in 32-bit words).
struct ScanScratch {
  unsigned *words = nullptr;
  size_t capacity = 0;
};

inline int seg_scan_huge(const char *what, const half8_t *in, uint4_t *out, uint16_t *totals, size_t num_segments, size_t S, bool nt, void *stream, ScanScratch scratch) {
  const size_t pps = S / kHugePartHalves, parts = num_segments * pps;
  if (parts > kMaxGrid || pps > 0xffffffffu) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": grid exceeds the launch limit");
  // ticket counter, then one 64-bit descriptor per partition, 256 bytes apart where the buffer has the room
  unsigned shift = desc_shift_for(parts);
  unsigned *ws = scratch.words;
  if (ws) {
    while (shift > 0 && look_back_words(parts, shift) > scratch.capacity) shift--;
    if (look_back_words(parts, shift) > scratch.capacity)
      return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": " + std::to_string(parts) + " partitions of 65536 halves exceed the built-in scratch buffer (at most " +
                                           std::to_string((scratch.capacity - 64) / 2) + " partitions, i.e. " + std::to_string((scratch.capacity - 64) / 2 * kHugePartHalves) + " halves per call)");
  }
  const size_t words = look_back_words(parts, shift);
  if (!ws) {
    ws = static_cast<unsigned *>(stream_alloc(words * sizeof(unsigned), stream));
    if (!ws) return fail(TCU_ERR_RUNTIME, std::string(what) + ": no temporary device memory for the partition descriptors");
  }
  const size_t n_chunks = num_segments * S / 8;
  launch(zero_look_back_kernel, (unsigned)((parts + 255) / 256), 256u, stream, ws, parts, shift);
  const int static_order = options().static_order ? 1 : 0;
  if (nt)
    launch(full_scan_kernel<8, false, true>, (unsigned)parts, 1024u, stream, in, out, n_chunks, ws, static_order, (unsigned)pps, totals, wait_policy(shift, ws));
  else
    launch(full_scan_kernel<8, false, false>, (unsigned)parts, 1024u, stream, in, out, n_chunks, ws, static_order, (unsigned)pps, totals, wait_policy(shift, ws));
  if (!scratch.words) stream_free(ws, stream);
  return TCU_OK;
}

inline int seg_reduce_dispatch(const void *d_in, void *d_out, size_t num_segments, size_t segment_size, int variant, int tiles_per_wave, int waves_per_block, void *stream) {
  SegArgs a{num_segments, segment_size, variant, tiles_per_wave, waves_per_block, false};
  bool generic = false;
  if (int rc = validate_segmented("tcu_seg_reduce_f16", d_in, d_out, a, &generic)) return rc;
  if (num_segments == 0) return TCU_OK;
  const size_t S = segment_size, N = num_segments * S;
  const half8_t *in = static_cast<const half8_t *>(d_in);
  uint16_t *out = static_cast<uint16_t *>(d_out);
  const bool nt = options().nontemporal;

  if (generic) {
    const int gw = waves_per_block ? waves_per_block : 4;
    const size_t grid = (num_segments + gw - 1) / gw;
    if (grid > kMaxGrid) return fail(TCU_ERR_UNSUPPORTED, "tcu_seg_reduce_f16: grid exceeds the launch limit");
    launch(seg_reduce_generic_kernel, (unsigned)grid, (unsigned)gw * 64u, stream, static_cast<const uint16_t *>(d_in), out, num_segments, S);
    return TCU_OK;
  }
  if (variant == TCU_VARIANT_AUTO && !tiles_per_wave && !waves_per_block && reduce_cuts_segments(S, num_segments)) return seg_reduce_huge(in, out, num_segments, S, nt, stream);
  const size_t n_chunks = N / 8;
  const Plan plan = auto_plan_reduce(S, N);
  // A segment shorter than a tile cannot be shared by the waves of a block: below 512 halves the block families
  // run the kernels whose waves take whole tiles, at the block's launch shape (waves per block x tiles per wave)
  const bool use_block = S >= kTileHalves && (variant == TCU_VARIANT_AUTO ? plan.block : is_block_variant(variant));
  // explicit families keep their own tuned shape; AUTO and matching families use the plan
  const bool plan_fits = variant == TCU_VARIANT_AUTO || plan.block == use_block;
  const int wpb = waves_per_block ? waves_per_block : (plan_fits ? plan.w : (use_block ? 8 : 4));
  const int u = tiles_per_wave ? tiles_per_wave : (plan_fits ? plan.u : (use_block ? 2 : block_family_tiles(variant, S, wpb, 4)));
  const unsigned block = (unsigned)wpb * 64u;
  const unsigned run = xcd_run_for(plan, plan_fits && u == plan.u && wpb == plan.w);

  if (use_block) {
    const size_t tiles_per_seg = S / kTileHalves;
    // the reference's 16n_block owns 16 segments per block
    const BlockShape shape = block_shape(tiles_per_seg, u, wpb, variant == TCU_VARIANT_MFMA_16N_BLOCK ? 16u : 1u);
    const size_t grid = (num_segments + shape.spb - 1) / shape.spb;
    if (grid > kMaxGrid) return fail(TCU_ERR_UNSUPPORTED, "tcu_seg_reduce_f16: grid exceeds the launch limit");
    TCU_SWITCH_U_MFMA_NT(seg_reduce_block_kernel, shape.u, a.mfma, nt, (unsigned)grid, block, stream, in, out, n_chunks, num_segments, tiles_per_seg, shape.spb, shape.group, run);
    return TCU_OK;
  }
  if (S <= 512) {
    const size_t tiles = (n_chunks + kTileChunks - 1) / kTileChunks;
    const size_t waves = (tiles + u - 1) / u;
    const size_t grid = (waves + wpb - 1) / wpb;
    if (grid > kMaxGrid) return fail(TCU_ERR_UNSUPPORTED, "tcu_seg_reduce_f16: grid exceeds the launch limit");
    const int lps_log2 = ilog2(S) - 3;
    if (a.mfma)
      launch_reduce_small_s<true>(lps_log2, u, (unsigned)grid, block, stream, in, out, n_chunks, num_segments, run);
    else
      launch_reduce_small_s<false>(lps_log2, u, (unsigned)grid, block, stream, in, out, n_chunks, num_segments, run);
    return TCU_OK;
  }
  // S >= 1024: each wave walks max(S, u tiles) of data
  const int tps_log2 = ilog2(S) - 9;
  const size_t tiles_per_seg = (size_t)1 << tps_log2;
  const size_t tiles = num_segments * tiles_per_seg;
  const size_t iters = tiles_per_seg > (size_t)u ? tiles_per_seg / u : 1;
  if (iters > 0xffffffffu) return fail(TCU_ERR_UNSUPPORTED, "tcu_seg_reduce_f16: segment too long for the wave-per-segment kernel; use a block variant");
  const size_t tiles_per_wave_total = iters * u;
  const size_t waves = (tiles + tiles_per_wave_total - 1) / tiles_per_wave_total;
  const size_t grid = (waves + wpb - 1) / wpb;
  if (grid > kMaxGrid) return fail(TCU_ERR_UNSUPPORTED, "tcu_seg_reduce_f16: grid exceeds the launch limit");
  TCU_SWITCH_U_MFMA_NT(seg_reduce_long_kernel, u, a.mfma, nt, (unsigned)grid, block, stream, in, out, n_chunks, num_segments, tps_log2, (unsigned)iters, run);
  return TCU_OK;
}

// ----- segmented reduction over an offsets array ------------------------------------------------

template <typename OFF>
inline int seg_reduce_offsets_typed(const uint16_t *in, uint16_t *out, size_t num_segments, const OFF *begin, const OFF *end, size_t expected, void *stream) {
  const int vector = aligned16(in) ? 1 : 0;
  const bool nt = options().nontemporal;
  // expected length of 2^17 halves and more: several 1024-thread blocks per segment (about
  // 65536 halves each), fp32 partials in stream-ordered temporary memory, then one small
  // block per segment adds them.  (A wave per segment: 158 us at 2^19, 57 ms for one 2^28 segment.)
  if (expected >= ((size_t)1 << 17)) {
    size_t slices = (expected + 65535) / 65536;
    if (slices > 65536) slices = 65536;  // one segment of 2^32 halves
    const size_t blocks = num_segments * slices;
    if (blocks > kMaxGrid) return fail(TCU_ERR_UNSUPPORTED, "tcu_seg_reduce_offsets_f16: grid exceeds the launch limit");
    float *partials = static_cast<float *>(stream_alloc(blocks * sizeof(float), stream));
    if (!partials) return fail(TCU_ERR_RUNTIME, "tcu_seg_reduce_offsets_f16: no temporary device memory for the partial sums");
    if (nt)
      launch(seg_reduce_offsets_sliced_kernel<OFF, true>, (unsigned)blocks, 1024u, stream, in, partials, begin, end, (unsigned)slices, vector);
    else
      launch(seg_reduce_offsets_sliced_kernel<OFF, false>, (unsigned)blocks, 1024u, stream, in, partials, begin, end, (unsigned)slices, vector);
    launch(segment_of_partials_kernel<uint16_t>, (unsigned)num_segments, 1024u, stream, static_cast<const float *>(partials), out, slices, blocks);
    stream_free(partials, stream);
    return TCU_OK;
  }
  // 4096 halves and more expected: a block per segment, about 32 halves per thread (128 to 512 threads, 1024 from 65536 halves on), the
  // result written by the block itself.  N = 2^28 against a wave per segment: S = 4096 76 vs 78.5 us, 16384 77.4 vs
  // 82.7, 65536 78.4 vs 89.5 (2^28 / S long-lived waves fill the chip unevenly); at 2048 the wave is faster (75.5 vs 88)
  if (expected >= 4096) {
    unsigned threads = 128;
    while (threads < 512 && (size_t)threads * 32 < expected) threads *= 2;
    if (expected >= 65536) threads = 1024;  // 1024 threads lose below that (S = 16384: 97 us)
    if (num_segments > kMaxGrid) return fail(TCU_ERR_UNSUPPORTED, "tcu_seg_reduce_offsets_f16: grid exceeds the launch limit");
    if (nt)
      launch(seg_reduce_offsets_sliced_kernel<OFF, true, true>, (unsigned)num_segments, threads, stream, in, reinterpret_cast<float *>(out), begin, end, 1u, vector);
    else
      launch(seg_reduce_offsets_sliced_kernel<OFF, false, true>, (unsigned)num_segments, threads, stream, in, reinterpret_cast<float *>(out), begin, end, 1u, vector);
    return TCU_OK;
  }
  // lanes per segment: about one 128-bit chunk per lane for the expected length, a whole wave when unknown
  int g_log2 = 6;
  if (expected) {
    g_log2 = 1;
    while (g_log2 < 6 && ((size_t)8 << g_log2) < expected) g_log2++;
  }
  // 128 to 512 halves expected: half as many lanes (at most 16), so that a segment takes two to four rounds and a
  // lane has as many loads in flight, while a round still reads 128 or 256 contiguous bytes (N = 2^28, S = 128 /
  // 256 / 512: 82 / 79 / 78 us against 104 / 102 / 102 with one chunk per lane; with 4 or 2 lanes, S = 64 / 32,
  // a round reads half a cache line per segment and the time goes up to 151 / 157 us from 105 / 108)
  if (expected >= 128 && expected <= 512) g_log2 = g_log2 - 1 < 4 ? g_log2 - 1 : 4;
  // one chunk per lane in flight is too little (120 us at N = 2^28): up to 1024 halves expected, a block takes two
  // runs of segments and has the first load of both in flight (107-111 us)
  const int passes = expected && expected <= 1024 ? 2 : 1;  // four passes measure worse (131 us: registers)
  const size_t segs_per_block = ((size_t)256 >> g_log2) * passes;
  const size_t grid = (num_segments + segs_per_block - 1) / segs_per_block;
  if (grid > kMaxGrid) return fail(TCU_ERR_UNSUPPORTED, "tcu_seg_reduce_offsets_f16: grid exceeds the launch limit");
#define TCU_OFFSETS_LAUNCH(GL, NT_, P_) launch(seg_reduce_offsets_kernel<OFF, GL, NT_, P_>, (unsigned)grid, 256u, stream, in, out, num_segments, begin, end, vector)
#define TCU_OFFSETS_CASE(GL)                                                      \
  case GL:                                                                       \
    if (nt) {                                                                    \
      if (passes == 2) TCU_OFFSETS_LAUNCH(GL, true, 2); else TCU_OFFSETS_LAUNCH(GL, true, 1);   \
    } else {                                                                     \
      if (passes == 2) TCU_OFFSETS_LAUNCH(GL, false, 2); else TCU_OFFSETS_LAUNCH(GL, false, 1); \
    }                                                                            \
    break
  switch (g_log2) {
    TCU_OFFSETS_CASE(1);
    TCU_OFFSETS_CASE(2);
    TCU_OFFSETS_CASE(3);
    TCU_OFFSETS_CASE(4);
    TCU_OFFSETS_CASE(5);
    default:
      TCU_OFFSETS_CASE(6);
  }
#undef TCU_OFFSETS_CASE
#undef TCU_OFFSETS_LAUNCH
  return TCU_OK;
}

inline int seg_reduce_offsets_dispatch(const void *d_in, void *d_out, size_t num_segments, const void *d_begin, const void *d_end, int offset_bits, size_t expected, void *stream) {
  const char *what = "tcu_seg_reduce_offsets_f16";
  if (offset_bits != 32 && offset_bits != 64) return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": offset_bits must be 32 or 64");
  if (num_segments == 0) return TCU_OK;
  if (!d_in || !d_out || !d_begin || !d_end) return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": null device pointer");
  if (num_segments > ((size_t)1 << 56)) return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": too many segments");
  const uint16_t *in = static_cast<const uint16_t *>(d_in);
  uint16_t *out = static_cast<uint16_t *>(d_out);
  if (offset_bits == 32) return seg_reduce_offsets_typed(in, out, num_segments, static_cast<const int32_t *>(d_begin), static_cast<const int32_t *>(d_end), expected, stream);
  return seg_reduce_offsets_typed(in, out, num_segments, static_cast<const int64_t *>(d_begin), static_cast<const int64_t *>(d_end), expected, stream);
}

// ----- segmented inclusive prefix sum -------------------------------------------------------

template <int LPS_LOG2, bool MFMA>
inline void launch_scan_wave_u(int u, int nt, unsigned grid, unsigned block, void *stream, const half8_t *in, uint4_t *out, uint16_t *totals, size_t n_chunks, size_t nseg, int tps_log2,
                               unsigned iters, unsigned run) {
#define TCU_SCAN_CASE(UU)                                                                                                                         \
  if (nt == kStoreAlternate)                                                                                                                      \
    launch(seg_scan_wave_kernel<LPS_LOG2, UU, MFMA, kStoreAlternate>, grid, block, stream, in, out, totals, n_chunks, nseg, tps_log2, iters, run); \
  else if (nt == kStoreStream)                                                                                                                    \
    launch(seg_scan_wave_kernel<LPS_LOG2, UU, MFMA, kStoreStream>, grid, block, stream, in, out, totals, n_chunks, nseg, tps_log2, iters, run);    \
  else                                                                                                                                            \
    launch(seg_scan_wave_kernel<LPS_LOG2, UU, MFMA, kStoreCached>, grid, block, stream, in, out, totals, n_chunks, nseg, tps_log2, iters, run);    \
  return
  switch (u) {
    case 1: TCU_SCAN_CASE(1);
    case 2: TCU_SCAN_CASE(2);
    case 4: TCU_SCAN_CASE(4);
    default: TCU_SCAN_CASE(8);
  }
#undef TCU_SCAN_CASE
}
template <bool MFMA>
inline void launch_scan_wave_s(int lps_log2, int u, int nt, unsigned grid, unsigned block, void *stream, const half8_t *in, uint4_t *out, uint16_t *totals, size_t n_chunks, size_t nseg,
                               int tps_log2, unsigned iters, unsigned run) {
  switch (lps_log2) {
    case 1: return launch_scan_wave_u<1, MFMA>(u, nt, grid, block, stream, in, out, totals, n_chunks, nseg, tps_log2, iters, run);
    case 2: return launch_scan_wave_u<2, MFMA>(u, nt, grid, block, stream, in, out, totals, n_chunks, nseg, tps_log2, iters, run);
    case 3: return launch_scan_wave_u<3, MFMA>(u, nt, grid, block, stream, in, out, totals, n_chunks, nseg, tps_log2, iters, run);
    case 4: return launch_scan_wave_u<4, MFMA>(u, nt, grid, block, stream, in, out, totals, n_chunks, nseg, tps_log2, iters, run);
    case 5: return launch_scan_wave_u<5, MFMA>(u, nt, grid, block, stream, in, out, totals, n_chunks, nseg, tps_log2, iters, run);
    default: return launch_scan_wave_u<6, MFMA>(u, nt, grid, block, stream, in, out, totals, n_chunks, nseg, tps_log2, iters, run);
  }
}

inline int seg_scan_dispatch(const void *d_in, void *d_out, void *d_totals, size_t num_segments, size_t segment_size, int variant, int tiles_per_wave, int waves_per_block, void *stream,
                             const char *what = "tcu_seg_scan_f16", ScanScratch scratch = ScanScratch{}) {
  SegArgs a{num_segments, segment_size, variant, tiles_per_wave, waves_per_block, false};
  bool generic = false;
  if (int rc = validate_segmented(what, d_in, d_out, a, &generic)) return rc;
  if (num_segments == 0) return TCU_OK;
  const size_t S = segment_size, N = num_segments * S;
  const half8_t *in = static_cast<const half8_t *>(d_in);
  uint4_t *out = static_cast<uint4_t *>(d_out);
  uint16_t *totals = static_cast<uint16_t *>(d_totals);
  const bool nt = options().nontemporal;
  const int policy = scan_store_policy();

  if (generic) {
    const int gw = waves_per_block ? waves_per_block : 4;
    const size_t grid = (num_segments + gw - 1) / gw;
    if (grid > kMaxGrid) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": grid exceeds the launch limit");
    launch(seg_scan_generic_kernel, (unsigned)grid, (unsigned)gw * 64u, stream, static_cast<const uint16_t *>(d_in), static_cast<uint16_t *>(d_out), totals, num_segments, S);
    return TCU_OK;
  }
  if (variant == TCU_VARIANT_AUTO && !tiles_per_wave && !waves_per_block && scan_cuts_segments(S, num_segments)) return seg_scan_huge(what, in, out, totals, num_segments, S, nt, stream, scratch);
  const size_t n_chunks = N / 8;
  const Plan plan = auto_plan_scan(S, N);
  const bool use_block = S >= kTileHalves && (variant == TCU_VARIANT_AUTO ? plan.block : is_block_variant(variant));  // as in the reduction
  const bool plan_fits = variant == TCU_VARIANT_AUTO || plan.block == use_block;
  const int wpb = waves_per_block ? waves_per_block : (plan_fits ? plan.w : (use_block ? 4 : 1));
  const int u = tiles_per_wave ? tiles_per_wave : (plan_fits ? plan.u : (use_block ? 4 : block_family_tiles(variant, S, wpb, 4)));
  const unsigned block = (unsigned)wpb * 64u;
  const unsigned run = xcd_run_for(plan, plan_fits && u == plan.u && wpb == plan.w);

  if (use_block) {
    const size_t tiles_per_seg = S / kTileHalves;
    const BlockShape shape = block_shape(tiles_per_seg, u, wpb, variant == TCU_VARIANT_MFMA_16N_BLOCK ? 16u : 1u);
    const size_t grid = (num_segments + shape.spb - 1) / shape.spb;
    if (grid > kMaxGrid) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": grid exceeds the launch limit");
    next_launch_lds_pad() = lds_pad_for(plan, plan_fits && u == plan.u && wpb == plan.w);
    if (policy == kStoreStream)
      TCU_SWITCH_U_MFMA(seg_scan_block_kernel, shape.u, a.mfma, kStoreStream, (unsigned)grid, block, stream, in, out, totals, n_chunks, num_segments, tiles_per_seg, shape.spb, shape.group, run);
    else if (policy == kStoreAlternate)
      TCU_SWITCH_U_MFMA(seg_scan_block_kernel, shape.u, a.mfma, kStoreAlternate, (unsigned)grid, block, stream, in, out, totals, n_chunks, num_segments, tiles_per_seg, shape.spb, shape.group, run);
    else
      TCU_SWITCH_U_MFMA(seg_scan_block_kernel, shape.u, a.mfma, kStoreCached, (unsigned)grid, block, stream, in, out, totals, n_chunks, num_segments, tiles_per_seg, shape.spb, shape.group, run);
    return TCU_OK;
  }
  int lps_log2, tps_log2 = 0;
  size_t iters = 1;
  const size_t tiles = (n_chunks + kTileChunks - 1) / kTileChunks;
  if (S < 512) {
    lps_log2 = ilog2(S) - 3;
  } else {
    lps_log2 = 6;
    tps_log2 = ilog2(S) - 9;
    const size_t tiles_per_seg = (size_t)1 << tps_log2;
    iters = tiles_per_seg > (size_t)u ? tiles_per_seg / u : 1;
    if (iters > 0xffffffffu) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": segment too long for the wave-per-segment kernel; use a block variant");
  }
  const size_t per_wave = iters * u;
  const size_t waves = (tiles + per_wave - 1) / per_wave;
  const size_t grid = (waves + wpb - 1) / wpb;
  if (grid > kMaxGrid) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": grid exceeds the launch limit");
  if (a.mfma)
    launch_scan_wave_s<true>(lps_log2, u, policy, (unsigned)grid, block, stream, in, out, totals, n_chunks, num_segments, tps_log2, (unsigned)iters, run);
  else
    launch_scan_wave_s<false>(lps_log2, u, policy, (unsigned)grid, block, stream, in, out, totals, n_chunks, num_segments, tps_log2, (unsigned)iters, run);
  return TCU_OK;
}

// ----- segmented inclusive prefix sum over an offsets array -----------------------------------

// rounds of 1024 chunks a slice of the chained kernel keeps in registers: 8 for the 65536 halves a slice is cut to,
// one more for segments that start off a chunk boundary or run up to an eighth over the expected length
constexpr int kOffsetsChainRounds = 9;

template <typename OFF>
inline int seg_scan_offsets_typed(const uint16_t *in, uint16_t *out, size_t num_segments, const OFF *begin, const OFF *end, size_t expected, void *stream) {
  // expected length of 1024 halves and more: a block per run of at most about 65536 halves of one
  // segment, one 128-bit chunk per thread and round (64 ... 1024 threads); with more than one run
  // per segment the runs' sums are taken first (fp32, stream-ordered temporary memory) and turned
  // into carry-ins.  (Groups of 16 lanes walking a segment: 226-313 us for 2048 ... 32768 at
  // N = 2^28 and milliseconds beyond, against 175-200 and 290 us this way.)
  if (expected >= 1024) {
    const int vec = aligned16(in) && aligned16(out) ? 1 : 0;
    const bool ntl = options().nontemporal;
    size_t slices = (expected + 65535) / 65536;
    if (slices > 65536) slices = 65536;  // one segment of 2^32 halves
    // two to four rounds per block measure best (N = 2^28: S = 1024 with 64 threads 165 us, 180 with groups of 16
    // lanes; S = 2048 with 128 threads 164, with 256 184; S = 4096 with 128 threads 167.5, with 256 173)
    const unsigned threads = expected < 2048 ? 64 : expected < 8192 ? 128 : expected <= 8192 ? 512 : 1024;
    const size_t blocks = num_segments * slices;
    if (blocks > kMaxGrid) return fail(TCU_ERR_UNSUPPORTED, "tcu_seg_scan_offsets_f16: grid exceeds the launch limit");
    if (slices > 1 && options().offsets_scan_chain) {
      // one pass: the slices of a segment meet through decoupled look-back (descriptors in stream-ordered temporary memory)
      const unsigned shift = desc_shift_for(blocks);
      const size_t words = look_back_words(blocks, shift);
      unsigned *ws = static_cast<unsigned *>(stream_alloc(words * sizeof(unsigned), stream));
      if (!ws) return fail(TCU_ERR_RUNTIME, "tcu_seg_scan_offsets_f16: no temporary device memory for the partition descriptors");
      launch(zero_look_back_kernel, (unsigned)((blocks + 255) / 256), 256u, stream, ws, blocks, shift);
      const int so = options().static_order ? 1 : 0;
      if (ntl)
        launch(seg_scan_offsets_chained_kernel<OFF, kOffsetsChainRounds, true>, (unsigned)blocks, 1024u, stream, in, out, begin, end, (unsigned)slices, vec, ws, so, wait_policy(shift, ws));
      else
        launch(seg_scan_offsets_chained_kernel<OFF, kOffsetsChainRounds, false>, (unsigned)blocks, 1024u, stream, in, out, begin, end, (unsigned)slices, vec, ws, so, wait_policy(shift, ws));
      stream_free(ws, stream);
      return TCU_OK;
    }
    float *sums = nullptr;
    if (slices > 1) {
      sums = static_cast<float *>(stream_alloc(blocks * sizeof(float), stream));
      if (!sums) return fail(TCU_ERR_RUNTIME, "tcu_seg_scan_offsets_f16: no temporary device memory for the slice sums");
      if (ntl)
        launch(seg_scan_offsets_slice_sums_kernel<OFF, true>, (unsigned)blocks, threads, stream, in, sums, begin, end, (unsigned)slices, vec);
      else
        launch(seg_scan_offsets_slice_sums_kernel<OFF, false>, (unsigned)blocks, threads, stream, in, sums, begin, end, (unsigned)slices, vec);
      launch(slice_prefix_kernel, (unsigned)num_segments, 64u, stream, sums, (unsigned)slices);
    }
    if (ntl)
      launch(seg_scan_offsets_sliced_kernel<OFF, true>, (unsigned)blocks, threads, stream, in, out, static_cast<const float *>(sums), begin, end, (unsigned)slices, vec);
    else
      launch(seg_scan_offsets_sliced_kernel<OFF, false>, (unsigned)blocks, threads, stream, in, out, static_cast<const float *>(sums), begin, end, (unsigned)slices, vec);
    if (sums) stream_free(sums, stream);
    return TCU_OK;
  }
  // lanes per segment: about one 128-bit chunk per lane and round for the expected length, at most 16
  int g_log2 = 4;
  if (expected) {
    g_log2 = 1;
    while (g_log2 < 4 && ((size_t)8 << g_log2) < expected) g_log2++;
  }
  // 65 to 128 halves expected: 8 lanes and two rounds instead of 16 and one (N = 2^28, S = 128: 168 vs 174 us;
  // fewer lanes lose at every other length: half a cache line per segment and round, or too many rounds)
  if (expected > 64 && expected <= 128) g_log2 = 3;
  const size_t threads = num_segments << g_log2;
  const size_t grid = (threads + 255) / 256;
  if (grid > kMaxGrid) return fail(TCU_ERR_UNSUPPORTED, "tcu_seg_scan_offsets_f16: grid exceeds the launch limit");
  const int vector = aligned16(in) && aligned16(out) ? 1 : 0;
  const bool nt = options().nontemporal;
#define TCU_OFFSETS_CASE(GL)                                                                                                          \
  case GL:                                                                                                                           \
    if (nt)                                                                                                                          \
      launch(seg_scan_offsets_kernel<OFF, GL, true>, (unsigned)grid, 256u, stream, in, out, num_segments, begin, end, vector);        \
    else                                                                                                                             \
      launch(seg_scan_offsets_kernel<OFF, GL, false>, (unsigned)grid, 256u, stream, in, out, num_segments, begin, end, vector);       \
    break
  switch (g_log2) {
    TCU_OFFSETS_CASE(1);
    TCU_OFFSETS_CASE(2);
    TCU_OFFSETS_CASE(3);
    default:
      TCU_OFFSETS_CASE(4);
  }
#undef TCU_OFFSETS_CASE
  return TCU_OK;
}

inline int seg_scan_offsets_dispatch(const void *d_in, void *d_out, size_t num_segments, const void *d_begin, const void *d_end, int offset_bits, size_t expected, void *stream) {
  const char *what = "tcu_seg_scan_offsets_f16";
  if (offset_bits != 32 && offset_bits != 64) return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": offset_bits must be 32 or 64");
  if (num_segments == 0) return TCU_OK;
  if (!d_in || !d_out || !d_begin || !d_end) return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": null device pointer");
  if (num_segments > ((size_t)1 << 56)) return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": too many segments");
  const uint16_t *in = static_cast<const uint16_t *>(d_in);
  uint16_t *out = static_cast<uint16_t *>(d_out);
  if (offset_bits == 32) return seg_scan_offsets_typed(in, out, num_segments, static_cast<const int32_t *>(d_begin), static_cast<const int32_t *>(d_end), expected, stream);
  return seg_scan_offsets_typed(in, out, num_segments, static_cast<const int64_t *>(d_begin), static_cast<const int64_t *>(d_end), expected, stream);
}

inline int add_partial_sums_dispatch(void *d_out, const void *d_ps, size_t num_segments, size_t segment_size, void *stream, bool shifted = false) {
  if (segment_size == 0) return fail(TCU_ERR_INVALID_ARG, "tcu_add_partial_sums_f16: segment_size must be positive");
  if (num_segments == 0) return TCU_OK;
  if (!d_out || !d_ps) return fail(TCU_ERR_INVALID_ARG, "tcu_add_partial_sums_f16: null device pointer");
  const size_t n = num_segments * segment_size;
  if (is_pow2(segment_size) && segment_size >= 8 && aligned16(d_out)) {
    const size_t n_chunks = n / 8;
    const size_t grid = (n_chunks + 255) / 256;
    if (grid > kMaxGrid) return fail(TCU_ERR_UNSUPPORTED, "tcu_add_partial_sums_f16: grid exceeds the launch limit");
    if (options().nontemporal)
      launch(add_partial_sums_kernel<true>, (unsigned)grid, 256u, stream, static_cast<uint4_t *>(d_out), static_cast<const uint16_t *>(d_ps), n_chunks, ilog2(segment_size) - 3, shifted ? 1 : 0);
    else
      launch(add_partial_sums_kernel<false>, (unsigned)grid, 256u, stream, static_cast<uint4_t *>(d_out), static_cast<const uint16_t *>(d_ps), n_chunks, ilog2(segment_size) - 3, shifted ? 1 : 0);
  } else {
    const size_t grid = (n + 255) / 256;
    if (grid > kMaxGrid) return fail(TCU_ERR_UNSUPPORTED, "tcu_add_partial_sums_f16: grid exceeds the launch limit");
    launch(add_partial_sums_generic_kernel, (unsigned)grid, 256u, stream, static_cast<uint16_t *>(d_out), static_cast<const uint16_t *>(d_ps), n, segment_size, shifted ? 1 : 0);
  }
  return TCU_OK;
}

// ----- full-array reduction / prefix sum ------------------------------------------------------

constexpr size_t kWorkspaceAlign = 256;
inline size_t round_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

struct FullPlan {
  int u, wpb;
  size_t part_halves;  // halves per block step / partition
};
// segment_size = halves one block takes per step (0 = default); must be wpb * u * 512 with u in {1,2,4,8}
inline int plan_full(const char *what, size_t segment_size, int waves_per_block, size_t default_part, FullPlan *p) {
  int wpb = waves_per_block ? waves_per_block : 4;
  if (!(wpb == 1 || wpb == 2 || wpb == 4 || wpb == 8 || wpb == 16)) return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": waves_per_block must be 0 (default), 1, 2, 4, 8 or 16");
  size_t part = segment_size ? segment_size : default_part;
  if (!is_pow2(part) || part < (size_t)wpb * 512) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": segment_size must be a power of two >= 512 * waves_per_block");
  size_t u = part / ((size_t)wpb * 512);
  while (u > 8 && wpb < 16) {  // more data per block than 8 tiles per wave: widen the block
    wpb *= 2;
    u /= 2;
  }
  if (u > 8) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": segment_size too large (at most 65536)");
  p->u = (int)u;
  p->wpb = wpb;
  p->part_halves = part;
  return TCU_OK;
}

inline int full_reduce_dispatch(const void *d_in, void *d_out, size_t n, void *d_ws, size_t *ws_bytes, int strategy, size_t segment_size, int waves_per_block, void *stream) {
  const char *what = "tcu_full_reduce_f16";
  if (!ws_bytes) return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": workspace_bytes must not be null");
  const bool mfma = (strategy & TCU_FULL_MFMA) != 0;
  strategy &= ~TCU_FULL_MFMA;
  if (strategy < TCU_FULL_AUTO || strategy > TCU_FULL_MULTI_KERNEL) return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": unknown strategy");
  // AUTO with the default partition: partition sums, then one block adds them
  const bool two_level = strategy == TCU_FULL_AUTO && segment_size == 0 && waves_per_block == 0 && !mfma;
  if (strategy == TCU_FULL_AUTO) strategy = TCU_FULL_SINGLE_PASS;
  const bool nt = options().nontemporal;
  if (strategy == TCU_FULL_SINGLE_PASS) {
    FullPlan p;
    if (int rc = plan_full(what, segment_size, waves_per_block ? waves_per_block : 16, 65536, &p)) return rc;
    const bool vec = n % 8 == 0 && aligned16(d_in);
    const size_t n_chunks = n / 8;
    const size_t n_tiles = (n_chunks + kTileChunks - 1) / kTileChunks;
    size_t grid = (n_tiles + (size_t)p.wpb * p.u - 1) / ((size_t)p.wpb * p.u);
    if (grid == 0) grid = 1;
    const size_t groups = (grid + kFullReduceGroup - 1) / kFullReduceGroup;
    const size_t counter_words = 64 + ((groups + 1) & ~(size_t)1);
    const size_t words = counter_words + 2 * (grid + groups);
    // the two-launch form keeps one float per 4096 halves in the workspace
    const size_t sum_parts = (n + kSumPartHalves - 1) / kSumPartHalves;
    const size_t sum_floats = sum_partials_floats(1, sum_parts ? sum_parts : 1);
    const size_t need = round_up(two_level && sum_floats > words ? 4 * sum_floats : 4 * words, kWorkspaceAlign);
    if (!d_ws) {
      *ws_bytes = need;
      return TCU_OK;
    }
    if (*ws_bytes < need) return fail(TCU_ERR_WORKSPACE, std::string(what) + ": workspace too small");
    if (!d_out || (n && !d_in)) return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": null device pointer");
    if (!vec) {
      // odd sizes: one block over scalar loads
      launch(sum_f16_kernel, 1u, 1024u, stream, static_cast<const uint16_t *>(d_in), static_cast<uint16_t *>(d_out), n);
      return TCU_OK;
    }
    if (grid > kMaxGrid) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": grid exceeds the launch limit");
    if (two_level) {
      if (sum_parts > kMaxGrid) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": grid exceeds the launch limit");
      float *partials = static_cast<float *>(d_ws);
      launch_partition_sums(nt, sum_parts ? sum_parts : 1, stream, static_cast<const half8_t *>(d_in), partials, n_chunks);
      launch_sum_of_partials(stream, partials, static_cast<uint16_t *>(d_out), 1, sum_parts ? sum_parts : 1);
      return TCU_OK;
    }
    unsigned *ws = static_cast<unsigned *>(d_ws);
    launch(zero_words_kernel, (unsigned)((words + 255) / 256), 256u, stream, ws, words);
    TCU_SWITCH_U_MFMA_NT(full_reduce_kernel, p.u, mfma, nt, (unsigned)grid, (unsigned)p.wpb * 64u, stream, static_cast<const half8_t *>(d_in), static_cast<uint16_t *>(d_out), n_chunks, ws, wait_policy(0, ws));
    return TCU_OK;
  }
  // the reference's two-kernel sequence: segmented reduction into fp16 totals, then a sum of the totals
  const size_t S = segment_size ? segment_size : 2048;
  if (!is_pow2(S) || S < 16) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": segment_size must be a power of two >= 16");
  if (n % S != 0) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": num_elements must be a multiple of segment_size");
  const size_t nseg = n / S;
  // The second step (the reference calls cub::DeviceReduce::Sum on the totals, src/reduction/wmma_2kers.cu:63-88): one block adds
  // fewer than `many_totals` totals (option, 65536); beyond that the totals go through the two-launch partition sums, whose partials lie behind them.
  const size_t totals_bytes = round_up(2 * (nseg ? nseg : 1), kWorkspaceAlign);
  const bool nested = nseg >= (size_t)options().many_totals;
  size_t nested_bytes = 0;
  if (nested)
    if (int rc = full_reduce_dispatch(nullptr, nullptr, nseg, nullptr, &nested_bytes, TCU_FULL_AUTO, 0, 0, nullptr)) return rc;
  const size_t need = totals_bytes + nested_bytes;
  if (!d_ws) {
    *ws_bytes = need;
    return TCU_OK;
  }
  if (*ws_bytes < need) return fail(TCU_ERR_WORKSPACE, std::string(what) + ": workspace too small");
  if (!d_out || (n && !d_in)) return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": null device pointer");
  if (int rc = seg_reduce_dispatch(d_in, d_ws, nseg, S, S == 16 ? TCU_VARIANT_MFMA_16 : TCU_VARIANT_MFMA_16N, 0, waves_per_block, stream)) return rc;  // the reference's sequence is built on its WMMA kernels
  if (nested) return full_reduce_dispatch(d_ws, d_out, nseg, static_cast<char *>(d_ws) + totals_bytes, &nested_bytes, TCU_FULL_AUTO, 0, 0, stream);
  launch(sum_f16_kernel, 1u, 1024u, stream, static_cast<const uint16_t *>(d_ws), static_cast<uint16_t *>(d_out), nseg);
  return TCU_OK;
}

inline int full_scan_dispatch(const void *d_in, void *d_out, size_t n, void *d_ws, size_t *ws_bytes, int strategy, size_t segment_size, int waves_per_block, void *stream) {
  const char *what = "tcu_full_scan_f16";
  if (!ws_bytes) return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": workspace_bytes must not be null");
  const bool mfma = (strategy & TCU_FULL_MFMA) != 0;
  strategy &= ~TCU_FULL_MFMA;
  if (strategy < TCU_FULL_AUTO || strategy > TCU_FULL_MULTI_KERNEL) return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": unknown strategy");
  // AUTO with the default partition: the kernel that parks 4 more tiles per wave in LDS, against the one that holds its tiles in registers only: 20.7 against 21.7 us at 2^24
  // elements, 61.2 against 62.1 at 2^26, 104.4 against 106.5 at 2^27, but 200.7 against 193.5 at 2^28, 381 against 366 at 2^29 and 733 against 711 at 2^30 (since a look-back
  // poll repeats only the reads that found nothing, the register kernel gained 3.5 % and the other 1 %), so up to 2^27
  const bool lds_pays = options().scan_lds_tiles < 0 ? n <= ((size_t)1 << 27) : options().scan_lds_tiles != 0;
  const bool lds_held = strategy == TCU_FULL_AUTO && segment_size == 0 && waves_per_block == 0 && lds_pays && !mfma;
  if (strategy == TCU_FULL_AUTO) strategy = TCU_FULL_SINGLE_PASS;
  const bool nt = options().nontemporal;
  if (strategy == TCU_FULL_SINGLE_PASS) {
    FullPlan p;
    if (int rc = plan_full(what, segment_size, waves_per_block ? waves_per_block : 16, 65536, &p)) return rc;
    if (n % 8 != 0 || !aligned16(d_in) || !aligned16(d_out)) {
      if (!d_ws) {
        *ws_bytes = kWorkspaceAlign;
        return TCU_OK;
      }
      if (!n) return TCU_OK;
      if (!d_in || !d_out) return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": null device pointer");
      launch(seg_scan_generic_kernel, 1u, 64u, stream, static_cast<const uint16_t *>(d_in), static_cast<uint16_t *>(d_out), static_cast<uint16_t *>(nullptr), (size_t)1, n);
      return TCU_OK;
    }
    const size_t n_chunks = n / 8;
    const size_t n_tiles = (n_chunks + kTileChunks - 1) / kTileChunks;
    const size_t parts = (n_tiles + (size_t)p.wpb * p.u - 1) / ((size_t)p.wpb * p.u);
    const unsigned shift = desc_shift_for(parts);
    const size_t need = round_up(4 * look_back_words(parts, shift), kWorkspaceAlign);
    if (!d_ws) {
      *ws_bytes = need;
      return TCU_OK;
    }
    if (*ws_bytes < need) return fail(TCU_ERR_WORKSPACE, std::string(what) + ": workspace too small");
    if (!n) return TCU_OK;
    if (!d_in || !d_out) return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": null device pointer");
    if (parts > kMaxGrid) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": grid exceeds the launch limit");
    unsigned *ws = static_cast<unsigned *>(d_ws);
    launch(zero_look_back_kernel, (unsigned)((parts + 255) / 256), 256u, stream, ws, parts, shift);
    if (lds_held) {  // partitions of 16 x 12 tiles: fewer than `parts`, same workspace layout
      const size_t big_parts = (n_tiles + 16 * 12 - 1) / (16 * 12);
      if (nt)
        launch(full_scan_lds_kernel<8, 4, true>, (unsigned)big_parts, 1024u, stream, static_cast<const half8_t *>(d_in), static_cast<uint4_t *>(d_out), n_chunks, ws, options().static_order ? 1 : 0, wait_policy(shift, ws));
      else
        launch(full_scan_lds_kernel<8, 4, false>, (unsigned)big_parts, 1024u, stream, static_cast<const half8_t *>(d_in), static_cast<uint4_t *>(d_out), n_chunks, ws, options().static_order ? 1 : 0, wait_policy(shift, ws));
      return TCU_OK;
    }
    TCU_SWITCH_U_MFMA_NT(full_scan_kernel, p.u, mfma, nt, (unsigned)parts, (unsigned)p.wpb * 64u, stream, static_cast<const half8_t *>(d_in), static_cast<uint4_t *>(d_out), n_chunks, ws, options().static_order ? 1 : 0, 0u, static_cast<uint16_t *>(nullptr), wait_policy(shift, ws));
    return TCU_OK;
  }
  // the reference's three-kernel sequence: segmented scan + totals, exclusive scan of the totals, add
  const size_t S = segment_size ? segment_size : 2048;
  if (!is_pow2(S) || S < 256) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": segment_size must be a power-of-two multiple of 256");
  if (n % S != 0) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": num_elements must be a multiple of segment_size");
  const size_t nseg = n / S;
  // The step in the middle (the reference calls cub::DeviceScan::ExclusiveSum on the totals, src/prefixsum/wmma_3kers.cu:60-82):
  // one block walks fewer than `many_totals` totals (option, 65536); beyond that the totals are scanned in place by the single-pass kernel
  // (inclusive sums; the third kernel then reads them one segment back), which needs its descriptors behind the totals.
  const size_t totals_bytes = round_up(2 * (nseg ? nseg : 1), kWorkspaceAlign);
  const bool nested = nseg >= (size_t)options().many_totals && nseg % 8 == 0;
  size_t nested_bytes = 0;
  if (nested)
    if (int rc = full_scan_dispatch(nullptr, nullptr, nseg, nullptr, &nested_bytes, TCU_FULL_AUTO, 0, 0, nullptr)) return rc;
  const size_t need = totals_bytes + nested_bytes;
  if (!d_ws) {
    *ws_bytes = need;
    return TCU_OK;
  }
  if (*ws_bytes < need) return fail(TCU_ERR_WORKSPACE, std::string(what) + ": workspace too small");
  if (!n) return TCU_OK;
  if (!d_in || !d_out) return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": null device pointer");
  if (int rc = seg_scan_dispatch(d_in, d_out, d_ws, nseg, S, TCU_VARIANT_MFMA_256N, 0, waves_per_block, stream)) return rc;
  if (nested) {
    if (int rc = full_scan_dispatch(d_ws, d_ws, nseg, static_cast<char *>(d_ws) + totals_bytes, &nested_bytes, TCU_FULL_AUTO, 0, 0, stream)) return rc;
    return add_partial_sums_dispatch(d_out, d_ws, nseg, S, stream, true);
  }
  launch(exclusive_scan_f16_kernel, 1u, 1024u, stream, static_cast<uint16_t *>(d_ws), nseg);
  return add_partial_sums_dispatch(d_out, d_ws, nseg, S, stream);
}

// ----- segments given by a key array ---------------------------------------------------------------

constexpr int kByKeyTiles = 4, kByKeyWaves = 16;                                   // per wave / per block
constexpr size_t kByKeyPartition = (size_t)kByKeyTiles * kByKeyWaves * kTileHalves;  // elements per block

template <typename KEY>
inline int by_key_typed(const char *what, bool reduce, const void *d_keys, const void *d_in, void *d_keys_out, void *d_out, void *d_num_runs, size_t n, void *d_ws, size_t *ws_bytes, void *stream) {
  if (!ws_bytes) return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": workspace_bytes must not be null");
  if (n >= ((size_t)1 << 32)) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": at most 2^32 - 1 elements (runs are counted in 32 bits)");
  const size_t parts = (n + kByKeyPartition - 1) / kByKeyPartition;
  const unsigned shift = desc_shift_for(parts) ? desc_shift_for(parts) : 1;  // a slot holds the value and the count descriptor: at least 16 bytes
  const size_t words = look_back_words(parts, shift);
  // the reduction's workspace serves either of its forms (the option may change between the query and the call)
  const KeyReduceLayout lay = key_reduce_layout(n, sizeof(KEY));
  const size_t need = round_up(reduce && lay.total > 4 * words ? lay.total : 4 * words, kWorkspaceAlign);
  if (!d_ws) {
    *ws_bytes = need;
    return TCU_OK;
  }
  if (*ws_bytes < need) return fail(TCU_ERR_WORKSPACE, std::string(what) + ": workspace too small");
  if (n == 0) {
    if (reduce && d_num_runs) launch(zero_words_kernel, 1u, 256u, stream, static_cast<unsigned *>(d_num_runs), (size_t)2);
    return TCU_OK;
  }
  if (!d_keys || !d_in || !d_out) return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": null device pointer");
  if (!aligned16(d_keys) || !aligned16(d_in) || (!reduce && !aligned16(d_out))) return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": keys, values and the scan's output must be 16-byte aligned");
  if ((reinterpret_cast<uintptr_t>(d_out) & 1u) || (reinterpret_cast<uintptr_t>(d_keys_out) & (sizeof(KEY) - 1)) || (reinterpret_cast<uintptr_t>(d_num_runs) & 7u))
    return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": misaligned output pointer");
  if (reduce && !options().by_key_reduce_chain) {
    if (!aligned16(d_ws)) return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": the workspace must be 16-byte aligned");
    char *w = static_cast<char *>(d_ws);
    unsigned long long *bits = reinterpret_cast<unsigned long long *>(w + lay.bits_at);
    KEY *list = d_keys_out ? reinterpret_cast<KEY *>(w + lay.list_at) : nullptr;
    unsigned *counts = reinterpret_cast<unsigned *>(w + lay.counts_at), *gprefix = reinterpret_cast<unsigned *>(w + lay.gprefix_at),
             *gflag = reinterpret_cast<unsigned *>(w + lay.gflag_at);
    float *lead = reinterpret_cast<float *>(w + lay.lead_at), *tail = reinterpret_cast<float *>(w + lay.tail_at), *gtail = reinterpret_cast<float *>(w + lay.gtail_at);
    const unsigned waves = options().by_key_waves > 0 ? (unsigned)options().by_key_waves : 1u;
    const size_t blocks = (lay.parts + waves - 1) / waves;
    if (blocks > kMaxGrid) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": grid exceeds the launch limit");
    const unsigned run = options().xcd_run >= 0 ? (unsigned)options().xcd_run : 0u;
    const unsigned group_blocks = (unsigned)((lay.groups + 3) / 4);  // the launches with a wave per group: 4 waves per block
    const KEY *keys = static_cast<const KEY *>(d_keys);
    const unsigned *ccounts = counts, *cgprefix = gprefix;
    uint16_t *out = static_cast<uint16_t *>(d_out);
    const int in_flight = options().by_key_key_tiles ? options().by_key_key_tiles : 16;  // KiB of keys a wave has in flight
#define TCU_KEY_HEADS(G_, NT_) launch(key_heads_kernel<KEY, G_, NT_>, (unsigned)blocks, waves * 64u, stream, keys, n, lay.parts, bits, counts, list, run)
    if (options().nontemporal) {
      if (in_flight == 4) TCU_KEY_HEADS(4, true);
      else if (in_flight == 8) TCU_KEY_HEADS(8, true);
      else TCU_KEY_HEADS(16, true);
    } else {
      if (in_flight == 4) TCU_KEY_HEADS(4, false);
      else if (in_flight == 8) TCU_KEY_HEADS(8, false);
      else TCU_KEY_HEADS(16, false);
    }
#undef TCU_KEY_HEADS
    launch(key_group_prefix_kernel, 1u, 1024u, stream, ccounts, gprefix, lay.parts, lay.groups);
    if (options().nontemporal)
      launch(reduce_by_heads_kernel<KEY, true>, (unsigned)blocks, waves * 64u, stream, static_cast<const uint16_t *>(d_in), static_cast<const unsigned long long *>(bits), ccounts, cgprefix, keys,
             static_cast<const KEY *>(list), out, static_cast<KEY *>(d_keys_out), lead, tail, n, lay.parts, run);
    else
      launch(reduce_by_heads_kernel<KEY, false>, (unsigned)blocks, waves * 64u, stream, static_cast<const uint16_t *>(d_in), static_cast<const unsigned long long *>(bits), ccounts, cgprefix, keys,
             static_cast<const KEY *>(list), out, static_cast<KEY *>(d_keys_out), lead, tail, n, lay.parts, run);
    launch(key_group_tails_kernel, group_blocks, 256u, stream, ccounts, static_cast<const float *>(tail), gflag, gtail, lay.parts, lay.groups);
    launch(close_boundary_runs_kernel, group_blocks, 256u, stream, ccounts, cgprefix, static_cast<const float *>(lead), static_cast<const float *>(tail), static_cast<const unsigned *>(gflag),
           static_cast<const float *>(gtail), out, static_cast<unsigned long long *>(d_num_runs), lay.parts, lay.groups);
    return TCU_OK;
  }
  unsigned *ws = static_cast<unsigned *>(d_ws);
  launch(zero_look_back_kernel, (unsigned)((parts + 255) / 256), 256u, stream, ws, parts, shift);
  const int so = options().static_order ? 1 : 0;
  const unsigned grid = (unsigned)parts, block = (unsigned)kByKeyWaves * 64u;
  const KEY *keys = static_cast<const KEY *>(d_keys);
  const uint16_t *in = static_cast<const uint16_t *>(d_in);
  uint16_t *out = static_cast<uint16_t *>(d_out);
  KEY *keys_out = static_cast<KEY *>(d_keys_out);
  unsigned long long *num_runs = static_cast<unsigned long long *>(d_num_runs);
  const bool nt = options().nontemporal;
  if (reduce) {
    if (nt) launch(by_key_kernel<KEY, kByKeyTiles, true, true>, grid, block, stream, keys, in, out, keys_out, num_runs, n, ws, so, wait_policy(shift, ws));
    else launch(by_key_kernel<KEY, kByKeyTiles, true, false>, grid, block, stream, keys, in, out, keys_out, num_runs, n, ws, so, wait_policy(shift, ws));
  } else {
    if (nt) launch(by_key_kernel<KEY, kByKeyTiles, false, true>, grid, block, stream, keys, in, out, keys_out, num_runs, n, ws, so, wait_policy(shift, ws));
    else launch(by_key_kernel<KEY, kByKeyTiles, false, false>, grid, block, stream, keys, in, out, keys_out, num_runs, n, ws, so, wait_policy(shift, ws));
  }
  return TCU_OK;
}

inline int seg_scan_by_key_dispatch(const void *d_keys, const void *d_in, void *d_out, size_t n, int key_bits, void *d_ws, size_t *ws_bytes, void *stream) {
  const char *what = "tcu_seg_scan_by_key_f16";
  if (key_bits == 32) return by_key_typed<int32_t>(what, false, d_keys, d_in, nullptr, d_out, nullptr, n, d_ws, ws_bytes, stream);
  if (key_bits == 64) return by_key_typed<int64_t>(what, false, d_keys, d_in, nullptr, d_out, nullptr, n, d_ws, ws_bytes, stream);
  return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": key_bits must be 32 or 64");
}
inline int seg_reduce_by_key_dispatch(const void *d_keys, const void *d_in, void *d_keys_out, void *d_out, void *d_num_runs, size_t n, int key_bits, void *d_ws, size_t *ws_bytes, void *stream) {
  const char *what = "tcu_seg_reduce_by_key_f16";
  if (key_bits == 32) return by_key_typed<int32_t>(what, true, d_keys, d_in, d_keys_out, d_out, d_num_runs, n, d_ws, ws_bytes, stream);
  if (key_bits == 64) return by_key_typed<int64_t>(what, true, d_keys, d_in, d_keys_out, d_out, d_num_runs, n, d_ws, ws_bytes, stream);
  return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": key_bits must be 32 or 64");
}

// ----- GEMV / GEMM -----------------------------------------------------------------------------

// OUT = float: tcu_gemv_f16_f32; OUT = half_t: tcu_gemv_f16_f16 (y in fp16)
template <typename OUT>
inline int gemv_dispatch_typed(const char *what, const void *A, const void *x, void *y, size_t M, size_t K, float alpha, float beta, int variant, void *stream) {
  if (!(variant == TCU_VARIANT_AUTO || variant == TCU_VARIANT_WAVE_SHUFFLE || variant == TCU_VARIANT_MFMA_16N || variant == TCU_VARIANT_MFMA_256N))
    return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": variant must be AUTO, WAVE_SHUFFLE, MFMA_16N or MFMA_256N");
  const bool trace = variant == TCU_VARIANT_MFMA_256N;  // row tile x x tile on the matrix unit, same launch shapes as the dot-product form
  if (M == 0) return TCU_OK;
  if (!y || (K && (!A || !x))) return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": null device pointer");
  const bool vec_ok = K % 8 == 0 && K > 0 && aligned16(A) && aligned16(x);
  const bool nt = options().nontemporal;
  const unsigned block = 256;
  if (!vec_ok) {
    if (variant != TCU_VARIANT_AUTO) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": K must be a positive multiple of 8 and A, x 16-byte aligned");
    const size_t grid = (M + 3) / 4;
    if (grid > kMaxGrid) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": grid exceeds the launch limit");
    launch(gemv_generic_kernel<OUT>, (unsigned)grid, block, stream, static_cast<const uint16_t *>(A), static_cast<const uint16_t *>(x), static_cast<OUT *>(y), M, K, alpha, beta);
    return TCU_OK;
  }
  const half8_t *a = static_cast<const half8_t *>(A), *xv = static_cast<const half8_t *>(x);
  OUT *yy = static_cast<OUT *>(y);
  if (variant == TCU_VARIANT_MFMA_16N) {
    // a block per 16-row strip; its waves split K, at least two steps of 256 k each (16384 x 16384: 1 wave 109 us,
    // 2 waves 112, 4 waves 108, 8 waves 124, 16 waves 117; one wave per strip and 16-byte pieces per row and load: 171)
    const size_t grid = (M + 15) / 16, steps = (K + 255) / 256;
    if (grid > kMaxGrid) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": grid exceeds the launch limit");
    int wpb = options().gemv_waves;
    if (K % 512 == 0 && options().gemv_strip_lds) {  // whole steps of 512 k: the strip goes through LDS
      if (!(wpb == 1 || wpb == 2 || wpb == 4)) wpb = 4;
      while (wpb > 1 && (size_t)wpb > K / 512) wpb /= 2;
      launch(gemv_strip_lds_kernel<OUT>, (unsigned)grid, (unsigned)wpb * 64u, stream, a, xv, yy, M, K / 8, alpha, beta);
      return TCU_OK;
    }
    if (!(wpb == 1 || wpb == 2 || wpb == 4 || wpb == 8 || wpb == 16)) {
      wpb = 4;
      while (wpb > 1 && (size_t)wpb * 2 > steps) wpb /= 2;
    }
    if (nt)
      launch(gemv_mfma_kernel<true, OUT>, (unsigned)grid, (unsigned)wpb * 64u, stream, a, xv, yy, M, K / 8, alpha, beta);
    else
      launch(gemv_mfma_kernel<false, OUT>, (unsigned)grid, (unsigned)wpb * 64u, stream, a, xv, yy, M, K / 8, alpha, beta);
    return TCU_OK;
  }
  const size_t k_tiles = (K / 8 + 63) / 64;
  if (k_tiles >= 8) {  // rows of 8 KiB and more: a block per group of rows
    // measured at 16384^2 (48 shapes, randomised order): 2 rows x 2 tiles x 16 waves 81.5 us, 2 x 1 x 16 81.6,
    // 2 x 1 x 8 81.7 ... 2 x 4 x 8 89.7, 4 rows 84.7+, 1 row 88+: as many waves as the row has tiles
    const int rows = options().gemv_rows ? options().gemv_rows : 2, bu = options().gemv_tiles ? options().gemv_tiles : (k_tiles >= 32 ? 2 : 1);
    const size_t fit = k_tiles / (size_t)bu;
    const unsigned bw = options().gemv_waves ? (unsigned)options().gemv_waves : (fit >= 16 ? 16u : fit >= 8 ? 8u : 4u);
    const size_t bgrid = (M + rows - 1) / rows;
    if (bgrid > kMaxGrid) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": grid exceeds the launch limit");
    if (trace) {  // the default shapes only
      if (rows != 2 || bu > 2) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": the MFMA_256N form takes gemv_rows = 2 and gemv_tiles <= 2");
      if (bu == 2) {
        if (nt) launch(gemv_block_kernel<2, 2, true, OUT, true>, (unsigned)bgrid, bw * 64u, stream, a, xv, yy, M, K / 8, alpha, beta);
        else launch(gemv_block_kernel<2, 2, false, OUT, true>, (unsigned)bgrid, bw * 64u, stream, a, xv, yy, M, K / 8, alpha, beta);
      } else {
        if (nt) launch(gemv_block_kernel<2, 1, true, OUT, true>, (unsigned)bgrid, bw * 64u, stream, a, xv, yy, M, K / 8, alpha, beta);
        else launch(gemv_block_kernel<2, 1, false, OUT, true>, (unsigned)bgrid, bw * 64u, stream, a, xv, yy, M, K / 8, alpha, beta);
      }
      return TCU_OK;
    }
#define TCU_GEMV_BLOCK(R_, U_)                                                                                              \
  if (rows == R_ && bu == U_) {                                                                                            \
    if (nt)                                                                                                                \
      launch(gemv_block_kernel<R_, U_, true, OUT>, (unsigned)bgrid, bw * 64u, stream, a, xv, yy, M, K / 8, alpha, beta);         \
    else                                                                                                                   \
      launch(gemv_block_kernel<R_, U_, false, OUT>, (unsigned)bgrid, bw * 64u, stream, a, xv, yy, M, K / 8, alpha, beta);        \
    return TCU_OK;                                                                                                         \
  }
    TCU_GEMV_BLOCK(1, 1) TCU_GEMV_BLOCK(1, 2) TCU_GEMV_BLOCK(1, 4) TCU_GEMV_BLOCK(1, 8)
    TCU_GEMV_BLOCK(2, 1) TCU_GEMV_BLOCK(2, 2) TCU_GEMV_BLOCK(2, 4)
    TCU_GEMV_BLOCK(4, 1) TCU_GEMV_BLOCK(4, 2) TCU_GEMV_BLOCK(4, 4)
    TCU_GEMV_BLOCK(8, 1) TCU_GEMV_BLOCK(8, 2)
#undef TCU_GEMV_BLOCK
    return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": unsupported gemv_rows / gemv_tiles option");
  }
  constexpr int ROWS = 2, UK = 4;
  const size_t waves = (M + ROWS - 1) / ROWS;
  const size_t grid = (waves + 3) / 4;
  if (grid > kMaxGrid) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": grid exceeds the launch limit");
  if (trace) {
    if (nt) launch(gemv_dot_kernel<ROWS, UK, true, OUT, true>, (unsigned)grid, block, stream, a, xv, yy, M, K / 8, alpha, beta);
    else launch(gemv_dot_kernel<ROWS, UK, false, OUT, true>, (unsigned)grid, block, stream, a, xv, yy, M, K / 8, alpha, beta);
    return TCU_OK;
  }
  if (nt)
    launch(gemv_dot_kernel<ROWS, UK, true, OUT>, (unsigned)grid, block, stream, a, xv, yy, M, K / 8, alpha, beta);
  else
    launch(gemv_dot_kernel<ROWS, UK, false, OUT>, (unsigned)grid, block, stream, a, xv, yy, M, K / 8, alpha, beta);
  return TCU_OK;
}
// A column-major (tcu_gemv_col_major_f16_f32 / _f16)
template <typename OUT>
inline int gemv_col_major_dispatch(const char *what, const void *A, size_t lda, const void *x, void *y, size_t M, size_t K, float alpha, float beta, void *stream) {
  if (M == 0) return TCU_OK;
  if (!y || (K && (!A || !x))) return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": null device pointer");
  if (lda < M) return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": lda must be at least M");
  const uint16_t *a = static_cast<const uint16_t *>(A);
  OUT *yy = static_cast<OUT *>(y);
  const bool vec_ok = K > 0 && K % 8 == 0 && lda % 8 == 0 && aligned16(A) && aligned16(x);
  if (!vec_ok) {
    const size_t grid = (M + 255) / 256;
    if (grid > kMaxGrid) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": grid exceeds the launch limit");
    launch(gemv_col_generic_kernel<OUT>, (unsigned)grid, 256u, stream, a, lda, static_cast<const uint16_t *>(x), yy, M, K, alpha, beta);
    return TCU_OK;
  }
  // slabs of 512 rows; K is cut into stretches so that about 1024 blocks of 8 waves run and a wave still takes two rounds or
  // more (16384 x 16384: 32 slabs x 32 stretches of 512 columns; 1024 ... 8192 blocks of 4 or 8 waves: 88-106 us)
  const int shape = options().gemv_col_shape;  // waves per block * 10 + groups of 8 columns per wave and round
  const unsigned waves = shape / 10 == 8 ? 8u : 4u, groups = shape % 10 == 1 ? 1u : 2u;
  const size_t round = (size_t)8 * groups * waves;  // columns per round of a block
  const size_t slabs = (M + kColSlabRows - 1) / kColSlabRows;
  size_t stretches = ((size_t)options().gemv_col_blocks + slabs - 1) / slabs;
  const size_t most = (K + 2 * round - 1) / (2 * round);
  if (stretches > most) stretches = most;
  if (stretches < 1) stretches = 1;
  size_t cols = (K + stretches - 1) / stretches;
  cols = (cols + round - 1) / round * round;  // whole rounds of the block's waves
  stretches = (K + cols - 1) / cols;
  if (slabs * stretches > kMaxGrid || slabs > 0xffffffffu) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": grid exceeds the launch limit");
  float *partials = static_cast<float *>(stream_alloc(stretches * M * sizeof(float), stream));
  if (!partials) return fail(TCU_ERR_RUNTIME, std::string(what) + ": no temporary device memory for the partial sums");
  const unsigned grid = (unsigned)(slabs * stretches);
  const half8_t *xv = static_cast<const half8_t *>(x);
#define TCU_GEMV_COL(W_, G_)                                                                                                              \
  do {                                                                                                                                    \
    if (options().nontemporal) launch(gemv_col_partials_kernel<W_, G_, true>, grid, W_ * 64u, stream, a, lda, xv, partials, M, K, (unsigned)slabs, cols); \
    else launch(gemv_col_partials_kernel<W_, G_, false>, grid, W_ * 64u, stream, a, lda, xv, partials, M, K, (unsigned)slabs, cols);      \
  } while (0)
  if (waves == 8 && groups == 1) TCU_GEMV_COL(8, 1);
  else if (waves == 8) TCU_GEMV_COL(8, 2);
  else if (groups == 1) TCU_GEMV_COL(4, 1);
  else TCU_GEMV_COL(4, 2);
#undef TCU_GEMV_COL
  launch(gemv_col_finish_kernel<OUT>, (unsigned)((M + 255) / 256), 256u, stream, static_cast<const float *>(partials), yy, M, (unsigned)stretches, alpha, beta);
  stream_free(partials, stream);
  return TCU_OK;
}

inline int gemv_dispatch(const void *A, const void *x, void *y, size_t M, size_t K, float alpha, float beta, int variant, void *stream) {
  return gemv_dispatch_typed<float>("tcu_gemv_f16_f32", A, x, y, M, K, alpha, beta, variant, stream);
}
inline int hgemv_dispatch(const void *A, const void *x, void *y, size_t M, size_t K, float alpha, float beta, int variant, void *stream) {
  return gemv_dispatch_typed<half_t>("tcu_gemv_f16_f16", A, x, y, M, K, alpha, beta, variant, stream);
}

// OUT = float: tcu_gemm_f16_f32; OUT = half_t: tcu_gemm_f16_f16 (C and D in fp16)
template <typename OUT>
inline int gemm_dispatch_typed(const char *what, const void *A, const void *B, const void *C, void *D, size_t M, size_t N, size_t K, float alpha, float beta, int variant, void *stream) {
  if (!(variant == TCU_VARIANT_AUTO || variant == TCU_VARIANT_BLOCK_LDS || variant == TCU_VARIANT_MFMA_16N)) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": variant must be AUTO, BLOCK_LDS or MFMA_16N");
  if (M == 0 || N == 0) return TCU_OK;
  if (!D || (K && (!A || !B)) || (beta != 0.0f && !C)) return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": null device pointer");
  // the tiled kernels move fp16 outputs as 32-bit pairs
  const bool al = aligned16(A) && aligned16(B) && (sizeof(OUT) == 4 || ((reinterpret_cast<uintptr_t>(C) | reinterpret_cast<uintptr_t>(D)) & 3u) == 0);
  const bool lds_ok = al && M % kGemmBM == 0 && N % kGemmBN == 0 && K % kGemmBK == 0 && K > 0;
  const bool direct_ok = al && M % 32 == 0 && N % 32 == 0 && K % 16 == 0 && K > 0;
  const half8_t *a = static_cast<const half8_t *>(A), *b = static_cast<const half8_t *>(B);
  const OUT *c = static_cast<const OUT *>(C);
  OUT *d = static_cast<OUT *>(D);
  if (variant == TCU_VARIANT_BLOCK_LDS && !lds_ok) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": the LDS kernel needs M, N multiples of 128 and K a multiple of 32");
  if (variant == TCU_VARIANT_MFMA_16N && !direct_ok) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": the direct kernel needs M, N multiples of 32 and K a multiple of 16");
  // fewer than 128 tiles of 256 x 256 leave more than half of the 256 compute units idle: the
  // 128 x 128 kernel then wins (2048^3: 37.8 vs 51.9 us; 2560^3, 100 tiles: 55.8 vs 62.4; 3072^3, 144 tiles: 126 vs 72.5)
  const bool big_tiles = options().gemm_big_tiles > 0 || (options().gemm_big_tiles < 0 && (M / kGemmBigBM) * (N / kGemmBigBN) >= 128);
  // 192 x 192 tiles where they fill the chip's rounds better than the 256 x 256 ones: a round of them costs
  // 0.5625 of the work and 17 % for the smaller tile (9216^3: 157 against 240 us per round); the big tiles are priced
  // with their split tail (a last round at most a third full costs its share and a fix-up).  3072^3: 256 tiles in one
  // round, 61.9 us, against 144 of 256 compute units busy for 70.5 (fp16 outputs 56.4 against 63.4); 6144^3 and up: level
  // or behind.  gemm_big_tiles = 192 forces them, 0 and 1 leave them out.
  if (al && K > 0 && variant != TCU_VARIANT_MFMA_16N && M % 192 == 0 && N % 192 == 0 && K % 64 == 0 && K <= ((size_t)1 << 22) && options().gemm_direct_lds < 0 &&
      ((reinterpret_cast<uintptr_t>(C) | reinterpret_cast<uintptr_t>(D)) & (4 * sizeof(OUT) - 1)) == 0) {
    const size_t units = (size_t)options().compute_units, t192 = (M / 192) * (N / 192);
    bool take = options().gemm_big_tiles == 192;
    if (options().gemm_big_tiles < 0 && M % kGemmBigBM == 0 && N % kGemmBigBN == 0) {
      const size_t t256 = (M / kGemmBigBM) * (N / kGemmBigBN), full = t256 / units, tail = t256 % units;
      if (t256 >= 128) {
        const double last = tail == 0 ? 0.0 : ((tail * 3 <= units && K >= 4096) ? (double)tail / (double)units + 0.15 : 1.0);
        const double cost256 = ((double)full + last) * 65536.0, cost192 = (double)((t192 + units - 1) / units) * 36864.0 * 1.17;
        take = cost192 < cost256;
      }
    }
    if (take) {
      if (t192 > kMaxGrid) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": grid exceeds the launch limit");
      const bool staged = options().gemm_staged_epilogue && ((reinterpret_cast<uintptr_t>(C) | reinterpret_cast<uintptr_t>(D)) & 15u) == 0;
      if (staged)
        launch(gemm_dlds_a3b2_m16_t192_kernel<OUT, true>, (unsigned)t192, 256u, stream, a, b, c, d, M, N, K, alpha, beta);
      else
        launch(gemm_dlds_a3b2_m16_t192_kernel<OUT, false>, (unsigned)t192, 256u, stream, a, b, c, d, M, N, K, alpha, beta);
      return TCU_OK;
    }
  }
  if (lds_ok && variant != TCU_VARIANT_MFMA_16N && M % kGemmBigBM == 0 && N % kGemmBigBN == 0 && big_tiles) {
    const size_t grid = (M / kGemmBigBM) * (N / kGemmBigBN);
    if (grid > kMaxGrid) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": grid exceeds the launch limit");
    // measured (2048^3 ... 16384^3, K = 4096 ... 16448): the transfer kernels with K step 64 (whole
    // 128-byte lines per row and transfer) beat the K-step-32 and the register-staged forms at
    // every size (8192^3: 1305 vs 1225 vs 1128 TFLOP/s), and of the two the one with three A and
    // two B buffers is equal or faster everywhere (16384^3: 1313 vs 1083).  The same kernel on
    // 16x16x32 MFMAs (66) draws less power per multiply-add and is the default: 8192^3 with fp16
    // outputs 783 vs 852 us, fp32 outputs 850 vs 866; 16384^3 fp16 6.36 vs 6.80 ms (same run)
    const int direct_lds = options().gemm_direct_lds >= 0 ? options().gemm_direct_lds : (K % 64 == 0 ? 66 : 4);
    if (direct_lds > 0 && K <= ((size_t)1 << 22)) {
      // the 16x16x32 kernel moves four adjacent outputs per access (16 bytes of fp32, 8 of fp16)
      const bool al4 = ((reinterpret_cast<uintptr_t>(C) | reinterpret_cast<uintptr_t>(D)) & (4 * sizeof(OUT) - 1)) == 0;
      if (direct_lds == 66 && K % 64 == 0 && al4) {
        // the epilogue that turns the outputs through LDS moves 16 bytes per lane: whole rows of a wave's 128 columns per store
        // instead of 64 (fp32) / 32 (fp16) bytes of 16 rows (8192^3, alpha 1.1, beta 1.2 / 0, events around the call, same run:
        // fp32 outputs 830-858 -> 794-809 / 774-789 -> 762 us, fp16 outputs 807 -> 757 / 776 -> 746 us; 4096^3 fp16 134-151 -> 121 / 126 -> 110)
        const bool staged = options().gemm_staged_epilogue && ((reinterpret_cast<uintptr_t>(C) | reinterpret_cast<uintptr_t>(D)) & 15u) == 0;
        // the tiles of a last, sparsely filled round of the grid: their K steps are spread evenly over all compute
        // units, in runs of at least 8 steps.  The shares cost up to 2 x 256 KiB of fp32 per block written and read
        // back, which pays while the round is at most a third full and a tile takes long enough (8192^3 sizes, same
        // run, with / without: 7168^3, 784 tiles on 256 units, 625 / 698 us; 6144^3 413 / 455; 9216^3 1300 / 1382;
        // but 5120^3, 400 tiles, 340 / 262; 3072^3 128 / 87; 9728^3 1600 / 1522)
        const size_t units = (size_t)options().compute_units, tail = grid % units, steps = K / 64;
        const int mode = options().gemm_split_tail;  // 0 never, 1 by the rule above, 2 whenever there is a tail
        if (tail && steps >= 16 && (mode == 2 || (mode == 1 && tail * 3 <= units && steps >= 64))) {
          const size_t full = grid - tail, total = tail * steps;
          size_t blocks = total / 8 < units ? total / 8 : units;
          const size_t run = (total + blocks - 1) / blocks;  // <= steps, as tail < units
          blocks = (total + run - 1) / run;
          float *ws = static_cast<float *>(stream_alloc(2 * blocks * (size_t)(kGemmBigBM * kGemmBigBN) * sizeof(float), stream));
          if (ws) {
            if (staged)
              launch(gemm_dlds_a3b2_m16_kernel<OUT, true>, (unsigned)(full + blocks), 256u, stream, a, b, c, d, M, N, K, alpha, beta, (unsigned)full, (unsigned)run, ws);
            else
              launch(gemm_dlds_a3b2_m16_kernel<OUT, false>, (unsigned)(full + blocks), 256u, stream, a, b, c, d, M, N, K, alpha, beta, (unsigned)full, (unsigned)run, ws);
            launch(gemm_split_fixup_kernel<OUT>, (unsigned)(tail * 64), 256u, stream, static_cast<const float *>(ws), c, d, M, N, K, alpha, beta, (unsigned)full, (unsigned)run);
            stream_free(ws, stream);
            return TCU_OK;
          }
        }
        if (staged)
          launch(gemm_dlds_a3b2_m16_kernel<OUT, true>, (unsigned)grid, 256u, stream, a, b, c, d, M, N, K, alpha, beta, (unsigned)grid, 1u, static_cast<float *>(nullptr));
        else
          launch(gemm_dlds_a3b2_m16_kernel<OUT, false>, (unsigned)grid, 256u, stream, a, b, c, d, M, N, K, alpha, beta, (unsigned)grid, 1u, static_cast<float *>(nullptr));
      }
      else if (direct_lds >= 65 && K % 64 == 0)
        launch(gemm_dlds_a3b2_kernel<OUT>, (unsigned)grid, 256u, stream, a, b, c, d, M, N, K, alpha, beta);
      else if (direct_lds >= 64 && K % 64 == 0)
        launch(gemm_dlds_kernel<64, 2, OUT>, (unsigned)grid, 256u, stream, a, b, c, d, M, N, K, alpha, beta);
      else if (direct_lds == 3)
        launch(gemm_dlds_kernel<32, 3, OUT>, (unsigned)grid, 256u, stream, a, b, c, d, M, N, K, alpha, beta);
      else
        launch(gemm_dlds_kernel<32, 4, OUT>, (unsigned)grid, 256u, stream, a, b, c, d, M, N, K, alpha, beta);
      return TCU_OK;
    }
    const bool bk64 = K % 64 == 0 && options().gemm_bk64;
    const size_t steps = K / (bk64 ? 64 : 32);
    int depth = options().gemm_depth < 1 ? 1 : (options().gemm_depth > 4 ? 4 : options().gemm_depth);
    if (bk64 && depth > 2) depth = 2;
    while (steps % (size_t)depth) depth--;  // the kernels take whole groups of `depth` steps
#define TCU_GEMM256(BK_, D_) launch(gemm_lds256_kernel<BK_, D_, OUT>, (unsigned)grid, 256u, stream, a, b, c, d, M, N, K, alpha, beta)
    if (bk64) {
      if (depth == 2) TCU_GEMM256(64, 2); else TCU_GEMM256(64, 1);
    } else {
      switch (depth) {
        case 4: TCU_GEMM256(32, 4); break;
        case 3: TCU_GEMM256(32, 3); break;
        case 2: TCU_GEMM256(32, 2); break;
        default: TCU_GEMM256(32, 1); break;
      }
    }
#undef TCU_GEMM256
  } else if (lds_ok && variant != TCU_VARIANT_MFMA_16N) {
    const size_t grid = (M / kGemmBM) * (N / kGemmBN);
    if (grid > kMaxGrid) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": grid exceeds the launch limit");
    // the transfer kernel with 128 x 128 tiles (two blocks per compute unit) unless the register-staged
    // kernel is asked for (gemm_direct_lds = 0) or K is beyond the 32-bit lane offsets
    if (options().gemm_direct_lds != 0 && K <= ((size_t)1 << 22)) {
      // K a multiple of 64 and outputs aligned to four: the three-A-two-B-buffer loop on 16x16x32 MFMAs with the
      // epilogue through LDS, as for the big tiles (gemm_direct_lds = 64 keeps the 32x32x16 kernel selectable)
      const bool al4 = ((reinterpret_cast<uintptr_t>(C) | reinterpret_cast<uintptr_t>(D)) & (4 * sizeof(OUT) - 1)) == 0;
      const int direct_lds = options().gemm_direct_lds;
      if ((direct_lds < 0 || direct_lds == 66) && K % 64 == 0 && al4) {
        const bool staged = options().gemm_staged_epilogue && ((reinterpret_cast<uintptr_t>(C) | reinterpret_cast<uintptr_t>(D)) & 15u) == 0;
        if (staged)
          launch(gemm_dlds_a3b2_m16_t128_kernel<OUT, true>, (unsigned)grid, 256u, stream, a, b, c, d, M, N, K, alpha, beta);
        else
          launch(gemm_dlds_a3b2_m16_t128_kernel<OUT, false>, (unsigned)grid, 256u, stream, a, b, c, d, M, N, K, alpha, beta);
      } else if (K % 64 == 0)
        launch(gemm_dlds_kernel<64, 2, OUT, 128>, (unsigned)grid, 256u, stream, a, b, c, d, M, N, K, alpha, beta);
      else
        launch(gemm_dlds_kernel<32, 4, OUT, 128>, (unsigned)grid, 256u, stream, a, b, c, d, M, N, K, alpha, beta);
      return TCU_OK;
    }
    launch(gemm_lds_kernel<OUT>, (unsigned)grid, 256u, stream, a, b, c, d, M, N, K, alpha, beta);
  } else if (direct_ok) {
    const size_t tiles = (M / 32) * (N / 32);
    const size_t grid = (tiles + 3) / 4;
    if (grid > kMaxGrid) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": grid exceeds the launch limit");
    launch(gemm_direct_kernel<OUT>, (unsigned)grid, 256u, stream, a, b, c, d, M, N, K, alpha, beta);
  } else {
    const size_t grid = (M * N + 255) / 256;
    if (grid > kMaxGrid) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": grid exceeds the launch limit");
    launch(gemm_generic_kernel<OUT>, (unsigned)grid, 256u, stream, static_cast<const uint16_t *>(A), static_cast<const uint16_t *>(B), c, d, M, N, K, alpha, beta);
  }
  return TCU_OK;
}
inline int gemm_dispatch(const void *A, const void *B, const void *C, void *D, size_t M, size_t N, size_t K, float alpha, float beta, int variant, void *stream) {
  return gemm_dispatch_typed<float>("tcu_gemm_f16_f32", A, B, C, D, M, N, K, alpha, beta, variant, stream);
}
inline int hgemm_dispatch(const void *A, const void *B, const void *C, void *D, size_t M, size_t N, size_t K, float alpha, float beta, int variant, void *stream) {
  return gemm_dispatch_typed<half_t>("tcu_gemm_f16_f16", A, B, C, D, M, N, K, alpha, beta, variant, stream);
}

// ----- fills, conversions, inputs, probes --------------------------------------------------------

inline unsigned fill_grid(size_t n) {
  size_t g = (n + 255) / 256;
  return (unsigned)(g > 65536 ? 65536 : (g ? g : 1));
}
inline int fill_dispatch(void *d, float value, size_t n, void *stream) {
  if (!n) return TCU_OK;
  if (!d) return fail(TCU_ERR_INVALID_ARG, "tcu_fill_f16: null device pointer");
  launch(fill_f16_kernel, fill_grid(n), 256u, stream, static_cast<uint16_t *>(d), value, n);
  return TCU_OK;
}
inline int convert_dispatch(void *d_out, const void *d_in, size_t n, void *stream) {
  if (!n) return TCU_OK;
  if (!d_out || !d_in) return fail(TCU_ERR_INVALID_ARG, "tcu_convert_f32_to_f16: null device pointer");
  launch(convert_f32_to_f16_kernel, fill_grid(n), 256u, stream, static_cast<uint16_t *>(d_out), static_cast<const float *>(d_in), n);
  return TCU_OK;
}
inline int generate_dispatch(void *d, size_t n, uint64_t seed, int dist, size_t first, void *stream) {
  if (dist < TCU_DIST_UNIFORM || dist > TCU_DIST_SMALLINT) return fail(TCU_ERR_INVALID_ARG, "tcu_generate_f16: unknown distribution");
  if (!n) return TCU_OK;
  if (!d) return fail(TCU_ERR_INVALID_ARG, "tcu_generate_f16: null device pointer");
  launch(generate_f16_kernel, fill_grid(n), 256u, stream, static_cast<uint16_t *>(d), n, seed, dist, first);
  return TCU_OK;
}

template <int U>
inline void launch_probe(int mode, int nt, unsigned grid, unsigned block, void *stream, uint4_t *dst, const half8_t *src, size_t n_chunks) {
#define TCU_PROBE_CASE(MODE)                                                                             \
  if (nt == kStoreAlternate)                                                                             \
    launch(stream_probe_kernel<U, MODE, kStoreAlternate>, grid, block, stream, dst, src, n_chunks);      \
  else if (nt == kStoreStream)                                                                           \
    launch(stream_probe_kernel<U, MODE, kStoreStream>, grid, block, stream, dst, src, n_chunks);         \
  else                                                                                                   \
    launch(stream_probe_kernel<U, MODE, kStoreCached>, grid, block, stream, dst, src, n_chunks);         \
  return
  switch (mode) {
    case 0: TCU_PROBE_CASE(0);
    case 1: TCU_PROBE_CASE(1);
    default: TCU_PROBE_CASE(2);
  }
#undef TCU_PROBE_CASE
}
inline int stream_probe_dispatch(void *d_dst, const void *d_src, size_t bytes, int mode, int tiles_per_wave, int waves_per_block, void *stream) {
  const char *what = "tcu_stream_probe";
  if (mode < 0 || mode > 2) return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": mode must be 0, 1 or 2");
  if (bytes % 16 != 0) return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": bytes must be a multiple of 16");
  const int u = tiles_per_wave ? tiles_per_wave : 4, wpb = waves_per_block ? waves_per_block : 4;
  if (!(u == 1 || u == 2 || u == 4 || u == 8) || !(wpb == 1 || wpb == 2 || wpb == 4 || wpb == 8 || wpb == 16)) return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": bad tiles_per_wave / waves_per_block");
  if (!bytes) return TCU_OK;
  if (!d_dst || (mode != 2 && !d_src) || !aligned16(d_dst) || !aligned16(d_src)) return fail(TCU_ERR_INVALID_ARG, std::string(what) + ": null or misaligned device pointer");
  const size_t n_chunks = bytes / 16;
  const size_t tiles = (n_chunks + kTileChunks - 1) / kTileChunks;
  const size_t waves = (tiles + u - 1) / u;
  const size_t grid = (waves + wpb - 1) / wpb;
  if (grid > kMaxGrid) return fail(TCU_ERR_UNSUPPORTED, std::string(what) + ": grid exceeds the launch limit");
  const int nt = scan_store_policy();
  uint4_t *dst = static_cast<uint4_t *>(d_dst);
  const half8_t *src = static_cast<const half8_t *>(d_src);
  switch (u) {
    case 1: launch_probe<1>(mode, nt, (unsigned)grid, wpb * 64u, stream, dst, src, n_chunks); break;
    case 2: launch_probe<2>(mode, nt, (unsigned)grid, wpb * 64u, stream, dst, src, n_chunks); break;
    case 4: launch_probe<4>(mode, nt, (unsigned)grid, wpb * 64u, stream, dst, src, n_chunks); break;
    default: launch_probe<8>(mode, nt, (unsigned)grid, wpb * 64u, stream, dst, src, n_chunks); break;
  }
  return TCU_OK;
}
inline int lane_probe_dispatch(void *d_out, size_t *out_words, void *stream) {
  if (!out_words) return fail(TCU_ERR_INVALID_ARG, "tcu_lane_probe: out_words must not be null");
  if (!d_out) {
    *out_words = kLaneProbeWords;
    return TCU_OK;
  }
  if (*out_words < kLaneProbeWords) return fail(TCU_ERR_WORKSPACE, "tcu_lane_probe: output buffer too small");
  launch(lane_probe_kernel, 1u, 64u, stream, static_cast<unsigned *>(d_out));
  return TCU_OK;
}

}  // namespace tcu
