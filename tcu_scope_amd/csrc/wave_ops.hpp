// Wave64 primitives for gfx950 (CDNA4): DPP cross-lane moves, lane swaps, fp16 MFMA,
// packed fp16 dot products, 128-bit global accesses and device-scope atomics.
//
// Every kernel in this directory is written against these wrappers only.  Lane
// numbering: lane = threadIdx.x & 63; a DPP "row" is 16 consecutive lanes.
//
// MFMA operand layouts used throughout (v_mfma_f32_16x16x32_f16, D = A*B + C):
//   A (16 x 32): lane l holds A[l % 16][8*(l/16) .. 8*(l/16)+7]   (8 halves)
//   B (32 x 16): lane l holds B[8*(l/16) .. 8*(l/16)+7][l % 16]   (8 halves)
//   C/D (16x16): lane l holds D[4*(l/16) + i][l % 16], i = 0..3   (4 floats)
// v_mfma_f32_32x32x16_f16:
//   A (32 x 16): lane l holds A[l % 32][8*(l/32) .. +7]
//   B (16 x 32): lane l holds B[8*(l/32) .. +7][l % 32]
//   C/D (32x32): lane l, register i (0..15) holds D[8*(i/4) + 4*(l/32) + i%4][l % 32]
#ifndef TCU_WAVE_OPS_HPP
#define TCU_WAVE_OPS_HPP

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace tcu {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float2_t __attribute__((ext_vector_type(2)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef unsigned uint2_t __attribute__((ext_vector_type(2)));
typedef unsigned uint4_t __attribute__((ext_vector_type(4)));

#define TCU_DEVICE __device__ __forceinline__

constexpr int kWave = 64;

// DPP control words
constexpr int DPP_QUAD_XOR1 = 0xB1;        // quad_perm:[1,0,3,2]
constexpr int DPP_QUAD_XOR2 = 0x4E;        // quad_perm:[2,3,0,1]
constexpr int DPP_ROW_SHR0 = 0x110;        // + d, d = 1..15
constexpr int DPP_WAVE_SHR1 = 0x138;
constexpr int DPP_ROW_MIRROR = 0x140;
constexpr int DPP_ROW_HALF_MIRROR = 0x141;
constexpr int DPP_ROW_BCAST15 = 0x142;
constexpr int DPP_ROW_BCAST31 = 0x143;

TCU_DEVICE int lane_id() { return (int)(threadIdx.x & 63u); }
TCU_DEVICE int wave_in_block() { return (int)(threadIdx.x >> 6); }

// dst = (lane enabled by masks) ? (source lane valid ? src[source lane] : (BOUND_CTRL ? 0 : old)) : old
template <int CTRL, int ROW_MASK = 0xf, int BANK_MASK = 0xf, bool BOUND_CTRL = true>
TCU_DEVICE float dpp(float old, float src) {
  return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(old), __float_as_int(src), CTRL, ROW_MASK, BANK_MASK, BOUND_CTRL));
}
template <int CTRL, int ROW_MASK = 0xf, int BANK_MASK = 0xf, bool BOUND_CTRL = true>
TCU_DEVICE unsigned dpp_u32(unsigned old, unsigned src) {
  return (unsigned)__builtin_amdgcn_update_dpp((int)old, (int)src, CTRL, ROW_MASK, BANK_MASK, BOUND_CTRL);
}

// value of `x` in lane `l` (l must be wave-uniform)
TCU_DEVICE float readlane(float x, int l) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(x), l)); }
TCU_DEVICE unsigned readlane_u32(unsigned x, int l) { return (unsigned)__builtin_amdgcn_readlane((int)x, l); }

// bit l of the result = `pred` of lane l
TCU_DEVICE unsigned long long ballot(bool pred) { return __builtin_amdgcn_ballot_w64(pred); }

// a[lanes 16..31] <-> b[lanes 0..15] and a[48..63] <-> b[32..47]
TCU_DEVICE void permlane16_swap(unsigned &a, unsigned &b) {
  uint2_t r = __builtin_amdgcn_permlane16_swap(a, b, false, false);
  a = r.x;
  b = r.y;
}
// a[lanes 32..63] <-> b[lanes 0..31]
TCU_DEVICE void permlane32_swap(unsigned &a, unsigned &b) {
  uint2_t r = __builtin_amdgcn_permlane32_swap(a, b, false, false);
  a = r.x;
  b = r.y;
}
// x + (x of lane ^ 16), x + (x of lane ^ 32): exact fp32 pair sums across DPP rows
TCU_DEVICE float add_xor16(float x) {
  unsigned a = __float_as_uint(x), b = a;
  permlane16_swap(a, b);
  return __uint_as_float(a) + __uint_as_float(b);
}
TCU_DEVICE float add_xor32(float x) {
  unsigned a = __float_as_uint(x), b = a;
  permlane32_swap(a, b);
  return __uint_as_float(a) + __uint_as_float(b);
}

TCU_DEVICE float4_t mfma_16x16x32(half8_t a, half8_t b, float4_t c) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0); }
TCU_DEVICE float16_t mfma_32x32x16(half8_t a, half8_t b, float16_t c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }

// c + a.x*b.x + a.y*b.y with an fp32 accumulator
TCU_DEVICE float fdot2(half2_t a, half2_t b, float c) { return __builtin_amdgcn_fdot2(a, b, c, false); }

// sum of the 8 halves of one 128-bit chunk, fp32 accumulate
TCU_DEVICE float sum8(half8_t v, float acc) {
  const half2_t ones = {(half_t)1.0f, (half_t)1.0f};
  acc = fdot2(__builtin_shufflevector(v, v, 0, 1), ones, acc);
  acc = fdot2(__builtin_shufflevector(v, v, 2, 3), ones, acc);
  acc = fdot2(__builtin_shufflevector(v, v, 4, 5), ones, acc);
  acc = fdot2(__builtin_shufflevector(v, v, 6, 7), ones, acc);
  return acc;
}

TCU_DEVICE half8_t splat8(float v) {
  half_t h = (half_t)v;
  half8_t r = {h, h, h, h, h, h, h, h};
  return r;
}

// two floats -> packed fp16 pair, round to nearest even
TCU_DEVICE unsigned pack_f16x2(float lo, float hi) {
  half2_t h = {(half_t)lo, (half_t)hi};
  return __builtin_bit_cast(unsigned, h);
}
TCU_DEVICE uint16_t f16_bits(float v) {
  half_t h = (half_t)v;
  return __builtin_bit_cast(uint16_t, h);
}

// 128-bit global accesses.  Streaming data is touched once: non-temporal hints keep it
// from displacing anything in L2 / Infinity Cache.
template <bool NT>
TCU_DEVICE half8_t load_chunk(const half8_t *p) {
  if constexpr (NT) return __builtin_nontemporal_load(p);
  return *p;
}
#ifndef TCU_STORE_NT
#define TCU_STORE_NT 1
#endif
template <bool NT>
TCU_DEVICE void store_chunk(uint4_t *p, uint4_t v) {
  if constexpr (NT && TCU_STORE_NT)
    __builtin_nontemporal_store(v, p);
  else
    *p = v;
}

// Store policies of the scan kernels and of the copy probe (the value of their NT template argument; all loads are
// non-temporal unless it is 0): 0 = every access through the cache, 1 = tile 0, 2, ... of a wave stored
// non-temporally and tile 1, 3, ... through the cache, 2 = every store non-temporal (the default).
// What the alternation buys depends on where the output goes.  Segmented scan of 2^28 halves, kernel times: with ONE
// 512 MiB output buffer that every launch rewrites, alternating stores run at 143-146 us against 160-169 us for
// all non-temporal -- the cached half of the output is exactly the 256 MiB of the memory-side cache, stays there
// dirty and is overwritten by the next launch before it has to be written to HBM.  With three or five output
// buffers taken in turn (or one 2 GiB output at 2^30 halves), i.e. when every byte written has to reach HBM, the
// same kernels take 161-174 us alternating and 160-169 us all non-temporal, and 172-182 us all cached.  Policy 1
// is therefore kept for callers whose output is consumed from that cache, and is not the default.
constexpr int kStoreCached = 0, kStoreAlternate = 1, kStoreStream = 2;
template <int NT, int J>
constexpr bool kTileStoreNT = NT == kStoreStream || (NT == kStoreAlternate && J % 2 == 0);

// f(Int<0>{}), f(Int<1>{}), ..., f(Int<N-1>{}): a loop whose index is a compile-time constant in the body
template <int V>
struct Int {
  static constexpr int value = V;
};
template <int N, int J = 0, class F>
TCU_DEVICE void static_for(F &&f) {
  if constexpr (J < N) {
    f(Int<J>{});
    static_for<N, J + 1>(f);
  }
}

// Global -> LDS without a register round trip: lane l of the wave moves the 16 bytes at its
// own global address `src` to lds_base + 16 * l (lds_base is the same for the whole wave).
// Written as inline assembly on purpose: for the compiler's own form of this instruction the
// wait-count pass drains every transfer in flight before the next LDS read it cannot prove
// disjoint, which would undo a multi-stage prefetch.  The price: the compiler knows nothing
// of these transfers, so the reader orders them by hand: wait_vector_loads<N>() for the
// wave's own, then a barrier for everybody's.
// An LDS location is named by its byte offset inside the block's LDS (lds_addr_t), which
// keeps the address arithmetic of a transfer in scalar integer registers.
using lds_addr_t = uint32_t;
// tells the compiler that a value is the same in every lane (it then lives in a scalar register)
TCU_DEVICE uint32_t wave_uniform(uint32_t x) { return (uint32_t)__builtin_amdgcn_readfirstlane(x); }
TCU_DEVICE lds_addr_t lds_address_of(const half_t *lds_pointer) {
  using lds_ptr_t = const __attribute__((address_space(3))) half_t *;
  return (lds_addr_t)(uintptr_t)(lds_ptr_t)lds_pointer;
}
// The global address is wave_base (the same for the whole wave, kept in scalar registers)
// plus the lane's own byte offset.
TCU_DEVICE void load_chunk_to_lds(const void *wave_base, uint32_t lane_byte_offset, lds_addr_t lds_base) {
  const uint32_t base = wave_uniform(lds_base);
  const uint64_t g = (uint64_t)wave_base;
  // (the builtin returns a signed int: widen through uint32_t, or bit 31 of the low word smears over the high one)
  const uint32_t g_lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)g), g_hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(g >> 32));
  const uint64_t gs = ((uint64_t)g_hi << 32) | (uint64_t)g_lo;
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(base), "v"(lane_byte_offset), "s"(gs) : "memory", "m0");
}
// blocks until at most N of this wave's vector memory loads are still in flight (they
// complete in issue order); N <= 63
template <int N>
TCU_DEVICE void wait_vector_loads() {
  static_assert(N >= 0 && N <= 63, "vmcnt has 6 bits");
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
  asm volatile("" ::: "memory");  // later reads of what the loads wrote stay behind the wait
}

// Block barrier for code that orders its own memory traffic: waits for this wave's LDS
// operations only (not for vector memory loads in flight, which __syncthreads() would drain)
// and keeps the compiler from moving memory accesses across it.
TCU_DEVICE void block_barrier_lds_only() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt((63 & 15) | ((63 >> 4) << 14) | (7 << 4) | (0 << 8));  // lgkmcnt(0)
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// stops the instruction scheduler from moving anything across this point
TCU_DEVICE void sched_fence() { __builtin_amdgcn_sched_barrier(0); }
// Instruction-mix hints for the scheduler inside one region: "next, COUNT instructions of KIND".
enum : int { kSchedMfma = 0x008, kSchedVmem = 0x010, kSchedVmemRead = 0x020, kSchedDsRead = 0x100, kSchedDsWrite = 0x200 };
template <int KIND, int COUNT>
TCU_DEVICE void sched_group() {
  __builtin_amdgcn_sched_group_barrier(KIND, COUNT, 0);
}

// orders LDS traffic between the lanes of one wave (no s_barrier: a wave runs in lockstep)
TCU_DEVICE void wave_lds_fence() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// device-scope atomics for single-pass full-array kernels
TCU_DEVICE unsigned atomic_add_u32(unsigned *p, unsigned v) { return __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
TCU_DEVICE unsigned atomic_add_u32_acq_rel(unsigned *p, unsigned v) { return __hip_atomic_fetch_add(p, v, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT); }
TCU_DEVICE float atomic_add_f32(float *p, float v) { return __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
TCU_DEVICE unsigned long long atomic_load_u64(const unsigned long long *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
TCU_DEVICE void atomic_store_u64(unsigned long long *p, unsigned long long v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
TCU_DEVICE float atomic_load_f32(const float *p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
TCU_DEVICE void device_fence_release() { __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent"); }
TCU_DEVICE void device_fence_acquire() { __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent"); }
TCU_DEVICE void spin_pause() { __builtin_amdgcn_s_sleep(1); }

}  // namespace tcu
#endif  // TCU_WAVE_OPS_HPP
