// Fills, conversions, seeded input generation, streaming probes and the lane probe.
#pragma once

#include <math.h>

#include "seg_reduce.hpp"

namespace tcu {

// out[i] = (half) value; the reference's setFP16 (src/utils/cuda_helpers.cuh:123-132)
__global__ __launch_bounds__(256) void fill_f16_kernel(uint16_t *out, float value, size_t n) {
  const uint16_t h = f16_bits(value);
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) out[i] = h;
}
// the reference's convertFp32ToFp16 (src/utils/cuda_helpers.cuh:116-121)
__global__ __launch_bounds__(256) void convert_f32_to_f16_kernel(uint16_t *out, const float *in, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) out[i] = f16_bits(in[i]);
}

TCU_DEVICE uint64_t mix64(uint64_t z) {
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
// Element i of stream `seed` = output i of SplitMix64 started at seed, mapped per `dist`.
__global__ __launch_bounds__(256) void generate_f16_kernel(uint16_t *out, size_t n, uint64_t seed, int dist, size_t first) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    const uint64_t z = mix64(seed + (uint64_t)(first + i + 1) * 0x9E3779B97F4A7C15ull);
    uint16_t h;
    if (dist == 0) {  // uniform [-1,1): 24 bits, exact in fp32, one rounding to fp16, never +1
      const float xf = (float)(uint32_t)(z >> 40) * 0x1p-23f - 1.0f;
      h = f16_bits(xf);
      if (h == 0x3c00u) h = 0x3bffu;
    } else if (dist == 1) {  // k/2048
      h = f16_bits((float)((int)(z >> 52) - 2048) * 0x1p-11f);
    } else if (dist == 2) {  // Box-Muller
      const uint64_t z2 = mix64(z + 0x9E3779B97F4A7C15ull);
      const double u1 = ((double)(z >> 40) + 1.0) * 0x1p-24;
      const double u2 = (double)(z2 >> 40) * 0x1p-24;
      h = f16_bits((float)(sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925286766559 * u2)));
    } else {  // {0,1,2}
      h = f16_bits((float)(uint32_t)((z >> 33) % 3u));
    }
    out[i] = h;
  }
}

// Streaming probes with the access shape of the reduction / scan kernels: each wave takes
// U consecutive tiles.  MODE 0 copy, 1 read only, 2 write only.
template <int U, int MODE, int NT>
__global__ __launch_bounds__(kMaxBlock) void stream_probe_kernel(uint4_t *dst, const half8_t *src, size_t n_chunks) {
  const int lane = lane_id();
  const size_t gw = (size_t)blockIdx.x * (blockDim.x >> 6) + wave_in_block();
  const size_t chunk0 = gw * (size_t)(U * kTileChunks);
  if (chunk0 >= n_chunks) return;
  half8_t v[U];
  if constexpr (MODE != 2) {
    load_tiles<U, NT != 0>(v, src, chunk0, n_chunks, lane);
  } else {
#pragma unroll
    for (int j = 0; j < U; j++) v[j] = splat8((float)lane);
  }
  if constexpr (MODE == 1) {
    float acc = 0.0f;
#pragma unroll
    for (int j = 0; j < U; j++) acc = sum8(v[j], acc);
    // keeps the loads alive; one word per wave only when the data says so (never for finite sums)
    if (acc == 123456.0f) reinterpret_cast<float *>(dst)[gw] = acc;
  } else {
    static_for<U>([&](auto J) {
      constexpr int j = decltype(J)::value;
      const size_t c = chunk0 + (size_t)j * kTileChunks + lane;
      if (c < n_chunks) store_chunk<kTileStoreNT<NT, j>>(dst + c, __builtin_bit_cast(uint4_t, v[j]));
    });
  }
}

// Lane probe: one wave.  Record layout (32-bit words, 64 per record unless noted):
//   0: mfma16 D regs (4 records)  A[m][k] = m + 1 (k == probe_k), B[k][n] = n + 1 (k == probe_k)
//      for probe_k = 0 -> D[m][n] = (m+1)(n+1) if the layouts hold
//   4: mfma16 with A = one-hot row 3 / k 17, B = one-hot k 17 / col 5 -> single 1 at D[3][5]
//   8: mfma32 D regs (16 records), A[m][k] = [k == 9] * (m + 1), B[k][n] = [k == 9] * (n + 1)
//  24: dpp quad_xor1, quad_xor2, row_half_mirror, row_mirror of lane id (4 records, as float)
//  28: row_shr:1, row_shr:3, wave_shr:1 (bound_ctrl zero fill), row_bcast15 (mask 0xA, old = -1),
//      row_bcast31 (mask 0xC, old = -1) (5 records)
//  33: permlane16_swap a,b and permlane32_swap a,b with a = lane, b = 100 + lane (4 records, u32)
//  37: ballot(lane % 3 == 0) low, high (2 records), readlane(lane*2, 37) (1 record)
constexpr size_t kLaneProbeWords = 40 * 64;
__global__ __launch_bounds__(64) void lane_probe_kernel(unsigned *out) {
  const int lane = lane_id();
  auto put_f = [&](int rec, float v) { out[rec * 64 + lane] = __float_as_uint(v); };
  auto put_u = [&](int rec, unsigned v) { out[rec * 64 + lane] = v; };
  {
    // operand element (row/col = lane%16, k = 8*(lane/16) + e)
    half8_t a, b;
    for (int e = 0; e < 8; e++) {
      const int k = 8 * (lane >> 4) + e;
      a[e] = (half_t)(k == 0 ? (float)((lane & 15) + 1) : 0.0f);
      b[e] = (half_t)(k == 0 ? (float)((lane & 15) + 1) : 0.0f);
    }
    float4_t d = mfma_16x16x32(a, b, float4_t{0, 0, 0, 0});
    for (int i = 0; i < 4; i++) put_f(0 + i, d[i]);
    for (int e = 0; e < 8; e++) {
      const int k = 8 * (lane >> 4) + e;
      a[e] = (half_t)((k == 17 && (lane & 15) == 3) ? 1.0f : 0.0f);
      b[e] = (half_t)((k == 17 && (lane & 15) == 5) ? 1.0f : 0.0f);
    }
    d = mfma_16x16x32(a, b, float4_t{0, 0, 0, 0});
    for (int i = 0; i < 4; i++) put_f(4 + i, d[i]);
  }
  {
    half8_t a, b;
    for (int e = 0; e < 8; e++) {
      const int k = 8 * (lane >> 5) + e;
      a[e] = (half_t)(k == 9 ? (float)((lane & 31) + 1) : 0.0f);
      b[e] = (half_t)(k == 9 ? (float)((lane & 31) + 1) : 0.0f);
    }
    float16_t c;
    for (int e = 0; e < 16; e++) c[e] = 0.0f;
    float16_t d = mfma_32x32x16(a, b, c);
    for (int i = 0; i < 16; i++) put_f(8 + i, d[i]);
  }
  const float fl = (float)lane;
  put_f(24, dpp<DPP_QUAD_XOR1>(fl, fl));
  put_f(25, dpp<DPP_QUAD_XOR2>(fl, fl));
  put_f(26, dpp<DPP_ROW_HALF_MIRROR>(fl, fl));
  put_f(27, dpp<DPP_ROW_MIRROR>(fl, fl));
  put_f(28, dpp<DPP_ROW_SHR0 + 1>(-1.0f, fl + 1.0f));
  put_f(29, dpp<DPP_ROW_SHR0 + 3>(-1.0f, fl + 1.0f));
  put_f(30, dpp<DPP_WAVE_SHR1>(-1.0f, fl + 1.0f));
  put_f(31, dpp<DPP_ROW_BCAST15, 0xA, 0xF, false>(-1.0f, fl + 1.0f));
  put_f(32, dpp<DPP_ROW_BCAST31, 0xC, 0xF, false>(-1.0f, fl + 1.0f));
  {
    unsigned a = (unsigned)lane, b = 100u + (unsigned)lane;
    permlane16_swap(a, b);
    put_u(33, a);
    put_u(34, b);
    a = (unsigned)lane;
    b = 100u + (unsigned)lane;
    permlane32_swap(a, b);
    put_u(35, a);
    put_u(36, b);
  }
  const unsigned long long bal = ballot(lane % 3 == 0);
  put_u(37, (unsigned)bal);
  put_u(38, (unsigned)(bal >> 32));
  put_u(39, readlane_u32((unsigned)lane * 2u, 37));
}

}  // namespace tcu
