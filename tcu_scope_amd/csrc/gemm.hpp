// D = alpha * A B + beta * C.  A: M x K row-major fp16; B: K x N column-major fp16 (stored
// as N rows of K, so both operands are K-contiguous); C, D: M x N row-major fp32.
// Operand layouts of the reference's compute_gemm (src/gemm/wmma.cu:15-18).
//
//   gemm_lds_kernel    : 128 x 128 block tile, K step 32, 4 waves in a 2 x 2 grid, each wave
//                        a 64 x 64 tile = 2 x 2 v_mfma_f32_32x32x16_f16 accumulators.
//                        A/B tiles go global -> registers -> LDS (rows padded to 40 halves
//                        so that the 128-bit fragment reads of 16 lanes hit distinct banks)
//                        with the next step's global loads in flight during the MFMAs and
//                        two LDS buffers (one barrier per step).  Counterpart of the
//                        reference's shared-memory kernels (src/gemm/wmma.cu:171-365,
//                        wmma_sharedmem.cu:43-123).
//   gemm_lds256_kernel, gemm_dlds_kernel, gemm_dlds_a3b2_kernel, gemm_dlds_a3b2_m16_kernel :
//                        256 x 256 block tile, 4 waves of 128 x 128 (all 256 accumulation
//                        registers), hand-pipelined; operands staged through registers or
//                        moved global -> LDS directly (described at the kernels); the last
//                        one on v_mfma_f32_16x16x32_f16 (less power per multiply-add), the
//                        others on 32x32x16.  gemm_dlds_a3b2_m16_t128_kernel (and gemm_dlds_kernel
//                        with TILE = 128) run the same loops on 128 x 128 block tiles, two blocks per
//                        compute unit, for outputs too small to fill the chip with the big tiles;
//                        gemm_dlds_a3b2_m16_t192_kernel on 192 x 192 tiles where those fill it better.
//   gemm_direct_kernel : one 32 x 32 tile per wave, fragments loaded straight from global
//                        memory (reference compute_gemm_naive, src/gemm/wmma_naive.cu:33-88).
//   gemm_generic_kernel: any M, N, K; one thread per output element.
#pragma once

#include <type_traits>

#include "wave_ops.hpp"

namespace tcu {

constexpr int kGemmBM = 128, kGemmBN = 128, kGemmBK = 32;
constexpr int kGemmLdsStride = 40;  // halves per LDS row (32 + 8 pad)

TCU_DEVICE void gemm_tile_of_block(size_t tiles_m, size_t tiles_n, size_t b, size_t *tile_m, size_t *tile_n);

// D and C are streamed once: non-temporal accesses keep them from displacing the A and B
// panels that other tiles reuse from L2.  All of a tile's C values are read before its first
// store, so the loads overlap and C may be the same buffer as D.
// OUT = float: a lane owns column (lane & 31) of rows 8*(i/4) + 4*(lane >> 5) + i%4.
// OUT = half_t (C and D in fp16, the layout of the reference's compute_hgemm,
// src/gemm/wmma.cu:367-560; products still accumulate in fp32, the only accumulator width the
// MFMA unit has): neighbouring lanes trade one value of each pair of rows, so that an even lane
// owns two adjacent columns of the even row and the odd lane the same columns of the odd row,
// and every access moves a 32-bit pair.
// alpha * a + beta * c in one fixed rounding sequence (alpha * a rounded, then one fused multiply-add with beta * c).  Left
// to the compiler, which of the two products is folded into the addition depends on the code around it, and two epilogues of
// the same accumulators then differ in the last bit; with this every GEMM kernel and epilogue gives the same bits.
// gemm_add_scaled takes the rounded product alpha * a (the epilogue that goes through LDS parks it there).
TCU_DEVICE float gemm_add_scaled(float alpha_a, float beta, float c) { return __builtin_fmaf(beta, c, alpha_a); }
TCU_DEVICE float gemm_axpby(float alpha, float a, float beta, float c) { return gemm_add_scaled(alpha * a, beta, c); }
TCU_DEVICE float4_t gemm_add_scaled(float4_t alpha_a, float beta, float4_t c) {
  float4_t r;
#pragma unroll
  for (int e = 0; e < 4; e++) r[e] = gemm_add_scaled(alpha_a[e], beta, c[e]);
  return r;
}
TCU_DEVICE float4_t gemm_axpby(float alpha, float4_t a, float beta, float4_t c) { return gemm_add_scaled(alpha * a, beta, c); }

template <typename OUT>
TCU_DEVICE void gemm_store_tile(OUT *D, const OUT *C, size_t ldc, size_t row0, size_t col0, const float16_t &acc, int lane, float alpha, float beta) {
  if constexpr (sizeof(OUT) == 4) {
    const size_t base = (row0 + 4 * (lane >> 5)) * ldc + col0 + (lane & 31);
    if (beta == 0.0f) {
#pragma unroll
      for (int i = 0; i < 16; i++) __builtin_nontemporal_store(alpha * acc[i], D + base + (size_t)(8 * (i / 4) + (i % 4)) * ldc);
    } else {
      float c[16];
#pragma unroll
      for (int i = 0; i < 16; i++) c[i] = __builtin_nontemporal_load(C + base + (size_t)(8 * (i / 4) + (i % 4)) * ldc);
#pragma unroll
      for (int i = 0; i < 16; i++) __builtin_nontemporal_store(gemm_axpby(alpha, acc[i], beta, c[i]), D + base + (size_t)(8 * (i / 4) + (i % 4)) * ldc);
    }
  } else {
    const bool odd = (lane & 1) != 0;
    // 32-bit word index of this lane's pair in row (row0 + 4*(lane >> 5) + (lane & 1)); ldc and col0 are even
    const size_t base = ((row0 + 4 * (lane >> 5) + (lane & 1)) * ldc + col0 + (lane & 30)) >> 1;
    const size_t ldw = ldc >> 1;
    uint32_t *d32 = reinterpret_cast<uint32_t *>(D);
    const uint32_t *c32 = reinterpret_cast<const uint32_t *>(C);
    float lo[8], hi[8];
#pragma unroll
    for (int p = 0; p < 8; p++) {  // rows 8*(p/2) + 2*(p%2) + {0, 1} of the lane's group of four
      const float send = odd ? acc[2 * p] : acc[2 * p + 1];
      const float recv = dpp<DPP_QUAD_XOR1>(send, send);
      lo[p] = odd ? recv : acc[2 * p];
      hi[p] = odd ? acc[2 * p + 1] : recv;
    }
    if (beta == 0.0f) {
#pragma unroll
      for (int p = 0; p < 8; p++) __builtin_nontemporal_store(pack_f16x2(alpha * lo[p], alpha * hi[p]), d32 + base + (size_t)(8 * (p / 2) + 2 * (p % 2)) * ldw);
    } else {
      uint32_t c[8];
#pragma unroll
      for (int p = 0; p < 8; p++) c[p] = __builtin_nontemporal_load(c32 + base + (size_t)(8 * (p / 2) + 2 * (p % 2)) * ldw);
#pragma unroll
      for (int p = 0; p < 8; p++) {
        const half2_t cv = __builtin_bit_cast(half2_t, c[p]);
        __builtin_nontemporal_store(pack_f16x2(gemm_axpby(alpha, lo[p], beta, (float)cv[0]), gemm_axpby(alpha, hi[p], beta, (float)cv[1])), d32 + base + (size_t)(8 * (p / 2) + 2 * (p % 2)) * ldw);
      }
    }
  }
}

// M % 128 == 0, N % 128 == 0, K % 32 == 0; 256 threads.
template <typename OUT>
__global__ __launch_bounds__(256) void gemm_lds_kernel(const half8_t *__restrict__ A, const half8_t *__restrict__ B, const OUT *C, OUT *D, size_t M, size_t N, size_t K, float alpha, float beta) {
  __shared__ __attribute__((aligned(16))) half_t lds_a[2][kGemmBM * kGemmLdsStride];
  __shared__ __attribute__((aligned(16))) half_t lds_b[2][kGemmBN * kGemmLdsStride];
  const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  size_t tile_m, tile_n;
  gemm_tile_of_block(M / kGemmBM, N / kGemmBN, blockIdx.x, &tile_m, &tile_n);
  const size_t k_chunks = K / 8;
  // global -> LDS copy assignment: 128 rows x 4 chunks = 512 chunks per operand, 2 per thread
  const int crow = tid >> 2, cchunk = tid & 3;  // rows crow and crow + 64
  const half8_t *ga0 = A + (tile_m * kGemmBM + crow) * k_chunks + cchunk;
  const half8_t *ga1 = ga0 + 64 * k_chunks;
  const half8_t *gb0 = B + (tile_n * kGemmBN + crow) * k_chunks + cchunk;
  const half8_t *gb1 = gb0 + 64 * k_chunks;
  const int so0 = crow * kGemmLdsStride + cchunk * 8, so1 = so0 + 64 * kGemmLdsStride;

  float16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;

  half8_t ra0 = ga0[0], ra1 = ga1[0], rb0 = gb0[0], rb1 = gb1[0];
  *reinterpret_cast<half8_t *>(&lds_a[0][so0]) = ra0;
  *reinterpret_cast<half8_t *>(&lds_a[0][so1]) = ra1;
  *reinterpret_cast<half8_t *>(&lds_b[0][so0]) = rb0;
  *reinterpret_cast<half8_t *>(&lds_b[0][so1]) = rb1;
  __syncthreads();

  const size_t steps = K / kGemmBK;
  // fragment read offsets: lane l -> row l%32 of the 32-row tile, halves 8*(l/32) .. +7 of a 16-k substep
  const int frow = lane & 31, fk = (lane >> 5) * 8;
  for (size_t s = 0; s < steps; s++) {
    const int cur = (int)(s & 1);
    if (s + 1 < steps) {
      const size_t o = (s + 1) * (kGemmBK / 8);
      ra0 = ga0[o];
      ra1 = ga1[o];
      rb0 = gb0[o];
      rb1 = gb1[o];
    }
#pragma unroll
    for (int kk = 0; kk < 2; kk++) {
      half8_t fa[2], fb[2];
#pragma unroll
      for (int i = 0; i < 2; i++) fa[i] = *reinterpret_cast<const half8_t *>(&lds_a[cur][(wm * 64 + i * 32 + frow) * kGemmLdsStride + kk * 16 + fk]);
#pragma unroll
      for (int j = 0; j < 2; j++) fb[j] = *reinterpret_cast<const half8_t *>(&lds_b[cur][(wn * 64 + j * 32 + frow) * kGemmLdsStride + kk * 16 + fk]);
#pragma unroll
      for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) acc[i][j] = mfma_32x32x16(fa[i], fb[j], acc[i][j]);
    }
    if (s + 1 < steps) {
      const int nxt = cur ^ 1;
      *reinterpret_cast<half8_t *>(&lds_a[nxt][so0]) = ra0;
      *reinterpret_cast<half8_t *>(&lds_a[nxt][so1]) = ra1;
      *reinterpret_cast<half8_t *>(&lds_b[nxt][so0]) = rb0;
      *reinterpret_cast<half8_t *>(&lds_b[nxt][so1]) = rb1;
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++) gemm_store_tile(D, C, N, tile_m * kGemmBM + wm * 64 + i * 32, tile_n * kGemmBN + wn * 64 + j * 32, acc[i][j], lane, alpha, beta);
}

// Block -> tile: the hardware deals consecutive block ids round-robin to the 8 XCDs, each
// with its own L2.  Block ids are first regrouped so that an XCD owns a contiguous range of
// tile ids, and tile ids walk bands of 4 tile rows column by column, so that the ~32 blocks
// an XCD runs at a time form a 4 x 8 patch sharing A row panels and B column panels in L2.
TCU_DEVICE void gemm_tile_of_block(size_t tiles_m, size_t tiles_n, size_t b, size_t *tile_m, size_t *tile_n) {
  const size_t nb = tiles_m * tiles_n;
  const size_t nb8 = nb & ~(size_t)7;  // the last nb % 8 blocks keep their ids
  const size_t id = b < nb8 ? (b % 8) * (nb8 / 8) + b / 8 : b;
  constexpr size_t GM = 4;
  const size_t band = id / (GM * tiles_n);
  const size_t rows = tiles_m - band * GM < GM ? tiles_m - band * GM : GM;
  const size_t r = id - band * GM * tiles_n;
  *tile_m = band * GM + r % rows;
  *tile_n = r / rows;
}

// M % 256 == 0, N % 256 == 0, K % (BK * DEPTH) == 0; 256 threads.  256 x 256 x BK block tile, 2 x 2
// waves of 128 x 128 (4 x 4 MFMA 32x32x16 accumulators = 256 registers, one wave per SIMD):
// per 16-wide k substep a wave reads 8 fragments from LDS for 16 MFMAs.  With one wave per
// SIMD nothing else hides latency, so the kernel is software-pipelined by hand:
//   - global loads run DEPTH steps ahead in DEPTH register stages (the loop is unrolled
//     DEPTH times to keep stage indices static);
//   - the stage of step s+1 is written to the other LDS buffer during the second-last
//     substep of step s, the one barrier of the step sits before the last substep, and the
//     fragments of step s+1's first substep are read behind that barrier while the last 16
//     MFMAs of step s run; inside a step the fragments of substep kk+1 are read while the
//     MFMAs of substep kk run.
// LDS rows are padded by 8 halves (the 128-bit fragment reads of 16 lanes hit distinct
// banks).
constexpr int kGemmBigBM = 256, kGemmBigBN = 256;
template <int BK, int DEPTH, typename OUT>
__global__ __launch_bounds__(256) void gemm_lds256_kernel(const half8_t *__restrict__ A, const half8_t *__restrict__ B, const OUT *C, OUT *D, size_t M, size_t N, size_t K, float alpha,
                                                          float beta) {
  constexpr int STRIDE = BK + 8;            // halves per LDS row
  constexpr int CPR = BK / 8;               // chunks per row
  constexpr int RPP = 256 / CPR;            // rows copied per pass of the block
  constexpr int PASSES = kGemmBigBM / RPP;  // passes per operand
  __shared__ __attribute__((aligned(16))) half_t lds_a[2][kGemmBigBM * STRIDE];
  __shared__ __attribute__((aligned(16))) half_t lds_b[2][kGemmBigBN * STRIDE];
  const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  size_t tile_m, tile_n;
  gemm_tile_of_block(M / kGemmBigBM, N / kGemmBigBN, blockIdx.x, &tile_m, &tile_n);
  const size_t k_chunks = K / 8;
  // Copy assignment: CPR consecutive lanes take one row's BK halves (one or two full cache
  // lines of global memory), 16 consecutive lanes 16 / CPR consecutive rows.  Inside LDS the
  // rows of every aligned group of 16 are permuted (lds_row): the 16 / CPR rows that 16
  // lanes store in one go land CPR positions apart, which puts their 128-bit stores into 16
  // different groups of four banks (row stride = 2 * CPR + 1 such groups, odd), and 16
  // consecutive rows read by 16 lanes still occupy 16 different positions.
  const int crow = tid / CPR, cchunk = tid % CPR;  // rows crow + RPP*i
  constexpr int ROT = CPR == 8 ? 1 : 2;  // rotate the low 4 bits of the row index right by ROT
  auto lds_row = [](int r) { return (r & ~15) | ((r & 15) >> ROT) | ((r << (4 - ROT)) & 15); };
  const half8_t *ga = A + (tile_m * kGemmBigBM + crow) * k_chunks + cchunk;
  const half8_t *gb = B + (tile_n * kGemmBigBN + crow) * k_chunks + cchunk;
  const int so = lds_row(crow) * STRIDE + cchunk * 8;
  const size_t steps = K / BK;

  float16_t acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
      for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;

  // Step 0 goes straight to LDS; register stage d then holds the steps t with (t - 1) % DEPTH
  // == d, i.e. during step s the stages hold the steps s+1 .. s+DEPTH.  The loop body is free
  // of branches (steps % DEPTH == 0 is the caller's duty; loads past the last step re-read
  // the last step and are never used), which keeps every stage in registers.
  half8_t ra[DEPTH][PASSES], rb[DEPTH][PASSES];
  {
    half8_t ta[PASSES], tb[PASSES];
#pragma unroll
    for (int i = 0; i < PASSES; i++) {
      ta[i] = ga[(size_t)i * RPP * k_chunks];
      tb[i] = gb[(size_t)i * RPP * k_chunks];
    }
#pragma unroll
    for (int d = 0; d < DEPTH; d++) {
      const size_t t = (size_t)d + 1 < steps ? (size_t)d + 1 : steps - 1;
#pragma unroll
      for (int i = 0; i < PASSES; i++) {
        ra[d][i] = ga[(size_t)i * RPP * k_chunks + t * CPR];
        rb[d][i] = gb[(size_t)i * RPP * k_chunks + t * CPR];
      }
    }
#pragma unroll
    for (int i = 0; i < PASSES; i++) {
      *reinterpret_cast<half8_t *>(&lds_a[0][so + i * RPP * STRIDE]) = ta[i];
      *reinterpret_cast<half8_t *>(&lds_b[0][so + i * RPP * STRIDE]) = tb[i];
    }
  }
  __syncthreads();

  const int frow = lane & 31, fk = (lane >> 5) * 8;
  constexpr int SUB = BK / 16;  // 16-wide k substeps per step (even: fragment parity carries over steps)
  const int fao = (wm * 128 + lds_row(frow)) * STRIDE + fk, fbo = (wn * 128 + lds_row(frow)) * STRIDE + fk;
  half8_t fa[2][4], fb[2][4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    fa[0][i] = *reinterpret_cast<const half8_t *>(&lds_a[0][fao + i * 32 * STRIDE]);
    fb[0][i] = *reinterpret_cast<const half8_t *>(&lds_b[0][fbo + i * 32 * STRIDE]);
  }
  for (size_t s0 = 0; s0 < steps; s0 += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; d++) {
      const size_t s = s0 + d;
      const int cur = (DEPTH & 1) ? (int)(s & 1) : (d & 1);
      const int nxt = cur ^ 1;
      const size_t sn = s + 1 + DEPTH < steps ? s + 1 + DEPTH : steps - 1;
      const size_t o = sn * CPR;
#pragma unroll
      for (int kk = 0; kk < SUB; kk++) {
        const int p = kk & 1, q = p ^ 1;
        if (kk == SUB - 1) {
          // the LDS writes of this step are visible behind the barrier; the fragments of the
          // next step's first substep are read while the MFMAs of this step's last one run
          __syncthreads();
          sched_fence();
#pragma unroll
          for (int i = 0; i < 4; i++) {
            fa[q][i] = *reinterpret_cast<const half8_t *>(&lds_a[nxt][fao + i * 32 * STRIDE]);
            fb[q][i] = *reinterpret_cast<const half8_t *>(&lds_b[nxt][fbo + i * 32 * STRIDE]);
          }
          // stage d went to LDS before the barrier: refill it with step s + 1 + DEPTH
#pragma unroll
          for (int i = 0; i < PASSES; i++) {
            ra[d][i] = ga[(size_t)i * RPP * k_chunks + o];
            rb[d][i] = gb[(size_t)i * RPP * k_chunks + o];
          }
        } else {
#pragma unroll
          for (int i = 0; i < 4; i++) {
            fa[q][i] = *reinterpret_cast<const half8_t *>(&lds_a[cur][fao + i * 32 * STRIDE + (kk + 1) * 16]);
            fb[q][i] = *reinterpret_cast<const half8_t *>(&lds_b[cur][fbo + i * 32 * STRIDE + (kk + 1) * 16]);
          }
        }
        // the next step's data (stage d) goes to the other LDS buffer, whose readers all
        // passed the barrier of the previous step: A and B in different substeps where the
        // step has enough of them, so that LDS is not flooded just before the barrier
        constexpr int WA = SUB >= 4 ? SUB - 3 : SUB - 2, WB = SUB - 2;
        if (kk == WA) {
#pragma unroll
          for (int i = 0; i < PASSES; i++) *reinterpret_cast<half8_t *>(&lds_a[nxt][so + i * RPP * STRIDE]) = ra[d][i];
        }
        if (kk == WB) {
#pragma unroll
          for (int i = 0; i < PASSES; i++) *reinterpret_cast<half8_t *>(&lds_b[nxt][so + i * RPP * STRIDE]) = rb[d][i];
        }
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
          for (int j = 0; j < 4; j++) acc[i][j] = mfma_32x32x16(fa[p][i], fb[p][j], acc[i][j]);
        // issue order of the substep: the 8 fragment reads lead, one per MFMA, then the
        // LDS writes or global loads of the substep spread over the remaining MFMAs
#pragma unroll
        for (int t = 0; t < 8; t++) {
          sched_group<kSchedDsRead, 1>();
          sched_group<kSchedMfma, 1>();
        }
        if (kk == WA || kk == WB) {
          constexpr int W = (WA == WB ? 2 : 1) * PASSES;  // 8 writes in every case
#pragma unroll
          for (int t = 0; t < 8; t++) {
            sched_group<kSchedDsWrite, W / 8>();
            sched_group<kSchedMfma, 1>();
          }
        } else if (kk == SUB - 1) {
#pragma unroll
          for (int t = 0; t < 8; t++) {
            sched_group<kSchedVmemRead, PASSES / 4>();
            sched_group<kSchedMfma, 1>();
          }
        } else {
          sched_group<kSchedMfma, 8>();
        }
        sched_fence();
      }
    }
  }
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) gemm_store_tile(D, C, N, tile_m * kGemmBigBM + wm * 128 + i * 32, tile_n * kGemmBigBN + wn * 128 + j * 32, acc[i][j], lane, alpha, beta);
}

// M % TILE == 0, N % TILE == 0, K % BK == 0, K <= 2^22 (lane offsets are 32-bit); 256 threads.
// TILE = 256: same tiling as gemm_lds256_kernel (256 x 256 x BK block tile, 2 x 2 waves of
// 128 x 128); TILE = 128: 2 x 2 waves of 64 x 64, 64 KiB of LDS, two blocks per compute unit
// (outputs too small to fill the chip with 256 x 256 tiles).  In both,
// the operands travel from global memory straight into LDS (load_chunk_to_lds), NBUF K steps
// deep: no staging registers, no LDS store instructions, prefetch distance NBUF - 1 steps.
// LDS rows are dense (BK halves = CPR chunks of 16 bytes).  A transfer instruction fills
// 1 KiB = 64 / CPR rows in lane order, so the swizzle that keeps the fragment reads free of
// bank conflicts is applied on the global side: LDS slot c of row r holds the row's chunk
// c ^ f(r), f(r) = (r / rows per 256 bytes) % CPR; the 16 rows that 16 lanes read for one k
// chunk then fall into 16 different groups of four banks.
// Step s (buffer s % NBUF): in every substep but the last, the fragments of the next substep
// are read under the first 8 MFMAs and up to 8 transfers of step s + NBUF - 1 (into the
// buffer of step s - 1, free since that step's barrier) are issued under the other 8;
// before the last substep a wave waits for its own transfers of step s + 1, the barrier
// publishes everybody's, the fragments of step s + 1, substep 0, are read while the last 16
// MFMAs of step s run, and the first half of the transfers of step s + NBUF already go out
// into the buffer that barrier has just freed (measured: every substep of extra flight time
// is worth 2-7 %; issuing more than half of a step's transfers in that one substep loses it
// again).
template <int BK, int NBUF, typename OUT, int TILE = kGemmBigBM>
__global__ __launch_bounds__(256) void gemm_dlds_kernel(const half8_t *__restrict__ A, const half8_t *__restrict__ B, const OUT *C, OUT *D, size_t M, size_t N, size_t K, float alpha, float beta) {
  constexpr int ROWH = BK;                           // halves per LDS row
  constexpr int CPR = BK / 8;                        // chunks per row
  constexpr int RPT = 64 / CPR;                      // rows per transfer instruction
  constexpr int RS = CPR == 4 ? 2 : 1;               // f(r) = (r >> RS) & (CPR - 1)
  constexpr int SUB = BK / 16;                       // 16-wide k substeps per step
  constexpr int W = TILE / 64;                       // 32 x 32 accumulators per wave and dimension (wave tile TILE/2 x TILE/2)
  constexpr int HALF = W * W / 2;                    // MFMAs per half substep
  constexpr int OPH = TILE * ROWH;                   // halves per operand per stage
  constexpr int P = NBUF - 1;                        // prefetch distance in steps
  constexpr int TPW = TILE / RPT / 4;                // transfer instructions per wave, operand and step
  constexpr int EARLY = TPW < HALF ? TPW : HALF;     // transfers of a step issued one substep ahead of the others
  static_assert((TILE == 128 || TILE == 256) && (BK == 32 || BK == 64) && 2 * TPW - EARLY <= HALF * (SUB - 1) && 2 * TPW * (P - 1) + EARLY <= 63, "transfers must fit the substeps and the counter");
  __shared__ __attribute__((aligned(1024))) half_t lds_a[NBUF][OPH];
  __shared__ __attribute__((aligned(1024))) half_t lds_b[NBUF][OPH];
  const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  size_t tile_m, tile_n;
  gemm_tile_of_block(M / TILE, N / TILE, blockIdx.x, &tile_m, &tile_n);
  const size_t k_chunks = K / 8;
  const size_t steps = K / BK;
  // transfer t of this wave (t = 0 .. TPW-1) fills rows RPT * (wave * TPW + t) .. + RPT-1; the
  // lane supplies row +lane/CPR, LDS slot lane%CPR, i.e. global chunk (lane%CPR) ^ f(row)
  // (the same lane offsets serve A and B: both have K columns).  Global addresses are a scalar
  // base per operand and step plus one of TPW 32-bit lane offsets.
  uint32_t goff[TPW];
#pragma unroll
  for (int t = 0; t < TPW; t++) {
    const int row = (wave * TPW + t) * RPT + lane / CPR;
    const int chunk = (lane % CPR) ^ ((row >> RS) & (CPR - 1));
    goff[t] = (uint32_t)(((size_t)row * k_chunks + chunk) * 16);
  }
  const char *ga = reinterpret_cast<const char *>(A + tile_m * TILE * k_chunks);
  const char *gb = reinterpret_cast<const char *>(B + tile_n * TILE * k_chunks);
  constexpr lds_addr_t STAGE = OPH * 2, TBYTES = 1024, STEPB = BK * 2;  // bytes per stage and operand, per transfer, per step and row
  const lds_addr_t ta = wave_uniform(lds_address_of(&lds_a[0][0]) + wave * TPW * TBYTES);
  const lds_addr_t tb = wave_uniform(lds_address_of(&lds_b[0][0]) + wave * TPW * TBYTES);
  // transfer x (0 .. 2*TPW-1) of a step: operand x % 2, rows of transfer x / 2
  auto issue = [&](size_t step, int buf, int x) {
    const size_t st = step < steps ? step : steps - 1;  // past the end: a harmless re-read into a free buffer
    if (x % 2 == 0)
      load_chunk_to_lds(ga + st * STEPB, goff[x / 2], ta + buf * STAGE + (x / 2) * TBYTES);
    else
      load_chunk_to_lds(gb + st * STEPB, goff[x / 2], tb + buf * STAGE + (x / 2) * TBYTES);
  };

  float16_t acc[W][W];
#pragma unroll
  for (int i = 0; i < W; i++)
#pragma unroll
    for (int j = 0; j < W; j++)
#pragma unroll
      for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;

#pragma unroll
  for (int d = 0; d < P; d++)
#pragma unroll
    for (int x = 0; x < 2 * TPW; x++) issue((size_t)d, d, x);
#pragma unroll
  for (int x = 0; x < EARLY; x++) issue((size_t)P, P, x);
  wait_vector_loads<2 * TPW * (P - 1) + EARLY>();
  block_barrier_lds_only();

  // fragment of row r, k chunk kc: slot kc ^ f(r); rows of a lane differ by multiples of 32
  const int frow = lane & 31, khalf = lane >> 5, fsw = (frow >> RS) & (CPR - 1);
  const int fa0 = (wm * (TILE / 2) + frow) * ROWH, fb0 = (wn * (TILE / 2) + frow) * ROWH;
  int ko[SUB];
#pragma unroll
  for (int kk = 0; kk < SUB; kk++) ko[kk] = ((2 * kk + khalf) ^ fsw) * 8;
  half8_t fa[2][W], fb[2][W];
#pragma unroll
  for (int i = 0; i < W; i++) {
    fa[0][i] = *reinterpret_cast<const half8_t *>(&lds_a[0][fa0 + i * 32 * ROWH + ko[0]]);
    fb[0][i] = *reinterpret_cast<const half8_t *>(&lds_b[0][fb0 + i * 32 * ROWH + ko[0]]);
  }
  int cur = 0;  // s % NBUF
  for (size_t s = 0; s < steps; s++) {
    const int nxt = cur + 1 == NBUF ? 0 : cur + 1;
    const int fill = cur == 0 ? NBUF - 1 : cur - 1;  // buffer of step s - 1 = buffer of step s + P
#pragma unroll
    for (int kk = 0; kk < SUB; kk++) {
      const int p = kk & 1, q = p ^ 1;
      if (kk < SUB - 1) {
        sched_fence();
#pragma unroll
        for (int i = 0; i < W; i++) {
          fa[q][i] = *reinterpret_cast<const half8_t *>(&lds_a[cur][fa0 + i * 32 * ROWH + ko[kk + 1]]);
          fb[q][i] = *reinterpret_cast<const half8_t *>(&lds_b[cur][fb0 + i * 32 * ROWH + ko[kk + 1]]);
        }
        // first half of the MFMAs with the fragment reads, second half with one transfer each
        // (the transfers are opaque to the scheduler, so fences pin them in place)
#pragma unroll
        for (int i = 0; i < W / 2; i++)
#pragma unroll
          for (int j = 0; j < W; j++) acc[i][j] = mfma_32x32x16(fa[p][i], fb[p][j], acc[i][j]);
#pragma unroll
        for (int t = 0; t < HALF; t++) {
          sched_group<kSchedDsRead, 2 * W / HALF>();
          sched_group<kSchedMfma, 1>();
        }
        sched_fence();
#pragma unroll
        for (int t = 0; t < HALF; t++) {
          const int i = W / 2 + t / W, j = t % W, x = EARLY + kk * HALF + t;
          if (x < 2 * TPW) issue(s + P, fill, x);
          acc[i][j] = mfma_32x32x16(fa[p][i], fb[p][j], acc[i][j]);
          sched_fence();
        }
      } else {
        // own transfers of step s + 1 done, barrier, fragments of step s + 1
        wait_vector_loads<2 * TPW * (P - 1)>();
        block_barrier_lds_only();
        sched_fence();
#pragma unroll
        for (int i = 0; i < W; i++) {
          fa[q][i] = *reinterpret_cast<const half8_t *>(&lds_a[nxt][fa0 + i * 32 * ROWH + ko[0]]);
          fb[q][i] = *reinterpret_cast<const half8_t *>(&lds_b[nxt][fb0 + i * 32 * ROWH + ko[0]]);
        }
        // the buffer of step s is free from this barrier on: the first transfers of step
        // s + NBUF go out here, one substep ahead of the rest
#pragma unroll
        for (int i = 0; i < W / 2; i++)
#pragma unroll
          for (int j = 0; j < W; j++) acc[i][j] = mfma_32x32x16(fa[p][i], fb[p][j], acc[i][j]);
#pragma unroll
        for (int t = 0; t < HALF; t++) {
          sched_group<kSchedDsRead, 2 * W / HALF>();
          sched_group<kSchedMfma, 1>();
        }
        sched_fence();
#pragma unroll
        for (int t = 0; t < HALF; t++) {
          const int i = W / 2 + t / W, j = t % W;
          if (t < EARLY) issue(s + NBUF, cur, t);
          acc[i][j] = mfma_32x32x16(fa[p][i], fb[p][j], acc[i][j]);
          sched_fence();
        }
      }
    }
    cur = nxt;
  }
  wait_vector_loads<0>();  // the re-reads past the last step must land before the block's LDS is released
#pragma unroll
  for (int i = 0; i < W; i++)
#pragma unroll
    for (int j = 0; j < W; j++) gemm_store_tile(D, C, N, tile_m * TILE + wm * (TILE / 2) + i * 32, tile_n * TILE + wn * (TILE / 2) + j * 32, acc[i][j], lane, alpha, beta);
}

// M % 256 == 0, N % 256 == 0, K % 64 == 0, K <= 2^22; 256 threads.
// gemm_dlds_kernel<64, 2> with the whole 160 KiB of LDS in use: three buffers for A, two for
// B.  After the barrier of step s the B tile of step s + 2 goes out into the B buffer the
// barrier has freed (all of it under the last 8 MFMAs of the step); the A tile of step s + 3
// follows under substeps 0 and 1 of step s + 1, into the A buffer of step s.  Every transfer
// then has at least a whole step (four substeps) of flight time, those of A almost two
// (measured against gemm_dlds_kernel<64, 2>: +1.5-3 % at 8192^3, +7 % at 12288^3, +17-21 % at
// 16384^3, where rows a multiple of 32 KiB apart make the loads slow; spreading the A tile
// over substeps 0-2 or 1-2 instead measures the same, all of it in substep 0 1 % less).
template <typename OUT>
__global__ __launch_bounds__(256) void gemm_dlds_a3b2_kernel(const half8_t *__restrict__ A, const half8_t *__restrict__ B, const OUT *C, OUT *D, size_t M, size_t N, size_t K, float alpha, float beta) {
  constexpr int BK = 64, ROWH = BK, CPR = 8, RPT = 8, RS = 1, SUB = 4, NA = 3, NB = 2;
  constexpr int OPH = kGemmBigBM * ROWH;     // halves per operand per stage
  constexpr int TPW = kGemmBigBM / RPT / 4;  // transfer instructions per wave, operand and step (8)
  __shared__ __attribute__((aligned(1024))) half_t lds_a[NA][OPH];
  __shared__ __attribute__((aligned(1024))) half_t lds_b[NB][OPH];
  const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  size_t tile_m, tile_n;
  gemm_tile_of_block(M / kGemmBigBM, N / kGemmBigBN, blockIdx.x, &tile_m, &tile_n);
  const size_t k_chunks = K / 8;
  const size_t steps = K / BK;
  uint32_t goff[TPW];
#pragma unroll
  for (int t = 0; t < TPW; t++) {
    const int row = (wave * TPW + t) * RPT + lane / CPR;
    const int chunk = (lane % CPR) ^ ((row >> RS) & (CPR - 1));
    goff[t] = (uint32_t)(((size_t)row * k_chunks + chunk) * 16);
  }
  const char *ga = reinterpret_cast<const char *>(A + tile_m * kGemmBigBM * k_chunks);
  const char *gb = reinterpret_cast<const char *>(B + tile_n * kGemmBigBN * k_chunks);
  constexpr lds_addr_t STAGE = OPH * 2, TBYTES = 1024, STEPB = BK * 2;
  const lds_addr_t ta = wave_uniform(lds_address_of(&lds_a[0][0]) + wave * TPW * TBYTES);
  const lds_addr_t tb = wave_uniform(lds_address_of(&lds_b[0][0]) + wave * TPW * TBYTES);
  // steps past the end: a harmless re-read of the last step into a free buffer
  auto issue_a = [&](size_t step, int buf, int t) { load_chunk_to_lds(ga + (step < steps ? step : steps - 1) * STEPB, goff[t], ta + buf * STAGE + t * TBYTES); };
  auto issue_b = [&](size_t step, int buf, int t) { load_chunk_to_lds(gb + (step < steps ? step : steps - 1) * STEPB, goff[t], tb + buf * STAGE + t * TBYTES); };

  float16_t acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
      for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;

  // in flight at the first barrier: A0 B0 | A1 B1 (the wave's counter returns in issue order)
#pragma unroll
  for (int t = 0; t < TPW; t++) issue_a(0, 0, t);
#pragma unroll
  for (int t = 0; t < TPW; t++) issue_b(0, 0, t);
#pragma unroll
  for (int t = 0; t < TPW; t++) issue_a(1, 1, t);
#pragma unroll
  for (int t = 0; t < TPW; t++) issue_b(1, 1, t);
  wait_vector_loads<2 * TPW>();
  block_barrier_lds_only();

  const int frow = lane & 31, khalf = lane >> 5, fsw = (frow >> RS) & (CPR - 1);
  const int fa0 = (wm * 128 + frow) * ROWH, fb0 = (wn * 128 + frow) * ROWH;
  int ko[SUB];
#pragma unroll
  for (int kk = 0; kk < SUB; kk++) ko[kk] = ((2 * kk + khalf) ^ fsw) * 8;
  half8_t fa[2][4], fb[2][4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    fa[0][i] = *reinterpret_cast<const half8_t *>(&lds_a[0][fa0 + i * 32 * ROWH + ko[0]]);
    fb[0][i] = *reinterpret_cast<const half8_t *>(&lds_b[0][fb0 + i * 32 * ROWH + ko[0]]);
  }
  int ca = 0, cb = 0;  // s % NA, s % NB
  for (size_t s = 0; s < steps; s++) {
    const int na = ca + 1 == NA ? 0 : ca + 1, nb = cb ^ 1;
    const int fill_a = ca == 0 ? NA - 1 : ca - 1;  // A buffer of step s - 1 = of step s + 2
#pragma unroll
    for (int kk = 0; kk < SUB; kk++) {
      const int p = kk & 1, q = p ^ 1;
      if (kk < SUB - 1) {
        sched_fence();
#pragma unroll
        for (int i = 0; i < 4; i++) {
          fa[q][i] = *reinterpret_cast<const half8_t *>(&lds_a[ca][fa0 + i * 32 * ROWH + ko[kk + 1]]);
          fb[q][i] = *reinterpret_cast<const half8_t *>(&lds_b[cb][fb0 + i * 32 * ROWH + ko[kk + 1]]);
        }
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
          for (int j = 0; j < 4; j++) acc[i][j] = mfma_32x32x16(fa[p][i], fb[p][j], acc[i][j]);
#pragma unroll
        for (int t = 0; t < 8; t++) {
          sched_group<kSchedDsRead, 1>();
          sched_group<kSchedMfma, 1>();
        }
        sched_fence();
#pragma unroll
        for (int t = 0; t < 8; t++) {
          const int i = 2 + t / 4, j = t % 4;
          if (kk < 2 && t % 2 == 0) issue_a(s + 2, fill_a, kk * 4 + t / 2);  // A tile of step s + 2: four transfers in each of substeps 0 and 1
          acc[i][j] = mfma_32x32x16(fa[p][i], fb[p][j], acc[i][j]);
          sched_fence();
        }
      } else {
        // own transfers of step s + 1 done (the A tile of step s + 2 may still fly), barrier,
        // fragments of step s + 1, B tile of step s + 2 into the B buffer of step s
        wait_vector_loads<TPW>();
        block_barrier_lds_only();
        sched_fence();
#pragma unroll
        for (int i = 0; i < 4; i++) {
          fa[q][i] = *reinterpret_cast<const half8_t *>(&lds_a[na][fa0 + i * 32 * ROWH + ko[0]]);
          fb[q][i] = *reinterpret_cast<const half8_t *>(&lds_b[nb][fb0 + i * 32 * ROWH + ko[0]]);
        }
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
          for (int j = 0; j < 4; j++) acc[i][j] = mfma_32x32x16(fa[p][i], fb[p][j], acc[i][j]);
#pragma unroll
        for (int t = 0; t < 8; t++) {
          sched_group<kSchedDsRead, 1>();
          sched_group<kSchedMfma, 1>();
        }
        sched_fence();
#pragma unroll
        for (int t = 0; t < 8; t++) {
          const int i = 2 + t / 4, j = t % 4;
          issue_b(s + 2, cb, t);
          acc[i][j] = mfma_32x32x16(fa[p][i], fb[p][j], acc[i][j]);
          sched_fence();
        }
      }
    }
    ca = na;
    cb = nb;
  }
  wait_vector_loads<0>();  // the re-reads past the last step must land before the block's LDS is released
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) gemm_store_tile(D, C, N, tile_m * kGemmBigBM + wm * 128 + i * 32, tile_n * kGemmBigBN + wn * 128 + j * 32, acc[i][j], lane, alpha, beta);
}

// Epilogue of a 128-column strip of 16 x 16 tiles whose accumulators came from mfma_16x16x32
// with the B fragment as the first operand (the product is formed transposed): the lane owns
// row (lane & 15) and the four adjacent columns 4 * (lane >> 4) .. + 3 of every tile, i.e. one
// 128-bit (fp32) or 64-bit (fp16) access per tile.  CRow16 holds a lane's C values of one row
// of eight tiles.
template <typename OUT, int W8>
struct CRow16 {
  using word_t = typename std::conditional<sizeof(OUT) == 4, float4_t, uint2_t>::type;
  word_t v[W8];
};
template <typename OUT, int W8>
TCU_DEVICE void gemm_load_c_row16(CRow16<OUT, W8> &c, const OUT *C, size_t ldc, size_t row0, size_t col0, int lane) {
  using word_t = typename CRow16<OUT, W8>::word_t;
  const word_t *p = reinterpret_cast<const word_t *>(C + (row0 + (lane & 15)) * ldc + col0 + 4 * (lane >> 4));
#pragma unroll
  for (int j = 0; j < W8; j++) c.v[j] = __builtin_nontemporal_load(p + j * 4);
}
// D = alpha * acc + beta * c for one row of W8 tiles; c is not read when beta == 0
template <typename OUT, int W8>
TCU_DEVICE void gemm_store_row16(OUT *D, size_t ldc, size_t row0, size_t col0, const float4_t (&acc)[W8], const CRow16<OUT, W8> &c, int lane, float alpha, float beta) {
  using word_t = typename CRow16<OUT, W8>::word_t;
  word_t *p = reinterpret_cast<word_t *>(D + (row0 + (lane & 15)) * ldc + col0 + 4 * (lane >> 4));
#pragma unroll
  for (int j = 0; j < W8; j++) {
    float4_t r = alpha * acc[j];
    if constexpr (sizeof(OUT) == 4) {
      if (beta != 0.0f) r = gemm_axpby(alpha, acc[j], beta, c.v[j]);
      __builtin_nontemporal_store(r, p + j * 4);
    } else {
      if (beta != 0.0f) {
        const uint32_t w01 = c.v[j][0], w23 = c.v[j][1];  // scalars first: a bit cast straight from a vector element reads element 0
        const half2_t c01 = __builtin_bit_cast(half2_t, w01), c23 = __builtin_bit_cast(half2_t, w23);
        r = gemm_axpby(alpha, acc[j], beta, float4_t{(float)c01[0], (float)c01[1], (float)c23[0], (float)c23[1]});
      }
      uint2_t v;
      v[0] = pack_f16x2(r[0], r[1]);
      v[1] = pack_f16x2(r[2], r[3]);
      __builtin_nontemporal_store(v, p + j * 4);
    }
  }
}
// The whole strip: W8 rows of W8 tiles, each row's C values read just before its stores (C may
// be the same buffer as D: a lane reads only elements it will itself write).  Reading one to
// three rows ahead of the stores measured the same or up to 1 % slower (8192^3, same run).
template <typename OUT, int W8>
TCU_DEVICE void gemm_store_strip16(OUT *D, const OUT *C, size_t ldc, size_t row0, size_t col0, const float4_t (&acc)[W8][W8], int lane, float alpha, float beta) {
#pragma unroll
  for (int i = 0; i < W8; i++) {
    CRow16<OUT, W8> c;
    if (beta != 0.0f) gemm_load_c_row16(c, C, ldc, row0 + i * 16, col0, lane);
    gemm_store_row16(D, ldc, row0 + i * 16, col0, acc[i], c, lane, alpha, beta);
  }
}

// The same strip with every row of tiles turned through LDS first, so that global memory sees whole rows: a
// row of W8 tiles is 16 rows of 16 * W8 outputs; the lanes park alpha * acc in `stage` (two buffers of
// gemm_stage_row_floats(W8) * 16 floats per wave, rows padded by four floats), and read it back with consecutive
// lanes along a row.  W8 = 8: 32 lanes x 4 fp32 outputs (512 bytes of one row, two rows per instruction) or 16 lanes
// x 8 fp16 outputs (256 bytes, four rows per instruction); W8 = 4: 256 bytes of four rows or 128 bytes of eight;
// the direct form writes 64 / 32 bytes of 16 rows per instruction.  C is read in the same shape, by the lane that
// writes the same elements of D.
constexpr int gemm_stage_row_floats(int w8) { return 16 * w8 + 4; }
constexpr int gemm_stage_wave_floats(int w8) { return 2 * 16 * gemm_stage_row_floats(w8); }
template <typename OUT, int W8>
TCU_DEVICE void gemm_store_strip16_staged(OUT *D, const OUT *C, size_t ldc, size_t row0, size_t col0, const float4_t (&acc)[W8][W8], int lane, float alpha, float beta, float *stage) {
  constexpr int kStageRowFloats = gemm_stage_row_floats(W8);
  constexpr int PER_LANE = sizeof(OUT) == 4 ? 4 : 8;       // outputs per lane and access (16 bytes)
  constexpr int LANES_PER_ROW = 16 * W8 / PER_LANE;        // W8 = 8: 32 or 16; W8 = 4: 16 or 8; W8 = 6: 24 or 12
  constexpr int ROWS_PER_ACCESS = 64 / LANES_PER_ROW >= 8 ? 8 : 64 / LANES_PER_ROW >= 4 ? 4 : 2;  // 2 or 4; 4 or 8; 2 or 4
  constexpr int ACCESSES = 16 / ROWS_PER_ACCESS;           // per row of tiles: 8 or 4; 4 or 2; 8 or 4
  constexpr int ACTIVE = ROWS_PER_ACCESS * LANES_PER_ROW;  // lanes that move outputs: all 64, or 48 of them where W8 = 6
  using word_t = typename std::conditional<sizeof(OUT) == 4, float4_t, uint4_t>::type;
  const int wr = lane & 15, wq = lane >> 4;  // accumulator layout: row, group of four columns
  const bool active = ACTIVE == 64 || lane < ACTIVE;
  const int rr = active ? lane / LANES_PER_ROW : 0, rc = (lane % LANES_PER_ROW) * PER_LANE;  // an idle lane keeps its addresses inside the tile
  const size_t at0 = (row0 + rr) * ldc + col0 + rc;  // access t of row of tiles i: at0 + (16 i + ROWS_PER_ACCESS t) * ldc
  // the C values of a row of tiles are requested one row of tiles ahead, all at once (one wait per load would
  // leave the epilogue bound by latency); C may be D: a lane reads only what it will itself write, rows later
  word_t c[2][ACCESSES];
  if (beta != 0.0f && active) {
#pragma unroll
    for (int t = 0; t < ACCESSES; t++) c[0][t] = __builtin_nontemporal_load(reinterpret_cast<const word_t *>(C + at0 + (size_t)(ROWS_PER_ACCESS * t) * ldc));
  }
#pragma unroll
  for (int i = 0; i < W8; i++) {
    float *buf = stage + (i & 1) * (16 * kStageRowFloats);
    if (beta != 0.0f && i + 1 < W8 && active) {
#pragma unroll
      for (int t = 0; t < ACCESSES; t++) c[(i + 1) & 1][t] = __builtin_nontemporal_load(reinterpret_cast<const word_t *>(C + at0 + (size_t)(16 * (i + 1) + ROWS_PER_ACCESS * t) * ldc));
    }
#pragma unroll
    for (int j = 0; j < W8; j++) *reinterpret_cast<float4_t *>(buf + wr * kStageRowFloats + 16 * j + 4 * wq) = alpha * acc[i][j];
    wave_lds_fence();
    if (active) {
#pragma unroll
    for (int t = 0; t < ACCESSES; t++) {
      const int r = t * ROWS_PER_ACCESS + rr;
      word_t *d = reinterpret_cast<word_t *>(D + at0 + (size_t)(16 * i + ROWS_PER_ACCESS * t) * ldc);
      float4_t v0 = *reinterpret_cast<const float4_t *>(buf + r * kStageRowFloats + rc);
      if constexpr (sizeof(OUT) == 4) {
        if (beta != 0.0f) v0 = gemm_add_scaled(v0, beta, c[i & 1][t]);
        __builtin_nontemporal_store(v0, d);
      } else {
        float4_t v1 = *reinterpret_cast<const float4_t *>(buf + r * kStageRowFloats + rc + 4);
        if (beta != 0.0f) {
          const uint32_t w0 = c[i & 1][t][0], w1 = c[i & 1][t][1], w2 = c[i & 1][t][2], w3 = c[i & 1][t][3];  // scalars first: a bit cast straight from a vector element reads element 0
          const half2_t c0 = __builtin_bit_cast(half2_t, w0), c1 = __builtin_bit_cast(half2_t, w1), c2 = __builtin_bit_cast(half2_t, w2), c3 = __builtin_bit_cast(half2_t, w3);
          v0 = gemm_add_scaled(v0, beta, float4_t{(float)c0[0], (float)c0[1], (float)c1[0], (float)c1[1]});
          v1 = gemm_add_scaled(v1, beta, float4_t{(float)c2[0], (float)c2[1], (float)c3[0], (float)c3[1]});
        }
        uint4_t o;
        o[0] = pack_f16x2(v0[0], v0[1]);
        o[1] = pack_f16x2(v0[2], v0[3]);
        o[2] = pack_f16x2(v1[0], v1[1]);
        o[3] = pack_f16x2(v1[2], v1[3]);
        __builtin_nontemporal_store(o, d);
      }
    }
    }
  }
}

// gemm_dlds_a3b2_kernel on v_mfma_f32_16x16x32_f16: the same block tile, buffers and transfer
// schedule, but a wave's 128 x 128 tile is 8 x 8 accumulators of 16 x 16 and a K step of 64 is
// two substeps of 32, each 16 fragment reads for 64 MFMAs.  Per multiply-add this shape reads
// the A/B fragment registers twice as often and the accumulator registers half as often as
// 32x32x16; the accumulators being four times as many words, the register traffic is lower,
// and so is the power: with operands held in registers the chip sustains 1865 TFLOP/s in this
// shape against 1600 in the other (normally distributed inputs, 40 ms launches), and the
// kernel is limited by power, not by issue slots.  C and D must be aligned to four outputs
// (16 bytes of fp32, 8 of fp16).
// One tile (or, with share != nullptr, the K steps step0 .. step0 + steps - 1 of one tile, whose raw fp32
// accumulators go to `share` as a 256 x 256 row-major tile).  May be called several times by a block:
// every wave waits for its own transfers before it leaves, and nothing reads LDS after the last barrier.
// W8 = 8: the 256 x 256 block tile; W8 = 4: a 128 x 128 block tile (waves of 64 x 64 = 4 x 4 accumulators, 80 KiB of
// LDS, two blocks per compute unit), for outputs too small to fill the chip with the big tiles; W8 = 6: a 192 x 192
// block tile (waves of 96 x 96, 120 KiB of LDS), for outputs that 256 x 256 tiles cut into much less than a round of
// the chip and 192 x 192 tiles into about one (3072^2: 144 against 256 tiles on 256 compute units).
template <typename OUT, bool STAGED, int W8 = 8>
TCU_DEVICE void gemm_a3b2_m16_tile(const half8_t *__restrict__ A, const half8_t *__restrict__ B, const OUT *C, OUT *D, size_t N, size_t K, size_t tile_m, size_t tile_n, size_t step0, size_t steps,
                                   float *share, float alpha, float beta) {
  constexpr int BK = 64, ROWH = BK, CPR = 8, RPT = 8, RS = 1, SUB = 2, NA = 3, NB = 2;
  constexpr int TILE = 32 * W8, WT = 16 * W8;  // block tile, wave tile
  constexpr int NM = W8 * W8;                  // MFMAs per substep
  constexpr int OPH = TILE * ROWH;             // halves per operand per stage
  constexpr int TPW = TILE / RPT / 4;          // transfer instructions per wave, operand and step (8 or 4)
  constexpr int TEVERY = NM / 2 / TPW;         // one transfer every so many MFMAs of a substep's second half
  static_assert(W8 == 8 || W8 == 6 || W8 == 4, "fragment reads (one before every other MFMA) and transfers must fit a substep");
  static_assert(4 * W8 <= NM && (NM / 2) % TPW == 0, "fragment reads and transfers per substep");
  __shared__ __attribute__((aligned(1024))) half_t lds_a[NA][OPH];
  __shared__ __attribute__((aligned(1024))) half_t lds_b[NB][OPH];
  const int tid = (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const size_t k_chunks = K / 8;
  uint32_t goff[TPW];
#pragma unroll
  for (int t = 0; t < TPW; t++) {
    const int row = (wave * TPW + t) * RPT + lane / CPR;
    const int chunk = (lane % CPR) ^ ((row >> RS) & (CPR - 1));
    goff[t] = (uint32_t)(((size_t)row * k_chunks + chunk) * 16);
  }
  constexpr lds_addr_t STAGE = OPH * 2, TBYTES = 1024, STEPB = BK * 2;
  const char *ga = reinterpret_cast<const char *>(A + tile_m * TILE * k_chunks) + step0 * STEPB;
  const char *gb = reinterpret_cast<const char *>(B + tile_n * TILE * k_chunks) + step0 * STEPB;
  const lds_addr_t ta = wave_uniform(lds_address_of(&lds_a[0][0]) + wave * TPW * TBYTES);
  const lds_addr_t tb = wave_uniform(lds_address_of(&lds_b[0][0]) + wave * TPW * TBYTES);
  auto issue_a = [&](size_t step, int buf, int t) { load_chunk_to_lds(ga + (step < steps ? step : steps - 1) * STEPB, goff[t], ta + buf * STAGE + t * TBYTES); };
  auto issue_b = [&](size_t step, int buf, int t) { load_chunk_to_lds(gb + (step < steps ? step : steps - 1) * STEPB, goff[t], tb + buf * STAGE + t * TBYTES); };

  float4_t acc[W8][W8];
#pragma unroll
  for (int i = 0; i < W8; i++)
#pragma unroll
    for (int j = 0; j < W8; j++)
#pragma unroll
      for (int e = 0; e < 4; e++) acc[i][j][e] = 0.0f;

  // in flight at the first barrier: A0 B0 | A1 B1 (the wave's counter returns in issue order)
#pragma unroll
  for (int t = 0; t < TPW; t++) issue_a(0, 0, t);
#pragma unroll
  for (int t = 0; t < TPW; t++) issue_b(0, 0, t);
#pragma unroll
  for (int t = 0; t < TPW; t++) issue_a(1, 1, t);
#pragma unroll
  for (int t = 0; t < TPW; t++) issue_b(1, 1, t);
  wait_vector_loads<2 * TPW>();
  block_barrier_lds_only();

  // fragment of row r, k chunk kc: slot kc ^ f(r); the lane supplies row (lane & 15) of a
  // 16-row tile and chunk (lane >> 4) of the substep's four; rows of a lane differ by multiples of 16
  const int frow = lane & 15, kq = lane >> 4, fsw = (frow >> RS) & (CPR - 1);
  const int fa0 = (wm * WT + frow) * ROWH, fb0 = (wn * WT + frow) * ROWH;
  int ko[SUB];
#pragma unroll
  for (int kk = 0; kk < SUB; kk++) ko[kk] = ((4 * kk + kq) ^ fsw) * 8;
  half8_t fa[2][W8], fb[2][W8];
#pragma unroll
  for (int i = 0; i < W8; i++) {
    fa[0][i] = *reinterpret_cast<const half8_t *>(&lds_a[0][fa0 + i * 16 * ROWH + ko[0]]);
    fb[0][i] = *reinterpret_cast<const half8_t *>(&lds_b[0][fb0 + i * 16 * ROWH + ko[0]]);
  }
  int ca = 0, cb = 0;  // s % NA, s % NB
  for (size_t s = 0; s < steps; s++) {
    const int na = ca + 1 == NA ? 0 : ca + 1, nb = cb ^ 1;
    const int fill_a = ca == 0 ? NA - 1 : ca - 1;  // A buffer of step s - 1 = of step s + 2
    // substep 0: MFMA t works on tile (t / W8, t % W8); fragment k of substep 1 (order: A0 B0..B7 A1..A7 for
    // W8 = 8) is read before MFMA 2k
#pragma unroll
    for (int t = 0; t < NM; t++) {
      if (t < 4 * W8 && t % 2 == 0) {
        const int k = t / 2;
        if (k == 0) fa[1][0] = *reinterpret_cast<const half8_t *>(&lds_a[ca][fa0 + ko[1]]);
        else if (k <= W8) fb[1][k - 1] = *reinterpret_cast<const half8_t *>(&lds_b[cb][fb0 + (k - 1) * 16 * ROWH + ko[1]]);
        else fa[1][k - W8] = *reinterpret_cast<const half8_t *>(&lds_a[ca][fa0 + (k - W8) * 16 * ROWH + ko[1]]);
      }
      if (t >= NM / 2 && (t - NM / 2) % TEVERY == 0) issue_a(s + 2, fill_a, (t - NM / 2) / TEVERY);  // A tile of step s + 2 under the second half
      acc[t / W8][t % W8] = mfma_16x16x32(fb[0][t % W8], fa[0][t / W8], acc[t / W8][t % W8]);
      sched_fence();
    }
    // substep 1: own transfers of step s + 1 done (the A tile of step s + 2 may still fly), barrier,
    // fragments of step s + 1.  (Measured and dropped: the B tile under the first half of this
    // substep, and the A tile a substep earlier, three steps ahead: 0-2 % slower.)
    wait_vector_loads<TPW>();
    block_barrier_lds_only();
    sched_fence();
#pragma unroll
    for (int t = 0; t < NM; t++) {
      if (t < 4 * W8 && t % 2 == 0) {
        const int k = t / 2;
        if (k == 0) fa[0][0] = *reinterpret_cast<const half8_t *>(&lds_a[na][fa0 + ko[0]]);
        else if (k <= W8) fb[0][k - 1] = *reinterpret_cast<const half8_t *>(&lds_b[nb][fb0 + (k - 1) * 16 * ROWH + ko[0]]);
        else fa[0][k - W8] = *reinterpret_cast<const half8_t *>(&lds_a[na][fa0 + (k - W8) * 16 * ROWH + ko[0]]);
      }
      if (t >= NM / 2 && (t - NM / 2) % TEVERY == 0) issue_b(s + 2, cb, (t - NM / 2) / TEVERY);  // B tile of step s + 2 into the B buffer of step s
      acc[t / W8][t % W8] = mfma_16x16x32(fb[1][t % W8], fa[1][t / W8], acc[t / W8][t % W8]);
      sched_fence();
    }
    ca = na;
    cb = nb;
  }
  wait_vector_loads<0>();  // the re-reads past the last step must land before the block's LDS is released
  constexpr int kStageWaveFloats = gemm_stage_wave_floats(W8);
  if (share != nullptr) {
    if constexpr (STAGED) {  // raw accumulators, whole rows of the TILE x TILE share (it is 16-byte aligned)
      block_barrier_lds_only();
      gemm_store_strip16_staged<float>(share, nullptr, TILE, wm * WT, wn * WT, acc, lane, 1.0f, 0.0f, reinterpret_cast<float *>(&lds_a[0][0]) + wave * kStageWaveFloats);
      block_barrier_lds_only();  // the block's next piece of work starts its transfers only after every wave has read its outputs back
    } else {
      gemm_store_strip16<float>(share, nullptr, TILE, wm * WT, wn * WT, acc, lane, 1.0f, 0.0f);
    }
  } else if constexpr (STAGED) {
    block_barrier_lds_only();  // the other waves have read their last fragments: the A buffers can hold outputs now
    static_assert(4 * kStageWaveFloats * sizeof(float) <= sizeof(lds_a), "staging area of four waves");
    gemm_store_strip16_staged(D, C, N, tile_m * TILE + wm * WT, tile_n * TILE + wn * WT, acc, lane, alpha, beta, reinterpret_cast<float *>(&lds_a[0][0]) + wave * kStageWaveFloats);
    block_barrier_lds_only();  // a block that goes on to another piece of work starts its transfers only after every wave has read its outputs back
  } else {
    gemm_store_strip16(D, C, N, tile_m * TILE + wm * WT, tile_n * TILE + wn * WT, acc, lane, alpha, beta);
  }
}

// The same loop on 192 x 192 block tiles (M and N multiples of 192, K of 64, C and D aligned to four outputs): one tile
// per block, one block per compute unit.
template <typename OUT, bool STAGED>
__global__ __launch_bounds__(256) void gemm_dlds_a3b2_m16_t192_kernel(const half8_t *__restrict__ A, const half8_t *__restrict__ B, const OUT *C, OUT *D, size_t M, size_t N, size_t K, float alpha, float beta) {
  size_t tile_m, tile_n;
  gemm_tile_of_block(M / 192, N / 192, blockIdx.x, &tile_m, &tile_n);
  gemm_a3b2_m16_tile<OUT, STAGED, 6>(A, B, C, D, N, K, tile_m, tile_n, 0, K / 64, static_cast<float *>(nullptr), alpha, beta);
}

// The same loop on 128 x 128 block tiles (M and N multiples of 128, K of 64, C and D aligned to four outputs): one tile
// per block, two blocks per compute unit.
template <typename OUT, bool STAGED>
__global__ __launch_bounds__(256, 2) void gemm_dlds_a3b2_m16_t128_kernel(const half8_t *__restrict__ A, const half8_t *__restrict__ B, const OUT *C, OUT *D, size_t M, size_t N, size_t K, float alpha, float beta) {
  size_t tile_m, tile_n;
  gemm_tile_of_block(M / 128, N / 128, blockIdx.x, &tile_m, &tile_n);
  gemm_a3b2_m16_tile<OUT, STAGED, 4>(A, B, C, D, N, K, tile_m, tile_n, 0, K / 64, static_cast<float *>(nullptr), alpha, beta);
}

// Blocks 0 .. full_tiles-1 take one tile each.  With T tiles on a chip that runs `units` blocks at a
// time, the last T % units tiles would cost a whole round of the kernel's time however few they are:
// their K steps, laid end to end (tile after tile), are instead cut into runs of `run` steps, one per
// block of the rest of the grid, so that every compute unit gets the same share of the tail.  A run
// covers the end of one tile and the start of the next at most (run <= K steps per tile); block j of
// the tail stores its raw accumulators for the two at ws + (2 j + 0 or 1) * 65536 floats, and
// gemm_split_fixup_kernel adds the shares of a tile in a fixed order and applies alpha, beta and C.
// full_tiles = grid size turns this off.
template <typename OUT, bool STAGED = false>
__global__ __launch_bounds__(256) void gemm_dlds_a3b2_m16_kernel(const half8_t *__restrict__ A, const half8_t *__restrict__ B, const OUT *C, OUT *D, size_t M, size_t N, size_t K, float alpha, float beta,
                                                                 unsigned full_tiles, unsigned run, float *ws) {
  const size_t tiles_m = M / kGemmBigBM, tiles_n = N / kGemmBigBN, steps = K / 64;
  size_t tile_m, tile_n;
  if (blockIdx.x < full_tiles) {  // block-uniform
    gemm_tile_of_block(tiles_m, tiles_n, blockIdx.x, &tile_m, &tile_n);
    gemm_a3b2_m16_tile<OUT, STAGED>(A, B, C, D, N, K, tile_m, tile_n, 0, steps, static_cast<float *>(nullptr), alpha, beta);
    return;
  }
  const size_t j = blockIdx.x - full_tiles, total = (tiles_m * tiles_n - full_tiles) * steps;
  size_t at = j * run;
  const size_t end = at + run < total ? at + run : total;
  for (int part = 0; at < end; part++) {
    const size_t t = at / steps, k0 = at % steps;
    const size_t len = end - at < steps - k0 ? end - at : steps - k0;
    gemm_tile_of_block(tiles_m, tiles_n, full_tiles + t, &tile_m, &tile_n);
    gemm_a3b2_m16_tile<OUT, STAGED>(A, B, C, D, N, K, tile_m, tile_n, k0, len, ws + (2 * j + part) * (size_t)(kGemmBigBM * kGemmBigBN), alpha, beta);
    at += len;
  }
}

// Second half of the K-split tail: tail tile t (tile id full_tiles + t) = alpha * (sum of its shares, in a
// fixed order) + beta * C.  One thread per four adjacent outputs, 64 blocks of 256 threads per tile.
template <typename OUT>
__global__ __launch_bounds__(256) void gemm_split_fixup_kernel(const float *__restrict__ ws, const OUT *C, OUT *D, size_t M, size_t N, size_t K, float alpha, float beta, unsigned full_tiles, unsigned run) {
  const size_t t = blockIdx.x / 64, steps = K / 64;
  const int row = (int)(blockIdx.x % 64) * 4 + (int)(threadIdx.x >> 6), col = (int)(threadIdx.x & 63) * 4;
  size_t tile_m, tile_n;
  gemm_tile_of_block(M / kGemmBigBM, N / kGemmBigBN, full_tiles + t, &tile_m, &tile_n);
  const size_t first = t * steps / run, last = ((t + 1) * steps - 1) / run;  // blocks of the tail with a share of this tile
  // only block `first` can have begun in the previous tile (this tile is then the second it touches); four
  // independent partial sums keep four loads in flight, combined in a fixed order
  constexpr size_t SHARE = (size_t)kGemmBigBM * kGemmBigBN;
  const float *p = ws + (size_t)row * kGemmBigBN + col;
  float4_t s0 = *reinterpret_cast<const float4_t *>(p + (2 * first + (first * run < t * steps ? 1 : 0)) * SHARE);
  float4_t s1 = {0.0f, 0.0f, 0.0f, 0.0f}, s2 = s1, s3 = s1;
  size_t j = first + 1;
  for (; j + 3 <= last; j += 4) {
    s1 += *reinterpret_cast<const float4_t *>(p + 2 * j * SHARE);
    s2 += *reinterpret_cast<const float4_t *>(p + 2 * (j + 1) * SHARE);
    s3 += *reinterpret_cast<const float4_t *>(p + 2 * (j + 2) * SHARE);
    s0 += *reinterpret_cast<const float4_t *>(p + 2 * (j + 3) * SHARE);
  }
  for (; j <= last; j++) s1 += *reinterpret_cast<const float4_t *>(p + 2 * j * SHARE);
  const float4_t sum = (s0 + s1) + (s2 + s3);
  const size_t o = (tile_m * kGemmBigBM + row) * N + tile_n * kGemmBigBN + col;
  float4_t r = alpha * sum;
  if constexpr (sizeof(OUT) == 4) {
    if (beta != 0.0f) r = gemm_axpby(alpha, sum, beta, *reinterpret_cast<const float4_t *>(C + o));
    *reinterpret_cast<float4_t *>(D + o) = r;
  } else {
    if (beta != 0.0f) {
      const uint2_t c = *reinterpret_cast<const uint2_t *>(C + o);
      const uint32_t w01 = c[0], w23 = c[1];
      const half2_t c01 = __builtin_bit_cast(half2_t, w01), c23 = __builtin_bit_cast(half2_t, w23);
      r = gemm_axpby(alpha, sum, beta, float4_t{(float)c01[0], (float)c01[1], (float)c23[0], (float)c23[1]});
    }
    uint2_t v;
    v[0] = pack_f16x2(r[0], r[1]);
    v[1] = pack_f16x2(r[2], r[3]);
    *reinterpret_cast<uint2_t *>(D + o) = v;
  }
}

// M % 32 == 0, N % 32 == 0, K % 16 == 0; one 32 x 32 tile per wave.
template <typename OUT>
__global__ __launch_bounds__(kWave * 4) void gemm_direct_kernel(const half8_t *__restrict__ A, const half8_t *__restrict__ B, const OUT *C, OUT *D, size_t M, size_t N, size_t K, float alpha,
                                                                 float beta) {
  const int lane = lane_id();
  const size_t tiles_m = M / 32, tiles_n = N / 32;
  const size_t tile = (size_t)blockIdx.x * (blockDim.x >> 6) + wave_in_block();
  if (tile >= tiles_m * tiles_n) return;
  const size_t tile_m = tile % tiles_m, tile_n = tile / tiles_m;
  const size_t k_chunks = K / 8;
  const half8_t *ga = A + (tile_m * 32 + (lane & 31)) * k_chunks + (lane >> 5);
  const half8_t *gb = B + (tile_n * 32 + (lane & 31)) * k_chunks + (lane >> 5);
  float16_t acc;
#pragma unroll
  for (int e = 0; e < 16; e++) acc[e] = 0.0f;
  for (size_t c = 0; c < k_chunks; c += 2) acc = mfma_32x32x16(ga[c], gb[c], acc);
  gemm_store_tile(D, C, N, tile_m * 32, tile_n * 32, acc, lane, alpha, beta);
}

template <typename OUT>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const uint16_t *__restrict__ A, const uint16_t *__restrict__ B, const OUT *C, OUT *D, size_t M, size_t N, size_t K, float alpha,
                                                            float beta) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= M * N) return;
  const size_t m = idx / N, n = idx % N;
  float acc = 0.0f;
  for (size_t k = 0; k < K; k++) acc += (float)__builtin_bit_cast(half_t, A[m * K + k]) * (float)__builtin_bit_cast(half_t, B[n * K + k]);
  D[idx] = (OUT)(beta == 0.0f ? alpha * acc : gemm_axpby(alpha, acc, beta, (float)C[idx]));
}

}  // namespace tcu
