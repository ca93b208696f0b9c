// GEMM / GEMV benchmarks under the reference's names (src/gemm/wmma.cu:776-777,
// wmma_naive.cu:339-340, wmma_sharedmem.cu, src/gemv/wmma_naive.cu:357-358, wmma_sharedmem.cu;
// the H* names keep C, D or y in fp16), the accuracy comparisons (src/gemm/accuracy.cu:277,
// src/gemv/accuracy.cu:332) and the timed CPU path.
#include "args.hpp"
#include "harness.hpp"

static void CUDA_WMMA_GEMM(benchmark::State &state) { harness::run_gemm(state, TCU_VARIANT_BLOCK_LDS, "CUDA_WMMA_GEMM"); }
static void CUDA_WMMA_GEMM_SHAREDMEM(benchmark::State &state) { harness::run_gemm(state, TCU_VARIANT_BLOCK_LDS, "CUDA_WMMA_GEMM_SHAREDMEM"); }
static void CUDA_WMMA_GEMM_NAIVE(benchmark::State &state) { harness::run_gemm(state, TCU_VARIANT_MFMA_16N, "CUDA_WMMA_GEMM_NAIVE"); }
static void CUDA_WMMA_HGEMM(benchmark::State &state) { harness::run_gemm(state, TCU_VARIANT_BLOCK_LDS, "CUDA_WMMA_HGEMM", true); }
static void CUDA_WMMA_HGEMM_NAIVE(benchmark::State &state) { harness::run_gemm(state, TCU_VARIANT_MFMA_16N, "CUDA_WMMA_HGEMM_NAIVE", true); }
static void CUDA_WMMA_GEMM_ACCURACY(benchmark::State &state) { harness::run_gemm_accuracy(state, "CUDA_WMMA_GEMM_ACCURACY"); }
BENCHMARK(CUDA_WMMA_GEMM)->Apply(GemmArgs)->UseManualTime();
BENCHMARK(CUDA_WMMA_HGEMM)->Apply(GemmArgs)->UseManualTime();
BENCHMARK(CUDA_WMMA_HGEMM_NAIVE)->Apply(GemmArgs)->UseManualTime();
BENCHMARK(CUDA_WMMA_GEMM_ACCURACY)->Apply(GemmArgs)->UseManualTime();
BENCHMARK(CUDA_WMMA_GEMM_SHAREDMEM)->Apply(GemmArgs)->UseManualTime();
BENCHMARK(CUDA_WMMA_GEMM_NAIVE)->Apply(GemmArgs)->UseManualTime();

static void CUDA_WMMA_GEMV_NAIVE(benchmark::State &state) { harness::run_gemv(state, TCU_VARIANT_MFMA_16N, "CUDA_WMMA_GEMV_NAIVE"); }
// the reference's second GEMV kernel stages tiles through shared memory to make its loads contiguous
// (src/gemv/wmma_sharedmem.cu:43-137); the MFMA form with contiguous loads here is the trace form
static void CUDA_WMMA_GEMV_SHAREDMEM(benchmark::State &state) { harness::run_gemv(state, TCU_VARIANT_MFMA_256N, "CUDA_WMMA_GEMV_SHAREDMEM"); }
static void TCU_WAVE_GEMV(benchmark::State &state) { harness::run_gemv(state, TCU_VARIANT_WAVE_SHUFFLE, "TCU_WAVE_GEMV"); }
static void CUDA_WMMA_HGEMV_NAIVE(benchmark::State &state) { harness::run_gemv(state, TCU_VARIANT_MFMA_16N, "CUDA_WMMA_HGEMV_NAIVE", true); }
static void TCU_WAVE_HGEMV(benchmark::State &state) { harness::run_gemv(state, TCU_VARIANT_WAVE_SHUFFLE, "TCU_WAVE_HGEMV", true); }
static void CUDA_WMMA_GEMV_ACCURACY(benchmark::State &state) { harness::run_gemv_accuracy(state, "CUDA_WMMA_GEMV_ACCURACY"); }
BENCHMARK(CUDA_WMMA_GEMV_NAIVE)->Apply(GemvArgs)->UseManualTime();
BENCHMARK(CUDA_WMMA_HGEMV_NAIVE)->Apply(GemvArgs)->UseManualTime();
BENCHMARK(TCU_WAVE_HGEMV)->Apply(GemvArgs)->UseManualTime();
BENCHMARK(CUDA_WMMA_GEMV_ACCURACY)->Apply(GemvArgs)->UseManualTime();
BENCHMARK(CUDA_WMMA_GEMV_SHAREDMEM)->Apply(GemvArgs)->UseManualTime();
BENCHMARK(TCU_WAVE_GEMV)->Apply(GemvArgs)->UseManualTime();
// the same product with A in the reference's own layout (column-major, lda = M: src/gemv/wmma_naive.cu:33-36)
static void TCU_COL_MAJOR_GEMV(benchmark::State &state) { harness::run_gemv(state, TCU_VARIANT_AUTO, "TCU_COL_MAJOR_GEMV", false, true); }
static void TCU_COL_MAJOR_HGEMV(benchmark::State &state) { harness::run_gemv(state, TCU_VARIANT_AUTO, "TCU_COL_MAJOR_HGEMV", true, true); }
BENCHMARK(TCU_COL_MAJOR_GEMV)->Apply(GemvArgs)->UseManualTime();
BENCHMARK(TCU_COL_MAJOR_HGEMV)->Apply(GemvArgs)->UseManualTime();

// The reference's CPU verification loop as a benchmark: N = 2^20 in segments of 16 (seed 0),
// one thread (as the reference wrote it) and all host threads.
static void CPU_SEQUENTIAL_SEGMENTED_REDUCTION(benchmark::State &state) { harness::run_cpu_segmented(state, false, 1); }
static void CPU_THREADED_SEGMENTED_REDUCTION(benchmark::State &state) { harness::run_cpu_segmented(state, false, 0); }
static void CPU_SEQUENTIAL_SEGMENTED_PREFIXSUM(benchmark::State &state) { harness::run_cpu_segmented(state, true, 1); }
static void CPU_THREADED_SEGMENTED_PREFIXSUM(benchmark::State &state) { harness::run_cpu_segmented(state, true, 0); }
static void CpuArgs(benchmark::internal::Benchmark *b) {
  b->Args({65536, 16, 1 << 20});
  for (int64_t seg : {16, 256, 1024, 4096, 16384}) b->Args({(int64_t(1) << 26) / seg, seg, int64_t(1) << 26});
  b->ArgNames({"num_segments", "segment_size", "num_elements"});
}
BENCHMARK(CPU_SEQUENTIAL_SEGMENTED_REDUCTION)->Apply(CpuArgs)->UseManualTime();
BENCHMARK(CPU_THREADED_SEGMENTED_REDUCTION)->Apply(CpuArgs)->UseManualTime();
BENCHMARK(CPU_SEQUENTIAL_SEGMENTED_PREFIXSUM)->Apply(CpuArgs)->UseManualTime();
BENCHMARK(CPU_THREADED_SEGMENTED_PREFIXSUM)->Apply(CpuArgs)->UseManualTime();
