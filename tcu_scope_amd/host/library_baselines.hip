// Library comparators measured beside the hand-written kernels, under the names of the
// reference's library baselines: CUB_FULL_REDUCTION / CUB_FULL_PREFIXSUM
// (src/reduction/cub.cu, src/prefixsum/cub.cu: cub::DeviceReduce::Sum,
// cub::DeviceScan::InclusiveSum), CUB_DEVICE_SEGMENTED_REDUCTION and its TUNE sweep
// (src/reduction/seg_cub_device.cu:18-63: cub::DeviceSegmentedReduce::Sum over an offsets
// array), CUBLAS_WMMA_GEMM (src/gemm/cublas.cu:65: cublasGemmEx, fp16 in, fp32 out) and
// CUBLAS_GEMV.  Here they run hipCUB (rocPRIM) and rocBLAS, the libraries this GPU ships with;
// HIPBLASLT_GEMM / HIPBLASLT_HGEMM time the same products through hipBLASLt (hipblasLtMatmul with
// the algorithm its heuristic ranks first), the library PyTorch calls for fp16 matrix products.
// Nothing of the product calls these libraries; the file only feeds the benchmark executable.
// Arithmetic: the reductions and the scan read fp16, accumulate in fp32 and write fp16 (the
// reference's patched CUB adds in fp16), so they move the same bytes as the kernels they are
// compared with.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <hipblaslt/hipblaslt.h>
#include <hipcub/hipcub.hpp>
#include <rocblas/rocblas.h>

#include <vector>

#include "args.hpp"
#include "harness.hpp"

using harness::DeviceBuffer;
using harness::EventPair;

namespace {

struct HalfToFloat {
  __host__ __device__ float operator()(const __half &h) const { return __half2float(h); }
};
using HalfAsFloat = hipcub::TransformInputIterator<float, HalfToFloat, const __half *>;

// an fp16 destination that takes fp32 values (rocPRIM assigns its accumulator type to *out)
struct HalfOut {
  __half *p;
  struct Ref {
    __half *p;
    __host__ __device__ Ref &operator=(float v) {
      *p = __float2half(v);
      return *this;
    }
  };
  using iterator_category = std::random_access_iterator_tag;
  using value_type = float;
  using difference_type = std::ptrdiff_t;
  using pointer = void;
  using reference = Ref;
  __host__ __device__ Ref operator*() const { return Ref{p}; }
  __host__ __device__ Ref operator[](difference_type i) const { return Ref{p + i}; }
  __host__ __device__ HalfOut operator+(difference_type i) const { return HalfOut{p + i}; }
  __host__ __device__ HalfOut &operator+=(difference_type i) {
    p += i;
    return *this;
  }
};

template <class Body>
void guarded(benchmark::State &state, Body body) {
  try {
    body();
  } catch (const std::exception &e) {
    state.SkipWithError(e.what());
  } catch (...) {
    state.SkipWithError("unknown exception");
  }
}

template <class Launch>
void timed_loop(benchmark::State &state, Launch launch) {
  EventPair ev;
  size_t it = 0;
  // one untimed call first, as the harness gives the hand-written kernels: the first launch out of a code object loads it
  launch(it++);
  PRINT_IF_ERROR(hipDeviceSynchronize());
  for (auto _ : state) {
    ev.start();
    launch(it++);
    const float ms = ev.stop_ms();
    state.PauseTiming();
    state.SetIterationTime(ms / 1000);
    state.ResumeTiming();
  }
}

void counters(benchmark::State &state, size_t num_segments, size_t segment_size, size_t num_elements, double bytes) {
  state.counters.insert({{"num_segments", (double)num_segments},
                         {"segment_size", (double)segment_size},
                         {"num_elements", (double)num_elements},
                         {"flops", {state.iterations() * 1.0 * num_elements, benchmark::Counter::kAvgThreadsRate}},
                         {"bytes_per_second", {state.iterations() * bytes, benchmark::Counter::kAvgThreadsRate}},
                         {"hbm_peak_fraction", {state.iterations() * bytes / 8e12, benchmark::Counter::kAvgThreadsRate}}});
}

}  // namespace

static void CUB_FULL_REDUCTION(benchmark::State &state) {
  guarded(state, [&] {
    const size_t n = state.range(0);
    const int nin = n <= ((size_t)1 << 29) ? 2 : 1;
    DeviceBuffer in[2] = {DeviceBuffer(n * 2), DeviceBuffer(nin == 2 ? n * 2 : 16)};
    DeviceBuffer out(16);
    for (int i = 0; i < nin; i++) harness::fill_input(in[i].get(), n, harness::flags().seed + i);
    size_t temp_bytes = 0;
    HalfAsFloat src0(static_cast<const __half *>(in[0].get()), HalfToFloat());
    PRINT_IF_ERROR(hipcub::DeviceReduce::Sum(nullptr, temp_bytes, src0, HalfOut{static_cast<__half *>(out.get())}, (int)n));
    DeviceBuffer temp(temp_bytes ? temp_bytes : 16);
    timed_loop(state, [&](size_t it) {
      HalfAsFloat src(static_cast<const __half *>(in[it % nin].get()), HalfToFloat());
      PRINT_IF_ERROR(hipcub::DeviceReduce::Sum(temp.get(), temp_bytes, src, HalfOut{static_cast<__half *>(out.get())}, (int)n));
    });
    counters(state, 1, n, n, 2.0 * n);
  });
}
BENCHMARK(CUB_FULL_REDUCTION)->ARGS()->UseManualTime();

static void CUB_FULL_PREFIXSUM(benchmark::State &state) {
  guarded(state, [&] {
    const size_t n = state.range(0);
    const int nin = n <= ((size_t)1 << 29) ? 2 : 1;
    DeviceBuffer in[2] = {DeviceBuffer(n * 2), DeviceBuffer(nin == 2 ? n * 2 : 16)};
    DeviceBuffer out(n * 2);
    for (int i = 0; i < nin; i++) harness::fill_input(in[i].get(), n, harness::flags().seed + i);
    size_t temp_bytes = 0;
    HalfAsFloat src0(static_cast<const __half *>(in[0].get()), HalfToFloat());
    PRINT_IF_ERROR(hipcub::DeviceScan::InclusiveSum(nullptr, temp_bytes, src0, HalfOut{static_cast<__half *>(out.get())}, (int)n));
    DeviceBuffer temp(temp_bytes ? temp_bytes : 16);
    timed_loop(state, [&](size_t it) {
      HalfAsFloat src(static_cast<const __half *>(in[it % nin].get()), HalfToFloat());
      PRINT_IF_ERROR(hipcub::DeviceScan::InclusiveSum(temp.get(), temp_bytes, src, HalfOut{static_cast<__half *>(out.get())}, (int)n));
    });
    counters(state, 1, n, n, 4.0 * n);
  });
}
BENCHMARK(CUB_FULL_PREFIXSUM)->ARGS()->UseManualTime();

static void run_device_segmented_reduction(benchmark::State &state) {
  guarded(state, [&] {
    const size_t num_segments = state.range(0), segment_size = state.range(1), n = num_segments * segment_size;
    if (n >= ((size_t)1 << 31) || num_segments >= ((size_t)1 << 31)) {
      state.SkipWithError("offsets are 32-bit integers");
      return;
    }
    const int nin = n <= ((size_t)1 << 29) ? 2 : 1;
    DeviceBuffer in[2] = {DeviceBuffer(n * 2), DeviceBuffer(nin == 2 ? n * 2 : 16)};
    DeviceBuffer out(num_segments * 2), offsets((num_segments + 1) * sizeof(int));
    for (int i = 0; i < nin; i++) harness::fill_input(in[i].get(), n, harness::flags().seed + i);
    {
      std::vector<int> h(num_segments + 1);
      for (size_t j = 0; j <= num_segments; j++) h[j] = (int)(j * segment_size);
      PRINT_IF_ERROR(hipMemcpy(offsets.get(), h.data(), h.size() * sizeof(int), hipMemcpyHostToDevice));
    }
    const int *off = static_cast<const int *>(offsets.get());
    size_t temp_bytes = 0;
    HalfAsFloat src0(static_cast<const __half *>(in[0].get()), HalfToFloat());
    PRINT_IF_ERROR(hipcub::DeviceSegmentedReduce::Sum(nullptr, temp_bytes, src0, HalfOut{static_cast<__half *>(out.get())}, (int)num_segments, off, off + 1));
    DeviceBuffer temp(temp_bytes ? temp_bytes : 16);
    timed_loop(state, [&](size_t it) {
      HalfAsFloat src(static_cast<const __half *>(in[it % nin].get()), HalfToFloat());
      PRINT_IF_ERROR(hipcub::DeviceSegmentedReduce::Sum(temp.get(), temp_bytes, src, HalfOut{static_cast<__half *>(out.get())}, (int)num_segments, off, off + 1));
    });
    counters(state, num_segments, segment_size, n, 2.0 * n + 2.0 * num_segments + 4.0 * num_segments);
  });
}
static void CUB_DEVICE_SEGMENTED_REDUCTION(benchmark::State &state) { run_device_segmented_reduction(state); }
static void CUB_DEVICE_TUNE_SEGMENTED_REDUCTION(benchmark::State &state) { run_device_segmented_reduction(state); }
BENCHMARK(CUB_DEVICE_SEGMENTED_REDUCTION)->SEG_16_ARGS()->UseManualTime();
BENCHMARK(CUB_DEVICE_SEGMENTED_REDUCTION)->SEG_32_ARGS()->UseManualTime();
BENCHMARK(CUB_DEVICE_SEGMENTED_REDUCTION)->SEG_64_ARGS()->UseManualTime();
BENCHMARK(CUB_DEVICE_SEGMENTED_REDUCTION)->SEG_128_ARGS()->UseManualTime();
BENCHMARK(CUB_DEVICE_SEGMENTED_REDUCTION)->SEG_256_ARGS()->UseManualTime();
BENCHMARK(CUB_DEVICE_SEGMENTED_REDUCTION)->SEG_512_ARGS()->UseManualTime();
BENCHMARK(CUB_DEVICE_SEGMENTED_REDUCTION)->SEG_1024_ARGS()->UseManualTime();
BENCHMARK(CUB_DEVICE_SEGMENTED_REDUCTION)->SEG_2048_ARGS()->UseManualTime();
BENCHMARK(CUB_DEVICE_SEGMENTED_REDUCTION)->SEG_4096_ARGS()->UseManualTime();
BENCHMARK(CUB_DEVICE_SEGMENTED_REDUCTION)->SEG_8192_ARGS()->UseManualTime();
BENCHMARK(CUB_DEVICE_SEGMENTED_REDUCTION)->SEG_16384_ARGS()->UseManualTime();
// the reference registers the sweeps over 2^22 and 2^30 elements (src/reduction/seg_cub_device.cu:153-155) and its
// figure specifications also ask for 2^14, 2^18 and 2^26 (figures/spec/tune_segmented_reduction*.yml); 2^28 is what
// this build's measurements are quoted on
BENCHMARK(CUB_DEVICE_TUNE_SEGMENTED_REDUCTION)->Apply(Tuning16_x_14)->UseManualTime();
BENCHMARK(CUB_DEVICE_TUNE_SEGMENTED_REDUCTION)->Apply(Tuning16_x_18)->UseManualTime();
BENCHMARK(CUB_DEVICE_TUNE_SEGMENTED_REDUCTION)->Apply(Tuning16_x_22)->UseManualTime();
BENCHMARK(CUB_DEVICE_TUNE_SEGMENTED_REDUCTION)->Apply(Tuning16_x_26)->UseManualTime();
BENCHMARK(CUB_DEVICE_TUNE_SEGMENTED_REDUCTION)->Apply(Tuning16_x_28)->UseManualTime();
BENCHMARK(CUB_DEVICE_TUNE_SEGMENTED_REDUCTION)->Apply(Tuning16_x_30)->UseManualTime();

// The reference builds every CUB baseline twice: against its patched copy of CUB (fp16 shuffle specialisations,
// CUB_HALF_OPTIMIZATION) and, under the ORIGINAL_CUB_* names, against the unpatched one
// (src/reduction/cub_original.cu:106, seg_cub_device_original.cu:131-148, src/prefixsum/cub_original.cu:98).  The
// library this build compares with is hipCUB as ROCm ships it, i.e. unpatched: the ORIGINAL_* device-wide names run
// the same calls as their twins above.
static void ORIGINAL_CUB_FULL_REDUCTION(benchmark::State &state) { CUB_FULL_REDUCTION(state); }
static void ORIGINAL_CUB_FULL_PREFIXSUM(benchmark::State &state) { CUB_FULL_PREFIXSUM(state); }
static void ORIGINAL_CUB_DEVICE_SEGMENTED_REDUCTION(benchmark::State &state) { run_device_segmented_reduction(state); }
static void ORIGINAL_CUB_DEVICE_TUNE_SEGMENTED_REDUCTION(benchmark::State &state) { run_device_segmented_reduction(state); }
BENCHMARK(ORIGINAL_CUB_FULL_REDUCTION)->ARGS()->UseManualTime();
BENCHMARK(ORIGINAL_CUB_FULL_PREFIXSUM)->ARGS()->UseManualTime();
BENCHMARK(ORIGINAL_CUB_DEVICE_SEGMENTED_REDUCTION)->SEG_16_ARGS()->UseManualTime();
BENCHMARK(ORIGINAL_CUB_DEVICE_SEGMENTED_REDUCTION)->SEG_32_ARGS()->UseManualTime();
BENCHMARK(ORIGINAL_CUB_DEVICE_SEGMENTED_REDUCTION)->SEG_64_ARGS()->UseManualTime();
BENCHMARK(ORIGINAL_CUB_DEVICE_SEGMENTED_REDUCTION)->SEG_128_ARGS()->UseManualTime();
BENCHMARK(ORIGINAL_CUB_DEVICE_SEGMENTED_REDUCTION)->SEG_256_ARGS()->UseManualTime();
BENCHMARK(ORIGINAL_CUB_DEVICE_SEGMENTED_REDUCTION)->SEG_512_ARGS()->UseManualTime();
BENCHMARK(ORIGINAL_CUB_DEVICE_SEGMENTED_REDUCTION)->SEG_1024_ARGS()->UseManualTime();
BENCHMARK(ORIGINAL_CUB_DEVICE_SEGMENTED_REDUCTION)->SEG_2048_ARGS()->UseManualTime();
BENCHMARK(ORIGINAL_CUB_DEVICE_SEGMENTED_REDUCTION)->SEG_4096_ARGS()->UseManualTime();
BENCHMARK(ORIGINAL_CUB_DEVICE_SEGMENTED_REDUCTION)->SEG_8192_ARGS()->UseManualTime();
BENCHMARK(ORIGINAL_CUB_DEVICE_SEGMENTED_REDUCTION)->SEG_16384_ARGS()->UseManualTime();
BENCHMARK(ORIGINAL_CUB_DEVICE_TUNE_SEGMENTED_REDUCTION)->Apply(Tuning16_x_14)->UseManualTime();
BENCHMARK(ORIGINAL_CUB_DEVICE_TUNE_SEGMENTED_REDUCTION)->Apply(Tuning16_x_18)->UseManualTime();
BENCHMARK(ORIGINAL_CUB_DEVICE_TUNE_SEGMENTED_REDUCTION)->Apply(Tuning16_x_22)->UseManualTime();
BENCHMARK(ORIGINAL_CUB_DEVICE_TUNE_SEGMENTED_REDUCTION)->Apply(Tuning16_x_26)->UseManualTime();
BENCHMARK(ORIGINAL_CUB_DEVICE_TUNE_SEGMENTED_REDUCTION)->Apply(Tuning16_x_28)->UseManualTime();
BENCHMARK(ORIGINAL_CUB_DEVICE_TUNE_SEGMENTED_REDUCTION)->Apply(Tuning16_x_30)->UseManualTime();

// ---- rocBLAS ------------------------------------------------------------------------------------
namespace {
rocblas_handle blas() {
  static rocblas_handle h = [] {
    rocblas_handle x = nullptr;
    if (rocblas_create_handle(&x) != rocblas_status_success) throw std::runtime_error("rocblas_create_handle failed");
    return x;
  }();
  return h;
}
void check_blas(rocblas_status s, const char *what) {
  if (s != rocblas_status_success) throw std::runtime_error(std::string(what) + ": rocBLAS status " + std::to_string((int)s));
}
}  // namespace

// D (M x N row-major) = alpha * A (M x K row-major) * B (K x N column-major) + beta * C, the
// layouts of tcu_gemm_f16_f32 / tcu_gemm_f16_f16 (half_out: C and D in fp16, as the reference's
// CUBLAS_WMMA_HGEMM, src/gemm/cublas.cu:623; fp32 accumulation either way).  In rocBLAS's
// column-major terms: D^T (N x M) = op(B) * A'.
static void blas_gemm(benchmark::State &state, bool half_out) {
  guarded(state, [&] {
    const size_t M = state.range(0), N = state.range(1), K = state.range(2);
    const float alpha = 1.1f, beta = 1.2f;
    const size_t out_size = half_out ? 2 : 4;
    const rocblas_datatype out_type = half_out ? rocblas_datatype_f16_r : rocblas_datatype_f32_r;
    DeviceBuffer A(M * K * 2), B(N * K * 2), C(M * N * out_size), D(M * N * out_size);
    TCU_CHECK(tcu_generate_f16(A.get(), M * K, harness::flags().seed, TCU_DIST_NORMAL, 0, nullptr));
    TCU_CHECK(tcu_generate_f16(B.get(), N * K, harness::flags().seed + 1, TCU_DIST_NORMAL, 0, nullptr));
    PRINT_IF_ERROR(hipMemset(C.get(), 0, M * N * out_size));
    auto run = [&] {
      check_blas(rocblas_gemm_ex(blas(), rocblas_operation_transpose, rocblas_operation_none, (rocblas_int)N, (rocblas_int)M, (rocblas_int)K, &alpha, B.get(), rocblas_datatype_f16_r, (rocblas_int)K, A.get(),
                                 rocblas_datatype_f16_r, (rocblas_int)K, &beta, C.get(), out_type, (rocblas_int)N, D.get(), out_type, (rocblas_int)N, rocblas_datatype_f32_r, rocblas_gemm_algo_standard, 0, 0),
                 "rocblas_gemm_ex");
    };
    run();
    PRINT_IF_ERROR(hipDeviceSynchronize());
    timed_loop(state, [&](size_t) { run(); });
    state.counters.insert({{"M", (double)M},
                           {"N", (double)N},
                           {"K", (double)K},
                           {"flops", {state.iterations() * 2.0 * M * N * K, benchmark::Counter::kAvgThreadsRate}},
                           {"mfma_peak_fraction", {state.iterations() * 2.0 * M * N * K / 2.5e15, benchmark::Counter::kAvgThreadsRate}}});
  });
}
static void CUBLAS_WMMA_GEMM(benchmark::State &state) { blas_gemm(state, false); }
static void CUBLAS_WMMA_HGEMM(benchmark::State &state) { blas_gemm(state, true); }
// The reference times every product twice, with tensor-core math switched on (CUBLAS_WMMA_*) and off (CUBLAS_GEMM,
// CUBLAS_HGEMM), and the fp16-output product also through cublasGemmEx (src/gemm/cublas.cu:618-627).  rocBLAS has no
// such switch and one entry point for these types, so the names below time the same library call as their twins.
static void CUBLAS_GEMM(benchmark::State &state) { blas_gemm(state, false); }
static void CUBLAS_HGEMM(benchmark::State &state) { blas_gemm(state, true); }
static void CUBLAS_WMMA_HGEMM_GemmEx(benchmark::State &state) { blas_gemm(state, true); }
static void CUBLAS_HGEMM_GemmEx(benchmark::State &state) { blas_gemm(state, true); }
BENCHMARK(CUBLAS_GEMM)->Apply(GemmArgs)->UseManualTime();
BENCHMARK(CUBLAS_WMMA_GEMM)->Apply(GemmArgs)->UseManualTime();
BENCHMARK(CUBLAS_HGEMM)->Apply(GemmArgs)->UseManualTime();
BENCHMARK(CUBLAS_WMMA_HGEMM)->Apply(GemmArgs)->UseManualTime();
BENCHMARK(CUBLAS_WMMA_HGEMM_GemmEx)->Apply(GemmArgs)->UseManualTime();
BENCHMARK(CUBLAS_HGEMM_GemmEx)->Apply(GemmArgs)->UseManualTime();

// The same product through hipBLASLt: in its column-major terms D^T (N x M) = B^T (N x K) * A' (K x M).
static void lt_check(hipblasStatus_t s, const char *what) {
  if (s != HIPBLAS_STATUS_SUCCESS) throw std::runtime_error(std::string(what) + ": hipBLASLt status " + std::to_string((int)s));
}
static void blaslt_gemm(benchmark::State &state, bool half_out) {
  guarded(state, [&] {
    const size_t M = state.range(0), N = state.range(1), K = state.range(2);
    const float alpha = 1.1f, beta = 1.2f;
    const size_t out_size = half_out ? 2 : 4;
    const hipDataType out_type = half_out ? HIP_R_16F : HIP_R_32F;
    DeviceBuffer A(M * K * 2), B(N * K * 2), C(M * N * out_size), D(M * N * out_size);
    TCU_CHECK(tcu_generate_f16(A.get(), M * K, harness::flags().seed, TCU_DIST_NORMAL, 0, nullptr));
    TCU_CHECK(tcu_generate_f16(B.get(), N * K, harness::flags().seed + 1, TCU_DIST_NORMAL, 0, nullptr));
    PRINT_IF_ERROR(hipMemset(C.get(), 0, M * N * out_size));
    static hipblasLtHandle_t lt = [] {
      hipblasLtHandle_t h = nullptr;
      lt_check(hipblasLtCreate(&h), "hipblasLtCreate");
      return h;
    }();
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t la = nullptr, lb = nullptr, lc = nullptr, ld = nullptr;
    hipblasLtMatmulPreference_t pref = nullptr;
    lt_check(hipblasLtMatmulDescCreate(&desc, HIPBLAS_COMPUTE_32F, HIP_R_32F), "hipblasLtMatmulDescCreate");
    const hipblasOperation_t op_t = HIPBLAS_OP_T, op_n = HIPBLAS_OP_N;
    lt_check(hipblasLtMatmulDescSetAttribute(desc, HIPBLASLT_MATMUL_DESC_TRANSA, &op_t, sizeof(op_t)), "TRANSA");
    lt_check(hipblasLtMatmulDescSetAttribute(desc, HIPBLASLT_MATMUL_DESC_TRANSB, &op_n, sizeof(op_n)), "TRANSB");
    lt_check(hipblasLtMatrixLayoutCreate(&la, HIP_R_16F, K, N, K), "layout of B");
    lt_check(hipblasLtMatrixLayoutCreate(&lb, HIP_R_16F, K, M, K), "layout of A");
    lt_check(hipblasLtMatrixLayoutCreate(&lc, out_type, N, M, N), "layout of C");
    lt_check(hipblasLtMatrixLayoutCreate(&ld, out_type, N, M, N), "layout of D");
    lt_check(hipblasLtMatmulPreferenceCreate(&pref), "hipblasLtMatmulPreferenceCreate");
    size_t ws_bytes = (size_t)128 << 20;
    lt_check(hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &ws_bytes, sizeof(ws_bytes)), "workspace preference");
    DeviceBuffer ws(ws_bytes);
    hipblasLtMatmulHeuristicResult_t found[1];
    int n_found = 0;
    lt_check(hipblasLtMatmulAlgoGetHeuristic(lt, desc, la, lb, lc, ld, pref, 1, found, &n_found), "hipblasLtMatmulAlgoGetHeuristic");
    if (n_found == 0) throw std::runtime_error("hipBLASLt offers no algorithm for this product");
    auto run = [&] {
      lt_check(hipblasLtMatmul(lt, desc, &alpha, B.get(), la, A.get(), lb, &beta, C.get(), lc, D.get(), ld, &found[0].algo, ws.get(), ws_bytes, nullptr), "hipblasLtMatmul");
    };
    run();
    PRINT_IF_ERROR(hipDeviceSynchronize());
    timed_loop(state, [&](size_t) { run(); });
    state.counters.insert({{"M", (double)M},
                           {"N", (double)N},
                           {"K", (double)K},
                           {"flops", {state.iterations() * 2.0 * M * N * K, benchmark::Counter::kAvgThreadsRate}},
                           {"mfma_peak_fraction", {state.iterations() * 2.0 * M * N * K / 2.5e15, benchmark::Counter::kAvgThreadsRate}}});
    hipblasLtMatmulPreferenceDestroy(pref);
    hipblasLtMatrixLayoutDestroy(la);
    hipblasLtMatrixLayoutDestroy(lb);
    hipblasLtMatrixLayoutDestroy(lc);
    hipblasLtMatrixLayoutDestroy(ld);
    hipblasLtMatmulDescDestroy(desc);
  });
}
static void HIPBLASLT_GEMM(benchmark::State &state) { blaslt_gemm(state, false); }
static void HIPBLASLT_HGEMM(benchmark::State &state) { blaslt_gemm(state, true); }
BENCHMARK(HIPBLASLT_GEMM)->Apply(GemmArgs)->UseManualTime();
BENCHMARK(HIPBLASLT_HGEMM)->Apply(GemmArgs)->UseManualTime();

// y (M) = alpha * A (M x K row-major) x + beta * y as a one-column GEMM (fp16 in, fp32 accumulate; y in fp32 or fp16):
// what the reference's CUDA_WMMA_GEMV_CUBLAS / CUDA_WMMA_HGEMV_CUBLAS do with cuBLAS (src/gemv/wmma_cublas.cu:245-246) and,
// in fp32, its CUBLAS_GEMV (src/gemv/cublas.cu:88)
static void blas_gemv(benchmark::State &state, bool half_out) {
  guarded(state, [&] {
    const size_t M = state.range(0), K = state.range(1);
    const float alpha = 1.0f, beta = 0.0f;
    const size_t out_size = half_out ? 2 : 4;
    const rocblas_datatype out_type = half_out ? rocblas_datatype_f16_r : rocblas_datatype_f32_r;
    DeviceBuffer A(M * K * 2), x(K * 2), y(M * out_size);
    TCU_CHECK(tcu_generate_f16(A.get(), M * K, harness::flags().seed, TCU_DIST_NORMAL, 0, nullptr));
    TCU_CHECK(tcu_generate_f16(x.get(), K, harness::flags().seed + 1, TCU_DIST_NORMAL, 0, nullptr));
    PRINT_IF_ERROR(hipMemset(y.get(), 0, M * out_size));
    auto run = [&] {
      check_blas(rocblas_gemm_ex(blas(), rocblas_operation_transpose, rocblas_operation_none, (rocblas_int)M, 1, (rocblas_int)K, &alpha, A.get(), rocblas_datatype_f16_r, (rocblas_int)K, x.get(),
                                 rocblas_datatype_f16_r, (rocblas_int)K, &beta, y.get(), out_type, (rocblas_int)M, y.get(), out_type, (rocblas_int)M, rocblas_datatype_f32_r,
                                 rocblas_gemm_algo_standard, 0, 0),
                 "rocblas_gemm_ex");
    };
    run();
    PRINT_IF_ERROR(hipDeviceSynchronize());
    timed_loop(state, [&](size_t) { run(); });
    const double bytes = 2.0 * M * K + 2.0 * K + (double)out_size * M;
    state.counters.insert({{"M", (double)M},
                           {"N", (double)K},
                           {"flops", {state.iterations() * 2.0 * M * K, benchmark::Counter::kAvgThreadsRate}},
                           {"bytes_per_second", {state.iterations() * bytes, benchmark::Counter::kAvgThreadsRate}},
                           {"hbm_peak_fraction", {state.iterations() * bytes / 8e12, benchmark::Counter::kAvgThreadsRate}}});
  });
}
static void CUBLAS_GEMV(benchmark::State &state) { blas_gemv(state, false); }
static void CUDA_WMMA_GEMV_CUBLAS(benchmark::State &state) { blas_gemv(state, false); }
static void CUDA_WMMA_HGEMV_CUBLAS(benchmark::State &state) { blas_gemv(state, true); }
BENCHMARK(CUBLAS_GEMV)->Apply(GemvArgs)->UseManualTime();
BENCHMARK(CUDA_WMMA_GEMV_CUBLAS)->Apply(GemvArgs)->UseManualTime();
BENCHMARK(CUDA_WMMA_HGEMV_CUBLAS)->Apply(GemvArgs)->UseManualTime();
