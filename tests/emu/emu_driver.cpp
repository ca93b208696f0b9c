// Builds the kernel sources of tcu_scope_amd/csrc against the CPU lane emulator and
// exports the same dispatch functions the GPU library wraps (TEST INFRASTRUCTURE ONLY).
#include "wave_ops_emu.hpp"
//
#include "../../tcu_scope_amd/csrc/dispatch.hpp"

extern "C" {
int emu_seg_reduce_f16(const void *in, void *out, size_t nseg, size_t seg, int variant, int u, int wpb) { return tcu::seg_reduce_dispatch(in, out, nseg, seg, variant, u, wpb, nullptr); }
int emu_seg_scan_f16(const void *in, void *out, void *totals, size_t nseg, size_t seg, int variant, int u, int wpb) {
  return tcu::seg_scan_dispatch(in, out, totals, nseg, seg, variant, u, wpb, nullptr);
}
int emu_seg_reduce_offsets_f16(const void *in, void *out, size_t nseg, const void *begin, const void *end, int bits, size_t expected) { return tcu::seg_reduce_offsets_dispatch(in, out, nseg, begin, end, bits, expected, nullptr); }
int emu_seg_scan_offsets_f16(const void *in, void *out, size_t nseg, const void *begin, const void *end, int bits, size_t expected) { return tcu::seg_scan_offsets_dispatch(in, out, nseg, begin, end, bits, expected, nullptr); }
int emu_add_partial_sums_f16(void *out, const void *ps, size_t nseg, size_t seg) { return tcu::add_partial_sums_dispatch(out, ps, nseg, seg, nullptr); }
const char *emu_last_error() { return tcu::last_error_string().c_str(); }
int emu_set_option(const char *name, int value) { return tcu::set_option(name, value); }
}
extern "C" {
int emu_full_reduce_f16(const void *in, void *out, size_t n, void *ws, size_t *ws_bytes, int strategy, size_t seg, int wpb) {
  return tcu::full_reduce_dispatch(in, out, n, ws, ws_bytes, strategy, seg, wpb, nullptr);
}
int emu_full_scan_f16(const void *in, void *out, size_t n, void *ws, size_t *ws_bytes, int strategy, size_t seg, int wpb) {
  return tcu::full_scan_dispatch(in, out, n, ws, ws_bytes, strategy, seg, wpb, nullptr);
}
int emu_gemv_f16_f32(const void *A, const void *x, void *y, size_t M, size_t K, float alpha, float beta, int variant) { return tcu::gemv_dispatch(A, x, y, M, K, alpha, beta, variant, nullptr); }
int emu_gemv_col_major_f16_f32(const void *A, size_t lda, const void *x, void *y, size_t M, size_t K, float alpha, float beta) {
  return tcu::gemv_col_major_dispatch<float>("tcu_gemv_col_major_f16_f32", A, lda, x, y, M, K, alpha, beta, nullptr);
}
int emu_gemv_col_major_f16_f16(const void *A, size_t lda, const void *x, void *y, size_t M, size_t K, float alpha, float beta) {
  return tcu::gemv_col_major_dispatch<tcu::half_t>("tcu_gemv_col_major_f16_f16", A, lda, x, y, M, K, alpha, beta, nullptr);
}
int emu_gemv_f16_f16(const void *A, const void *x, void *y, size_t M, size_t K, float alpha, float beta, int variant) { return tcu::hgemv_dispatch(A, x, y, M, K, alpha, beta, variant, nullptr); }
int emu_gemm_f16_f16(const void *A, const void *B, const void *C, void *D, size_t M, size_t N, size_t K, float alpha, float beta, int variant) {
  return tcu::hgemm_dispatch(A, B, C, D, M, N, K, alpha, beta, variant, nullptr);
}
int emu_gemm_f16_f32(const void *A, const void *B, const void *C, void *D, size_t M, size_t N, size_t K, float alpha, float beta, int variant) {
  return tcu::gemm_dispatch(A, B, C, D, M, N, K, alpha, beta, variant, nullptr);
}
int emu_seg_scan_by_key_f16(const void *keys, const void *in, void *out, size_t n, int bits, void *ws, size_t *ws_bytes) {
  return tcu::seg_scan_by_key_dispatch(keys, in, out, n, bits, ws, ws_bytes, nullptr);
}
int emu_seg_reduce_by_key_f16(const void *keys, const void *in, void *keys_out, void *out, void *num_runs, size_t n, int bits, void *ws, size_t *ws_bytes) {
  return tcu::seg_reduce_by_key_dispatch(keys, in, keys_out, out, num_runs, n, bits, ws, ws_bytes, nullptr);
}
int emu_fill_f16(void *d, float v, size_t n) { return tcu::fill_dispatch(d, v, n, nullptr); }
int emu_convert_f32_to_f16(void *o, const void *i, size_t n) { return tcu::convert_dispatch(o, i, n, nullptr); }
int emu_generate_f16(void *d, size_t n, uint64_t seed, int dist, size_t first) { return tcu::generate_dispatch(d, n, seed, dist, first, nullptr); }
int emu_stream_probe(void *dst, const void *src, size_t bytes, int mode, int u, int wpb) { return tcu::stream_probe_dispatch(dst, src, bytes, mode, u, wpb, nullptr); }
int emu_lane_probe(void *out, size_t *words) { return tcu::lane_probe_dispatch(out, words, nullptr); }
}
