// extern "C" surface of libtokenweave_amd.so (declared in
// include/tokenweave_amd.h): argument mapping only, kernels live in
// tw_norm.hip and tw_gemm.hip.
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>

#include "tw_common.h"

namespace tw {

static thread_local char g_last_error[512] = "";

int set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  return code;
}

hipError_t& launch_status() {
  static thread_local hipError_t status = hipSuccess;
  return status;
}

int finish_launch(const char* what) {
  const hipError_t e = launch_status();
  if (e != hipSuccess)
    return set_error(TW_ERR_LAUNCH, "%s: kernel launch failed: %s", what, hipGetErrorString(e));
  return TW_OK;
}

int device_compute_units() {
  constexpr int kMaxDevices = 64;
  static int cache[kMaxDevices];  // 0 = not queried yet
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return -1;
  int v = __atomic_load_n(&cache[dev], __ATOMIC_RELAXED);
  if (v == 0) {
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        cus <= 0)
      return -1;
    __atomic_store_n(&cache[dev], cus, __ATOMIC_RELAXED);
    v = cus;
  }
  return v;
}

static int strided_partials(const char* what, uint64_t mcptr, int64_t stride, int rank,
                            int world_size, const void** out) {
  if (world_size < 1 || world_size > TW_MAX_PARTIALS)
    return set_error(TW_ERR_INVALID_ARGUMENT, "%s: world_size %d not in [1, %d]", what, world_size,
                     TW_MAX_PARTIALS);
  if (rank < 0 || rank >= world_size)
    return set_error(TW_ERR_INVALID_ARGUMENT, "%s: Invalid rank %d, must be in [0, %d]", what, rank,
                     world_size - 1);
  if (mcptr == 0) return set_error(TW_ERR_INVALID_ARGUMENT, "%s: mcptr is null", what);
  if (stride % 16 != 0)
    return set_error(TW_ERR_ALIGNMENT, "%s: peer stride %lld is not a multiple of 16 bytes", what,
                     (long long)stride);
  for (int p = 0; p < world_size; ++p)
    out[p] = reinterpret_cast<const void*>(mcptr + (uint64_t)((int64_t)p * stride));
  return TW_OK;
}

}  // namespace tw

extern "C" {

int tw_version(void) { return 100; }

const char* tw_last_error(void) { return tw::g_last_error; }

int tw_num_compute_units(void) { return tw::device_compute_units(); }

int tw_fused_add_rms_norm(void* input, void* residual, const void* weight, int64_t num_tokens,
                          int64_t hidden_size, float epsilon, int dtype, void* stream) {
  if (!residual && num_tokens > 0)
    return tw::set_error(TW_ERR_INVALID_ARGUMENT, "fused_add_rms_norm: residual is null");
  const void* parts[1] = {input};
  return tw::run_row_norm("fused_add_rms_norm", parts, 1, input, residual, nullptr, weight, nullptr,
                          num_tokens, hidden_size, epsilon, dtype, 0, false, stream);
}

int tw_rms_norm(void* out, const void* input, const void* weight, int64_t num_tokens,
                int64_t hidden_size, float epsilon, int dtype, void* stream) {
  const void* parts[1] = {input};
  return tw::run_row_norm("rms_norm", parts, 1, out, nullptr, nullptr, weight, nullptr, num_tokens,
                          hidden_size, epsilon, dtype, 0, false, stream);
}

int tw_rms_norm_inplace(void* out, void* input, const void* weight, int64_t num_tokens,
                        int64_t hidden_size, float epsilon, int dtype, void* stream) {
  if (!out && num_tokens > 0)
    return tw::set_error(TW_ERR_INVALID_ARGUMENT, "rms_norm_inplace: out is null");
  if (out == input && num_tokens > 0)
    return tw::set_error(TW_ERR_INVALID_ARGUMENT, "rms_norm_inplace: out must not alias input");
  const void* parts[1] = {input};
  return tw::run_row_norm("rms_norm_inplace", parts, 1, input, nullptr, out, weight, nullptr, num_tokens,
                          hidden_size, epsilon, dtype, 0, false, stream);
}

int tw_fused_add_rms_norm_cta(void* input, void* residual, const void* weight,
                              int64_t num_tokens, int64_t hidden_size, int max_ctas,
                              float epsilon, void* stream) {
  if (!residual && num_tokens > 0)
    return tw::set_error(TW_ERR_INVALID_ARGUMENT, "fused_add_rms_norm_cta: residual is null");
  const void* parts[1] = {input};
  return tw::run_row_norm("fused_add_rms_norm_cta", parts, 1, input, residual, nullptr, weight, nullptr,
                          num_tokens, hidden_size, epsilon, TW_DTYPE_BF16, max_ctas, true, stream);
}

int tw_reduce_add_rms_norm(const void* const* partials, int num_partials, void* y, void* residual,
                           const void* weight, int64_t num_tokens, int64_t hidden_size,
                           int max_ctas, float epsilon, void* stream) {
  if (!residual && num_tokens > 0)
    return tw::set_error(TW_ERR_INVALID_ARGUMENT, "reduce_add_rms_norm: residual is null");
  return tw::run_row_norm("reduce_add_rms_norm", partials, num_partials, y, residual, nullptr,
                          weight, nullptr, num_tokens, hidden_size, epsilon, TW_DTYPE_BF16, max_ctas, true,
                          stream);
}

int tw_fused_rs_ln_cta(void* input, void* residual, const void* weight, uint64_t mcptr,
                       int64_t peer_stride_bytes, int rank, int world_size, int max_ctas,
                       float epsilon, int64_t num_tokens, int64_t hidden_size, void* stream) {
  const void* parts[TW_MAX_PARTIALS];
  int rc = tw::strided_partials("fused_rs_ln_cta", mcptr, peer_stride_bytes, rank, world_size,
                                parts);
  if (rc != TW_OK) return rc;
  if (!residual && num_tokens > 0)
    return tw::set_error(TW_ERR_INVALID_ARGUMENT, "fused_rs_ln_cta: residual is null");
  return tw::run_row_norm("fused_rs_ln_cta", parts, world_size, input, residual, nullptr, weight, nullptr,
                          num_tokens, hidden_size, epsilon, TW_DTYPE_BF16, max_ctas, true, stream);
}

int tw_fused_rs_ln_ag_cta(void* input, void* residual, const void* weight, uint64_t mcptr,
                          int64_t peer_stride_bytes, int rank, int world_size, int max_ctas,
                          float epsilon, int64_t num_tokens, int64_t hidden_size, void* stream) {
  const void* parts[TW_MAX_PARTIALS];
  int rc = tw::strided_partials("fused_rs_ln_ag_cta", mcptr, peer_stride_bytes, rank, world_size,
                                parts);
  if (rc != TW_OK) return rc;
  if (!residual && num_tokens > 0)
    return tw::set_error(TW_ERR_INVALID_ARGUMENT, "fused_rs_ln_ag_cta: residual is null");
  return tw::run_row_norm("fused_rs_ln_ag_cta", parts, world_size, input, residual, nullptr,
                          weight, nullptr, num_tokens, hidden_size, epsilon, TW_DTYPE_BF16, max_ctas, true,
                          stream);
}

static int check_workspace(const char* what, const void* workspace, int64_t workspace_bytes) {
  if (workspace && workspace_bytes < TW_SPLIT_WORKSPACE_BYTES)
    return tw::set_error(TW_ERR_INVALID_ARGUMENT, "%s: workspace of %lld bytes, need %d", what,
                         (long long)workspace_bytes, TW_SPLIT_WORKSPACE_BYTES);
  return TW_OK;
}

int tw_reduce_add_rms_norm_ws(const void* const* partials, int num_partials, void* y, void* residual,
                              const void* weight, int64_t num_tokens, int64_t hidden_size,
                              int max_ctas, float epsilon, void* workspace, int64_t workspace_bytes,
                              void* stream) {
  if (int rc = check_workspace("reduce_add_rms_norm_ws", workspace, workspace_bytes)) return rc;
  if (!residual && num_tokens > 0)
    return tw::set_error(TW_ERR_INVALID_ARGUMENT, "reduce_add_rms_norm_ws: residual is null");
  return tw::run_row_norm_ws("reduce_add_rms_norm_ws", partials, num_partials, y, residual, weight,
                             num_tokens, hidden_size, epsilon, max_ctas, workspace, stream);
}

int tw_fused_rs_ln_ag_cta_ws(void* input, void* residual, const void* weight, uint64_t mcptr,
                             int64_t peer_stride_bytes, int rank, int world_size, int max_ctas,
                             float epsilon, int64_t num_tokens, int64_t hidden_size, void* workspace,
                             int64_t workspace_bytes, void* stream) {
  if (int rc = check_workspace("fused_rs_ln_ag_cta_ws", workspace, workspace_bytes)) return rc;
  const void* parts[TW_MAX_PARTIALS];
  int rc = tw::strided_partials("fused_rs_ln_ag_cta_ws", mcptr, peer_stride_bytes, rank, world_size,
                                parts);
  if (rc != TW_OK) return rc;
  if (!residual && num_tokens > 0)
    return tw::set_error(TW_ERR_INVALID_ARGUMENT, "fused_rs_ln_ag_cta_ws: residual is null");
  return tw::run_row_norm_ws("fused_rs_ln_ag_cta_ws", parts, world_size, input, residual, weight,
                             num_tokens, hidden_size, epsilon, max_ctas, workspace, stream);
}

int tw_reduce_add_rms_norm_noalloc(const void* const* partials, int num_partials, void* y, void* residual,
                                   const void* weight, int64_t num_tokens, int64_t hidden_size,
                                   int max_ctas, float epsilon, void* stream) {
  if (!residual && num_tokens > 0)
    return tw::set_error(TW_ERR_INVALID_ARGUMENT, "reduce_add_rms_norm_noalloc: residual is null");
  return tw::run_row_norm_noalloc("reduce_add_rms_norm_noalloc", partials, num_partials, y, residual, weight,
                                  num_tokens, hidden_size, epsilon, max_ctas, stream);
}

int tw_split_segments(int64_t num_tokens, int64_t hidden_size, int max_ctas) {
  return tw::split_segments(num_tokens, hidden_size, max_ctas);
}

int tw_rms_norm_static_fp8_quant(void* out, const void* input, const void* weight,
                                 const float* scale, int64_t num_tokens, int64_t hidden_size,
                                 float epsilon, int dtype, void* stream) {
  if (!scale && num_tokens > 0)
    return tw::set_error(TW_ERR_INVALID_ARGUMENT, "rms_norm_static_fp8_quant: scale is null");
  const void* parts[1] = {input};
  return tw::run_row_norm("rms_norm_static_fp8_quant", parts, 1, out, nullptr, nullptr, weight, scale,
                          num_tokens, hidden_size, epsilon, dtype, 0, false, stream);
}

int tw_fused_add_rms_norm_static_fp8_quant(void* out, const void* input, void* residual,
                                           const void* weight, const float* scale,
                                           int64_t num_tokens, int64_t hidden_size, float epsilon,
                                           int dtype, void* stream) {
  if ((!scale || !residual) && num_tokens > 0)
    return tw::set_error(TW_ERR_INVALID_ARGUMENT,
                         "fused_add_rms_norm_static_fp8_quant: scale or residual is null");
  const void* parts[1] = {input};
  return tw::run_row_norm("fused_add_rms_norm_static_fp8_quant", parts, 1, out, residual, nullptr,
                          weight, scale, num_tokens, hidden_size, epsilon, dtype, 0, false, stream);
}

int tw_reduce_add_rms_norm_static_fp8_quant(const void* const* partials, int num_partials, void* out,
                                            void* residual, const void* weight, const float* scale,
                                            int64_t num_tokens, int64_t hidden_size, int max_ctas,
                                            float epsilon, void* stream) {
  if ((!scale || !residual) && num_tokens > 0)
    return tw::set_error(TW_ERR_INVALID_ARGUMENT,
                         "reduce_add_rms_norm_static_fp8_quant: scale or residual is null");
  return tw::run_row_norm("reduce_add_rms_norm_static_fp8_quant", partials, num_partials, out,
                          residual, nullptr, weight, scale, num_tokens, hidden_size, epsilon,
                          TW_DTYPE_BF16, max_ctas, true, stream);
}

static int dyn_quant_kind(const char* what, int out_kind, int* quant) {
  if (out_kind == TW_QUANT_FP8_E4M3FN) *quant = 2;
  else if (out_kind == TW_QUANT_INT8) *quant = 3;
  else return tw::set_error(TW_ERR_DTYPE, "%s: unknown output kind %d", what, out_kind);
  return TW_OK;
}

int tw_rms_norm_dynamic_per_token_quant(void* out, const void* input, const void* weight,
                                        float* scales, const float* scale_ub, void* residual,
                                        int64_t num_tokens, int64_t hidden_size, float epsilon,
                                        int dtype, int out_kind, void* stream) {
  int quant;
  if (int rc = dyn_quant_kind("rms_norm_dynamic_per_token_quant", out_kind, &quant)) return rc;
  const void* parts[1] = {input};
  return tw::run_row_norm_q("rms_norm_dynamic_per_token_quant", parts, 1, out, residual, nullptr,
                            weight, quant, scale_ub, scales, num_tokens, hidden_size, epsilon, dtype,
                            0, false, stream);
}

int tw_reduce_add_rms_norm_dynamic_per_token_quant(const void* const* partials, int num_partials,
                                                   void* out, float* scales, void* residual,
                                                   const void* weight, const float* scale_ub,
                                                   int64_t num_tokens, int64_t hidden_size,
                                                   int max_ctas, float epsilon, int out_kind,
                                                   void* stream) {
  int quant;
  if (int rc = dyn_quant_kind("reduce_add_rms_norm_dynamic_per_token_quant", out_kind, &quant)) return rc;
  return tw::run_row_norm_q("reduce_add_rms_norm_dynamic_per_token_quant", partials, num_partials, out,
                            residual, nullptr, weight, quant, scale_ub, scales, num_tokens,
                            hidden_size, epsilon, TW_DTYPE_BF16, max_ctas, true, stream);
}

int tw_gemm_bf16_nt(void* out, const void* a, const void* b, int64_t M, int64_t N, int64_t K,
                    int64_t ldc, int max_cus, void* stream) {
  return tw::run_gemm_bf16_nt(out, a, b, nullptr, M, N, K, ldc, max_cus, stream);
}

int tw_gemm_bf16_nt_bias(void* out, const void* a, const void* b, const void* bias, int64_t M, int64_t N,
                         int64_t K, int64_t ldc, int max_cus, void* stream) {
  return tw::run_gemm_bf16_nt(out, a, b, bias, M, N, K, ldc, max_cus, stream);
}

int tw_gemm_bf16_nt_partials(void* const* outs, const void* const* as, const void* const* bs,
                             int num_partials, int64_t M, int64_t N, int64_t K, int64_t ldc, int max_cus,
                             void* stream) {
  return tw::run_gemm_bf16_nt_partials(outs, as, bs, nullptr, num_partials, M, N, K, ldc, max_cus, stream);
}

int tw_gemm_bf16_nt_partials_bias(void* const* outs, const void* const* as, const void* const* bs,
                                  const void* const* biases, int num_partials, int64_t M, int64_t N,
                                  int64_t K, int64_t ldc, int max_cus, void* stream) {
  return tw::run_gemm_bf16_nt_partials(outs, as, bs, biases, num_partials, M, N, K, ldc, max_cus, stream);
}

}  // extern "C"
