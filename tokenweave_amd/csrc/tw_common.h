// Shared between the translation units of libtokenweave_amd.so: error
// reporting and the per-device property cache.  Not part of the public ABI.
#ifndef TW_COMMON_H
#define TW_COMMON_H

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <tuple>
#include <utility>

#include "../../include/tokenweave_amd.h"

namespace tw {

// Records a printf-style message for tw_last_error() and returns `code`.
int set_error(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

// Compute units of the current device, queried once per device; <= 0 on error.
int device_compute_units();

// Status of this thread's most recent launch_kernel call.
hipError_t& launch_status();

// Enqueues `kernel` and records the status of THIS launch in launch_status().  The
// runtime's per-thread "last error" is neither read nor cleared, so an error left there
// by other code in the process is not mistaken for ours and is not swallowed.
template <typename... KArgs, typename... Args>
inline void launch_kernel(void (*kernel)(KArgs...), dim3 grid, dim3 block, size_t lds_bytes,
                          hipStream_t stream, Args&&... args) {
  static_assert(sizeof...(KArgs) == sizeof...(Args), "argument count differs from the kernel's");
  std::tuple<KArgs...> vals{static_cast<KArgs>(std::forward<Args>(args))...};
  std::apply(
      [&](auto&... v) {
        void* ptrs[] = {static_cast<void*>(&v)...};
        launch_status() = hipLaunchKernel(reinterpret_cast<const void*>(kernel), grid, block, ptrs,
                                          lds_bytes, stream);
      },
      vals);
}

// TW_OK, or TW_ERR_LAUNCH with the runtime's message when the last launch_kernel failed.
int finish_launch(const char* what);

int run_row_norm(const char* what, const void* const* partials, int np, void* y,
                 void* residual, void* copy_out, const void* weight, const float* quant_scale,
                 int64_t T, int64_t H, float eps, int dtype, int max_ctas, bool require_vec,
                 void* stream);

// quant: 0 none, 1 static fp8, 2 dynamic per-token fp8, 3 dynamic per-token int8.
int run_row_norm_q(const char* what, const void* const* partials, int np, void* y,
                   void* residual, void* copy_out, const void* weight, int quant,
                   const float* quant_scale, float* row_scales, int64_t T, int64_t H, float eps,
                   int dtype, int max_ctas, bool require_vec, void* stream);

// The P-partial op with the split-row kernel where it pays; `workspace` is
// TW_SPLIT_WORKSPACE_BYTES of zeroed device memory (or null: never split).
int run_row_norm_ws(const char* what, const void* const* partials, int np, void* y, void* residual,
                    const void* weight, int64_t T, int64_t H, float eps, int max_ctas,
                    void* workspace, void* stream);

// run_row_norm_ws on the library's static workspace; refuses T > TW_SPLIT_MAX_TOKENS.
int run_row_norm_noalloc(const char* what, const void* const* partials, int np, void* y, void* residual,
                         const void* weight, int64_t T, int64_t H, float eps, int max_ctas, void* stream);

// Segments per row the split-row kernel would use for this shape on the current device
// (1 = the one-workgroup-per-row kernel runs instead).
int split_segments(int64_t T, int64_t H, int max_ctas);

// bias: [N] bf16 added to every row of the product, or null.
int run_gemm_bf16_nt(void* out, const void* a, const void* b, const void* bias, int64_t M, int64_t N,
                     int64_t K, int64_t ldc, int max_cus, void* stream);

// biases: null, or `count` pointers each of which may be null.
int run_gemm_bf16_nt_partials(void* const* outs, const void* const* as, const void* const* bs,
                              const void* const* biases, int count, int64_t M, int64_t N, int64_t K,
                              int64_t ldc, int max_cus, void* stream);

}  // namespace tw

#endif
