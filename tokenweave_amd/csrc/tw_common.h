// Shared between the translation units of libtokenweave_amd.so: error
// reporting and the per-device property cache.  Not part of the public ABI.
#ifndef TW_COMMON_H
#define TW_COMMON_H

#include <stdint.h>

#include "../../include/tokenweave_amd.h"

namespace tw {

// Records a printf-style message for tw_last_error() and returns `code`.
int set_error(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

// Compute units of the current device, queried once per device; <= 0 on error.
int device_compute_units();

int run_row_norm(const char* what, const void* const* partials, int np, void* y,
                 void* residual, void* copy_out, const void* weight, const float* quant_scale,
                 int64_t T, int64_t H, float eps, int dtype, int max_ctas, bool require_vec,
                 void* stream);

// quant: 0 none, 1 static fp8, 2 dynamic per-token fp8, 3 dynamic per-token int8.
int run_row_norm_q(const char* what, const void* const* partials, int np, void* y,
                   void* residual, void* copy_out, const void* weight, int quant,
                   const float* quant_scale, float* row_scales, int64_t T, int64_t H, float eps,
                   int dtype, int max_ctas, bool require_vec, void* stream);

int run_copy16(void* dst, const void* src, int64_t nbytes, void* stream);

int run_gemm_bf16_nt(void* out, const void* a, const void* b, int64_t M, int64_t N,
                     int64_t K, int64_t ldc, int max_cus, void* stream);

}  // namespace tw

#endif
