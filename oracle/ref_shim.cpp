// TEST INFRASTRUCTURE ONLY — never linked into or called by the product path.
//
// C-ABI shim around the reference's own CPU implementation of the path,
// csrc/cpu/layernorm.cpp (rms_norm :91-103, fused_add_rms_norm :105-117).
// That translation unit is compiled where it lies under the reference tree
// (see oracle/Makefile); this file only declares its two entry points and
// hands them tensors that alias the caller's bf16 buffers, so the reference
// arithmetic runs unmodified.  Output: oracle/_ref/libtw_ref.so.
#include <torch/all.h>

#include <cstdint>

// Defined in the reference's csrc/cpu/layernorm.cpp (signatures also listed in
// csrc/ops.h:64-70).
void rms_norm(torch::Tensor& out, torch::Tensor& input, torch::Tensor& weight,
              double epsilon);
void fused_add_rms_norm(torch::Tensor& input, torch::Tensor& residual,
                        torch::Tensor& weight, double epsilon);

namespace {
torch::Tensor alias_bf16(void* p, int64_t rows, int64_t cols) {
  auto opt = torch::TensorOptions().dtype(torch::kBFloat16).device(torch::kCPU);
  if (rows < 0) return torch::from_blob(p, {cols}, opt);
  return torch::from_blob(p, {rows, cols}, opt);
}
}  // namespace

extern "C" {

// x <- RMSNorm(x + r) * w ; r <- x + r      (reference: layernorm.cpp:105-117)
int tw_ref_fused_add_rms_norm(void* x, void* r, const void* w, int64_t T,
                              int64_t H, double eps) {
  try {
    auto tx = alias_bf16(x, T, H);
    auto tr = alias_bf16(r, T, H);
    auto tw = alias_bf16(const_cast<void*>(w), -1, H);
    fused_add_rms_norm(tx, tr, tw, eps);
    return 0;
  } catch (...) {
    return -1;
  }
}

// out <- RMSNorm(x) * w                     (reference: layernorm.cpp:91-103)
int tw_ref_rms_norm(void* out, const void* x, const void* w, int64_t T,
                    int64_t H, double eps) {
  try {
    auto to = alias_bf16(out, T, H);
    auto tx = alias_bf16(const_cast<void*>(x), T, H);
    auto tw = alias_bf16(const_cast<void*>(w), -1, H);
    rms_norm(to, tx, tw, eps);
    return 0;
  } catch (...) {
    return -1;
  }
}

}  // extern "C"
