// libtokenweave_amd_torch.so — the norm ops registered with torch's dispatcher under
// the reference's schema strings (csrc/torch_bindings.cpp:135-171, 199-219), namespace
// `tokenweave_amd`, each forwarding to the C ABI of libtokenweave_amd.so.  This is the
// binding the reference itself uses for these ops (TORCH_LIBRARY + ops.impl(...,
// torch::kCUDA, ...)); a call from Python goes torch.ops -> dispatcher -> here -> one
// kernel launch, with no Python in between.
//
// Host-side checks are what the HIP kernels assume (device, dtype, row contiguity,
// shapes); their messages follow the reference's where it has one.  CPU tensors reach
// the CPU registration, which only raises: there is no CPU implementation.
#include <ATen/ATen.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <hip/hip_runtime_api.h>
#include <torch/library.h>

#include <map>
#include <mutex>
#include <string>
#include <unordered_map>

#include "../../include/tokenweave_amd.h"

namespace {

using at::Tensor;

void check_rc(int rc) {
  if (rc == TW_OK) return;
  TORCH_CHECK_NOT_IMPLEMENTED(rc != TW_ERR_DTYPE, tw_last_error());
  TORCH_CHECK(false, tw_last_error());
}

std::string dtype_name(at::ScalarType t) { return std::string("torch.") + c10::toString(t); }

// AT_DISPATCH_SWITCH wording (csrc/dispatch_utils.h:14-21)
int dtype_code(const char* kernel, const Tensor& t) {
  switch (t.scalar_type()) {
    case at::kBFloat16: return TW_DTYPE_BF16;
    case at::kHalf: return TW_DTYPE_F16;
    case at::kFloat: return TW_DTYPE_F32;
    default:
      TORCH_CHECK_NOT_IMPLEMENTED(false, "\"", kernel, "\" not implemented for '", dtype_name(t.scalar_type()), "'");
  }
  return -1;
}

// csrc/dispatch_utils.h:23-27: the TokenWeave kernels dispatch bf16 only
void require_bf16(const char* kernel, const Tensor& t) {
  TORCH_CHECK_NOT_IMPLEMENTED(t.scalar_type() == at::kBFloat16, "\"", kernel, "\" not implemented for '",
                              dtype_name(t.scalar_type()), "'");
}

void check_tensor(const char* name, const Tensor& t, at::ScalarType dtype, const c10::Device& device) {
  if (t.is_cuda() && t.scalar_type() == dtype && t.device() == device && t.is_contiguous()) return;
  TORCH_CHECK(t.is_cuda(), name, " is on ", t.device(),
              ": tokenweave_amd ops run on the GPU only (there is no CPU implementation)");
  TORCH_CHECK(t.device() == device, name, " is on ", t.device(), ", expected ", device);
  TORCH_CHECK(t.scalar_type() == dtype, name, " has dtype ", dtype_name(t.scalar_type()), ", expected ",
              dtype_name(dtype));
  TORCH_CHECK(t.is_contiguous(), name,
              " must be row-contiguous (stride(-1) == 1, stride(-2) == hidden_size); got shape ", t.sizes(),
              " stride ", t.strides());
}

void check_weight(const Tensor& weight, int64_t hidden, at::ScalarType dtype, const c10::Device& device) {
  check_tensor("weight", weight, dtype, device);
  TORCH_CHECK(weight.numel() == hidden, "weight has ", weight.numel(), " elements, expected hidden_size ", hidden);
}

// (num_tokens, hidden_size) as the reference computes them (csrc/layernorm_kernels.cu:198-199)
struct Rows {
  int64_t T, H;
};
Rows rows_of(const Tensor& t) {
  TORCH_CHECK(t.dim() >= 1, "expected a tensor with at least one dimension");
  const int64_t H = t.size(-1);
  return {H ? t.numel() / H : 0, H};
}

// Device guard + the current stream of the tensor's device (OptionalCUDAGuard and
// getCurrentCUDAStream in the reference, csrc/tokenweave_fused_kernels.cu:239-240).
struct Launch {
  c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard;
  void* stream;
  explicit Launch(const Tensor& t) : guard(t.device()) {
    stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(t.device().index()).stream();
  }
};

// ---------------------------------------------------------------------------
// One-GPU stand-in for the symmetric-memory address space: the P ranks' staging
// buffers are equally spaced slots of one allocation, and a registered region tells
// the op the distance between them so that mcptr + p * stride is partial p.
// ---------------------------------------------------------------------------
struct Region {
  uint64_t base;
  int64_t stride, slots, usable, token;
};
std::mutex g_regions_mutex;
std::map<uint64_t, Region> g_regions;  // by base address

// `token` names one registration: a region is dropped only by the token that made it, so
// the late clean-up of a freed buffer cannot remove a newer buffer at the same address.
void register_partials_region(int64_t base, int64_t stride, int64_t slots, int64_t usable, int64_t token) {
  TORCH_CHECK(stride > 0 && stride % 16 == 0, "slot stride must be a positive multiple of 16");
  TORCH_CHECK(slots >= 1 && slots <= TW_MAX_PARTIALS, "slots must be in [1, ", TW_MAX_PARTIALS, "]");
  TORCH_CHECK(usable > 0 && usable <= stride, "usable bytes of a slot must fit its stride");
  std::lock_guard<std::mutex> lock(g_regions_mutex);
  g_regions[(uint64_t)base] = Region{(uint64_t)base, stride, slots, usable, token};
}

void unregister_partials_region(int64_t base, int64_t token) {
  std::lock_guard<std::mutex> lock(g_regions_mutex);
  auto it = g_regions.find((uint64_t)base);
  if (it != g_regions.end() && it->second.token == token) g_regions.erase(it);
}

bool find_region(uint64_t mcptr, Region* out) {
  std::lock_guard<std::mutex> lock(g_regions_mutex);
  auto it = g_regions.upper_bound(mcptr);
  if (it == g_regions.begin()) return false;
  --it;
  const Region& r = it->second;
  if (mcptr < r.base || mcptr >= r.base + (uint64_t)r.stride) return false;
  *out = r;
  return true;
}

int64_t peer_stride(uint64_t mcptr, int64_t world_size, int64_t nbytes) {
  if (world_size == 1) return 16;  // unused: there is only partial 0
  Region r;
  TORCH_CHECK(find_region(mcptr, &r), "mcptr 0x", std::hex, mcptr, std::dec,
              " is not inside slot 0 of a registered partials region "
              "(allocate the staging buffers with tokenweave_amd.PartialsBuffer)");
  TORCH_CHECK(world_size <= r.slots, "world_size ", world_size, " exceeds the ", r.slots,
              " slots of the partials region");
  TORCH_CHECK((int64_t)(mcptr - r.base) + nbytes <= r.usable, "the rows of this call (", nbytes,
              " bytes at offset ", mcptr - r.base, ") reach past the ", r.usable,
              " usable bytes of a staging slot");
  return r.stride;
}

// ---------------------------------------------------------------------------
// Workspace of the split-row kernel: one zeroed buffer per (device, stream), made on
// the first decode-size call on that stream — never while the stream is being captured
// into a graph — and kept for the life of the process.
// ---------------------------------------------------------------------------
std::mutex g_ws_mutex;
std::unordered_map<uint64_t, Tensor> g_workspaces;

bool stream_is_capturing(void* stream) {
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  // a failing query leaves the capture (if any) alone; treat it as "capturing": do not allocate
  if (hipStreamIsCapturing(static_cast<hipStream_t>(stream), &status) != hipSuccess) return true;
  return status != hipStreamCaptureStatusNone;
}

// The workspace of (device, stream), or null when there is none yet and the stream is
// being captured: allocating then would draw from the graph's private pool and record the
// fill kernel.  The caller runs the one-workgroup-per-row kernel instead (same bits); a
// workspace made beforehand (prepare_split_workspace or any eager decode-size call on the
// stream) is used by captured calls too.
void* split_workspace(const c10::Device& device, void* stream) {
  const uint64_t key = ((uint64_t)(uintptr_t)stream << 8) ^ (uint64_t)(device.index() & 0xff);
  std::lock_guard<std::mutex> lock(g_ws_mutex);
  auto it = g_workspaces.find(key);
  if (it == g_workspaces.end()) {
    if (stream_is_capturing(stream)) return nullptr;
    Tensor ws = at::zeros({(int64_t)TW_SPLIT_WORKSPACE_BYTES}, at::TensorOptions().device(device).dtype(at::kByte));
    TORCH_CHECK(((uintptr_t)ws.data_ptr() & 255u) == 0, "workspace allocation is not 256-byte aligned");
    it = g_workspaces.emplace(key, std::move(ws)).first;
  }
  return it->second.data_ptr();
}

// Creates the workspace of the current stream of device `device_index` now (before a capture).
void prepare_split_workspace(int64_t device_index) {
  const c10::Device device(c10::DeviceType::CUDA, (c10::DeviceIndex)device_index);
  c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(device);
  void* stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(device.index()).stream();
  TORCH_CHECK(split_workspace(device, stream) != nullptr,
              "prepare_split_workspace: the current stream is being captured; call it before the capture begins");
}

// ---------------------------------------------------------------------------
// layer norm ops (vllm/_custom_ops.py:176-207 -> csrc/torch_bindings.cpp:135-171)
// ---------------------------------------------------------------------------
void rms_norm(Tensor& out, Tensor& input, Tensor& weight, double epsilon) {
  const int code = dtype_code("rms_norm_kernel", input);
  const auto dt = input.scalar_type();
  const auto dev = input.device();
  check_tensor("input", input, dt, dev);
  check_tensor("out", out, dt, dev);
  const Rows r = rows_of(input);
  TORCH_CHECK(out.sizes() == input.sizes(), "out and input must have the same shape");
  check_weight(weight, r.H, dt, dev);
  Launch l(input);
  check_rc(tw_rms_norm(out.data_ptr(), input.data_ptr(), weight.data_ptr(), r.T, r.H, (float)epsilon, code,
                       l.stream));
}

void fused_add_rms_norm(Tensor& input, Tensor& residual, Tensor& weight, double epsilon) {
  const int code = dtype_code("fused_add_rms_norm_kernel", input);
  const auto dt = input.scalar_type();
  const auto dev = input.device();
  check_tensor("input", input, dt, dev);
  check_tensor("residual", residual, dt, dev);
  const Rows r = rows_of(input);
  TORCH_CHECK(residual.sizes() == input.sizes(), "input and residual must have the same shape");
  check_weight(weight, r.H, dt, dev);
  Launch l(input);
  check_rc(tw_fused_add_rms_norm(input.data_ptr(), residual.data_ptr(), weight.data_ptr(), r.T, r.H,
                                 (float)epsilon, code, l.stream));
}

void rms_norm_inplace(Tensor& out, Tensor& input, Tensor& weight, double epsilon) {
  const int code = dtype_code("rms_norm_inplace_kernel", input);
  const auto dt = input.scalar_type();
  const auto dev = input.device();
  check_tensor("input", input, dt, dev);
  check_tensor("out", out, dt, dev);
  const Rows r = rows_of(input);
  TORCH_CHECK(out.sizes() == input.sizes(), "out and input must have the same shape");
  check_weight(weight, r.H, dt, dev);
  Launch l(input);
  check_rc(tw_rms_norm_inplace(out.data_ptr(), input.data_ptr(), weight.data_ptr(), r.T, r.H, (float)epsilon,
                               code, l.stream));
}

void fused_add_rms_norm_cta(Tensor& input, Tensor& residual, Tensor& weight, int64_t max_ctas, double epsilon) {
  require_bf16("fused_add_rms_norm_cta_kernel", input);
  const auto dev = input.device();
  check_tensor("input", input, at::kBFloat16, dev);
  check_tensor("residual", residual, at::kBFloat16, dev);
  const Rows r = rows_of(input);
  TORCH_CHECK(residual.sizes() == input.sizes(), "input and residual must have the same shape");
  check_weight(weight, r.H, at::kBFloat16, dev);
  Launch l(input);
  check_rc(tw_fused_add_rms_norm_cta(input.data_ptr(), residual.data_ptr(), weight.data_ptr(), r.T, r.H,
                                     (int)max_ctas, (float)epsilon, l.stream));
}

void fused_rs_ln(bool all_gather, const char* kernel, Tensor& input, Tensor& residual, Tensor& weight,
                 int64_t mcptr, int64_t rank, int64_t world_size, int64_t max_ctas, double epsilon) {
  require_bf16(kernel, input);
  const auto dev = input.device();
  check_tensor("input", input, at::kBFloat16, dev);
  check_tensor("residual", residual, at::kBFloat16, dev);
  const Rows r = rows_of(input);
  TORCH_CHECK(residual.sizes() == input.sizes(), "input and residual must have the same shape");
  check_weight(weight, r.H, at::kBFloat16, dev);
  TORCH_CHECK(rank >= 0 && rank < world_size, "Invalid rank ", rank, ", must be in [0, ", world_size - 1, "]");
  const int64_t stride = peer_stride((uint64_t)mcptr, world_size, r.T * r.H * 2);
  Launch l(input);
  if (max_ctas <= 0 && r.T > 0 && r.T <= 2 * TW_SPLIT_MAX_TOKENS) {
    // decode-size batch, or a few more rows than compute units: the workspace entry point
    // cuts rows into several workgroups where that pays
    if (void* ws = split_workspace(dev, l.stream)) {
      check_rc(tw_fused_rs_ln_ag_cta_ws(input.data_ptr(), residual.data_ptr(), weight.data_ptr(), (uint64_t)mcptr,
                                        stride, (int)rank, (int)world_size, 0, (float)epsilon, r.T, r.H, ws,
                                        TW_SPLIT_WORKSPACE_BYTES, l.stream));
      return;
    }
  }
  auto fn = all_gather ? tw_fused_rs_ln_ag_cta : tw_fused_rs_ln_cta;
  check_rc(fn(input.data_ptr(), residual.data_ptr(), weight.data_ptr(), (uint64_t)mcptr, stride, (int)rank,
              (int)world_size, (int)max_ctas, (float)epsilon, r.T, r.H, l.stream));
}

void fused_rs_ln_ag_cta(Tensor& input, Tensor& residual, Tensor& weight, int64_t mcptr, int64_t /*signal_pads*/,
                        int64_t rank, int64_t world_size, int64_t max_ctas, double epsilon) {
  fused_rs_ln(true, "fused_rs_ln_ag_cta_kernel", input, residual, weight, mcptr, rank, world_size, max_ctas,
              epsilon);
}

void fused_rs_ln_cta(Tensor& input, Tensor& residual, Tensor& weight, int64_t mcptr, int64_t /*signal_pads*/,
                     int64_t rank, int64_t world_size, int64_t max_ctas, double epsilon) {
  fused_rs_ln(false, "fused_rs_ln_cta_kernel", input, residual, weight, mcptr, rank, world_size, max_ctas,
              epsilon);
}

// ---------------------------------------------------------------------------
// norm + quantisation (csrc/torch_bindings.cpp:199-219)
// ---------------------------------------------------------------------------
void check_fp8_out(const Tensor& out, const Tensor& like) {
  TORCH_CHECK(out.is_cuda() && out.device() == like.device(), "result is on ", out.device(), ", expected ",
              like.device());
  TORCH_CHECK_NOT_IMPLEMENTED(out.scalar_type() == at::kFloat8_e4m3fn,
                              "\"rms_norm_kernel_fp8_type\" not implemented for '", dtype_name(out.scalar_type()),
                              "'");
  TORCH_CHECK(out.is_contiguous() && out.sizes() == like.sizes(),
              "result must be a contiguous fp8 tensor with the input's shape");
}

void check_scale(const Tensor& scale, const c10::Device& dev) {
  TORCH_CHECK(scale.is_cuda() && scale.device() == dev, "scale must be a tensor on the input's device");
  TORCH_CHECK(scale.scalar_type() == at::kFloat && scale.numel() == 1, "scale must hold one float32 value");
}

void rms_norm_static_fp8_quant(Tensor& out, Tensor& input, Tensor& weight, Tensor& scale, double epsilon) {
  const int code = dtype_code("rms_norm_kernel_scalar_type", input);
  const auto dt = input.scalar_type();
  const auto dev = input.device();
  check_tensor("input", input, dt, dev);
  check_fp8_out(out, input);
  const Rows r = rows_of(input);
  check_weight(weight, r.H, dt, dev);
  check_scale(scale, dev);
  Launch l(input);
  check_rc(tw_rms_norm_static_fp8_quant(out.data_ptr(), input.data_ptr(), weight.data_ptr(),
                                        scale.data_ptr<float>(), r.T, r.H, (float)epsilon, code, l.stream));
}

void fused_add_rms_norm_static_fp8_quant(Tensor& out, Tensor& input, Tensor& residual, Tensor& weight,
                                         Tensor& scale, double epsilon) {
  const int code = dtype_code("fused_add_rms_norm_kernel_scalar_type", input);
  const auto dt = input.scalar_type();
  const auto dev = input.device();
  check_tensor("input", input, dt, dev);
  check_tensor("residual", residual, dt, dev);
  check_fp8_out(out, input);
  const Rows r = rows_of(input);
  TORCH_CHECK(residual.sizes() == input.sizes(), "input and residual must have the same shape");
  check_weight(weight, r.H, dt, dev);
  check_scale(scale, dev);
  Launch l(input);
  check_rc(tw_fused_add_rms_norm_static_fp8_quant(out.data_ptr(), input.data_ptr(), residual.data_ptr(),
                                                  weight.data_ptr(), scale.data_ptr<float>(), r.T, r.H,
                                                  (float)epsilon, code, l.stream));
}

// The launcher's checks (fused_layernorm_dynamic_per_token_quant.cu:139-147).
void rms_norm_dynamic_per_token_quant(Tensor& out, const Tensor& input, const Tensor& weight, Tensor& scales,
                                      double epsilon, std::optional<Tensor> scale_ub,
                                      std::optional<Tensor> residual) {
  const int code = dtype_code("rms_norm_dynamic_per_token_quant_dispatch", input);
  const auto dt = input.scalar_type();
  const auto dev = input.device();
  check_tensor("input", input, dt, dev);
  const Rows r = rows_of(input);
  TORCH_CHECK(out.is_cuda() && out.device() == dev, "result is on ", out.device(), ", expected ", dev);
  const bool fp8 = out.scalar_type() == at::kFloat8_e4m3fn;
  TORCH_CHECK(fp8 || out.scalar_type() == at::kChar, "result must be torch.float8_e4m3fn or torch.int8, got ",
              dtype_name(out.scalar_type()));
  TORCH_CHECK(out.is_contiguous() && out.sizes() == input.sizes(),
              "result must be contiguous and have the input's shape");
  TORCH_CHECK(scales.is_cuda() && scales.device() == dev && scales.scalar_type() == at::kFloat,
              "scales must be a float32 tensor on the input's device");
  TORCH_CHECK(scales.is_contiguous() && scales.numel() == r.T, "scales must hold ", r.T, " contiguous values");
  const float* ub = nullptr;
  if (scale_ub.has_value()) {
    TORCH_CHECK(fp8, "scale_ub is defined for fp8 output only");
    check_scale(*scale_ub, dev);
    ub = scale_ub->data_ptr<float>();
  }
  check_weight(weight, r.H, dt, dev);
  void* res = nullptr;
  if (residual.has_value()) {
    check_tensor("residual", *residual, dt, dev);
    TORCH_CHECK(residual->sizes() == input.sizes(), "input and residual must have the same shape");
    res = residual->data_ptr();
  }
  Launch l(input);
  check_rc(tw_rms_norm_dynamic_per_token_quant(out.data_ptr(), input.data_ptr(), weight.data_ptr(),
                                               scales.data_ptr<float>(), ub, res, r.T, r.H, (float)epsilon, code,
                                               fp8 ? TW_QUANT_FP8_E4M3FN : TW_QUANT_INT8, l.stream));
}

[[noreturn]] void no_cpu(const char* name) {
  TORCH_CHECK(false, "tokenweave_amd::", name,
              " has no CPU implementation: tokenweave_amd ops run on the GPU only; pass tensors that live on "
              "the MI355X");
}

}  // namespace

// Schema strings of the reference (csrc/torch_bindings.cpp:135-171, 199-219).
TORCH_LIBRARY(tokenweave_amd, m) {
  m.def("rms_norm(Tensor! result, Tensor input, Tensor weight, float epsilon) -> ()");
  m.def("fused_add_rms_norm(Tensor! input, Tensor! residual, Tensor weight, float epsilon) -> ()");
  m.def("rms_norm_inplace(Tensor! result, Tensor! input, Tensor weight, float epsilon) -> ()");
  m.def(
      "fused_rs_ln_ag_cta(Tensor! input, Tensor! residual, Tensor weight, int mcptr, int signal_pads, int rank, "
      "int world_size, int MAX_CTAS, float epsilon) -> ()");
  m.def("fused_add_rms_norm_cta(Tensor! input, Tensor! residual, Tensor weight, int MAX_CTAS, float epsilon) -> ()");
  m.def(
      "fused_rs_ln_cta(Tensor! input, Tensor! residual, Tensor weight, int mcptr, int signal_pads, int rank, "
      "int world_size, int MAX_CTAS, float epsilon) -> ()");
  m.def("rms_norm_static_fp8_quant(Tensor! result, Tensor input, Tensor weight, Tensor scale, float epsilon) -> ()");
  m.def(
      "fused_add_rms_norm_static_fp8_quant(Tensor! result, Tensor input, Tensor! residual, Tensor weight, "
      "Tensor scale, float epsilon) -> ()");
  m.def(
      "rms_norm_dynamic_per_token_quant(Tensor! result, Tensor input, Tensor weight, Tensor! scale, "
      "float epsilon, Tensor? scale_ub, Tensor!? residual) -> ()");
  // the staging regions behind `mcptr` (no tensors: registered for every backend)
  m.def("register_partials_region(int base, int stride_bytes, int slots, int usable_bytes, int token) -> ()",
        &register_partials_region);
  m.def("unregister_partials_region(int base, int token) -> ()", &unregister_partials_region);
  // the split-row workspace of the current stream, ahead of a graph capture
  m.def("prepare_split_workspace(int device_index) -> ()", &prepare_split_workspace);
}

TORCH_LIBRARY_IMPL(tokenweave_amd, CUDA, m) {
  m.impl("rms_norm", &rms_norm);
  m.impl("fused_add_rms_norm", &fused_add_rms_norm);
  m.impl("rms_norm_inplace", &rms_norm_inplace);
  m.impl("fused_rs_ln_ag_cta", &fused_rs_ln_ag_cta);
  m.impl("fused_add_rms_norm_cta", &fused_add_rms_norm_cta);
  m.impl("fused_rs_ln_cta", &fused_rs_ln_cta);
  m.impl("rms_norm_static_fp8_quant", &rms_norm_static_fp8_quant);
  m.impl("fused_add_rms_norm_static_fp8_quant", &fused_add_rms_norm_static_fp8_quant);
  m.impl("rms_norm_dynamic_per_token_quant", &rms_norm_dynamic_per_token_quant);
}

// CPU tensors: the dtype is judged first (as a dispatch over floating types would), then
// the call is refused.
TORCH_LIBRARY_IMPL(tokenweave_amd, CPU, m) {
  m.impl("rms_norm", [](Tensor&, Tensor& input, Tensor&, double) {
    dtype_code("rms_norm_kernel", input);
    no_cpu("rms_norm");
  });
  m.impl("fused_add_rms_norm", [](Tensor& input, Tensor&, Tensor&, double) {
    dtype_code("fused_add_rms_norm_kernel", input);
    no_cpu("fused_add_rms_norm");
  });
  m.impl("rms_norm_inplace", [](Tensor&, Tensor& input, Tensor&, double) {
    dtype_code("rms_norm_inplace_kernel", input);
    no_cpu("rms_norm_inplace");
  });
  m.impl("fused_rs_ln_ag_cta",
         [](Tensor& input, Tensor&, Tensor&, int64_t, int64_t, int64_t, int64_t, int64_t, double) {
           require_bf16("fused_rs_ln_ag_cta_kernel", input);
           no_cpu("fused_rs_ln_ag_cta");
         });
  m.impl("fused_add_rms_norm_cta", [](Tensor& input, Tensor&, Tensor&, int64_t, double) {
    require_bf16("fused_add_rms_norm_cta_kernel", input);
    no_cpu("fused_add_rms_norm_cta");
  });
  m.impl("fused_rs_ln_cta",
         [](Tensor& input, Tensor&, Tensor&, int64_t, int64_t, int64_t, int64_t, int64_t, double) {
           require_bf16("fused_rs_ln_cta_kernel", input);
           no_cpu("fused_rs_ln_cta");
         });
  m.impl("rms_norm_static_fp8_quant", [](Tensor&, Tensor& input, Tensor&, Tensor&, double) {
    dtype_code("rms_norm_kernel_scalar_type", input);
    no_cpu("rms_norm_static_fp8_quant");
  });
  m.impl("fused_add_rms_norm_static_fp8_quant", [](Tensor&, Tensor& input, Tensor&, Tensor&, Tensor&, double) {
    dtype_code("fused_add_rms_norm_kernel_scalar_type", input);
    no_cpu("fused_add_rms_norm_static_fp8_quant");
  });
  m.impl("rms_norm_dynamic_per_token_quant", [](Tensor&, const Tensor& input, const Tensor&, Tensor&, double,
                                                std::optional<Tensor>, std::optional<Tensor>) {
    dtype_code("rms_norm_dynamic_per_token_quant_dispatch", input);
    no_cpu("rms_norm_dynamic_per_token_quant");
  });
}
