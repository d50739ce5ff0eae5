/*
 * TEST INFRASTRUCTURE ONLY.  CPU restatement of the reference's fp32-accumulate
 * residual-add + RMSNorm path, extended to P partial-sum buffers.  Only tests,
 * the smoke check and the benchmark's cpu_baseline leg may load this library;
 * the product (tokenweave_amd) never does.
 *
 * Reference followed, line by line:
 *   csrc/cpu/layernorm.cpp:44-88   fused_add_rms_norm_impl  (operation order,
 *                                  which value is squared, which is re-read)
 *   csrc/cpu/layernorm.cpp:4-41    rms_norm_impl
 *   csrc/cpu/cpu_types_x86.hpp:208-241  FP32Vec8: 8 independent fp32 lane
 *                                  accumulators, reduce_sum = lanes 0..7 in order
 *   csrc/cpu/cpu_types_x86.hpp:229-231  bf16 -> f32 is a 16-bit left shift
 *   csrc/cpu/cpu_types_x86.hpp:647-698  f32 -> bf16: round-to-nearest-even when
 *                                  built with AVX512-BF16, truncation otherwise
 *   csrc/custom_all_reduce.cuh:286-294  P-way sum: fp32, fixed order p = 0..P-1,
 *                                  one down-cast at the end
 *   csrc/tokenweave_fused_kernels.cu:37-72  rms_norm_inplace (copy + normalise)
 *   csrc/quantization/fp8/common.cuh:38-56  static-scale fp8 conversion (the
 *                                  reference has no CPU twin of the norm+quant ops)
 *
 * Pinned by (tests/test_oracle_*.py): bit equality with the reference's own
 * layernorm.cpp compiled from its sources (oracle/_ref, truncating build) on the
 * reference's test grid; closed forms (constant / one-hot / zero rows); an
 * independent numpy fp32 restatement of RMSNorm.forward_native; float64 witness;
 * the fp8 conversion against torch's own CPU cast over every bf16 bit pattern;
 * the dynamic per-token quantisation against the composition the reference's own
 * test uses (tests/kernels/test_fused_quant_layernorm.py:51-72): forward_native
 * in numpy, then per-token scales and torch's CPU fp8 cast / numpy rint.
 *
 * Every function is built with -ffp-contract=off: the reference's vector code is
 * separate multiplies and adds (no FMA in its AVX2 build).
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#define TW_ROUND_RNE 0   /* AVX512-BF16 build of the reference */
#define TW_ROUND_TRUNC 1 /* every other x86 build of the reference */

static inline float bf16_to_f32(uint16_t v) {
  uint32_t u = (uint32_t)v << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

static inline uint16_t f32_to_bf16(float f, int mode) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if (mode == TW_ROUND_TRUNC) return (uint16_t)(u >> 16);
  if ((u & 0x7fffffffu) > 0x7f800000u) /* NaN: keep it quiet, as vcvtneps2bf16 */
    return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

/* Row kernel shared by every entry point.
 *   np == 0 : s = x            (rms_norm: nothing added, nothing written back)
 *   np >= 1 : s = (((p0 + p1) + ...) + p_{np-1}) + r   in fp32, r optional
 * sum of squares uses the UNROUNDED fp32 s (layernorm.cpp:65-67);
 * the normalised output re-reads the ROUNDED residual (layernorm.cpp:78-83). */
static void row_reduce_add_norm(const uint16_t* const* parts, int np,
                                int64_t row_off, uint16_t* res_row,
                                uint16_t* y_row, const uint16_t* w, float eps,
                                int H, int mode) {
  float lane[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  for (int j = 0; j < H; j += 8) {
    for (int k = 0; k < 8; ++k) {
      float s = bf16_to_f32(parts[0][row_off + j + k]);
      for (int p = 1; p < np; ++p) s = s + bf16_to_f32(parts[p][row_off + j + k]);
      if (res_row) s = s + bf16_to_f32(res_row[j + k]);
      float sq = s * s;
      lane[k] = lane[k] + sq;
      if (res_row) res_row[j + k] = f32_to_bf16(s, mode);
    }
  }
  float ss = 0.0f;
  for (int k = 0; k < 8; ++k) ss += lane[k];
  float mean = ss / (float)H;
  float inv = 1.0f / sqrtf(mean + eps);
  const uint16_t* src = res_row ? res_row : parts[0] + row_off;
  /* y_row may alias parts[*] + row_off: all reads of the row are done. */
  for (int j = 0; j < H; ++j) {
    float t = bf16_to_f32(src[j]) * inv;
    t = t * bf16_to_f32(w[j]);
    y_row[j] = f32_to_bf16(t, mode);
  }
}

/* x <- norm(x + r) * w ; r <- x + r.  layernorm.cpp:44-88. */
int tw_oracle_fused_add_rms_norm(uint16_t* x, uint16_t* r, const uint16_t* w,
                                 int64_t T, int64_t H, float eps, int mode) {
  if (H % 8 != 0 || H <= 0 || T < 0) return -1; /* TORCH_CHECK layernorm.cpp:52 */
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < T; ++i) {
    const uint16_t* parts[1] = {x};
    row_reduce_add_norm(parts, 1, i * H, r + i * H, x + i * H, w, eps, (int)H, mode);
  }
  return 0;
}

/* y <- norm(sum_p partial_p + r) * w ; r <- sum_p partial_p + r.
 * y may alias any partials[p].  P=1 with y == partials[0] is the function above. */
int tw_oracle_reduce_add_rms_norm(const uint16_t* const* partials, int P,
                                  uint16_t* y, uint16_t* r, const uint16_t* w,
                                  int64_t T, int64_t H, float eps, int mode) {
  if (H % 8 != 0 || H <= 0 || T < 0 || P < 1 || P > 64) return -1;
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < T; ++i)
    row_reduce_add_norm(partials, P, i * H, r + i * H, y + i * H, w, eps, (int)H, mode);
  return 0;
}

/* out <- norm(x) * w.  layernorm.cpp:4-41. */
int tw_oracle_rms_norm(uint16_t* out, const uint16_t* x, const uint16_t* w,
                       int64_t T, int64_t H, float eps, int mode) {
  if (H % 8 != 0 || H <= 0 || T < 0) return -1; /* TORCH_CHECK layernorm.cpp:11 */
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < T; ++i) {
    const uint16_t* parts[1] = {x};
    row_reduce_add_norm(parts, 0, i * H, 0, out + i * H, w, eps, (int)H, mode);
  }
  return 0;
}

/* out <- x (becomes the residual) ; x <- norm(x) * w.
 * tokenweave_fused_kernels.cu:37-72 with the CPU path's single rounding. */
int tw_oracle_rms_norm_inplace(uint16_t* out, uint16_t* x, const uint16_t* w,
                               int64_t T, int64_t H, float eps, int mode) {
  if (H % 8 != 0 || H <= 0 || T < 0) return -1;
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < T; ++i) {
    memcpy(out + i * H, x + i * H, (size_t)H * 2);
    const uint16_t* parts[1] = {x};
    row_reduce_add_norm(parts, 0, i * H, 0, x + i * H, w, eps, (int)H, mode);
  }
  return 0;
}

/* f32 -> OCP float8 e4m3fn (1-4-3, bias 7, max 448, no infinities), round to
 * nearest even, for |x| <= 448 (callers clamp first).  Normal numbers:
 * x = (1 + q/8) 2^e; subnormals: x = q 2^-9; in both cases the code is the
 * rounded significand added to the exponent field, so a carry out of the
 * mantissa lands in the exponent. */
static inline uint8_t f32_to_e4m3fn(float x) {
  uint32_t u;
  memcpy(&u, &x, 4);
  const uint8_t sign = (uint8_t)((u >> 24) & 0x80);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint8_t)(sign | 0x7f);
  float a = fabsf(x);
  int code;
  if (a < 0.015625f) { /* below 2^-6: subnormal grid of 2^-9 */
    code = (int)rintf(a * 512.0f);
  } else {
    int e;
    float m = frexpf(a, &e); /* a = m 2^e, m in [0.5, 1) */
    code = ((e - 1 + 7) << 3) + (int)rintf((m * 2.0f - 1.0f) * 8.0f);
  }
  if (code > 0x7e) code = 0x7e;
  return (uint8_t)(sign | code);
}

/* Static-scale quantisation of a bf16 tensor, scaled_fp8_conversion<true> of
 * csrc/quantization/fp8/common.cuh:38-56: x = f32(y) * (1.0f / scale), clamped to
 * +-448, converted with round-to-nearest-even.  This is what the reference's
 * unit test composes after the unquantised norm
 * (tests/kernels/test_layernorm.py:113-131). */
int tw_oracle_static_fp8_quant(uint8_t* out, const uint16_t* y, int64_t n, float scale) {
  if (n < 0) return -1;
  const float inv = 1.0f / scale;
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    float x = bf16_to_f32(y[i]) * inv;
    x = fmaxf(-448.0f, fminf(x, 448.0f));
    out[i] = f32_to_e4m3fn(x);
  }
  return 0;
}

/* Residual-add + RMSNorm + dynamic per-token quantisation, P partials.
 * Follows the reference's fused kernel, scalar path
 * (csrc/quantization/fused_kernels/layernorm_utils.cuh:19-126, called from
 * fused_layernorm_dynamic_per_token_quant.cu:64-83); the reference has no CPU twin.
 *   x      = sum_p f32(partial_p) + f32(r)                    (fp32; :28-31)
 *   rms    = 1/sqrt(sum x^2 / H + eps)   (unrounded x; :34,43 uses rsqrtf, whose CUDA
 *            implementation is within 2 ulp of this correctly rounded value)
 *   n      = f32( bf16( f32(bf16(x * rms)) * f32(w) ) )       (two roundings; :68,114)
 *   scale  = max( min(max_j |n_j|, *scale_ub) / qmax, min_scale )   (:80-88)
 *            qmax = 448, min_scale = 1/(448*512) for fp8 (csrc/quantization/utils.cuh:48-52);
 *            qmax = 127, min_scale = FLT_EPSILON for int8 (:55-59)
 *   r      <- bf16(x)                                         (:111)
 *   out    = fp8_rne(clamp(n / scale, +-448))   (division: quant_conversions.cuh:34-39,62-69)
 *          | int8_sat(rint(n * (1/scale)))      (fused_layernorm_..._quant.cu:32-36,
 *                                                quant_conversions.cuh:14-32,47-52)
 * The sum of squares is accumulated as in row_reduce_add_norm (the reference's GPU
 * order is a cub block reduction of unspecified association).
 * qkind: 0 = fp8 e4m3fn, 1 = int8.  r and scale_ub may be NULL. */
int tw_oracle_rms_norm_dynamic_per_token_quant(
    uint8_t* out, float* scales, const uint16_t* const* partials, int P, uint16_t* r,
    const uint16_t* w, const float* scale_ub, int64_t T, int64_t H, float eps, int qkind) {
  if (H <= 0 || T < 0 || P < 1 || P > 64 || (qkind != 0 && qkind != 1)) return -1;
  const float qmax = qkind == 0 ? 448.0f : 127.0f;
  const float min_scale = qkind == 0 ? 1.0f / (448.0f * 512.0f) : 1.1920928955078125e-07f;
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < T; ++i) {
    const int64_t off = i * H;
    float lane[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int64_t j = 0; j < H; ++j) {
      float x = bf16_to_f32(partials[0][off + j]);
      for (int p = 1; p < P; ++p) x = x + bf16_to_f32(partials[p][off + j]);
      if (r) x = x + bf16_to_f32(r[off + j]);
      float sq = x * x;
      lane[j & 7] = lane[j & 7] + sq;
    }
    float ss = 0.0f;
    for (int k = 0; k < 8; ++k) ss += lane[k];
    const float rms = 1.0f / sqrtf(ss / (float)H + eps);
    float amax = 0.0f;
    for (int pass = 0; pass < 2; ++pass) {
      float scale = 0.0f, scale_inv = 0.0f;
      if (pass == 1) {
        scale = scale_ub ? fminf(amax, *scale_ub) : amax;
        scale = fmaxf(scale / qmax, min_scale);
        scales[i] = scale;
        scale_inv = 1.0f / scale;
      }
      for (int64_t j = 0; j < H; ++j) {
        float x = bf16_to_f32(partials[0][off + j]);
        for (int p = 1; p < P; ++p) x = x + bf16_to_f32(partials[p][off + j]);
        if (r) x = x + bf16_to_f32(r[off + j]);
        float t = bf16_to_f32(f32_to_bf16(x * rms, TW_ROUND_RNE));
        float n = bf16_to_f32(f32_to_bf16(t * bf16_to_f32(w[j]), TW_ROUND_RNE));
        if (pass == 0) {
          amax = fmaxf(amax, fabsf(n));
        } else {
          if (r) r[off + j] = f32_to_bf16(x, TW_ROUND_RNE);
          if (qkind == 0) {
            float q = fmaxf(-448.0f, fminf(n / scale, 448.0f));
            out[off + j] = f32_to_e4m3fn(q);
          } else {
            float q = rintf(n * scale_inv);
            q = fmaxf(-128.0f, fminf(q, 127.0f));
            out[off + j] = (uint8_t)(int8_t)q;
          }
        }
      }
    }
  }
  return 0;
}

/* out[M,N] = bf16( sum_k f32(a[M,K]) * f32(b[N,K]) ), fp32 accumulate, k ascending.
 * Semantics of torch.matmul(x, W.t(), out=) at
 * vllm/model_executor/layers/linear.py:224 (accumulation order is the BLAS's
 * there; this is the plain order, compared under tolerance only). */
int tw_oracle_gemm_bf16_nt(uint16_t* out, const uint16_t* a, const uint16_t* b,
                           int64_t M, int64_t N, int64_t K, int mode) {
  if (M < 0 || N <= 0 || K <= 0) return -1;
#pragma omp parallel for schedule(static)
  for (int64_t m = 0; m < M; ++m) {
    for (int64_t n = 0; n < N; ++n) {
      float acc = 0.0f;
      for (int64_t k = 0; k < K; ++k)
        acc = acc + bf16_to_f32(a[m * K + k]) * bf16_to_f32(b[n * K + k]);
      out[m * N + n] = f32_to_bf16(acc, mode);
    }
  }
  return 0;
}
