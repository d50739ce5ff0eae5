// Fused P-partial reduce + residual-add + RMSNorm for gfx950 (MI355X, wave64).
//
// One workgroup owns one token row at a time and keeps the whole row in
// registers between the sum-of-squares reduction and the normalised store:
// every byte is read once and written once.  At hidden size 8192 and 224 rows or
// more a workgroup is 256 lanes (4 waves), each lane owning four 16-byte vectors
// (8 bf16 each) of the row in every buffer; it issues its 4*(P+1) loads back to
// back, so a row keeps (P+1)*16 KiB of HBM reads in flight.  With fewer rows a
// row is spread over 512 or 1024 lanes (two or one vector each).
//
// Memory policy, measured on MI355X with operands rotated through > 1 GiB:
//   * partial and residual loads carry the non-temporal bit: the data is used
//     once, and streaming it past the L2 / last-level cache replacement is worth
//     ~20 % of bandwidth against default loads;
//   * residual and output stores carry it too: the lines leave the L2 while the
//     kernel runs instead of in the write-back at its end (~10 % at 2048 rows);
//   * the weight row is loaded with the default policy and stays cached.
// Rows are addressed through buffer descriptors whose base is the row and whose
// extent is one row, so lanes past the end of a short row read zeros and their
// stores are dropped by the hardware: no tail branches.
//
// Rows are walked with stride gridDim.x, so the same kernel serves the
// one-workgroup-per-row launch (the default: fastest at every size measured) and
// the capped launch that leaves compute units to a concurrent GEMM.
//
// What this replaces in the reference: fused_rs_ln_ag_cta_kernel
// (csrc/tokenweave_fused_kernels.cu:80-155), fused_rs_ln_cta_kernel and
// fused_add_rms_norm_cta_kernel (csrc/tokenweave_artifact_kernels.cu:129-204,
// :38-104), fused_add_rms_norm_kernel / rms_norm_kernel
// (csrc/layernorm_kernels.cu:62-158, :22-54) and rms_norm_inplace_kernel
// (csrc/tokenweave_fused_kernels.cu:37-72).  Arithmetic follows the reference's
// CPU path (csrc/cpu/layernorm.cpp:44-88): fp32 sum, sum of squares of the
// unrounded sum, output computed from the rounded residual with one rounding.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "tw_common.h"

namespace tw {

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));

struct PartialPtrs {
  const void* p[TW_MAX_PARTIALS];
};

// Timeline stamps of the vector kernel.  They exist only in the measurement build of this
// file (the benchmark's own library defines TW_TRACE before including it): per token
// row, the constant-rate wall clock at a few program points and the hardware ids of
// the compute unit, written by lane 0 to a buffer the benchmark supplies.  The drained
// form first waits for the wave's outstanding memory operations.
#ifdef TW_TRACE
__device__ unsigned long long* g_trace;
constexpr int kTraceSlots = 8;
// The stamps of a row are collected in registers and written out after its last one, so
// that neither the trace pointer's load nor the stamp stores sit in the row's way.
#define TW_STAMP_BEGIN unsigned long long tw_stamps[kTraceSlots] = {}
#define TW_STAMP(row, i) tw_stamps[i] = wall_clock64()
#define TW_STAMP_DRAINED(row, i)                                                                 \
  do {                                                                                           \
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");                                             \
    TW_STAMP(row, i);                                                                            \
  } while (0)
#define TW_STAMP_HWID(row, i)                                                                    \
  tw_stamps[i] = ((unsigned long long)__builtin_amdgcn_s_getreg((4 - 1) << 11 | 20) << 32) |     \
                 (unsigned)__builtin_amdgcn_s_getreg((32 - 1) << 11 | 4)
#define TW_STAMP_END(row)                                                                        \
  do {                                                                                           \
    unsigned long long* tw_buf = g_trace; /* null outside a traced burst: nothing is written */  \
    if (threadIdx.x == 0 && tw_buf) {                                                            \
      for (int tw_i = 0; tw_i < kTraceSlots; ++tw_i)                                             \
        tw_buf[(size_t)(row) * kTraceSlots + tw_i] = tw_stamps[tw_i];                            \
    }                                                                                            \
  } while (0)
#else
#define TW_STAMP_BEGIN
#define TW_STAMP(row, i)
#define TW_STAMP_DRAINED(row, i)
#define TW_STAMP_HWID(row, i)
#define TW_STAMP_END(row)
#endif

// ---------------------------------------------------------------------------
// bf16 helpers.  A 32-bit word holds two bf16: element 2i in the low half.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float bf16_lo(uint32_t u) { return __uint_as_float(u << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t u) { return __uint_as_float(u & 0xffff0000u); }

// Round-to-nearest-even pack (v_cvt_pk_bf16_f32 on gfx950).
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

__device__ __forceinline__ void unpack8(const uint4& v, float (&f)[8]) {
  f[0] = bf16_lo(v.x); f[1] = bf16_hi(v.x);
  f[2] = bf16_lo(v.y); f[3] = bf16_hi(v.y);
  f[4] = bf16_lo(v.z); f[5] = bf16_hi(v.z);
  f[6] = bf16_lo(v.w); f[7] = bf16_hi(v.w);
}

__device__ __forceinline__ void add8(const uint4& v, float (&f)[8]) {
  f[0] += bf16_lo(v.x); f[1] += bf16_hi(v.x);
  f[2] += bf16_lo(v.y); f[3] += bf16_hi(v.y);
  f[4] += bf16_lo(v.z); f[5] += bf16_hi(v.z);
  f[6] += bf16_lo(v.w); f[7] += bf16_hi(v.w);
}

// The vector kernel's view of a 16-bit element type: widen a 32-bit word (element
// 2i in the low half) and narrow two floats with round-to-nearest-even.
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));

template <typename E> struct Pk;
template <> struct Pk<__bf16> {
  static __device__ __forceinline__ float lo(uint32_t u) { return bf16_lo(u); }
  static __device__ __forceinline__ float hi(uint32_t u) { return bf16_hi(u); }
  static __device__ __forceinline__ uint32_t pack(float a, float b) { return pack_bf16(a, b); }
};
template <> struct Pk<_Float16> {
  static __device__ __forceinline__ float lo(uint32_t u) { return (float)__builtin_bit_cast(f16x2_t, u).x; }
  static __device__ __forceinline__ float hi(uint32_t u) { return (float)__builtin_bit_cast(f16x2_t, u).y; }
  static __device__ __forceinline__ uint32_t pack(float a, float b) {
    f32x2_t v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2_t));
  }
};

template <typename E>
__device__ __forceinline__ void unpack8e(const uint4& v, float (&f)[8]) {
  f[0] = Pk<E>::lo(v.x); f[1] = Pk<E>::hi(v.x);
  f[2] = Pk<E>::lo(v.y); f[3] = Pk<E>::hi(v.y);
  f[4] = Pk<E>::lo(v.z); f[5] = Pk<E>::hi(v.z);
  f[6] = Pk<E>::lo(v.w); f[7] = Pk<E>::hi(v.w);
}

template <typename E>
__device__ __forceinline__ void add8e(const uint4& v, float (&f)[8]) {
  f[0] += Pk<E>::lo(v.x); f[1] += Pk<E>::hi(v.x);
  f[2] += Pk<E>::lo(v.y); f[3] += Pk<E>::hi(v.y);
  f[4] += Pk<E>::lo(v.z); f[5] += Pk<E>::hi(v.z);
  f[6] += Pk<E>::lo(v.w); f[7] += Pk<E>::hi(v.w);
}

// ---------------------------------------------------------------------------
// Sums with a fixed association order.
//
// wave_sum: 64 lanes -> the same total in every lane.  xor-1, xor-2 (quad
//   permutes), half-row mirror, row mirror on DPP leave every lane of a 16-lane
//   row with that row's sum; the four row sums are added as ((r0+r1)+r2)+r3
//   through v_readlane.
// block_sum (element-wise kernel): wave sums through one LDS slot per wave, one
//   barrier, every lane adds the slots in wave order.
// row_sum_chunks (vector kernel): the row is cut into chunks of 64 consecutive
//   16-byte vectors; chunk c is reduced with wave_sum by whichever wave owns it,
//   and the (at most 64) chunk sums, one per lane, are reduced with wave_sum again.  Lane t of a workgroup of
//   nt lanes owns vectors t, t + nt, ... (nt a multiple of 64), so the chunk of
//   its k-th vector is k * nt/64 + wave.  The result therefore depends only on
//   the row's data — not on the workgroup size or the vectors per lane — which
//   lets the launcher pick the workgroup shape per token count.
// LDS slots must not be reused before the next barrier (callers alternate
// between two slot arrays).
// ---------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
  int moved = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true);
  return v + __int_as_float(moved);
}

__device__ __forceinline__ float wave_sum(float v) {
  v = dpp_add<0xB1>(v);   // quad_perm:[1,0,3,2]
  v = dpp_add<0x4E>(v);   // quad_perm:[2,3,0,1]
  v = dpp_add<0x141>(v);  // row_half_mirror
  v = dpp_add<0x140>(v);  // row_mirror
  float r0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
  float r1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
  float r2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
  float r3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
  return ((r0 + r1) + r2) + r3;
}

__device__ __forceinline__ float block_sum(float v, float* slots, int nwaves) {
  v = wave_sum(v);
  if (nwaves == 1) return v;
  if ((threadIdx.x & 63) == 0) slots[threadIdx.x >> 6] = v;
  __syncthreads();
  float total = slots[0];
  for (int i = 1; i < nwaves; ++i) total += slots[i];
  return total;
}

// Maximum of non-negative values: the same DPP steps as wave_sum, then the
// workgroup's wave maxima through LDS (one slot per wave, at most 16).
template <int CTRL>
__device__ __forceinline__ float dpp_max(float v) {
  int moved = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true);
  return fmaxf(v, __int_as_float(moved));
}

__device__ __forceinline__ float wave_max(float v) {
  v = dpp_max<0xB1>(v);
  v = dpp_max<0x4E>(v);
  v = dpp_max<0x141>(v);
  v = dpp_max<0x140>(v);
  float r0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
  float r1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
  float r2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
  float r3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
  return fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
}

__device__ __forceinline__ float block_max(float v, float* slots, int nwaves) {
  v = wave_max(v);
  if (nwaves == 1) return v;
  const int lane = threadIdx.x & 63;
  if (lane == 0) slots[threadIdx.x >> 6] = v;
  __syncthreads();
  return wave_max(lane < nwaves ? slots[lane] : 0.0f);
}

constexpr int kMaxChunks = 64;  // 4096 vectors = hidden size 32768

template <int VPT>
__device__ __forceinline__ float row_sum_chunks(const float (&per_vec)[VPT], float* slots,
                                                int nwaves, int nchunks) {
  const int wave = threadIdx.x >> 6;
  float c[VPT];
#pragma unroll
  for (int k = 0; k < VPT; ++k) c[k] = wave_sum(per_vec[k]);
  if (VPT == 1 && nwaves == 1) return c[0];
  if ((threadIdx.x & 63) == 0) {
#pragma unroll
    for (int k = 0; k < VPT; ++k) slots[k * nwaves + wave] = c[k];
  }
  __syncthreads();
  const int lane = threadIdx.x & 63;
  return wave_sum(lane < nchunks ? slots[lane] : 0.0f);
}

__device__ __forceinline__ float inv_rms(float ss, float hidden, float eps) {
  // Same expression as csrc/cpu/layernorm.cpp:72-73; hipcc keeps fp32 division
  // and sqrt correctly rounded.
  return 1.0f / sqrtf(ss / hidden + eps);
}

// ---------------------------------------------------------------------------
// Row addressing: one buffer descriptor per (tensor, row).  Offsets inside a row
// are 32-bit; an access that does not fit inside the row's extent reads zeros /
// is not written.  Cache-policy bits of the raw buffer intrinsics on gfx950:
// 1 = sc0, 2 = nt, 16 = sc1.
// ---------------------------------------------------------------------------
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
constexpr int kLoadStream = 2;    // nt
constexpr int kLoadCached = 0;
constexpr int kStoreStream = 2;  // nt

__device__ __forceinline__ __amdgpu_buffer_rsrc_t row_desc(const void* base, size_t row,
                                                           uint32_t row_bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(
      const_cast<char*>(static_cast<const char*>(base)) + row * row_bytes, 0, row_bytes, 0x00020000);
}

template <int AUX>
__device__ __forceinline__ uint4 load16(__amdgpu_buffer_rsrc_t d, uint32_t off) {
  u32x4_t t = __builtin_amdgcn_raw_buffer_load_b128(d, off, 0, AUX);
  return make_uint4(t.x, t.y, t.z, t.w);
}

// Static-scale fp8 (OCP e4m3fn) quantisation of four values: multiply by the
// inverted scale, clamp to the finite range, round to nearest even
// (v_cvt_pk_fp8_f32).  scaled_fp8_conversion<true> of the reference
// (csrc/quantization/fp8/common.cuh:38-56).
constexpr float kFp8Max = 448.0f;
__device__ __forceinline__ uint32_t quant4_fp8(float a, float b, float c, float d, float scale_inv) {
  a = fmaxf(-kFp8Max, fminf(a * scale_inv, kFp8Max));
  b = fmaxf(-kFp8Max, fminf(b * scale_inv, kFp8Max));
  c = fmaxf(-kFp8Max, fminf(c * scale_inv, kFp8Max));
  d = fmaxf(-kFp8Max, fminf(d * scale_inv, kFp8Max));
  int r = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
  r = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, r, true);
  return (uint32_t)r;
}

// Output kinds.  Static fp8 quantises the bf16 result of the unquantised op with a
// caller-supplied scale.  The two dynamic kinds follow the reference's fused kernel
// (csrc/quantization/fused_kernels/layernorm_utils.cuh:51-124): the normalised value
// is n = bf16(bf16(s * inv) * w) computed from the unrounded fp32 sum s, the row's
// scale is max(min(max|n|, ub) / qmax, floor), and the codes are
// fp8(clamp(n / scale)) or int8(sat(rint(n * (1 / scale)))).
constexpr int kQNone = 0, kQStaticFp8 = 1, kQDynFp8 = 2, kQDynInt8 = 3;
constexpr float kFp8MinScale = 1.0f / (448.0f * 512.0f);  // csrc/quantization/utils.cuh:48-52
constexpr float kInt8MinScale = 1.1920928955078125e-07f;  // FLT_EPSILON, utils.cuh:55-59

__device__ __forceinline__ float dyn_scale(float amax, const float* scale_ub, bool int8) {
  float sc = scale_ub ? fminf(amax, *scale_ub) : amax;
  return int8 ? fmaxf(sc / 127.0f, kInt8MinScale) : fmaxf(sc / kFp8Max, kFp8MinScale);
}

// Four values -> four fp8 codes, true division by the scale
// (quant_conversions.cuh:34-39,62-69).
__device__ __forceinline__ uint32_t quant4_fp8_div(float a, float b, float c, float d, float scale) {
  a = fmaxf(-kFp8Max, fminf(a / scale, kFp8Max));
  b = fmaxf(-kFp8Max, fminf(b / scale, kFp8Max));
  c = fmaxf(-kFp8Max, fminf(c / scale, kFp8Max));
  d = fmaxf(-kFp8Max, fminf(d / scale, kFp8Max));
  int r = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
  r = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, r, true);
  return (uint32_t)r;
}

// Round to nearest even, saturate (quant_conversions.cuh:14-32).
__device__ __forceinline__ uint32_t quant1_int8(float x, float scale_inv) {
  float q = fmaxf(-128.0f, fminf(__builtin_rintf(x * scale_inv), 127.0f));
  return (uint32_t)(int)q & 0xffu;
}

__device__ __forceinline__ uint32_t quant4_int8(float a, float b, float c, float d, float scale_inv) {
  return quant1_int8(a, scale_inv) | (quant1_int8(b, scale_inv) << 8) |
         (quant1_int8(c, scale_inv) << 16) | (quant1_int8(d, scale_inv) << 24);
}

typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void store8(__amdgpu_buffer_rsrc_t d, uint32_t off, uint32_t lo, uint32_t hi) {
  u32x2_t t = {lo, hi};
  __builtin_amdgcn_raw_buffer_store_b64(t, d, off, 0, kStoreStream);
}

__device__ __forceinline__ void store16(__amdgpu_buffer_rsrc_t d, uint32_t off, const uint4& v) {
  u32x4_t t = {v.x, v.y, v.z, v.w};
  __builtin_amdgcn_raw_buffer_store_b128(t, d, off, 0, kStoreStream);
}

// ---------------------------------------------------------------------------
// Vector kernel, 16-bit element types (bf16; fp16 for the P = 1 ops).
//   NP       number of partial buffers known at compile time, 0 = use np_rt
//   VPT      16-byte vectors per lane per buffer; lane t owns vectors
//            t, t + blockDim, ... (row length <= VPT * blockDim * 8 elements)
//   HAS_RES  add the residual and write the rounded sum back to it
//   COPY     also store the untouched first partial to `copy_out`
//            (rms_norm_inplace: the copy becomes the residual stream)
// y may alias any partial: a lane stores y only to vector slots it has already
// read in every buffer.  blockDim.x must be a multiple of 64.
// ---------------------------------------------------------------------------
//   Q        output kind (kQNone .. kQDynInt8); quant_scale is the static scale
//            (kQStaticFp8) or the optional upper bound of the row scale (kQDynFp8)
//   E        element type of every tensor (__bf16 or _Float16)
template <typename E, int NP, int VPT, int MAXNT, bool HAS_RES, bool COPY, int Q>
__device__ __forceinline__ void row_norm_vec_body(
    const PartialPtrs& parts, int np_rt, void* y_out, void* residual, void* copy_out,
    const void* __restrict__ weight, const float* __restrict__ quant_scale,
    float* __restrict__ row_scales, float eps, int num_tokens, int vec_per_row, float hidden, int nt, int grid,
    float (*slots)[kMaxChunks], float (*max_slots)[16]) {
  constexpr bool FP8 = Q == kQStaticFp8;
  // nt = lanes per workgroup and grid = workgroups come as kernel arguments, and the
  // launcher never starts more workgroups than there are rows (the row loop tests at
  // its end): read from the dispatch packet's hidden arguments (blockDim, gridDim), and
  // with a test of the row count ahead of the first row, the kernel would make two more
  // dependent memory round trips before the row's first load can go out.
  const int nwaves = nt >> 6;
  const int nchunks = (vec_per_row + 63) >> 6;  // <= VPT * nwaves
  const int np = NP > 0 ? NP : np_rt;
  const uint32_t row_bytes = (uint32_t)vec_per_row * 16u;
  uint32_t off[VPT];
#pragma unroll
  for (int k = 0; k < VPT; ++k) off[k] = (threadIdx.x + k * nt) * 16u;

  const __amdgpu_buffer_rsrc_t dw = row_desc(weight, 0, row_bytes);
  // The static scale / the optional bound of the dynamic scale: one scalar, read ahead
  // of the row loop so that its latency is not behind the reduction.
  float qparam = __builtin_inff();
  if (Q != kQNone && quant_scale) qparam = *quant_scale;

  int phase = 0;
  int row = blockIdx.x;
  do {
    float s[VPT][8];
    uint4 first[VPT];
    uint4 wv[VPT];     // the weight row is fetched per token row, behind the row's own loads
    TW_STAMP_BEGIN;
    TW_STAMP(row, 0);  // row begins
    TW_STAMP_HWID(row, 6);
    const __amdgpu_buffer_rsrc_t dr = row_desc(HAS_RES ? residual : parts.p[0], row, row_bytes);

    if (NP > 0 && (VPT <= 2 || MAXNT <= 256)) {
      // Issue every load of the row before the first use.  (Four vectors per lane
      // in a workgroup of more than 256 lanes would not fit the register file;
      // those rows accumulate one partial at a time below.)
      uint4 a[VPT][NP > 0 ? NP : 1];
      uint4 rv[VPT];
#pragma unroll
      for (int p = 0; p < NP; ++p) {
        const __amdgpu_buffer_rsrc_t dp = row_desc(parts.p[p], row, row_bytes);
#pragma unroll
        for (int k = 0; k < VPT; ++k) a[k][p] = load16<kLoadStream>(dp, off[k]);
      }
      if (HAS_RES) {
#pragma unroll
        for (int k = 0; k < VPT; ++k) rv[k] = load16<kLoadStream>(dr, off[k]);
      }
      // Nothing below may be scheduled above this point and no load of the row below
      // it: the compiler would otherwise trade loads in flight for registers.
      __builtin_amdgcn_sched_barrier(0);
      // The weight row goes last: an L2 hit after the first workgroups, and its
      // (cold) latency must not sit ahead of the row's own loads.  (Issued ahead of
      // the barrier it costs the P = 1 op 8 % at 512 rows.)
#pragma unroll
      for (int k = 0; k < VPT; ++k) wv[k] = load16<kLoadCached>(dw, off[k]);
      // Accumulate stream by stream, in the order the loads were issued: the arithmetic
      // on the first partials runs while the later ones are still on their way.  (Per
      // element the order of the additions is p = 0 .. P-1, then the residual, either way.)
#pragma unroll
      for (int k = 0; k < VPT; ++k) {
        first[k] = a[k][0];
        unpack8e<E>(a[k][0], s[k]);
      }
#pragma unroll
      for (int p = 1; p < NP; ++p) {
#pragma unroll
        for (int k = 0; k < VPT; ++k) add8e<E>(a[k][p], s[k]);
      }
      if (HAS_RES) {
#pragma unroll
        for (int k = 0; k < VPT; ++k) add8e<E>(rv[k], s[k]);
      }
    } else {
      {
        const __amdgpu_buffer_rsrc_t dp = row_desc(parts.p[0], row, row_bytes);
#pragma unroll
        for (int k = 0; k < VPT; ++k) {
          first[k] = load16<kLoadStream>(dp, off[k]);
          unpack8e<E>(first[k], s[k]);
        }
      }
      for (int p = 1; p < np; ++p) {
        const __amdgpu_buffer_rsrc_t dp = row_desc(parts.p[p], row, row_bytes);
#pragma unroll
        for (int k = 0; k < VPT; ++k) add8e<E>(load16<kLoadStream>(dp, off[k]), s[k]);
      }
      if (HAS_RES) {
#pragma unroll
        for (int k = 0; k < VPT; ++k) add8e<E>(load16<kLoadStream>(dr, off[k]), s[k]);
      }
#pragma unroll
      for (int k = 0; k < VPT; ++k) wv[k] = load16<kLoadCached>(dw, off[k]);
    }

    TW_STAMP_DRAINED(row, 1);  // every load of the row (and the weight) has returned
    if (COPY) {
      const __amdgpu_buffer_rsrc_t dc = row_desc(copy_out, row, row_bytes);
#pragma unroll
      for (int k = 0; k < VPT; ++k) store16(dc, off[k], first[k]);
    }

    // Sum of squares of the unrounded fp32 sum, one running sum per vector; round
    // the residual once.  (Lanes past the row's end hold zeros and add nothing.)
    float ss[VPT];
    uint4 rnew[VPT];
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
      ss[k] = 0.0f;
#pragma unroll
      for (int e = 0; e < 8; ++e) ss[k] += s[k][e] * s[k][e];
      rnew[k].x = Pk<E>::pack(s[k][0], s[k][1]);
      rnew[k].y = Pk<E>::pack(s[k][2], s[k][3]);
      rnew[k].z = Pk<E>::pack(s[k][4], s[k][5]);
      rnew[k].w = Pk<E>::pack(s[k][6], s[k][7]);
      if (HAS_RES) store16(dr, off[k], rnew[k]);
    }

    TW_STAMP(row, 2);  // residual stores issued
    const float total = row_sum_chunks<VPT>(ss, slots[phase], nwaves, nchunks);
    const float inv = inv_rms(total, hidden, eps);
    TW_STAMP(row, 3);  // row sum known

    // bf16 output: 16 bytes per vector; fp8 output: the bf16 result quantised, 8 bytes
    // per vector in rows of half the size.
    const __amdgpu_buffer_rsrc_t dy = row_desc(y_out, row, Q != kQNone ? row_bytes / 2 : row_bytes);
    if (Q == kQDynFp8 || Q == kQDynInt8) {
      uint4 nv[VPT];
      float amax = 0.0f;
#pragma unroll
      for (int k = 0; k < VPT; ++k) {
        float w[8], t[8];
        unpack8e<E>(wv[k], w);
        uint4 tv;
        tv.x = Pk<E>::pack(s[k][0] * inv, s[k][1] * inv);
        tv.y = Pk<E>::pack(s[k][2] * inv, s[k][3] * inv);
        tv.z = Pk<E>::pack(s[k][4] * inv, s[k][5] * inv);
        tv.w = Pk<E>::pack(s[k][6] * inv, s[k][7] * inv);
        unpack8e<E>(tv, t);
        nv[k].x = Pk<E>::pack(t[0] * w[0], t[1] * w[1]);
        nv[k].y = Pk<E>::pack(t[2] * w[2], t[3] * w[3]);
        nv[k].z = Pk<E>::pack(t[4] * w[4], t[5] * w[5]);
        nv[k].w = Pk<E>::pack(t[6] * w[6], t[7] * w[7]);
        unpack8e<E>(nv[k], t);
#pragma unroll
        for (int e = 0; e < 8; ++e) amax = fmaxf(amax, fabsf(t[e]));
      }
      amax = block_max(amax, max_slots[phase], nwaves);
      const float scale = dyn_scale(fminf(amax, qparam), nullptr, Q == kQDynInt8);
      if (threadIdx.x == 0) row_scales[row] = scale;
      const float sinv = 1.0f / scale;
#pragma unroll
      for (int k = 0; k < VPT; ++k) {
        float n[8];
        unpack8e<E>(nv[k], n);
        if (Q == kQDynInt8)
          store8(dy, off[k] / 2, quant4_int8(n[0], n[1], n[2], n[3], sinv),
                 quant4_int8(n[4], n[5], n[6], n[7], sinv));
        else
          store8(dy, off[k] / 2, quant4_fp8_div(n[0], n[1], n[2], n[3], scale),
                 quant4_fp8_div(n[4], n[5], n[6], n[7], scale));
      }
    } else {
      const float scale_inv = 1.0f / qparam;
#pragma unroll
      for (int k = 0; k < VPT; ++k) {
        float r[8], w[8];
        unpack8e<E>(rnew[k], r);
        unpack8e<E>(wv[k], w);
        uint4 o;
        o.x = Pk<E>::pack(r[0] * inv * w[0], r[1] * inv * w[1]);
        o.y = Pk<E>::pack(r[2] * inv * w[2], r[3] * inv * w[3]);
        o.z = Pk<E>::pack(r[4] * inv * w[4], r[5] * inv * w[5]);
        o.w = Pk<E>::pack(r[6] * inv * w[6], r[7] * inv * w[7]);
        if (FP8) {
          float y[8];
          unpack8e<E>(o, y);
          store8(dy, off[k] / 2, quant4_fp8(y[0], y[1], y[2], y[3], scale_inv),
                 quant4_fp8(y[4], y[5], y[6], y[7], scale_inv));
        } else {
          store16(dy, off[k], o);
        }
      }
    }
    TW_STAMP(row, 4);          // y stores issued
    TW_STAMP_DRAINED(row, 5);  // every store of the row acknowledged
    TW_STAMP_END(row);
    row += grid;
    phase ^= 1;
  } while (row < num_tokens);
}

template <int NP, int VPT, int MAXNT, bool HAS_RES, bool COPY, int Q>
__global__ __launch_bounds__(MAXNT) void row_norm_bf16_kernel(
    PartialPtrs parts, int np_rt, void* y_out, void* residual, void* copy_out,
    const void* __restrict__ weight, const float* __restrict__ quant_scale,
    float* __restrict__ row_scales, float eps, int num_tokens, int vec_per_row, float hidden, int nt, int grid) {
  __shared__ float slots[2][kMaxChunks];
  __shared__ float max_slots[2][16];
  row_norm_vec_body<__bf16, NP, VPT, MAXNT, HAS_RES, COPY, Q>(parts, np_rt, y_out, residual, copy_out, weight,
                                                            quant_scale, row_scales, eps, num_tokens,
                                                            vec_per_row, hidden, nt, grid, slots, max_slots);
}

// fp16 tensors reach the library through the P = 1 ops only.
template <int VPT, int MAXNT, bool HAS_RES, bool COPY, int Q>
__global__ __launch_bounds__(MAXNT) void row_norm_f16_kernel(
    PartialPtrs parts, void* y_out, void* residual, void* copy_out, const void* __restrict__ weight,
    const float* __restrict__ quant_scale, float* __restrict__ row_scales, float eps, int num_tokens,
    int vec_per_row, float hidden, int nt, int grid) {
  __shared__ float slots[2][kMaxChunks];
  __shared__ float max_slots[2][16];
  row_norm_vec_body<_Float16, 1, VPT, MAXNT, HAS_RES, COPY, Q>(parts, 1, y_out, residual, copy_out, weight,
                                                             quant_scale, row_scales, eps, num_tokens,
                                                             vec_per_row, hidden, nt, grid, slots, max_slots);
}

// ---------------------------------------------------------------------------
// Split rows: few token rows, many compute units (decode batches).
//
// A row is cut into `segs` segments of whole 64-vector chunks and every segment
// gets its own workgroup (one vector per lane, one chunk per wave), so one row's
// (P + 1) input streams are pulled by several compute units at once.  A segment
// workgroup does the first half of the row kernel on its vectors — fp32 sum,
// rounded residual stored, one sum of squares per chunk by wave_sum — and leaves
// its chunk sums in the row's slot of a small workspace.  It then counts itself in
// on the row's arrival counter.  The workgroup that arrives last finds every chunk
// sum of the row there, reduces them exactly as row_sum_chunks does (chunk c in
// lane c, one wave_sum), and writes y for the WHOLE row from the rounded residual
// it re-reads — the same operands in the same order as the one-workgroup kernel,
// hence the same bits.  Nobody waits for anybody: a workgroup that is not last is
// finished, so the kernel makes progress whatever the dispatch order and needs no
// co-residency.
//
// The last workgroup of a row resets the row's counter, so the counters are zero
// again when the kernel ends; calls that share a workspace must not overlap in time.
//
// XCD_ROWS: workgroup b serves row 8 (b / (8 segs)) + b % 8, segment (b / 8) % segs,
// so the segments of one row have equal b % 8 and — with the dispatcher handing
// consecutive workgroups to consecutive XCDs — run on one XCD, whose L2 then holds
// the residual for the last workgroup's re-read (0.1 - 0.3 us).  That placement is
// a speed matter only: the hand-over below is written for segments on different
// XCDs, and the form without the remap (row = b / segs, segments of a row spread
// over XCDs) is compiled into the measurement library and checked by the tests
// against the same bits.
// ---------------------------------------------------------------------------
struct SplitRow {
  float sums[kMaxChunks];  // chunk sums of squares of the row in flight (two 128-byte lines)
  uint32_t arrived;        // segment workgroups that have delivered theirs (a line of its own)
  uint32_t pad[31];
};
static_assert(sizeof(SplitRow) * TW_SPLIT_MAX_TOKENS == TW_SPLIT_WORKSPACE_BYTES,
              "workspace layout and the public size disagree");

constexpr int kLoadDevice = 16;   // sc1: coherent at device scope
constexpr int kStoreDevice = 16;  // sc1: written through to device scope

__device__ __forceinline__ void store16_device(__amdgpu_buffer_rsrc_t d, uint32_t off, const uint4& v) {
  u32x4_t t = {v.x, v.y, v.z, v.w};
  __builtin_amdgcn_raw_buffer_store_b128(t, d, off, 0, kStoreDevice);
}

// One segment of a split row: VPT * nwaves whole chunks starting at chunk `chunk0` of row
// `row` (wave w of the workgroup owns chunks chunk0 + k * nwaves + w, k < VPT: the same
// lane-to-vector assignment as the row kernel's, segment by segment).  `lds_flag` is one
// LDS word of the caller's.
template <int NP, int VPT>
__device__ __forceinline__ void split_segment(
    const PartialPtrs& parts, int np_rt, void* y_out, void* residual, const void* __restrict__ weight,
    SplitRow* __restrict__ slot, float eps, int row, int chunk0, int vec_per_row, float hidden, int segs, int nt,
    uint32_t* lds_flag) {
  const int nwaves = nt >> 6;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int nchunks = (vec_per_row + 63) >> 6;
  const int np = NP > 0 ? NP : np_rt;
  const uint32_t row_bytes = (uint32_t)vec_per_row * 16u;
  uint32_t off[VPT];
#pragma unroll
  for (int k = 0; k < VPT; ++k) off[k] = (uint32_t)((chunk0 + k * nwaves + wave) * 64 + lane) * 16u;

  const __amdgpu_buffer_rsrc_t dr = row_desc(residual, row, row_bytes);
  float s[VPT][8];
  if (NP > 0) {
    uint4 a[VPT][NP > 0 ? NP : 1];
    uint4 rv[VPT];
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      const __amdgpu_buffer_rsrc_t dp = row_desc(parts.p[p], row, row_bytes);
#pragma unroll
      for (int k = 0; k < VPT; ++k) a[k][p] = load16<kLoadStream>(dp, off[k]);
    }
#pragma unroll
    for (int k = 0; k < VPT; ++k) rv[k] = load16<kLoadStream>(dr, off[k]);
#pragma unroll
    for (int k = 0; k < VPT; ++k) unpack8(a[k][0], s[k]);
#pragma unroll
    for (int p = 1; p < NP; ++p) {
#pragma unroll
      for (int k = 0; k < VPT; ++k) add8(a[k][p], s[k]);
    }
#pragma unroll
    for (int k = 0; k < VPT; ++k) add8(rv[k], s[k]);
  } else {
    {
      const __amdgpu_buffer_rsrc_t dp = row_desc(parts.p[0], row, row_bytes);
#pragma unroll
      for (int k = 0; k < VPT; ++k) unpack8(load16<kLoadStream>(dp, off[k]), s[k]);
    }
    for (int p = 1; p < np; ++p) {
      const __amdgpu_buffer_rsrc_t dp = row_desc(parts.p[p], row, row_bytes);
#pragma unroll
      for (int k = 0; k < VPT; ++k) add8(load16<kLoadStream>(dp, off[k]), s[k]);
    }
#pragma unroll
    for (int k = 0; k < VPT; ++k) add8(load16<kLoadStream>(dr, off[k]), s[k]);
  }

#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    float ss = 0.0f;
#pragma unroll
    for (int e = 0; e < 8; ++e) ss += s[k][e] * s[k][e];
    uint4 rnew;
    rnew.x = pack_bf16(s[k][0], s[k][1]);
    rnew.y = pack_bf16(s[k][2], s[k][3]);
    rnew.z = pack_bf16(s[k][4], s[k][5]);
    rnew.w = pack_bf16(s[k][6], s[k][7]);
    store16_device(dr, off[k], rnew);
    const float c = wave_sum(ss);
    const int chunk = chunk0 + k * nwaves + wave;
    if (lane == 0 && chunk < nchunks)
      __hip_atomic_store(&slot->sums[chunk], c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }

  // The hand-over, instruction by instruction.  It is built from device-scope accesses
  // and explicit waits instead of release / acquire fences, because a fence at agent
  // scope is an L2 write-back (buffer_wbl2) per wave, serialised per XCD: 2 - 20x the
  // kernel's whole duration.  What it relies on is stated here so that it can be checked:
  //  (1) Everything another workgroup will read — the rounded residual (store16_device)
  //      and the chunk sums (relaxed agent-scope atomic stores) — is written with sc1
  //      stores: the data is written through this XCD's L2 to memory, and the store's
  //      acknowledgement (what vmcnt counts) comes back only after that.  No dirty line
  //      is left behind in an L2 that another XCD cannot see, so nothing needs writing back.
  //  (2) s_waitcnt vmcnt(0): this wave goes on only when every one of its stores has
  //      been acknowledged.  s_barrier: every wave of the workgroup has done so.
  //  (3) Only then thread 0 counts the workgroup in, with an agent-scope atomic
  //      read-modify-write (performed at the memory side, one total order per counter).
  //      A workgroup that reads segs - 1 therefore knows that every other segment's
  //      stores of (1) were acknowledged before that segment's increment, which precedes
  //      its own in the counter's order.
  //  (4) The last workgroup's reads of the chunk sums and of the residual are issued after
  //      the atomic's value has come back (the branch below depends on it; vector memory
  //      instructions are issued in program order, never speculatively), and they are sc1
  //      loads: served from memory at device scope, not from a line an earlier access may
  //      have left in this compute unit's cache or this XCD's L2.  The residual lines are
  //      read before that only by the segment that overwrites them, with streaming loads.
  //  The weight row and y are ordinary traffic: nobody else reads or writes them here.
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (threadIdx.x == 0)
    *lds_flag = __hip_atomic_fetch_add(&slot->arrived, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __syncthreads();
  if (*lds_flag != (uint32_t)(segs - 1)) return;

  // Last workgroup of the row: all chunk sums are in the slot.
  if (threadIdx.x == 0) __hip_atomic_store(&slot->arrived, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const float cs = lane < nchunks
                       ? __hip_atomic_load(&slot->sums[lane], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                       : 0.0f;
  const float inv = inv_rms(wave_sum(cs), hidden, eps);

  const __amdgpu_buffer_rsrc_t dw = row_desc(weight, 0, row_bytes);
  const __amdgpu_buffer_rsrc_t dy = row_desc(y_out, row, row_bytes);
  constexpr int U = 4;  // vectors in flight per lane
  for (int v0 = threadIdx.x; v0 < vec_per_row; v0 += U * nt) {
    uint4 rv[U], wv[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t o = (uint32_t)(v0 + u * nt) * 16u;  // past the row's end: zeros, store dropped
      rv[u] = load16<kLoadDevice>(dr, o);
      wv[u] = load16<kLoadCached>(dw, o);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      float r[8], w[8];
      unpack8(rv[u], r);
      unpack8(wv[u], w);
      uint4 o;
      o.x = pack_bf16(r[0] * inv * w[0], r[1] * inv * w[1]);
      o.y = pack_bf16(r[2] * inv * w[2], r[3] * inv * w[3]);
      o.z = pack_bf16(r[4] * inv * w[4], r[5] * inv * w[5]);
      o.w = pack_bf16(r[6] * inv * w[6], r[7] * inv * w[7]);
      store16(dy, (uint32_t)(v0 + u * nt) * 16u, o);
    }
  }
}

template <int NP, bool XCD_ROWS>
__global__ __launch_bounds__(1024) void row_norm_split_kernel(
    PartialPtrs parts, int np_rt, void* y_out, void* residual, const void* __restrict__ weight,
    SplitRow* __restrict__ ws, float eps, int num_tokens, int vec_per_row, float hidden, int segs, int nt) {
  __shared__ uint32_t arrivals_before;
  // nt = lanes per workgroup, as a kernel argument (see row_norm_vec_body)
  const int per_group = 8 * segs;
  const int row = XCD_ROWS ? (blockIdx.x / per_group) * 8 + (blockIdx.x & 7) : blockIdx.x / segs;
  const int seg = XCD_ROWS ? (blockIdx.x % per_group) >> 3 : blockIdx.x % segs;
  // The first partial's pointer is demanded here so that its load goes out with the
  // row count's: one round trip to the kernel arguments ahead of the test, and the loads
  // that follow find their cache lines there.
  asm volatile("" ::"s"(parts.p[0]));
  if (row >= num_tokens) return;
  split_segment<NP, 1>(parts, np_rt, y_out, residual, weight, ws + row, eps, row, seg * (nt >> 6), vec_per_row,
                       hidden, segs, nt, &arrivals_before);
}

// ---------------------------------------------------------------------------
// Mixed launch: a few more rows than compute units.
//
// With one workgroup per row, row counts just above the number of compute units leave
// some units with two rows and the rest with one, and the launch takes as long as two
// rows on one unit: 257 .. 400 rows all cost what 512 do.  Here the first `full` rows (one
// per compute unit) go to one workgroup each as usual, and the excess rows are cut into
// `segs` segments (halves or quarters of a row), each a workgroup of its own, handed over
// through the workspace like the split rows above: every unit then carries its row plus
// at most one segment (the launcher offers this up to a quarter more rows than units).  Same
// bits as the one-workgroup kernel (the chunk sums are reduced
// in the same order).  Workgroup b >= full serves excess row 8 ((b - full) / (8 segs)) +
// b % 8, segment ((b - full) / 8) % segs (`full` is a multiple of 8: the segments of a row
// share an XCD).
// ---------------------------------------------------------------------------
template <int NP, int SEG_VPT>
__global__ __launch_bounds__(256) void row_norm_mixed_kernel(
    PartialPtrs parts, int np_rt, void* y_out, void* residual, const void* __restrict__ weight,
    SplitRow* __restrict__ ws, float eps, int num_tokens, int vec_per_row, float hidden, int full, int segs,
    int nt) {
  __shared__ float slots[2][kMaxChunks];
  __shared__ float max_slots[2][16];
  __shared__ uint32_t arrivals_before;
  if ((int)blockIdx.x < full) {
    // rows [0, full): exactly one row per workgroup (row loop with stride = row count)
    row_norm_vec_body<__bf16, NP, 4, 256, true, false, kQNone>(parts, np_rt, y_out, residual, nullptr, weight,
                                                              nullptr, nullptr, eps, full, vec_per_row, hidden, nt,
                                                              full, slots, max_slots);
    return;
  }
  const int b = (int)blockIdx.x - full;
  const int per_group = 8 * segs;
  const int row = full + (b / per_group) * 8 + (b & 7);
  const int seg = (b % per_group) >> 3;
  if (row >= num_tokens) return;
  split_segment<NP, SEG_VPT>(parts, np_rt, y_out, residual, weight, ws + (row - full), eps, row,
                             seg * SEG_VPT * (nt >> 6), vec_per_row, hidden, segs, nt, &arrivals_before);
}

// ---------------------------------------------------------------------------
// Element-wise kernel: any hidden size, any alignment, bf16 / fp16 / fp32.
// Two passes over the row; the second re-reads the rounded residual (or the
// input when there is none), like the reference's generic kernel
// (csrc/layernorm_kernels.cu:122-158).
// ---------------------------------------------------------------------------
template <typename T> struct Elem;
template <> struct Elem<__bf16> {
  static __device__ __forceinline__ float load(const __bf16* p) {
    return __uint_as_float((uint32_t)(*reinterpret_cast<const uint16_t*>(p)) << 16);
  }
  static __device__ __forceinline__ __bf16 round(float f) { return (__bf16)f; }
};
template <> struct Elem<_Float16> {
  static __device__ __forceinline__ float load(const _Float16* p) { return (float)*p; }
  static __device__ __forceinline__ _Float16 round(float f) { return (_Float16)f; }
};
template <> struct Elem<float> {
  static __device__ __forceinline__ float load(const float* p) { return *p; }
  static __device__ __forceinline__ float round(float f) { return f; }
};

template <typename T, bool HAS_RES, bool COPY, bool FP8>
__global__ __launch_bounds__(1024) void row_norm_elem_kernel(
    PartialPtrs parts, int np, void* y_out, T* residual, T* copy_out,
    const T* __restrict__ weight, const float* __restrict__ quant_scale, float eps,
    int num_tokens, int hidden_size) {
  __shared__ float slots[2][16];
  const int tid = threadIdx.x;
  const int nt = blockDim.x;
  const int nwaves = nt >> 6;
  float scale_inv = 1.0f;
  if (FP8) scale_inv = 1.0f / *quant_scale;
  int phase = 0;
  for (int row = blockIdx.x; row < num_tokens; row += gridDim.x, phase ^= 1) {
    const size_t base = (size_t)row * hidden_size;
    float ss = 0.0f;
    for (int j = tid; j < hidden_size; j += nt) {
      float s = Elem<T>::load(static_cast<const T*>(parts.p[0]) + base + j);
      for (int p = 1; p < np; ++p)
        s += Elem<T>::load(static_cast<const T*>(parts.p[p]) + base + j);
      if (HAS_RES) {
        s += Elem<T>::load(residual + base + j);
        residual[base + j] = Elem<T>::round(s);
      }
      ss += s * s;
    }
    const float total = block_sum(ss, slots[phase], nwaves);
    const float inv = inv_rms(total, (float)hidden_size, eps);
    const T* src = HAS_RES ? residual : static_cast<const T*>(parts.p[0]);
    for (int j = tid; j < hidden_size; j += nt) {
      const T raw = src[base + j];
      const float r = Elem<T>::load(&raw);
      if (COPY) copy_out[base + j] = raw;
      const T y = Elem<T>::round(r * inv * Elem<T>::load(weight + j));
      if (FP8) {
        const float q = fmaxf(-kFp8Max, fminf(Elem<T>::load(&y) * scale_inv, kFp8Max));
        static_cast<uint8_t*>(y_out)[base + j] =
            (uint8_t)(__builtin_amdgcn_cvt_pk_fp8_f32(q, q, 0, false) & 0xff);
      } else {
        static_cast<T*>(y_out)[base + j] = y;
      }
    }
  }
}

// Element-wise kernel with dynamic per-token quantisation: three passes over the
// row, like the reference's scalar path (layernorm_utils.cuh:19-124) — sum of
// squares, row maximum of the normalised value, quantise (+ residual write-back).
// The sum is recomputed from the inputs in every pass: the residual is overwritten
// only in the last one, by the lane that read it.
template <typename T, bool HAS_RES, bool INT8>
__global__ __launch_bounds__(1024) void row_norm_dyn_elem_kernel(
    PartialPtrs parts, int np, uint8_t* out, float* __restrict__ row_scales, T* residual,
    const T* __restrict__ weight, const float* __restrict__ scale_ub, float eps, int num_tokens,
    int hidden_size) {
  __shared__ float slots[2][16];
  __shared__ float max_slots[2][16];
  const int tid = threadIdx.x;
  const int nt = blockDim.x;
  const int nwaves = nt >> 6;
  int phase = 0;
  for (int row = blockIdx.x; row < num_tokens; row += gridDim.x, phase ^= 1) {
    const size_t base = (size_t)row * hidden_size;
    auto sum_at = [&](int j) {
      float s = Elem<T>::load(static_cast<const T*>(parts.p[0]) + base + j);
      for (int p = 1; p < np; ++p) s += Elem<T>::load(static_cast<const T*>(parts.p[p]) + base + j);
      if (HAS_RES) s += Elem<T>::load(residual + base + j);
      return s;
    };
    auto normed = [&](float s, float inv, int j) {
      const T t = Elem<T>::round(s * inv);
      const T n = Elem<T>::round(Elem<T>::load(&t) * Elem<T>::load(weight + j));
      return Elem<T>::load(&n);
    };
    float ss = 0.0f;
    for (int j = tid; j < hidden_size; j += nt) {
      const float s = sum_at(j);
      ss += s * s;
    }
    const float inv = inv_rms(block_sum(ss, slots[phase], nwaves), (float)hidden_size, eps);
    float amax = 0.0f;
    for (int j = tid; j < hidden_size; j += nt) amax = fmaxf(amax, fabsf(normed(sum_at(j), inv, j)));
    amax = block_max(amax, max_slots[phase], nwaves);
    const float scale = dyn_scale(amax, scale_ub, INT8);
    if (tid == 0) row_scales[row] = scale;
    const float sinv = 1.0f / scale;
    for (int j = tid; j < hidden_size; j += nt) {
      const float s = sum_at(j);
      if (HAS_RES) residual[base + j] = Elem<T>::round(s);
      const float n = normed(s, inv, j);
      if (INT8) {
        out[base + j] = (uint8_t)quant1_int8(n, sinv);
      } else {
        const float q = fmaxf(-kFp8Max, fminf(n / scale, kFp8Max));
        out[base + j] = (uint8_t)(__builtin_amdgcn_cvt_pk_fp8_f32(q, q, 0, false) & 0xff);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------
static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

static int default_grid(int64_t num_tokens) {
  // One workgroup per row.  Measured against grids capped at 1x .. 8x the
  // compute-unit count, the uncapped launch is as fast or faster at every size
  // from 1 to 8192 rows: the hardware dispatcher refills a compute unit as soon as
  // a row retires, which beats a fixed row-to-workgroup assignment.
  return (int)(num_tokens < INT32_MAX ? num_tokens : INT32_MAX);
}

// Workgroup shape for rows of V 16-byte vectors and T rows.  Results do not
// depend on the shape (row_sum_chunks), so it is chosen for speed alone, from
// sweeps at hidden size 8192 / 6144 with cold operands:
//   * T < 48: as many lanes per row as the row has vectors (up to 1024), one
//     vector each — the shortest path from launch to the last store when the
//     call is latency bound;
//   * 48 <= T < 224: two vectors per lane (512 lanes at hidden size 8192), 3-5 %
//     ahead of both neighbours while there are fewer rows than compute units;
//   * T >= 224: four vectors per lane in workgroups of at most 256 lanes, every
//     load of the row in flight at once (fastest from 256 to 8192 rows); the P = 1
//     ops, half of whose traffic is stores, run 0.3 - 2.5 % faster with two vectors
//     per lane from 1024 rows on (512 lanes at hidden size 8192); rows between 512
//     and 1024 vectors, whose quarter does not fill a 256-lane workgroup, do so from
//     8192 rows on (hidden size 6144: 2.5 - 2.9 % faster at 8192 and 16384 rows, 5 %
//     slower at 1024 and 2048; hidden size 8192 is 2 - 6 % slower that way at any size);
//   * rows longer than 1024 vectors: two vectors per lane up to 2048 vectors, four
//     up to 4096 (one partial at a time).  Longer rows take the element-wise kernel.
struct VecShape { int vpt, nt, maxnt; };

static bool vec_shape(int V, int64_t T, int np, VecShape* sh) {
  int vpt, maxnt = 1024;
  if (V <= 1024) {
    if (T < 48 || V < 128) vpt = 1;
    else if (T < 224 || V < 256) vpt = 2;
    else if (np == 1 && T >= 1024 && V >= 512) vpt = 2;
    else if (T >= 8192 && V > 512 && V < 1024) vpt = 2;
    else { vpt = 4; maxnt = 256; }
  } else if (V <= 2048) vpt = 2;
  else if (V <= 4096) vpt = 4;
  else return false;
  int lanes = (V + vpt - 1) / vpt;
  sh->vpt = vpt;
  sh->nt = ((lanes + 63) / 64) * 64;
  sh->maxnt = maxnt;
  return true;
}

struct RowNormArgs {
  PartialPtrs parts;
  int np;
  void* y;
  void* residual;
  void* copy_out;
  const void* weight;
  bool f16;                  // tensors are fp16 (vector kernel, P = 1 only); bf16 otherwise
  int q;                     // output kind (kQNone ..)
  const float* quant_scale;  // static fp8: the scale; dynamic fp8: optional upper bound (may be null)
  float* row_scales;         // dynamic kinds: one scale per row (output)
  SplitRow* split_ws;        // workspace of the split-row kernel, or null
  int64_t T, H;
  float eps;
  int grid;
  hipStream_t stream;
};

template <int NP, bool HAS_RES, bool COPY, int Q>
static int launch_vec(const RowNormArgs& a) {
  const int V = (int)(a.H / 8);
  VecShape sh;
  // The shape follows the number of rows in flight: under a grid cap that is the grid.
  if (!vec_shape(V, a.grid < a.T ? a.grid : a.T, a.np, &sh)) return 1;  // caller falls back to the element-wise kernel
  dim3 g(a.grid), b(sh.nt);
  if (a.f16) {
    if (NP != 1) return 1;
#define TW_LAUNCH_F16(VPT, MAXNT)                                                                \
  launch_kernel(row_norm_f16_kernel<VPT, MAXNT, HAS_RES, COPY, Q>, g, b, 0, a.stream,            \
                     a.parts, a.y, a.residual, a.copy_out, a.weight, a.quant_scale,              \
                     a.row_scales, a.eps, (int)a.T, V, (float)a.H, sh.nt, a.grid)
    if (sh.vpt == 1) TW_LAUNCH_F16(1, 1024);
    else if (sh.vpt == 2) TW_LAUNCH_F16(2, 1024);
    else if (sh.maxnt == 256) TW_LAUNCH_F16(4, 256);
    else TW_LAUNCH_F16(4, 1024);
#undef TW_LAUNCH_F16
    return 0;
  }
#define TW_LAUNCH(VPT, MAXNT)                                                                    \
  launch_kernel(row_norm_bf16_kernel<NP, VPT, MAXNT, HAS_RES, COPY, Q>, g, b, 0,                 \
                     a.stream, a.parts, a.np, a.y, a.residual, a.copy_out, a.weight,             \
                     a.quant_scale, a.row_scales, a.eps, (int)a.T, V, (float)a.H, sh.nt, a.grid)
  if (sh.vpt == 1) TW_LAUNCH(1, 1024);
  else if (sh.vpt == 2) TW_LAUNCH(2, 1024);
  else if (sh.maxnt == 256) TW_LAUNCH(4, 256);
  else TW_LAUNCH(4, 1024);
#undef TW_LAUNCH
  return 0;
}

// The split-row kernel exists for the fused op proper: bf16 vector rows, residual
// add, bf16 output.
static bool splittable(bool vec_ok, int dtype, const void* residual, const void* copy_out, int quant) {
  return vec_ok && dtype == TW_DTYPE_BF16 && residual && !copy_out && quant == kQNone;
}

// Segments per row and workgroup shape of the split-row kernel, or false when the
// one-workgroup-per-row kernel is the better (or only) choice.  A segment is
// nwaves whole chunks, one per wave.
struct SplitPlan { int nwaves, segs; };

static bool split_plan(int V, int64_t T, int cus, SplitPlan* sp) {
  const int nchunks = (V + 63) / 64;
  if (T < 1 || T > TW_SPLIT_MAX_TOKENS || nchunks < 2 || nchunks > kMaxChunks || cus <= 0) return false;
  // Measured with cold operands at hidden sizes 4096 .. 16384 and 1 .. 128 rows, over
  // segments of 1 .. 16 chunks with 1, 2 or 4 vectors per lane: segments of four chunks
  // with one vector per lane (256 lanes) are the fastest split; they beat one workgroup
  // per row by 0.3 - 0.8 us at hidden size 8192 and by 2 - 3 us at 16384 up to 48 rows,
  // draw level at 64 rows, and lose at 128 rows and for rows shorter than 16 chunks (the
  // hand-over costs more than the shorter load phase saves).  Eight-chunk segments take
  // over when four-chunk ones would make more workgroups than there are compute units.
  if (T > 48 || nchunks < 16) return false;
  sp->nwaves = T * ((nchunks + 3) / 4) <= cus ? 4 : 8;
  sp->segs = (nchunks + sp->nwaves - 1) / sp->nwaves;
  return sp->segs >= 2;
}

template <int NP>
static void launch_split(const RowNormArgs& a, const SplitPlan& sp) {
  const int V = (int)(a.H / 8);
  const int groups = (int)((a.T + 7) / 8);
  dim3 g((unsigned)(groups * 8 * sp.segs)), b((unsigned)(sp.nwaves * 64));
  launch_kernel(row_norm_split_kernel<NP, true>, g, b, 0, a.stream, a.parts, a.np, a.y, a.residual, a.weight,
                a.split_ws, a.eps, (int)a.T, V, (float)a.H, sp.segs, sp.nwaves * 64);
}

// Mixed launch (row_norm_mixed_kernel) for cus < T <= cus + cus / 4 rows of at most 1024
// vectors: `full` = cus rows with a workgroup each, the T - cus excess rows in quarters (halves
// for rows too short to quarter), so that no compute unit gets more than one segment beside
// its row.  Measured at hidden size 8192, eight partials, cold operands, 256 compute units:
// 257 / 288 / 320 rows 11.0 / 11.8 / 12.1 us against 12.3 / 13.3 / 13.0 us with one workgroup
// per row.  Beyond cus / 4 excess rows it stops paying: quarters then queue two deep on a unit
// (321 rows 12.5 against 13.0 us, 352 rows 13.5 against 13.1, 376 rows 14.3 against 13.4), and
// halves — one per unit up to cus / 2 excess rows — lose from the start (376 rows 14.0 against
// 13.4 us): the workgroup that arrives last re-reads and normalises the whole row, which puts
// nearly a second row's traffic back on its unit.  The workgroup shape is the row kernel's for
// these sizes: four vectors per lane.
struct MixedPlan { int full, segs, nt; };

static bool mixed_plan(int V, int64_t T, int np, int cus, MixedPlan* mp) {
  if (cus < 8 || cus % 8 != 0 || T <= cus || T > cus + cus / 4 || T - cus > TW_SPLIT_MAX_TOKENS) return false;
  VecShape sh;
  if (!vec_shape(V, T, np, &sh) || sh.vpt != 4 || sh.maxnt != 256) return false;
  const int nwaves = sh.nt / 64;
  const int nchunks = (V + 63) / 64;
  if (nchunks < 2 * nwaves) return false;  // a half row must be whole chunks of its own
  mp->full = cus;
  mp->segs = nchunks > 3 * nwaves ? 4 : 2;
  mp->nt = sh.nt;
  return true;
}

template <int NP>
static void launch_mixed(const RowNormArgs& a, const MixedPlan& mp) {
  const int V = (int)(a.H / 8);
  const int excess = (int)a.T - mp.full;
  const int groups = (excess + 7) / 8;
  dim3 g((unsigned)(mp.full + groups * 8 * mp.segs)), b((unsigned)mp.nt);
#define TW_LAUNCH_MIXED(SEG_VPT)                                                                             \
  launch_kernel(row_norm_mixed_kernel<NP, SEG_VPT>, g, b, 0, a.stream, a.parts, a.np, a.y, a.residual,       \
                a.weight, a.split_ws, a.eps, (int)a.T, V, (float)a.H, mp.full, mp.segs, mp.nt)
  if (mp.segs == 4) TW_LAUNCH_MIXED(1);
  else TW_LAUNCH_MIXED(2);
#undef TW_LAUNCH_MIXED
}

static void launch_mixed_np(const RowNormArgs& a, const MixedPlan& mp) {
  switch (a.np) {
    case 1: launch_mixed<1>(a, mp); break;
    case 2: launch_mixed<2>(a, mp); break;
    case 4: launch_mixed<4>(a, mp); break;
    case 8: launch_mixed<8>(a, mp); break;
    default: launch_mixed<0>(a, mp); break;
  }
}

static void launch_split_np(const RowNormArgs& a, const SplitPlan& sp) {
  switch (a.np) {
    case 1: launch_split<1>(a, sp); break;
    case 2: launch_split<2>(a, sp); break;
    case 4: launch_split<4>(a, sp); break;
    case 8: launch_split<8>(a, sp); break;
    default: launch_split<0>(a, sp); break;
  }
}

// mode: residual given -> add + write back; copy_out given -> rms_norm_inplace;
// neither -> rms_norm.  Only the P = 1 kernels exist without a residual.
template <int NP, bool HAS_RES>
static int launch_vec_q(const RowNormArgs& a) {
  switch (a.q) {
    case kQNone: return launch_vec<NP, HAS_RES, false, kQNone>(a);
    case kQStaticFp8: return launch_vec<NP, HAS_RES, false, kQStaticFp8>(a);
    case kQDynFp8: return launch_vec<NP, HAS_RES, false, kQDynFp8>(a);
    default: return launch_vec<NP, HAS_RES, false, kQDynInt8>(a);
  }
}

template <int NP>
static int launch_vec_mode(const RowNormArgs& a) {
  if (a.residual) return launch_vec_q<NP, true>(a);
  if (a.copy_out) return (NP == 1 && a.q == kQNone) ? launch_vec<1, false, true, kQNone>(a) : 1;
  // Without a residual only P = 1 and the dynamic kinds (whose P-partial form may come
  // without one) have vector kernels.
  if (NP == 1) return launch_vec_q<1, false>(a);
  if (a.q == kQDynFp8) return launch_vec<NP, false, false, kQDynFp8>(a);
  if (a.q == kQDynInt8) return launch_vec<NP, false, false, kQDynInt8>(a);
  return 1;
}

template <typename T>
static void launch_elem(const RowNormArgs& a) {
  int nt = a.H < 1024 ? (int)((a.H + 63) / 64) * 64 : 1024;
  dim3 g(a.grid), b(nt);
#define TW_LAUNCH(HAS_RES, COPY, FP8)                                                            \
  launch_kernel(row_norm_elem_kernel<T, HAS_RES, COPY, FP8>, g, b, 0, a.stream, a.parts,         \
                     a.np, a.y, static_cast<T*>(a.residual), static_cast<T*>(a.copy_out),        \
                     static_cast<const T*>(a.weight), a.quant_scale, a.eps, (int)a.T, (int)a.H)
  if (a.q == kQDynFp8 || a.q == kQDynInt8) {
#define TW_LAUNCH_DYN(HAS_RES, INT8)                                                             \
  launch_kernel(row_norm_dyn_elem_kernel<T, HAS_RES, INT8>, g, b, 0, a.stream, a.parts,          \
                     a.np, static_cast<uint8_t*>(a.y), a.row_scales, static_cast<T*>(a.residual), \
                     static_cast<const T*>(a.weight), a.quant_scale, a.eps, (int)a.T, (int)a.H)
    if (a.residual) { if (a.q == kQDynInt8) TW_LAUNCH_DYN(true, true); else TW_LAUNCH_DYN(true, false); }
    else { if (a.q == kQDynInt8) TW_LAUNCH_DYN(false, true); else TW_LAUNCH_DYN(false, false); }
#undef TW_LAUNCH_DYN
    return;
  }
  const bool fp8 = a.q == kQStaticFp8;
  if (a.residual) { if (fp8) TW_LAUNCH(true, false, true); else TW_LAUNCH(true, false, false); }
  else if (a.copy_out) TW_LAUNCH(false, true, false);
  else { if (fp8) TW_LAUNCH(false, false, true); else TW_LAUNCH(false, false, false); }
#undef TW_LAUNCH
}

// Shared by every entry point.  residual == nullptr: no residual add;
// copy_out != nullptr: rms_norm_inplace; quant: 0 = y in the input's type, 1 = fp8
// with the static scale *quant_scale, 2 / 3 = dynamic per-token fp8 / int8 (row scales
// to row_scales, quant_scale = optional upper bound).
// require_vec: refuse instead of falling back to the element-wise kernel (the
// *_cta contract).
static int run_row_norm_any(const char* what, const void* const* partials, int np, void* y,
                            void* residual, void* copy_out, const void* weight, int quant,
                            const float* quant_scale, float* row_scales, int64_t T, int64_t H, float eps,
                            int dtype, int max_ctas, bool require_vec, void* split_workspace,
                            void* stream_v) {
  if (np < 1 || np > TW_MAX_PARTIALS)
    return set_error(TW_ERR_INVALID_ARGUMENT, "%s: number of partials %d not in [1, %d]", what, np,
                     TW_MAX_PARTIALS);
  if (T < 0 || H <= 0 || T > INT32_MAX || H > INT32_MAX)
    return set_error(TW_ERR_INVALID_ARGUMENT, "%s: bad shape num_tokens=%lld hidden_size=%lld", what,
                     (long long)T, (long long)H);
  if (dtype != TW_DTYPE_BF16 && dtype != TW_DTYPE_F16 && dtype != TW_DTYPE_F32)
    return set_error(TW_ERR_DTYPE, "%s: unknown dtype code %d", what, dtype);
  if (T == 0) return TW_OK;
  if (!y || !weight || !partials)
    return set_error(TW_ERR_INVALID_ARGUMENT, "%s: null pointer argument", what);
  if (quant < kQNone || quant > kQDynInt8)
    return set_error(TW_ERR_INVALID_ARGUMENT, "%s: unknown output kind %d", what, quant);
  if (quant != kQNone && copy_out)
    return set_error(TW_ERR_INVALID_ARGUMENT, "%s: quantised output is not defined for the in-place op", what);
  if ((quant == kQStaticFp8 && !quant_scale) || (quant >= kQDynFp8 && !row_scales))
    return set_error(TW_ERR_INVALID_ARGUMENT, "%s: scale pointer is null", what);
  if (quant == kQDynInt8 && quant_scale)
    return set_error(TW_ERR_INVALID_ARGUMENT, "%s: an upper bound of the scale is defined for fp8 output only",
                     what);
  RowNormArgs a = {};
  bool aligned = aligned16(y) && aligned16(weight) && (!residual || aligned16(residual)) &&
                 (!copy_out || aligned16(copy_out));
  for (int p = 0; p < np; ++p) {
    if (!partials[p])
      return set_error(TW_ERR_INVALID_ARGUMENT, "%s: partial %d is a null pointer", what, p);
    a.parts.p[p] = partials[p];
    aligned = aligned && aligned16(partials[p]);
  }
  // fp8 rows are H bytes: H % 16 keeps every row of the output 16-byte aligned too
  const bool vec_ok = aligned && (H % 8 == 0) && (quant == kQNone || H % 16 == 0);
  if (require_vec && (!vec_ok || dtype != TW_DTYPE_BF16)) {
    if (dtype != TW_DTYPE_BF16)
      return set_error(TW_ERR_DTYPE, "%s: only bf16 is supported", what);
    // Message of the reference's launcher (csrc/tokenweave_fused_kernels.cu:259).
    return set_error(TW_ERR_ALIGNMENT,
                     "Input, residual, and weight tensors must be 16-byte aligned and "
                     "hidden_size must be divisible by 8 for optimized kernel.");
  }
  int grid = max_ctas > 0 ? max_ctas : default_grid(T);
  if (grid > T) grid = (int)T;
  a.np = np;
  a.y = y;
  a.residual = residual;
  a.copy_out = copy_out;
  a.weight = weight;
  a.f16 = dtype == TW_DTYPE_F16;
  a.q = quant;
  a.quant_scale = quant_scale;
  a.row_scales = row_scales;
  a.T = T;
  a.H = H;
  a.eps = eps;
  a.grid = grid;
  a.stream = static_cast<hipStream_t>(stream_v);

  // Few rows and a workspace: several workgroups per row.  A grid cap is a compute-unit
  // budget and is honoured by not splitting.
  if (split_workspace && max_ctas <= 0 && splittable(vec_ok, dtype, residual, copy_out, quant)) {
    SplitPlan sp;
    MixedPlan mp;
    if (split_plan((int)(H / 8), T, device_compute_units(), &sp)) {
      a.split_ws = static_cast<SplitRow*>(split_workspace);
      launch_split_np(a, sp);
      return finish_launch(what);
    }
    if (mixed_plan((int)(H / 8), T, np, device_compute_units(), &mp)) {
      a.split_ws = static_cast<SplitRow*>(split_workspace);
      launch_mixed_np(a, mp);
      return finish_launch(what);
    }
  }

  if (vec_ok && (dtype == TW_DTYPE_BF16 || (dtype == TW_DTYPE_F16 && np == 1))) {
    int fell = 1;
    switch (np) {
      case 1: fell = launch_vec_mode<1>(a); break;
      case 2: fell = launch_vec_mode<2>(a); break;
      case 4: fell = launch_vec_mode<4>(a); break;
      case 8: fell = launch_vec_mode<8>(a); break;
      default: fell = launch_vec_mode<0>(a); break;
    }
    if (fell == 0) return finish_launch(what);
    // rows longer than 4 vectors per lane (or a mode without a vector kernel):
    // the element-wise kernel below
  }
  switch (dtype) {
    case TW_DTYPE_BF16: launch_elem<__bf16>(a); break;
    case TW_DTYPE_F16: launch_elem<_Float16>(a); break;
    default: launch_elem<float>(a); break;
  }
  return finish_launch(what);
}

int run_row_norm_q(const char* what, const void* const* partials, int np, void* y,
                   void* residual, void* copy_out, const void* weight, int quant,
                   const float* quant_scale, float* row_scales, int64_t T, int64_t H, float eps,
                   int dtype, int max_ctas, bool require_vec, void* stream) {
  return run_row_norm_any(what, partials, np, y, residual, copy_out, weight, quant, quant_scale, row_scales,
                          T, H, eps, dtype, max_ctas, require_vec, nullptr, stream);
}

int run_row_norm_ws(const char* what, const void* const* partials, int np, void* y, void* residual,
                    const void* weight, int64_t T, int64_t H, float eps, int max_ctas,
                    void* workspace, void* stream) {
  if (workspace && (reinterpret_cast<uintptr_t>(workspace) & 255u))
    return set_error(TW_ERR_ALIGNMENT, "%s: the workspace must be 256-byte aligned", what);
  return run_row_norm_any(what, partials, np, y, residual, nullptr, weight, kQNone, nullptr, nullptr, T, H,
                          eps, TW_DTYPE_BF16, max_ctas, true, workspace, stream);
}

// ---------------------------------------------------------------------------
// The split-row workspace as a static device array, for callers that cannot
// allocate.  Every GPU the library runs on holds its own copy at its own address
// until the process ends; the address is resolved once per device, with that
// device current, and the kernels receive it as an argument exactly as they
// receive a caller's workspace.  The array is zero when the code object is loaded
// and every call's kernel leaves the arrival counters zero again, which is all that
// must be zero at the start of a call; the chunk sums are rewritten before they are
// read.  All calls on one GPU share the array: calls that overlap in time race.
// ---------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[TW_SPLIT_WORKSPACE_BYTES];

static int static_scratch(const char* what, void** out) {
  constexpr int kMaxDevices = 64;
  static std::atomic<void*> resolved[kMaxDevices];
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
    return set_error(TW_ERR_LAUNCH, "%s: no current device", what);
  void* ptr = resolved[dev].load(std::memory_order_acquire);
  if (!ptr) {
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr)
      return set_error(TW_ERR_LAUNCH, "%s: could not resolve the static workspace on device %d: %s", what, dev,
                       hipGetErrorString(e));
    resolved[dev].store(ptr, std::memory_order_release);
  }
  *out = ptr;
  return TW_OK;
}

int run_row_norm_noalloc(const char* what, const void* const* partials, int np, void* y, void* residual,
                         const void* weight, int64_t T, int64_t H, float eps, int max_ctas, void* stream) {
  if (T > TW_SPLIT_MAX_TOKENS)
    return set_error(TW_ERR_INVALID_ARGUMENT,
                     "%s: num_tokens %lld exceeds the %d rows the static workspace holds "
                     "(larger batches need no workspace: call tw_reduce_add_rms_norm)",
                     what, (long long)T, TW_SPLIT_MAX_TOKENS);
  void* ws = nullptr;
  if (int rc = static_scratch(what, &ws)) return rc;
  return run_row_norm_any(what, partials, np, y, residual, nullptr, weight, kQNone, nullptr, nullptr, T, H,
                          eps, TW_DTYPE_BF16, max_ctas, true, ws, stream);
}

int split_segments(int64_t T, int64_t H, int max_ctas) {
  SplitPlan sp;
  MixedPlan mp;
  if (max_ctas > 0 || H <= 0 || H % 8 != 0 || H / 8 > INT32_MAX) return 1;
  if (split_plan((int)(H / 8), T, device_compute_units(), &sp)) return sp.segs;
  // (the mixed plan's shape does not depend on the number of partials for these row counts)
  return mixed_plan((int)(H / 8), T, 8, device_compute_units(), &mp) ? mp.segs : 1;
}

int run_row_norm(const char* what, const void* const* partials, int np, void* y,
                 void* residual, void* copy_out, const void* weight, const float* quant_scale,
                 int64_t T, int64_t H, float eps, int dtype, int max_ctas, bool require_vec,
                 void* stream) {
  return run_row_norm_q(what, partials, np, y, residual, copy_out, weight,
                        quant_scale ? kQStaticFp8 : kQNone, quant_scale, nullptr, T, H, eps, dtype,
                        max_ctas, require_vec, stream);
}

}  // namespace tw
