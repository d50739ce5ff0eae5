// bf16 "NT" GEMM on gfx950 MFMA:  out[M, N] = a[M, K] * b[N, K]^T, fp32
// accumulate, bf16 out.  This is the row-parallel o_proj / down_proj that
// produces one rank's partial sum in the token-weave schedule; the reference
// runs it as torch.matmul(x, W.t(), out=) (vllm/model_executor/layers/
// linear.py:203-228).
//
// Both operands are K-contiguous, so the 8 consecutive k a lane feeds to
// v_mfma_f32_32x32x16_bf16 are one 16-byte chunk of a row of `a` or `b`.  The
// MFMA is issued with `b` rows as its first operand, which leaves every lane
// with 4 consecutive n per accumulator quad: 8-byte row-major stores.
//
// Two kernels:
//  * gemm_bf16_nt_big_kernel (K % 64 == 0): 256 x 256 x 64 tiles, 8 waves
//    (2 x 4, two per SIMD), each wave 128 x 64 (128 fp32 accumulators).  Operand
//    slabs go from global memory straight into LDS (buffer_load ... lds: no
//    staging registers, no LDS store instructions), two LDS stages of 64 KiB.
//    A wave instruction fills 1 KiB = 8 LDS rows of 128 bytes; row r keeps its
//    16-byte chunk c at position c ^ ((r >> 1) & 7), which makes the 16-byte
//    fragment reads of 16 consecutive rows conflict-free on the 64-bank LDS
//    (counter-verified) without padding.  The descriptor's extent is the
//    operand's size, so tile rows past M or N read as zeros.  Fragments are
//    double-buffered in registers; the next k-step's LDS reads are issued
//    between the two halves of the current step's MFMAs.
//  * gemm_bf16_nt_kernel (any K % 8 == 0): 128 x 128 x 64 tiles, 4 waves,
//    register-staged loads into padded LDS; the general fallback.
// Workgroups walk the tile list with stride gridDim.x (grid cap = compute-unit
// budget of the weave schedule), and tile ids are remapped so that the
// workgroups of one XCD (blockIdx % 8) share operand panels in that XCD's L2.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "tw_common.h"

namespace tw {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));

constexpr int BM = 128, BN = 128, BK = 64;
constexpr int LDS_ROW = BK + 8;  // elements; 144-byte row pitch
constexpr int GEMM_THREADS = 256;
constexpr int CHUNKS_PER_ROW = BK / 8;                           // 16-byte chunks per tile row
constexpr int LOADS_PER_THREAD = BM * CHUNKS_PER_ROW / GEMM_THREADS;  // 4
constexpr int GROUP_M = 8;  // tile rows per column sweep (operand reuse in L2)

__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

__global__ __launch_bounds__(GEMM_THREADS) void gemm_bf16_nt_kernel(
    uint16_t* __restrict__ out, const uint16_t* __restrict__ a, const uint16_t* __restrict__ b,
    int M, int N, int K, int64_t ldc, int tiles_m, int tiles_n) {
  __shared__ __attribute__((aligned(16))) uint16_t lds_a[2][BM * LDS_ROW];
  __shared__ __attribute__((aligned(16))) uint16_t lds_b[2][BN * LDS_ROW];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int l32 = lane & 31, lhi = lane >> 5;
  const int num_tiles = tiles_m * tiles_n;
  const int nk = (K + BK - 1) / BK;

  for (int t = blockIdx.x; t < num_tiles; t += gridDim.x) {
    // XCD-aware remap: ids congruent mod 8 run on one XCD; give each XCD a
    // contiguous range of the grouped tile order.
    int pid = t;
    {
      const int per_xcd = num_tiles / 8;
      const int body = per_xcd * 8;
      if (t < body) pid = (t & 7) * per_xcd + (t >> 3);
    }
    const int group_size = GROUP_M * tiles_n;
    const int group = pid / group_size;
    const int first_m = group * GROUP_M;
    const int rows_in_group = min(tiles_m - first_m, GROUP_M);
    const int tm_idx = first_m + (pid % group_size) % rows_in_group;
    const int tn_idx = (pid % group_size) / rows_in_group;
    const int m0 = tm_idx * BM, n0 = tn_idx * BN;

    f32x16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    uint4 ra[LOADS_PER_THREAD], rb[LOADS_PER_THREAD];
    auto fetch = [&](int kt) {
#pragma unroll
      for (int i = 0; i < LOADS_PER_THREAD; ++i) {
        const int c = tid + i * GEMM_THREADS;
        const int row = c / CHUNKS_PER_ROW, kc = c % CHUNKS_PER_ROW;
        const int k = kt * BK + kc * 8;
        const int am = min(m0 + row, M - 1);  // rows past M are computed, never stored
        const int bn = min(n0 + row, N - 1);
        if (k < K) {
          ra[i] = *reinterpret_cast<const uint4*>(a + (size_t)am * K + k);
          rb[i] = *reinterpret_cast<const uint4*>(b + (size_t)bn * K + k);
        } else {
          ra[i] = make_uint4(0, 0, 0, 0);
          rb[i] = make_uint4(0, 0, 0, 0);
        }
      }
    };
    auto stash = [&](int buf) {
#pragma unroll
      for (int i = 0; i < LOADS_PER_THREAD; ++i) {
        const int c = tid + i * GEMM_THREADS;
        const int row = c / CHUNKS_PER_ROW, kc = c % CHUNKS_PER_ROW;
        *reinterpret_cast<uint4*>(&lds_a[buf][row * LDS_ROW + kc * 8]) = ra[i];
        *reinterpret_cast<uint4*>(&lds_b[buf][row * LDS_ROW + kc * 8]) = rb[i];
      }
    };

    fetch(0);
    __syncthreads();  // previous tile's readers are done with both buffers
    stash(0);
    __syncthreads();

    for (int kt = 0; kt < nk; ++kt) {
      const int buf = kt & 1;
      if (kt + 1 < nk) fetch(kt + 1);
#pragma unroll
      for (int kk = 0; kk < BK / 16; ++kk) {
        bf16x8_t fa[2], fb[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          const int ar = wm * 64 + i * 32 + l32;
          const int br = wn * 64 + i * 32 + l32;
          fa[i] = __builtin_bit_cast(
              bf16x8_t, *reinterpret_cast<const uint4*>(&lds_a[buf][ar * LDS_ROW + kk * 16 + lhi * 8]));
          fb[i] = __builtin_bit_cast(
              bf16x8_t, *reinterpret_cast<const uint4*>(&lds_b[buf][br * LDS_ROW + kk * 16 + lhi * 8]));
        }
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[j], fa[i], acc[i][j], 0, 0, 0);
      }
      if (kt + 1 < nk) stash(buf ^ 1);
      __syncthreads();
    }

    // acc[i][j][4*q + e] = out[m0 + wm*64 + i*32 + l32][n0 + wn*64 + j*32 + 8*q + 4*lhi + e]
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int m = m0 + wm * 64 + i * 32 + l32;
      if (m >= M) continue;
#pragma unroll
      for (int j = 0; j < 2; ++j) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n = n0 + wn * 64 + j * 32 + 8 * q + 4 * lhi;
          if (n < N) {
            uint2 v;
            v.x = pack2(acc[i][j][4 * q + 0], acc[i][j][4 * q + 1]);
            v.y = pack2(acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]);
            *reinterpret_cast<uint2*>(out + (size_t)m * ldc + n) = v;
          }
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------
// 256 x 256 x 64 tiles, direct-to-LDS operand slabs (see the file comment).
// ---------------------------------------------------------------------------
typedef __attribute__((address_space(3))) void lds_void_t;
constexpr int BIG_BM = 256, BIG_BN = 256, BIG_BK = 64;
constexpr int BIG_THREADS = 512;
constexpr int BIG_ROWB = BIG_BK * 2;             // bytes per LDS row
constexpr int BIG_PANEL = BIG_BM * BIG_ROWB;     // 32 KiB: one operand, one stage
constexpr int BIG_STAGE = 2 * BIG_PANEL;         // a-panel then b-panel
constexpr int BIG_LDS_BYTES = 2 * BIG_STAGE;     // two stages
constexpr int BIG_GROUP_M = 4;

__global__ __launch_bounds__(BIG_THREADS) void gemm_bf16_nt_big_kernel(
    uint16_t* __restrict__ out, const uint16_t* __restrict__ a, const uint16_t* __restrict__ b,
    int M, int N, int K, int64_t ldc, int tiles_m, int tiles_n) {
  constexpr int TM = 4, TN = 2;  // 32 x 32 MFMA tiles per wave: 128 x 64
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds_big[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 2, wn = wave & 3, l32 = lane & 31, lhi = lane >> 5;
  const int num_tiles = tiles_m * tiles_n;
  const int nk = K / BIG_BK;
  // Loader: wave instruction j of wave w fills LDS rows [(4w + j) * 8, +8); lane l
  // lands at row l / 8, position l % 8, so it must fetch chunk (l % 8) ^ key(row).
  const int ld_row = lane >> 3;
  const int ld_key = lane >> 4;                     // key of rows in an even 8-row block
  const int ld_chunk_even = (lane & 7) ^ ld_key;
  const int ld_chunk_odd = (lane & 7) ^ (ld_key | 4);  // odd block: rows 8..15 of a 16-row group
  // Reader: lane row l32 (+ 32 i), chunk 2 kk + lhi.
  uint32_t roff[4];
#pragma unroll
  for (int kk = 0; kk < 4; ++kk)
    roff[kk] = l32 * BIG_ROWB + ((((kk << 1) | lhi) ^ ((l32 >> 1) & 7)) << 4);

  const __amdgpu_buffer_rsrc_t da = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t*>(a), 0, (uint32_t)((size_t)M * K * 2), 0x00020000);
  const __amdgpu_buffer_rsrc_t db = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t*>(b), 0, (uint32_t)((size_t)N * K * 2), 0x00020000);

  for (int t = blockIdx.x; t < num_tiles; t += gridDim.x) {
    int pid = t;
    {
      const int per_xcd = num_tiles / 8;
      const int body = per_xcd * 8;
      if (t < body) pid = (t & 7) * per_xcd + (t >> 3);
    }
    const int group_size = BIG_GROUP_M * tiles_n;
    const int group = pid / group_size;
    const int first_m = group * BIG_GROUP_M;
    const int rows_in_group = min(tiles_m - first_m, BIG_GROUP_M);
    const int tm_idx = first_m + (pid % group_size) % rows_in_group;
    const int tn_idx = (pid % group_size) / rows_in_group;
    const int m0 = tm_idx * BIG_BM, n0 = tn_idx * BIG_BN;

    uint32_t va[4], vb[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int r = (wave * 4 + j) * 8 + ld_row;
      const int chunk = (j & 1) ? ld_chunk_odd : ld_chunk_even;  // 4 * wave is even
      va[j] = (uint32_t)(((size_t)(m0 + r) * K + chunk * 8) * 2);
      vb[j] = (uint32_t)(((size_t)(n0 + r) * K + chunk * 8) * 2);
    }
    auto issue = [&](int kt, int stage) {
      uint8_t* sa = lds_big + stage * BIG_STAGE + (wave * 4) * 1024;
      uint8_t* sb = sa + BIG_PANEL;
      const uint32_t koff = (uint32_t)kt * BIG_ROWB;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        __builtin_amdgcn_raw_ptr_buffer_load_lds(da, (lds_void_t*)(sa + j * 1024), 16, va[j], koff, 0, 0);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(db, (lds_void_t*)(sb + j * 1024), 16, vb[j], koff, 0, 0);
      }
    };

    f32x16_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    __syncthreads();  // the previous tile's fragment reads are finished
    issue(0, 0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    for (int kt = 0; kt < nk; ++kt) {
      const int stage = kt & 1;
      if (kt + 1 < nk) issue(kt + 1, stage ^ 1);
      const uint8_t* pa = lds_big + stage * BIG_STAGE + (wm * 128) * BIG_ROWB;
      const uint8_t* pb = lds_big + stage * BIG_STAGE + BIG_PANEL + (wn * 64) * BIG_ROWB;
      bf16x8_t fa[2][TM], fb[2][TN];
#pragma unroll
      for (int i = 0; i < TM; ++i)
        fa[0][i] = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const uint4*>(pa + i * 32 * BIG_ROWB + roff[0]));
#pragma unroll
      for (int j = 0; j < TN; ++j)
        fb[0][j] = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const uint4*>(pb + j * 32 * BIG_ROWB + roff[0]));
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
        const int cur = kk & 1, nxt = cur ^ 1;
        // First half of this step's MFMAs, the next step's fragment reads, second
        // half: the reads complete in the shadow of the second half.  The
        // scheduling barriers keep the compiler from sinking the reads to their use.
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < TM / 2; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[cur][j], fa[cur][i], acc[i][j], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (kk < 3) {
#pragma unroll
          for (int i = 0; i < TM; ++i)
            fa[nxt][i] = __builtin_bit_cast(
                bf16x8_t, *reinterpret_cast<const uint4*>(pa + i * 32 * BIG_ROWB + roff[kk + 1]));
#pragma unroll
          for (int j = 0; j < TN; ++j)
            fb[nxt][j] = __builtin_bit_cast(
                bf16x8_t, *reinterpret_cast<const uint4*>(pb + j * 32 * BIG_ROWB + roff[kk + 1]));
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = TM / 2; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[cur][j], fa[cur][i], acc[i][j], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
      // the next slab has landed (this wave's share), and after the barrier every
      // wave's share has; nobody still reads the stage that gets overwritten next
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
    }

    // acc[i][j][4 q + e] = out[m0 + wm*128 + i*32 + l32][n0 + wn*64 + j*32 + 8 q + 4 lhi + e]
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int m = m0 + wm * 128 + i * 32 + l32;
      if (m >= M) continue;
#pragma unroll
      for (int j = 0; j < TN; ++j) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n = n0 + wn * 64 + j * 32 + 8 * q + 4 * lhi;
          if (n < N) {
            uint2 v;
            v.x = pack2(acc[i][j][4 * q + 0], acc[i][j][4 * q + 1]);
            v.y = pack2(acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]);
            *reinterpret_cast<uint2*>(out + (size_t)m * ldc + n) = v;
          }
        }
      }
    }
  }
}

int run_gemm_bf16_nt(void* out, const void* a, const void* b, int64_t M, int64_t N, int64_t K,
                     int64_t ldc, int max_cus, void* stream) {
  if (M < 0 || N <= 0 || K <= 0 || M > INT32_MAX || N > INT32_MAX || K > INT32_MAX || ldc < N)
    return set_error(TW_ERR_INVALID_ARGUMENT, "gemm_bf16_nt: bad shape M=%lld N=%lld K=%lld ldc=%lld",
                     (long long)M, (long long)N, (long long)K, (long long)ldc);
  if (M == 0) return TW_OK;
  if (!out || !a || !b) return set_error(TW_ERR_INVALID_ARGUMENT, "gemm_bf16_nt: null pointer argument");
  auto al = [](const void* p, unsigned n) { return (reinterpret_cast<uintptr_t>(p) & (n - 1)) == 0; };
  if (K % 8 != 0 || N % 4 != 0 || ldc % 4 != 0 || !al(a, 16) || !al(b, 16) || !al(out, 8))
    return set_error(TW_ERR_ALIGNMENT,
                     "gemm_bf16_nt: needs K %% 8 == 0, N %% 4 == 0, ldc %% 4 == 0, 16-byte aligned "
                     "a and b, 8-byte aligned out");
  hipStream_t hs = static_cast<hipStream_t>(stream);
  // The 256 x 256 kernel needs whole 64-wide k-slabs, 32-bit byte offsets into both
  // operands and enough tiles to be worth its larger prologue.
  const bool big = (K % BIG_BK == 0) && ((uint64_t)M * K < (1ull << 31)) && ((uint64_t)N * K < (1ull << 31)) &&
                   M >= 192 && N >= 192;
  if (big) {
    static bool lds_ok = false;  // benign race: the attribute call is idempotent
    if (!lds_ok) {
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_bf16_nt_big_kernel),
                              hipFuncAttributeMaxDynamicSharedMemorySize, BIG_LDS_BYTES) != hipSuccess)
        return set_error(TW_ERR_LAUNCH, "gemm_bf16_nt: the device refused %d bytes of LDS", BIG_LDS_BYTES);
      lds_ok = true;
    }
    const int tiles_m = (int)((M + BIG_BM - 1) / BIG_BM), tiles_n = (int)((N + BIG_BN - 1) / BIG_BN);
    int64_t grid = (int64_t)tiles_m * tiles_n;
    if (max_cus > 0 && grid > max_cus) grid = max_cus;
    hipLaunchKernelGGL(gemm_bf16_nt_big_kernel, dim3((unsigned)grid), dim3(BIG_THREADS), BIG_LDS_BYTES, hs,
                       static_cast<uint16_t*>(out), static_cast<const uint16_t*>(a),
                       static_cast<const uint16_t*>(b), (int)M, (int)N, (int)K, ldc, tiles_m, tiles_n);
  } else {
    const int tiles_m = (int)((M + BM - 1) / BM), tiles_n = (int)((N + BN - 1) / BN);
    int64_t grid = (int64_t)tiles_m * tiles_n;
    if (max_cus > 0 && grid > max_cus) grid = max_cus;
    if (grid > INT32_MAX) grid = INT32_MAX;
    hipLaunchKernelGGL(gemm_bf16_nt_kernel, dim3((unsigned)grid), dim3(GEMM_THREADS), 0, hs,
                       static_cast<uint16_t*>(out), static_cast<const uint16_t*>(a),
                       static_cast<const uint16_t*>(b), (int)M, (int)N, (int)K, ldc, tiles_m, tiles_n);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess)
    return set_error(TW_ERR_LAUNCH, "gemm_bf16_nt: kernel launch failed: %s", hipGetErrorString(e));
  return TW_OK;
}

}  // namespace tw
