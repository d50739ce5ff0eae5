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
// Workgroup: 256 lanes (4 waves, 2 x 2), tile 128 x 128 x 64, each wave 64 x 64
// (2 x 2 MFMA tiles, 64 fp32 accumulators per lane).  Tiles are double-buffered
// in LDS; the next k-slab is fetched into registers while the current one is
// multiplied.  LDS rows are padded by 16 bytes so the 16-byte fragment reads of
// 32 consecutive rows fall in distinct banks.  Workgroups walk the tile list
// with stride gridDim.x (grid cap = compute-unit budget of the weave schedule),
// and tile ids are remapped so that the workgroups of one XCD (blockIdx % 8)
// share operand panels in that XCD's L2.
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
  const int tiles_m = (int)((M + BM - 1) / BM), tiles_n = (int)((N + BN - 1) / BN);
  const int64_t tiles = (int64_t)tiles_m * tiles_n;
  int64_t grid = tiles;
  if (max_cus > 0 && grid > max_cus) grid = max_cus;
  if (grid > INT32_MAX) grid = INT32_MAX;
  hipLaunchKernelGGL(gemm_bf16_nt_kernel, dim3((unsigned)grid), dim3(GEMM_THREADS), 0,
                     static_cast<hipStream_t>(stream), static_cast<uint16_t*>(out),
                     static_cast<const uint16_t*>(a), static_cast<const uint16_t*>(b), (int)M, (int)N,
                     (int)K, ldc, tiles_m, tiles_n);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess)
    return set_error(TW_ERR_LAUNCH, "gemm_bf16_nt: kernel launch failed: %s", hipGetErrorString(e));
  return TW_OK;
}

}  // namespace tw
