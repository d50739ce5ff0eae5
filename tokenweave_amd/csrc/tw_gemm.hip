// bf16 "NT" GEMM on gfx950 MFMA:  out[M, N] = a[M, K] * b[N, K]^T, fp32
// accumulate, bf16 out.  This is the row-parallel o_proj / down_proj that
// produces one rank's partial sum in the token-weave schedule; the reference
// runs it as torch.matmul(x, W.t(), out=) (vllm/model_executor/layers/
// linear.py:203-228).
//
// Both operands are K-contiguous, so the 8 consecutive k a lane feeds to
// v_mfma_f32_32x32x16_bf16 are one 16-byte chunk of a row of `a` or `b`.  The
// MFMA is issued with `b` rows as its first operand, which leaves every lane
// with 4 consecutive n per accumulator quad: 8-byte row-major stores, or, in the
// big kernel when the output allows 16-byte stores, a transpose through LDS into
// whole 128-byte lines per row.
//
// Two kernels:
//  * gemm_bf16_nt_big_kernel<TM, TN> (K >= 64; a last partial k-slab is zero-filled): (64 TM) x (128 TN) x 64 tiles,
//    8 waves (2 x 4, two per SIMD), each wave (32 TM) x (32 TN): 128/192/256/320 x 256
//    (TN = 2) chosen per problem so that the tile count wastes the fewest workgroup
//    rounds (M = 2458: 320-row tiles make exactly 256 tiles; M = 1024: 128-row tiles
//    give every compute unit one), or 256 x 384.
//    Operand slabs go from global memory straight into LDS (buffer_load ... lds:
//    no staging registers, no LDS store instructions), two LDS stages.
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

#include <atomic>

#include "tw_common.h"

namespace tw {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

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

// The optional bias of the in-place linear is added the way the reference adds it
// (vllm/model_executor/layers/linear.py:224-228: torch.matmul(..., out=output), then
// output += bias): to the product already rounded to bf16, in fp32, rounded again.
// `packed` and `bias2` hold two bf16 each, element 2i in the low half.
__device__ __forceinline__ uint32_t add_bias2(uint32_t packed, uint32_t bias2) {
  const float lo = __uint_as_float(packed << 16) + __uint_as_float(bias2 << 16);
  const float hi = __uint_as_float(packed & 0xffff0000u) + __uint_as_float(bias2 & 0xffff0000u);
  return pack2(lo, hi);
}

__global__ __launch_bounds__(GEMM_THREADS) void gemm_bf16_nt_kernel(
    uint16_t* __restrict__ out, const uint16_t* __restrict__ a, const uint16_t* __restrict__ b,
    const uint16_t* __restrict__ bias, int M, int N, int K, int64_t ldc, int tiles_m, int tiles_n) {
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
            if (bias) {  // N % 4 == 0: the four columns lie inside the row; bias is 8-byte aligned
              const uint2 bv = *reinterpret_cast<const uint2*>(bias + n);
              v.x = add_bias2(v.x, bv.x);
              v.y = add_bias2(v.y, bv.y);
            }
            *reinterpret_cast<uint2*>(out + (size_t)m * ldc + n) = v;
          }
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------
// (32 TM x 2) x 256 x 64 tiles, direct-to-LDS operand slabs (see the file
// comment).  TM = 32-row MFMA tiles per wave along M: 4 -> 256-row tiles,
// 5 -> 320-row tiles, 3 -> 192-row tiles.  The launcher picks the height that
// wastes the fewest workgroup rounds for the given M.
// ---------------------------------------------------------------------------
typedef __attribute__((address_space(3))) void lds_void_t;
constexpr int BIG_BK = 64;
constexpr int BIG_THREADS = 512;
constexpr int BIG_ROWB = BIG_BK * 2;             // bytes per LDS row
constexpr int BIG_GROUP_M = 4;
constexpr int big_lds_bytes(int tm, int tn) { return 2 * (tm * 64 + tn * 128) * BIG_ROWB; }

// One k-slab of both operands, global memory -> LDS: this wave's LA + LB wave
// instructions of 1 KiB each.  (A free function, not a lambda: the kernel is a
// template, and the host pass must be able to instantiate its stub without
// compiling device builtins.)
template <int LA, int LB>
__device__ __forceinline__ void big_issue_slab(__amdgpu_buffer_rsrc_t da, __amdgpu_buffer_rsrc_t db,
                                               const uint32_t (&va)[LA], const uint32_t (&vb)[LB],
                                               uint8_t* sa, uint8_t* sb, uint32_t koff) {
#pragma unroll
  for (int j = 0; j < LA; ++j)
    __builtin_amdgcn_raw_ptr_buffer_load_lds(da, (lds_void_t*)(sa + j * 1024), 16, va[j], koff, 0, 0);
#pragma unroll
  for (int j = 0; j < LB; ++j)
    __builtin_amdgcn_raw_ptr_buffer_load_lds(db, (lds_void_t*)(sb + j * 1024), 16, vb[j], koff, 0, 0);
}

// The last k-slab of an inner dimension that is not a multiple of 64 (but of 8): the 16-byte
// chunks that lie past K must land in LDS as zeros.  A lane's chunk is c ^ 4 in odd 8-row
// blocks and c in even ones (the swizzle above), so two flags per lane say whether its chunk
// is inside; a chunk outside is requested at an offset past the descriptor's extent, which
// the hardware answers with zeros.
constexpr uint32_t BIG_OUT_OF_RANGE = 0x80000000u;  // operands are smaller than 2 GiB

template <int LA, int LB>
__device__ __forceinline__ void big_issue_slab_tail(__amdgpu_buffer_rsrc_t da, __amdgpu_buffer_rsrc_t db,
                                                    const uint32_t (&va)[LA], const uint32_t (&vb)[LB],
                                                    uint8_t* sa, uint8_t* sb, uint32_t koff, int blk_a, int blk_b,
                                                    bool in_even, bool in_odd) {
#pragma unroll
  for (int j = 0; j < LA; ++j) {
    const bool in = ((blk_a + j) & 1) ? in_odd : in_even;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(da, (lds_void_t*)(sa + j * 1024), 16, in ? va[j] : BIG_OUT_OF_RANGE, koff,
                                             0, 0);
  }
#pragma unroll
  for (int j = 0; j < LB; ++j) {
    const bool in = ((blk_b + j) & 1) ? in_odd : in_even;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(db, (lds_void_t*)(sb + j * 1024), 16, in ? vb[j] : BIG_OUT_OF_RANGE, koff,
                                             0, 0);
  }
}

// `count` independent products of one shape in one launch: out[p] = a[p] * b[p]^T.  The
// token-weave producer uses it for the P row-parallel partial sums of a token split,
// each written into its rank's staging slot; a plain GEMM is count = 1.
struct GemmBatch {
  uint16_t* out[TW_MAX_PARTIALS];
  const uint16_t* a[TW_MAX_PARTIALS];
  const uint16_t* b[TW_MAX_PARTIALS];
  const uint16_t* bias[TW_MAX_PARTIALS];  // [N] bf16 or null: added to that product only
};

template <int TM, int TN>
__global__ __launch_bounds__(BIG_THREADS) void gemm_bf16_nt_big_kernel(
    GemmBatch batch, int count, int M, int N, int K, int64_t ldc, int tiles_m, int tiles_n, int wide_store) {
  constexpr int WM = 32 * TM, WN = 32 * TN;  // wave tile
  constexpr int BM = 2 * WM, BN = 4 * WN;    // workgroup tile: the 8 waves as 2 x 4
  constexpr int PANEL_A = BM * BIG_ROWB;
  constexpr int STAGE = PANEL_A + BN * BIG_ROWB;  // a-panel then b-panel
  constexpr int LA = BM / 64;           // a-panel loads per wave per slab (8 rows x 8 waves each)
  constexpr int LB = BN / 64;           // b-panel loads per wave per slab
  constexpr int H1 = (TM + 1) / 2;      // MFMA rows issued before the next fragments are fetched
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds_big[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 2, wn = wave & 3, l32 = lane & 31, lhi = lane >> 5;
  const int tiles_per_product = tiles_m * tiles_n;
  const int num_tiles = count * tiles_per_product;
  const int nk = (K + BIG_BK - 1) / BIG_BK;
  const int tail_chunks = (K % BIG_BK) / 8;  // 16-byte chunks of the last slab that lie inside K (0: all eight)
  // Loader: wave instruction j of wave w fills the 8-row LDS block w * L + j; lane l
  // lands at row l / 8, position l % 8 of that block, so it must fetch the chunk
  // (l % 8) ^ key(row), key(r) = (r >> 1) & 7 = ((block & 1) << 2) | (l >> 4).
  const int ld_row = lane >> 3;
  const int ld_key = lane >> 4;
  const bool tail_in_even = ((lane & 7) ^ ld_key) < tail_chunks;
  const bool tail_in_odd = ((lane & 7) ^ ld_key ^ 4) < tail_chunks;
  // Reader: lane row l32 (+ 32 i; wave offsets are multiples of 16 rows, which do not
  // change the key), chunk 2 kk + lhi.
  uint32_t roff[4];
#pragma unroll
  for (int kk = 0; kk < 4; ++kk)
    roff[kk] = l32 * BIG_ROWB + ((((kk << 1) | lhi) ^ ((l32 >> 1) & 7)) << 4);

  for (int t = blockIdx.x; t < num_tiles; t += gridDim.x) {
    // Every XCD (workgroup ids congruent mod 8) gets a contiguous range of the tile order:
    // with eight products, one product each.
    int pid = t;
    {
      const int per_xcd = num_tiles / 8;
      const int body = per_xcd * 8;
      if (t < body) pid = (t & 7) * per_xcd + (t >> 3);
    }
    const int product = pid / tiles_per_product;
    pid -= product * tiles_per_product;
    uint16_t* __restrict__ out = batch.out[product];
    const uint16_t* __restrict__ bias = batch.bias[product];
    const __amdgpu_buffer_rsrc_t da = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t*>(batch.a[product]), 0, (uint32_t)((size_t)M * K * 2), 0x00020000);
    const __amdgpu_buffer_rsrc_t db = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t*>(batch.b[product]), 0, (uint32_t)((size_t)N * K * 2), 0x00020000);
    const int group_size = BIG_GROUP_M * tiles_n;
    const int group = pid / group_size;
    const int first_m = group * BIG_GROUP_M;
    const int rows_in_group = min(tiles_m - first_m, BIG_GROUP_M);
    const int tm_idx = first_m + (pid % group_size) % rows_in_group;
    const int tn_idx = (pid % group_size) / rows_in_group;
    const int m0 = tm_idx * BM, n0 = tn_idx * BN;

    uint32_t va[LA], vb[LB];
#pragma unroll
    for (int j = 0; j < LA; ++j) {
      const int blk = wave * LA + j;
      const int chunk = (lane & 7) ^ (((blk & 1) << 2) | ld_key);
      va[j] = (uint32_t)(((size_t)(m0 + blk * 8 + ld_row) * K + chunk * 8) * 2);
    }
#pragma unroll
    for (int j = 0; j < LB; ++j) {
      const int blk = wave * LB + j;
      const int chunk = (lane & 7) ^ (((blk & 1) << 2) | ld_key);
      vb[j] = (uint32_t)(((size_t)(n0 + blk * 8 + ld_row) * K + chunk * 8) * 2);
    }
    f32x16_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    __syncthreads();  // the previous tile's fragment reads are finished
    big_issue_slab<LA, LB>(da, db, va, vb, lds_big + (wave * LA) * 1024,
                           lds_big + PANEL_A + (wave * LB) * 1024, 0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    for (int kt = 0; kt < nk; ++kt) {
      const int stage = kt & 1;
      if (kt + 2 < nk || (kt + 2 == nk && tail_chunks == 0))
        big_issue_slab<LA, LB>(da, db, va, vb, lds_big + (stage ^ 1) * STAGE + (wave * LA) * 1024,
                               lds_big + (stage ^ 1) * STAGE + PANEL_A + (wave * LB) * 1024,
                               (uint32_t)(kt + 1) * BIG_ROWB);
      else if (kt + 2 == nk)
        big_issue_slab_tail<LA, LB>(da, db, va, vb, lds_big + (stage ^ 1) * STAGE + (wave * LA) * 1024,
                                    lds_big + (stage ^ 1) * STAGE + PANEL_A + (wave * LB) * 1024,
                                    (uint32_t)(kt + 1) * BIG_ROWB, wave * LA, wave * LB, tail_in_even, tail_in_odd);
      const uint8_t* pa = lds_big + stage * STAGE + (wm * WM) * BIG_ROWB;
      const uint8_t* pb = lds_big + stage * STAGE + PANEL_A + (wn * WN) * BIG_ROWB;
      if constexpr (TN == 3) {
        // 192 accumulators leave no room for two copies of both fragment sets: `a`
        // fragments are single-buffered and refilled for the next step right after
        // their last use in this one (half of them in the middle of the step, half
        // at its end); only the `b` fragments are double-buffered.
        bf16x8_t fa[TM], fb[2][TN];
#pragma unroll
        for (int i = 0; i < TM; ++i)
          fa[i] = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const uint4*>(pa + i * 32 * BIG_ROWB + roff[0]));
#pragma unroll
        for (int j = 0; j < TN; ++j)
          fb[0][j] = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const uint4*>(pb + j * 32 * BIG_ROWB + roff[0]));
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
          const int cur = kk & 1, nxt = cur ^ 1;
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int i = 0; i < H1; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
              acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[cur][j], fa[i], acc[i][j], 0, 0, 0);
          __builtin_amdgcn_sched_barrier(0);
          if (kk < 3) {
#pragma unroll
            for (int i = 0; i < H1; ++i)
              fa[i] = __builtin_bit_cast(
                  bf16x8_t, *reinterpret_cast<const uint4*>(pa + i * 32 * BIG_ROWB + roff[kk + 1]));
#pragma unroll
            for (int j = 0; j < TN; ++j)
              fb[nxt][j] = __builtin_bit_cast(
                  bf16x8_t, *reinterpret_cast<const uint4*>(pb + j * 32 * BIG_ROWB + roff[kk + 1]));
          }
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int i = H1; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
              acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[cur][j], fa[i], acc[i][j], 0, 0, 0);
          __builtin_amdgcn_sched_barrier(0);
          if (kk < 3) {
#pragma unroll
            for (int i = H1; i < TM; ++i)
              fa[i] = __builtin_bit_cast(
                  bf16x8_t, *reinterpret_cast<const uint4*>(pa + i * 32 * BIG_ROWB + roff[kk + 1]));
          }
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        continue;
      }
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
        // First part of this step's MFMAs, the next step's fragment reads, the rest:
        // the reads complete in the shadow of the rest.  The scheduling barriers keep
        // the compiler from sinking the reads to their use.
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < H1; ++i)
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
        for (int i = H1; i < TM; ++i)
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

    // acc[i][j][4 q + e] = out[m0 + wm*WM + i*32 + l32][n0 + wn*WN + j*32 + 8 q + 4 lhi + e]
    if (wide_store) {
      // Through LDS, 32 rows of the wave tile at a time (a wave-private 32 x WN patch,
      // rows padded by 8 bytes): lanes write their 4-element groups, then read the patch
      // back row-contiguously, 16 bytes per lane, so that a wave store covers whole
      // 128-byte lines of 8 output rows instead of 16-byte pieces of 32 rows.  The slab
      // stages are free: every wave passed the barrier that ends the k loop.
      constexpr int PATCH_ROW = WN * 2 + 8;            // bytes
      constexpr int CHUNKS = WN / 8;                   // 16-byte chunks per patch row
      constexpr int ROWS_PER_PASS = 64 / CHUNKS;       // 8 (WN = 64) or 5 (WN = 96: 4 lanes idle)
      uint8_t* patch = lds_big + wave * (32 * PATCH_ROW);
      const int rd_row = lane / CHUNKS, rd_chunk = lane % CHUNKS;
      const bool rd_lane = rd_row < ROWS_PER_PASS;
      const int n = n0 + wn * WN + rd_chunk * 8;
      // this lane's eight columns are the same in every pass: their bias is fetched once
      uint4 bv = make_uint4(0, 0, 0, 0);
      if (bias && rd_lane && n < N) bv = *reinterpret_cast<const uint4*>(bias + n);
#pragma unroll
      for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            uint2 v;
            v.x = pack2(acc[i][j][4 * q + 0], acc[i][j][4 * q + 1]);
            v.y = pack2(acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]);
            *reinterpret_cast<uint2*>(patch + l32 * PATCH_ROW + (j * 32 + 8 * q + 4 * lhi) * 2) = v;
          }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int r = 0; r < 32; r += ROWS_PER_PASS) {
          const int row = min(r + rd_row, 31);
          const int m = m0 + wm * WM + i * 32 + row;
          // 8-byte LDS reads: the padded row pitch keeps rows 8-byte, not 16-byte, aligned
          const uint2 lo = *reinterpret_cast<const uint2*>(patch + row * PATCH_ROW + rd_chunk * 16);
          const uint2 hi = *reinterpret_cast<const uint2*>(patch + row * PATCH_ROW + rd_chunk * 16 + 8);
          // streaming stores: the tile is not read again by this kernel, and whoever reads
          // it next (the norm kernel) runs on other XCDs; 1 - 3.5 % faster than default stores
          if (rd_lane && r + rd_row < 32 && m < M && n < N) {
            u32x4_t v = {lo.x, lo.y, hi.x, hi.y};
            if (bias) v = u32x4_t{add_bias2(lo.x, bv.x), add_bias2(lo.y, bv.y), add_bias2(hi.x, bv.z),
                                  add_bias2(hi.y, bv.w)};
            __builtin_nontemporal_store(v, reinterpret_cast<u32x4_t*>(out + (size_t)m * ldc + n));
          }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      }
      continue;
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int m = m0 + wm * WM + i * 32 + l32;
      if (m >= M) continue;
#pragma unroll
      for (int j = 0; j < TN; ++j) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n = n0 + wn * WN + j * 32 + 8 * q + 4 * lhi;
          if (n < N) {
            uint2 v;
            v.x = pack2(acc[i][j][4 * q + 0], acc[i][j][4 * q + 1]);
            v.y = pack2(acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]);
            if (bias) {
              const uint2 bv = *reinterpret_cast<const uint2*>(bias + n);
              v.x = add_bias2(v.x, bv.x);
              v.y = add_bias2(v.y, bv.y);
            }
            *reinterpret_cast<uint2*>(out + (size_t)m * ldc + n) = v;
          }
        }
      }
    }
  }
}

template <int TM, int TN>
static int launch_big(const GemmBatch& batch, int count, int64_t M, int64_t N, int64_t K, int64_t ldc,
                      int max_cus, hipStream_t hs) {
  constexpr int BM = 64 * TM, BN = 128 * TN;
  constexpr int LDS = big_lds_bytes(TM, TN);
  // the attribute belongs to the function on one device: set it once per device
  constexpr int kMaxDevices = 64;
  static std::atomic<bool> lds_ok[kMaxDevices];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
    return set_error(TW_ERR_LAUNCH, "gemm_bf16_nt: no current device");
  if (!lds_ok[dev].load(std::memory_order_acquire)) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_bf16_nt_big_kernel<TM, TN>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, LDS) != hipSuccess)
      return set_error(TW_ERR_LAUNCH, "gemm_bf16_nt: the device refused %d bytes of LDS", LDS);
    lds_ok[dev].store(true, std::memory_order_release);
  }
  const int tiles_m = (int)((M + BM - 1) / BM), tiles_n = (int)((N + BN - 1) / BN);
  int64_t grid = (int64_t)count * tiles_m * tiles_n;
  if (max_cus > 0 && grid > max_cus) grid = max_cus;
  // 16-byte stores need 16-byte aligned row segments that end inside the row
  int wide_store = (N % 8 == 0 && ldc % 8 == 0) ? 1 : 0;
  for (int p = 0; p < count; ++p)
    if ((reinterpret_cast<uintptr_t>(batch.out[p]) | reinterpret_cast<uintptr_t>(batch.bias[p])) & 15u) wide_store = 0;
  launch_kernel(gemm_bf16_nt_big_kernel<TM, TN>, dim3((unsigned)grid), dim3(BIG_THREADS), LDS, hs, batch, count,
                (int)M, (int)N, (int)K, ldc, tiles_m, tiles_n, wide_store);
  return TW_OK;
}

// Workgroup tile for the problem, (64 TM) x (128 TN).  Cost = rounds x (tile area /
// relative throughput + a fixed part per round); ties go to the earlier entry.  The
// 64-wide wave tiles come in four heights so that a tile count can be made to fit the
// compute units exactly (M = 2458: 320-row tiles make 256 tiles; the 128-row tile loads
// 30 % more operand bytes per flop than the 192-row one and is rated 0.85); 256 x 384 (96-wide
// wave tiles, 192 accumulators, exactly 160 KiB of LDS) wins where its fewer, larger
// rounds fit.  96 x 96 wave tiles (192 x 384) were measured no faster per area than
// 256 x 256 and are not offered.
struct BigTile { int tm, tn; };

static BigTile pick_big_tile(int64_t M, int64_t N, int count, int cus) {
  // Relative throughput per tile area, measured: the 256 x 384 tile loads a fifth fewer
  // operand bytes per flop and runs a round in 1.35x the time of a 256 x 256 round.
  static const struct { int tm, tn; double eff; } kTiles[] = {
      {2, 2, 0.85}, {3, 2, 1.0}, {4, 2, 1.0}, {5, 2, 1.0}, {4, 3, 1.1}};
  BigTile best = {4, 2};
  double best_cost = 1e300;
  for (const auto& t : kTiles) {
    const int64_t tiles = count * ((M + 64 * t.tm - 1) / (64 * t.tm)) * ((N + 128 * t.tn - 1) / (128 * t.tn));
    const int64_t rounds = (tiles + cus - 1) / cus;
    const double cost = (double)rounds * (64.0 * t.tm * 128.0 * t.tn / t.eff + 2048.0);
    if (cost < best_cost) {
      best_cost = cost;
      best = BigTile{t.tm, t.tn};
    }
  }
  return best;
}

// The tile shape never changes a result bit: every output element is the same sequence of
// MFMA k-steps whatever tile it lies in.
static bool big_kernel_fits(int64_t M, int64_t N, int64_t K) {
  // at least one whole 64-wide k-slab, 32-bit byte offsets into both operands (below the
  // out-of-range marker when a last partial slab has to be zero-filled), and enough rows and
  // columns to be worth the larger prologue
  const uint64_t limit = (K % BIG_BK == 0) ? (1ull << 31) : (1ull << 30);  // elements per operand
  return K >= BIG_BK && (uint64_t)M * K < limit && (uint64_t)N * K < limit && M >= 192 && N >= 192;
}

static int launch_big_for(const GemmBatch& batch, int count, int64_t M, int64_t N, int64_t K, int64_t ldc,
                          int max_cus, hipStream_t hs) {
  int cus = max_cus > 0 ? max_cus : device_compute_units();
  if (cus <= 0) cus = 256;
  const BigTile bt = pick_big_tile(M, N, count, cus);
  if (bt.tn == 3) return launch_big<4, 3>(batch, count, M, N, K, ldc, max_cus, hs);
  if (bt.tm == 2) return launch_big<2, 2>(batch, count, M, N, K, ldc, max_cus, hs);
  if (bt.tm == 3) return launch_big<3, 2>(batch, count, M, N, K, ldc, max_cus, hs);
  if (bt.tm == 5) return launch_big<5, 2>(batch, count, M, N, K, ldc, max_cus, hs);
  return launch_big<4, 2>(batch, count, M, N, K, ldc, max_cus, hs);
}

static int check_gemm_shape(const char* what, int64_t M, int64_t N, int64_t K, int64_t ldc) {
  if (M < 0 || N <= 0 || K <= 0 || M > INT32_MAX || N > INT32_MAX || K > INT32_MAX || ldc < N)
    return set_error(TW_ERR_INVALID_ARGUMENT, "%s: bad shape M=%lld N=%lld K=%lld ldc=%lld", what, (long long)M,
                     (long long)N, (long long)K, (long long)ldc);
  if (K % 8 != 0 || N % 4 != 0 || ldc % 4 != 0)
    return set_error(TW_ERR_ALIGNMENT, "%s: needs K %% 8 == 0, N %% 4 == 0, ldc %% 4 == 0", what);
  return TW_OK;
}

static int check_gemm_pointers(const char* what, const void* out, const void* a, const void* b,
                               const void* bias) {
  if (!out || !a || !b) return set_error(TW_ERR_INVALID_ARGUMENT, "%s: null pointer argument", what);
  auto al = [](const void* p, unsigned n) { return (reinterpret_cast<uintptr_t>(p) & (n - 1)) == 0; };
  if (!al(a, 16) || !al(b, 16) || !al(out, 8) || !al(bias, 8))
    return set_error(TW_ERR_ALIGNMENT, "%s: needs 16-byte aligned a and b, 8-byte aligned out and bias", what);
  return TW_OK;
}

int run_gemm_bf16_nt(void* out, const void* a, const void* b, const void* bias, int64_t M, int64_t N,
                     int64_t K, int64_t ldc, int max_cus, void* stream) {
  if (int rc = check_gemm_shape("gemm_bf16_nt", M, N, K, ldc)) return rc;
  if (M == 0) return TW_OK;
  if (int rc = check_gemm_pointers("gemm_bf16_nt", out, a, b, bias)) return rc;
  hipStream_t hs = static_cast<hipStream_t>(stream);
  if (big_kernel_fits(M, N, K)) {
    GemmBatch batch = {};
    batch.out[0] = static_cast<uint16_t*>(out);
    batch.a[0] = static_cast<const uint16_t*>(a);
    batch.b[0] = static_cast<const uint16_t*>(b);
    batch.bias[0] = static_cast<const uint16_t*>(bias);
    if (int rc = launch_big_for(batch, 1, M, N, K, ldc, max_cus, hs)) return rc;
  } else {
    const int tiles_m = (int)((M + BM - 1) / BM), tiles_n = (int)((N + BN - 1) / BN);
    int64_t grid = (int64_t)tiles_m * tiles_n;
    if (max_cus > 0 && grid > max_cus) grid = max_cus;
    if (grid > INT32_MAX) grid = INT32_MAX;
    launch_kernel(gemm_bf16_nt_kernel, dim3((unsigned)grid), dim3(GEMM_THREADS), 0, hs,
                  static_cast<uint16_t*>(out), static_cast<const uint16_t*>(a),
                  static_cast<const uint16_t*>(b), static_cast<const uint16_t*>(bias), (int)M, (int)N, (int)K, ldc,
                  tiles_m, tiles_n);
  }
  return finish_launch("gemm_bf16_nt");
}

// outs[p][M, N] (row stride ldc) = as[p][M, K] * bs[p][N, K]^T (+ biases[p] when `biases` and
// that entry are non-null) for p < count: one launch over count x tiles when the shape fits
// the big kernel, one launch per product otherwise.
int run_gemm_bf16_nt_partials(void* const* outs, const void* const* as, const void* const* bs,
                              const void* const* biases, int count, int64_t M, int64_t N, int64_t K,
                              int64_t ldc, int max_cus, void* stream) {
  const char* what = "gemm_bf16_nt_partials";
  if (count < 1 || count > TW_MAX_PARTIALS)
    return set_error(TW_ERR_INVALID_ARGUMENT, "%s: number of partials %d not in [1, %d]", what, count,
                     TW_MAX_PARTIALS);
  if (int rc = check_gemm_shape(what, M, N, K, ldc)) return rc;
  if (M == 0) return TW_OK;
  if (!outs || !as || !bs) return set_error(TW_ERR_INVALID_ARGUMENT, "%s: null pointer argument", what);
  GemmBatch batch = {};
  for (int p = 0; p < count; ++p) {
    const void* bias = biases ? biases[p] : nullptr;
    if (int rc = check_gemm_pointers(what, outs[p], as[p], bs[p], bias)) return rc;
    batch.bias[p] = static_cast<const uint16_t*>(bias);
    batch.out[p] = static_cast<uint16_t*>(outs[p]);
    batch.a[p] = static_cast<const uint16_t*>(as[p]);
    batch.b[p] = static_cast<const uint16_t*>(bs[p]);
  }
  if (big_kernel_fits(M, N, K)) {
    if (int rc = launch_big_for(batch, count, M, N, K, ldc, max_cus, static_cast<hipStream_t>(stream))) return rc;
    return finish_launch(what);
  }
  for (int p = 0; p < count; ++p)
    if (int rc = run_gemm_bf16_nt(outs[p], as[p], bs[p], batch.bias[p], M, N, K, ldc, max_cus, stream)) return rc;
  return TW_OK;
}

}  // namespace tw
