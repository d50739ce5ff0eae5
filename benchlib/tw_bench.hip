// libtw_bench.so — kernels that exist for MEASUREMENT and TESTING only; bench.py and the
// tests load this library, the product (libtokenweave_amd.so and the Python package)
// never does.  The library's own sources are compiled into it, but none of the tw_*
// entry points is exported from here: only the twb_* functions below are.
//
//  * the library's own norm kernels compiled with timeline stamps (TW_TRACE): the
//    same source, plus per-row wall-clock stamps written to a caller's buffer;
//  * memory-system yardsticks with the launch shape of the headline norm kernel (one
//    workgroup of 256 lanes per 16 KiB row, four 16-byte vectors per lane per stream):
//    a read-only stream over the row's nine input streams, a stand-in that moves the
//    norm kernel's exact traffic (nine streams read, two written in place) without
//    arithmetic, reduction or barrier, a plain copy with default cache policy whose
//    traffic is known exactly (hardware counters are scaled against it), and an empty
//    kernel (launch-to-launch floor);
//  * the main loop of the big GEMM kernel put together from its parts (MFMAs, fragment
//    reads from LDS, operand slabs global -> LDS, the barrier per k-slab) on operands that
//    stay in the L2s, and the rate at which waves get 16-byte LDS reads through: what the
//    loop itself can reach on this machine, apart from tile prologue and epilogue;
//  * the split-row kernel WITHOUT its row-to-XCD placement (the segments of a row spread
//    over the XCDs), which the product never launches: the tests run it against the same
//    bits to pin that the cross-workgroup hand-over does not depend on the placement.
#define TW_TRACE 1
#define TW_API __attribute__((visibility("hidden")))
#define TWB_API __attribute__((visibility("default")))
#include "tw_api.hip"
#include "tw_gemm.hip"
#include "tw_norm.hip"

namespace twb {

// host copy of the device-side trace pointer (tw::g_trace): null outside a traced burst
static unsigned long long* g_trace_current = nullptr;

using tw::kLoadStream;
using tw::load16;
using tw::row_desc;
using tw::store16;

struct Streams {
  const void* p[9];
};

// One workgroup per row (the launchers start exactly `rows` workgroups, so the kernels
// neither test nor loop: like the norm kernel they make one round trip to their
// arguments before the first load).
// Per row: nine streams read with the norm kernel's loads.  MODE 0: read them (nothing is
// written unless the data matches a pattern that random inputs never produce); 1: read
// them and store the folded value over the row in streams 0 and 8 (the norm's y and
// residual); 2: overwrite streams 0 and 8 and read nothing (what the memory system gives
// the stores by themselves).
template <int MODE>
__global__ __launch_bounds__(256) void stream_rows_kernel(Streams st, uint4* sink, int vec_per_row) {
  // all kernel arguments are demanded here, so that they are fetched in one round trip
  asm volatile("" ::"s"(st.p[0]), "s"(st.p[1]), "s"(st.p[2]), "s"(st.p[3]), "s"(st.p[4]), "s"(st.p[5]),
               "s"(st.p[6]), "s"(st.p[7]), "s"(st.p[8]), "s"(vec_per_row));
  const uint32_t row_bytes = (uint32_t)vec_per_row * 16u;
  const int row = blockIdx.x;  // launched with one workgroup per row: no test, no loop
  if (MODE == 2) {
    const __amdgpu_buffer_rsrc_t d0 = row_desc(st.p[0], row, row_bytes);
    const __amdgpu_buffer_rsrc_t d8 = row_desc(st.p[8], row, row_bytes);
    const uint4 v = make_uint4(row, threadIdx.x, 0x3f803f80u, 0x3f803f80u);
#pragma unroll
    for (int k = 0; k < 4; ++k) store16(d8, (threadIdx.x + k * 256) * 16u, v);
#pragma unroll
    for (int k = 0; k < 4; ++k) store16(d0, (threadIdx.x + k * 256) * 16u, v);
    return;
  }
  uint4 a[4][9];
#pragma unroll
  for (int s = 0; s < 9; ++s) {
    const __amdgpu_buffer_rsrc_t d = row_desc(st.p[s], row, row_bytes);
#pragma unroll
    for (int k = 0; k < 4; ++k) a[k][s] = load16<kLoadStream>(d, (threadIdx.x + k * 256) * 16u);
  }
  // every load of the row is in flight before the first use, as in the norm kernel
  __builtin_amdgcn_sched_barrier(0);
  uint4 f[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    f[k] = a[k][0];
#pragma unroll
    for (int s = 1; s < 9; ++s) {
      f[k].x ^= a[k][s].x;
      f[k].y ^= a[k][s].y;
      f[k].z ^= a[k][s].z;
      f[k].w ^= a[k][s].w;
    }
  }
  if (MODE == 1) {
    const __amdgpu_buffer_rsrc_t d0 = row_desc(st.p[0], row, row_bytes);
    const __amdgpu_buffer_rsrc_t d8 = row_desc(st.p[8], row, row_bytes);
#pragma unroll
    for (int k = 0; k < 4; ++k) store16(d8, (threadIdx.x + k * 256) * 16u, f[k]);
#pragma unroll
    for (int k = 0; k < 4; ++k) store16(d0, (threadIdx.x + k * 256) * 16u, f[k]);
  } else {
#pragma unroll
    for (int k = 0; k < 4; ++k)
      if (f[k].x == 0x5eed5eedu && f[k].y == 0x0badf00du && f[k].z == 0x12345678u && f[k].w == 0x9abcdef0u)
        sink[threadIdx.x] = f[k];
  }
}

// The read-and-write form with arrival stamps: trace[row][0] = row begins, [1 + s] =
// stream s has returned (in issue order), [10] = stores issued, [11] = stores
// acknowledged; 16 slots per row, wall clock in 10 ns units.
template <int N>
__device__ __forceinline__ void wait_loads_outstanding() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

__global__ __launch_bounds__(256) void stream_rows_trace_kernel(Streams st, unsigned long long* trace, int rows,
                                                                int vec_per_row) {
  const uint32_t row_bytes = (uint32_t)vec_per_row * 16u;
  {
    const int row = blockIdx.x;  // launched with one workgroup per row: no test, no loop
    unsigned long long* t = trace + (size_t)row * 16;
    const bool rec = threadIdx.x == 0;
    if (rec) t[0] = wall_clock64();
    uint4 a[4][9];
#pragma unroll
    for (int s = 0; s < 9; ++s) {
      const __amdgpu_buffer_rsrc_t d = row_desc(st.p[s], row, row_bytes);
#pragma unroll
      for (int k = 0; k < 4; ++k) a[k][s] = load16<kLoadStream>(d, (threadIdx.x + k * 256) * 16u);
    }
    __builtin_amdgcn_sched_barrier(0);
    uint4 f[4];
#define TWB_ARRIVED(S)                                  \
  wait_loads_outstanding<4 * (8 - S)>();                \
  if (rec) t[1 + S] = wall_clock64();                   \
  _Pragma("unroll") for (int k = 0; k < 4; ++k) {       \
    if (S == 0) f[k] = a[k][0];                         \
    else {                                              \
      f[k].x ^= a[k][S].x; f[k].y ^= a[k][S].y;         \
      f[k].z ^= a[k][S].z; f[k].w ^= a[k][S].w;         \
    }                                                   \
  }                                                     \
  __builtin_amdgcn_sched_barrier(0);
    TWB_ARRIVED(0) TWB_ARRIVED(1) TWB_ARRIVED(2) TWB_ARRIVED(3) TWB_ARRIVED(4)
    TWB_ARRIVED(5) TWB_ARRIVED(6) TWB_ARRIVED(7) TWB_ARRIVED(8)
#undef TWB_ARRIVED
    const __amdgpu_buffer_rsrc_t d0 = row_desc(st.p[0], row, row_bytes);
    const __amdgpu_buffer_rsrc_t d8 = row_desc(st.p[8], row, row_bytes);
#pragma unroll
    for (int k = 0; k < 4; ++k) store16(d8, (threadIdx.x + k * 256) * 16u, f[k]);
#pragma unroll
    for (int k = 0; k < 4; ++k) store16(d0, (threadIdx.x + k * 256) * 16u, f[k]);
    if (rec) t[10] = wall_clock64();
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (rec) t[11] = wall_clock64();
  }
}

__global__ __launch_bounds__(256) void copy16_kernel(uint4* __restrict__ dst, const uint4* __restrict__ src,
                                                     size_t n) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) dst[i] = src[i];
}

__global__ void empty_kernel() {}

// Reads one dword every `step` bytes of two regions, from every XCD (workgroup b runs on
// XCD b % 8 and takes the addresses of slice b / 8): afterwards the address translations
// of the regions are in the translation caches of every XCD while (with step >= 4 KiB)
// next to none of their data is in any cache.  Streaming loads, nothing written unless the
// data matches a pattern that random inputs never produce.
__global__ __launch_bounds__(64) void touch_pages_kernel(const uint8_t* a, uint64_t a_bytes, const uint8_t* b,
                                                         uint64_t b_bytes, uint32_t step, uint32_t* sink) {
  const uint64_t slices = gridDim.x >> 3, slice = blockIdx.x >> 3;
  uint32_t v = 0;
  for (uint64_t off = (slice * 64 + threadIdx.x) * (uint64_t)step; off < a_bytes; off += slices * 64 * step)
    v ^= __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(a + off));
  for (uint64_t off = (slice * 64 + threadIdx.x) * (uint64_t)step; off < b_bytes; off += slices * 64 * step)
    v ^= __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(b + off));
  if (v == 0x5eed5eedu) sink[threadIdx.x] = v;
}

// One lane reads `count` dwords, `stride` bytes apart from base + offset, one after the
// other (each read waits for the previous one), and notes how long each took on the
// constant-rate wall clock (10 ns units): out[k] = latency of read k.  Streaming loads:
// nothing is kept in a cache on the way.
__global__ __launch_bounds__(64) void latency_chain_kernel(const uint8_t* base, uint64_t stride, int count,
                                                           uint64_t offset, uint32_t* out, uint32_t* sink) {
  if (threadIdx.x != 0) return;
  uint32_t acc = 0;
  for (int k = 0; k < count; ++k) {
    const uint32_t* p = reinterpret_cast<const uint32_t*>(base + (uint64_t)k * stride + offset);
    const unsigned long long t0 = wall_clock64();
    const uint32_t v = __builtin_nontemporal_load(p);
    asm volatile("s_waitcnt vmcnt(0)" ::"v"(v) : "memory");
    const unsigned long long t1 = wall_clock64();
    acc ^= v;
    out[k] = (uint32_t)(t1 - t0);
  }
  if (acc == 0x5eed5eedu) sink[0] = acc;
}

// One wave that watches both clocks for `ticks` units of the constant-rate wall clock
// (10 ns each): out[0] = shader-clock cycles, out[1] = wall-clock ticks that went by.  The
// ratio is the shader clock the compute unit ran at during the window.
__global__ __launch_bounds__(64) void clock_probe_kernel(long long* out, long long ticks) {
  const long long t0 = wall_clock64();
  const long long c0 = __builtin_readcyclecounter();
  long long t1 = t0;
  // bounded: the wall clock advances whatever else happens, so the wave always leaves
  while (t1 - t0 < ticks) t1 = wall_clock64();
  const long long c1 = __builtin_readcyclecounter();
  if (threadIdx.x == 0) {
    out[0] = c1 - c0;
    out[1] = t1 - t0;
  }
}


// The k loop of gemm_bf16_nt_big_kernel<5, 2> (eight waves, 160 x 64 wave tiles, 320 x 256 x 64
// slabs, two LDS stages) assembled from switchable parts; the arithmetic result is
// meaningless.  parts bit 0: fragment reads from LDS (else the MFMAs reuse their first
// operands); bit 1: the slab loads global -> LDS (from a `window`-byte region per XCD, so
// the L2s serve them); bit 2: issue the slab's loads over the four k-steps instead of at
// the slab's head.  Every variant keeps the wait + barrier per slab, which also keeps the
// two waves of a SIMD in step, so that wave 0's clock stamps stand for the workgroup.
// out[2 b] = shader-clock cycles, out[2 b + 1] = wall clock (10 ns) of workgroup b.
__global__ __launch_bounds__(512) void gemm_loop_kernel(int slabs, int parts, uint32_t window, const uint8_t* src,
                                                        long long* out, float* sink) {
  constexpr int TM = 5, TN = 2, STAGE = (320 + 256) * 128, LOADS = 9;
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int l32 = lane & 31, lhi = lane >> 5;
  const bool reads = parts & 1, loads = parts & 2, spread = parts & 4;
  for (int i = threadIdx.x; i < 2 * STAGE / 4; i += blockDim.x)
    reinterpret_cast<uint32_t*>(lds)[i] = 0x3c003c00u + (i & 3);
  __syncthreads();
  uint32_t roff[4];
  for (int kk = 0; kk < 4; ++kk) roff[kk] = l32 * 128 + ((((kk << 1) | lhi) ^ ((l32 >> 1) & 7)) << 4);
  const uint8_t* pa = lds + (wave >> 2) * (32 * TM) * 128;
  const uint8_t* pb = lds + 320 * 128 + (wave & 3) * (32 * TN) * 128;
  const __amdgpu_buffer_rsrc_t d = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint8_t*>(src) + (size_t)(blockIdx.x & 7) * window, 0, window, 0x00020000);
  tw::f32x16_t acc[TM][TN];
  for (int i = 0; i < TM; ++i)
    for (int j = 0; j < TN; ++j)
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;
  tw::bf16x8_t fa[2][TM], fb[2][TN];
  for (int i = 0; i < TM; ++i)
    fa[0][i] = fa[1][i] = __builtin_bit_cast(tw::bf16x8_t, *reinterpret_cast<const uint4*>(pa + i * 4096 + roff[0]));
  for (int j = 0; j < TN; ++j)
    fb[0][j] = fb[1][j] = __builtin_bit_cast(tw::bf16x8_t, *reinterpret_cast<const uint4*>(pb + j * 4096 + roff[0]));
  __syncthreads();
  const long long t0 = wall_clock64();
  const long long c0 = __builtin_readcyclecounter();
  for (int s = 0; s < slabs; ++s) {
    const int stage = s & 1;
    // a different slab-sized piece of the window per workgroup and slab
    uint32_t base = (uint32_t)(((blockIdx.x >> 3) * STAGE + s * STAGE * 7) & (window - 1)) & ~1023u;
    if (base > window - STAGE) base = window - STAGE;  // the whole slab lies inside the window
    uint8_t* dst = lds + (stage ^ 1) * STAGE + wave * LOADS * 1024;
    const uint8_t* qa = pa + stage * STAGE;
    const uint8_t* qb = pb + stage * STAGE;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      const int cur = kk & 1, nxt = cur ^ 1;
      if (loads) {
#pragma unroll
        for (int j = 0; j < LOADS; ++j)
          if (spread ? (j * 4) / LOADS == kk : kk == 0)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(d, (tw::lds_void_t*)(dst + j * 1024), 16,
                                                     (uint32_t)(lane * 16 + (wave * LOADS + j) * 1024), base, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < (TM + 1) / 2; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[cur][j], fa[cur][i], acc[i][j], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      if (reads) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
          fa[nxt][i] = __builtin_bit_cast(tw::bf16x8_t,
                                          *reinterpret_cast<const uint4*>(qa + i * 4096 + roff[(kk + 1) & 3]));
#pragma unroll
        for (int j = 0; j < TN; ++j)
          fb[nxt][j] = __builtin_bit_cast(tw::bf16x8_t,
                                          *reinterpret_cast<const uint4*>(qb + j * 4096 + roff[(kk + 1) & 3]));
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = (TM + 1) / 2; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[cur][j], fa[cur][i], acc[i][j], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  }
  const long long c1 = __builtin_readcyclecounter();
  const long long t1 = wall_clock64();
  float t = 0.0f;
  for (int i = 0; i < TM; ++i)
    for (int j = 0; j < TN; ++j)
      for (int e = 0; e < 16; ++e) t += acc[i][j][e];
  if (t == 12345.678f) sink[threadIdx.x] = t;  // keeps the MFMAs alive; never true
  if (threadIdx.x == 0) {
    out[blockIdx.x * 2] = c1 - c0;
    out[blockIdx.x * 2 + 1] = t1 - t0;
  }
}

// 16-byte LDS reads with the GEMM's fragment addressing, 28 per wave and iteration (one
// k-slab's worth), by blockDim / 64 waves; dma: each wave also brings nine 1 KiB pieces
// global -> LDS per iteration (the slab loads).  out[b] = shader-clock cycles of workgroup b.
__global__ __launch_bounds__(1024) void lds_read_rate_kernel(int iters, int dma, const uint8_t* src, long long* out,
                                                             uint32_t* sink) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int l32 = lane & 31, lhi = lane >> 5;
  for (int i = threadIdx.x; i < 147456 / 4; i += blockDim.x) reinterpret_cast<uint32_t*>(lds)[i] = i;
  uint32_t roff[4];
  for (int kk = 0; kk < 4; ++kk) roff[kk] = l32 * 128 + ((((kk << 1) | lhi) ^ ((l32 >> 1) & 7)) << 4);
  const uint8_t* base = lds + (wave % 8) * 8192;
  const __amdgpu_buffer_rsrc_t d = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(src), 0, 1u << 20, 0x00020000);
  uint4 acc = make_uint4(0, 0, 0, 0);
  __syncthreads();
  const long long c0 = __builtin_readcyclecounter();
  for (int it = 0; it < iters; ++it) {
    if (dma && wave < 8) {
#pragma unroll
      for (int j = 0; j < 9; ++j)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(d, (tw::lds_void_t*)(lds + 73728 + (wave * 9 + j) * 1024), 16,
                                                 (uint32_t)(lane * 16 + (wave * 9 + j) * 1024), 0, 0, 0);
    }
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
#pragma unroll
      for (int f = 0; f < 7; ++f) {
        const uint4 v = *reinterpret_cast<const uint4*>(base + f * 4096 + roff[kk]);
        acc.x ^= v.x; acc.y ^= v.y; acc.z ^= v.z; acc.w ^= v.w;
      }
    }
  }
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
  __syncthreads();
  const long long c1 = __builtin_readcyclecounter();
  if (threadIdx.x == 0) out[blockIdx.x] = c1 - c0;
  if (acc.x == 0x12345u && acc.y == 7u) sink[threadIdx.x] = acc.z + acc.w;  // never true for the fill above
}

}  // namespace twb

extern "C" {

// dst[0, nbytes) <- src[0, nbytes): grid-stride copy, 16 bytes per lane, default cache policy.
TWB_API int twb_copy_bytes(void* dst, const void* src, int64_t nbytes, void* stream) {
  if (nbytes < 0 || nbytes % 16 != 0 || !dst || !src ||
      ((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) & 15u))
    return tw::set_error(TW_ERR_INVALID_ARGUMENT, "copy: needs 16-byte aligned pointers and size");
  const size_t n = (size_t)nbytes / 16;
  if (n == 0) return TW_OK;
  const int cus = tw::device_compute_units();
  size_t blocks = (n + 255) / 256;
  const size_t cap = (size_t)(cus > 0 ? cus : 256) * 16;
  if (blocks > cap) blocks = cap;
  tw::launch_kernel(twb::copy16_kernel, dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                    static_cast<uint4*>(dst), static_cast<const uint4*>(src), n);
  return tw::finish_launch("copy");
}

// streams: HOST array of nine device pointers, each [rows, hidden_size] bf16 (16 KiB rows
// at most: hidden_size <= 8192, hidden_size % 8 == 0).  write = 0: read the nine streams;
// 1: read them and overwrite streams 0 and 8; 2: overwrite streams 0 and 8, read nothing.
// sink: 4 KiB of device memory (never written with random data).
TWB_API int twb_stream_rows(const void* const* streams, void* sink, int64_t rows, int64_t hidden_size,
                           int write, void* stream) {
  if (!streams || !sink || rows < 1 || rows > INT32_MAX || hidden_size < 8 || hidden_size > 8192 ||
      hidden_size % 8 != 0)
    return tw::set_error(TW_ERR_INVALID_ARGUMENT, "stream_rows: bad argument");
  twb::Streams st;
  for (int s = 0; s < 9; ++s) {
    if (!streams[s] || (reinterpret_cast<uintptr_t>(streams[s]) & 15u))
      return tw::set_error(TW_ERR_INVALID_ARGUMENT, "stream_rows: stream %d null or misaligned", s);
    st.p[s] = streams[s];
  }
  const dim3 g((unsigned)rows), b(256);
  hipStream_t hs = static_cast<hipStream_t>(stream);
  uint4* sk = static_cast<uint4*>(sink);
  const int vec = (int)(hidden_size / 8);
  if (write == 2) tw::launch_kernel(twb::stream_rows_kernel<2>, g, b, 0, hs, st, sk, vec);
  else if (write) tw::launch_kernel(twb::stream_rows_kernel<1>, g, b, 0, hs, st, sk, vec);
  else tw::launch_kernel(twb::stream_rows_kernel<0>, g, b, 0, hs, st, sk, vec);
  return tw::finish_launch("stream_rows");
}

// twb_stream_rows(write = 1) with arrival stamps; trace: rows x 16 uint64 of device memory.
TWB_API int twb_trace_stream_rows(const void* const* streams, void* trace, int64_t rows, int64_t hidden_size,
                                 void* stream) {
  if (!streams || !trace || rows < 1 || rows > INT32_MAX || hidden_size < 8 || hidden_size > 8192 ||
      hidden_size % 8 != 0)
    return tw::set_error(TW_ERR_INVALID_ARGUMENT, "trace_stream_rows: bad argument");
  twb::Streams st;
  for (int s = 0; s < 9; ++s) {
    if (!streams[s] || (reinterpret_cast<uintptr_t>(streams[s]) & 15u))
      return tw::set_error(TW_ERR_INVALID_ARGUMENT, "trace_stream_rows: stream %d null or misaligned", s);
    st.p[s] = streams[s];
  }
  tw::launch_kernel(twb::stream_rows_trace_kernel, dim3((unsigned)rows), dim3(256), 0,
                    static_cast<hipStream_t>(stream), st, static_cast<unsigned long long*>(trace), (int)rows,
                    (int)(hidden_size / 8));
  return tw::finish_launch("trace_stream_rows");
}

TWB_API int twb_empty(int grid, int block, void* stream) {
  if (grid < 1 || block < 1 || block > 1024) return tw::set_error(TW_ERR_INVALID_ARGUMENT, "empty: bad launch shape");
  tw::launch_kernel(twb::empty_kernel, dim3((unsigned)grid), dim3((unsigned)block), 0,
                    static_cast<hipStream_t>(stream));
  return tw::finish_launch("empty");
}

// See touch_pages_kernel.  a, b: device regions (b may be null), sizes in bytes; step: a
// multiple of 4, at least 128; sink: 256 bytes of device memory; grid = 8 * slices workgroups.
TWB_API int twb_touch_pages(const void* a, int64_t a_bytes, const void* b, int64_t b_bytes, int step, int slices,
                            void* sink, void* stream) {
  if (!a || a_bytes < 4 || (b && b_bytes < 4) || step < 128 || step % 4 != 0 || slices < 1 || slices > 4096 ||
      !sink || (reinterpret_cast<uintptr_t>(a) & 3u) || (reinterpret_cast<uintptr_t>(b) & 3u))
    return tw::set_error(TW_ERR_INVALID_ARGUMENT, "touch_pages: bad argument");
  // the last dword read of a region starts at a multiple of step below bytes - 3
  tw::launch_kernel(twb::touch_pages_kernel, dim3((unsigned)(8 * slices)), dim3(64), 0,
                    static_cast<hipStream_t>(stream), static_cast<const uint8_t*>(a), (uint64_t)(a_bytes - 3),
                    static_cast<const uint8_t*>(b), (uint64_t)(b ? b_bytes - 3 : 0), (uint32_t)step,
                    static_cast<uint32_t*>(sink));
  return tw::finish_launch("touch_pages");
}

// See latency_chain_kernel.  base: device region of at least (count - 1) * stride + offset + 4
// bytes; out: count uint32 of device memory; sink: 4 bytes.
TWB_API int twb_latency_chain(const void* base, int64_t stride, int count, int64_t offset, void* out, void* sink,
                              void* stream) {
  if (!base || !out || !sink || stride < 4 || stride % 4 != 0 || offset < 0 || offset % 4 != 0 || count < 1 ||
      count > (1 << 20) || (reinterpret_cast<uintptr_t>(base) & 3u))
    return tw::set_error(TW_ERR_INVALID_ARGUMENT, "latency_chain: bad argument");
  tw::launch_kernel(twb::latency_chain_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream),
                    static_cast<const uint8_t*>(base), (uint64_t)stride, count, (uint64_t)offset,
                    static_cast<uint32_t*>(out), static_cast<uint32_t*>(sink));
  return tw::finish_launch("latency_chain");
}

// Shader clock over a window of `microseconds` (1 .. 1000) on one compute unit: out is two
// int64 of device memory, {shader cycles, 10 ns wall-clock ticks}.
TWB_API int twb_clock_probe(void* out, int microseconds, void* stream) {
  if (!out || microseconds < 1 || microseconds > 1000)
    return tw::set_error(TW_ERR_INVALID_ARGUMENT, "clock_probe: bad argument");
  tw::launch_kernel(twb::clock_probe_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream),
                    static_cast<long long*>(out), (long long)microseconds * 100);
  return tw::finish_launch("clock_probe");
}

// tw_reduce_add_rms_norm with timeline stamps: trace is num_tokens x 8 uint64 of device
// memory.  Per row: [0] row begins, [1] all loads returned, [2] residual stores issued,
// [3] row sum known, [4] y stores issued, [5] all stores acknowledged (wall clock, 10 ns
// units), [6] XCC id << 32 | HW_ID, [7] unused.  The first call with a given trace buffer
// is synchronous on entry (it sets a device global); further calls with the same buffer
// are asynchronous, so a burst of launches runs back to back and leaves the stamps of its
// last launch.  Call twb_trace_end() before the trace buffer is freed.
TWB_API int twb_trace_reduce_add_rms_norm(const void* const* partials, int num_partials, void* y, void* residual,
                                         const void* weight, int64_t num_tokens, int64_t hidden_size,
                                         int max_ctas, float epsilon, void* trace, void* stream) {
  if (!trace) return tw::set_error(TW_ERR_INVALID_ARGUMENT, "trace: null trace buffer");
  unsigned long long* buf = static_cast<unsigned long long*>(trace);
  if (buf != twb::g_trace_current) {  // bench.py calls from one thread, on one device
    if (hipMemcpyToSymbol(HIP_SYMBOL(tw::g_trace), &buf, sizeof(buf)) != hipSuccess)
      return tw::set_error(TW_ERR_LAUNCH, "trace: could not set the trace pointer");
    twb::g_trace_current = buf;
  }
  return tw::run_row_norm("trace_reduce_add_rms_norm", partials, num_partials, y, residual, nullptr, weight,
                          nullptr, num_tokens, hidden_size, epsilon, TW_DTYPE_BF16, max_ctas, true, stream);
}


// Ends a traced burst: kernels launched after this write no stamps (the trace buffer may
// be freed).  Synchronous.
TWB_API int twb_trace_end(void) {
  unsigned long long* none = nullptr;
  if (hipMemcpyToSymbol(HIP_SYMBOL(tw::g_trace), &none, sizeof(none)) != hipSuccess)
    return tw::set_error(TW_ERR_LAUNCH, "trace: could not clear the trace pointer");
  twb::g_trace_current = nullptr;
  return TW_OK;
}

TWB_API const char* twb_last_error(void) { return tw_last_error(); }

// tw_reduce_add_rms_norm_ws through the split-row kernel with `segs_nwaves` waves per
// segment (4 or 8), the segments of a row placed on CONSECUTIVE workgroups — hence on
// different XCDs — instead of on one XCD: the form the product does not launch.  Requires
// what the split-row kernel requires (bf16, 16-byte alignment, hidden_size % 8 == 0,
// 1 <= num_tokens <= TW_SPLIT_MAX_TOKENS, a zeroed 256-byte aligned workspace of
// TW_SPLIT_WORKSPACE_BYTES) and at least two segments per row.
TWB_API int twb_reduce_add_rms_norm_split_spread(const void* const* partials, int num_partials, void* y,
                                                 void* residual, const void* weight, int64_t num_tokens,
                                                 int64_t hidden_size, float epsilon, int seg_waves,
                                                 void* workspace, void* stream) {
  const char* what = "reduce_add_rms_norm_split_spread";
  if (!partials || !y || !residual || !weight || !workspace || num_partials < 1 || num_partials > TW_MAX_PARTIALS ||
      num_tokens < 1 || num_tokens > TW_SPLIT_MAX_TOKENS || hidden_size < 8 || hidden_size % 8 != 0 ||
      (seg_waves != 4 && seg_waves != 8))
    return tw::set_error(TW_ERR_INVALID_ARGUMENT, "%s: bad argument", what);
  const int V = (int)(hidden_size / 8);
  const int nchunks = (V + 63) / 64;
  const int segs = (nchunks + seg_waves - 1) / seg_waves;
  if (nchunks > tw::kMaxChunks || segs < 2)
    return tw::set_error(TW_ERR_INVALID_ARGUMENT, "%s: the row has %d chunks, need 2 .. %d segments' worth", what,
                         nchunks, tw::kMaxChunks);
  auto misaligned = [](const void* p, unsigned n) { return (reinterpret_cast<uintptr_t>(p) & (n - 1)) != 0; };
  tw::PartialPtrs parts = {};
  bool bad = misaligned(y, 16) || misaligned(residual, 16) || misaligned(weight, 16) || misaligned(workspace, 256);
  for (int p = 0; p < num_partials; ++p) {
    if (!partials[p]) return tw::set_error(TW_ERR_INVALID_ARGUMENT, "%s: partial %d is null", what, p);
    bad = bad || misaligned(partials[p], 16);
    parts.p[p] = partials[p];
  }
  if (bad) return tw::set_error(TW_ERR_ALIGNMENT, "%s: misaligned pointer", what);
  const dim3 g((unsigned)(num_tokens * segs)), b((unsigned)(seg_waves * 64));
  hipStream_t hs = static_cast<hipStream_t>(stream);
  tw::SplitRow* ws = static_cast<tw::SplitRow*>(workspace);
#define TWB_SPREAD(NP)                                                                                          \
  tw::launch_kernel(tw::row_norm_split_kernel<NP, false>, g, b, 0, hs, parts, num_partials, y, residual, weight, \
                    ws, epsilon, (int)num_tokens, V, (float)hidden_size, segs, seg_waves * 64)
  switch (num_partials) {
    case 1: TWB_SPREAD(1); break;
    case 2: TWB_SPREAD(2); break;
    case 4: TWB_SPREAD(4); break;
    case 8: TWB_SPREAD(8); break;
    default: TWB_SPREAD(0); break;
  }
#undef TWB_SPREAD
  return tw::finish_launch(what);
}

// tw_gemm_bf16_nt with the big kernel's workgroup tile forced to (64 tm) x (128 tn), one
// workgroup per tile and no compute-unit budget, instead of the tile the library's cost
// model picks: the 192 x 256 and 128 x 256 tiles leave registers for a norm workgroup on
// the same compute unit, which the 320 x 256 tile does not.  Same operand rules as the
// library call; the shape must fit the big kernel.
TWB_API int twb_gemm_bf16_nt_tile(void* out, const void* a, const void* b, int64_t M, int64_t N, int64_t K,
                                  int64_t ldc, int tm, int tn, void* stream) {
  const char* what = "gemm_bf16_nt_tile";
  if (int rc = tw::check_gemm_shape(what, M, N, K, ldc)) return rc;
  if (int rc = tw::check_gemm_pointers(what, out, a, b, nullptr)) return rc;
  if (M == 0) return TW_OK;
  if (!tw::big_kernel_fits(M, N, K)) return tw::set_error(TW_ERR_INVALID_ARGUMENT, "%s: shape outside the big kernel", what);
  tw::GemmBatch batch = {};
  batch.out[0] = static_cast<uint16_t*>(out);
  batch.a[0] = static_cast<const uint16_t*>(a);
  batch.b[0] = static_cast<const uint16_t*>(b);
  hipStream_t hs = static_cast<hipStream_t>(stream);
  int rc = TW_ERR_INVALID_ARGUMENT;
  if (tm == 2 && tn == 2) rc = tw::launch_big<2, 2>(batch, 1, M, N, K, ldc, 0, hs);
  else if (tm == 3 && tn == 2) rc = tw::launch_big<3, 2>(batch, 1, M, N, K, ldc, 0, hs);
  else if (tm == 4 && tn == 2) rc = tw::launch_big<4, 2>(batch, 1, M, N, K, ldc, 0, hs);
  else if (tm == 5 && tn == 2) rc = tw::launch_big<5, 2>(batch, 1, M, N, K, ldc, 0, hs);
  else if (tm == 4 && tn == 3) rc = tw::launch_big<4, 3>(batch, 1, M, N, K, ldc, 0, hs);
  else return tw::set_error(TW_ERR_INVALID_ARGUMENT, "%s: no %d x %d tile", what, 64 * tm, 128 * tn);
  return rc ? rc : tw::finish_launch(what);
}

static int bench_lds_limit(const void* fn, int bytes) {
  return hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) == hipSuccess ? TW_OK
             : tw::set_error(TW_ERR_LAUNCH, "the device refused %d bytes of LDS", bytes);
}

// The GEMM's k loop from its parts (see gemm_loop_kernel).  src: 8 * window bytes of device
// memory, window a power of two >= 128 KiB; out: 2 * grid int64; sink: 512 floats.
TWB_API int twb_gemm_loop(int slabs, int parts, int64_t window, const void* src, void* out, void* sink, int grid,
                         void* stream) {
  if (slabs < 1 || grid < 1 || !src || !out || !sink || window < (128 << 10) || window > (1ll << 30) ||
      (window & (window - 1)))
    return tw::set_error(TW_ERR_INVALID_ARGUMENT, "gemm_loop: bad argument");
  if (int rc = bench_lds_limit(reinterpret_cast<const void*>(twb::gemm_loop_kernel), 147456)) return rc;
  tw::launch_kernel(twb::gemm_loop_kernel, dim3((unsigned)grid), dim3(512), 147456, static_cast<hipStream_t>(stream),
                    slabs, parts, (uint32_t)window, static_cast<const uint8_t*>(src), static_cast<long long*>(out),
                    static_cast<float*>(sink));
  return tw::finish_launch("gemm_loop");
}

// src: 1 MiB of device memory; out: grid int64; sink: 1024 uint32.
TWB_API int twb_lds_read_rate(int iters, int waves, int dma, const void* src, void* out, void* sink, int grid,
                             void* stream) {
  if (iters < 1 || waves < 1 || waves > 16 || grid < 1 || !src || !out || !sink)
    return tw::set_error(TW_ERR_INVALID_ARGUMENT, "lds_read_rate: bad argument");
  if (int rc = bench_lds_limit(reinterpret_cast<const void*>(twb::lds_read_rate_kernel), 147456)) return rc;
  tw::launch_kernel(twb::lds_read_rate_kernel, dim3((unsigned)grid), dim3((unsigned)waves * 64), 147456,
                    static_cast<hipStream_t>(stream), iters, dma, static_cast<const uint8_t*>(src),
                    static_cast<long long*>(out), static_cast<uint32_t*>(sink));
  return tw::finish_launch("lds_read_rate");
}

}  // extern "C"
