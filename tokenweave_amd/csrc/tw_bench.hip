// libtw_bench.so — kernels that exist for MEASUREMENT only; bench.py loads this
// library, the product (libtokenweave_amd.so and the Python package) never does.
//
//  * the library's own norm kernels compiled with timeline stamps (TW_TRACE): the
//    same source, plus per-row wall-clock stamps written to a caller's buffer;
//  * memory-system yardsticks with the launch shape of the headline norm kernel (one
//    workgroup of 256 lanes per 16 KiB row, four 16-byte vectors per lane per stream):
//    a read-only stream over the row's nine input streams, a stand-in that moves the
//    norm kernel's exact traffic (nine streams read, two written in place) without
//    arithmetic, reduction or barrier, a plain copy with default cache policy whose
//    traffic is known exactly (hardware counters are scaled against it), and an empty
//    kernel (launch-to-launch floor).
#define TW_TRACE 1
#include "tw_api.hip"
#include "tw_gemm.hip"
#include "tw_norm.hip"

namespace twb {

using tw::kLoadStream;
using tw::load16;
using tw::row_desc;
using tw::store16;

struct Streams {
  const void* p[9];
};

// Per row: nine streams read with the norm kernel's loads.  WRITE: the folded value is
// stored over the row in streams 0 and 8 (the norm's y and residual); otherwise nothing
// is written unless the data matches a pattern that random inputs never produce.
template <bool WRITE>
__global__ __launch_bounds__(256) void stream_rows_kernel(Streams st, uint4* sink, int rows, int vec_per_row,
                                                          int write_only) {
  const uint32_t row_bytes = (uint32_t)vec_per_row * 16u;
  if (WRITE && write_only) {
    // the two written streams alone: what the memory system gives the stores by themselves
    for (int row = blockIdx.x; row < rows; row += gridDim.x) {
      const __amdgpu_buffer_rsrc_t d0 = row_desc(st.p[0], row, row_bytes);
      const __amdgpu_buffer_rsrc_t d8 = row_desc(st.p[8], row, row_bytes);
      const uint4 v = make_uint4(row, threadIdx.x, 0x3f803f80u, 0x3f803f80u);
#pragma unroll
      for (int k = 0; k < 4; ++k) store16(d8, (threadIdx.x + k * 256) * 16u, v);
#pragma unroll
      for (int k = 0; k < 4; ++k) store16(d0, (threadIdx.x + k * 256) * 16u, v);
    }
    return;
  }
  for (int row = blockIdx.x; row < rows; row += gridDim.x) {
    uint4 a[4][9];
#pragma unroll
    for (int s = 0; s < 9; ++s) {
      const __amdgpu_buffer_rsrc_t d = row_desc(st.p[s], row, row_bytes);
#pragma unroll
      for (int k = 0; k < 4; ++k) a[k][s] = load16<kLoadStream>(d, (threadIdx.x + k * 256) * 16u);
    }
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
    if (WRITE) {
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
  for (int row = blockIdx.x; row < rows; row += gridDim.x) {
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

}  // namespace twb

extern "C" {

// dst[0, nbytes) <- src[0, nbytes): grid-stride copy, 16 bytes per lane, default cache policy.
TW_API int twb_copy_bytes(void* dst, const void* src, int64_t nbytes, void* stream) {
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
TW_API int twb_stream_rows(const void* const* streams, void* sink, int64_t rows, int64_t hidden_size,
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
  if (write)
    tw::launch_kernel(twb::stream_rows_kernel<true>, g, b, 0, hs, st, static_cast<uint4*>(sink), (int)rows,
                      (int)(hidden_size / 8), write == 2 ? 1 : 0);
  else
    tw::launch_kernel(twb::stream_rows_kernel<false>, g, b, 0, hs, st, static_cast<uint4*>(sink), (int)rows,
                      (int)(hidden_size / 8), 0);
  return tw::finish_launch("stream_rows");
}

// twb_stream_rows(write = 1) with arrival stamps; trace: rows x 16 uint64 of device memory.
TW_API int twb_trace_stream_rows(const void* const* streams, void* trace, int64_t rows, int64_t hidden_size,
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

TW_API int twb_empty(int grid, int block, void* stream) {
  if (grid < 1 || block < 1 || block > 1024) return tw::set_error(TW_ERR_INVALID_ARGUMENT, "empty: bad launch shape");
  tw::launch_kernel(twb::empty_kernel, dim3((unsigned)grid), dim3((unsigned)block), 0,
                    static_cast<hipStream_t>(stream));
  return tw::finish_launch("empty");
}

// tw_reduce_add_rms_norm with timeline stamps: trace is num_tokens x 8 uint64 of device
// memory.  Per row: [0] row begins, [1] all loads returned, [2] residual stores issued,
// [3] row sum known, [4] y stores issued, [5] all stores acknowledged (wall clock, 10 ns
// units), [6] XCC id << 32 | HW_ID, [7] unused.  Synchronous on entry (it sets a device
// global), asynchronous afterwards.
TW_API int twb_trace_reduce_add_rms_norm(const void* const* partials, int num_partials, void* y, void* residual,
                                         const void* weight, int64_t num_tokens, int64_t hidden_size,
                                         int max_ctas, float epsilon, void* trace, void* stream) {
  if (!trace) return tw::set_error(TW_ERR_INVALID_ARGUMENT, "trace: null trace buffer");
  unsigned long long* buf = static_cast<unsigned long long*>(trace);
  if (hipMemcpyToSymbol(HIP_SYMBOL(tw::g_trace), &buf, sizeof(buf)) != hipSuccess)
    return tw::set_error(TW_ERR_LAUNCH, "trace: could not set the trace pointer");
  return tw::run_row_norm("trace_reduce_add_rms_norm", partials, num_partials, y, residual, nullptr, weight,
                          nullptr, num_tokens, hidden_size, epsilon, TW_DTYPE_BF16, max_ctas, true, stream);
}

}  // extern "C"
