/*
 * tokenweave_amd — C ABI of the MI355X (gfx950) fused
 * P-partial reduce + residual-add + RMSNorm path.
 *
 * One rank, one GPU.  Every pointer is a DEVICE pointer to row-major,
 * row-contiguous memory ([num_tokens, hidden_size], element stride 1, row
 * stride hidden_size) unless stated otherwise.  Every call only ENQUEUES work
 * on `stream` (a hipStream_t; NULL = the default stream) of the device that is
 * current on the calling thread: no allocation, no host synchronisation, safe
 * under stream capture.  Return value: TW_OK, or a negative TW_ERR_* code with
 * a message retrievable from tw_last_error() on the same thread.  Nothing
 * throws across this boundary.
 *
 * Arithmetic (identical for every entry point; the reference's CPU path,
 * csrc/cpu/layernorm.cpp:44-88, with round-to-nearest-even stores):
 *   S   = sum_{p=0}^{P-1} f32(partial_p)        fp32, fixed order p = 0..P-1
 *   s   = S + f32(residual)                      fp32
 *   r'  = bf16_rne(s)                            -> residual (in place)
 *   inv = 1 / sqrt( sum_j s_j^2 / H + eps )      fp32, unrounded s
 *   y   = bf16_rne( f32(r') * inv * f32(w) )     -> output
 * Row results do not depend on num_tokens, on max_ctas or on which other rows
 * are in the call.
 */
#ifndef TOKENWEAVE_AMD_H
#define TOKENWEAVE_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Exported from the shared library.  (A build that compiles the sources into another
 * library may define TW_API beforehand to keep these names out of its own exports.) */
#ifndef TW_API
#define TW_API __attribute__((visibility("default")))
#endif

#define TW_OK 0
#define TW_ERR_INVALID_ARGUMENT (-1) /* null pointer, negative size, bad P / rank */
#define TW_ERR_ALIGNMENT (-2)        /* 16-byte alignment or H % 8 violated      */
#define TW_ERR_DTYPE (-3)            /* dtype not supported by this entry point   */
#define TW_ERR_LAUNCH (-4)           /* the HIP runtime refused the launch        */

/* Element types of the baseline ops (the reference dispatches them with
 * VLLM_DISPATCH_FLOATING_TYPES, csrc/dispatch_utils.h:14-21).  The *_cta and
 * reduce entry points are bf16 only, like the reference's
 * VLLM_BF16_DISPATCH_FLOATING_TYPES (csrc/dispatch_utils.h:23-27). */
#define TW_DTYPE_BF16 0
#define TW_DTYPE_F16 1
#define TW_DTYPE_F32 2

/* Output kinds of the dynamic per-token quantisation ops. */
#define TW_QUANT_FP8_E4M3FN 0
#define TW_QUANT_INT8 1

#define TW_MAX_PARTIALS 16

/* Library version (major*10000 + minor*100 + patch). */
TW_API int tw_version(void);

/* Message for the last non-TW_OK return on this thread ("" if none). */
TW_API const char* tw_last_error(void);

/* Number of compute units of the current device (<0 on error). */
TW_API int tw_num_compute_units(void);

/* input <- RMSNorm(input + residual) * weight ; residual <- input + residual.
 * Replaces ::fused_add_rms_norm (csrc/layernorm_kernels.cu:194-231, schema at
 * csrc/torch_bindings.cpp:141-144; CPU twin csrc/cpu/layernorm.cpp:105-117).
 * Any hidden_size and alignment are accepted: rows that are not 16-byte
 * aligned or hidden_size % 8 != 0 take an element-wise kernel, as the
 * reference's launcher does (layernorm_kernels.cu:223-230). */
TW_API int tw_fused_add_rms_norm(void* input, void* residual, const void* weight,
                          int64_t num_tokens, int64_t hidden_size,
                          float epsilon, int dtype, void* stream);

/* out <- RMSNorm(input) * weight.
 * Replaces ::rms_norm (csrc/layernorm_kernels.cu:165-181, schema at
 * csrc/torch_bindings.cpp:135-138; CPU twin csrc/cpu/layernorm.cpp:91-103). */
TW_API int tw_rms_norm(void* out, const void* input, const void* weight,
                int64_t num_tokens, int64_t hidden_size, float epsilon,
                int dtype, void* stream);

/* out <- input (the copy becomes the residual stream) ;
 * input <- RMSNorm(input) * weight.
 * Replaces ::rms_norm_inplace (csrc/tokenweave_fused_kernels.cu:186-202,
 * schema at csrc/torch_bindings.cpp:147-150). */
TW_API int tw_rms_norm_inplace(void* out, void* input, const void* weight,
                        int64_t num_tokens, int64_t hidden_size, float epsilon,
                        int dtype, void* stream);

/* tw_fused_add_rms_norm on a grid capped at max_ctas workgroups that walk the
 * rows with stride max_ctas (max_ctas <= 0: library default).  bf16 only;
 * pointers must be 16-byte aligned and hidden_size % 8 == 0, else
 * TW_ERR_ALIGNMENT.
 * Replaces ::fused_add_rms_norm_cta (csrc/tokenweave_artifact_kernels.cu:
 * 717-754, schema at csrc/torch_bindings.cpp:160-164). */
TW_API int tw_fused_add_rms_norm_cta(void* input, void* residual, const void* weight,
                              int64_t num_tokens, int64_t hidden_size,
                              int max_ctas, float epsilon, void* stream);

/* The fused op restricted to one GPU, general form.
 *   partials : HOST array of P device pointers, each [num_tokens, hidden_size]
 *              bf16 (this rank's row shard of every tensor-parallel partial sum)
 *   y        : [num_tokens, hidden_size] bf16 output; may alias any partials[p]
 *   residual : read and overwritten with r'
 * 1 <= P <= TW_MAX_PARTIALS.  bf16; 16-byte alignment and H % 8 == 0 required.
 * This is the body of fused_rs_ln_ag_cta_kernel
 * (csrc/tokenweave_fused_kernels.cu:106-152) with the switch-side
 * multimem.ld_reduce replaced by P loads from local HBM. */
TW_API int tw_reduce_add_rms_norm(const void* const* partials, int num_partials,
                           void* y, void* residual, const void* weight,
                           int64_t num_tokens, int64_t hidden_size,
                           int max_ctas, float epsilon, void* stream);

/* Same op with the reference's argument list.  `mcptr` is the device address
 * of this rank's row shard inside partial buffer 0; partial p lives at
 * mcptr + p * peer_stride_bytes (the one-GPU stand-in for "the same offset in
 * every peer's symmetric buffer").  y is written to `input`, which normally is
 * the shard of partial `rank` (mcptr + rank * peer_stride_bytes), as the
 * reference stores y over its own staging rows.  signal pads do not exist on
 * one GPU and are not part of this ABI.
 * Replaces ::fused_rs_ln_cta (csrc/tokenweave_artifact_kernels.cu:772-813,
 * schema at csrc/torch_bindings.cpp:166-171). */
TW_API int tw_fused_rs_ln_cta(void* input, void* residual, const void* weight,
                       uint64_t mcptr, int64_t peer_stride_bytes, int rank,
                       int world_size, int max_ctas, float epsilon,
                       int64_t num_tokens, int64_t hidden_size, void* stream);

/* Identical to tw_fused_rs_ln_cta on one GPU: the all-gather that distinguishes
 * the reference op is the store of y to the peers, and there are none.
 * Replaces ::fused_rs_ln_ag_cta (csrc/tokenweave_fused_kernels.cu:220-261,
 * schema at csrc/torch_bindings.cpp:152-157). */
TW_API int tw_fused_rs_ln_ag_cta(void* input, void* residual, const void* weight,
                          uint64_t mcptr, int64_t peer_stride_bytes, int rank,
                          int world_size, int max_ctas, float epsilon,
                          int64_t num_tokens, int64_t hidden_size,
                          void* stream);

/* Workspace of the *_ws entry points: TW_SPLIT_WORKSPACE_BYTES of device memory,
 * 256-byte aligned, all zeros before the first call that uses it.  Every call
 * leaves it ready for the next one (its arrival counters back at zero) when its
 * kernel has finished.  Calls that share a workspace must not overlap in time
 * (same stream, or ordered by events).  It holds the hand-over slots of
 * TW_SPLIT_MAX_TOKENS rows that are cut into segments. */
#define TW_SPLIT_MAX_TOKENS 256
#define TW_SPLIT_WORKSPACE_BYTES (TW_SPLIT_MAX_TOKENS * 384)

/* tw_reduce_add_rms_norm for decode-size batches.  With few token rows and many
 * compute units a row is cut into segments of whole 64-vector chunks, one
 * workgroup per segment; the segments leave their partial sums of squares in
 * `workspace`, and the workgroup that arrives last normalises the row.  Results
 * are bit-identical to tw_reduce_add_rms_norm.  The split is used when
 * max_ctas <= 0, num_tokens <= TW_SPLIT_MAX_TOKENS and tw_split_segments() says
 * more than one segment.  The workspace also serves batches of a few more rows
 * than the device has compute units (C < num_tokens <= C + C/4): one workgroup
 * per row would give some units two rows and the others one, so the first C rows
 * get a workgroup each and the excess rows are cut into quarters, a workgroup
 * each, handed over the same way (bit-identical again).  Otherwise, or
 * with workspace == NULL, the call IS tw_reduce_add_rms_norm.
 * workspace_bytes < TW_SPLIT_WORKSPACE_BYTES is an error.
 * The reference sizes its persistent grids per batch so that its kernels are not
 * starved of CTAs (grid = min(MAX_CTAS, rows), block = hidden_size / 8:
 * csrc/tokenweave_fused_kernels.cu:241-244, vllm/model_executor/models/
 * tokenweave_utils.py:86); on 256 compute units a decode batch of 1-32 rows needs
 * more than one workgroup per row to do the same. */
TW_API int tw_reduce_add_rms_norm_ws(const void* const* partials, int num_partials,
                              void* y, void* residual, const void* weight,
                              int64_t num_tokens, int64_t hidden_size,
                              int max_ctas, float epsilon, void* workspace,
                              int64_t workspace_bytes, void* stream);

/* tw_fused_rs_ln_ag_cta (= tw_fused_rs_ln_cta on one GPU) with the workspace of
 * tw_reduce_add_rms_norm_ws: the reference's argument list for decode-size
 * batches.  Replaces ::fused_rs_ln_ag_cta / ::fused_rs_ln_cta as above. */
TW_API int tw_fused_rs_ln_ag_cta_ws(void* input, void* residual, const void* weight,
                             uint64_t mcptr, int64_t peer_stride_bytes, int rank,
                             int world_size, int max_ctas, float epsilon,
                             int64_t num_tokens, int64_t hidden_size,
                             void* workspace, int64_t workspace_bytes,
                             void* stream);

/* tw_reduce_add_rms_norm_ws without a workspace argument and without any
 * allocation: the workspace is a static array in the library's device code
 * (TW_SPLIT_WORKSPACE_BYTES = 96 KiB on every GPU the library is used on, held
 * until the process ends).  No counterpart in the reference; it is for callers
 * that cannot allocate device memory — code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  num_tokens above
 * TW_SPLIT_MAX_TOKENS is refused with TW_ERR_INVALID_ARGUMENT (such batches need
 * no workspace: use tw_reduce_add_rms_norm).  The first call on a device resolves
 * the array's address (not a stream operation: make it before capturing).  All
 * calls on one GPU share the one array: calls that overlap in time on the same GPU
 * (different streams, no ordering) race; order them or use the *_ws form with a
 * workspace per stream. */
TW_API int tw_reduce_add_rms_norm_noalloc(const void* const* partials, int num_partials,
                                   void* y, void* residual, const void* weight,
                                   int64_t num_tokens, int64_t hidden_size,
                                   int max_ctas, float epsilon, void* stream);

/* Segments per row the *_ws entry points use for this shape on the current
 * device: 1 = one workgroup per row (no workspace traffic).  For a batch of a few
 * more rows than compute units it is the number of segments of each excess row. */
TW_API int tw_split_segments(int64_t num_tokens, int64_t hidden_size, int max_ctas);

/* out[M, N] = a[M, K] * b[N, K]^T, bf16 in, fp32 accumulate on MFMA, bf16 out.
 * `ldc` is the row stride of out in elements (>= N), so the result can land in
 * a row slice of a wider staging buffer.  Required: K % 8 == 0, N % 4 == 0,
 * ldc % 4 == 0, 16-byte aligned a and b, 8-byte aligned out.  max_cus > 0
 * limits the grid to that many workgroups so a concurrent kernel keeps the
 * remaining compute units.
 * Replaces UnquantizedLinearMethod.apply_inplace = torch.matmul(x, W.t(), out=)
 * (vllm/model_executor/layers/linear.py:203-228) for the row-parallel o_proj /
 * down_proj that produces one rank's partial sum. */
TW_API int tw_gemm_bf16_nt(void* out, const void* a, const void* b, int64_t M,
                    int64_t N, int64_t K, int64_t ldc, int max_cus,
                    void* stream);

/* tw_gemm_bf16_nt with the linear layer's optional bias: bias is [N] bf16 in device
 * memory (8-byte aligned) or NULL.  It is added as the reference adds it — to the
 * product already rounded to bf16, in fp32, rounded again:
 *   out = bf16_rne( f32(bf16_rne(a * b^T)) + f32(bias) )
 * (torch.matmul(x, W.t(), out=output); output += bias,
 * vllm/model_executor/layers/linear.py:224-228).  In a tensor-parallel layer only
 * rank 0 passes its bias (linear.py:1306-1308), so the P-way sum holds it once. */
TW_API int tw_gemm_bf16_nt_bias(void* out, const void* a, const void* b, const void* bias,
                         int64_t M, int64_t N, int64_t K, int64_t ldc, int max_cus,
                         void* stream);

/* The producer of the fused op's input: the P row-parallel partial sums of one
 * token split in ONE launch, outs[p][M, N] = as[p][M, K] * bs[p][N, K]^T for
 * p < num_partials, each written straight into its rank's staging rows (outs[p] =
 * slot p of the staging buffer at the split's first row, ldc = the slot's row
 * stride in elements) — the layout tw_reduce_add_rms_norm / tw_fused_rs_ln_ag_cta
 * read, with no copy in between.  outs, as, bs are HOST arrays of num_partials
 * device pointers; shapes, alignment and max_cus as for tw_gemm_bf16_nt; results are
 * bit-identical to num_partials calls of tw_gemm_bf16_nt.  Workgroups walk
 * num_partials x tiles; with eight partials every XCD computes one of them.
 * Replaces the row-parallel o_proj / down_proj writing in place into the symmetric
 * staging buffer: UnquantizedLinearMethod.apply_inplace and
 * RowParallelLinear.forward_inplace (vllm/model_executor/layers/linear.py:203-228,
 * 1310-1321), called from vllm/model_executor/models/llama.py:99-103,248-249 —
 * there one GEMM per rank, here (one GPU standing in for the ranks) all of them. */
TW_API int tw_gemm_bf16_nt_partials(void* const* outs, const void* const* as,
                             const void* const* bs, int num_partials, int64_t M,
                             int64_t N, int64_t K, int64_t ldc, int max_cus,
                             void* stream);

/* Norm with static-scale fp8 output.  out is [num_tokens, hidden_size] of OCP
 * float8 e4m3fn (1 byte per element): out = fp8_rne(clamp(y / *scale, +-448)),
 * where y is the bf16 (or `dtype`) result the unquantised op would store, and
 * `scale` points to ONE fp32 value in device memory.  input is not modified.
 * Replaces ::rms_norm_static_fp8_quant (csrc/layernorm_quant_kernels.cu:165-190,
 * schema at csrc/torch_bindings.cpp:199-205). */
TW_API int tw_rms_norm_static_fp8_quant(void* out, const void* input, const void* weight,
                                        const float* scale, int64_t num_tokens,
                                        int64_t hidden_size, float epsilon, int dtype,
                                        void* stream);

/* residual <- input + residual ; out <- fp8 quantisation (as above) of
 * RMSNorm(residual) * weight.  input is not modified.
 * Replaces ::fused_add_rms_norm_static_fp8_quant
 * (csrc/layernorm_quant_kernels.cu:203-245, schema at
 * csrc/torch_bindings.cpp:207-213). */
TW_API int tw_fused_add_rms_norm_static_fp8_quant(void* out, const void* input, void* residual,
                                                  const void* weight, const float* scale,
                                                  int64_t num_tokens, int64_t hidden_size,
                                                  float epsilon, int dtype, void* stream);

/* tw_reduce_add_rms_norm with the fp8 output above: the fused P-partial op
 * feeding an fp8 GEMM.  bf16 in; 16-byte alignment and hidden_size % 16 == 0
 * required.  No counterpart in the reference (its TokenWeave kernels emit bf16);
 * it composes the two reference ops it is named after. */
TW_API int tw_reduce_add_rms_norm_static_fp8_quant(const void* const* partials, int num_partials,
                                                   void* out, void* residual, const void* weight,
                                                   const float* scale, int64_t num_tokens,
                                                   int64_t hidden_size, int max_ctas,
                                                   float epsilon, void* stream);

/* Residual-add (optional) + RMSNorm + dynamic per-token quantisation:
 *   x = input + residual (fp32) ; residual <- x ; rms = 1/sqrt(mean(x^2) + epsilon)
 *   n = round(round(x * rms) * weight)            (both roundings to the input type)
 *   scales[t] = max(min(max_j |n[t][j]|, *scale_ub) / qmax, floor)
 *   out = fp8_e4m3fn(clamp(n / scales[t], +-448))     qmax 448, floor 1/(448 * 512)
 *       | int8(saturate(rint(n * (1 / scales[t]))))   qmax 127, floor FLT_EPSILON
 * out: [num_tokens, hidden_size] bytes; scales: num_tokens floats (device);
 * scale_ub: NULL or one device float (fp8 only); residual: NULL or
 * [num_tokens, hidden_size], updated in place.  input is not modified.  Any
 * hidden_size / alignment (vector kernel for bf16 and fp16, 16-byte aligned, hidden_size % 16 == 0).
 * Replaces ::rms_norm_dynamic_per_token_quant
 * (csrc/quantization/fused_kernels/fused_layernorm_dynamic_per_token_quant.cu:131-155,
 * schema at csrc/torch_bindings.cpp:216-221). */
TW_API int tw_rms_norm_dynamic_per_token_quant(void* out, const void* input, const void* weight,
                                               float* scales, const float* scale_ub,
                                               void* residual, int64_t num_tokens,
                                               int64_t hidden_size, float epsilon, int dtype,
                                               int out_kind, void* stream);

/* The op above over P partial buffers: x = sum_p partials[p] + residual in fp32,
 * fixed order.  bf16 in; 16-byte alignment and hidden_size % 16 == 0 required;
 * residual may be NULL.  No counterpart in the reference (its TokenWeave kernels
 * emit bf16); it fuses the reference's all-reduce + the op above. */
TW_API int tw_reduce_add_rms_norm_dynamic_per_token_quant(
    const void* const* partials, int num_partials, void* out, float* scales, void* residual,
    const void* weight, const float* scale_ub, int64_t num_tokens, int64_t hidden_size,
    int max_ctas, float epsilon, int out_kind, void* stream);

/* tw_gemm_bf16_nt_partials with a bias per product: biases is NULL or a HOST array of
 * num_partials device pointers, each [N] bf16 or NULL (one GPU standing in for the ranks
 * passes rank 0's bias in biases[0] and NULL elsewhere, linear.py:1306-1308).  Same
 * arithmetic as tw_gemm_bf16_nt_bias; bit-identical to num_partials calls of it. */
TW_API int tw_gemm_bf16_nt_partials_bias(void* const* outs, const void* const* as,
                                  const void* const* bs, const void* const* biases,
                                  int num_partials, int64_t M, int64_t N, int64_t K,
                                  int64_t ldc, int max_cus, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TOKENWEAVE_AMD_H */
