/*
 * rg_hip.h — C ABI of the gfx950 (MI355X) kernel library behind RefactorGraph's
 * 04kernel plugin surface.
 *
 * The reference links its CUDA kernels as C++ into the kernel library; here the
 * device code lives in one shared object (librg_hip.so) and the host-side
 * `Kernel::lower(Resources&)` closures are its only callers.  Each entry point
 * below names the reference interface it stands in for (paths relative to the
 * reference tree).
 *
 * Conventions
 *   - every pointer named y/x/a/b/... is a DEVICE address unless said otherwise;
 *   - `dtype` is the reference's DataType code
 *     (src/00common/include/common/data_type.h:19-36): F32=1 U8=2 I8=3 U16=4
 *     I16=5 I32=6 I64=7 Bool=9 FP16=10 F64=11 U32=12 U64=13 BF16=16;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream, which
 *     is what a Routine uses: src/03runtime/src/stream.cc:60-69);
 *   - launchers only enqueue work: no synchronisation, no allocation, no throw;
 *   - the return value is a hipError_t as int (0 = success), or one of the
 *     negative RG_HIP_E_* codes for requests the library does not handle.
 */
#ifndef RG_HIP_H
#define RG_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
    RG_F32 = 1, RG_U8 = 2, RG_I8 = 3, RG_U16 = 4, RG_I16 = 5, RG_I32 = 6, RG_I64 = 7,
    RG_BOOL = 9, RG_FP16 = 10, RG_F64 = 11, RG_U32 = 12, RG_U64 = 13, RG_BF16 = 16,
};

enum {
    RG_HIP_E_UNSUPPORTED = -1, /* dtype / shape combination has no kernel */
    RG_HIP_E_ARGUMENT = -2,    /* null pointer, zero/odd size, misaligned operand */
    RG_HIP_E_WORKSPACE = -3,   /* workspace smaller than the matching *_workspace() query */
};

/* ---- device + memory: what a hardware::Device / hardware::Memory backend needs -------------
 * replaces the CUDA runtime calls in src/02hardware/src/devices/nvidia/device.cc:17-47
 * (cudaGetDeviceCount, cudaSetDevice, cudaMemGetInfo, cudaGetDeviceProperties) and
 * src/02hardware/src/devices/nvidia/memory.cc:14-38 (cudaMalloc, cudaFree, cudaMemcpy x3);
 * rg_hip_sync stands in for kernel::cuda::sync (src/04kernel/cuda/src/functions.cu:13-15). */
int rg_hip_device_count(int *count);
int rg_hip_set_device(int card);
int rg_hip_mem_info(size_t *free_bytes, size_t *total_bytes);
int rg_hip_device_name(char *buf, size_t len);
int rg_hip_malloc(void **ptr, size_t bytes);
int rg_hip_free(void *ptr);
int rg_hip_memcpy_h2d(void *dst, const void *src, size_t bytes); /* blocking, like cudaMemcpy */
int rg_hip_memcpy_d2h(void *dst, const void *src, size_t bytes); /* blocking */
int rg_hip_memcpy_d2d(void *dst, const void *src, size_t bytes); /* blocking */
int rg_hip_memcpy_d2d_async(void *dst, const void *src, size_t bytes, void *stream);
int rg_hip_sync(void);
const char *rg_hip_error_string(int status);

/* ---- streams and captured graphs ---------------------------------------------------------
 * No counterpart in the reference, whose routines all use the default stream and are enqueued one
 * by one on every run (src/03runtime/src/stream.cc:60-69).  A stream created here (default flags
 * and priority: it stays ordered with the default stream's blocking copies) can be handed to every
 * launcher above; between rg_hip_graph_begin and rg_hip_graph_end the launches on it are recorded
 * instead of run, and the executable graph that rg_hip_graph_end returns replays them with one
 * call.  A replay uses the addresses and scalar arguments of the recording. */
int rg_hip_stream_create(void **stream);
int rg_hip_stream_destroy(void *stream);
int rg_hip_stream_sync(void *stream);
int rg_hip_graph_begin(void *stream);
int rg_hip_graph_end(void *stream, void **graph_exec);
int rg_hip_graph_launch(void *graph_exec, void *stream);
int rg_hip_graph_destroy(void *graph_exec);

/* ---- RmsNormalization --------------------------------------------------------------------
 * replaces the NVRTC kernel + launch of
 * src/04kernel/src/kernels/rms_normalization/cuda_kernel.cc:53-88,128-130;
 * arithmetic contract: src/04kernel/src/kernels/rms_normalization/cpu_kernel.cc:47-65.
 * y[r,:] = x[r,:] * rsqrt(mean(x[r,:]^2) + eps) * w.  dtype: F32, F64, FP16, BF16
 * (sums in float for FP16/BF16).  y may alias x. */
int rg_hip_rms_norm(void *y, const void *x, const void *w,
                    size_t rows, size_t cols, float eps, int dtype, void *stream);

/* RmsNormalization whose output goes on into DynamicQuantizeLinear (the head of a quantised linear layer):
 * y as rg_hip_rms_norm writes it for F32, and yq / scale / zero_point as rg_hip_dynamic_quantize_linear
 * computes them from y, bit for bit (contracts: src/04kernel/src/kernels/rms_normalization/cpu_kernel.cc:47-65
 * and src/04kernel/src/kernels/dynamic_quantize_linear/cpu_kernel.cc:25-70).  No counterpart in the reference,
 * which runs the two operators one after the other: here the normalising launch leaves the least and the
 * greatest value of every workgroup's rows in the workspace, so the quantising launch is the only one that reads
 * y (two launches instead of three; y read once instead of twice).
 * rg_hip_rms_norm_quantize_workspace returns 0 for shapes the pair is not fused for (rows that are no whole
 * 16-byte vectors, fewer than 132 or more than 8192 columns, more than 4096 workgroups): run the two
 * operators then.  Pointers 16-byte aligned. */
size_t rg_hip_rms_norm_quantize_workspace(size_t rows, size_t cols);
int rg_hip_rms_norm_quantize(uint8_t *yq, float *scale, uint8_t *zero_point, float *y, const float *x,
                             const float *w, size_t rows, size_t cols, float eps,
                             void *workspace, size_t workspace_bytes, void *stream);

/* ---- Softmax -----------------------------------------------------------------------------
 * replaces src/04kernel/src/kernels/softmax/cuda_kernel.cu:21-125 (and the cuDNN path
 * cudnn_kernel.cc:37-76); shape digest as SoftmaxInfo
 * (src/04kernel/src/attributes/softmax_info.cc:6-13): softmax along `mid` of [pre, mid, post].
 * dtype: F32, F64, FP16, BF16 (exp/sum in float for FP16/BF16).
 * causal_rows == 0: plain softmax.  causal_rows == R > 0 (requires post == 1, pre % R == 0,
 * mid >= R): rows are grouped in [R, mid] matrices and row r keeps columns
 * c <= r + (mid - R); masked inputs are not read and masked outputs are exactly 0. */
int rg_hip_softmax(void *y, const void *x, size_t pre, size_t mid, size_t post,
                   int dtype, size_t causal_rows, void *stream);

/* ---- RotaryEmbedding ---------------------------------------------------------------------
 * no counterpart exists in the reference (no rotary operator or kernel anywhere in src/);
 * rotate-half pairing (i, i + dim/2), angle = pos * theta^(-2i/dim), on x[batch, seq, heads, dim].
 * pos: int64 [batch, seq] when pos_per_batch != 0, else [seq].  dtype: FP16, BF16, F32.
 * dim even, <= 512.  y may alias x. */
int rg_hip_rope(void *y, const void *x, const int64_t *pos, int pos_per_batch,
                size_t batch, size_t seq, size_t heads, size_t dim,
                float theta, int dtype, void *stream);

/* ---- DequantizeLinear --------------------------------------------------------------------
 * replaces src/04kernel/src/kernels/dequantize_linear/cuda_kernel.cc:50-86; arithmetic
 * contract src/04kernel/src/kernels/dequantize_linear/cpu_kernel.cc:43-56:
 * y = (float)((int)x - (int)zp) * scale.  x viewed as [outer, axis_len, inner];
 * per_axis == 0: scale/zp hold one element (the reference path);
 * per_axis != 0: scale/zp hold axis_len elements.  zp may be NULL (= 0).
 * in_dtype: U8, I8, U16, I16, I32; output float. */
int rg_hip_dequantize_linear(float *y, const void *x, const float *scale, const void *zp,
                             size_t outer, size_t axis_len, size_t inner,
                             int in_dtype, int per_axis, void *stream);

/* ---- DynamicQuantizeLinear -------------------------------------------------------------
 * replaces src/04kernel/src/kernels/dynamic_quantize_linear/cuda_kernel.cu:48-136 (Thrust map +
 * cub::DeviceReduce + quantize kernel); arithmetic contract
 * src/04kernel/src/kernels/dynamic_quantize_linear/cpu_kernel.cc:25-70 (float in, uint8 out):
 * len = max(0, max x) - min(0, min x); scale = len / 255; zp = saturate(0 - min x * 255 / len);
 * y = saturate(round(x / scale) + zp).  Bit-identical to the CPU kernel, including its running
 * maximum that starts at FLT_MIN (an all-zero input gives scale FLT_MIN / 255, zp 0, y 0).
 * Outputs in operator order: y [size] uint8, scale [1] float, zero_point [1] uint8.
 * workspace: rg_hip_dynamic_quantize_linear_workspace(size) bytes, 4-byte aligned. */
size_t rg_hip_dynamic_quantize_linear_workspace(size_t size);
int rg_hip_dynamic_quantize_linear(uint8_t *y, float *scale, uint8_t *zero_point, const float *x,
                                   size_t size, void *workspace, size_t workspace_bytes, void *stream);

/* ---- Cast -------------------------------------------------------------------------------
 * replaces src/04kernel/src/kernels/cast/cuda_kernel.cc:38-124 (a kernel generated and compiled at
 * run time per type pair); arithmetic contract: for U8/U16/U32/U64/I8/I16/I32/I64/F32/F64/Bool the
 * `static_cast<U>(a)` of src/04kernel/src/kernels/cast/cpu_kernel.cc:28-40; for pairs with FP16 or
 * BF16 the expressions of cuda_kernel.cc:55-96 (to FP16/BF16: floats round to nearest even, a double
 * through float first, integers are taken as `int` and rounded toward zero; from FP16/BF16 to
 * integers: truncated as `int`), except that `-> Bool` is `x != 0` for every source type (the
 * reference's generated code tests `== 0` for floating sources).  Bool is one byte holding 0 or 1.
 * Out-of-range float -> integer conversions saturate.  from_dtype == to_dtype copies (nothing is
 * done when y == x).  y, x: `size` elements each. */
int rg_hip_cast(void *y, const void *x, size_t size, int from_dtype, int to_dtype, void *stream);

/* ---- MatMul -----------------------------------------------------------------------------
 * replaces src/04kernel/src/kernels/mat_mul/cublas_kernel.cu:9-108 (cublasGemmEx /
 * cublasGemmStridedBatchedEx after an Expand of the bias into Y); arithmetic contract
 * src/04kernel/src/kernels/mat_mul_common/cpu_template.hpp:19-31:
 * Y = alpha * op(A) @ op(B) + beta * C.  dtype F32, F64, FP16 or BF16 for all operands; a is
 * [a_batch, m, k] ([a_batch, k, m] when trans_a), b [b_batch, k, n] ([b_batch, n, k] when trans_b),
 * y [batch, m, n], row-major.  alpha and beta are converted to dtype first, like the reference;
 * sums are accumulated in float (double for F64).
 * a_index / b_index: as for rg_hip_matmul_integer (HOST arrays of `batch` matrix indices, or NULL
 * for matrix i; one B for consecutive matrices of A runs as one product of batch * m rows, groups of consecutive
 * matrices of A with one B each as one product per group).  c may be NULL (then beta is ignored); otherwise the bias element of
 * Y[batch b, row i, column j] is c[b * c_stride_batch + i * c_stride_m + j * c_stride_n] (strides
 * in elements, 0 broadcasts), which covers every bias the reference expands when its batch
 * dimensions are all 1 or equal to the output's. */
int rg_hip_matmul(void *y, const void *a, const void *b, const void *c, int dtype, int trans_a, int trans_b,
                  float alpha, float beta, size_t batch, size_t m, size_t k, size_t n,
                  const uint32_t *a_index, const uint32_t *b_index, size_t c_stride_batch,
                  size_t c_stride_m, size_t c_stride_n, void *stream);
/* The same product with a workspace, as the reference's routine receives one from its lowering
 * (src/04kernel/src/kernels/mat_mul/cublas_kernel.cu:12,38: `lower` returns a RoutineWorkspace and the routine is
 * handed `void *workspace`).  rg_hip_matmul_workspace() says how many bytes help for a shape (0: none do, and
 * rg_hip_matmul_ws then runs exactly what rg_hip_matmul runs).  With at least that many bytes (16-byte aligned,
 * contents arbitrary, nothing to clear; not to be shared by calls that may overlap), one to four rows of A
 * against FP16 / BF16 weights kept as [k, n] - a decode step on the layout ONNX MatMul stores - run with k shared
 * between workgroups that each read 512 contiguous bytes of a k-row; their float sums meet in the workspace and
 * are added in a fixed order, so results do not depend on timing.  A smaller or NULL workspace is not an error. */
size_t rg_hip_matmul_workspace(int dtype, int trans_a, int trans_b, size_t batch, size_t m, size_t k, size_t n);
int rg_hip_matmul_ws(void *y, const void *a, const void *b, const void *c, int dtype, int trans_a, int trans_b,
                     float alpha, float beta, size_t batch, size_t m, size_t k, size_t n,
                     const uint32_t *a_index, const uint32_t *b_index, size_t c_stride_batch,
                     size_t c_stride_m, size_t c_stride_n, void *workspace, size_t workspace_bytes, void *stream);

/* ---- Transpose ----------------------------------------------------------------------------
 * replaces src/04kernel/cuda/src/transpose.cu + src/04kernel/src/kernels/transpose/cuda_kernel.cu:8-30;
 * contract src/04kernel/src/kernels/transpose/cpu_kernel.cc:27-37: the output is block_count blocks
 * of block_size bytes, output block i is input block locate(i) with
 * locate (src/04kernel/src/attributes/transpose_info.cc:117-126): for d = 0 .. dims-1:
 * q = i / stride_o[d]; ans += q * stride_i[d]; i -= q * stride_o[d].
 * stride_i / stride_o: HOST arrays [dims] (TransposeInfo::dims), dims <= 8; y != x.  Tensors of up
 * to 2^32 - 1 blocks and words (16 bytes, or the widest power of two that divides block_size and
 * both addresses). */
int rg_hip_transpose(void *y, const void *x, const uint32_t *stride_i, const uint32_t *stride_o,
                     size_t dims, size_t block_size, size_t block_count, void *stream);

/* ---- Split / Concat ----------------------------------------------------------------------
 * replace src/04kernel/cuda/src/split.cu:7-50 and concat.cu:7-50 (+ the launchers in
 * src/04kernel/src/kernels/{split,concat}/cuda_kernel.cc); contract
 * src/04kernel/src/kernels/{split,concat}/cpu_kernel.cc with SplitInfo
 * (src/04kernel/src/attributes/split_info.cc:5-30): the joined tensor is block_count blocks of `sum`
 * bytes, block i being the segments of the `count` parts one after the other; part j holds
 * block_count segments of segments[j] bytes.  outputs / inputs and segments: HOST arrays [count]
 * (device pointers, bytes); the segments add up to `sum`. */
int rg_hip_split(void *const *outputs, const void *x, const uint32_t *segments, size_t count,
                 size_t block_count, size_t sum, void *stream);
int rg_hip_concat(void *y, const void *const *inputs, const uint32_t *segments, size_t count,
                  size_t block_count, size_t sum, void *stream);

/* ---- Expand ------------------------------------------------------------------------------
 * replaces src/04kernel/cuda/src/expand.cu:1-56 + src/04kernel/src/kernels/expand/cuda_kernel.cu:9-26;
 * contract src/04kernel/src/kernels/expand/cpu_kernel.cc:27-46 with ExpandInfo
 * (src/04kernel/src/attributes/expand_info.cc:14-60): output block i (block_size bytes) is input
 * block j, where for d = 0 .. dims-1: j += (rem / stride_o[d]) * stride_i[d]; rem %= stride_o[d]
 * (stride_i[d] == 0 where the input is broadcast).  stride_i / stride_o: HOST arrays [dims],
 * dims <= 8; dims == 0 copies.  y != x. */
int rg_hip_expand(void *y, const void *x, const uint32_t *stride_i, const uint32_t *stride_o,
                  size_t dims, size_t block_size, size_t block_count, void *stream);

/* ---- Where -------------------------------------------------------------------------------
 * replaces src/04kernel/cuda/src/where.cu:1-62 + src/04kernel/src/kernels/where/where_cuda.cu;
 * contract src/04kernel/src/kernels/where/cpu_kernel.cc:32-47: output element i (element_size
 * bytes: 1, 2, 4 or 8) is x[at1] where condition[at0] != 0 (one byte per element), else y[at2],
 * with (at0, at1, at2) = Broadcaster::locate(i) (src/04kernel/src/attributes/broadcaster.cc:87-100).
 * strides: HOST array [dims][4] = per merged dimension the strides of condition, x, y and of the
 * output (Broadcaster::strides as it stands); dims == 0: nothing is broadcast, at = (i, i, i). */
int rg_hip_where(void *out, const void *condition, const void *x, const void *y, const uint32_t *strides,
                 size_t dims, size_t outputs_count, size_t element_size, void *stream);

/* ---- MatMulInteger -----------------------------------------------------------------------
 * replaces src/04kernel/src/kernels/mat_mul_integer/cublas_kernel.cu:87-184 (Thrust
 * zero-point pre-pass + cublasGemmEx); arithmetic contract
 * src/04kernel/src/kernels/mat_mul_integer/cpu_kernel.cc:26-146:
 * Y[i,j] = sum_k int8(A[i,k] - a_zp) * int8(B[k,j] - b_zp), differences taken modulo 256.
 * a [a_batch, m, k], b [b_batch, k, n] bytes (row-major), y int32 [batch, m, n].
 * a_zp / b_zp: NULL, or device pointers to one byte (RG_MMI_*_ZP_SCALAR) or to one byte per
 * (batch, row) of the operand, as the reference's CPU kernel reads them.
 * a_index / b_index: HOST arrays [batch] giving the operand matrix used by each output batch
 * (the Broadcaster's locate(), src/04kernel/src/attributes/broadcaster.cc:87-100); NULL = i.
 * The zero points are fused into the tile loads: no workspace is needed and
 * rg_hip_matmul_integer_workspace() returns 0 (the reference needs m*k [+ k*n] bytes).
 * Integer sums are exact in any order, so every path (matrix cores on 256 x 256 tiles, with k split
 * between workgroups when the tiles are few, also for 65 to 255 rows; weight streaming for up to 64
 * rows; vector-ALU dot products for one to four rows; 128 x 128 tiles for other shapes with k a
 * multiple of 16) returns the same bits. */
enum {
    RG_MMI_A_ZP_SCALAR = 1u,
    RG_MMI_B_ZP_SCALAR = 2u,
};
size_t rg_hip_matmul_integer_workspace(size_t batch, size_t m, size_t k, size_t n, unsigned flags);
int rg_hip_matmul_integer(int32_t *y, const void *a, const void *b,
                          const void *a_zp, const void *b_zp, unsigned flags,
                          size_t batch, size_t m, size_t k, size_t n,
                          const uint32_t *a_index, const uint32_t *b_index,
                          void *workspace, void *stream);
/* MatMulInteger with DequantizeLinear folded into its epilogue: y[b,i,j] = float(sum) * scale[j or 0],
 * i.e. the result of rg_hip_matmul_integer followed by the reference's DequantizeLinear without zero
 * point (src/04kernel/src/kernels/dequantize_linear/cpu_kernel.cc:17-28: one int -> float
 * conversion, one multiplication) on the last axis, bit for bit, without the int32 tensor ever
 * reaching memory (with fewer than 256 rows, or few output tiles, partial sums of ranges of k meet in
 * y itself as int32 and a finishing launch converts them in place: y is the only memory used).
 * No counterpart in the reference, which runs the two operators one after the other.
 * scale: device pointer to one float, or to n floats when scale_per_column != 0. */
int rg_hip_matmul_integer_dequantize(float *y, const void *a, const void *b, const void *a_zp,
                                     const void *b_zp, unsigned flags, size_t batch, size_t m,
                                     size_t k, size_t n, const uint32_t *a_index,
                                     const uint32_t *b_index, const float *scale, int scale_per_column,
                                     void *workspace, void *stream);

/* ---- Attention with KV cache ---------------------------------------------------------------
 * the reference declares this kernel but never defines it
 * (src/04kernel/src/kernels/attention/cuda_kernel.hh:10-25); the parameter block follows
 * AttentionCuda::info and the tensor layouts follow src/08-01llm/README.md:29-63:
 *   q, o [N, n_head, seq, D]; k, v [N, n_kv_head, seq, D]; caches [N, n_kv_head, cap, D].
 * For batch row b with past = past_lens[past_per_row ? b : 0] (int64, read on the device):
 *   the new k/v rows are written to cache[b, :, past .. past+seq), then query row r attends
 *   cache positions 0 .. past + r with scores scaled by `scale` (causal decoder mask);
 *   cache rows >= past + seq are left untouched.  The lengths live on the device, so the host
 *   cannot refuse them: a negative past counts as 0 and a past above cap - seq is moved back to
 *   cap - seq (the new rows then replace the last seq rows of the cache and the queries see the
 *   history shortened accordingly); nothing is ever read or written outside the caches.
 * k_cache == v_cache == NULL: no cache (past = 0, attends k/v directly).  past_lens == NULL: 0.
 * n_head % n_kv_head == 0; D in {64, 80, 96, 128}; dtype FP16 or BF16; fp32 softmax / accumulation.
 * workspace: rg_hip_attention_kvcache_workspace() bytes (partial results of key ranges, of either
 *   kernel: up to 35 MiB at D = 128), contents irrelevant.
 * sync_state: NULL, or rg_hip_attention_kvcache_state_bytes() bytes of device memory that the
 *   caller zeroed once and keeps for this purpose (a runtime::Resource of the stream, like the
 *   reference's library handles, src/04kernel/src/utilities/cuda/cublas_context.cu:18-31); the
 *   kernel uses it for ticket counters and leaves it zero.  With it the whole call is one
 *   kernel launch; without it a small clearing launch precedes the kernel.  Calls that share
 *   one sync_state must not overlap (a Stream runs its routines in order on one queue). */
size_t rg_hip_attention_kvcache_workspace(size_t N, size_t n_head, size_t n_kv_head,
                                          size_t seq, size_t cap, size_t D);
size_t rg_hip_attention_kvcache_state_bytes(void);
int rg_hip_attention_kvcache(void *o, const void *q, const void *k, const void *v,
                             void *k_cache, void *v_cache,
                             const int64_t *past_lens, int past_per_row,
                             size_t N, size_t n_head, size_t n_kv_head,
                             size_t seq, size_t cap, size_t D,
                             float scale, int dtype,
                             void *workspace, size_t workspace_bytes, void *sync_state,
                             void *stream);

/* The same operation for callers that cannot allocate device memory or hand over a workspace:
 * code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  No
 * counterpart in the reference (every reference kernel gets its workspace from the stack that
 * kernel::Graph::lower allocates).  The split-KV partials and ticket counters live in a fixed
 * array of rg_hip_attention_kvcache_static_scratch_bytes() bytes (2 KiB + 2.03 MiB) inside the
 * library's device image, one copy per GPU, held until the process ends; the call allocates
 * nothing and frees nothing, and the counters are cleared by a small fill kernel at the start of
 * every call (not a memset, so the call can be captured).  Limits: those of
 * rg_hip_attention_kvcache (D in {64, 80, 96, 128}, the head dims 80 and 96 on the tiled kernel only
 * and without key ranges shared between workgroups; a larger D is refused with RG_HIP_E_WORKSPACE, the
 * partial slots being sized for D <= 128); the launch uses at most 512 workgroups, which is what
 * the array holds partials for (the tiled kernel shares an item's keys between workgroups only
 * as far as 2 MiB of records reach).  All calls on one GPU share the array: calls that overlap on one
 * GPU (two streams, two threads) race and must be serialised by the caller.  Same kernels as
 * rg_hip_attention_kvcache: the caches come out bit-identical, the output within the rounding of
 * the summation order (which work a wavefront pulls is decided at run time in either entry). */
size_t rg_hip_attention_kvcache_static_scratch_bytes(void);
int rg_hip_attention_kvcache_static(void *o, const void *q, const void *k, const void *v,
                                    void *k_cache, void *v_cache,
                                    const int64_t *past_lens, int past_per_row,
                                    size_t N, size_t n_head, size_t n_kv_head,
                                    size_t seq, size_t cap, size_t D,
                                    float scale, int dtype, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* RG_HIP_H */
