/*
 * CPU oracle for the LLM-operator hot path.
 *
 * TEST INFRASTRUCTURE ONLY. Nothing on the product path (the HIP library, the
 * host plugin layer, the Python package) links, loads or calls this file. It
 * is used by tests/, by __graft_entry__.smoke() and by the cpu_baseline leg of
 * bench.py as the checker / the timed CPU baseline.
 *
 * Every function restates, in plain C, the arithmetic of one CPU kernel of
 * InfiniTensor/RefactorGraph (paths relative to the reference tree):
 *
 *   oracle_rms_norm_*          src/04kernel/src/kernels/rms_normalization/cpu_kernel.cc:38-67
 *   oracle_softmax_*           src/04kernel/src/kernels/softmax/cpu_kernel.cc:27-60
 *                              (with the accumulator typed T instead of int; the
 *                              literal int-accumulator behaviour is kept as
 *                              oracle_softmax_literal_f32 for a regression fixture)
 *   oracle_matmul_integer      src/04kernel/src/kernels/mat_mul_integer/cpu_kernel.cc:26-149
 *                              + src/04kernel/src/kernels/mat_mul_common/cpu_template.hpp:18-30
 *   oracle_dequantize_linear   src/04kernel/src/kernels/dequantize_linear/cpu_kernel.cc:40-74
 *                              (scalar scale = the reference path; per-axis scale is this
 *                              build's extension with the same one-subtract-one-multiply form)
 *   oracle_dynamic_quantize_linear
 *                              src/04kernel/src/kernels/dynamic_quantize_linear/cpu_kernel.cc:25-70
 *                              (the running maximum starts at FLT_MIN as in the reference, so an
 *                              all-zero input gives scale FLT_MIN / 255, zero point 0, y 0)
 *   oracle_matmul_f32          src/04kernel/src/kernels/mat_mul/cpu_kernel.cc:28-68
 *                              + mat_mul_common/cpu_template.hpp:18-30 (beta == 0: y ignored)
 *   oracle_mul_f32             src/04kernel/src/kernels/simple_binary/cpu_kernel.cc:33-48,90
 *   oracle_attention_head_f32  no reference kernel exists
 *                              (src/04kernel/src/collectors/attention.cc:13-46 is a stub);
 *                              composition MatMul(transB) -> Mul(scale) -> causal mask ->
 *                              softmax -> MatMul of the functions above, on the layouts of
 *                              src/08-01llm/README.md:29-63.  PARITY UNPINNED by the reference.
 *   oracle_rope_f32            no reference item exists; closed-form rotate-half rotary
 *                              embedding.  PARITY UNPINNED by the reference.
 *   oracle_split / _concat     src/04kernel/src/kernels/{split,concat}/cpu_kernel.cc + attributes/split_info.cc
 *   oracle_expand(_info)       src/04kernel/src/kernels/expand/cpu_kernel.cc + attributes/expand_info.cc
 *   oracle_where, _broadcaster src/04kernel/src/kernels/where/cpu_kernel.cc + attributes/broadcaster.cc
 *   oracle_transpose(_info)    src/04kernel/src/attributes/transpose_info.cc:7-126
 *                              + src/04kernel/src/kernels/transpose/cpu_kernel.cc:27-37
 *
 * Pinning (see tests/test_oracle_*.py): every function is checked against the
 * known-answer vectors of the reference's own tests where they exist, and
 * against independent mathematics (float64 brute force, closed forms,
 * invariants, torch/numpy library routines) elsewhere.
 *
 * Built with -ffp-contract=off so results do not depend on FMA availability.
 */
#ifndef RG_ORACLE_H
#define RG_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ONNX element type codes, as src/00common/include/common/data_type.h:19-36 */
enum {
    ORACLE_F32 = 1,
    ORACLE_U8 = 2,
    ORACLE_I8 = 3,
    ORACLE_U16 = 4,
    ORACLE_I16 = 5,
    ORACLE_I32 = 6,
    ORACLE_F64 = 11,
};

/* y[r, :] = x[r, :] * rsqrt(mean(x[r, :]^2) + eps) * w ; sum accumulated serially in T.
 * threads <= 1 runs serially, otherwise rows are split over that many threads
 * (identical arithmetic per row). */
void oracle_rms_norm_f32(float *y, const float *x, const float *w,
                         size_t rows, size_t cols, float eps, int threads);
void oracle_rms_norm_f64(double *y, const double *x, const double *w,
                         size_t rows, size_t cols, float eps, int threads);

/* softmax along the middle axis of a [pre, mid, post] view. */
void oracle_softmax_f32(float *y, const float *x, size_t pre, size_t mid, size_t post, int threads);
void oracle_softmax_f64(double *y, const double *x, size_t pre, size_t mid, size_t post, int threads);
/* the reference's as-written behaviour: exp(x-max) / (int-truncated running sum). */
void oracle_softmax_literal_f32(float *y, const float *x, size_t pre, size_t mid, size_t post);
/* last-axis softmax over [batch, rows, cols] where row r keeps columns
 * c <= r + (cols - rows); everything else is exactly 0. */
void oracle_softmax_causal_f32(float *y, const float *x, size_t batch, size_t rows, size_t cols, int threads);

/* Zero-point handling as the reference CPU kernel:
 *   *_zp == NULL          no zero point: operand bytes are reinterpreted as int8
 *   *_zp_signed           zero-point dtype is I8 (else U8); decides how the operand byte is read
 *   *_zp_scalar           one element; otherwise A: one per (batch,row) [batch*m],
 *                         B: one per (batch, row of B) [batch*k] (as written in the reference)
 * a_off/b_off: per-output-batch operand matrix indices (NULL = identity). */
void oracle_matmul_integer(int32_t *y, const void *a, const void *b,
                           const void *a_zp, int a_zp_signed, int a_zp_scalar,
                           const void *b_zp, int b_zp_signed, int b_zp_scalar,
                           size_t batch, size_t m, size_t k, size_t n,
                           const uint32_t *a_off, const uint32_t *b_off,
                           size_t a_batch, size_t b_batch, int threads);

/* y[o, a, i] = (float)((int)x[o, a, i] - (int)zp[..]) * scale[..];
 * scale_count == 1: scalar scale/zp (reference path), else scale_count == axis_len (per-axis).
 * zp may be NULL. Returns 0, or -1 for an unsupported dtype. */
int oracle_dequantize_linear(float *y, const void *x, const float *scale, const void *zp,
                             size_t outer, size_t axis_len, size_t inner,
                             int in_dtype, size_t scale_count, int threads);

/* y = saturate(round(x / scale) + zp) with scale = (max(0, max x) - min(0, min x)) / 255 and
 * zp = saturate(0 - min x * 255 / len), all in float; outputs in operator order. */
void oracle_dynamic_quantize_linear(uint8_t *y, float *scale_out, uint8_t *zp_out,
                                    const float *x, size_t n);

/* y[M,N] = alpha * sum_k a[i*sa0 + k*sa1] * b[k*sb0 + j*sb1], serial k order, float accumulate. */
void oracle_matmul_f32(float *y, const float *a, const float *b,
                       size_t M, size_t K, size_t N,
                       size_t sa0, size_t sa1, size_t sb0, size_t sb1, float alpha);
/* mat_mul_common/cpu_template.hpp:19-31 with the bias already expanded into y (mat_mul/cpu_kernel.cc:36-37) */
void oracle_matmul_bias_f32(float *y, const float *a, const float *b, size_t M, size_t K, size_t N,
                            size_t sa0, size_t sa1, size_t sb0, size_t sb1, float alpha, float beta);
void oracle_matmul_bias_f64(double *y, const double *a, const double *b, size_t M, size_t K, size_t N,
                            size_t sa0, size_t sa1, size_t sb0, size_t sb1, double alpha, double beta);
void oracle_mul_f32(float *y, const float *a, const float *b, size_t n_a, size_t n_b);

/* One (batch row, query head) of causal attention over a KV history.
 *   q [seq, D]; kc, vc [len, D] with len = past + seq (cache rows already holding the new K/V);
 *   row r attends columns 0 .. past + r; o [seq, D]; scratch >= 2*seq*len floats.
 * causal == 0 lets every row attend all len columns. */
void oracle_attention_head_f32(float *o, const float *q, const float *kc, const float *vc,
                               size_t seq, size_t past, size_t D, float scale, int causal,
                               float *scratch);

/* Rotate-half rotary embedding on [batch, seq, heads, D] (float, already up-cast):
 *   inv_freq[i] = (float) pow(theta, -2 i / D)  (computed in double, rounded once)
 *   angle = (float)pos * inv_freq[i]            (one float multiply)
 *   c, s = (float)cos((double)angle), (float)sin((double)angle)
 *   y[i] = x[i]*c - x[i+D/2]*s ; y[i+D/2] = x[i+D/2]*c + x[i]*s   (float, unfused)
 * pos is [batch, seq] when pos_per_batch != 0, else [seq]. */
void oracle_rope_f32(float *y, const float *x, const int64_t *pos, int pos_per_batch,
                     size_t batch, size_t seq, size_t heads, size_t D, float theta, int threads);

/* Transpose (permutation of dimensions) as the reference computes it:
 * src/04kernel/src/attributes/transpose_info.cc:7-115 digests (shape, perm) — dimensions of size 1
 * dropped, dimensions that stay neighbours merged, a last dimension that stays last folded into the
 * block size — into per-output-dimension (strideI, strideO) pairs; the kernel
 * (src/04kernel/src/kernels/transpose/cpu_kernel.cc:27-37) copies, for every output block i, the
 * input block locate(i).  oracle_transpose_info returns the digest (dims <= rank pairs written to
 * stride_i/stride_o, *block_size in bytes, *block_count) and the number of pairs;
 * oracle_transpose runs the copy.  rank <= 8.  Pinned by the reference's digest vectors
 * (src/04kernel/test/attributes/test_transpose_info.cpp:7-43) and by numpy.transpose. */
int oracle_transpose_info(uint32_t *stride_i, uint32_t *stride_o, uint32_t *block_size, uint32_t *block_count,
                          const uint32_t *shape, const uint32_t *perm, int rank, uint32_t elem_size);
void oracle_transpose(void *y, const void *x, const uint32_t *shape, const uint32_t *perm, int rank,
                      uint32_t elem_size);

/* Split / Concat as the reference computes them: src/04kernel/src/attributes/split_info.cc:5-24
 * (digest) and src/04kernel/src/kernels/{split,concat}/cpu_kernel.cc:27-42 (copies).  shapes: `count`
 * rows of `rank` entries (the parts).  Pinned by the reference's vectors
 * (src/04kernel/test/attributes/test_split_info.cpp:7-30, test/kernels/{split,concat}/test_cpu.cpp)
 * and by numpy.split / numpy.concatenate. */
void oracle_split_info(uint32_t *block_count, uint32_t *sum, uint32_t *segments, const uint32_t *shapes, int count,
                       int rank, int axis, uint32_t elem_size);
void oracle_split(void *const *outputs, const void *x, const uint32_t *segments, size_t count, size_t block_count,
                  size_t sum);
void oracle_concat(void *y, const void *const *inputs, const uint32_t *segments, size_t count, size_t block_count,
                   size_t sum);

/* Expand: src/04kernel/src/attributes/expand_info.cc:14-60 (digest; returns the number of stride pairs)
 * and src/04kernel/src/kernels/expand/cpu_kernel.cc:27-46.  Pinned by
 * src/04kernel/test/attributes/test_expand_info.cpp:7-18, test/kernels/expand/test_cpu.cpp and
 * numpy.broadcast_to. */
int oracle_expand_info(uint32_t *stride_i, uint32_t *stride_o, uint32_t *block_size, uint32_t *block_count,
                       const uint32_t *input, int in_rank, const uint32_t *output, int out_rank, uint32_t elem_size);
void oracle_expand(void *y, const void *x, const uint32_t *stride_i, const uint32_t *stride_o, int dims,
                   uint32_t block_size, uint32_t block_count);

/* Broadcaster (src/04kernel/src/attributes/broadcaster.cc:17-100; shapes: rows of 8 entries, at most 8
 * inputs; returns the number of merged dimensions) and Where
 * (src/04kernel/src/kernels/where/cpu_kernel.cc:32-47; strides rows of 4).  Pinned by
 * src/04kernel/test/attributes/test_broadcaster.cpp:7-36, test/kernels/where/test_cpu.cpp and numpy.where. */
int oracle_broadcaster(uint32_t *strides, uint32_t *outputs_count, const uint32_t *shapes, const int *ranks, int inputs);
void oracle_where(void *out, const uint8_t *c, const void *x, const void *y, const uint32_t *strides, int dims,
                  uint32_t count, uint32_t elem_size);

#ifdef __cplusplus
}
#endif
#endif
