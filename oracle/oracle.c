/*
 * CPU oracle (test infrastructure, never on the product path): see oracle.h for
 * the reference file:line each function follows and for what pins it.
 */
#include "oracle.h"

#include <float.h>
#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ threads */

typedef void (*range_fn)(size_t begin, size_t end, void *ctx);

struct span_job {
    range_fn fn;
    void *ctx;
    size_t begin, end;
};

static void *span_entry(void *p) {
    struct span_job *j = (struct span_job *) p;
    j->fn(j->begin, j->end, j->ctx);
    return NULL;
}

/* Split [0, n) into contiguous spans, one per thread. The arithmetic done for
 * an index never depends on the split. */
static void for_spans(size_t n, int threads, range_fn fn, void *ctx) {
    if (threads <= 1 || n < 2) {
        fn(0, n, ctx);
        return;
    }
    if ((size_t) threads > n) threads = (int) n;
    pthread_t *tid = (pthread_t *) malloc(sizeof(pthread_t) * (size_t) threads);
    struct span_job *jobs = (struct span_job *) malloc(sizeof(struct span_job) * (size_t) threads);
    size_t chunk = (n + (size_t) threads - 1) / (size_t) threads;
    int started = 0;
    for (int t = 0; t < threads; ++t) {
        size_t b = (size_t) t * chunk, e = b + chunk > n ? n : b + chunk;
        if (b >= e) break;
        jobs[t].fn = fn;
        jobs[t].ctx = ctx;
        jobs[t].begin = b;
        jobs[t].end = e;
        if (pthread_create(&tid[t], NULL, span_entry, &jobs[t]) != 0) {
            fn(b, e, ctx);
            tid[t] = 0;
            jobs[t].fn = NULL;
        }
        started = t + 1;
    }
    for (int t = 0; t < started; ++t)
        if (jobs[t].fn) pthread_join(tid[t], NULL);
    free(jobs);
    free(tid);
}

/* ----------------------------------------------------------------- rms norm */

struct rms_ctx {
    void *y;
    const void *x, *w;
    size_t cols;
    float eps;
};

static void rms_rows_f32(size_t r0, size_t r1, void *p) {
    struct rms_ctx *c = (struct rms_ctx *) p;
    const float *w = (const float *) c->w;
    for (size_t r = r0; r < r1; ++r) {
        const float *x = (const float *) c->x + r * c->cols;
        float *y = (float *) c->y + r * c->cols;
        float ss = 0.0f;
        for (size_t j = 0; j < c->cols; ++j) ss = ss + x[j] * x[j];
        ss = ss / (float) c->cols;
        ss = ss + c->eps;
        /* double division of 1 by the float square root, rounded back to float */
        ss = (float) (1.0 / (double) sqrtf(ss));
        for (size_t j = 0; j < c->cols; ++j) y[j] = x[j] * ss * w[j];
    }
}

static void rms_rows_f64(size_t r0, size_t r1, void *p) {
    struct rms_ctx *c = (struct rms_ctx *) p;
    const double *w = (const double *) c->w;
    for (size_t r = r0; r < r1; ++r) {
        const double *x = (const double *) c->x + r * c->cols;
        double *y = (double *) c->y + r * c->cols;
        double ss = 0.0;
        for (size_t j = 0; j < c->cols; ++j) ss = ss + x[j] * x[j];
        ss = ss / (double) c->cols;
        ss = ss + (double) c->eps;
        ss = 1.0 / sqrt(ss);
        for (size_t j = 0; j < c->cols; ++j) y[j] = x[j] * ss * w[j];
    }
}

void oracle_rms_norm_f32(float *y, const float *x, const float *w,
                         size_t rows, size_t cols, float eps, int threads) {
    struct rms_ctx c = {y, x, w, cols, eps};
    for_spans(rows, threads, rms_rows_f32, &c);
}

void oracle_rms_norm_f64(double *y, const double *x, const double *w,
                         size_t rows, size_t cols, float eps, int threads) {
    struct rms_ctx c = {y, x, w, cols, eps};
    for_spans(rows, threads, rms_rows_f64, &c);
}

/* ------------------------------------------------------------------ softmax */

struct softmax_ctx {
    void *y;
    const void *x;
    size_t mid, post;
    size_t rows, cols; /* causal form */
};

/* slice i of pre*post: first element at (i - i%post)*mid + i%post, step post */
#define SOFTMAX_BODY(T, EXP)                                                   \
    struct softmax_ctx *c = (struct softmax_ctx *) p;                          \
    const T *x = (const T *) c->x;                                             \
    T *y = (T *) c->y;                                                         \
    size_t mid = c->mid, post = c->post;                                       \
    for (size_t i = i0; i < i1; ++i) {                                         \
        size_t base = (i - i % post) * mid + i % post;                         \
        size_t arg = 0;                                                        \
        for (size_t j = 1; j < mid; ++j)                                       \
            if (x[base + arg * post] < x[base + j * post]) arg = j;            \
        T mx = x[base + arg * post];                                           \
        T sum = 0;                                                             \
        for (size_t j = 0; j < mid; ++j) {                                     \
            T e = EXP(x[base + j * post] - mx);                                \
            y[base + j * post] = e;                                            \
            sum = sum + e;                                                     \
        }                                                                      \
        for (size_t j = 0; j < mid; ++j) y[base + j * post] = y[base + j * post] / sum; \
    }

static void softmax_slices_f32(size_t i0, size_t i1, void *p) { SOFTMAX_BODY(float, expf) }
static void softmax_slices_f64(size_t i0, size_t i1, void *p) { SOFTMAX_BODY(double, exp) }

void oracle_softmax_f32(float *y, const float *x, size_t pre, size_t mid, size_t post, int threads) {
    struct softmax_ctx c = {y, x, mid, post, 0, 0};
    for_spans(pre * post, threads, softmax_slices_f32, &c);
}

void oracle_softmax_f64(double *y, const double *x, size_t pre, size_t mid, size_t post, int threads) {
    struct softmax_ctx c = {y, x, mid, post, 0, 0};
    for_spans(pre * post, threads, softmax_slices_f64, &c);
}

void oracle_softmax_literal_f32(float *y, const float *x, size_t pre, size_t mid, size_t post) {
    for (size_t i = 0; i < pre * post; ++i) {
        size_t base = (i - i % post) * mid + i % post;
        size_t arg = 0;
        for (size_t j = 1; j < mid; ++j)
            if (x[base + arg * post] < x[base + j * post]) arg = j;
        float mx = x[base + arg * post];
        int sum = 0; /* the reference's accumulator type: every addend < 1 is truncated away */
        for (size_t j = 0; j < mid; ++j) {
            float e = expf(x[base + j * post] - mx);
            y[base + j * post] = e;
            sum = (int) ((float) sum + e);
        }
        for (size_t j = 0; j < mid; ++j) y[base + j * post] = y[base + j * post] / (float) sum;
    }
}

static void softmax_causal_rows_f32(size_t i0, size_t i1, void *p) {
    struct softmax_ctx *c = (struct softmax_ctx *) p;
    size_t rows = c->rows, cols = c->cols;
    for (size_t i = i0; i < i1; ++i) {
        const float *x = (const float *) c->x + i * cols;
        float *y = (float *) c->y + i * cols;
        size_t r = i % rows;
        size_t keep = r + (cols - rows) + 1; /* columns 0 .. r + (cols - rows) */
        if (keep > cols) keep = cols;
        float mx = x[0];
        for (size_t j = 1; j < keep; ++j)
            if (mx < x[j]) mx = x[j];
        float sum = 0.0f;
        for (size_t j = 0; j < keep; ++j) {
            float e = expf(x[j] - mx);
            y[j] = e;
            sum = sum + e;
        }
        for (size_t j = 0; j < keep; ++j) y[j] = y[j] / sum;
        for (size_t j = keep; j < cols; ++j) y[j] = 0.0f;
    }
}

void oracle_softmax_causal_f32(float *y, const float *x, size_t batch, size_t rows, size_t cols, int threads) {
    struct softmax_ctx c = {y, x, 0, 0, rows, cols};
    for_spans(batch * rows, threads, softmax_causal_rows_f32, &c);
}

/* ----------------------------------------------------------- matmul integer */

/* the reference's subtraction: int8 - int8 wraps to int8; uint8 - uint8 goes
 * through int16 and is truncated to int8. Both are "difference modulo 256". */
static int8_t zp_sub(int is_signed, uint8_t v, uint8_t z) {
    if (is_signed) return (int8_t) ((int) (int8_t) v - (int) (int8_t) z);
    return (int8_t) (int16_t) ((int16_t) v - (int16_t) z);
}

struct mmi_ctx {
    int32_t *y;
    const int8_t *a, *b;
    size_t m, k, n;
};

static void mmi_rows(size_t i0, size_t i1, void *p) {
    struct mmi_ctx *c = (struct mmi_ctx *) p;
    size_t k = c->k, n = c->n;
    for (size_t i = i0; i < i1; ++i)
        for (size_t j = 0; j < n; ++j) {
            int32_t sum = 0;
            for (size_t q = 0; q < k; ++q)
                sum += (int32_t) ((int) c->a[i * k + q] * (int) c->b[q * n + j]);
            c->y[i * n + j] = sum;
        }
}

void oracle_matmul_integer(int32_t *y, const void *a_, const void *b_,
                           const void *a_zp_, int a_zp_signed, int a_zp_scalar,
                           const void *b_zp_, int b_zp_signed, int b_zp_scalar,
                           size_t batch, size_t m, size_t k, size_t n,
                           const uint32_t *a_off, const uint32_t *b_off,
                           size_t a_batch, size_t b_batch, int threads) {
    const uint8_t *a = (const uint8_t *) a_, *b = (const uint8_t *) b_;
    const uint8_t *a_zp = (const uint8_t *) a_zp_, *b_zp = (const uint8_t *) b_zp_;
    int8_t *aw = NULL, *bw = NULL; /* the reference's workspace: zero-point-adjusted copies */
    if (a_zp) {
        aw = (int8_t *) malloc(a_batch * m * k + 1);
        for (size_t i = 0; i < a_batch; ++i)
            for (size_t r = 0; r < m; ++r)
                for (size_t q = 0; q < k; ++q) {
                    uint8_t z = a_zp_scalar ? a_zp[0] : a_zp[i * m + r];
                    aw[(i * m + r) * k + q] = zp_sub(a_zp_signed, a[(i * m + r) * k + q], z);
                }
    }
    if (b_zp) {
        bw = (int8_t *) malloc(b_batch * k * n + 1);
        for (size_t i = 0; i < b_batch; ++i)
            for (size_t r = 0; r < k; ++r)
                for (size_t q = 0; q < n; ++q) {
                    /* as written in the reference: one zero point per ROW of B */
                    uint8_t z = b_zp_scalar ? b_zp[0] : b_zp[i * k + r];
                    bw[(i * k + r) * n + q] = zp_sub(b_zp_signed, b[(i * k + r) * n + q], z);
                }
    }
    const int8_t *as = aw ? aw : (const int8_t *) a;
    const int8_t *bs = bw ? bw : (const int8_t *) b;
    for (size_t i = 0; i < batch; ++i) {
        size_t ia = a_off ? a_off[i] : i, ib = b_off ? b_off[i] : i;
        struct mmi_ctx c = {y + i * m * n, as + ia * m * k, bs + ib * k * n, m, k, n};
        for_spans(m, threads, mmi_rows, &c);
    }
    free(aw);
    free(bw);
}

/* -------------------------------------------------------- dequantize linear */

struct dq_ctx {
    float *y;
    const void *x, *zp;
    const float *scale;
    size_t axis_len, inner, scale_count;
    int dtype;
};

#define DQ_LOOP(TI)                                                            \
    {                                                                          \
        const TI *x = (const TI *) c->x;                                       \
        const TI *zp = (const TI *) c->zp;                                     \
        for (size_t e = e0; e < e1; ++e) {                                     \
            size_t a = c->scale_count == 1 ? 0 : (e / c->inner) % c->axis_len; \
            float s = c->scale[a];                                             \
            /* the zero constant of the reference is an int when absent */     \
            if (zp) c->y[e] = (float) (x[e] - zp[a]) * s;                      \
            else c->y[e] = (float) (x[e] - 0) * s;                             \
        }                                                                      \
    }

static void dq_span(size_t e0, size_t e1, void *p) {
    struct dq_ctx *c = (struct dq_ctx *) p;
    switch (c->dtype) {
        case ORACLE_U8: DQ_LOOP(uint8_t) break;
        case ORACLE_I8: DQ_LOOP(int8_t) break;
        case ORACLE_U16: DQ_LOOP(uint16_t) break;
        case ORACLE_I16: DQ_LOOP(int16_t) break;
        case ORACLE_I32: DQ_LOOP(int32_t) break;
        default: break;
    }
}

int oracle_dequantize_linear(float *y, const void *x, const float *scale, const void *zp,
                             size_t outer, size_t axis_len, size_t inner,
                             int in_dtype, size_t scale_count, int threads) {
    switch (in_dtype) {
        case ORACLE_U8: case ORACLE_I8: case ORACLE_U16: case ORACLE_I16: case ORACLE_I32: break;
        default: return -1;
    }
    if (scale_count != 1 && scale_count != axis_len) return -1;
    struct dq_ctx c = {y, x, zp, scale, axis_len, inner, scale_count, in_dtype};
    for_spans(outer * axis_len * inner, threads, dq_span, &c);
    return 0;
}

/* ------------------------------------------------------- dynamic quantize linear */

/* saturate<uint8_t>: src/04kernel/src/kernels/dynamic_quantize_linear/cpu_kernel.cc:25-31 */
static uint8_t dql_saturate(float v) {
    v = v < 0.0f ? 0.0f : v;       /* std::clamp(x, QMIN, QMAX) */
    v = 255.0f < v ? 255.0f : v;
    return (uint8_t) roundf(v);    /* std::round: half away from zero */
}

void oracle_dynamic_quantize_linear(uint8_t *y, float *scale_out, uint8_t *zp_out,
                                    const float *x, size_t n) {
    /* cpu_kernel.cc:38-57: the accumulation starts from {max float, min positive float} */
    float mn = FLT_MAX, mx = FLT_MIN;
    for (size_t i = 0; i < n; ++i) {
        mn = x[i] < mn ? x[i] : mn;   /* std::min(min, it) */
        mx = mx < x[i] ? x[i] : mx;   /* std::max(max, it) */
    }
    /* cpu_kernel.cc:58-60 */
    const float len = (0.0f < mx ? mx : 0.0f) - (mn < 0.0f ? mn : 0.0f);
    const float scale = len / 255.0f;
    *scale_out = scale;
    if (!(len > 0.0f)) { /* cannot happen for finite input (mx >= FLT_MIN); NaN-only input */
        *zp_out = 0;
        memset(y, 0, n);
        return;
    }
    const uint8_t zp = dql_saturate(0.0f - mn * 255.0f / len);
    *zp_out = zp;
    /* cpu_kernel.cc:62-66 */
    for (size_t i = 0; i < n; ++i) y[i] = dql_saturate(roundf(x[i] / scale) + (float) zp);
}

/* ------------------------------------------------------- float matmul + mul */

void oracle_matmul_f32(float *y, const float *a, const float *b,
                       size_t M, size_t K, size_t N,
                       size_t sa0, size_t sa1, size_t sb0, size_t sb1, float alpha) {
    for (size_t i = 0; i < M; ++i)
        for (size_t j = 0; j < N; ++j) {
            float sum = 0.0f;
            for (size_t q = 0; q < K; ++q) sum += a[i * sa0 + q * sa1] * b[q * sb0 + j * sb1];
            y[i * N + j] = alpha * sum; /* beta == 0: the stale y is not read */
        }
}

/* MatMul with bias: src/04kernel/src/kernels/mat_mul_common/cpu_template.hpp:19-31, T = float or
 * double.  y holds the expanded bias on entry (mat_mul/cpu_kernel.cc:36-37 expands C into Y first);
 * beta must be 0 when there is no bias (cpu_kernel.cc:48). */
void oracle_matmul_bias_f32(float *y, const float *a, const float *b,
                            size_t M, size_t K, size_t N,
                            size_t sa0, size_t sa1, size_t sb0, size_t sb1, float alpha, float beta) {
    for (size_t i = 0; i < M; ++i)
        for (size_t j = 0; j < N; ++j) {
            float sum = 0.0f;
            for (size_t q = 0; q < K; ++q) sum += a[i * sa0 + q * sa1] * b[q * sb0 + j * sb1];
            y[i * N + j] = beta * y[i * N + j] + alpha * sum;
        }
}

void oracle_matmul_bias_f64(double *y, const double *a, const double *b,
                            size_t M, size_t K, size_t N,
                            size_t sa0, size_t sa1, size_t sb0, size_t sb1, double alpha, double beta) {
    for (size_t i = 0; i < M; ++i)
        for (size_t j = 0; j < N; ++j) {
            double sum = 0.0;
            for (size_t q = 0; q < K; ++q) sum += a[i * sa0 + q * sa1] * b[q * sb0 + j * sb1];
            y[i * N + j] = beta * y[i * N + j] + alpha * sum;
        }
}

void oracle_mul_f32(float *y, const float *a, const float *b, size_t n_a, size_t n_b) {
    size_t n = n_a > n_b ? n_a : n_b;
    for (size_t i = 0; i < n; ++i) y[i] = a[n_a == 1 ? 0 : i] * b[n_b == 1 ? 0 : i];
}

/* ---------------------------------------------------------------- attention */

void oracle_attention_head_f32(float *o, const float *q, const float *kc, const float *vc,
                               size_t seq, size_t past, size_t D, float scale, int causal,
                               float *scratch) {
    size_t len = past + seq;
    float *s = scratch, *pbuf = scratch + seq * len;
    /* S = Q K^T (transB), then the "scale" kernel */
    oracle_matmul_f32(s, q, kc, seq, D, len, D, 1, 1, D, 1.0f);
    oracle_mul_f32(s, s, &scale, seq * len, 1);
    if (causal)
        for (size_t r = 0; r < seq; ++r)
            for (size_t cidx = past + r + 1; cidx < len; ++cidx) s[r * len + cidx] = -INFINITY;
    oracle_softmax_f32(pbuf, s, seq, len, 1, 1);
    /* O = P V */
    oracle_matmul_f32(o, pbuf, vc, seq, len, D, len, 1, D, 1, 1.0f);
}

/* --------------------------------------------------------------------- rope */

struct rope_ctx {
    float *y;
    const float *x;
    const int64_t *pos;
    const float *inv_freq;
    int pos_per_batch;
    size_t seq, heads, D;
};

static void rope_tokens(size_t t0, size_t t1, void *p) {
    struct rope_ctx *c = (struct rope_ctx *) p;
    size_t half = c->D / 2;
    for (size_t t = t0; t < t1; ++t) {
        size_t s = t % c->seq;
        int64_t position = c->pos_per_batch ? c->pos[t] : c->pos[s];
        for (size_t i = 0; i < half; ++i) {
            float angle = (float) position * c->inv_freq[i];
            float cs = (float) cos((double) angle), sn = (float) sin((double) angle);
            for (size_t h = 0; h < c->heads; ++h) {
                const float *x = c->x + (t * c->heads + h) * c->D;
                float *y = c->y + (t * c->heads + h) * c->D;
                float lo = x[i], hi = x[i + half];
                y[i] = lo * cs - hi * sn;
                y[i + half] = hi * cs + lo * sn;
            }
        }
    }
}

void oracle_rope_f32(float *y, const float *x, const int64_t *pos, int pos_per_batch,
                     size_t batch, size_t seq, size_t heads, size_t D, float theta, int threads) {
    size_t half = D / 2;
    float *inv_freq = (float *) malloc(sizeof(float) * (half ? half : 1));
    for (size_t i = 0; i < half; ++i)
        inv_freq[i] = (float) pow((double) theta, -2.0 * (double) i / (double) D);
    struct rope_ctx c = {y, x, pos, inv_freq, pos_per_batch, seq, heads, D};
    for_spans(batch * seq, threads, rope_tokens, &c);
    free(inv_freq);
}

/* ------------------------------------------------------- transpose */

int oracle_transpose_info(uint32_t *stride_i, uint32_t *stride_o, uint32_t *block_size, uint32_t *block_count,
                          const uint32_t *shape_, const uint32_t *perm_, int rank, uint32_t elem_size) {
    uint32_t shape[8], perm[8];
    int map[8];
    uint32_t count = 1;
    for (int i = 0; i < rank; ++i) count *= shape_[i];
    *block_size = elem_size;
    *block_count = count;
    /* transpose_info.cc:19-40: dimensions of size 1 go */
    int r = 0;
    for (int i = 0; i < rank; ++i) {
        if (shape_[i] != 1) { map[i] = r; shape[r++] = shape_[i]; } else map[i] = -1;
    }
    int p = 0;
    for (int i = 0; i < rank; ++i)
        if (map[perm_[i]] >= 0) perm[p++] = (uint32_t) map[perm_[i]];
    rank = r;
    if (rank <= 1) goto whole;
    /* transpose_info.cc:47-79: input dimensions that stay neighbours in the output become one */
    {
        int keep[8];
        for (int i = 0; i < rank; ++i) keep[i] = 1;
        for (int i = 1; i < rank; ++i)
            if (perm[i] == perm[i - 1] + 1) keep[perm[i]] = 0;
        int to[8], j = -1;
        for (int i = 0; i < rank; ++i) {
            if (keep[i] || i == 0) { shape[++j] = shape[i]; to[i] = j; keep[i] = 1; }
            else { shape[j] *= shape[i]; to[i] = -1; }
        }
        int q = 0;
        for (int i = 0; i < rank; ++i)
            if (to[perm[i]] >= 0 && keep[perm[i]]) perm[q++] = (uint32_t) to[perm[i]];
        rank = j + 1;
    }
    if (rank <= 1) goto whole;
    /* transpose_info.cc:87-93: a last dimension that stays last is part of the block */
    if (perm[rank - 1] == (uint32_t) (rank - 1)) {
        *block_size *= shape[rank - 1];
        *block_count /= shape[rank - 1];
        --rank;
    }
    /* transpose_info.cc:94-112: strides of the input, taken in output order, and of the output */
    {
        uint32_t in_stride[8];
        in_stride[rank - 1] = 1;
        for (int i = rank - 1; i > 0; --i) in_stride[i - 1] = in_stride[i] * shape[i];
        stride_o[rank - 1] = 1;
        for (int i = rank - 1; i > 0; --i) stride_o[i - 1] = stride_o[i] * shape[perm[i]];
        for (int i = 0; i < rank; ++i) stride_i[i] = in_stride[perm[i]];
    }
    return rank;
whole:
    stride_i[0] = stride_o[0] = 1;
    *block_size *= *block_count;
    *block_count = 1;
    return 1;
}

void oracle_transpose(void *y, const void *x, const uint32_t *shape, const uint32_t *perm, int rank,
                      uint32_t elem_size) {
    uint32_t si[8], so[8], block, count;
    const int dims = oracle_transpose_info(si, so, &block, &count, shape, perm, rank, elem_size);
    for (uint32_t i = 0; i < count; ++i) {
        /* transpose_info.cc:117-126 (locate) */
        uint32_t from = 0, rem = i;
        for (int d = 0; d < dims; ++d) {
            from += rem / so[d] * si[d];
            rem %= so[d];
        }
        memcpy((uint8_t *) y + (size_t) i * block, (const uint8_t *) x + (size_t) from * block, block);
    }
}


/* ------------------------------------------------------- split / concat */

/* split_info.cc:5-24: blockCount = product of the dimensions before the axis, segment j = shape_j[axis] times
 * the bytes behind the axis, sum = their total.  shapes: count rows of `rank` entries. */
void oracle_split_info(uint32_t *block_count, uint32_t *sum, uint32_t *segments, const uint32_t *shapes, int count,
                       int rank, int axis, uint32_t elem_size) {
    uint32_t blocks = 1, postfix = elem_size, total = 0;
    for (int d = 0; d < axis; ++d) blocks *= shapes[d];
    for (int d = axis + 1; d < rank; ++d) postfix *= shapes[d];
    for (int j = 0; j < count; ++j) {
        segments[j] = shapes[j * rank + axis] * postfix;
        total += segments[j];
    }
    *block_count = blocks;
    *sum = total;
}

/* split/cpu_kernel.cc:27-42 */
void oracle_split(void *const *outputs, const void *x, const uint32_t *segments, size_t count, size_t block_count,
                  size_t sum) {
    for (size_t i = 0; i < block_count; ++i) {
        size_t offset = i * sum;
        for (size_t j = 0; j < count; ++j) {
            const size_t len = segments[j];
            memcpy((uint8_t *) outputs[j] + i * len, (const uint8_t *) x + offset, len);
            offset += len;
        }
    }
}

/* concat/cpu_kernel.cc:27-42 */
void oracle_concat(void *y, const void *const *inputs, const uint32_t *segments, size_t count, size_t block_count,
                   size_t sum) {
    for (size_t i = 0; i < block_count; ++i) {
        size_t offset = i * sum;
        for (size_t j = 0; j < count; ++j) {
            const size_t len = segments[j];
            memcpy((uint8_t *) y + offset, (const uint8_t *) inputs[j] + i * len, len);
            offset += len;
        }
    }
}

/* ------------------------------------------------------- expand */

/* expand_info.cc:14-60.  Returns the number of (i, o) stride pairs (0: nothing is broadcast). */
int oracle_expand_info(uint32_t *stride_i, uint32_t *stride_o, uint32_t *block_size, uint32_t *block_count,
                       const uint32_t *input, int in_rank, const uint32_t *output, int out_rank, uint32_t elem_size) {
    uint32_t si[18], so[18];
    int n = 1;
    si[0] = so[0] = 1;
    uint32_t count = 1, stride = 1;
    int i = in_rank;
    for (int o = out_rank; o != 0;) {
        const uint32_t i_ = i == 0 ? 1 : input[--i], o_ = output[--o];
        if (o_ == 1) continue;
        if (i_ == 1) {
            if (si[n - 1]) { si[n] = 0; so[n] = count; ++n; }
        } else {
            if (!si[n - 1]) { si[n] = stride; so[n] = count; ++n; }
            stride *= i_;
        }
        count *= o_;
    }
    *block_size = elem_size;
    if (n == 1) {  /* nothing is broadcast */
        *block_size *= count;
        *block_count = 1;
        return 0;
    }
    /* reversed, the initial {1, 1} dropped; the last pair left is a broadcast one and becomes the block */
    int dims = n - 1;
    for (int d = 0; d < dims; ++d) { stride_i[d] = si[n - 1 - d]; stride_o[d] = so[n - 1 - d]; }
    const uint32_t tail_o = stride_o[dims - 1];
    *block_size *= tail_o;
    *block_count = count / tail_o;
    for (int d = 0; d < dims; ++d) { stride_i[d] /= tail_o; stride_o[d] /= tail_o; }
    return dims;
}

/* expand/cpu_kernel.cc:27-46 */
void oracle_expand(void *y, const void *x, const uint32_t *stride_i, const uint32_t *stride_o, int dims,
                   uint32_t block_size, uint32_t block_count) {
    for (uint32_t k = 0; k < block_count; ++k) {
        long rem = k, j = 0;
        for (int d = 0; d < dims; ++d) {
            if (stride_i[d]) {
                j += rem / stride_o[d] * stride_i[d];
                rem %= stride_o[d];
            } else {
                rem %= stride_o[d];
            }
        }
        memcpy((uint8_t *) y + (size_t) k * block_size, (const uint8_t *) x + (size_t) j * block_size, block_size);
    }
}

/* ------------------------------------------------------- broadcaster / where */

/* broadcaster.cc:17-79: shapes of `inputs` tensors (ranks[i] entries each, rows of 8).  strides receives
 * dims x (inputs + 1) values; returns dims (0: nothing is broadcast) and the output element count. */
int oracle_broadcaster(uint32_t *strides, uint32_t *outputs_count, const uint32_t *shapes, const int *ranks, int inputs) {
    uint32_t rev[16 * 9];
    int used = 0, end[8], state[8], next[8];
    uint32_t muls[8], count = 1;
    for (int i = 0; i < inputs; ++i) { end[i] = ranks[i]; state[i] = 0; muls[i] = 1; }
    for (;;) {
        uint32_t shape = 1;
        int all_end = 1;
        for (int i = 0; i < inputs; ++i) next[i] = 0;
        for (int i = 0; i < inputs; ++i) {
            if (end[i] == 0) continue;
            const uint32_t dim = shapes[i * 8 + --end[i]];
            next[i] = dim != 1;
            if (next[i]) shape = dim;  /* (a mismatch between inputs is the caller's error) */
            all_end = 0;
        }
        if (all_end) break;
        if (shape == 1) continue;
        int same = 1;
        for (int i = 0; i < inputs; ++i) same &= next[i] == state[i];
        if (!same) {
            /* a new group of (inputs + 1) strides, written back to front: output stride first */
            for (int i = 0; i < inputs; ++i) state[i] = next[i];
            uint32_t *group = rev + used;
            used += inputs + 1;
            for (int i = 0; i < inputs; ++i) {
                group[i] = 0;
                if (state[inputs - 1 - i]) { group[i] = muls[inputs - 1 - i]; muls[inputs - 1 - i] *= shape; }
            }
            group[inputs] = count;
        } else {
            for (int i = 0; i < inputs; ++i)
                if (state[i]) muls[i] *= shape;
        }
        count *= shape;
    }
    *outputs_count = count;
    /* `rev` holds what the reference's vector holds read from its end; reversing the whole vector gives, per
     * group from the slowest dimension on, the input strides in input order followed by the output stride */
    int all_one = used == inputs + 1;
    for (int t = 0; t < used && all_one; ++t) all_one = rev[t] == 1;
    if (all_one || used == 0) return 0;
    const int dims = used / (inputs + 1);
    for (int g = 0; g < dims; ++g) {
        const uint32_t *group = rev + (dims - 1 - g) * (inputs + 1);
        for (int i = 0; i < inputs; ++i) strides[g * (inputs + 1) + i] = group[inputs - 1 - i];
        strides[g * (inputs + 1) + inputs] = group[inputs];
    }
    return dims;
}

/* where/cpu_kernel.cc:32-47 with broadcaster.cc:87-100 */
void oracle_where(void *out, const uint8_t *c, const void *x, const void *y, const uint32_t *strides, int dims,
                  uint32_t count, uint32_t elem_size) {
    for (uint32_t i = 0; i < count; ++i) {
        uint32_t at[3] = {i, i, i};
        if (dims) {
            long rem = i;
            at[0] = at[1] = at[2] = 0;
            for (int d = 0; d < dims; ++d) {
                const uint32_t *dim = strides + 4 * d;
                const long q = rem / dim[3];
                for (int j = 0; j < 3; ++j) at[j] += dim[j] * (uint32_t) q;
                rem %= dim[3];
            }
        }
        memcpy((uint8_t *) out + (size_t) i * elem_size,
               c[at[0]] ? (const uint8_t *) x + (size_t) at[1] * elem_size : (const uint8_t *) y + (size_t) at[2] * elem_size,
               elem_size);
    }
}
