// Rotary position embedding (rotate-half pairing) for gfx950.
//
// The reference has no rotary operator; the contract is the closed form
//   inv_freq[i] = theta^(-2i/D),  angle = pos * inv_freq[i]   (i < D/2)
//   y[i]       = x[i]       * cos(angle) - x[i + D/2] * sin(angle)
//   y[i + D/2] = x[i + D/2] * cos(angle) + x[i]       * sin(angle)
// on x[batch, seq, heads, D].  HBM-bound (one read, one write).  The D/2 (cos, sin) pairs of a
// token are shared by all its heads, so they are evaluated once per token into LDS instead of
// once per element: the trigonometric work drops by the head count and stays off the critical
// path of the 128-bit loads, which are issued before the table is built.
#include "common.hpp"

#include <cmath>

namespace rg {
namespace {

constexpr int kMaxHalf = 256;   // D <= 512
constexpr int kMaxTokens = 8;   // tokens per workgroup

// inv_freq is computed on the host in double and rounded once to float, so device and host
// evaluations of the angle use bit-identical factors.  Passed by value in the kernel arguments.
struct InvFreq {
    float f[kMaxHalf];
};

// Workgroup: `tokens` consecutive tokens; a work unit is one (token, head, 16-byte slice of
// the lower half) plus its partner slice in the upper half.  ITER units per thread are loaded
// before the table is built.
template <class T, int ITER>
__global__ __launch_bounds__(256) void rope_tokens(T *__restrict__ y, const T *__restrict__ x,
                                                   const int64_t *__restrict__ pos,
                                                   int pos_per_batch, uint64_t n_tokens,
                                                   uint32_t seq, uint32_t heads, uint32_t D,
                                                   uint32_t tokens, const InvFreq inv_freq) {
    constexpr int VEC = Vec16<T>::N;
    __shared__ float tab_cos[kMaxTokens * kMaxHalf];
    __shared__ float tab_sin[kMaxTokens * kMaxHalf];

    const uint32_t half = D / 2;
    const uint32_t slices = half / VEC;             // 16-byte slices per half head
    const uint32_t units_per_token = heads * slices;
    const uint64_t tok0 = static_cast<uint64_t>(blockIdx.x) * tokens;
    const uint32_t live_tokens =
        static_cast<uint32_t>(n_tokens - tok0 < tokens ? n_tokens - tok0 : tokens);
    const uint32_t total_units = live_tokens * units_per_token;

    Vec16<T> lo[ITER], hi[ITER];
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
        const uint32_t u = threadIdx.x + it * 256;
        if (u < total_units) {
            const uint32_t tk = u / units_per_token, r = u % units_per_token;
            const uint32_t h = r / slices, sl = r % slices;
            const T *p = x + ((tok0 + tk) * heads + h) * D + sl * VEC;
            lo[it] = load16_stream(p);
            hi[it] = load16_stream(p + half);
        }
    }

    for (uint32_t e = threadIdx.x; e < live_tokens * half; e += 256) {
        const uint32_t tk = e / half, i = e % half;
        const uint64_t token = tok0 + tk;
        const int64_t position = pos_per_batch ? pos[token] : pos[token % seq];
        const float angle = static_cast<float>(position) * inv_freq.f[i];
        float sn, cs;
        sincosf(angle, &sn, &cs);
        tab_cos[tk * half + i] = cs;
        tab_sin[tk * half + i] = sn;
    }
    __syncthreads();

#pragma unroll
    for (int it = 0; it < ITER; ++it) {
        const uint32_t u = threadIdx.x + it * 256;
        if (u < total_units) {
            const uint32_t tk = u / units_per_token, r = u % units_per_token;
            const uint32_t h = r / slices, sl = r % slices;
            Vec16<T> olo, ohi;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const float cs = tab_cos[tk * half + sl * VEC + e];
                const float sn = tab_sin[tk * half + sl * VEC + e];
                const float a = to_compute(lo[it].v[e]), b = to_compute(hi[it].v[e]);
                olo.v[e] = from_compute<T>(a * cs - b * sn);
                ohi.v[e] = from_compute<T>(b * cs + a * sn);
            }
            T *q = y + ((tok0 + tk) * heads + h) * D + sl * VEC;
            store16_stream(q, olo);
            store16_stream(q + half, ohi);
        }
    }
}

// Any D (even) / alignment: one thread per (token, head, i) pair.
template <class T>
__global__ __launch_bounds__(256) void rope_generic(T *__restrict__ y, const T *__restrict__ x,
                                                    const int64_t *__restrict__ pos,
                                                    int pos_per_batch, uint64_t n_pairs,
                                                    uint32_t seq, uint32_t heads, uint32_t D,
                                                    const InvFreq inv_freq) {
    const uint64_t g = static_cast<uint64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (g >= n_pairs) return;
    const uint32_t half = D / 2;
    const uint32_t i = static_cast<uint32_t>(g % half);
    const uint64_t th = g / half;  // token * heads + head
    const uint64_t token = th / heads;
    const int64_t position = pos_per_batch ? pos[token] : pos[token % seq];
    const float angle = static_cast<float>(position) * inv_freq.f[i];
    float sn, cs;
    sincosf(angle, &sn, &cs);
    const float a = to_compute(x[th * D + i]), b = to_compute(x[th * D + i + half]);
    y[th * D + i] = from_compute<T>(a * cs - b * sn);
    y[th * D + i + half] = from_compute<T>(b * cs + a * sn);
}

template <class T, int ITER>
void launch_tokens(T *y, const T *x, const int64_t *pos, int ppb, uint64_t n_tokens, size_t seq,
                   size_t heads, size_t D, uint32_t tokens, const InvFreq &f, hipStream_t s) {
    const uint64_t grid = (n_tokens + tokens - 1) / tokens;
    rope_tokens<T, ITER><<<static_cast<unsigned>(grid), 256, 0, s>>>(
        y, x, pos, ppb, n_tokens, static_cast<uint32_t>(seq), static_cast<uint32_t>(heads),
        static_cast<uint32_t>(D), tokens, f);
}

template <class T>
int dispatch(void *y_, const void *x_, const int64_t *pos, int ppb, size_t batch, size_t seq,
             size_t heads, size_t D, float theta, hipStream_t s) {
    auto *y = static_cast<T *>(y_);
    auto *x = static_cast<const T *>(x_);
    InvFreq f;
    const size_t half = D / 2;
    for (size_t i = 0; i < half; ++i)
        f.f[i] = static_cast<float>(std::pow(static_cast<double>(theta),
                                             -2.0 * static_cast<double>(i) / static_cast<double>(D)));
    for (size_t i = half; i < kMaxHalf; ++i) f.f[i] = 0.0f;

    constexpr size_t VEC = Vec16<T>::N;
    const uint64_t n_tokens = static_cast<uint64_t>(batch) * seq;
    const size_t units = half % VEC == 0 ? heads * (half / VEC) : 0;
    if (units && units <= 2048 && aligned16(y) && aligned16(x)) {
        // as many whole tokens as fit 1024 work units (4 per thread), at most kMaxTokens
        if (units <= 1024) {
            uint32_t tokens = static_cast<uint32_t>(1024 / units);
            if (tokens > kMaxTokens) tokens = kMaxTokens;
            if (n_tokens / tokens < 1024 && tokens > 1) tokens = 1;  // small inputs: more workgroups
            const size_t per_block = tokens * units;
            if (per_block <= 256) launch_tokens<T, 1>(y, x, pos, ppb, n_tokens, seq, heads, D, tokens, f, s);
            else if (per_block <= 512) launch_tokens<T, 2>(y, x, pos, ppb, n_tokens, seq, heads, D, tokens, f, s);
            else launch_tokens<T, 4>(y, x, pos, ppb, n_tokens, seq, heads, D, tokens, f, s);
        } else {
            launch_tokens<T, 8>(y, x, pos, ppb, n_tokens, seq, heads, D, 1, f, s);
        }
    } else {
        const uint64_t n_pairs = n_tokens * heads * half;
        const uint64_t grid = (n_pairs + 255) / 256;
        if (grid > 0x7fffffffu) return RG_HIP_E_UNSUPPORTED;
        rope_generic<T><<<static_cast<unsigned>(grid), 256, 0, s>>>(
            y, x, pos, ppb, n_pairs, static_cast<uint32_t>(seq), static_cast<uint32_t>(heads),
            static_cast<uint32_t>(D), f);
    }
    return launch_status();
}

}  // namespace
}  // namespace rg

extern "C" int rg_hip_rope(void *y, const void *x, const int64_t *pos, int pos_per_batch,
                           size_t batch, size_t seq, size_t heads, size_t dim, float theta,
                           int dtype, void *stream) {
    if (!y || !x || !pos) return RG_HIP_E_ARGUMENT;
    if (dim % 2 != 0 || dim > 2 * rg::kMaxHalf) return RG_HIP_E_UNSUPPORTED;
    if (batch == 0 || seq == 0 || heads == 0 || dim == 0) return 0;
    if (seq > 0x7fffffffu || heads > 0x7fffffffu) return RG_HIP_E_UNSUPPORTED;
    hipStream_t s = rg::as_stream(stream);
    switch (dtype) {
        case RG_FP16: return rg::dispatch<__half>(y, x, pos, pos_per_batch, batch, seq, heads, dim, theta, s);
        case RG_BF16: return rg::dispatch<__hip_bfloat16>(y, x, pos, pos_per_batch, batch, seq, heads, dim, theta, s);
        case RG_F32: return rg::dispatch<float>(y, x, pos, pos_per_batch, batch, seq, heads, dim, theta, s);
        default: return RG_HIP_E_UNSUPPORTED;
    }
}
