// DynamicQuantizeLinear for gfx950: float tensor -> uint8 tensor + scale + zero point.
//
// Arithmetic contract: src/04kernel/src/kernels/dynamic_quantize_linear/cpu_kernel.cc:25-70 of
// the reference, operation by operation in float:
//   (min, max) over x, started from (FLT_MAX, FLT_MIN);
//   len = max(0, max) - min(0, min);  scale = len / 255;
//   zp = saturate(0 - min * 255 / len);  y = saturate(round(x / scale) + zp);
//   saturate(v) = (uint8) round(clamp(v, 0, 255)), round = half away from zero.
// Divisions are the correctly rounded ones and denormals are kept, so the results are
// bit-identical to the CPU kernel's (an all-zero input gives scale FLT_MIN / 255, zp 0, y 0).
//
// Two launches, HBM-bound (5 bytes per element; the second read of x comes from the memory-side
// cache for tensors that fit it): per-workgroup (min, max) partials into the workspace, then every
// workgroup of the second launch reduces those partials itself — no atomics, nothing to clear, the
// result does not depend on timing.  Both launches keep eight 128-bit loads per thread in flight;
// the second replaces the division by a multiplication wherever that provably gives the same
// integer (see Quantiser::pack).
#include <cfloat>

#include "common.hpp"

namespace rg {
namespace {

constexpr uint32_t kMaxPartials = 1024;  // workgroups of the first launch
constexpr int UNROLL = 8;                // 128-bit loads a thread has in flight
constexpr uint64_t kTile = 256 * UNROLL; // vectors a workgroup takes per step
typedef float f32x4 __attribute__((ext_vector_type(4)));

struct OpMin {
    __device__ __forceinline__ float operator()(float a, float b) const { return b < a ? b : a; }
};
struct OpMax2 {
    __device__ __forceinline__ float operator()(float a, float b) const { return a < b ? b : a; }
};

__device__ __forceinline__ float block_min(float v, float *smem) {
    return block_allreduce<4>(v, smem, [](float w) { return wave_allreduce(w, OpMin{}); }, OpMin{});
}
__device__ __forceinline__ float block_max(float v, float *smem) {
    return block_allreduce<4>(v, smem, [](float w) { return wave_allreduce(w, OpMax2{}); }, OpMax2{});
}

__device__ __forceinline__ uint32_t saturate_u8(float v) {
    v = v < 0.f ? 0.f : v;
    v = 255.f < v ? 255.f : v;
    return static_cast<uint32_t>(roundf(v));
}

// scale and zero point from the extrema, and the quantisation of elements
struct Quantiser {
    float scale, zp_f, inv_scale;
    bool degenerate;
    __device__ __forceinline__ Quantiser(float mn, float mx) {
        const float len = (0.f < mx ? mx : 0.f) - (mn < 0.f ? mn : 0.f);
        scale = len / 255.f;
        degenerate = !(len > 0.f);
        zp_f = degenerate ? 0.f : static_cast<float>(saturate_u8(0.f - mn * 255.f / len));
        inv_scale = 1.f / scale;
    }
    // round(x / scale) + zp is integer-valued (or infinite), so is its clamp to [0, 255]: the second
    // rounding of the reference's saturate() changes nothing and is left out
    __device__ __forceinline__ uint32_t operator()(float v) const {
        float t = roundf(v / scale) + zp_f;
        t = t < 0.f ? 0.f : t;
        t = 255.f < t ? 255.f : t;
        return degenerate ? 0u : static_cast<uint32_t>(t);
    }
    // Four elements into one word.  The division is replaced by a multiplication where that provably
    // cannot change the result: q' = v * (1 / scale), two roundings, lies within |q'| 2^-22 of the
    // correctly rounded quotient q; if no half-integer lies within twice that distance of q', both
    // round to the same integer whichever way ties go, and that integer is the one nearest to q'.
    // Otherwise (also for NaN, infinities and a scale whose reciprocal overflows) the four elements
    // are quantised with the division.
    __device__ __forceinline__ uint32_t pack(f32x4 v) const {
        uint32_t w = 0;
        bool sure = true;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float q = v[e] * inv_scale;
            const float r = __builtin_rintf(q);
            sure = sure && __builtin_fabsf(__builtin_fabsf(q - r) - 0.5f) > __builtin_fabsf(q) * 0x1p-21f;
            float t = r + zp_f;
            t = t < 0.f ? 0.f : t;
            t = 255.f < t ? 255.f : t;
            w |= static_cast<uint32_t>(t) << (8 * e);
        }
        if (!sure || degenerate)
            w = (*this)(v[0]) | ((*this)(v[1]) << 8) | ((*this)(v[2]) << 16) | ((*this)(v[3]) << 24);
        return w;
    }
};

// (min, max) of a contiguous share of x per workgroup; vec: x is 16-byte aligned.
__global__ __launch_bounds__(256) void dql_minmax(float *__restrict__ partials, const float *__restrict__ x,
                                                  uint64_t n, int vec) {
    float mn = FLT_MAX, mx = FLT_MIN;
    const uint64_t stride = static_cast<uint64_t>(gridDim.x) * 256;
    const uint64_t t = static_cast<uint64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (vec) {
        // (ordinary loads: the second launch should find x in the memory-side cache)
        const uint64_t n4 = n / 4;
        const f32x4 *x4 = reinterpret_cast<const f32x4 *>(x);
        for (uint64_t base = blockIdx.x * kTile; base < n4; base += gridDim.x * kTile) {
            f32x4 v[UNROLL];
#pragma unroll
            for (int j = 0; j < UNROLL; ++j) {
                const uint64_t i = base + j * 256 + threadIdx.x;
                v[j] = i < n4 ? x4[i] : f32x4{FLT_MAX, FLT_MAX, FLT_MAX, FLT_MAX};
            }
#pragma unroll
            for (int j = 0; j < UNROLL; ++j) {
                if (base + j * 256 + threadIdx.x < n4) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        mn = v[j][e] < mn ? v[j][e] : mn;
                        mx = mx < v[j][e] ? v[j][e] : mx;
                    }
                }
            }
        }
        for (uint64_t i = n4 * 4 + t; i < n; i += stride) {
            mn = x[i] < mn ? x[i] : mn;
            mx = mx < x[i] ? x[i] : mx;
        }
    } else {
        for (uint64_t i = t; i < n; i += stride) {
            mn = x[i] < mn ? x[i] : mn;
            mx = mx < x[i] ? x[i] : mx;
        }
    }
    __shared__ float scratch[8];
    mn = block_min(mn, scratch);
    mx = block_max(mx, scratch + 4);
    if (threadIdx.x == 0) {
        partials[2 * blockIdx.x] = mn;
        partials[2 * blockIdx.x + 1] = mx;
    }
}

__global__ __launch_bounds__(256) void dql_quantize(uint8_t *__restrict__ y, float *__restrict__ scale_out,
                                                    uint8_t *__restrict__ zp_out, const float *__restrict__ x,
                                                    const float *__restrict__ partials, uint32_t n_partials,
                                                    uint64_t n, int vec) {
    float mn = FLT_MAX, mx = FLT_MIN;
    for (uint32_t i = threadIdx.x; i < n_partials; i += 256) {
        const float a = partials[2 * i], b = partials[2 * i + 1];
        mn = a < mn ? a : mn;
        mx = mx < b ? b : mx;
    }
    __shared__ float scratch[8];
    mn = block_min(mn, scratch);
    mx = block_max(mx, scratch + 4);

    const Quantiser quant(mn, mx);
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        *scale_out = quant.scale;
        *zp_out = static_cast<uint8_t>(quant.zp_f);
    }

    const uint64_t stride = static_cast<uint64_t>(gridDim.x) * 256;
    const uint64_t t = static_cast<uint64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (vec) {
        const uint64_t n4 = n / 4;
        const f32x4 *x4 = reinterpret_cast<const f32x4 *>(x);
        uint32_t *y4 = reinterpret_cast<uint32_t *>(y);
        for (uint64_t base = blockIdx.x * kTile; base < n4; base += gridDim.x * kTile) {
            f32x4 v[UNROLL];
#pragma unroll
            for (int j = 0; j < UNROLL; ++j) {
                const uint64_t i = base + j * 256 + threadIdx.x;
                if (i < n4) v[j] = __builtin_nontemporal_load(x4 + i);
            }
#pragma unroll
            for (int j = 0; j < UNROLL; ++j) {
                const uint64_t i = base + j * 256 + threadIdx.x;
                if (i < n4) __builtin_nontemporal_store(quant.pack(v[j]), y4 + i);
            }
        }
        for (uint64_t i = n4 * 4 + t; i < n; i += stride) y[i] = static_cast<uint8_t>(quant(x[i]));
    } else {
        for (uint64_t i = t; i < n; i += stride) y[i] = static_cast<uint8_t>(quant(x[i]));
    }
}

}  // namespace

// The quantising launch on extrema that another kernel has left (RmsNormalization with its output's least and
// greatest value per workgroup): x is read once here.
int quantize_with_partials(uint8_t *y, float *scale, uint8_t *zero_point, const float *x, size_t size, const float *partials,
                           size_t n_partials, hipStream_t s) {
    const int vec = aligned16(x) && (reinterpret_cast<uintptr_t>(y) & 3u) == 0;
    uint64_t grid = (size + 4 * kTile - 1) / (4 * kTile);
    if (grid > 8192) grid = 8192;
    if (grid == 0) grid = 1;
    dql_quantize<<<static_cast<unsigned>(grid), 256, 0, s>>>(y, scale, zero_point, x, partials,
                                                             static_cast<uint32_t>(n_partials), size, vec);
    return launch_status();
}

}  // namespace rg

extern "C" size_t rg_hip_dynamic_quantize_linear_workspace(size_t) {
    return static_cast<size_t>(rg::kMaxPartials) * 2 * sizeof(float);
}

extern "C" int rg_hip_dynamic_quantize_linear(uint8_t *y, float *scale, uint8_t *zero_point, const float *x,
                                              size_t size, void *workspace, size_t workspace_bytes,
                                              void *stream) {
    using namespace rg;
    if (!y || !scale || !zero_point || !x) return RG_HIP_E_ARGUMENT;
    if (size == 0) return RG_HIP_E_ARGUMENT;
    if (!workspace || workspace_bytes < rg_hip_dynamic_quantize_linear_workspace(size)) return RG_HIP_E_WORKSPACE;
    if (reinterpret_cast<uintptr_t>(workspace) % alignof(float) != 0) return RG_HIP_E_ARGUMENT;
    hipStream_t s = as_stream(stream);
    const int vec = aligned16(x) && (reinterpret_cast<uintptr_t>(y) & 3u) == 0;
    // a workgroup takes kTile vectors (4 kTile elements) per step
    uint64_t wgs = (size + 4 * kTile - 1) / (4 * kTile);
    if (wgs > kMaxPartials) wgs = kMaxPartials;
    if (wgs == 0) wgs = 1;
    float *partials = static_cast<float *>(workspace);
    dql_minmax<<<static_cast<unsigned>(wgs), 256, 0, s>>>(partials, x, size, vec);
    int rc = launch_status();
    if (rc) return rc;
    uint64_t grid = (size + 4 * kTile - 1) / (4 * kTile);
    if (grid > 8192) grid = 8192;
    if (grid == 0) grid = 1;
    dql_quantize<<<static_cast<unsigned>(grid), 256, 0, s>>>(y, scale, zero_point, x, partials,
                                                             static_cast<uint32_t>(wgs), size, vec);
    return launch_status();
}
