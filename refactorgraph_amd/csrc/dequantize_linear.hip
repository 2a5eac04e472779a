// DequantizeLinear for gfx950: y = (float)((int)x - (int)zp) * scale.
//
// Arithmetic contract: src/04kernel/src/kernels/dequantize_linear/cpu_kernel.cc:43-56 of the
// reference (one integer subtract, one int->float convert, one float multiply: bit-exact in any
// IEEE implementation).  The reference handles a scalar scale only; a per-axis scale over
// x[outer, axis_len, inner] uses the same form with scale[a] / zp[a].
// HBM-bound, 5 bytes per 8-bit element: every store instruction writes 1 KiB contiguous per
// wavefront (float4 per lane) and the matching loads are 4-byte lanes of a contiguous 256 B.
#include "common.hpp"

namespace rg {
namespace {

struct alignas(4) Bytes4 {
    uint8_t b[4];
};
struct alignas(16) Float4 {
    float v[4];
};
typedef float f32x4 __attribute__((ext_vector_type(4)));

template <class TI> __device__ __forceinline__ int widen(uint8_t raw);
template <> __device__ __forceinline__ int widen<uint8_t>(uint8_t raw) { return raw; }
template <> __device__ __forceinline__ int widen<int8_t>(uint8_t raw) { return static_cast<int8_t>(raw); }

// 8-bit input, groups of 4 consecutive elements that share (scalar) or vector-load (per-axis,
// inner == 1) their scale.  UNROLL groups per thread, 256 lanes apart, so each load/store
// instruction of a wavefront is contiguous.
// PER_AXIS: 0 one scale; 1 the innermost axis carries the scales (a group of 4 takes 4 of them); 2 an axis in front of
// `inner4` groups of 4 carries them (a group takes one: rows of a weight matrix with a scale each)
template <class TI, int PER_AXIS, int UNROLL>
__global__ __launch_bounds__(256) void dequant8_vec(float *__restrict__ y, const TI *__restrict__ x,
                                                    const float *__restrict__ scale,
                                                    const TI *__restrict__ zp, uint64_t groups,
                                                    uint32_t axis_len, uint32_t inner4) {
    const uint64_t g0 = static_cast<uint64_t>(blockIdx.x) * (256 * UNROLL) + threadIdx.x;
    Bytes4 in[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const uint64_t g = g0 + u * 256;
        if (g < groups)
            in[u] = __builtin_bit_cast(Bytes4, __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(x + g * 4)));
    }
    float s_scalar = 0.f;
    int z_scalar = 0;
    if constexpr (PER_AXIS == 0) {
        s_scalar = scale[0];
        z_scalar = zp ? static_cast<int>(zp[0]) : 0;
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const uint64_t g = g0 + u * 256;
        if (g < groups) {
            Float4 out;
            if constexpr (PER_AXIS == 2) {
                const uint32_t a = (static_cast<uint32_t>(g) / inner4) % axis_len;  // (the host keeps groups below 2^32)
                const float sa = scale[a];
                const int za = zp ? widen<TI>(reinterpret_cast<const uint8_t *>(zp)[a]) : 0;
#pragma unroll
                for (int e = 0; e < 4; ++e) out.v[e] = static_cast<float>(widen<TI>(in[u].b[e]) - za) * sa;
            } else if constexpr (PER_AXIS == 1) {
                const uint32_t a0 = static_cast<uint32_t>((g * 4) % axis_len);
                const Float4 s = *reinterpret_cast<const Float4 *>(scale + a0);
                int z[4] = {0, 0, 0, 0};
                if (zp) {
                    const Bytes4 zb = *reinterpret_cast<const Bytes4 *>(zp + a0);
#pragma unroll
                    for (int e = 0; e < 4; ++e) z[e] = widen<TI>(zb.b[e]);
                }
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    out.v[e] = static_cast<float>(widen<TI>(in[u].b[e]) - z[e]) * s.v[e];
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    out.v[e] = static_cast<float>(widen<TI>(in[u].b[e]) - z_scalar) * s_scalar;
            }
            __builtin_nontemporal_store(__builtin_bit_cast(f32x4, out), reinterpret_cast<f32x4 *>(y + g * 4));
        }
    }
}

// 32-bit input (the sums of a MatMulInteger), groups of 4 consecutive elements: 16 bytes in, 16 bytes out per lane,
// UNROLL groups per thread 256 lanes apart.  Same arithmetic, same sharing of the scale as above.
typedef int i32x4 __attribute__((ext_vector_type(4)));
template <int PER_AXIS, int UNROLL>
__global__ __launch_bounds__(256) void dequant32_vec(float *__restrict__ y, const int32_t *__restrict__ x,
                                                     const float *__restrict__ scale, const int32_t *__restrict__ zp,
                                                     uint64_t groups, uint32_t axis_len, uint32_t inner4) {
    const uint64_t g0 = static_cast<uint64_t>(blockIdx.x) * (256 * UNROLL) + threadIdx.x;
    i32x4 in[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const uint64_t g = g0 + u * 256;
        if (g < groups) in[u] = __builtin_nontemporal_load(reinterpret_cast<const i32x4 *>(x + g * 4));
    }
    float s_scalar = 0.f;
    int z_scalar = 0;
    if constexpr (PER_AXIS == 0) {
        s_scalar = scale[0];
        z_scalar = zp ? zp[0] : 0;
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const uint64_t g = g0 + u * 256;
        if (g < groups) {
            Float4 out;
            if constexpr (PER_AXIS == 2) {
                const uint32_t a = (static_cast<uint32_t>(g) / inner4) % axis_len;
                const float sa = scale[a];
                const int za = zp ? zp[a] : 0;
#pragma unroll
                for (int e = 0; e < 4; ++e) out.v[e] = static_cast<float>(in[u][e] - za) * sa;
            } else if constexpr (PER_AXIS == 1) {
                const uint32_t a0 = static_cast<uint32_t>((g * 4) % axis_len);
                const Float4 s = *reinterpret_cast<const Float4 *>(scale + a0);
                i32x4 z = {0, 0, 0, 0};
                if (zp) z = *reinterpret_cast<const i32x4 *>(zp + a0);
#pragma unroll
                for (int e = 0; e < 4; ++e) out.v[e] = static_cast<float>(in[u][e] - z[e]) * s.v[e];
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) out.v[e] = static_cast<float>(in[u][e] - z_scalar) * s_scalar;
            }
            __builtin_nontemporal_store(__builtin_bit_cast(f32x4, out), reinterpret_cast<f32x4 *>(y + g * 4));
        }
    }
}

// 16-bit input, groups of 4 consecutive elements: 8 bytes in, 16 bytes out per lane.  Same arithmetic, same sharing of the
// scale (PER_AXIS as above).
template <class TI, int PER_AXIS, int UNROLL>
__global__ __launch_bounds__(256) void dequant16_vec(float *__restrict__ y, const TI *__restrict__ x,
                                                     const float *__restrict__ scale, const TI *__restrict__ zp,
                                                     uint64_t groups, uint32_t axis_len, uint32_t inner4) {
    struct alignas(8) Elems4 {
        TI v[4];
    };
    const uint64_t g0 = static_cast<uint64_t>(blockIdx.x) * (256 * UNROLL) + threadIdx.x;
    Elems4 in[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const uint64_t g = g0 + u * 256;
        if (g < groups) in[u] = __builtin_bit_cast(Elems4, __builtin_nontemporal_load(reinterpret_cast<const uint64_t *>(x + g * 4)));
    }
    float s_scalar = 0.f;
    int z_scalar = 0;
    if constexpr (PER_AXIS == 0) {
        s_scalar = scale[0];
        z_scalar = zp ? static_cast<int>(zp[0]) : 0;
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const uint64_t g = g0 + u * 256;
        if (g < groups) {
            Float4 out;
            if constexpr (PER_AXIS == 2) {
                const uint32_t a = (static_cast<uint32_t>(g) / inner4) % axis_len;  // (the host keeps groups below 2^32)
                const float sa = scale[a];
                const int za = zp ? static_cast<int>(zp[a]) : 0;
#pragma unroll
                for (int e = 0; e < 4; ++e) out.v[e] = static_cast<float>(static_cast<int>(in[u].v[e]) - za) * sa;
            } else if constexpr (PER_AXIS == 1) {
                const uint32_t a0 = static_cast<uint32_t>((g * 4) % axis_len);
                const Float4 s = *reinterpret_cast<const Float4 *>(scale + a0);
                Elems4 z = {};
                if (zp) z = *reinterpret_cast<const Elems4 *>(zp + a0);
#pragma unroll
                for (int e = 0; e < 4; ++e) out.v[e] = static_cast<float>(static_cast<int>(in[u].v[e]) - static_cast<int>(z.v[e])) * s.v[e];
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) out.v[e] = static_cast<float>(static_cast<int>(in[u].v[e]) - z_scalar) * s_scalar;
            }
            __builtin_nontemporal_store(__builtin_bit_cast(f32x4, out), reinterpret_cast<f32x4 *>(y + g * 4));
        }
    }
}

// Every other case: one element per thread-iteration.
template <class TI>
__global__ __launch_bounds__(256) void dequant_generic(float *__restrict__ y, const TI *__restrict__ x,
                                                       const float *__restrict__ scale,
                                                       const TI *__restrict__ zp, uint64_t n,
                                                       uint64_t axis_len, uint64_t inner, int per_axis) {
    const uint64_t stride = static_cast<uint64_t>(gridDim.x) * 256;
    for (uint64_t e = static_cast<uint64_t>(blockIdx.x) * 256 + threadIdx.x; e < n; e += stride) {
        const uint64_t a = per_axis ? (e / inner) % axis_len : 0;
        const int z = zp ? static_cast<int>(zp[a]) : 0;
        y[e] = static_cast<float>(static_cast<int>(x[e]) - z) * scale[a];
    }
}

template <class TI>
int dispatch8(float *y, const void *x_, const float *scale, const void *zp_, size_t outer,
              size_t axis_len, size_t inner, int per_axis, hipStream_t s) {
    auto *x = static_cast<const TI *>(x_);
    auto *zp = static_cast<const TI *>(zp_);
    const uint64_t n = static_cast<uint64_t>(outer) * axis_len * inner;
    constexpr int UNROLL = 8;  // 32 KiB written per workgroup; 4 gave 8 % less throughput on 4096 x 4096
    const bool base_ok = n % 4 == 0 && aligned16(y) && (reinterpret_cast<uintptr_t>(x) & 3u) == 0;
    const uint64_t groups = n / 4;
    const uint64_t grid = (groups + 256 * UNROLL - 1) / (256 * UNROLL);
    if (base_ok && grid <= 0x7fffffffu) {
        if (!per_axis) {
            dequant8_vec<TI, 0, UNROLL><<<static_cast<unsigned>(grid), 256, 0, s>>>(
                y, x, scale, zp, groups, 1, 1);
            return launch_status();
        }
        if (inner == 1 && axis_len % 4 == 0 && aligned16(scale) &&
            (!zp || (reinterpret_cast<uintptr_t>(zp) & 3u) == 0) && axis_len <= 0xffffffffu) {
            dequant8_vec<TI, 1, UNROLL><<<static_cast<unsigned>(grid), 256, 0, s>>>(
                y, x, scale, zp, groups, static_cast<uint32_t>(axis_len), 1);
            return launch_status();
        }
        // the scales belong to an axis in front of runs of whole groups (per-row scales of a weight matrix)
        if (inner % 4 == 0 && groups <= 0xffffffffu && axis_len <= 0xffffffffu && inner / 4 <= 0xffffffffu) {
            dequant8_vec<TI, 2, UNROLL><<<static_cast<unsigned>(grid), 256, 0, s>>>(
                y, x, scale, zp, groups, static_cast<uint32_t>(axis_len), static_cast<uint32_t>(inner / 4));
            return launch_status();
        }
    }
    uint64_t g = (n + 255) / 256;
    if (g > 65536) g = 65536;
    dequant_generic<TI><<<static_cast<unsigned>(g), 256, 0, s>>>(y, x, scale, zp, n, axis_len, inner, per_axis);
    return launch_status();
}

template <class TI>
int dispatch_wide(float *y, const void *x, const float *scale, const void *zp, size_t outer,
                  size_t axis_len, size_t inner, int per_axis, hipStream_t s) {
    const uint64_t n = static_cast<uint64_t>(outer) * axis_len * inner;
    if constexpr (sizeof(TI) == 4) {
        constexpr int UNROLL = 4;
        const uint64_t groups = n / 4;
        const uint64_t grid = (groups + 256 * UNROLL - 1) / (256 * UNROLL);
        if (n % 4 == 0 && aligned16(y) && aligned16(x) && grid <= 0x7fffffffu) {
            auto *xi = static_cast<const int32_t *>(x);
            auto *zi = static_cast<const int32_t *>(zp);
            if (!per_axis) {
                dequant32_vec<0, UNROLL><<<static_cast<unsigned>(grid), 256, 0, s>>>(y, xi, scale, zi, groups, 1, 1);
                return launch_status();
            }
            if (inner == 1 && axis_len % 4 == 0 && aligned16(scale) && (!zp || aligned16(zp)) && axis_len <= 0xffffffffu) {
                dequant32_vec<1, UNROLL><<<static_cast<unsigned>(grid), 256, 0, s>>>(y, xi, scale, zi, groups,
                                                                                      static_cast<uint32_t>(axis_len), 1);
                return launch_status();
            }
            if (inner % 4 == 0 && groups <= 0xffffffffu && axis_len <= 0xffffffffu && inner / 4 <= 0xffffffffu) {
                dequant32_vec<2, UNROLL><<<static_cast<unsigned>(grid), 256, 0, s>>>(
                    y, xi, scale, zi, groups, static_cast<uint32_t>(axis_len), static_cast<uint32_t>(inner / 4));
                return launch_status();
            }
        }
    }
    if constexpr (sizeof(TI) == 2) {
        constexpr int UNROLL = 4;
        const uint64_t groups = n / 4;
        const uint64_t grid = (groups + 256 * UNROLL - 1) / (256 * UNROLL);
        auto *xi = static_cast<const TI *>(x);
        auto *zi = static_cast<const TI *>(zp);
        if (n % 4 == 0 && aligned16(y) && (reinterpret_cast<uintptr_t>(x) & 7u) == 0 && grid <= 0x7fffffffu) {
            if (!per_axis) {
                dequant16_vec<TI, 0, UNROLL><<<static_cast<unsigned>(grid), 256, 0, s>>>(y, xi, scale, zi, groups, 1, 1);
                return launch_status();
            }
            if (inner == 1 && axis_len % 4 == 0 && aligned16(scale) && (!zp || (reinterpret_cast<uintptr_t>(zp) & 7u) == 0) &&
                axis_len <= 0xffffffffu) {
                dequant16_vec<TI, 1, UNROLL><<<static_cast<unsigned>(grid), 256, 0, s>>>(y, xi, scale, zi, groups,
                                                                                          static_cast<uint32_t>(axis_len), 1);
                return launch_status();
            }
            if (inner % 4 == 0 && groups <= 0xffffffffu && axis_len <= 0xffffffffu && inner / 4 <= 0xffffffffu) {
                dequant16_vec<TI, 2, UNROLL><<<static_cast<unsigned>(grid), 256, 0, s>>>(
                    y, xi, scale, zi, groups, static_cast<uint32_t>(axis_len), static_cast<uint32_t>(inner / 4));
                return launch_status();
            }
        }
    }
    uint64_t g = (n + 255) / 256;
    if (g > 65536) g = 65536;
    dequant_generic<TI><<<static_cast<unsigned>(g), 256, 0, s>>>(
        y, static_cast<const TI *>(x), scale, static_cast<const TI *>(zp), n, axis_len, inner, per_axis);
    return launch_status();
}

}  // namespace
}  // namespace rg

extern "C" int rg_hip_dequantize_linear(float *y, const void *x, const float *scale, const void *zp,
                                        size_t outer, size_t axis_len, size_t inner, int in_dtype,
                                        int per_axis, void *stream) {
    if (!y || !x || !scale) return RG_HIP_E_ARGUMENT;
    if (outer == 0 || axis_len == 0 || inner == 0) return 0;
    hipStream_t s = rg::as_stream(stream);
    switch (in_dtype) {
        case RG_U8: return rg::dispatch8<uint8_t>(y, x, scale, zp, outer, axis_len, inner, per_axis, s);
        case RG_I8: return rg::dispatch8<int8_t>(y, x, scale, zp, outer, axis_len, inner, per_axis, s);
        case RG_U16: return rg::dispatch_wide<uint16_t>(y, x, scale, zp, outer, axis_len, inner, per_axis, s);
        case RG_I16: return rg::dispatch_wide<int16_t>(y, x, scale, zp, outer, axis_len, inner, per_axis, s);
        case RG_I32: return rg::dispatch_wide<int32_t>(y, x, scale, zp, outer, axis_len, inner, per_axis, s);
        default: return RG_HIP_E_UNSUPPORTED;
    }
}
