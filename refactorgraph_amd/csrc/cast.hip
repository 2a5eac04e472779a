// Cast for gfx950: element-wise conversion between the reference's numeric data types.
//
// Arithmetic contract:
//   - pairs of U8/U16/U32/U64/I8/I16/I32/I64/F32/F64/Bool: `static_cast<U>(a)` of
//     src/04kernel/src/kernels/cast/cpu_kernel.cc:28-40 of the reference (integer narrowing wraps,
//     float -> integer truncates toward zero, integer -> float rounds to nearest even, anything
//     -> Bool is `a != 0`, Bool is one byte holding 0 or 1);
//   - pairs with FP16/BF16: the expressions of src/04kernel/src/kernels/cast/cuda_kernel.cc:55-96
//     (float/double -> half or bfloat16: round to nearest even, a double going through float first;
//     integer -> half/bfloat16: the value as `int`, rounded toward zero; half/bfloat16 -> integer:
//     truncated toward zero as `int`), except `-> Bool`, which the reference writes as `x == 0`
//     (true for zeros): this library keeps `x != 0` like every other source type.
// A float -> integer conversion of a value outside the target's range has no defined result in the
// reference (C++); here it saturates (NaN gives 0), as the hardware conversion does.
//
// HBM-bound: sizeof(from) + sizeof(to) bytes per element.  A thread converts groups of E = 16 /
// max(sizeof) consecutive elements, so the wider side moves 16 bytes per lane; UNROLL groups per
// thread sit 256 lanes apart, so every load and store instruction of a wavefront is contiguous.
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include "common.hpp"

namespace rg {
namespace {

struct BoolByte {
    uint8_t v;
};

template <class T> struct IsNarrowFloat { static constexpr bool value = false; };
template <> struct IsNarrowFloat<__half> { static constexpr bool value = true; };
template <> struct IsNarrowFloat<__hip_bfloat16> { static constexpr bool value = true; };

__device__ __forceinline__ float widen(__half v) { return __half2float(v); }
__device__ __forceinline__ float widen(__hip_bfloat16 v) { return __bfloat162float(v); }

template <class TO> __device__ __forceinline__ TO narrow_rn(float v);
template <> __device__ __forceinline__ __half narrow_rn<__half>(float v) { return __float2half(v); }
template <> __device__ __forceinline__ __hip_bfloat16 narrow_rn<__hip_bfloat16>(float v) { return __float2bfloat16(v); }

// int -> float rounded toward zero (exact below 2^24; above, the low bits are dropped)
__device__ __forceinline__ float int_to_float_rz(int v) {
    const float f = static_cast<float>(v);  // nearest
    // step back when rounding went away from zero
    const long long back = static_cast<long long>(f);
    const long long x = v;
    if ((x >= 0 && back > x) || (x < 0 && back < x))
        return __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, f) - 1u);
    return f;
}
template <class TO> __device__ __forceinline__ TO narrow_rz(float v);
template <> __device__ __forceinline__ __half narrow_rz<__half>(float v) { return __float2half_rz(v); }
template <> __device__ __forceinline__ __hip_bfloat16 narrow_rz<__hip_bfloat16>(float v) {
    // truncation of the float's low 16 bits is rounding toward zero
    const uint16_t bits = static_cast<uint16_t>(__builtin_bit_cast(uint32_t, v) >> 16);
    return __builtin_bit_cast(__hip_bfloat16, bits);
}

template <class T> struct IsFloating { static constexpr bool value = false; };
template <> struct IsFloating<float> { static constexpr bool value = true; };
template <> struct IsFloating<double> { static constexpr bool value = true; };

template <class TO, class TI> __device__ __forceinline__ TO convert(TI v) {
    if constexpr (__is_same(TI, BoolByte)) {
        const int b = v.v != 0;
        if constexpr (__is_same(TO, BoolByte)) return BoolByte{static_cast<uint8_t>(b)};
        else if constexpr (IsNarrowFloat<TO>::value) return narrow_rn<TO>(static_cast<float>(b));
        else return static_cast<TO>(b);
    } else if constexpr (__is_same(TO, BoolByte)) {
        if constexpr (IsNarrowFloat<TI>::value) return BoolByte{static_cast<uint8_t>(widen(v) != 0.f)};
        else return BoolByte{static_cast<uint8_t>(v != 0)};
    } else if constexpr (IsNarrowFloat<TI>::value) {
        const float f = widen(v);
        if constexpr (IsNarrowFloat<TO>::value) return narrow_rn<TO>(f);            // half <-> bfloat16 through float
        else if constexpr (IsFloating<TO>::value) return static_cast<TO>(f);         // exact
        else return static_cast<TO>(static_cast<int>(f));                            // as int, toward zero
    } else if constexpr (IsNarrowFloat<TO>::value) {
        if constexpr (IsFloating<TI>::value) {
            float f = static_cast<float>(v);  // a double is rounded to float first, then to the narrow type
            if constexpr (sizeof(TI) == 8) asm volatile("" : "+v"(f));  // keeps the two roundings apart (not merged into one)
            return narrow_rn<TO>(f);
        }
        else return narrow_rz<TO>(int_to_float_rz(static_cast<int>(v)));              // as int, toward zero
    } else {
        return static_cast<TO>(v);
    }
}

template <class T, int N> struct alignas(sizeof(T) * N) Pack {
    T e[N];
};

// A pack moves as one 2-, 4-, 8- or 16-byte access with the streaming hint (every element is read
// once and written once).
template <int BYTES> struct Mover;
template <> struct Mover<2> { typedef uint16_t type; };
template <> struct Mover<4> { typedef uint32_t type; };
template <> struct Mover<8> { typedef uint32_t type __attribute__((ext_vector_type(2))); };
template <> struct Mover<16> { typedef uint32_t type __attribute__((ext_vector_type(4))); };

template <class P> __device__ __forceinline__ P load_streaming(const void *p) {
    typedef typename Mover<sizeof(P)>::type M;
    return __builtin_bit_cast(P, __builtin_nontemporal_load(static_cast<const M *>(p)));
}
template <class P> __device__ __forceinline__ void store_streaming(void *p, const P &v) {
    typedef typename Mover<sizeof(P)>::type M;
    __builtin_nontemporal_store(__builtin_bit_cast(M, v), static_cast<M *>(p));
}

template <class TO, class TI, int E, int UNROLL>
__global__ __launch_bounds__(256) void cast_vec(TO *__restrict__ y, const TI *__restrict__ x, uint64_t groups) {
    const uint64_t g0 = static_cast<uint64_t>(blockIdx.x) * (256 * UNROLL) + threadIdx.x;
    Pack<TI, E> in[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const uint64_t g = g0 + u * 256;
        if (g < groups) in[u] = load_streaming<Pack<TI, E>>(x + g * E);
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const uint64_t g = g0 + u * 256;
        if (g < groups) {
            Pack<TO, E> out;
#pragma unroll
            for (int e = 0; e < E; ++e) out.e[e] = convert<TO, TI>(in[u].e[e]);
            store_streaming(y + g * E, out);
        }
    }
}

template <class TO, class TI>
__global__ __launch_bounds__(256) void cast_scalar(TO *__restrict__ y, const TI *__restrict__ x, uint64_t first,
                                                   uint64_t n) {
    const uint64_t stride = static_cast<uint64_t>(gridDim.x) * 256;
    for (uint64_t i = first + static_cast<uint64_t>(blockIdx.x) * 256 + threadIdx.x; i < n; i += stride)
        y[i] = convert<TO, TI>(x[i]);
}

template <class TO, class TI>
int launch_pair(void *y_, const void *x_, uint64_t n, hipStream_t s) {
    auto *y = static_cast<TO *>(y_);
    auto *x = static_cast<const TI *>(x_);
    constexpr int WIDE = sizeof(TI) > sizeof(TO) ? sizeof(TI) : sizeof(TO);
    constexpr int E = 16 / WIDE;
    constexpr int UNROLL = 8;
    uint64_t done = 0;
    if (reinterpret_cast<uintptr_t>(x) % (sizeof(TI) * E) == 0 && reinterpret_cast<uintptr_t>(y) % (sizeof(TO) * E) == 0 &&
        n >= static_cast<uint64_t>(E)) {
        const uint64_t groups = n / E;
        const uint64_t grid = (groups + 256 * UNROLL - 1) / (256 * UNROLL);
        if (grid <= 0x7fffffffu) {
            cast_vec<TO, TI, E, UNROLL><<<static_cast<unsigned>(grid), 256, 0, s>>>(y, x, groups);
            const int rc = launch_status();
            if (rc) return rc;
            done = groups * E;
        }
    }
    if (done < n) {
        uint64_t g = (n - done + 255) / 256;
        if (g > 65536) g = 65536;
        cast_scalar<TO, TI><<<static_cast<unsigned>(g), 256, 0, s>>>(y, x, done, n);
        return launch_status();
    }
    return 0;
}

template <class TI>
int launch_from(void *y, const void *x, uint64_t n, int to, hipStream_t s) {
    switch (to) {
        case RG_U8: return launch_pair<uint8_t, TI>(y, x, n, s);
        case RG_U16: return launch_pair<uint16_t, TI>(y, x, n, s);
        case RG_U32: return launch_pair<uint32_t, TI>(y, x, n, s);
        case RG_U64: return launch_pair<uint64_t, TI>(y, x, n, s);
        case RG_I8: return launch_pair<int8_t, TI>(y, x, n, s);
        case RG_I16: return launch_pair<int16_t, TI>(y, x, n, s);
        case RG_I32: return launch_pair<int32_t, TI>(y, x, n, s);
        case RG_I64: return launch_pair<int64_t, TI>(y, x, n, s);
        case RG_F32: return launch_pair<float, TI>(y, x, n, s);
        case RG_F64: return launch_pair<double, TI>(y, x, n, s);
        case RG_BOOL: return launch_pair<BoolByte, TI>(y, x, n, s);
        case RG_FP16: return launch_pair<__half, TI>(y, x, n, s);
        case RG_BF16: return launch_pair<__hip_bfloat16, TI>(y, x, n, s);
        default: return RG_HIP_E_UNSUPPORTED;
    }
}

size_t dtype_size(int dt) {
    switch (dt) {
        case RG_U8: case RG_I8: case RG_BOOL: return 1;
        case RG_U16: case RG_I16: case RG_FP16: case RG_BF16: return 2;
        case RG_U32: case RG_I32: case RG_F32: return 4;
        case RG_U64: case RG_I64: case RG_F64: return 8;
        default: return 0;
    }
}

}  // namespace
}  // namespace rg

extern "C" int rg_hip_cast(void *y, const void *x, size_t size, int from_dtype, int to_dtype, void *stream) {
    using namespace rg;
    if (!y || !x) return RG_HIP_E_ARGUMENT;
    const size_t from_size = dtype_size(from_dtype), to_size = dtype_size(to_dtype);
    if (!from_size || !to_size) return RG_HIP_E_UNSUPPORTED;
    if (size == 0) return 0;
    hipStream_t s = as_stream(stream);
    if (from_dtype == to_dtype) {  // the reference copies (cuda_kernel.cc:101-107); nothing to do in place
        if (y == x) return 0;
        return static_cast<int>(hipMemcpyAsync(y, x, size * from_size, hipMemcpyDeviceToDevice, s));
    }
    switch (from_dtype) {
        case RG_U8: return launch_from<uint8_t>(y, x, size, to_dtype, s);
        case RG_U16: return launch_from<uint16_t>(y, x, size, to_dtype, s);
        case RG_U32: return launch_from<uint32_t>(y, x, size, to_dtype, s);
        case RG_U64: return launch_from<uint64_t>(y, x, size, to_dtype, s);
        case RG_I8: return launch_from<int8_t>(y, x, size, to_dtype, s);
        case RG_I16: return launch_from<int16_t>(y, x, size, to_dtype, s);
        case RG_I32: return launch_from<int32_t>(y, x, size, to_dtype, s);
        case RG_I64: return launch_from<int64_t>(y, x, size, to_dtype, s);
        case RG_F32: return launch_from<float>(y, x, size, to_dtype, s);
        case RG_F64: return launch_from<double>(y, x, size, to_dtype, s);
        case RG_BOOL: return launch_from<BoolByte>(y, x, size, to_dtype, s);
        case RG_FP16: return launch_from<__half>(y, x, size, to_dtype, s);
        case RG_BF16: return launch_from<__hip_bfloat16>(y, x, size, to_dtype, s);
        default: return RG_HIP_E_UNSUPPORTED;
    }
}
