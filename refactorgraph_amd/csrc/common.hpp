// Shared device helpers for the gfx950 kernels: 64-lane wavefront reductions built on DPP,
// 128-bit vector access, storage-type conversion.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <hip/hip_bf16.h>
#include <stdint.h>

#include "rg_hip.h"

namespace rg {

constexpr int kWave = 64;

// ---------------------------------------------------------------- launch helpers

inline hipStream_t as_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

inline int launch_status() { return static_cast<int>(hipGetLastError()); }

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---------------------------------------------------------------- DPP lane exchange
// dpp_ctrl encodings (GCN3+ ISA): quad_perm = perm bits, row_half_mirror = 0x141,
// row_mirror = 0x140.  Four DPP steps leave every lane of a 16-lane row holding the row's
// reduction; two cross-row exchanges (ds_bpermute via __shfl_xor) finish the wavefront.

template <int Ctrl>
__device__ __forceinline__ float dpp_f32(float v) {
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), Ctrl, 0xf, 0xf, true));
}

struct OpSum {
    __device__ __forceinline__ float operator()(float a, float b) const { return a + b; }
};
struct OpMax {
    __device__ __forceinline__ float operator()(float a, float b) const { return fmaxf(a, b); }
};

template <class Op>
__device__ __forceinline__ float row16_allreduce(float v, Op op) {
    v = op(v, dpp_f32<0xB1>(v));   // quad_perm [1,0,3,2]
    v = op(v, dpp_f32<0x4E>(v));   // quad_perm [2,3,0,1]
    v = op(v, dpp_f32<0x141>(v));  // row_half_mirror
    v = op(v, dpp_f32<0x140>(v));  // row_mirror
    return v;
}

template <class Op>
__device__ __forceinline__ float wave_allreduce(float v, Op op) {
    v = row16_allreduce(v, op);
    v = op(v, __shfl_xor(v, 16, kWave));
    v = op(v, __shfl_xor(v, 32, kWave));
    return v;
}

__device__ __forceinline__ float wave_sum(float v) { return wave_allreduce(v, OpSum{}); }
__device__ __forceinline__ float wave_max(float v) { return wave_allreduce(v, OpMax{}); }

__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
    for (int m = 1; m < kWave; m <<= 1) v += __shfl_xor(v, m, kWave);
    return v;
}
__device__ __forceinline__ double wave_max(double v) {
#pragma unroll
    for (int m = 1; m < kWave; m <<= 1) v = fmax(v, __shfl_xor(v, m, kWave));
    return v;
}

// Reduction over a workgroup of NWAVES wavefronts; every thread receives the result.
// `smem` must hold NWAVES elements and may be reused after the call returns.
template <int NWAVES, class T, class WaveOp, class Op>
__device__ __forceinline__ T block_allreduce(T v, T *smem, WaveOp wave_op, Op op) {
    v = wave_op(v);
    if constexpr (NWAVES == 1) return v;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    __syncthreads();  // protects smem against a previous use
    if (lane == 0) smem[wave] = v;
    __syncthreads();
    T r = smem[0];
#pragma unroll
    for (int i = 1; i < NWAVES; ++i) r = op(r, smem[i]);
    return r;
}

// ---------------------------------------------------------------- 128-bit vectors

template <class T>
struct alignas(16) Vec16 {
    static constexpr int N = 16 / sizeof(T);
    T v[N];
};

template <class T>
__device__ __forceinline__ Vec16<T> load16(const T *p) {
    return *reinterpret_cast<const Vec16<T> *>(p);
}
template <class T>
__device__ __forceinline__ void store16(T *p, const Vec16<T> &v) {
    *reinterpret_cast<Vec16<T> *>(p) = v;
}

// Streaming variants: data touched once, marked non-temporal so it does not displace reusable
// lines in L2 / the memory-side cache.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
// Sixteen bytes from an address of any alignment: five aligned 32-bit loads and four byte alignments.  `last_word` is
// the last aligned word of the buffer; words behind it are not read (the bytes they would have given are arbitrary),
// and the word in front of an unaligned `p` shares its first byte's word, so nothing outside the buffer's own words
// is touched.
__device__ __forceinline__ u32x4 load16_any(const void *p, const void *last_word) {
    const uint64_t bits = reinterpret_cast<uint64_t>(p), last = reinterpret_cast<uint64_t>(last_word);
    const uint32_t shift = static_cast<uint32_t>(bits) & 3u;
    const uint64_t first = bits & ~3ull;
    uint32_t w[5];
#pragma unroll
    for (int i = 0; i < 5; ++i) {
        const uint64_t at = first + 4 * i < last ? first + 4 * i : last;
        w[i] = *reinterpret_cast<const uint32_t *>(at);
    }
    u32x4 v;
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = __builtin_amdgcn_alignbyte(w[i + 1], w[i], shift);
    return v;
}
template <class T>
__device__ __forceinline__ Vec16<T> load16_stream(const T *p) {
    const u32x4 raw = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
    return __builtin_bit_cast(Vec16<T>, raw);
}
template <class T>
__device__ __forceinline__ void store16_stream(T *p, const Vec16<T> &v) {
    __builtin_nontemporal_store(__builtin_bit_cast(u32x4, v), reinterpret_cast<u32x4 *>(p));
}

// ---------------------------------------------------------------- storage <-> compute type

template <class T> struct Compute { using type = float; };
template <> struct Compute<double> { using type = double; };

__device__ __forceinline__ float to_compute(float v) { return v; }
__device__ __forceinline__ double to_compute(double v) { return v; }
__device__ __forceinline__ float to_compute(__half v) { return __half2float(v); }
__device__ __forceinline__ float to_compute(__hip_bfloat16 v) { return __bfloat162float(v); }

template <class T> __device__ __forceinline__ T from_compute(typename Compute<T>::type v);
template <> __device__ __forceinline__ float from_compute<float>(float v) { return v; }
template <> __device__ __forceinline__ double from_compute<double>(double v) { return v; }
template <> __device__ __forceinline__ __half from_compute<__half>(float v) { return __float2half_rn(v); }
template <> __device__ __forceinline__ __hip_bfloat16 from_compute<__hip_bfloat16>(float v) {
    return __float2bfloat16(v);
}

}  // namespace rg
