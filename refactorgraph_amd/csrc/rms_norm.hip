// RmsNormalization for gfx950.
//
// Arithmetic contract: src/04kernel/src/kernels/rms_normalization/cpu_kernel.cc:47-65 of the
// reference (y = x * 1/sqrt(mean(x^2) + eps) * w, normalised over the last axis).
// HBM-bound: one read of x, one write of y.  A row is held in registers between the
// sum-of-squares pass and the scaling pass, so x is fetched from memory exactly once;
// all global accesses are 128-bit and wave-contiguous.
#include <cfloat>

#include "common.hpp"

namespace rg {
namespace {

// GROUP threads (one wavefront, or the whole 256-thread workgroup) own one row and keep up to
// NV 16-byte vectors of it per thread.
// MINMAX (float only): the workgroup also leaves the least and the greatest value it has written in
// partials[2 blockIdx.x], [2 blockIdx.x + 1], started from (FLT_MAX, FLT_MIN) like the reference's
// DynamicQuantizeLinear (src/04kernel/src/kernels/dynamic_quantize_linear/cpu_kernel.cc:25-70), whose first
// pass over this output it replaces.
template <class T, int GROUP, int NV, bool MINMAX = false>
__global__ __launch_bounds__(256) void rms_norm_rows(T *__restrict__ y, const T *__restrict__ x,
                                                     const T *__restrict__ w, uint32_t rows,
                                                     uint32_t cols, float eps, float *__restrict__ partials = nullptr) {
    using CT = typename Compute<T>::type;
    constexpr int VEC = Vec16<T>::N;
    constexpr int ROWS_PER_BLOCK = 256 / GROUP;
    __shared__ CT smem[4];

    const uint32_t t = threadIdx.x % GROUP;
    const size_t row = static_cast<size_t>(blockIdx.x) * ROWS_PER_BLOCK + threadIdx.x / GROUP;
    const bool live = row < rows;  // only ever false for GROUP <= 64 (no block barrier there)
    const uint32_t nvec = cols / VEC;
    const T *xr = x + row * cols;
    T *yr = y + row * cols;

    Vec16<T> xv[NV];
    CT acc = 0;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const uint32_t idx = t + i * GROUP;
        if (live && idx < nvec) {
            xv[i] = load16_stream(xr + static_cast<size_t>(idx) * VEC);
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const CT f = to_compute(xv[i].v[e]);
                acc += f * f;
            }
        }
    }
    if constexpr (GROUP < kWave) {  // short rows (a head's 128 elements): several to a wavefront
#pragma unroll
        for (int o = GROUP / 2; o > 0; o >>= 1) acc += __shfl_xor(acc, o, kWave);
    } else if constexpr (GROUP == kWave) {
        acc = wave_sum(acc);
    } else {
        acc = block_allreduce<GROUP / kWave>(
            acc, smem, [](CT v) { return wave_sum(v); }, [](CT a, CT b) { return a + b; });
    }
    const CT scale = CT(1) / sqrt(acc / static_cast<CT>(cols) + static_cast<CT>(eps));
    float mn = FLT_MAX, mx = FLT_MIN;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const uint32_t idx = t + i * GROUP;
        if (live && idx < nvec) {
            const Vec16<T> wv = load16(w + static_cast<size_t>(idx) * VEC);
            Vec16<T> out;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                out.v[e] = from_compute<T>(to_compute(xv[i].v[e]) * scale * to_compute(wv.v[e]));
                if constexpr (MINMAX) {
                    const float v = static_cast<float>(out.v[e]);
                    mn = v < mn ? v : mn;
                    mx = mx < v ? v : mx;
                }
            }
            // (ordinary stores where a second kernel reads the output next: it should find it in the memory-side cache)
            if constexpr (MINMAX) store16(yr + static_cast<size_t>(idx) * VEC, out);
            else store16_stream(yr + static_cast<size_t>(idx) * VEC, out);
        }
    }
    if constexpr (MINMAX) {
        static_assert(!MINMAX || GROUP >= kWave, "whole wavefronts per row");
        __shared__ float ext[8];
        mn = wave_allreduce(mn, [](float a, float b) { return b < a ? b : a; });
        mx = wave_allreduce(mx, [](float a, float b) { return a < b ? b : a; });
        const uint32_t lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
        if (lane == 0) {
            ext[wave] = mn;
            ext[4 + wave] = mx;
        }
        __syncthreads();
        if (threadIdx.x == 0) {
#pragma unroll
            for (int i = 1; i < 4; ++i) {
                mn = ext[i] < mn ? ext[i] : mn;
                mx = mx < ext[4 + i] ? ext[4 + i] : mx;
            }
            partials[2 * blockIdx.x] = mn;
            partials[2 * blockIdx.x + 1] = mx;
        }
    }
}

// Any row length / alignment: one workgroup per row, two passes over x (second one from cache).
template <class T>
__global__ __launch_bounds__(256) void rms_norm_generic(T *__restrict__ y, const T *__restrict__ x,
                                                        const T *__restrict__ w, uint32_t cols,
                                                        float eps) {
    using CT = typename Compute<T>::type;
    __shared__ CT smem[4];
    const T *xr = x + static_cast<size_t>(blockIdx.x) * cols;
    T *yr = y + static_cast<size_t>(blockIdx.x) * cols;
    CT acc = 0;
    for (uint32_t j = threadIdx.x; j < cols; j += 256) {
        const CT f = to_compute(xr[j]);
        acc += f * f;
    }
    acc = block_allreduce<4>(
        acc, smem, [](CT v) { return wave_sum(v); }, [](CT a, CT b) { return a + b; });
    const CT scale = CT(1) / sqrt(acc / static_cast<CT>(cols) + static_cast<CT>(eps));
    for (uint32_t j = threadIdx.x; j < cols; j += 256)
        yr[j] = from_compute<T>(to_compute(xr[j]) * scale * to_compute(w[j]));
}

template <class T, int GROUP, int NV>
void launch_rows(T *y, const T *x, const T *w, size_t rows, size_t cols, float eps, hipStream_t s) {
    constexpr int ROWS_PER_BLOCK = 256 / GROUP;
    const unsigned grid = static_cast<unsigned>((rows + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK);
    rms_norm_rows<T, GROUP, NV><<<grid, 256, 0, s>>>(y, x, w, static_cast<uint32_t>(rows),
                                                     static_cast<uint32_t>(cols), eps);
}

template <class T>
int dispatch(void *y_, const void *x_, const void *w_, size_t rows, size_t cols, float eps,
             hipStream_t s) {
    auto *y = static_cast<T *>(y_);
    auto *x = static_cast<const T *>(x_);
    auto *w = static_cast<const T *>(w_);
    constexpr size_t VEC = Vec16<T>::N;
    const bool vec_ok = cols % VEC == 0 && aligned16(y) && aligned16(x) && aligned16(w);
    const size_t nvec = cols / VEC;
    if (vec_ok && nvec <= 32) {
        // rows of a few vectors (normalisation per head: 128 elements): 4 to 32 lanes per row instead of 64
        if (nvec <= 4) launch_rows<T, 4, 1>(y, x, w, rows, cols, eps, s);
        else if (nvec <= 8) launch_rows<T, 8, 1>(y, x, w, rows, cols, eps, s);
        else if (nvec <= 16) launch_rows<T, 16, 1>(y, x, w, rows, cols, eps, s);
        else launch_rows<T, 32, 1>(y, x, w, rows, cols, eps, s);
    } else if (vec_ok && nvec <= (rows < 1024 ? 64 * 4 : sizeof(T) == 2 ? 64 * 8 : 64 * 16)) {
        // one wavefront per row: no workgroup barrier, up to 16 loads in flight per lane.  Long rows go to a workgroup
        // each where that ends earlier: few rows (8 rows of 4096 floats 6.1 -> 2.8 us) and 16-bit rows of more than 512
        // vectors, whose 16 vectors per lane as floats cost the occupancy (4096 rows of 8192 halves from HBM
        // 34 -> 26 us, of 5120 22 -> 17 us; rows of floats are level: 4096 x 4096 24.0 and 24.1 us)
        if (nvec <= 64) launch_rows<T, 64, 1>(y, x, w, rows, cols, eps, s);
        else if (nvec <= 128) launch_rows<T, 64, 2>(y, x, w, rows, cols, eps, s);
        else if (nvec <= 256) launch_rows<T, 64, 4>(y, x, w, rows, cols, eps, s);
        else if (nvec <= 512) launch_rows<T, 64, 8>(y, x, w, rows, cols, eps, s);
        else launch_rows<T, 64, 16>(y, x, w, rows, cols, eps, s);
    } else if (vec_ok && nvec <= 256 * 8) {
        if (nvec <= 256) launch_rows<T, 256, 1>(y, x, w, rows, cols, eps, s);
        else if (nvec <= 512) launch_rows<T, 256, 2>(y, x, w, rows, cols, eps, s);
        else if (nvec <= 1024) launch_rows<T, 256, 4>(y, x, w, rows, cols, eps, s);
        else launch_rows<T, 256, 8>(y, x, w, rows, cols, eps, s);
    } else {
        rms_norm_generic<T><<<static_cast<unsigned>(rows), 256, 0, s>>>(
            y, x, w, static_cast<uint32_t>(cols), eps);
    }
    return launch_status();
}

// The float rows that the fused RmsNormalization -> DynamicQuantizeLinear pair takes: whole 16-byte vectors, one
// wavefront or one workgroup per row as in dispatch<float> above, and at most kMaxMinMaxGroups workgroups (each
// workgroup of the quantising launch reduces all of their extrema itself).  Returns the workgroups, 0: not taken.
constexpr size_t kMaxMinMaxGroups = 4096;
size_t minmax_groups(size_t rows, size_t cols) {
    if (cols % 4 != 0 || rows == 0) return 0;
    const size_t nvec = cols / 4;
    if (nvec <= 32 || nvec > 256 * 8) return 0;
    const bool wave_rows = nvec <= (rows < 1024 ? 64 * 4 : 64 * 16);
    const size_t groups = wave_rows ? (rows + 3) / 4 : rows;
    return groups <= kMaxMinMaxGroups ? groups : 0;
}

template <int GROUP, int NV>
void launch_minmax(float *y, const float *x, const float *w, size_t rows, size_t cols, float eps, float *partials, hipStream_t s) {
    constexpr int ROWS_PER_BLOCK = 256 / GROUP;
    const unsigned grid = static_cast<unsigned>((rows + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK);
    rms_norm_rows<float, GROUP, NV, true><<<grid, 256, 0, s>>>(y, x, w, static_cast<uint32_t>(rows),
                                                                static_cast<uint32_t>(cols), eps, partials);
}

int dispatch_minmax(float *y, const float *x, const float *w, size_t rows, size_t cols, float eps, float *partials, hipStream_t s) {
    const size_t nvec = cols / 4;
    if (nvec <= (rows < 1024 ? 64 * 4 : 64 * 16)) {
        if (nvec <= 64) launch_minmax<64, 1>(y, x, w, rows, cols, eps, partials, s);
        else if (nvec <= 128) launch_minmax<64, 2>(y, x, w, rows, cols, eps, partials, s);
        else if (nvec <= 256) launch_minmax<64, 4>(y, x, w, rows, cols, eps, partials, s);
        else if (nvec <= 512) launch_minmax<64, 8>(y, x, w, rows, cols, eps, partials, s);
        else launch_minmax<64, 16>(y, x, w, rows, cols, eps, partials, s);
    } else {
        if (nvec <= 256) launch_minmax<256, 1>(y, x, w, rows, cols, eps, partials, s);
        else if (nvec <= 512) launch_minmax<256, 2>(y, x, w, rows, cols, eps, partials, s);
        else if (nvec <= 1024) launch_minmax<256, 4>(y, x, w, rows, cols, eps, partials, s);
        else launch_minmax<256, 8>(y, x, w, rows, cols, eps, partials, s);
    }
    return launch_status();
}

}  // namespace

// defined with DynamicQuantizeLinear: its second launch on extrema that somebody else has left in `partials`
int quantize_with_partials(uint8_t *y, float *scale, uint8_t *zero_point, const float *x, size_t size, const float *partials,
                           size_t n_partials, hipStream_t s);

}  // namespace rg

extern "C" size_t rg_hip_rms_norm_quantize_workspace(size_t rows, size_t cols) {
    return rg::minmax_groups(rows, cols) * 2 * sizeof(float);
}

extern "C" int rg_hip_rms_norm_quantize(uint8_t *yq, float *scale, uint8_t *zero_point, float *y, const float *x,
                                        const float *w, size_t rows, size_t cols, float eps, void *workspace,
                                        size_t workspace_bytes, void *stream) {
    using namespace rg;
    if (!yq || !scale || !zero_point || !y || !x || !w) return RG_HIP_E_ARGUMENT;
    if (rows > 0x7fffffffu || cols > 0x7fffffffu) return RG_HIP_E_UNSUPPORTED;
    const size_t groups = minmax_groups(rows, cols);
    if (groups == 0 || !aligned16(y) || !aligned16(x) || !aligned16(w)) return RG_HIP_E_UNSUPPORTED;
    if (!workspace || workspace_bytes < groups * 2 * sizeof(float)) return RG_HIP_E_WORKSPACE;
    if (reinterpret_cast<uintptr_t>(workspace) % alignof(float) != 0) return RG_HIP_E_ARGUMENT;
    hipStream_t s = as_stream(stream);
    float *partials = static_cast<float *>(workspace);
    const int rc = dispatch_minmax(y, x, w, rows, cols, eps, partials, s);
    if (rc) return rc;
    return quantize_with_partials(yq, scale, zero_point, y, rows * cols, partials, groups, s);
}

extern "C" int rg_hip_rms_norm(void *y, const void *x, const void *w, size_t rows, size_t cols,
                               float eps, int dtype, void *stream) {
    if (!y || !x || !w) return RG_HIP_E_ARGUMENT;
    if (rows == 0 || cols == 0) return 0;
    if (rows > 0x7fffffffu || cols > 0x7fffffffu) return RG_HIP_E_UNSUPPORTED;
    hipStream_t s = rg::as_stream(stream);
    switch (dtype) {
        case RG_F32: return rg::dispatch<float>(y, x, w, rows, cols, eps, s);
        case RG_F64: return rg::dispatch<double>(y, x, w, rows, cols, eps, s);
        case RG_FP16: return rg::dispatch<__half>(y, x, w, rows, cols, eps, s);
        case RG_BF16: return rg::dispatch<__hip_bfloat16>(y, x, w, rows, cols, eps, s);
        default: return RG_HIP_E_UNSUPPORTED;
    }
}
