// Softmax along one axis of a [pre, mid, post] view, optional causal mask, for gfx950.
//
// Arithmetic contract: src/04kernel/src/kernels/softmax/cpu_kernel.cc:27-60 of the reference,
// with a floating accumulator (the reference's own CUDA kernel, cuda_kernel.cu:29-55, computes
// the same true softmax).  HBM-bound: a row is read once with 128-bit loads, kept in registers
// through max / exp / sum, and written once.  FP16/BF16 rows are evaluated in float and rounded
// once on store.
#include "common.hpp"

namespace rg {
namespace {

template <class CT> __device__ __forceinline__ CT neg_inf();
template <> __device__ __forceinline__ float neg_inf<float>() { return -__builtin_inff(); }
template <> __device__ __forceinline__ double neg_inf<double>() { return -__builtin_inf(); }

// exp(d) for d <= 0.  16-bit storage: hardware exp2 on d*log2(e) (relative error ~1e-6 at
// |d| < 30, far below the storage precision); F32/F64: the library routine.
template <class T> struct Exp {
    static __device__ __forceinline__ float eval(float d) {
        return __builtin_amdgcn_exp2f(d * 1.4426950408889634f);
    }
};
template <> struct Exp<float> {
    static __device__ __forceinline__ float eval(float d) { return expf(d); }
};
template <> struct Exp<double> {
    static __device__ __forceinline__ double eval(double d) { return exp(d); }
};

// e / sum.  16-bit storage multiplies by one reciprocal per row (the extra rounding is ~1e-7
// relative); F32/F64 divide, as the reference does.
template <class T> struct Normalise {
    float inv;
    __device__ __forceinline__ explicit Normalise(float sum) : inv(1.0f / sum) {}
    __device__ __forceinline__ float operator()(float e) const { return e * inv; }
};
template <> struct Normalise<float> {
    float sum;
    __device__ __forceinline__ explicit Normalise(float s) : sum(s) {}
    __device__ __forceinline__ float operator()(float e) const { return e / sum; }
};
template <> struct Normalise<double> {
    double sum;
    __device__ __forceinline__ explicit Normalise(double s) : sum(s) {}
    __device__ __forceinline__ double operator()(double e) const { return e / sum; }
};

// GROUP threads own one contiguous row (post == 1), NV 16-byte vectors per thread.
// causal_rows == 0: plain.  Otherwise row r of each [causal_rows, mid] matrix keeps the first
// r + (mid - causal_rows) + 1 columns; vectors wholly beyond that are neither loaded nor
// computed, only zero-filled.
template <class T, int GROUP, int NV>
__global__ __launch_bounds__(256) void softmax_rows(T *__restrict__ y, const T *__restrict__ x,
                                                    uint64_t rows, uint32_t mid,
                                                    uint32_t causal_rows) {
    using CT = typename Compute<T>::type;
    constexpr int VEC = Vec16<T>::N;
    constexpr int ROWS_PER_BLOCK = 256 / GROUP;
    __shared__ CT smem[4];

    const uint32_t t = threadIdx.x % GROUP;
    const uint64_t row = static_cast<uint64_t>(blockIdx.x) * ROWS_PER_BLOCK + threadIdx.x / GROUP;
    const bool live = row < rows;
    const uint32_t nvec = mid / VEC;
    uint32_t keep = mid;  // number of unmasked leading columns
    if (causal_rows) keep = static_cast<uint32_t>(row % causal_rows) + (mid - causal_rows) + 1;
    const T *xr = x + row * mid;
    T *yr = y + row * mid;

    CT f[NV][VEC];
    CT mx = neg_inf<CT>();
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const uint32_t idx = t + i * GROUP;
        const uint32_t c0 = idx * VEC;
        if (live && idx < nvec && c0 < keep) {
            const Vec16<T> xv = load16_stream(xr + c0);
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                f[i][e] = c0 + e < keep ? to_compute(xv.v[e]) : neg_inf<CT>();
                mx = mx < f[i][e] ? f[i][e] : mx;
            }
        } else {
#pragma unroll
            for (int e = 0; e < VEC; ++e) f[i][e] = neg_inf<CT>();
        }
    }
    auto wmax = [](CT v) { return wave_max(v); };
    auto wsum = [](CT v) { return wave_sum(v); };
    if constexpr (GROUP < kWave) {  // short rows: several to a wavefront, reduced among GROUP neighbouring lanes
#pragma unroll
        for (int o = GROUP / 2; o > 0; o >>= 1) {
            const CT other = __shfl_xor(mx, o, kWave);
            mx = mx < other ? other : mx;
        }
    } else if constexpr (GROUP == kWave) mx = wave_max(mx);
    else mx = block_allreduce<GROUP / kWave>(mx, smem, wmax, [](CT a, CT b) { return a < b ? b : a; });

    CT sum = 0;
#pragma unroll
    for (int i = 0; i < NV; ++i)
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            // masked / padding slots hold -inf: exp gives exactly 0
            f[i][e] = Exp<T>::eval(f[i][e] - mx);
            sum += f[i][e];
        }
    if constexpr (GROUP < kWave) {
#pragma unroll
        for (int o = GROUP / 2; o > 0; o >>= 1) sum += __shfl_xor(sum, o, kWave);
    } else if constexpr (GROUP == kWave) sum = wave_sum(sum);
    else sum = block_allreduce<GROUP / kWave>(sum, smem, wsum, [](CT a, CT b) { return a + b; });

    const Normalise<T> norm(sum);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const uint32_t idx = t + i * GROUP;
        if (live && idx < nvec) {
            Vec16<T> out;
#pragma unroll
            for (int e = 0; e < VEC; ++e) out.v[e] = from_compute<T>(norm(f[i][e]));
            store16_stream(yr + static_cast<size_t>(idx) * VEC, out);
        }
    }
}

// Rows too long for the register kernel (more than 1024 16-byte vectors; post == 1): one workgroup of 1024
// threads per row.  One sweep over the row keeps a running (max, sum of exp) per thread, rescaling the sum
// when the maximum rises, and leaves the first 64 KiB of the row in LDS as read; the threads' pairs are merged
// once; the second sweep takes the row from LDS (what did not fit, from memory again) and writes the result.
// A thread visits the same vectors in both sweeps, so the LDS copy needs no barrier of its own.  CACHED is
// 4096 vectors (two workgroups per CU) for rows that fit in them, else 8192.
template <class T, uint32_t CACHED>
__global__ __launch_bounds__(1024) void softmax_long(T *__restrict__ y, const T *__restrict__ x, uint32_t mid,
                                                     uint32_t causal_rows) {
    using CT = typename Compute<T>::type;
    constexpr int VEC = Vec16<T>::N;
    constexpr uint32_t THREADS = 1024, AHEAD = 4;
    __shared__ Vec16<T> cache[CACHED];
    __shared__ CT smem[THREADS / kWave];

    const uint32_t t = threadIdx.x;
    const uint64_t row = blockIdx.x;
    const uint32_t nvec = mid / VEC;
    uint32_t keep = mid;
    if (causal_rows) keep = static_cast<uint32_t>(row % causal_rows) + (mid - causal_rows) + 1;
    const uint32_t kvec = (keep + VEC - 1) / VEC;  // vectors that hold at least one kept column
    const T *xr = x + row * mid;
    T *yr = y + row * mid;

    CT mx = neg_inf<CT>(), sum = 0;
    for (uint32_t i0 = t; i0 < kvec; i0 += THREADS * AHEAD) {
        Vec16<T> xv[AHEAD];
#pragma unroll
        for (uint32_t a = 0; a < AHEAD; ++a) {
            const uint32_t idx = i0 + a * THREADS;
            if (idx < kvec) xv[a] = load16_stream(xr + static_cast<size_t>(idx) * VEC);
        }
#pragma unroll
        for (uint32_t a = 0; a < AHEAD; ++a) {
            const uint32_t idx = i0 + a * THREADS;
            if (idx >= kvec) break;
            if (idx < CACHED) cache[idx] = xv[a];
            CT f[VEC], vm = neg_inf<CT>();
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                f[e] = idx * VEC + e < keep ? to_compute(xv[a].v[e]) : neg_inf<CT>();
                vm = vm < f[e] ? f[e] : vm;
            }
            if (mx < vm) {  // exp(-inf - vm) = 0 clears the (still zero) sum of a thread that had no maximum yet
                sum *= Exp<T>::eval(mx - vm);
                mx = vm;
            }
            if (mx > neg_inf<CT>()) {
#pragma unroll
                for (int e = 0; e < VEC; ++e) sum += Exp<T>::eval(f[e] - mx);
            }
        }
    }
    auto wmax = [](CT v) { return wave_max(v); };
    auto wsum = [](CT v) { return wave_sum(v); };
    const CT row_max = block_allreduce<THREADS / kWave>(mx, smem, wmax, [](CT a, CT b) { return a < b ? b : a; });
    // a thread without a maximum contributes 0 * exp(-inf) = 0; a row of -inf only gives NaN throughout, as
    // in the kernel above and in the reference
    const CT share = sum * Exp<T>::eval(mx - row_max);
    const CT total = block_allreduce<THREADS / kWave>(share, smem, wsum, [](CT a, CT b) { return a + b; });
    const Normalise<T> norm(total);

    for (uint32_t i0 = t; i0 < nvec; i0 += THREADS * AHEAD) {
        Vec16<T> xv[AHEAD];
#pragma unroll
        for (uint32_t a = 0; a < AHEAD; ++a) {
            const uint32_t idx = i0 + a * THREADS;
            if (idx < kvec) xv[a] = idx < CACHED ? cache[idx] : load16_stream(xr + static_cast<size_t>(idx) * VEC);
        }
#pragma unroll
        for (uint32_t a = 0; a < AHEAD; ++a) {
            const uint32_t idx = i0 + a * THREADS;
            if (idx >= nvec) break;
            Vec16<T> out;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const bool kept = idx < kvec && idx * VEC + e < keep;
                out.v[e] = from_compute<T>(kept ? norm(Exp<T>::eval(to_compute(xv[a].v[e]) - row_max)) : CT(0));
            }
            store16_stream(yr + static_cast<size_t>(idx) * VEC, out);
        }
    }
}

// Contiguous rows (post == 1) whose length or addresses do not fit 128-bit vectors throughout (a row of scores
// over a history of 1025 positions, a vocabulary of 50257): THREADS threads per row, the row swept twice (a running
// maximum and sum per thread, merged once; then the results - the second read comes from L2).  The middle of a row,
// from the first 16-byte boundary of its addresses on, still moves in aligned 128-bit vectors; only the elements
// before and after go one by one (all of them when x and y are aligned differently).
template <class T, int THREADS>
__global__ __launch_bounds__(THREADS < 256 ? 256 : THREADS) void softmax_ragged(T *__restrict__ y, const T *__restrict__ x,
                                                                               uint64_t rows, uint32_t mid, uint32_t causal_rows) {
    using CT = typename Compute<T>::type;
    constexpr int VEC = Vec16<T>::N;
    constexpr int BLOCK = THREADS < 256 ? 256 : THREADS, RPB = BLOCK / THREADS;
    static_assert((THREADS <= kWave && kWave % THREADS == 0) || THREADS == BLOCK, "a row belongs to a part of a wavefront or to the whole workgroup");
    __shared__ CT smem[BLOCK / kWave];
    const uint32_t t = threadIdx.x % THREADS;
    const uint64_t row = static_cast<uint64_t>(blockIdx.x) * RPB + threadIdx.x / THREADS;
    const bool live = row < rows;
    uint32_t keep = mid;
    if (causal_rows) keep = static_cast<uint32_t>(row % causal_rows) + (mid - causal_rows) + 1;
    if (!live) keep = 0;  // (a workgroup's surplus rows take part in the barriers only)
    const T *xr = x + (live ? row : 0) * mid;
    T *yr = y + (live ? row : 0) * mid;
    const uint32_t to_boundary = static_cast<uint32_t>((16 - (reinterpret_cast<uintptr_t>(xr) & 15)) & 15) / sizeof(T);
    const bool same = ((reinterpret_cast<uintptr_t>(xr) ^ reinterpret_cast<uintptr_t>(yr)) & 15) == 0;
    const uint32_t head = same && to_boundary < mid ? to_boundary : mid;  // elements before the first vector
    const uint32_t vecs = (mid - head) / VEC, tail = head + vecs * VEC;  // elements from `tail` on follow the last vector

    CT mx = neg_inf<CT>(), sum = 0;
    auto take = [&](CT f) {
        if (mx < f) {  // exp(-inf - f) = 0 clears the (still zero) sum of a thread that had no maximum yet
            sum *= Exp<T>::eval(mx - f);
            mx = f;
        }
        if (mx > neg_inf<CT>()) sum += Exp<T>::eval(f - mx);
    };
    for (uint32_t i = t; i < head; i += THREADS)
        if (i < keep) take(to_compute(xr[i]));
    for (uint32_t i = tail + t; i < mid; i += THREADS)
        if (i < keep) take(to_compute(xr[i]));
#pragma unroll 4
    for (uint32_t v = t; v < vecs; v += THREADS) {
        const uint32_t c0 = head + v * VEC;
        if (c0 >= keep) break;  // this thread's further vectors lie beyond the kept columns as well
        const Vec16<T> xv = load16_stream(xr + c0);
        CT f[VEC], vm = neg_inf<CT>();
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            f[e] = c0 + e < keep ? to_compute(xv.v[e]) : neg_inf<CT>();
            vm = vm < f[e] ? f[e] : vm;
        }
        if (mx < vm) {
            sum *= Exp<T>::eval(mx - vm);
            mx = vm;
        }
        if (mx > neg_inf<CT>()) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) sum += Exp<T>::eval(f[e] - mx);
        }
    }
    auto wmax = [](CT v) { return wave_max(v); };
    auto wsum = [](CT v) { return wave_sum(v); };
    CT row_max, total;
    if constexpr (THREADS <= kWave) {  // (short rows: several to a wavefront, so that it has several rows' loads in flight)
        row_max = mx;
#pragma unroll
        for (int off = THREADS / 2; off > 0; off >>= 1) {
            const CT other = __shfl_xor(row_max, off, kWave);
            row_max = row_max < other ? other : row_max;
        }
        total = sum * Exp<T>::eval(mx - row_max);
#pragma unroll
        for (int off = THREADS / 2; off > 0; off >>= 1) total += __shfl_xor(total, off, kWave);
    } else {
        row_max = block_allreduce<THREADS / kWave>(mx, smem, wmax, [](CT a, CT b) { return a < b ? b : a; });
        total = block_allreduce<THREADS / kWave>(sum * Exp<T>::eval(mx - row_max), smem, wsum, [](CT a, CT b) { return a + b; });
    }
    if (!live) return;
    const Normalise<T> norm(total);
    auto result = [&](T v, uint32_t i) {
        return from_compute<T>(i < keep ? norm(Exp<T>::eval(to_compute(v) - row_max)) : CT(0));
    };
    for (uint32_t i = t; i < head; i += THREADS) yr[i] = result(xr[i], i);
    for (uint32_t i = tail + t; i < mid; i += THREADS) yr[i] = result(xr[i], i);
#pragma unroll 4
    for (uint32_t v = t; v < vecs; v += THREADS) {
        const uint32_t c0 = head + v * VEC;
        Vec16<T> out;
        if (c0 < keep) {
            const Vec16<T> xv = load16_stream(xr + c0);
#pragma unroll
            for (int e = 0; e < VEC; ++e) out.v[e] = result(xv.v[e], c0 + e);
        } else {
#pragma unroll
            for (int e = 0; e < VEC; ++e) out.v[e] = from_compute<T>(CT(0));
        }
        store16_stream(yr + c0, out);
    }
}

// Contiguous rows of up to 32 elements that fit no vectors (two classes, seven experts): one thread per row, the row in
// registers (64 threads per row left 62 of them idle: 4 M rows of two fp16 elements 732 us).
template <class T>
__global__ __launch_bounds__(256) void softmax_tiny(T *__restrict__ y, const T *__restrict__ x, uint64_t rows, uint32_t mid,
                                                    uint32_t causal_rows) {
    using CT = typename Compute<T>::type;
    const uint64_t row = static_cast<uint64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (row >= rows) return;
    uint32_t keep = mid;
    if (causal_rows) keep = static_cast<uint32_t>(row % causal_rows) + (mid - causal_rows) + 1;
    const T *xr = x + row * mid;
    T *yr = y + row * mid;
    CT f[32], mx = neg_inf<CT>();
#pragma unroll
    for (int e = 0; e < 32; ++e) {
        f[e] = static_cast<uint32_t>(e) < keep ? to_compute(xr[e]) : neg_inf<CT>();
        mx = mx < f[e] ? f[e] : mx;
    }
    CT sum = 0;
#pragma unroll
    for (int e = 0; e < 32; ++e) {
        f[e] = Exp<T>::eval(f[e] - mx);  // (slots beyond the row hold -inf: exactly 0)
        sum += f[e];
    }
    const Normalise<T> norm(sum);
#pragma unroll
    for (int e = 0; e < 32; ++e)
        if (static_cast<uint32_t>(e) < mid) yr[e] = from_compute<T>(static_cast<uint32_t>(e) < keep ? norm(f[e]) : CT(0));
}

// A few very long contiguous rows (logits over a vocabulary): one workgroup per row leaves the chip idle (a row of
// 128256 floats 47 us).  The row is cut into chunks, one workgroup each, in three launches that need no workspace:
// (1) a chunk's maximum and its sum relative to it go, as two floats, into the first 8 bytes of the chunk's place in
// y; (2) one workgroup per row combines them and writes the row's maximum and sum into every chunk's first 8 bytes;
// (3) a chunk reads its 8 bytes, then its elements of x, and writes its outputs over them.  Only for y and x that
// do not overlap (in place, step 1 would destroy inputs).  CT is float for every T but double.
constexpr int kChunkThreads = 1024;

template <class T>
__global__ __launch_bounds__(kChunkThreads) void softmax_chunk_stats(T *__restrict__ y, const T *__restrict__ x, uint32_t mid,
                                                                     uint32_t chunk) {
    using CT = typename Compute<T>::type;
    __shared__ CT smem[kChunkThreads / kWave];
    const uint64_t row = blockIdx.y;
    const uint32_t c0 = blockIdx.x * chunk, c1 = blockIdx.x + 1 == gridDim.x ? mid : c0 + chunk;  // (the last chunk takes the rest)
    const T *xr = x + row * mid;
    CT m = neg_inf<CT>();
    for (uint32_t j = c0 + threadIdx.x; j < c1; j += kChunkThreads) {
        const CT v = to_compute(xr[j]);
        m = m < v ? v : m;
    }
    m = block_allreduce<kChunkThreads / kWave>(m, smem, [](CT v) { return wave_max(v); }, [](CT a, CT b) { return a < b ? b : a; });
    CT sum = 0;
    if (m > neg_inf<CT>())
        for (uint32_t j = c0 + threadIdx.x; j < c1; j += kChunkThreads) sum += Exp<T>::eval(to_compute(xr[j]) - m);
    sum = block_allreduce<kChunkThreads / kWave>(sum, smem, [](CT v) { return wave_sum(v); }, [](CT a, CT b) { return a + b; });
    if (threadIdx.x == 0) {
        const float pair[2] = {static_cast<float>(m), static_cast<float>(sum)};
        __builtin_memcpy(reinterpret_cast<char *>(y + row * mid + c0), pair, 8);  // (any alignment)
    }
}

template <class T>
__global__ __launch_bounds__(256) void softmax_chunk_combine(T *__restrict__ y, uint32_t mid, uint32_t chunk, uint32_t chunks) {
    __shared__ float smem[4];
    const uint64_t row = blockIdx.x;
    char *yr = reinterpret_cast<char *>(y + row * mid);
    float m = -__builtin_inff();
    for (uint32_t c = threadIdx.x; c < chunks; c += 256) {
        float pair[2];
        __builtin_memcpy(pair, yr + static_cast<uint64_t>(c) * chunk * sizeof(T), 8);
        m = fmaxf(m, pair[0]);
    }
    m = block_allreduce<4>(m, smem, [](float v) { return wave_max(v); }, [](float a, float b) { return fmaxf(a, b); });
    float sum = 0.f;
    for (uint32_t c = threadIdx.x; c < chunks; c += 256) {
        float pair[2];
        __builtin_memcpy(pair, yr + static_cast<uint64_t>(c) * chunk * sizeof(T), 8);
        if (pair[0] > -__builtin_inff()) sum += pair[1] * expf(pair[0] - m);
    }
    sum = block_allreduce<4>(sum, smem, [](float v) { return wave_sum(v); }, [](float a, float b) { return a + b; });
    const float pair[2] = {m, sum};
    for (uint32_t c = threadIdx.x; c < chunks; c += 256) __builtin_memcpy(yr + static_cast<uint64_t>(c) * chunk * sizeof(T), pair, 8);
}

template <class T>
__global__ __launch_bounds__(kChunkThreads) void softmax_chunk_write(T *__restrict__ y, const T *__restrict__ x, uint32_t mid,
                                                                     uint32_t chunk) {
    using CT = typename Compute<T>::type;
    const uint64_t row = blockIdx.y;
    const uint32_t c0 = blockIdx.x * chunk, c1 = blockIdx.x + 1 == gridDim.x ? mid : c0 + chunk;  // (the last chunk takes the rest)
    const T *xr = x + row * mid;
    T *yr = y + row * mid;
    float pair[2];
    __builtin_memcpy(pair, reinterpret_cast<const char *>(yr + c0), 8);
    __syncthreads();  // everybody has the row's maximum and sum before the first output lands on them
    const CT m = static_cast<CT>(pair[0]);
    const Normalise<T> norm(static_cast<CT>(pair[1]));
    for (uint32_t j = c0 + threadIdx.x; j < c1; j += kChunkThreads) yr[j] = from_compute<T>(norm(Exp<T>::eval(to_compute(xr[j]) - m)));
}

// Any mid / post / alignment: one thread per (pre, post) slice, three passes, neighbouring
// threads touch neighbouring `post` positions.
template <class T>
__global__ __launch_bounds__(256) void softmax_generic(T *__restrict__ y, const T *__restrict__ x,
                                                       uint64_t slices, uint32_t mid, uint64_t post,
                                                       uint32_t causal_rows) {
    using CT = typename Compute<T>::type;
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i >= slices) return;
    const uint64_t base = (i - i % post) * mid + i % post;
    uint32_t keep = mid;
    if (causal_rows) keep = static_cast<uint32_t>(i % causal_rows) + (mid - causal_rows) + 1;
    CT mx = neg_inf<CT>();
    for (uint32_t j = 0; j < keep; ++j) {
        const CT v = to_compute(x[base + j * post]);
        mx = mx < v ? v : mx;
    }
    CT sum = 0;
    for (uint32_t j = 0; j < keep; ++j) sum += Exp<T>::eval(to_compute(x[base + j * post]) - mx);
    for (uint32_t j = 0; j < keep; ++j)
        y[base + j * post] = from_compute<T>(Exp<T>::eval(to_compute(x[base + j * post]) - mx) / sum);
    for (uint32_t j = keep; j < mid; ++j) y[base + j * post] = from_compute<T>(CT(0));
}

// An axis that is not the innermost one (post > 1) with a mid worth sharing: a workgroup takes 32 neighbouring
// (pre, post) slices and SEG threads per slice, which walk mid in steps of SEG (the 32 lanes of a step read
// neighbouring addresses), keep a running maximum and a sum relative to it (one exponential per element), meet in LDS
// and walk their elements once more to write.  One thread per slice, as above, left a [4096, 4096] tensor along axis 0
// to 16 workgroups and 3.7 ms.
template <class T, int SEG>
__global__ __launch_bounds__(32 * SEG) void softmax_columns(T *__restrict__ y, const T *__restrict__ x, uint64_t slices,
                                                            uint32_t mid, uint64_t post) {
    using CT = typename Compute<T>::type;
    __shared__ CT sh_m[SEG][32], sh_s[SEG][32];
    const uint32_t col = threadIdx.x % 32, seg = threadIdx.x / 32;
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * 32 + col;
    const bool live = i < slices;
    const uint64_t base = live ? (i - i % post) * mid + i % post : 0;
    CT m = neg_inf<CT>(), sum = 0;
    if (live) {
        for (uint32_t j = seg; j < mid; j += SEG) {
            const CT v = to_compute(x[base + j * post]);
            if (v > m) {  // (the first finite value lands here: the old sum is 0 and exp(-inf) is 0)
                sum = sum * Exp<T>::eval(m - v) + CT(1);
                m = v;
            } else if (v > neg_inf<CT>()) {
                sum += Exp<T>::eval(v - m);
            }
        }
    }
    sh_m[seg][col] = m;
    sh_s[seg][col] = sum;
    __syncthreads();
    CT all_m = neg_inf<CT>(), all_s = 0;
#pragma unroll
    for (int k = 0; k < SEG; ++k) all_m = sh_m[k][col] > all_m ? sh_m[k][col] : all_m;
#pragma unroll
    for (int k = 0; k < SEG; ++k)
        if (sh_m[k][col] > neg_inf<CT>()) all_s += sh_s[k][col] * Exp<T>::eval(sh_m[k][col] - all_m);
    if (!live) return;
    const Normalise<T> norm(all_s);
    for (uint32_t j = seg; j < mid; j += SEG)
        y[base + j * post] = from_compute<T>(norm(Exp<T>::eval(to_compute(x[base + j * post]) - all_m)));
}

template <class T, int GROUP, int NV>
void launch_rows(T *y, const T *x, size_t rows, size_t mid, size_t causal_rows, hipStream_t s) {
    constexpr int ROWS_PER_BLOCK = 256 / GROUP;
    const unsigned grid = static_cast<unsigned>((rows + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK);
    softmax_rows<T, GROUP, NV><<<grid, 256, 0, s>>>(y, x, rows, static_cast<uint32_t>(mid),
                                                    static_cast<uint32_t>(causal_rows));
}

template <class T>
int dispatch(void *y_, const void *x_, size_t pre, size_t mid, size_t post, size_t causal_rows,
             hipStream_t s) {
    auto *y = static_cast<T *>(y_);
    auto *x = static_cast<const T *>(x_);
    constexpr size_t VEC = Vec16<T>::N;
    const size_t nvec = mid / VEC;
    // a few very long rows: chunks of a row to a workgroup each (not for double: the chunk results travel as floats)
    if (post == 1 && causal_rows == 0 && sizeof(T) <= 4 && mid >= 32768 && mid <= 0xffffffffu && pre * (mid / 8192) <= 2048 && pre <= 65535) {
        const char *xb = reinterpret_cast<const char *>(x), *yb = reinterpret_cast<const char *>(y);
        const size_t bytes = pre * mid * sizeof(T);
        const bool apart = xb + bytes <= yb || yb + bytes <= xb;
        size_t chunks = 512 / pre;
        if (chunks > mid / 4096) chunks = mid / 4096;
        if (apart && chunks >= 4) {
            // chunks of a multiple of 8 elements; the last one takes what is left (never less than a chunk, so that
            // its first 8 bytes are its own)
            const uint32_t chunk = static_cast<uint32_t>(mid / chunks) / 8 * 8;
            const uint32_t n_chunks = static_cast<uint32_t>(mid / chunk);
            const dim3 grid(n_chunks, static_cast<unsigned>(pre));
            softmax_chunk_stats<T><<<grid, kChunkThreads, 0, s>>>(y, x, static_cast<uint32_t>(mid), chunk);
            int rc = launch_status();
            if (rc) return rc;
            softmax_chunk_combine<T><<<static_cast<unsigned>(pre), 256, 0, s>>>(y, static_cast<uint32_t>(mid), chunk, n_chunks);
            rc = launch_status();
            if (rc) return rc;
            softmax_chunk_write<T><<<grid, kChunkThreads, 0, s>>>(y, x, static_cast<uint32_t>(mid), chunk);
            return launch_status();
        }
    }
    const bool rows_ok = post == 1 && mid % VEC == 0 && aligned16(y) && aligned16(x) &&
                         (pre + 3) / 4 <= 0x7fffffffu;
    if (rows_ok && nvec <= 16 && (pre + 15) / 16 <= 0x7fffffffu) {
        // rows of a few vectors (scores over a handful of experts or classes): 1 to 16 lanes per row instead of 64
        if (nvec <= 1) launch_rows<T, 1, 1>(y, x, pre, mid, causal_rows, s);
        else if (nvec <= 2) launch_rows<T, 2, 1>(y, x, pre, mid, causal_rows, s);
        else if (nvec <= 4) launch_rows<T, 4, 1>(y, x, pre, mid, causal_rows, s);
        else if (nvec <= 8) launch_rows<T, 8, 1>(y, x, pre, mid, causal_rows, s);
        else launch_rows<T, 16, 1>(y, x, pre, mid, causal_rows, s);
    } else if (rows_ok && nvec <= 64 * 4) {
        if (nvec <= 64) launch_rows<T, 64, 1>(y, x, pre, mid, causal_rows, s);
        else if (nvec <= 128) launch_rows<T, 64, 2>(y, x, pre, mid, causal_rows, s);
        else launch_rows<T, 64, 4>(y, x, pre, mid, causal_rows, s);
    } else if (rows_ok && nvec <= 256 * 4) {
        if (nvec <= 256) launch_rows<T, 256, 1>(y, x, pre, mid, causal_rows, s);
        else if (nvec <= 512) launch_rows<T, 256, 2>(y, x, pre, mid, causal_rows, s);
        else launch_rows<T, 256, 4>(y, x, pre, mid, causal_rows, s);
    } else if (rows_ok && pre <= 0x7fffffffu) {
        if (nvec <= 4096)
            softmax_long<T, 4096><<<static_cast<unsigned>(pre), 1024, 0, s>>>(y, x, static_cast<uint32_t>(mid),
                                                                             static_cast<uint32_t>(causal_rows));
        else
            softmax_long<T, 8192><<<static_cast<unsigned>(pre), 1024, 0, s>>>(y, x, static_cast<uint32_t>(mid),
                                                                             static_cast<uint32_t>(causal_rows));
    } else if (post == 1 && pre <= 0x7fffffffu) {
        const uint32_t m32 = static_cast<uint32_t>(mid), c32 = static_cast<uint32_t>(causal_rows);
        if (mid <= 32) softmax_tiny<T><<<static_cast<unsigned>((pre + 255) / 256), 256, 0, s>>>(y, x, pre, m32, c32);
        else if (mid / Vec16<T>::N <= 48) softmax_ragged<T, 16><<<static_cast<unsigned>((pre + 15) / 16), 256, 0, s>>>(y, x, pre, m32, c32);
        else if (mid / Vec16<T>::N <= 96) softmax_ragged<T, 32><<<static_cast<unsigned>((pre + 7) / 8), 256, 0, s>>>(y, x, pre, m32, c32);
        else if (mid <= 2048) softmax_ragged<T, 64><<<static_cast<unsigned>((pre + 3) / 4), 256, 0, s>>>(y, x, pre, m32, c32);
        else if (mid <= 32768) softmax_ragged<T, 256><<<static_cast<unsigned>(pre), 256, 0, s>>>(y, x, pre, m32, c32);
        else softmax_ragged<T, 1024><<<static_cast<unsigned>(pre), 1024, 0, s>>>(y, x, pre, m32, c32);
    } else if (post > 1 && mid >= 32 && causal_rows == 0 && (static_cast<uint64_t>(pre) * post + 31) / 32 <= 0x7fffffffu) {
        const uint64_t slices = static_cast<uint64_t>(pre) * post;
        const unsigned grid = static_cast<unsigned>((slices + 31) / 32);
        if (mid >= 1024) softmax_columns<T, 32><<<grid, 1024, 0, s>>>(y, x, slices, static_cast<uint32_t>(mid), post);
        else softmax_columns<T, 8><<<grid, 256, 0, s>>>(y, x, slices, static_cast<uint32_t>(mid), post);
    } else {
        const uint64_t slices = static_cast<uint64_t>(pre) * post;
        const uint64_t grid = (slices + 255) / 256;
        if (grid > 0x7fffffffu) return RG_HIP_E_UNSUPPORTED;
        softmax_generic<T><<<static_cast<unsigned>(grid), 256, 0, s>>>(
            y, x, slices, static_cast<uint32_t>(mid), post, static_cast<uint32_t>(causal_rows));
    }
    return launch_status();
}

}  // namespace
}  // namespace rg

extern "C" int rg_hip_softmax(void *y, const void *x, size_t pre, size_t mid, size_t post,
                              int dtype, size_t causal_rows, void *stream) {
    if (!y || !x) return RG_HIP_E_ARGUMENT;
    if (pre == 0 || mid == 0 || post == 0) return 0;
    if (mid > 0x7fffffffu) return RG_HIP_E_UNSUPPORTED;
    if (causal_rows && (post != 1 || pre % causal_rows != 0 || mid < causal_rows))
        return RG_HIP_E_ARGUMENT;
    hipStream_t s = rg::as_stream(stream);
    switch (dtype) {
        case RG_F32: return rg::dispatch<float>(y, x, pre, mid, post, causal_rows, s);
        case RG_F64: return rg::dispatch<double>(y, x, pre, mid, post, causal_rows, s);
        case RG_FP16: return rg::dispatch<__half>(y, x, pre, mid, post, causal_rows, s);
        case RG_BF16: return rg::dispatch<__hip_bfloat16>(y, x, pre, mid, post, causal_rows, s);
        default: return RG_HIP_E_UNSUPPORTED;
    }
}
