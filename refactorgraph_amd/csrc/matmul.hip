// MatMul (GEMM) for gfx950: Y = alpha * op(A) @ op(B) + beta * C, C broadcast over Y.
//
// Contract: src/04kernel/src/kernels/mat_mul/cublas_kernel.cu:9-108 of the reference (row-major
// A [m,k] or [k,m] when transposed, B [k,n] or [n,k], batches strided or broadcast, alpha / beta
// converted to the data type, bias expanded into Y before the product is added) and, for the
// arithmetic, src/04kernel/src/kernels/mat_mul_common/cpu_template.hpp:19-31
// (y = beta * c + alpha * sum_k a*b).  Floating-point sums are accumulated in float (double for
// F64) in an order that differs from the CPU loop, so results agree to rounding, not bit for bit.
// The bias is read through strides inside the epilogue instead of being expanded into Y first.
//
// Fast path (FP16 / BF16, A not transposed, m and n multiples of 256, k multiple of 64): one
// 256x256 tile of Y per workgroup of four wavefronts (128x128 each, 4x4 blocks of
// v_mfma_f32_32x32x16), k-tiles of 64 copied from global memory straight into two LDS buffers
// with global_load_lds_dwordx4, fragments double buffered by k-step, one MFMA per scheduling slot:
// the structure of the MatMulInteger kernel with 16-bit operands.
//   A tile (and B given as [n,k]): rows of 128 bytes, chunk c of row r at chunk position
//           c ^ (r & 7) ^ ((r >> 3) & 1); fragments by 128-bit reads.
//   B given as [k,n]: 64 k-rows of 512 bytes, chunk c of k-row r at c ^ swz(r & 3); the operand
//           (8 consecutive k of one column per lane) is formed by two ds_read_b64_tr_b16, which
//           transpose 16-bit elements inside 16 lanes (lane i receives element i % 4 of the 8-byte
//           pieces addressed by lanes i / 4, i / 4 + 4, i / 4 + 8, i / 4 + 12).
// Few rows of A with the weights as [n, k] (a decode step) are bound by reading the weights once: one row goes
// through a matrix-vector kernel on the vector ALUs, 2 to 16 rows through 4x4x4 block products whose operands
// come straight from global memory, up to 255 rows through 32x32x16 products with the tiles passed through LDS.
// With the weights as [k, n] the block products sit behind a transposition in registers (32 rows a pass).  Where
// those passes would take longer than one launch of the 256 x 256 tiles, fewer than 256 rows run on one row of tiles.
// F32 (A not transposed) has 128 x 128 tiles of 32x32x2 products and the block-product kernels for few rows.
// Everything else (F64, transposed A, other shapes) goes through a plain tiled kernel.
#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>

#include <type_traits>
#include <utility>

#include "common.hpp"
#include "split_handoff.hpp"

namespace rg {
namespace {

// Where the bias element of Y[batch b, row i, column j] lives: c + b*sb + i*sm + j*sn (elements);
// a stride of 0 broadcasts.  c == nullptr: no bias.
struct Bias {
    const void *ptr;
    uint64_t sb, sm, sn;
};

template <class T> struct Acc { typedef float type; };
template <> struct Acc<double> { typedef double type; };

template <class T> __device__ __forceinline__ typename Acc<T>::type up(T v) { return static_cast<typename Acc<T>::type>(v); }
template <> __device__ __forceinline__ float up<__half>(__half v) { return __half2float(v); }
template <> __device__ __forceinline__ float up<__hip_bfloat16>(__hip_bfloat16 v) { return __bfloat162float(v); }
template <class T> __device__ __forceinline__ T down(typename Acc<T>::type v) { return static_cast<T>(v); }
template <> __device__ __forceinline__ __half down<__half>(float v) { return __float2half(v); }
template <> __device__ __forceinline__ __hip_bfloat16 down<__hip_bfloat16>(float v) { return __float2bfloat16(v); }

// alpha and beta are converted to the data type first, as the reference does
template <class T> typename Acc<T>::type through(float v) { return static_cast<typename Acc<T>::type>(static_cast<T>(v)); }
template <> float through<__half>(float v) { return __half2float(__float2half(v)); }
template <> float through<__hip_bfloat16>(float v) { return __bfloat162float(__float2bfloat16(v)); }

// ---------------------------------------------------------------- generic kernel
// 16x16 outputs per workgroup, one per thread; k walked in LDS tiles of 16; element (i, kk) of
// op(A) is a[i*sa0 + kk*sa1], element (kk, j) of op(B) is b[kk*sb0 + j*sb1].
template <class T>
__global__ __launch_bounds__(256) void mm_generic(T *__restrict__ y, const T *__restrict__ a, const T *__restrict__ b,
                                                  Bias bias, uint32_t m, uint32_t k, uint32_t n, uint64_t sa0,
                                                  uint64_t sa1, uint64_t sb0, uint64_t sb1,
                                                  typename Acc<T>::type alpha, typename Acc<T>::type beta,
                                                  uint32_t a_matrix0, uint32_t b_matrix0, uint32_t y_matrix0) {
    typedef typename Acc<T>::type A_t;
    __shared__ A_t ta[16][17];
    __shared__ A_t tb[16][17];
    const uint32_t bz = blockIdx.z;
    const uint64_t am = a_matrix0 + bz, bm = b_matrix0 + bz, ym = y_matrix0 + bz;
    const T *A = a + am * m * k;
    const T *B = b + bm * static_cast<uint64_t>(k) * n;
    const uint32_t tx = threadIdx.x % 16, ty = threadIdx.x / 16;
    const uint32_t row = blockIdx.y * 16 + ty, col = blockIdx.x * 16 + tx;
    A_t acc = 0;
    for (uint32_t k0 = 0; k0 < k; k0 += 16) {
        A_t va = 0, vb = 0;
        if (row < m && k0 + tx < k) va = up(A[row * sa0 + (k0 + tx) * sa1]);
        if (k0 + ty < k && col < n) vb = up(B[(k0 + ty) * sb0 + col * sb1]);
        ta[ty][tx] = va;
        tb[ty][tx] = vb;
        __syncthreads();
#pragma unroll
        for (int q = 0; q < 16; ++q) acc += ta[ty][q] * tb[q][tx];
        __syncthreads();
    }
    if (row < m && col < n) {
        A_t r = alpha * acc;
        if (bias.ptr) r += beta * up(static_cast<const T *>(bias.ptr)[ym * bias.sb + row * bias.sm + col * bias.sn]);
        y[(ym * m + row) * n + col] = down<T>(r);
    }
}

// ---------------------------------------------------------------- MFMA kernel (FP16 / BF16)

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef __bf16 b8 __attribute__((ext_vector_type(8)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef short s4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// ---------------------------------------------------------------- F32 on the matrix cores
//
// Y = alpha * A @ op(B) (+ bias) for float operands, A not transposed, k a multiple of 16: 128 x 128 outputs per
// workgroup of four wavefronts (64 x 64 each, 2 x 2 blocks of v_mfma_f32_32x32x2_f32, whose operands are one float
// per lane: row or column lane % 32, k lane / 32).  k is walked in tiles of 16 through two LDS buffers, filled from
// registers (128-bit loads a tile ahead); tiles that come as [row][k] are kept with a pitch of 20 floats, B as
// [k, n] with a pitch of 132.  Rows and columns beyond the matrix are loaded from its last ones and not stored.
constexpr int FT = 128, FK = 16, FP_RK = 20, FP_KN = 132;

template <bool TRANS_B>
__global__ __launch_bounds__(256) void mm_f32_tiles(float *__restrict__ y, const float *__restrict__ a,
                                                    const float *__restrict__ b, Bias bias, uint32_t m, uint32_t k, uint32_t n,
                                                    float alpha, float beta, uint32_t a_matrix0, uint32_t b_matrix0,
                                                    uint32_t y_matrix0) {
    constexpr int B_TILE = TRANS_B ? FT * FP_RK : FK * FP_KN;
    __shared__ __align__(16) float As[2][FT * FP_RK];
    __shared__ __align__(16) float Bs[2][B_TILE];
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
    const uint32_t bz = blockIdx.z;
    const uint64_t am = a_matrix0 + bz, bm = b_matrix0 + bz, ym = y_matrix0 + bz;
    const uint32_t row0 = blockIdx.y * FT, col0 = blockIdx.x * FT;
    const float *A = a + am * m * static_cast<uint64_t>(k);
    const float *B = b + bm * static_cast<uint64_t>(k) * n;

    // a thread's pieces of a tile: [row][k] tiles: rows tid / 4 and + 64, k 4 (tid % 4) .. + 3;
    // B as [k, n]: k-rows tid / 32 and + 8, columns 4 (tid % 32) .. + 3
    const uint32_t pr = tid >> 2, pk = 4 * (tid & 3);
    const float *a_src[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const uint32_t r = row0 + pr + 64 * i;
        a_src[i] = A + static_cast<uint64_t>(r < m ? r : m - 1) * k + pk;
    }
    const float *b_src[2];
    if constexpr (TRANS_B) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const uint32_t c = col0 + pr + 64 * i;
            b_src[i] = B + static_cast<uint64_t>(c < n ? c : n - 1) * k + pk;
        }
    } else {
        const uint32_t c = col0 + 4 * (tid & 31);
        const uint32_t cc = c + 4 <= n ? c : n - 4;  // n is a multiple of 4
#pragma unroll
        for (int i = 0; i < 2; ++i) b_src[i] = B + static_cast<uint64_t>((tid >> 5) + 8 * i) * n + cc;
    }
    f32x4 ra[2], rb[2];
    auto fetch = [&](uint32_t k0) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            ra[i] = *reinterpret_cast<const f32x4 *>(a_src[i] + k0);
            rb[i] = *reinterpret_cast<const f32x4 *>(TRANS_B ? b_src[i] + k0 : b_src[i] + static_cast<uint64_t>(k0) * n);
        }
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            *reinterpret_cast<f32x4 *>(&As[buf][(pr + 64 * i) * FP_RK + pk]) = ra[i];
            if constexpr (TRANS_B) *reinterpret_cast<f32x4 *>(&Bs[buf][(pr + 64 * i) * FP_RK + pk]) = rb[i];
            else *reinterpret_cast<f32x4 *>(&Bs[buf][((tid >> 5) + 8 * i) * FP_KN + 4 * (tid & 31)]) = rb[i];
        }
    };

    f16v acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    const uint32_t l32 = lane & 31, kh = lane >> 5;
    const uint32_t tiles = k / FK;
    fetch(0);
    for (uint32_t t = 0; t < tiles; ++t) {
        const int buf = t & 1;
        stash(buf);
        __syncthreads();  // the tile is complete; the other buffer's readers of two tiles ago have passed this point
        if (t + 1 < tiles) fetch((t + 1) * FK);
#pragma unroll
        for (int kk = 0; kk < FK; kk += 2) {
            float fa[2], fb[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) fa[i] = As[buf][(wm * 64 + 32 * i + l32) * FP_RK + kk + kh];
#pragma unroll
            for (int j = 0; j < 2; ++j)
                fb[j] = TRANS_B ? Bs[buf][(wn * 64 + 32 * j + l32) * FP_RK + kk + kh] : Bs[buf][(kk + kh) * FP_KN + wn * 64 + 32 * j + l32];
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
    }
    // accumulator: column lane % 32 of the block, register e holds row 8 (e / 4) + 4 (lane / 32) + e % 4
    const float *C = static_cast<const float *>(bias.ptr);
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const uint32_t row = row0 + wm * 64 + 32 * i + 8 * (e / 4) + 4 * kh + (e % 4);
                const uint32_t col = col0 + wn * 64 + 32 * j + l32;
                if (row < m && col < n) {
                    float v = alpha * acc[i][j][e];
                    if (C) v += beta * C[ym * bias.sb + row * bias.sm + col * bias.sn];
                    y[(ym * m + row) * n + col] = v;
                }
            }
}

template <class T> struct Mfma;
template <> struct Mfma<__half> {
    static __device__ __forceinline__ f16v run(u32x4 a, u32x4 b, f16v c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(h8, a), __builtin_bit_cast(h8, b), c, 0, 0, 0);
    }
};
template <> struct Mfma<__hip_bfloat16> {
    static __device__ __forceinline__ f16v run(u32x4 a, u32x4 b, f16v c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(b8, a), __builtin_bit_cast(b8, b), c, 0, 0, 0);
    }
};

constexpr int BM = 256, BN = 256, BK = 64;   // BK in elements: 128 bytes
constexpr int M_TILE = 32768;                // one A or B tile in LDS
constexpr int M_STAGE = 2 * M_TILE;

__device__ __forceinline__ uint32_t n_swizzle(uint32_t r) { return 4 * (r & 1) + 10 * ((r >> 1) & 1); }  // r < 4

// A, B: byte pointers to this workgroup's first row / first column; pitches in bytes.  SHORT_M: A has only
// a_rows < 256 rows; the tile's rows beyond them are copied from the last one (their results are not stored).
template <class T, bool TRANS_B, bool SHORT_M>
__device__ __forceinline__ void mm_tile_loop(f16v (&acc)[4][4], uint8_t *lds0, uint8_t *lds1, const uint8_t *A,
                                             const uint8_t *B, uint32_t k, uint32_t pitch_a, uint32_t pitch_b,
                                             uint32_t a_rows) {
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t wm = wave >> 1, wn = wave & 1, h = lane >> 5;
    // copy q < 8: A rows 8 (8 wave + q) .. + 7, this lane row + lane / 8, chunk position lane % 8.
    // copy 8 + p, B as [n,k]: the same for B's rows (columns of Y); B as [k,n]: k-rows
    // 2 (8 wave + p) and the next, this lane k-row + lane / 32, chunk position lane % 32.
    const uint8_t *a_wave = A + static_cast<uint64_t>(wave * 64) * pitch_a;
    const uint32_t a_lane = (lane >> 3) * pitch_a + 16 * ((lane & 7) ^ (lane >> 3));
    const uint8_t *b_wave = B + static_cast<uint64_t>(wave * (TRANS_B ? 64 : 16)) * pitch_b;
    uint32_t b_lane[2];
    if constexpr (TRANS_B) {
        b_lane[0] = b_lane[1] = (lane >> 3) * pitch_b + 16 * ((lane & 7) ^ (lane >> 3));
    } else {
#pragma unroll
        for (int p = 0; p < 2; ++p) b_lane[p] = (lane >> 5) * pitch_b + 16 * ((lane & 31) ^ n_swizzle(2 * p + (lane >> 5)));
    }
    auto copy = [&](uint8_t *base, uint32_t kt, int q) {
        const uint8_t *src;
        uint8_t *dst;
        if (q < 8) {
            if constexpr (SHORT_M) {
                const uint32_t row = wave * 64 + 8 * q + (lane >> 3);
                src = A + ((row < a_rows ? row : a_rows - 1) * pitch_a + kt * 128 + (16 * ((lane & 7) ^ (lane >> 3) ^ (q & 1))));
            } else {
                src = a_wave + (kt * 128 + 8 * q * pitch_a) + (a_lane ^ (16 * (q & 1)));
            }
            dst = base + (wave * 8 + q) * 1024;
        } else if constexpr (TRANS_B) {
            src = b_wave + (kt * 128 + 8 * (q - 8) * pitch_b) + (b_lane[0] ^ (16 * (q & 1)));
            dst = base + M_TILE + (wave * 8 + (q - 8)) * 1024;
        } else {
            src = b_wave + static_cast<uint64_t>(kt * BK + 2 * (q - 8)) * pitch_b + b_lane[q & 1];
            dst = base + M_TILE + (wave * 8 + (q - 8)) * 1024;
        }
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)src,
                                         (__attribute__((address_space(3))) void *)dst, 16, 0, 0);
    };
    // A fragment i of k-step ks: row wm 128 + 32 i + lane % 32, chunk 2 ks + h
    const uint32_t a_off = (wm * 128 + (lane & 31)) * 128 + 16 * (h ^ (lane & 7) ^ ((lane >> 3) & 1));
    auto read_a = [&](const uint8_t *base, int ks, int i) -> u32x4 {
        return *reinterpret_cast<const u32x4 *>(base + (a_off ^ (32 * ks)) + i * 4096);
    };
    // B fragment j of k-step ks, B as [n,k]: like A with row wn 128 + 32 j + lane % 32.
    // B as [k,n]: column wn 128 + 32 j + lane % 32, k 16 ks + 8 h .. + 7 in two transposing reads:
    // lane a of a group of 16 addresses k-row + a / 4, columns 4 (a % 4) .. + 3 of the group's 16.
    uint32_t b_off;
    if constexpr (TRANS_B) {
        b_off = M_TILE + (wn * 128 + (lane & 31)) * 128 + 16 * (h ^ (lane & 7) ^ ((lane >> 3) & 1));
    } else {
        const uint32_t a16 = lane & 15, r = a16 >> 2;
        const uint32_t chunk = wn * 16 + 2 * ((lane >> 4) & 1) + ((a16 & 3) >> 1);  // + 4 j: bits 6-7 of the byte offset
        b_off = M_TILE + (8 * h + r) * 512 + 16 * (chunk ^ n_swizzle(r)) + 8 * (a16 & 1);
    }
    auto read_b = [&](const uint8_t *base, int ks, int j, int half, u32x4 &f) {
        if constexpr (TRANS_B) {
            if (half == 0) f = *reinterpret_cast<const u32x4 *>(base + (b_off ^ (32 * ks)) + j * 4096);
        } else {
            const s4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (s4 __attribute__((address_space(3))) *)(base + (b_off ^ (64 * j)) + (16 * ks + 4 * half) * 512));
            const u32x2 w = __builtin_bit_cast(u32x2, v);
            f[2 * half] = w[0];
            f[2 * half + 1] = w[1];
        }
    };

    const uint32_t k_tiles = k / BK;
    u32x4 fa[2][4], fb[2][4];
#pragma unroll
    for (int q = 0; q < 16; ++q) copy(lds0, 0, q);
#pragma unroll
    for (int q = 0; q < 16; ++q) copy(lds1, k_tiles > 1 ? 1 : 0, q);  // k_tiles == 1: tile 0 again, never multiplied
    asm volatile("s_waitcnt vmcnt(16)" ::: "memory");  // tile 0 (the 16 older copies)
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) fa[0][i] = read_a(lds0, 0, i);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        read_b(lds0, 0, j, 0, fb[0][j]);
        read_b(lds0, 0, j, 1, fb[0][j]);
    }

    // Tile kt is in buffer RB, tile kt+1 arrives in WB.
    auto step = [&](uint32_t kt_, uint8_t *RB, const uint8_t *WB) __attribute__((always_inline)) {
        const bool more = kt_ + 2 < k_tiles;  // uniform
        auto slot = [&]<int s>() __attribute__((always_inline)) {
            // rows walk the columns back and forth, so that only one operand changes between MFMAs
            constexpr int ks = s / 16, o = s % 16, row = o / 4, col = (row & 1) ? 3 - o % 4 : o % 4;
            constexpr int cur = ks & 1, nxt = cur ^ 1;
            if constexpr (s == 48) {
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wavefront's part of tile kt+1
                __syncthreads();                                  // tile kt+1 complete, RB no longer read
            }
            acc[row][col] = Mfma<T>::run(fa[cur][row], fb[cur][col], acc[row][col]);
            const uint8_t *src = ks == 3 ? WB : RB;
            constexpr int nks = (ks + 1) % 4;
            if constexpr (o < 4) fa[nxt][o] = read_a(src, nks, o);
            else if constexpr (o < 12) read_b(src, nks, (o - 4) / 2, (o - 4) % 2, fb[nxt][(o - 4) / 2]);
            if constexpr (s >= 48) if (more) copy(RB, kt_ + 2, s - 48);
            __builtin_amdgcn_sched_barrier(0);
        };
        [&]<int... I>(std::integer_sequence<int, I...>) __attribute__((always_inline)) {
            (slot.template operator()<I>(), ...);
        }(std::make_integer_sequence<int, 64>{});
    };
    uint32_t kt = 0;
    for (; kt + 2 <= k_tiles; kt += 2) {
        step(kt, lds0, lds1);
        step(kt + 1, lds1, lds0);
    }
    if (kt < k_tiles) step(kt, lds0, lds1);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no copy may land after the workgroup's LDS is released
}

template <class T, bool TRANS_B, bool SHORT_M = false>  // SHORT_M: fewer than 256 rows of A, one row of tiles
__global__ __launch_bounds__(256, 1) void mm_mfma_256x256(T *__restrict__ y, const T *__restrict__ a,
                                                          const T *__restrict__ b, Bias bias, uint32_t m, uint32_t k,
                                                          uint32_t n, float alpha, float beta, uint32_t a_matrix0,
                                                          uint32_t b_matrix0, uint32_t y_matrix0) {
    __shared__ __align__(1024) uint8_t lds0[M_STAGE];
    __shared__ __align__(1024) uint8_t lds1[M_STAGE];

    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t bz = blockIdx.z;
    const uint64_t am = a_matrix0 + bz, bm = b_matrix0 + bz, ym = y_matrix0 + bz;

    // XCD-aware tile order: consecutive workgroup ids are dealt round-robin to the 8 XCDs, so
    // give each XCD a contiguous block of tiles (they then share A row-panels / B column-panels
    // in that XCD's L2); within it walk tiles in column-major groups of 4 rows to keep panels hot.
    const uint32_t tiles_n = (n + BN - 1) / BN, tiles_m = (m + BM - 1) / BM, n_tiles = tiles_m * tiles_n;
    uint32_t t = blockIdx.x;
    if (n_tiles % 8 == 0) t = (t % 8) * (n_tiles / 8) + t / 8;
    const uint32_t group = 4 * tiles_n;
    const uint32_t g = t / group, r = t % group;
    const uint32_t rows_here = tiles_m - g * 4 < 4 ? tiles_m - g * 4 : 4;
    const uint32_t tile_m = g * 4 + r % rows_here, tile_n = r / rows_here;

    // m and n need not be multiples of the tile: the last tile of a row or column of tiles is moved back
    // so that it ends with the matrix (m, n >= 256); the outputs it shares with its neighbour are
    // computed twice, to the same values
    const uint32_t tile_row0 = SHORT_M ? 0 : tile_m * BM + BM <= m ? tile_m * BM : m - BM;
    const uint32_t tile_col0 = tile_n * BN + BN <= n ? tile_n * BN : n - BN;
    const uint8_t *A = reinterpret_cast<const uint8_t *>(a + (am * m + tile_row0) * k);
    const T *b_matrix = b + bm * static_cast<uint64_t>(k) * n;
    const uint8_t *B = reinterpret_cast<const uint8_t *>(
        TRANS_B ? b_matrix + static_cast<uint64_t>(tile_col0) * k : b_matrix + tile_col0);

    f16v acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    mm_tile_loop<T, TRANS_B, SHORT_M>(acc, lds0, lds1, A, B, k, 2 * k, TRANS_B ? 2 * k : 2 * n, m);

    // 32x32 accumulator layout: lane holds column (lane % 32); register e holds row
    // 8*(e/4) + 4*(lane/32) + e%4.  The 128x128 block of a wavefront is transposed through LDS (its
    // own 32 KiB of the tile buffers, free now) so that Y is written with 128-bit row-contiguous
    // stores: neighbouring lanes first exchange two of their four rows, so that every lane writes
    // two adjacent columns (one dword) of two rows; chunk c of row r sits at chunk position c ^ (r & 15).
    const uint32_t wm = wave >> 1, wn = wave & 1;
    const uint32_t row0 = tile_row0 + wm * 128, col0 = tile_col0 + wn * 128;
    const T *C = static_cast<const T *>(bias.ptr);
    __syncthreads();  // every wavefront has read its last fragments
    uint8_t *stage = (wave & 2 ? lds1 : lds0) + (wave & 1) * 32768;
    const bool odd = lane & 1;
    const uint32_t col_pair = (lane & 31) & ~1u;  // first of the two columns this lane writes
    // a bias per column (the usual one of a linear layer) is the same for every row: four loads per lane instead
    // of one per output (4096^3: 133 -> 118 us)
    const bool column_bias = C && bias.sm == 0;
    float cb[4] = {0.f, 0.f, 0.f, 0.f};
    if (column_bias) {
#pragma unroll
        for (int j = 0; j < 4; ++j) cb[j] = beta * up(C[ym * bias.sb + (col0 + j * 32 + (lane & 31)) * bias.sn]);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            // any other bias: the sixteen values of a block are requested together, ahead of their use (one at a
            // time each addition waited for its own load: 4096^3 with a bias per output 160 us)
            T bv[16];
            const bool other_bias = C && !column_bias;
            if (other_bias) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    uint32_t row = row0 + i * 32 + 8 * (e / 4) + 4 * (lane >> 5) + e % 4;
                    if (SHORT_M && row >= m) row = m - 1;
                    bv[e] = C[ym * bias.sb + row * bias.sm + (col0 + j * 32 + (lane & 31)) * bias.sn];
                }
            }
#pragma unroll
            for (int eg = 0; eg < 4; ++eg) {
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    v[e] = alpha * acc[i][j][4 * eg + e];
                    if (column_bias) v[e] += cb[j];
                    else if (other_bias) v[e] += beta * up(bv[4 * eg + e]);
                }
                // even lanes keep rows 0 and 1, odd lanes rows 2 and 3 of the group of four
                const float give0 = odd ? v[0] : v[2], give1 = odd ? v[1] : v[3];
                const float got0 = __shfl_xor(give0, 1, kWave), got1 = __shfl_xor(give1, 1, kWave);
                const float lo0 = odd ? got0 : v[0], hi0 = odd ? v[2] : got0;
                const float lo1 = odd ? got1 : v[1], hi1 = odd ? v[3] : got1;
                const uint32_t r_first = i * 32 + 8 * eg + 4 * (lane >> 5) + (odd ? 2 : 0);
                const uint32_t byte_col = 2 * (j * 32 + col_pair);
                auto put = [&](uint32_t row, float lo, float hi) {
                    const T pair[2] = {down<T>(lo), down<T>(hi)};
                    *reinterpret_cast<uint32_t *>(stage + row * 256 + (byte_col ^ (16 * (row & 15)))) =
                        __builtin_bit_cast(uint32_t, pair);
                };
                put(r_first, lo0, hi0);
                put(r_first + 1, lo1, hi1);
            }
        }
    // (each wavefront reads back only what it wrote itself: no barrier)
    T *Y = y + (ym * m + row0) * n + col0;
#pragma unroll
    for (int it = 0; it < 32; ++it) {
        const uint32_t idx = lane + 64 * it, row = idx / 16, chunk = idx % 16;
        const u32x4 v = *reinterpret_cast<const u32x4 *>(stage + row * 256 + 16 * (chunk ^ (row & 15)));
        if (!SHORT_M || row0 + row < m)
            __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(Y + static_cast<uint64_t>(row) * n + chunk * 8));
    }
}

// ---------------------------------------------------------------- FP16 / BF16: any shape on the matrix cores
//
// What the kernels above do not take (fewer than 256 columns, column counts that are no multiple of 8, k that is
// no multiple of 64, ...) as long as A is not transposed and k is a multiple of 8: 128 x 128 outputs per workgroup
// of four wavefronts (64 x 64 each, 2 x 2 blocks of v_mfma_f32_32x32x16), k in tiles of 64 through two LDS
// buffers filled from registers that are loaded three tiles ahead.  Both tiles are kept as [row or column][k] with a
// pitch of 72 elements, so every fragment is one 128-bit read; B as [k, n] is turned on its way into LDS (two k-rows
// of eight columns become eight 32-bit writes).  Loads are unconditional, from addresses clamped into the matrix,
// so that the wait for a tile does not wait for the later ones as well; what lies beyond k is replaced by zeros,
// rows and columns beyond the matrix are not stored.  Where rows of B as [k, n] are not 16-byte aligned, eight
// elements come from five aligned words.
constexpr int HT = 128, HK = 64, HP = 72, HF = 3;
constexpr size_t kHalfTiles = 128;   // tiles of 128 rows up to which tiles of 64 rows are launched instead
constexpr size_t kSmallGrid = 384;  // workgroups up to which these tiles replace the 256 x 256 ones
constexpr size_t kSkinnyPassesSmall = 12000, kRowsKnPassesSmall = 10500;

// TM: rows of a tile, 128 or 64 (a wavefront then has 32 rows of 64 columns: twice the workgroups for few tiles)
template <class T, bool TRANS_B, bool B_VEC, int TM>  // B_VEC: rows of B as [k, n] start on 16-byte boundaries, n >= 8
__global__ __launch_bounds__(256, 2) void mm_tiles16(T *__restrict__ y, const T *__restrict__ a, const T *__restrict__ b, Bias bias,
                                                  uint32_t m, uint32_t k, uint32_t n, float alpha, float beta,
                                                  uint32_t a_matrix0, uint32_t b_matrix0, uint32_t y_matrix0) {
    constexpr int MI = TM / 64, AI = TM / 32;  // row blocks of a wavefront, loads of A per thread and tile
    __shared__ __align__(16) uint16_t As[2][TM * HP];
    __shared__ __align__(16) uint16_t Bs[2][HT * HP];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
    const uint32_t bz = blockIdx.z;
    const uint64_t am = a_matrix0 + bz, bm = b_matrix0 + bz, ym = y_matrix0 + bz;
    // Tile order: consecutive workgroup ids go round-robin to the 8 XCDs, so each XCD gets a contiguous run of tiles,
    // walked down the rows of one column panel after the other: the workgroups of an XCD share a panel of B in its L2.
    const uint32_t row_tiles = (m + TM - 1) / TM, n_tiles = row_tiles * ((n + HT - 1) / HT);
    uint32_t tile = blockIdx.x;
    if (n_tiles % 8 == 0) tile = (tile % 8) * (n_tiles / 8) + tile / 8;
    const uint32_t row0 = (tile % row_tiles) * TM, col0 = (tile / row_tiles) * HT;
    const uint16_t *A = reinterpret_cast<const uint16_t *>(a) + am * m * static_cast<uint64_t>(k);
    const uint16_t *B = reinterpret_cast<const uint16_t *>(b) + bm * static_cast<uint64_t>(k) * n;

    // [row][k] tiles: rows tid / 8 + 32 i, k 8 (tid % 8) .. + 7 (a row of a tile is one 128-byte line).
    // B as [k, n]: k-rows 2 (tid / 16) + 32 (i / 2) + i % 2, columns 8 (tid % 16) .. + 7
    const uint32_t pr = tid >> 3, pk = 8 * (tid & 7);
    const uint16_t *a_src[AI], *b_src[4];
#pragma unroll
    for (int i = 0; i < AI; ++i) {
        const uint32_t r = row0 + pr + 32 * i;
        a_src[i] = A + static_cast<uint64_t>(r < m ? r : m - 1) * k;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t c = col0 + pr + 32 * i;
        b_src[i] = B + static_cast<uint64_t>(c < n ? c : n - 1) * k;  // (B as [n, k] only)
    }
    const uint32_t bk = tid >> 4, bc = col0 + 8 * (tid & 15);
    const uint32_t bc_load = bc + 8 <= n ? bc : (n >= 8 ? n - 8 : 0);  // (vector loads only)
    const uint16_t *b_last = reinterpret_cast<const uint16_t *>((reinterpret_cast<uint64_t>(B + static_cast<uint64_t>(k) * n) - 1) & ~3ull);
    const u32x4 zero4 = {0u, 0u, 0u, 0u};
    u32x4 ra[HF][AI], rb[HF][4];  // HF tiles in flight
    auto fetch = [&](auto set, uint32_t k0) {
        constexpr int P = decltype(set)::value;
        const uint32_t kq = k0 + pk < k ? k0 + pk : k - 8;  // k is a multiple of 8
#pragma unroll
        for (int i = 0; i < AI; ++i) ra[P][i] = *reinterpret_cast<const u32x4 *>(a_src[i] + kq);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if constexpr (TRANS_B) {
                rb[P][i] = *reinterpret_cast<const u32x4 *>(b_src[i] + kq);
            } else {
                const uint32_t kr = k0 + 2 * bk + 32 * (i / 2) + i % 2;
                const uint16_t *src = B + static_cast<uint64_t>(kr < k ? kr : k - 1) * n;
                if constexpr (B_VEC) {
                    rb[P][i] = *reinterpret_cast<const u32x4 *>(src + bc_load);
                } else {
                    rb[P][i] = load16_any(src + bc, b_last);  // (columns beyond n: arbitrary values, not stored)
                }
            }
        }
    };
    // (the tile that reaches beyond k takes a branch of its own: selects in the common path were scheduled ahead of
    // the barrier before them, where they waited for loads a step early)
    auto stash_part = [&](auto set, auto whole, int buf, uint32_t k0) {
        constexpr int P = decltype(set)::value;
        constexpr bool WHOLE = decltype(whole)::value;
        const bool k_in = WHOLE || k0 + pk < k;
#pragma unroll
        for (int i = 0; i < AI; ++i) *reinterpret_cast<u32x4 *>(&As[buf][(pr + 32 * i) * HP + pk]) = k_in ? ra[P][i] : zero4;
        if constexpr (TRANS_B) {
#pragma unroll
            for (int i = 0; i < 4; ++i) *reinterpret_cast<u32x4 *>(&Bs[buf][(pr + 32 * i) * HP + pk]) = k_in ? rb[P][i] : zero4;
        }
        if constexpr (!TRANS_B) {
            // the two k-rows of a lane's eight columns as one 32-bit word per column.  The eight 16-byte pieces of a
            // column's k are kept in an order that depends on the column (piece ^ (column / 16) % 8): the writes of
            // a wavefront then fall into 64 different LDS banks
#pragma unroll
            for (int ii = 0; ii < 2; ++ii) {
                const bool rows_in = WHOLE || k0 + 2 * bk + 32 * ii < k;  // (k is even: both rows of the pair are in or out)
                const uint32_t word = (bk + 16 * ii) ^ (((tid >> 1) & 7) << 2);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint32_t col = 8 * (tid & 15) + 2 * j;
                    const uint32_t even = __builtin_amdgcn_perm(rb[P][2 * ii + 1][j], rb[P][2 * ii][j], 0x05040100u);
                    const uint32_t odd = __builtin_amdgcn_perm(rb[P][2 * ii + 1][j], rb[P][2 * ii][j], 0x07060302u);
                    *reinterpret_cast<uint32_t *>(&Bs[buf][col * HP + 2 * word]) = rows_in ? even : 0u;
                    *reinterpret_cast<uint32_t *>(&Bs[buf][(col + 1) * HP + 2 * word]) = rows_in ? odd : 0u;
                }
            }
        }
    };
    auto stash = [&](auto set, int buf, uint32_t k0) {
        if (k0 + HK <= k) stash_part(set, std::true_type{}, buf, k0);
        else stash_part(set, std::false_type{}, buf, k0);
    };

    f16v acc[MI][2];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    const uint32_t l32 = lane & 31, kh = lane >> 5;
    const uint32_t tiles = (k + HK - 1) / HK;
    // Step t: (barrier) request tile t + 3 into the registers tile t has left, write tile t + 1 into the buffer
    // tile t - 1 was read from, multiply tile t.  The barrier says both that tile t is complete in its buffer and
    // that everybody has finished reading tile t - 1; the LDS writes ride along with the products instead of
    // standing between two of them.
    auto step = [&](auto set_free, auto set_next, uint32_t t) {
        const int buf = t & 1;
        __syncthreads();
        fetch(set_free, (t + HF) * HK);
        stash(set_next, buf ^ 1, (t + 1) * HK);
#pragma unroll
        for (int ks = 0; ks < HK / 16; ++ks) {
            u32x4 fa[MI], fb[2];
#pragma unroll
            for (int i = 0; i < MI; ++i) fa[i] = *reinterpret_cast<const u32x4 *>(&As[buf][(wm * (TM / 2) + 32 * i + l32) * HP + 16 * ks + 8 * kh]);
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const uint32_t piece = TRANS_B ? 2 * ks + kh : (2 * ks + kh) ^ ((4 * wn + 2 * j + (l32 >> 4)) & 7);
                fb[j] = *reinterpret_cast<const u32x4 *>(&Bs[buf][(wn * 64 + 32 * j + l32) * HP + 8 * piece]);
            }
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = Mfma<T>::run(fa[i], fb[j], acc[i][j]);
        }
    };
    const std::integral_constant<int, 0> s0;
    const std::integral_constant<int, 1> s1;
    const std::integral_constant<int, 2> s2;
    fetch(s0, 0);
    fetch(s1, HK);
    fetch(s2, 2 * HK);
    stash(s0, 0, 0);
    uint32_t t = 0;
    for (; t + HF <= tiles; t += HF) {  // no branch inside: the waits count the loads of the later tiles exactly
        step(s0, s1, t);
        step(s1, s2, t + 1);
        step(s2, s0, t + 2);
    }
    if (t < tiles) step(s0, s1, t);
    if (t + 1 < tiles) step(s1, s2, t + 1);
    // accumulator: column lane % 32 of the block, register e holds row 8 (e / 4) + 4 (lane / 32) + e % 4
    const T *C = static_cast<const T *>(bias.ptr);
    // (a bias per column is the same for every row: one load per column block instead of one per output)
    const bool column_bias = C && bias.sm == 0;
    float cb[2] = {0.f, 0.f};
    if (column_bias) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const uint32_t col = col0 + wn * 64 + 32 * j + l32;
            cb[j] = beta * up(C[ym * bias.sb + (col < n ? col : n - 1) * bias.sn]);
        }
    }
    // with an even n (and Y on a 4-byte boundary) neighbouring lanes exchange two of their four rows, so that a lane
    // stores two adjacent columns of two rows with 32-bit stores; otherwise element by element
    const bool pairs = n % 2 == 0 && (reinterpret_cast<uintptr_t>(y) & 3u) == 0;
    const bool odd = lane & 1;
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int eg = 0; eg < 4; ++eg) {
                const uint32_t row_eg = row0 + wm * (TM / 2) + 32 * i + 8 * eg + 4 * kh;
                const uint32_t col = col0 + wn * 64 + 32 * j + l32;
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    v[e] = alpha * acc[i][j][4 * eg + e];
                    if (column_bias) v[e] += cb[j];
                    else if (C && row_eg + e < m && col < n) v[e] += beta * up(C[ym * bias.sb + (row_eg + e) * bias.sm + col * bias.sn]);
                }
                if (pairs) {
                    // even lanes keep rows 0 and 1, odd lanes rows 2 and 3 of the group of four
                    const float give0 = odd ? v[0] : v[2], give1 = odd ? v[1] : v[3];
                    const float got0 = __shfl_xor(give0, 1, kWave), got1 = __shfl_xor(give1, 1, kWave);
                    const float lo0 = odd ? got0 : v[0], hi0 = odd ? v[2] : got0;
                    const float lo1 = odd ? got1 : v[1], hi1 = odd ? v[3] : got1;
                    const uint32_t row = row_eg + (odd ? 2 : 0), col_pair = col & ~1u;
                    if (col_pair < n) {  // (n is even: both columns are in or out)
                        const T p0[2] = {down<T>(lo0), down<T>(hi0)}, p1[2] = {down<T>(lo1), down<T>(hi1)};
                        if (row < m) *reinterpret_cast<uint32_t *>(y + (ym * m + row) * n + col_pair) = __builtin_bit_cast(uint32_t, p0);
                        if (row + 1 < m) *reinterpret_cast<uint32_t *>(y + (ym * m + row + 1) * n + col_pair) = __builtin_bit_cast(uint32_t, p1);
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (row_eg + e < m && col < n) y[(ym * m + row_eg + e) * n + col] = down<T>(v[e]);
                }
            }
}

// ---------------------------------------------------------------- few rows of A (decode): weight streaming
//
// Y[m, n] = alpha * A[m, k] @ W[n, k]^T (+ bias) for m <= 32 SLABS, FP16 / BF16: bound by reading W once
// from HBM.  A workgroup owns 32 rows of W (32 columns of Y); its four wavefronts each take a
// quarter of k.  A wavefront loads a 32 x 128 tile of W and the matching tile of A (one per slab of
// 32 rows) with coalesced 128-bit loads (4 rows of 256 bytes per instruction: longer runs per row
// serve the DRAM pages better than 128 bytes did) two tiles ahead into registers, passes a tile
// through its own 8 KiB of LDS (chunk-swizzled rows) to bring it into MFMA operand layout, and
// multiplies with v_mfma_f32_32x32x16 (W rows as the first operand, so a lane holds one row of A in
// the result; with two slabs the W fragments are read once for both).  No barrier in the loop: a wavefront only reads what it wrote itself.  The four
// partial sums meet once at the end.  (Copying the tiles straight into LDS, as the big kernels
// do, is slower here: that path moves about 24 bytes per clock and CU, a third of what plain
// loads reach, and this kernel has nothing else to hide behind.)
constexpr int SK_DEPTH = 2;   // tiles in flight per wavefront
constexpr int SK_TK = 128;    // k elements per tile (256 bytes per row)
constexpr int SK_LOADS = 8;   // 128-bit loads per lane and operand tile

template <class T, int SLABS>  // slabs of 32 rows of A that share one pass over W
__global__ __launch_bounds__(256) void mm_skinny(T *__restrict__ y, const T *__restrict__ a, const T *__restrict__ w,
                                                 Bias bias, uint32_t m, uint32_t m_total, uint32_t row_first,
                                                 uint32_t k, uint32_t n, float alpha, float beta, uint32_t a_matrix0,
                                                 uint32_t b_matrix0, uint32_t y_matrix0) {
    constexpr int WAVE_LDS = 8192 * (1 + SLABS);  // the tile of W and one tile of A per slab
    __shared__ __align__(16) uint8_t lds[4 * WAVE_LDS + 4 * 32 * SLABS * 33 * 4];
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t bz = blockIdx.z;
    const uint64_t am = a_matrix0 + bz, bm = b_matrix0 + bz, ym = y_matrix0 + bz;
    const uint32_t n0 = blockIdx.x * 32;
    const uint64_t pitch = 2ull * k;  // bytes of a row of A or W
    const uint8_t *W = reinterpret_cast<const uint8_t *>(w + (bm * n + n0) * static_cast<uint64_t>(k));
    const uint8_t *A = reinterpret_cast<const uint8_t *>(a + (am * m_total + row_first) * static_cast<uint64_t>(k));

    // this wavefront's k-tiles (128 elements = 256 bytes each)
    const uint32_t k_tiles = k / SK_TK;
    const uint32_t t0 = k_tiles * wave / 4, t1 = k_tiles * (wave + 1) / 4;

    // load i of a tile brings rows 4 i .. 4 i + 3: this lane row + lane / 16, 16-byte chunk lane % 16,
    // kept in LDS at chunk position (lane % 16) ^ (row & 15); rows of A beyond m repeat its last row
    // (their results are not stored)
    const uint32_t ld_row = lane >> 4, ld_chunk = lane & 15;
    const uint8_t *w_src = W + ld_row * pitch + 16 * ld_chunk;
    uint32_t a_row[SLABS][SK_LOADS];
#pragma unroll
    for (int sl = 0; sl < SLABS; ++sl)
#pragma unroll
        for (int i = 0; i < SK_LOADS; ++i) a_row[sl][i] = 32 * sl + 4 * i + ld_row < m ? 32 * sl + 4 * i + ld_row : m - 1;
    struct Tile {
        u32x4 w[SK_LOADS], a[SLABS][SK_LOADS];
    };
    auto load = [&](Tile &t, uint32_t kt) {
#pragma unroll
        for (int i = 0; i < SK_LOADS; ++i)
            t.w[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(w_src + 4 * i * pitch + kt * 256));
#pragma unroll
        for (int sl = 0; sl < SLABS; ++sl)
#pragma unroll
            for (int i = 0; i < SK_LOADS; ++i)
                t.a[sl][i] = *reinterpret_cast<const u32x4 *>(A + a_row[sl][i] * pitch + 16 * ld_chunk + kt * 256);
    };
    // fragment of k-step ks: row lane % 32, chunk 2 ks + lane / 32
    const uint32_t r = lane & 31, h = lane >> 5;
    const uint32_t f_off = r * 256 + 16 * (h ^ (r & 15));
    uint8_t *mine = lds + wave * WAVE_LDS;

    f16v acc0[SLABS], acc1[SLABS];
#pragma unroll
    for (int sl = 0; sl < SLABS; ++sl)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc0[sl][e] = acc1[sl][e] = 0.f;
    auto multiply = [&](const Tile &t) {
#pragma unroll
        for (int i = 0; i < SK_LOADS; ++i) {
            const uint32_t row = 4 * i + ld_row, off = row * 256 + 16 * (ld_chunk ^ (row & 15));
            *reinterpret_cast<u32x4 *>(mine + off) = t.w[i];
#pragma unroll
            for (int sl = 0; sl < SLABS; ++sl) *reinterpret_cast<u32x4 *>(mine + 8192 * (1 + sl) + off) = t.a[sl][i];
        }
#pragma unroll
        for (int ks = 0; ks < SK_TK / 16; ks += 2) {
            const u32x4 w0 = *reinterpret_cast<const u32x4 *>(mine + (f_off ^ (32 * ks)));
            const u32x4 w1 = *reinterpret_cast<const u32x4 *>(mine + (f_off ^ (32 * (ks + 1))));
#pragma unroll
            for (int sl = 0; sl < SLABS; ++sl) {
                const u32x4 a0 = *reinterpret_cast<const u32x4 *>(mine + 8192 * (1 + sl) + (f_off ^ (32 * ks)));
                const u32x4 a1 = *reinterpret_cast<const u32x4 *>(mine + 8192 * (1 + sl) + (f_off ^ (32 * (ks + 1))));
                acc0[sl] = Mfma<T>::run(w0, a0, acc0[sl]);
                acc1[sl] = Mfma<T>::run(w1, a1, acc1[sl]);
            }
        }
    };

    // No branch around a load while the ring is full: with loads under a branch the compiler's wait for one tile
    // becomes a wait for every tile in flight.  The first loads take the last tile again where the wavefront has
    // fewer than SK_DEPTH of them; the branches are left to the last two rounds.
    Tile tile[SK_DEPTH];
    if (t0 < t1) {
#pragma unroll
        for (int i = 0; i < SK_DEPTH; ++i) load(tile[i], t0 + i < t1 ? t0 + i : t1 - 1);
        uint32_t t = t0;
        for (; t + 2 * SK_DEPTH <= t1; t += SK_DEPTH) {
#pragma unroll
            for (int i = 0; i < SK_DEPTH; ++i) {
                multiply(tile[i]);
                load(tile[i], t + i + SK_DEPTH);
            }
        }
        for (; t < t1; t += SK_DEPTH) {
#pragma unroll
            for (int i = 0; i < SK_DEPTH; ++i) {
                if (t + i < t1) {
                    multiply(tile[i]);
                    if (t + i + SK_DEPTH < t1) load(tile[i], t + i + SK_DEPTH);
                }
            }
        }
    }

    // partial sums: lane holds row (lane % 32) of A, register e column 8 (e/4) + 4 (lane/32) + e%4 of the block
    float *part = reinterpret_cast<float *>(lds + 4 * WAVE_LDS);  // [wave][row of A][column], pitch 33
#pragma unroll
    for (int sl = 0; sl < SLABS; ++sl)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const uint32_t col = 8 * (e / 4) + 4 * h + (e % 4);
            part[(wave * 32 * SLABS + 32 * sl + r) * 33 + col] = acc0[sl][e] + acc1[sl][e];
        }
    __syncthreads();
    const T *C = static_cast<const T *>(bias.ptr);
#pragma unroll
    for (int q = 0; q < 4 * SLABS; ++q) {
        const uint32_t idx = tid + 256 * q, row = idx / 32, col = idx % 32;
        if (row < m) {
            float v = 0.f;
#pragma unroll
            for (int wv = 0; wv < 4; ++wv) v += part[(wv * 32 * SLABS + row) * 33 + col];
            v *= alpha;
            const uint64_t yrow = row_first + row;
            if (C) v += beta * up(C[ym * bias.sb + yrow * bias.sm + (n0 + col) * bias.sn]);
            y[(ym * m_total + yrow) * n + n0 + col] = down<T>(v);
        }
    }
}

// ---------------------------------------------------------------- two to sixteen rows of A: blocks of k
//
// Y[m, n] = alpha * A[m, k] @ W[n, k]^T (+ bias) for m <= 16, FP16 / BF16, with operands that need no pass through
// LDS.  v_mfma_f32_4x4x4 multiplies sixteen independent 4x4 blocks; here the sixteen blocks stand for sixteen
// pieces of k.  Lane l holds row l % 4 of a group of four rows and the eight elements of k-piece l / 4, so one
// 128-bit load per lane (four rows of 256 contiguous bytes per instruction) is already the operand of two
// instructions, for W (rows of W as the first operand) and for A (rows of A as the second) alike.  A workgroup
// owns 16 rows of W, its wavefronts each a share of k; a wavefront keeps 4 x G accumulators of four registers
// (rows of W 4 r + register index, row of A 4 g + l % 4, block l / 4) and streams steps of 128 k, DEPTH ahead.
// At the end the sixteen blocks are added by two halving lane swaps and two rotations inside the 16-lane rows,
// and the wavefronts' sums meet in LDS.  Every workgroup reads all of A from L2, and that traffic adds to the
// time: beyond 16 rows of A the kernel above, with half as many workgroups, is faster.
typedef float f4v __attribute__((ext_vector_type(4)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
// Block products on a 128-bit piece of each operand (the sixteen blocks are sixteen pieces of k): PARTS
// instructions, part q on the q-th share of the piece.
template <class T> struct Mfma4;
template <> struct Mfma4<__half> {
    static constexpr int PARTS = 2;
    template <int Q> static __device__ __forceinline__ f4v part(const u32x4 &a, const u32x4 &b, f4v c) {
        return __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(h4, u32x2{a[2 * Q], a[2 * Q + 1]}),
                                                  __builtin_bit_cast(h4, u32x2{b[2 * Q], b[2 * Q + 1]}), c, 0, 0, 0);
    }
    static __device__ __forceinline__ f4v run(u32x2 a, u32x2 b, f4v c) {
        return __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(h4, a), __builtin_bit_cast(h4, b), c, 0, 0, 0);
    }
};
template <> struct Mfma4<__hip_bfloat16> {
    static constexpr int PARTS = 2;
    template <int Q> static __device__ __forceinline__ f4v part(const u32x4 &a, const u32x4 &b, f4v c) {
        return __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(s4, u32x2{a[2 * Q], a[2 * Q + 1]}),
                                                      __builtin_bit_cast(s4, u32x2{b[2 * Q], b[2 * Q + 1]}), c, 0, 0, 0);
    }
    static __device__ __forceinline__ f4v run(u32x2 a, u32x2 b, f4v c) {
        return __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(s4, a), __builtin_bit_cast(s4, b), c, 0, 0, 0);
    }
};
template <> struct Mfma4<float> {  // v_mfma_f32_4x4x1_16B_f32: one k per block and instruction
    static constexpr int PARTS = 4;
    template <int Q> static __device__ __forceinline__ f4v part(const u32x4 &a, const u32x4 &b, f4v c) {
        // (elements copied into scalars first: reinterpreting a vector element in place reads element 0)
        const uint32_t ua = a[Q], ub = b[Q];
        return __builtin_amdgcn_mfma_f32_4x4x1f32(__builtin_bit_cast(float, ua), __builtin_bit_cast(float, ub), c, 0, 0, 0);
    }
};
// lanes 0-31 receive lo_keeps summed over both halves of the wavefront, lanes 32-63 hi_keeps
__device__ __forceinline__ float swap32_sum(float lo_keeps, float hi_keeps) {
    const auto r = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(uint32_t, lo_keeps),
                                                    __builtin_bit_cast(uint32_t, hi_keeps), false, false);
    const uint32_t r0 = r[0], r1 = r[1];
    return __builtin_bit_cast(float, r0) + __builtin_bit_cast(float, r1);
}
// the same between neighbouring rows of 16 lanes: even rows receive even_keeps, odd rows odd_keeps
__device__ __forceinline__ float swap16_sum(float even_keeps, float odd_keeps) {
    const auto r = __builtin_amdgcn_permlane16_swap(__builtin_bit_cast(uint32_t, even_keeps),
                                                    __builtin_bit_cast(uint32_t, odd_keeps), false, false);
    const uint32_t r0 = r[0], r1 = r[1];
    return __builtin_bit_cast(float, r0) + __builtin_bit_cast(float, r1);
}

template <class T, int G, int WAVES, int DEPTH>  // G groups of four rows of A
__global__ __launch_bounds__(64 * WAVES) void mm_rows(T *__restrict__ y, const T *__restrict__ a, const T *__restrict__ w,
                                                      Bias bias, uint32_t m, uint32_t m_total, uint32_t row_first, uint32_t k,
                                                      uint32_t n, float alpha, float beta, uint32_t a_matrix0,
                                                      uint32_t b_matrix0, uint32_t y_matrix0) {
    // rows row_first .. row_first + m - 1 of each m_total-row matrix
    constexpr int ROWS = 4 * G, PITCH = 20;  // floats per row of a partial block [row of A][16 columns]
    __shared__ __align__(16) float part[WAVES * ROWS * PITCH];
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t bz = blockIdx.z;
    const uint64_t am = a_matrix0 + bz, bm = b_matrix0 + bz, ym = y_matrix0 + bz;
    const uint32_t n0 = blockIdx.x * 16;
    const uint32_t pitch = sizeof(T) * k;
    const uint8_t *W = reinterpret_cast<const uint8_t *>(w + (bm * n + n0) * static_cast<uint64_t>(k));
    const uint8_t *A = reinterpret_cast<const uint8_t *>(a + (am * m_total + row_first) * static_cast<uint64_t>(k));
    const uint32_t steps = pitch / 256;  // a step is 256 bytes of every row: 128 or (float) 64 k
    const uint32_t s0 = steps * wave / WAVES, s1 = steps * (wave + 1) / WAVES, cnt = s1 - s0;
    const uint32_t i4 = lane & 3, blk = lane >> 2;
    uint32_t w_off[4], a_off[G];
#pragma unroll
    for (int r = 0; r < 4; ++r) w_off[r] = (4 * r + i4) * pitch + 16 * blk + 256 * s0;
#pragma unroll
    for (int g = 0; g < G; ++g) a_off[g] = (4 * g + i4 < m ? 4 * g + i4 : m - 1) * pitch + 16 * blk + 256 * s0;
    struct Step {
        u32x4 w[4], a[G];
    };
    auto load = [&](Step &t, uint32_t j) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
            t.w[r] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(W + (w_off[r] + 256 * j)));
#pragma unroll
        for (int g = 0; g < G; ++g) t.a[g] = *reinterpret_cast<const u32x4 *>(A + (a_off[g] + 256 * j));
    };
    f4v acc[4][G];
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int g = 0; g < G; ++g) acc[r][g] = f4v{0.f, 0.f, 0.f, 0.f};
    auto multiply = [&](const Step &t) {
        auto sweep = [&]<int Q>() __attribute__((always_inline)) {
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int g = 0; g < G; ++g) acc[r][g] = Mfma4<T>::template part<Q>(t.w[r], t.a[g], acc[r][g]);
        };
        sweep.template operator()<0>();
        sweep.template operator()<1>();
        if constexpr (Mfma4<T>::PARTS == 4) {
            sweep.template operator()<2>();
            sweep.template operator()<3>();
        }
    };
    Step st[DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d)
        if (d < cnt) load(st[d], d);
    for (uint32_t j = 0; j < cnt; j += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            if (j + d < cnt) {
                multiply(st[d]);
                if (j + d + DEPTH < cnt) load(st[d], j + d + DEPTH);
            }
        }
    }
    // The sixteen blocks of a register hold sixteen parts of k.  Two halving exchanges leave a lane with the sums
    // over the four rows of 16 lanes, for the rows of W 4 rr .. 4 rr + 3; two rotations inside the row of lanes
    // add the four blocks that are left.
    const uint32_t rr = 2 * (lane >> 5) + ((lane >> 4) & 1);
#pragma unroll
    for (int g = 0; g < G; ++g) {
        f4v t;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float u0 = swap32_sum(acc[0][g][e], acc[2][g][e]);
            const float u1 = swap32_sum(acc[1][g][e], acc[3][g][e]);
            float v = swap16_sum(u0, u1);
            v += dpp_f32<0x124>(v);  // row_ror:4
            v += dpp_f32<0x128>(v);  // row_ror:8
            t[e] = v;
        }
        if ((blk & 3) == 0) *reinterpret_cast<f4v *>(part + (wave * ROWS + 4 * g + i4) * PITCH + 4 * rr) = t;
    }
    __syncthreads();
    const T *C = static_cast<const T *>(bias.ptr);
    for (uint32_t idx = tid; idx < ROWS * 16; idx += 64 * WAVES) {
        const uint32_t row = idx >> 4, col = idx & 15;
        if (row < m) {
            float v = 0.f;
#pragma unroll
            for (int p = 0; p < WAVES; ++p) v += part[(p * ROWS + row) * PITCH + col];
            v *= alpha;
            const uint64_t yrow = row_first + row;
            if (C) v += beta * up(C[ym * bias.sb + yrow * bias.sm + (n0 + col) * bias.sn]);
            y[(ym * m_total + yrow) * n + n0 + col] = down<T>(v);
        }
    }
}

// ---------------------------------------------------------------- up to 32 rows of A, weights as [k, n]: blocks of k
//
// The same block products with the weights as ONNX MatMul stores them, B [k, n]: Y[rows <= 32, n] = alpha * A @ B
// (+ bias).  The contraction index runs down the columns of B, so a lane cannot load an operand (four
// consecutive k of one column) in one piece; it loads CW columns of eight consecutive k-rows (eight loads of 8 or
// 16 bytes; four lanes cover a strip of 4 CW columns, the sixteen blocks sixteen groups of eight k-rows) and
// transposes them in registers, two byte permutes per operand.  A (rows of A as the first operand) is loaded as
// in mm_rows.  A workgroup owns a strip and all of k, its wavefronts a share of k each, so no sums cross
// workgroups: strips of 16 columns (32-byte pieces of a row of B) where that is needed to cover the chip, of 32
// columns for wide B.  Strips are numbered so that neighbours, which share 128-byte lines, run on the same XCD.
// More than 32 rows take several passes over B.
template <int BYTES> struct ColumnWord;  // CW columns of one k-row
template <> struct ColumnWord<8> { typedef u32x2 type; };
template <> struct ColumnWord<16> { typedef u32x4 type; };

template <class T, int G, int WAVES, int CW>  // G groups of four rows of A; CW columns per lane (4 or 8)
__global__ __launch_bounds__(64 * WAVES) void mm_rows_kn(T *__restrict__ y, const T *__restrict__ a, const T *__restrict__ b,
                                                         Bias bias, uint32_t m, uint32_t m_total, uint32_t row_first, uint32_t k,
                                                         uint32_t n, float alpha, float beta, uint32_t a_matrix0,
                                                         uint32_t b_matrix0, uint32_t y_matrix0) {
    constexpr int ROWS = 4 * G, SW = 4 * CW, PITCH = SW + 1;  // strip width; floats per row of a partial block
    constexpr int DEPTH = 2;  // steps of 128 k in flight
    constexpr bool F32 = sizeof(T) == 4;  // floats: four columns per lane, one k per block and instruction, no transposition
    static_assert(!F32 || CW == 4, "floats come four columns to a lane");
    constexpr int AW = F32 ? 2 : 1;       // 128-bit pieces of a row of A per step: eight k
    typedef typename ColumnWord<sizeof(T) * CW>::type Word;
    __shared__ float part[WAVES * ROWS * PITCH];
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t bz = blockIdx.z;
    const uint64_t am = a_matrix0 + bz, bm = b_matrix0 + bz, ym = y_matrix0 + bz;
    uint32_t strip = blockIdx.x;
    if (gridDim.x % 8 == 0) strip = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
    const uint32_t n0 = strip * SW;
    const uint32_t pitch_a = sizeof(T) * k, pitch_b = sizeof(T) * n;
    const uint8_t *B = reinterpret_cast<const uint8_t *>(b + bm * k * static_cast<uint64_t>(n) + n0);
    const uint8_t *A = reinterpret_cast<const uint8_t *>(a + (am * m_total + row_first) * static_cast<uint64_t>(k));
    const uint32_t steps = k / 128;
    const uint32_t s0 = steps * wave / WAVES, s1 = steps * (wave + 1) / WAVES, cnt = s1 - s0;
    const uint32_t j4 = lane & 3, blk = lane >> 2;
    // this lane: k-rows 128 s + 8 blk .. + 7, columns n0 + CW j4 .. + CW - 1 of B; rows 4 g + j4 of A at the same k
    const uint32_t b_off = (128 * s0 + 8 * blk) * pitch_b + sizeof(T) * CW * j4;
    uint32_t a_off[G];
#pragma unroll
    for (int g = 0; g < G; ++g)
        a_off[g] = (4 * g + j4 < m ? 4 * g + j4 : m - 1) * pitch_a + 16 * AW * blk + 256 * AW * s0;
    struct Step {
        Word w[8];
        u32x4 a[G][AW];
    };
    auto load = [&](Step &t, uint32_t j) {
#pragma unroll
        for (int r = 0; r < 8; ++r)
            t.w[r] = __builtin_nontemporal_load(reinterpret_cast<const Word *>(B + (b_off + (128 * j + r) * pitch_b)));
#pragma unroll
        for (int g = 0; g < G; ++g)
#pragma unroll
            for (int x = 0; x < AW; ++x) t.a[g][x] = *reinterpret_cast<const u32x4 *>(A + (a_off[g] + 256 * AW * j + 16 * x));
    };
    f4v acc[CW][G];
#pragma unroll
    for (int c = 0; c < CW; ++c)
#pragma unroll
        for (int g = 0; g < G; ++g) acc[c][g] = f4v{0.f, 0.f, 0.f, 0.f};
    auto multiply = [&](const Step &t) {
        if constexpr (F32) {
#pragma unroll
            for (int r = 0; r < 8; ++r)
#pragma unroll
                for (int c = 0; c < CW; ++c) {
                    const uint32_t wv = t.w[r][c];
#pragma unroll
                    for (int g = 0; g < G; ++g) {
                        const uint32_t av = t.a[g][r / 4][r % 4];
                        acc[c][g] = __builtin_amdgcn_mfma_f32_4x4x1f32(__builtin_bit_cast(float, av), __builtin_bit_cast(float, wv),
                                                                       acc[c][g], 0, 0, 0);
                    }
                }
        } else {
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            // four k-rows of CW columns become CW columns of four k
            u32x2 col[CW];
#pragma unroll
            for (int p = 0; p < CW / 2; ++p) {
                const uint32_t d0 = t.w[4 * q][p], d1 = t.w[4 * q + 1][p], d2 = t.w[4 * q + 2][p], d3 = t.w[4 * q + 3][p];
                col[2 * p] = u32x2{__builtin_amdgcn_perm(d1, d0, 0x05040100u), __builtin_amdgcn_perm(d3, d2, 0x05040100u)};
                col[2 * p + 1] = u32x2{__builtin_amdgcn_perm(d1, d0, 0x07060302u), __builtin_amdgcn_perm(d3, d2, 0x07060302u)};
            }
#pragma unroll
            for (int c = 0; c < CW; ++c)
#pragma unroll
                for (int g = 0; g < G; ++g)
                    acc[c][g] = Mfma4<T>::run(u32x2{t.a[g][0][2 * q], t.a[g][0][2 * q + 1]}, col[c], acc[c][g]);
        }
        }
    };
    Step st[DEPTH];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d)
        if (d < cnt) load(st[d], d);
    for (uint32_t j = 0; j < cnt; j += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            if (j + d < cnt) {
                multiply(st[d]);
                if (j + d + DEPTH < cnt) load(st[d], j + d + DEPTH);
            }
        }
    }
    // sixteen blocks = sixteen parts of k: two halving swaps leave a lane with the columns
    // (CW / 4) (2 (lane / 32) + (lane / 16) % 2) + x of its CW, two rotations inside the 16-lane row add the four
    // blocks that remain
    constexpr int Q = CW / 4;
    const uint32_t cc = Q * (2 * (lane >> 5) + ((lane >> 4) & 1));
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
        for (int e = 0; e < 4; ++e)
#pragma unroll
            for (int x = 0; x < Q; ++x) {
                const float u0 = swap32_sum(acc[x][g][e], acc[2 * Q + x][g][e]);
                const float u1 = swap32_sum(acc[Q + x][g][e], acc[3 * Q + x][g][e]);
                float v = swap16_sum(u0, u1);
                v += dpp_f32<0x124>(v);  // row_ror:4
                v += dpp_f32<0x128>(v);  // row_ror:8
                if ((blk & 3) == 0) part[(wave * ROWS + 4 * g + e) * PITCH + CW * j4 + cc + x] = v;
            }
    __syncthreads();
    const T *C = static_cast<const T *>(bias.ptr);
    for (uint32_t idx = tid; idx < ROWS * SW; idx += 64 * WAVES) {
        const uint32_t row = idx / SW, col = idx % SW;
        if (row < m) {
            float v = 0.f;
#pragma unroll
            for (int p = 0; p < WAVES; ++p) v += part[(p * ROWS + row) * PITCH + col];
            v *= alpha;
            const uint64_t yrow = row_first + row;
            if (C) v += beta * up(C[ym * bias.sb + yrow * bias.sm + (n0 + col) * bias.sn]);
            y[(ym * m_total + yrow) * n + n0 + col] = down<T>(v);
        }
    }
}

// ---------------------------------------------------------------- one to four rows of A: matrix-vector products
//
// Y[m, n] = alpha * A[m, k] @ W[n, k]^T (+ bias) for m <= 4, FP16 / BF16.  A matrix core would spend
// 32 rows of work on these few, so the products are formed by the vector ALUs instead and the
// kernel is a plain stream over W: a wavefront owns R rows of W, a lane reads 16 bytes (8
// elements) of each per step, GV_LOADS / R steps ahead, and multiplies them (two elements per
// instruction, sums in FP32) with the matching 8 elements of every row of A, which the
// workgroup keeps in LDS (consecutive lanes read consecutive 16 bytes; at most 64 KiB, a longer k
// is walked in segments).  The 64 partial sums
// of a row meet in a butterfly of lane exchanges at the end.  The first loads of W are issued
// before A is staged, so the copy of A costs no memory latency of its own.
constexpr int GV_LOADS = 8;  // 128-bit loads in flight per lane

// acc + w.x * a.x + w.y * a.y on a pair of 16-bit elements held in one register (v_dot2_f32_f16 / v_dot2_f32_bf16)
template <class T> __device__ __forceinline__ float dot2(uint32_t w, uint32_t a, float acc);
template <> __device__ __forceinline__ float dot2<__half>(uint32_t w, uint32_t a, float acc) {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, w), __builtin_bit_cast(h2, a), acc, false);
}
template <> __device__ __forceinline__ float dot2<__hip_bfloat16>(uint32_t w, uint32_t a, float acc) {
    typedef __bf16 b2 __attribute__((ext_vector_type(2)));
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(b2, w), __builtin_bit_cast(b2, a), acc, false);
}

template <class T, int M, int R, bool LONG>  // LONG: k in more than one segment
__global__ __launch_bounds__(1024) void mm_gemv(T *__restrict__ y, const T *__restrict__ a, const T *__restrict__ w,
                                               Bias bias, uint32_t m, uint32_t k, uint32_t n, uint32_t segment, float alpha,
                                               float beta, uint32_t a_matrix0, uint32_t b_matrix0, uint32_t y_matrix0) {
    constexpr int DEPTH = GV_LOADS / R;  // steps of loads in flight
    extern __shared__ __align__(16) uint8_t gv_lds[];  // M rows of A, one segment of k each
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t bz = blockIdx.z;
    const uint64_t am = a_matrix0 + bz, bm = b_matrix0 + bz, ym = y_matrix0 + bz;
    const uint32_t pieces = k / 8;  // 16-byte pieces of a row
    // A workgroup walks several blocks of rows of W when there are more blocks than the launch has workgroups (a
    // vocabulary's worth of rows): A is copied into LDS once, not once per 16 rows (the short-lived workgroups of
    // one block each left [1,4096] x [32000,4096]^T at 2.7 TB/s).
    const uint32_t row_blocks = (n + (blockDim.x / 64) * R - 1) / ((blockDim.x / 64) * R);
    bool a_in_lds = false;
    for (uint32_t rb = blockIdx.x; rb < row_blocks; rb += gridDim.x) {
    const uint32_t row0 = (rb * (blockDim.x / 64) + wave) * R;

    const u32x4 *W[R];
#pragma unroll
    for (int j = 0; j < R; ++j) {
        const uint32_t row = row0 + j < n ? row0 + j : n - 1;  // rows beyond n repeat the last one and are not stored
        W[j] = reinterpret_cast<const u32x4 *>(w + (bm * n + row) * static_cast<uint64_t>(k));
    }
    const u32x4 *A = reinterpret_cast<const u32x4 *>(a + am * m * static_cast<uint64_t>(k));
    u32x4 *sa = reinterpret_cast<u32x4 *>(gv_lds);
    float acc[R][M];
#pragma unroll
    for (int j = 0; j < R; ++j)
#pragma unroll
        for (int i = 0; i < M; ++i) acc[j][i] = 0.f;

    // k in segments of which M rows of A fit into LDS (one segment unless k is very long; that case is compiled
    // without the loop, which costs a fifth of the speed)
    uint32_t p0 = 0;
    do {
        const uint32_t len = !LONG ? pieces : pieces - p0 < segment ? pieces - p0 : segment;
        const uint32_t steps = (len + 63) / 64;  // a wavefront covers 64 pieces per step
        u32x4 buf[DEPTH][R];
        // No branch around a load (with one, the compiler's wait for one step becomes a wait for every step in flight):
        // lanes and steps beyond the row's end fetch its last piece again and are left out of the products.
        auto load = [&](int slot, uint32_t step) {
            step = step < steps ? step : steps - 1;
            uint32_t c = step * 64 + lane;
            c = c < len ? c : len - 1;
#pragma unroll
            for (int j = 0; j < R; ++j) buf[slot][j] = __builtin_nontemporal_load(W[j] + p0 + c);
        };
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) load(d, d);

        // A into LDS while the first pieces of W are on their way; rows beyond m are zero
        if (LONG || !a_in_lds) {
            if (LONG && (p0 || a_in_lds)) __syncthreads();  // everybody has finished with the segment before
#pragma unroll
            for (int i = 0; i < M; ++i)
                for (uint32_t c = tid; c < len; c += blockDim.x) {
                    u32x4 v = {0u, 0u, 0u, 0u};
                    if (static_cast<uint32_t>(i) < m) v = A[static_cast<uint64_t>(i) * pieces + p0 + c];
                    sa[i * len + c] = v;
                }
            __syncthreads();
            a_in_lds = true;
        }

        auto multiply = [&](int d, uint32_t step) {
            const uint32_t c = step * 64 + lane;
            if (step < steps && c < len) {
#pragma unroll
                for (int i = 0; i < M; ++i) {
                    const u32x4 av = sa[i * len + c];
#pragma unroll
                    for (int j = 0; j < R; ++j)
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc[j][i] = dot2<T>(buf[d][j][e], av[e], acc[j][i]);
                }
            }
        };
        auto last_round = [&](uint32_t s) {
#pragma unroll
            for (int d = 0; d < DEPTH; ++d) multiply(d, s + d);
        };
        uint32_t s = 0;
        for (; s + 2 * DEPTH <= steps; s += DEPTH) {  // the ring stays full
#pragma unroll
            for (int d = 0; d < DEPTH; ++d) {
                multiply(d, s + d);
                load(d, s + d + DEPTH);
            }
        }
        if (s + DEPTH < steps) {  // one more round with loads (some of them beyond the end), then the last one
#pragma unroll
            for (int d = 0; d < DEPTH; ++d) {
                multiply(d, s + d);
                load(d, s + d + DEPTH);
            }
            last_round(s + DEPTH);
        } else {
            last_round(s);
        }
    } while (LONG && (p0 += segment) < pieces);

    // every lane ends with all sums; lane j * M + i keeps and stores the one of (row j of W, row i of A)
    float mine = 0.f;
#pragma unroll
    for (int j = 0; j < R; ++j)
#pragma unroll
        for (int i = 0; i < M; ++i) {
            float v = acc[j][i];
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
            if (lane == static_cast<uint32_t>(j * M + i)) mine = v;
        }
    if (lane < R * M) {
        const uint32_t j = lane / M, i = lane % M, col = row0 + j;
        if (col < n && i < m) {
            float v = alpha * mine;
            const T *C = static_cast<const T *>(bias.ptr);
            if (C) v += beta * up(C[ym * bias.sb + i * bias.sm + col * bias.sn]);
            y[(ym * m + i) * n + col] = down<T>(v);
        }
    }
    }  // row blocks
}

// ---------------------------------------------------------------- one to four rows of A, B as [k, n]
//
// Y[m <= 4, n] = alpha * A[m, k] @ B[k, n] (+ bias), FP16 / BF16, for weights kept the way ONNX MatMul
// has them.  The sum runs down the columns of B, so a lane owns 8 columns (one 128-bit load per
// k-row) and L lanes cover a strip of 8 L columns; the 64 / L lane groups of a wavefront and the 16
// wavefronts of a workgroup take different k-rows, 8 loads per lane in flight.  A workgroup walks
// all of k for its strip, so the sums need no atomics and no workspace and come out in a fixed
// order: FP32 FMAs per lane, an exchange between the lane groups, then the 16 wavefronts' sums added
// in order through LDS.  A (4096 k at a time) sits in LDS as it is in memory.  Strips narrower than
// a 128-byte line (L < 8) share lines with their neighbours: workgroups are dealt to the eight XCDs
// in turn, so the strips are numbered such that neighbours run on the same XCD at the same time and
// the second one finds the line in that XCD's L2.
constexpr int KN_SEG = 4096;  // k per segment of A in LDS
constexpr int KN_DEPTH = 8;   // loads in flight per lane

template <class T> __device__ __forceinline__ void widen8(const u32x4 &c, float (&f)[8]);
template <> __device__ __forceinline__ void widen8<__half>(const u32x4 &c, float (&f)[8]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t v = c[j];
        const __half2 h = *reinterpret_cast<const __half2 *>(&v);
        f[2 * j] = __low2float(h);
        f[2 * j + 1] = __high2float(h);
    }
}
template <> __device__ __forceinline__ void widen8<__hip_bfloat16>(const u32x4 &c, float (&f)[8]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        f[2 * j] = __uint_as_float(c[j] << 16);
        f[2 * j + 1] = __uint_as_float(c[j] & 0xffff0000u);
    }
}

template <class T, int M, int L>
__global__ __launch_bounds__(1024) void mm_gemv_kn(T *__restrict__ y, const T *__restrict__ a, const T *__restrict__ b,
                                                  Bias bias, uint32_t m, uint32_t k, uint32_t n, float alpha, float beta,
                                                  uint32_t a_matrix0, uint32_t b_matrix0, uint32_t y_matrix0, uint32_t row0,
                                                  uint32_t rows) {
    // rows row0 .. row0 + rows - 1 (rows <= M) of each m-row matrix
    constexpr int G = 64 / L, SW = 8 * L;  // lane groups per wavefront, columns per strip
    constexpr int A_BYTES = M * KN_SEG * 2, P_BYTES = 16 * M * SW * 4;
    __shared__ __align__(16) uint8_t lds[A_BYTES > P_BYTES ? A_BYTES : P_BYTES];
    T(*sa)[KN_SEG] = reinterpret_cast<T(*)[KN_SEG]>(lds);  // rows of A, one segment of k
    float *part = reinterpret_cast<float *>(lds);          // afterwards: [wavefront][row of A][column of the strip]
    const uint32_t tid = threadIdx.x, lane = tid & 63, c = lane % L, g = lane / L;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t bz = blockIdx.z;
    const uint64_t am = a_matrix0 + bz, bm = b_matrix0 + bz, ym = y_matrix0 + bz;
    uint32_t strip = blockIdx.x;
    if (gridDim.x % 8 == 0) strip = (blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3);
    const uint32_t col0 = strip * SW + 8 * c;  // this lane's 8 columns
    const bool live = col0 < n;
    const T *B = b + bm * k * static_cast<uint64_t>(n) + col0;
    const T *A = a + (am * m + row0) * static_cast<uint64_t>(k);

    float acc[M][8];
#pragma unroll
    for (int i = 0; i < M; ++i)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[i][e] = 0.f;

    for (uint32_t k0 = 0; k0 < k; k0 += KN_SEG) {
        const uint32_t len = k - k0 < KN_SEG ? k - k0 : KN_SEG;
        const uint32_t steps = (len + 16 * G - 1) / (16 * G);  // the workgroup covers 16 G k-rows per step
        // step s: this lane reads k-row k0 + (16 s + wave) G + g
        // A first (the loads return in order, so the wait for A leaves the loads of B in flight): the two
        // halves of the workgroup take rows 0, 2 and 1, 3, a thread 16 bytes of each of its rows
        constexpr int ROWS = (M + 1) / 2;
        const uint32_t ap = 8 * (tid & 511), ai = tid >> 9;
        u32x4 av[ROWS];
#pragma unroll
        for (int j = 0; j < ROWS; ++j) {
            av[j] = u32x4{0u, 0u, 0u, 0u};  // rows beyond the last are zero
            if (2 * j + ai < rows && ap < len) av[j] = *reinterpret_cast<const u32x4 *>(A + static_cast<uint64_t>(2 * j + ai) * k + k0 + ap);
        }
        u32x4 buf[KN_DEPTH];
        auto load = [&](int slot, uint32_t step) {
            const uint32_t r = (16 * step + wave) * G + g;
            if (live && r < len) buf[slot] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(B + static_cast<uint64_t>(k0 + r) * n));
        };
#pragma unroll
        for (int d = 0; d < KN_DEPTH; ++d)
            if (static_cast<uint32_t>(d) < steps) load(d, d);

        if (k0) __syncthreads();  // everybody has finished with the segment before
#pragma unroll
        for (int j = 0; j < ROWS; ++j)
            if (2 * j + ai < M && ap < len) *reinterpret_cast<u32x4 *>(&sa[2 * j + ai][ap]) = av[j];
        __syncthreads();

        for (uint32_t s = 0; s < steps; s += KN_DEPTH) {
#pragma unroll
            for (int d = 0; d < KN_DEPTH; ++d) {
                if (s + d < steps) {
                    const uint32_t r = (16 * (s + d) + wave) * G + g;
                    if (live && r < len) {
                        float wf[8];
                        widen8<T>(buf[d], wf);
#pragma unroll
                        for (int i = 0; i < M; ++i) {
                            const float ai = up(sa[i][r]);
#pragma unroll
                            for (int e = 0; e < 8; ++e) acc[i][e] = fmaf(wf[e], ai, acc[i][e]);
                        }
                    }
                    if (s + d + KN_DEPTH < steps) load(d, s + d + KN_DEPTH);
                }
            }
        }
    }

    // The lane groups of a wavefront (lane bits from L up), then the wavefronts in order.  While a lane
    // still holds more than one sum, a stage halves them: the lane keeps the lower or the upper half (by its
    // lane bit) and gets the partner's share of that half, so V sums cost about V exchanges, not V log2 G;
    // from one sum per lane on, both partners add and hold the same.
    constexpr int V = M * 8;
    float *v = &acc[0][0];
    uint32_t first = 0, twin = 0;  // the lane ends with sums first .. ; twin != 0: another lane writes them
#pragma unroll
    for (int t = 0; (L << t) < 64; ++t) {
        const int off = L << t;
        const int nv = (V >> t) > 1 ? (V >> t) : 1;
        if (nv > 1) {
            const int half = nv / 2;
            const bool hi = lane & off;
#pragma unroll
            for (int j = 0; j < half; ++j) {
                const float keep = hi ? v[j + half] : v[j];
                const float send = hi ? v[j] : v[j + half];
                v[j] = keep + __shfl_xor(send, off, 64);
            }
            if (hi) first += half;
        } else {
            v[0] += __shfl_xor(v[0], off, 64);
            twin |= lane & off;
        }
    }
    constexpr int STAGES = __builtin_ctz(64 / L);
    constexpr int LEFT = (V >> STAGES) > 1 ? (V >> STAGES) : 1;  // sums a lane holds at the end
    __syncthreads();  // A is no longer read
    if (!twin) {
#pragma unroll
        for (int j = 0; j < LEFT; ++j) {
            const uint32_t f = first + j;  // sum f: row f / 8 of A, column f % 8 of the lane's eight
            part[(wave * M + f / 8) * SW + 8 * c + f % 8] = v[j];
        }
    }
    __syncthreads();
    for (uint32_t t = tid; t < M * SW; t += 1024) {
        const uint32_t i = t / SW, cc = t % SW, col = strip * SW + cc;
        if (i < rows && col < n) {
            float v = 0.f;
#pragma unroll
            for (int wv = 0; wv < 16; ++wv) v += part[(wv * M + i) * SW + cc];
            v *= alpha;
            const T *C = static_cast<const T *>(bias.ptr);
            if (C) v += beta * up(C[ym * bias.sb + (row0 + i) * bias.sm + col * bias.sn]);
            y[(ym * m + row0 + i) * n + col] = down<T>(v);
        }
    }
}

// ---------------------------------------------------------------- one to four rows of A, B as [k, n], k shared between workgroups
//
// The kernel above walks all of k in one workgroup, so its strips must be narrow for the launch to cover the chip:
// at n = 4096 a workgroup reads 32 to 128 bytes of every k-row, and runs that short cost DRAM and L2 efficiency
// (one row against [4096, 4096]: 15.5 us where W as [n, k] takes 7).  With a workspace the strip can be wide
// instead: a workgroup takes 256 columns (512 contiguous bytes of a k-row, two k-rows per wavefront load) and a
// share of k, keeps its whole share in flight at once when that is at most 256 k-rows (8 loads per lane), and
// leaves its float sums in the workspace; the workgroup that finds every share of its strip delivered adds the shares
// in their fixed order and stores.  The result therefore does not depend on which workgroup that is.
// (the hand-off, shares_complete below, needs nothing cleared beforehand)
constexpr int KSP_COLS = 256;   // columns of a strip
constexpr int KSP_ROWS = 32;    // k-rows a workgroup's 16 wavefronts load per instruction
constexpr int KSP_DEPTH = 8;    // loads per lane in flight
constexpr int KSP_MAX_KR = 2048;  // k-rows of a share

template <class T, int M>
__global__ __launch_bounds__(1024) void mm_kn_split(T *__restrict__ y, const T *__restrict__ a, const T *__restrict__ b, Bias bias,
                                                   uint32_t m, uint32_t k, uint32_t n, float alpha, float beta, uint32_t kr,
                                                   uint32_t shares, float *__restrict__ part, unsigned long long *__restrict__ sync,
                                                   unsigned long long launch_no) {
    // kr: k-rows per share, a multiple of KSP_ROWS * KSP_DEPTH; k is even
    __shared__ __align__(16) float sums[16 * M * KSP_COLS];  // [wavefront][row of A][column of the strip]
    const uint32_t tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, half = lane >> 5;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t strip = blockIdx.x, share = blockIdx.y;
    const uint32_t col0 = strip * KSP_COLS, k0 = share * kr;
    const uint32_t k_here = k - k0 < kr ? k - k0 : kr;           // k-rows of this share that exist (even)
    const bool live = col0 + 8 * l32 < n;
    const T *bcol = b + (live ? col0 + 8 * l32 : 0);
    const uint32_t my_row = 2 * wave + half;                     // + KSP_ROWS * j

    float acc[M][8];
#pragma unroll
    for (int i = 0; i < M; ++i)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[i][e] = 0.f;

    // The wavefront's two k-rows of a load are neighbours, so their elements of a row of A are one aligned 32-bit
    // word at a wave-uniform address: scalar loads, which neither wait for the loads of B nor make them wait.
    struct Round {
        u32x4 v[KSP_DEPTH];
        uint32_t pa[M][KSP_DEPTH];
    };
    auto load = [&](Round &t, uint32_t base) {
#pragma unroll
        for (int i = 0; i < M; ++i)
#pragma unroll
            for (int j = 0; j < KSP_DEPTH; ++j) {
                const uint32_t r = base + KSP_ROWS * j + 2 * wave;
                const bool have = static_cast<uint32_t>(i) < m && r < k_here;
                const uint32_t word = *reinterpret_cast<const uint32_t *>(a + static_cast<uint64_t>(have ? i : 0) * k + k0 + (have ? r : 0));
                t.pa[i][j] = have ? word : 0u;
            }
#pragma unroll
        for (int j = 0; j < KSP_DEPTH; ++j) {
            // rows beyond the share repeat its last row; their factor from A is zero
            const uint32_t r = base + KSP_ROWS * j + my_row, rr = r < k_here ? r : k_here - 1;
            t.v[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(bcol + static_cast<uint64_t>(k0 + rr) * n));
        }
    };
    auto multiply = [&](const Round &t) {
#pragma unroll
        for (int j = 0; j < KSP_DEPTH; ++j) {
            float f[8];
            widen8<T>(t.v[j], f);
#pragma unroll
            for (int i = 0; i < M; ++i) {
                const uint16_t bits = static_cast<uint16_t>(half ? t.pa[i][j] >> 16 : t.pa[i][j] & 0xffffu);
                const float av = up(__builtin_bit_cast(T, bits));
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[i][e] = fmaf(av, f[e], acc[i][e]);
            }
        }
    };

    constexpr uint32_t STEP = KSP_ROWS * KSP_DEPTH;
    Round r0, r1;
    load(r0, 0);
    for (uint32_t base = 0; base < kr; base += 2 * STEP) {
        const bool more = base + STEP < kr;
        if (more) load(r1, base + STEP);
        multiply(r0);
        if (more) {
            if (base + 2 * STEP < kr) load(r0, base + 2 * STEP);
            multiply(r1);
        }
    }

    // the two halves of a wavefront hold different k-rows of the same columns
#pragma unroll
    for (int i = 0; i < M; ++i)
#pragma unroll
        for (int e = 0; e < 8; e += 2) {
            const float t = swap32_sum(acc[i][e], acc[i][e + 1]);  // lower half: column e, upper half: column e + 1
            sums[(wave * M + i) * KSP_COLS + 8 * l32 + e + half] = t;
        }
    __syncthreads();
    const T *C = static_cast<const T *>(bias.ptr);
    auto finish = [&](uint32_t i, uint32_t col, float v) {
        v *= alpha;
        if (C) v += beta * up(C[i * bias.sm + col * bias.sn]);
        y[static_cast<uint64_t>(i) * n + col] = down<T>(v);
    };
#pragma unroll
    for (int q = 0; q < (M * KSP_COLS + 1023) / 1024; ++q) {
        const uint32_t t = tid + 1024 * q, i = t / KSP_COLS, cc = t % KSP_COLS;
        float v = 0.f;
        if (t < M * KSP_COLS) {
#pragma unroll
            for (int wv = 0; wv < 16; ++wv) v += sums[(wv * M + i) * KSP_COLS + cc];
            if (shares == 1) {
                if (i < m && col0 + cc < n) finish(i, col0 + cc, v);
            } else {
                store_through(part + (static_cast<uint64_t>(strip) * shares + share) * (M * KSP_COLS) + t, v);
            }
        }
    }
    if (shares == 1) return;
    if (!shares_complete(sync + strip, sync + gridDim.x + static_cast<uint64_t>(strip) * shares, share, shares, launch_no, tid)) return;
    const float *strip_part = part + static_cast<uint64_t>(strip) * shares * (M * KSP_COLS);
#pragma unroll
    for (int q = 0; q < (M * KSP_COLS + 1023) / 1024; ++q) {
        const uint32_t t = tid + 1024 * q, i = t / KSP_COLS, cc = t % KSP_COLS;
        if (t < M * KSP_COLS) {
            // eight shares' sums are requested by one piece of assembly that also waits for them (as separate
            // device-scope loads each would be followed by a wait of its own), then added in the shares' order
            float v = 0.f;
            if constexpr (M == 1) {
                // one row of A: the shares' sums are 1 KiB apart, so sixteen of them are four addresses with four
                // immediate offsets each - one request, one wait (a strip's last group may reach into the next
                // strip's sums or the padding behind the last one; those values are not used)
                for (uint32_t sh = 0; sh < shares; sh += 16) {
                    float g[16];
                    const uint32_t o0 = (sh * KSP_COLS + t) * 4, o1 = o0 + 4096, o2 = o0 + 8192, o3 = o0 + 12288;
                    asm volatile("global_load_dword %0, %16, %20 sc1\n\t"
                                 "global_load_dword %1, %16, %20 offset:1024 sc1\n\t"
                                 "global_load_dword %2, %16, %20 offset:2048 sc1\n\t"
                                 "global_load_dword %3, %16, %20 offset:3072 sc1\n\t"
                                 "global_load_dword %4, %17, %20 sc1\n\t"
                                 "global_load_dword %5, %17, %20 offset:1024 sc1\n\t"
                                 "global_load_dword %6, %17, %20 offset:2048 sc1\n\t"
                                 "global_load_dword %7, %17, %20 offset:3072 sc1\n\t"
                                 "global_load_dword %8, %18, %20 sc1\n\t"
                                 "global_load_dword %9, %18, %20 offset:1024 sc1\n\t"
                                 "global_load_dword %10, %18, %20 offset:2048 sc1\n\t"
                                 "global_load_dword %11, %18, %20 offset:3072 sc1\n\t"
                                 "global_load_dword %12, %19, %20 sc1\n\t"
                                 "global_load_dword %13, %19, %20 offset:1024 sc1\n\t"
                                 "global_load_dword %14, %19, %20 offset:2048 sc1\n\t"
                                 "global_load_dword %15, %19, %20 offset:3072 sc1\n\t"
                                 "s_waitcnt vmcnt(0)"
                                 : "=&v"(g[0]), "=&v"(g[1]), "=&v"(g[2]), "=&v"(g[3]), "=&v"(g[4]), "=&v"(g[5]), "=&v"(g[6]), "=&v"(g[7]),
                                   "=&v"(g[8]), "=&v"(g[9]), "=&v"(g[10]), "=&v"(g[11]), "=&v"(g[12]), "=&v"(g[13]), "=&v"(g[14]), "=&v"(g[15])
                                 : "v"(o0), "v"(o1), "v"(o2), "v"(o3), "s"(strip_part)
                                 : "memory");
#pragma unroll
                    for (int j = 0; j < 16; ++j)
                        if (sh + j < shares) v += g[j];
                }
            } else
            for (uint32_t sh = 0; sh < shares; sh += 8) {
                uint32_t off[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) off[j] = ((sh + j < shares ? sh + j : shares - 1) * (M * KSP_COLS) + t) * 4;
                float g0, g1, g2, g3, g4, g5, g6, g7;
                asm volatile("global_load_dword %0, %8, %16 sc1\n\t"
                             "global_load_dword %1, %9, %16 sc1\n\t"
                             "global_load_dword %2, %10, %16 sc1\n\t"
                             "global_load_dword %3, %11, %16 sc1\n\t"
                             "global_load_dword %4, %12, %16 sc1\n\t"
                             "global_load_dword %5, %13, %16 sc1\n\t"
                             "global_load_dword %6, %14, %16 sc1\n\t"
                             "global_load_dword %7, %15, %16 sc1\n\t"
                             "s_waitcnt vmcnt(0)"
                             : "=&v"(g0), "=&v"(g1), "=&v"(g2), "=&v"(g3), "=&v"(g4), "=&v"(g5), "=&v"(g6), "=&v"(g7)
                             : "v"(off[0]), "v"(off[1]), "v"(off[2]), "v"(off[3]), "v"(off[4]), "v"(off[5]), "v"(off[6]), "v"(off[7]),
                               "s"(strip_part)
                             : "memory");
                const float got[8] = {g0, g1, g2, g3, g4, g5, g6, g7};
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    if (sh + j < shares) v += got[j];
            }
            if (i < m && col0 + cc < n) finish(i, col0 + cc, v);
        }
    }
}

// Shares of k for the kernel above: about one workgroup per CU, shares of whole load rounds, at most 255.
struct KnSplitPlan {
    uint32_t strips, shares, kr;
    size_t ticket_bytes, bytes;
};
inline KnSplitPlan kn_split_plan(size_t k, size_t n, uint32_t rows_padded) {
    KnSplitPlan p{};
    p.strips = static_cast<uint32_t>((n + KSP_COLS - 1) / KSP_COLS);
    static int cus = 0;
    if (cus == 0) {
        int dev = 0, c = 0;
        if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&c, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && c > 0) cus = c;
        else cus = 256;
    }
    constexpr uint32_t STEP = KSP_ROWS * KSP_DEPTH;
    uint32_t shares = (static_cast<uint32_t>(cus) + p.strips / 2) / p.strips;
    if (shares < 1) shares = 1;
    uint32_t kr = static_cast<uint32_t>((k + shares - 1) / shares);
    kr = (kr + STEP - 1) / STEP * STEP;
    if (kr > KSP_MAX_KR) kr = KSP_MAX_KR;
    shares = static_cast<uint32_t>((k + kr - 1) / kr);
    p.shares = shares;
    p.kr = kr;
    p.ticket_bytes = (static_cast<size_t>(p.strips) * (shares + 1) * 8 + 255) / 256 * 256;  // a counter per strip, a flag per share
    p.bytes = p.ticket_bytes + static_cast<size_t>(p.strips) * shares * rows_padded * KSP_COLS * sizeof(float) + 16384;  // (padding: see the kernel)
    return p;
}

// ---------------------------------------------------------------- up to 32 rows of A, B as [k, n], k shared between workgroups
//
// The same sharing for the matrix cores.  A workgroup of four wavefronts takes a strip of 64 columns and at most 1024
// k-rows: that part of B (128 KiB) is requested in one go, straight into LDS, so every byte the workgroup will ever
// read is in flight from its first microsecond.  Wavefront w copies and multiplies a quarter of the k-rows for both
// column blocks of the strip, so it waits for its own copies only.  LDS layout: k-rows of 128 bytes, chunk c of row r
// at chunk position c ^ 4 ((r >> 1) & 1): the four rows x 64 bytes that 32 lanes of a transposing 64-bit read touch
// then lie on 64 different banks.  A product's first operand comes from two such reads (k-rows 8 h .. 8 h + 7 of the
// step for half h of the wavefront), its second operand is one 128-bit load of A from global memory (row lane % 32,
// the same eight k), issued before the copies so that it arrives before them.  The four wavefronts' sums meet in
// LDS, the shares of k in the workspace as above; the finished tile leaves through LDS in whole 128-byte rows.
// Measured on the way here ([32, 4096] x [4096, 4096], 23.0 us before): with strips of 128 columns, 16 wavefronts
// and shares of 512 k-rows 15.2 us, of which the copies alone 7.1, the products 0.4, the sixteen wavefronts' sums
// through LDS 1.8, 4 MB of float sums into the workspace 1.1, the hand-off 1.2 and the one workgroup per strip that
// adds up 128 KiB and stores 4096 scattered 16-bit values 3.6.  As built now 13.3 us: the copies alone 7.8 (128-byte
// pieces of B's rows), A's operands 1.4 (32-byte pieces of 32 rows per load, twice as many strips ask for them),
// the products 1.2, and 3.0 for everything behind them.
constexpr int KM_COLS = 64;       // columns of a strip (128 bytes of a k-row)
constexpr int KM_ROWB = 128;      // bytes of a k-row of the strip in LDS
constexpr int KM_MAX_KR = 1024;   // k-rows of a share: 128 KiB of LDS
constexpr int KM_PART = 2048;     // floats a workgroup leaves: 32 rows of A x 64 columns
template <class T>
__global__ __launch_bounds__(256) void mm_kn_mfma_split(T *__restrict__ y, const T *__restrict__ a, const T *__restrict__ b, Bias bias,
                                                       uint32_t m, uint32_t k, uint32_t n, float alpha, float beta, uint32_t kr,
                                                       uint32_t shares, float *__restrict__ part, unsigned long long *__restrict__ sync,
                                                       unsigned long long launch_no) {
    // kr: k-rows per share, a multiple of 256, at most KM_MAX_KR; k a multiple of 8, n of 64
    // sync: one arrival counter per strip, then one flag per strip and share
    __shared__ __align__(1024) uint8_t lds[KM_MAX_KR * KM_ROWB];
    const uint32_t tid = threadIdx.x, lane = tid & 63, l32 = lane & 31, half = lane >> 5;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t strip = blockIdx.x, share = blockIdx.y;
    const uint32_t col0 = strip * KM_COLS, k0 = share * kr;
    const uint32_t k_here = k - k0 < kr ? k - k0 : kr;  // k-rows of this share that exist (a multiple of 8)
    const uint32_t kq = kr / 4, row0 = wave * kq;        // this wavefront's k-rows of the share: a multiple of 64

    // the operand from A first: row l32 (rows beyond m repeat the last one, their results are not stored), k-rows
    // row0 + 16 ks + 8 half .. + 7; beyond the share's last k-row the operand is zero
    constexpr int MAX_STEPS = KM_MAX_KR / 4 / 16;
    u32x4 af[MAX_STEPS];
    {
        const T *arow = a + static_cast<uint64_t>(l32 < m ? l32 : m - 1) * k + k0;
#pragma unroll
        for (int ks = 0; ks < MAX_STEPS; ++ks) {
            const uint32_t kk = row0 + 16 * ks + 8 * half;
            const bool have = 16 * ks < kq && kk < k_here;
            const u32x4 v = *reinterpret_cast<const u32x4 *>(arow + (have ? kk : 0));
            af[ks] = have ? v : u32x4{0, 0, 0, 0};
        }
    }
    // the copies: eight k-rows of 128 bytes per instruction; lane L fills chunk position L % 8 of row L / 8 of them,
    // which holds chunk (L % 8) ^ 4 ((L / 8 >> 1) & 1).  Rows beyond the share's last one repeat it (A's operand is
    // zero there).
    {
        const uint32_t cp_r = lane >> 3, chunk = (lane & 7) ^ (4 * ((cp_r >> 1) & 1));
        const T *src0 = b + col0 + 8 * chunk;
#pragma unroll 4
        for (uint32_t r0 = row0; r0 < row0 + kq; r0 += 8) {
            const uint32_t r = r0 + cp_r, rr = r < k_here ? r : k_here - 1;
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(src0 + static_cast<uint64_t>(k0 + rr) * n),
                                             (__attribute__((address_space(3))) void *)(lds + r0 * KM_ROWB), 16, 0, 0);
        }
    }
    f16v acc[2];
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[j][e] = 0.f;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // a wavefront reads only what it has copied itself: no barrier
    {
        // transposing read: lane s of a group of 16 addresses k-row s / 4, columns 4 (s % 4) .. + 3 of the group's 16;
        // the other column block of the strip is reached by XOR with 64 (bit 2 of the chunk position)
        const uint32_t s16 = lane & 15, v_r = s16 >> 2;
        const uint32_t chunk = 2 * ((lane >> 4) & 1) + ((s16 & 3) >> 1);
        const uint32_t f_off = (row0 + 8 * half + v_r) * KM_ROWB + 16 * (chunk ^ (4 * ((v_r >> 1) & 1))) + 8 * (s16 & 1);
        // the reads of four k-steps are issued together, ahead of their products: read by read behind its product,
        // a wavefront that is alone on its SIMD waits out the LDS latency 64 times over (4.5 us instead of 0.5)
        auto read4 = [&](u32x4 (&bf)[4][2], int ks0) {
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const uint32_t o = f_off + 16 * (ks0 + q) * KM_ROWB;
                    const s4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s4 __attribute__((address_space(3))) *)(lds + (o ^ (64 * j))));
                    const s4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (s4 __attribute__((address_space(3))) *)(lds + ((o + 4 * KM_ROWB) ^ (64 * j))));
                    const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
                    bf[q][j] = u32x4{l2[0], l2[1], h2[0], h2[1]};
                }
        };
        u32x4 bf[2][4][2];
        if (kq > 0) read4(bf[0], 0);
#pragma unroll
        for (int g = 0; g < MAX_STEPS / 4; ++g) {
            if (64 * g < kq) {
                if (64 * (g + 1) < kq && g + 1 < MAX_STEPS / 4) read4(bf[(g + 1) & 1], 4 * (g + 1));
#pragma unroll
                for (int q = 0; q < 4; ++q)
#pragma unroll
                    for (int j = 0; j < 2; ++j) acc[j] = Mfma<T>::run(bf[g & 1][q][j], af[4 * g + q], acc[j]);
            }
        }
    }
    // lane holds row l32 of A; register e column 8 (e / 4) + 4 half + e % 4 of column block j.  The four wavefronts'
    // sums meet in the tile's memory: element x = 1024 j + 64 e + lane of wavefront w at float 2048 w + x.
    float *sums = reinterpret_cast<float *>(lds);
    __syncthreads();  // every wavefront has read its fragments
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) sums[wave * KM_PART + j * 1024 + e * 64 + lane] = acc[j][e];
    __syncthreads();
    // thread t owns elements 8 t .. 8 t + 7
    f4v mine[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        mine[h] = *reinterpret_cast<const f4v *>(sums + 8 * tid + 4 * h);
#pragma unroll
        for (int w = 1; w < 4; ++w) mine[h] += *reinterpret_cast<const f4v *>(sums + w * KM_PART + 8 * tid + 4 * h);
    }
    if (shares > 1) {
        const float *strip_part = part + static_cast<uint64_t>(strip) * shares * KM_PART;
        const uint32_t my_off = (share * KM_PART + 8 * tid) * 4;
        asm volatile("global_store_dwordx4 %0, %1, %3 sc1\n\tglobal_store_dwordx4 %0, %2, %3 offset:16 sc1"
                     : : "v"(my_off), "v"(mine[0]), "v"(mine[1]), "s"(strip_part) : "memory");
        if (!shares_complete(sync + strip, sync + gridDim.x + static_cast<uint64_t>(strip) * shares, share, shares, launch_no, tid)) return;
        mine[0] = mine[1] = f4v{0.f, 0.f, 0.f, 0.f};
        for (uint32_t sh = 0; sh < shares; sh += 4) {
            uint32_t off[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) off[j] = ((sh + j < shares ? sh + j : shares - 1) * KM_PART + 8 * tid) * 4;
            f4v g0, g1, g2, g3, g4, g5, g6, g7;
            asm volatile("global_load_dwordx4 %0, %8, %12 sc1\n\t"
                         "global_load_dwordx4 %1, %8, %12 offset:16 sc1\n\t"
                         "global_load_dwordx4 %2, %9, %12 sc1\n\t"
                         "global_load_dwordx4 %3, %9, %12 offset:16 sc1\n\t"
                         "global_load_dwordx4 %4, %10, %12 sc1\n\t"
                         "global_load_dwordx4 %5, %10, %12 offset:16 sc1\n\t"
                         "global_load_dwordx4 %6, %11, %12 sc1\n\t"
                         "global_load_dwordx4 %7, %11, %12 offset:16 sc1\n\t"
                         "s_waitcnt vmcnt(0)"
                         : "=&v"(g0), "=&v"(g1), "=&v"(g2), "=&v"(g3), "=&v"(g4), "=&v"(g5), "=&v"(g6), "=&v"(g7)
                         : "v"(off[0]), "v"(off[1]), "v"(off[2]), "v"(off[3]), "s"(strip_part)
                         : "memory");
            const f4v got[8] = {g0, g1, g2, g3, g4, g5, g6, g7};
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (sh + j < shares) {
                    mine[0] += got[2 * j];
                    mine[1] += got[2 * j + 1];
                }
        }
    }
    // the tile leaves through LDS: [row of A][64 columns] of T, then 16 bytes per thread
    __syncthreads();  // the sums in LDS have been read
    T *tile = reinterpret_cast<T *>(lds);
    const T *C = static_cast<const T *>(bias.ptr);
#pragma unroll
    for (int v = 0; v < 8; ++v) {
        const uint32_t x = 8 * tid + v, e = (x >> 6) & 15, i = x & 31, c = 32 * (x >> 10) + 8 * (e >> 2) + 4 * ((x >> 5) & 1) + (e & 3);
        float r = mine[v / 4][v % 4] * alpha;
        if (C && i < m) r += beta * up(C[i * bias.sm + (col0 + c) * bias.sn]);
        tile[i * KM_COLS + c] = down<T>(r);
    }
    __syncthreads();
    {
        const uint32_t i = tid >> 3, c8 = tid & 7;
        if (i < m) *reinterpret_cast<u32x4 *>(y + static_cast<uint64_t>(i) * n + col0 + 8 * c8) = *reinterpret_cast<const u32x4 *>(tile + i * KM_COLS + 8 * c8);
    }
}

inline KnSplitPlan kn_mfma_split_plan(size_t k, size_t n) {
    KnSplitPlan p{};
    p.strips = static_cast<uint32_t>(n / KM_COLS);
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
        cus = 256;
    uint32_t shares = (static_cast<uint32_t>(cus) + p.strips / 2) / p.strips;
    if (shares < 1) shares = 1;
    uint32_t kr = static_cast<uint32_t>((k + shares - 1) / shares);
    kr = (kr + 255) / 256 * 256;  // a wavefront's quarter in groups of four k-steps
    if (kr > KM_MAX_KR) kr = KM_MAX_KR;
    p.shares = static_cast<uint32_t>((k + kr - 1) / kr);
    p.kr = kr;
    p.ticket_bytes = (static_cast<size_t>(p.strips) * (p.shares + 1) * 8 + 255) / 256 * 256;  // a counter per strip, a flag per share
    p.bytes = p.ticket_bytes + static_cast<size_t>(p.strips) * p.shares * KM_PART * sizeof(float);
    return p;
}

template <class T>
int launch_kn_split(T *y, const T *a, const T *b, Bias bias, uint32_t m, uint32_t k, uint32_t n, float alpha, float beta,
                    void *workspace, const KnSplitPlan &plan, hipStream_t s) {
    auto *flags = static_cast<unsigned long long *>(workspace);
    float *part = reinterpret_cast<float *>(static_cast<uint8_t *>(workspace) + plan.ticket_bytes);
    const dim3 grid(plan.strips, plan.shares, 1);
    const unsigned long long no = next_launch_number();
    if (m <= 1) mm_kn_split<T, 1><<<grid, 1024, 0, s>>>(y, a, b, bias, m, k, n, alpha, beta, plan.kr, plan.shares, part, flags, no);
    else if (m <= 2) mm_kn_split<T, 2><<<grid, 1024, 0, s>>>(y, a, b, bias, m, k, n, alpha, beta, plan.kr, plan.shares, part, flags, no);
    else mm_kn_split<T, 4><<<grid, 1024, 0, s>>>(y, a, b, bias, m, k, n, alpha, beta, plan.kr, plan.shares, part, flags, no);
    return launch_status();
}

template <class T>
int launch_kn_mfma_split(T *y, const T *a, const T *b, Bias bias, uint32_t m, uint32_t k, uint32_t n, float alpha, float beta,
                         void *workspace, const KnSplitPlan &plan, hipStream_t s) {
    if constexpr (sizeof(T) == 2) {
        auto *sync = static_cast<unsigned long long *>(workspace);
        float *part = reinterpret_cast<float *>(static_cast<uint8_t *>(workspace) + plan.ticket_bytes);
        mm_kn_mfma_split<T><<<dim3(plan.strips, plan.shares, 1), 256, 0, s>>>(y, a, b, bias, m, k, n, alpha, beta, plan.kr, plan.shares,
                                                                                part, sync, next_launch_number());
        return launch_status();
    } else {
        return RG_HIP_E_UNSUPPORTED;
    }
}

template <class T, int M, int L>
int launch_gemv_kn_l(T *y, const T *a, const T *b, Bias bias, uint32_t m, uint32_t k, uint32_t n, float alpha, float beta,
                     uint32_t am0, uint32_t bm0, uint32_t ym0, uint32_t count, uint32_t row0, uint32_t rows, hipStream_t s) {
    const dim3 grid((n + 8 * L - 1) / (8 * L), 1, count);
    mm_gemv_kn<T, M, L><<<grid, 1024, 0, s>>>(y, a, b, bias, m, k, n, alpha, beta, am0, bm0, ym0, row0, rows);
    return launch_status();
}

// The widest strip (8, 4 or 2 lanes of 8 columns) that still gives some 160 workgroups: a wide strip reads
// whole 128-byte lines and has fewer lane groups to add up, but one workgroup per CU keeps only so many
// bytes in flight, so the chip has to be covered first.
template <class T, int M>
int launch_gemv_kn(T *y, const T *a, const T *b, Bias bias, uint32_t m, uint32_t k, uint32_t n, float alpha, float beta,
                   uint32_t am0, uint32_t bm0, uint32_t ym0, uint32_t count, uint32_t row0, uint32_t rows, hipStream_t s) {
    auto groups = [&](uint32_t lanes) { return static_cast<uint64_t>((n + 8 * lanes - 1) / (8 * lanes)) * count; };
    if (groups(8) >= 160) return launch_gemv_kn_l<T, M, 8>(y, a, b, bias, m, k, n, alpha, beta, am0, bm0, ym0, count, row0, rows, s);
    if (groups(4) >= 160) return launch_gemv_kn_l<T, M, 4>(y, a, b, bias, m, k, n, alpha, beta, am0, bm0, ym0, count, row0, rows, s);
    return launch_gemv_kn_l<T, M, 2>(y, a, b, bias, m, k, n, alpha, beta, am0, bm0, ym0, count, row0, rows, s);
}

template <class T, int G, int WAVES, int DEPTH>
int launch_rows(T *y, const T *a, const T *b, Bias bias, uint32_t rows, uint32_t m, uint32_t row_first, uint32_t k, uint32_t n,
                float al, float be, uint32_t am0, uint32_t bm0, uint32_t ym0, uint32_t count, hipStream_t s) {
    const dim3 grid(n / 16, 1, count);
    mm_rows<T, G, WAVES, DEPTH><<<grid, 64 * WAVES, 0, s>>>(y, a, b, bias, rows, m, row_first, k, n, al, be, am0, bm0, ym0);
    return launch_status();
}

template <class T, int G, int WAVES, int CW>
int launch_rows_kn(T *y, const T *a, const T *b, Bias bias, uint32_t rows, uint32_t m, uint32_t row_first, uint32_t k, uint32_t n,
                   float al, float be, uint32_t am0, uint32_t bm0, uint32_t ym0, uint32_t count, hipStream_t s) {
    const dim3 grid(n / (4 * CW), 1, count);
    mm_rows_kn<T, G, WAVES, CW><<<grid, 64 * WAVES, 0, s>>>(y, a, b, bias, rows, m, row_first, k, n, al, be, am0, bm0, ym0);
    return launch_status();
}

constexpr uint32_t GV_LDS_BYTES = 64 * 1024;  // of A per workgroup at most
constexpr uint32_t kGemvMaxGrid = 512;     // workgroups of a launch: two per CU

template <class T, int M>
int launch_gemv(T *y, const T *a, const T *w, Bias bias, uint32_t m, uint32_t k, uint32_t n, float alpha, float beta,
                uint32_t am0, uint32_t bm0, uint32_t ym0, uint32_t count, hipStream_t s) {
    constexpr int R = 1;  // rows of W per wavefront: more of them share the reads of A from LDS, and measured slower
    constexpr uint32_t segment_limit = GV_LDS_BYTES / (16 * M);  // 16-byte pieces of a row of A
    const uint32_t segment = k / 8 < segment_limit ? k / 8 : segment_limit;
    const size_t lds = static_cast<size_t>(M) * segment * 16;
    // the wavefronts of a workgroup share one copy of A: as many as still leave a workgroup for every CU
    uint32_t waves = 16;
    while (waves > 4 && static_cast<uint64_t>((n + waves * R - 1) / (waves * R)) * count < 256) waves /= 2;
    uint32_t blocks = (n + waves * R - 1) / (waves * R);
    if (blocks > kGemvMaxGrid) blocks = kGemvMaxGrid;  // (the rest of the row blocks in turns)
    const dim3 grid(blocks, 1, count);
    if (segment == k / 8) mm_gemv<T, M, R, false><<<grid, 64 * waves, lds, s>>>(y, a, w, bias, m, k, n, segment, alpha, beta, am0, bm0, ym0);
    else mm_gemv<T, M, R, true><<<grid, 64 * waves, lds, s>>>(y, a, w, bias, m, k, n, segment, alpha, beta, am0, bm0, ym0);
    return launch_status();
}

template <class T>
int launch_typed(void *y_, const void *a_, const void *b_, Bias bias, int trans_a, int trans_b, float alpha, float beta,
                 size_t batch, size_t m, size_t k, size_t n, const uint32_t *a_index, const uint32_t *b_index,
                 hipStream_t s, void *workspace = nullptr, size_t workspace_bytes = 0) {
    auto *y = static_cast<T *>(y_);
    auto *a = static_cast<const T *>(a_);
    auto *b = static_cast<const T *>(b_);
    typedef typename Acc<T>::type A_t;
    const A_t al = through<T>(alpha), be = bias.ptr ? through<T>(beta) : A_t(0);
    constexpr bool narrow = sizeof(T) == 2;
    // rows of B as [k, n] and of Y start on 16-byte boundaries when n is a multiple of 8; tiles that are moved
    // back overlap their neighbours, which a bias that is the output itself does not allow
    const bool ragged = m % BM != 0 || n % BN != 0;
    const bool fast = narrow && !trans_a && m >= BM && n >= BN && n % 8 == 0 && k % BK == 0 && k > 0 && aligned16(a) &&
                      aligned16(b) && aligned16(y_) && !(ragged && bias.ptr == y_);

    // fewer rows than a tile, weights as [n, k]: stream W once per slab of 32 rows of A
    const bool skinny = narrow && !fast && !trans_a && trans_b && m < BM && n % 32 == 0 && k % SK_TK == 0 &&
                        aligned16(a) && aligned16(b);

    // one row (and up to four where the block-product kernel below does not apply): matrix-vector products on the
    // vector ALUs, A (padded to 1, 2 or 4 rows) in LDS
    const uint32_t gv_m = m <= 1 ? 1 : m <= 2 ? 2 : 4;
    const bool gemv = narrow && !trans_a && trans_b && m <= 4 && k > 0 && k % 8 == 0 && aligned16(a) && aligned16(b);

    // the same with B as [k, n]; up to 32 rows go four at a time, each pass reading B again at the same cost
    // (20 us per pass at 4096 x 4096: 8 rows in a fifth, 32 rows in six sevenths of the plain kernel's time,
    // which is what is left for these shapes otherwise)
    const bool gemv_kn = narrow && !trans_a && !trans_b && m <= 32 && k > 0 && k % 8 == 0 && n % 8 == 0 && aligned16(a) &&
                         aligned16(b);

    // two to sixteen rows, weights as [n, k]: operands straight from global memory into 4x4x4 block products
    // (a single row too when k is long: the matrix-vector kernel keeps a whole row of W per wavefront in flight,
    // which stops paying beyond 16 KiB; and when k is short, where a wavefront of that kernel ends a row after few
    // loads, at k = 128 with 16 of its lanes: [1, 1024] x [65536, 1024]^T 40 -> 28 us, 32 products of
    // [1, 128] x [4096, 128]^T 67 -> 24 us, [1, 2048] x [4096, 2048]^T 4.8 -> 4.3 us)
    const bool rows = narrow && !trans_a && trans_b && (m >= 2 || k > 8192 || k <= 2048) && m <= 16 && n % 16 == 0 && k % 128 == 0 &&
                      k > 0 && k < (1u << 26) && aligned16(a) && aligned16(b);

    // fewer than 256 rows, weights as [k, n]: the same block products behind a transposition in registers, 32 rows a
    // pass (one to four rows against a wide B stay with the matrix-vector kernel, which is a little faster there)
    const bool rows_kn = narrow && !trans_a && !trans_b && m < BM && !(m <= 4 && n >= 8192) && n % 16 == 0 && k % 128 == 0 &&
                         k > 0 && static_cast<uint64_t>(k) * n < (1ull << 31) && k < (1u << 26) && aligned16(a) && aligned16(b);

    // fewer than 256 rows on the 256 x 256 tiles (one row of tiles, A's missing rows repeated, their results not
    // stored): a launch costs what a full tile costs, about 93 us at k = 4096, whatever m is, so it is taken where
    // the passes of the few-rows kernels would take longer (measured per pass at k = 4096: 5.5 ns per column for 32
    // rows with B as [k, n], 3.4 to 4.7 ns for 64 rows with B as [n, k]) and where the plain kernel is the alternative
    const bool short_ok = narrow && !trans_a && m < BM && n >= BN && n % 8 == 0 && k % BK == 0 && k > 0 && aligned16(a) &&
                          aligned16(b) && aligned16(y_) && !(n % BN != 0 && bias.ptr == y_) &&
                          k < (1u << 22);  // a lane's offset into A (up to 255 rows) stays below 2^31
    // FP16 / BF16 shapes that none of the kernels above takes, more than 8 rows: 128 x 128 tiles, any m and n.
    // They also take the shapes of the 256 x 256 tiles when those are few: a workgroup's walk through k is a chain
    // of dependent steps (1.33 us per 64 of k on the large tile, 0.83 us on the small one), so while the small tiles
    // find a CU each, or nearly, the launch ends earlier (k = 4096: 85 -> 53 us up to 64 large tiles, 85 -> 78 at 86,
    // level at 128)
    // Up to 8 rows only where the plain kernel is expected to take longer (it needs 2.9 ns per thousand elements of B,
    // 596 us for [8, 4096] x [4096, 50257]; a tile launch about 4 us and 0.83 us per 64 of k).
    const bool tiles16_rows = m > 8 || static_cast<uint64_t>(n) * k > 1400000u + 4500u * static_cast<uint64_t>(k);
    const bool tiles16 = narrow && !trans_a && k % 8 == 0 && k > 0 && tiles16_rows && aligned16(a) && (!trans_b || aligned16(b));
    const bool small_grid = tiles16 && ((m + HT - 1) / HT) * ((n + HT - 1) / HT) * (a_index || b_index ? 1 : batch) <= kSmallGrid;
    bool short_tile = false;
    if (short_ok || small_grid) {
        // (the tile launch that the passes of the few-rows kernels are weighed against is cheaper on the small tiles;
        // there the matrices of a batch count too, all of them being tiles of one launch that find a CU each)
        // (one to four rows against W as [n, k] read W once at the speed of the memory whatever n is: never a tile)
        const uint64_t columns = small_grid ? n * (a_index || b_index ? 1 : batch) : n;
        // passes of four rows over B as [k, n] against one launch of small tiles (a pass: 4.3 us or B at 5 TB/s)
        const double b_us = 2.0 * static_cast<double>(k) * static_cast<double>(columns) / 5.0e6;
        const double gemv_kn_us = static_cast<double>((m + 3) / 4) * (b_us > 4.3 ? b_us : 4.3);
        const bool gemv_kn_slow = small_grid && m > 4 && 4.0 + 0.83 * static_cast<double>((k + HK - 1) / HK) < gemv_kn_us;
        if (trans_b) short_tile = rows || gemv ? false : skinny ? ((m + 63) / 64) * columns > (small_grid ? kSkinnyPassesSmall : 23000u) : true;
        else short_tile = rows_kn ? ((m + 31) / 32) * columns > (small_grid ? kRowsKnPassesSmall : 17000u)
                                  : gemv_kn ? (short_ok && m > 16) || gemv_kn_slow : true;
    }
    // A short k leaves a tile little to do between fetching its operands and storing its results, and two small tiles
    // per CU overlap the one's stores with the other's loads: with k <= 128 the small tiles take a full grid too
    // ([4096, 128] x [128, 4096] 24.7 -> 22.9 us, [8192, 128] x [128, 8192] 93 -> 76 us, 32 products of
    // [512, 128] x [512, 128]^T 21 -> 13.5 us; at k = 256 they lose, 28 -> 31 us), and with k <= 512 every short tile
    // is a small one and taken before the few-rows kernels (32 products [128, 128] x [4096, 128]^T 110 -> 25 us)
    const bool short_k = tiles16 && m > 16 && ((fast && k <= 128) || (short_ok && k <= 512));

    // F32 on the matrix cores.  A launch of the 128 x 128 tiles walks all of k in every workgroup and takes about
    // 300 us at k = 4096 however few tiles there are; up to that cost few rows go through the block products of
    // mm_rows / mm_rows_kn (one k per block and instruction; no transposition needed for B as [k, n], an operand
    // being one float), 32 rows a pass: 27 us (B as [n, k]) and 33 us (as [k, n]) per pass and 4096 columns.
    constexpr bool is_f32 = std::is_same<T, float>::value;
    const bool f32_tiles_ok = is_f32 && !trans_a && k % FK == 0 && k > 0 && aligned16(a) && aligned16(b) &&
                              (trans_b || (n % 4 == 0 && n >= 4));
    const bool rows_f32_ok = is_f32 && !trans_a && trans_b && n % 16 == 0 && k % 64 == 0 && k > 0 && k < (1u << 25) &&
                             aligned16(a) && aligned16(b);
    const bool rows_kn_f32_ok = is_f32 && !trans_a && !trans_b && n % 16 == 0 && k % 128 == 0 && k > 0 &&
                                static_cast<uint64_t>(k) * n < (1ull << 30) && k < (1u << 25) && aligned16(a) && aligned16(b);
    // (microseconds, from those figures, with 3 us for a launch; 768 tiles run side by side)
    const double kn4096 = static_cast<double>(n) / 4096 * static_cast<double>(k) / 4096;
    const double f32_tile_rounds = static_cast<double>((((m + FT - 1) / FT) * ((n + FT - 1) / FT) + 767) / 768);
    const double f32_cost_tiles = f32_tiles_ok ? 3.0 + 300.0 * static_cast<double>(k) / 4096 * f32_tile_rounds : 1e30;
    const double f32_passes = static_cast<double>((m + 31) / 32);
    const bool rows_f32 = rows_f32_ok && f32_passes * (3.0 + 27.0 * kn4096) <= f32_cost_tiles;
    const bool rows_kn_f32 = rows_kn_f32_ok && f32_passes * (3.0 + 33.0 * kn4096) <= f32_cost_tiles;
    const bool f32_tiles = f32_tiles_ok && m > 8;

    auto launch_tiles16 = [&](uint32_t am0, uint32_t bm0, uint32_t ym0, uint32_t count) -> int {
        if constexpr (narrow) {
            // tiles of 64 rows while those of 128 would leave half of the CUs without one
            const bool half = ((m + HT - 1) / HT) * ((n + HT - 1) / HT) * count <= kHalfTiles;
            const size_t tm = half ? HT / 2 : HT;
            const uint64_t tiles = ((m + tm - 1) / tm) * ((n + HT - 1) / HT);
            if (tiles > 0x7fffffffu) return RG_HIP_E_UNSUPPORTED;
            const dim3 grid(static_cast<unsigned>(tiles), 1, count);
            const uint32_t m32 = static_cast<uint32_t>(m), k32 = static_cast<uint32_t>(k), n32 = static_cast<uint32_t>(n);
            const bool vec = n % 8 == 0 && n >= 8 && aligned16(b);
#define RG_TILES16(TB, VEC)                                                                                              \
    (half ? mm_tiles16<T, TB, VEC, HT / 2><<<grid, 256, 0, s>>>(y, a, b, bias, m32, k32, n32, al, be, am0, bm0, ym0)      \
          : mm_tiles16<T, TB, VEC, HT><<<grid, 256, 0, s>>>(y, a, b, bias, m32, k32, n32, al, be, am0, bm0, ym0))
            if (trans_b) RG_TILES16(true, true);
            else if (vec) RG_TILES16(false, true);
            else RG_TILES16(false, false);
#undef RG_TILES16
            return launch_status();
        } else {
            return RG_HIP_E_UNSUPPORTED;
        }
    };

    auto launch = [&](uint32_t am0, uint32_t bm0, uint32_t ym0, uint32_t count) -> int {
        if constexpr (narrow) {
            // five to 32 rows against weights as [k, n] with a workspace at hand: the same sharing on the matrix cores
            if (workspace && !trans_a && !trans_b && m > 4 && m <= 32 && batch == 1 && count == 1 && n % KM_COLS == 0 && k > 0 &&
                k % 8 == 0 && static_cast<uint64_t>(k) * n >= (1u << 20) && aligned16(b) && aligned16(a) && aligned16(y_) &&
                reinterpret_cast<uintptr_t>(workspace) % 16 == 0) {
                const KnSplitPlan plan = kn_mfma_split_plan(k, n);
                if (plan.shares <= 255 && plan.bytes <= workspace_bytes)
                    return launch_kn_mfma_split<T>(y + static_cast<uint64_t>(ym0) * m * n, a + static_cast<uint64_t>(am0) * m * k,
                                                   b + static_cast<uint64_t>(bm0) * k * n, bias, static_cast<uint32_t>(m),
                                                   static_cast<uint32_t>(k), static_cast<uint32_t>(n), al, be, workspace, plan, s);
            }
            // one to four rows against weights as [k, n] with a workspace at hand: wide strips, k shared between
            // workgroups (from 2 MB of weights on; below that the launch is all there is to either kernel)
            if (workspace && !trans_a && !trans_b && m <= 4 && batch == 1 && count == 1 && n % 8 == 0 && k > 0 && k % 2 == 0 &&
                static_cast<uint64_t>(k) * n >= (1u << 20) && aligned16(b) && reinterpret_cast<uintptr_t>(a) % 4 == 0 &&
                reinterpret_cast<uintptr_t>(workspace) % 8 == 0) {
                const KnSplitPlan plan = kn_split_plan(k, n, m <= 1 ? 1 : m <= 2 ? 2 : 4);
                if (plan.shares <= 255 && plan.bytes <= workspace_bytes)
                    return launch_kn_split<T>(y + static_cast<uint64_t>(ym0) * m * n, a + static_cast<uint64_t>(am0) * m * k,
                                              b + static_cast<uint64_t>(bm0) * k * n, bias, static_cast<uint32_t>(m),
                                              static_cast<uint32_t>(k), static_cast<uint32_t>(n), al, be, workspace, plan, s);
            }
            if ((small_grid && (short_tile || fast)) || short_k) return launch_tiles16(am0, bm0, ym0, count);
            if (short_tile) {
                const dim3 grid(static_cast<unsigned>((n + BN - 1) / BN), 1, count);
                if (trans_b)
                    mm_mfma_256x256<T, true, true><<<grid, 256, 0, s>>>(y, a, b, bias, static_cast<uint32_t>(m), static_cast<uint32_t>(k),
                                                                        static_cast<uint32_t>(n), al, be, am0, bm0, ym0);
                else
                    mm_mfma_256x256<T, false, true><<<grid, 256, 0, s>>>(y, a, b, bias, static_cast<uint32_t>(m), static_cast<uint32_t>(k),
                                                                         static_cast<uint32_t>(n), al, be, am0, bm0, ym0);
                return launch_status();
            }
            if (rows_kn) {
                const uint32_t m32 = static_cast<uint32_t>(m), k32 = static_cast<uint32_t>(k), n32 = static_cast<uint32_t>(n);
                const bool wide = n % 32 == 0 && n >= 8192;
                for (uint32_t r0 = 0; r0 < m32; r0 += 32) {
                    const uint32_t rows = m32 - r0 < 32 ? m32 - r0 : 32;
                    int e;
#define RG_ROWS_KN(G, CW) launch_rows_kn<T, G, 8, CW>(y, a, b, bias, rows, m32, r0, k32, n32, al, be, am0, bm0, ym0, count, s)
                    if (rows <= 4) e = wide ? RG_ROWS_KN(1, 8) : RG_ROWS_KN(1, 4);
                    else if (rows <= 8) e = wide ? RG_ROWS_KN(2, 8) : RG_ROWS_KN(2, 4);
                    else if (rows <= 16) e = wide ? RG_ROWS_KN(4, 8) : RG_ROWS_KN(4, 4);
                    else e = RG_ROWS_KN(8, 4);
#undef RG_ROWS_KN
                    if (e) return e;
                }
                return 0;
            }
            if (rows) {
                const uint32_t m32 = static_cast<uint32_t>(m), k32 = static_cast<uint32_t>(k), n32 = static_cast<uint32_t>(n);
                if (m <= 4 && k > 8192) return launch_rows<T, 1, 16, 2>(y, a, b, bias, m32, m32, 0, k32, n32, al, be, am0, bm0, ym0, count, s);
                if (m <= 4) return launch_rows<T, 1, 16, 1>(y, a, b, bias, m32, m32, 0, k32, n32, al, be, am0, bm0, ym0, count, s);
                if (m <= 8) return launch_rows<T, 2, 16, 1>(y, a, b, bias, m32, m32, 0, k32, n32, al, be, am0, bm0, ym0, count, s);
                // many workgroups per CU: small ones, several of which run side by side
                if (n / 16 > 384) return launch_rows<T, 4, 4, 3>(y, a, b, bias, m32, m32, 0, k32, n32, al, be, am0, bm0, ym0, count, s);
                return launch_rows<T, 4, 16, 1>(y, a, b, bias, m32, m32, 0, k32, n32, al, be, am0, bm0, ym0, count, s);
            }
            if (gemv_kn) {
                const uint32_t m32 = static_cast<uint32_t>(m), k32 = static_cast<uint32_t>(k), n32 = static_cast<uint32_t>(n);
                for (uint32_t r0 = 0; r0 < m32; r0 += 4) {
                    const uint32_t rows = m32 - r0 < 4 ? m32 - r0 : 4;
                    int e;
                    switch (rows) {
                        case 1: e = launch_gemv_kn<T, 1>(y, a, b, bias, m32, k32, n32, al, be, am0, bm0, ym0, count, r0, rows, s); break;
                        case 2: e = launch_gemv_kn<T, 2>(y, a, b, bias, m32, k32, n32, al, be, am0, bm0, ym0, count, r0, rows, s); break;
                        default: e = launch_gemv_kn<T, 4>(y, a, b, bias, m32, k32, n32, al, be, am0, bm0, ym0, count, r0, rows, s);
                    }
                    if (e) return e;
                }
                return 0;
            }
            if (gemv) {
                const uint32_t m32 = static_cast<uint32_t>(m), k32 = static_cast<uint32_t>(k), n32 = static_cast<uint32_t>(n);
                switch (gv_m) {
                    case 1: return launch_gemv<T, 1>(y, a, b, bias, m32, k32, n32, al, be, am0, bm0, ym0, count, s);
                    case 2: return launch_gemv<T, 2>(y, a, b, bias, m32, k32, n32, al, be, am0, bm0, ym0, count, s);
                    default: return launch_gemv<T, 4>(y, a, b, bias, m32, k32, n32, al, be, am0, bm0, ym0, count, s);
                }
            }
            if (skinny) {
                // two slabs of 32 rows share one pass over W
                for (size_t r0 = 0; r0 < m; r0 += 64) {
                    const uint32_t rows = static_cast<uint32_t>(m - r0 < 64 ? m - r0 : 64);
                    const dim3 grid(static_cast<unsigned>(n / 32), 1, count);
                    if (rows <= 32)
                        mm_skinny<T, 1><<<grid, 256, 0, s>>>(y, a, b, bias, rows, static_cast<uint32_t>(m), static_cast<uint32_t>(r0),
                                                             static_cast<uint32_t>(k), static_cast<uint32_t>(n), al, be, am0, bm0, ym0);
                    else
                        mm_skinny<T, 2><<<grid, 256, 0, s>>>(y, a, b, bias, rows, static_cast<uint32_t>(m), static_cast<uint32_t>(r0),
                                                             static_cast<uint32_t>(k), static_cast<uint32_t>(n), al, be, am0, bm0, ym0);
                    const int rc = launch_status();
                    if (rc) return rc;
                }
                return 0;
            }
            if (fast) {
                const dim3 grid(static_cast<unsigned>(((m + BM - 1) / BM) * ((n + BN - 1) / BN)), 1, count);
                if (trans_b)
                    mm_mfma_256x256<T, true><<<grid, 256, 0, s>>>(y, a, b, bias, static_cast<uint32_t>(m), static_cast<uint32_t>(k),
                                                                  static_cast<uint32_t>(n), al, be, am0, bm0, ym0);
                else
                    mm_mfma_256x256<T, false><<<grid, 256, 0, s>>>(y, a, b, bias, static_cast<uint32_t>(m), static_cast<uint32_t>(k),
                                                                   static_cast<uint32_t>(n), al, be, am0, bm0, ym0);
                return launch_status();
            }
        }
        if constexpr (narrow) {
            if (tiles16) return launch_tiles16(am0, bm0, ym0, count);
        }
        if constexpr (std::is_same<T, float>::value) {
            if (rows_f32) {
                const uint32_t m32 = static_cast<uint32_t>(m), k32 = static_cast<uint32_t>(k), n32 = static_cast<uint32_t>(n);
                for (uint32_t r0 = 0; r0 < m32; r0 += 32) {
                    const uint32_t rows = m32 - r0 < 32 ? m32 - r0 : 32;
                    int e;
#define RG_ROWS_F32(G, W, DP) launch_rows<T, G, W, DP>(y, a, b, bias, rows, m32, r0, k32, n32, al, be, am0, bm0, ym0, count, s)
                    if (rows <= 4) e = RG_ROWS_F32(1, 16, 1);
                    else if (rows <= 8) e = RG_ROWS_F32(2, 16, 1);
                    else if (rows <= 16) e = n / 16 > 384 ? RG_ROWS_F32(4, 4, 3) : RG_ROWS_F32(4, 16, 1);
                    else e = RG_ROWS_F32(8, 4, 3);
#undef RG_ROWS_F32
                    if (e) return e;
                }
                return 0;
            }
            if (rows_kn_f32) {
                const uint32_t m32 = static_cast<uint32_t>(m), k32 = static_cast<uint32_t>(k), n32 = static_cast<uint32_t>(n);
                for (uint32_t r0 = 0; r0 < m32; r0 += 32) {
                    const uint32_t rows = m32 - r0 < 32 ? m32 - r0 : 32;
                    int e;
#define RG_ROWS_KN_F32(G, W) launch_rows_kn<T, G, W, 4>(y, a, b, bias, rows, m32, r0, k32, n32, al, be, am0, bm0, ym0, count, s)
                    if (rows <= 4) e = RG_ROWS_KN_F32(1, 8);
                    else if (rows <= 8) e = RG_ROWS_KN_F32(2, 8);
                    else if (rows <= 16) e = RG_ROWS_KN_F32(4, 8);
                    else e = RG_ROWS_KN_F32(8, 4);  // 128 accumulators and two steps of operands: one wavefront per SIMD
#undef RG_ROWS_KN_F32
                    if (e) return e;
                }
                return 0;
            }
            if (f32_tiles) {
                const dim3 grid(static_cast<unsigned>((n + FT - 1) / FT), static_cast<unsigned>((m + FT - 1) / FT), count);
                if (grid.y > 65535) return RG_HIP_E_UNSUPPORTED;
                if (trans_b) mm_f32_tiles<true><<<grid, 256, 0, s>>>(y, a, b, bias, static_cast<uint32_t>(m), static_cast<uint32_t>(k),
                                                                    static_cast<uint32_t>(n), al, be, am0, bm0, ym0);
                else mm_f32_tiles<false><<<grid, 256, 0, s>>>(y, a, b, bias, static_cast<uint32_t>(m), static_cast<uint32_t>(k),
                                                              static_cast<uint32_t>(n), al, be, am0, bm0, ym0);
                return launch_status();
            }
        }
        const dim3 grid(static_cast<unsigned>((n + 15) / 16), static_cast<unsigned>((m + 15) / 16), count);
        mm_generic<T><<<grid, 256, 0, s>>>(y, a, b, bias, static_cast<uint32_t>(m), static_cast<uint32_t>(k),
                                           static_cast<uint32_t>(n), trans_a ? 1 : k, trans_a ? m : 1, trans_b ? 1 : n,
                                           trans_b ? k : 1, al, be, am0, bm0, ym0);
        return launch_status();
    };

    if (!a_index && !b_index) {
        for (size_t i = 0; i < batch; i += 65535) {  // grid.z is limited to 65535
            const uint32_t count = static_cast<uint32_t>(batch - i < 65535 ? batch - i : 65535);
            const int rc = launch(static_cast<uint32_t>(i), static_cast<uint32_t>(i), static_cast<uint32_t>(i), count);
            if (rc) return rc;
        }
        return 0;
    }
    // runs of matrices that follow each other in both operands are one launch each
    auto at = [](const uint32_t *index, size_t i) { return index ? index[i] : static_cast<uint32_t>(i); };
    for (size_t i = 0; i < batch;) {
        size_t run = 1;
        while (i + run < batch && run < 65535 && at(a_index, i + run) == at(a_index, i) + run &&
               at(b_index, i + run) == at(b_index, i) + run)
            ++run;
        const int rc = launch(at(a_index, i), at(b_index, i), static_cast<uint32_t>(i), static_cast<uint32_t>(run));
        if (rc) return rc;
        i += run;
    }
    return 0;
}

}  // namespace
}  // namespace rg

extern "C" size_t rg_hip_matmul_workspace(int dtype, int trans_a, int trans_b, size_t batch, size_t m, size_t k, size_t n) {
    using namespace rg;
    if ((dtype != RG_FP16 && dtype != RG_BF16) || trans_a || trans_b || batch != 1 || m == 0 || m > 32 || k == 0 ||
        k > 0x7fffffffu || n > 0x7fffffffu || static_cast<uint64_t>(k) * n < (1u << 20))
        return 0;
    if (m > 4) {
        if (n % KM_COLS != 0 || k % 8 != 0) return 0;
        const KnSplitPlan plan = kn_mfma_split_plan(k, n);
        return plan.shares <= 255 ? plan.bytes : 0;
    }
    if (n % 8 != 0 || k % 2 != 0) return 0;
    const KnSplitPlan plan = kn_split_plan(k, n, m <= 1 ? 1 : m <= 2 ? 2 : 4);
    return plan.shares <= 255 ? plan.bytes : 0;
}

extern "C" int rg_hip_matmul(void *y, const void *a, const void *b, const void *c, int dtype, int trans_a, int trans_b,
                             float alpha, float beta, size_t batch, size_t m, size_t k, size_t n,
                             const uint32_t *a_index, const uint32_t *b_index, size_t c_stride_batch,
                             size_t c_stride_m, size_t c_stride_n, void *stream) {
    return rg_hip_matmul_ws(y, a, b, c, dtype, trans_a, trans_b, alpha, beta, batch, m, k, n, a_index, b_index, c_stride_batch,
                            c_stride_m, c_stride_n, nullptr, 0, stream);
}

extern "C" int rg_hip_matmul_ws(void *y, const void *a, const void *b, const void *c, int dtype, int trans_a, int trans_b,
                                float alpha, float beta, size_t batch, size_t m, size_t k, size_t n,
                                const uint32_t *a_index, const uint32_t *b_index, size_t c_stride_batch,
                                size_t c_stride_m, size_t c_stride_n, void *workspace, size_t workspace_bytes, void *stream) {
    using namespace rg;
    if (!y || !a || !b) return RG_HIP_E_ARGUMENT;
    if (batch == 0 || m == 0 || n == 0) return 0;
    if (m > 0x7fffffffu || n > 0x7fffffffu || k > 0x7fffffffu || batch > 0xffffffffu) return RG_HIP_E_UNSUPPORTED;
    hipStream_t s = as_stream(stream);
    Bias bias{c, c_stride_batch, c_stride_m, c_stride_n};
    // One B for consecutive matrices of A (activations [batch, m, k] against weights): the batch is more rows of one
    // product, not `batch` launches that each read B again (64 x [1,4096] against [4096,4096]: 337 -> 12 us).
    // The same for groups of consecutive matrices of A that share one B each, the B's consecutive too (the query
    // heads of a key / value head): a batch of as many products as there are groups, in one launch
    // (8 groups of 4 matrices [1,4096] against [4096,128]: 427 -> 21 us).
    // (up to 2^20 rows: every kernel's grid takes that many)
    if (batch > 1 && b_index && !trans_a) {
        size_t group = 1;
        while (group < batch && b_index[group] == b_index[0]) ++group;
        bool fold = batch % group == 0 && group * m <= (1u << 20) && (group > 1 || !a_index) &&
                    (!c || c_stride_batch == m * c_stride_m || group == 1);
        for (size_t i = 0; i < batch && fold; ++i)
            fold = b_index[i] == b_index[0] + i / group && (a_index ? a_index[i] == a_index[0] + i : true);
        if (fold) {
            const size_t element = dtype == RG_F64 ? 8 : dtype == RG_F32 ? 4 : 2;
            a = static_cast<const uint8_t *>(a) + static_cast<size_t>(a_index ? a_index[0] : 0) * m * k * element;
            b = static_cast<const uint8_t *>(b) + static_cast<size_t>(b_index[0]) * k * n * element;
            m *= group;
            batch /= group;
            a_index = b_index = nullptr;
            bias.sb *= group;
        }
    }
    switch (dtype) {
        case RG_F32: return launch_typed<float>(y, a, b, bias, trans_a, trans_b, alpha, beta, batch, m, k, n, a_index, b_index, s);
        case RG_F64: return launch_typed<double>(y, a, b, bias, trans_a, trans_b, alpha, beta, batch, m, k, n, a_index, b_index, s);
        case RG_FP16:
            return launch_typed<__half>(y, a, b, bias, trans_a, trans_b, alpha, beta, batch, m, k, n, a_index, b_index, s, workspace,
                                        workspace_bytes);
        case RG_BF16:
            return launch_typed<__hip_bfloat16>(y, a, b, bias, trans_a, trans_b, alpha, beta, batch, m, k, n, a_index, b_index, s,
                                                workspace, workspace_bytes);
        default: return RG_HIP_E_UNSUPPORTED;
    }
}
