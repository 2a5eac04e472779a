// MatMulInteger for gfx950: Y[i,j] = sum_k int8(A[i,k] - a_zp) * int8(B[k,j] - b_zp), int32.
//
// Arithmetic contract: src/04kernel/src/kernels/mat_mul_integer/cpu_kernel.cc:26-146 of the
// reference.  Operands are bytes; a zero point is subtracted modulo 256 and the difference is
// read as int8 (for both the I8 and the U8 flavour of the reference's `sub`, so the zero-point
// dtype does not change the result byte).  Integer accumulation is exact, so any summation
// order is bit-identical to the reference's serial loop.
//
// Fast path (m, n multiples of 256, k multiple of 64): one 256x256 output tile per workgroup of
// four wavefronts, int8 MFMA 32x32x32, LDS double-buffered k-tiles of 64.  B [k,n] is byte-
// transposed on its way into LDS so that both MFMA operands are k-contiguous.  Zero points are
// folded into the staging step (XOR / packed byte subtract), so there is no pre-pass over A or
// B and no workspace.  Everything else goes through a plain tiled kernel.
#include "common.hpp"

namespace rg {
namespace {

// ---------------------------------------------------------------- zero points

// One zero-point byte per (matrix, row) of an operand, or one for the whole operand, or none.
struct ZeroPoint {
    const uint8_t *ptr;  // nullptr: none
    uint32_t per_row;    // 0: scalar
};

__device__ __forceinline__ uint32_t zp_byte(const ZeroPoint &z, uint64_t matrix_row) {
    if (!z.ptr) return 0;
    return z.per_row ? z.ptr[matrix_row] : z.ptr[0];
}

// Four lane-wise byte subtractions modulo 256 (SWAR): x - z per byte.
__device__ __forceinline__ uint32_t sub_bytes(uint32_t x, uint32_t z) {
    constexpr uint32_t H = 0x80808080u;
    return ((x | H) - (z & ~H)) ^ ((x ^ ~z) & H);
}

__device__ __forceinline__ uint32_t splat(uint32_t byte) { return byte * 0x01010101u; }

// ---------------------------------------------------------------- generic kernel
// 16x16 outputs per workgroup, one per thread; k walked in LDS tiles of 16.

__global__ __launch_bounds__(256) void mmi_generic(int32_t *__restrict__ y,
                                                   const uint8_t *__restrict__ a,
                                                   const uint8_t *__restrict__ b, ZeroPoint za,
                                                   ZeroPoint zb, uint32_t m, uint32_t k, uint32_t n,
                                                   uint32_t a_matrix0, uint32_t b_matrix0,
                                                   uint32_t y_matrix0) {
    __shared__ int8_t ta[16][17];
    __shared__ int8_t tb[16][17];
    const uint32_t bz = blockIdx.z;
    const uint64_t am = a_matrix0 + bz, bm = b_matrix0 + bz, ym = y_matrix0 + bz;
    const uint8_t *A = a + am * m * k;
    const uint8_t *B = b + bm * static_cast<uint64_t>(k) * n;
    const uint32_t tx = threadIdx.x % 16, ty = threadIdx.x / 16;
    const uint32_t row = blockIdx.y * 16 + ty, col = blockIdx.x * 16 + tx;
    int32_t acc = 0;
    for (uint32_t k0 = 0; k0 < k; k0 += 16) {
        // A tile element (ty, tx): row `row`, k index k0+tx
        int8_t va = 0, vb = 0;
        if (row < m && k0 + tx < k)
            va = static_cast<int8_t>(A[static_cast<uint64_t>(row) * k + k0 + tx] - zp_byte(za, am * m + row));
        // B tile element (ty, tx): k index k0+ty, column `col`
        if (k0 + ty < k && col < n)
            vb = static_cast<int8_t>(B[static_cast<uint64_t>(k0 + ty) * n + col] - zp_byte(zb, bm * k + k0 + ty));
        ta[ty][tx] = va;
        tb[ty][tx] = vb;
        __syncthreads();
#pragma unroll
        for (int q = 0; q < 16; ++q) acc += static_cast<int32_t>(ta[ty][q]) * static_cast<int32_t>(tb[q][tx]);
        __syncthreads();
    }
    if (row < m && col < n) y[(ym * m + row) * n + col] = acc;
}

// ---------------------------------------------------------------- MFMA kernel
//
// Workgroup = 256 threads = four wavefronts (one per SIMD), one 256x256 tile of Y; wavefront
// (wm, wn) owns the 128x128 quadrant as 4x4 blocks of v_mfma_i32_32x32x32_i8 (256 accumulator
// registers).  k is walked in tiles of 64:
//   A tile: 256 rows x 64 bytes, k-contiguous as in memory, LDS rows padded to 80 bytes so the
//           128-bit fragment reads of consecutive rows fall into different banks;
//   B tile: 64 k-rows x 256 columns in memory; every thread takes 4 k-rows x 16 columns
//           (four 128-bit loads), byte-transposes the four 4x4 blocks with v_perm_b32 and
//           writes 64 contiguous bytes into LDS laid out [k/4][column][4 k-bytes].  A fragment
//           (16 consecutive k of one column) is then four 32-bit LDS reads 1 KiB apart.
// Both operands present the same k order to the MFMA, so the contraction is exact.
// Global loads run two k-tiles ahead in registers (three register stages), LDS is double
// buffered, and the staging work of tile kt+1 (zero-point subtract, transposition, LDS writes)
// is in the same basic block as the MFMAs of tile kt so that it issues in their shadow.

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int A_ROW = BK + 16;                       // padded LDS row of the A tile, bytes
constexpr int A_TILE = BM * A_ROW;                   // 20480
constexpr int B_TILE = (BK / 4) * BN * 4;            // 16384
constexpr int STAGE_BYTES = A_TILE + B_TILE;         // one LDS buffer
constexpr int LDS_BYTES = 2 * STAGE_BYTES;

// 4x4 byte transpose: in[r] holds bytes (r,0..3); out[c] holds bytes (0..3,c).
__device__ __forceinline__ void transpose4x4(uint32_t i0, uint32_t i1, uint32_t i2, uint32_t i3,
                                             uint32_t out[4]) {
    // v_perm_b32(s0, s1, sel): result byte i = byte sel[i] of the 8 bytes {s1 (0-3), s0 (4-7)}
    const uint32_t t0 = __builtin_amdgcn_perm(i1, i0, 0x05010400u);  // r0b0 r1b0 r0b1 r1b1
    const uint32_t t1 = __builtin_amdgcn_perm(i1, i0, 0x07030602u);  // r0b2 r1b2 r0b3 r1b3
    const uint32_t t2 = __builtin_amdgcn_perm(i3, i2, 0x05010400u);  // r2b0 r3b0 r2b1 r3b1
    const uint32_t t3 = __builtin_amdgcn_perm(i3, i2, 0x07030602u);  // r2b2 r3b2 r2b3 r3b3
    out[0] = __builtin_amdgcn_perm(t2, t0, 0x05040100u);  // r0b0 r1b0 r2b0 r3b0
    out[1] = __builtin_amdgcn_perm(t2, t0, 0x07060302u);
    out[2] = __builtin_amdgcn_perm(t3, t1, 0x05040100u);
    out[3] = __builtin_amdgcn_perm(t3, t1, 0x07060302u);
}

struct alignas(16) U4 {
    uint32_t v[4];
};

// Register-staged global loads of one k-tile for one thread.
struct Stage {
    U4 a[4];  // rows tid/4 + 64*i, bytes (tid%4)*16 .. +15 of the k-tile
    U4 b[4];  // k-rows 4*(tid/16) + i, columns 16*(tid%16) .. +15
};

// A_MODE 0: zero point absent, 0 or 128 (one XOR mask); 1: any scalar / per-row zero point.
template <int A_MODE, bool B_ZP>
__device__ __forceinline__ void mmi_tile_loop(v16i (&acc)[4][4], uint8_t *lds, const uint8_t *A,
                                              const uint8_t *B, uint32_t k, uint32_t n,
                                              uint32_t a_xor, const uint32_t (&za_w)[4],
                                              ZeroPoint zb, uint64_t zb_row0) {
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t wm = wave >> 1, wn = wave & 1;
    const uint8_t *a_src = A + static_cast<uint64_t>(tid >> 2) * k + (tid & 3) * 16;
    const uint8_t *b_src = B + static_cast<uint64_t>(4 * (tid >> 4)) * n + (tid & 15) * 16;
    const uint32_t a_dst = (tid >> 2) * A_ROW + (tid & 3) * 16;
    const uint32_t b_dst = A_TILE + (tid >> 4) * (BN * 4) + (tid & 15) * 64;
    const uint32_t a_frag = (wm * 128 + (lane & 31)) * A_ROW + (lane >> 5) * 16;
    const uint32_t b_frag = A_TILE + (lane >> 5) * (4 * BN * 4) + (wn * 128 + (lane & 31)) * 4;

    auto load_stage = [&](Stage &st, uint32_t k0) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            st.a[i] = *reinterpret_cast<const U4 *>(a_src + static_cast<uint64_t>(64 * i) * k + k0);
#pragma unroll
        for (int i = 0; i < 4; ++i)
            st.b[i] = *reinterpret_cast<const U4 *>(b_src + static_cast<uint64_t>(k0 + i) * n);
    };

    auto store_stage = [&](const Stage &st, uint32_t buf, uint32_t k0) {
        uint8_t *base = lds + buf * STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            U4 v = st.a[i];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if constexpr (A_MODE == 0) v.v[e] ^= a_xor;
                else v.v[e] = sub_bytes(v.v[e], za_w[i]);
            }
            *reinterpret_cast<U4 *>(base + a_dst + 64 * i * A_ROW) = v;
        }
        uint32_t r[4][4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t zw = 0;
            if constexpr (B_ZP) zw = splat(zp_byte(zb, zb_row0 + k0 + 4 * (tid >> 4) + i));
#pragma unroll
            for (int q = 0; q < 4; ++q) r[i][q] = B_ZP ? sub_bytes(st.b[i].v[q], zw) : st.b[i].v[q];
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            U4 out;
            transpose4x4(r[0][q], r[1][q], r[2][q], r[3][q], out.v);
            *reinterpret_cast<U4 *>(base + b_dst + q * 16) = out;
        }
    };

    auto compute = [&](uint32_t buf) {
        const uint8_t *base = lds + buf * STAGE_BYTES;
#pragma unroll
        for (int ks = 0; ks < BK / 32; ++ks) {
            v4i fa[4], fb[4];
#pragma unroll
            for (int i = 0; i < 4; ++i)
                fa[i] = *reinterpret_cast<const v4i *>(base + a_frag + i * 32 * A_ROW + ks * 32);
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    fb[j][q] = *reinterpret_cast<const int *>(base + b_frag + (ks * 8 + q) * (BN * 4) + j * 128);
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
    };

    const uint32_t k_tiles = k / BK;
    Stage s0, s1, s2;
    load_stage(s0, 0);
    if (k_tiles > 1) load_stage(s1, BK);
    store_stage(s0, 0, 0);
    __syncthreads();

    // tile j lives in register stage j % 3 and LDS buffer j % 2
#define RG_MMI_STEP(KT, S_NEXT2, S_NEXT1)                                   \
    {                                                                       \
        const uint32_t kt_ = (KT);                                          \
        if (kt_ + 2 < k_tiles) load_stage(S_NEXT2, (kt_ + 2) * BK);         \
        compute(kt_ & 1);                                                   \
        if (kt_ + 1 < k_tiles) store_stage(S_NEXT1, (kt_ + 1) & 1, (kt_ + 1) * BK); \
        __syncthreads();                                                    \
    }
    uint32_t kt = 0;
    for (; kt + 3 <= k_tiles; kt += 3) {
        RG_MMI_STEP(kt, s2, s1)
        RG_MMI_STEP(kt + 1, s0, s2)
        RG_MMI_STEP(kt + 2, s1, s0)
    }
    if (kt < k_tiles) {
        RG_MMI_STEP(kt, s2, s1)
        ++kt;
    }
    if (kt < k_tiles) {
        RG_MMI_STEP(kt, s0, s2)
    }
#undef RG_MMI_STEP
}

__global__ __launch_bounds__(256, 1) void mmi_mfma_256x256(int32_t *__restrict__ y,
                                                           const uint8_t *__restrict__ a,
                                                           const uint8_t *__restrict__ b,
                                                           ZeroPoint za, ZeroPoint zb, uint32_t m,
                                                           uint32_t k, uint32_t n,
                                                           uint32_t a_matrix0, uint32_t b_matrix0,
                                                           uint32_t y_matrix0) {
    extern __shared__ __align__(16) uint8_t lds[];

    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t bz = blockIdx.z;
    const uint64_t am = a_matrix0 + bz, bm = b_matrix0 + bz, ym = y_matrix0 + bz;

    // XCD-aware tile order: consecutive workgroup ids are dealt round-robin to the 8 XCDs, so
    // give each XCD a contiguous block of tiles (they then share A row-panels / B column-panels
    // in that XCD's L2).
    const uint32_t tiles_n = n / BN, tiles_m = m / BM, n_tiles = tiles_m * tiles_n;
    uint32_t t = blockIdx.x;
    if (n_tiles % 8 == 0) t = (t % 8) * (n_tiles / 8) + t / 8;
    // within the linear order walk tiles in column-major groups of 4 rows to keep panels hot
    const uint32_t group = 4 * tiles_n;
    const uint32_t g = t / group, r = t % group;
    const uint32_t rows_here = tiles_m - g * 4 < 4 ? tiles_m - g * 4 : 4;
    const uint32_t tile_m = g * 4 + r % rows_here, tile_n = r / rows_here;

    const uint8_t *A = a + (am * m + static_cast<uint64_t>(tile_m) * BM) * k;
    const uint8_t *B = b + bm * static_cast<uint64_t>(k) * n + static_cast<uint64_t>(tile_n) * BN;

    v16i acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

    // zero points of this thread's staged A rows; scalar 0 / 128 (or none) reduce to one XOR mask
    uint32_t za_w[4] = {0, 0, 0, 0};
    uint32_t a_xor = 0;
    bool a_simple = true;
    if (za.ptr) {
        if (za.per_row) {
            a_simple = false;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                za_w[i] = splat(za.ptr[am * m + static_cast<uint64_t>(tile_m) * BM + (tid >> 2) + 64 * i]);
        } else {
            const uint32_t z = za.ptr[0];
            if (z == 0 || z == 128) {
                a_xor = splat(z);
            } else {
                a_simple = false;
#pragma unroll
                for (int i = 0; i < 4; ++i) za_w[i] = splat(z);
            }
        }
    }
    // a scalar zero point of 0 on B is the common case: skip the subtract entirely
    bool b_zp = zb.ptr != nullptr;
    if (b_zp && !zb.per_row && zb.ptr[0] == 0) b_zp = false;
    const uint64_t zb_row0 = bm * k;

    if (a_simple) {
        if (!b_zp) mmi_tile_loop<0, false>(acc, lds, A, B, k, n, a_xor, za_w, zb, zb_row0);
        else mmi_tile_loop<0, true>(acc, lds, A, B, k, n, a_xor, za_w, zb, zb_row0);
    } else {
        if (!b_zp) mmi_tile_loop<1, false>(acc, lds, A, B, k, n, a_xor, za_w, zb, zb_row0);
        else mmi_tile_loop<1, true>(acc, lds, A, B, k, n, a_xor, za_w, zb, zb_row0);
    }

    // 32x32 accumulator layout: lane holds column (lane % 32); register e holds row
    // 8*(e/4) + 4*(lane/32) + e%4.  Y is written once and not re-read: streaming stores.
    const uint32_t wm = wave >> 1, wn = wave & 1;
    int32_t *Y = y + (ym * m + static_cast<uint64_t>(tile_m) * BM + wm * 128) * n +
                 static_cast<uint64_t>(tile_n) * BN + wn * 128;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const uint32_t row = i * 32 + 8 * (e / 4) + 4 * (lane >> 5) + (e % 4);
                const uint32_t col = j * 32 + (lane & 31);
                __builtin_nontemporal_store(acc[i][j][e], Y + static_cast<uint64_t>(row) * n + col);
            }
}

}  // namespace
}  // namespace rg

extern "C" size_t rg_hip_matmul_integer_workspace(size_t, size_t, size_t, size_t, unsigned) {
    return 0;
}

extern "C" int rg_hip_matmul_integer(int32_t *y, const void *a, const void *b, const void *a_zp,
                                     const void *b_zp, unsigned flags, size_t batch, size_t m,
                                     size_t k, size_t n, const uint32_t *a_index,
                                     const uint32_t *b_index, void * /*workspace*/, void *stream) {
    using namespace rg;
    if (!y || !a || !b) return RG_HIP_E_ARGUMENT;
    if (batch == 0 || m == 0 || n == 0) return 0;
    if (m > 0x7fffffffu || n > 0x7fffffffu || k > 0x7fffffffu || batch > 0xffffffffu)
        return RG_HIP_E_UNSUPPORTED;
    hipStream_t s = as_stream(stream);
    const ZeroPoint za{static_cast<const uint8_t *>(a_zp), (flags & RG_MMI_A_ZP_SCALAR) ? 0u : 1u};
    const ZeroPoint zb{static_cast<const uint8_t *>(b_zp), (flags & RG_MMI_B_ZP_SCALAR) ? 0u : 1u};
    const bool fast = m % BM == 0 && n % BN == 0 && k % BK == 0 && k > 0 && aligned16(a) && aligned16(b);

    auto launch = [&](uint32_t am0, uint32_t bm0, uint32_t ym0, uint32_t count) -> int {
        if (fast) {
            static bool attr_set = false;
            constexpr size_t lds_bytes = LDS_BYTES;
            if (!attr_set) {
                hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(mmi_mfma_256x256),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize,
                                                   static_cast<int>(lds_bytes));
                if (e != hipSuccess) return static_cast<int>(e);
                attr_set = true;
            }
            const dim3 grid(static_cast<unsigned>((m / BM) * (n / BN)), 1, count);
            mmi_mfma_256x256<<<grid, 256, lds_bytes, s>>>(
                y, static_cast<const uint8_t *>(a), static_cast<const uint8_t *>(b), za, zb,
                static_cast<uint32_t>(m), static_cast<uint32_t>(k), static_cast<uint32_t>(n), am0, bm0, ym0);
        } else {
            const dim3 grid(static_cast<unsigned>((n + 15) / 16), static_cast<unsigned>((m + 15) / 16), count);
            mmi_generic<<<grid, 256, 0, s>>>(
                y, static_cast<const uint8_t *>(a), static_cast<const uint8_t *>(b), za, zb,
                static_cast<uint32_t>(m), static_cast<uint32_t>(k), static_cast<uint32_t>(n), am0, bm0, ym0);
        }
        return launch_status();
    };

    if (!a_index && !b_index) {
        // grid.z is limited to 65535
        for (size_t i = 0; i < batch; i += 65535) {
            const uint32_t count = static_cast<uint32_t>(batch - i < 65535 ? batch - i : 65535);
            const int rc = launch(static_cast<uint32_t>(i), static_cast<uint32_t>(i), static_cast<uint32_t>(i), count);
            if (rc) return rc;
        }
        return 0;
    }
    for (size_t i = 0; i < batch; ++i) {
        const int rc = launch(a_index ? a_index[i] : static_cast<uint32_t>(i),
                              b_index ? b_index[i] : static_cast<uint32_t>(i), static_cast<uint32_t>(i), 1);
        if (rc) return rc;
    }
    return 0;
}
