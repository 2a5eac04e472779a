// MatMulInteger for gfx950: Y[i,j] = sum_k int8(A[i,k] - a_zp) * int8(B[k,j] - b_zp), int32.
//
// Arithmetic contract: src/04kernel/src/kernels/mat_mul_integer/cpu_kernel.cc:26-146 of the
// reference.  Operands are bytes; a zero point is subtracted modulo 256 and the difference is
// read as int8 (for both the I8 and the U8 flavour of the reference's `sub`, so the zero-point
// dtype does not change the result byte).  Integer accumulation is exact, so any summation
// order is bit-identical to the reference's serial loop.
//
// Fast path (m, n multiples of 256, k multiple of 128): one 256x256 output tile per workgroup of
// four wavefronts, int8 MFMA 32x32x32, LDS double-buffered k-tiles of 128.  B [k,n] is byte-
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
// registers).  k is walked in tiles of 128 (64 MFMAs per wavefront between barriers):
//   A tile: 256 rows x 128 bytes, k-contiguous as in memory (each row segment is one full
//           128-byte line), LDS rows padded to 144 bytes so that the 128-bit fragment reads of
//           consecutive rows fall into different banks;
//   B tile: 128 k-rows x 256 columns in memory; a thread takes 4 k-rows x 16 columns (four
//           128-bit loads) and byte-transposes the four 4x4 blocks with v_perm_b32, which leaves
//           one dword (4 consecutive k) per column.  The four lanes 16 apart hold the four
//           k-quads of one 16-k group for the same columns; a 4x4 dword transpose across them
//           (v_permlane32_swap + v_permlane16_swap) gives each lane 16 consecutive k of four
//           columns, written with 128-bit stores into LDS laid out [k/16][column][16 k-bytes].
//           The 16-byte slot of a column inside its 256-byte block is XOR-swizzled with the
//           block index so that both these writes and the 128-bit fragment reads are free of
//           bank conflicts.
// Both operands present the same k order to the MFMA, so the contraction is exact.
// Global loads run ahead in registers (two register stages: a tile is loaded one and a half
// iterations before it is written to LDS), LDS is double buffered, and the staging work of
// tile kt+1 (zero-point subtract, transposition, LDS writes) sits in the same basic block as
// the MFMAs of tile kt, with scheduling-group hints that issue it in their shadow.

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int BM = 256, BN = 256, BK = 128;
constexpr int A_ROW = BK + 16;                       // padded LDS row of the A tile, bytes
constexpr int A_TILE = BM * A_ROW;                   // 36864
constexpr int KG_BYTES = BN * 16;                    // one 16-k group of the B tile: [column][16 k-bytes]
constexpr int B_TILE = (BK / 16) * KG_BYTES;         // 32768
constexpr int STAGE_BYTES = A_TILE + B_TILE;         // one LDS buffer (69632)
constexpr int LDS_BYTES = 2 * STAGE_BYTES;           // 139264 of the 160 KiB per CU
constexpr int A_LOADS = BM * BK / (256 * 16);        // 8 128-bit loads per thread per tile
constexpr int B_LOADS = BK * BN / (256 * 16);        // 8


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
    U4 a[A_LOADS];  // rows tid/8 + 32*i, bytes (tid%8)*16 .. +15 of the k-tile
    U4 b[B_LOADS];  // k-rows 64*(i/4) + 4*(tid/16) + i%4, columns 16*(tid%16) .. +15
};

// A_MODE 0: zero point absent, 0 or 128 (one XOR mask); 1: any scalar / per-row zero point.
template <int A_MODE, bool B_ZP>
__device__ __forceinline__ void mmi_tile_loop(v16i (&acc)[4][4], uint8_t *lds, const uint8_t *A,
                                              const uint8_t *B, uint32_t k, uint32_t n,
                                              uint32_t a_xor, const uint32_t (&za_w)[A_LOADS],
                                              ZeroPoint zb, uint64_t zb_row0) {
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t wm = wave >> 1, wn = wave & 1;
    const uint8_t *a_src = A + static_cast<uint64_t>(tid >> 3) * k + (tid & 7) * 16;
    const uint8_t *b_src = B + static_cast<uint64_t>(4 * (tid >> 4)) * n + (tid & 15) * 16;
    const uint32_t a_dst = (tid >> 3) * A_ROW + (tid & 7) * 16;
    // B staging: this lane ends up with columns 16*nb + 4*r + c (c = 0..3) of 16-k group wave + 4h
    const uint32_t nb = tid & 15, r_grp = lane >> 4;
    uint32_t b_dst[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) b_dst[c] = A_TILE + wave * KG_BYTES + 256 * nb + 16 * ((4 * r_grp + c) ^ nb);
    const uint32_t a_frag = (wm * 128 + (lane & 31)) * A_ROW + (lane >> 5) * 16;
    // B fragment j: column wn*128 + 32*j + lane%32 of 16-k group 2*ks + lane/32
    uint32_t b_frag[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t blk = 8 * wn + 2 * j + ((lane >> 4) & 1);
        b_frag[j] = A_TILE + (lane >> 5) * KG_BYTES + 256 * blk + 16 * ((lane & 15) ^ (blk & 15));
    }

    auto load_stage = [&](Stage &st, uint32_t k0) {
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i)
            st.a[i] = *reinterpret_cast<const U4 *>(a_src + static_cast<uint64_t>(32 * i) * k + k0);
#pragma unroll
        for (int i = 0; i < B_LOADS; ++i)
            st.b[i] = *reinterpret_cast<const U4 *>(
                b_src + static_cast<uint64_t>(k0 + 64 * (i / 4) + (i % 4)) * n);
    };

    auto store_stage = [&](const Stage &st, uint32_t buf, uint32_t k0) {
        uint8_t *base = lds + buf * STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i) {
            U4 v = st.a[i];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if constexpr (A_MODE == 0) v.v[e] ^= a_xor;
                else v.v[e] = sub_bytes(v.v[e], za_w[i]);
            }
            *reinterpret_cast<U4 *>(base + a_dst + 32 * i * A_ROW) = v;
        }
#pragma unroll
        for (int h = 0; h < B_LOADS / 4; ++h) {
            uint32_t r[4][4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                uint32_t zw = 0;
                if constexpr (B_ZP) zw = splat(zp_byte(zb, zb_row0 + k0 + 64 * h + 4 * (tid >> 4) + i));
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    r[i][q] = B_ZP ? sub_bytes(st.b[4 * h + i].v[q], zw) : st.b[4 * h + i].v[q];
            }
            uint32_t d[4][4];  // d[q][c]: this lane's k-quad of column 4q + c
#pragma unroll
            for (int q = 0; q < 4; ++q) transpose4x4(r[0][q], r[1][q], r[2][q], r[3][q], d[q]);
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                // 4x4 dword transpose across the lane groups 0-15 / 16-31 / 32-47 / 48-63:
                // afterwards lane group g holds k-quads 0..3 of column 4g + c in d[0..3][c]
                auto s02 = __builtin_amdgcn_permlane32_swap(d[0][c], d[2][c], false, false);
                auto s13 = __builtin_amdgcn_permlane32_swap(d[1][c], d[3][c], false, false);
                auto t01 = __builtin_amdgcn_permlane16_swap(s02[0], s13[0], false, false);
                auto t23 = __builtin_amdgcn_permlane16_swap(s02[1], s13[1], false, false);
                U4 out;
                out.v[0] = t01[0];
                out.v[1] = t01[1];
                out.v[2] = t23[0];
                out.v[3] = t23[1];
                *reinterpret_cast<U4 *>(base + b_dst[c] + 4 * h * KG_BYTES) = out;
            }
        }
    };

    // Fragments: the four B fragments of a k-step stay live through its 16 MFMAs and are double
    // buffered; an A fragment is dead after its row of four MFMAs and is refilled in place with
    // the next k-step's fragment.
    auto read_a = [&](uint32_t buf, int ks, int i) -> v4i {
        return *reinterpret_cast<const v4i *>(lds + buf * STAGE_BYTES + a_frag + i * 32 * A_ROW + ks * 32);
    };
    auto read_b = [&](uint32_t buf, int ks, v4i (&fb)[4]) {
        const uint8_t *base = lds + buf * STAGE_BYTES;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            fb[j] = *reinterpret_cast<const v4i *>(base + b_frag[j] + ks * 2 * KG_BYTES);
    };
    // one k-step: 16 MFMAs; NEXT_KS < 0: no refill (the tile ends)
    auto kstep = [&](v4i (&fa)[4], const v4i (&fb)[4], uint32_t buf, int next_ks) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
            if (next_ks >= 0) fa[i] = read_a(buf, next_ks, i);
        }
    };
    // Issue order requested from the scheduler for one tile (64 MFMAs): fragment reads, the global
    // loads of tile kt+2 and the register part of the staging of tile kt+1 (zero point,
    // transposition) behind the first 48, its LDS writes behind the last 16.  The LDS writes
    // follow the tile's last fragment read in program order because the compiler cannot prove
    // that the two LDS buffers do not alias.
    auto interleave = [&]() {
#pragma unroll
        for (int i = 0; i < 48; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // MFMA
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // DS read
            __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // VMEM read
            __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);  // VALU
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // MFMA
            __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);  // DS write
            __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);  // VALU
        }
    };

    const uint32_t k_tiles = k / BK;
    Stage s0, s1;
    v4i fa[4], fb0[4], fb1[4];
    load_stage(s0, 0);
    store_stage(s0, 0, 0);
    if (k_tiles > 1) load_stage(s1, BK);
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) fa[i] = read_a(0, 0, i);
    read_b(0, 0, fb0);

    // tile j lives in register stage j % 2 and LDS buffer j % 2; fa / fb0 hold the ks = 0
    // fragments of the tile about to be multiplied.  S_FREE is the stage whose tile (kt) is
    // already in LDS.
#define RG_MMI_STEP(KT, S_FREE, S_NEXT1, HAS2, HAS1)                        \
    {                                                                       \
        const uint32_t kt_ = (KT), buf_ = kt_ & 1;                          \
        if (HAS2) load_stage(S_FREE, (kt_ + 2) * BK);                       \
        read_b(buf_, 1, fb1);                                               \
        kstep(fa, fb0, buf_, 1);                                            \
        read_b(buf_, 2, fb0);                                               \
        kstep(fa, fb1, buf_, 2);                                            \
        read_b(buf_, 3, fb1);                                               \
        kstep(fa, fb0, buf_, 3);                                            \
        /* every LDS read of this tile is issued: the LDS writes may follow */ \
        if (HAS1) store_stage(S_NEXT1, buf_ ^ 1, (kt_ + 1) * BK);           \
        kstep(fa, fb1, buf_, -1);                                           \
        interleave();                                                       \
        __syncthreads();                                                    \
        if (HAS1) {                                                         \
            _Pragma("unroll") for (int i = 0; i < 4; ++i) fa[i] = read_a(buf_ ^ 1, 0, i); \
            read_b(buf_ ^ 1, 0, fb0);                                       \
        }                                                                   \
    }
    uint32_t kt = 0;
    for (; kt + 4 <= k_tiles; kt += 2) {  // both steps here have two more tiles behind them
        RG_MMI_STEP(kt, s0, s1, true, true)
        RG_MMI_STEP(kt + 1, s1, s0, true, true)
    }
    // up to three remaining tiles, register stages continuing the alternation
    if (kt < k_tiles) { RG_MMI_STEP(kt, s0, s1, kt + 2 < k_tiles, kt + 1 < k_tiles) ++kt; }
    if (kt < k_tiles) { RG_MMI_STEP(kt, s1, s0, kt + 2 < k_tiles, kt + 1 < k_tiles) ++kt; }
    if (kt < k_tiles) { RG_MMI_STEP(kt, s0, s1, kt + 2 < k_tiles, kt + 1 < k_tiles) ++kt; }
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
    uint32_t za_w[A_LOADS] = {};
    uint32_t a_xor = 0;
    bool a_simple = true;
    if (za.ptr) {
        if (za.per_row) {
            a_simple = false;
#pragma unroll
            for (int i = 0; i < A_LOADS; ++i)
                za_w[i] = splat(za.ptr[am * m + static_cast<uint64_t>(tile_m) * BM + (tid >> 3) + 32 * i]);
        } else {
            const uint32_t z = za.ptr[0];
            if (z == 0 || z == 128) {
                a_xor = splat(z);
            } else {
                a_simple = false;
#pragma unroll
                for (int i = 0; i < A_LOADS; ++i) za_w[i] = splat(z);
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
