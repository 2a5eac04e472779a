// MatMulInteger for gfx950: Y[i,j] = sum_k int8(A[i,k] - a_zp) * int8(B[k,j] - b_zp), int32.
//
// Arithmetic contract: src/04kernel/src/kernels/mat_mul_integer/cpu_kernel.cc:26-146 of the
// reference.  Operands are bytes; a zero point is subtracted modulo 256 and the difference is
// read as int8 (for both the I8 and the U8 flavour of the reference's `sub`, so the zero-point
// dtype does not change the result byte).  Integer accumulation is exact, so any summation
// order is bit-identical to the reference's serial loop.
//
// Fast path (m, n multiples of 256, k multiple of 128): one 256x256 output tile per workgroup of
// four wavefronts, int8 MFMA 32x32x32, k-tiles of 128 copied from global memory straight into two
// LDS buffers.  B [k,n] stays as in memory and is byte-transposed by the LDS read, so that both
// MFMA operands are k-contiguous.  Zero points are applied to the operand fragments, so there is
// no pre-pass over A or B and no workspace.  Everything else goes through a plain tiled kernel.
#include <type_traits>
#include <utility>

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

// Optional epilogue: the int32 sum leaves as float(sum) * scale (DequantizeLinear without zero point,
// src/04kernel/src/kernels/dequantize_linear/cpu_kernel.cc:17-28: one conversion, one multiplication),
// with one scale for the tensor or one per column of Y.
struct Dequant {
    const float *scale;
    uint32_t per_column;
};
template <bool DEQ>
__device__ __forceinline__ int32_t finish(int32_t sum, float scale) {
    if constexpr (DEQ) return __builtin_bit_cast(int32_t, static_cast<float>(sum) * scale);
    else return sum;
}

// ---------------------------------------------------------------- generic kernel
// 16x16 outputs per workgroup, one per thread; k walked in LDS tiles of 16.

template <bool DEQ>
__global__ __launch_bounds__(256) void mmi_generic(int32_t *__restrict__ y,
                                                   const uint8_t *__restrict__ a,
                                                   const uint8_t *__restrict__ b, ZeroPoint za,
                                                   ZeroPoint zb, Dequant dq, uint32_t m, uint32_t k, uint32_t n,
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
    if (row < m && col < n) y[(ym * m + row) * n + col] = finish<DEQ>(acc, DEQ ? dq.scale[dq.per_column ? col : 0] : 0.f);
}

// ---------------------------------------------------------------- MFMA kernel
//
// Workgroup = 256 threads = four wavefronts (one per SIMD), one 256x256 tile of Y; wavefront
// (wm, wn) owns the 128x128 quadrant as 4x4 blocks of v_mfma_i32_32x32x32_i8 (256 accumulator
// registers).  k is walked in tiles of 128 (64 MFMAs per wavefront) through two LDS buffers.
// There is no register staging: both tiles go from global memory into LDS with
// global_load_lds_dwordx4 (lane L of a wavefront-wide copy fills bytes 16 L .. 16 L + 15 behind a
// wave-uniform LDS base, from a global address of its own), 16 copies per wavefront and k-tile.
//   A tile: 256 rows of 128 bytes, unpadded; the 16-byte chunk c of row r sits at chunk position
//           c ^ (r & 7) ^ ((r >> 3) & 1), which spreads the 128-bit fragment reads of 8 as well
//           as of 16 consecutive rows over all banks.
//   B tile: as in memory, 128 k-rows of 256 bytes; chunk c of k-row r sits at chunk position
//           c ^ swz(r & 7).  The MFMA operand (16 consecutive k of one column per lane) is formed
//           by ds_read_b64_tr_b8: within 16 lanes, lane i receives byte i % 8 of the 8-byte pieces
//           addressed by lanes i / 8, i / 8 + 2, ..., so lanes 2 j and 2 j + 1 address the two
//           halves of the 16 columns in k-row j and every lane gets 8 consecutive k of its column.
// Both operands present the same k order to the MFMA, so the contraction is exact.  Zero points
// are applied to the fragments (one XOR mask, or a packed byte subtract), so there is no pre-pass
// over A or B and no workspace.  One k-tile is 64 MFMAs per wavefront in a fixed order (a
// scheduling barrier after each with its share of LDS reads and copies); fragments are double
// buffered by k-step.  The barrier of a tile sits before its last k-step: after it the buffer
// just multiplied is refilled with tile kt+2 while the last 16 MFMAs run from registers and the
// first fragments of tile kt+1 arrive.

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int BM = 256, BN = 256, BK = 128;
constexpr int D_TILE = 32768;            // A 256 x 128 or B 128 x 256
constexpr int D_STAGE = 2 * D_TILE;      // one LDS buffer

__device__ __forceinline__ uint32_t b_swizzle(uint32_t x) { return ((x & 3) << 1) | ((x >> 2) * 9); }  // x < 8

// A wave-uniform pointer, moved to scalar registers (so that what is added to it later is scalar arithmetic).
// (The builtin returns int: without the casts the low word would be sign-extended over the high one.)
__device__ __forceinline__ const uint8_t *scalar_pointer(const uint8_t *p) {
    const uint64_t bits = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<uint32_t>(bits)));
    const uint32_t hi = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<uint32_t>(bits >> 32)));
    return reinterpret_cast<const uint8_t *>((static_cast<uint64_t>(hi) << 32) | lo);
}

// SHORT_M: A has only a_rows < 256 rows; the tile's rows beyond them are copied from the last one (their results
// are not stored).
template <int A_MODE, bool B_ZP, bool SHORT_M>
__device__ __forceinline__ void mmi_tile_loop(v16i (&acc)[4][4], uint8_t *lds0, uint8_t *lds1,
                                              const uint8_t *A, const uint8_t *B, uint32_t k, uint32_t lda, uint32_t n,
                                              uint32_t a_xor, const uint32_t (&za_f)[4], ZeroPoint zb,
                                              uint64_t zb_row0, uint32_t a_rows, uint8_t *zlds) {
    // k: length of the range of k walked here (A, B and zb_row0 point at its start); lda: bytes per row of A
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t wm = wave >> 1, wn = wave & 1, h = lane >> 5;
    // copy q < 8: A rows 8 (8 wave + q) .. + 7, this lane row + lane / 8, chunk position lane % 8;
    // copy 8 + p: B k-rows 4 (8 wave + p) .. + 3, this lane k-row + lane / 16, chunk position lane % 16
    const uint8_t *a_wave = scalar_pointer(A + static_cast<uint64_t>(wave * 64) * lda);
    const uint32_t a_lane = (lane >> 3) * lda + 16 * ((lane & 7) ^ (lane >> 3));
    const uint8_t *b_wave = scalar_pointer(B + static_cast<uint64_t>(wave * 32) * n);
    uint32_t b_lane[2];
#pragma unroll
    for (int p = 0; p < 2; ++p) b_lane[p] = (lane >> 4) * n + 16 * ((lane & 15) ^ b_swizzle(4 * p + (lane >> 4)));
    // The copies are issued as assembly, a scalar base plus a 32-bit lane offset (the host keeps 8 rows of A and
    // 4 k-rows of B below 2^31 bytes): no vector arithmetic per copy, and the compiler, which then does not know
    // that a vector-memory instruction writes LDS, adds no waits of its own; the waits for copies in this file are
    // the explicit ones in front of the barriers.  (Writing M0 needs one wait state before the copy reads it.)
    const uint32_t a_lane2[2] = {a_lane, a_lane ^ 16u};
    const uint32_t lds_addr[2] = {
        static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) uint8_t *)lds0)),
        static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) uint8_t *)lds1))};
    auto copy = [&](uint8_t *base, uint32_t k0, int q) {
        const uint32_t to = base == lds0 ? lds_addr[0] : lds_addr[1];
        const uint8_t *src;
        uint32_t lane_off, dst;
        if (q < 8) {
            if constexpr (SHORT_M) {
                const uint32_t row = wave * 64 + 8 * q + (lane >> 3);
                src = A + k0;
                lane_off = (row < a_rows ? row : a_rows - 1) * lda + 16 * ((lane & 7) ^ (lane >> 3) ^ (q & 1));
            } else {
                src = a_wave + (k0 + static_cast<uint64_t>(8 * q) * lda);
                lane_off = a_lane2[q & 1];
            }
            dst = to + (wave * 8 + q) * 1024;
        } else {
            src = b_wave + static_cast<uint64_t>(k0 + 4 * (q - 8)) * n;
            lane_off = b_lane[q & 1];
            dst = to + D_TILE + (wave * 8 + (q - 8)) * 1024;
        }
        src = scalar_pointer(src);
        dst = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(dst));
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                     :
                     : "v"(lane_off), "s"(src), "s"(dst)
                     : "memory", "m0");
    };
    // A fragment i of k-step ks: row wm 128 + 32 i + lane % 32, chunk 2 ks + h
    const uint32_t a_off = (wm * 128 + (lane & 31)) * 128 + 16 * (h ^ (lane & 7) ^ ((lane >> 3) & 1));
    auto read_a = [&](const uint8_t *base, int ks, int i) -> v4i {
        return *reinterpret_cast<const v4i *>(base + (a_off ^ (32 * ks)) + i * 4096);
    };
    // B fragment j of k-step ks: column wn 128 + 32 j + lane % 32, k 16 (2 ks + h) .. + 15 in two reads
    uint32_t b_off[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t a16 = lane & 15, chunk = wn * 8 + 2 * j + ((lane >> 4) & 1);
        b_off[j] = D_TILE + (16 * h + (a16 >> 1)) * 256 + 16 * (chunk ^ b_swizzle(a16 >> 1)) + 8 * (a16 & 1);
    }
    typedef int v2i __attribute__((ext_vector_type(2)));
    auto read_b = [&](const uint8_t *base, int ks, int j, int half, v4i &f) {
        const v2i r = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
            (__attribute__((address_space(3))) v2i *)(base + b_off[j] + (32 * ks + 8 * half) * 256));
        f[2 * half] = r[0];
        f[2 * half + 1] = r[1];
    };
    auto fix_a = [&](v4i &f, int i) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if constexpr (A_MODE == 0) f[e] ^= static_cast<int>(a_xor);
            else f[e] = static_cast<int>(sub_bytes(static_cast<uint32_t>(f[e]), za_f[i]));
        }
    };
    // B's zero points (one per k-row) of the sixteen k of a fragment, held in registers a k-step ahead like the
    // fragments.  No global load may stand in the loop: its wait would be a wait for every copy in flight (the
    // counter is shared), which doubled the time of a launch.  A scalar zero point is read once; per-row ones
    // travel with their tile, one more copy per wavefront and tile (128 bytes into a slot of the wavefront's own),
    // when their address is a multiple of 4; otherwise they are loaded from memory as before.
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const int z_mode = !B_ZP ? 1 : !zb.per_row ? 1 : (reinterpret_cast<uintptr_t>(zb.ptr) & 3u) == 0 ? 2 : 0;
    const uint32_t z_lds = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) uint8_t *)zlds));
    u32x4 zr[2];
    if (B_ZP && !zb.per_row) {
        const uint32_t z = splat(zb.ptr[0]);
        zr[0] = zr[1] = u32x4{z, z, z, z};
    } else {
        zr[0] = zr[1] = u32x4{0u, 0u, 0u, 0u};
    }
    auto copy_z = [&](int stage, uint32_t k0) {  // 128 zero points of the k-rows k0 .. k0 + 127 into this wavefront's slot
        const uint8_t *src = scalar_pointer(zb.ptr + zb_row0 + k0);
        const uint32_t dst = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(z_lds + (stage * 4 + wave) * 256));
        const uint32_t lane_off = 4 * (lane & 31);  // (the upper half of the wavefront fetches the same bytes again)
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1"
                     :
                     : "v"(lane_off), "s"(src), "s"(dst)
                     : "memory", "m0");
    };
    auto read_z = [&](int stage, uint32_t k0, int ks, u32x4 &z) {
        if constexpr (B_ZP) {
            if (z_mode == 2) z = *reinterpret_cast<const u32x4 *>(zlds + (stage * 4 + wave) * 256 + 16 * (2 * ks + h));
            else if (z_mode == 0) __builtin_memcpy(&z, zb.ptr + zb_row0 + k0 + 16 * (2 * ks + h), 16);
        }
    };
    auto fix_b = [&](v4i &f, const u32x4 &z) {
        if constexpr (B_ZP) {
#pragma unroll
            for (int e = 0; e < 4; ++e) f[e] = static_cast<int>(sub_bytes(static_cast<uint32_t>(f[e]), z[e]));
        }
    };

    const uint32_t k_tiles = k / BK;
    v4i fa[2][4], fb[2][4];
#pragma unroll
    for (int q = 0; q < 16; ++q) copy(lds0, 0, q);
    if (z_mode == 2) copy_z(0, 0);
#pragma unroll
    for (int q = 0; q < 16; ++q) copy(lds1, k_tiles > 1 ? BK : 0, q);  // k_tiles == 1: tile 0 again, never multiplied
    if (z_mode == 2) {
        copy_z(1, k_tiles > 1 ? BK : 0);
        asm volatile("s_waitcnt vmcnt(17)" ::: "memory");  // tile 0 (the 17 older copies)
    } else {
        asm volatile("s_waitcnt vmcnt(16)" ::: "memory");  // tile 0 (the 16 older copies)
    }
    __syncthreads();
    read_z(0, 0, 0, zr[0]);
#pragma unroll
    for (int i = 0; i < 4; ++i) fa[0][i] = read_a(lds0, 0, i);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        read_b(lds0, 0, j, 0, fb[0][j]);
        read_b(lds0, 0, j, 1, fb[0][j]);
    }

    // Tile kt is in buffer RB, tile kt+1 arrives in WB.
    auto step = [&](uint32_t kt_, uint8_t *RB, const uint8_t *WB) __attribute__((always_inline)) {
        // the tile after next; behind the end, tile 0 once more (never multiplied): no branch around the copies
        const uint32_t k_cp = kt_ + 2 < k_tiles ? (kt_ + 2) * BK : 0;
        auto slot = [&]<int s>() __attribute__((always_inline)) {
            // rows walk the columns back and forth, so that only one operand changes between MFMAs
            constexpr int ks = s / 16, o = s % 16, row = o / 4, col = (row & 1) ? 3 - o % 4 : o % 4;
            constexpr int cur = ks & 1, nxt = cur ^ 1;
            if constexpr (s == 48) {
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wavefront's part of tile kt+1
                __syncthreads();                                  // tile kt+1 complete, RB no longer read
            }
            if constexpr (o % 4 == 0) fix_a(fa[cur][row], row);
            if constexpr (row == 0) fix_b(fb[cur][col], zr[cur]);
            acc[row][col] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[cur][row], fb[cur][col], acc[row][col], 0, 0, 0);
            const uint8_t *src = ks == 3 ? WB : RB;
            constexpr int nks = (ks + 1) % 4;
            if constexpr (o < 4) fa[nxt][o] = read_a(src, nks, o);
            else if constexpr (o < 12) read_b(src, nks, (o - 4) / 2, (o - 4) % 2, fb[nxt][(o - 4) / 2]);
            else if constexpr (o == 12) read_z(src == lds0 ? 0 : 1, (ks == 3 ? kt_ + 1 : kt_) * BK, nks, zr[nxt]);
            if constexpr (s >= 48) copy(RB, k_cp, s - 48);
            if constexpr (s == 63 && B_ZP) {
                if (z_mode == 2) copy_z(RB == lds0 ? 0 : 1, k_cp);
            }
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

// The walk through k for the common case (a scalar zero point of 0 or 128 for A, none for B, full tiles), laid out
// for a wavefront that is alone on its SIMD: whatever it issues besides its products has to fit behind them.
// Measured on this part: a product occupies the matrix pipe for 32 clocks, in which the wavefront issues up to six
// more vector or scalar instructions (or two LDS reads) without delaying the next product; a seventh costs its own
// four clocks, dependent scalar arithmetic eight clocks an instruction, and the four wavefronts' copies share one
// address unit (16 clocks per 1 KiB copy), so a burst of sixteen copies per wavefront in sixteen consecutive slots
// queues up there and holds the wavefronts.  Hence:
//   * a copy is one scalar add into M0 and the copy itself: its source is one scalar base per operand and tile plus
//     a per-copy lane offset that stays in a register;
//   * the XOR of an A fragment's four words is dealt to four consecutive slots, ahead of the fragment's first use;
//   * fragment reads are issued in pairs in the first six slots of a k-step;
//   * the copies of a tile are dealt over a whole tile's worth of slots, one every fourth slot, through a ring of
//     four 32 KiB stages of 64 k each (A 256 x 64 at +0, B 64 x 256 at +16384).
// Tile t lives in stage t % 4; its stage is free again after the barrier in the middle of tile t (all its fragment
// reads are issued in the first half of the tile), from where the A part of tile t + 4 is copied into it (slots 16,
// 20, 24, 28) and then the B part (slots 0, 4, 8, 12 of tile t + 1).  The same barrier, behind a wait for all but the
// 16 newest copies, makes tile t + 1 visible to every wavefront.
//   A stage: row r at r * 64, chunk c of it at position c ^ ((r >> 2) & 3)
//   B stage: k-row r at r * 256, chunk c at position c ^ b_swizzle(r & 7)
// (2,630 clocks per 128 of k against 3,030 for the two-buffer loop below, which the other cases keep.  On uniform
// random bytes the part is power-limited and gives the clocks back as a lower frequency, 1.61 against 1.77 GHz inside
// the loop; operands that toggle fewer bits keep the gain: all-zero operands 52.5 -> 46.1 us at 4096^3.)
__device__ __forceinline__ void mmi_tile_loop_ring(v16i (&acc)[4][4], uint8_t *lds, const uint8_t *A, const uint8_t *B,
                                                   uint32_t k, uint32_t lda, uint32_t n, uint32_t a_xor) {
    constexpr uint32_t RK = 64, R_STAGE = 32768, R_B = 16384;
    const uint32_t tid = threadIdx.x, lane = tid & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t wm = wave >> 1, wn = wave & 1, h = lane >> 5;
    const uint8_t *a_wave = scalar_pointer(A + static_cast<uint64_t>(wave * 64) * lda);
    const uint8_t *b_wave = scalar_pointer(B + static_cast<uint64_t>(wave * 16) * n);
    // copy q < 4: A rows 16 (4 wave + q) .. + 15, this lane row + lane / 4, chunk position lane % 4;
    // copy 4 + p: B k-rows 4 (4 wave + p) .. + 3, this lane k-row + lane / 16, chunk position lane % 16
    uint32_t voff[8];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        voff[q] = (16 * q + (lane >> 2)) * lda + 16 * ((lane & 3) ^ ((lane >> 4) & 3));
        voff[4 + q] = (4 * q + (lane >> 4)) * n + 16 * ((lane & 15) ^ b_swizzle(4 * (q & 1) + (lane >> 4)));
    }
    const uint32_t lds_wave = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(
        static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) uint8_t *)lds)) + wave * 4096));
    const uint32_t k_tiles = k / RK;
    // copy Q (0..7) of tile `tile` (clamped to tile 0 behind the end: copied, never multiplied) into stage ST
    auto tile_a = [&](uint32_t tile) { return scalar_pointer(a_wave + (tile < k_tiles ? tile * RK : 0)); };
    auto tile_b = [&](uint32_t tile) { return scalar_pointer(b_wave + static_cast<uint64_t>(tile < k_tiles ? tile * RK : 0) * n); };
    auto copy = [&]<int Q, int ST>(const uint8_t *from) __attribute__((always_inline)) {
        constexpr uint32_t to = ST * R_STAGE + (Q < 4 ? Q * 1024 : R_B + (Q - 4) * 1024);
        const uint32_t lane_off = voff[Q], lds_to = lds_wave;
        asm volatile("s_add_u32 m0, %2, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                     :
                     : "v"(lane_off), "s"(from), "s"(lds_to), "n"(to)
                     : "memory", "m0", "scc");
    };
    const uint32_t a_off = (wm * 128 + (lane & 31)) * 64 + 16 * (h ^ ((lane >> 2) & 3));
    auto read_a = [&](int stage, int ks, int i) -> v4i {
        return *reinterpret_cast<const v4i *>(lds + stage * R_STAGE + (a_off ^ (32 * ks)) + i * 2048);
    };
    uint32_t b_off[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t a16 = lane & 15, chunk = wn * 8 + 2 * j + ((lane >> 4) & 1);
        b_off[j] = R_B + (16 * h + (a16 >> 1)) * 256 + 16 * (chunk ^ b_swizzle(a16 >> 1)) + 8 * (a16 & 1);
    }
    typedef int v2i __attribute__((ext_vector_type(2)));
    auto read_b = [&](int stage, int ks, int j, int half, v4i &f) {
        const v2i r = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
            (__attribute__((address_space(3))) v2i *)(lds + stage * R_STAGE + b_off[j] + (32 * ks + 8 * half) * 256));
        f[2 * half] = r[0];
        f[2 * half + 1] = r[1];
    };

    v4i fa[2][4], fb[2][4];
    // tiles 0, 1, 2 and the A part of tile 3 (its B part follows in the first half of tile 0)
    {
        const uint8_t *a0 = tile_a(0), *b0 = tile_b(0), *a1 = tile_a(1), *b1 = tile_b(1), *a2 = tile_a(2), *b2 = tile_b(2),
                      *a3 = tile_a(3);
        [&]<int... Q>(std::integer_sequence<int, Q...>) __attribute__((always_inline)) {
            (copy.template operator()<Q, 0>(Q < 4 ? a0 : b0), ...);
            (copy.template operator()<Q, 1>(Q < 4 ? a1 : b1), ...);
            (copy.template operator()<Q, 2>(Q < 4 ? a2 : b2), ...);
        }(std::make_integer_sequence<int, 8>{});
        [&]<int... Q>(std::integer_sequence<int, Q...>) __attribute__((always_inline)) {
            (copy.template operator()<Q, 3>(a3), ...);
        }(std::make_integer_sequence<int, 4>{});
    }
    asm volatile("s_waitcnt vmcnt(20)" ::: "memory");  // tile 0 (the 8 oldest of 28 copies)
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) fa[0][i] = read_a(0, 0, i);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        read_b(0, 0, j, 0, fb[0][j]);
        read_b(0, 0, j, 1, fb[0][j]);
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) fa[0][i][e] ^= static_cast<int>(a_xor);

    // tile `t` is in stage ST
    auto step = [&]<int ST>(uint32_t t) __attribute__((always_inline)) {
        const uint8_t *b_cp = tile_b(t + 3), *a_cp = tile_a(t + 4);
        auto slot = [&]<int s>() __attribute__((always_inline)) {
            // rows walk the columns back and forth, so that only one operand changes between MFMAs
            constexpr int ks = s / 16, o = s % 16, row = o / 4, col = (row & 1) ? 3 - o % 4 : o % 4;
            constexpr int cur = ks & 1, nxt = cur ^ 1;
            if constexpr (s == 16) {
                // tile t + 1 has landed (all but the 16 newest copies) and this wavefront's reads of stage ST are done
                asm volatile("s_waitcnt vmcnt(16) lgkmcnt(0)" ::: "memory");
                __syncthreads();  // tile t + 1 complete for everybody, stage ST no longer read
            }
            acc[row][col] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[cur][row], fb[cur][col], acc[row][col], 0, 0, 0);
            constexpr int src = ks == 1 ? (ST + 1) % 4 : ST;
            constexpr int nks = ks ^ 1;
            if constexpr (o < 2) {
                fa[nxt][2 * o] = read_a(src, nks, 2 * o);
                fa[nxt][2 * o + 1] = read_a(src, nks, 2 * o + 1);
            } else if constexpr (o < 6) {
                read_b(src, nks, o - 2, 0, fb[nxt][o - 2]);
                read_b(src, nks, o - 2, 1, fb[nxt][o - 2]);
            }
            // the XOR of A's zero point, one word per slot: fragments 2 and 3 of this k-step (first used in slots 8
            // and 12), then fragments 0 and 1 of the next
            if constexpr (o < 8) fa[cur][2 + o / 4][o % 4] ^= static_cast<int>(a_xor);
            else fa[nxt][(o - 8) / 4][o % 4] ^= static_cast<int>(a_xor);
            if constexpr (s % 4 == 0) {
                if constexpr (s < 16) copy.template operator()<4 + s / 4, (ST + 3) % 4>(b_cp);   // B part of tile t + 3
                else copy.template operator()<(s - 16) / 4, ST>(a_cp);                           // A part of tile t + 4
            }
            __builtin_amdgcn_sched_barrier(0);
        };
        [&]<int... I>(std::integer_sequence<int, I...>) __attribute__((always_inline)) {
            (slot.template operator()<I>(), ...);
        }(std::make_integer_sequence<int, 32>{});
    };
    uint32_t t = 0;
    for (; t + 4 <= k_tiles; t += 4) {
        step.template operator()<0>(t);
        step.template operator()<1>(t + 1);
        step.template operator()<2>(t + 2);
        step.template operator()<3>(t + 3);
    }
    if (t < k_tiles) {  // k is a multiple of 128: two tiles are left
        step.template operator()<0>(t);
        step.template operator()<1>(t + 1);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no copy may land after the workgroup's LDS is released
}

// SPLIT: blockIdx.y picks a range of `split_tiles` k-tiles and the sums are added to a zeroed Y with integer atomics
// (exact in any order): for products with too few output tiles to occupy the chip.
// SHORT_M: fewer than 256 rows of A, one row of tiles.
template <bool DEQ, bool SPLIT, bool SHORT_M = false>
__global__ __launch_bounds__(256, 1) void mmi_mfma_256x256(int32_t *__restrict__ y, const uint8_t *__restrict__ a,
                                                           const uint8_t *__restrict__ b, ZeroPoint za, ZeroPoint zb,
                                                           Dequant dq, uint32_t m, uint32_t k, uint32_t n, uint32_t split_tiles,
                                                           uint32_t a_matrix0, uint32_t b_matrix0, uint32_t y_matrix0) {
    static_assert(!(DEQ && SPLIT), "partial sums cannot be dequantised");
    __shared__ __align__(1024) uint8_t lds_all[2 * D_STAGE];
    uint8_t *const lds0 = lds_all, *const lds1 = lds_all + D_STAGE;
    __shared__ __align__(256) uint8_t zlds[2 * 4 * 256];  // B's zero points of a tile: a slot per buffer and wavefront

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
    const uint32_t row0 = SHORT_M ? 0 : tile_m * BM + BM <= m ? tile_m * BM : m - BM;
    const uint32_t col0 = tile_n * BN + BN <= n ? tile_n * BN : n - BN;
    uint32_t k_begin = 0, k_len = k;
    if constexpr (SPLIT) {
        k_begin = blockIdx.y * split_tiles * BK;
        k_len = k - k_begin < split_tiles * BK ? k - k_begin : split_tiles * BK;
    }
    const uint8_t *A = a + (am * m + row0) * k + k_begin;
    const uint8_t *B = b + (bm * k + k_begin) * static_cast<uint64_t>(n) + col0;

    v16i acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

    const uint32_t wm = wave >> 1, wn = wave & 1;
    // zero points of the rows of this lane's A fragments; scalar 0 / 128 (or none) reduce to one XOR mask
    uint32_t za_f[4] = {};
    uint32_t a_xor = 0;
    bool a_simple = true;
    if (za.ptr) {
        if (za.per_row) {
            a_simple = false;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                uint32_t row = row0 + wm * 128 + 32 * i + (lane & 31);
                if (SHORT_M && row >= m) row = m - 1;
                za_f[i] = splat(za.ptr[am * m + row]);
            }
        } else {
            const uint32_t z = za.ptr[0];
            if (z == 0 || z == 128) {
                a_xor = splat(z);
            } else {
                a_simple = false;
#pragma unroll
                for (int i = 0; i < 4; ++i) za_f[i] = splat(z);
            }
        }
    }
    bool b_zp = zb.ptr != nullptr;
    if (b_zp && !zb.per_row && zb.ptr[0] == 0) b_zp = false;
    const uint64_t zb_row0 = bm * k + k_begin;

    if (a_simple && !b_zp && !SHORT_M && k < (1u << 26)) {  // (63 rows of A stay below 2^32 bytes: lane offsets of the copies)
        mmi_tile_loop_ring(acc, lds_all, A, B, k_len, k, n, a_xor);
    } else if (a_simple) {
        if (!b_zp) mmi_tile_loop<0, false, SHORT_M>(acc, lds0, lds1, A, B, k_len, k, n, a_xor, za_f, zb, zb_row0, m, zlds);
        else mmi_tile_loop<0, true, SHORT_M>(acc, lds0, lds1, A, B, k_len, k, n, a_xor, za_f, zb, zb_row0, m, zlds);
    } else {
        if (!b_zp) mmi_tile_loop<1, false, SHORT_M>(acc, lds0, lds1, A, B, k_len, k, n, a_xor, za_f, zb, zb_row0, m, zlds);
        else mmi_tile_loop<1, true, SHORT_M>(acc, lds0, lds1, A, B, k_len, k, n, a_xor, za_f, zb, zb_row0, m, zlds);
    }

    int32_t *Y = y + (ym * m + row0 + wm * 128) * n + col0 + wn * 128;
    float scale[4] = {};  // of this lane's four columns
    if constexpr (DEQ) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
            scale[j] = dq.scale[dq.per_column ? col0 + wn * 128 + j * 32 + (lane & 31) : 0];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const uint32_t row = i * 32 + 8 * (e / 4) + 4 * (lane >> 5) + (e % 4);
                const uint32_t col = j * 32 + (lane & 31);
                if (SHORT_M && wm * 128 + row >= m) continue;
                if constexpr (SPLIT)
                    __hip_atomic_fetch_add(Y + static_cast<uint64_t>(row) * n + col, acc[i][j][e], __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
                else
                    __builtin_nontemporal_store(finish<DEQ>(acc[i][j][e], scale[j]), Y + static_cast<uint64_t>(row) * n + col);
            }
}

}  // namespace
}  // namespace rg

extern "C" size_t rg_hip_matmul_integer_workspace(size_t, size_t, size_t, size_t, unsigned) {
    return 0;
}

namespace rg {
namespace {

// ---------------------------------------------------------------- few rows of A (decode): weight streaming
//
// Y[m <= 128, n] for up to four slabs of 32 rows: bound by reading B ([k, n], the weights) once.  A workgroup
// takes 256 columns and a few k-tiles of 128 (32 KiB of B each, coalesced 256-byte row pieces
// through registers into LDS, rows padded by 16 bytes, the next tile's loads in flight while one is
// multiplied), forms the MFMA operand with the transposing 64-bit LDS read as the big kernel
// does, takes its A fragments (16 consecutive k of a row per lane) straight from global memory,
// and adds its partial sums (32 x 256 per slab) to Y with integer atomics: the k-range of a column block is
// spread over workgroups, and integer addition gives the same result in any order.  Y is zeroed
// by a launch of its own before.  Zero points as in the big kernel.
constexpr int SK_PITCH = 256 + 16;
// Splitting k between workgroups when there are few output tiles: up to kSplitMax ranges, as many as bring the
// launch to about kSplitFill workgroups.  Every range adds one atomic per output, which costs about as much as
// the idle CUs gain from 64 tiles on ([256,4096] x [4096,4096]: 49.6 us unsplit, 35 / 29 / 27 / 32 us with 2 / 3 /
// 4 / 8 ranges; 512 rows: 49.6 unsplit, 37.5 / 35.7 / 37.3 / 53; 86 tiles in two ranges 58.6 against 49.3).
constexpr uint64_t kSplitFill = 128;
constexpr uint32_t kSplitMax = 4;
constexpr uint64_t kSkinnyWorkgroups = 256;  // per launch: one per CU (512 and 128 were measured: slower)

// ---------------------------------------------------------------- any shape on the matrix cores
//
// What the kernels around it do not take (fewer than 256 columns, column counts that are no multiple of 16, k that
// is no multiple of 128) as long as k is a multiple of 16: 128 x 128 outputs per workgroup of four wavefronts
// (64 x 64 each, 2 x 2 blocks of v_mfma_i32_32x32x32_i8), k in tiles of 128 through two LDS buffers filled from
// registers that are loaded two tiles ahead.  Both tiles are kept as [row or column][k] with a pitch of 144 bytes,
// so every fragment is one 128-bit read; B ([k, n] in memory) is turned on its way into LDS: four k-rows of sixteen
// columns become sixteen 32-bit writes.  The zero points are subtracted (bytes, modulo 256) as the tiles pass
// through registers.  Loads are unconditional, from addresses clamped into the matrices, so that the wait for a
// tile does not wait for the later ones as well; what lies beyond k is replaced by zeros (after the subtraction),
// rows and columns beyond the matrices are not stored.  Where rows of B are not 16-byte aligned, sixteen bytes
// come from five aligned words.
constexpr int GT = 128, GK = 128, GP = 144;

template <bool DEQ, bool B_VEC>  // B_VEC: rows of B start on 16-byte boundaries, n >= 16
__global__ __launch_bounds__(256, 2) void mmi_tiles(int32_t *__restrict__ y, const uint8_t *__restrict__ a, const uint8_t *__restrict__ b,
                                                 ZeroPoint za, ZeroPoint zb, Dequant dq, uint32_t m, uint32_t k, uint32_t n,
                                                 uint32_t a_matrix0, uint32_t b_matrix0, uint32_t y_matrix0) {
    __shared__ __align__(16) uint8_t As[2][GT * GP];
    __shared__ __align__(16) uint8_t Bs[2][GT * GP];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
    const uint32_t bz = blockIdx.z;
    const uint64_t am = a_matrix0 + bz, bm = b_matrix0 + bz, ym = y_matrix0 + bz;
    // Tile order: consecutive workgroup ids go round-robin to the 8 XCDs, so each XCD gets a contiguous run of tiles,
    // walked down the rows of one column panel after the other: the workgroups of an XCD share a panel of B in its L2.
    const uint32_t row_tiles = (m + GT - 1) / GT, n_tiles = row_tiles * ((n + GT - 1) / GT);
    uint32_t tile_id = blockIdx.x;
    if (n_tiles % 8 == 0) tile_id = (tile_id % 8) * (n_tiles / 8) + tile_id / 8;
    const uint32_t row0 = (tile_id % row_tiles) * GT, col0 = (tile_id / row_tiles) * GT;
    const uint8_t *A = a + am * m * static_cast<uint64_t>(k);
    const uint8_t *B = b + bm * static_cast<uint64_t>(k) * n;

    // A tile: rows tid / 8 + 32 i, k 16 (tid % 8) .. + 15 (a row of a tile is one 128-byte line).
    // B tile: k-rows 4 (tid / 8) + i, columns 16 (tid % 8) .. + 15
    const uint32_t pr = tid >> 3, pk = 16 * (tid & 7);
    const uint8_t *a_src[4];
    uint32_t a_zero[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t r = row0 + pr + 32 * i, row = r < m ? r : m - 1;
        a_src[i] = A + static_cast<uint64_t>(row) * k;
        a_zero[i] = splat(zp_byte(za, am * m + row));
    }
    const uint32_t bq = tid >> 3, bc = col0 + 16 * (tid & 7);
    const uint32_t bc_load = bc + 16 <= n ? bc : (n >= 16 ? n - 16 : 0);  // (vector loads only)
    const uint8_t *b_last = reinterpret_cast<const uint8_t *>((reinterpret_cast<uint64_t>(B) + static_cast<uint64_t>(k) * n - 1) & ~3ull);
    // B's zero points are loaded with the tiles, without a branch (a load under a branch makes the wait for one tile
    // a wait for all): without zero points the loads read some byte of B and are masked away
    const uint8_t *zb_base = zb.ptr ? zb.ptr + (zb.per_row ? bm * k : 0) : B;
    const uint32_t zb_step = zb.ptr && zb.per_row ? 1u : 0u, zb_keep = zb.ptr ? 0xffffffffu : 0u;
    const u32x4 zero4 = {0u, 0u, 0u, 0u};
    u32x4 ra[2][4], rb[2][4];  // two tiles in flight (a third set of registers spills)
    uint32_t b_zero[2][4];
    auto fetch = [&](auto set, uint32_t k0) {
        constexpr int P = decltype(set)::value;
        const uint32_t kq = k0 + pk < k ? k0 + pk : k - 16;  // k is a multiple of 16
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            ra[P][i] = *reinterpret_cast<const u32x4 *>(a_src[i] + kq);
            const uint32_t kr0 = k0 + 4 * bq + i, kr = kr0 < k ? kr0 : k - 1;
            const uint8_t *src = B + static_cast<uint64_t>(kr) * n;
            b_zero[P][i] = splat(zb_base[static_cast<uint64_t>(kr) * zb_step]) & zb_keep;
            if constexpr (B_VEC) {
                rb[P][i] = *reinterpret_cast<const u32x4 *>(src + bc_load);
            } else {
                rb[P][i] = load16_any(src + bc, b_last);  // (columns beyond n: arbitrary bytes, not stored)
            }
        }
    };
    // (the tile that reaches beyond k takes a branch of its own: selects in the common path get scheduled ahead of
    // the barrier before them, where they wait for loads a step early)
    auto stash_part = [&](auto set, auto whole, int buf, uint32_t k0) {
        constexpr int P = decltype(set)::value;
        constexpr bool WHOLE = decltype(whole)::value;
        const bool k_in = WHOLE || k0 + pk < k;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            u32x4 v;
#pragma unroll
            for (int j = 0; j < 4; ++j) v[j] = sub_bytes(ra[P][i][j], a_zero[i]);
            *reinterpret_cast<u32x4 *>(&As[buf][(pr + 32 * i) * GP + pk]) = k_in ? v : zero4;
        }
        // four k-rows of sixteen columns -> per column one word of four consecutive k.  The eight 16-byte pieces
        // of a column's k are kept in an order that depends on the column (piece ^ (column / 16) % 8), which
        // spreads the eight column groups of a wavefront over the LDS banks
        const bool rows_in = WHOLE || k0 + 4 * bq < k;  // (k is a multiple of 4: all four rows are in or out)
        const uint32_t word = bq ^ ((tid & 7) << 2);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            uint32_t r[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) r[i] = sub_bytes(rb[P][i][j], b_zero[P][i]);
            const uint32_t lo01 = __builtin_amdgcn_perm(r[1], r[0], 0x05010400u), hi01 = __builtin_amdgcn_perm(r[1], r[0], 0x07030602u);
            const uint32_t lo23 = __builtin_amdgcn_perm(r[3], r[2], 0x05010400u), hi23 = __builtin_amdgcn_perm(r[3], r[2], 0x07030602u);
            const uint32_t c[4] = {__builtin_amdgcn_perm(lo23, lo01, 0x05040100u), __builtin_amdgcn_perm(lo23, lo01, 0x07060302u),
                                   __builtin_amdgcn_perm(hi23, hi01, 0x05040100u), __builtin_amdgcn_perm(hi23, hi01, 0x07060302u)};
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint32_t col = 16 * (tid & 7) + 4 * j + q;
                *reinterpret_cast<uint32_t *>(&Bs[buf][col * GP + 4 * word]) = rows_in ? c[q] : 0u;
            }
        }
    };
    auto stash = [&](auto set, int buf, uint32_t k0) {
        if (k0 + GK <= k) stash_part(set, std::true_type{}, buf, k0);
        else stash_part(set, std::false_type{}, buf, k0);
    };

    v16i acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

    const uint32_t l32 = lane & 31, kh = lane >> 5;
    const uint32_t tiles = (k + GK - 1) / GK;
    // Step t: (barrier) request tile t + 2 into the registers tile t has left, write tile t + 1 into the buffer
    // tile t - 1 was read from, multiply tile t.  The barrier says both that tile t is complete in its buffer and
    // that everybody has finished reading tile t - 1.
    auto step = [&](auto set_free, auto set_next, uint32_t t) {
        const int buf = t & 1;
        __syncthreads();
        fetch(set_free, (t + 2) * GK);
        stash(set_next, buf ^ 1, (t + 1) * GK);
#pragma unroll
        for (int ks = 0; ks < GK / 32; ++ks) {
            v4i fa[2], fb[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) fa[i] = *reinterpret_cast<const v4i *>(&As[buf][(wm * 64 + 32 * i + l32) * GP + 32 * ks + 16 * kh]);
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const uint32_t piece = (2 * ks + kh) ^ ((4 * wn + 2 * j + (l32 >> 4)) & 7);
                fb[j] = *reinterpret_cast<const v4i *>(&Bs[buf][(wn * 64 + 32 * j + l32) * GP + 16 * piece]);
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
    };
    const std::integral_constant<int, 0> s0;
    const std::integral_constant<int, 1> s1;
    fetch(s0, 0);
    fetch(s1, GK);
    stash(s0, 0, 0);
    uint32_t t = 0;
    for (; t + 2 <= tiles; t += 2) {  // no branch inside: the waits count the loads of the later tile exactly
        step(s0, s1, t);
        step(s1, s0, t + 1);
    }
    if (t < tiles) step(s0, s1, t);
    // accumulator: column lane % 32 of the block, register e holds row 8 (e / 4) + 4 (lane / 32) + e % 4
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const uint32_t col = col0 + wn * 64 + 32 * j + l32;
        const float scale = DEQ && col < n ? dq.scale[dq.per_column ? col : 0] : 0.f;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const uint32_t row = row0 + wm * 64 + 32 * i + 8 * (e / 4) + 4 * kh + (e % 4);
                if (row < m && col < n) y[(ym * m + row) * n + col] = finish<DEQ>(acc[i][j][e], scale);
            }
    }
}

__global__ __launch_bounds__(256) void mmi_zero(int32_t *__restrict__ y, uint64_t count) {
    for (uint64_t i = static_cast<uint64_t>(blockIdx.x) * 256 + threadIdx.x; i < count; i += static_cast<uint64_t>(gridDim.x) * 256)
        y[i] = 0;
}

// The dequantising form of the few-rows path: the int32 sums, complete in Y, become float(sum) * scale in place.
__global__ __launch_bounds__(256) void mmi_dequantize_in_place(int32_t *__restrict__ y, Dequant dq, uint64_t rows, uint32_t n) {
    const uint64_t count = rows * n;
    for (uint64_t i = static_cast<uint64_t>(blockIdx.x) * 256 + threadIdx.x; i < count; i += static_cast<uint64_t>(gridDim.x) * 256)
        y[i] = finish<true>(y[i], dq.scale[dq.per_column ? static_cast<uint32_t>(i % n) : 0]);
}

template <int SLABS>  // slabs of 32 rows of A that share one pass over B
__global__ __launch_bounds__(256) void mmi_skinny(int32_t *__restrict__ y, const uint8_t *__restrict__ a,
                                                  const uint8_t *__restrict__ b, ZeroPoint za, ZeroPoint zb, uint32_t rows,
                                                  uint32_t m, uint32_t row_first, uint32_t k, uint32_t n, uint32_t tiles,
                                                  uint32_t a_matrix0, uint32_t b_matrix0, uint32_t y_matrix0) {
    __shared__ __align__(16) uint8_t tile[BK * SK_PITCH];
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, h = lane >> 5;
    const uint32_t bz = blockIdx.z;
    const uint64_t am = a_matrix0 + bz, bm = b_matrix0 + bz, ym = y_matrix0 + bz;
    const uint32_t col0 = blockIdx.x * 256;
    const uint32_t t_first = blockIdx.y * tiles, k_tiles = k / BK;
    const uint32_t t_end = t_first + tiles < k_tiles ? t_first + tiles : k_tiles;
    const uint8_t *B = b + bm * k * static_cast<uint64_t>(n) + col0;

    // B tile: 128 k-rows of 256 bytes, 16 lanes per row, 16 rows per pass of the workgroup
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    u32x4 w[8];
    auto load_b = [&](uint32_t t) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint64_t r = static_cast<uint64_t>(t) * BK + 16 * i + (tid >> 4);
            w[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(B + r * n + 16 * (tid & 15)));
        }
    };
    // A fragments of the four k-steps of a tile: row lane % 32 of the slab (rows beyond it repeat the last one),
    // k 32 ks + 16 h .. + 15
    uint64_t a_row[SLABS];
    uint32_t za_splat[SLABS];
#pragma unroll
    for (int sl = 0; sl < SLABS; ++sl) {
        const uint32_t row = 32 * sl + (lane & 31) < rows ? 32 * sl + (lane & 31) : rows - 1;
        a_row[sl] = am * m + row_first + row;
        za_splat[sl] = za.ptr ? splat(za.per_row ? za.ptr[a_row[sl]] : za.ptr[0]) : 0;
    }
    const bool b_zp = zb.ptr != nullptr;
    typedef int v2i __attribute__((ext_vector_type(2)));
    const uint32_t a16 = lane & 15;
    v16i acc[SLABS][2];
#pragma unroll
    for (int sl = 0; sl < SLABS; ++sl)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[sl][j][e] = 0;

    // B's zero points of a tile's k-steps are loaded with its A fragments, without a branch (a load under a branch
    // turns the compiler's wait for it into a wait for everything in flight): without zero points the loads read
    // bytes of B and are masked away; a scalar one is read once
    const uint8_t *zb_base = b_zp && zb.per_row ? zb.ptr + bm * k : B;
    const uint32_t zb_keep = b_zp && zb.per_row ? 0xffffffffu : 0u;
    const uint32_t zb_scalar = b_zp && !zb.per_row ? splat(zb.ptr[0]) : 0u;
    load_b(t_first);
    // (the next tile's load has no branch around it either: the last tile takes a body of its own)
    auto tile_step = [&](uint32_t t, auto more) {
        const uint32_t k0 = t * BK;
        v4i fa[SLABS][4];
        u32x4 zk[4];
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) __builtin_memcpy(&zk[ks], zb_base + k0 + 32 * ks + 16 * h, 16);  // (any alignment)
#pragma unroll
        for (int sl = 0; sl < SLABS; ++sl)
#pragma unroll
            for (int ks = 0; ks < 4; ++ks)
                fa[sl][ks] = *reinterpret_cast<const v4i *>(a + a_row[sl] * k + k0 + 32 * ks + 16 * h);
#pragma unroll
        for (int i = 0; i < 8; ++i)
            *reinterpret_cast<u32x4 *>(tile + (16 * i + (tid >> 4)) * SK_PITCH + 16 * (tid & 15)) = w[i];
        __syncthreads();
        if constexpr (decltype(more)::value) load_b(t + 1);  // in flight while this tile is multiplied
        if (za.ptr) {
#pragma unroll
            for (int sl = 0; sl < SLABS; ++sl)
#pragma unroll
                for (int ks = 0; ks < 4; ++ks)
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        fa[sl][ks][e] = static_cast<int>(sub_bytes(static_cast<uint32_t>(fa[sl][ks][e]), za_splat[sl]));
        }
        // B fragment of column block j (32 columns) and k-step ks: column lane % 32, k 32 ks + 16 h .. + 15 in two
        // transposing reads of 8 k each; lane a of a group of 16 addresses k-row a / 2, columns 8 (a % 2) .. + 7
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            uint32_t z[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) z[e] = (zk[ks][e] & zb_keep) | zb_scalar;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const uint32_t cols = 64 * wave + 32 * j + 16 * ((lane >> 4) & 1);
                const uint8_t *src = tile + (32 * ks + 16 * h + (a16 >> 1)) * SK_PITCH + cols + 8 * (a16 & 1);
                const v2i lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) v2i *)(src));
                const v2i hi = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) v2i *)(src + 8 * SK_PITCH));
                v4i fb = {lo[0], lo[1], hi[0], hi[1]};
                if (b_zp) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) fb[e] = static_cast<int>(sub_bytes(static_cast<uint32_t>(fb[e]), z[e]));
                }
#pragma unroll
                for (int sl = 0; sl < SLABS; ++sl)
                    acc[sl][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[sl][ks], fb, acc[sl][j], 0, 0, 0);
            }
        }
        __syncthreads();  // the tile is rewritten
    };
    for (uint32_t t = t_first; t + 1 < t_end; ++t) tile_step(t, std::true_type{});
    tile_step(t_end - 1, std::false_type{});
    // accumulator: column lane % 32 of the block, register e holds row 8 (e / 4) + 4 h + e % 4
    int32_t *Y = y + (ym * m + row_first) * n + col0 + 64 * wave;
#pragma unroll
    for (int sl = 0; sl < SLABS; ++sl)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const uint32_t r = 32 * sl + 8 * (e / 4) + 4 * h + (e % 4);
                if (r < rows)
                    __hip_atomic_fetch_add(Y + static_cast<uint64_t>(r) * n + 32 * j + (lane & 31), acc[sl][j][e],
                                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
}

// ---------------------------------------------------------------- one to four rows of A: matrix-vector products
//
// Y[m <= 4, n]: the matrix cores would spend 32 rows of work on these few, so the products are
// formed by v_dot4_i32_i8 on the vector ALUs and the kernel is a plain stream over B ([k, n]).
// A workgroup takes a strip of 256 columns and a range of k; a lane owns 16 columns (one 128-bit
// load per k-row) and, per step, four consecutive k-rows (lane / 16 picks which four of the step's
// 16), GEMV_DEPTH steps of loads in flight.  The four rows are transposed inside the lane with byte
// permutes, so that a register holds the four k of one column, which is the order of four
// consecutive bytes of a row of A.  Zero points are subtracted from the bytes before (modulo 256,
// as everywhere).  The 16 partial sums per column (4 wavefronts x 4 row groups) meet in LDS; the
// k-ranges of different workgroups meet in Y by integer atomics, as in the few-rows kernel above,
// unless one workgroup covers all of k: then Y is stored and needs no zeroing.
constexpr uint64_t kGemvWorkgroups = 512;  // aimed at per launch
constexpr int GEMV_DEPTH = 2;               // steps of loads in flight per wavefront

template <int M>
__global__ __launch_bounds__(256) void mmi_gemv(int32_t *__restrict__ y, const uint8_t *__restrict__ a,
                                                const uint8_t *__restrict__ b, ZeroPoint za, ZeroPoint zb, uint32_t m,
                                                uint32_t k, uint32_t n, uint32_t steps_per_wave, uint32_t a_matrix0,
                                                uint32_t b_matrix0, uint32_t y_matrix0) {
    __shared__ __align__(16) int32_t part[16 * M * 256];  // [wavefront * 4 + row group][row of A][column of the strip]
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const uint32_t tid = threadIdx.x, lane = tid & 63, g = lane >> 4, c = lane & 15;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t bz = blockIdx.z;
    const uint64_t am = a_matrix0 + bz, bm = b_matrix0 + bz, ym = y_matrix0 + bz;
    const uint32_t col0 = blockIdx.x * 256 + 16 * c;  // this lane's 16 columns
    const bool live = col0 < n;
    const uint32_t total_steps = k / 16, step0 = blockIdx.y * 4 * steps_per_wave;
    const uint8_t *B = b + bm * k * static_cast<uint64_t>(n) + col0;
    const uint8_t *A[M];
    uint32_t za_splat[M];
#pragma unroll
    for (int i = 0; i < M; ++i) {
        const uint64_t row = am * m + (static_cast<uint32_t>(i) < m ? i : m - 1);  // rows beyond m repeat the last one
        A[i] = a + row * k;
        za_splat[i] = za.ptr ? splat(za.per_row ? za.ptr[row] : za.ptr[0]) : 0;
    }

    int32_t acc[M][16];
#pragma unroll
    for (int i = 0; i < M; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][e] = 0;

    // step s of this wavefront: k-rows 16 (step0 + 4 s + wave) .. + 15, this lane 4 g .. 4 g + 3 of them
    // the four bytes of every row of A and of the zero points of B that go with the k-rows travel with them:
    // loads return in the order issued, so one issued only when it is needed would wait for everything ahead of it
    u32x4 buf[GEMV_DEPTH][4];
    uint32_t a_quad[GEMV_DEPTH][M], z_quad[GEMV_DEPTH];
    const uint8_t *Z = zb.ptr && zb.per_row ? zb.ptr + bm * k : nullptr;
    auto load = [&](int slot, uint32_t step) {
        const uint64_t kk = 16ull * step + 4 * g;
        if (live) {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                buf[slot][r] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(B + (kk + r) * n));
#pragma unroll
            for (int i = 0; i < M; ++i) a_quad[slot][i] = *reinterpret_cast<const uint32_t *>(A[i] + kk);
            if (Z) z_quad[slot] = *reinterpret_cast<const uint32_t *>(Z + kk);
        }
    };
    const uint32_t z_all = zb.ptr && !zb.per_row ? splat(zb.ptr[0]) : 0;
#pragma unroll
    for (int d = 0; d < GEMV_DEPTH; ++d)
        if (static_cast<uint32_t>(d) < steps_per_wave && step0 + 4 * d + wave < total_steps) load(d, step0 + 4 * d + wave);

    for (uint32_t s = 0; s < steps_per_wave; s += GEMV_DEPTH) {
#pragma unroll
        for (int d = 0; d < GEMV_DEPTH; ++d) {
            const uint32_t step = step0 + 4 * (s + d) + wave;
            if (s + d < steps_per_wave && step < total_steps) {
                if (live) {
                    uint32_t aq[M];  // bytes: A[i][kk .. kk + 3] minus the zero point
#pragma unroll
                    for (int i = 0; i < M; ++i) aq[i] = za.ptr ? sub_bytes(a_quad[d][i], za_splat[i]) : a_quad[d][i];
                    u32x4 rows[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        rows[r] = buf[d][r];
                        if (Z || z_all) {  // a zero point of zero changes nothing
                            const uint32_t z = Z ? splat((z_quad[d] >> (8 * r)) & 0xffu) : z_all;
#pragma unroll
                            for (int e = 0; e < 4; ++e) rows[r][e] = sub_bytes(rows[r][e], z);
                        }
                    }
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        // 4 x 4 bytes (k-row r, column 4 e + j) -> register j holds the four k of column 4 e + j;
                        // v_perm_b32 picks result bytes from {second operand: indices 0-3, first operand: 4-7}
                        const uint32_t t_lo = __builtin_amdgcn_perm(rows[1][e], rows[0][e], 0x05010400u);
                        const uint32_t t_hi = __builtin_amdgcn_perm(rows[1][e], rows[0][e], 0x07030602u);
                        const uint32_t u_lo = __builtin_amdgcn_perm(rows[3][e], rows[2][e], 0x05010400u);
                        const uint32_t u_hi = __builtin_amdgcn_perm(rows[3][e], rows[2][e], 0x07030602u);
                        const uint32_t col[4] = {__builtin_amdgcn_perm(u_lo, t_lo, 0x05040100u),
                                                 __builtin_amdgcn_perm(u_lo, t_lo, 0x07060302u),
                                                 __builtin_amdgcn_perm(u_hi, t_hi, 0x05040100u),
                                                 __builtin_amdgcn_perm(u_hi, t_hi, 0x07060302u)};
#pragma unroll
                        for (int i = 0; i < M; ++i)
#pragma unroll
                            for (int j = 0; j < 4; ++j)
                                acc[i][4 * e + j] = __builtin_amdgcn_sdot4(static_cast<int>(aq[i]), static_cast<int>(col[j]),
                                                                           acc[i][4 * e + j], false);
                    }
                }
                const uint32_t next = step + 4 * GEMV_DEPTH;
                if (s + d + GEMV_DEPTH < steps_per_wave && next < total_steps) load(d, next);
            }
        }
    }

    if (live) {
#pragma unroll
        for (int i = 0; i < M; ++i)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const v4i v = {acc[i][4 * e], acc[i][4 * e + 1], acc[i][4 * e + 2], acc[i][4 * e + 3]};
                *reinterpret_cast<v4i *>(part + ((wave * 4 + g) * M + i) * 256 + 16 * c + 4 * e) = v;
            }
    }
    __syncthreads();
    const uint32_t col = blockIdx.x * 256 + tid;
    if (col < n) {
#pragma unroll
        for (int i = 0; i < M; ++i) {
            if (static_cast<uint32_t>(i) < m) {
                int32_t sum = 0;
#pragma unroll
                for (int p = 0; p < 16; ++p) sum += part[(p * M + i) * 256 + tid];
                int32_t *dst = y + (ym * m + i) * n + col;
                if (gridDim.y == 1) *dst = sum;
                else __hip_atomic_fetch_add(dst, sum, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
}

template <int M>
int launch_gemv(int32_t *y, const uint8_t *a, const uint8_t *b, ZeroPoint za, ZeroPoint zb, uint32_t m, uint32_t k, uint32_t n,
                uint32_t am0, uint32_t bm0, uint32_t ym0, uint32_t count, hipStream_t s) {
    const uint32_t strips = (n + 255) / 256, total_steps = k / 16;
    // steps per wavefront: as few as keep about kGemvWorkgroups workgroups (the more a workgroup sums itself,
    // the fewer atomics per output)
    uint64_t per_wave = static_cast<uint64_t>(total_steps) * strips * count / (4 * kGemvWorkgroups);
    per_wave = per_wave < 1 ? 1 : per_wave;
    const uint32_t splits = static_cast<uint32_t>((total_steps + 4 * per_wave - 1) / (4 * per_wave));
    if (splits > 1) {
        const uint64_t outputs = static_cast<uint64_t>(count) * m * n;
        const uint64_t zero_grid = (outputs + 1023) / 1024;
        mmi_zero<<<static_cast<unsigned>(zero_grid > 4096 ? 4096 : zero_grid), 256, 0, s>>>(y + static_cast<uint64_t>(ym0) * m * n,
                                                                                           outputs);
        const int rc = launch_status();
        if (rc) return rc;
    }
    mmi_gemv<M><<<dim3(strips, splits, count), 256, 0, s>>>(y, a, b, za, zb, m, k, n, static_cast<uint32_t>(per_wave), am0, bm0,
                                                          ym0);
    return launch_status();
}

template <bool DEQ>
int mmi_launch(int32_t *y, const void *a, const void *b, const void *a_zp, const void *b_zp, unsigned flags,
               size_t batch, size_t m, size_t k, size_t n, const uint32_t *a_index, const uint32_t *b_index,
               Dequant dq, void *stream) {
    if (!y || !a || !b) return RG_HIP_E_ARGUMENT;
    if (batch == 0 || m == 0 || n == 0) return 0;
    if (m > 0x7fffffffu || n > 0x7fffffffu || k > 0x7fffffffu || batch > 0xffffffffu)
        return RG_HIP_E_UNSUPPORTED;
    // One B for consecutive matrices of A (activations [batch, m, k] against weights): the batch is more rows of one
    // product, not `batch` launches that each read B again.  The zero points per (matrix, row) follow: A's are
    // consecutive like its rows, B's are those of the one matrix.
    // (up to 2^20 rows: every kernel's grid takes that many)
    if (batch > 1 && b_index && batch * m <= (1u << 20)) {
        bool fold = true;
        for (size_t i = 0; i < batch && fold; ++i)
            fold = b_index[i] == b_index[0] && (a_index ? a_index[i] == a_index[0] + i : true);
        if (fold) {
            const size_t a0 = a_index ? a_index[0] : 0, b0 = b_index[0];
            a = static_cast<const uint8_t *>(a) + a0 * m * k;
            b = static_cast<const uint8_t *>(b) + b0 * k * n;
            if (a_zp && !(flags & RG_MMI_A_ZP_SCALAR)) a_zp = static_cast<const uint8_t *>(a_zp) + a0 * m;
            if (b_zp && !(flags & RG_MMI_B_ZP_SCALAR)) b_zp = static_cast<const uint8_t *>(b_zp) + b0 * k;
            m *= batch;
            batch = 1;
            a_index = b_index = nullptr;
        }
    }
    hipStream_t s = as_stream(stream);
    const ZeroPoint za{static_cast<const uint8_t *>(a_zp), (flags & RG_MMI_A_ZP_SCALAR) ? 0u : 1u};
    const ZeroPoint zb{static_cast<const uint8_t *>(b_zp), (flags & RG_MMI_B_ZP_SCALAR) ? 0u : 1u};
    // B rows start on 16-byte boundaries when n is a multiple of 16
    const bool fast = m >= BM && n >= BN && n % 16 == 0 && k % BK == 0 && k > 0 && aligned16(a) && aligned16(b) &&
                      k < (1u << 27) && n < (1u << 28);  // lane offsets of the tile copies stay below 2^31

    // fewer rows than a tile: stream B once per slab of 32 rows
    const bool skinny = !fast && m < BM && n % 256 == 0 && k % BK == 0 && k > 0 && aligned16(a) &&
                        aligned16(b);

    // fewer than 256 rows on one row of 256 x 256 tiles (A's missing rows repeated, their results not stored): for
    // more than 64 rows (at 4096 x 4096: 128 rows 31 us through the weight-streaming kernel, 255 rows, two passes,
    // 60 us, against 22 to 25 us here) and for shapes that kernel does not fit
    const bool short_ok = m < BM && n >= BN && n % 16 == 0 && k % BK == 0 && k > 0 && aligned16(a) && aligned16(b) &&
                          k < (1u << 23) && n < (1u << 28);

    // one to four rows: matrix-vector products on the vector ALUs
    const bool gemv = m <= 4 && n % 16 == 0 && k % 16 == 0 && k > 0 && aligned16(b) && (reinterpret_cast<uintptr_t>(a) & 3u) == 0 &&
                      (!zb.ptr || !zb.per_row || (reinterpret_cast<uintptr_t>(zb.ptr) & 3u) == 0);

    const bool short_tile = short_ok && !gemv && (skinny ? m > 64 : true);

    // the 256 x 256 tiles, with k split between workgroups when the tiles are few
    auto launch_tiles = [&](auto short_m, uint32_t am0, uint32_t bm0, uint32_t ym0, uint32_t count) -> int {
        constexpr bool SHORT = decltype(short_m)::value;
        const uint64_t tiles = ((m + BM - 1) / BM) * ((n + BN - 1) / BN);
        const uint32_t k_tiles = static_cast<uint32_t>(k / BK);
        // too few tiles for the chip: split k as well, up to kSplitMax ways with at least two k-tiles each
        uint32_t splits = static_cast<uint32_t>(kSplitFill / (tiles * count));
        splits = splits > kSplitMax ? kSplitMax : splits;
        splits = splits > k_tiles / 2 ? k_tiles / 2 : splits;
        // tiles moved back overlap: their outputs would be added twice
        if ((!SHORT && m % BM != 0) || n % BN != 0) splits = 1;
        if (splits > 1) {
            const uint32_t split_tiles = (k_tiles + splits - 1) / splits;
            splits = (k_tiles + split_tiles - 1) / split_tiles;
            const uint64_t outputs = static_cast<uint64_t>(count) * m * n, zero_grid = (outputs + 1023) / 1024;
            int32_t *y0 = y + static_cast<uint64_t>(ym0) * m * n;
            mmi_zero<<<static_cast<unsigned>(zero_grid > 4096 ? 4096 : zero_grid), 256, 0, s>>>(y0, outputs);
            int rc = launch_status();
            if (rc) return rc;
            mmi_mfma_256x256<false, true, SHORT><<<dim3(static_cast<unsigned>(tiles), splits, count), 256, 0, s>>>(
                y, static_cast<const uint8_t *>(a), static_cast<const uint8_t *>(b), za, zb, dq,
                static_cast<uint32_t>(m), static_cast<uint32_t>(k), static_cast<uint32_t>(n), split_tiles, am0, bm0, ym0);
            rc = launch_status();
            if (rc) return rc;
            if constexpr (DEQ) {
                mmi_dequantize_in_place<<<static_cast<unsigned>(zero_grid > 4096 ? 4096 : zero_grid), 256, 0, s>>>(
                    y0, dq, static_cast<uint64_t>(count) * m, static_cast<uint32_t>(n));
                return launch_status();
            }
            return 0;
        }
        const dim3 grid(static_cast<unsigned>(tiles), 1, count);
        mmi_mfma_256x256<DEQ, false, SHORT><<<grid, 256, 0, s>>>(
            y, static_cast<const uint8_t *>(a), static_cast<const uint8_t *>(b), za, zb, dq,
            static_cast<uint32_t>(m), static_cast<uint32_t>(k), static_cast<uint32_t>(n), 0, am0, bm0, ym0);
        return launch_status();
    };

    // The 128 x 128 tiles instead of the 256 x 256 ones where the launch is expected to end earlier: a workgroup's
    // walk through k is a chain of dependent steps (1.6 us per 128 of k on the large tile, 1.12 us on the small one),
    // and sharing k between workgroups costs a zeroing pass and one atomic per output and range (measured: 9 us and
    // 4.3 us per million outputs), so few large tiles with a short k lose to four times as many small ones
    // (2048^3: 40 -> 24 us; 1024 x 4096 x 4096: 52 -> 39 us; 256 x 4096 x 4096 stays: 27 against 37 us).
    auto small_tiles_pay = [&](bool short_m, uint32_t count) {
        const double large = static_cast<double>(((m + BM - 1) / BM) * ((n + BN - 1) / BN)) * count;
        const double small = static_cast<double>(((m + GT - 1) / GT) * ((n + GT - 1) / GT)) * count;
        const uint32_t k_tiles = static_cast<uint32_t>(k / BK);
        uint32_t splits = static_cast<uint32_t>(kSplitFill / large);
        splits = splits > kSplitMax ? kSplitMax : splits;
        splits = splits > k_tiles / 2 ? k_tiles / 2 : splits;
        if ((!short_m && m % BM != 0) || n % BN != 0 || splits < 1) splits = 1;
        const double outputs = 1e-6 * static_cast<double>(m) * static_cast<double>(n) * count;
        const double steps = (k_tiles + splits - 1) / splits;
        const double large_us = splits > 1 ? 1.6 * steps + 9 + 4.3 * outputs + (DEQ ? 2 + 2.5 * outputs : 0)
                                           : 1.6 * steps * static_cast<double>((static_cast<uint64_t>(large) + 255) / 256) + 3;
        const double small_us = 6 + 1.12 * k_tiles * (small > 256 ? small / 256 : 1.0);
        return small_us < large_us;
    };
    auto launch_small_tiles = [&](uint32_t am0, uint32_t bm0, uint32_t ym0, uint32_t count) -> int {
        const dim3 grid(static_cast<unsigned>(((m + GT - 1) / GT) * ((n + GT - 1) / GT)), 1, count);
        const auto *a8 = static_cast<const uint8_t *>(a);
        const auto *b8 = static_cast<const uint8_t *>(b);
        const uint32_t m32 = static_cast<uint32_t>(m), k32 = static_cast<uint32_t>(k), n32 = static_cast<uint32_t>(n);
        if (n % 16 == 0 && aligned16(b)) mmi_tiles<DEQ, true><<<grid, 256, 0, s>>>(y, a8, b8, za, zb, dq, m32, k32, n32, am0, bm0, ym0);
        else mmi_tiles<DEQ, false><<<grid, 256, 0, s>>>(y, a8, b8, za, zb, dq, m32, k32, n32, am0, bm0, ym0);
        return launch_status();
    };
    // (up to 8 rows only where the plain kernel is expected to take longer: it needs 3.3 ns per thousand elements of B,
    // 675 us for [8, 4096] x [4096, 50257]; a launch of these tiles about 6 us and 1.12 us per 128 of k)
    const bool small_tiles_rows = m > 8 || static_cast<uint64_t>(n) * k > 1800000u + 2650u * static_cast<uint64_t>(k);
    const bool small_tiles_ok = k % 16 == 0 && k > 0 && small_tiles_rows && aligned16(a) && ((m + GT - 1) / GT) * ((n + GT - 1) / GT) <= 0x7fffffffu;

    auto launch = [&](uint32_t am0, uint32_t bm0, uint32_t ym0, uint32_t count) -> int {
        if (small_tiles_ok && (short_tile || (fast && !gemv && !skinny)) && small_tiles_pay(short_tile, count))
            return launch_small_tiles(am0, bm0, ym0, count);
        if (short_tile) return launch_tiles(std::true_type{}, am0, bm0, ym0, count);
        if (gemv) {
            const auto *a8 = static_cast<const uint8_t *>(a);
            const auto *b8 = static_cast<const uint8_t *>(b);
            const uint32_t m32 = static_cast<uint32_t>(m), k32 = static_cast<uint32_t>(k), n32 = static_cast<uint32_t>(n);
            int rc = m <= 1   ? launch_gemv<1>(y, a8, b8, za, zb, m32, k32, n32, am0, bm0, ym0, count, s)
                     : m <= 2 ? launch_gemv<2>(y, a8, b8, za, zb, m32, k32, n32, am0, bm0, ym0, count, s)
                              : launch_gemv<4>(y, a8, b8, za, zb, m32, k32, n32, am0, bm0, ym0, count, s);
            if (rc) return rc;
            if constexpr (DEQ) {
                const uint64_t outputs = static_cast<uint64_t>(count) * m * n, grid = (outputs + 1023) / 1024;
                mmi_dequantize_in_place<<<static_cast<unsigned>(grid > 4096 ? 4096 : grid), 256, 0, s>>>(
                    y + static_cast<uint64_t>(ym0) * m * n, dq, static_cast<uint64_t>(count) * m, static_cast<uint32_t>(n));
                return launch_status();
            }
            return 0;
        }
        if (skinny) {
            const uint64_t outputs = static_cast<uint64_t>(count) * m * n;
            uint64_t zero_grid = (outputs + 1023) / 1024;
            mmi_zero<<<static_cast<unsigned>(zero_grid > 4096 ? 4096 : zero_grid), 256, 0, s>>>(y + static_cast<uint64_t>(ym0) * m * n,
                                                                                               outputs);
            int rc = launch_status();
            if (rc) return rc;
            // up to four slabs of 32 rows share one pass over B
            for (size_t r0 = 0; r0 < m; r0 += 128) {
                const uint32_t rows = static_cast<uint32_t>(m - r0 < 128 ? m - r0 : 128);
                // k-tiles per workgroup: as few as keep about kSkinnyWorkgroups workgroups per launch (fewer atomics per
                // output the more tiles a workgroup sums itself; with two and four slabs half as many workgroups and
                // twice as many were measured: both slower)
                const uint64_t target = kSkinnyWorkgroups;
                const uint32_t k_tiles = static_cast<uint32_t>(k / BK);
                uint32_t tiles = static_cast<uint32_t>((static_cast<uint64_t>(k_tiles) * (n / 256) * count + target - 1) / target);
                tiles = tiles < 1 ? 1 : tiles > k_tiles ? k_tiles : tiles;
                const unsigned splits = (k_tiles + tiles - 1) / tiles;
                const dim3 grid(static_cast<unsigned>(n / 256), splits, count);
                const auto *a8 = static_cast<const uint8_t *>(a);
                const auto *b8 = static_cast<const uint8_t *>(b);
                const uint32_t m32 = static_cast<uint32_t>(m), r32 = static_cast<uint32_t>(r0), k32 = static_cast<uint32_t>(k),
                               n32 = static_cast<uint32_t>(n);
                if (rows <= 32) mmi_skinny<1><<<grid, 256, 0, s>>>(y, a8, b8, za, zb, rows, m32, r32, k32, n32, tiles, am0, bm0, ym0);
                else if (rows <= 64) mmi_skinny<2><<<grid, 256, 0, s>>>(y, a8, b8, za, zb, rows, m32, r32, k32, n32, tiles, am0, bm0, ym0);
                else mmi_skinny<4><<<grid, 256, 0, s>>>(y, a8, b8, za, zb, rows, m32, r32, k32, n32, tiles, am0, bm0, ym0);
                rc = launch_status();
                if (rc) return rc;
            }
            if constexpr (DEQ) {
                mmi_dequantize_in_place<<<static_cast<unsigned>(zero_grid > 4096 ? 4096 : zero_grid), 256, 0, s>>>(
                    y + static_cast<uint64_t>(ym0) * m * n, dq, static_cast<uint64_t>(count) * m, static_cast<uint32_t>(n));
                return launch_status();
            }
            return 0;
        }
        if (fast) {
            return launch_tiles(std::false_type{}, am0, bm0, ym0, count);
        } else if (small_tiles_ok) {
            return launch_small_tiles(am0, bm0, ym0, count);
        } else {
            const dim3 grid(static_cast<unsigned>((n + 15) / 16), static_cast<unsigned>((m + 15) / 16), count);
            mmi_generic<DEQ><<<grid, 256, 0, s>>>(
                y, static_cast<const uint8_t *>(a), static_cast<const uint8_t *>(b), za, zb, dq,
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
}  // namespace
}  // namespace rg

extern "C" int rg_hip_matmul_integer(int32_t *y, const void *a, const void *b, const void *a_zp,
                                     const void *b_zp, unsigned flags, size_t batch, size_t m,
                                     size_t k, size_t n, const uint32_t *a_index,
                                     const uint32_t *b_index, void * /*workspace*/, void *stream) {
    return rg::mmi_launch<false>(y, a, b, a_zp, b_zp, flags, batch, m, k, n, a_index, b_index, rg::Dequant{nullptr, 0},
                                 stream);
}

extern "C" int rg_hip_matmul_integer_dequantize(float *y, const void *a, const void *b, const void *a_zp,
                                                const void *b_zp, unsigned flags, size_t batch, size_t m,
                                                size_t k, size_t n, const uint32_t *a_index,
                                                const uint32_t *b_index, const float *scale, int scale_per_column,
                                                void * /*workspace*/, void *stream) {
    if (!scale) return RG_HIP_E_ARGUMENT;
    return rg::mmi_launch<true>(reinterpret_cast<int32_t *>(y), a, b, a_zp, b_zp, flags, batch, m, k, n, a_index, b_index,
                                rg::Dequant{scale, scale_per_column ? 1u : 0u}, stream);
}
