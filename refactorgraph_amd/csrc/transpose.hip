// Transpose (permutation of dimensions) for gfx950: pure data movement, HBM-bound.
//
// Contract: src/04kernel/src/kernels/transpose/cpu_kernel.cc:27-37 with the digest of
// src/04kernel/src/attributes/transpose_info.cc:7-126 — the output is `block_count` blocks of
// `block_size` bytes; output block i is input block locate(i), where locate() peels the output
// strides off i from the slowest dimension on and adds up the matching input strides.
//
// One kernel for every shape: the tensor is moved in words of W bytes, W the widest of 16, 8, 4, 2, 1
// that divides the block size and both addresses; word g of the output (consecutive lanes, consecutive
// words: stores are always contiguous) comes from word g % (block / W) of input block
// locate(g / (block / W)).  Blocks of 256 bytes and more (a head's row that keeps its place while
// sequence and head dimensions swap) read whole cache lines too; when it is two neighbouring
// dimensions that change places in front of such blocks, a workgroup takes 8 x 8 of them so that
// both sides move in runs of 8 blocks (transpose_tiles).  When the innermost dimension itself moves
// and a block is one element, tiles of 64 x 64 (32 x 32 for 8- and 16-byte elements) go through LDS,
// read in runs along the input's innermost dimension and written in runs along the output's
// (transpose_tile2d).  Only blocks of several words that are smaller than 64 bytes still gather.
// Divisions by the strides are multiplications by 2^64 / d rounded up (exact for 32-bit dividends).
#include "common.hpp"

namespace rg {
namespace {

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
constexpr int kMaxDims = 8;
constexpr int UNROLL = 4;  // words a thread has in flight
constexpr uint32_t TILE_H = 8, TILE_S = 8;   // blocks of a tile along the two dimensions that change places

struct Divisor {
    uint64_t magic;  // ceil(2^64 / d); 0 stands for d == 1
    uint32_t d;
    __device__ __forceinline__ uint32_t div(uint32_t n) const {
        return magic ? static_cast<uint32_t>(__umul64hi(static_cast<uint64_t>(n), magic)) : n;
    }
};

Divisor make_divisor(uint32_t d) {
    Divisor r;
    r.d = d;
    r.magic = d <= 1 ? 0 : ~0ull / d + 1;  // floor((2^64 - 1) / d) + 1 == ceil(2^64 / d) unless d divides 2^64,
                                           // where it is 2^64 / d as well
    return r;
}

struct Plan {
    Divisor stride_o[kMaxDims];
    uint32_t stride_i[kMaxDims];
    Divisor words_per_block;
    uint32_t dims;
    uint64_t words;  // of the whole tensor
};

template <class Word>
__global__ __launch_bounds__(256) void transpose_words(Word *__restrict__ y, const Word *__restrict__ x, const Plan p) {
    const uint64_t base = (static_cast<uint64_t>(blockIdx.x) * UNROLL) * 256 + threadIdx.x;
    Word v[UNROLL];
#pragma unroll
    for (int j = 0; j < UNROLL; ++j) {
        const uint64_t g = base + j * 256;
        if (g < p.words) {
            const uint32_t g32 = static_cast<uint32_t>(g);
            const uint32_t block = p.words_per_block.div(g32), word = g32 - block * p.words_per_block.d;
            uint32_t from = 0, rem = block;
            for (uint32_t d = 0; d < p.dims; ++d) {
                const uint32_t q = p.stride_o[d].div(rem);
                from += q * p.stride_i[d];
                rem -= q * p.stride_o[d].d;
            }
            v[j] = __builtin_nontemporal_load(x + static_cast<uint64_t>(from) * p.words_per_block.d + word);
        }
    }
#pragma unroll
    for (int j = 0; j < UNROLL; ++j) {
        const uint64_t g = base + j * 256;
        if (g < p.words) __builtin_nontemporal_store(v[j], y + g);
    }
}

// Expand whose innermost output dimension is broadcast from single elements (a column [n, 1] spread over rows, a scalar
// over a vector): a row of the output is one element repeated, so the output goes out in 16-byte words of copies of
// that element instead of one element per store (1.6 TB/s for 16-bit elements).  The plan's blocks are the rows (its
// dimensions those in front of the innermost one, output strides in rows), words_per_block their 16-byte words.
template <class Elem>
__global__ __launch_bounds__(256) void expand_splat(u32x4_t *__restrict__ y, const Elem *__restrict__ x, const Plan p) {
    const uint64_t base = (static_cast<uint64_t>(blockIdx.x) * UNROLL) * 256 + threadIdx.x;
#pragma unroll
    for (int j = 0; j < UNROLL; ++j) {
        const uint64_t g = base + j * 256;
        if (g < p.words) {
            const uint32_t row = p.words_per_block.div(static_cast<uint32_t>(g));
            uint32_t from = 0, rem = row;
            for (uint32_t d = 0; d < p.dims; ++d) {
                const uint32_t q = p.stride_o[d].div(rem);
                from += q * p.stride_i[d];
                rem -= q * p.stride_o[d].d;
            }
            const uint64_t e = x[from];
            uint64_t lo = e;
            if constexpr (sizeof(Elem) < 8) {
#pragma unroll
                for (unsigned bits = 8 * sizeof(Elem); bits < 64; bits *= 2) lo |= lo << bits;
            }
            u32x4_t v = {static_cast<uint32_t>(lo), static_cast<uint32_t>(lo >> 32), static_cast<uint32_t>(lo), static_cast<uint32_t>(lo >> 32)};
            __builtin_nontemporal_store(v, y + g);
        }
    }
}

// The common case of two neighbouring dimensions changing places in front of blocks that stay whole
// (digest: the last output dimension S has output stride 1, the one before it, H, input stride 1).
// A workgroup moves a tile of 8 x 8 blocks: it reads 8 runs of 8 neighbouring input blocks and
// writes 8 runs of 8 neighbouring output blocks, so both sides of the copy work on runs of 2 KiB
// (for 256-byte blocks) where the word kernel reads single blocks far apart.  (8 x 16 tiles with
// twice the loads in flight were not faster.)
struct TilePlan {
    Plan plan;           // for the dimensions in front of H and S
    uint32_t extent_h, extent_s, stride_i_s;  // stride_i of H is 1, stride_o of S is 1
    uint32_t tiles_s;    // extent_s / TILE_S
    Divisor tiles_per_outer;
};

template <class Word>
__global__ __launch_bounds__(256) void transpose_tiles(Word *__restrict__ y, const Word *__restrict__ x, const TilePlan t) {
    const Plan &p = t.plan;
    const uint32_t wpb = p.words_per_block.d;
    // tile -> (outer index, tile row of H, tile column of S); all wave-uniform
    const uint32_t tile = blockIdx.x;
    const uint32_t outer = t.tiles_per_outer.div(tile), r = tile - outer * t.tiles_per_outer.d;
    const uint32_t th = r / t.tiles_s, ts = r - th * t.tiles_s;
    const uint32_t out0 = outer * t.extent_h * t.extent_s;  // first output block of this outer index
    uint32_t in0 = 0, rem = out0;
    for (uint32_t d = 0; d + 2 < p.dims; ++d) {
        const uint32_t q = p.stride_o[d].div(rem);
        in0 += q * p.stride_i[d];
        rem -= q * p.stride_o[d].d;
    }
    const uint32_t words = TILE_H * TILE_S * wpb;  // of the tile
    for (uint32_t w0 = 0; w0 < words; w0 += 256 * UNROLL) {
        Word v[UNROLL];
        uint32_t row[UNROLL], col[UNROLL];
#pragma unroll
        for (int j = 0; j < UNROLL; ++j) {
            const uint32_t w = w0 + j * 256 + threadIdx.x;
            row[j] = p.words_per_block.div(w);  // TILE_H ss + hh: neighbouring rows are neighbouring input blocks
            col[j] = w - row[j] * wpb;
            if (w < words) {
                const uint32_t hh = row[j] % TILE_H, ss = row[j] / TILE_H;
                const uint64_t from = in0 + (th * TILE_H + hh) + static_cast<uint64_t>(ts * TILE_S + ss) * t.stride_i_s;
                v[j] = __builtin_nontemporal_load(x + from * wpb + col[j]);
            }
        }
#pragma unroll
        for (int j = 0; j < UNROLL; ++j) {
            const uint32_t w = w0 + j * 256 + threadIdx.x;
            if (w < words) {
                const uint32_t hh = row[j] % TILE_H, ss = row[j] / TILE_H;
                const uint64_t to = out0 + static_cast<uint64_t>(th * TILE_H + hh) * t.extent_s + (ts * TILE_S + ss);
                __builtin_nontemporal_store(v[j], y + to * wpb + col[j]);
            }
        }
    }
}

// The innermost dimension itself moves (blocks of one element): an LDS tile turns the gather into
// two coalesced sides.  F is the dimension that is innermost in the input (input stride 1), L the one
// that is innermost in the output; a workgroup reads a T x T tile in runs along F, writes it in runs
// along L, and the other dimensions are peeled off the workgroup index.
constexpr int kMaxOuter = kMaxDims - 2;
struct Tile2dPlan {
    uint32_t outer_dims;
    uint32_t outer_extent[kMaxOuter], outer_si[kMaxOuter], outer_so[kMaxOuter];
    uint32_t extent_f, extent_l;  // elements along F and L
    uint32_t si_l, so_f;          // input stride of L, output stride of F (those of F resp. L are 1)
    uint32_t tiles_f, tiles_l;
};

template <class Word, int T>
__global__ __launch_bounds__(256) void transpose_tile2d(Word *__restrict__ y, const Word *__restrict__ x, const Tile2dPlan p) {
    __shared__ Word tile[T][T + 1];
    uint32_t b = blockIdx.x;
    const uint32_t tl = b % p.tiles_l;
    b /= p.tiles_l;
    const uint32_t tf = b % p.tiles_f;
    b /= p.tiles_f;
    uint64_t in0 = 0, out0 = 0;
    for (uint32_t d = 0; d < p.outer_dims; ++d) {
        const uint32_t i = b % p.outer_extent[d];
        b /= p.outer_extent[d];
        in0 += static_cast<uint64_t>(i) * p.outer_si[d];
        out0 += static_cast<uint64_t>(i) * p.outer_so[d];
    }
    const uint32_t f0 = tf * T, l0 = tl * T;
    constexpr int ROWS_PER_PASS = 256 / T;
    const uint32_t fast = threadIdx.x % T, slow = threadIdx.x / T;
#pragma unroll
    for (int j = 0; j < T / ROWS_PER_PASS; ++j) {
        const uint32_t l = slow + ROWS_PER_PASS * j;
        if (f0 + fast < p.extent_f && l0 + l < p.extent_l)
            tile[l][fast] = x[in0 + static_cast<uint64_t>(l0 + l) * p.si_l + f0 + fast];
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < T / ROWS_PER_PASS; ++j) {
        const uint32_t f = slow + ROWS_PER_PASS * j;
        if (f0 + f < p.extent_f && l0 + fast < p.extent_l)
            y[out0 + static_cast<uint64_t>(f0 + f) * p.so_f + l0 + fast] = tile[fast][f];
    }
}

// Fills the plan if the digest describes single-element blocks with an innermost input dimension that
// is not the innermost output dimension; returns the grid size or 0.
uint64_t plan_tile2d(Tile2dPlan &t, const uint32_t *stride_i, const uint32_t *stride_o, size_t dims, uint64_t block_count,
                     uint32_t tile) {
    if (dims < 2 || stride_o[dims - 1] != 1) return 0;
    const size_t l = dims - 1;
    size_t f = dims;
    for (size_t d = 0; d + 1 < dims; ++d)
        if (stride_i[d] == 1) f = d;
    if (f == dims) return 0;
    auto extent = [&](size_t d) { return static_cast<uint32_t>((d == 0 ? block_count : stride_o[d - 1]) / stride_o[d]); };
    t = Tile2dPlan{};
    t.extent_f = extent(f);
    t.extent_l = extent(l);
    t.si_l = stride_i[l];
    t.so_f = stride_o[f];
    t.tiles_f = (t.extent_f + tile - 1) / tile;
    t.tiles_l = (t.extent_l + tile - 1) / tile;
    uint64_t grid = static_cast<uint64_t>(t.tiles_f) * t.tiles_l;
    for (size_t d = 0; d < dims; ++d) {
        if (d == f || d == l) continue;
        t.outer_extent[t.outer_dims] = extent(d);
        t.outer_si[t.outer_dims] = stride_i[d];
        t.outer_so[t.outer_dims] = stride_o[d];
        grid *= t.outer_extent[t.outer_dims++];
    }
    return grid;
}

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// The same for elements of ES = 1 or 2 bytes whose rows start on 16-byte boundaries on both sides: tiles of T x T
// elements with T = 128 / ES, so that a row of a tile is one 128-byte line either way.  A thread loads 4 / ES
// neighbouring rows of 16 bytes along F, turns them in registers (v_perm_b32) into one 32-bit word per F index that
// holds 4 / ES neighbouring L indices, and writes those words into an LDS tile kept as [F][L] (the eight 16-byte
// pieces of a row XOR-swizzled by F / (16 / ES), which spreads a wavefront's writes over the banks); the way out is
// one 128-bit LDS read and one 128-bit store per thread and piece.  One element per instruction, as above, ran at
// 2.3 (8-bit) and 3.7 TB/s (16-bit).
template <int ES>
__global__ __launch_bounds__(256) void transpose_tile2d_vec(uint8_t *__restrict__ y, const uint8_t *__restrict__ x, const Tile2dPlan p) {
    constexpr int V = 16 / ES, T = 128 / ES, R = 4 / ES;  // elements of a vector, tile edge, rows a thread loads
    __shared__ __align__(16) uint8_t tile[T * 128];
    uint32_t b = blockIdx.x;
    const uint32_t tl = b % p.tiles_l;
    b /= p.tiles_l;
    const uint32_t tf = b % p.tiles_f;
    b /= p.tiles_f;
    uint64_t in0 = 0, out0 = 0;  // in elements
    for (uint32_t d = 0; d < p.outer_dims; ++d) {
        const uint32_t i = b % p.outer_extent[d];
        b /= p.outer_extent[d];
        in0 += static_cast<uint64_t>(i) * p.outer_si[d];
        out0 += static_cast<uint64_t>(i) * p.outer_so[d];
    }
    const uint32_t f0 = tf * T, l0 = tl * T;
    const uint32_t g = threadIdx.x >> 3, c = threadIdx.x & 7;  // rows R g .. R g + R - 1 of L, F indices V c .. V c + V - 1
    u32x4 r[R];
#pragma unroll
    for (int i = 0; i < R; ++i) r[i] = u32x4{0u, 0u, 0u, 0u};
    if (f0 + V * c < p.extent_f && l0 + R * g < p.extent_l) {  // (the extents are multiples of V: whole vectors, whole groups)
#pragma unroll
        for (int i = 0; i < R; ++i)
            r[i] = *reinterpret_cast<const u32x4 *>(x + (in0 + static_cast<uint64_t>(l0 + R * g + i) * p.si_l + f0 + V * c) * ES);
    }
    // word g of row f: byte 16 ((g / 4) ^ (f / V % 8)) + 4 (g % 4) of the row
    const uint32_t at = 16 * ((g >> 2) ^ c) + 4 * (g & 3);
    if constexpr (ES == 2) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            *reinterpret_cast<uint32_t *>(tile + (V * c + 2 * j) * 128 + at) = __builtin_amdgcn_perm(r[1][j], r[0][j], 0x05040100u);
            *reinterpret_cast<uint32_t *>(tile + (V * c + 2 * j + 1) * 128 + at) = __builtin_amdgcn_perm(r[1][j], r[0][j], 0x07060302u);
        }
    } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t lo01 = __builtin_amdgcn_perm(r[1][j], r[0][j], 0x05010400u), hi01 = __builtin_amdgcn_perm(r[1][j], r[0][j], 0x07030602u);
            const uint32_t lo23 = __builtin_amdgcn_perm(r[3][j], r[2][j], 0x05010400u), hi23 = __builtin_amdgcn_perm(r[3][j], r[2][j], 0x07030602u);
            *reinterpret_cast<uint32_t *>(tile + (V * c + 4 * j) * 128 + at) = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u);
            *reinterpret_cast<uint32_t *>(tile + (V * c + 4 * j + 1) * 128 + at) = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u);
            *reinterpret_cast<uint32_t *>(tile + (V * c + 4 * j + 2) * 128 + at) = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u);
            *reinterpret_cast<uint32_t *>(tile + (V * c + 4 * j + 3) * 128 + at) = __builtin_amdgcn_perm(hi23, hi01, 0x07060302u);
        }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < T / 32; ++i) {
        const uint32_t f = g + 32 * i;  // piece c of row f: L indices V c .. V c + V - 1
        const u32x4 v = *reinterpret_cast<const u32x4 *>(tile + f * 128 + 16 * (c ^ ((f / V) & 7)));
        if (f0 + f < p.extent_f && l0 + V * c < p.extent_l)
            *reinterpret_cast<u32x4 *>(y + (out0 + static_cast<uint64_t>(f0 + f) * p.so_f + l0 + V * c) * ES) = v;
    }
}

// True when transpose_tile2d_vec applies: every row of either side starts on a 16-byte boundary.
template <int ES>
bool tile2d_vec_fits(const Tile2dPlan &t, const void *y, const void *x) {
    constexpr uint32_t V = 16 / ES;
    bool ok = aligned16(x) && aligned16(y) && t.extent_f % V == 0 && t.extent_l % V == 0 && t.si_l % V == 0 && t.so_f % V == 0;
    for (uint32_t d = 0; d < t.outer_dims; ++d) ok = ok && t.outer_si[d] % V == 0 && t.outer_so[d] % V == 0;
    return ok;
}

template <class Word>
int launch(void *y, const void *x, const Plan &p, const uint32_t *stride_i, const uint32_t *stride_o, uint64_t block_count,
           hipStream_t s) {
    // blocks of one element of 8 or 16 bits with aligned rows: the vector form of the LDS tile
    if constexpr (sizeof(Word) <= 2) {
        if (p.words_per_block.d == 1) {
            constexpr int ES = sizeof(Word);
            Tile2dPlan t;
            const uint64_t grid = plan_tile2d(t, stride_i, stride_o, p.dims, block_count, 128 / ES);
            if (grid && grid <= 0x7fffffffull && tile2d_vec_fits<ES>(t, y, x)) {
                transpose_tile2d_vec<ES><<<static_cast<unsigned>(grid), 256, 0, s>>>(static_cast<uint8_t *>(y),
                                                                                     static_cast<const uint8_t *>(x), t);
                return launch_status();
            }
        }
    }
    // blocks of one element: through an LDS tile
    if (p.words_per_block.d == 1) {
        constexpr int T = sizeof(Word) <= 4 ? 64 : 32;
        Tile2dPlan t;
        const uint64_t grid = plan_tile2d(t, stride_i, stride_o, p.dims, block_count, T);
        if (grid && grid <= 0x7fffffffull) {
            transpose_tile2d<Word, T><<<static_cast<unsigned>(grid), 256, 0, s>>>(static_cast<Word *>(y),
                                                                                 static_cast<const Word *>(x), t);
            return launch_status();
        }
    }
    // two neighbouring dimensions change places in front of whole blocks of 64 bytes or more
    if (p.dims >= 2 && p.stride_i[p.dims - 2] == 1 && p.words_per_block.d * sizeof(Word) >= 64) {
        const uint32_t extent_s = p.stride_o[p.dims - 2].d;
        const uint64_t outer_blocks = p.dims >= 3 ? p.stride_o[p.dims - 3].d : block_count;
        const uint32_t extent_h = static_cast<uint32_t>(outer_blocks / extent_s);
        if (extent_s % TILE_S == 0 && extent_h % TILE_H == 0 && outer_blocks % extent_s == 0) {
            TilePlan t{};
            t.plan = p;
            t.extent_h = extent_h;
            t.extent_s = extent_s;
            t.stride_i_s = p.stride_i[p.dims - 1];
            t.tiles_s = extent_s / TILE_S;
            t.tiles_per_outer = make_divisor((extent_h / TILE_H) * (extent_s / TILE_S));
            const uint64_t tiles = block_count / (TILE_H * TILE_S);
            if (tiles <= 0x7fffffffull) {
                transpose_tiles<Word><<<static_cast<unsigned>(tiles), 256, 0, s>>>(static_cast<Word *>(y),
                                                                                  static_cast<const Word *>(x), t);
                return launch_status();
            }
        }
    }
    const uint64_t per_wg = 256ull * UNROLL;
    const uint64_t grid = (p.words + per_wg - 1) / per_wg;
    if (grid > 0x7fffffffull) return RG_HIP_E_UNSUPPORTED;
    transpose_words<Word><<<static_cast<unsigned>(grid), 256, 0, s>>>(static_cast<Word *>(y), static_cast<const Word *>(x), p);
    return launch_status();
}

}  // namespace
}  // namespace rg

// Expand (one-directional broadcast), contract src/04kernel/src/kernels/expand/cpu_kernel.cc:27-46 with the
// digest of src/04kernel/src/attributes/expand_info.cc:14-60: output block i is input block
// j = sum over the dimensions of (rem / o) * i, rem %= o — the arithmetic of the transposition's locate()
// with input strides that are 0 where the input is broadcast, so the word kernel above serves as it is.
extern "C" int rg_hip_expand(void *y, const void *x, const uint32_t *stride_i, const uint32_t *stride_o, size_t dims,
                             size_t block_size, size_t block_count, void *stream) {
    using namespace rg;
    if (!y || !x || (dims && (!stride_i || !stride_o))) return RG_HIP_E_ARGUMENT;
    if (dims > static_cast<size_t>(kMaxDims)) return RG_HIP_E_UNSUPPORTED;
    if (block_size == 0 || block_count == 0) return 0;
    if (y == x) return RG_HIP_E_ARGUMENT;
    const uint64_t bytes = static_cast<uint64_t>(block_size) * block_count;
    if (block_count > 0xffffffffull) return RG_HIP_E_UNSUPPORTED;
    hipStream_t s = as_stream(stream);
    if (dims == 0) return static_cast<int>(hipMemcpyAsync(y, x, bytes, hipMemcpyDeviceToDevice, s));  // nothing is broadcast
    // single elements repeated along the innermost output dimension, rows of whole 16-byte words
    if (stride_i[dims - 1] == 0 && stride_o[dims - 1] == 1 && (block_size == 1 || block_size == 2 || block_size == 4 || block_size == 8) &&
        aligned16(y) && (reinterpret_cast<uintptr_t>(x) & (block_size - 1)) == 0) {
        const uint64_t row = dims >= 2 ? stride_o[dims - 2] : block_count;  // elements of a row
        bool ok = row > 0 && (row * block_size) % 16 == 0 && bytes / 16 <= 0xffffffffull;
        for (size_t d = 0; d + 1 < dims && ok; ++d) ok = stride_o[d] != 0 && stride_o[d] % row == 0;
        if (ok) {
            Plan p{};
            p.dims = static_cast<uint32_t>(dims - 1);
            p.words = bytes / 16;
            p.words_per_block = make_divisor(static_cast<uint32_t>(row * block_size / 16));
            for (size_t d = 0; d + 1 < dims; ++d) {
                p.stride_o[d] = make_divisor(static_cast<uint32_t>(stride_o[d] / row));
                p.stride_i[d] = stride_i[d];
            }
            const uint64_t grid = (p.words + 256ull * UNROLL - 1) / (256ull * UNROLL);
            if (grid <= 0x7fffffffull) {
                const unsigned g = static_cast<unsigned>(grid);
                u32x4_t *out = static_cast<u32x4_t *>(y);
                switch (block_size) {
                    case 1: expand_splat<uint8_t><<<g, 256, 0, s>>>(out, static_cast<const uint8_t *>(x), p); break;
                    case 2: expand_splat<uint16_t><<<g, 256, 0, s>>>(out, static_cast<const uint16_t *>(x), p); break;
                    case 4: expand_splat<uint32_t><<<g, 256, 0, s>>>(out, static_cast<const uint32_t *>(x), p); break;
                    default: expand_splat<uint64_t><<<g, 256, 0, s>>>(out, static_cast<const uint64_t *>(x), p); break;
                }
                return launch_status();
            }
        }
    }
    const uintptr_t misalign = reinterpret_cast<uintptr_t>(y) | reinterpret_cast<uintptr_t>(x) | block_size;
    uint32_t w = 16;
    while (misalign & (w - 1)) w >>= 1;
    const uint64_t words = bytes / w;
    if (words > 0xffffffffull) return RG_HIP_E_UNSUPPORTED;
    Plan p{};
    p.dims = static_cast<uint32_t>(dims);
    p.words = words;
    p.words_per_block = make_divisor(static_cast<uint32_t>(block_size / w));
    for (size_t d = 0; d < dims; ++d) {
        if (stride_o[d] == 0) return RG_HIP_E_ARGUMENT;
        p.stride_o[d] = make_divisor(stride_o[d]);
        p.stride_i[d] = stride_i[d];
    }
    const uint64_t grid = (p.words + 256ull * UNROLL - 1) / (256ull * UNROLL);
    if (grid > 0x7fffffffull) return RG_HIP_E_UNSUPPORTED;
    const unsigned g = static_cast<unsigned>(grid);
    switch (w) {
        case 16: transpose_words<u32x4><<<g, 256, 0, s>>>(static_cast<u32x4 *>(y), static_cast<const u32x4 *>(x), p); break;
        case 8: transpose_words<uint64_t><<<g, 256, 0, s>>>(static_cast<uint64_t *>(y), static_cast<const uint64_t *>(x), p); break;
        case 4: transpose_words<uint32_t><<<g, 256, 0, s>>>(static_cast<uint32_t *>(y), static_cast<const uint32_t *>(x), p); break;
        case 2: transpose_words<uint16_t><<<g, 256, 0, s>>>(static_cast<uint16_t *>(y), static_cast<const uint16_t *>(x), p); break;
        default: transpose_words<uint8_t><<<g, 256, 0, s>>>(static_cast<uint8_t *>(y), static_cast<const uint8_t *>(x), p); break;
    }
    return launch_status();
}

extern "C" int rg_hip_transpose(void *y, const void *x, const uint32_t *stride_i, const uint32_t *stride_o,
                                size_t dims, size_t block_size, size_t block_count, void *stream) {
    using namespace rg;
    if (!y || !x || !stride_i || !stride_o) return RG_HIP_E_ARGUMENT;
    if (dims == 0 || dims > static_cast<size_t>(kMaxDims)) return RG_HIP_E_UNSUPPORTED;
    if (block_size == 0 || block_count == 0) return 0;
    if (y == x) return RG_HIP_E_ARGUMENT;  // not an in-place operation
    const uint64_t bytes = static_cast<uint64_t>(block_size) * block_count;
    if (block_count > 0xffffffffull) return RG_HIP_E_UNSUPPORTED;
    hipStream_t s = as_stream(stream);
    if (block_count == 1) return static_cast<int>(hipMemcpyAsync(y, x, bytes, hipMemcpyDeviceToDevice, s));

    const uintptr_t misalign = reinterpret_cast<uintptr_t>(y) | reinterpret_cast<uintptr_t>(x) | block_size;
    uint32_t w = 16;
    while (misalign & (w - 1)) w >>= 1;
    const uint64_t words = bytes / w;
    if (words > 0xffffffffull) return RG_HIP_E_UNSUPPORTED;  // word indices are 32-bit in the kernel

    Plan p{};
    p.dims = static_cast<uint32_t>(dims);
    p.words = words;
    p.words_per_block = make_divisor(static_cast<uint32_t>(block_size / w));
    for (size_t d = 0; d < dims; ++d) {
        if (stride_o[d] == 0) return RG_HIP_E_ARGUMENT;
        p.stride_o[d] = make_divisor(stride_o[d]);
        p.stride_i[d] = stride_i[d];
    }
    switch (w) {
        case 16: return launch<u32x4>(y, x, p, stride_i, stride_o, block_count, s);
        case 8: return launch<uint64_t>(y, x, p, stride_i, stride_o, block_count, s);
        case 4: return launch<uint32_t>(y, x, p, stride_i, stride_o, block_count, s);
        case 2: return launch<uint16_t>(y, x, p, stride_i, stride_o, block_count, s);
        default: return launch<uint8_t>(y, x, p, stride_i, stride_o, block_count, s);
    }
}
