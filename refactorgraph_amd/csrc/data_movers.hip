// Split, Concat and Where for gfx950: pure data movement, HBM-bound.
//
// Split / Concat contract: src/04kernel/src/kernels/{split,concat}/cpu_kernel.cc with the digest of
// src/04kernel/src/attributes/split_info.cc:5-30 — the joined tensor is `block_count` blocks of `sum`
// bytes; block i is the concatenation of `count` segments, segment j being bytes
// [i * len_j, (i + 1) * len_j) of part j.  The reference's CUDA kernels (src/04kernel/cuda/src/
// split.cu:7-50, concat.cu:7-50) stage the part pointers in shared memory and copy units of at most
// 16 bytes found by a gcd; here pointers and segment bounds travel in the kernel arguments (16 parts
// a launch), the unit is the widest power of two up to 16 bytes that divides every segment length
// and address, and a thread walks the joined tensor linearly, so that the joined side moves in
// whole lines and each part's side in runs of its segment length.
//
// Where contract: src/04kernel/src/kernels/where/cpu_kernel.cc:32-47 — output element i is element
// locate(i)[1] of x where element locate(i)[0] of the condition is true, else element locate(i)[2]
// of y; locate is the Broadcaster's (src/04kernel/src/attributes/broadcaster.cc:87-100).
#include "common.hpp"

namespace rg {
namespace {

constexpr int kMaxParts = 16;
constexpr int UNROLL = 1;  // words per thread and pass: more of them in flight per thread were slower (4: 62 %, 2: 72 %, 1: 74 % of HBM)

struct Parts {
    uint64_t ptr[kMaxParts];       // part tensors
    uint32_t begin[kMaxParts + 1]; // byte offset of each part's segment within a block of the joined tensor
    uint32_t count;
    uint32_t sum;                  // bytes of a block of the joined tensor
    uint32_t block_count;
    uint32_t words;                // words of the segments covered by this launch, per block
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// CONCAT: parts -> joined, else joined -> parts.  A workgroup covers 256 >> rows_log2 words of
// 1 << rows_log2 blocks at a time (short blocks: several blocks per workgroup).
template <class Word, bool CONCAT>
__global__ __launch_bounds__(256) void parts_copy(uint8_t *__restrict__ joined, const Parts p, uint32_t rows_log2) {
    const uint32_t cols = 256u >> rows_log2;
    const uint32_t col = threadIdx.x & (cols - 1), row_in_wg = threadIdx.x >> (8 - rows_log2);
    for (uint32_t row = (blockIdx.y << rows_log2) + row_in_wg; row < p.block_count; row += gridDim.y << rows_log2) {
        for (uint32_t w0 = blockIdx.x * cols * UNROLL; w0 < p.words; w0 += gridDim.x * cols * UNROLL) {
            Word v[UNROLL];
            uint8_t *to[UNROLL];
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                const uint32_t w = w0 + u * cols + col;
                to[u] = nullptr;
                if (w < p.words) {
                    const uint32_t off = p.begin[0] + w * static_cast<uint32_t>(sizeof(Word));
                    uint32_t j = 0;
#pragma unroll
                    for (int s = 1; s < kMaxParts; ++s) j += (s < static_cast<int>(p.count) && off >= p.begin[s]) ? 1u : 0u;
                    const uint32_t len = p.begin[j + 1] - p.begin[j];
                    uint8_t *part = reinterpret_cast<uint8_t *>(p.ptr[j]) + static_cast<uint64_t>(row) * len + (off - p.begin[j]);
                    uint8_t *whole = joined + static_cast<uint64_t>(row) * p.sum + off;
                    const uint8_t *from = CONCAT ? part : whole;
                    to[u] = CONCAT ? whole : part;
                    v[u] = *reinterpret_cast<const Word *>(from);  // (plain loads, streaming stores: the fastest of the four combinations)
                }
            }
#pragma unroll
            for (int u = 0; u < UNROLL; ++u)
                if (to[u]) __builtin_nontemporal_store(v[u], reinterpret_cast<Word *>(to[u]));
        }
    }
}

template <class Word, bool CONCAT>
int launch_parts(uint8_t *joined, const Parts &p, hipStream_t s) {
    // short blocks share a workgroup: as many blocks as keep a row of the workgroup at 8 words or more
    uint32_t rows_log2 = 0;
    while (rows_log2 < 5 && (256u >> (rows_log2 + 1)) * UNROLL >= p.words && (1u << rows_log2) < p.block_count) ++rows_log2;
    const uint32_t cols = 256u >> rows_log2;
    uint64_t gx = (static_cast<uint64_t>(p.words) + cols * UNROLL - 1) / (cols * UNROLL);
    uint64_t gy = (static_cast<uint64_t>(p.block_count) + (1u << rows_log2) - 1) >> rows_log2;
    if (gy > 65535) gy = 65535;
    if (gx > 65535) gx = 65535;
    parts_copy<Word, CONCAT><<<dim3(static_cast<unsigned>(gx), static_cast<unsigned>(gy)), 256, 0, s>>>(joined, p, rows_log2);
    return launch_status();
}

template <bool CONCAT>
int parts_entry(void *joined, const void *const *parts, const uint32_t *segments, size_t count, size_t block_count,
                size_t sum, hipStream_t s) {
    if (!joined || !parts || !segments) return RG_HIP_E_ARGUMENT;
    if (count == 0 || block_count == 0 || sum == 0) return 0;
    if (block_count > 0xffffffffull || sum > 0xffffffffull) return RG_HIP_E_UNSUPPORTED;
    uint64_t total = 0;
    uintptr_t misalign = reinterpret_cast<uintptr_t>(joined) | sum;
    for (size_t j = 0; j < count; ++j) {
        if (segments[j] && !parts[j]) return RG_HIP_E_ARGUMENT;
        total += segments[j];
        misalign |= reinterpret_cast<uintptr_t>(parts[j]) | segments[j];
    }
    if (total != sum) return RG_HIP_E_ARGUMENT;
    uint32_t w = 16;
    while (misalign & (w - 1)) w >>= 1;
    uint32_t begin = 0;
    for (size_t j0 = 0; j0 < count; j0 += kMaxParts) {
        Parts p{};
        p.count = static_cast<uint32_t>(count - j0 < kMaxParts ? count - j0 : kMaxParts);
        p.sum = static_cast<uint32_t>(sum);
        p.block_count = static_cast<uint32_t>(block_count);
        for (uint32_t j = 0; j < p.count; ++j) {
            p.ptr[j] = reinterpret_cast<uint64_t>(parts[j0 + j]);
            p.begin[j] = begin;
            begin += segments[j0 + j];
        }
        for (uint32_t j = p.count; j <= kMaxParts; ++j) p.begin[j] = begin;
        p.words = (begin - p.begin[0]) / w;
        if (p.words == 0) continue;
        int rc;
        uint8_t *jn = static_cast<uint8_t *>(joined);
        switch (w) {
            case 16: rc = launch_parts<u32x4, CONCAT>(jn, p, s); break;
            case 8: rc = launch_parts<uint64_t, CONCAT>(jn, p, s); break;
            case 4: rc = launch_parts<uint32_t, CONCAT>(jn, p, s); break;
            case 2: rc = launch_parts<uint16_t, CONCAT>(jn, p, s); break;
            default: rc = launch_parts<uint8_t, CONCAT>(jn, p, s); break;
        }
        if (rc) return rc;
    }
    return 0;
}

// ---------------------------------------------------------------- Where

constexpr int kMaxDims = 8;
struct WherePlan {
    uint64_t magic[kMaxDims];      // ceil(2^64 / output stride); 0 stands for stride 1
    uint32_t stride_o[kMaxDims];
    uint32_t stride_in[kMaxDims][3];
    uint32_t dims;
    uint32_t count;
};

template <class Elem>
__global__ __launch_bounds__(256) void where_elements(Elem *__restrict__ out, const uint8_t *__restrict__ c,
                                                      const Elem *__restrict__ x, const Elem *__restrict__ y, const WherePlan p) {
    for (uint32_t i = blockIdx.x * 256 + threadIdx.x; i < p.count; i += gridDim.x * 256) {
        uint32_t at[3] = {i, i, i};
        if (p.dims) {
            at[0] = at[1] = at[2] = 0;
            uint32_t rem = i;
            for (uint32_t d = 0; d < p.dims; ++d) {
                const uint32_t q = p.magic[d] ? static_cast<uint32_t>(__umul64hi(static_cast<uint64_t>(rem), p.magic[d])) : rem;
                rem -= q * p.stride_o[d];
#pragma unroll
                for (int j = 0; j < 3; ++j) at[j] += q * p.stride_in[d][j];
            }
        }
        out[i] = c[at[0]] ? x[at[1]] : y[at[2]];
    }
}

// No broadcasting and everything 16-byte aligned: 16 bytes of output per thread.
template <class Elem>
__global__ __launch_bounds__(256) void where_vec(Elem *__restrict__ out, const uint8_t *__restrict__ c,
                                                 const Elem *__restrict__ x, const Elem *__restrict__ y, uint64_t groups) {
    constexpr int E = 16 / sizeof(Elem);
    struct alignas(16) Group {
        Elem v[E];
    };
    struct alignas(E) Flags {
        uint8_t v[E];
    };
    for (uint64_t g = static_cast<uint64_t>(blockIdx.x) * 256 + threadIdx.x; g < groups; g += static_cast<uint64_t>(gridDim.x) * 256) {
        const Flags f = reinterpret_cast<const Flags *>(c)[g];
        const Group a = reinterpret_cast<const Group *>(x)[g], b = reinterpret_cast<const Group *>(y)[g];
        Group r;
#pragma unroll
        for (int e = 0; e < E; ++e) r.v[e] = f.v[e] ? a.v[e] : b.v[e];
        reinterpret_cast<Group *>(out)[g] = r;
    }
}

// Broadcasting whose innermost dimension is a multiple of 16 bytes long: a thread still produces 16 bytes of
// output, divides once for all of them, and reads from each input either the 16 bytes (flags: E bytes) beside
// them (innermost stride 1) or the one element they all share (innermost stride 0).
template <class Elem>
__global__ __launch_bounds__(256) void where_groups(Elem *__restrict__ out, const uint8_t *__restrict__ c,
                                                    const Elem *__restrict__ x, const Elem *__restrict__ y, const WherePlan p,
                                                    uint32_t groups) {
    constexpr int E = 16 / sizeof(Elem);
    struct alignas(16) Group {
        Elem v[E];
    };
    struct alignas(E) Flags {
        uint8_t v[E];
    };
    const uint32_t last = p.dims - 1;
    const bool run_c = p.stride_in[last][0], run_x = p.stride_in[last][1], run_y = p.stride_in[last][2];
    for (uint32_t g = blockIdx.x * 256 + threadIdx.x; g < groups; g += gridDim.x * 256) {
        uint32_t at[3] = {0, 0, 0};
        uint32_t rem = g * E;
        for (uint32_t d = 0; d < p.dims; ++d) {
            const uint32_t q = p.magic[d] ? static_cast<uint32_t>(__umul64hi(static_cast<uint64_t>(rem), p.magic[d])) : rem;
            rem -= q * p.stride_o[d];
#pragma unroll
            for (int j = 0; j < 3; ++j) at[j] += q * p.stride_in[d][j];
        }
        Flags f;
        Group a, b, r;
        if (run_c) {
            f = *reinterpret_cast<const Flags *>(c + at[0]);
        } else {
            const uint8_t one = c[at[0]];
#pragma unroll
            for (int e = 0; e < E; ++e) f.v[e] = one;
        }
        if (run_x) {
            a = *reinterpret_cast<const Group *>(x + at[1]);
        } else {
            const Elem one = x[at[1]];
#pragma unroll
            for (int e = 0; e < E; ++e) a.v[e] = one;
        }
        if (run_y) {
            b = *reinterpret_cast<const Group *>(y + at[2]);
        } else {
            const Elem one = y[at[2]];
#pragma unroll
            for (int e = 0; e < E; ++e) b.v[e] = one;
        }
#pragma unroll
        for (int e = 0; e < E; ++e) r.v[e] = f.v[e] ? a.v[e] : b.v[e];
        reinterpret_cast<Group *>(out)[g] = r;
    }
}

template <class Elem>
int launch_where(void *out, const void *c, const void *x, const void *y, const WherePlan &p, hipStream_t s) {
    constexpr uint32_t E = 16 / sizeof(Elem);
    const uintptr_t mis = reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y);
    if (p.dims == 0 && p.count % E == 0 && (mis & 15) == 0 && (reinterpret_cast<uintptr_t>(c) & (E - 1)) == 0) {
        const uint64_t groups = p.count / E;
        uint64_t grid = (groups + 255) / 256;
        if (grid > 1u << 20) grid = 1u << 20;
        where_vec<Elem><<<static_cast<unsigned>(grid), 256, 0, s>>>(static_cast<Elem *>(out), static_cast<const uint8_t *>(c),
                                                                    static_cast<const Elem *>(x), static_cast<const Elem *>(y), groups);
        return launch_status();
    }
    if (p.dims) {
        // groups of E outputs never straddle the innermost dimension, and an input that runs along it (stride 1)
        // has every outer stride a multiple of its length: aligned bases then make every group access aligned
        const uint32_t last = p.dims - 1;
        const uint32_t inner = p.dims == 1 ? p.count : p.stride_o[last - 1];
        bool ok = p.stride_o[last] == 1 && inner % E == 0 && p.count % E == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0;
        const uintptr_t base[3] = {reinterpret_cast<uintptr_t>(c), reinterpret_cast<uintptr_t>(x), reinterpret_cast<uintptr_t>(y)};
        for (int j = 0; j < 3 && ok; ++j) {
            const uint32_t st = p.stride_in[last][j];
            ok = st == 0 || (st == 1 && (base[j] & (j == 0 ? E - 1 : 15)) == 0);
            for (uint32_t d = 0; d < last && ok && st == 1; ++d) ok = p.stride_in[d][j] % E == 0;
        }
        if (ok) {
            const uint32_t groups = p.count / E;
            uint32_t grid = (groups + 255) / 256;
            if (grid > 1u << 20) grid = 1u << 20;
            where_groups<Elem><<<grid, 256, 0, s>>>(static_cast<Elem *>(out), static_cast<const uint8_t *>(c),
                                                    static_cast<const Elem *>(x), static_cast<const Elem *>(y), p, groups);
            return launch_status();
        }
    }
    uint64_t grid = (static_cast<uint64_t>(p.count) + 255) / 256;
    if (grid > 1u << 20) grid = 1u << 20;
    where_elements<Elem><<<static_cast<unsigned>(grid), 256, 0, s>>>(static_cast<Elem *>(out), static_cast<const uint8_t *>(c),
                                                                     static_cast<const Elem *>(x), static_cast<const Elem *>(y), p);
    return launch_status();
}

}  // namespace
}  // namespace rg

extern "C" int rg_hip_split(void *const *outputs, const void *x, const uint32_t *segments, size_t count, size_t block_count,
                            size_t sum, void *stream) {
    return rg::parts_entry<false>(const_cast<void *>(x), outputs, segments, count, block_count, sum, rg::as_stream(stream));
}

extern "C" int rg_hip_concat(void *y, const void *const *inputs, const uint32_t *segments, size_t count, size_t block_count,
                             size_t sum, void *stream) {
    return rg::parts_entry<true>(y, inputs, segments, count, block_count, sum, rg::as_stream(stream));
}

extern "C" int rg_hip_where(void *out, const void *condition, const void *x, const void *y, const uint32_t *strides, size_t dims,
                            size_t outputs_count, size_t element_size, void *stream) {
    using namespace rg;
    if (!out || !condition || !x || !y || (dims && !strides)) return RG_HIP_E_ARGUMENT;
    if (dims > static_cast<size_t>(kMaxDims)) return RG_HIP_E_UNSUPPORTED;
    if (outputs_count == 0) return 0;
    if (outputs_count > 0xffffffffull) return RG_HIP_E_UNSUPPORTED;
    WherePlan p{};
    p.dims = static_cast<uint32_t>(dims);
    p.count = static_cast<uint32_t>(outputs_count);
    for (size_t d = 0; d < dims; ++d) {
        const uint32_t so = strides[4 * d + 3];
        if (so == 0) return RG_HIP_E_ARGUMENT;
        p.stride_o[d] = so;
        p.magic[d] = so <= 1 ? 0 : ~0ull / so + 1;
        for (int j = 0; j < 3; ++j) p.stride_in[d][j] = strides[4 * d + j];
    }
    hipStream_t s = as_stream(stream);
    switch (element_size) {
        case 1: return launch_where<uint8_t>(out, condition, x, y, p, s);
        case 2: return launch_where<uint16_t>(out, condition, x, y, p, s);
        case 4: return launch_where<uint32_t>(out, condition, x, y, p, s);
        case 8: return launch_where<uint64_t>(out, condition, x, y, p, s);
        default: return RG_HIP_E_UNSUPPORTED;
    }
}
