// Causal multi-head / grouped-query attention with a KV cache, for gfx950.
//
// The reference declares this kernel but never defines it
// (src/04kernel/src/kernels/attention/cuda_kernel.hh:10-25); tensor layouts and cache modes
// follow src/08-01llm/README.md:29-63:
//   q, o [N, H, seq, D]; k, v [N, Hkv, seq, D]; caches [N, Hkv, cap, D]; head h uses kv head
//   h / (H / Hkv); query row r of batch row b (absolute position past_b + r) attends cache
//   positions 0 .. past_b + r; the new k/v rows are appended at past_b .. past_b + seq - 1.
//
// Split-KV kernel (all shapes; the decode path).  HBM-bound: every K and V byte is read once
// per kv head and shared by the G query heads of its group.  The key space of all
// (batch row, query row, kv head) segments is laid end to end and cut into equal ranges, one
// per resident workgroup, so ragged per-row history lengths cannot unbalance the CUs.  A range
// is walked 16 keys per step: each lane owns a 16-byte slice of one key row, so a wavefront
// load is 1 KiB contiguous.  QK^T uses packed-half dot products followed by a DPP reduction
// over the 16 lanes of a key row, which leaves every lane holding the scores it needs for the
// PV update of its own slice of the head dimension; softmax is the online (running max / sum)
// form in float.  A segment that ends up in more than one range leaves (max, sum, unnormalised
// O) partials; the workgroup that finishes such a segment last (a ticket counter per segment)
// merges them, so one launch does everything.
#include "attention_prefill.hpp"
#include "common.hpp"

#include <mutex>

namespace rg {
namespace {

constexpr int kMaxBatch = 1024;     // rows of the batch whose lengths a workgroup scans
constexpr float kMinusBig = -1e30f; // running-max sentinel (finite: keeps exp2 arguments defined)
constexpr float kSlack = 6.0f;      // log2 headroom of the softmax reference before it is raised

struct AttnParams {
    const void *q, *k, *v;
    void *o, *kc, *vc;
    const int64_t *past;
    int past_per_row;
    uint32_t N, H, Hkv, seq, cap;
    uint32_t group;      // H / Hkv
    uint32_t head0;      // first query head (within each kv group) handled by this launch
    int append;          // write the new k/v rows into the caches
    float scale_log2e;   // scale * log2(e)
    float *part;         // partial slots: 2 per workgroup, each G*(D+2) floats
    uint32_t *counters;  // one ticket counter per workgroup, zero between launches
    uint32_t n_workgroups;
};

// ---------------------------------------------------------------- key-space partition
// Batch row b contributes seq query rows; query row r has L = base_b + r + 1 keys for each of
// the Hkv kv heads.  Order: b, then r, then kv head, then key position.

struct Partition {
    uint64_t *prefix;   // [N + 1] keys before batch row b
    uint32_t *base;     // [N] clamped history length of batch row b
};

// Every segment is laid out with kPiecePad positions that hold no key in front of its keys.  A
// range of the laid-out space is a share of the work, and starting a segment costs a workgroup
// about as much as streaming that many keys (query rows, a state to merge, a partial to write).
constexpr uint32_t kPiecePad = 128;

__device__ __forceinline__ uint64_t keys_before_row(uint32_t Hkv, uint32_t base, uint32_t r) {
    // Hkv * sum_{i<r} (base + i + 1 + kPiecePad)
    return static_cast<uint64_t>(Hkv) *
           (static_cast<uint64_t>(r) * (base + 1 + kPiecePad) + static_cast<uint64_t>(r) * (r - 1) / 2);
}

// Fills `part` (shared memory) and returns the total key count.  Called by every thread.
__device__ uint64_t build_partition(const AttnParams &p, Partition part) {
    const uint32_t t = threadIdx.x;
    // clamp so that the seq new rows always fit the cache; no cache: no history
    for (uint32_t b = t; b < p.N; b += blockDim.x) {
        int64_t raw = 0;
        if (p.kc && p.past) raw = p.past[p.past_per_row ? b : 0];
        if (raw < 0) raw = 0;
        const int64_t room = static_cast<int64_t>(p.cap) - static_cast<int64_t>(p.seq);
        if (p.kc && raw > room) raw = room < 0 ? 0 : room;
        part.base[b] = static_cast<uint32_t>(raw);
    }
    __syncthreads();
    // exclusive scan of per-batch-row key counts by the first wavefront: each lane sums a
    // contiguous run of rows, the lane totals are scanned with shuffles
    if (t < kWave) {
        const uint32_t per_lane = (p.N + kWave - 1) / kWave;
        const uint32_t b0 = t * per_lane;
        uint64_t mine = 0;
        for (uint32_t i = 0; i < per_lane; ++i)
            if (b0 + i < p.N) mine += keys_before_row(p.Hkv, part.base[b0 + i], p.seq);
        uint64_t incl = mine;
#pragma unroll
        for (int d = 1; d < kWave; d <<= 1) {
            const uint64_t up = __shfl_up(incl, d, kWave);
            if (t >= static_cast<uint32_t>(d)) incl += up;
        }
        uint64_t run = incl - mine;
        for (uint32_t i = 0; i < per_lane; ++i)
            if (b0 + i < p.N) {
                part.prefix[b0 + i] = run;
                run += keys_before_row(p.Hkv, part.base[b0 + i], p.seq);
            }
        if (t == kWave - 1) part.prefix[p.N] = incl;
    }
    __syncthreads();
    return part.prefix[p.N];
}

// Quotient of key counts; almost always both fit 32 bits, where the division is several times
// cheaper than the emulated 64-bit one.
__device__ __forceinline__ uint64_t udiv(uint64_t a, uint64_t b) {
    if (((a | b) >> 32) == 0) return static_cast<uint32_t>(a) / static_cast<uint32_t>(b);
    return a / b;
}

// The same partition for at most 64 batch rows, built by one wavefront without barriers: a later
// read of `part` or `*total_out` by this wavefront sees the values (shared memory accesses of a
// wavefront complete in program order); other wavefronts need a barrier first.
__device__ void build_partition_wave(const AttnParams &p, Partition part, uint32_t lane, uint64_t *total_out) {
    uint32_t base = 0;
    uint64_t mine = 0;
    if (lane < p.N) {
        int64_t raw = 0;
        if (p.kc && p.past) raw = p.past[p.past_per_row ? lane : 0];
        if (raw < 0) raw = 0;
        const int64_t room = static_cast<int64_t>(p.cap) - static_cast<int64_t>(p.seq);
        if (p.kc && raw > room) raw = room < 0 ? 0 : room;
        base = static_cast<uint32_t>(raw);
        mine = keys_before_row(p.Hkv, base, p.seq);
    }
    uint64_t incl = mine;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        const uint64_t up = __shfl_up(incl, d, kWave);
        if (lane >= static_cast<uint32_t>(d)) incl += up;
    }
    if (lane < p.N) {
        part.base[lane] = base;
        part.prefix[lane] = incl - mine;
    }
    if (lane == kWave - 1) {
        part.prefix[p.N] = incl;
        *total_out = incl;
    }
}

struct Segment {
    uint32_t b, r, kvh;
    uint32_t base;       // history length of batch row b
    uint32_t len;        // keys of this segment = base + r + 1
    uint64_t start;      // position of the segment (its padding first) in the laid-out space
};

// Segment containing laid-out key f.
__device__ Segment locate(const AttnParams &p, const Partition &part, uint64_t f) {
    uint32_t lo = 0, hi = p.N;  // largest b with prefix[b] <= f
    while (hi - lo > 1) {
        const uint32_t mid = (lo + hi) / 2;
        if (part.prefix[mid] <= f) lo = mid;
        else hi = mid;
    }
    Segment s;
    s.b = lo;
    s.base = part.base[lo];
    const uint64_t u = f - part.prefix[lo];
    // largest r with keys_before_row(r) <= u
    uint32_t rlo = 0, rhi = p.seq;
    while (rhi - rlo > 1) {
        const uint32_t mid = (rlo + rhi) / 2;
        if (keys_before_row(p.Hkv, s.base, mid) <= u) rlo = mid;
        else rhi = mid;
    }
    s.r = rlo;
    s.len = s.base + s.r + 1;
    const uint32_t span = s.len + kPiecePad;
    const uint64_t u2 = u - keys_before_row(p.Hkv, s.base, s.r);
    s.kvh = static_cast<uint32_t>(udiv(u2, span));
    s.start = part.prefix[lo] + keys_before_row(p.Hkv, s.base, s.r) + static_cast<uint64_t>(s.kvh) * span;
    return s;
}

__device__ __forceinline__ uint64_t range_width(uint64_t total, uint32_t n_workgroups) {
    uint64_t w = udiv(total + n_workgroups - 1, n_workgroups);
    w = (w + 15) / 16 * 16;
    return w < 64 ? 64 : w;
}

// ---------------------------------------------------------------- element helpers

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf2_t __attribute__((ext_vector_type(2)));

struct alignas(16) Raw16 {
    uint32_t w[4];
};

template <class T> struct Elem;
template <> struct Elem<__half> {
    static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, a), __builtin_bit_cast(half2_t, b), c, false);
    }
    static __device__ __forceinline__ float lo(uint32_t w) {
        return static_cast<float>(__builtin_bit_cast(half2_t, w)[0]);
    }
    static __device__ __forceinline__ float hi(uint32_t w) {
        return static_cast<float>(__builtin_bit_cast(half2_t, w)[1]);
    }
    static __device__ __forceinline__ uint16_t pack(float f) {
        return __builtin_bit_cast(uint16_t, static_cast<_Float16>(f));
    }
};
template <> struct Elem<__hip_bfloat16> {
    static __device__ __forceinline__ float lo(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
    static __device__ __forceinline__ float hi(uint32_t w) { return __builtin_bit_cast(float, w & 0xffff0000u); }
    static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
        return fmaf(hi(a), hi(b), fmaf(lo(a), lo(b), c));
    }
    static __device__ __forceinline__ uint16_t pack(float f) {
        return __builtin_bit_cast(uint16_t, __float2bfloat16(f));
    }
};

// 16-byte streaming load from global memory (the address space is stated so that a pointer
// chosen at run time between two buffers does not fall back to generic addressing)
typedef const u32x4 __attribute__((address_space(1))) *GlobalVec16;
__device__ __forceinline__ Raw16 load_stream_global(const void *p) {
    return __builtin_bit_cast(Raw16, __builtin_nontemporal_load((GlobalVec16)p));
}

// reduction over the LPR (8 or 16) lanes that share a key row
template <int LPR>
__device__ __forceinline__ float row_sum(float v) {
    v += dpp_f32<0xB1>(v);
    v += dpp_f32<0x4E>(v);
    v += dpp_f32<0x141>(v);
    if constexpr (LPR == 16) v += dpp_f32<0x140>(v);
    return v;
}

// Device-scope (all XCDs) visible accesses for the split-KV partials: the store is written
// through, the load does not hit a stale line of another XCD's L2.
__device__ __forceinline__ void store_coherent(float *p, float v) {
    __hip_atomic_store(reinterpret_cast<uint32_t *>(p), __builtin_bit_cast(uint32_t, v), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void store_coherent2(float *p, float a, float b) {  // p 8-byte aligned
    const uint64_t v = (static_cast<uint64_t>(__builtin_bit_cast(uint32_t, b)) << 32) | __builtin_bit_cast(uint32_t, a);
    __hip_atomic_store(reinterpret_cast<uint64_t *>(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_coherent(const float *p) {
    return __builtin_bit_cast(float, __hip_atomic_load(reinterpret_cast<const uint32_t *>(p), __ATOMIC_RELAXED,
                                                       __HIP_MEMORY_SCOPE_AGENT));
}

// ---------------------------------------------------------------- split kernel

// Merge of the partials of one cut segment (pieces held by workgroups first..last), one
// (head, d) output per thread iteration.  Loads of a batch of partials are independent.
template <class T, int D, int G>
__device__ void merge_segment(const AttnParams &p, const Segment &sg, uint64_t W, uint64_t first,
                              uint64_t last) {
    T *O = static_cast<T *>(p.o);
    constexpr int B = 8;
    for (uint32_t idx = threadIdx.x; idx < G * D; idx += blockDim.x) {
        const uint32_t g = idx / D, d = idx % D;
        float M = kMinusBig, o_sum = 0.f, l_sum = 0.f;
        for (uint64_t w0 = first; w0 <= last; w0 += B) {
            float pm[B], po[B], pl[B];
#pragma unroll
            for (int j = 0; j < B; ++j) {
                const uint64_t w = w0 + j;
                pm[j] = kMinusBig;
                po[j] = 0.f;
                pl[j] = 0.f;
                if (w <= last) {
                    const uint64_t piece_start = sg.start > w * W ? sg.start : w * W;
                    const uint64_t slot = w * 2 + (piece_start == w * W ? 0 : 1);
                    const float *ps = p.part + slot * (G * (D + 2)) + g * (D + 2);
                    pm[j] = load_coherent(ps + D);
                    po[j] = load_coherent(ps + d);
                    pl[j] = load_coherent(ps + D + 1);
                }
            }
            float mn = M;
#pragma unroll
            for (int j = 0; j < B; ++j) mn = fmaxf(mn, pm[j]);
            const float alpha = __builtin_amdgcn_exp2f(M - mn);
            o_sum *= alpha;
            l_sum *= alpha;
            M = mn;
#pragma unroll
            for (int j = 0; j < B; ++j) {
                const float wgt = __builtin_amdgcn_exp2f(pm[j] - mn);
                o_sum = fmaf(wgt, po[j], o_sum);
                l_sum = fmaf(wgt, pl[j], l_sum);
            }
        }
        const uint32_t h = sg.kvh * p.group + p.head0 + g;
        T *dst = O + ((static_cast<uint64_t>(sg.b) * p.H + h) * p.seq + sg.r) * D + d;
        *reinterpret_cast<uint16_t *>(dst) = Elem<T>::pack(o_sum / l_sum);
    }
}

// Sums (or maxima) over the four 16-lane groups of a wavefront with lane swaps.  The two
// results of a swap are copied into scalars before they are reinterpreted as floats.
struct SwapPair {
    float a, b;
};
__device__ __forceinline__ SwapPair swap32(float x, float y) {
    const auto r = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(uint32_t, x), __builtin_bit_cast(uint32_t, y),
                                                    false, false);
    const uint32_t r0 = r[0], r1 = r[1];
    return {__builtin_bit_cast(float, r0), __builtin_bit_cast(float, r1)};
}
__device__ __forceinline__ SwapPair swap16(float x, float y) {
    const auto r = __builtin_amdgcn_permlane16_swap(__builtin_bit_cast(uint32_t, x), __builtin_bit_cast(uint32_t, y),
                                                    false, false);
    const uint32_t r0 = r[0], r1 = r[1];
    return {__builtin_bit_cast(float, r0), __builtin_bit_cast(float, r1)};
}
__device__ __forceinline__ float swap32_sum(float lo_keeps, float hi_keeps) {
    // lanes 0-31 receive lo_keeps summed over both halves, lanes 32-63 hi_keeps
    const SwapPair r = swap32(lo_keeps, hi_keeps);
    return r.a + r.b;
}
__device__ __forceinline__ float swap16_sum(float even_keeps, float odd_keeps) {
    // even 16-lane groups receive even_keeps summed over the group pair, odd ones odd_keeps
    const SwapPair r = swap16(even_keeps, odd_keeps);
    return r.a + r.b;
}
__device__ __forceinline__ float swap_sum(float v) {
    const float h = swap32_sum(v, v);
    return swap16_sum(h, h);
}
__device__ __forceinline__ float swap_max(float v) {
    const SwapPair r = swap32(v, v);
    const float h = fmaxf(r.a, r.b);
    const SwapPair q = swap16(h, h);
    return fmaxf(q.a, q.b);
}

constexpr int kSplitThreads = 512;                   // one workgroup per CU at two wavefronts per SIMD
constexpr int kSplitWaves = kSplitThreads / kWave;
constexpr int kMaxPieces = 4;                        // pieces of a range handled per pass

// One piece = the part of a segment that falls into a workgroup's range.
struct PieceRec {
    uint64_t start;      // position of key 0 of the segment in the laid-out space
    uint64_t hist_row0;  // cache row of key 0 of the kv head
    int64_t new_row0;    // input row that key 0 would have (key `base` is the first real one)
    uint32_t b, r, kvh, base, len;  // the segment
    uint32_t pos0, end;  // keys [pos0, end) of the segment
    uint32_t blk0;       // first block of the piece within the pass
    uint32_t flags;      // 1: the whole segment, 2: appends the new rows, 4: begins where the range does
    uint32_t pad;
};

__device__ __forceinline__ uint32_t uni(uint32_t v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ uint64_t uni(uint64_t v) {
    return (static_cast<uint64_t>(uni(static_cast<uint32_t>(v >> 32))) << 32) | uni(static_cast<uint32_t>(v));
}

// What a wavefront needs of a piece to load and consume its blocks (wave-uniform registers).
struct PieceView {
    uint64_t hist_row0;
    int64_t new_row0;
    uint32_t base, pos0, end, blk0, flags;
};

template <class T, int D, int G>
__global__ __launch_bounds__(kSplitThreads) void attn_split(const AttnParams p) {
    constexpr int LPR = D / 8;          // lanes per key row
    constexpr int KPW = kWave / LPR;    // key rows per wavefront load
    constexpr int U = 4;                // loads per register set
    constexpr uint32_t BK = KPW * U;    // keys per block: the unit a wavefront pulls
    constexpr int NSET = 1;             // blocks a wavefront keeps in flight (more did not pay: the
                                        // other wavefront of the SIMD covers the wait)
    constexpr int NW = kSplitWaves;

    __shared__ uint64_t sh_prefix[kMaxBatch + 1];
    __shared__ uint32_t sh_base[kMaxBatch];
    __shared__ PieceRec sh_pc[kMaxPieces];
    __shared__ uint64_t sh_f;
    __shared__ uint32_t sh_np, sh_nblk;
    __shared__ unsigned long long sh_taken;  // blocks handed out: from the front (low word), from the back (high word)
    __shared__ uint32_t sh_has[kMaxPieces];  // wavefronts that hold a state of the piece (bit mask)
    __shared__ uint32_t sh_last[kMaxPieces];
    __shared__ alignas(16) uint32_t sh_q[kMaxPieces][G][D / 2];
    __shared__ alignas(16) float sh_o[kMaxPieces][NW][G][D];
    __shared__ alignas(16) float sh_m[kMaxPieces][G][NW];
    __shared__ alignas(16) float sh_l[kMaxPieces][G][NW];

    __shared__ uint64_t sh_total;

    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const Partition part{sh_prefix, sh_base};
    if (p.N <= kWave) {
        if (wave == 0) build_partition_wave(p, part, lane, &sh_total);
    } else {
        const uint64_t t = build_partition(p, part);
        if (threadIdx.x == 0) sh_total = t;
    }
    const uint32_t row = lane / LPR, chunk = lane % LPR;  // key row within a wavefront load, 16-byte slice
    const T *Q = static_cast<const T *>(p.q);
    const T *Kn = static_cast<const T *>(p.k);
    const T *Vn = static_cast<const T *>(p.v);
    T *Kc = static_cast<T *>(p.kc);
    T *Vc = static_cast<T *>(p.vc);
    T *O = static_cast<T *>(p.o);

    uint32_t qv[G][4];  // this lane's slice of the G query rows
    float m[G], l[G], acc[G][8];
    bool empty = true;  // this lane's key rows have not held a valid key yet

    // Online-softmax update with one block; keys >= the end of the piece are masked out.  The
    // running reference m[g] is only moved (and the accumulators rescaled) when some score
    // exceeds it by more than kSlack or a lane meets its first valid key, a rare event after the
    // first block; otherwise p = exp2(s - m) <= 2^kSlack is accumulated directly.  A lane that
    // has seen no valid key keeps m = 0 with empty accumulators.
    auto consume = [&](const PieceView &pc, uint32_t key0, const Raw16(&kk)[U], const Raw16(&vv)[U]) {
        const uint32_t limit = pc.end;
        // the segment of the last query row writes the new rows it reads into the caches
        if ((pc.flags & 2) && key0 + BK > pc.base) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const uint32_t key = key0 + u * KPW + row;
                if (key >= pc.base && key < limit) {
                    const uint64_t coff = (pc.hist_row0 + key) * D + chunk * 8;
                    *reinterpret_cast<Raw16 *>(Kc + coff) = kk[u];
                    *reinterpret_cast<Raw16 *>(Vc + coff) = vv[u];
                }
            }
        }
        float t[U][G];  // score - reference, log2 units
        float over = -__builtin_inff();
        const bool valid0 = key0 + row < limit;  // keys ascend with u
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const bool valid = key0 + u * KPW + row < limit;
#pragma unroll
            for (int g = 0; g < G; ++g) {
                float d = 0.f;
#pragma unroll
                for (int e = 0; e < 4; ++e) d = Elem<T>::dot2(qv[g][e], kk[u].w[e], d);
                d = fmaf(row_sum<LPR>(d), p.scale_log2e, -m[g]);
                t[u][g] = valid ? d : -__builtin_inff();
                over = fmaxf(over, t[u][g]);
            }
        }
        if (__builtin_amdgcn_ballot_w64(over > kSlack || (empty && valid0)) != 0) {
#pragma unroll
            for (int g = 0; g < G; ++g) {
                // how far the reference moves: to the block maximum at the lane's first valid
                // key (the accumulators are still empty), never down afterwards
                float up = t[0][g];
#pragma unroll
                for (int u = 1; u < U; ++u) up = fmaxf(up, t[u][g]);
                up = empty ? (valid0 ? up : 0.f) : fmaxf(up, 0.f);
                const float alpha = empty ? 1.f : __builtin_amdgcn_exp2f(-up);
                m[g] += up;
                l[g] *= alpha;
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[g][e] *= alpha;
#pragma unroll
                for (int u = 0; u < U; ++u) t[u][g] -= up;
            }
            empty = empty && !valid0;
        }
#pragma unroll
        for (int g = 0; g < G; ++g) {
            float pr[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                pr[u] = __builtin_amdgcn_exp2f(t[u][g]);
                l[g] += pr[u];
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float a0 = acc[g][2 * e], a1 = acc[g][2 * e + 1];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    a0 = fmaf(pr[u], Elem<T>::lo(vv[u].w[e]), a0);
                    a1 = fmaf(pr[u], Elem<T>::hi(vv[u].w[e]), a1);
                }
                acc[g][2 * e] = a0;
                acc[g][2 * e + 1] = a1;
            }
        }
    };

    // Leaves this wavefront's state of piece j in shared memory.  The key rows of the wavefront
    // are summed with lane swaps that halve the number of values per step (a lane group keeps
    // the sums it will store and hands the rest over), ending with two output columns per lane.
    auto flush = [&](uint32_t j) {
        const uint32_t quarter = lane >> 4;  // 16-lane group
#pragma unroll
        for (int g = 0; g < G; ++g) {
            float mg = empty ? kMinusBig : m[g];  // lanes without a valid key drop out of the maxima
            float M = mg;
            if constexpr (LPR == 8) M = fmaxf(M, dpp_f32<0x128>(M));
            M = swap_max(M);
            const float w = __builtin_amdgcn_exp2f(mg - M);
            float lv = l[g] * w;
            if constexpr (LPR == 8) lv += dpp_f32<0x128>(lv);
            lv = swap_sum(lv);
            float a[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                a[e] = acc[g][e] * w;
                if constexpr (LPR == 8) a[e] += dpp_f32<0x128>(a[e]);
            }
            float s4[4], s2[2];
#pragma unroll
            for (int e = 0; e < 4; ++e) s4[e] = swap32_sum(a[e], a[e + 4]);  // lanes 32-63 keep columns 4-7
#pragma unroll
            for (int e = 0; e < 2; ++e) s2[e] = swap16_sum(s4[e], s4[e + 2]);  // odd 16-lane groups keep +2
            // this lane now holds columns chunk*8 + 2*quarter + {0, 1} of the wavefront's sum
            if (LPR == 16 || (lane & 8) == 0) {
                float *dst = &sh_o[j][wave][g][(lane & (LPR - 1)) * 8 + 2 * quarter];
                dst[0] = s2[0];
                dst[1] = s2[1];
            }
            if (lane == 0) {
                sh_m[j][g][wave] = M;
                sh_l[j][g][wave] = lv;
            }
        }
        if (lane == 0) atomicOr(&sh_has[j], 1u << wave);
    };

    // ---- one thread lays out the next pieces of the range and numbers their blocks
    Segment sg{};  // walked by thread 0 only
    auto build_tables = [&](uint64_t pass_begin, uint64_t range_begin, uint64_t range_end) {
        uint64_t f = pass_begin;
        uint32_t np = 0, nblk = 0;
        while (np < kMaxPieces && f < range_end) {
            if (f == range_begin) {
                sg = locate(p, part, f);
            } else {  // the previous piece ended with its segment: step to the next one
                sg.start += sg.len + kPiecePad;
                if (++sg.kvh == p.Hkv) {
                    sg.kvh = 0;
                    if (++sg.r == p.seq) {
                        sg.r = 0;
                        sg.base = sh_base[++sg.b];
                    }
                    sg.len = sg.base + sg.r + 1;
                }
            }
            // positions [at, at + width) of the padded segment are in the range; the keys among them
            const uint32_t at = static_cast<uint32_t>(f - sg.start);
            const uint64_t left = range_end - f;
            const uint32_t span = sg.len + kPiecePad;
            const uint32_t width = static_cast<uint32_t>(left < span - at ? left : span - at);
            const uint32_t pos0 = at > kPiecePad ? at - kPiecePad : 0;
            const uint32_t end = at + width > kPiecePad ? at + width - kPiecePad : 0;
            f += width;
            if (end <= pos0) continue;  // padding only
            PieceRec rc;
            rc.start = sg.start + kPiecePad;
            rc.b = sg.b; rc.r = sg.r; rc.kvh = sg.kvh; rc.base = sg.base; rc.len = sg.len;
            rc.pos0 = pos0;
            rc.end = end;
            const uint64_t kv_head = static_cast<uint64_t>(sg.b) * p.Hkv + sg.kvh;
            rc.hist_row0 = kv_head * p.cap;
            rc.new_row0 = static_cast<int64_t>(kv_head * p.seq) - static_cast<int64_t>(sg.base);
            rc.blk0 = nblk;
            rc.flags = ((pos0 == 0 && end == sg.len) ? 1u : 0u) |
                       ((p.append && Kc && sg.r + 1 == p.seq) ? 2u : 0u) |
                       (rc.start + pos0 == range_begin ? 4u : 0u);
            rc.pad = 0;
            sh_pc[np] = rc;
            nblk += (end - pos0 + BK - 1) / BK;
            ++np;
        }
        sh_np = np;
        sh_nblk = nblk;
        sh_taken = 0;
        sh_f = f;
    };
    // The thread that builds the first tables belongs to the wavefront that built the partition
    // (or comes after the barriers of the many-row path), so one barrier covers both.
    if (threadIdx.x == 0) {
        const uint64_t total0 = sh_total;
        const uint64_t W0 = range_width(total0, p.n_workgroups);
        const uint64_t begin0 = static_cast<uint64_t>(blockIdx.x) * W0;
        if (begin0 < total0) build_tables(begin0, begin0, begin0 + W0 < total0 ? begin0 + W0 : total0);
    }
    if (threadIdx.x < kMaxPieces) sh_has[threadIdx.x] = 0;
    __syncthreads();
    const uint64_t total = uni(sh_total);
    const uint64_t W = range_width(total, p.n_workgroups);
    const uint64_t range_begin = static_cast<uint64_t>(blockIdx.x) * W;
    if (range_begin >= total) return;
    const uint64_t range_end = range_begin + W < total ? range_begin + W : total;

    for (;;) {
        const uint32_t np = uni(sh_np), nblk = uni(sh_nblk);
        const uint64_t next_begin = uni(sh_f);
        // a range that only holds padding has nothing to stream
        if (np > 0) [&]() {
        const uint32_t c1 = np > 1 ? uni(sh_pc[1].blk0) : 0xffffffffu;
        const uint32_t c2 = np > 2 ? uni(sh_pc[2].blk0) : 0xffffffffu;
        const uint32_t c3 = np > 3 ? uni(sh_pc[3].blk0) : 0xffffffffu;
        auto piece_of = [&](uint32_t blk) -> uint32_t { return (blk >= c1) + (blk >= c2) + (blk >= c3); };
        auto view = [&](uint32_t j) {
            PieceView v;
            const PieceRec &rc = sh_pc[j];
            v.hist_row0 = uni(rc.hist_row0);
            v.new_row0 = static_cast<int64_t>(uni(static_cast<uint64_t>(rc.new_row0)));
            v.base = uni(rc.base);
            v.pos0 = uni(rc.pos0);
            v.end = uni(rc.end);
            v.blk0 = uni(rc.blk0);
            v.flags = uni(rc.flags);
            return v;
        };
        // Blocks are handed out through a shared counter, so a wavefront that is served faster
        // simply takes more of them.  Half of the wavefronts take blocks from the front of the
        // list, the others from its back: most of them then stay inside one piece and never
        // have to set a state aside to start another.
        constexpr uint32_t kNoBlock = 0xffffffffu;
        auto grab = [&]() -> uint32_t {
            const bool from_back = wave >= NW / 2;
            unsigned long long old = 0;
            if (lane == 0) old = atomicAdd(&sh_taken, from_back ? (1ull << 32) : 1ull);
            const uint32_t front = uni(static_cast<uint32_t>(old)), back = uni(static_cast<uint32_t>(old >> 32));
            if (front + back >= nblk) return kNoBlock;
            return from_back ? nblk - 1 - back : front;
        };

        // Loads one block: keys below the history length come from the caches, later ones from
        // the k/v inputs.  Unconditional (a block beyond the last re-reads the last one and is
        // never consumed), clamped to the last key of the piece, streaming.
        PieceView iss{};
        uint32_t iss_j = 0xffffffffu;
        auto issue = [&](uint32_t blk, Raw16(&kk)[U], Raw16(&vv)[U]) {
            blk = blk < nblk ? blk : nblk - 1;
            const uint32_t j = piece_of(blk);
            if (j != iss_j) {
                iss = view(j);
                iss_j = j;
            }
            const uint32_t key0 = iss.pos0 + (blk - iss.blk0) * BK;
            if (key0 + BK <= iss.base) {  // history only (wave-uniform): one base address
                const T *kb = Kc + iss.hist_row0 * D + chunk * 8;
                const T *vb = Vc + iss.hist_row0 * D + chunk * 8;
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    uint32_t key = key0 + u * KPW + row;
                    key = key < iss.end ? key : iss.end - 1;
                    const uint64_t off = static_cast<uint64_t>(key) * D;
                    kk[u] = load_stream_global(kb + off);
                    vv[u] = load_stream_global(vb + off);
                }
            } else {
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    uint32_t key = key0 + u * KPW + row;
                    key = key < iss.end ? key : iss.end - 1;
                    const bool hist = key < iss.base;
                    const int64_t krow = (hist ? static_cast<int64_t>(iss.hist_row0) : iss.new_row0) + key;
                    const int64_t off = krow * D + chunk * 8;
                    kk[u] = load_stream_global((hist ? Kc : Kn) + off);
                    vv[u] = load_stream_global((hist ? Vc : Vn) + off);
                }
            }
        };

        Raw16 kbuf[NSET][U], vbuf[NSET][U];
        uint32_t blk[NSET];
#pragma unroll
        for (int s = 0; s < NSET; ++s) {
            blk[s] = grab();
            issue(blk[s], kbuf[s], vbuf[s]);
        }
        // ---- the query rows of the pieces go to shared memory while the first blocks arrive
        for (uint32_t idx = threadIdx.x; idx < np * G * LPR; idx += kSplitThreads) {
            const uint32_t j = idx / (G * LPR), g = (idx / LPR) % G, c = idx % LPR;
            const PieceRec &rc = sh_pc[j];
            const uint32_t h = rc.kvh * p.group + p.head0 + g;
            const Raw16 raw = *reinterpret_cast<const Raw16 *>(
                Q + ((static_cast<uint64_t>(rc.b) * p.H + h) * p.seq + rc.r) * D + c * 8);
            *reinterpret_cast<Raw16 *>(&sh_q[j][g][c * 4]) = raw;
        }
        __syncthreads();

        // ---- each wavefront consumes the blocks it pulled
        PieceView cur{};
        uint32_t cur_j = 0xffffffffu;
        bool live = true;
        while (live) {
#pragma unroll
            for (int s = 0; s < NSET; ++s) {
                if (!live) break;
                if (blk[s] >= nblk) {
                    live = false;
                    break;
                }
                const uint32_t j = piece_of(blk[s]);
                if (j != cur_j) {
                    if (cur_j != 0xffffffffu) flush(cur_j);
                    cur = view(j);
                    cur_j = j;
#pragma unroll
                    for (int g = 0; g < G; ++g) {
                        const Raw16 raw = *reinterpret_cast<const Raw16 *>(&sh_q[j][g][chunk * 4]);
#pragma unroll
                        for (int e = 0; e < 4; ++e) qv[g][e] = raw.w[e];
                        m[g] = 0.f;
                        l[g] = 0.f;
#pragma unroll
                        for (int e = 0; e < 8; ++e) acc[g][e] = 0.f;
                    }
                    empty = true;
                }
                consume(cur, cur.pos0 + (blk[s] - cur.blk0) * BK, kbuf[s], vbuf[s]);
                blk[s] = grab();
                issue(blk[s], kbuf[s], vbuf[s]);
            }
        }
        if (cur_j != 0xffffffffu) flush(cur_j);
        __syncthreads();

        // ---- merge the wavefronts' states of all pieces at once, four output columns per
        // thread; whole segments give output rows, cut ones leave a partial
        bool any_cut = false;
        for (uint32_t j = 0; j < np; ++j) any_cut = any_cut || !(sh_pc[j].flags & 1);
        for (uint32_t idx = threadIdx.x; idx < np * G * (D / 4); idx += kSplitThreads) {
            const uint32_t j = idx / (G * (D / 4)), g = (idx / (D / 4)) % G, d = (idx % (D / 4)) * 4;
            const PieceRec &rc = sh_pc[j];
            const uint32_t has = sh_has[j];
            float mw[NW], lw[NW];
#pragma unroll
            for (int w4 = 0; w4 < NW; w4 += 4) {
                const f32x4 mv = *reinterpret_cast<const f32x4 *>(&sh_m[j][g][w4]);
                const f32x4 lv = *reinterpret_cast<const f32x4 *>(&sh_l[j][g][w4]);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const bool on = (has >> (w4 + i)) & 1;
                    mw[w4 + i] = on ? mv[i] : kMinusBig;
                    lw[w4 + i] = on ? lv[i] : 0.f;
                }
            }
            float M = kMinusBig;
#pragma unroll
            for (int w = 0; w < NW; ++w) M = fmaxf(M, mw[w]);
            float o_sum[4] = {0.f, 0.f, 0.f, 0.f}, l_sum = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w) {
                const bool on = (has >> w) & 1;
                const float wgt = on ? __builtin_amdgcn_exp2f(mw[w] - M) : 0.f;
                const f32x4 ov = *reinterpret_cast<const f32x4 *>(&sh_o[j][w][g][d]);
                l_sum = fmaf(wgt, lw[w], l_sum);
#pragma unroll
                for (int i = 0; i < 4; ++i) o_sum[i] = fmaf(wgt, on ? ov[i] : 0.f, o_sum[i]);
            }
            if (rc.flags & 1) {
                const uint32_t h = rc.kvh * p.group + p.head0 + g;
                T *dst = O + ((static_cast<uint64_t>(rc.b) * p.H + h) * p.seq + rc.r) * D + d;
                const float inv = 1.f / l_sum;
                const uint32_t lo = Elem<T>::pack(o_sum[0] * inv) | (static_cast<uint32_t>(Elem<T>::pack(o_sum[1] * inv)) << 16);
                const uint32_t hi = Elem<T>::pack(o_sum[2] * inv) | (static_cast<uint32_t>(Elem<T>::pack(o_sum[3] * inv)) << 16);
                *reinterpret_cast<uint2 *>(dst) = make_uint2(lo, hi);
            } else {
                const uint64_t slot = static_cast<uint64_t>(blockIdx.x) * 2 + ((rc.flags & 4) ? 0 : 1);
                float *ps = p.part + slot * (G * (D + 2)) + g * (D + 2);
                store_coherent2(ps + d, o_sum[0], o_sum[1]);
                store_coherent2(ps + d + 2, o_sum[2], o_sum[3]);
                if (d == 0) store_coherent2(ps + D, M, l_sum);
            }
        }
        if (any_cut) {
            // The workgroup that completes a cut segment last merges its partials.  Ordering of
            // the hand-off, writer side: the partials are device-scope write-through stores; every
            // wavefront waits until all of its vector-memory operations have been acknowledged
            // (vmcnt counts stores on this target and a write-through store is acknowledged once
            // it has left the XCD's L2), then the barrier collects the wavefronts, and only then
            // is the ticket taken.  Reader side: the ticket's value decides `sh_last`, which the
            // merging threads read after another barrier, so their device-scope loads (which
            // bypass the XCD-local L2) are issued after the ticket add has returned and therefore
            // after every other piece's stores were acknowledged.  A workgroup-scope fence alone
            // would not do: it emits no wait for outstanding stores.  No cache-wide write-back or
            // invalidate is needed (one per workgroup cost 3.5x).
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            if (threadIdx.x < kMaxPieces) {
                uint32_t is_last = 0;
                if (threadIdx.x < np && !(sh_pc[threadIdx.x].flags & 1)) {
                    const PieceRec &rc = sh_pc[threadIdx.x];
                    const uint64_t first = udiv(rc.start, W), last = udiv(rc.start + rc.len - 1, W);
                    const uint32_t ticket = __hip_atomic_fetch_add(p.counters + first, 1u, __ATOMIC_RELAXED,
                                                                   __HIP_MEMORY_SCOPE_AGENT);
                    is_last = ticket == static_cast<uint32_t>(last - first);
                    if (is_last) p.counters[first] = 0;  // leave the counters as they were found
                }
                sh_last[threadIdx.x] = is_last;
            }
            __syncthreads();
            for (uint32_t j = 0; j < np; ++j) {
                if (!sh_last[j]) continue;
                const PieceRec &rc = sh_pc[j];
                Segment sg;
                sg.b = rc.b; sg.r = rc.r; sg.kvh = rc.kvh; sg.base = rc.base; sg.len = rc.len; sg.start = rc.start;
                merge_segment<T, D, G>(p, sg, W, udiv(sg.start, W), udiv(sg.start + sg.len - 1, W));
            }
        }
        }();
        if (next_begin >= range_end) break;
        __syncthreads();  // the tables are rewritten for the next pass
        if (threadIdx.x == 0) build_tables(next_begin, range_begin, range_end);
        if (threadIdx.x < kMaxPieces) sh_has[threadIdx.x] = 0;
        __syncthreads();
    }
}

// Zeroes the ticket counters when the caller supplies no persistent (already zero) ones.
__global__ __launch_bounds__(256) void attn_clear(uint32_t *counters, uint32_t n) {
    for (uint32_t i = blockIdx.x * 256 + threadIdx.x; i < n; i += gridDim.x * 256) counters[i] = 0;
}

// ---------------------------------------------------------------- host side

struct DeviceInfo {
    int cus = 0;
};

const DeviceInfo &device_info() {
    static DeviceInfo info = [] {
        DeviceInfo d;
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess)
            d.cus = prop.multiProcessorCount;
        if (d.cus <= 0) d.cus = 256;
        return d;
    }();
    return info;
}

template <class T, int D, int G>
uint32_t resident_workgroups() {
    static uint32_t cached = [] {
        int per_cu = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, attn_split<T, D, G>, kSplitThreads, 0) != hipSuccess ||
            per_cu <= 0)
            per_cu = 1;
        return static_cast<uint32_t>(per_cu) * static_cast<uint32_t>(device_info().cus);
    }();
    return cached;
}

constexpr uint32_t kMaxWorkgroups = 4096;  // bound used by the workspace query
// Several query rows per batch row: the tiled kernel stages K/V once per 32 query rows x 4 heads, but an item walks
// all of its keys by itself, while the split kernel reads K/V once per query row and spreads the keys over every
// CU.  With the history length h: tiled about rounds * h * 0.020 us (rounds = items over the 512 workgroups that
// are resident), split about N * Hkv * seq * h * 512 B at 7 TB/s; h cancels.  Measured at N = 32, 8 kv heads,
// h = 4000: 4 rows 109 us tiled against 318 us split, 2 rows 108 against 159; at N = 1: 4 rows 84 against 20.
constexpr size_t kPrefillAlways = 32;  // query rows from which the tiled kernel is used whatever the batch

bool prefill_pays(size_t N, size_t n_head, size_t n_kv_head, size_t seq, size_t cap, size_t D, bool ranges_fit) {
    if (seq >= kPrefillAlways) return true;
    const size_t group = n_head / n_kv_head, heads_per_item = group == 1 ? 1 : group == 2 ? 2 : 4;
    // the split kernel takes eight, four, two or one heads of a group per launch and reads K/V again in every launch
    // (a group of 7: three times), while the chunks of a group on the tiled kernel find them in L2
    size_t split_launches = 0;
    for (size_t left = group; left > 0; left -= left >= 8 ? 8 : left >= 4 ? 4 : left >= 2 ? 2 : 1) ++split_launches;
    if (seq < 2 && split_launches < 2) return false;
    const size_t rows_per_item = 32 * (4 / heads_per_item);
    const size_t items = N * n_kv_head * ((group + heads_per_item - 1) / heads_per_item) * ((seq + rows_per_item - 1) / rows_per_item);
    // Few items: the tiled kernel shares an item's keys between workgroups (head dims 64 and 128, records in the
    // workspace), and then costs about 17.5 us + 9.4e-5 us per kv head and key, against 8 us + 7.3e-5 us per
    // kv head, key and query row on the split kernel (N = 1, 8 kv heads, 8 new rows: history 1000 13.9 us split
    // against 18.1 tiled, 4000 26.1 against 22.7, 32768 154 against 46).  The history is device data and the host
    // may not read it, so half of the capacity stands for it.  Both costs are linear in the history with the
    // tiled kernel's slope the smaller one, so the wrong choice costs most at the ends: with a history near
    // nothing where the rule chose tiled (about 10 us lost, the difference of the constant terms), with a full
    // cache where it chose split (the slopes' difference times the capacity).  Half the capacity makes these two
    // worst cases meet as closely as one fixed value can.
    if (ranges_fit && seq == 1 && split_launches >= 2 && (D == 64 || D == 128)) return true;  // (16 x 28/4 heads, history 4000: 80 -> 52 us)
    if (ranges_fit && seq >= 2 && items * 2 <= 512 && cap >= 1024 && (D == 64 || D == 128)) {
        const double keys = static_cast<double>(N * n_kv_head) * static_cast<double>(cap) / 2;
        return 9.5 < keys * (7.3e-5 * static_cast<double>(seq * split_launches) - 9.4e-5);
    }
    const size_t rounds = (items + 511) / 512;
    return N * n_kv_head * seq * split_launches >= 280 * rounds;
}

template <class T, int D, int G>
int launch(AttnParams p, hipStream_t s) {
    uint32_t wgs = resident_workgroups<T, D, G>();
    if (wgs > p.n_workgroups) wgs = p.n_workgroups;  // what the partial slots and counters are sized for
    p.n_workgroups = wgs;
    attn_split<T, D, G><<<wgs, kSplitThreads, 0, s>>>(p);
    return launch_status();
}

template <class T, int D>
int dispatch_group(AttnParams p, hipStream_t s) {
    // heads of a kv group are processed G at a time (G in {8, 4, 2, 1})
    uint32_t done = 0;
    while (done < p.group) {
        const uint32_t left = p.group - done;
        p.head0 = done;
        p.append = done == 0;
        int rc;
        if (left >= 8) {
            // eight heads read their K/V once instead of twice (64/8 heads, 64 sequences, history 4096: 337 -> 238 us)
            AttnParams p8 = p;
            p8.n_workgroups = p.n_workgroups / 2;  // (the partial slots are sized for groups of four)
            rc = launch<T, D, 8>(p8, s);
            done += 8;
        } else if (left >= 4) {
            rc = launch<T, D, 4>(p, s);
            done += 4;
        } else if (left >= 2) {
            rc = launch<T, D, 2>(p, s);
            done += 2;
        } else {
            rc = launch<T, D, 1>(p, s);
            done += 1;
        }
        if (rc) return rc;
    }
    return 0;
}

constexpr size_t kCounterBytes = kMaxWorkgroups * sizeof(uint32_t);

size_t workspace_bytes(size_t D) {
    // ticket counters (used when the caller passes no persistent ones), then two partial slots
    // per workgroup sized for the widest head group (4)
    // (the tiled kernel's records of key ranges use the same area, never in the same call)
    const size_t split = static_cast<size_t>(kMaxWorkgroups) * 2 * 4 * (D + 2) * sizeof(float);
    const size_t tiled = prefill_part_bytes(static_cast<uint32_t>(D));
    return kCounterBytes + (split > tiled ? split : tiled);
}

// ---------------------------------------------------------------- library-owned scratch
// Split-KV partials and ticket counters for callers that may not allocate: a fixed array in
// device memory, one copy per GPU the library is loaded on.  In host code the array's name is
// only a handle for hipGetSymbolAddress; the address it returns for the current device is what
// kernels and fill launches are given.
constexpr uint32_t kStaticWorkgroups = 512;                      // the launch is capped at this many
constexpr size_t kStaticCounterBytes = kStaticWorkgroups * sizeof(uint32_t);
constexpr size_t kStaticPartBytes = static_cast<size_t>(kStaticWorkgroups) * 2 * 4 * (128 + 2) * sizeof(float);
constexpr size_t kStaticBytes = kStaticCounterBytes + kStaticPartBytes;  // 2 KiB + 2.03 MiB

__device__ __align__(256) unsigned char scratch[kStaticBytes];

constexpr int kMaxDevices = 64;
std::mutex scratch_mutex;
void *scratch_of_device[kMaxDevices] = {};

// Address of the current device's copy of `scratch` (looked up once per device).
int static_scratch(void **out) {
    int dev = -1;
    const hipError_t rc = hipGetDevice(&dev);
    if (rc != hipSuccess) return static_cast<int>(rc);
    if (dev < 0 || dev >= kMaxDevices) return RG_HIP_E_UNSUPPORTED;
    std::lock_guard<std::mutex> lock(scratch_mutex);
    if (!scratch_of_device[dev]) {
        void *ptr = nullptr;
        const hipError_t rs = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (rs != hipSuccess) return static_cast<int>(rs);
        if (!ptr) return RG_HIP_E_WORKSPACE;
        scratch_of_device[dev] = ptr;
    }
    *out = scratch_of_device[dev];
    return 0;
}

// Argument checks and dispatch shared by the entry points.  `part` holds two partial slots per
// workgroup for at most `max_workgroups` workgroups; `counters` one ticket counter per workgroup,
// zero on entry unless `clear_counters` asks for the clearing launch.
int attention_call(void *o, const void *q, const void *k, const void *v, void *k_cache, void *v_cache,
                   const int64_t *past_lens, int past_per_row, size_t N, size_t n_head, size_t n_kv_head,
                   size_t seq, size_t cap, size_t D, float scale, int dtype, float *part, size_t part_bytes,
                   uint32_t *counters, uint32_t max_workgroups, bool clear_counters, hipStream_t s) {
    if (!o || !q || !k || !v) return RG_HIP_E_ARGUMENT;
    if ((k_cache == nullptr) != (v_cache == nullptr)) return RG_HIP_E_ARGUMENT;
    if (N == 0 || n_head == 0 || seq == 0) return 0;
    if (n_kv_head == 0 || n_head % n_kv_head != 0) return RG_HIP_E_ARGUMENT;
    // head dims 64 and 128 have both kernels; 80 and 96 the tiled one only (the split kernel gives 8 or 16 lanes to a row)
    const bool split_ok = D == 64 || D == 128;
    if (!split_ok && D != 80 && D != 96) return RG_HIP_E_UNSUPPORTED;
    if (dtype != RG_FP16 && dtype != RG_BF16) return RG_HIP_E_UNSUPPORTED;
    if (N > kMaxBatch || seq > 0xffffu || cap > 0x3fffffffu || n_head > 0xffffu) return RG_HIP_E_UNSUPPORTED;
    if (k_cache && cap < seq) return RG_HIP_E_ARGUMENT;
    if (N * seq * n_kv_head > 0x7fffffffu) return RG_HIP_E_UNSUPPORTED;
    if (!part || !counters) return RG_HIP_E_WORKSPACE;
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o) ||
        (k_cache && (!aligned16(k_cache) || !aligned16(v_cache))))
        return RG_HIP_E_ARGUMENT;

    // many query rows per batch row: the tiled MFMA kernel (K/V staged once per query tile)
    if (prefill_supported(static_cast<uint32_t>(n_head), static_cast<uint32_t>(n_kv_head), static_cast<uint32_t>(D)) &&
        (!split_ok || prefill_pays(N, n_head, n_kv_head, seq, cap, D, part_bytes >= prefill_part_bytes(static_cast<uint32_t>(D))))) {
        PrefillArgs a{};
        a.q = q; a.k = k; a.v = v; a.o = o; a.kc = k_cache; a.vc = v_cache;
        a.past = past_lens;
        a.past_per_row = past_per_row;
        a.N = static_cast<uint32_t>(N);
        a.H = static_cast<uint32_t>(n_head);
        a.Hkv = static_cast<uint32_t>(n_kv_head);
        a.seq = static_cast<uint32_t>(seq);
        a.cap = static_cast<uint32_t>(cap);
        a.D = static_cast<uint32_t>(D);
        a.scale = scale;
        a.dtype = dtype;
        a.part = part;
        a.part_bytes = part_bytes;
        return launch_prefill(a, s);
    }

    AttnParams p{};
    p.q = q; p.k = k; p.v = v; p.o = o; p.kc = k_cache; p.vc = v_cache;
    p.past = past_lens;
    p.past_per_row = past_per_row;
    p.N = static_cast<uint32_t>(N);
    p.H = static_cast<uint32_t>(n_head);
    p.Hkv = static_cast<uint32_t>(n_kv_head);
    p.seq = static_cast<uint32_t>(seq);
    p.cap = static_cast<uint32_t>(cap);
    p.group = p.H / p.Hkv;
    p.scale_log2e = scale * 1.4426950408889634f;
    p.part = part;
    p.counters = counters;
    p.n_workgroups = max_workgroups;  // upper bound; launch() lowers it to what is resident
    if (clear_counters) {
        attn_clear<<<1, 256, 0, s>>>(counters, max_workgroups);
        const int rc = launch_status();
        if (rc) return rc;
    }
    if (dtype == RG_FP16) {
        return D == 128 ? dispatch_group<__half, 128>(p, s) : dispatch_group<__half, 64>(p, s);
    }
    return D == 128 ? dispatch_group<__hip_bfloat16, 128>(p, s) : dispatch_group<__hip_bfloat16, 64>(p, s);
}

}  // namespace
}  // namespace rg

extern "C" size_t rg_hip_attention_kvcache_workspace(size_t, size_t, size_t, size_t, size_t, size_t D) {
    return rg::workspace_bytes(D);
}

extern "C" size_t rg_hip_attention_kvcache_state_bytes(void) { return rg::kCounterBytes; }

extern "C" int rg_hip_attention_kvcache(void *o, const void *q, const void *k, const void *v,
                                        void *k_cache, void *v_cache, const int64_t *past_lens,
                                        int past_per_row, size_t N, size_t n_head, size_t n_kv_head,
                                        size_t seq, size_t cap, size_t D, float scale, int dtype,
                                        void *workspace, size_t workspace_bytes, void *sync_state,
                                        void *stream) {
    using namespace rg;
    // a workspace that is missing or too small is reported after the argument checks
    const bool usable = workspace && D <= 128 && workspace_bytes >= rg::workspace_bytes(D);
    float *part = usable ? reinterpret_cast<float *>(static_cast<char *>(workspace) + kCounterBytes) : nullptr;
    uint32_t *counters = static_cast<uint32_t *>(sync_state ? sync_state : workspace);
    return attention_call(o, q, k, v, k_cache, v_cache, past_lens, past_per_row, N, n_head, n_kv_head, seq, cap, D,
                          scale, dtype, part, usable ? workspace_bytes - kCounterBytes : 0, counters, kMaxWorkgroups,
                          sync_state == nullptr, as_stream(stream));
}

extern "C" size_t rg_hip_attention_kvcache_static_scratch_bytes(void) { return rg::kStaticBytes; }

extern "C" int rg_hip_attention_kvcache_static(void *o, const void *q, const void *k, const void *v,
                                               void *k_cache, void *v_cache, const int64_t *past_lens,
                                               int past_per_row, size_t N, size_t n_head, size_t n_kv_head,
                                               size_t seq, size_t cap, size_t D, float scale, int dtype,
                                               void *stream) {
    using namespace rg;
    // the scratch is sized for head dimensions up to 128 and head groups of four per launch
    if (D > 128) return RG_HIP_E_WORKSPACE;
    void *base = nullptr;
    const int rc = static_scratch(&base);
    if (rc) return rc;
    uint32_t *counters = static_cast<uint32_t *>(base);
    float *part = reinterpret_cast<float *>(static_cast<char *>(base) + kStaticCounterBytes);
    // The counters are cleared by a small fill kernel on every call (no memset: the call may be
    // under stream capture), so that whatever an earlier call left there cannot matter.
    return attention_call(o, q, k, v, k_cache, v_cache, past_lens, past_per_row, N, n_head, n_kv_head, seq, cap, D,
                          scale, dtype, part, kStaticPartBytes, counters, kStaticWorkgroups, true, as_stream(stream));
}
