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
// form in float.  Segments that end up in more than one range leave (max, sum, unnormalised O)
// partials that a second small kernel merges.
#include "common.hpp"

namespace rg {
namespace {

constexpr int kMaxBatch = 1024;     // rows of the batch whose lengths a workgroup scans
constexpr float kMinusBig = -1e30f; // running-max sentinel (finite: keeps exp2 arguments defined)

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
    uint32_t n_workgroups;
};

// ---------------------------------------------------------------- key-space partition
// Batch row b contributes seq query rows; query row r has L = base_b + r + 1 keys for each of
// the Hkv kv heads.  Order: b, then r, then kv head, then key position.

struct Partition {
    uint64_t *prefix;   // [N + 1] keys before batch row b
    uint32_t *base;     // [N] clamped history length of batch row b
};

__device__ __forceinline__ uint64_t keys_before_row(uint32_t Hkv, uint32_t base, uint32_t r) {
    // Hkv * sum_{i<r} (base + i + 1)
    return static_cast<uint64_t>(Hkv) * (static_cast<uint64_t>(r) * (base + 1) + static_cast<uint64_t>(r) * (r - 1) / 2);
}

// Fills `part` (shared memory) and returns the total key count.  Called by every thread.
__device__ uint64_t build_partition(const AttnParams &p, Partition part, uint64_t *scan_tmp) {
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
    // exclusive scan of per-batch-row key counts; N <= kMaxBatch, blockDim.x-strided chunks
    if (t == 0) {
        uint64_t run = 0;
        for (uint32_t b = 0; b < p.N; ++b) {
            part.prefix[b] = run;
            run += keys_before_row(p.Hkv, part.base[b], p.seq);
        }
        part.prefix[p.N] = run;
    }
    (void) scan_tmp;
    __syncthreads();
    return part.prefix[p.N];
}

struct Segment {
    uint32_t b, r, kvh;
    uint32_t base;       // history length of batch row b
    uint32_t len;        // keys of this segment = base + r + 1
    uint64_t start;      // position of key 0 of the segment in the laid-out key space
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
    const uint64_t u2 = u - keys_before_row(p.Hkv, s.base, s.r);
    s.kvh = static_cast<uint32_t>(u2 / s.len);
    s.start = part.prefix[lo] + keys_before_row(p.Hkv, s.base, s.r) + static_cast<uint64_t>(s.kvh) * s.len;
    return s;
}

__device__ __forceinline__ uint64_t range_width(uint64_t total, uint32_t n_workgroups) {
    uint64_t w = (total + n_workgroups - 1) / n_workgroups;
    w = (w + 15) / 16 * 16;
    return w < 64 ? 64 : w;
}

// ---------------------------------------------------------------- element helpers

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

// reduction over the LPR (8 or 16) lanes that share a key row
template <int LPR>
__device__ __forceinline__ float row_sum(float v) {
    v += dpp_f32<0xB1>(v);
    v += dpp_f32<0x4E>(v);
    v += dpp_f32<0x141>(v);
    if constexpr (LPR == 16) v += dpp_f32<0x140>(v);
    return v;
}

// ---------------------------------------------------------------- split kernel

template <class T, int D, int G>
__global__ __launch_bounds__(256) void attn_split(const AttnParams p) {
    constexpr int LPR = D / 8;          // lanes per key row
    constexpr int KPW = kWave / LPR;    // key rows per wavefront load
    constexpr int KPB = KPW * 4;        // key rows per workgroup step
    constexpr int STATES = KPB;         // independent online-softmax states per workgroup
    constexpr int U = 4;                // steps in flight

    __shared__ uint64_t sh_prefix[kMaxBatch + 1];
    __shared__ uint32_t sh_base[kMaxBatch];
    __shared__ float sh_o[STATES][G][D];
    __shared__ float sh_m[STATES][G];
    __shared__ float sh_l[STATES][G];

    const Partition part{sh_prefix, sh_base};
    const uint64_t total = build_partition(p, part, nullptr);
    const uint64_t W = range_width(total, p.n_workgroups);
    const uint64_t range_begin = static_cast<uint64_t>(blockIdx.x) * W;
    if (range_begin >= total) return;
    const uint64_t range_end = range_begin + W < total ? range_begin + W : total;

    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t row = lane / LPR, chunk = lane % LPR;  // key row within a wavefront load, 16-byte slice
    const T *Q = static_cast<const T *>(p.q);
    const T *Kn = static_cast<const T *>(p.k);
    const T *Vn = static_cast<const T *>(p.v);
    T *Kc = static_cast<T *>(p.kc);
    T *Vc = static_cast<T *>(p.vc);
    T *O = static_cast<T *>(p.o);

    uint64_t f = range_begin;
    while (f < range_end) {
        const Segment sg = locate(p, part, f);
        const uint32_t pos0 = static_cast<uint32_t>(f - sg.start);
        const uint64_t left = range_end - f;
        const uint32_t len = static_cast<uint32_t>(left < sg.len - pos0 ? left : sg.len - pos0);
        const bool whole = pos0 == 0 && len == sg.len;

        // this lane's slice of the G query rows
        uint32_t qv[G][4];
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const uint32_t h = sg.kvh * p.group + p.head0 + g;
            const Raw16 raw = *reinterpret_cast<const Raw16 *>(
                Q + ((static_cast<uint64_t>(sg.b) * p.H + h) * p.seq + sg.r) * D + chunk * 8);
#pragma unroll
            for (int e = 0; e < 4; ++e) qv[g][e] = raw.w[e];
        }
        const uint64_t kv_head = static_cast<uint64_t>(sg.b) * p.Hkv + sg.kvh;
        const T *k_hist = Kc ? Kc + kv_head * p.cap * D : nullptr;
        const T *v_hist = Vc ? Vc + kv_head * p.cap * D : nullptr;
        const T *k_new = Kn + kv_head * p.seq * D;
        const T *v_new = Vn + kv_head * p.seq * D;
        // only the last query row's segment appends, and only on the launch that owns it
        const bool do_append = p.append && Kc && sg.r + 1 == p.seq;

        float m[G], l[G], acc[G][8];
#pragma unroll
        for (int g = 0; g < G; ++g) {
            m[g] = kMinusBig;
            l[g] = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[g][e] = 0.f;
        }

        const uint32_t end = pos0 + len;
        for (uint32_t step0 = pos0; step0 < end; step0 += KPB * U) {
            Raw16 kk[U], vv[U];
            bool valid[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const uint32_t key = step0 + u * KPB + wave * KPW + row;
                valid[u] = key < end;
                kk[u] = Raw16{{0, 0, 0, 0}};
                vv[u] = Raw16{{0, 0, 0, 0}};
                if (valid[u]) {
                    if (key >= sg.base) {  // one of the new rows
                        const uint64_t off = static_cast<uint64_t>(key - sg.base) * D + chunk * 8;
                        kk[u] = *reinterpret_cast<const Raw16 *>(k_new + off);
                        vv[u] = *reinterpret_cast<const Raw16 *>(v_new + off);
                        if (do_append) {
                            const uint64_t coff = (kv_head * p.cap + key) * D + chunk * 8;
                            *reinterpret_cast<Raw16 *>(Kc + coff) = kk[u];
                            *reinterpret_cast<Raw16 *>(Vc + coff) = vv[u];
                        }
                    } else {
                        const uint64_t off = static_cast<uint64_t>(key) * D + chunk * 8;
                        kk[u] = *reinterpret_cast<const Raw16 *>(k_hist + off);
                        vv[u] = *reinterpret_cast<const Raw16 *>(v_hist + off);
                    }
                }
            }
            float s[U][G];
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int g = 0; g < G; ++g) {
                    float d = 0.f;
#pragma unroll
                    for (int e = 0; e < 4; ++e) d = Elem<T>::dot2(qv[g][e], kk[u].w[e], d);
                    d = row_sum<LPR>(d) * p.scale_log2e;
                    s[u][g] = valid[u] ? d : -__builtin_inff();
                }
#pragma unroll
            for (int g = 0; g < G; ++g) {
                float mn = m[g];
#pragma unroll
                for (int u = 0; u < U; ++u) mn = fmaxf(mn, s[u][g]);
                const float alpha = __builtin_amdgcn_exp2f(m[g] - mn);
                m[g] = mn;
                float pr[U], ps = 0.f;
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    pr[u] = __builtin_amdgcn_exp2f(s[u][g] - mn);
                    ps += pr[u];
                }
                l[g] = l[g] * alpha + ps;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float a0 = acc[g][2 * e] * alpha, a1 = acc[g][2 * e + 1] * alpha;
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        a0 = fmaf(pr[u], Elem<T>::lo(vv[u].w[e]), a0);
                        a1 = fmaf(pr[u], Elem<T>::hi(vv[u].w[e]), a1);
                    }
                    acc[g][2 * e] = a0;
                    acc[g][2 * e + 1] = a1;
                }
            }
        }

        // merge the STATES row states of the workgroup
        const uint32_t st = wave * KPW + row;
        __syncthreads();  // previous piece finished reading
#pragma unroll
        for (int g = 0; g < G; ++g) {
#pragma unroll
            for (int e = 0; e < 8; ++e) sh_o[st][g][chunk * 8 + e] = acc[g][e];
            if (chunk == 0) {
                sh_m[st][g] = m[g];
                sh_l[st][g] = l[g];
            }
        }
        __syncthreads();
        const uint64_t slot = static_cast<uint64_t>(blockIdx.x) * 2 + (f == range_begin ? 0 : 1);
        float *pslot = p.part + slot * (G * (D + 2));
        for (uint32_t idx = threadIdx.x; idx < G * D; idx += 256) {
            const uint32_t g = idx / D, d = idx % D;
            float M = kMinusBig;
#pragma unroll
            for (int s2 = 0; s2 < STATES; ++s2) M = fmaxf(M, sh_m[s2][g]);
            float o_sum = 0.f, l_sum = 0.f;
#pragma unroll
            for (int s2 = 0; s2 < STATES; ++s2) {
                const float w = __builtin_amdgcn_exp2f(sh_m[s2][g] - M);
                o_sum = fmaf(w, sh_o[s2][g][d], o_sum);
                l_sum = fmaf(w, sh_l[s2][g], l_sum);
            }
            if (whole) {
                const uint32_t h = sg.kvh * p.group + p.head0 + g;
                T *dst = O + ((static_cast<uint64_t>(sg.b) * p.H + h) * p.seq + sg.r) * D + d;
                *reinterpret_cast<uint16_t *>(dst) = Elem<T>::pack(o_sum / l_sum);
            } else {
                pslot[g * (D + 2) + d] = o_sum;
                if (d == 0) {
                    pslot[g * (D + 2) + D] = M;
                    pslot[g * (D + 2) + D + 1] = l_sum;
                }
            }
        }
        f += len;
    }
}

// One workgroup per segment; merges the partials of segments that were cut.
template <class T, int D, int G>
__global__ __launch_bounds__(256) void attn_merge(const AttnParams p) {
    __shared__ uint64_t sh_prefix[kMaxBatch + 1];
    __shared__ uint32_t sh_base[kMaxBatch];
    const Partition part{sh_prefix, sh_base};
    const uint64_t total = build_partition(p, part, nullptr);
    const uint64_t W = range_width(total, p.n_workgroups);

    const uint32_t kvh = blockIdx.x % p.Hkv;
    const uint32_t br = blockIdx.x / p.Hkv;
    const uint32_t r = br % p.seq, b = br / p.seq;
    const uint32_t base = part.base[b];
    const uint32_t len = base + r + 1;
    const uint64_t start = part.prefix[b] + keys_before_row(p.Hkv, base, r) + static_cast<uint64_t>(kvh) * len;
    const uint64_t first = start / W, last = (start + len - 1) / W;
    if (first == last) return;  // finished by the split kernel

    T *O = static_cast<T *>(p.o);
    for (uint32_t idx = threadIdx.x; idx < G * D; idx += 256) {
        const uint32_t g = idx / D, d = idx % D;
        float M = kMinusBig;
        for (uint64_t w = first; w <= last; ++w) {
            const uint64_t piece_start = start > w * W ? start : w * W;
            const uint64_t slot = w * 2 + (piece_start == w * W ? 0 : 1);
            M = fmaxf(M, p.part[slot * (G * (D + 2)) + g * (D + 2) + D]);
        }
        float o_sum = 0.f, l_sum = 0.f;
        for (uint64_t w = first; w <= last; ++w) {
            const uint64_t piece_start = start > w * W ? start : w * W;
            const uint64_t slot = w * 2 + (piece_start == w * W ? 0 : 1);
            const float *ps = p.part + slot * (G * (D + 2)) + g * (D + 2);
            const float wgt = __builtin_amdgcn_exp2f(ps[D] - M);
            o_sum = fmaf(wgt, ps[d], o_sum);
            l_sum = fmaf(wgt, ps[D + 1], l_sum);
        }
        const uint32_t h = kvh * p.group + p.head0 + g;
        T *dst = O + ((static_cast<uint64_t>(b) * p.H + h) * p.seq + r) * D + d;
        *reinterpret_cast<uint16_t *>(dst) = Elem<T>::pack(o_sum / l_sum);
    }
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
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, attn_split<T, D, G>, 256, 0) != hipSuccess ||
            per_cu <= 0)
            per_cu = 2;
        return static_cast<uint32_t>(per_cu) * static_cast<uint32_t>(device_info().cus);
    }();
    return cached;
}

constexpr uint32_t kMaxWorkgroups = 4096;  // bound used by the workspace query

template <class T, int D, int G>
int launch(AttnParams p, hipStream_t s) {
    uint32_t wgs = resident_workgroups<T, D, G>();
    if (wgs > kMaxWorkgroups) wgs = kMaxWorkgroups;
    p.n_workgroups = wgs;
    attn_split<T, D, G><<<wgs, 256, 0, s>>>(p);
    int rc = launch_status();
    if (rc) return rc;
    const uint64_t segments = static_cast<uint64_t>(p.N) * p.seq * p.Hkv;
    attn_merge<T, D, G><<<static_cast<unsigned>(segments), 256, 0, s>>>(p);
    return launch_status();
}

template <class T, int D>
int dispatch_group(AttnParams p, hipStream_t s) {
    // heads of a kv group are processed G at a time (G in {4, 2, 1})
    uint32_t done = 0;
    while (done < p.group) {
        const uint32_t left = p.group - done;
        p.head0 = done;
        p.append = done == 0;
        int rc;
        if (left >= 4) {
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

size_t workspace_bytes(size_t D) {
    // two partial slots per workgroup, sized for the widest head group (4)
    return static_cast<size_t>(kMaxWorkgroups) * 2 * 4 * (D + 2) * sizeof(float);
}

}  // namespace
}  // namespace rg

extern "C" size_t rg_hip_attention_kvcache_workspace(size_t, size_t, size_t, size_t, size_t, size_t D) {
    return rg::workspace_bytes(D);
}

extern "C" int rg_hip_attention_kvcache(void *o, const void *q, const void *k, const void *v,
                                        void *k_cache, void *v_cache, const int64_t *past_lens,
                                        int past_per_row, size_t N, size_t n_head, size_t n_kv_head,
                                        size_t seq, size_t cap, size_t D, float scale, int dtype,
                                        void *workspace, size_t workspace_bytes, void *stream) {
    using namespace rg;
    if (!o || !q || !k || !v) return RG_HIP_E_ARGUMENT;
    if ((k_cache == nullptr) != (v_cache == nullptr)) return RG_HIP_E_ARGUMENT;
    if (N == 0 || n_head == 0 || seq == 0) return 0;
    if (n_kv_head == 0 || n_head % n_kv_head != 0) return RG_HIP_E_ARGUMENT;
    if (D != 64 && D != 128) return RG_HIP_E_UNSUPPORTED;
    if (dtype != RG_FP16 && dtype != RG_BF16) return RG_HIP_E_UNSUPPORTED;
    if (N > kMaxBatch || seq > 0xffffu || cap > 0x3fffffffu || n_head > 0xffffu) return RG_HIP_E_UNSUPPORTED;
    if (k_cache && cap < seq) return RG_HIP_E_ARGUMENT;
    if (N * seq * n_kv_head > 0x7fffffffu) return RG_HIP_E_UNSUPPORTED;
    if (!workspace || workspace_bytes < rg::workspace_bytes(D)) return RG_HIP_E_WORKSPACE;
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o) ||
        (k_cache && (!aligned16(k_cache) || !aligned16(v_cache))))
        return RG_HIP_E_ARGUMENT;

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
    p.part = static_cast<float *>(workspace);
    hipStream_t s = as_stream(stream);
    if (dtype == RG_FP16) {
        return D == 128 ? dispatch_group<__half, 128>(p, s) : dispatch_group<__half, 64>(p, s);
    }
    return D == 128 ? dispatch_group<__hip_bfloat16, 128>(p, s) : dispatch_group<__hip_bfloat16, 64>(p, s);
}
