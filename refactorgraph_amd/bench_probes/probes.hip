// Measurement aids for bench.py, not operators and not part of the boundary library: they are built into
// librg_probe.so, which only the benchmark loads.  Each one measures what the part itself sustains with nothing
// else to do, so that a kernel's rate can be quoted against a ceiling measured in the same run:
//   rg_probe_mfma_i8    a loop of int8 matrix-core products on operands that stay in registers (the chip lowers
//                       its clock under matrix-core load, and by how much depends on how many bits toggle,
//                       i.e. on the data);
//   rg_probe_hbm_read   a plain stream of 128-bit non-temporal loads,
//   rg_probe_hbm_write  a plain stream of 128-bit non-temporal stores,
//   rg_probe_hbm_copy   both.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <utility>

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// One wavefront per SIMD (256 accumulator registers), like the GEMM kernel's 4 x 4 blocks of
// v_mfma_i32_32x32x32_i8; `operands` holds 8 fragments of 16 bytes per lane.
__global__ __launch_bounds__(256, 1) void probe_mfma_i8(int32_t *__restrict__ out, const v4i *__restrict__ operands,
                                                        uint32_t iters) {
    const uint32_t lane = threadIdx.x & 63;
    v4i a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        a[i] = operands[lane * 8 + i];
        b[i] = operands[lane * 8 + 4 + i];
    }
    v16i acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;
    for (uint32_t it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[(i & 1) ? 3 - j : j], acc[i][j], 0, 0, 0);
    }
    int32_t sum = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) sum += acc[i][j][e];
    out[blockIdx.x * 256 + threadIdx.x] = sum;
}

// Streams: a workgroup of 256 threads owns consecutive blocks of 8 x 4 KiB (eight 128-bit accesses per thread in
// flight, each wavefront access 1 KiB contiguous) and walks the buffer with the grid's stride.
constexpr uint32_t kUnroll = 8;
constexpr uint64_t kBlockVecs = 256ull * kUnroll;   // 16-byte vectors per workgroup and pass

template <bool READ, bool WRITE>
__global__ __launch_bounds__(256) void probe_stream(u32x4 *__restrict__ dst, const u32x4 *__restrict__ src, uint64_t vecs,
                                                    uint32_t *__restrict__ sink) {
    u32x4 keep = {0u, 0u, 0u, 0u};
    for (uint64_t base = blockIdx.x * kBlockVecs; base < vecs; base += gridDim.x * kBlockVecs) {
        u32x4 v[kUnroll];
#pragma unroll
        for (uint32_t u = 0; u < kUnroll; ++u) {
            const uint64_t at = base + u * 256 + threadIdx.x;
            if constexpr (READ) v[u] = at < vecs ? __builtin_nontemporal_load(src + at) : u32x4{0u, 0u, 0u, 0u};
            else v[u] = u32x4{static_cast<uint32_t>(at), 1u, 2u, 3u};
        }
#pragma unroll
        for (uint32_t u = 0; u < kUnroll; ++u) {
            const uint64_t at = base + u * 256 + threadIdx.x;
            if constexpr (WRITE) {
                if (at < vecs) __builtin_nontemporal_store(v[u], dst + at);
            } else {
                keep ^= v[u];
            }
        }
    }
    if constexpr (!WRITE) {
        // never true for the benchmark's data; keeps the loads alive
        if ((keep[0] ^ keep[1] ^ keep[2] ^ keep[3]) == 0x9e3779b9u) *sink = keep[0];
    }
}

int status() { return static_cast<int>(hipGetLastError()); }

// workgroups == 0: one workgroup per 32 KiB block (the dispatcher deals them out); otherwise that many
// workgroups walk the buffer with the grid's stride.
unsigned stream_grid(uint64_t vecs, size_t workgroups) {
    uint64_t blocks = (vecs + kBlockVecs - 1) / kBlockVecs;
    if (blocks == 0) blocks = 1;
    if (blocks > 0x7fffffffull) blocks = 0x7fffffffull;
    if (workgroups != 0 && workgroups < blocks) blocks = workgroups;
    return static_cast<unsigned>(blocks);
}

}  // namespace

// `workgroups` workgroups of four wavefronts (one per SIMD) each run `iterations` x 16 v_mfma_i32_32x32x32_i8 on
// operands that stay in registers (2 * 32^3 integer operations per product and wavefront) and write one int32 per
// thread to out [workgroups * 256].  operands: 8 KiB (64 lanes x 8 fragments x 16 bytes, 16-byte aligned).
extern "C" int rg_probe_mfma_i8(int32_t *out, const void *operands, size_t workgroups, size_t iterations, void *stream) {
    if (!out || !operands || workgroups == 0 || workgroups > 0x7fffffffu || iterations > 0xffffffffu) return 1;
    if (reinterpret_cast<uintptr_t>(operands) & 15u) return 1;
    probe_mfma_i8<<<static_cast<unsigned>(workgroups), 256, 0, reinterpret_cast<hipStream_t>(stream)>>>(
        out, static_cast<const v4i *>(operands), static_cast<uint32_t>(iterations));
    return status();
}

// bytes: a multiple of 16; pointers 16-byte aligned.  sink: 4 bytes the read probe may write (it never does for
// data whose words do not XOR to one particular constant).
extern "C" int rg_probe_hbm_read(void *sink, const void *src, size_t bytes, size_t workgroups, void *stream) {
    if (!sink || !src || bytes % 16 || (reinterpret_cast<uintptr_t>(src) & 15u)) return 1;
    const uint64_t vecs = bytes / 16;
    probe_stream<true, false><<<stream_grid(vecs, workgroups), 256, 0, reinterpret_cast<hipStream_t>(stream)>>>(
        nullptr, static_cast<const u32x4 *>(src), vecs, static_cast<uint32_t *>(sink));
    return status();
}

extern "C" int rg_probe_hbm_write(void *dst, size_t bytes, size_t workgroups, void *stream) {
    if (!dst || bytes % 16 || (reinterpret_cast<uintptr_t>(dst) & 15u)) return 1;
    const uint64_t vecs = bytes / 16;
    probe_stream<false, true><<<stream_grid(vecs, workgroups), 256, 0, reinterpret_cast<hipStream_t>(stream)>>>(
        static_cast<u32x4 *>(dst), nullptr, vecs, nullptr);
    return status();
}

extern "C" int rg_probe_hbm_copy(void *dst, const void *src, size_t bytes, size_t workgroups, void *stream) {
    if (!dst || !src || bytes % 16 || ((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) & 15u)) return 1;
    const uint64_t vecs = bytes / 16;
    probe_stream<true, true><<<stream_grid(vecs, workgroups), 256, 0, reinterpret_cast<hipStream_t>(stream)>>>(
        static_cast<u32x4 *>(dst), static_cast<const u32x4 *>(src), vecs, nullptr);
    return status();
}

// ---------------------------------------------------------------- calibration probes (bench.py --calibrate)
//
// rg_probe_issue_shadow: what a wavefront that is alone on its SIMD can issue behind a matrix product without
// delaying the next one.  Workgroups of four wavefronts run a loop of v_mfma_i32_32x32x32_i8 (zero operands, so the
// clock stays up and clocks are what is measured) with `count` instructions of one kind behind every product, and
// report the shader clocks per product.  kind: 0 v_xor_b32, 1 s_nop, 2 ds_read_b128, 3 dependent s_add_u32,
// 4 v_exp_f32, 5 v_cvt_pk_f16_f32, 6 v_dot2c_f32_f16, 7 v_max3_f32, 8 v_fma_f32, 9 ds_read_b64_tr_b16.
// rg_probe_copy_rate: bytes per shader clock that a CU takes from L2 with `waves` wavefronts that keep `depth`
// 1 KiB transfers in flight each: global_load_lds_dwordx4 (into LDS) or global_load_dwordx4 (into registers).
namespace {

// (LDS reads name their target as read and written: the register stays the read's own until the sum at the end, so
// the compiler puts nothing else where data still on its way will land)
template <int KIND, int N>
__device__ __forceinline__ void shadow_filler(int (&x)[8], v4i (&r)[8], const __attribute__((address_space(3))) v4i *lp, unsigned &s) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
        if constexpr (KIND == 0) asm volatile("v_xor_b32 %0, %0, %1" : "+v"(x[i % 8]) : "v"(x[(i + 1) % 8]));
        else if constexpr (KIND == 1) asm volatile("s_nop 0");
        else if constexpr (KIND == 2) asm volatile("ds_read_b128 %0, %1 offset:%2" : "+v"(r[i % 8]) : "v"(lp), "n"((i % 8) * 1024));
        else if constexpr (KIND == 3) asm volatile("s_add_u32 %0, %0, 1" : "+s"(s) : : "scc");
        else if constexpr (KIND == 4) asm volatile("v_exp_f32 %0, %0" : "+v"(x[i % 8]));
        else if constexpr (KIND == 5) asm volatile("v_cvt_pk_f16_f32 %0, %0, %1" : "+v"(x[i % 8]) : "v"(x[(i + 1) % 8]));
        else if constexpr (KIND == 6) asm volatile("v_dot2c_f32_f16 %0, %1, %2" : "+v"(x[i % 8]) : "v"(x[(i + 1) % 8]), "v"(x[(i + 2) % 8]));
        else if constexpr (KIND == 7) asm volatile("v_max3_f32 %0, %0, %1, %2" : "+v"(x[i % 8]) : "v"(x[(i + 1) % 8]), "v"(x[(i + 2) % 8]));
        else if constexpr (KIND == 8) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(x[i % 8]) : "v"(x[(i + 1) % 8]), "v"(x[(i + 2) % 8]));
        else if constexpr (KIND == 9) asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "+v"(*reinterpret_cast<long long *>(&r[i % 8])) : "v"(lp), "n"((i % 8) * 512));
    }
}

template <int KIND, int N>
__global__ __launch_bounds__(256, 1) void probe_shadow(unsigned long long *out, int iters) {
    __shared__ v4i lds[2048];
    const unsigned lane = threadIdx.x & 63;
    for (int i = threadIdx.x; i < 2048; i += 256) lds[i] = v4i{0, 0, 0, 0};
    __syncthreads();
    v4i a[4], b[4];
    for (int i = 0; i < 4; ++i) { a[i] = v4i{0, 0, 0, 0}; b[i] = v4i{0, 0, 0, 0}; }
    v16i acc[4][4];
    for (int i = 0; i < 4; ++i) for (int j = 0; j < 4; ++j) for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;
    int x[8];
    for (int i = 0; i < 8; ++i) x[i] = lane + i;
    v4i r[8];
    for (int i = 0; i < 8; ++i) r[i] = v4i{0, 0, 0, 0};
    unsigned s = 0;
    const __attribute__((address_space(3))) v4i *lp = (const __attribute__((address_space(3))) v4i *)lds + lane;
    const unsigned long long t0 = __builtin_readcyclecounter();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[j], acc[i][j], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
                shadow_filler<KIND, N>(x, r, lp, s);
                __builtin_amdgcn_sched_barrier(0);
            }
        if constexpr (KIND == 2 || KIND == 9) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }
    const unsigned long long t1 = __builtin_readcyclecounter();
    int sum = s;
    for (int i = 0; i < 8; ++i) sum += x[i] + r[i][0] + r[i][1] + r[i][2] + r[i][3];
    for (int i = 0; i < 4; ++i) for (int j = 0; j < 4; ++j) for (int e = 0; e < 16; ++e) sum += acc[i][j][e];
    if (threadIdx.x == 0) out[blockIdx.x] = t1 - t0;
    if (sum == 0x12345678) out[4096 + threadIdx.x] = sum;
}

template <int KIND, int... Ns>
bool shadow_dispatch(int count, unsigned long long *out, unsigned grid, int iters, hipStream_t s, std::integer_sequence<int, Ns...>) {
    bool hit = false;
    ((count == Ns ? (probe_shadow<KIND, Ns><<<grid, 256, 0, s>>>(out, iters), hit = true) : false), ...);
    return hit;
}

// DEPTH 0: into LDS, `depth` transfers per wavefront and round; DEPTH > 0: into registers, DEPTH transfers per round
// (ordinary loads, so that the compiler knows which registers the transfers in flight still own)
template <int DEPTH>
__global__ __launch_bounds__(512) void probe_copy(unsigned long long *out, const unsigned char *src, int iters, int depth) {
    __shared__ __align__(1024) unsigned char lds[65536];
    const unsigned tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), waves = blockDim.x / 64;
    // four workgroups walk one 1 MiB region, 32 regions: what an XCD's workgroups touch stays in its L2
    const unsigned char *base = src + static_cast<size_t>(blockIdx.x % 8 + 8 * ((blockIdx.x / 8) % 4)) * (1 << 20);
    const unsigned lds_base = static_cast<unsigned>(reinterpret_cast<size_t>((__attribute__((address_space(3))) unsigned char *)lds)) + wave * 8192;
    v4i acc = {0, 0, 0, 0};
    const unsigned long long t0 = __builtin_readcyclecounter();
    for (int it = 0; it < iters; ++it) {
        if constexpr (DEPTH == 0) {
            for (int u0 = 0; u0 < depth; u0 += 4) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const unsigned off = ((it * depth + u0 + j) * waves + wave) * 1024 % (1 << 20);
                    const unsigned long long pb = reinterpret_cast<unsigned long long>(base + off);
                    const unsigned char *p = reinterpret_cast<const unsigned char *>(
                        (static_cast<unsigned long long>(__builtin_amdgcn_readfirstlane(static_cast<unsigned>(pb >> 32))) << 32) |
                        static_cast<unsigned>(__builtin_amdgcn_readfirstlane(static_cast<unsigned>(pb))));
                    const unsigned to = __builtin_amdgcn_readfirstlane(lds_base + ((u0 + j) & 7) * 1024);
                    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(lane * 16), "s"(p), "s"(to) : "memory", "m0");
                }
            }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        } else {
            v4i t[DEPTH];
#pragma unroll
            for (int u = 0; u < DEPTH; ++u) {
                const unsigned off = ((it * DEPTH + u) * waves + wave) * 1024 % (1 << 20);
                t[u] = *reinterpret_cast<const v4i *>(base + off + lane * 16);
            }
#pragma unroll
            for (int u = 0; u < DEPTH; ++u) acc += t[u];
        }
    }
    const unsigned long long t1 = __builtin_readcyclecounter();
    if (tid == 0) out[blockIdx.x] = t1 - t0;
    if (acc[0] == 0x12345678) out[4096] = acc[1] + lds[tid];
}

}  // namespace

// out: device memory for 8192 unsigned 64-bit words; word w < workgroups: shader clocks of the timed loop of workgroup w
extern "C" int rg_probe_issue_shadow(void *out, int kind, int count, size_t workgroups, size_t iterations, void *stream) {
    if (!out || workgroups == 0 || workgroups > 4096 || iterations == 0 || iterations > 0x7fffffff) return 1;
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    auto *o = static_cast<unsigned long long *>(out);
    const unsigned g = static_cast<unsigned>(workgroups);
    const int it = static_cast<int>(iterations);
    using Counts = std::integer_sequence<int, 0, 1, 2, 3, 4, 6, 8, 12>;
    bool hit = false;
    switch (kind) {
        case 0: hit = shadow_dispatch<0>(count, o, g, it, s, Counts{}); break;
        case 1: hit = shadow_dispatch<1>(count, o, g, it, s, Counts{}); break;
        case 2: hit = shadow_dispatch<2>(count, o, g, it, s, Counts{}); break;
        case 3: hit = shadow_dispatch<3>(count, o, g, it, s, Counts{}); break;
        case 4: hit = shadow_dispatch<4>(count, o, g, it, s, Counts{}); break;
        case 5: hit = shadow_dispatch<5>(count, o, g, it, s, Counts{}); break;
        case 6: hit = shadow_dispatch<6>(count, o, g, it, s, Counts{}); break;
        case 7: hit = shadow_dispatch<7>(count, o, g, it, s, Counts{}); break;
        case 8: hit = shadow_dispatch<8>(count, o, g, it, s, Counts{}); break;
        case 9: hit = shadow_dispatch<9>(count, o, g, it, s, Counts{}); break;
        default: break;
    }
    return hit ? status() : 1;
}

// src: at least 32 MiB of device memory; out as above
extern "C" int rg_probe_copy_rate(void *out, const void *src, int to_lds, size_t waves, size_t depth, size_t workgroups,
                                  size_t iterations, void *stream) {
    if (!out || !src || (waves != 4 && waves != 8) || depth == 0 || depth > 64 || depth % 4 != 0 || workgroups == 0 || workgroups > 4096 ||
        iterations == 0 || iterations > 0x7fffffff)
        return 1;
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    auto *o = static_cast<unsigned long long *>(out);
    const unsigned g = static_cast<unsigned>(workgroups), b = static_cast<unsigned>(waves * 64);
    const auto *from = static_cast<const unsigned char *>(src);
    const int it = static_cast<int>(iterations), d = static_cast<int>(depth);
    if (to_lds) probe_copy<0><<<g, b, 0, s>>>(o, from, it, d);
    else if (depth == 4) probe_copy<4><<<g, b, 0, s>>>(o, from, it, d);
    else if (depth == 8) probe_copy<8><<<g, b, 0, s>>>(o, from, it, d);
    else if (depth == 16) probe_copy<16><<<g, b, 0, s>>>(o, from, it, d);
    else if (depth == 32) probe_copy<32><<<g, b, 0, s>>>(o, from, it, d);
    else return 1;
    return status();
}
