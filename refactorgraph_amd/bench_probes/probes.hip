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
