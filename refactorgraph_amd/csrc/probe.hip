// Measurement aid, not an operator: a loop of int8 matrix-core products on operands that stay in
// registers.  What it sustains is the ceiling of any MatMulInteger kernel on this part for the same
// operand values (the chip lowers its clock under matrix-core load, and by how much depends on how
// many bits toggle, i.e. on the data), so bench.py quotes the GEMM kernel against it.
#include "common.hpp"

namespace rg {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

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

}  // namespace
}  // namespace rg

extern "C" int rg_hip_probe_mfma_i8(int32_t *out, const void *operands, size_t workgroups, size_t iterations, void *stream) {
    using namespace rg;
    if (!out || !operands || workgroups == 0 || workgroups > 0x7fffffffu || iterations > 0xffffffffu) return RG_HIP_E_ARGUMENT;
    if (!aligned16(operands)) return RG_HIP_E_ARGUMENT;
    probe_mfma_i8<<<static_cast<unsigned>(workgroups), 256, 0, as_stream(stream)>>>(
        out, static_cast<const v4i *>(operands), static_cast<uint32_t>(iterations));
    return launch_status();
}
