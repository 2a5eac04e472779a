// Hand-off between workgroups that share a sum: each leaves its part in a workspace, the one that finds all parts
// delivered adds them up.  Used where a reduction dimension is split between workgroups of one launch and the result
// must neither depend on timing nor need a clearing launch (few rows of MatMul and MatMulInteger).
#pragma once

#include <atomic>
#include <chrono>

#include "common.hpp"

namespace rg {

constexpr unsigned long long kCounterAtRest = 0x5DEECE66D1CE4E5Bull;  // what a strip's arrival counter holds between launches

// The workgroup's sums have been stored (written through).  Returns true in the workgroup that has to add the
// strip's shares up.  Every wavefront waits until its stores have been acknowledged and the barrier collects them;
// then one thread counts this share in.  The counter rests at a fixed 64-bit value between launches (the workgroup
// that counts in last puts it back), so the arrival that reads that value + shares - 1 is the last one: one round
// trip.  A counter that reads anything else - the workspace is handed over with arbitrary contents - says nothing,
// and then, for every share of that launch alike, flags decide: this share's flag is set to the launch's number and
// acknowledged, the strip's flags are read (loads that bypass the XCD's L2), and a workgroup that finds them all
// set adds up.  The workgroup whose flag reached memory last is certain to; another one that arrived at almost the
// same time may too, and then both store the same values.  Flags holding anything else than this launch's number
// count as not set; whoever adds up clears them and puts the counter to rest.  No clearing launch, no dependence
// of the result on who is last.
__device__ __forceinline__ bool shares_complete(unsigned long long *counter, unsigned long long *strip_flags, uint32_t share,
                                                uint32_t shares, unsigned long long launch_no, uint32_t tid) {
    __shared__ int state;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) {
        const unsigned long long d = __hip_atomic_fetch_add(counter, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - kCounterAtRest;
        state = d < shares ? (d == shares - 1 ? 2 : 1) : 0;
        if (d == shares - 1) __hip_atomic_store(counter, kCounterAtRest, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (d >= shares) {
            __hip_atomic_store(strip_flags + share, launch_no, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
    }
    __syncthreads();
    const int st = state;
    if (st != 0) return st == 2;
    int set = 1;
    for (uint32_t f = tid; f < shares; f += blockDim.x)
        set &= __hip_atomic_load(strip_flags + f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == launch_no;
    if (!__syncthreads_and(set)) return false;
    for (uint32_t f = tid; f < shares; f += blockDim.x) __hip_atomic_store(strip_flags + f, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (tid == 0) __hip_atomic_store(counter, kCounterAtRest, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return true;
}

// A number no other launch of this process carries (started from the clock so that what an earlier process
// left in a reused allocation does not match either).
inline unsigned long long next_launch_number() {
    static std::atomic<unsigned long long> counter{
        static_cast<unsigned long long>(std::chrono::steady_clock::now().time_since_epoch().count()) * 0x9E3779B97F4A7C15ull};
    return counter.fetch_add(1, std::memory_order_relaxed) | (1ull << 63);  // never 0, which stands for a cleared flag
}


// Device-scope accesses for the parts: the store is written through, the load does not hit a stale line of another
// XCD's L2.
__device__ __forceinline__ void store_through(float *p, float v) {
    __hip_atomic_store(reinterpret_cast<uint32_t *>(p), __builtin_bit_cast(uint32_t, v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_through(const float *p) {
    return __builtin_bit_cast(float, __hip_atomic_load(reinterpret_cast<const uint32_t *>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
}

}  // namespace rg
