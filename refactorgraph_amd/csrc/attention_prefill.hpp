// Interface between the attention entry point and the tiled (MFMA) prefill kernel.
#pragma once

#include "common.hpp"

namespace rg {

struct PrefillArgs {
    const void *q, *k, *v;
    void *o, *kc, *vc;
    const int64_t *past;
    int past_per_row;
    uint32_t N, H, Hkv, seq, cap, D;
    float scale;
    int dtype;  // RG_FP16 or RG_BF16
    float *part;        // workspace for the partial results of key ranges (may be null: no ranges then)
    size_t part_bytes;
};

// Bytes of `part` with which every launch that shares keys between workgroups finds room.
size_t prefill_part_bytes(uint32_t D);

// True when launch_prefill handles the shape (head dim 64, 80, 96 or 128, any group size).
bool prefill_supported(uint32_t H, uint32_t Hkv, uint32_t D);

// Enqueues the kernel; returns a hipError_t as int.
int launch_prefill(const PrefillArgs &a, hipStream_t s);

}  // namespace rg
