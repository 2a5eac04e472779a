// Tiled causal attention for many query rows per batch row (prefill), head dim 128 or 64, gfx950.
//
// Same contract as the split-KV kernel (layouts of src/08-01llm/README.md:29-63 of the
// reference: q, o [N, H, seq, D]; k, v [N, Hkv, seq, D]; caches [N, Hkv, cap, D]; query row r
// attends positions 0 .. past + r; new rows appended at past .. past + seq - 1).
//
// A workgroup of four wavefronts works on one kv head at a time: wavefront w owns 32 query rows of
// one of the query heads that share this kv head (GQA), so a K/V tile staged once in LDS serves up
// to four query heads.  Keys are walked 64 at a time; a tile of K and V rows is copied from global
// memory straight into one of two LDS buffers (global_load_lds_dwordx4: lane L of a wavefront-wide
// copy fills bytes 16 L .. 16 L + 15 behind a wave-uniform LDS base from an address of its own),
// one tile ahead of its use, with the 16-byte chunks of a row XOR-swizzled so that the fragment
// reads below are free of bank conflicts.  Both products run on the fp16/bf16 MFMA
// (v_mfma_f32_32x32x16) in transposed form:
//     S^T[key, q] = K[key, :] . Q[q, :]       A = K rows (LDS, 128-bit reads), B = Q rows (registers)
//     O^T[d, q]  += V^T[d, key] . P^T[key, q] A = V columns (LDS, transposing 64-bit reads), B = P (registers)
// In this form a lane holds one query row of S^T / O^T in its accumulator registers, so the
// softmax row statistics need no cross-lane reduction beyond one exchange between the two
// half-wavefronts, and P^T is already in B-operand position.  Softmax is online in float with
// the lazily raised reference of the split kernel.
//
// The workgroups are persistent.  The unit of work is an item = 32 query rows x 4 heads of one
// (batch row, kv head) stream; moving the query rows in and the output rows out is pure memory
// latency, which a workgroup that did one item would pay in full (a launch of one-item workgroups
// spent two thirds of its time there).  So a workgroup walks a list of items, and the two LDS
// buffers carry one continuous sequence of slots across them: [Q of item 0] [tile 0] [tile 1] ...
// [Q of item 1] [tile 0] ...  While a slot is worked on, the next one is copied in; the query rows
// of the next item therefore arrive under the last key tile of the current one, the output rows
// leave from registers (16-byte stores, no staging) while tile 0 of the next item is on its way,
// and nothing waits for memory except the very first slot.  Items are dealt so that every
// workgroup gets the same number of key tiles (query tile t is paired with tile q_tiles - 1 - t)
// and so that the workgroups of an XCD walk few streams at a time, which keeps the K/V rows that
// the query tiles of a stream share in that XCD's L2.
#include "attention_prefill.hpp"

namespace rg {
namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef __bf16 b8 __attribute__((ext_vector_type(8)));
typedef float f16v __attribute__((ext_vector_type(16)));

constexpr int BN = 64;                 // keys per tile: two blocks of 32
constexpr int KB = BN / 32;            // blocks of 32 keys per tile
constexpr int CPI = BN / 16;           // K (and V) copy instructions per wavefront and tile
constexpr int ROWB = 256;              // bytes of a K, V or Q row in LDS: head dim 128, unpadded.  Head dim 64 keeps
                                       // this pitch and the layout below and uses chunks 0-7 of a row only (the
                                       // copies fill the other positions with chunks they fetch a second time)
constexpr int TILE = BN * ROWB;        // 16384: one K or V tile
constexpr int BUF_BYTES = 2 * TILE;    // K tile + V tile; two such buffers, reused for the output transposition
constexpr float kSlack = 6.0f;
constexpr float kMinusBig = -1e30f;
constexpr uint64_t kSplitMinTiles = 8;  // key tiles of the capacity per range of a SPLIT launch, at least
constexpr uint64_t kSplitMax = 32;      // ranges per item, at most

// LDS layout of a tile: the 16-byte chunk c of K row r sits at chunk position c ^ (r & 15), which
// puts the 128-bit fragment reads of 8 or 16 consecutive rows on distinct banks; chunk c of V row r
// sits at c ^ v_swizzle(r & 3), which does the same for the transposing 64-bit reads (4 rows x 32
// or 64 bytes per group of lanes).
__device__ __forceinline__ uint32_t v_swizzle(uint32_t r) { return 4 * (r & 1) + 10 * ((r >> 1) & 1); }

struct alignas(16) Raw16 {
    uint32_t w[4];
};

struct U2 {
    uint32_t w[2];
};
// 64-bit LDS read that transposes 16-bit elements inside each group of 16 lanes: lane i of a group
// receives element i % 4 of what lanes i / 4, i / 4 + 4, i / 4 + 8 and i / 4 + 12 address.
typedef short s4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ U2 read_tr16(const uint8_t *p) {
    const s4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s4 __attribute__((address_space(3))) *)(p));
    return __builtin_bit_cast(U2, v);
}

template <class T> struct Ops;
template <> struct Ops<__half> {
    static __device__ __forceinline__ f16v mfma(const Raw16 &a, const Raw16 &b, f16v c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(h8, a), __builtin_bit_cast(h8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        const h2 v = {static_cast<_Float16>(lo), static_cast<_Float16>(hi)};
        return __builtin_bit_cast(uint32_t, v);
    }
    // running row sum: the two rounded probabilities of a packed word, exactly as the PV product sees them
    static __device__ __forceinline__ float add_pair(float sum, uint32_t packed, float, float) {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        const h2 ones = {static_cast<_Float16>(1.f), static_cast<_Float16>(1.f)};
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, packed), ones, sum, false);
    }
};
template <> struct Ops<__hip_bfloat16> {
    static __device__ __forceinline__ f16v mfma(const Raw16 &a, const Raw16 &b, f16v c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(b8, a), __builtin_bit_cast(b8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        const uint32_t l = __builtin_bit_cast(uint16_t, __float2bfloat16(lo));
        const uint32_t h = __builtin_bit_cast(uint16_t, __float2bfloat16(hi));
        return l | (h << 16);
    }
    static __device__ __forceinline__ float add_pair(float sum, uint32_t, float p0, float p1) { return sum + (p0 + p1); }
};

// Sum and maximum over the two half-wavefronts (lanes i and i + 32), on the vector ALU.
struct HalfPair {
    float a, b;
};
__device__ __forceinline__ HalfPair half_swap(float x, float y) {
    // a: lanes 0-31 keep x, lanes 32-63 receive y of lanes 0-31; b: lanes 0-31 receive x of lanes 32-63, 32-63 keep y
    const auto r = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(uint32_t, x), __builtin_bit_cast(uint32_t, y), false, false);
    const uint32_t r0 = r[0], r1 = r[1];
    return {__builtin_bit_cast(float, r0), __builtin_bit_cast(float, r1)};
}
__device__ __forceinline__ float half_max(float v) {
    const HalfPair r = half_swap(v, v);
    return fmaxf(r.a, r.b);
}
__device__ __forceinline__ float half_sum(float v) {
    const HalfPair r = half_swap(v, v);
    return r.a + r.b;
}

__device__ __forceinline__ uint32_t uni(uint32_t v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ uint32_t div_magic(uint32_t x, uint32_t magic) { return magic ? uni(__umulhi(x, magic)) : x; }

// How the items are dealt to the workgroups (computed on the host).
struct PrefillPlan {
    uint32_t group;        // query heads per kv head
    uint32_t head_chunks;  // group / HW
    uint32_t q_tiles;      // query tiles (of ROWS rows) per stream
    uint32_t pairs;        // (q_tiles + 1) / 2: workgroups that share a stream
    uint32_t xcds;         // 8 when the streams divide evenly over the XCDs, else 1
    uint32_t spx;          // streams per XCD
    uint32_t groups;       // sets of `pairs` workgroups per XCD; set g walks streams g, g + groups, ...
    // floor(2^32 / d) + 1 for d = head_chunks and d = Hkv: x / d = mulhi(x, magic) for every x with
    // x * d < 2^32, which the host checks (0 stands for d = 1)
    uint32_t magic_chunks, magic_hkv;
    // key ranges per item (SPLIT instances): the streams above are then (stream, range) pairs, range fastest
    uint32_t splits, magic_splits;
    float *part;  // partial results of the ranges, kPartFloats(DH) per item and range
};

// Partial result of one key range of one item: per thread its accumulator registers of O^T, then m and l.
__host__ __device__ constexpr uint32_t part_floats(uint32_t dh) { return 256u * (((dh + 31) / 32) * 16 + 2); }

// One item: query tile qt of stream (kv head `kvhead` = b * Hkv + kvh of the batch, head chunk hc).
// Kept to four scalars: the workgroup holds two of them across its whole life.
constexpr uint32_t kNoItem = 0xffffffffu;
struct Item {
    uint32_t kvhead, hc;
    uint32_t qt;    // kNoItem: there is no such item
    uint32_t base;  // history length of the batch row, moved into [0, cap - seq]
    uint32_t ks;    // key range of the item this workgroup walks (SPLIT instances; else 0)
    __device__ bool valid() const { return qt != kNoItem; }
};

// Copy of 16 bytes per lane from global memory into LDS (lane L of the wavefront fills bytes
// 16 L .. 16 L + 15 behind the wave-uniform LDS address; OFFSET is added to the global address and
// to the LDS address alike).  Issued as inline assembly: the compiler
// then does not know that a vector-memory operation writes LDS and adds no waits of its own between
// the copies and the LDS reads; every wait for a copy in this file is an explicit s_waitcnt before a
// barrier.  (Writing M0 needs one wait state before the copy reads it.)
template <int OFFSET>
__device__ __forceinline__ void copy16(const void *sbase, uint32_t voffset, uint32_t lds_addr) {
    // the base and the LDS address are wave-uniform by construction; they are pinned to scalar registers
    // here because the assembly needs them there, wherever the compiler has computed them
    const uint64_t b = reinterpret_cast<uint64_t>(sbase);
    sbase = reinterpret_cast<const void *>((static_cast<uint64_t>(uni(static_cast<uint32_t>(b >> 32))) << 32) |
                                           uni(static_cast<uint32_t>(b)));
    lds_addr = uni(lds_addr);
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 offset:%3"
                 :
                 : "v"(voffset), "s"(sbase), "s"(lds_addr), "n"(OFFSET)
                 : "memory", "m0");
}

#define RG_SCHED_FENCE() __builtin_amdgcn_sched_barrier(0)

// HW: query heads per workgroup (1, 2 or 4); the other 4 / HW wavefronts take further 32-row
// query sub-tiles of the same heads.
// SPLIT: an item's keys are shared between plan.splits workgroups (few items with a long history: chunked prefill,
// a new turn of a conversation); each leaves its unnormalised O^T, m and l in plan.part and attn_prefill_merge
// finishes the item.  The tiles of an item are dealt in equal counts; a range beyond the item's last tile walks
// tile 0 with every key masked (history lengths are device data: the host sizes the ranges by the capacity).
template <class T, int HW, int DH, bool SPLIT>
__global__ __launch_bounds__(256, 2) void attn_prefill(const PrefillArgs a, const PrefillPlan plan) {
    constexpr int QS = 4 / HW;      // query sub-tiles per workgroup
    constexpr int ROWS = 32 * QS;   // query rows per item
    constexpr int GROWB = 2 * DH;   // bytes of a row in memory
    constexpr int KSTEPS = DH / 16; // products of a S^T block
    constexpr int DBLK = (DH + 31) / 32;  // blocks of 32 rows of O^T (the last one half used at head dim 80)
    constexpr uint32_t NCH = DH / 8;      // 16-byte chunks of a row in memory; a copy's lanes beyond them fetch
                                          // chunk (position's chunk) % NCH of the same row a second time
    constexpr int OWN_PASSES = (ROWS * NCH + 255) / 256;  // the new rows on their way to the caches: chunks per thread
    static_assert(DH % 16 == 0 && DH >= 64 && DH <= 128, "head dim 64 to 128 in steps of 16");
    __shared__ __align__(1024) uint8_t lds[2 * BUF_BYTES];
    const uint32_t lds_addr0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
        (__attribute__((address_space(3))) uint8_t *)lds));

    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t half = lane >> 5, l32 = lane & 31;
    const uint32_t wave_u = uni(wave);

    // Workgroup w: consecutive ids are dealt round-robin to the XCDs.  Within an XCD, set g of
    // `pairs` workgroups walks the XCD's streams g, g + groups, ...; member j of a set takes query
    // tiles q_tiles - 1 - j and j of each of them (the heavy one first).
    const uint32_t xcd = uni(blockIdx.x % plan.xcds), lw = uni(blockIdx.x / plan.xcds);
    const uint32_t pj = uni(lw % plan.pairs), set = uni(lw / plan.pairs);
    uint32_t en_k = set, en_sub = 0;
    // The history length of an item's batch row is read when the item is enumerated and clamped
    // when the item becomes the current one (an item later), so that nobody waits for the load.
    auto next_item = [&](uint64_t &raw_past) __attribute__((always_inline)) -> Item {
        Item it{0, 0, kNoItem, 0, 0};
        raw_past = 0;
        while (en_k < plan.spx) {
            const uint32_t heavy = plan.q_tiles - 1 - pj;
            const uint32_t qt = en_sub == 0 ? heavy : pj;
            const bool ok = en_sub == 0 || pj != heavy;
            uint32_t stream = en_k * plan.xcds + xcd;
            if constexpr (SPLIT) {
                const uint32_t whole = div_magic(stream, plan.magic_splits);
                it.ks = stream - whole * plan.splits;
                stream = whole;
            }
            if (en_sub == 0) {
                en_sub = 1;
            } else {
                en_sub = 0;
                en_k += plan.groups;
            }
            if (!ok) continue;
            // (a plain integer division would run on the vector ALU and leave its results, and every
            // address derived from them, in vector registers)
            it.kvhead = div_magic(stream, plan.magic_chunks);
            it.hc = stream - it.kvhead * plan.head_chunks;
            it.qt = qt;
            if (a.kc && a.past) raw_past = static_cast<uint64_t>(a.past[a.past_per_row ? div_magic(it.kvhead, plan.magic_hkv) : 0]);
            break;
        }
        return it;
    };
    auto clamp_past = [&](uint64_t raw) __attribute__((always_inline)) -> uint32_t {
        // the two words are moved to scalar registers one by one and compared there (a 64-bit signed
        // comparison would be done on the vector ALU and drag everything that depends on the history
        // length into vector registers)
        const uint32_t lo = uni(static_cast<uint32_t>(raw)), hi = uni(static_cast<uint32_t>(raw >> 32));
        const uint32_t room = a.cap > a.seq ? a.cap - a.seq : 0;
        const uint32_t len = hi == 0 ? lo : (hi >> 31 ? 0u : room);  // negative: 0; beyond 32 bits: the upper end
        return len < room ? len : room;
    };

    const uint8_t *Q = static_cast<const uint8_t *>(a.q);
    const uint8_t *Kn = static_cast<const uint8_t *>(a.k);
    const uint8_t *Vn = static_cast<const uint8_t *>(a.v);
    uint8_t *Kc = static_cast<uint8_t *>(a.kc);
    uint8_t *Vc = static_cast<uint8_t *>(a.vc);
    T *O = static_cast<T *>(a.o);
    const float c_log2e = a.scale * 1.4426950408889634f;

    // ---- copies.  Tile: wavefront w copies key rows 16 w .. 16 w + 15 of K and of V, four rows
    // (1 KiB) per instruction; this lane brings chunk position lane % 16 of row 16 w + 4 i + lane / 16.
    // A tile that lies inside the history or inside the new rows is addressed as a uniform base plus
    // a per-lane byte offset prepared once (rows of the new tensors beyond the last key are read
    // along: they are masked); only a tile that straddles the two tensors or the end of the new rows
    // computes its addresses row by row.  The tensors' addresses are formed from the kernel arguments
    // by scalar arithmetic at every call: scalar registers are what this kernel is short of, scalar
    // instructions it has to spare.
    const uint32_t cp_row = (BN / 4) * wave_u + (lane >> 4);
    const uint32_t v_lane = cp_row * ROWB + 16 * ((lane & 15) ^ v_swizzle(lane >> 4));
    // K: chunk position lane % 16 of row r holds chunk (lane % 16) ^ (r & 15); rows 4 i further on flip
    // bits 2-3 of the chunk index, i.e. bits 6-7 of the byte offset
    const uint32_t k_lane = cp_row * ROWB + 16 * ((lane & 15) ^ (cp_row & 15));
    auto copy_tile = [&](const Item &it, uint32_t kt, uint32_t buf) __attribute__((always_inline)) {
        const uint32_t first = kt * BN, total_keys = it.base + a.seq;
        const bool in_hist = first + BN <= it.base, in_new = first >= it.base && first + BN <= total_keys;
        const uint32_t kdst = lds_addr0 + buf + CPI * wave_u * 1024, vdst = kdst + TILE;
        if (in_hist || in_new) {  // uniform
            const uint64_t row0 = in_hist ? static_cast<uint64_t>(it.kvhead) * a.cap + first
                                          : static_cast<uint64_t>(it.kvhead) * a.seq + (first - it.base);
            const uint8_t *kb_ = (in_hist ? Kc : Kn) + row0 * GROWB;
            const uint8_t *vb_ = (in_hist ? Vc : Vn) + row0 * GROWB;
            static_assert(CPI == 4, "four copies of four rows per wavefront and tensor");
            if constexpr (DH == 128) {
                // (the instruction's offset moves the global and the LDS address alike: four rows are 1 KiB in both)
                copy16<0>(kb_, k_lane, kdst);
                copy16<0>(vb_, v_lane, vdst);
                copy16<4 * ROWB>(kb_, k_lane ^ 64, kdst);
                copy16<4 * ROWB>(vb_, v_lane, vdst);
                copy16<8 * ROWB>(kb_, k_lane ^ 128, kdst);
                copy16<8 * ROWB>(vb_, v_lane, vdst);
                copy16<12 * ROWB>(kb_, k_lane ^ 192, kdst);
                copy16<12 * ROWB>(vb_, v_lane, vdst);
            } else {
#pragma unroll
                for (int i = 0; i < CPI; ++i) {
                    const uint32_t r = cp_row + 4 * i;
                    copy16<0>(kb_, r * GROWB + 16 * (((lane & 15) ^ (r & 15)) % NCH), kdst + i * 1024);
                    copy16<0>(vb_, r * GROWB + 16 * (((lane & 15) ^ v_swizzle(lane >> 4)) % NCH), vdst + i * 1024);
                }
            }
        } else {
            const uint8_t *kh = Kc + static_cast<uint64_t>(it.kvhead) * a.cap * GROWB;
            const uint8_t *vh = Vc + static_cast<uint64_t>(it.kvhead) * a.cap * GROWB;
            const uint8_t *kn = Kn + static_cast<uint64_t>(it.kvhead) * a.seq * GROWB;
            const uint8_t *vn = Vn + static_cast<uint64_t>(it.kvhead) * a.seq * GROWB;
#pragma unroll
            for (int i = 0; i < CPI; ++i) {
                uint32_t pos = first + cp_row + 4 * i;
                pos = pos < total_keys ? pos : total_keys - 1;
                // a wavefront's 16 rows may lie on both sides of the seam: the side is chosen per lane
                // by handing the copy the lane's full address (no scalar base)
                const bool old = pos < it.base;
                const uint32_t row_off = (old ? pos : pos - it.base) * GROWB;  // within one kv head: below 2^32
                const uint32_t kc = ((lane & 15) ^ ((cp_row + 4 * i) & 15)) % NCH, vc = ((lane & 15) ^ v_swizzle(lane >> 4)) % NCH;
                const uint8_t *ksrc = (old ? kh : kn) + (row_off + 16 * kc);
                const uint8_t *vsrc = (old ? vh : vn) + (row_off + 16 * vc);
                asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(ksrc), "s"(kdst + i * 1024) : "memory", "m0");
                asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(vsrc), "s"(vdst + i * 1024) : "memory", "m0");
            }
        }
    };
    // This wavefront's head within the group of the item's kv head.  A group that is no multiple of HW leaves the
    // last chunk short: the wavefronts beyond it repeat the group's last head and store nothing.
    auto head_in_group = [&](const Item &it) __attribute__((always_inline)) -> uint32_t {
        const uint32_t h = it.hc * HW + wave_u % HW;
        return h < plan.group ? h : plan.group - 1;
    };
    // Query rows of an item: every wavefront copies its own 32 rows (8 KiB, contiguous in memory)
    // into its quarter of the buffer, laid out like a K tile (chunk c of row r at position c ^ (r & 15)).
    auto copy_q = [&](const Item &it, uint32_t buf) __attribute__((always_inline)) {
        // (b * H + head) = kvhead * group + the head's index within the group
        const uint32_t bh = uni(it.kvhead * plan.group + head_in_group(it));
        const uint32_t r0 = it.qt * ROWS + 32 * (wave_u / HW);
        const uint8_t *qh = Q + static_cast<uint64_t>(bh) * a.seq * GROWB;
        const uint32_t dst = lds_addr0 + buf + wave_u * (32 * ROWB);
        if (r0 + 32 <= a.seq) {
            // rows 4 i + lane / 16: the same offset pattern as a K tile's
            const uint8_t *qb = qh + static_cast<uint64_t>(r0) * GROWB;
            if constexpr (DH == 128) {
                const uint32_t q_lane = (lane >> 4) * ROWB + 16 * ((lane & 15) ^ (lane >> 4));
                copy16<0>(qb, q_lane, dst);
                copy16<4 * ROWB>(qb, q_lane ^ 64, dst);
                copy16<8 * ROWB>(qb, q_lane ^ 128, dst);
                copy16<12 * ROWB>(qb, q_lane ^ 192, dst);
                const uint8_t *qb2 = qb + 16 * ROWB;  // (the instruction's offset field ends at 4095)
                copy16<0>(qb2, q_lane, dst + 4096);
                copy16<4 * ROWB>(qb2, q_lane ^ 64, dst + 4096);
                copy16<8 * ROWB>(qb2, q_lane ^ 128, dst + 4096);
                copy16<12 * ROWB>(qb2, q_lane ^ 192, dst + 4096);
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const uint32_t row = 4 * i + (lane >> 4);
                    copy16<0>(qb, row * GROWB + 16 * (((lane & 15) ^ (row & 15)) % NCH), dst + i * 1024);
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const uint32_t row = 4 * i + (lane >> 4);
                uint32_t grow = r0 + row;
                grow = grow < a.seq ? grow : a.seq - 1;
                copy16<0>(qh, grow * GROWB + 16 * (((lane & 15) ^ (row & 15)) % NCH), dst + i * 1024);  // within one head: below 2^32
            }
        }
    };

    // fragment addresses inside a buffer: K (or Q) row l32 (+ 32 kb), chunk 2 kk + half; V see below
    const uint32_t k_off = l32 * ROWB + 16 * (half ^ (l32 & 15));
    // V piece of block db: row 4 half + r (+ 32 kb + 16 jj, + 8), chunk 4 db + cl; the swizzle leaves
    // 4 db to bits 6-7 of the byte offset, so a block is reached by XOR with 64 db
    const uint32_t s16 = lane & 15, v_r = s16 >> 2, v_cl = 2 * ((lane >> 4) & 1) + ((s16 & 3) >> 1);
    const uint32_t v_off = TILE + (4 * half + v_r) * ROWB + 16 * (v_cl ^ v_swizzle(v_r)) + 8 * (s16 & 1);

    // ---- state of the item being worked on
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    Raw16 qf[KSTEPS];   // Q fragments (B operand): lane holds query row r0 + l32, d = 16 kk + 8 half .. +7
    f16v o[DBLK];
    float m = 0.f, l = 0.f;
    bool fresh = true;
    Item cur{0, 0, kNoItem, 0, 0};
    uint64_t nxt_raw = 0, nn_raw = 0;
    Item nxt = next_item(nxt_raw);
    if (!nxt.valid()) return;
    nxt.base = clamp_past(nxt_raw);
    // n_tiles: the tile after the last one this workgroup walks for the item, t_first the first one (0 and the
    // item's tile count unless SPLIT); qlim: the first key this lane's query row does not see
    uint32_t r0 = 0, n_tiles = 0, wave_tiles = 0, qlim = 0, t_first = 0;
    bool mask_all = false, last_range = true;
    auto key_range = [&](const Item &it, uint32_t &first, uint32_t &end, bool &dummy) __attribute__((always_inline)) {
        const uint32_t rows_end = (it.qt + 1) * ROWS < a.seq ? (it.qt + 1) * ROWS : a.seq;
        const uint32_t tiles = uni((it.base + rows_end - 1) / BN + 1);
        first = 0;
        end = tiles;
        dummy = false;
        if constexpr (SPLIT) {
            const uint32_t share = div_magic(tiles + plan.splits - 1, plan.magic_splits);  // tiles per range, rounded up
            first = it.ks * share;
            if (first >= tiles) {
                first = 0;
                end = 1;
                dummy = true;
            } else {
                end = first + share < tiles ? first + share : tiles;
            }
        }
    };
    auto begin_item = [&]() __attribute__((always_inline)) {
        r0 = cur.qt * ROWS + 32 * (wave_u / HW);
        const uint32_t rows_end = (cur.qt + 1) * ROWS < a.seq ? (cur.qt + 1) * ROWS : a.seq;
        const uint32_t all_tiles = uni((cur.base + rows_end - 1) / BN + 1);
        key_range(cur, t_first, n_tiles, mask_all);
        last_range = !mask_all && n_tiles == all_tiles;
        const uint32_t wave_last_row = r0 + 31 < a.seq ? r0 + 31 : a.seq - 1;
        wave_tiles = uni(r0 < a.seq ? (cur.base + wave_last_row) / BN + 1 : 0);
        qlim = mask_all ? 0u : cur.base + r0 + l32 + 1;  // absolute position of this lane's query row, plus one
#pragma unroll
        for (int db = 0; db < DBLK; ++db)
#pragma unroll
            for (int e = 0; e < 16; ++e) o[db][e] = 0.f;
        m = 0.f;
        l = 0.f;
        fresh = true;
    };

    // ---- the new k/v rows that correspond to an item's query rows go to the caches (once per kv head):
    // thread owns 16-byte chunk tid % 16 of rows tid / 16 + 16 j.  They are picked up behind the
    // item's last key tile, whose buffer still holds them unless the item's rows straddle two tiles
    // (then they are loaded from the inputs again), and stored when the item goes out.
    auto load_own_rows = [&](const Item &it, uint32_t buf, u32x4 (&ak)[ROWS / 16], u32x4 (&av)[ROWS / 16]) __attribute__((always_inline)) {
        if (!(Kc && it.hc == 0)) return;
        if (SPLIT && !last_range) return;  // (the range that ends with the item's last tile appends)
        const uint32_t rows_end = (it.qt + 1) * ROWS < a.seq ? (it.qt + 1) * ROWS : a.seq;
        const uint32_t lo = it.qt * ROWS;
        const uint32_t tile_first = (n_tiles - 1) * BN;  // first key of the last tile
        uint32_t tid = threadIdx.x;  // (opaque copy, see finish_item)
        asm volatile("" : "+v"(tid));
        // thread tid takes chunks tid, tid + 256, ... of the ROWS x NCH chunks of the item's rows
        if (it.base + lo >= tile_first) {
            const uint8_t *tb = lds + buf;
#pragma unroll
            for (int jr = 0; jr < OWN_PASSES; ++jr) {
                const uint32_t idx = tid + 256 * jr;
                uint32_t row = lo + idx / NCH;
                row = row < rows_end ? row : rows_end - 1;  // reads stay unconditional, the stores are guarded
                const uint32_t r = it.base + row - tile_first, c = idx % NCH;
                ak[jr] = *reinterpret_cast<const u32x4 *>(tb + r * ROWB + 16 * (c ^ (r & 15)));
                av[jr] = *reinterpret_cast<const u32x4 *>(tb + TILE + r * ROWB + 16 * (c ^ v_swizzle(r & 3)));
            }
        } else {
            const uint8_t *k_new = Kn + static_cast<uint64_t>(it.kvhead) * a.seq * GROWB;
            const uint8_t *v_new = Vn + static_cast<uint64_t>(it.kvhead) * a.seq * GROWB;
#pragma unroll
            for (int jr = 0; jr < OWN_PASSES; ++jr) {
                const uint32_t idx = tid + 256 * jr;
                uint32_t row = lo + idx / NCH;
                row = row < rows_end ? row : rows_end - 1;
                const uint32_t off = row * GROWB + (idx % NCH) * 16;
                ak[jr] = *reinterpret_cast<const u32x4 *>(k_new + off);
                av[jr] = *reinterpret_cast<const u32x4 *>(v_new + off);
            }
        }
    };

    // ---- output of a finished item: normalise and transpose through LDS, so that a store instruction
    // covers four whole rows (1 KiB contiguous) instead of 64 scattered pieces.  The wavefront uses
    // its own quarter of the query buffer (`stage`), which nobody else touches and whose query rows
    // it has already taken: chunk c of row r at chunk position c ^ (r & 15).  Then the item's own new rows.
    auto finish_item = [&](const Item &it, const u32x4 (&ak)[ROWS / 16], const u32x4 (&av)[ROWS / 16], uint8_t *stage) __attribute__((always_inline)) {
        const uint32_t bh = uni(it.kvhead * plan.group + head_in_group(it));
        const bool head_ok = it.hc * HW + wave_u % HW < plan.group;  // else a repeated head: nothing to store
        const uint32_t fr0 = it.qt * ROWS + 32 * (wave_u / HW);
        const uint32_t rows_end = (it.qt + 1) * ROWS < a.seq ? (it.qt + 1) * ROWS : a.seq;
        const bool do_append = Kc && it.hc == 0 && (!SPLIT || last_range);
        const uint32_t own_lo = it.base + it.qt * ROWS, own_hi = it.base + rows_end;
        // (lane indices from an opaque copy: the addresses below are then formed here, once per item, and
        // not ahead of the loops, where they would occupy registers all the time)
        uint32_t tid = threadIdx.x;
        asm volatile("" : "+v"(tid));
        const uint32_t lane = tid & 63, l32 = tid & 31, half = (tid >> 5) & 1;
        if constexpr (SPLIT) {
            if (fr0 < a.seq && head_ok) {
                // record of (item, range): register r of thread t at r * 256 + t.  A wavefront that met no tile of
                // its own in the range (or only masked keys) leaves a maximum far below any real one.
                const uint32_t stream = it.kvhead * plan.head_chunks + it.hc;
                float *rec = plan.part + (static_cast<uint64_t>(stream * plan.q_tiles + it.qt) * plan.splits + it.ks) * part_floats(DH);
#pragma unroll
                for (int db = 0; db < DBLK; ++db)
#pragma unroll
                    for (int e = 0; e < 16; ++e) rec[(db * 16 + e) * 256 + tid] = o[db][e];
                rec[(DBLK * 16) * 256 + tid] = fresh ? kMinusBig : m;
                rec[(DBLK * 16 + 1) * 256 + tid] = l;
            }
        } else if (fr0 < a.seq && head_ok) {
            const float inv = 1.f / half_sum(l);
#pragma unroll
            for (int db = 0; db < DBLK; ++db)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    if (4 * db + g >= static_cast<int>(NCH)) continue;  // (head dim 80: the second half of the last block)
                    // registers 4 g .. 4 g + 3 of a block: d = 32 db + 8 g + 4 half + 0..3 of row l32
                    const uint2 w = make_uint2(Ops<T>::pack2(o[db][4 * g] * inv, o[db][4 * g + 1] * inv),
                                               Ops<T>::pack2(o[db][4 * g + 2] * inv, o[db][4 * g + 3] * inv));
                    *reinterpret_cast<uint2 *>(stage + l32 * ROWB + 16 * ((4 * db + g) ^ (l32 & 15)) + 8 * half) = w;
                }
            // (each wavefront reads back only what it wrote itself: no barrier)
            uint8_t *op = reinterpret_cast<uint8_t *>(O) + (static_cast<uint64_t>(bh) * a.seq + fr0) * GROWB;
            // lane takes chunks lane, lane + 64, ... of the 32 x NCH chunks of the wavefront's rows
#pragma unroll
            for (int i = 0; i < (32 * static_cast<int>(NCH) + 63) / 64; ++i) {
                const uint32_t idx = lane + 64 * i, row = idx / NCH, c = idx % NCH;
                if (idx < 32 * NCH) {
                    const u32x4 v = *reinterpret_cast<const u32x4 *>(stage + row * ROWB + 16 * (c ^ (row & 15)));
                    if (fr0 + row < a.seq) *reinterpret_cast<u32x4 *>(op + row * GROWB + 16 * c) = v;
                }
            }
        }
        if (do_append) {
#pragma unroll
            for (int jr = 0; jr < OWN_PASSES; ++jr) {
                const uint32_t idx = tid + 256 * jr, pos = own_lo + idx / NCH;
                if (pos < own_hi) {  // (chunks beyond the item's ROWS rows fall beyond own_hi as well)
                    const uint64_t dst = (static_cast<uint64_t>(it.kvhead) * a.cap + pos) * GROWB + (idx % NCH) * 16;
                    *reinterpret_cast<u32x4 *>(Kc + dst) = ak[jr];
                    *reinterpret_cast<u32x4 *>(Vc + dst) = av[jr];
                }
            }
        }
    };

    // ---- one key tile in buffer `buf` (byte offset of the buffer within `lds`).  The scheduling
    // fences keep the order written here: fragment reads four ahead of the products that use them.
    auto tile = [&](uint32_t buf, uint32_t kt) __attribute__((always_inline)) {
        const uint32_t other = buf ^ BUF_BYTES;
        // The copy of the next slot (the next key tile, or the next item's query rows) is issued in
        // eight parts, one behind each of the first eight products: a copy instruction that finds the
        // memory pipeline busy holds the wavefront, and there it waits under a product instead of
        // ahead of them.  Both kinds of copy have the same shape: parts 0, 2, 4, 6 take four rows each
        // from `base_a`, parts 1, 3, 5, 7 from `base_b`.  A key tile that straddles the seam between
        // history and new rows, or ragged query rows, are copied at once (mode 2).
        uint32_t mode = 0, dst_a = 0, dst_b = 0;
        bool is_q = false;
        const uint8_t *base_a = nullptr, *base_b = nullptr;
        const uint32_t q_lane = (lane >> 4) * ROWB + 16 * ((lane & 15) ^ (lane >> 4));
        const uint32_t vq_lane = (lane >> 4) * ROWB + 16 * ((lane & 15) ^ v_swizzle(lane >> 4));
        if (kt + 1 < n_tiles) {
            const uint32_t first = (kt + 1) * BN, total_keys = cur.base + a.seq;
            const bool in_hist = first + BN <= cur.base, in_new = first >= cur.base && first + BN <= total_keys;
            if (in_hist || in_new) {
                const uint64_t row0 = (in_hist ? static_cast<uint64_t>(cur.kvhead) * a.cap + first
                                               : static_cast<uint64_t>(cur.kvhead) * a.seq + (first - cur.base)) +
                                      (BN / 4) * wave_u;
                base_a = (in_hist ? Kc : Kn) + row0 * GROWB;
                base_b = (in_hist ? Vc : Vn) + row0 * GROWB;
                dst_a = lds_addr0 + other + CPI * wave_u * 1024;
                dst_b = dst_a + TILE;
                mode = 1;
            } else {
                mode = 2;
            }
        } else if (nxt.valid()) {
            const uint32_t nr0 = nxt.qt * ROWS + 32 * (wave_u / HW);
            if (nr0 + 32 <= a.seq) {
                const uint32_t bh = uni(nxt.kvhead * plan.group + head_in_group(nxt));
                base_a = Q + (static_cast<uint64_t>(bh) * a.seq + nr0) * GROWB;
                base_b = base_a + 16 * GROWB;
                dst_a = lds_addr0 + other + wave_u * (32 * ROWB);
                dst_b = dst_a + 16 * ROWB;
                is_q = true;
                mode = 1;
            } else {
                mode = 2;
            }
        }
        auto copy_part = [&]<int I>() __attribute__((always_inline)) {
            if (mode != 1) return;
            constexpr int J = I / 2;
            if constexpr (DH == 128) {
                if (I % 2 == 0) copy16<J * 4 * ROWB>(base_a, q_lane ^ (64 * J), dst_a);
                else copy16<J * 4 * ROWB>(base_b, is_q ? q_lane ^ (64 * J) : vq_lane, dst_b);
            } else {
                // rows 4 J + lane / 16 of the wavefront's sixteen: K and Q rows swizzled by the row, V rows by lane / 16
                const uint32_t row = 4 * J + (lane >> 4);
                const uint32_t k_like = row * GROWB + 16 * (((lane & 15) ^ (row & 15)) % NCH);
                const uint32_t v_like = row * GROWB + 16 * (((lane & 15) ^ v_swizzle(lane >> 4)) % NCH);
                if (I % 2 == 0) copy16<0>(base_a, k_like, dst_a + 1024 * J);
                else copy16<0>(base_b, is_q ? k_like : v_like, dst_b + 1024 * J);
            }
        };
        auto copy_rest = [&]() __attribute__((always_inline)) {  // what the parts do not cover
            if (mode != 2) return;
            if (kt + 1 < n_tiles) copy_tile(cur, kt + 1, other);
            else copy_q(nxt, other);
        };
        if (kt >= wave_tiles) {
            copy_part.template operator()<0>();
            copy_part.template operator()<1>();
            copy_part.template operator()<2>();
            copy_part.template operator()<3>();
            copy_part.template operator()<4>();
            copy_part.template operator()<5>();
            copy_part.template operator()<6>();
            copy_part.template operator()<7>();
            copy_rest();
            return;
        }
        const uint8_t *const tb = lds + buf;
        // a block entirely above the diagonal is skipped
        const bool second = KB > 1 && kt * BN + 32 <= cur.base + r0 + 31;
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) {
            if (kb == 1 && !second) break;
            // S^T block kb: keys BN kt + 32 kb + (8 (e/4) + 4 half + e%4), query row l32
            Raw16 kf[4];
            const uint8_t *kb_base = tb + 32 * kb * ROWB;
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) kf[kk] = *reinterpret_cast<const Raw16 *>(kb_base + (k_off ^ (32 * kk)));
            if (kb == 0) copy_rest();
            RG_SCHED_FENCE();
            f16v sc;
#pragma unroll
            for (int e = 0; e < 16; ++e) sc[e] = 0.f;
            auto product = [&]<int KK>() __attribute__((always_inline)) {
                sc = Ops<T>::mfma(kf[KK % 4], qf[KK], sc);
                if constexpr (KK + 4 < KSTEPS) kf[KK % 4] = *reinterpret_cast<const Raw16 *>(kb_base + (k_off ^ (32 * (KK + 4))));
                if (kb == 0) {  // the eight parts of the copy spread over the products
                    constexpr int P0 = KK * 8 / KSTEPS, P1 = (KK + 1) * 8 / KSTEPS;
                    copy_part.template operator()<P0>();
                    if constexpr (P1 - P0 > 1) copy_part.template operator()<P0 + 1>();
                    static_assert(P1 - P0 <= 2, "at most two parts behind a product");
                }
                RG_SCHED_FENCE();
            };
            product.template operator()<0>();
            product.template operator()<1>();
            product.template operator()<2>();
            product.template operator()<3>();
            if constexpr (KSTEPS > 4) product.template operator()<4>();
            if constexpr (KSTEPS > 5) product.template operator()<5>();
            if constexpr (KSTEPS > 6) product.template operator()<6>();
            if constexpr (KSTEPS > 7) product.template operator()<7>();
            // O^T block db: rows d = 32 db + l32; A element i of MFMA (kb, jj) is V[key(i), d] with
            // key(i) = 32 kb + 16 jj + (i < 4 ? 4 half + i : 8 + 4 half + i - 4), the key order of pf.
            // A transposing read hands the 16 lanes of a group (16 consecutive d) four consecutive
            // keys each: lane s of the group addresses key s / 4, columns 4 (s % 4) .. +3.
            // (product index i = DBLK jj + db; the first four fragments are requested before the softmax)
            auto read_v = [&](int i) __attribute__((always_inline)) {
                const int jj = i / DBLK, db = i % DBLK;
                const uint8_t *vp = tb + (32 * kb + 16 * jj) * ROWB + (v_off ^ (64 * db));
                const U2 lo = read_tr16(vp), hi = read_tr16(vp + 8 * ROWB);
                return Raw16{{lo.w[0], lo.w[1], hi.w[0], hi.w[1]}};
            };
            Raw16 vf[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) vf[i] = read_v(i);
            RG_SCHED_FENCE();
            // scale, causal mask (only blocks that reach past the wavefront's first query position)
            const bool need_mask = kt * BN + 32 * kb + 31 > cur.base + r0 || (SPLIT && mask_all);
            float over = -__builtin_inff();
            if (need_mask) {  // wave-uniform: only the blocks on the diagonal pay for the comparisons
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const uint32_t key = kt * BN + 32 * kb + 8 * (e / 4) + 4 * half + (e % 4);
                    const float t = key >= qlim ? -__builtin_inff() : fmaf(sc[e], c_log2e, -m);
                    sc[e] = t;
                    over = fmaxf(over, t);
                }
            } else {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const float t = fmaf(sc[e], c_log2e, -m);
                    sc[e] = t;
                    over = fmaxf(over, t);
                }
            }
            over = half_max(over);  // both halves hold the same query row
            if (fresh || __builtin_amdgcn_ballot_w64(over > kSlack) != 0) {
                const float up = fresh ? fmaxf(over, kMinusBig) : fmaxf(over, 0.f);
                const float alpha = fresh ? 1.f : __builtin_amdgcn_exp2f(-up);
                m += up;
                l *= alpha;
#pragma unroll
                for (int db = 0; db < DBLK; ++db)
#pragma unroll
                    for (int e = 0; e < 16; ++e) o[db][e] *= alpha;
#pragma unroll
                for (int e = 0; e < 16; ++e) sc[e] -= up;
                fresh = false;
            }
            // P^T in B-operand position: element i of MFMA (kb, jj) is accumulator register 8 jj + i
            Raw16 pf[2];
#pragma unroll
            for (int jj = 0; jj < 2; ++jj)
#pragma unroll
                for (int i2 = 0; i2 < 4; ++i2) {
                    const float p0 = __builtin_amdgcn_exp2f(sc[8 * jj + 2 * i2]);
                    const float p1 = __builtin_amdgcn_exp2f(sc[8 * jj + 2 * i2 + 1]);
                    pf[jj].w[i2] = Ops<T>::pack2(p0, p1);
                    l = Ops<T>::add_pair(l, pf[jj].w[i2], p0, p1);
                }
            RG_SCHED_FENCE();
#pragma unroll
            for (int i = 0; i < 2 * DBLK; ++i) {
                o[i % DBLK] = Ops<T>::mfma(vf[i % 4], pf[i / DBLK], o[i % DBLK]);
                if (i + 4 < 2 * DBLK) vf[i % 4] = read_v(i + 4);
                RG_SCHED_FENCE();
            }
        }
    };

    // ---- the slot of the next item's query rows (in buffer `buf`; the other buffer still holds the
    // last key tile of the item just finished): every wavefront takes its query fragments and the
    // finished item's own new rows out of LDS; after a barrier tile 0 of the next item is requested
    // into the buffer thus freed, and the finished item goes out while it travels
    bool have_cur = false;
    auto q_slot = [&](uint32_t buf) __attribute__((always_inline)) -> bool {
        Item nn{0, 0, kNoItem, 0, 0};
        u32x4 ak[ROWS / 16], av[ROWS / 16];
        if (have_cur) load_own_rows(cur, buf ^ BUF_BYTES, ak, av);
        if (nxt.valid()) {
            const uint8_t *qb = lds + buf + wave_u * (32 * ROWB);
#pragma unroll
            for (int kk = 0; kk < KSTEPS; ++kk) qf[kk] = *reinterpret_cast<const Raw16 *>(qb + (k_off ^ (32 * kk)));
            if (have_cur) {
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                __builtin_amdgcn_s_barrier();
            }
            uint32_t first = 0, end = 0;
            bool dummy = false;
            key_range(nxt, first, end, dummy);
            copy_tile(nxt, first, buf ^ BUF_BYTES);
            nn = next_item(nn_raw);  // its history length is on its way while the output goes out
        }
        if (have_cur) finish_item(cur, ak, av, lds + buf + wave_u * (32 * ROWB));
        if (!nxt.valid()) return false;
        cur = nxt;
        nxt = nn;
        nxt.base = clamp_past(nn_raw);
        have_cur = true;
        begin_item();
        return true;
    };
    auto end_slot = [&]() __attribute__((always_inline)) {
        // this wavefront's copies for the next slot have landed and its reads of this slot's buffer
        // are done; after the barrier that holds for the workgroup
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
    };

    // slot sequence: the query slot of an item, then its key tiles; the buffer alternates with every slot
    copy_q(nxt, 0);
    end_slot();
    uint32_t buf = 0;
    for (;;) {
        if (!q_slot(buf)) break;
        end_slot();
        buf ^= BUF_BYTES;
        for (uint32_t kt = t_first; kt < n_tiles; ++kt) {
            tile(buf, kt);
            end_slot();
            buf ^= BUF_BYTES;
        }
    }
}

// Finishes the items of a SPLIT launch: workgroups with the threads of attn_prefill (wavefront = head and query
// sub-tile, lane = query row and half of the keys), each taking eight of a thread's accumulator registers
// (blockIdx.y: two groups of four consecutive d), add the ranges' records weighted by 2^(m_range - m_max), normalise
// and store four consecutive d per instruction.
constexpr int kMergeRegs = 8;
template <class T, int HW, int DH>
__global__ __launch_bounds__(256) void attn_prefill_merge(const PrefillArgs a, const PrefillPlan plan) {
    constexpr int QS = 4 / HW, ROWS = 32 * QS, DBLK = (DH + 31) / 32;
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5, l32 = lane & 31;
    const uint32_t qt = blockIdx.x % plan.q_tiles, stream = blockIdx.x / plan.q_tiles;
    const uint32_t kvhead = stream / plan.head_chunks, hc = stream % plan.head_chunks;
    const uint32_t h = hc * HW + wave % HW;
    const uint32_t fr0 = qt * ROWS + 32 * (wave / HW);
    if (h >= plan.group || fr0 >= a.seq) return;  // (whole wavefronts)
    const float *rec = plan.part + static_cast<uint64_t>(blockIdx.x) * plan.splits * part_floats(DH);
    const uint32_t e0 = blockIdx.y * kMergeRegs;
    float m_max = kMinusBig;
    for (uint32_t r = 0; r < plan.splits; ++r) m_max = fmaxf(m_max, rec[r * part_floats(DH) + (DBLK * 16) * 256 + tid]);
    float o[kMergeRegs], l = 0.f;
#pragma unroll
    for (int e = 0; e < kMergeRegs; ++e) o[e] = 0.f;
#pragma unroll 4
    for (uint32_t r = 0; r < plan.splits; ++r) {
        const float *p = rec + r * part_floats(DH);
        const float w = __builtin_amdgcn_exp2f(p[(DBLK * 16) * 256 + tid] - m_max);
        l += w * p[(DBLK * 16 + 1) * 256 + tid];
#pragma unroll
        for (int e = 0; e < kMergeRegs; ++e) o[e] += w * p[(e0 + e) * 256 + tid];
    }
    const float inv = 1.f / half_sum(l);
    const uint32_t row = fr0 + l32;
    if (row >= a.seq) return;
    T *out = static_cast<T *>(a.o) + (static_cast<uint64_t>(kvhead * plan.group + h) * a.seq + row) * DH;
#pragma unroll
    for (int gg = 0; gg < kMergeRegs / 4; ++gg) {
        // registers 4 g .. 4 g + 3 of block db: d = 32 db + 8 g + 4 half + 0..3
        const uint32_t e = e0 + 4 * gg, db = e / 16, g = (e % 16) / 4, d = 32 * db + 8 * g + 4 * half;
        if (d >= DH) continue;  // (head dim 80: the second half of the last block)
        const uint2 w = make_uint2(Ops<T>::pack2(o[4 * gg] * inv, o[4 * gg + 1] * inv), Ops<T>::pack2(o[4 * gg + 2] * inv, o[4 * gg + 3] * inv));
        *reinterpret_cast<uint2 *>(out + d) = w;
    }
}

template <class T, int HW, int DH>
uint32_t resident_prefill_workgroups() {
    static uint32_t cached = [] {
        int per_cu = 0, dev = 0, cus = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, attn_prefill<T, HW, DH, false>, 256, 0) != hipSuccess || per_cu <= 0)
            per_cu = 2;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess) cus = prop.multiProcessorCount;
        if (cus <= 0) cus = 256;
        return static_cast<uint32_t>(per_cu) * static_cast<uint32_t>(cus);
    }();
    return cached;
}

template <class T, int HW, int DH>
int launch_hw(const PrefillArgs &a, hipStream_t s) {
    constexpr uint32_t ROWS = 32 * (4 / HW);
    PrefillPlan plan{};
    plan.group = a.H / a.Hkv;
    plan.head_chunks = (plan.group + HW - 1) / HW;
    plan.q_tiles = (a.seq + ROWS - 1) / ROWS;
    plan.pairs = (plan.q_tiles + 1) / 2;
    uint64_t streams = static_cast<uint64_t>(a.N) * a.Hkv * plan.head_chunks;
    if (streams * plan.pairs > 0x7fffffffu) return RG_HIP_E_UNSUPPORTED;
    // Few items and room for a long history: the keys of an item are shared between workgroups, as many as bring
    // the launch to the workgroups that are resident together, each with at least kSplitMinTiles tiles of the
    // capacity, while the records fit the workspace (head dims 64 and 128)
    plan.splits = 1;
    const uint64_t items = streams * plan.q_tiles;
    if constexpr (DH == 64 || DH == 128) {
        const uint64_t resident = resident_prefill_workgroups<T, HW, DH>();
        const uint64_t cap_tiles = (static_cast<uint64_t>(a.cap) + BN - 1) / BN;
        uint64_t splits = items ? resident / items : 1;
        if (splits > cap_tiles / kSplitMinTiles) splits = cap_tiles / kSplitMinTiles;
        if (splits > kSplitMax) splits = kSplitMax;
        const uint64_t room = a.part ? a.part_bytes / (items * part_floats(DH) * sizeof(float)) : 0;
        if (splits > room) splits = room;
        if (splits >= 2 && streams * splits * plan.pairs <= 0x7fffffffu) plan.splits = static_cast<uint32_t>(splits);
    }
    plan.magic_splits = plan.splits > 1 ? static_cast<uint32_t>((1ull << 32) / plan.splits + 1) : 0;
    plan.part = a.part;
    const uint64_t whole_streams = streams;
    streams *= plan.splits;
    plan.xcds = streams % 8 == 0 ? 8 : 1;
    plan.spx = static_cast<uint32_t>(streams / plan.xcds);
    // as many sets of `pairs` workgroups per XCD as stay resident together (at least one)
    const uint32_t per_xcd = resident_prefill_workgroups<T, HW, DH>() / plan.xcds;
    uint32_t groups = per_xcd / plan.pairs;
    if (groups < 1) groups = 1;
    if (groups > plan.spx) groups = plan.spx;
    plan.groups = groups;
    uint64_t widest = plan.head_chunks > a.Hkv ? plan.head_chunks : a.Hkv;
    if (plan.splits > widest) widest = plan.splits;
    if (streams * widest >= (1ull << 32)) return RG_HIP_E_UNSUPPORTED;
    plan.magic_chunks = plan.head_chunks > 1 ? static_cast<uint32_t>((1ull << 32) / plan.head_chunks + 1) : 0;
    plan.magic_hkv = a.Hkv > 1 ? static_cast<uint32_t>((1ull << 32) / a.Hkv + 1) : 0;
    const uint32_t grid = plan.xcds * plan.groups * plan.pairs;
    if constexpr (DH == 64 || DH == 128) {
        if (plan.splits > 1) {
            attn_prefill<T, HW, DH, true><<<grid, 256, 0, s>>>(a, plan);
            const int rc = launch_status();
            if (rc) return rc;
            constexpr unsigned parts = ((DH + 31) / 32) * 16 / kMergeRegs;
            attn_prefill_merge<T, HW, DH><<<dim3(static_cast<unsigned>(whole_streams * plan.q_tiles), parts), 256, 0, s>>>(a, plan);
            return launch_status();
        }
    }
    (void)whole_streams;
    attn_prefill<T, HW, DH, false><<<grid, 256, 0, s>>>(a, plan);
    return launch_status();
}

template <class T, int DH>
int launch_d(const PrefillArgs &a, hipStream_t s) {
    const uint32_t group = a.H / a.Hkv;
    if (group == 1) return launch_hw<T, 1, DH>(a, s);
    if (group == 2) return launch_hw<T, 2, DH>(a, s);
    return launch_hw<T, 4, DH>(a, s);  // chunks of four heads; the last one is short when group % 4 != 0
}

template <class T>
int launch_t(const PrefillArgs &a, hipStream_t s) {
    switch (a.D) {
        case 64: return launch_d<T, 64>(a, s);
        case 80: return launch_d<T, 80>(a, s);
        case 96: return launch_d<T, 96>(a, s);
        case 128: return launch_d<T, 128>(a, s);
        default: return RG_HIP_E_UNSUPPORTED;
    }
}

}  // namespace

size_t prefill_part_bytes(uint32_t D_) {
    // a launch shares keys only while (items x ranges) stay within the workgroups resident together: two per CU
    return D_ == 64 || D_ == 128 ? static_cast<size_t>(512) * part_floats(D_) * sizeof(float) : 0;
}

bool prefill_supported(uint32_t H, uint32_t Hkv, uint32_t D_) {
    return (D_ == 128 || D_ == 96 || D_ == 80 || D_ == 64) && Hkv != 0 && H % Hkv == 0;
}

int launch_prefill(const PrefillArgs &a, hipStream_t s) {
    if (a.dtype == RG_FP16) return launch_t<__half>(a, s);
    return launch_t<__hip_bfloat16>(a, s);
}

}  // namespace rg
