// Tiled causal attention for many query rows per batch row (prefill), head dim 128, gfx950.
//
// Same contract as the split-KV kernel (layouts of src/08-01llm/README.md:29-63 of the
// reference: q, o [N, H, seq, D]; k, v [N, Hkv, seq, D]; caches [N, Hkv, cap, D]; query row r
// attends positions 0 .. past + r; new rows appended at past .. past + seq - 1).
//
// A workgroup of four wavefronts works on one kv head: wavefront w owns 32 query rows of one of
// the query heads that share this kv head (GQA), so a K/V tile staged once in LDS serves up to
// four query heads.  Keys are walked 32 at a time; a tile of K and V rows is copied from global
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
// the lazily raised reference of the split kernel.  O^T is transposed through LDS at the end so
// that the global stores are 128-bit and row-contiguous.
#include "attention_prefill.hpp"

namespace rg {
namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef __bf16 b8 __attribute__((ext_vector_type(8)));
typedef float f16v __attribute__((ext_vector_type(16)));

constexpr int D = 128;
constexpr int BN = 32;                 // keys per tile (32 or 64); 32 keeps the kernel within the registers and
                                       // LDS of three workgroups per CU, which hides more of the memory latency
constexpr int KB = BN / 32;            // blocks of 32 keys per tile
constexpr int CPI = BN / 16;           // K (and V) copy instructions per wavefront and tile
constexpr int ROWB = 2 * D;            // bytes of a K or V row (unpadded in LDS)
constexpr int TILE = BN * ROWB;        // 16384: one K or V tile
constexpr int BUF_BYTES = 2 * TILE;    // K tile + V tile; two such buffers, reused for the output transposition
constexpr float kSlack = 6.0f;
constexpr float kMinusBig = -1e30f;

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
};

// HW: query heads per workgroup (1, 2 or 4); the other 4 / HW wavefronts take further 32-row
// query sub-tiles of the same heads.
template <class T, int HW>
__global__ __launch_bounds__(256, 3) void attn_prefill(const PrefillArgs a, uint32_t group,
                                                    uint32_t q_tiles, uint32_t head_chunks) {
    constexpr int QS = 4 / HW;      // query sub-tiles per workgroup
    constexpr int ROWS = 32 * QS;   // query rows per workgroup
    __shared__ __align__(1024) uint8_t lds0[BUF_BYTES];
    __shared__ __align__(1024) uint8_t lds1[BUF_BYTES];

    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t half = lane >> 5, l32 = lane & 31;

    // Workgroup order: consecutive workgroup ids are dealt round-robin to the 8 XCDs, so every
    // XCD is given whole (batch row, kv head, head chunk) streams, one after the other and the
    // heaviest query tile (longest key range) of each first.  The query tiles of a stream then
    // run close together on one XCD and find the K/V rows they share in its L2.
    const uint32_t n_rest = a.N * a.Hkv * head_chunks;
    uint32_t rest, qt;
    if (n_rest % 8 == 0) {
        const uint32_t xcd = blockIdx.x % 8, slot = blockIdx.x / 8;
        rest = (slot / q_tiles) * 8 + xcd;
        qt = q_tiles - 1 - slot % q_tiles;
    } else {
        rest = blockIdx.x / q_tiles;
        qt = q_tiles - 1 - blockIdx.x % q_tiles;
    }
    const uint32_t hc = rest % head_chunks;
    rest /= head_chunks;
    const uint32_t kvh = rest % a.Hkv, b = rest / a.Hkv;

    const T *Q = static_cast<const T *>(a.q);
    const T *Kn = static_cast<const T *>(a.k);
    const T *Vn = static_cast<const T *>(a.v);
    T *Kc = static_cast<T *>(a.kc);
    T *Vc = static_cast<T *>(a.vc);
    T *O = static_cast<T *>(a.o);
    const uint64_t kv_head = static_cast<uint64_t>(b) * a.Hkv + kvh;
    const T *k_new = Kn + kv_head * a.seq * D;
    const T *v_new = Vn + kv_head * a.seq * D;
    const T *k_hist = Kc ? Kc + kv_head * a.cap * D : nullptr;
    const T *v_hist = Vc ? Vc + kv_head * a.cap * D : nullptr;

    const uint32_t head = kvh * group + hc * HW + wave % HW;
    const uint32_t r0 = qt * ROWS + 32 * (wave / HW);  // first query row of this wavefront
    const bool wave_active = r0 < a.seq;
    const uint32_t wg_rows_end = (qt + 1) * ROWS < a.seq ? (qt + 1) * ROWS : a.seq;

    // Q fragments (B operand): lane holds query row r0 + l32, d = 16 kk + 8 half .. +7
    Raw16 qf[8];
    {
        const uint32_t qrow = r0 + l32 < a.seq ? r0 + l32 : a.seq - 1;
        const T *qp = Q + ((static_cast<uint64_t>(b) * a.H + head) * a.seq + qrow) * D + 8 * half;
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) qf[kk] = *reinterpret_cast<const Raw16 *>(qp + 16 * kk);
    }

    // history length of this batch row, clamped so that the new rows fit the cache (read after the
    // query loads are on their way: they do not depend on it)
    uint32_t base = 0;
    if (a.kc && a.past) {
        int64_t raw = a.past[a.past_per_row ? b : 0];
        if (raw < 0) raw = 0;
        const int64_t room = static_cast<int64_t>(a.cap) - static_cast<int64_t>(a.seq);
        if (raw > room) raw = room < 0 ? 0 : room;
        base = static_cast<uint32_t>(raw);
    }

    const uint32_t wg_last_key = base + wg_rows_end - 1;  // inclusive
    const uint32_t n_tiles = wg_last_key / BN + 1;
    const uint32_t wave_last_row = r0 + 31 < a.seq ? r0 + 31 : a.seq - 1;
    const uint32_t wave_tiles = wave_active ? (base + wave_last_row) / BN + 1 : 0;
    const uint32_t qpos = base + r0 + l32;  // absolute position of this lane's query row
    const float c_log2e = a.scale * 1.4426950408889634f;

    // Tile copies: wavefront w copies key rows 16 w .. 16 w + 15 of K and of V, four rows (1 KiB)
    // per instruction; this lane brings chunk position lane % 16 of row 16 w + 4 i + lane / 16.
    // A tile that lies inside the history or inside the new rows is addressed as a uniform base
    // plus a per-lane byte offset prepared once (rows of the new tensors beyond the workgroup's last
    // key are read along: they are masked); only a tile that straddles the two tensors or the end
    // of the new rows computes its addresses row by row.
    const uint32_t wave_u = __builtin_amdgcn_readfirstlane(wave);
    const uint32_t cp_row = (BN / 4) * wave_u + (lane >> 4);
    const uint32_t v_lane = cp_row * ROWB + 16 * ((lane & 15) ^ v_swizzle(lane >> 4));
    // K: chunk position lane % 16 of row r holds chunk (lane % 16) ^ (r & 15); rows 4 i further on flip
    // bits 2-3 of the chunk index, i.e. bits 6-7 of the byte offset
    const uint32_t k_lane = cp_row * ROWB + 16 * ((lane & 15) ^ (cp_row & 15));
    const uint32_t total_keys = base + a.seq;
    typedef const __attribute__((address_space(1))) void *GlobalPtr;
    typedef __attribute__((address_space(3))) void *LdsPtr;
    auto copy_tile = [&](uint32_t kt, uint8_t *buf) {
        const uint32_t first = kt * BN;
        const bool in_hist = first + BN <= base, in_new = first >= base && first + BN <= total_keys;
        if (in_hist || in_new) {  // uniform
            const uint64_t tile_off = static_cast<uint64_t>(in_hist ? first : first - base) * ROWB;
            const uint8_t *kb_ = reinterpret_cast<const uint8_t *>(in_hist ? k_hist : k_new) + tile_off;
            const uint8_t *vb_ = reinterpret_cast<const uint8_t *>(in_hist ? v_hist : v_new) + tile_off;
#pragma unroll
            for (int i = 0; i < CPI; ++i) {
                __builtin_amdgcn_global_load_lds((GlobalPtr)(kb_ + ((k_lane ^ (64 * i)) + 4 * i * ROWB)), (LdsPtr)(buf + (CPI * wave_u + i) * 1024), 16, 0, 0);
                __builtin_amdgcn_global_load_lds((GlobalPtr)(vb_ + v_lane + 4 * i * ROWB), (LdsPtr)(buf + TILE + (CPI * wave_u + i) * 1024), 16, 0, 0);
            }
        } else {
#pragma unroll
            for (int i = 0; i < CPI; ++i) {
                uint32_t pos = first + cp_row + 4 * i;
                pos = pos < total_keys ? pos : total_keys - 1;
                const bool old = pos < base;
                const uint64_t row_off = static_cast<uint64_t>(old ? pos : pos - base) * D;
                const uint32_t kc = (lane & 15) ^ ((cp_row + 4 * i) & 15), vc = (lane & 15) ^ v_swizzle(lane >> 4);
                const T *ksrc = (old ? k_hist : k_new) + row_off + 8 * kc;
                const T *vsrc = (old ? v_hist : v_new) + row_off + 8 * vc;
                __builtin_amdgcn_global_load_lds((GlobalPtr)ksrc, (LdsPtr)(buf + (CPI * wave_u + i) * 1024), 16, 0, 0);
                __builtin_amdgcn_global_load_lds((GlobalPtr)vsrc, (LdsPtr)(buf + TILE + (CPI * wave_u + i) * 1024), 16, 0, 0);
            }
        }
    };

    f16v o[4];
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int e = 0; e < 16; ++e) o[db][e] = 0.f;
    float m = 0.f, l = 0.f;
    bool fresh = true;

    copy_tile(0, lds0);
    // query fragments and tile 0 have landed
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();

    // fragment addresses inside a buffer: K row l32 (+ 32 kb), chunk 2 kk + half; V see below
    const uint32_t k_off = l32 * ROWB + 16 * (half ^ (l32 & 15));
    // V piece of block db: row 4 half + r (+ 32 kb + 16 jj, + 8), chunk 4 db + cl; the swizzle leaves
    // 4 db to bits 6-7 of the byte offset, so a block is reached by XOR with 64 db
    const uint32_t s16 = lane & 15, v_r = s16 >> 2, v_cl = 2 * ((lane >> 4) & 1) + ((s16 & 3) >> 1);
    const uint32_t v_off = TILE + (4 * half + v_r) * ROWB + 16 * (v_cl ^ v_swizzle(v_r)) + 8 * (s16 & 1);

    auto tile = [&]<int P>(uint32_t kt) __attribute__((always_inline)) {
        uint8_t *const buf = P ? lds1 : lds0, *const other = P ? lds0 : lds1;
        // The copy of tile kt+1 into the other buffer (free since the barrier that ended tile kt-1)
        // is issued behind this tile's first fragment reads: the compiler waits for every copy in
        // flight before the first read of a buffer that a copy has written, and at that point
        // none is.
        if (kt >= wave_tiles && kt + 1 < n_tiles) copy_tile(kt + 1, other);
        if (kt < wave_tiles) {
            // S^T block kb: keys BN kt + 32 kb + (8 (e/4) + 4 half + e%4), query row l32.  With two
            // blocks per tile (BN = 64) both are issued first; the softmax of a block then runs on
            // the VALU while the matrix core still works on the next product (S^T of block 1, or
            // the PV update of block 0), and a block entirely above the diagonal is skipped.
            const bool second = KB > 1 && kt * BN + 32 <= base + r0 + 31;
            f16v s[KB];
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) {
#pragma unroll
                for (int e = 0; e < 16; ++e) s[kb][e] = 0.f;
                if (kb == 0 || second) {
#pragma unroll
                    for (int kk = 0; kk < 8; ++kk) {
                        const Raw16 kf = *reinterpret_cast<const Raw16 *>(buf + 32 * kb * ROWB + (k_off ^ (32 * kk)));
                        s[kb] = Ops<T>::mfma(kf, qf[kk], s[kb]);
                    }
                }
            }
            if (kt + 1 < n_tiles) copy_tile(kt + 1, other);
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) {
                if (kb == 1 && !second) break;
                // scale, causal mask (only blocks that reach past the wavefront's first query position)
                const bool need_mask = kt * BN + 32 * kb + 31 > base + r0;
                float over = -__builtin_inff();
                if (need_mask) {  // wave-uniform: only the blocks on the diagonal pay for the comparisons
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        const uint32_t key = kt * BN + 32 * kb + 8 * (e / 4) + 4 * half + (e % 4);
                        const float t = key > qpos ? -__builtin_inff() : fmaf(s[kb][e], c_log2e, -m);
                        s[kb][e] = t;
                        over = fmaxf(over, t);
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        const float t = fmaf(s[kb][e], c_log2e, -m);
                        s[kb][e] = t;
                        over = fmaxf(over, t);
                    }
                }
                over = fmaxf(over, __shfl_xor(over, 32, kWave));  // both halves hold the same query row
                if (fresh || __builtin_amdgcn_ballot_w64(over > kSlack) != 0) {
                    const float up = fresh ? fmaxf(over, kMinusBig) : fmaxf(over, 0.f);
                    const float alpha = fresh ? 1.f : __builtin_amdgcn_exp2f(-up);
                    m += up;
                    l *= alpha;
#pragma unroll
                    for (int db = 0; db < 4; ++db)
#pragma unroll
                        for (int e = 0; e < 16; ++e) o[db][e] *= alpha;
#pragma unroll
                    for (int e = 0; e < 16; ++e) s[kb][e] -= up;
                    fresh = false;
                }
                // P^T in B-operand position: element i of MFMA (kb, jj) is accumulator register 8 jj + i
                Raw16 pf[2];
#pragma unroll
                for (int jj = 0; jj < 2; ++jj)
#pragma unroll
                    for (int i2 = 0; i2 < 4; ++i2) {
                        const float p0 = __builtin_amdgcn_exp2f(s[kb][8 * jj + 2 * i2]);
                        const float p1 = __builtin_amdgcn_exp2f(s[kb][8 * jj + 2 * i2 + 1]);
                        l += p0 + p1;
                        pf[jj].w[i2] = Ops<T>::pack2(p0, p1);
                    }
                // O^T block db: rows d = 32 db + l32; A element i of MFMA (kb, jj) is V[key(i), d] with
                // key(i) = 32 kb + 16 jj + (i < 4 ? 4 half + i : 8 + 4 half + i - 4), the key order of pf.
                // A transposing read hands the 16 lanes of a group (16 consecutive d) four consecutive
                // keys each: lane s of the group addresses key s / 4, columns 4 (s % 4) .. +3.
#pragma unroll
                for (int db = 0; db < 4; ++db)
#pragma unroll
                    for (int jj = 0; jj < 2; ++jj) {
                        const uint8_t *vp = buf + (32 * kb + 16 * jj) * ROWB + (v_off ^ (64 * db));
                        const U2 lo = read_tr16(vp), hi = read_tr16(vp + 8 * ROWB);
                        const Raw16 vf{{lo.w[0], lo.w[1], hi.w[0], hi.w[1]}};
                        o[db] = Ops<T>::mfma(vf, pf[jj], o[db]);
                    }
            }
        }

        // This wavefront's copies of tile kt+1 have landed and its reads of this buffer are done;
        // after the barrier that holds for the workgroup.
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
    };
    for (uint32_t kt = 0; kt < n_tiles; kt += 2) {
        tile.template operator()<0>(kt);
        if (kt + 1 < n_tiles) tile.template operator()<1>(kt + 1);
    }

    // The new rows that correspond to this workgroup's query rows are appended to the caches (once
    // per kv head): thread owns 16-byte chunk tid % 16 of rows tid / 16 + 16 j.  The loads are
    // issued here and the stores follow the output write-out, which hides their latency.
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const bool do_append = Kc && hc == 0;
    const uint32_t own_lo = base + qt * ROWS, own_hi = base + wg_rows_end;
    u32x4 ak[ROWS / 16], av[ROWS / 16];
    if (do_append) {
#pragma unroll
        for (int j = 0; j < ROWS / 16; ++j) {
            uint32_t pos = own_lo + (tid >> 4) + 16 * j;
            pos = pos < own_hi ? pos : own_hi - 1;  // loads stay unconditional, the stores are guarded
            const uint64_t off = static_cast<uint64_t>(pos - base) * D + (tid & 15) * 8;
            ak[j] = *reinterpret_cast<const u32x4 *>(k_new + off);
            av[j] = *reinterpret_cast<const u32x4 *>(v_new + off);
        }
    }

    // ---- normalise, transpose O^T -> O through LDS, 128-bit row-contiguous stores
    l += __shfl_xor(l, 32, kWave);
    const float inv = 1.f / l;
    // the K/V tiles are no longer needed (barrier above, no copy in flight): two wavefronts per buffer
    uint8_t *ldsO = (wave & 2 ? lds1 : lds0) + (wave & 1) * (32 * ROWB);  // chunk c of row r at chunk position c ^ (r & 15)
    if (wave_active) {
#pragma unroll
        for (int db = 0; db < 4; ++db)
#pragma unroll
            for (int e = 0; e < 16; e += 2) {
                const uint32_t d = 32 * db + 8 * (e / 4) + 4 * half + (e % 4);
                *reinterpret_cast<uint32_t *>(ldsO + l32 * ROWB + ((2 * d) ^ (16 * (l32 & 15)))) =
                    Ops<T>::pack2(o[db][e] * inv, o[db][e + 1] * inv);
            }
    }
    // (each wavefront reads back only what it wrote itself: no barrier)
    if (wave_active) {
        // computed afresh from an opaque copy of the wavefront index: otherwise the address is built in the
        // prologue, next to the query pointer it resembles, and kept in scratch memory across the tile loop
        uint32_t wave_e = wave;
        asm volatile("" : "+v"(wave_e));
        const uint32_t head_e = kvh * group + hc * HW + wave_e % HW, r0_e = qt * ROWS + 32 * (wave_e / HW);
        T *op = O + ((static_cast<uint64_t>(b) * a.H + head_e) * a.seq + r0_e) * D;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t idx = lane + 64 * i, row = idx / 16, c = idx % 16;
            if (r0 + row < a.seq)
                *reinterpret_cast<Raw16 *>(op + static_cast<uint64_t>(row) * D + c * 8) =
                    *reinterpret_cast<const Raw16 *>(ldsO + row * ROWB + 16 * (c ^ (row & 15)));
        }
    }
    if (do_append) {
#pragma unroll
        for (int j = 0; j < ROWS / 16; ++j) {
            const uint32_t pos = own_lo + (tid >> 4) + 16 * j;
            if (pos < own_hi) {
                const uint64_t dst = (kv_head * a.cap + pos) * D + (tid & 15) * 8;
                *reinterpret_cast<u32x4 *>(Kc + dst) = ak[j];
                *reinterpret_cast<u32x4 *>(Vc + dst) = av[j];
            }
        }
    }
}

template <class T, int HW>
int launch_hw(const PrefillArgs &a, hipStream_t s) {
    const uint32_t group = a.H / a.Hkv;
    const uint32_t head_chunks = group / HW;
    constexpr uint32_t ROWS = 32 * (4 / HW);
    const uint32_t q_tiles = (a.seq + ROWS - 1) / ROWS;
    const uint64_t grid = static_cast<uint64_t>(a.N) * a.Hkv * head_chunks * q_tiles;
    if (grid > 0x7fffffffu) return RG_HIP_E_UNSUPPORTED;
    attn_prefill<T, HW><<<static_cast<unsigned>(grid), 256, 0, s>>>(a, group, q_tiles, head_chunks);
    return launch_status();
}

template <class T>
int launch_t(const PrefillArgs &a, hipStream_t s) {
    const uint32_t group = a.H / a.Hkv;
    if (group % 4 == 0) return launch_hw<T, 4>(a, s);
    if (group == 2) return launch_hw<T, 2>(a, s);
    return launch_hw<T, 1>(a, s);
}

}  // namespace

bool prefill_supported(uint32_t H, uint32_t Hkv, uint32_t D_) {
    const uint32_t group = H / Hkv;
    return D_ == D && (group % 4 == 0 || group == 2 || group == 1);
}

int launch_prefill(const PrefillArgs &a, hipStream_t s) {
    if (a.dtype == RG_FP16) return launch_t<__half>(a, s);
    return launch_t<__hip_bfloat16>(a, s);
}

}  // namespace rg
