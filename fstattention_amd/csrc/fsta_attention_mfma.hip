// Matrix-core tree attention kernel for gfx950: bf16 / fp16, head_dim 32/64/128,
// query blocks of 32/64/128 rows.
//
// One workgroup owns one query block of one (batch, head) slice; each of its
// M/32 waves owns 32 query rows and keeps their state in registers for the whole
// kernel.  The block's own rows (the "leaf" diagonal of reference
// fstattention.py:86-91,104-107: one key per query) never go through LDS: every
// lane dots its Q registers with its own leaf row and seeds the running softmax
// with it.  All other keys are processed in tiles of 32: first the block's unique
// ancestors under the packed tree mask, then the dense shared prefix
// (fstattention.py:113-136).  Work per tile:
//
//   S^T[key, q] = K_tile . Q^T        v_mfma_f32_32x32x16, K fragments from LDS,
//                                     Q fragments loaded once from HBM into VGPRs
//   mask, online softmax (base 2)     in the accumulator layout: a lane holds 16
//                                     keys of ONE query, so row statistics need a
//                                     single cross-lane exchange (lane ^ 32)
//   O^T[d, q] += V_tile^T . P^T       V fragments through ds_read_b64_tr_b16, P^T
//                                     straight from the softmax registers
//
// Computing the transposed products makes the softmax output land exactly in the
// B-operand layout of the second product, so P never touches LDS.  For bf16 the
// weights are fed as a hi+lo pair of bf16 values (two MFMAs) unless
// FSTA_FLAG_FAST_PV asks for one; fp16 weights are precise enough as they are.
// The running maximum is only raised when a row's new maximum exceeds it by more
// than 2^8, so the accumulator rescale is rare; weights stay below 2^8.
//
// K/V rows are gathered from HBM straight into LDS (global_load_lds_dwordx4: 16
// bytes per lane, one row = D*2 bytes = a run of consecutive lanes, no register
// staging).  LDS holds a ring of `stages` tiles; the gathers of the next
// stages-1 tiles are in flight while the current one is multiplied, which is
// what keeps enough bytes outstanding to use HBM.  The tiles are XOR-swizzled by
// choosing which 16-byte chunk of its row a lane fetches.
#include "fsta_common.h"

namespace fsta {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

constexpr int kTileN = 32;     // keys per tile
constexpr int kXcds = 8;       // L2 domains of an MI355X; workgroup i runs on XCD i % 8
constexpr int kMaxStages = 4;  // ring depth limit (LDS per workgroup = stages * 4 * 32 * D bytes)
constexpr float kRescaleSlack = 8.f;  // log2 of the largest weight kept without raising the maximum

template <bool BF16> struct Mma;
template <> struct Mma<true> {
    using elem = __bf16;
    using elem2 = bf16x2;
    using frag = bf16x8;
    static __device__ __forceinline__ f32x16 mfma(frag a, frag b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ float dot2(elem2 a, elem2 b, float c) {
        return __builtin_amdgcn_fdot2_f32_bf16(a, b, c, false);
    }
};
template <> struct Mma<false> {
    using elem = _Float16;
    using elem2 = f16x2;
    using frag = f16x8;
    static __device__ __forceinline__ f32x16 mfma(frag a, frag b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ float dot2(elem2 a, elem2 b, float c) {
        return __builtin_amdgcn_fdot2(a, b, c, false);
    }
};

__host__ __device__ constexpr int anc_tile_capacity(int max_anc) { return (max_anc + kTileN - 1) / kTileN; }

// LDS of one workgroup: ring of K|V tiles, then per ancestor tile 32 sanitised keys,
// one validity word and M mask words.
template <int D, int M>
__host__ __device__ constexpr size_t mfma_lds_bytes(int max_anc, int stages) {
    return (size_t)stages * 2 * kTileN * D * 2 +
           (size_t)anc_tile_capacity(max_anc) * (kTileN * 4 + 4 + M * 4);
}

template <int N> __device__ __forceinline__ void wait_vmcnt() {
    // s_waitcnt immediate on gfx9: vmcnt = [3:0] and [15:14], expcnt = [6:4], lgkmcnt = [11:8];
    // the other two counters are left at "do not wait"
    static_assert(N >= 0 && N < 64, "vmcnt has 6 bits");
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

// Waits until at most `tiles` tiles' worth of this wave's global->LDS transfers
// (kPerTile instructions each, retired in order) are still outstanding.
template <int kPerTile> __device__ __forceinline__ void wait_tiles_outstanding(int tiles) {
    static_assert((kMaxStages - 2) * kPerTile < 64, "ring too deep for vmcnt");
    switch (tiles) {
        case 0: wait_vmcnt<0>(); break;
        case 1: wait_vmcnt<kPerTile>(); break;
        default: wait_vmcnt<2 * kPerTile>(); break;
    }
}

// 32-bit LDS address of a pointer into the dynamic shared segment
__device__ __forceinline__ uint32_t lds_addr(const void* ptr) {
    return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) char*)ptr;
}

// ds_read_b64_tr_b16: within each group of 16 lanes, lane i supplies the address of
// 4 consecutive 16-bit elements (think row i/4, column block i%4 of a 4 x 16 tile)
// and receives element column i of rows 0..3, i.e. component j comes from lane
// 4j + i/4, element i%4.  It is issued as inline assembly on purpose: the compiler
// orders the builtin form behind every outstanding global->LDS transfer
// (s_waitcnt vmcnt(0)), which would drain the gather ring on every tile.  The
// result is only valid after wait_lds() has been applied to it.
__device__ __forceinline__ s16x4 lds_read_tr16(uint32_t addr) {
    s16x4 out;
    asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(out) : "v"(addr) : "memory");
    return out;
}

struct VPair { s16x4 a, b; };   // 8 consecutive k-indices of one A-operand row

// Waits for every outstanding LDS access and ties the fragments to the wait, so no
// use of them can be scheduled ahead of it.
template <int N> __device__ __forceinline__ void wait_lds(VPair (&f)[2][N]);
template <> __device__ __forceinline__ void wait_lds<1>(VPair (&f)[2][1]) {
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(f[0][0].a), "+v"(f[0][0].b), "+v"(f[1][0].a), "+v"(f[1][0].b) :: "memory");
}
template <> __device__ __forceinline__ void wait_lds<2>(VPair (&f)[2][2]) {
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(f[0][0].a), "+v"(f[0][0].b), "+v"(f[0][1].a), "+v"(f[0][1].b),
                   "+v"(f[1][0].a), "+v"(f[1][0].b), "+v"(f[1][1].a), "+v"(f[1][1].b) :: "memory");
}
template <> __device__ __forceinline__ void wait_lds<4>(VPair (&f)[2][4]) {
    asm volatile("s_waitcnt lgkmcnt(0)"
                 : "+v"(f[0][0].a), "+v"(f[0][0].b), "+v"(f[0][1].a), "+v"(f[0][1].b),
                   "+v"(f[0][2].a), "+v"(f[0][2].b), "+v"(f[0][3].a), "+v"(f[0][3].b),
                   "+v"(f[1][0].a), "+v"(f[1][0].b), "+v"(f[1][1].a), "+v"(f[1][1].b),
                   "+v"(f[1][2].a), "+v"(f[1][2].b), "+v"(f[1][3].a), "+v"(f[1][3].b) :: "memory");
}

// 16-byte chunk position of (row, chunk) inside an LDS tile.  K is read as whole
// 16-byte fragments by 32 different rows at once, V as 4-row x 64-byte groups by
// the transposing read; each gets the XOR pattern that spreads its access over
// all 64 banks.
template <int D> __device__ __forceinline__ int k_chunk(int row, int c) {
    constexpr int cpr = D / 8, rpb = 16 / cpr;
    return c ^ ((row / rpb) % cpr);
}
template <int D> __device__ __forceinline__ int v_chunk(int row, int c) {
    constexpr int qpr = D / 32, rpb = 4 / qpr;
    return c ^ (4 * ((row / rpb) % qpr));
}

template <bool BF16, int D, int M, bool SPLIT>
__global__ __launch_bounds__(M * 2, 2) void attn_mfma_kernel(AttnParams p, int stages) {
    using MM = Mma<BF16>;
    using T = typename MM::elem;
    using T2 = typename MM::elem2;
    using Frag = typename MM::frag;
    constexpr int kWaves = M / 32;
    constexpr int kThreads = kWaves * 64;
    constexpr int kCpr = D / 8;                   // 16-byte chunks per row
    constexpr int kRowsPerDma = 64 / kCpr;        // rows one wave-wide 1 KiB transfer covers
    constexpr int kDmaPerTile = 2 * kTileN / kRowsPerDma;   // K and V transfers of one tile
    constexpr int kDmaPerWave = kDmaPerTile / kWaves;
    static_assert(kDmaPerWave * kWaves == kDmaPerTile, "transfers must split evenly over the waves");
    constexpr int kRowGroups = (kDmaPerWave + 1) / 2;   // row groups a wave touches per tile
    constexpr int kSteps = D / 16;                // QK^T MFMAs per tile
    constexpr int kDTiles = D / 32;               // 32-row tiles of O^T
    constexpr int kTileElems = kTileN * D;

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    T* ring = reinterpret_cast<T*>(smem);                 // [stages][K tile | V tile]
    int* key_s = reinterpret_cast<int*>(ring + stages * 2 * kTileElems);
    const int cap = anc_tile_capacity(p.max_anc);                            // listed tiles
    uint32_t* valid_s = reinterpret_cast<uint32_t*>(key_s + cap * kTileN);   // [cap]
    uint32_t* mask_s = valid_s + cap;                                        // [cap][M]

    // Workgroup -> (slice, block): consecutive workgroup ids rotate over the 8
    // XCDs, so give every XCD whole (batch, head) slices; all query blocks of a
    // slice then share one L2 for the K/V rows they have in common.
    const int xcd = blockIdx.x % kXcds;
    const int within = blockIdx.x / kXcds;
    const int hz = (within / p.nb) * kXcds + xcd;
    const int j = within % p.nb;
    if (hz >= p.heads_total) return;

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int ql = lane & 31;        // query (column of S^T / O^T) of this lane
    const int h = lane >> 5;         // which half of the rows of the accumulator tile
    const int row_in_block = wave * 32 + ql;
    const int qrow = j * M + row_in_block;
    const bool q_ok = qrow < p.nq;

    const T* qb = static_cast<const T*>(p.q) + (size_t)hz * p.nq * D;
    const T* kb = static_cast<const T*>(p.k) + (size_t)hz * p.nk * D;
    const T* vb = static_cast<const T*>(p.v) + (size_t)hz * p.nk * D;

    // ---- block metadata: the loads nothing else depends on go out first --------
    int n_anc = p.anc_count ? p.anc_count[j] : p.max_anc;
    const int64_t leaf64 = p.leaf_idx[(size_t)j * M + row_in_block];
    // Sanitised ancestor list.  An empty or out-of-range slot is given the row of the
    // first valid key of its tile (row 0 if the tile has none): the transfer count per
    // tile stays fixed, the slot's mask bits are cleared through valid_s, and the data
    // it brings in is data the tile holds anyway.
    for (int c = tid; c < cap * kTileN; c += kThreads) {
        int64_t idx = -1;
        if (c < p.max_anc) idx = p.ancestor_idx[(size_t)j * p.max_anc + c];
        const bool ok = idx >= 0 && idx < p.nk;
        const uint64_t vote = __ballot(ok);
        const uint32_t mine = (uint32_t)(vote >> (lane & 32));
        const int first = mine ? (lane & 32) + __ffs(mine) - 1 : lane;
        const int fallback = __shfl(ok ? (int)idx : 0, first);
        key_s[c] = ok ? (int)idx : fallback;
        if ((lane & 31) == 0) valid_s[c >> 5] = mine;
    }
    {
        const uint32_t* src = p.mask_bits + (size_t)j * p.mask_words * M;
        for (int e = tid; e < p.mask_words * M; e += kThreads) mask_s[e] = src[e];
    }
    n_anc = min(max(n_anc, 0), p.max_anc);
    const int listed_tiles = (n_anc + kTileN - 1) / kTileN;
    const int total_tiles = listed_tiles + (p.prefix + kTileN - 1) / kTileN;
    const int ahead = stages - 1;   // tiles kept in flight beyond the one in use
    __syncthreads();

    // ---- gather: HBM -> LDS, 16 bytes per lane, no registers in between --------
    // Transfer g of a tile moves row group g/2 = rows [kRowsPerDma*(g/2), +kRowsPerDma) of K
    // (g even) or V (g odd); wave w issues transfers [w*kDmaPerWave, +kDmaPerWave).  Lane i
    // lands at LDS byte 16*i of the transfer, i.e. row i / kCpr, chunk slot i % kCpr, and
    // fetches the chunk that the XOR swizzle assigns to that slot.  Every wave issues exactly
    // kDmaPerWave transfers per tile: the vmcnt bookkeeping below counts on it.
    const int dma_row = lane / kCpr, dma_slot = lane % kCpr;
    auto issue = [&](int t, int stage) {
        T* dst_tile = ring + stage * 2 * kTileElems;
        int rows[kRowGroups];
#pragma unroll
        for (int i = 0; i < kRowGroups; ++i) {
            const int r = ((wave * kDmaPerWave) / 2 + i) * kRowsPerDma + dma_row;
            if (t < listed_tiles) rows[i] = key_s[t * kTileN + r];
            else rows[i] = min((t - listed_tiles) * kTileN + r, p.prefix - 1);
        }
#pragma unroll
        for (int i = 0; i < kDmaPerWave; ++i) {
            const int g = wave * kDmaPerWave + i;
            const int u = g >> 1;
            const bool is_v = g & 1;
            const int r = u * kRowsPerDma + dma_row;
            const size_t row_off = (size_t)rows[u - (wave * kDmaPerWave) / 2] * D;
            const T* src = is_v ? vb + row_off + v_chunk<D>(r, dma_slot) * 8
                                : kb + row_off + k_chunk<D>(r, dma_slot) * 8;
            __builtin_amdgcn_global_load_lds(
                (const void __attribute__((address_space(1)))*)src,
                (void __attribute__((address_space(3)))*)(dst_tile + (is_v ? kTileElems : 0) + u * 512),
                16, 0, 0);
        }
    };
    for (int t = 0; t < ahead; ++t)
        if (t < total_tiles) issue(t, t);

    // ---- Q fragments: B operand of S^T = K.Q^T, lane holds Q[q][16s + 8h .. +7] --
    Frag qf[kSteps];
#pragma unroll
    for (int s = 0; s < kSteps; ++s) {
        u32x4 raw = {0u, 0u, 0u, 0u};
        if (q_ok) raw = *reinterpret_cast<const u32x4*>(qb + (size_t)qrow * D + 16 * s + 8 * h);
        qf[s] = __builtin_bit_cast(Frag, raw);
    }

    // ---- leaf (diagonal) path seeds the running softmax -----------------------
    // reference fstattention.py:86-91,104-107: row r also attends to K/V row leaf_idx[j, r].
    // One key per query: every lane dots its Q registers with its own row, no LDS.
    float m_i = -INFINITY, l_i = 0.f;
    f32x16 o[kDTiles];
    {
        const bool leaf_ok = leaf64 >= 0 && leaf64 < p.nk;
        const size_t leaf = leaf_ok ? (size_t)leaf64 : 0;
        u32x4 kraw[kSteps];
        u32x2 vraw[kDTiles][4];
#pragma unroll
        for (int s = 0; s < kSteps; ++s) {
            kraw[s] = u32x4{0u, 0u, 0u, 0u};
            if (leaf_ok) kraw[s] = *reinterpret_cast<const u32x4*>(kb + leaf * D + 16 * s + 8 * h);
        }
#pragma unroll
        for (int dt = 0; dt < kDTiles; ++dt)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                // accumulator rows 8g + 4h .. +3 of tile dt are 4 consecutive head dims
                vraw[dt][g] = u32x2{0u, 0u};
                if (leaf_ok) vraw[dt][g] = *reinterpret_cast<const u32x2*>(vb + leaf * D + 32 * dt + 8 * g + 4 * h);
            }
        float part = 0.f;
#pragma unroll
        for (int s = 0; s < kSteps; ++s) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const T2 a = {qf[s][2 * e], qf[s][2 * e + 1]};
                const Frag kf = __builtin_bit_cast(Frag, kraw[s]);
                const T2 b = {kf[2 * e], kf[2 * e + 1]};
                part = MM::dot2(a, b, part);
            }
        }
        const float dot = part + __shfl_xor(part, 32);
        if (leaf_ok) { m_i = dot * p.scale_log2e; l_i = h == 0 ? 1.f : 0.f; }
#pragma unroll
        for (int dt = 0; dt < kDTiles; ++dt)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                typedef T t4 __attribute__((ext_vector_type(4)));
                const t4 vv = __builtin_bit_cast(t4, vraw[dt][g]);
#pragma unroll
                for (int e = 0; e < 4; ++e) o[dt][4 * g + e] = (float)vv[e];
            }
    }

    int stage = 0;                      // ring slot of tile t
    int fill = ahead % stages;          // ring slot the next issued tile goes to (= slot of tile t-1)
    for (int t = 0; t < total_tiles; ++t) {
        // tile t has landed once at most the transfers of the tiles issued after it are outstanding
        wait_tiles_outstanding<kDmaPerWave>(min(total_tiles - 1 - t, ahead - 1));
        __syncthreads();   // everyone's share of tile t is in LDS; everyone is done with tile t-1
        if (t + ahead < total_tiles) issue(t + ahead, fill);
        const T* kt = ring + stage * 2 * kTileElems;
        const T* vt = kt + kTileElems;
        fill = stage;
        stage = stage + 1 == stages ? 0 : stage + 1;

        uint32_t word;
        if (t < listed_tiles) {
            word = mask_s[t * M + row_in_block] & valid_s[t];
        } else {
            const int left = p.prefix - (t - listed_tiles) * kTileN;
            word = left >= 32 ? 0xffffffffu : ((1u << left) - 1u);
        }
        if (__ballot(word != 0u) == 0ull) continue;   // none of this wave's queries attends to the tile

        // S^T = K_tile . Q^T
        f32x16 s;
#pragma unroll
        for (int r = 0; r < 16; ++r) s[r] = 0.f;
#pragma unroll
        for (int ks = 0; ks < kSteps; ++ks) {
            const u32x4 raw = *reinterpret_cast<const u32x4*>(kt + ql * D + k_chunk<D>(ql, 2 * ks + h) * 8);
            s = MM::mfma(__builtin_bit_cast(Frag, raw), qf[ks], s);
        }
        // V fragments (A operand of O^T += V^T.P^T: rows are head dims) through the
        // transposing read; issued now so that LDS latency hides behind the softmax
        VPair vfrag[2][kDTiles];
        {
            const int tr_row = (lane & 15) >> 2;                          // key within a group of 4
            const int tr_col = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);   // head dim within the 32-row tile
#pragma unroll
            for (int kk = 0; kk < 2; ++kk) {
#pragma unroll
                for (int dt = 0; dt < kDTiles; ++dt) {
                    const int col = 32 * dt + tr_col;
                    const int r0 = 16 * kk + 4 * h + tr_row;      // keys 16kk+4h .. +3
                    const int r1 = r0 + 8;                         // keys 16kk+8+4h .. +3
                    vfrag[kk][dt].a = lds_read_tr16(lds_addr(vt + r0 * D + v_chunk<D>(r0, col >> 3) * 8 + (col & 7)));
                    vfrag[kk][dt].b = lds_read_tr16(lds_addr(vt + r1 * D + v_chunk<D>(r1, col >> 3) * 8 + (col & 7)));
                }
            }
        }
        // mask + online softmax; accumulator register r is key 8*(r/4) + 4h + r%4
        const uint32_t wsh = word >> (4 * h);
        float sv[16];
        float mx = -INFINITY;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const bool on = (wsh >> (8 * (r / 4) + (r % 4))) & 1u;
            sv[r] = on ? s[r] * p.scale_log2e : -INFINITY;
            mx = fmaxf(mx, sv[r]);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        // Raise the running maximum only for rows that would otherwise produce a weight
        // above 2^kRescaleSlack (always when the row had no key so far); rare after the
        // first tiles, so the rescale of the accumulators is a wave-uniform branch.
        const bool raise = mx > m_i + kRescaleSlack || (m_i == -INFINITY && mx > -INFINITY);
        if (__ballot(raise) != 0ull) {
            const float alpha = raise ? __builtin_amdgcn_exp2f(m_i - mx) : 1.f;   // exp2(-inf) = 0
            if (raise) m_i = mx;
            l_i *= alpha;
#pragma unroll
            for (int dt = 0; dt < kDTiles; ++dt)
#pragma unroll
                for (int r = 0; r < 16; ++r) o[dt][r] *= alpha;
        }
        const float m_safe = m_i == -INFINITY ? 0.f : m_i;
        float rowsum = 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            sv[r] = __builtin_amdgcn_exp2f(sv[r] - m_safe);
            rowsum += sv[r];
        }
        l_i += rowsum;
        // P^T fragments: registers 8kk .. 8kk+7 are the 8 k-indices this lane feeds to MFMA kk
        Frag ph[2], pl[2];
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
#pragma unroll
            for (int e = 0; e < 8; e += 2) {
                const f32x2 w = {sv[8 * kk + e], sv[8 * kk + e + 1]};
                const T2 hi = __builtin_convertvector(w, T2);
                ph[kk][e] = hi[0];
                ph[kk][e + 1] = hi[1];
                if (SPLIT) {
                    const f32x2 rest = w - __builtin_convertvector(hi, f32x2);
                    const T2 lo = __builtin_convertvector(rest, T2);
                    pl[kk][e] = lo[0];
                    pl[kk][e + 1] = lo[1];
                }
            }
        }
        // O^T += V_tile^T . P^T ; hi weights of all head-dim tiles first, then lo, so that
        // MFMAs on the same accumulator are several instructions apart
        wait_lds(vfrag);
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
#pragma unroll
            for (int dt = 0; dt < kDTiles; ++dt)
                o[dt] = MM::mfma(__builtin_bit_cast(Frag, vfrag[kk][dt]), ph[kk], o[dt]);
            if (SPLIT) {
#pragma unroll
                for (int dt = 0; dt < kDTiles; ++dt)
                    o[dt] = MM::mfma(__builtin_bit_cast(Frag, vfrag[kk][dt]), pl[kk], o[dt]);
            }
        }
    }

    // ---- epilogue: normalise, write O once (and the base-2 log-sum-exp) --------
    const float l_tot = l_i + __shfl_xor(l_i, 32);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    if (q_ok) {
        if (p.lse && h == 0)
            p.lse[(size_t)hz * p.nq + qrow] = l_tot > 0.f ? m_i + log2f(l_tot) : -INFINITY;
        const size_t base = ((size_t)hz * p.nq + qrow) * D;
#pragma unroll
        for (int dt = 0; dt < kDTiles; ++dt) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                // accumulator rows 8g + 4h .. +3 of tile dt are 4 consecutive head dims
                const int d = 32 * dt + 8 * g + 4 * h;
                float4 val;
                val.x = o[dt][4 * g + 0] * inv;
                val.y = o[dt][4 * g + 1] * inv;
                val.z = o[dt][4 * g + 2] * inv;
                val.w = o[dt][4 * g + 3] * inv;
                if (p.out_f32) {
                    *reinterpret_cast<float4*>(static_cast<float*>(p.o) + base + d) = val;
                } else {
                    typedef T t4 __attribute__((ext_vector_type(4)));
                    const T2 lo = __builtin_convertvector((f32x2){val.x, val.y}, T2);
                    const T2 hi = __builtin_convertvector((f32x2){val.z, val.w}, T2);
                    t4 packed;
                    packed[0] = lo[0]; packed[1] = lo[1]; packed[2] = hi[0]; packed[3] = hi[1];
                    *reinterpret_cast<t4*>(static_cast<T*>(p.o) + base + d) = packed;
                }
            }
        }
    }
}

template <bool BF16, int D, int M, bool SPLIT>
int launch_one(const AttnParams& p, hipStream_t stream) {
    // ring depth: everything in flight at once for short tile lists, else the limit
    const int tiles = anc_tile_capacity(p.max_anc) + (p.prefix + kTileN - 1) / kTileN;
    int stages = tiles < 2 ? 2 : (tiles > kMaxStages ? kMaxStages : tiles);
    size_t lds = mfma_lds_bytes<D, M>(p.max_anc, stages);
    while (lds > 160 * 1024 && stages > 2) lds = mfma_lds_bytes<D, M>(p.max_anc, --stages);
    if (lds > 160 * 1024)
        return fail(FSTA_EUNSUPPORTED, "max_ancestors=%d needs %zu bytes of LDS (limit 163840)", p.max_anc, lds);
    if (lds > 64 * 1024)
        FSTA_HIP_OK(hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_mfma_kernel<BF16, D, M, SPLIT>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    const int slices_per_xcd = (p.heads_total + kXcds - 1) / kXcds;
    const unsigned grid = (unsigned)(kXcds * slices_per_xcd * p.nb);
    hipLaunchKernelGGL((attn_mfma_kernel<BF16, D, M, SPLIT>), dim3(grid), dim3(M * 2), lds, stream, p, stages);
    FSTA_HIP_OK(hipGetLastError());
    return FSTA_OK;
}

template <bool BF16, int D, bool SPLIT>
int launch_m(const AttnParams& p, hipStream_t stream) {
    switch (p.block_m) {
        case 32: return launch_one<BF16, D, 32, SPLIT>(p, stream);
        case 64: return launch_one<BF16, D, 64, SPLIT>(p, stream);
        case 128: return launch_one<BF16, D, 128, SPLIT>(p, stream);
    }
    return fail(FSTA_EUNSUPPORTED, "matrix-core kernel: block_m=%d", p.block_m);
}

template <bool BF16, bool SPLIT>
int launch_d(const AttnParams& p, int head_dim, hipStream_t stream) {
    switch (head_dim) {
        case 32: return launch_m<BF16, 32, SPLIT>(p, stream);
        case 64: return launch_m<BF16, 64, SPLIT>(p, stream);
        case 128: return launch_m<BF16, 128, SPLIT>(p, stream);
    }
    return fail(FSTA_EUNSUPPORTED, "matrix-core kernel: head_dim=%d", head_dim);
}

}  // namespace

bool mfma_supported(int dtype, int head_dim, int block_m) {
    return (dtype == FSTA_F16 || dtype == FSTA_BF16) &&
           (head_dim == 32 || head_dim == 64 || head_dim == 128) &&
           (block_m == 32 || block_m == 64 || block_m == 128);
}

int launch_attention_mfma(const AttnParams& p, int dtype, int head_dim, bool fast_pv, hipStream_t stream) {
    if (dtype == FSTA_F16) return launch_d<false, false>(p, head_dim, stream);
    if (fast_pv) return launch_d<true, false>(p, head_dim, stream);
    return launch_d<true, true>(p, head_dim, stream);
}

}  // namespace fsta
