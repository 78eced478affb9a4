// Matrix-core tree attention kernel for gfx950: bf16 / fp16, head_dim 32/64/128,
// query blocks of 32/64/128 rows.
//
// One workgroup owns one query block of one (batch, head) slice; each of its
// M/32 waves owns 32 query rows and keeps their state in registers for the whole
// kernel.  Work per 32-key tile:
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
//
// K/V rows are gathered from HBM straight into LDS (global_load_lds_dwordx4: 16
// bytes per lane, one row = D*2 bytes = a run of consecutive lanes, no register
// staging).  LDS holds a ring of STAGES tiles; the gathers of the next STAGES-1
// tiles are in flight while the current one is multiplied, which is what keeps
// enough bytes outstanding to use HBM.  The tiles are XOR-swizzled by choosing
// which 16-byte chunk of its row a lane fetches.  The block's own rows (the
// "leaf" diagonal of reference fstattention.py:86-91,104-107) never go through
// LDS: every lane dots its Q registers with its own leaf row and seeds the
// running softmax with it.
#include "fsta_common.h"

namespace fsta {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

constexpr int kTileN = 32;   // keys per tile
constexpr int kXcds = 8;     // L2 domains of an MI355X; workgroup i runs on XCD i % 8

template <bool BF16> struct Mma;
template <> struct Mma<true> {
    using elem = __bf16;
    using frag = bf16x8;
    static __device__ __forceinline__ f32x16 mfma(frag a, frag b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ float to_f32(elem x) { return (float)x; }
};
template <> struct Mma<false> {
    using elem = _Float16;
    using frag = f16x8;
    static __device__ __forceinline__ f32x16 mfma(frag a, frag b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ float to_f32(elem x) { return (float)x; }
};

__host__ __device__ constexpr int anc_tile_capacity(int max_anc) { return (max_anc + kTileN - 1) / kTileN; }

template <int D, int M, int STAGES>
__host__ __device__ constexpr size_t mfma_lds_bytes(int max_anc) {
    // ring of K|V tiles, then per ancestor tile: 32 sanitised keys, one validity word, M mask words
    return (size_t)STAGES * 2 * kTileN * D * 2 + (size_t)anc_tile_capacity(max_anc) * (kTileN * 4 + 4 + M * 4);
}

template <int N> __device__ __forceinline__ void wait_vmcnt() {
    // s_waitcnt immediate on gfx9: vmcnt = [3:0] and [15:14], expcnt = [6:4], lgkmcnt = [11:8];
    // the other two counters are left at "do not wait"
    static_assert(N >= 0 && N < 64, "vmcnt has 6 bits");
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
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

constexpr int stages_for(int block_m) { return block_m == 128 ? 4 : 3; }

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
__global__ __launch_bounds__(M * 2, 2) void attn_mfma_kernel(AttnParams p) {
    using MM = Mma<BF16>;
    using T = typename MM::elem;
    using Frag = typename MM::frag;
    constexpr int kStages = stages_for(M);
    constexpr int kAhead = kStages - 1;           // tiles in flight beyond the one being used
    constexpr int kWaves = M / 32;
    constexpr int kThreads = kWaves * 64;
    constexpr int kCpr = D / 8;                   // 16-byte chunks per row
    constexpr int kRowsPerDma = 64 / kCpr;        // rows one wave-wide 1 KiB transfer covers
    constexpr int kDmaPerTile = 2 * kTileN / kRowsPerDma;   // K and V transfers of one tile
    constexpr int kDmaPerWave = kDmaPerTile / kWaves;
    static_assert(kDmaPerWave * kWaves == kDmaPerTile, "transfers must split evenly over the waves");
    constexpr int kSteps = D / 16;                // QK^T MFMAs per tile
    constexpr int kDTiles = D / 32;               // 32-row tiles of O^T
    constexpr int kTileElems = kTileN * D;

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    T* ring = reinterpret_cast<T*>(smem);                 // [kStages][K tile | V tile]
    int* key_s = reinterpret_cast<int*>(ring + kStages * 2 * kTileElems);
    const int cap = anc_tile_capacity(p.max_anc);
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

    int n_anc = p.anc_count ? p.anc_count[j] : p.max_anc;
    n_anc = min(max(n_anc, 0), p.max_anc);
    const int anc_tiles = (n_anc + kTileN - 1) / kTileN;
    const int prefix_tiles = (p.prefix + kTileN - 1) / kTileN;
    const int total_tiles = anc_tiles + prefix_tiles;

    // ---- everything that does not depend on other loads goes out first ---------
    const int64_t leaf64 = p.leaf_idx[(size_t)j * M + row_in_block];
    // Q fragments: B operand of S^T = K.Q^T, lane holds Q[q][16s + 8h .. +7]
    Frag qf[kSteps];
#pragma unroll
    for (int s = 0; s < kSteps; ++s) {
        u32x4 raw = {0u, 0u, 0u, 0u};
        if (q_ok) raw = *reinterpret_cast<const u32x4*>(qb + (size_t)qrow * D + 16 * s + 8 * h);
        qf[s] = __builtin_bit_cast(Frag, raw);
    }
    // sanitised ancestor list, per-tile validity words, this block's mask words
    for (int c = tid; c < anc_tiles * kTileN; c += kThreads) {
        int64_t idx = -1;
        if (c < n_anc) idx = p.ancestor_idx[(size_t)j * p.max_anc + c];
        const bool ok = idx >= 0 && idx < p.nk;
        key_s[c] = ok ? (int)idx : -1;
        const uint64_t vote = __ballot(ok);
        if (lane == 0) valid_s[c >> 5] = (uint32_t)vote;
        if (lane == 32) valid_s[c >> 5] = (uint32_t)(vote >> 32);
    }
    {
        const uint32_t* src = p.mask_bits + (size_t)j * p.mask_words * M;
        for (int e = tid; e < anc_tiles * M; e += kThreads) mask_s[e] = src[e];
    }
    // Rows of a partly filled tile are not transferred; whatever a V buffer holds
    // there meets a weight of exactly 0, so it only has to be finite: start from zeros.
    for (int e = tid; e < kStages * kTileElems / 8; e += kThreads) {
        const int stage = e / (kTileElems / 8), off = e % (kTileElems / 8);
        *reinterpret_cast<u32x4*>(ring + (stage * 2 + 1) * kTileElems + off * 8) = u32x4{0u, 0u, 0u, 0u};
    }
    __syncthreads();

    // ---- gather: HBM -> LDS, 16 bytes per lane, no registers in between --------
    // Transfer g of a tile moves rows [kRowsPerDma*u, +kRowsPerDma) of K (g < half) or V.
    // Lane i lands at LDS byte 16*i of the transfer, i.e. row i / kCpr, chunk slot i % kCpr;
    // it fetches the chunk that the XOR swizzle assigns to that slot.
    auto issue = [&](int t) {
        T* stage = ring + (t % kStages) * 2 * kTileElems;
#pragma unroll
        for (int i = 0; i < kDmaPerWave; ++i) {
            const int g = wave * kDmaPerWave + i;
            const bool is_v = g >= kDmaPerTile / 2;
            const int u = is_v ? g - kDmaPerTile / 2 : g;
            const int r = u * kRowsPerDma + lane / kCpr;
            const int slot = lane % kCpr;
            int row;
            if (t < anc_tiles) row = key_s[t * kTileN + r];
            else { row = (t - anc_tiles) * kTileN + r; if (row >= p.prefix) row = -1; }
            const int c = is_v ? v_chunk<D>(r, slot) : k_chunk<D>(r, slot);
            const T* src = (is_v ? vb : kb) + (size_t)max(row, 0) * D + c * 8;
            T* dst = stage + (is_v ? kTileElems : 0) + u * 512;
            if (row >= 0)
                __builtin_amdgcn_global_load_lds(
                    (const void __attribute__((address_space(1)))*)src,
                    (void __attribute__((address_space(3)))*)dst, 16, 0, 0);
        }
    };

    // ---- leaf (diagonal) path seeds the running softmax -----------------------
    // reference fstattention.py:86-91,104-107: row r also attends to K/V row leaf_idx[j, r]
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
        // the first tiles start moving before the leaf rows are used
#pragma unroll
        for (int t = 0; t < kAhead; ++t)
            if (t < total_tiles) issue(t);

        float part = 0.f;
#pragma unroll
        for (int s = 0; s < kSteps; ++s) {
            const Frag kf = __builtin_bit_cast(Frag, kraw[s]);
#pragma unroll
            for (int e = 0; e < 8; ++e) part += MM::to_f32(qf[s][e]) * MM::to_f32(kf[e]);
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
                for (int e = 0; e < 4; ++e) o[dt][4 * g + e] = MM::to_f32(vv[e]);
            }
    }

    for (int t = 0; t < total_tiles; ++t) {
        // tile t has landed once at most the transfers of the tiles behind it are outstanding
        if (total_tiles - 1 - t >= kAhead - 1) wait_vmcnt<(kAhead - 1) * kDmaPerWave>();
        else wait_vmcnt<0>();
        __syncthreads();   // everyone's share of tile t is in LDS; everyone is done with tile t-1
        if (t + kAhead < total_tiles) issue(t + kAhead);   // reuses the buffer of tile t-1

        const T* kt = ring + (t % kStages) * 2 * kTileElems;
        const T* vt = kt + kTileElems;
        uint32_t word;
        if (t < anc_tiles) {
            word = mask_s[t * M + row_in_block] & valid_s[t];
        } else {
            const int left = p.prefix - (t - anc_tiles) * kTileN;
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
        const float m_new = fmaxf(m_i, mx);
        const float m_safe = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = __builtin_amdgcn_exp2f(m_i - m_safe);
        float rowsum = 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            sv[r] = __builtin_amdgcn_exp2f(sv[r] - m_safe);
            rowsum += sv[r];
        }
        l_i = l_i * alpha + rowsum;
        m_i = m_new;
        if (__ballot(alpha != 1.f) != 0ull) {
#pragma unroll
            for (int dt = 0; dt < kDTiles; ++dt)
#pragma unroll
                for (int r = 0; r < 16; ++r) o[dt][r] *= alpha;
        }
        // P^T fragments: registers 8kk .. 8kk+7 are the 8 k-indices this lane feeds to MFMA kk
        Frag ph[2], pl[2];
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float w = sv[8 * kk + e];
                const T hi = (T)w;
                ph[kk][e] = hi;
                if (SPLIT) pl[kk][e] = (T)(w - MM::to_f32(hi));
            }
        }
        // O^T += V_tile^T . P^T ; hi weights of all head-dim tiles first, then lo, so that
        // MFMAs on the same accumulator are four instructions apart
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
                    t4 packed;
                    packed[0] = (T)val.x; packed[1] = (T)val.y; packed[2] = (T)val.z; packed[3] = (T)val.w;
                    *reinterpret_cast<t4*>(static_cast<T*>(p.o) + base + d) = packed;
                }
            }
        }
    }
}

template <bool BF16, int D, int M, bool SPLIT>
int launch_one(const AttnParams& p, hipStream_t stream) {
    const size_t lds = mfma_lds_bytes<D, M, stages_for(M)>(p.max_anc);
    if (lds > 160 * 1024)
        return fail(FSTA_EUNSUPPORTED, "max_ancestors=%d needs %zu bytes of LDS (limit 163840)", p.max_anc, lds);
    if (lds > 64 * 1024)
        FSTA_HIP_OK(hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_mfma_kernel<BF16, D, M, SPLIT>),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    const int slices_per_xcd = (p.heads_total + kXcds - 1) / kXcds;
    const unsigned grid = (unsigned)(kXcds * slices_per_xcd * p.nb);
    hipLaunchKernelGGL((attn_mfma_kernel<BF16, D, M, SPLIT>), dim3(grid), dim3(M * 2), lds, stream, p);
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
