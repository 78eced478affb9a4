// Matrix-core tree attention kernel for gfx950: bf16 / fp16, head_dim 32/64/128,
// query blocks of 32/64/128 rows.
//
// One workgroup owns one query block of one (batch, head) slice; each of its
// M/32 waves owns 32 query rows and keeps their state in registers for the whole
// kernel.  Keys come in tiles of 32 rows, gathered through LDS.  The tile list is
//
//   [ M/32 leaf tiles | ancestor tiles | shared-prefix tiles ]
//
// Leaf tile w holds K/V rows leaf_idx[j, 32w .. 32w+31] (the diagonal of reference
// fstattention.py:86-91,104-107: one key per query); wave w takes one dot product
// per query from it on the vector ALU and seeds its running softmax.  Ancestor
// tiles carry the packed tree mask, prefix tiles are dense
// (fstattention.py:113-136); work per such tile:
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
#include "fsta_mfma_common.h"

namespace fsta {
namespace {

using namespace mfma;

// Key-split factor: how many waves share one group of 32 query rows, each taking every
// KS-th tile with its own running softmax; the partial results are merged through LDS at
// the end.  Blocks of 64 and 32 rows would otherwise run on 2 or 1 waves.
constexpr int key_split_for(int block_m) { return block_m >= 128 ? 1 : 2; }
// Leaf tiles consumed per step (each by a different wave).
constexpr int leaf_group_for(int block_m) { return block_m >= 64 ? 2 : 1; }

template <bool BF16, int D, int M, bool SPLIT>
__global__ __launch_bounds__(M * 2 * key_split_for(M), 2) void attn_mfma_kernel(AttnParams p, int stages) {
    using MM = Mma<BF16>;
    using T = typename MM::elem;
    using T2 = typename MM::elem2;
    using Frag = typename MM::frag;
    constexpr int kQGroups = M / 32;              // groups of 32 query rows
    constexpr int kSplit = key_split_for(M);
    constexpr int kLeafGroup = leaf_group_for(M);
    constexpr int kWaves = kQGroups * kSplit;
    constexpr int kThreads = kWaves * 64;
    constexpr int kCpr = D / 8;                   // 16-byte chunks per row
    constexpr int kRowsPerDma = 64 / kCpr;        // rows one wave-wide 1 KiB transfer covers
    constexpr int kDmaPerTile = 2 * kTileN / kRowsPerDma;   // K and V transfers of one tile
    constexpr int kDmaWaves = kDmaPerTile < kWaves ? kDmaPerTile : kWaves;   // waves that gather
    constexpr int kDmaPerWave = kDmaPerTile / kDmaWaves;
    static_assert(kDmaPerWave * kDmaWaves == kDmaPerTile, "transfers must split evenly over the waves");
    constexpr int kRowGroups = (kDmaPerWave + 1) / 2;   // row groups a wave touches per tile
    constexpr int kSteps = D / 16;                // QK^T MFMAs per tile
    constexpr int kDTiles = D / 32;               // 32-row tiles of O^T
    constexpr int kTileElems = kTileN * D;

    // (all kernel arguments in one batch of scalar loads instead of one round trip per first use)
    asm volatile("" ::"s"(p.q), "s"(p.k), "s"(p.v), "s"(p.o), "s"(p.lse), "s"(p.ancestor_idx), "s"(p.mask_bits),
                 "s"(p.anc_count), "s"(p.leaf_idx), "s"(p.nq), "s"(p.nk), "s"(p.prefix), "s"(p.max_anc),
                 "s"(p.mask_words), "s"(p.nb), "s"(p.heads_total), "s"(p.out_f32), "s"(p.scale_log2e), "s"(stages));
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    T* ring = reinterpret_cast<T*>(smem);                 // [stages][K tile | V tile]
    int* key_s = reinterpret_cast<int*>(ring + stages * 2 * kTileElems);
    const int cap = kQGroups + anc_tile_capacity(p.max_anc);                 // listed tiles
    uint32_t* valid_s = reinterpret_cast<uint32_t*>(key_s + cap * kTileN);   // [cap]
    uint32_t* mask_s = valid_s + ((cap + 3) & ~3);                           // [ancestor tiles][M], 16-byte aligned

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
    const int qgroup = wave % kQGroups;   // which 32 query rows
    const int split = wave / kQGroups;    // which share of the tiles
    const int lane = tid & 63;
    const int ql = lane & 31;        // query (column of S^T / O^T) of this lane
    const int h = lane >> 5;         // which half of the rows of the accumulator tile
    const int row_in_block = qgroup * 32 + ql;
    const int qrow = j * M + row_in_block;
    const bool q_ok = qrow < p.nq;

    const T* qb = static_cast<const T*>(p.q) + (size_t)hz * p.nq * D;
    const T* kb = static_cast<const T*>(p.k) + (size_t)hz * p.nk * D;
    const T* vb = static_cast<const T*>(p.v) + (size_t)hz * p.nk * D;

    // ---- block metadata: the loads nothing else depends on go out first --------
    int n_anc = p.anc_count ? p.anc_count[j] : p.max_anc;
    const int64_t leaf64 = p.leaf_idx[(size_t)j * M + row_in_block];
    const bool leaf_ok = leaf64 >= 0 && leaf64 < p.nk;
    // This block's mask words go to LDS as they are: a straight global->LDS copy, 16 bytes
    // per lane, the 1 KiB pieces dealt round-robin to the waves.
    {
        const int mask_bytes = p.mask_words * M * 4;   // multiple of 128
        const char* src = reinterpret_cast<const char*>(p.mask_bits) + (size_t)j * mask_bytes;
        for (int piece = wave; piece * 1024 < mask_bytes; piece += kWaves) {
            if (piece * 1024 + lane * 16 < mask_bytes)
                __builtin_amdgcn_global_load_lds(
                    (const void __attribute__((address_space(1)))*)(src + piece * 1024 + lane * 16),
                    (void __attribute__((address_space(3)))*)(reinterpret_cast<char*>(mask_s) + piece * 1024),
                    16, 0, 0);
        }
    }
    // Sanitised key lists: the block's M leaf slots (tiles 0 .. kQGroups-1), then the
    // ancestor slots.  An empty or out-of-range slot is given the row of the first valid
    // key of its tile (row 0 if the tile has none): the transfer count per tile stays
    // fixed, the slot's mask bits are cleared through valid_s, and the data it brings in
    // is data the tile holds anyway.  The ids are requested kKeyBatch at a time before any
    // is used, so the list costs one memory round trip, not one per pass.
    constexpr int kKeyBatch = 4;
    for (int c0 = tid; c0 < cap * kTileN; c0 += kKeyBatch * kThreads) {
        int64_t ids[kKeyBatch];
#pragma unroll
        for (int i = 0; i < kKeyBatch; ++i) {
            const int c = c0 + i * kThreads;
            ids[i] = -1;
            if (c < M) ids[i] = p.leaf_idx[(size_t)j * M + c];
            else if (c - M < p.max_anc) ids[i] = p.ancestor_idx[(size_t)j * p.max_anc + (c - M)];
        }
#pragma unroll
        for (int i = 0; i < kKeyBatch; ++i) {
            const int c = c0 + i * kThreads;
            if (c < cap * kTileN) {
                const bool ok = ids[i] >= 0 && ids[i] < p.nk;
                const uint64_t vote = __ballot(ok);
                const uint32_t mine = (uint32_t)(vote >> (lane & 32));
                const int first = mine ? (lane & 32) + __ffs(mine) - 1 : lane;
                const int fallback = __shfl(ok ? (int)ids[i] : 0, first);
                key_s[c] = ok ? (int)ids[i] : fallback;
                if ((lane & 31) == 0) valid_s[c >> 5] = mine;
            }
        }
    }
    // Q fragments: B operand of S^T = K.Q^T, lane holds Q[q][16s + 8h .. +7].  Requested
    // after the lists so that waiting for the lists does not wait for Q.
    Frag qf[kSteps];
#pragma unroll
    for (int s = 0; s < kSteps; ++s) {
        u32x4 raw = {0u, 0u, 0u, 0u};
        if (q_ok) raw = *reinterpret_cast<const u32x4*>(qb + (size_t)qrow * D + 16 * s + 8 * h);
        qf[s] = __builtin_bit_cast(Frag, raw);
    }
    n_anc = min(max(n_anc, 0), p.max_anc);
    const int listed_tiles = kQGroups + (n_anc + kTileN - 1) / kTileN;
    const int total_tiles = listed_tiles + (p.prefix + kTileN - 1) / kTileN;
    __syncthreads();

    // ---- gather: HBM -> LDS, 16 bytes per lane, no registers in between --------
    // Transfer g of a tile moves row group g/2 = rows [kRowsPerDma*(g/2), +kRowsPerDma) of K
    // (g even) or V (g odd); wave w < kDmaWaves issues transfers [w*kDmaPerWave, +kDmaPerWave).
    // Lane i lands at LDS byte 16*i of the transfer, i.e. row i / kCpr, chunk slot i % kCpr,
    // and fetches the chunk that the XOR swizzle assigns to that slot.  Every gathering wave
    // issues exactly kDmaPerWave transfers per tile: the vmcnt bookkeeping counts on it.
    const int dma_row = lane / kCpr, dma_slot = lane % kCpr;
    auto issue = [&](int t, int slot) {
        if (kDmaWaves < kWaves && wave >= kDmaWaves) return;
        T* dst_tile = ring + slot * 2 * kTileElems;
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
            // V of a leaf tile is read row-wise like K (no transposing read), so it takes K's swizzle
            const T* src = is_v ? vb + row_off + (t < kQGroups ? k_chunk<D>(r, dma_slot) : v_chunk<D>(r, dma_slot)) * 8
                                : kb + row_off + k_chunk<D>(r, dma_slot) * 8;
            __builtin_amdgcn_global_load_lds(
                (const void __attribute__((address_space(1)))*)src,
                (void __attribute__((address_space(3)))*)(dst_tile + (is_v ? kTileElems : 0) + u * 512),
                16, 0, 0);
        }
    };

    // Ring bookkeeping, in tiles: `issued` gathers started, `consumed` tiles everyone is done
    // with; tile i lives in slot i % stages.  begin_step(g) makes tiles [consumed, consumed+g)
    // usable: wait until at most the gathers issued after them are outstanding (they retire in
    // order), barrier (everyone's share has landed, everyone is done with the tiles before),
    // then refill the slots that barrier freed.
    int issued = 0, issue_slot = 0, consumed = 0, slot = 0;
    auto refill = [&]() {
        while (issued < total_tiles && issued < consumed + stages) {
            issue(issued, issue_slot);
            ++issued;
            issue_slot = issue_slot + 1 == stages ? 0 : issue_slot + 1;
        }
    };
    auto begin_step = [&](int g) {
        if (issued < min(consumed + g, total_tiles)) {
            // ring too shallow (long ancestor lists leave little LDS) for this step's tiles to be
            // in flight already: free the slots first, then request them
            ring_barrier();
            refill();
        }
        wait_tiles_outstanding<kDmaPerWave>(max(issued - consumed - g, 0));
        ring_barrier();
        refill();
    };
    auto end_step = [&](int g) {
        consumed += g;
        slot += g;
        if (slot >= stages) slot -= stages;
    };
    auto tile_ptr = [&](int i) {   // K tile of the i-th tile of the current step; V follows it
        int sl = slot + i;
        if (sl >= stages) sl -= stages;
        return ring + sl * 2 * kTileElems;
    };
    refill();

    float m_i = -INFINITY, l_i = 0.f;
    f32x16 o[kDTiles];
#pragma unroll
    for (int dt = 0; dt < kDTiles; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[dt][r] = 0.f;

    // Leaf tile i = the block's own rows 32i .. 32i+31 (reference
    // fstattention.py:86-91,104-107): query r sees exactly row r of it, so this is one
    // dot product per lane pair for one wave, no matrix core; it seeds that wave's
    // running softmax.  kLeafGroup leaf tiles are taken per step, by different waves.
    for (int base = 0; base < kQGroups; base += kLeafGroup) {
        begin_step(kLeafGroup);
        if (split == 0 && qgroup >= base && qgroup < base + kLeafGroup && __ballot(leaf_ok) != 0ull) {
            const T* kt = tile_ptr(qgroup - base);
            const T* vt = kt + kTileElems;
            float part[2] = {0.f, 0.f};
            {
                u32x4 kraw[kSteps];
#pragma unroll
                for (int ks = 0; ks < kSteps; ++ks)
                    kraw[ks] = lds_read_b128(lds_addr(kt + ql * D + k_chunk<D>(ql, 2 * ks + h) * 8));
                lds_wait();
#pragma unroll
                for (int ks = 0; ks < kSteps; ++ks) {
                    lds_tie(kraw[ks]);
                    const Frag kf = __builtin_bit_cast(Frag, kraw[ks]);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const T2 a = {qf[ks][2 * e], qf[ks][2 * e + 1]};
                        const T2 b = {kf[2 * e], kf[2 * e + 1]};
                        part[e & 1] = MM::dot2(a, b, part[e & 1]);
                    }
                }
            }
            const float half_dot = part[0] + part[1];
            const float dot = half_dot + __shfl_xor(half_dot, 32);
            u32x2 vraw[kDTiles][4];
#pragma unroll
            for (int dt = 0; dt < kDTiles; ++dt)
#pragma unroll
                for (int g = 0; g < 4; ++g)   // accumulator rows 8g + 4h .. +3 of tile dt: 4 head dims
                    vraw[dt][g] = lds_read_b64(lds_addr(vt + ql * D + k_chunk<D>(ql, 4 * dt + g) * 8 + 4 * h));
            lds_wait();
#pragma unroll
            for (int dt = 0; dt < kDTiles; ++dt)
#pragma unroll
                for (int g = 0; g < 4; ++g) lds_tie(vraw[dt][g]);
            if (leaf_ok) {
                m_i = dot * p.scale_log2e;
                l_i = h == 0 ? 1.f : 0.f;
#pragma unroll
                for (int dt = 0; dt < kDTiles; ++dt)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const uint32_t w0 = vraw[dt][g][0], w1 = vraw[dt][g][1];
                        o[dt][4 * g + 0] = MM::low(w0);
                        o[dt][4 * g + 1] = MM::high(w0);
                        o[dt][4 * g + 2] = MM::low(w1);
                        o[dt][4 * g + 3] = MM::high(w1);
                    }
            }
        }
        end_step(kLeafGroup);
    }

    // Ancestor tiles under the packed tree mask, then the dense shared prefix; kSplit tiles
    // per step, tile consumed+s by the waves of share s.  A tile none of a wave's queries
    // attends to is not skipped: with an all-zero mask word it adds exact zeros, and a
    // branch-free body spares the accumulators a copy per step.
    const int tr_row = (lane & 15) >> 2;                          // key within a group of 4
    const int tr_col = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);   // head dim within the 32-row tile
    while (consumed < total_tiles) {
        begin_step(kSplit);
        const int t = consumed + split;
        const T* kt = tile_ptr(split);
        const T* vt = kt + kTileElems;
        end_step(kSplit);
        uint32_t word = 0u;
        if (t < listed_tiles) {
            word = mask_s[(t - kQGroups) * M + row_in_block] & valid_s[t];
        } else if (t < total_tiles) {
            const int left = p.prefix - (t - listed_tiles) * kTileN;
            word = left >= 32 ? 0xffffffffu : ((1u << left) - 1u);
        }
        if (kSplit > 1 && t >= total_tiles) continue;   // this share has no tile in the last step

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
        // transposing read.  The first half of the keys is requested now, so that LDS
        // latency hides behind the softmax; the second half behind the first MFMAs.
        auto read_v = [&](VPair (&f)[kDTiles], int kk) {
#pragma unroll
            for (int dt = 0; dt < kDTiles; ++dt) {
                const int col = 32 * dt + tr_col;
                const int r0 = 16 * kk + 4 * h + tr_row;      // keys 16kk+4h .. +3
                const int r1 = r0 + 8;                         // keys 16kk+8+4h .. +3
                f[dt].a = lds_read_tr16(lds_addr(vt + r0 * D + v_chunk<D>(r0, col >> 3) * 8 + (col & 7)));
                f[dt].b = lds_read_tr16(lds_addr(vt + r1 * D + v_chunk<D>(r1, col >> 3) * 8 + (col & 7)));
            }
        };
        auto tie_v = [&](VPair (&f)[kDTiles]) {
            lds_wait();
#pragma unroll
            for (int dt = 0; dt < kDTiles; ++dt) { lds_tie(f[dt].a); lds_tie(f[dt].b); }
        };
        VPair v0[kDTiles], v1[kDTiles];
        read_v(v0, 0);
        // mask + online softmax; accumulator register r is key 8*(r/4) + 4h + r%4.  The
        // maximum is taken over the raw scores (the scale is positive here, the launcher sends
        // other scales to the scalar kernel) and the scale rides in the FMA under the exp2.
        const uint32_t wsh = word >> (4 * h);
        float sv[16];
        float mx_raw = -INFINITY;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const bool on = (wsh >> (8 * (r / 4) + (r % 4))) & 1u;
            sv[r] = on ? s[r] : -INFINITY;
            mx_raw = fmaxf(mx_raw, sv[r]);
        }
        mx_raw = fmaxf(mx_raw, __shfl_xor(mx_raw, 32));
        const float mx = mx_raw * p.scale_log2e;
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
        const float neg_m = m_i == -INFINITY ? 0.f : -m_i;
        float rowsum = 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            sv[r] = __builtin_amdgcn_exp2f(__builtin_fmaf(sv[r], p.scale_log2e, neg_m));
            rowsum += sv[r];
        }
        l_i += rowsum;
        // P^T fragments: registers 8kk .. 8kk+7 are the 8 k-indices this lane feeds to MFMA kk
        Frag ph[2], pl[2];
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
            u32x4 hi4, lo4;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float a = sv[8 * kk + 2 * e], b = sv[8 * kk + 2 * e + 1];
                const uint32_t hi = MM::pack(a, b);
                hi4[e] = hi;
                if (SPLIT) lo4[e] = MM::pack(a - MM::low(hi), b - MM::high(hi));
            }
            ph[kk] = __builtin_bit_cast(Frag, hi4);
            if (SPLIT) pl[kk] = __builtin_bit_cast(Frag, lo4);
        }
        // O^T += V_tile^T . P^T ; hi weights of all head-dim tiles first, then lo, so that
        // MFMAs on the same accumulator are several instructions apart
        tie_v(v0);
        read_v(v1, 1);
#pragma unroll
        for (int dt = 0; dt < kDTiles; ++dt)
            o[dt] = MM::mfma(__builtin_bit_cast(Frag, v0[dt]), ph[0], o[dt]);
        if (SPLIT) {
#pragma unroll
            for (int dt = 0; dt < kDTiles; ++dt)
                o[dt] = MM::mfma(__builtin_bit_cast(Frag, v0[dt]), pl[0], o[dt]);
        }
        tie_v(v1);
#pragma unroll
        for (int dt = 0; dt < kDTiles; ++dt)
            o[dt] = MM::mfma(__builtin_bit_cast(Frag, v1[dt]), ph[1], o[dt]);
        if (SPLIT) {
#pragma unroll
            for (int dt = 0; dt < kDTiles; ++dt)
                o[dt] = MM::mfma(__builtin_bit_cast(Frag, v1[dt]), pl[1], o[dt]);
        }
    }

    // ---- merge the shares of a query group (same lanes, same layout) through LDS ----
    if (kSplit > 1) {
        __syncthreads();   // the ring is free: every tile has been consumed
        float* xch = reinterpret_cast<float*>(smem) + (size_t)qgroup * (2 + 16 * kDTiles) * 64;
        if (split == 1) {
            xch[lane] = m_i;
            xch[64 + lane] = l_i;
#pragma unroll
            for (int dt = 0; dt < kDTiles; ++dt)
#pragma unroll
                for (int r = 0; r < 16; ++r) xch[(2 + 16 * dt + r) * 64 + lane] = o[dt][r];
        }
        __syncthreads();
        if (split != 0) return;
        const float m_b = xch[lane], l_b = xch[64 + lane];
        const float m_new = fmaxf(m_i, m_b);
        const float m_safe = m_new == -INFINITY ? 0.f : m_new;
        const float a_own = __builtin_amdgcn_exp2f(m_i - m_safe);
        const float a_oth = __builtin_amdgcn_exp2f(m_b - m_safe);
        l_i = l_i * a_own + l_b * a_oth;
        m_i = m_new;
#pragma unroll
        for (int dt = 0; dt < kDTiles; ++dt)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                o[dt][r] = o[dt][r] * a_own + xch[(2 + 16 * dt + r) * 64 + lane] * a_oth;
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
                    const u32x2 packed = {MM::pack(val.x, val.y), MM::pack(val.z, val.w)};
                    *reinterpret_cast<u32x2*>(static_cast<T*>(p.o) + base + d) = packed;
                }
            }
        }
    }
}

template <bool BF16, int D, int M, bool SPLIT>
int launch_one(const AttnParams& p, hipStream_t stream) {
    // ring depth: everything in flight at once for short tile lists, else the limit
    const int tiles = M / 32 + anc_tile_capacity(p.max_anc) + (p.prefix + kTileN - 1) / kTileN;
    int stages = tiles < 2 ? 2 : (tiles > kMaxStages ? kMaxStages : tiles);
    size_t lds = mfma_lds_bytes<D, M>(p.max_anc, stages);
    while (lds > 160 * 1024 && stages > 2) lds = mfma_lds_bytes<D, M>(p.max_anc, --stages);
    if (lds > 160 * 1024)
        return fail(FSTA_EUNSUPPORTED, "max_ancestors=%d needs %zu bytes of LDS (limit 163840)", p.max_anc, lds);
    if (lds > 64 * 1024) {
        const int rc = allow_full_lds<&attn_mfma_kernel<BF16, D, M, SPLIT>>();
        if (rc != FSTA_OK) return rc;
    }
    const int slices_per_xcd = (p.heads_total + kXcds - 1) / kXcds;
    const unsigned grid = (unsigned)(kXcds * slices_per_xcd * p.nb);
    hipLaunchKernelGGL((attn_mfma_kernel<BF16, D, M, SPLIT>), dim3(grid), dim3(M * 2 * key_split_for(M)), lds,
                       stream, p, stages);
    FSTA_HIP_OK(hipGetLastError());
    note_launch({"attn_mfma_kernel", BF16 ? "true" : "false", {D, M, SPLIT ? 1 : 0, 0, 0}, 3, 0x4u, 0, 0});
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
