// Streaming tree attention kernel for gfx950: launches with many more (query block, slice) pairs
// than the GPU holds workgroups.
//
// The kernel of fsta_attention_mfma16.hip gives every (block, slice) pair a workgroup of its own.
// Such a workgroup spends a third of its life on a chain of dependent memory round trips before
// its first matrix instruction (block plan -> K/V rows named by the plan -> first tile in LDS) and
// ends with stores nobody overlaps; only the other workgroup on the same CU covers for it.  Here a
// workgroup STAYS: the grid is as many workgroups as the GPU holds at once, each walks a list of
// (block, slice) pairs, and the gather ring never drains in between.  While the matrix cores work
// on the last tiles of one pair, the ring already holds the Q rows and first tiles of the next,
// whose plan was requested a whole pair earlier.  What makes this possible on a machine with one
// in-order counter (vmcnt) for loads AND stores:
//   * every wave counts the vector-memory instructions it issues (`ops`) and remembers the count
//     after each tile's transfers; "tile X has landed" is then "at most ops - ops_after(X)
//     instructions outstanding", whatever was issued in between (stores of the previous pair, the
//     request for the next plan).  Stores that are still on their way no longer hold up the wait
//     for a tile that was requested before them;
//   * the output leaves straight from the accumulators (two lane-row swaps make 16 contiguous
//     bytes per lane), so the epilogue needs neither LDS nor a barrier and the ring stays as it is;
//   * Q travels through the ring like a tile, and the block's own rows ("leaf tiles") are spread
//     between the ancestor tiles instead of in front of them: the four cheap leaf steps of a
//     128-row block would otherwise eat the ring's whole lookahead at the start of every pair.
//
// Measured (MI355X): parity-green and SLOWER than one workgroup per pair -- 2048-node trees x 512 slices, blocks of
// 128 rows: 440 against 300 us; the reference's benchmark shapes: twice the time.  The instrumented build
// (`python -m fstattention_amd.timeline --stream`) says why: of a step's ~4700 cycles a wave spends ~1000 waiting for
// its tile, ~950 at the barrier and ~1250 in the scalar bookkeeping that requests one tile (all eight waves of a
// workgroup walk the same ~250 scalar instructions per step in lockstep, at one instruction per four cycles and
// wave), against ~2000 in the arithmetic of a tile.  The library therefore never chooses this kernel by itself;
// FSTA_FLAG_STREAM selects it.
//
// Tile list of one pair: [Q (M/64 tiles) | A0 L0 A1 L1 ... then whatever is left of either kind].
// Arithmetic of a tile (S^T = K.Q^T on v_mfma_f32_16x16x32, packed tree mask, base-2 online softmax,
// O^T += V^T.P^T) is that of fsta_attention_mfma16.hip with one wave per group of 16 query rows.
#include "fsta_mfma_common.h"

namespace fsta {
namespace {

using namespace mfma;

constexpr int kStreamMaxStages = 8;

#ifdef FSTA_TIMELINE
__device__ unsigned long long* g_stream_profile = nullptr;   // [workgroup][wave][10 cycle sums, 10 counts], set by fsta_stream_profile_buffer
#endif

__device__ __forceinline__ int pick(bool c, int a, int b) { return c ? a : b; }

// s_waitcnt vmcnt(n) for a run-time n (the instruction takes an immediate): five compares down a binary tree;
// n above 31 waits for 31 (a stronger wait than asked for, never a weaker one).
template <int LO, int HI> __device__ __forceinline__ void wait_ops_in(int n) {
    if constexpr (LO == HI) {
        wait_vmcnt<LO>();
    } else {
        constexpr int kMid = (LO + HI) / 2;
        if (n <= kMid) wait_ops_in<LO, kMid>(n);
        else wait_ops_in<kMid + 1, HI>(n);
    }
}
__device__ __forceinline__ void wait_ops_outstanding(int n) { wait_ops_in<0, 31>(n); }

template <int D, int M>
__host__ __device__ inline size_t stream_plan_bytes(int max_anc) {
    return ((size_t)plan_layout(M, max_anc).block_words * 4 + 15) & ~(size_t)15;
}
template <int D, int M>
__host__ __device__ inline size_t stream_lds_bytes(int max_anc, int stages, int plan_bufs) {
    return (size_t)stages * 2 * kTileN * D * 2 + plan_bufs * stream_plan_bytes<D, M>(max_anc);
}

template <bool BF16, int D, int M, bool SPLIT>
__global__ __launch_bounds__(M * 4, 4) void attn_stream_kernel(AttnParams p, int stages, int wg_per_xcd, int plan_bufs) {
#ifdef FSTA_TIMELINE
    // instrumented build only (-DFSTA_TIMELINE): shader-clock cycles per kind of segment, summed per wave
    unsigned long long pacc[10] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0}, pcnt[10] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    unsigned long long plast = __builtin_amdgcn_s_memtime();
#define FSTA_MARK(seg) do { const unsigned long long t_ = __builtin_amdgcn_s_memtime(); pacc[seg] += t_ - plast; pcnt[seg] += 1; plast = t_; } while (0)
#else
#define FSTA_MARK(seg) do { } while (0)
#endif
    using MM = Mma<BF16>;
    using T = typename MM::elem;
    using T2 = typename MM::elem2;
    using Frag = typename MM::frag;
    constexpr int kWaves = M / 16;                // one wave per group of 16 query rows
    constexpr int kLeafTiles = M / 32;            // 32-row tiles holding the block's own rows
    constexpr int kQTiles = M / 64;               // ring tiles the block's Q rows take (a tile = 64 rows of D elements)
    constexpr int kCpr = D / 8;                   // 16-byte chunks per row
    constexpr int kRowBytes = 2 * D;
    constexpr int kRowsPerDma = 64 / kCpr;        // rows one wave-wide 1 KiB transfer covers
    constexpr int kDmaPerTile = 2 * kTileN / kRowsPerDma;   // K and V transfers of one tile
    static_assert(kDmaPerTile % kWaves == 0, "every wave issues the same number of transfers per tile");
    constexpr int kDmaPerWave = kDmaPerTile / kWaves;
    static_assert(kDmaPerWave == 1 || kDmaPerWave % 2 == 0, "a wave's transfers are K/V pairs of whole row groups");
    constexpr int kRowGroups = (kDmaPerWave + 1) / 2;
    constexpr int kSteps = D / 32;                // MFMAs per 16-key half of S^T
    constexpr int kOTiles = D / 16;               // 16-row tiles of O^T
    constexpr int kTileElems = kTileN * D;
    constexpr float kTrustedSum = BF16 ? 16777216.f : 32768.f;
    static_assert(M == 64 || M == 128, "blocks of 64 or 128 rows");

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    T* ring = reinterpret_cast<T*>(smem);
    const int ring_bytes = stages * 2 * kTileElems * 2;
    const int anc_cap = anc_tile_capacity(p.max_anc);
    const int common_words = kPlanHeaderWords + anc_cap * kTileN;
    const int group_words = kTileN * (1 + anc_cap);
    const int plan_words = common_words + kLeafTiles * group_words;
    const int plan_stride = (int)stream_plan_bytes<D, M>(p.max_anc);
    // plan records of the pairs at list positions r, r + 1 (, r + 2): position r sits in buffer r % plan_bufs
    unsigned char* const plan_area = smem + ring_bytes;
    auto buf_of = [&](int r) __attribute__((always_inline)) { return plan_bufs == 2 ? (r & 1) : r % 3; };

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63;
    const int ql = lane & 15;        // query (column of S^T / O^T) of this lane
    const int g = lane >> 4;         // which quarter of the rows of an accumulator tile
    const float sc = p.scale_log2e;

    // ---- this workgroup's list of (block, slice) pairs ---------------------------------------------
    // Workgroup w runs on XCD w % 8 and takes slices hz = 8 sx + xcd only, so that the blocks of a slice
    // share one L2 for the ancestors they have in common.  The pairs of an XCD are numbered slice by
    // slice; the workgroups of the XCD take them round-robin, so that at any moment they work on a few
    // neighbouring slices.  Inside a slice the block numbers are rotated by the round the slice starts
    // in: block j costs about as much as block j of any other slice (long ancestor lists sit at the end
    // of a tree), and without the rotation a workgroup would meet the same j in every round.
    const int xcd = blockIdx.x % kXcds;
    const int wg_in_xcd = blockIdx.x / kXcds;
    const int slices_here = (p.heads_total - xcd + kXcds - 1) / kXcds;
    const int pairs_here = slices_here * p.nb;
    const int n_mine = wg_in_xcd < pairs_here ? (pairs_here - wg_in_xcd + wg_per_xcd - 1) / wg_per_xcd : 0;
    if (n_mine == 0) return;

    // list position r -> (slice, block)
    auto pair_at = [&](int r, int& hz, int& block) __attribute__((always_inline)) {
        const int idx = wg_in_xcd + r * wg_per_xcd;
        const int sx = idx / p.nb, jj = idx - sx * p.nb;
        const int rot = (sx * p.nb) / wg_per_xcd;
        block = (jj + rot) % p.nb;
        hz = sx * kXcds + xcd;
    };

    // ---- the ring and its bookkeeping ---------------------------------------------------------------
    // Tiles are numbered through all pairs of the list; tile i lives in slot i % stages.  `issued` tiles
    // have been requested, `consumed` tiles everyone is done with.
    // Byte k of `behind` = vector-memory instructions this wave has issued after the transfers of the tile
    // that has k newer tiles behind it (one 64-bit scalar: no array, no selects; the counts stay far below 256).
    uint64_t behind = 0ull;
    uint32_t behind_plan0 = 0u, behind_plan1 = 0u;   // ... issued after the requests for the plans of list positions plan_ready + 1, + 2
    static_assert(kStreamMaxStages == 8, "one byte per ring stage");
    auto count_ops = [&](int n) __attribute__((always_inline)) {
        behind += (uint64_t)n * 0x0101010101010101ull;
        behind_plan0 += n;
        behind_plan1 += n;
    };
    auto ops_after_tile = [&](int newer) __attribute__((always_inline)) { return (int)((behind >> (8 * newer)) & 0xffu); };
    int issued = 0, consumed = 0, issue_slot = 0, slot = 0;

    // pairs: `cur` is being consumed (position r of the list), `nxt` follows it
    int cur_hz, cur_block, nxt_hz, nxt_block;
    pair_at(0, cur_hz, cur_block);
    pair_at(n_mine > 1 ? 1 : 0, nxt_hz, nxt_block);
    int cur_row_base = cur_block * M, nxt_row_base = nxt_block * M;
    int r_cur = 0;
    int cur_base = 0;                 // number of the first tile of cur
    int cur_total = 1 << 28;          // tiles of cur (known once its plan has landed)
    int cur_anc = 0, nxt_anc = 0;     // ancestor tiles
    int nxt_total = 1 << 28;
    int plan_ready = -1;              // last list position whose plan is known to have landed for every wave
    int plan_asked = -1;              // last list position whose plan has been requested
    const int plan_ahead = plan_bufs - 1;      // the plan of position r + plan_ahead is requested while r is worked on

    const int dma_row = lane / kCpr, dma_slot = lane % kCpr;
    uint32_t dma_leaf[kDmaPerWave], dma_flip[kDmaPerWave];
#pragma unroll
    for (int i = 0; i < kDmaPerWave; ++i) {
        const int t2 = wave * kDmaPerWave + i;
        const int r = (t2 >> 1) * kRowsPerDma + dma_row;
        dma_leaf[i] = (uint32_t)k_chunk<D>(r, dma_slot) * 16u;
        dma_flip[i] = (t2 & 1) ? ((uint32_t)v16_chunk<D>(r, dma_slot) * 16u) ^ dma_leaf[i] : 0u;
    }

    auto request_plan = [&](int block, int r_of_x) __attribute__((always_inline)) {
        const int parity = buf_of(r_of_x);
        // the waves share the copy of the record: piece k (1 KiB) by wave k % kWaves
        const char* rec = reinterpret_cast<const char*>(p.plan) + (size_t)block * (size_t)plan_words * 4;
        const int chunks = plan_words / 4;
        for (int piece = wave; piece * 64 < chunks; piece += kWaves) {
            const int c = piece * 64 + lane;
            if (c < chunks)
                __builtin_amdgcn_global_load_lds(
                    (const void __attribute__((address_space(1)))*)(rec + (size_t)((uint32_t)c * 16u)),
                    (void __attribute__((address_space(3)))*)(plan_area + parity * plan_stride + piece * 1024), 16, 0, 0);
            count_ops(1);
        }
        // (a wave without a piece of the record waits for nobody's: the barrier covers the others')
        const uint32_t mine = wave * 64 < chunks ? 0u : 0x7fffu;
        if (plan_asked == plan_ready) behind_plan0 = mine;
        else behind_plan1 = mine;
        plan_asked = r_of_x;
    };

    // Requests tile `local` of pair x (list position parity `parity`, `anc` ancestor tiles) into ring slot `sl`.
    auto issue_tile = [&](int hz, int row_base, int parity, int anc, int local, int sl) __attribute__((always_inline)) {
        unsigned char* dst_tile = reinterpret_cast<unsigned char*>(ring + sl * 2 * kTileElems);
        if (local < kQTiles) {
            // 64 Q rows, row-major with K's swizzle; transfer t2 moves rows [t2 * kRowsPerDma, +kRowsPerDma)
            const char* qb = reinterpret_cast<const char*>(p.q) + (size_t)hz * p.nq * kRowBytes;
            int lane_o = lane;
            asm volatile("" : "+v"(lane_o));
            const int dma_row = lane_o / kCpr, dma_slot = lane_o % kCpr;     // (shadow the kernel-wide copies: see the Q step)
#pragma unroll
            for (int i = 0; i < kDmaPerWave; ++i) {
                const int t2 = wave * kDmaPerWave + i;
                const int rr = t2 * kRowsPerDma + dma_row;
                const int grow = min(row_base + local * 64 + rr, p.nq - 1);
                const uint32_t off = (uint32_t)grow * (uint32_t)kRowBytes + (uint32_t)k_chunk<D>(rr, dma_slot) * 16u;
                __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1)))*)(qb + (size_t)off),
                                                 (void __attribute__((address_space(3)))*)(dst_tile + t2 * 1024), 16, 0, 2);   // (non-temporal: read once)
            }
        } else {
            const int pos = local - kQTiles;
            const int both = min(anc, kLeafTiles);
            bool leaf;
            int idx;
            if (pos < 2 * both) {
                leaf = pos & 1;
                idx = pos >> 1;
            } else {
                leaf = anc < kLeafTiles;
                idx = pos - both;
            }
            const uint32_t* plan_s = reinterpret_cast<const uint32_t*>(plan_area + parity * plan_stride);
            const uint32_t* keys = leaf ? plan_s + common_words + idx * group_words
                                        : plan_s + kPlanHeaderWords + idx * kTileN;
            const unsigned char* kb = static_cast<const unsigned char*>(p.k) + (size_t)hz * p.nk * kRowBytes;
            const unsigned char* vb = static_cast<const unsigned char*>(p.v) + (size_t)hz * p.nk * kRowBytes;
            int rows[kRowGroups];
#pragma unroll
            for (int i = 0; i < kRowGroups; ++i)
                rows[i] = min((int)keys[((wave * kDmaPerWave) / 2 + i) * kRowsPerDma + dma_row] + p.key_shift, p.nk - 1);
            const uint32_t anc_tile = leaf ? 0u : 0xffffffffu;
#pragma unroll
            for (int i = 0; i < kDmaPerWave; ++i) {
                const int t2 = wave * kDmaPerWave + i;
                const int u = t2 >> 1;
                const bool is_v = t2 & 1;
                const uint32_t off = (uint32_t)rows[i >> 1] * (uint32_t)kRowBytes + (dma_leaf[i] ^ (dma_flip[i] & anc_tile));
                const char* src = reinterpret_cast<const char*>(is_v ? vb : kb) + (size_t)off;
                __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1)))*)src,
                                                 (void __attribute__((address_space(3)))*)(dst_tile + (is_v ? kTileElems * 2 : 0) + u * 1024),
                                                 16, 0, 0);
            }
        }
        count_ops(kDmaPerWave);
        behind <<= 8;     // the new tile is the newest: nothing issued after it yet
    };

    // Requests tiles while the ring has room: tiles of cur, then of nxt; a tile that needs a plan which
    // has not landed yet stops the refill (the Q tiles need none).
    auto refill = [&]() __attribute__((always_inline)) {
        while (issued < consumed + stages) {
            int local = issued - cur_base;
            const bool in_cur = local < cur_total;
            if (!in_cur) {
                if (r_cur + 1 >= n_mine) break;
                local -= cur_total;
                if (local >= nxt_total) break;
            }
            const int r_of = in_cur ? r_cur : r_cur + 1;
            if (local >= kQTiles && plan_ready < r_of) break;
            // (pick() takes values: `c ? a : b` on two variables selects between their ADDRESSES, which keeps both in memory)
            issue_tile(pick(in_cur, cur_hz, nxt_hz), pick(in_cur, cur_row_base, nxt_row_base), buf_of(r_of),
                       pick(in_cur, cur_anc, nxt_anc), local, issue_slot);
            ++issued;
            issue_slot = issue_slot + 1 == stages ? 0 : issue_slot + 1;
        }
    };
    auto anc_tiles_of = [&](int parity) __attribute__((always_inline)) {   // ancestor tiles of the pair whose plan sits in buffer `parity`
        uint32_t head = lds_read_b32(lds_addr(plan_area + parity * plan_stride));
        lds_wait();
        lds_tie(head);
        const int n_anc = min(max(__builtin_amdgcn_readfirstlane((int)head), 0), p.max_anc);
        return (n_anc + kTileN - 1) / kTileN;
    };

    // Makes tiles [consumed, consumed + n) usable: waits until they have landed (instructions issued after
    // them may stay outstanding), barrier (everyone's share has landed, everyone is done with the tiles
    // before), then refills the slots that barrier freed.  When the refill is about to reach tiles that
    // need a plan which has been requested but not awaited yet, the same wait covers that request and the
    // barrier makes the plan visible to all waves.  `ask_next`: request the plan of nxt behind the barrier
    // (its buffer was the plan of the pair before cur, which every wave has left by then).
    auto begin_step = [&](int n, bool ask_next) __attribute__((always_inline)) {
        int allow = ops_after_tile(issued - consumed - n);
        const int waiting = plan_ready + 1;     // list position of the first pair whose plan has not been awaited
        const int first_needing = waiting == r_cur ? cur_base + kQTiles : cur_base + cur_total + kQTiles;
        const bool publish = plan_asked >= waiting && waiting <= r_cur + 1 && consumed + stages > first_needing;
        if (publish) allow = min(allow, (int)behind_plan0);
        wait_ops_outstanding(allow);
        FSTA_MARK(0);
        ring_barrier();
        FSTA_MARK(1);
        if (publish) {
            plan_ready = waiting;
            behind_plan0 = behind_plan1;
            const bool is_cur = waiting == r_cur;
            const int anc = anc_tiles_of(buf_of(waiting));
            const int total = kQTiles + kLeafTiles + anc;
            cur_anc = pick(is_cur, anc, cur_anc);
            cur_total = pick(is_cur, total, cur_total);
            nxt_anc = pick(is_cur, nxt_anc, anc);
            nxt_total = pick(is_cur, nxt_total, total);
        }
        if (ask_next && r_cur + plan_ahead < n_mine) {
            int hz_a, block_a;
            pair_at(r_cur + plan_ahead, hz_a, block_a);
            request_plan(block_a, r_cur + plan_ahead);
        }
        refill();
        FSTA_MARK(2);
    };
    auto end_step = [&](int n) __attribute__((always_inline)) {
        consumed += n;
        slot += n;
        if (slot >= stages) slot -= stages;
    };

    // lane constants of the fragment reads (see fsta_attention_mfma16.hip)
    constexpr int kHalfTileBytes = 16 * D * 2;
    const uint32_t k_lane0 = (uint32_t)(ql * D + k_chunk<D>(ql, g) * 8) * 2;
    const int tr_r0 = 4 * g + (ql >> 2);
    const int tr_col = 4 * (ql & 3);
    const uint32_t v_lane0 = (uint32_t)(tr_r0 * D + v16_chunk<D>(tr_r0, tr_col >> 3) * 8 + (tr_col & 7)) * 2;

    // ---- start: plan of the first pair, its Q tiles ---------------------------------------------------
    request_plan(cur_block, 0);
    if (plan_ahead > 1 && n_mine > 1) request_plan(nxt_block, 1);
    refill();

    for (;;) {
        // ---- Q step: the block's Q rows are in the ring; every wave takes its 16 rows as B operands ----
        begin_step(kQTiles, true);
        Frag qf[kSteps];
        {
            int sl = slot + wave / 4;               // 64 rows per Q tile = 4 waves
            if (sl >= stages) sl -= stages;
            const T* qt = ring + sl * 2 * kTileElems;
            // (addresses used once per pair are derived from an opaque copy of the lane number, so that they are
            // worked out here and not kept in registers through the whole kernel)
            int lane_o = lane;
            asm volatile("" : "+v"(lane_o));
            const int ql_o = lane_o & 15, g_o = lane_o >> 4;
            const int row = (wave & 3) * 16 + ql_o;
            u32x4 qraw[kSteps];
#pragma unroll
            for (int s = 0; s < kSteps; ++s)
                qraw[s] = lds_read_b128(lds_addr(qt + row * D + k_chunk<D>(row, 4 * s + g_o) * 8));
            lds_wait();
#pragma unroll
            for (int s = 0; s < kSteps; ++s) {
                lds_tie(qraw[s]);
                qf[s] = __builtin_bit_cast(Frag, qraw[s]);
            }
        }
        end_step(kQTiles);
        FSTA_MARK(3);
        // (the Q step's barrier published this pair's plan at the latest)
        const uint32_t* plan_s = reinterpret_cast<const uint32_t*>(plan_area + buf_of(r_cur) * plan_stride);
        const uint32_t* group_s = plan_s + common_words;
        // this row's mask words, one per ancestor tile (rows 32 i .. 32 i + 31 of the block are group i: waves 2 i, 2 i + 1)
        const uint32_t* my_mask;
        {
            int lane_o = lane;
            asm volatile("" : "+v"(lane_o));
            my_mask = group_s + (wave >> 1) * group_words + kTileN + (wave & 1) * 16 + (lane_o & 15);
        }

        float m_i = -INFINITY, l_i = 0.f;
        f32x4 o[kOTiles];
#pragma unroll
        for (int dt = 0; dt < kOTiles; ++dt) o[dt] = f32x4{0.f, 0.f, 0.f, 0.f};

        const int both = min(cur_anc, kLeafTiles);
        for (int local = kQTiles; local < cur_total; ++local) {
            begin_step(1, false);
            const T* kt = ring + slot * 2 * kTileElems;
            const T* vt = kt + kTileElems;
            end_step(1);
            const int pos = local - kQTiles;
            bool leaf;
            int idx;
            if (pos < 2 * both) {
                leaf = pos & 1;
                idx = pos >> 1;
            } else {
                leaf = cur_anc < kLeafTiles;
                idx = pos - both;
            }
            if (leaf) {
                // Leaf tile idx = the block's own rows 32 idx .. 32 idx + 31 (reference fstattention.py:86-91,104-107):
                // query r sees exactly row r of it.  The two waves owning those rows take one dot product per query
                // on the vector ALU and add that key to their running softmax.
                if ((wave >> 1) != idx) { FSTA_MARK(5); continue; }
                int lane_o = lane;
                asm volatile("" : "+v"(lane_o));
                const int ql_o = lane_o & 15, g_o = lane_o >> 4;
                const int row = (wave & 1) * 16 + ql_o;
                const uint32_t valid = __builtin_amdgcn_readfirstlane((int)plan_s[kPlanLeafValid + idx]);   // leaf slots of these 32 rows
                if (((valid >> ((wave & 1) * 16)) & 0xffffu) == 0u) { FSTA_MARK(5); continue; }      // none of this wave's rows has a leaf key
                const bool leaf_ok = (valid >> row) & 1u;
                float part[2] = {0.f, 0.f};
                u32x2 vraw[kOTiles];
                {
                    u32x4 kraw[kSteps];
#pragma unroll
                    for (int ks = 0; ks < kSteps; ++ks)
                        kraw[ks] = lds_read_b128(lds_addr(kt + row * D + k_chunk<D>(row, 4 * ks + g_o) * 8));
#pragma unroll
                    for (int dt = 0; dt < kOTiles; ++dt)   // accumulator rows 4g .. 4g+3 of tile dt: 4 head dims
                        vraw[dt] = lds_read_b64(lds_addr(vt + row * D + k_chunk<D>(row, 2 * dt + (g_o >> 1)) * 8 + 4 * (g_o & 1)));
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
                const float sl2 = sum_quarters(part[0] + part[1]) * sc;
#pragma unroll
                for (int dt = 0; dt < kOTiles; ++dt) lds_tie(vraw[dt]);
                // one more key for the row: raise the maximum if this key needs it, weight 2^(s - m)
                const bool raise = leaf_ok && (sl2 > m_i + kRescaleSlack || m_i == -INFINITY);
                const float m_new = raise ? sl2 : m_i;
                const float alpha = raise ? __builtin_amdgcn_exp2f(m_i - m_new) : 1.f;     // exp2(-inf) = 0
                const float w = leaf_ok ? __builtin_amdgcn_exp2f(sl2 - m_new) : 0.f;
                m_i = m_new;
                l_i = l_i * alpha + (g_o == 0 ? w : 0.f);
#pragma unroll
                for (int dt = 0; dt < kOTiles; ++dt) {
                    o[dt][0] = __builtin_fmaf(w, MM::low(vraw[dt][0]), o[dt][0] * alpha);
                    o[dt][1] = __builtin_fmaf(w, MM::high(vraw[dt][0]), o[dt][1] * alpha);
                    o[dt][2] = __builtin_fmaf(w, MM::low(vraw[dt][1]), o[dt][2] * alpha);
                    o[dt][3] = __builtin_fmaf(w, MM::high(vraw[dt][1]), o[dt][3] * alpha);
                }
                FSTA_MARK(4);
                continue;
            }
            // ---- ancestor tile idx under the packed tree mask ----
            const uint32_t word = my_mask[idx * kTileN];
            if (__ballot(word != 0u) == 0ull) { FSTA_MARK(7); continue; }     // none of this wave's 16 queries attends to this tile

            typedef const u32x4 __attribute__((address_space(3))) * lds_u32x4;
            const uint32_t k_addr0 = lds_addr(kt) + k_lane0;
            f32x4 s[2];
#pragma unroll
            for (int sub = 0; sub < 2; ++sub) {
                s[sub] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < kSteps; ++ks) {
                    const u32x4 raw = *(lds_u32x4)(uintptr_t)((k_addr0 ^ (uint32_t)(ks << 6)) + sub * kHalfTileBytes);
                    s[sub] = mfma16(__builtin_bit_cast(Frag, raw), qf[ks], s[sub]);
                }
            }
            // V fragments (A operand of O^T += V^T.P^T) through the transposing read, a quarter of the head-dim tiles at
            // a time: the first quarter is requested now (its latency hides behind the softmax), each further one
            // behind the products of the one before.
            constexpr int kBatch = kOTiles / 4;
            const uint32_t v_addr0 = lds_addr(vt) + v_lane0;
            auto read_v = [&](VPair (&f)[kBatch], int first_dt) __attribute__((always_inline)) {
#pragma unroll
                for (int i = 0; i < kBatch; ++i) {
                    const uint32_t addr = v_addr0 ^ (uint32_t)((first_dt + i) << 5);
                    f[i].a = lds_read_tr16(addr);
                    f[i].b = lds_read_tr16_at<kHalfTileBytes>(addr);
                }
            };
            auto tie_v = [&](VPair (&f)[kBatch]) __attribute__((always_inline)) {
                lds_wait();
#pragma unroll
                for (int i = 0; i < kBatch; ++i) { lds_tie(f[i].a); lds_tie(f[i].b); }
            };
            VPair va[kBatch], vb[kBatch];
            read_v(va, 0);
            const uint32_t wsh = word >> (4 * g);
            float sv[8];
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                const uint32_t keep = (uint32_t)__builtin_amdgcn_sbfe((int)wsh, 16 * (r / 4) + (r % 4), 1);
                const float score = s[r / 4][r % 4];
                const uint32_t bits = __builtin_bit_cast(uint32_t, score);
                sv[r] = __builtin_bit_cast(float, (bits & keep) | (0xff800000u & ~keep));
            }
            float pw[8];
            float rowsum = 0.f;
            {
                const float neg_m = m_i == -INFINITY ? 0.f : -m_i;
#pragma unroll
                for (int r = 0; r < 8; ++r) {
                    pw[r] = __builtin_amdgcn_exp2f(__builtin_fmaf(sv[r], sc, neg_m));
                    rowsum += pw[r];
                }
            }
            const bool redo = !(rowsum <= kTrustedSum) || (m_i == -INFINITY && (wsh & 0x000f000fu) != 0u);
            if (__ballot(redo) != 0ull) {
                float mx_raw = fmaxf(fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3])),
                                     fmaxf(fmaxf(sv[4], sv[5]), fmaxf(sv[6], sv[7])));
                mx_raw = max_quarters(mx_raw);
                const float mx = mx_raw * sc;
                const bool raise = mx > m_i + kRescaleSlack || (m_i == -INFINITY && mx > -INFINITY);
                const float alpha = raise ? __builtin_amdgcn_exp2f(m_i - mx) : 1.f;
                if (raise) m_i = mx;
                l_i *= alpha;
#pragma unroll
                for (int dt = 0; dt < kOTiles; ++dt)
#pragma unroll
                    for (int r = 0; r < 4; ++r) o[dt][r] *= alpha;
                const float neg_m = m_i == -INFINITY ? 0.f : -m_i;
                rowsum = 0.f;
#pragma unroll
                for (int r = 0; r < 8; ++r) {
                    pw[r] = __builtin_amdgcn_exp2f(__builtin_fmaf(sv[r], sc, neg_m));
                    rowsum += pw[r];
                }
            }
            l_i += rowsum;
            u32x4 hi4, lo4;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float a = pw[2 * e], b = pw[2 * e + 1];
                const uint32_t hi = MM::pack(a, b);
                hi4[e] = hi;
                if (SPLIT) lo4[e] = MM::pack(a - MM::low(hi), b - MM::high(hi));
            }
            const Frag ph = __builtin_bit_cast(Frag, hi4);
            Frag pl;
            if (SPLIT) pl = __builtin_bit_cast(Frag, lo4);
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                VPair (&now)[kBatch] = (b & 1) ? vb : va;
                VPair (&then)[kBatch] = (b & 1) ? va : vb;
                tie_v(now);
                if (b < 3) read_v(then, (b + 1) * kBatch);
#pragma unroll
                for (int i = 0; i < kBatch; ++i) o[b * kBatch + i] = mfma16(__builtin_bit_cast(Frag, now[i]), ph, o[b * kBatch + i]);
                if (SPLIT) {
#pragma unroll
                    for (int i = 0; i < kBatch; ++i) o[b * kBatch + i] = mfma16(__builtin_bit_cast(Frag, now[i]), pl, o[b * kBatch + i]);
                }
            }
            FSTA_MARK(6);
        }

        // ---- end of the pair: normalise and store straight from the accumulators ----------------------
        // Lane (g, ql) holds head dims 16 dt + 4g .. + 3 of row ql for every tile dt.  For 16-bit output a
        // lane-row swap between g and g ^ 1 pairs the pieces of two tiles up, so that every lane stores 16
        // contiguous bytes and the four lanes of a row 64: tiles 2a and 2a+1 leave in one instruction.
        {
            const float l_tot = sum_quarters(l_i);
            const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
            const float lse_val = l_tot > 0.f ? m_i + log2f(l_tot) : -INFINITY;
            const int first_row = cur_row_base + wave * 16;
            int lane_o = lane;
            asm volatile("" : "+v"(lane_o));
            const int ql = lane_o & 15, g = lane_o >> 4;     // (shadow the kernel-wide copies: see the Q step)
            const int row = first_row + ql;
            if (first_row < p.nq) {       // (wave-uniform: the stores below are issued, and counted, exactly when this holds)
                if (p.lse) {
                    if (g == 0 && row < p.nq) p.lse[(size_t)cur_hz * p.nq + row] = lse_val;
                    count_ops(1);
                }
                if (p.out_f32) {
                    float* ob = static_cast<float*>(p.o) + ((size_t)cur_hz * p.nq + row) * D + 4 * g;
#pragma unroll
                    for (int dt = 0; dt < kOTiles; ++dt) {
                        const f32x4 val = {o[dt][0] * inv, o[dt][1] * inv, o[dt][2] * inv, o[dt][3] * inv};
                        if (row < p.nq) __builtin_nontemporal_store(val, reinterpret_cast<f32x4*>(ob + 16 * dt));
                    }
                    count_ops(kOTiles);
                } else {
                    T* ob = static_cast<T*>(p.o) + ((size_t)cur_hz * p.nq + row) * D + ((g & 1) ? 16 + 4 * (g - 1) : 4 * g);
#pragma unroll
                    for (int a = 0; a < kOTiles / 2; ++a) {
                        const f32x4& x = o[2 * a];
                        const f32x4& y = o[2 * a + 1];
                        const uint32_t x0 = MM::pack(x[0] * inv, x[1] * inv), x1 = MM::pack(x[2] * inv, x[3] * inv);
                        const uint32_t y0 = MM::pack(y[0] * inv, y[1] * inv), y1 = MM::pack(y[2] * inv, y[3] * inv);
                        const u32x2 s0 = __builtin_amdgcn_permlane16_swap(x0, y0, false, false);
                        const u32x2 s1 = __builtin_amdgcn_permlane16_swap(x1, y1, false, false);
                        const uint32_t a0 = s0[0], b0 = s0[1], a1 = s1[0], b1 = s1[1];
                        const u32x4 val = {a0, a1, b0, b1};
                        if (row < p.nq) __builtin_nontemporal_store(val, reinterpret_cast<u32x4*>(ob + 32 * a));
                    }
                    count_ops(kOTiles / 2);
                }
            }
        }

        // ---- next pair ------------------------------------------------------------------------------------
        FSTA_MARK(8);
        if (r_cur + 1 >= n_mine) break;
        cur_base += cur_total;
        ++r_cur;
        cur_hz = nxt_hz;
        cur_block = nxt_block;
        cur_row_base = nxt_row_base;
        cur_total = nxt_total;      // (known if its plan has been awaited already; else the Q step's barrier publishes it)
        cur_anc = nxt_anc;
        nxt_total = 1 << 28;
        nxt_anc = 0;
        if (r_cur + 1 < n_mine) {
            pair_at(r_cur + 1, nxt_hz, nxt_block);
            nxt_row_base = nxt_block * M;
        }
    }
#ifdef FSTA_TIMELINE
    if (g_stream_profile && lane == 0) {
        unsigned long long* out = g_stream_profile + ((size_t)blockIdx.x * kWaves + wave) * 20;
        for (int i = 0; i < 10; ++i) { out[i] = pacc[i]; out[10 + i] = pcnt[i]; }
    }
#endif
}

template <bool BF16, int D, int M, bool SPLIT>
int launch_stream(const AttnParams& p, hipStream_t stream) {
    constexpr int kQTiles = M / 64, kLeafTiles = M / 32;
    constexpr size_t kTileBytes = (size_t)2 * kTileN * D * 2;
    // Two workgroups per CU (80 KB of LDS each): the deepest ring that fits beside the plan records, at least four
    // stages; a third plan buffer (plans requested two pairs ahead: short lists leave one pair's time too short
    // for the round trip) where that still leaves four stages.
    constexpr size_t kHalfCu = 80 * 1024;
    int plan_bufs = stream_lds_bytes<D, M>(p.max_anc, 4, 3) <= kHalfCu ? 3 : 2;
    int stages = kStreamMaxStages;
    while (stages > 4 && stream_lds_bytes<D, M>(p.max_anc, stages, plan_bufs) > kHalfCu) --stages;
    size_t lds = stream_lds_bytes<D, M>(p.max_anc, stages, plan_bufs);
    if (lds > kHalfCu) return FSTA_EUNSUPPORTED;      // ancestor lists too long: the other kernel
    const int per_cu = 2;
    (void)kTileBytes; (void)kQTiles; (void)kLeafTiles;
    const int wg_per_xcd = per_cu * (kCus / kXcds);
    const int slices_per_xcd = (p.heads_total + kXcds - 1) / kXcds;
    const long long pairs_per_xcd = (long long)slices_per_xcd * p.nb;
    (void)pairs_per_xcd;
    if (p.dry_run) return FSTA_OK;
    if (lds > 64 * 1024) {
        const int rc = allow_full_lds<&attn_stream_kernel<BF16, D, M, SPLIT>>();
        if (rc != FSTA_OK) return rc;
    }
    hipLaunchKernelGGL((attn_stream_kernel<BF16, D, M, SPLIT>), dim3((unsigned)(kXcds * wg_per_xcd)), dim3(M * 4), lds, stream, p,
                       stages, wg_per_xcd, plan_bufs);
    FSTA_HIP_OK(hipGetLastError());
    note_launch({"attn_stream_kernel", BF16 ? "true" : "false", {D, M, SPLIT ? 1 : 0, 0, 0, 0}, 3, 0x4u, 0, 0});
    return FSTA_OK;
}

template <bool BF16, bool SPLIT>
int launch_stream_dm(const AttnParams& p, int head_dim, hipStream_t stream) {
    if (head_dim == 128 && p.block_m == 128) return launch_stream<BF16, 128, 128, SPLIT>(p, stream);
    if (head_dim == 64 && p.block_m == 128) return launch_stream<BF16, 64, 128, SPLIT>(p, stream);
    if (head_dim == 128 && p.block_m == 64) return launch_stream<BF16, 128, 64, SPLIT>(p, stream);
    if (head_dim == 64 && p.block_m == 64) return launch_stream<BF16, 64, 64, SPLIT>(p, stream);
    return FSTA_EUNSUPPORTED;
}

}  // namespace

// On request (AttnParams::stream_mode > 0), no shared prefix, a block plan, blocks of 64 or 128 rows, head dim 64 or 128:
// FSTA_EUNSUPPORTED for everything else (the caller then takes the kernel with one workgroup per pair).
int launch_attention_stream(const AttnParams& p, int dtype, int head_dim, bool fast_pv, hipStream_t stream) {
    if (p.stream_mode <= 0) return FSTA_EUNSUPPORTED;       // measured slower than one workgroup per pair: on request only
    if (!p.plan || p.prefix != 0 || p.part_o || p.k_scale || p.v_scale) return FSTA_EUNSUPPORTED;
    if ((uint64_t)p.nk * (uint64_t)head_dim * 2u > 0xffffffffull) return FSTA_EUNSUPPORTED;
    if (dtype == FSTA_F16) return launch_stream_dm<false, false>(p, head_dim, stream);
    if (dtype == FSTA_BF16) return fast_pv ? launch_stream_dm<true, false>(p, head_dim, stream) : launch_stream_dm<true, true>(p, head_dim, stream);
    return FSTA_EUNSUPPORTED;
}

}  // namespace fsta

#ifdef FSTA_TIMELINE
// Instrumented build only: device buffer of (workgroups x waves x 20) uint64 that every launch of the streaming
// kernel fills (cycles spent in ten kinds of segment, then how often each was passed), or NULL.
extern "C" int fsta_stream_profile_buffer(unsigned long long* device_buffer) {
    FSTA_HIP_OK(hipMemcpyToSymbol(HIP_SYMBOL(fsta::g_stream_profile), &device_buffer, sizeof(device_buffer)));
    return FSTA_OK;
}
#endif
