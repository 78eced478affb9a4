// Matrix-core tree attention kernel for gfx950, 16 query rows per wave
// (v_mfma_f32_16x16x32): bf16 / fp16, head_dim 32/64/128, query blocks of 32/64/128 rows.
//
// Same structure as the 32-rows-per-wave kernel (tile list [leaf tiles | ancestor tiles |
// prefix tiles], K/V gathered straight into an LDS ring, transposed products S^T = K.Q^T and
// O^T += V^T.P^T, base-2 online softmax in the accumulator layout), but a wave keeps only 16
// query rows: 32 accumulator registers for O^T instead of 64 and 16 for Q instead of 32.  The
// kernel fits in 128 VGPRs, so four waves share a SIMD and cover each other's waits
// (gathers, LDS, the serial MFMA -> softmax -> MFMA chain of one tile); the price is that every
// K/V fragment is read from LDS by twice as many waves.
//
// Layouts of v_mfma_f32_16x16x32 (lane = 16*g + i): A holds row i, k = 8g .. 8g+7; B holds
// k = 8g .. 8g+7, column i; C holds rows 4g .. 4g+3 of column i.  With S^T the column is the
// query, so a lane owns keys 4g .. 4g+3 of each 16-key half of a tile for ONE query, and the
// 8 weights it ends up with are exactly its 8 k-slots of the B operand of O^T += V^T.P^T.
#include "fsta_mfma_common.h"
#include <type_traits>

// Cache policy (`aux` operand of the global->LDS transfers, 2 = non-temporal): rows that no other workgroup will ask
// for again go past the caches' retention -- the Q rows, the output rows (non-temporal stores) and, in a launch whose
// workgroups all run at once, the leaf tiles requested ahead of the plan.  K/V rows of larger launches are left alone:
// a block's own rows are the ancestors of later blocks, which find them in L2 (non-temporal leaf rows: +13 % on the
// reference's benchmark shape, measured).  Measured with Q and O non-temporal: cfg4 26.6 -> 23.5 us, cfg3 14.0 -> 13.0,
// the reference's benchmark at N = 2048 41.4 -> 38.4, cfg2 5.28 -> 5.14 (5.10 with the early leaf tiles as well).
constexpr int kStreamOnce = 2;

namespace fsta {
namespace {

using namespace mfma;

// Instrumented build (-DFSTA_TIMELINE, `python -m fstattention_amd.build --timeline`): every wave
// notes the 100 MHz clock at fixed points of the kernel and writes the notes out at the end;
// `python -m fstattention_amd.timeline` turns them into the mean time between the points.  The
// regular library contains none of this.
#ifdef FSTA_TIMELINE
constexpr int kStamps = 16;
__device__ uint64_t* g_timeline = nullptr;     // [workgroup][wave][kStamps + 2], set by fsta_timeline_buffer
__device__ __forceinline__ uint32_t stamp_clock() {
    // the constant 100 MHz clock (10 ns per tick, the same on every CU)
    return (uint32_t)__builtin_amdgcn_s_memrealtime();
}
#define FSTA_STAMP(i) do { if (lane == 0) tl_s[wave][i] = stamp_clock(); } while (0)
#else
#define FSTA_STAMP(i) do { } while (0)
#endif

constexpr int leaf_group16_for(int block_m) { return block_m >= 64 ? 2 : 1; }

// LDS of one workgroup: the ring of K|V tiles, then the workgroup's part of the block plan
// (header and ancestor keys, then leaf keys and mask words of its M/32 groups of 32 rows).
template <int D, int M>
__host__ __device__ inline size_t mfma16_lds_bytes(int max_anc, int stages) {
    const PlanLayout l = plan_layout(M, max_anc);
    return (size_t)stages * 2 * kTileN * D * 2 + (size_t)l.block_words * 4;
}

// 16 staged rows of W bytes each (LDS, `stride` apart) -> global rows `pitch` apart, 16 bytes per
// lane, whole rows per instruction; rows at or past rows_valid are not written.
template <int W>
__device__ __forceinline__ void flush_rows(const unsigned char* stage, int stride, unsigned char* dst, size_t pitch,
                                           int lane, int rows_valid) {
    constexpr int kLanesPerRow = W / 16;
    constexpr int kRowsPerStore = 64 / kLanesPerRow;
    constexpr int kIters = kRowsPerStore >= 16 ? 1 : 16 / kRowsPerStore;
    const int st_row = lane / kLanesPerRow, st_piece = lane % kLanesPerRow;
#pragma unroll
    for (int i = 0; i < kIters; ++i) {
        const int r = i * kRowsPerStore + st_row;
        if (r < 16 && r < rows_valid) {
            const u32x4 val = *reinterpret_cast<const u32x4*>(stage + r * stride + st_piece * 16);
            __builtin_nontemporal_store(val, reinterpret_cast<u32x4*>(dst + r * pitch + st_piece * 16));
        }
    }
}

// KS > 0: waves that share one group of 16 query rows, each taking every KS-th tile with its own
// running softmax (merged through LDS at the end).  KS = -2: two waves share a group of rows by
// the head dimension instead: both walk every tile and form the same weights, each accumulates
// and stores its half of O.  Nothing is exchanged or merged at the end, which shortens the chain
// of a launch with one or two ancestor tiles per block; the duplicated S and softmax work makes
// it the wrong choice for long tile lists.
// RUNS = the launch writes partial results into a workspace (AttnParams::part_o): workgroup `ksp` of a block
// takes the ksp-th run of prefix tiles (key_splits runs of split_tiles tiles; none at all with split_tiles = 0,
// when the prefix is another kernel's), workgroup 0 also the tree part.
// KV8 = K and V are stored as 8-bit floats (OCP e4m3) with one scale per (batch, head) slice each:
// rows are gathered as they are (half the bytes) into a staging ring; the workgroup widens every
// tile once into one of two 16-bit tiles in LDS (exact: e4m3 is a subset of both 16-bit types),
// one step ahead of its use, and the products run on those as they do for 16-bit K/V.  Widening a
// tile once per workgroup costs an eighth of widening the fragments in every wave.
template <bool BF16, int D, int M, bool SPLIT, int KS, bool RUNS, bool KV8 = false>
__global__ __launch_bounds__(M * 4 * (KS < 0 ? -KS : KS), 4) void attn_mfma16_kernel(AttnParams p, int stages, int early_leaf, int sub_shift) {
    using MM = Mma<BF16>;
    using T = typename MM::elem;
    using T2 = typename MM::elem2;
    using Frag = typename MM::frag;
    constexpr int kQGroups = M / 16;              // groups of 16 query rows
    constexpr int kLeafTiles = M / 32;            // 32-row tiles holding the block's own rows
    constexpr bool kDShare = KS < 0;              // the waves of a row group share the head dimension
    constexpr int kSplit = kDShare ? 1 : KS;      // tiles per step, dealt to the waves of a row group
    constexpr int kShares = kDShare ? -KS : KS;   // waves per row group
    static_assert(!kDShare || (KS == -2 && D >= 64), "head-dimension halves need two accumulator tiles each");
    static_assert(!KV8 || (KS == 1 && !RUNS), "8-bit K/V: one wave per row group, no key runs");
    constexpr int kLeafGroup = KV8 ? 1 : leaf_group16_for(M);
    constexpr int kWaves = kQGroups * kShares;
    constexpr int kThreads = kWaves * 64;
    constexpr int kCpr = D / 8;                   // 16-byte chunks per 16-bit row (Q rows, tiles in LDS)
    constexpr int kKvRowBytes = KV8 ? D : 2 * D;  // a K/V row in memory
    constexpr int kKvCpr = kKvRowBytes / 16;      // 16-byte chunks per gathered row
    constexpr int kRowsPerDma = 64 / kKvCpr;      // rows one wave-wide 1 KiB transfer covers
    constexpr int kDmaPerTile = 2 * kTileN / kRowsPerDma;   // K and V transfers of one tile
    constexpr int kDmaWaves = kDmaPerTile < kWaves ? kDmaPerTile : kWaves;   // waves that gather
    constexpr int kDmaPerWave = kDmaPerTile / kDmaWaves;
    static_assert(kDmaPerWave * kDmaWaves == kDmaPerTile, "transfers must split evenly over the waves");
    static_assert(kDmaPerWave == 1 || kDmaPerWave % 2 == 0, "a wave's transfers are K/V pairs of whole row groups");
    constexpr int kRowGroups = (kDmaPerWave + 1) / 2;   // row groups a wave touches per tile
    constexpr int kSteps = D / 32;                // MFMAs per 16-key half of S^T
    constexpr int kDTiles = D / 16;               // 16-row tiles of O^T
    constexpr int kOTiles = kDShare ? kDTiles / 2 : kDTiles;   // ... of which a wave accumulates these
    constexpr int kTileElems = kTileN * D;
    // Largest sum of a lane's 8 weights accepted without looking at the row maximum: far from
    // float overflow in l and O, and every single weight still converts to the 16-bit type.
    constexpr float kTrustedSum = BF16 ? 16777216.f : 32768.f;

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    // 16-bit K/V: ring [stages][K tile | V tile].  8-bit K/V: two widened tiles [2][K tile | V tile],
    // then the staging ring [stages][K rows | V rows] of bytes.
    T* ring = reinterpret_cast<T*>(smem);
    constexpr int kStageBytes = 2 * kTileN * D;           // one staged 8-bit tile
    unsigned char* stage8 = smem + 2 * 2 * kTileElems * 2;
    const int ring_bytes = KV8 ? 2 * 2 * kTileElems * 2 + stages * kStageBytes : stages * 2 * kTileElems * 2;
    // this workgroup's part of the block plan: header | ancestor keys | per 32 rows: leaf keys, mask words
    const int anc_cap = anc_tile_capacity(p.max_anc);
    const int common_words = kPlanHeaderWords + anc_cap * kTileN;
    const int group_words = kTileN * (1 + anc_cap);
    uint32_t* plan_s = reinterpret_cast<uint32_t*>(smem + ring_bytes);
    uint32_t* group_s = plan_s + common_words;            // [kLeafTiles][group_words]

    // All kernel arguments are fetched by ONE batch of scalar loads.  Left to itself the compiler
    // loads each field just before its first use, which puts four dependent round trips to the
    // argument segment in front of the first memory request of the workgroup.
    asm volatile("" ::"s"(p.q), "s"(p.k), "s"(p.v), "s"(p.o), "s"(p.lse), "s"(p.plan), "s"(p.key_shift),
                 "s"(p.nq), "s"(p.nk), "s"(p.prefix), "s"(p.max_anc), "s"(p.nb), "s"(p.heads_total), "s"(p.out_f32),
                 "s"(p.scale_log2e), "s"(stages), "s"(early_leaf), "s"(sub_shift));

    // Workgroup -> (slice, block), XCD-aware: every XCD gets whole (batch, head) slices, so all
    // query blocks of a slice share one L2 for the K/V rows they have in common.  The grid is
    // (8 XCDs x key runs, blocks, slices per XCD): workgroups go to the XCDs round-robin in x-fastest
    // order and the x extent is a multiple of 8, so blockIdx.x % 8 is the XCD, and the blocks of
    // a slice are dispatched next to each other.  (Grids past the y/z limits come as one long x
    // axis in the same order: `linear_grid`.)
    // Key runs (long shared prefix, few blocks): workgroup `ksp` of a block takes the ksp-th run
    // of prefix tiles, workgroup 0 also the tree part; each writes a normalised partial result
    // and its log-sum-exp, which a merge kernel joins.
    // A workgroup takes M consecutive rows: a whole block of the caller's, or (sub_shift = 1, small
    // grids) one half of a block of 2M rows, so that twice as many CUs share the launch.  The
    // half-block reads the block's ancestor list and its own rows of the mask and leaf list.
    const int linear_grid = (sub_shift >> 8) & 1;
    const int late_first = (sub_shift >> 9) & 1;
    sub_shift &= 0xff;
    const int xcd = blockIdx.x % kXcds;
    int ksp = 0, hz, part;
    if (linear_grid) {
        int within = blockIdx.x / kXcds;
        if constexpr (RUNS) {
            ksp = within % p.key_splits;
            within /= p.key_splits;
        }
        const int parts = p.nb << sub_shift;
        hz = (within / parts) * kXcds + xcd;
        part = within % parts;
    } else {
        if constexpr (RUNS) ksp = blockIdx.x / kXcds;
        hz = blockIdx.z * kXcds + xcd;
        part = blockIdx.y;
        if (late_first) {
            // (8 XCDs, slices per XCD, blocks): the late blocks of every slice, which have the longest
            // ancestor lists, are dispatched first, so that the two workgroups that come to share a CU in a
            // launch of more than one and at most two per CU are one of the long and one of the short half.
            hz = blockIdx.y * kXcds + xcd;
            part = gridDim.z - 1 - blockIdx.z;
        }
    }
    const bool tree = !RUNS || ksp == 0;
    const int j = part >> sub_shift;                                        // block of the caller's lists
    const int block_rows = M << sub_shift;                                  // rows per such block
    const int row_base = j * block_rows + (part & ((1 << sub_shift) - 1)) * M;   // first query row of this workgroup
    if (hz >= p.heads_total) return;

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
#ifdef FSTA_TIMELINE
    __shared__ uint32_t tl_s[16][kStamps];
    const uint64_t tl_begin = __builtin_amdgcn_s_memrealtime();     // 100 MHz, the same clock on every CU
    if ((tid & 63) < kStamps) tl_s[wave][tid & 63] = 0u;
    { const int lane = tid & 63; FSTA_STAMP(0); }
#endif
    const int qgroup = wave % kQGroups;   // which 16 query rows
    const int split = wave / kQGroups;    // which share of the tiles (of the head dimension)
    const int dt0 = kDShare ? split * kOTiles : 0;   // first accumulator tile of this wave
    const int lane = tid & 63;
    const int ql = lane & 15;        // query (column of S^T / O^T) of this lane
    const int g = lane >> 4;         // which quarter of the rows of an accumulator tile
    const int row_in_block = qgroup * 16 + ql;

    const T* qb = static_cast<const T*>(p.q) + (size_t)hz * p.nq * D;
    const unsigned char* kb = static_cast<const unsigned char*>(p.k) + (size_t)hz * p.nk * kKvRowBytes;
    const unsigned char* vb = static_cast<const unsigned char*>(p.v) + (size_t)hz * p.nk * kKvRowBytes;
    // scale under the exp2: softmax scale, log2(e) and, for 8-bit K, the slice's K scale
    float sc = p.scale_log2e;
    if (KV8 && p.k_scale) sc *= p.k_scale[hz];

    // ---- start-up: every request that needs no metadata goes out together with the metadata ----
    // Loads and transfers retire in issue order.  The block plan goes first (the ancestor requests
    // hang on it), then the Q rows and, in a launch whose workgroups all run at once, the first
    // leaf tiles.  The number of transfers issued after the plan is a compile-time constant: the
    // wait for the plan can then leave exactly those in flight.
    // The plan holds what a workgroup needs of the tree in the form it is used in: 32-bit K/V rows
    // per tile slot (empty slots repeat a row), leaf validity, mask words per (ancestor tile, row).
    // Record of block j: common part, then one group per 32 rows; this workgroup takes the
    // common part and its own M/32 groups, which land next to each other in LDS.
    // In a small launch (`early_leaf`) every wave copies the whole piece for itself (it is a few
    // hundred bytes, all waves write the same values to the same place): a wave then depends on
    // no other wave until the first tile is consumed.  Otherwise the waves share the copy and
    // meet at a barrier.
    {
        const int block_groups = block_rows / kTileN;
        const char* rec = reinterpret_cast<const char*>(p.plan) +
                          (size_t)j * (size_t)(common_words + block_groups * group_words) * 4;
        const int common_chunks = common_words / 4;                       // 16-byte pieces
        const int chunks = common_chunks + kLeafTiles * (group_words / 4);
        const uint32_t group_skip = (uint32_t)(((row_base - j * block_rows) / kTileN) * group_words * 4);
        for (int piece = early_leaf ? 0 : wave; piece * 64 < chunks; piece += early_leaf ? 1 : kWaves) {
            const int c = piece * 64 + lane;
            if (c < chunks)
                __builtin_amdgcn_global_load_lds(
                    (const void __attribute__((address_space(1)))*)(rec + (size_t)((uint32_t)c * 16u + (c >= common_chunks ? group_skip : 0u))),
                    (void __attribute__((address_space(3)))*)(reinterpret_cast<char*>(plan_s) + piece * 1024),
                    16, 0, 0);
        }
    }
    // Q rows of this wave: whole rows straight into LDS, K-tile swizzle, parked in the last ring
    // slots until the fragments have been read; the first tiles are requested into the other slots
    // as soon as the plan is there, without waiting for the Q rows.  Rows past the end of
    // a ragged last block are read as the last row and never stored.
    const int q_row = lane / kCpr, q_slot = lane % kCpr;           // Q rows are 16-bit
    const int dma_row = lane / kKvCpr, dma_slot = lane % kKvCpr;   // K/V rows as stored
    constexpr int kQRowsPerDma = 64 / kCpr;
    constexpr int kQDma = 16 / kQRowsPerDma;
    static_assert(kQDma >= 1, "a transfer covers at most the wave's 16 rows");
    // (a small grid has LDS to spare: Q then gets an area of its own behind the plan, the
    // whole ring is free from the start and the fragments are read after the ancestor tiles have
    // been requested instead of in front of the first barrier)
    // (8-bit K/V: Q waits in the widened tiles, which are first written behind the first barrier)
    T* qstage = early_leaf ? reinterpret_cast<T*>(group_s + kLeafTiles * group_words) + wave * 16 * D
                : KV8      ? ring + wave * 16 * D
                           : ring + (size_t)stages * 2 * kTileElems - (kWaves - wave) * 16 * D;
    static_assert(!KV8 || kWaves * 16 <= 4 * kTileN, "Q must fit into the two widened tiles");
#pragma unroll
    for (int i = 0; i < kQDma; ++i) {
        const int r = i * kQRowsPerDma + q_row;
        const int grow = min(row_base + qgroup * 16 + r, p.nq - 1);
        const uint32_t off = (uint32_t)grow * (uint32_t)(D * sizeof(T)) + (uint32_t)k_chunk<D>(r, q_slot) * 16u;
        __builtin_amdgcn_global_load_lds(
            (const void __attribute__((address_space(1)))*)(reinterpret_cast<const char*>(qb) + (size_t)off),
            (void __attribute__((address_space(3)))*)(qstage + i * 512), 16, 0, kStreamOnce);
    }

    // ---- gather: HBM -> LDS, 16 bytes per lane, no registers in between --------
    // Transfer t2 of a tile moves row group t2/2 = rows [kRowsPerDma*(t2/2), +kRowsPerDma) of K
    // (t2 even) or V (t2 odd); wave w < kDmaWaves issues transfers [w*kDmaPerWave, +kDmaPerWave).
    // Lane i lands at LDS byte 16*i of the transfer, i.e. row i / kCpr, chunk slot i % kCpr, and
    // fetches the chunk that the XOR swizzle assigns to that slot.  Every gathering wave issues
    // exactly kDmaPerWave transfers per tile: the vmcnt bookkeeping counts on it.
    // A lane's address is slice base (uniform) + a 32-bit byte offset: row * row pitch + the chunk
    // its slot holds.  The chunk offsets are fixed for the kernel's life (dma_anc / dma_leaf); a
    // request then costs one multiply-add per transfer.  (The launcher keeps slices below 4 GiB.)
    // (dma_flip = ancestor-tile offset XOR leaf-tile offset, applied under an all-ones / all-zeros
    // word: a select between elements of two arrays makes the compiler address the arrays through a
    // selected pointer, i.e. keep them in scratch memory, whose reloads share vmcnt with the ring)
    uint32_t dma_leaf[kDmaPerWave], dma_flip[kDmaPerWave];
#pragma unroll
    for (int i = 0; i < kDmaPerWave; ++i) {
        const int t2 = wave * kDmaPerWave + i;
        const int r = (t2 >> 1) * kRowsPerDma + dma_row;
        // V of a leaf tile is read row-wise like K (no transposing read), so it takes K's swizzle
        if constexpr (KV8) {   // staged as stored (chunk = slot); the swizzle is applied when the tile is widened
            dma_leaf[i] = 0u;
            dma_flip[i] = 0u;
        } else {
            dma_leaf[i] = (uint32_t)k_chunk<D>(r, dma_slot) * 16u;
            dma_flip[i] = (t2 & 1) ? ((uint32_t)v16_chunk<D>(r, dma_slot) * 16u) ^ dma_leaf[i] : 0u;
        }
    }
    auto issue_rows = [&](int t, int slot, const int (&rows)[kRowGroups], bool once) {
        unsigned char* dst_tile = KV8 ? stage8 + slot * kStageBytes : reinterpret_cast<unsigned char*>(ring + slot * 2 * kTileElems);
        constexpr int kHalf = KV8 ? kStageBytes / 2 : kTileElems * 2;   // bytes from the K part to the V part
        const uint32_t anc_tile = t < kLeafTiles ? 0u : 0xffffffffu;
#pragma unroll
        for (int i = 0; i < kDmaPerWave; ++i) {
            const int t2 = wave * kDmaPerWave + i;
            const int u = t2 >> 1;
            const bool is_v = t2 & 1;
            const uint32_t off = (uint32_t)rows[i >> 1] * (uint32_t)kKvRowBytes +
                                 (KV8 ? (uint32_t)dma_slot * 16u : dma_leaf[i] ^ (dma_flip[i] & anc_tile));
            const char* src = reinterpret_cast<const char*>(is_v ? vb : kb) + (size_t)off;
            // (`once` is a constant at both call sites: one of the two forms remains)
            if (once)
                __builtin_amdgcn_global_load_lds(
                    (const void __attribute__((address_space(1)))*)src,
                    (void __attribute__((address_space(3)))*)(dst_tile + (is_v ? kHalf : 0) + u * 1024), 16, 0, kStreamOnce);
            else
                __builtin_amdgcn_global_load_lds(
                    (const void __attribute__((address_space(1)))*)src,
                    (void __attribute__((address_space(3)))*)(dst_tile + (is_v ? kHalf : 0) + u * 1024), 16, 0, 0);
        }
    };
    // A valid leaf slot of row r names r's own key (reference utils.py:121-122), so the first
    // leaf tiles are requested on that assumption, in the ring slots Q does not occupy, while
    // the lists are still on their way.  Lists that say otherwise are honoured below.
    // This shortens the start-up chain of a launch whose workgroups all run at once; a launch
    // with several rounds of workgroups hides that chain anyway and would only pay for the
    // rows of empty slots, so the launcher asks for it (`early_leaf`) for small grids only.
    constexpr int kEarlyTiles = kLeafTiles < 2 ? kLeafTiles : 2;   // the launcher provides ring slots for Q plus these
    const int n_spec = early_leaf ? kEarlyTiles : 0;
#pragma unroll
    for (int t = 0; t < kEarlyTiles; ++t) {
        if (t >= n_spec || (kDmaWaves < kWaves && wave >= kDmaWaves)) break;
        int rows[kRowGroups];
#pragma unroll
        for (int i = 0; i < kRowGroups; ++i)
            rows[i] = min(p.prefix + row_base + t * kTileN + ((wave * kDmaPerWave) / 2 + i) * kRowsPerDma + dma_row, p.nk - 1);
        issue_rows(t, t, rows, true);
    }

    FSTA_STAMP(1);    // all start-up requests are out
    const bool gathers = !(kDmaWaves < kWaves && wave >= kDmaWaves);
    // Q fragments: B operand of S^T = K.Q^T, lane holds Q[q][32s + 8g .. +7].  Only the leaf
    // tiles requested above were issued after the Q rows.
    Frag qf[kSteps];
    auto read_q = [&](int tiles_issued_since) {
        wait_tiles_outstanding<kDmaPerWave>(gathers ? tiles_issued_since : 0);
        u32x4 qraw[kSteps];
#pragma unroll
        for (int s = 0; s < kSteps; ++s)
            qraw[s] = lds_read_b128(lds_addr(qstage + ql * D + k_chunk<D>(ql, 4 * s + g) * 8));
        lds_wait();
#pragma unroll
        for (int s = 0; s < kSteps; ++s) {
            lds_tie(qraw[s]);
            qf[s] = __builtin_bit_cast(Frag, qraw[s]);
        }
    };
    if (early_leaf) {
        // this wave's own copy of the plan has landed; the Q rows and leaf tiles stay in flight
        if (gathers && n_spec) wait_vmcnt<kQDma + kEarlyTiles * kDmaPerWave>();
        else wait_vmcnt<kQDma>();
    } else {
        // the plan has landed (it usually comes from L2: every slice reads the same one); the Q rows, which come
        // from HBM, stay in flight while the first tiles are requested into the ring slots Q does not occupy
        wait_vmcnt<kQDma>();
        ring_barrier();   // everybody's pieces of the plan have landed
    }
    FSTA_STAMP(2);    // the plan is here
    // From the plan: ancestor count, validity of this lane's own leaf slot and, after early leaf
    // requests, whether any valid leaf slot names another row than the one requested (lane i looks
    // at slot i of the tiles requested: every wave sees all of them and decides alike).
    const int first_group = (row_base - j * block_rows) / kTileN;   // this workgroup's first group of 32 rows
    bool leaf_ok, restart = false;
    int n_anc;
    {
        uint32_t head = lds_read_b32(lds_addr(plan_s));
        uint32_t my_valid = lds_read_b32(lds_addr(plan_s + kPlanLeafValid + first_group + (row_in_block >> 5)));
        uint32_t spec_valid = 0u, spec_key = 0u;
        const bool checks = lane < n_spec * kTileN;
        if (checks) {
            spec_valid = lds_read_b32(lds_addr(plan_s + kPlanLeafValid + first_group + (lane >> 5)));
            spec_key = lds_read_b32(lds_addr(group_s + (lane >> 5) * group_words + (lane & 31)));
        }
        lds_wait();
        lds_tie(head);
        lds_tie(my_valid);
        lds_tie(spec_valid);
        lds_tie(spec_key);
        n_anc = __builtin_amdgcn_readfirstlane((int)head);
        leaf_ok = tree && ((my_valid >> (row_in_block & 31)) & 1u);
        const bool other = checks && ((spec_valid >> (lane & 31)) & 1u) &&
                           (int)spec_key + p.key_shift != p.prefix + row_base + lane;
        restart = __ballot(other) != 0ull;
    }
    n_anc = tree ? min(max(n_anc, 0), p.max_anc) : 0;
    const int listed_tiles = kLeafTiles + (n_anc + kTileN - 1) / kTileN;
    int prefix_first = 0, prefix_end = (p.prefix + kTileN - 1) / kTileN;   // this workgroup's prefix tiles
    if constexpr (RUNS) {
        prefix_first = min(ksp * p.split_tiles, prefix_end);
        prefix_end = min(prefix_first + p.split_tiles, prefix_end);
    }
    const int total_tiles = listed_tiles + prefix_end - prefix_first;
    const int prefix_shift = prefix_first - listed_tiles;   // list position t holds prefix tile t + prefix_shift

    auto issue = [&](int t, int slot) {
        if (kDmaWaves < kWaves && wave >= kDmaWaves) return;
        int rows[kRowGroups];
        if (kDShare || t < listed_tiles) {   // (head-dimension pairing is launched without a prefix)
            const uint32_t* keys = t < kLeafTiles ? group_s + t * group_words
                                                  : plan_s + kPlanHeaderWords + (t - kLeafTiles) * kTileN;
#pragma unroll
            for (int i = 0; i < kRowGroups; ++i)   // (the clamp keeps a plan made for more K/V rows from reaching past them)
                rows[i] = min((int)keys[((wave * kDmaPerWave) / 2 + i) * kRowsPerDma + dma_row] + p.key_shift, p.nk - 1);
        } else {
#pragma unroll
            for (int i = 0; i < kRowGroups; ++i)
                rows[i] = min((t + prefix_shift) * kTileN + ((wave * kDmaPerWave) / 2 + i) * kRowsPerDma + dma_row, p.prefix - 1);
        }
        issue_rows(t, slot, rows, false);
    };

    // Ring bookkeeping, in tiles: `issued` gathers started, `consumed` tiles everyone is done
    // with; tile i lives in slot i % stages.  begin_step(n) makes tiles [consumed, consumed+n)
    // usable: wait until at most the gathers issued after them are outstanding (they retire in
    // order), barrier (everyone's share has landed, everyone is done with the tiles before),
    // then refill the slots that barrier freed.
    int issued = n_spec, issue_slot = n_spec, consumed = 0, slot = 0;   // n_spec < stages
    if (!tree) issued = consumed = kLeafTiles;   // no tree part: the list starts behind the leaf tiles
    auto refill_to = [&](int limit) {   // requests tiles up to (not including) list position `limit`
        while (issued < total_tiles && issued < limit) {
            issue(issued, issue_slot);
            ++issued;
            issue_slot = issue_slot + 1 == stages ? 0 : issue_slot + 1;
        }
    };
    auto refill = [&]() { refill_to(consumed + stages); };
    // 8-bit K/V: tile t of the list waits in staging slot t % stages and is widened into 16-bit tile
    // t % 2.  Eight values (8 bytes) per piece: K rows land in the K swizzle, V rows of ancestor
    // and prefix tiles in the swizzle of the transposing read, V rows of leaf tiles in K's.
    int widened = consumed;     // tiles widened so far (by this wave's share; complete behind the next barrier)
    auto widen = [&](int t) {
        if constexpr (KV8) {
            const unsigned char* src = stage8 + (t % stages) * kStageBytes;
            T* dst = ring + (t & 1) * 2 * kTileElems;
            constexpr int kPieces = 2 * kTileN * D / 8;        // K pieces, then V pieces
            constexpr int kPerThread = kPieces / kThreads;     // (a power of two)
            static_assert(kPerThread * kThreads == kPieces, "pieces split evenly over the threads");
            const bool leaf_tile = t < kLeafTiles;
            // two pieces are requested before the first one is widened (more would not fit the registers
            // of the 64-row blocks): one LDS round trip per pair
            constexpr int kBatch = kPerThread >= 2 ? 2 : 1;
            static_assert(kPerThread % kBatch == 0, "pieces come in pairs (or one per thread)");
#pragma unroll 1
            for (int i0 = 0; i0 < kPerThread; i0 += kBatch) {
                u32x2 raw[kBatch];
#pragma unroll
                for (int i = 0; i < kBatch; ++i) {
                    const int piece = (i0 + i) * kThreads + tid;
                    const int is_v = piece >= kPieces / 2 ? 1 : 0;
                    const int idx = piece - is_v * (kPieces / 2);
                    raw[i] = lds_read_b64(lds_addr(src + is_v * (kStageBytes / 2) + (idx / kCpr) * D + (idx % kCpr) * 8));
                }
                lds_wait();
#pragma unroll
                for (int i = 0; i < kBatch; ++i) {
                    const int piece = (i0 + i) * kThreads + tid;
                    const int is_v = piece >= kPieces / 2 ? 1 : 0;
                    const int idx = piece - is_v * (kPieces / 2);
                    const int row = idx / kCpr, c = idx % kCpr;
                    lds_tie(raw[i]);
                    const uint32_t lo = raw[i][0], hi = raw[i][1];
                    u32x4 wide;
                    if constexpr (BF16) {
                        wide[0] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo, 1.0f, false));
                        wide[1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo, 1.0f, true));
                        wide[2] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi, 1.0f, false));
                        wide[3] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi, 1.0f, true));
                    } else {
                        wide[0] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(lo, 1.0f, false));
                        wide[1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(lo, 1.0f, true));
                        wide[2] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(hi, 1.0f, false));
                        wide[3] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(hi, 1.0f, true));
                    }
                    const int chunk = (is_v && !leaf_tile) ? v16_chunk<D>(row, c) : k_chunk<D>(row, c);
                    lds_write_b128(lds_addr(dst + is_v * kTileElems + row * D + chunk * 8), wide);
                }
            }
        }
    };
    bool all_landed = false;   // every tile of the list is in LDS and every wave knows it
    auto begin_step = [&](int n) {
        if constexpr (KV8) {
            // (n == 1) Tile `consumed` must be widened and visible; tile consumed + 1 is widened during
            // this step.  A staging slot is free again once its tile has been widened by everyone,
            // i.e. behind the barrier after that: the slots of tiles up to `consumed` here.
            if (widened == consumed) {   // first step: nothing widened yet
                wait_tiles_outstanding<kDmaPerWave>(max(issued - consumed - 1, 0));
                ring_barrier();
                widen(consumed);
                widened = consumed + 1;
            }
            const bool more = consumed + 1 < total_tiles;
            if (more && issued < consumed + 2) refill_to(consumed + 2);   // (a ring of one slot)
            if (more) wait_tiles_outstanding<kDmaPerWave>(max(issued - consumed - 2, 0));
            ring_barrier();
            refill_to(consumed + 1 + stages);
            if (more) {
                widen(consumed + 1);
                widened = consumed + 2;
            }
            return;
        }
        if (kDShare && all_landed) return;
        if (kDShare && issued == total_tiles && consumed >= kLeafTiles) {
            // short list, the last tiles are in flight: wait for all of them once instead of
            // passing a barrier per step
            wait_vmcnt<0>();
            ring_barrier();
            all_landed = true;
            return;
        }
        if (issued < min(consumed + n, total_tiles)) {
            // ring too shallow (long ancestor lists leave little LDS) for this step's tiles to be
            // in flight already: free the slots first, then request them
            ring_barrier();
            refill();
        }
        wait_tiles_outstanding<kDmaPerWave>(max(issued - consumed - n, 0));
        ring_barrier();
        refill();
    };
    auto end_step = [&](int n) {
        consumed += n;
        slot += n;
        if (slot >= stages) slot -= stages;
    };
    auto tile_ptr = [&](int i) {   // K tile of the i-th tile of the current step; V follows it
        if constexpr (KV8) return ring + ((consumed + i) & 1) * 2 * kTileElems;
        int sl = slot + i;
        if (sl >= stages) sl -= stages;
        return ring + sl * 2 * kTileElems;
    };
    if (restart) {   // a leaf list that names other rows than the ones requested: start the ring over
        wait_vmcnt<0>();
        __syncthreads();
        issued = consumed;
        issue_slot = 0;
    }
    if (!early_leaf) {
        // (Q is parked in the last ring slots -- 8-bit K/V: in the widened tiles, the whole staging ring is free)
        constexpr int kQSlots = KV8 ? 0 : (kWaves * 16 + 2 * kTileN - 1) / (2 * kTileN);
        refill_to(consumed + stages - kQSlots);
        read_q(issued - consumed);
        ring_barrier();   // everybody has read its Q rows: their slots are free
    }
    refill();
    FSTA_STAMP(3);    // ancestor tiles requested
    if (early_leaf) read_q(issued);
    FSTA_STAMP(4);    // Q fragments in registers

    float m_i = -INFINITY, l_i = 0.f;
    f32x4 o[kOTiles];
#pragma unroll
    for (int dt = 0; dt < kOTiles; ++dt) o[dt] = f32x4{0.f, 0.f, 0.f, 0.f};

    // Leaf tile i = the block's own rows 32i .. 32i+31 (reference fstattention.py:86-91,104-107):
    // query r sees exactly row r of it.  The two waves owning those rows take one dot product
    // per query from it on the vector ALU and seed their running softmax with it.
    for (int base = tree ? 0 : kLeafTiles; base < kLeafTiles; base += kLeafGroup) {
        begin_step(kLeafGroup);
        FSTA_STAMP(5);    // (last) leaf tile has landed
        const int my_tile = qgroup >> 1;
        if ((kDShare || split == 0) && my_tile >= base && my_tile < base + kLeafGroup && __ballot(leaf_ok) != 0ull) {
            const T* kt = tile_ptr(my_tile - base);
            const T* vt = kt + kTileElems;
            const int row = (qgroup & 1) * 16 + ql;   // this query's row of the leaf tile
            float part[2] = {0.f, 0.f};
            u32x2 vraw[kOTiles];   // the row's V values are requested together with its K values
            {
                u32x4 kraw[kSteps];
#pragma unroll
                for (int ks = 0; ks < kSteps; ++ks)
                    kraw[ks] = lds_read_b128(lds_addr(kt + row * D + k_chunk<D>(row, 4 * ks + g) * 8));
#pragma unroll
                for (int dt = 0; dt < kOTiles; ++dt)   // accumulator rows 4g .. 4g+3 of tile dt0 + dt: 4 head dims
                    vraw[dt] = lds_read_b64(lds_addr(vt + row * D + k_chunk<D>(row, 2 * (dt0 + dt) + (g >> 1)) * 8 + 4 * (g & 1)));
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
            const float dot = sum_quarters(part[0] + part[1]);
#pragma unroll
            for (int dt = 0; dt < kOTiles; ++dt) lds_tie(vraw[dt]);
            if (leaf_ok) {
                m_i = dot * sc;
                l_i = g == 0 ? 1.f : 0.f;
#pragma unroll
                for (int dt = 0; dt < kOTiles; ++dt) {
                    o[dt][0] = MM::low(vraw[dt][0]);
                    o[dt][1] = MM::high(vraw[dt][0]);
                    o[dt][2] = MM::low(vraw[dt][1]);
                    o[dt][3] = MM::high(vraw[dt][1]);
                }
            }
        }
        end_step(kLeafGroup);
    }
    FSTA_STAMP(6);    // leaf step done
#ifdef FSTA_TIMELINE
    int tl_tile = 0;
#endif

    // Ancestor tiles under the packed tree mask, then the dense shared prefix; kSplit tiles per
    // step, tile consumed+s by the waves of share s.
    // Byte offsets of this lane's fragments inside a tile.  The XOR swizzles only touch the
    // chunk bits, so the fragment of K-step ks / head-dim tile dt sits at offset0 ^ (ks << 6)
    // resp. offset0 ^ (dt << 5), and the rows 16 further down at a fixed distance.
    constexpr int kHalfTileBytes = 16 * D * 2;   // 16 rows
    const uint32_t k_lane0 = (uint32_t)(ql * D + k_chunk<D>(ql, g) * 8) * 2;
    const int tr_r0 = 4 * g + (ql >> 2);   // this lane's key row for the transposing read
    const int tr_col = 4 * (ql & 3);       // head dim within the 16-row tile
    const uint32_t v_lane0 = (uint32_t)(tr_r0 * D + v16_chunk<D>(tr_r0, tr_col >> 3) * 8 + (tr_col & 7)) * 2;
    // this row's mask words, one per ancestor tile (bits of empty slots are clear in the plan)
    const uint32_t* my_mask = group_s + (row_in_block >> 5) * group_words + kTileN + (row_in_block & 31);
    // One step of NT tiles (32 keys each) for this wave: S^T, mask, weights, O^T.  NT = 2 (the waves that share
    // the head dimension: short lists, every tile in LDS before the first step) treats two tiles as one of 64
    // keys: one pass through the weights, one check of the running maximum, one chain MFMA -> vector ALU -> MFMA
    // instead of two, which is what a lone wave on its SIMD waits for.
    typedef const u32x4 __attribute__((address_space(3))) * lds_u32x4;
    constexpr int kHalf = kOTiles / 2;
    auto step_tiles = [&](auto nt_tag, const T* const (&kts)[2], const uint32_t (&words)[2]) {
        constexpr int NT = decltype(nt_tag)::value;
        // S^T = K_tile . Q^T, two halves of 16 keys per tile
        f32x4 s[2 * NT];
#pragma unroll
        for (int tl = 0; tl < NT; ++tl) {
            const uint32_t k_addr0 = lds_addr(kts[tl]) + k_lane0;
#pragma unroll
            for (int sub = 0; sub < 2; ++sub) {
                s[2 * tl + sub] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < kSteps; ++ks) {
                    const u32x4 raw = *(lds_u32x4)(uintptr_t)((k_addr0 ^ (uint32_t)(ks << 6)) + sub * kHalfTileBytes);
                    s[2 * tl + sub] = mfma16(__builtin_bit_cast(Frag, raw), qf[ks], s[2 * tl + sub]);
                }
            }
        }
        // V fragments (A operand of O^T += V^T.P^T: rows are head dims) through the transposing
        // read: k-slots 8g .. 8g+3 are keys 4g .. 4g+3, k-slots 8g+4 .. 8g+7 keys 16+4g .. 16+4g+3.
        // Half of the head-dim tiles are requested now (LDS latency hides behind the softmax),
        // the other half behind the first MFMAs.
        auto read_v = [&](VPair (&f)[kHalf], const T* vt, int first_dt) {
            const uint32_t v_addr0 = lds_addr(vt) + v_lane0;
#pragma unroll
            for (int i = 0; i < kHalf; ++i) {
                const uint32_t addr = v_addr0 ^ (uint32_t)((first_dt + i) << 5);
                f[i].a = lds_read_tr16(addr);
                f[i].b = lds_read_tr16_at<kHalfTileBytes>(addr);
            }
        };
        auto tie_v = [&](VPair (&f)[kHalf]) {
            lds_wait();
#pragma unroll
            for (int i = 0; i < kHalf; ++i) { lds_tie(f[i].a); lds_tie(f[i].b); }
        };
        VPair v0[kHalf], v1[kHalf];
        read_v(v0, kts[0] + kTileElems, dt0);
        // mask + online softmax; register j of half `sub` is key 16*sub + 4g + j.  The scale rides
        // in the FMA under the exp2.
        float sv[8 * NT];
        uint32_t own_bits = 0u;   // mask bits of the keys this lane holds
#pragma unroll
        for (int tl = 0; tl < NT; ++tl) {
            const uint32_t wsh = words[tl] >> (4 * g);
            own_bits |= wsh & 0x000f000fu;
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                // bit -> all-ones / all-zeros (v_bfe_i32), then a bitwise select against -inf (v_bfi_b32)
                const uint32_t keep = (uint32_t)__builtin_amdgcn_sbfe((int)wsh, 16 * (r / 4) + (r % 4), 1);
                const float score = s[2 * tl + r / 4][r % 4];   // (a copy: bit_cast straight from a vector element reads element 0)
                const uint32_t bits = __builtin_bit_cast(uint32_t, score);
                sv[8 * tl + r] = __builtin_bit_cast(float, (bits & keep) | (0xff800000u & ~keep));
            }
        }
        // The weights are first taken against the running maximum as it stands: no row maximum,
        // no cross-lane exchange.  That is exact as long as no weight gets large (a power-of-two
        // factor on a row's weights cancels in O / l); the sum of the lane's weights is the check.
        // A row without a maximum so far, or a sum above the limit (or not a number), sends the
        // wave through the full update below: row maximum, raise, rescale, weights again.
        float pw[8 * NT];
        float rowsum = 0.f;
        {
            const float neg_m = m_i == -INFINITY ? 0.f : -m_i;
#pragma unroll
            for (int r = 0; r < 8 * NT; ++r) {
                pw[r] = __builtin_amdgcn_exp2f(__builtin_fmaf(sv[r], sc, neg_m));
                rowsum += pw[r];
            }
        }
        const bool redo = !(rowsum <= kTrustedSum) || (m_i == -INFINITY && own_bits != 0u);
        if (__ballot(redo) != 0ull) {
            float mx_raw = sv[0];
#pragma unroll
            for (int r = 1; r < 8 * NT; ++r) mx_raw = fmaxf(mx_raw, sv[r]);
            mx_raw = max_quarters(mx_raw);
            const float mx = mx_raw * sc;   // the scale is positive here
            // raise only rows that would otherwise keep a weight above 2^kRescaleSlack
            const bool raise = mx > m_i + kRescaleSlack || (m_i == -INFINITY && mx > -INFINITY);
            const float alpha = raise ? __builtin_amdgcn_exp2f(m_i - mx) : 1.f;   // exp2(-inf) = 0
            if (raise) m_i = mx;
            l_i *= alpha;
#pragma unroll
            for (int dt = 0; dt < kOTiles; ++dt)
#pragma unroll
                for (int r = 0; r < 4; ++r) o[dt][r] *= alpha;
            const float neg_m = m_i == -INFINITY ? 0.f : -m_i;
            rowsum = 0.f;
#pragma unroll
            for (int r = 0; r < 8 * NT; ++r) {
                pw[r] = __builtin_amdgcn_exp2f(__builtin_fmaf(sv[r], sc, neg_m));
                rowsum += pw[r];
            }
        }
        l_i += rowsum;
        // P^T fragments: the 8 weights of a tile are this lane's 8 k-slots
        Frag ph[NT], pl[NT];
#pragma unroll
        for (int tl = 0; tl < NT; ++tl) {
            u32x4 hi4, lo4;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float a = pw[8 * tl + 2 * e], b = pw[8 * tl + 2 * e + 1];
                const uint32_t hi = MM::pack(a, b);
                hi4[e] = hi;
                if (SPLIT) lo4[e] = MM::pack(a - MM::low(hi), b - MM::high(hi));
            }
            ph[tl] = __builtin_bit_cast(Frag, hi4);
            if (SPLIT) pl[tl] = __builtin_bit_cast(Frag, lo4);
        }
        // O^T += V_tile^T . P^T
#pragma unroll
        for (int tl = 0; tl < NT; ++tl) {
            tie_v(v0);
            read_v(v1, kts[tl] + kTileElems, dt0 + kHalf);
#pragma unroll
            for (int i = 0; i < kHalf; ++i) o[i] = mfma16(__builtin_bit_cast(Frag, v0[i]), ph[tl], o[i]);
            if (SPLIT) {
#pragma unroll
                for (int i = 0; i < kHalf; ++i) o[i] = mfma16(__builtin_bit_cast(Frag, v0[i]), pl[tl], o[i]);
            }
            tie_v(v1);
            if (tl + 1 < NT) read_v(v0, kts[tl + 1] + kTileElems, dt0);
#pragma unroll
            for (int i = 0; i < kHalf; ++i) o[kHalf + i] = mfma16(__builtin_bit_cast(Frag, v1[i]), ph[tl], o[kHalf + i]);
            if (SPLIT) {
#pragma unroll
                for (int i = 0; i < kHalf; ++i) o[kHalf + i] = mfma16(__builtin_bit_cast(Frag, v1[i]), pl[tl], o[kHalf + i]);
            }
        }
    };
    while (consumed < total_tiles) {
#ifdef FSTA_TIMELINE
        if (tl_tile < 5) { FSTA_STAMP(7 + tl_tile); }     // begin of ancestor / prefix step tl_tile
        ++tl_tile;
#endif
        if constexpr (kDShare) {
            // (no prefix, no skipping: the launch code sends only short ancestor lists here)
            const int n_here = total_tiles - consumed >= 2 ? 2 : 1;
            begin_step(n_here);
            const T* const kts[2] = {tile_ptr(0), tile_ptr(1)};
            const int t = consumed;
            end_step(n_here);
            const uint32_t w0 = t < listed_tiles ? my_mask[(t - kLeafTiles) * kTileN] : 0u;
            if (n_here == 2) {
                const uint32_t w1 = t + 1 < listed_tiles ? my_mask[(t + 1 - kLeafTiles) * kTileN] : 0u;
                const uint32_t words[2] = {w0, w1};
                step_tiles(std::integral_constant<int, 2>{}, kts, words);
            } else {
                const uint32_t words[2] = {w0, 0u};
                step_tiles(std::integral_constant<int, 1>{}, kts, words);
            }
        } else {
            begin_step(kSplit);
            const int t = consumed + split;
            const T* const kts[2] = {tile_ptr(split), nullptr};
            end_step(kSplit);
            uint32_t word = 0u;
            if (t < listed_tiles) {
                word = my_mask[(t - kLeafTiles) * kTileN];
            } else if (t < total_tiles) {
                const int left = p.prefix - (t + prefix_shift) * kTileN;
                word = left >= 32 ? 0xffffffffu : ((1u << left) - 1u);
            }
            if (kSplit > 1 && t >= total_tiles) continue;   // this share has no tile in the last step
            // A tile none of this wave's 16 queries attends to (10-30 % of the ancestor tiles of deep
            // trees) is skipped where a workgroup walks long lists.
            if (__ballot(word != 0u) == 0ull) continue;
            const uint32_t words[2] = {word, 0u};
            step_tiles(std::integral_constant<int, 1>{}, kts, words);
        }
    }

    FSTA_STAMP(12);   // all tiles done
    // ---- end of the tile list: normalise, write O once (and the base-2 log-sum-exp) --------
    // In the accumulator layout 16 neighbouring lanes hold 16 different rows of O, which the
    // memory pipeline would write as 64 separate 8-byte pieces per instruction.  A wave turns
    // its block around in LDS instead (the ring is free by now) and stores whole rows, 16 bytes
    // per lane; columns go in passes of at most 2*D bytes per row.
    constexpr int kStageStride = D * 2 + 16;     // bytes per staged row (padded against bank conflicts)
    const int first_row = row_base + qgroup * 16;
    // (with key runs: a partial result in the workspace, unless this launch is the one that joins the parts)
    const bool join = RUNS && p.merge_parts > 0;
    const bool partial = RUNS && !join;
    const int hz_out = partial ? hz + ksp * p.heads_total : hz;
    float* const lse_out = partial ? p.part_lse : p.lse;
    void* const o_out = partial ? static_cast<void*>(p.part_o) : p.o;
    const bool out_f32 = partial || p.out_f32;
    auto finish = [&](auto& vals, int col0, unsigned char* stage, bool write_lse) {
        constexpr int kTilesHere = (int)(sizeof(vals) / sizeof(vals[0]));
        const float l_tot = sum_quarters(l_i);
        float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
        if (KV8 && p.v_scale) inv *= p.v_scale[hz];   // O was accumulated on the stored V values
        float lse_val = l_tot > 0.f ? m_i + log2f(l_tot) : -INFINITY;
        // the row number is derived again from an opaque copy: kept from the start-up it
        // would occupy a register pair through the whole kernel
        int rib = row_in_block;
        asm volatile("" : "+v"(rib));
        const int row = row_base + rib;
        if constexpr (RUNS) {
            if (join) {
                // Join with the partial results of the prefix runs (normalised float32 rows with their base-2
                // log-sum-exps, written by the launch before this one): weights 2^(lse - max), the own part scaled
                // in place, the others added from memory (this lane's 4 head dims of each of its tiles).
                const size_t part_rows = (size_t)p.heads_total * p.nq;
                const size_t mine = (size_t)hz * p.nq + min(row, p.nq - 1);     // (rows past the end: read a real row, store nothing)
                float mx = lse_val;
                for (int pp = 1; pp <= p.merge_parts; ++pp) mx = fmaxf(mx, p.part_lse[pp * part_rows + mine]);
                const float mx_safe = mx == -INFINITY ? 0.f : mx;
                float wsum = __builtin_amdgcn_exp2f(lse_val - mx_safe);      // exp2(-inf) = 0
                const float own = wsum * inv;
#pragma unroll
                for (int i = 0; i < kTilesHere; ++i)
#pragma unroll
                    for (int r = 0; r < 4; ++r) vals[i][r] *= own;
                for (int pp = 1; pp <= p.merge_parts; ++pp) {
                    const float w = __builtin_amdgcn_exp2f(p.part_lse[pp * part_rows + mine] - mx_safe);
                    wsum += w;
                    const float* src = p.part_o + (pp * part_rows + mine) * D + col0 + 4 * g;
#pragma unroll
                    for (int i = 0; i < kTilesHere; ++i) {
                        const f32x4 x = *reinterpret_cast<const f32x4*>(src + 16 * i);
#pragma unroll
                        for (int r = 0; r < 4; ++r) vals[i][r] = __builtin_fmaf(w, x[r], vals[i][r]);
                    }
                }
                inv = wsum > 0.f ? 1.f / wsum : 0.f;
                lse_val = wsum > 0.f ? mx + log2f(wsum) : -INFINITY;
            }
        }
        if (write_lse && row < p.nq && lse_out && g == 0) lse_out[(size_t)hz_out * p.nq + row] = lse_val;
        const int rows_valid = p.nq - first_row;
        if (out_f32) {
            constexpr int kPass = kTilesHere < D / 32 ? kTilesHere : D / 32;   // tiles per pass
            float* ob = static_cast<float*>(o_out) + ((size_t)hz_out * p.nq + first_row) * D + col0;
#pragma unroll
            for (int h = 0; h < kTilesHere / kPass; ++h) {
#pragma unroll
                for (int i = 0; i < kPass; ++i) {
                    const f32x4& acc = vals[h * kPass + i];
                    const f32x4 val = {acc[0] * inv, acc[1] * inv, acc[2] * inv, acc[3] * inv};
                    *reinterpret_cast<f32x4*>(stage + ql * kStageStride + (16 * i + 4 * g) * 4) = val;
                }
                __builtin_amdgcn_wave_barrier();
                flush_rows<kPass * 64>(stage, kStageStride, reinterpret_cast<unsigned char*>(ob + h * kPass * 16),
                                       (size_t)D * 4, lane, rows_valid);
                __builtin_amdgcn_wave_barrier();
            }
        } else {
            T* ob = static_cast<T*>(o_out) + ((size_t)hz_out * p.nq + first_row) * D + col0;
#pragma unroll
            for (int i = 0; i < kTilesHere; ++i) {
                // accumulator rows 4g .. 4g+3 of a tile are 4 consecutive head dims
                const f32x4& acc = vals[i];
                const u32x2 packed = {MM::pack(acc[0] * inv, acc[1] * inv), MM::pack(acc[2] * inv, acc[3] * inv)};
                *reinterpret_cast<u32x2*>(stage + ql * kStageStride + (16 * i + 4 * g) * 2) = packed;
            }
            __builtin_amdgcn_wave_barrier();
            flush_rows<kTilesHere * 32>(stage, kStageStride, reinterpret_cast<unsigned char*>(ob), (size_t)D * 2, lane,
                                        rows_valid);
        }
    };
    if constexpr (kDShare) {
        __syncthreads();   // every wave is done with the last tile
        FSTA_STAMP(15);   // (head-dimension pairing) barrier in front of the epilogue passed
        finish(o, split * (D / 2), smem + (size_t)wave * 16 * kStageStride, split == 0);
    } else if constexpr (kSplit == 1) {
        __syncthreads();   // every wave is done with the last tile
        finish(o, 0, smem + (size_t)qgroup * 16 * kStageStride, true);
    } else {
        // Two waves share each group of query rows: they swap halves of the head dimension
        // through LDS (same lanes, same layout), and each merges, normalises and stores its half.
        constexpr int kH = kDTiles / 2;
        constexpr int kXchFloats = (2 + 4 * kH) * 64;
        __syncthreads();   // the ring is free: every tile has been consumed
        float* give = reinterpret_cast<float*>(smem) + (size_t)(qgroup * 2 + split) * kXchFloats;
        const float* take = reinterpret_cast<float*>(smem) + (size_t)(qgroup * 2 + (1 - split)) * kXchFloats;
        give[lane] = m_i;
        give[64 + lane] = l_i;
        f32x4 keep[kH];
        if (split == 0) {
#pragma unroll
            for (int i = 0; i < kH; ++i) {
                keep[i] = o[i];
#pragma unroll
                for (int r = 0; r < 4; ++r) give[(2 + 4 * i + r) * 64 + lane] = o[kH + i][r];
            }
        } else {
#pragma unroll
            for (int i = 0; i < kH; ++i) {
                keep[i] = o[kH + i];
#pragma unroll
                for (int r = 0; r < 4; ++r) give[(2 + 4 * i + r) * 64 + lane] = o[i][r];
            }
        }
        __syncthreads();
        const float m_b = take[lane], l_b = take[64 + lane];
        const float m_new = fmaxf(m_i, m_b);
        const float m_safe = m_new == -INFINITY ? 0.f : m_new;
        const float a_own = __builtin_amdgcn_exp2f(m_i - m_safe);
        const float a_oth = __builtin_amdgcn_exp2f(m_b - m_safe);
        l_i = l_i * a_own + l_b * a_oth;
        m_i = m_new;
#pragma unroll
        for (int i = 0; i < kH; ++i)
#pragma unroll
            for (int r = 0; r < 4; ++r) keep[i][r] = keep[i][r] * a_own + take[(2 + 4 * i + r) * 64 + lane] * a_oth;
        unsigned char* stage = smem + (size_t)kQGroups * 2 * kXchFloats * 4 + (size_t)wave * 16 * kStageStride;
        finish(keep, split * (D / 2), stage, split == 0);
    }
#ifdef FSTA_TIMELINE
    FSTA_STAMP(13);   // stores issued
    wait_vmcnt<0>();
    FSTA_STAMP(14);   // stores retired
    if (g_timeline && lane < kStamps + 2) {
        const uint64_t wg = (uint64_t)blockIdx.x + (uint64_t)gridDim.x * (blockIdx.y + (uint64_t)gridDim.y * blockIdx.z);
        uint64_t* out = g_timeline + (wg * kWaves + wave) * (kStamps + 2);
        out[lane] = lane < kStamps ? tl_s[wave][lane] : lane == kStamps ? tl_begin : __builtin_amdgcn_s_memrealtime();
    }
#endif
}

template <bool BF16, int D, int M, bool SPLIT, int KS>
int launch_ks(const AttnParams& p, int sub_shift, hipStream_t stream) {
    // ring depth: everything in flight at once for short tile lists, else the limit
    const int tiles = M / 32 + anc_tile_capacity(p.max_anc) + (p.prefix + kTileN - 1) / kTileN;
    int stages = tiles < 2 ? 2 : (tiles > kMaxStages ? kMaxStages : tiles);
    size_t lds = mfma16_lds_bytes<D, M>(p.max_anc, stages);
    while (lds > 160 * 1024 && stages > 2) lds = mfma16_lds_bytes<D, M>(p.max_anc, --stages);
    // the kernel's start-up parks Q in the last ring slots and requests up to two leaf tiles
    // into the first ones; ancestor lists too long to leave that much LDS go to the other kernel
    constexpr int kShares = KS < 0 ? -KS : KS;
    constexpr int kWaves = M / 16 * kShares, kQSlots = (kWaves * 16 + 2 * kTileN - 1) / (2 * kTileN);
    if (stages < kQSlots + (M / 32 < 2 ? M / 32 : 2)) {
        if (p.part_o) return FSTA_EUNSUPPORTED;   // the caller falls back to a launch without key splits
        return launch_attention_mfma(p, BF16 ? FSTA_BF16 : FSTA_F16, D, BF16 && !SPLIT, stream);
    }
    // the epilogue reuses the front of the segment: exchange area of a key split, row staging
    constexpr size_t kEpilogueBytes = KS > 1 ? (size_t)(M / 16) * 2 * ((2 + D / 8) * 256 + 16 * (D * 2 + 16))
                                             : (size_t)kWaves * 16 * (D * 2 + 16);
    if (lds < kEpilogueBytes) lds = kEpilogueBytes;
    if (lds > 160 * 1024)
        return fail(FSTA_EUNSUPPORTED, "max_ancestors=%d needs %zu bytes of LDS (limit 163840)", p.max_anc, lds);
    const int slices_per_xcd = (p.heads_total + kXcds - 1) / kXcds;
    const unsigned grid = (unsigned)(kXcds * slices_per_xcd * (p.nb << sub_shift) * p.key_splits);   // workgroups
    // (8 XCDs x key runs, blocks, slices per XCD) where the y and z extents allow it, else one axis
    const bool linear_grid = (p.nb << sub_shift) > 65535 || slices_per_xcd > 65535;
    // More than one and at most two workgroups per CU: late blocks first (see the kernel's mapping).
    const bool late_first = !linear_grid && !p.part_o && p.key_splits == 1 && grid > (unsigned)kCus && grid <= 2u * kCus;
    const dim3 grid3 = linear_grid  ? dim3(grid)
                       : late_first ? dim3((unsigned)kXcds, (unsigned)slices_per_xcd, (unsigned)(p.nb << sub_shift))
                                    : dim3((unsigned)(kXcds * p.key_splits), (unsigned)(p.nb << sub_shift), (unsigned)slices_per_xcd);
    const int shift_arg = sub_shift | (linear_grid ? 0x100 : 0) | (late_first ? 0x200 : 0);
    // a launch whose workgroups all run at once: leaf tiles requested early, Q in an area of its own
    constexpr size_t kQBytes = (size_t)kWaves * 16 * D * 2;
    const int early = grid <= kCus && !p.part_o && lds + kQBytes <= 160 * 1024 ? 1 : 0;
    if (early) lds += kQBytes;
    if (p.dry_run) return p.part_o && KS < 0 ? FSTA_EUNSUPPORTED : FSTA_OK;
    if (p.part_o) {
        if constexpr (KS > 0) {
            if (lds > 64 * 1024) {
                const int rc = allow_full_lds<&attn_mfma16_kernel<BF16, D, M, SPLIT, KS, true>>();
                if (rc != FSTA_OK) return rc;
            }
            hipLaunchKernelGGL((attn_mfma16_kernel<BF16, D, M, SPLIT, KS, true>), grid3, dim3(M * 4 * kShares),
                               lds, stream, p, stages, early, shift_arg);
        } else {
            return FSTA_EUNSUPPORTED;   // (key runs are never combined with head-dimension shares)
        }
    } else {
        if (lds > 64 * 1024) {
            const int rc = allow_full_lds<&attn_mfma16_kernel<BF16, D, M, SPLIT, KS, false>>();
            if (rc != FSTA_OK) return rc;
        }
        hipLaunchKernelGGL((attn_mfma16_kernel<BF16, D, M, SPLIT, KS, false>), grid3, dim3(M * 4 * kShares), lds,
                           stream, p, stages, early, shift_arg);
    }
    FSTA_HIP_OK(hipGetLastError());
    note_launch({"attn_mfma16_kernel", BF16 ? "true" : "false", {D, M, SPLIT ? 1 : 0, KS, p.part_o ? 1 : 0, 0}, 6,
                 0x34u, sub_shift, early});
    return FSTA_OK;
}

template <bool BF16, int D, int M, bool SPLIT>
int launch_one(const AttnParams& p, int sub_shift, hipStream_t stream) {
    // Key splitting pays when a wave would otherwise walk several ancestor / prefix tiles on
    // its own and the block is small (few waves); blocks of 128 rows fill the workgroup anyway.
    const int work_tiles = anc_tile_capacity(p.max_anc) + (p.prefix + kTileN - 1) / kTileN;
    if constexpr (M < 128) {
        if constexpr (D >= 64) {
            // Up to four ancestor tiles, no prefix, and a launch whose workgroups all run at once (its
            // time is the length of one workgroup's chain): the two waves of a row group share the
            // head dimension, with no exchange at the end, instead of the tiles.  With several rounds
            // of workgroups the duplicated work costs more than the shorter chain gains (cfg4: +50 %),
            // and so it does with longer lists (8 tiles: +10 %).
            const int slices_per_xcd = (p.heads_total + kXcds - 1) / kXcds;
            const bool one_round = kXcds * slices_per_xcd * (p.nb << sub_shift) <= kCus;
            if (one_round && work_tiles <= 4 && p.prefix == 0 && !p.part_o && !p.share_tiles)
                return launch_ks<BF16, D, M, SPLIT, -2>(p, sub_shift, stream);
        }
        if (work_tiles >= 2) return launch_ks<BF16, D, M, SPLIT, 2>(p, sub_shift, stream);
    }
    return launch_ks<BF16, D, M, SPLIT, 1>(p, sub_shift, stream);
}

template <bool BF16, int D, bool SPLIT>
int launch_m(const AttnParams& p, hipStream_t stream) {
    // Launches that would leave half of the CUs without a workgroup are cut into half-blocks.
    const int slices_per_xcd = (p.heads_total + kXcds - 1) / kXcds;
    // (also the launch that joins the partial results of a dense prefix: twice the CUs share the reading)
    const bool halve = (!p.part_o || p.merge_parts > 0) && kXcds * slices_per_xcd * p.nb * 2 <= kCus;
    switch (p.block_m) {
        case 32: return launch_one<BF16, D, 32, SPLIT>(p, 0, stream);
        case 64: return halve ? launch_one<BF16, D, 32, SPLIT>(p, 1, stream) : launch_one<BF16, D, 64, SPLIT>(p, 0, stream);
        case 128: return halve ? launch_one<BF16, D, 64, SPLIT>(p, 1, stream) : launch_one<BF16, D, 128, SPLIT>(p, 0, stream);
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

// 8-bit K/V: one wave per group of 16 rows, whole blocks, no key runs.
template <bool BF16, int D, int M>
int launch_kv8(const AttnParams& p, hipStream_t stream) {
    constexpr bool kSplitP = BF16;
    const int tiles = M / 32 + anc_tile_capacity(p.max_anc) + (p.prefix + kTileN - 1) / kTileN;
    int stages = tiles < 2 ? 2 : (tiles > kMaxStages ? kMaxStages : tiles);
    const size_t plan_bytes = (size_t)plan_layout(M, p.max_anc).block_words * 4;
    auto lds_for = [&](int st) { return (size_t)2 * 2 * kTileN * D * 2 + (size_t)st * 2 * kTileN * D + plan_bytes; };
    size_t lds = lds_for(stages);
    while (lds > 160 * 1024 && stages > 2) lds = lds_for(--stages);
    constexpr size_t kEpilogueBytes = (size_t)(M / 16) * 16 * (D * 2 + 16);
    if (lds < kEpilogueBytes) lds = kEpilogueBytes;
    if (lds > 160 * 1024)
        return fail(FSTA_EUNSUPPORTED, "8-bit K/V: max_ancestors=%d needs %zu bytes of LDS (limit 163840)", p.max_anc, lds);
    const int slices_per_xcd = (p.heads_total + kXcds - 1) / kXcds;
    const unsigned grid = (unsigned)(kXcds * slices_per_xcd * p.nb);
    const bool linear_grid = p.nb > 65535 || slices_per_xcd > 65535;
    const dim3 grid3 = linear_grid ? dim3(grid) : dim3((unsigned)kXcds, (unsigned)p.nb, (unsigned)slices_per_xcd);
    if (lds > 64 * 1024) {
        const int rc = allow_full_lds<&attn_mfma16_kernel<BF16, D, M, kSplitP, 1, false, true>>();
        if (rc != FSTA_OK) return rc;
    }
    hipLaunchKernelGGL((attn_mfma16_kernel<BF16, D, M, kSplitP, 1, false, true>), grid3, dim3(M * 4), lds, stream, p,
                       stages, 0, linear_grid ? 0x100 : 0);
    FSTA_HIP_OK(hipGetLastError());
    note_launch({"attn_mfma16_kernel", BF16 ? "true" : "false", {D, M, kSplitP ? 1 : 0, 1, 0, 1}, 6, 0x34u, 0, 0});
    return FSTA_OK;
}

template <bool BF16, int D>
int launch_kv8_m(const AttnParams& p, hipStream_t stream) {
    switch (p.block_m) {
        case 32: return launch_kv8<BF16, D, 32>(p, stream);
        case 64: return launch_kv8<BF16, D, 64>(p, stream);
        case 128: return launch_kv8<BF16, D, 128>(p, stream);
    }
    return fail(FSTA_EUNSUPPORTED, "8-bit K/V: block_m=%d (supported: 32, 64, 128)", p.block_m);
}

}  // namespace

int launch_attention_mfma16_kv8(const AttnParams& p, int dtype, int head_dim, hipStream_t stream) {
    if ((uint64_t)p.nk * (uint64_t)head_dim > 0xffffffffull || !p.plan)
        return fail(FSTA_EUNSUPPORTED, "8-bit K/V needs a block plan and slices below 4 GiB");
    const bool bf16 = dtype == FSTA_BF16;
    if (dtype != FSTA_BF16 && dtype != FSTA_F16) return fail(FSTA_EUNSUPPORTED, "8-bit K/V: q must be float16 or bfloat16");
    switch (head_dim) {
        case 64: return bf16 ? launch_kv8_m<true, 64>(p, stream) : launch_kv8_m<false, 64>(p, stream);
        case 128: return bf16 ? launch_kv8_m<true, 128>(p, stream) : launch_kv8_m<false, 128>(p, stream);
    }
    return fail(FSTA_EUNSUPPORTED, "8-bit K/V: head_dim=%d (supported: 64, 128)", head_dim);
}

int launch_attention_mfma16(const AttnParams& p, int dtype, int head_dim, bool fast_pv, hipStream_t stream) {
    // the gathers address a (batch, head) slice of K or V with 32-bit byte offsets
    if ((uint64_t)p.nk * (uint64_t)head_dim * 2u > 0xffffffffull || !p.plan) return FSTA_EUNSUPPORTED;
    if (dtype == FSTA_F16) return launch_d<false, false>(p, head_dim, stream);
    if (fast_pv) return launch_d<true, false>(p, head_dim, stream);
    return launch_d<true, true>(p, head_dim, stream);
}

}  // namespace fsta

#ifdef FSTA_TIMELINE
// Instrumented build only: device buffer of (workgroups x waves x 18) uint64 that every launch of
// the kernel above fills (16 stamps of the 100 MHz clock, then the full clock at entry and exit), or NULL.
extern "C" int fsta_timeline_buffer(uint64_t* device_buffer) {
    FSTA_HIP_OK(hipMemcpyToSymbol(HIP_SYMBOL(fsta::g_timeline), &device_buffer, sizeof(device_buffer)));
    return FSTA_OK;
}
#endif
