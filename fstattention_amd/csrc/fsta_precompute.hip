// Integer kernels of the tree precompute: per-block unique ancestors, leaves and
// ancestor mask (bit-exact with reference utils.py:104-129), mask packing, and
// parent[] -> lineage.  All of it is bit/byte work bound by memory latency; one
// workgroup owns one query block and keeps the block's ancestor set as a bitmap
// over node ids in LDS.
#include "fsta_common.h"

namespace fsta {
namespace {

constexpr int kThreads = 256;

constexpr int kMaxThreads = 1024;   // block_precompute_kernel runs with 256 or 1024 threads
constexpr int kBatch = 8;           // independent loads a thread has in flight

// Dynamic LDS of block_precompute_kernel (32-bit words):
//   bitmap[W] | rank_base[W] | mbits[mask_words * M] | lvl[M] | misc[4] | vals[staged]
// vals: the block's lineage rows as int32 (when they fit), so that the second pass over them
// reads LDS instead of going to memory again.
__host__ __device__ inline size_t precompute_lds_words(int64_t n_words, int mask_words, int block_m) {
    return (size_t)(2 * n_words) + (size_t)mask_words * block_m + block_m + 4;
}

__global__ __launch_bounds__(kMaxThreads) void block_precompute_kernel(
    int64_t* __restrict__ lineage, const int64_t* __restrict__ level_lookup,
    int64_t n_nodes, int64_t width, int block_m, int max_anc, int mask_words, int mutate, int staged,
    int64_t* __restrict__ ancestor_idx, uint8_t* __restrict__ ancestor_mask,
    int64_t* __restrict__ leaf_idx, uint32_t* __restrict__ mask_bits,
    int32_t* __restrict__ anc_count, uint32_t* __restrict__ plan, const int64_t* __restrict__ parent,
    uint32_t* __restrict__ status) {
    // `parent` != NULL (fsta_precompute_from_parents): the block's lineage rows are not read but built here, from the
    // parent array (copied into LDS as int32 behind the staged rows); `lineage` and `level_lookup` are then outputs
    // (each may be NULL) and `staged` is 1.
    extern __shared__ uint32_t lds[];
    const int n_words = (int)((n_nodes + 31) >> 5);
    uint32_t* bitmap = lds;                                   // ancestor set of this block
    uint32_t* rank_base = bitmap + n_words;                   // set bits in lower words
    uint32_t* mbits = rank_base + n_words;                    // [mask_words][block_m]
    int32_t* lvl_s = reinterpret_cast<int32_t*>(mbits + (size_t)mask_words * block_m);  // [block_m]
    uint32_t* misc = reinterpret_cast<uint32_t*>(lvl_s + block_m);   // [0] a -1 was seen, [2] total count, [3] a listed ancestor
    int32_t* vals_s = reinterpret_cast<int32_t*>(misc + 4);          // [rows * width] when staged

    const int tid = threadIdx.x;
    const int threads = blockDim.x;
    const int j = blockIdx.x;
    const int64_t lo = (int64_t)j * block_m;
    const int rows = (int)min((int64_t)block_m, n_nodes - lo);

    // The first kBatch lineage entries of every thread are requested before anything else; they
    // are on their way while the LDS tables are cleared.
    const int64_t* chunk = lineage + lo * width;
    const uint32_t n_elem = (uint32_t)rows * (uint32_t)width;   // the host checked that this fits
    auto load_batch = [&](uint32_t e0, int64_t (&val)[kBatch]) {
#pragma unroll
        for (int b = 0; b < kBatch; ++b) {
            const uint32_t e = e0 + (uint32_t)b * threads;
            val[b] = e < n_elem ? chunk[e] : 0;
        }
    };
    int64_t first[kBatch];
    if (!parent) load_batch(tid, first);
    int32_t* par_s = vals_s + (size_t)block_m * width;      // [n_nodes], from-parents mode only
    uint32_t err = 0u;
    if (parent) {
        for (int64_t i = tid; i < n_nodes; i += threads) {
            const int64_t pp = parent[i];
            const bool ok = pp >= -1 && pp < i;
            if (!ok) err |= FSTA_PRE_BAD_NODE_ID;
            par_s[i] = ok ? (int32_t)pp : -1;
        }
    }

    for (int w = tid; w < n_words; w += threads) bitmap[w] = 0u;
    for (int e = tid; e < mask_words * block_m; e += threads) mbits[e] = 0u;
    if (tid < 4) misc[tid] = 0u;
    if (parent) {
        __syncthreads();
        // One lane per row walks to the root once and notes the ancestors in hop order (every hop goes to a smaller
        // id, so the walk ends), then turns its row around into level order, -1 padded (layout of utils.py:66-75:
        // column l = the ancestor at level l; the node's own column holds -1 until the self entry goes in).
        for (int r = tid; r < block_m; r += threads) {
            int32_t lv = -1;
            if (r < rows) {
                int32_t* row = vals_s + (size_t)r * width;
                int32_t depth = 0;
                for (int32_t a = par_s[lo + r]; a >= 0; a = par_s[a]) {
                    if (depth < width) row[depth] = a;
                    ++depth;
                }
                if (depth >= width) {          // deeper than the rows are wide: flagged, the row counts as empty
                    err |= FSTA_PRE_BAD_LEVEL;
                    depth = 0;
                } else {
                    lv = depth;
                }
                for (int32_t a = 0, b = depth - 1; a < b; ++a, --b) {
                    const int32_t x = row[a];
                    row[a] = row[b];
                    row[b] = x;
                }
                for (int32_t l = depth; l < width; ++l) row[l] = -1;
                if (level_lookup) const_cast<int64_t*>(level_lookup)[lo + r] = lv >= 0 ? lv : 0;
            }
            lvl_s[r] = lv;
        }
    }
    for (int r = tid; r < block_m && !parent; r += threads) {
        int32_t lv = -1;  // -1 = nothing to insert (pad row or invalid level)
        if (r < rows) {
            int64_t l = level_lookup[lo + r];
            if (l < 0) l += width;  // negative levels index from the end, as a Python index does
            if (l < 0 || l >= width) err |= FSTA_PRE_BAD_LEVEL;
            else lv = (int32_t)l;
        }
        lvl_s[r] = lv;
    }
    __syncthreads();

    // 1. set a bit for every value of the block's lineage rows (utils.py:118-119); kBatch loads
    //    per thread go out before the first one is used
    bool saw_pad = false;
    auto take_batch = [&](uint32_t e0, const int64_t (&val)[kBatch]) {
#pragma unroll
        for (int b = 0; b < kBatch; ++b) {
            const uint32_t e = e0 + (uint32_t)b * threads;
            if (e >= n_elem) break;
            int32_t keep = -1;
            if (val[b] == -1) saw_pad = true;
            else if (val[b] < -1 || val[b] >= n_nodes) err |= FSTA_PRE_BAD_NODE_ID;
            else {
                // rows of one block share most of their ancestors: only a bit that is not there
                // yet goes through the (serialising) atomic
                keep = (int32_t)val[b];
                const uint32_t bit = 1u << (keep & 31);
                if (!(bitmap[keep >> 5] & bit)) atomicOr(&bitmap[keep >> 5], bit);
            }
            if (staged) vals_s[e] = keep;
        }
    };
    if (parent) {
        __syncthreads();      // the rows are complete
        for (uint32_t e = tid; e < n_elem; e += threads) {
            const int32_t v = vals_s[e];
            if (v < 0) saw_pad = true;
            else {
                const uint32_t bit = 1u << (v & 31);
                if (!(bitmap[v >> 5] & bit)) atomicOr(&bitmap[v >> 5], bit);
            }
            if (lineage) {      // the rows as the lineage tensor (with the self entries when asked for)
                const uint32_t r = e / (uint32_t)width, l = e - r * (uint32_t)width;
                lineage[lo * width + e] = (mutate && (int32_t)l == lvl_s[r]) ? lo + r : (int64_t)v;
            }
        }
    } else {
    take_batch(tid, first);
    for (uint32_t e0 = tid + (uint32_t)threads * kBatch; e0 < n_elem; e0 += (uint32_t)threads * kBatch) {
        int64_t val[kBatch];
        load_batch(e0, val);
        take_batch(e0, val);
    }
    }
    if (saw_pad) misc[0] = 1u;
    __syncthreads();

    // 2. exclusive prefix sum of the per-word popcounts -> rank of every ancestor; the first
    //    wave scans, each lane a run of consecutive words
    if (tid < 64) {
        // The reference drops the smallest unique value unconditionally (utils.py:119, the
        // `[1:]`); that is the -1 padding whenever one is present.  Without any -1 in the block
        // the smallest node id goes instead.  (Same wave as the scan: its LDS accesses stay in order.)
        if (tid == 0 && misc[0] == 0u) {
            for (int w = 0; w < n_words; ++w) {
                if (bitmap[w]) { bitmap[w] &= bitmap[w] - 1u; break; }
            }
        }
        __builtin_amdgcn_wave_barrier();
        const int per_lane = (n_words + 63) / 64;
        const int w_begin = min(tid * per_lane, n_words);
        const int w_end = min(w_begin + per_lane, n_words);
        uint32_t local = 0u;
        for (int w = w_begin; w < w_end; ++w) local += __popc(bitmap[w]);
        uint32_t incl = local;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const uint32_t up = __shfl_up(incl, d, 64);
            if (tid >= d) incl += up;
        }
        uint32_t run = incl - local;
        for (int w = w_begin; w < w_end; ++w) { rank_base[w] = run; run += __popc(bitmap[w]); }
        if (tid == 63) misc[2] = incl;
    }
    __syncthreads();
    const uint32_t total = misc[2];
    if (total > (uint32_t)max_anc) err |= FSTA_PRE_TOO_MANY_ANCESTORS;
    const int kept = (int)min(total, (uint32_t)max_anc);

    // 3. ancestor_idx: ascending ids, left aligned, -1 padded (utils.py:112,120); the block plan
    //    receives the same ids as 32-bit keys
    const PlanLayout layout = plan_layout(block_m, max_anc);
    uint32_t* rec = plan ? plan + (size_t)j * layout.block_words : nullptr;
    const uint32_t last_tile_first = kept > 0 ? (uint32_t)((kept - 1) & ~31) : 0xffffffffu;   // first slot of the last tile in use
    for (int c = kept + tid; c < max_anc; c += threads) ancestor_idx[(size_t)j * max_anc + c] = -1;
    for (int w = tid; w < n_words; w += threads) {
        uint32_t bits = bitmap[w];
        uint32_t r = rank_base[w];
        while (bits) {
            const int b = __ffs(bits) - 1;
            bits &= bits - 1u;
            if (r < (uint32_t)max_anc) {
                ancestor_idx[(size_t)j * max_anc + r] = (int64_t)w * 32 + b;
                if (rec) rec[kPlanHeaderWords + r] = (uint32_t)(w * 32 + b);
                if (r == last_tile_first) misc[3] = (uint32_t)(w * 32 + b);
            }
            ++r;
        }
    }
    if (anc_count && tid == 0) anc_count[j] = kept;

    // 4. leaves: ids of the block's range that are not in the set; the range is
    //    not clipped to n_nodes (utils.py:121-122)
    for (int r = tid; r < block_m; r += threads) {
        const int64_t id = lo + r;
        const bool is_anc = id < n_nodes && ((bitmap[id >> 5] >> (id & 31)) & 1u);
        leaf_idx[(size_t)j * block_m + r] = is_anc ? -1 : id;
    }

    // 5. mask: row r holds its lineage plus itself in its own level column
    //    (utils.py:124-127); membership of ancestor c in that row
    //    A thread walks a run of consecutive levels of one row.  Ancestors along a path have
    //    increasing ids, hence increasing ranks: the bits of a run fall into one or two mask words,
    //    which are collected in a register and merged with one atomic each.
    {
        const int segs_per_row = max(1, min((int)width, threads / max(rows, 1)));
        const int seg_len = ((int)width + segs_per_row - 1) / segs_per_row;
        for (int sidx = tid; sidx < rows * segs_per_row; sidx += threads) {
            const int r = sidx / segs_per_row;
            const int l0 = (sidx - r * segs_per_row) * seg_len;
            const int l1 = min(l0 + seg_len, (int)width);
            const int own = lvl_s[r];
            const uint32_t base = (uint32_t)r * (uint32_t)width;
            uint32_t cur = 0xffffffffu, acc = 0u;
            for (int l = l0; l < l1; ++l) {
                const int64_t val = l == own ? lo + r : (staged ? (int64_t)vals_s[base + l] : chunk[base + l]);
                if (val < 0 || val >= n_nodes) continue;
                const uint32_t word = bitmap[val >> 5];
                const uint32_t bit = 1u << (val & 31);
                if (!(word & bit)) continue;
                const uint32_t rank = rank_base[val >> 5] + __popc(word & (bit - 1u));
                if (rank >= (uint32_t)max_anc) continue;
                if ((rank >> 5) != cur) {
                    if (acc) atomicOr(&mbits[cur * block_m + r], acc);
                    cur = rank >> 5;
                    acc = 0u;
                }
                acc |= 1u << (rank & 31);
            }
            if (acc) atomicOr(&mbits[cur * block_m + r], acc);
        }
    }
    __syncthreads();

    if (mask_bits) {
        for (int e = tid; e < mask_words * block_m; e += threads)
            mask_bits[(size_t)j * mask_words * block_m + e] = mbits[e];
    }
    if (rec) {
        // Block plan: what the attention kernel would otherwise derive from the lists in every
        // workgroup.  An empty slot repeats a row its tile holds anyway (the first key of the last
        // ancestor tile in use, the first leaf of a group of 32 rows), so that every tile is
        // gathered with the same number of requests; its mask bits are zero by construction.
        const int tiles = layout.tiles, groups = block_m / 32;
        const uint32_t spare = kept > 0 ? misc[3] : (uint32_t)lo;
        for (int c = kept + tid; c < tiles * 32; c += threads) rec[kPlanHeaderWords + c] = spare;
        if (tid == 0) rec[0] = (uint32_t)kept;
        else if (tid < kPlanHeaderWords && (tid < kPlanLeafValid || tid - kPlanLeafValid >= groups)) rec[tid] = 0u;
        if (tid < block_m) {   // (block_m <= 128: the first two waves)
            const int64_t id = lo + tid;
            const bool is_anc = id < n_nodes && ((bitmap[id >> 5] >> (id & 31)) & 1u);
            const uint64_t vote = __ballot(!is_anc);
            const uint32_t mine = (tid & 32) ? (uint32_t)(vote >> 32) : (uint32_t)vote;   // this group of 32 rows
            const uint32_t first_leaf = mine ? (uint32_t)(lo + (tid & ~31) + __builtin_ctz(mine)) : (uint32_t)lo;
            uint32_t* grp = rec + layout.common_words + (tid >> 5) * layout.group_words;
            grp[tid & 31] = is_anc ? first_leaf : (uint32_t)id;
            if ((tid & 31) == 0) rec[kPlanLeafValid + (tid >> 5)] = mine;
        }
        for (int e = tid; e < groups * tiles * 32; e += threads) {
            const int g = e / (tiles * 32), rem = e - g * tiles * 32;   // rem = 32 * tile + row within the group
            rec[layout.common_words + g * layout.group_words + 32 + rem] = mbits[(rem >> 5) * block_m + g * 32 + (rem & 31)];
        }
    }
    if (ancestor_mask) {
        // one byte per (row, ancestor slot); 8 slots of a row per store where the layout allows
        uint8_t* out = ancestor_mask + (size_t)j * block_m * max_anc;
        if (max_anc % 8 == 0 && reinterpret_cast<uintptr_t>(out) % 8 == 0) {
            const int per_row = max_anc / 8;
            for (int e = tid; e < block_m * per_row; e += threads) {
                const int r = e / per_row, c = (e - r * per_row) * 8;
                const uint32_t bits = (mbits[(c >> 5) * block_m + r] >> (c & 31)) & 0xffu;
                // bit i -> byte i: three doubling steps spread the 8 bits over 64
                uint64_t x = bits;
                x = (x | (x << 28)) & 0x0000000f0000000full;
                x = (x | (x << 14)) & 0x0003000300030003ull;
                x = (x | (x << 7)) & 0x0101010101010101ull;
                reinterpret_cast<uint64_t*>(out)[e] = x;
            }
        } else {
            const int n_out = block_m * max_anc;
            for (int e = tid; e < n_out; e += threads) {
                const int r = e / max_anc, c = e - r * max_anc;
                out[e] = (uint8_t)((mbits[(c >> 5) * block_m + r] >> (c & 31)) & 1u);
            }
        }
    }

    // 6. the caller's lineage receives the self entries (utils.py:118,125)
    if (mutate && !parent) {
        for (int r = tid; r < rows; r += threads)
            if (lvl_s[r] >= 0) lineage[(lo + r) * width + lvl_s[r]] = lo + r;
    }
    if (err) atomicOr(status, err);
}

constexpr int kPackMaxTiles = 512;   // ancestor tiles a block plan written by pack_mask_kernel can have

__global__ __launch_bounds__(kThreads) void pack_mask_kernel(
    const int64_t* __restrict__ ancestor_idx, const uint8_t* __restrict__ ancestor_mask,
    const int64_t* __restrict__ leaf_idx, int block_m, int max_anc, int mask_words, int64_t key_limit,
    uint32_t* __restrict__ mask_bits, int32_t* __restrict__ anc_count, uint32_t* __restrict__ plan) {
    __shared__ int last_valid;
    __shared__ uint32_t tile_valid[kPackMaxTiles];   // plan only: slots of a tile whose id lies in [0, key_limit)
    const int tid = threadIdx.x;
    const int j = blockIdx.x;
    if (tid == 0) last_valid = -1;
    __syncthreads();
    const int64_t* idx = ancestor_idx + (size_t)j * max_anc;
    int mine = -1;
    for (int c = tid; c < max_anc; c += kThreads)
        if (idx[c] >= 0) mine = c;
    if (mine >= 0) atomicMax(&last_valid, mine);
    const PlanLayout layout = plan_layout(block_m, max_anc);
    uint32_t* rec = plan ? plan + (size_t)j * layout.block_words : nullptr;
    if (rec) {
        // keys of the ancestor slots, a half-wave per tile of 32: an empty or out-of-range slot
        // repeats the first valid key of its tile (row 0 if there is none)
        for (int c0 = 0; c0 < layout.tiles * 32; c0 += kThreads) {
            const int c = c0 + tid;
            if (c < layout.tiles * 32) {
                const int64_t id = c < max_anc ? idx[c] : -1;
                const bool ok = id >= 0 && id < key_limit;
                const uint64_t vote = __ballot(ok);
                const uint32_t half = (tid & 32) ? (uint32_t)(vote >> 32) : (uint32_t)vote;
                const uint32_t key = ok ? (uint32_t)id : 0u;
                const uint32_t first = __shfl(key, (tid & 32) + __builtin_ctz(half | 0x80000000u), 64);
                rec[kPlanHeaderWords + c] = ok ? key : first;
                if ((tid & 31) == 0) tile_valid[c >> 5] = half;
            }
        }
        if (tid < block_m) {   // leaf slots, a half-wave per group of 32 rows
            const int64_t id = leaf_idx[(size_t)j * block_m + tid];
            const bool ok = id >= 0 && id < key_limit;
            const uint64_t vote = __ballot(ok);
            const uint32_t half = (tid & 32) ? (uint32_t)(vote >> 32) : (uint32_t)vote;
            const uint32_t key = ok ? (uint32_t)id : 0u;
            const uint32_t first = __shfl(key, (tid & 32) + __builtin_ctz(half | 0x80000000u), 64);
            rec[layout.common_words + (tid >> 5) * layout.group_words + (tid & 31)] = ok ? key : first;
            if ((tid & 31) == 0) rec[kPlanLeafValid + (tid >> 5)] = half;
        }
        if (tid >= 1 && tid < kPlanHeaderWords && (tid < kPlanLeafValid || tid - kPlanLeafValid >= block_m / 32)) rec[tid] = 0u;
    }
    __syncthreads();
    const uint8_t* in = ancestor_mask + (size_t)j * block_m * max_anc;
    for (int e = tid; e < mask_words * block_m; e += kThreads) {
        const int w = e / block_m, r = e - w * block_m;
        uint32_t bits = 0u;
        const int c0 = w * 32;
        const int c1 = min(c0 + 32, max_anc);
        for (int c = c0; c < c1; ++c)
            if (in[(size_t)r * max_anc + c] && idx[c] >= 0) bits |= 1u << (c - c0);
        if (mask_bits) mask_bits[(size_t)j * mask_words * block_m + e] = bits;
        if (rec) rec[layout.common_words + (r >> 5) * layout.group_words + 32 + w * 32 + (r & 31)] = bits & tile_valid[w];
    }
    if (tid == 0) {
        if (anc_count) anc_count[j] = last_valid + 1;
        if (rec) rec[0] = (uint32_t)(last_valid + 1);
    }
}

// `lds_nodes` > 0: the workgroup first copies parent[0 .. lds_nodes) into LDS as int32 (the walks to
// the root are chains of dependent reads: an LDS access per hop instead of a trip to L2).
__global__ __launch_bounds__(kThreads) void lineage_from_parents_kernel(
    const int64_t* __restrict__ parent, int64_t n_nodes, int64_t width,
    int64_t* __restrict__ lineage, int64_t* __restrict__ level_lookup,
    uint32_t* __restrict__ status, int lds_nodes) {
    extern __shared__ int32_t par_s[];
    for (int x = threadIdx.x; x < lds_nodes; x += kThreads) {
        const int64_t v = parent[x];
        par_s[x] = (v >= -1 && v < x) ? (int32_t)v : -2;   // -2: malformed entry
    }
    const int64_t first = (int64_t)blockIdx.x * kThreads;
    const int64_t last = min(first + kThreads, n_nodes);
    if (lineage) {   // the rows of this workgroup's nodes are one contiguous piece: fill it with -1, coalesced
        int64_t* piece = lineage + first * width;
        for (int64_t e = threadIdx.x; e < (last - first) * width; e += kThreads) piece[e] = -1;
    }
    __syncthreads();
    const int64_t i = first + threadIdx.x;
    if (i >= n_nodes) return;
    auto up = [&](int64_t node) -> int64_t {   // parent of `node`, or -2 for an entry outside [-1, node)
        if (lds_nodes) return par_s[node];
        const int64_t v = parent[node];
        return (v >= -1 && v < node) ? v : -2;
    };
    uint32_t err = 0u;
    // pass 1: depth of node i; every hop goes to a smaller id, so the walk ends
    int64_t depth = 0;
    for (int64_t a = up(i); a != -1; a = up(a)) {
        if (a < -1) { err |= FSTA_PRE_BAD_NODE_ID; break; }
        ++depth;
    }
    level_lookup[i] = depth;
    if (lineage && !err) {
        if (depth >= width) {
            err |= FSTA_PRE_BAD_LEVEL;
        } else {
            // pass 2: the ancestor reached after s hops lives at level depth - s
            int64_t* row = lineage + i * width;
            int64_t a = up(i);
            for (int64_t l = depth - 1; l >= 0; --l) {
                row[l] = a;
                a = up(a);
            }
        }
    }
    if (err) atomicOr(status, err);
}

// The same result for trees whose parent array and a piece of the output fit into LDS: a
// workgroup owns `rows_per_wg` consecutive nodes.  One lane per node walks to the root ONCE,
// noting the ancestors in hop order in an LDS row; the depth is the hop count.  Then all lanes
// write the rows out, reversed into level order and padded with -1, as whole 512-byte pieces
// (the walk above stores 8 bytes per lane into 64 different rows per instruction).
__global__ __launch_bounds__(kThreads) void lineage_rows_kernel(
    const int64_t* __restrict__ parent, int n, int width, int rows_per_wg,
    int64_t* __restrict__ lineage, int64_t* __restrict__ level_lookup, uint32_t* __restrict__ status) {
    asm volatile("" ::"s"(parent), "s"(n), "s"(width), "s"(rows_per_wg), "s"(lineage), "s"(level_lookup), "s"(status));   // one batch of argument loads
    extern __shared__ int32_t rows_s[];
    int32_t* par_s = rows_s;                  // [n]
    int32_t* depth_s = par_s + n;             // [rows_per_wg], -1: the row stays empty
    int32_t* hops_s = depth_s + rows_per_wg;  // [rows_per_wg][width] ancestors, nearest first
    const int tid = threadIdx.x;
    for (int x = tid; x < n; x += kThreads) {
        const int64_t v = parent[x];
        par_s[x] = (v >= -1 && v < x) ? (int32_t)v : -2;   // -2: malformed entry
    }
    __syncthreads();
    const int first = blockIdx.x * rows_per_wg;
    const int rows = min(rows_per_wg, n - first);
    uint32_t err = 0u;
    for (int t = tid; t < rows; t += kThreads) {
        int32_t* mine = hops_s + (size_t)t * width;
        int hops = 0;
        int32_t a = par_s[first + t];
        for (; a >= 0; a = par_s[a]) {        // every hop goes to a smaller id, so the walk ends
            if (hops < width) mine[hops] = a;
            ++hops;
        }
        if (a < -1) err |= FSTA_PRE_BAD_NODE_ID;
        else if (hops >= width) err |= FSTA_PRE_BAD_LEVEL;
        level_lookup[first + t] = hops;
        depth_s[t] = (a < -1 || hops >= width) ? -1 : hops;
    }
    __syncthreads();
    int64_t* out = lineage + (size_t)first * width;
    const uint32_t n_out = (uint32_t)rows * (uint32_t)width;
    for (uint32_t e = tid; e < n_out; e += kThreads) {
        const uint32_t t = e / (uint32_t)width;
        const int l = (int)(e - t * (uint32_t)width);
        const int d = depth_s[t];
        out[e] = l < d ? (int64_t)hops_s[(size_t)t * width + (d - 1 - l)] : -1;
    }
    if (err) atomicOr(status, err);
}

}  // namespace
}  // namespace fsta

using namespace fsta;

extern "C" int32_t fsta_mask_words(int32_t max_ancestors) { return (max_ancestors + 31) / 32; }

extern "C" int fsta_precompute(int64_t* lineage, const int64_t* level_lookup, int64_t n_nodes,
                               int64_t width, int32_t block_m, int32_t max_ancestors,
                               int32_t mutate_lineage, int64_t* ancestor_idx,
                               uint8_t* ancestor_mask, int64_t* leaf_idx, uint32_t* mask_bits,
                               int32_t* anc_count, uint32_t* block_plan, uint32_t* status, void* stream) {
    if (n_nodes < 0 || width < 1 || block_m < 1 || max_ancestors < 1)
        return fail(FSTA_EINVAL, "fsta_precompute: n_nodes=%lld width=%lld block_m=%d max_ancestors=%d",
                    (long long)n_nodes, (long long)width, block_m, max_ancestors);
    if (n_nodes == 0) return FSTA_OK;
    if (!lineage || !level_lookup || !ancestor_idx || !leaf_idx || !status)
        return fail(FSTA_EINVAL, "fsta_precompute: null pointer");
    if (block_m > 4096) return fail(FSTA_EUNSUPPORTED, "fsta_precompute: block_m=%d > 4096", block_m);
    if (block_plan && !plan_block_size_ok(block_m))
        return fail(FSTA_EINVAL, "fsta_precompute: a block plan needs block_m 32, 64 or 128 (got %d)", block_m);
    if (block_plan && n_nodes + block_m > 0x7fffffff)
        return fail(FSTA_EUNSUPPORTED, "fsta_precompute: block plan keys are 32-bit (n_nodes=%lld)", (long long)n_nodes);
    if (misaligned(lineage, 8) || misaligned(level_lookup, 8) || misaligned(ancestor_idx, 8) || misaligned(leaf_idx, 8))
        return fail(FSTA_EINVAL, "fsta_precompute: lineage, level_lookup, ancestor_idx and leaf_idx must be 8-byte aligned");
    if (misaligned(mask_bits, 4) || misaligned(anc_count, 4) || misaligned(status, 4) || misaligned(block_plan, 16))
        return fail(FSTA_EINVAL, "fsta_precompute: mask_bits, anc_count and status must be 4-byte aligned, block_plan 16-byte");
    const int mask_words = fsta_mask_words(max_ancestors);
    const int64_t n_words = (n_nodes + 31) >> 5;
    if ((int64_t)block_m * width > 0x7fffffff)
        return fail(FSTA_EUNSUPPORTED, "fsta_precompute: block_m=%d x width=%lld entries per block", block_m,
                    (long long)width);
    size_t lds = sizeof(uint32_t) * precompute_lds_words(n_words, mask_words, block_m);
    if (lds > 160 * 1024)
        return fail(FSTA_EUNSUPPORTED,
                    "fsta_precompute: n_nodes=%lld block_m=%d max_ancestors=%d need %zu bytes of LDS (limit 163840)",
                    (long long)n_nodes, block_m, max_ancestors, lds);
    // the block's lineage rows stay in LDS between the two passes over them when they fit
    const size_t entries = (size_t)block_m * (size_t)width;
    const int staged = lds + entries * 4 <= 160 * 1024 ? 1 : 0;
    if (staged) lds += entries * 4;
    if (lds > 64 * 1024) {
        const int rc = allow_full_lds<&block_precompute_kernel>();
        if (rc != FSTA_OK) return rc;
    }
    const int64_t nb = (n_nodes + block_m - 1) / block_m;
    // a block with many entries is worked on by 16 waves, else by 4
    const int threads = entries >= 2048 || (size_t)block_m * max_ancestors >= 8192 ? kMaxThreads : kThreads;
    hipLaunchKernelGGL(block_precompute_kernel, dim3((unsigned)nb), dim3(threads), lds,
                       static_cast<hipStream_t>(stream), lineage, level_lookup, n_nodes, width,
                       block_m, max_ancestors, mask_words, mutate_lineage, staged, ancestor_idx,
                       ancestor_mask, leaf_idx, mask_bits, anc_count, block_plan, nullptr, status);
    FSTA_HIP_OK(hipGetLastError());
    return FSTA_OK;
}

extern "C" int fsta_precompute_from_parents(const int64_t* parent, int64_t n_nodes, int64_t width, int32_t block_m,
                                            int32_t max_ancestors, int32_t insert_self, int64_t* lineage,
                                            int64_t* level_lookup, int64_t* ancestor_idx, uint8_t* ancestor_mask,
                                            int64_t* leaf_idx, uint32_t* mask_bits, int32_t* anc_count,
                                            uint32_t* block_plan, uint32_t* status, void* stream) {
    if (n_nodes < 0 || width < 1 || block_m < 1 || max_ancestors < 1)
        return fail(FSTA_EINVAL, "fsta_precompute_from_parents: n_nodes=%lld width=%lld block_m=%d max_ancestors=%d",
                    (long long)n_nodes, (long long)width, block_m, max_ancestors);
    if (n_nodes == 0) return FSTA_OK;
    if (!parent || !ancestor_idx || !leaf_idx || !status) return fail(FSTA_EINVAL, "fsta_precompute_from_parents: null pointer");
    if (block_m > 4096) return fail(FSTA_EUNSUPPORTED, "fsta_precompute_from_parents: block_m=%d > 4096", block_m);
    if (block_plan && !plan_block_size_ok(block_m))
        return fail(FSTA_EINVAL, "fsta_precompute_from_parents: a block plan needs block_m 32, 64 or 128 (got %d)", block_m);
    if (misaligned(parent, 8) || misaligned(lineage, 8) || misaligned(level_lookup, 8) || misaligned(ancestor_idx, 8) ||
        misaligned(leaf_idx, 8))
        return fail(FSTA_EINVAL, "fsta_precompute_from_parents: parent, lineage, level_lookup, ancestor_idx and leaf_idx must be 8-byte aligned");
    if (misaligned(mask_bits, 4) || misaligned(anc_count, 4) || misaligned(status, 4) || misaligned(block_plan, 16))
        return fail(FSTA_EINVAL, "fsta_precompute_from_parents: mask_bits, anc_count and status must be 4-byte aligned, block_plan 16-byte");
    const int mask_words = fsta_mask_words(max_ancestors);
    const int64_t n_words = (n_nodes + 31) >> 5;
    // tables, the block's rows and the parent array, all in one workgroup's LDS
    const double need = 4.0 * ((double)precompute_lds_words(n_words, mask_words, block_m) + (double)block_m * (double)width + (double)n_nodes);
    if (need > 160.0 * 1024)
        return fail(FSTA_EUNSUPPORTED, "fsta_precompute_from_parents: n_nodes=%lld width=%lld block_m=%d max_ancestors=%d need %.0f "
                    "bytes of LDS (limit 163840): fsta_lineage_from_parents + fsta_precompute take any size",
                    (long long)n_nodes, (long long)width, block_m, max_ancestors, need);
    const size_t lds = (size_t)need;
    if (lds > 64 * 1024) {
        const int rc = allow_full_lds<&block_precompute_kernel>();
        if (rc != FSTA_OK) return rc;
    }
    const int64_t nb = (n_nodes + block_m - 1) / block_m;
    const size_t entries = (size_t)block_m * (size_t)width;
    const int threads = entries >= 2048 || (size_t)block_m * max_ancestors >= 8192 || n_nodes >= 2048 ? kMaxThreads : kThreads;
    hipLaunchKernelGGL(block_precompute_kernel, dim3((unsigned)nb), dim3(threads), lds, static_cast<hipStream_t>(stream), lineage,
                       level_lookup, n_nodes, width, block_m, max_ancestors, mask_words, insert_self ? 1 : 0, 1, ancestor_idx,
                       ancestor_mask, leaf_idx, mask_bits, anc_count, block_plan, parent, status);
    FSTA_HIP_OK(hipGetLastError());
    return FSTA_OK;
}

extern "C" size_t fsta_block_plan_bytes(int32_t num_blocks, int32_t block_m, int32_t max_ancestors) {
    if (num_blocks <= 0 || max_ancestors < 1 || !plan_block_size_ok(block_m)) return 0;
    return (size_t)num_blocks * (size_t)plan_layout(block_m, max_ancestors).block_words * sizeof(uint32_t);
}

extern "C" int fsta_pack_mask(const int64_t* ancestor_idx, const uint8_t* ancestor_mask, const int64_t* leaf_idx,
                              int32_t num_blocks, int32_t block_m, int32_t max_ancestors, int64_t key_limit,
                              uint32_t* mask_bits, int32_t* anc_count, uint32_t* block_plan, void* stream) {
    if (num_blocks < 0 || block_m < 1 || max_ancestors < 1)
        return fail(FSTA_EINVAL, "fsta_pack_mask: num_blocks=%d block_m=%d max_ancestors=%d",
                    num_blocks, block_m, max_ancestors);
    if (num_blocks == 0) return FSTA_OK;
    if (!ancestor_idx || !ancestor_mask || (!block_plan && (!mask_bits || !anc_count)))
        return fail(FSTA_EINVAL, "fsta_pack_mask: null pointer");
    if (block_plan) {
        if (!leaf_idx) return fail(FSTA_EINVAL, "fsta_pack_mask: a block plan needs leaf_idx");
        if (!plan_block_size_ok(block_m))
            return fail(FSTA_EINVAL, "fsta_pack_mask: a block plan needs block_m 32, 64 or 128 (got %d)", block_m);
        if (key_limit < 0 || key_limit > 0x7fffffff)
            return fail(FSTA_EINVAL, "fsta_pack_mask: key_limit=%lld outside [0, 2^31)", (long long)key_limit);
        if (fsta_mask_words(max_ancestors) > kPackMaxTiles)
            return fail(FSTA_EUNSUPPORTED, "fsta_pack_mask: block plan with max_ancestors=%d > %d", max_ancestors,
                        kPackMaxTiles * 32);
    }
    if (misaligned(ancestor_idx, 8) || misaligned(leaf_idx, 8))
        return fail(FSTA_EINVAL, "fsta_pack_mask: ancestor_idx and leaf_idx must be 8-byte aligned");
    if (misaligned(mask_bits, 4) || misaligned(anc_count, 4) || misaligned(block_plan, 16))
        return fail(FSTA_EINVAL, "fsta_pack_mask: mask_bits and anc_count must be 4-byte aligned, block_plan 16-byte");
    hipLaunchKernelGGL(pack_mask_kernel, dim3(num_blocks), dim3(kThreads), 0,
                       static_cast<hipStream_t>(stream), ancestor_idx, ancestor_mask, leaf_idx, block_m,
                       max_ancestors, fsta_mask_words(max_ancestors), key_limit, mask_bits, anc_count, block_plan);
    FSTA_HIP_OK(hipGetLastError());
    return FSTA_OK;
}

extern "C" int fsta_lineage_from_parents(const int64_t* parent, int64_t n_nodes, int64_t width,
                                         int64_t* lineage, int64_t* level_lookup, uint32_t* status,
                                         void* stream) {
    if (n_nodes < 0 || width < 1)
        return fail(FSTA_EINVAL, "fsta_lineage_from_parents: n_nodes=%lld width=%lld",
                    (long long)n_nodes, (long long)width);
    if (n_nodes == 0) return FSTA_OK;
    if (!parent || !level_lookup || !status)
        return fail(FSTA_EINVAL, "fsta_lineage_from_parents: null pointer");
    if (lineage && n_nodes <= 16384 && width <= 8192) {
        // rows of the output staged in LDS: as many nodes per workgroup as fit, in whole waves
        const size_t fixed = (size_t)n_nodes * 4;
        int rows_per_wg = (int)((160 * 1024 - fixed) / ((size_t)width * 4 + 4));
        rows_per_wg = rows_per_wg >= kThreads ? kThreads : rows_per_wg / 64 * 64;
        // small trees: still enough workgroups to spread the walks over the CUs
        while (rows_per_wg > 64 && (n_nodes + rows_per_wg - 1) / rows_per_wg < 16) rows_per_wg -= 64;
        if (rows_per_wg >= 64) {
            const size_t lds = fixed + (size_t)rows_per_wg * ((size_t)width * 4 + 4);
            if (lds > 64 * 1024) {
                const int rc = allow_full_lds<&lineage_rows_kernel>();
                if (rc != FSTA_OK) return rc;
            }
            const unsigned wgs = (unsigned)((n_nodes + rows_per_wg - 1) / rows_per_wg);
            hipLaunchKernelGGL(lineage_rows_kernel, dim3(wgs), dim3(kThreads), lds, static_cast<hipStream_t>(stream),
                               parent, (int)n_nodes, (int)width, rows_per_wg, lineage, level_lookup, status);
            FSTA_HIP_OK(hipGetLastError());
            return FSTA_OK;
        }
    }
    const unsigned grid = (unsigned)((n_nodes + kThreads - 1) / kThreads);
    const int lds_nodes = n_nodes <= 16384 ? (int)n_nodes : 0;   // 64 KB of int32
    hipLaunchKernelGGL(lineage_from_parents_kernel, dim3(grid), dim3(kThreads), (size_t)lds_nodes * 4,
                       static_cast<hipStream_t>(stream), parent, n_nodes, width, lineage,
                       level_lookup, status, lds_nodes);
    FSTA_HIP_OK(hipGetLastError());
    return FSTA_OK;
}
