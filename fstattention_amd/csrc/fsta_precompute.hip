// Integer kernels of the tree precompute: per-block unique ancestors, leaves and
// ancestor mask (bit-exact with reference utils.py:104-129), mask packing, and
// parent[] -> lineage.  All of it is bit/byte work bound by memory latency; one
// workgroup owns one query block and keeps the block's ancestor set as a bitmap
// over node ids in LDS.
#include "fsta_common.h"

namespace fsta {
namespace {

constexpr int kThreads = 256;

// Dynamic LDS of block_precompute_kernel:
//   bitmap[W] | rank_base[W] | mbits[mask_words * M] | lvl[M] | partial[kThreads] | misc[4]
__host__ __device__ inline size_t precompute_lds_words(int64_t n_words, int mask_words, int block_m) {
    return (size_t)(2 * n_words) + (size_t)mask_words * block_m + block_m + kThreads + 4;
}

__global__ __launch_bounds__(kThreads) void block_precompute_kernel(
    int64_t* __restrict__ lineage, const int64_t* __restrict__ level_lookup,
    int64_t n_nodes, int64_t width, int block_m, int max_anc, int mask_words, int mutate,
    int64_t* __restrict__ ancestor_idx, uint8_t* __restrict__ ancestor_mask,
    int64_t* __restrict__ leaf_idx, uint32_t* __restrict__ mask_bits,
    int32_t* __restrict__ anc_count, uint32_t* __restrict__ status) {
    extern __shared__ uint32_t lds[];
    const int n_words = (int)((n_nodes + 31) >> 5);
    uint32_t* bitmap = lds;                                   // ancestor set of this block
    uint32_t* rank_base = bitmap + n_words;                   // set bits in lower words
    uint32_t* mbits = rank_base + n_words;                    // [mask_words][block_m]
    int32_t* lvl_s = reinterpret_cast<int32_t*>(mbits + (size_t)mask_words * block_m);  // [block_m]
    uint32_t* partial = reinterpret_cast<uint32_t*>(lvl_s + block_m);                   // [kThreads]
    uint32_t* misc = partial + kThreads;  // [0] a -1 was seen, [1] error bits, [2] total count

    const int tid = threadIdx.x;
    const int j = blockIdx.x;
    const int64_t lo = (int64_t)j * block_m;
    const int rows = (int)min((int64_t)block_m, n_nodes - lo);

    for (int w = tid; w < n_words; w += kThreads) bitmap[w] = 0u;
    for (int e = tid; e < mask_words * block_m; e += kThreads) mbits[e] = 0u;
    if (tid < 4) misc[tid] = 0u;
    uint32_t err = 0u;
    for (int r = tid; r < block_m; r += kThreads) {
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

    // 1. set a bit for every value of the block's lineage rows (utils.py:118-119)
    const int64_t* chunk = lineage + lo * width;
    const int64_t n_elem = (int64_t)rows * width;
    bool saw_pad = false;
    for (int64_t e = tid; e < n_elem; e += kThreads) {
        const int64_t val = chunk[e];
        if (val == -1) saw_pad = true;
        else if (val < -1 || val >= n_nodes) err |= FSTA_PRE_BAD_NODE_ID;
        else atomicOr(&bitmap[val >> 5], 1u << (val & 31));
    }
    if (saw_pad) misc[0] = 1u;
    __syncthreads();

    // The reference drops the smallest unique value unconditionally (utils.py:119,
    // the `[1:]`); that is the -1 padding whenever one is present.  Without any
    // -1 in the block the smallest node id goes instead.
    if (tid == 0 && misc[0] == 0u) {
        for (int w = 0; w < n_words; ++w) {
            if (bitmap[w]) { bitmap[w] &= bitmap[w] - 1u; break; }
        }
    }
    __syncthreads();

    // 2. exclusive prefix sum of the per-word popcounts -> rank of every ancestor
    const int per_thread = (n_words + kThreads - 1) / kThreads;
    const int w_begin = min(tid * per_thread, n_words);
    const int w_end = min(w_begin + per_thread, n_words);
    uint32_t local = 0u;
    for (int w = w_begin; w < w_end; ++w) local += __popc(bitmap[w]);
    partial[tid] = local;
    __syncthreads();
    if (tid == 0) {
        uint32_t run = 0u;
        for (int t = 0; t < kThreads; ++t) { const uint32_t c = partial[t]; partial[t] = run; run += c; }
        misc[2] = run;
    }
    __syncthreads();
    {
        uint32_t run = partial[tid];
        for (int w = w_begin; w < w_end; ++w) { rank_base[w] = run; run += __popc(bitmap[w]); }
    }
    __syncthreads();
    const uint32_t total = misc[2];
    if (total > (uint32_t)max_anc) err |= FSTA_PRE_TOO_MANY_ANCESTORS;
    const int kept = (int)min(total, (uint32_t)max_anc);

    // 3. ancestor_idx: ascending ids, left aligned, -1 padded (utils.py:112,120)
    for (int c = kept + tid; c < max_anc; c += kThreads) ancestor_idx[(size_t)j * max_anc + c] = -1;
    for (int w = tid; w < n_words; w += kThreads) {
        uint32_t bits = bitmap[w];
        uint32_t r = rank_base[w];
        while (bits) {
            const int b = __ffs(bits) - 1;
            bits &= bits - 1u;
            if (r < (uint32_t)max_anc) ancestor_idx[(size_t)j * max_anc + r] = (int64_t)w * 32 + b;
            ++r;
        }
    }
    if (anc_count && tid == 0) anc_count[j] = kept;

    // 4. leaves: ids of the block's range that are not in the set; the range is
    //    not clipped to n_nodes (utils.py:121-122)
    for (int r = tid; r < block_m; r += kThreads) {
        const int64_t id = lo + r;
        const bool is_anc = id < n_nodes && ((bitmap[id >> 5] >> (id & 31)) & 1u);
        leaf_idx[(size_t)j * block_m + r] = is_anc ? -1 : id;
    }

    // 5. mask: row r holds its lineage plus itself in its own level column
    //    (utils.py:124-127); membership of ancestor c in that row
    for (int64_t e = tid; e < n_elem; e += kThreads) {
        const int r = (int)(e / width);
        const int l = (int)(e - (int64_t)r * width);
        const int64_t val = (l == lvl_s[r]) ? lo + r : chunk[e];
        if (val < 0 || val >= n_nodes) continue;
        const uint32_t word = bitmap[val >> 5];
        const uint32_t bit = 1u << (val & 31);
        if (!(word & bit)) continue;
        const uint32_t rank = rank_base[val >> 5] + __popc(word & (bit - 1u));
        if (rank < (uint32_t)max_anc) atomicOr(&mbits[(rank >> 5) * block_m + r], 1u << (rank & 31));
    }
    __syncthreads();

    if (mask_bits) {
        for (int e = tid; e < mask_words * block_m; e += kThreads)
            mask_bits[(size_t)j * mask_words * block_m + e] = mbits[e];
    }
    if (ancestor_mask) {
        uint8_t* out = ancestor_mask + (size_t)j * block_m * max_anc;
        const int n_out = block_m * max_anc;
        for (int e = tid; e < n_out; e += kThreads) {
            const int r = e / max_anc, c = e - r * max_anc;
            out[e] = (uint8_t)((mbits[(c >> 5) * block_m + r] >> (c & 31)) & 1u);
        }
    }

    // 6. the caller's lineage receives the self entries (utils.py:118,125)
    if (mutate) {
        for (int r = tid; r < rows; r += kThreads)
            if (lvl_s[r] >= 0) lineage[(lo + r) * width + lvl_s[r]] = lo + r;
    }
    if (err) atomicOr(status, err);
}

__global__ __launch_bounds__(kThreads) void pack_mask_kernel(
    const int64_t* __restrict__ ancestor_idx, const uint8_t* __restrict__ ancestor_mask,
    int block_m, int max_anc, int mask_words, uint32_t* __restrict__ mask_bits,
    int32_t* __restrict__ anc_count) {
    __shared__ int last_valid;
    const int tid = threadIdx.x;
    const int j = blockIdx.x;
    if (tid == 0) last_valid = -1;
    __syncthreads();
    const int64_t* idx = ancestor_idx + (size_t)j * max_anc;
    int mine = -1;
    for (int c = tid; c < max_anc; c += kThreads)
        if (idx[c] >= 0) mine = c;
    if (mine >= 0) atomicMax(&last_valid, mine);
    const uint8_t* in = ancestor_mask + (size_t)j * block_m * max_anc;
    for (int e = tid; e < mask_words * block_m; e += kThreads) {
        const int w = e / block_m, r = e - w * block_m;
        uint32_t bits = 0u;
        const int c0 = w * 32;
        const int c1 = min(c0 + 32, max_anc);
        for (int c = c0; c < c1; ++c)
            if (in[(size_t)r * max_anc + c] && idx[c] >= 0) bits |= 1u << (c - c0);
        mask_bits[(size_t)j * mask_words * block_m + e] = bits;
    }
    __syncthreads();
    if (tid == 0) anc_count[j] = last_valid + 1;
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

}  // namespace
}  // namespace fsta

using namespace fsta;

extern "C" int32_t fsta_mask_words(int32_t max_ancestors) { return (max_ancestors + 31) / 32; }

extern "C" int fsta_precompute(int64_t* lineage, const int64_t* level_lookup, int64_t n_nodes,
                               int64_t width, int32_t block_m, int32_t max_ancestors,
                               int32_t mutate_lineage, int64_t* ancestor_idx,
                               uint8_t* ancestor_mask, int64_t* leaf_idx, uint32_t* mask_bits,
                               int32_t* anc_count, uint32_t* status, void* stream) {
    if (n_nodes < 0 || width < 1 || block_m < 1 || max_ancestors < 1)
        return fail(FSTA_EINVAL, "fsta_precompute: n_nodes=%lld width=%lld block_m=%d max_ancestors=%d",
                    (long long)n_nodes, (long long)width, block_m, max_ancestors);
    if (n_nodes == 0) return FSTA_OK;
    if (!lineage || !level_lookup || !ancestor_idx || !leaf_idx || !status)
        return fail(FSTA_EINVAL, "fsta_precompute: null pointer");
    if (block_m > 4096) return fail(FSTA_EUNSUPPORTED, "fsta_precompute: block_m=%d > 4096", block_m);
    const int mask_words = fsta_mask_words(max_ancestors);
    const int64_t n_words = (n_nodes + 31) >> 5;
    const size_t lds = sizeof(uint32_t) * precompute_lds_words(n_words, mask_words, block_m);
    if (lds > 160 * 1024)
        return fail(FSTA_EUNSUPPORTED,
                    "fsta_precompute: n_nodes=%lld block_m=%d max_ancestors=%d need %zu bytes of LDS (limit 163840)",
                    (long long)n_nodes, block_m, max_ancestors, lds);
    if (lds > 64 * 1024) {
        const int rc = allow_full_lds<&block_precompute_kernel>();
        if (rc != FSTA_OK) return rc;
    }
    const int64_t nb = (n_nodes + block_m - 1) / block_m;
    hipLaunchKernelGGL(block_precompute_kernel, dim3((unsigned)nb), dim3(kThreads), lds,
                       static_cast<hipStream_t>(stream), lineage, level_lookup, n_nodes, width,
                       block_m, max_ancestors, mask_words, mutate_lineage, ancestor_idx,
                       ancestor_mask, leaf_idx, mask_bits, anc_count, status);
    FSTA_HIP_OK(hipGetLastError());
    return FSTA_OK;
}

extern "C" int fsta_pack_mask(const int64_t* ancestor_idx, const uint8_t* ancestor_mask,
                              int32_t num_blocks, int32_t block_m, int32_t max_ancestors,
                              uint32_t* mask_bits, int32_t* anc_count, void* stream) {
    if (num_blocks < 0 || block_m < 1 || max_ancestors < 1)
        return fail(FSTA_EINVAL, "fsta_pack_mask: num_blocks=%d block_m=%d max_ancestors=%d",
                    num_blocks, block_m, max_ancestors);
    if (num_blocks == 0) return FSTA_OK;
    if (!ancestor_idx || !ancestor_mask || !mask_bits || !anc_count)
        return fail(FSTA_EINVAL, "fsta_pack_mask: null pointer");
    hipLaunchKernelGGL(pack_mask_kernel, dim3(num_blocks), dim3(kThreads), 0,
                       static_cast<hipStream_t>(stream), ancestor_idx, ancestor_mask, block_m,
                       max_ancestors, fsta_mask_words(max_ancestors), mask_bits, anc_count);
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
    const unsigned grid = (unsigned)((n_nodes + kThreads - 1) / kThreads);
    const int lds_nodes = n_nodes <= 16384 ? (int)n_nodes : 0;   // 64 KB of int32
    hipLaunchKernelGGL(lineage_from_parents_kernel, dim3(grid), dim3(kThreads), (size_t)lds_nodes * 4,
                       static_cast<hipStream_t>(stream), parent, n_nodes, width, lineage,
                       level_lookup, status, lds_nodes);
    FSTA_HIP_OK(hipGetLastError());
    return FSTA_OK;
}
