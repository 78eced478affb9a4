// Depth-first (pre-order) renumbering of a forest on the device: parent[] -> perm / rank.
//
// The reference leaves "DFS ordering so that the nodes of a block share lineage" as an open
// item (README.md:19-20); the host version is trees.dfs_order.  Integer work: one launch of one
// workgroup for the trees of speculative decoding (a few thousand nodes), six launches of N
// threads for larger ones; siblings are found through per-parent child lists, not by a sort.
//
//   size[i]  nodes in the subtree of i                     (every node adds 1 to each ancestor)
//   off[i]   sum of size[s] over the siblings s visited before i (roots are siblings of each other)
//   pre[i]   = sum over a in {i and its ancestors} of (off[a] + 1), minus 1
//   perm[pre[i]] = i, rank[i] = pre[i]
#include <mutex>

#include "fsta_common.h"

namespace fsta {
namespace {

// Scratch of fsta_dfs_order_static: subtree sizes, sibling offsets and child lists of one tree.  Every GPU the
// library runs on holds its own copy of this array (384 KiB) at its own address until the process
// ends; in host code the name below is only a handle for hipGetSymbolAddress, never an address.
static __device__ __align__(256) int32_t scratch[FSTA_DFS_ORDER_WORKSPACE_INTS(FSTA_DFS_ORDER_STATIC_MAX_NODES)];

constexpr int kMaxDevices = 64;
int32_t* g_scratch_ptr[kMaxDevices] = {};   // device address of `scratch` on each device, once looked up
std::mutex g_scratch_mutex;

// Device address of the current device's copy of `scratch` (looked up on the first call per device).
int scratch_on_current_device(int32_t** out) {
    int dev = -1;
    FSTA_HIP_OK(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return fail(FSTA_EUNSUPPORTED, "fsta_dfs_order_static: device %d", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        FSTA_HIP_OK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        if (!ptr) return fail(FSTA_EHIP, "fsta_dfs_order_static: no address for the scratch array");
        g_scratch_ptr[dev] = static_cast<int32_t*>(ptr);
    }
    *out = g_scratch_ptr[dev];
    return FSTA_OK;
}

constexpr int kOrderThreads = 256;


// ---- trees too large for one workgroup's LDS (up to FSTA_DFS_ORDER_MAX_NODES) ----------------------
// Six launches of N threads over arrays in device memory (they stay in L2: 4 bytes per node each):
//   size[i]   every node adds 1 to each ancestor (a walk of depth(i) dependent reads)
//   kids[p]   number of children; the roots are the children of a virtual node N
//   first[p]  exclusive prefix sum of kids (one workgroup)
//   child[]   the children of every parent, next to each other (slot by atomic counter: any order)
//   off[i]    sum of size[s] over the siblings s that the order visits before i: a scan of the
//             parent's child list, i.e. work proportional to sum over parents of (children)^2
//   pre[i]    sum over i and its ancestors of (off + 1), minus 1
// Work O(N * depth + sum of children^2): linear for the trees of tree decoding (bounded fan-out,
// depth of tens of levels), and still finite for a star or a chain of 2^17 nodes.
// Every hop of a walk must go to a smaller id (or to -1), so the walks end whatever the input holds.
__device__ __forceinline__ int32_t checked_parent(const int64_t* __restrict__ parent, int32_t i) {
    const int64_t p = parent[i];
    return (p >= -1 && p < i) ? (int32_t)p : -2;   // -2: malformed entry
}

__global__ __launch_bounds__(kOrderThreads) void order_init_kernel(int32_t n, int32_t* size, int32_t* kids, int32_t* bad) {
    const int32_t i = blockIdx.x * kOrderThreads + threadIdx.x;
    if (i < n) size[i] = 1;
    if (i <= n) kids[i] = 0;
    if (i == 0) *bad = 0;
}

__global__ __launch_bounds__(kOrderThreads) void order_sizes_kernel(const int64_t* __restrict__ parent, int32_t n,
                                                                    int32_t* size, int32_t* kids, int32_t* bad,
                                                                    uint32_t* status) {
    const int32_t i = blockIdx.x * kOrderThreads + threadIdx.x;
    if (i >= n) return;
    int32_t a = checked_parent(parent, i);
    if (a >= -1) atomicAdd(&kids[a >= 0 ? a : n], 1);
    while (a >= 0) {
        // neighbouring ids often meet after a few hops: where all lanes of the wave that are still
        // walking stand on the same node, one of them adds for all (else the adds queue up at the roots)
        const uint64_t walking = __ballot(true);
        const int32_t first = __builtin_amdgcn_readfirstlane(a);
        if (__ballot(a != first) == 0ull) {
            if ((threadIdx.x & 63) == __ffsll((long long)walking) - 1) atomicAdd(&size[first], __popcll(walking));
        } else {
            atomicAdd(&size[a], 1);
        }
        a = checked_parent(parent, a);
    }
    // `bad` is this call's own flag (the status word may already carry bits of an earlier stage of a
    // front-end chain, which say nothing about this parent array)
    if (a < -1) {
        atomicOr(status, FSTA_PRE_BAD_NODE_ID);
        atomicOr(bad, 1);
    }
}

constexpr int kScanThreads = 1024;

// first[p] = kids[0] + ... + kids[p-1] for p = 0 .. n (n + 1 entries), cursor = a copy; one workgroup
__global__ __launch_bounds__(kScanThreads) void order_scan_kernel(int32_t n, const int32_t* __restrict__ kids,
                                                                  int32_t* __restrict__ first, int32_t* __restrict__ cursor) {
    __shared__ int32_t wave_sum[kScanThreads / 64];
    const int tid = threadIdx.x;
    const int per = (n + 1 + kScanThreads - 1) / kScanThreads;
    const int lo = min(tid * per, n + 1), hi = min(lo + per, n + 1);
    int32_t local = 0;
    for (int x = lo; x < hi; ++x) local += kids[x];
    int32_t incl = local;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int32_t up = __shfl_up(incl, d, 64);
        if ((tid & 63) >= d) incl += up;
    }
    if ((tid & 63) == 63) wave_sum[tid >> 6] = incl;
    __syncthreads();
    int32_t base = 0;
    for (int w = 0; w < (tid >> 6); ++w) base += wave_sum[w];
    int32_t run = base + incl - local;
    for (int x = lo; x < hi; ++x) {
        first[x] = run;
        cursor[x] = run;
        run += kids[x];
    }
}

__global__ __launch_bounds__(kOrderThreads) void order_fill_kernel(const int64_t* __restrict__ parent, int32_t n,
                                                                   int32_t* cursor, int32_t* __restrict__ child) {
    const int32_t i = blockIdx.x * kOrderThreads + threadIdx.x;
    if (i >= n) return;
    const int32_t p = checked_parent(parent, i);
    if (p < -1) return;     // (flagged by the size pass; the result is the identity)
    child[atomicAdd(&cursor[p >= 0 ? p : n], 1)] = i;
}

__global__ __launch_bounds__(kOrderThreads) void order_offsets_kernel(const int64_t* __restrict__ parent, int32_t n,
                                                                      int light_first, const int32_t* __restrict__ size,
                                                                      const int32_t* __restrict__ kids,
                                                                      const int32_t* __restrict__ first,
                                                                      const int32_t* __restrict__ child,
                                                                      int32_t* __restrict__ off) {
    const int32_t i = blockIdx.x * kOrderThreads + threadIdx.x;
    if (i >= n) return;
    const int32_t p = checked_parent(parent, i);
    int32_t acc = 0;
    if (p >= -1) {
        const int32_t pp = p >= 0 ? p : n;
        const int32_t begin = first[pp], count = kids[pp];
        // order key (size, id) in one comparison; plain index order compares ids only
        const int64_t my_key = light_first ? ((int64_t)size[i] << 32) | (uint32_t)i : (int64_t)i;
        for (int32_t c = 0; c < count; ++c) {
            const int32_t s = child[begin + c];
            const int32_t sz = size[s];
            const int64_t key = light_first ? ((int64_t)sz << 32) | (uint32_t)s : (int64_t)s;
            acc += key < my_key ? sz : 0;
        }
    }
    off[i] = acc;
}

__global__ __launch_bounds__(kOrderThreads) void order_finish_kernel(const int64_t* __restrict__ parent, int32_t n,
                                                                     const int32_t* __restrict__ off, int64_t* __restrict__ perm,
                                                                     int64_t* __restrict__ rank,
                                                                     const int32_t* bad) {
    const int32_t i = blockIdx.x * kOrderThreads + threadIdx.x;
    if (i >= n) return;
    if (*bad) {      // malformed parent array: identity, the caller reads the status word
        perm[i] = i;
        rank[i] = i;
        return;
    }
    int64_t pre = -1;
    for (int32_t cur = i; cur >= 0; cur = checked_parent(parent, cur)) pre += off[cur] + 1;
    perm[pre] = i;
    rank[i] = pre;
}

// Trees of a few thousand nodes (what speculative decoding builds) in ONE workgroup and launch:
// the four steps above with every array in LDS, so that a hop or a sibling visit is an LDS
// access and the steps are separated by barriers instead of kernel boundaries.  Siblings are
// found through per-parent child lists (built with atomic exchanges) instead of the all-pairs
// loop: a node visits its parent's other children only.  A list is a chain of dependent reads,
// so children of a parent with more than kListedChildren of them (no tree of speculative decoding
// has such nodes) scan the whole node array instead, whose reads are independent.
// (Tried and dropped: path sums by pointer doubling and sizes level by level.  Fewer dependent
// hops, but every round ends in a barrier of 16 waves, which costs more than the hops it saves
// on trees up to 160 levels deep.)
constexpr int kSmallThreads = 1024;
constexpr int kSmallMaxNodes = 4096;   // 6 int32 arrays of n (+1) entries: 96 KB of LDS
constexpr int kListedChildren = 64;

__global__ __launch_bounds__(kSmallThreads) void order_small_kernel(const int64_t* __restrict__ parent, int n,
                                                                    int light_first, int64_t* __restrict__ perm,
                                                                    int64_t* __restrict__ rank,
                                                                    uint32_t* __restrict__ status) {
    asm volatile("" ::"s"(parent), "s"(n), "s"(light_first), "s"(perm), "s"(rank), "s"(status));   // one batch of argument loads
    extern __shared__ int32_t small_s[];
    int32_t* par_s = small_s;          // [n]   parent, -1 for roots
    int32_t* size_s = par_s + n;       // [n]   nodes in the subtree
    int32_t* off_s = size_s + n;       // [n]   sizes of the siblings visited earlier
    int32_t* next_s = off_s + n;       // [n]   next child of the same parent
    int32_t* head_s = next_s + n;      // [n+1] first child; entry n: the roots
    int32_t* kids_s = head_s + n + 1;  // [n+1] number of children
    int32_t* bad_s = kids_s + n + 1;   // [1]   malformed input
    const int tid = threadIdx.x;
    if (tid == 0) *bad_s = 0;
    for (int i = tid; i <= n; i += kSmallThreads) {
        head_s[i] = -1;
        kids_s[i] = 0;
    }
    __syncthreads();
    for (int i = tid; i < n; i += kSmallThreads) {
        const int64_t p = parent[i];
        const bool ok = p >= -1 && p < i;     // every hop goes to a smaller id: the walks end
        par_s[i] = ok ? (int32_t)p : -1;
        size_s[i] = 1;
        if (!ok) *bad_s = 1;
    }
    __syncthreads();
    if (*bad_s) {      // malformed parent array: identity, the caller reads the status word
        for (int i = tid; i < n; i += kSmallThreads) {
            perm[i] = i;
            rank[i] = i;
        }
        if (tid == 0) atomicOr(status, FSTA_PRE_BAD_NODE_ID);
        return;
    }
    for (int i = tid; i < n; i += kSmallThreads) {
        const int32_t p = par_s[i];
        next_s[i] = atomicExch(&head_s[p >= 0 ? p : n], i);
        atomicAdd(&kids_s[p >= 0 ? p : n], 1);
        // Every node adds 1 to each of its ancestors.  Nodes with neighbouring ids meet after a
        // few hops: where all lanes of the wave that are still walking stand on the same node,
        // one of them adds for all (otherwise the adds of a shallow tree queue up at its root).
        for (int32_t a = p; a >= 0; a = par_s[a]) {
            const uint64_t walking = __ballot(true);
            const int32_t first = __builtin_amdgcn_readfirstlane(a);
            if (__ballot(a != first) == 0ull) {
                if ((tid & 63) == __ffsll((long long)walking) - 1) atomicAdd(&size_s[first], __popcll(walking));
            } else {
                atomicAdd(&size_s[a], 1);
            }
        }
    }
    __syncthreads();
    for (int i = tid; i < n; i += kSmallThreads) {
        const int32_t p = par_s[i];
        const int32_t my_key = light_first ? (size_s[i] << 13) | i : i;    // sizes and ids are below 2^13
        int32_t acc = 0;
        if (kids_s[p >= 0 ? p : n] <= kListedChildren) {
            for (int32_t s = head_s[p >= 0 ? p : n]; s >= 0; s = next_s[s]) {
                const int32_t sz = size_s[s];
                const int32_t key = light_first ? (sz << 13) | s : s;
                acc += key < my_key ? sz : 0;
            }
        } else {
#pragma unroll 4
            for (int32_t s = 0; s < n; ++s) {
                const int32_t sz = size_s[s];
                const int32_t key = light_first ? (sz << 13) | s : s;
                acc += (par_s[s] == p && key < my_key) ? sz : 0;
            }
        }
        off_s[i] = acc;
    }
    __syncthreads();
    for (int i = tid; i < n; i += kSmallThreads) {
        int32_t pre = -1;
        for (int32_t cur = i; cur >= 0; cur = par_s[cur]) pre += off_s[cur] + 1;
        perm[pre] = i;
        rank[i] = pre;
    }
}

// new_parent[rank[i]] = rank[parent[i]]: the same forest with node i renamed rank[i]
__global__ __launch_bounds__(kOrderThreads) void renumber_kernel(const int64_t* __restrict__ parent,
                                                                 const int64_t* __restrict__ rank, int64_t n,
                                                                 int64_t* __restrict__ new_parent) {
    const int64_t i = (int64_t)blockIdx.x * kOrderThreads + threadIdx.x;
    if (i >= n) return;
    const int64_t p = parent[i], r = rank[i];
    if (r < 0 || r >= n) return;                      // not a permutation: nothing written for this node
    new_parent[r] = (p >= 0 && p < n) ? rank[p] : -1;
}

}  // namespace
}  // namespace fsta

using namespace fsta;

extern "C" int fsta_renumber_parents(const int64_t* parent, const int64_t* rank, int64_t n_nodes,
                                     int64_t* new_parent, void* stream) {
    if (n_nodes < 0) return fail(FSTA_EINVAL, "fsta_renumber_parents: n_nodes=%lld", (long long)n_nodes);
    if (n_nodes == 0) return FSTA_OK;
    if (!parent || !rank || !new_parent) return fail(FSTA_EINVAL, "fsta_renumber_parents: null pointer");
    const int64_t blocks = (n_nodes + kOrderThreads - 1) / kOrderThreads;
    if (blocks > 0x7fffffff) return fail(FSTA_EUNSUPPORTED, "fsta_renumber_parents: n_nodes=%lld", (long long)n_nodes);
    hipLaunchKernelGGL(renumber_kernel, dim3((unsigned)blocks), dim3(kOrderThreads), 0, static_cast<hipStream_t>(stream),
                       parent, rank, n_nodes, new_parent);
    FSTA_HIP_OK(hipGetLastError());
    return FSTA_OK;
}

namespace {

// The launches of fsta_dfs_order; `workspace`: FSTA_DFS_ORDER_WORKSPACE_INTS(n_nodes) int32 of device
// memory (only trees too large for the single-workgroup kernel touch it).
int dfs_order_launch(const int64_t* parent, int64_t n_nodes, int32_t light_first, int64_t* perm, int64_t* rank,
                     int32_t* workspace, uint32_t* status, hipStream_t s) {
    if (n_nodes <= kSmallMaxNodes) {
        const size_t lds = (size_t)(6 * n_nodes + 3) * sizeof(int32_t);
        if (lds > 64 * 1024) {
            const int rc = allow_full_lds<&order_small_kernel>();
            if (rc != FSTA_OK) return rc;
        }
        hipLaunchKernelGGL(order_small_kernel, dim3(1), dim3(kSmallThreads), lds, s, parent, (int)n_nodes,
                           light_first ? 1 : 0, perm, rank, status);
        FSTA_HIP_OK(hipGetLastError());
        return FSTA_OK;
    }
    const int32_t n = (int32_t)n_nodes;
    int32_t* size = workspace;                 // [n]
    int32_t* off = size + n;                   // [n]
    int32_t* kids = off + n;                   // [n + 1]
    int32_t* first = kids + n + 1;             // [n + 1]
    int32_t* cursor = first + n + 1;           // [n + 1]
    int32_t* child = cursor + n + 1;           // [n]
    int32_t* bad = child + n;                  // [1] this call found a malformed parent entry
    const unsigned blocks = (unsigned)((n_nodes + kOrderThreads) / kOrderThreads);   // covers n + 1 entries
    // (every array is written by a kernel before it is read: nothing of an earlier call survives)
    hipLaunchKernelGGL(order_init_kernel, dim3(blocks), dim3(kOrderThreads), 0, s, n, size, kids, bad);
    hipLaunchKernelGGL(order_sizes_kernel, dim3(blocks), dim3(kOrderThreads), 0, s, parent, n, size, kids, bad, status);
    hipLaunchKernelGGL(order_scan_kernel, dim3(1), dim3(kScanThreads), 0, s, n, kids, first, cursor);
    hipLaunchKernelGGL(order_fill_kernel, dim3(blocks), dim3(kOrderThreads), 0, s, parent, n, cursor, child);
    hipLaunchKernelGGL(order_offsets_kernel, dim3(blocks), dim3(kOrderThreads), 0, s, parent, n, light_first ? 1 : 0,
                       size, kids, first, child, off);
    hipLaunchKernelGGL(order_finish_kernel, dim3(blocks), dim3(kOrderThreads), 0, s, parent, n, off, perm, rank, bad);
    FSTA_HIP_OK(hipGetLastError());
    return FSTA_OK;
}

}  // namespace

extern "C" int fsta_dfs_order(const int64_t* parent, int64_t n_nodes, int32_t light_first, int64_t* perm,
                              int64_t* rank, int32_t* workspace, uint32_t* status, void* stream) {
    if (n_nodes < 0) return fail(FSTA_EINVAL, "fsta_dfs_order: n_nodes=%lld", (long long)n_nodes);
    if (n_nodes > FSTA_DFS_ORDER_MAX_NODES)
        return fail(FSTA_EUNSUPPORTED, "fsta_dfs_order: n_nodes=%lld > %d", (long long)n_nodes, FSTA_DFS_ORDER_MAX_NODES);
    if (n_nodes == 0) return FSTA_OK;
    if (!parent || !perm || !rank || !workspace || !status)
        return fail(FSTA_EINVAL, "fsta_dfs_order: null pointer");
    return dfs_order_launch(parent, n_nodes, light_first, perm, rank, workspace, status, static_cast<hipStream_t>(stream));
}

extern "C" int fsta_dfs_order_static(const int64_t* parent, int64_t n_nodes, int32_t light_first, int64_t* perm,
                                     int64_t* rank, uint32_t* status, void* stream) {
    if (n_nodes < 0) return fail(FSTA_EINVAL, "fsta_dfs_order_static: n_nodes=%lld", (long long)n_nodes);
    if (n_nodes > FSTA_DFS_ORDER_STATIC_MAX_NODES)
        return fail(FSTA_EUNSUPPORTED, "fsta_dfs_order_static: n_nodes=%lld > %d (size of the library's own scratch array; "
                    "fsta_dfs_order takes a workspace of the caller's)", (long long)n_nodes, FSTA_DFS_ORDER_STATIC_MAX_NODES);
    if (n_nodes == 0) return FSTA_OK;
    if (!parent || !perm || !rank || !status) return fail(FSTA_EINVAL, "fsta_dfs_order_static: null pointer");
    int32_t* work = nullptr;
    const int rc = scratch_on_current_device(&work);
    if (rc != FSTA_OK) return rc;
    return dfs_order_launch(parent, n_nodes, light_first, perm, rank, work, status, static_cast<hipStream_t>(stream));
}
