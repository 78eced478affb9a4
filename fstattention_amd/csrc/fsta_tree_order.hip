// Depth-first (pre-order) renumbering of a forest on the device: parent[] -> perm / rank.
//
// The reference leaves "DFS ordering so that the nodes of a block share lineage" as an open
// item (README.md:19-20); the host version is trees.dfs_order.  Integer work, a few launches
// of N threads each; trees of speculative decoding have a few thousand nodes, so the
// sibling pass is a tiled all-pairs loop (N^2 / 2 comparisons) rather than a sort.
//
//   size[i]  nodes in the subtree of i                     (every node adds 1 to each ancestor)
//   off[i]   sum of size[s] over the siblings s visited before i (roots are siblings of each other)
//   pre[i]   = sum over a in {i and its ancestors} of (off[a] + 1), minus 1
//   perm[pre[i]] = i, rank[i] = pre[i]
#include "fsta_common.h"

namespace fsta {
namespace {

constexpr int kOrderThreads = 256;
constexpr int kSiblingTile = 1024;   // candidate siblings staged in LDS per step

__device__ __forceinline__ int32_t load_coherent(const int32_t* p) {
    // values produced by atomics of other workgroups: read past this CU's L1
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__global__ __launch_bounds__(kOrderThreads) void order_init_kernel(int64_t n, int32_t* size, int32_t* off) {
    const int64_t i = (int64_t)blockIdx.x * kOrderThreads + threadIdx.x;
    if (i < n) {
        size[i] = 1;
        off[i] = 0;
    }
}

// Every hop must go to a smaller id (or to -1), so the walks below end whatever the input holds.
__global__ __launch_bounds__(kOrderThreads) void order_sizes_kernel(const int64_t* __restrict__ parent, int64_t n,
                                                                    int32_t* size, uint32_t* status) {
    const int64_t i = (int64_t)blockIdx.x * kOrderThreads + threadIdx.x;
    if (i >= n) return;
    int64_t cur = i, p = parent[i];
    while (p != -1) {
        if (p < -1 || p >= cur) {
            atomicOr(status, FSTA_PRE_BAD_NODE_ID);
            return;
        }
        atomicAdd(&size[p], 1);
        cur = p;
        p = parent[cur];
    }
}

// grid (ceil(n / kOrderThreads), ceil(n / kSiblingTile)): thread i against the candidates of tile y
__global__ __launch_bounds__(kOrderThreads) void order_siblings_kernel(const int64_t* __restrict__ parent, int64_t n,
                                                                       int light_first, const int32_t* size,
                                                                       int32_t* off) {
    __shared__ int32_t par_s[kSiblingTile];
    __shared__ int32_t size_s[kSiblingTile];
    const int64_t i = (int64_t)blockIdx.x * kOrderThreads + threadIdx.x;
    const int64_t s0 = (int64_t)blockIdx.y * kSiblingTile;
    // a sibling has an id above the common parent; with plain index order it also lies below i
    const int64_t block_first = (int64_t)blockIdx.x * kOrderThreads;
    const int64_t block_last = min(block_first + kOrderThreads, n) - 1;
    if (!light_first && s0 > block_last) return;
    for (int t = threadIdx.x; t < kSiblingTile; t += kOrderThreads) {
        const int64_t s = s0 + t;
        par_s[t] = s < n ? (int32_t)parent[s] : -2;     // -2 never matches
        size_s[t] = s < n ? load_coherent(size + s) : 0;
    }
    __syncthreads();
    if (i >= n) return;
    const int32_t my_parent = (int32_t)parent[i];
    const int32_t my_size = load_coherent(size + i);
    const int count = (int)min((int64_t)kSiblingTile, n - s0);
    int32_t acc = 0;
    for (int t = 0; t < count; ++t) {
        const int64_t s = s0 + t;
        const bool sibling = par_s[t] == my_parent && s != i;
        const bool before = light_first ? (size_s[t] < my_size || (size_s[t] == my_size && s < i)) : s < i;
        acc += (sibling && before) ? size_s[t] : 0;
    }
    if (acc) atomicAdd(&off[i], acc);
}

__global__ __launch_bounds__(kOrderThreads) void order_finish_kernel(const int64_t* __restrict__ parent, int64_t n,
                                                                     const int32_t* off, int64_t* __restrict__ perm,
                                                                     int64_t* __restrict__ rank,
                                                                     const uint32_t* status) {
    const int64_t i = (int64_t)blockIdx.x * kOrderThreads + threadIdx.x;
    if (i >= n) return;
    if (*status) {      // malformed parent array: identity, the caller reads the status word
        perm[i] = i;
        rank[i] = i;
        return;
    }
    int64_t pre = -1, cur = i;
    while (cur >= 0) {
        pre += load_coherent(off + cur) + 1;
        const int64_t p = parent[cur];
        if (p >= cur) break;
        cur = p;
    }
    perm[pre] = i;
    rank[i] = pre;
}

}  // namespace
}  // namespace fsta

using namespace fsta;

extern "C" int fsta_dfs_order(const int64_t* parent, int64_t n_nodes, int32_t light_first, int64_t* perm,
                              int64_t* rank, int32_t* workspace, uint32_t* status, void* stream) {
    if (n_nodes < 0) return fail(FSTA_EINVAL, "fsta_dfs_order: n_nodes=%lld", (long long)n_nodes);
    if (n_nodes > FSTA_DFS_ORDER_MAX_NODES)
        return fail(FSTA_EUNSUPPORTED, "fsta_dfs_order: n_nodes=%lld > %d (all-pairs sibling pass)",
                    (long long)n_nodes, FSTA_DFS_ORDER_MAX_NODES);
    if (n_nodes == 0) return FSTA_OK;
    if (!parent || !perm || !rank || !workspace || !status)
        return fail(FSTA_EINVAL, "fsta_dfs_order: null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    int32_t* size = workspace;
    int32_t* off = workspace + n_nodes;
    const unsigned blocks = (unsigned)((n_nodes + kOrderThreads - 1) / kOrderThreads);
    const unsigned tiles = (unsigned)((n_nodes + kSiblingTile - 1) / kSiblingTile);
    hipLaunchKernelGGL(order_init_kernel, dim3(blocks), dim3(kOrderThreads), 0, s, n_nodes, size, off);
    hipLaunchKernelGGL(order_sizes_kernel, dim3(blocks), dim3(kOrderThreads), 0, s, parent, n_nodes, size, status);
    hipLaunchKernelGGL(order_siblings_kernel, dim3(blocks, tiles), dim3(kOrderThreads), 0, s, parent, n_nodes,
                       light_first ? 1 : 0, size, off);
    hipLaunchKernelGGL(order_finish_kernel, dim3(blocks), dim3(kOrderThreads), 0, s, parent, n_nodes, off, perm,
                       rank, status);
    FSTA_HIP_OK(hipGetLastError());
    return FSTA_OK;
}
