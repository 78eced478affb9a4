"""Host-side tree generators and the lineage layout contract.

A tree (forest) over node ids ``0..N-1`` is described either by a ``parent``
array (``parent[i] < i`` or ``-1`` for a root) or by the reference's
``(lineage, level_lookup)`` pair (reference ``utils.py:43-44,66-75``):

* ``level_lookup[i]``  level of node ``i`` (roots are level 0), int64 ``[N]``;
* ``lineage[i, l]``    id of node ``i``'s strict ancestor living at level ``l``,
  ``-1`` elsewhere, int64 ``[N, max_level + 1]``.  The column of a node's own
  level is ``-1`` until the block precompute writes the node id there
  (reference ``utils.py:125``).

Everything here is synthetic-input generation that runs on the host with numpy;
none of it is on the accelerated path.  The five ``config*`` generators build
the trees of the benchmark configurations, seeded with
``numpy.random.default_rng``.
"""
from __future__ import annotations

import itertools
import math
from dataclasses import dataclass

import numpy as np
import torch

# Sequence length -> tree depth / ancestor tile of the reference's own benchmark
# trees (reference ``utils.py:4-24``): 2**k tokens <-> depth k-3, always 64 ancestors.
DEPTH_MAPPING = {2 ** k: k - 3 for k in range(10, 18)}
MAX_ANCESTOR_MAPPING = {2 ** k: 64 for k in range(10, 18)}


# --------------------------------------------------------------------------- #
# parent array <-> lineage
# --------------------------------------------------------------------------- #
def levels_from_parents(parent: np.ndarray) -> np.ndarray:
    """Level of every node; requires ``parent[i] < i`` (roots: ``-1``)."""
    parent = np.asarray(parent, dtype=np.int64)
    n = parent.shape[0]
    if n and (parent >= np.arange(n)).any():
        raise ValueError("parent[i] must be < i (topological numbering)")
    if n and (parent < -1).any():
        raise ValueError("parent[i] must be >= -1")
    level = np.zeros(n, dtype=np.int64)
    for i in range(n):
        p = parent[i]
        level[i] = 0 if p < 0 else level[p] + 1
    return level


def lineage_from_parents(parent, min_width: int = 0):
    """``parent[N]`` -> ``(lineage int64 [N, max_level+1], level_lookup int64 [N])``.

    Follows the layout of reference ``utils.py:66-75``: a strict ancestor ``a``
    of node ``i`` is stored at ``lineage[i, level(a)]``.  The width leaves one
    column for the deepest node's own level so that every row holds at least
    one ``-1`` (reference ``utils.py:119`` depends on it).
    """
    parent = np.asarray(parent, dtype=np.int64)
    n = parent.shape[0]
    level = levels_from_parents(parent)
    width = max(int(level.max()) + 1 if n else 1, int(min_width), 1)
    lineage = np.full((n, width), -1, dtype=np.int64)
    for i in range(n):
        p = parent[i]
        if p >= 0:
            lp = level[p]
            lineage[i, :lp] = lineage[p, :lp]
            lineage[i, lp] = p
    return torch.from_numpy(lineage), torch.from_numpy(level)


def parents_from_lineage(lineage, level_lookup) -> np.ndarray:
    """Inverse of :func:`lineage_from_parents` (ignores a self entry if present)."""
    lin = np.asarray(lineage)
    lvl = np.asarray(level_lookup)
    n = lin.shape[0]
    parent = np.full(n, -1, dtype=np.int64)
    has = lvl > 0
    parent[has] = lin[np.nonzero(has)[0], lvl[has] - 1]
    return parent


# --------------------------------------------------------------------------- #
# lineage-aware node order (the reference's open item, README.md:19-20)
# --------------------------------------------------------------------------- #
def subtree_sizes(parent) -> np.ndarray:
    """Number of nodes in the subtree of every node (itself included)."""
    parent = np.asarray(parent, dtype=np.int64)
    size = np.ones(parent.shape[0], dtype=np.int64)
    for i in range(parent.shape[0] - 1, 0, -1):      # children come after their parents
        if parent[i] >= 0:
            size[parent[i]] += size[i]
    return size


def dfs_order(parent, children: str = "index") -> np.ndarray:
    """Depth-first (pre-order) numbering of a forest: ``perm[new_id] = old_id``.

    Blocks of consecutive ids then hold whole subtrees and paths, so the nodes
    of a block share most of their ancestors and the per-block ancestor lists
    (reference ``utils.py:116-120``) shrink.  Siblings (and roots) are visited
    by ascending id (``children="index"``) or smallest subtree first
    (``"light_first"``, ties by id), which leaves the long paths for last and
    packs the short ones next to their parent.  A parent still precedes its
    children, so the result is a valid numbering for every function here.
    """
    parent = np.asarray(parent, dtype=np.int64)
    n = parent.shape[0]
    if children not in ("index", "light_first"):
        raise ValueError(f"children={children!r}: expected 'index' or 'light_first'")
    levels_from_parents(parent)                      # validates parent[i] < i
    size = subtree_sizes(parent)
    kids = [[] for _ in range(n)]
    roots = []
    for i in range(n):
        (roots if parent[i] < 0 else kids[parent[i]]).append(i)
    if children == "light_first":
        key = lambda x: (size[x], x)
        roots.sort(key=key)
        for c in kids:
            c.sort(key=key)
    perm = np.empty(n, dtype=np.int64)
    stack = roots[::-1]
    filled = 0
    while stack:
        x = stack.pop()
        perm[filled] = x
        filled += 1
        stack.extend(kids[x][::-1])
    assert filled == n
    return perm


def renumber_parents(parent, perm):
    """The same forest with node ``perm[new]`` renamed ``new``: ``(new_parent, rank)``.

    ``rank[old] = new`` is the inverse of ``perm``.  Token tensors laid out in the
    old order are brought to the new one with ``x.index_select(2, perm)`` (q, and
    the tree part of k and v) and results back with ``o.index_select(2, rank)``.
    ``perm`` must keep parents in front of their children.
    """
    parent = np.asarray(parent, dtype=np.int64)
    perm = np.asarray(perm, dtype=np.int64)
    n = parent.shape[0]
    if perm.shape != (n,) or not np.array_equal(np.sort(perm), np.arange(n)):
        raise ValueError("perm is not a permutation of the node ids")
    rank = np.empty(n, dtype=np.int64)
    rank[perm] = np.arange(n, dtype=np.int64)
    old_parent = parent[perm]
    new_parent = np.where(old_parent >= 0, rank[np.maximum(old_parent, 0)], -1)
    if n and (new_parent >= np.arange(n)).any():
        raise ValueError("perm puts a child in front of its parent")
    return new_parent, rank


# --------------------------------------------------------------------------- #
# the reference's own benchmark tree
# --------------------------------------------------------------------------- #
def _level_starts(depth: int, topk: int, left_weight_factor: float) -> np.ndarray:
    starts = np.zeros(depth + 2, dtype=np.int64)
    size = topk
    starts[1] = topk
    for i in range(2, depth + 2):
        size = topk * int(size * left_weight_factor)
        starts[i] = starts[i - 1] + size
    return starts


def create_tree(depth: int = 7, topk: int = 4, left_weight_factor: float = 0.5):
    """Left-weighted top-k forest of reference ``utils.py:27-77``.

    Level ``l`` has ``topk * int(prev * left_weight_factor)`` nodes, numbered
    level by level; node ``i`` of level ``l >= 1`` hangs under
    ``start[l-1] + (i - start[l]) // topk``.  With the defaults the tree has
    ``2**(depth+3) - 4`` nodes.  Returns ``(lineage [N, depth+1], level_lookup [N])``
    as int64 torch tensors, the own-level column still ``-1``.
    """
    starts = _level_starts(depth, topk, left_weight_factor)
    n = int(starts[-1])
    idx = np.arange(n, dtype=np.int64)
    level = np.searchsorted(starts, idx, side="right").astype(np.int64) - 1
    lineage = np.full((n, depth + 1), -1, dtype=np.int64)
    for l in range(1, depth + 1):
        nodes = idx[level == l]
        if nodes.size == 0:
            continue
        par = starts[l - 1] + (nodes - starts[l]) // topk
        lineage[nodes, : l - 1] = lineage[par, : l - 1]
        lineage[nodes, l - 1] = par
    return torch.from_numpy(lineage), torch.from_numpy(level)


def create_full_attention_mask(lineage, pad_size: int = 4):
    """Dense ancestor-or-self mask with the reference's return convention.

    Reference ``utils.py:79-102`` returns a float32 ``[N+4, N+4]`` tensor whose
    trailing 4 rows/columns are zero.  This restatement ignores the ``-1``
    padding explicitly instead of letting it index column ``N-1``, so it is also
    right when the last node is somebody's ancestor.
    """
    lin = np.asarray(lineage)
    n = lin.shape[0]
    mask = np.zeros((n + pad_size, n + pad_size), dtype=np.float32)
    rows, cols = np.nonzero(lin >= 0)
    mask[rows, lin[rows, cols]] = 1.0
    mask[np.arange(n), np.arange(n)] = 1.0
    return torch.from_numpy(mask)


# --------------------------------------------------------------------------- #
# benchmark configurations
# --------------------------------------------------------------------------- #
@dataclass(frozen=True)
class TreeConfig:
    """One benchmark configuration: the tree plus the tensor shapes it runs on."""
    name: str
    parent: np.ndarray
    block_m: int
    batch: int
    heads: int
    head_dim: int
    dtype: torch.dtype
    tree_seed: int
    tensor_seed: int
    layers: int = 1
    pad_rows: int = 0          # q/k/v rows past the tree (the reference's tensors hold N_CTX = n_nodes + 4 rows)
    max_ancestors: int = 0     # 0: derived from the tree

    @property
    def n_nodes(self) -> int:
        return int(self.parent.shape[0])


def random_recursive_parents(n: int, seed: int, window: int | None = None) -> np.ndarray:
    """``parent[i] ~ U[max(0, i-window), i)``; ``window=None`` means ``U[0, i)``."""
    rng = np.random.default_rng(seed)
    parent = np.full(n, -1, dtype=np.int64)
    for i in range(1, n):
        lo = 0 if window is None else max(0, i - window)
        parent[i] = rng.integers(lo, i)
    return parent


def medusa_parents(n: int = 256, depths: int = 4, topk: int = 10,
                   alpha: float = 0.3, seed: int = 1002) -> np.ndarray:
    """Medusa-style static tree: keep the ``n-1`` most probable candidate paths.

    Each draft depth has ``topk`` ranked candidates whose probabilities are a
    seeded Dirichlet(alpha) draw sorted descending; a path ``(r1..rd)`` scores
    the product of its ranks' probabilities.  Node 0 is the root (empty path);
    the other nodes are the best ``n-1`` paths (the set is prefix-closed
    because a prefix never scores below its extensions; ties break on
    ``(depth, ranks)``), numbered by ``(depth, ranks)`` ascending so that
    ``parent < child``.
    """
    return medusa_parents_from_probs(medusa_probs(depths, topk, alpha, seed), n)


def medusa_probs(depths: int = 4, topk: int = 10, alpha: float = 0.3, seed: int = 1002) -> np.ndarray:
    """Seeded candidate probabilities ``[depths, topk]`` (float64), each row sorted descending."""
    rng = np.random.default_rng(seed)
    return np.stack([np.sort(rng.dirichlet(alpha * np.ones(topk)))[::-1] for _ in range(depths)])


def medusa_parents_from_probs(probs, n: int) -> np.ndarray:
    """Parent array of the tree of the ``n-1`` most probable paths for given ``probs [depths, topk]``."""
    probs = np.asarray(probs, dtype=np.float64)
    depths, topk = probs.shape
    cands = []
    for d in range(1, depths + 1):
        for ranks in itertools.product(range(topk), repeat=d):
            score = 1.0
            for h, r in enumerate(ranks):
                score *= probs[h][r]
            cands.append((-score, d, ranks))
    cands.sort()
    kept = sorted((d, ranks) for _, d, ranks in cands[: n - 1])
    # close under prefixes defensively (floating-point ties could break closure)
    have = {ranks for _, ranks in kept}
    for _, ranks in kept:
        if len(ranks) > 1 and ranks[:-1] not in have:
            raise AssertionError("kept path set is not prefix-closed")
    ids = {(): 0}
    for i, (_, ranks) in enumerate(kept, start=1):
        ids[ranks] = i
    parent = np.full(len(kept) + 1, -1, dtype=np.int64)
    for _, ranks in kept:
        parent[ids[ranks]] = ids[ranks[:-1]]
    return parent


def deep_narrow_parents(n: int = 1024, chain_depth: int = 128, p_branch: float = 0.25,
                        max_branch: int = 32, seed: int = 1003) -> np.ndarray:
    """Chain ``0..chain_depth`` plus side paths of length ``U{1..max_branch}``.

    The chain nodes are swept repeatedly; each sprouts a new path with
    probability ``p_branch``.  New nodes are appended to the id space; the last
    path is truncated when ``n`` nodes exist.
    """
    rng = np.random.default_rng(seed)
    parent = [-1] + list(range(chain_depth))
    while len(parent) < n:
        for c in range(chain_depth + 1):
            if len(parent) >= n:
                break
            if rng.random() < p_branch:
                length = int(rng.integers(1, max_branch + 1))
                prev = c
                for _ in range(length):
                    if len(parent) >= n:
                        break
                    parent.append(prev)
                    prev = len(parent) - 1
    return np.asarray(parent, dtype=np.int64)


def wide_shallow_parents(n: int = 4096, branching: int = 8) -> np.ndarray:
    """Complete ``branching``-ary tree in BFS order, truncated to ``n`` nodes."""
    i = np.arange(n, dtype=np.int64)
    parent = (i - 1) // branching
    parent[0] = -1
    return parent


def config(index: int, dtype: torch.dtype | None = None) -> TreeConfig:
    """The five benchmark configurations (1-based ``index``)."""
    if index == 1:
        return TreeConfig("cfg1_random64_fp32", random_recursive_parents(64, 1001), 16,
                          1, 8, 64, dtype or torch.float32, 1001, 2001)
    if index == 2:
        return TreeConfig("cfg2_medusa256", medusa_parents(256, seed=1002), 64,
                          1, 32, 128, dtype or torch.bfloat16, 1002, 2002)
    if index == 3:
        return TreeConfig("cfg3_deep1024", deep_narrow_parents(1024, seed=1003), 64,
                          1, 32, 128, dtype or torch.bfloat16, 1003, 2003)
    if index == 4:
        return TreeConfig("cfg4_wide4096", wide_shallow_parents(4096, 8), 64,
                          1, 32, 128, dtype or torch.bfloat16, 1004, 2004)
    if index == 5:
        return TreeConfig("cfg5_batched2048", random_recursive_parents(2048, 1005, window=64), 128,
                          8, 64, 128, dtype or torch.bfloat16, 1005, 2005, layers=32)
    raise ValueError(f"no such config: {index}")


def reference_benchmark_config(n_ctx: int) -> TreeConfig:
    """The workload of the reference's own benchmark (``fstattention.py:240-296``): batch 4, 48 heads,
    head dim 64, float16, ``create_tree(DEPTH_MAPPING[n_ctx])`` (``n_ctx - 4`` nodes in tensors of
    ``n_ctx`` rows), query blocks of 128 rows, 64 ancestor slots."""
    lineage, level = create_tree(DEPTH_MAPPING[n_ctx])
    parent = parents_from_lineage(lineage.numpy(), level.numpy())
    return TreeConfig(f"reference_benchmark_n{n_ctx}", parent, 128, 4, 48, 64, torch.float16, 0, 3000 + n_ctx,
                      pad_rows=n_ctx - parent.shape[0], max_ancestors=MAX_ANCESTOR_MAPPING[n_ctx])


def make_qkv(cfg: TreeConfig, layer: int = 0, device="cpu", prefix: int = 0):
    """CPU-seeded N(0,1) q/k/v of the configuration's shape, cast then moved."""
    g = torch.Generator().manual_seed(cfg.tensor_seed + layer)
    shape_q = (cfg.batch, cfg.heads, cfg.n_nodes, cfg.head_dim)
    shape_k = (cfg.batch, cfg.heads, cfg.n_nodes + prefix, cfg.head_dim)
    q = torch.randn(shape_q, generator=g, dtype=torch.float32).to(cfg.dtype)
    k = torch.randn(shape_k, generator=g, dtype=torch.float32).to(cfg.dtype)
    v = torch.randn(shape_k, generator=g, dtype=torch.float32).to(cfg.dtype)
    return q.to(device), k.to(device), v.to(device)


def required_max_ancestors(parent: np.ndarray, block_m: int, multiple: int = 16) -> int:
    """Largest per-block count of unique strict ancestors, rounded up."""
    parent = np.asarray(parent)
    n = parent.shape[0]
    worst = 1
    for start in range(0, n, block_m):
        seen = set()
        for i in range(start, min(start + block_m, n)):
            p = parent[i]
            while p >= 0 and p not in seen:
                seen.add(int(p))
                p = parent[p]
        worst = max(worst, len(seen))
    return int(math.ceil(worst / multiple) * multiple)
