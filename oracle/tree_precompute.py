"""CPU restatement of the per-block tree precompute (test infrastructure only).

``block_inputs`` follows reference ``utils.py:104-129`` step for step with numpy
in place of torch: ``numpy.unique`` is ascending like ``torch.unique``
(``utils.py:119``), ``numpy.isin`` is set membership like ``torch.isin``
(``utils.py:127``).  ``dense_tree_mask`` and ``block_inputs_bruteforce`` are
independent formulations used to pin it.
"""
from __future__ import annotations

import math

import numpy as np


def block_inputs(lineage: np.ndarray, level_lookup: np.ndarray, block_m: int = 64,
                 max_ancestors: int = 32, mutate: bool = True):
    """``(ancestor_idx int64 [NB,A], ancestor_mask bool [NB,M,A], leaf_idx int64 [NB,M])``.

    Per block of ``block_m`` consecutive node ids (reference ``utils.py:116-127``):

    * unique values of the block's lineage rows, ascending, first one dropped
      (it is the ``-1`` padding) -> left-aligned in ``ancestor_idx`` (``:119-120``);
      more than ``max_ancestors`` of them is an error like the reference's
      shape-mismatch ``RuntimeError``;
    * every id of ``arange(j*M, (j+1)*M)`` -- not clipped to ``N`` -- that is not
      in that set is a leaf, stored at its row (``:121-122``);
    * each real node is written into its own level column (``:124-125``) and
      ``ancestor_mask[j, r, c]`` says whether ancestor ``c`` occurs in row ``r``
      afterwards (``:126-127``).

    With ``mutate`` the caller's ``lineage`` receives the self entries, as the
    reference's view semantics do (``utils.py:118,125``).
    """
    if not mutate:
        lineage = lineage.copy()
    n = lineage.shape[0]
    nb = math.ceil(n / block_m)
    ancestor_idx = np.full((nb, max_ancestors), -1, dtype=np.int64)
    ancestor_mask = np.zeros((nb, block_m, max_ancestors), dtype=np.bool_)
    leaf_idx = np.full((nb, block_m), -1, dtype=np.int64)
    for j in range(nb):
        lo = j * block_m
        chunk = lineage[lo: lo + block_m]            # view, like utils.py:118
        uniq = np.unique(chunk.reshape(-1))[1:]
        if uniq.shape[0] > max_ancestors:
            raise RuntimeError(
                f"block {j}: {uniq.shape[0]} unique ancestors exceed max_ancestors={max_ancestors}")
        ancestor_idx[j, : uniq.shape[0]] = uniq
        members = set(uniq.tolist())
        for node in range(lo, lo + block_m):
            if node not in members:
                leaf_idx[j, node - lo] = node
        for node in range(lo, min(lo + block_m, n)):
            chunk[node - lo, level_lookup[node]] = node
        for r in range(chunk.shape[0]):
            ancestor_mask[j, r, : uniq.shape[0]] = np.isin(uniq, chunk[r])
    return ancestor_idx, ancestor_mask, leaf_idx


def ancestors_of(parent: np.ndarray, i: int):
    out = []
    p = int(parent[i])
    while p >= 0:
        out.append(p)
        p = int(parent[p])
    return out


def dense_tree_mask(parent: np.ndarray) -> np.ndarray:
    """bool ``[N,N]``: ``mask[i,a]`` iff ``a`` is ``i`` or a strict ancestor of ``i``."""
    parent = np.asarray(parent)
    n = parent.shape[0]
    mask = np.zeros((n, n), dtype=np.bool_)
    for i in range(n):
        mask[i, i] = True
        mask[i, ancestors_of(parent, i)] = True
    return mask


def block_inputs_bruteforce(parent: np.ndarray, block_m: int, max_ancestors: int):
    """Same three tensors, built from the parent array with Python sets only."""
    parent = np.asarray(parent)
    n = parent.shape[0]
    nb = math.ceil(n / block_m)
    ancestor_idx = np.full((nb, max_ancestors), -1, dtype=np.int64)
    ancestor_mask = np.zeros((nb, block_m, max_ancestors), dtype=np.bool_)
    leaf_idx = np.full((nb, block_m), -1, dtype=np.int64)
    for j in range(nb):
        lo = j * block_m
        rows = range(lo, min(lo + block_m, n))
        anc = {i: set(ancestors_of(parent, i)) for i in rows}
        union = sorted(set().union(*anc.values())) if anc else []
        if len(union) > max_ancestors:
            raise RuntimeError("too many ancestors")
        ancestor_idx[j, : len(union)] = union
        for r in range(block_m):
            if lo + r not in union:
                leaf_idx[j, r] = lo + r
        for i in rows:
            allowed = anc[i] | {i}
            for c, a in enumerate(union):
                ancestor_mask[j, i - lo, c] = a in allowed
    return ancestor_idx, ancestor_mask, leaf_idx


def reconstruct_dense_mask(ancestor_idx, ancestor_mask, leaf_idx, n: int) -> np.ndarray:
    """Scatter the block tensors back into a dense bool ``[n, n_cols]`` mask.

    Row ``i`` of block ``j`` allows column ``ancestor_idx[j,c]`` where
    ``ancestor_mask[j,r,c]`` is set, plus ``leaf_idx[j,r]`` when that is ``>= 0``.
    Columns reach as far as the largest index present (pad-row leaves of a
    ragged last block point past ``n``).
    """
    ancestor_idx = np.asarray(ancestor_idx)
    ancestor_mask = np.asarray(ancestor_mask)
    leaf_idx = np.asarray(leaf_idx)
    nb, m = leaf_idx.shape
    ncols = max(n, int(leaf_idx.max()) + 1, int(ancestor_idx.max()) + 1)
    out = np.zeros((nb * m, ncols), dtype=np.bool_)
    for j in range(nb):
        for r in range(m):
            cols = ancestor_idx[j][ancestor_mask[j, r]]
            out[j * m + r, cols] = True
            if leaf_idx[j, r] >= 0:
                out[j * m + r, leaf_idx[j, r]] = True
    return out


def kv_rows_loaded(ancestor_idx, leaf_idx) -> int:
    """``sum_j (n_anc[j] + n_leaf[j])``: K (or V) rows the op gathers per head."""
    return int((np.asarray(ancestor_idx) >= 0).sum() + (np.asarray(leaf_idx) >= 0).sum())


def attended_pairs(parent: np.ndarray) -> int:
    """``sum_i (depth(i) + 1)``: query/key pairs that are not masked."""
    parent = np.asarray(parent)
    depth = np.zeros(parent.shape[0], dtype=np.int64)
    for i in range(parent.shape[0]):
        depth[i] = 0 if parent[i] < 0 else depth[parent[i]] + 1
    return int(depth.sum() + parent.shape[0])
