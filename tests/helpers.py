"""Shared helpers of the GPU parity tests."""
import math

import numpy as np
import torch

from fstattention_amd import trees
from oracle import dense_attention as da
from oracle import tree_precompute as tp

TOL = {torch.float32: 1e-5, torch.float16: 2e-3, torch.bfloat16: 2e-3}


def oracle_inputs(parent, block_m, max_anc=None, multiple=16):
    """CPU oracle's (ancestor_idx, ancestor_mask, leaf_idx) as torch tensors + max_anc."""
    lineage, level = trees.lineage_from_parents(parent)
    if max_anc is None:
        max_anc = trees.required_max_ancestors(parent, block_m, multiple)
    a_idx, a_mask, l_idx = tp.block_inputs(lineage.numpy().copy(), level.numpy(), block_m, max_anc)
    return torch.from_numpy(a_idx), torch.from_numpy(a_mask), torch.from_numpy(l_idx), max_anc


def rand_qkv(z, h, nq, nk, d, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn((z, h, nq, d), generator=g, dtype=torch.float32).to(dtype)
    k = torch.randn((z, h, nk, d), generator=g, dtype=torch.float32).to(dtype)
    v = torch.randn((z, h, nk, d), generator=g, dtype=torch.float32).to(dtype)
    return q, k, v


def dense_oracle(q, k, v, parent, sm_scale, prefix=0, nq_pad=0):
    """float64 dense-masked attention over [prefix | tree (+ pad rows that see themselves)]."""
    mask = tp.dense_tree_mask(parent)
    n = mask.shape[0]
    if nq_pad:
        full = np.zeros((n + nq_pad, n + nq_pad), dtype=bool)
        full[:n, :n] = mask
        full[np.arange(n, n + nq_pad), np.arange(n, n + nq_pad)] = True
        mask = full
    mask = da.full_mask_with_prefix(mask, prefix)
    return da.dense_tree_attention(q, k, v, mask, sm_scale, dtype=torch.float64)


def assert_close(got, want, dtype, what=""):
    tol = TOL[dtype]
    got = got.detach().cpu().double()
    want = want.double()
    assert got.shape == want.shape, (got.shape, want.shape)
    assert torch.isfinite(got).all(), f"{what}: non-finite output"
    err = (got - want).abs()
    bound = tol + tol * want.abs()
    bad = err > bound
    assert not bad.any(), (f"{what}: {int(bad.sum())} of {bad.numel()} elements outside "
                           f"atol=rtol={tol}; max err {float(err.max()):.3e}")
    return float(err.max())
