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


def expected_plan(a_idx, a_mask, l_idx, key_limit=None):
    """The block plan (layout of include/fsta.h) of three index tensors (numpy), written from
    their definition: (words uint32 [NB, block_words], care bool of the same shape).  `care` is
    False on the keys of empty slots, which may repeat any row."""
    nb, m, a = a_mask.shape
    tiles, groups = (a + 31) // 32, m // 32
    common = 8 + 32 * tiles
    group = 32 * (1 + tiles)
    words = np.zeros((nb, common + groups * group), dtype=np.uint32)
    care = np.ones(words.shape, dtype=bool)
    limit = 2 ** 31 - 1 if key_limit is None else key_limit
    for j in range(nb):
        valid_a = (a_idx[j] >= 0) & (a_idx[j] < limit)
        words[j, 0] = np.flatnonzero(a_idx[j] >= 0).max(initial=-1) + 1
        for c in range(32 * tiles):
            if c < a and valid_a[c]:
                words[j, 8 + c] = a_idx[j, c]
            else:
                care[j, 8 + c] = False
        for r in range(m):
            g, r5 = divmod(r, 32)
            base = common + g * group
            ok = 0 <= l_idx[j, r] < limit
            if ok:
                words[j, base + r5] = l_idx[j, r]
                words[j, 4 + g] |= np.uint32(1 << r5)
            else:
                care[j, base + r5] = False
            for c in range(a):
                if a_mask[j, r, c] and valid_a[c]:
                    words[j, base + 32 + (c // 32) * 32 + r5] |= np.uint32(1 << (c % 32))
    return words, care
