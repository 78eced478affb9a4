"""Pins the dense-masked attention oracle (oracle/dense_attention.py)."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from fstattention_amd import trees
from oracle import dense_attention as da
from oracle import tree_precompute as tp


def _rand(shape, seed, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g, dtype=torch.float32).to(dtype)


def test_against_library_sdpa():
    parent = trees.random_recursive_parents(48, 21)
    mask = tp.dense_tree_mask(parent)
    q, k, v = (_rand((2, 3, 48, 32), s, torch.float64) for s in (1, 2, 3))
    scale = 0.37
    o, _ = da.dense_tree_attention(q, k, v, mask, scale)
    want = F.scaled_dot_product_attention(q, k, v, attn_mask=torch.from_numpy(mask), scale=scale)
    torch.testing.assert_close(o, want, atol=1e-12, rtol=1e-12)


def test_chain_tree_is_causal_attention():
    n = 40
    parent = np.arange(-1, n - 1)
    mask = tp.dense_tree_mask(parent)
    q, k, v = (_rand((1, 2, n, 16), s, torch.float64) for s in (4, 5, 6))
    o, _ = da.dense_tree_attention(q, k, v, mask, 0.25)
    want = F.scaled_dot_product_attention(q, k, v, is_causal=True, scale=0.25)
    torch.testing.assert_close(o, want, atol=1e-12, rtol=1e-12)


def test_prefix_mask_against_sdpa():
    parent = trees.random_recursive_parents(24, 2)
    mask = da.full_mask_with_prefix(tp.dense_tree_mask(parent), 16)
    assert mask.shape == (24, 40) and mask[:, :16].all()
    q = _rand((1, 2, 24, 16), 7, torch.float64)
    k, v = (_rand((1, 2, 40, 16), s, torch.float64) for s in (8, 9))
    o, _ = da.dense_tree_attention(q, k, v, mask, 0.5)
    want = F.scaled_dot_product_attention(q, k, v, attn_mask=torch.from_numpy(mask), scale=0.5)
    torch.testing.assert_close(o, want, atol=1e-12, rtol=1e-12)


def test_roots_return_their_own_value_row():
    parent = np.array([-1, -1, 0, 1, -1, 2])
    mask = tp.dense_tree_mask(parent)
    q, k, v = (_rand((1, 1, 6, 8), s) for s in (1, 2, 3))
    o, lse = da.dense_tree_attention(q, k, v, mask, 1.0, dtype=torch.float32)
    for r in (0, 1, 4):
        torch.testing.assert_close(o[0, 0, r], v[0, 0, r], atol=0, rtol=0)
        # one key: lse2 is that score in base-2 units
        s = float((q[0, 0, r] * k[0, 0, r]).sum()) * 1.4426950408889634
        assert abs(float(lse[0, 0, r]) - s) < 1e-5


def test_equal_keys_give_plain_mean_of_allowed_values():
    parent = trees.random_recursive_parents(30, 13)
    mask = tp.dense_tree_mask(parent)
    q = _rand((1, 2, 30, 8), 1, torch.float64)
    k = _rand((1, 2, 1, 8), 2, torch.float64).expand(1, 2, 30, 8).contiguous()
    v = _rand((1, 2, 30, 8), 3, torch.float64)
    o, _ = da.dense_tree_attention(q, k, v, mask, 0.7)
    m = torch.from_numpy(mask).double()
    want = (m @ v) / m.sum(-1, keepdim=True)
    torch.testing.assert_close(o, want, atol=1e-12, rtol=1e-12)


@pytest.mark.parametrize("prefix", [0, 5])
def test_scalar_double_loop(prefix):
    parent = trees.random_recursive_parents(12, 17)
    mask = da.full_mask_with_prefix(tp.dense_tree_mask(parent), prefix)
    q = _rand((1, 1, 12, 4), 1, torch.float64)
    k, v = (_rand((1, 1, 12 + prefix, 4), s, torch.float64) for s in (2, 3))
    o, _ = da.dense_tree_attention(q, k, v, mask, 0.9)
    want = da.scalar_tree_attention(q[0, 0].numpy(), k[0, 0].numpy(), v[0, 0].numpy(),
                                    parent, 0.9, prefix)
    np.testing.assert_allclose(o[0, 0].numpy(), want, atol=1e-12, rtol=1e-12)


def test_lse_is_base2_logsumexp_of_scaled_scores():
    parent = trees.random_recursive_parents(20, 19)
    mask = tp.dense_tree_mask(parent)
    q, k, v = (_rand((1, 2, 20, 8), s, torch.float64) for s in (1, 2, 3))
    scale = 0.3
    _, lse = da.dense_tree_attention(q, k, v, mask, scale)
    scores = (q @ k.transpose(-1, -2)) * scale
    scores = scores.masked_fill(~torch.from_numpy(mask), float("-inf"))
    torch.testing.assert_close(lse, torch.logsumexp(scores, -1) / math.log(2), atol=1e-12, rtol=1e-12)
    torch.testing.assert_close(da.lse_base2(scores), lse, atol=1e-12, rtol=1e-12)


def test_empty_rows_give_zero():
    mask = np.zeros((3, 3), dtype=bool)
    mask[0, 0] = True
    q, k, v = (_rand((1, 1, 3, 4), s) for s in (1, 2, 3))
    o, lse = da.dense_tree_attention(q, k, v, mask, 1.0)
    assert torch.equal(o[0, 0, 1:], torch.zeros(2, 4, dtype=o.dtype))
    assert torch.isinf(lse[0, 0, 1:]).all()


def test_low_precision_inputs_are_upcast_not_rerounded():
    parent = trees.random_recursive_parents(16, 23)
    mask = tp.dense_tree_mask(parent)
    q, k, v = (_rand((1, 1, 16, 8), s, torch.bfloat16) for s in (1, 2, 3))
    o, _ = da.dense_tree_attention(q, k, v, mask, 0.35)
    o64, _ = da.dense_tree_attention(q.double(), k.double(), v.double(), mask, 0.35)
    assert o.dtype == torch.float64
    torch.testing.assert_close(o, o64, atol=0, rtol=0)
