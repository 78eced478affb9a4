"""GPU parity of the streaming kernel (workgroups that stay and walk a list of query blocks) against the
dense-masked float64 oracle, and bit for bit against the kernel with one workgroup per block on the sizes it
is made for.  Same tolerances as the other attention tests: 2e-3 (float16 / bfloat16) on the float32 output."""
import math

import numpy as np
import pytest
import torch

from fstattention_amd import _lib, create_fst_attention_kernel_inputs, fst_attention, trees
from test_gpu_attention import run_tree, sampled_rows_check

pytestmark = pytest.mark.gpu

STREAM = "attn_stream_kernel"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("block_m", [64, 128])
def test_forced_on_small_trees(block_m, d, dtype):
    """Few blocks and slices: most workgroups get one pair or none, some XCDs no slice at all."""
    parent = trees.random_recursive_parents(700, 11 + d + block_m, window=40)
    run_tree(parent, block_m, 1, 3, d, dtype, 5, stream_blocks=True, native_out=True, want_kernel=STREAM)


@pytest.mark.parametrize("n, window, block_m, z, h", [
    (1, None, 128, 1, 1),            # a single node
    (129, 4, 128, 2, 5),             # ragged last block, deep chains: many ancestor tiles
    (2048, 64, 128, 2, 9),           # configuration 5's tree, 18 slices
    (1500, None, 64, 1, 16),         # shallow random tree, block of 64
    (900, 2, 64, 3, 4),              # nearly a chain: ancestor lists grow with the block number
])
def test_forced_shapes_against_oracle(n, window, block_m, z, h):
    parent = trees.random_recursive_parents(n, 100 + n, window=window)
    run_tree(parent, block_m, z, h, 128, torch.bfloat16, 9, stream_blocks=True, want_kernel=STREAM)


def test_forest_with_empty_leaf_slots_and_rows_without_ancestors():
    """Roots (no ancestors: the leaf key is the only key), inner nodes (no leaf key: the node itself comes through the
    ancestor list) and a float32 output."""
    parent = trees.random_recursive_parents(600, 3, window=16)
    parent[::37] = -1                     # more roots
    run_tree(parent, 128, 1, 8, 64, torch.float16, 21, stream_blocks=True, native_out=True, want_kernel=STREAM)


def test_long_lists_per_workgroup():
    """Many more pairs than workgroups (what the kernel is for): every workgroup walks a list of a dozen pairs; whole
    result compared with the kernel that gives every pair a workgroup of its own (the library's own choice)."""
    cfg = trees.config(5)
    m, d, n = cfg.block_m, cfg.head_dim, cfg.n_nodes
    lineage, level = trees.lineage_from_parents(cfg.parent)
    max_anc = trees.required_max_ancestors(cfg.parent, m, 16)
    inputs = create_fst_attention_kernel_inputs(lineage.cuda(), level.cuda(), m, max_anc)
    z, h = 8, 48
    g = torch.Generator(device="cuda").manual_seed(31)
    q, k, v = (torch.randn((z, h, n, d), generator=g, device="cuda", dtype=torch.float32).to(torch.bfloat16) for _ in range(3))
    scale = 1.0 / math.sqrt(d)
    o, lse = fst_attention(q, k, v, *inputs, scale, BLOCK_M=m, MAX_ANCESTORS=max_anc, out_dtype=torch.float32, return_lse=True,
                           stream_blocks=True)
    assert STREAM in _lib.load().fsta_last_attention_kernel().decode()
    o2, lse2 = fst_attention(q, k, v, *inputs, scale, BLOCK_M=m, MAX_ANCESTORS=max_anc, out_dtype=torch.float32,
                             return_lse=True)
    assert STREAM not in _lib.load().fsta_last_attention_kernel().decode()
    assert bool(torch.isfinite(o).all())
    # the two kernels take a row's keys in different orders: equal up to float32 rounding of the sums
    torch.testing.assert_close(o, o2, atol=2e-5, rtol=2e-5)
    torch.testing.assert_close(lse, lse2, atol=2e-5, rtol=2e-5)
    sampled_rows_check(q, k, v, cfg.parent, o, lse, scale, 0, 64, 77, torch.bfloat16, "cfg5 streaming")
    # and in the type of q
    o3 = fst_attention(q, k, v, *inputs, scale, BLOCK_M=m, MAX_ANCESTORS=max_anc, stream_blocks=True)
    torch.testing.assert_close(o3.float(), o.to(torch.bfloat16).float(), atol=0, rtol=2 ** -7)


def test_reference_benchmark_shape_fp16():
    """The reference's own benchmark workload (fstattention.py:240-296: batch 4, 48 heads, head dim 64, float16, blocks of
    128 rows, 64 ancestor slots) at N = 4096: short lists (at most two ancestor tiles), plans requested two pairs ahead."""
    cfg = trees.reference_benchmark_config(4096)
    m, d, n = cfg.block_m, cfg.head_dim, cfg.n_nodes + cfg.pad_rows
    lineage, level = trees.lineage_from_parents(cfg.parent)
    inputs = create_fst_attention_kernel_inputs(lineage.cuda(), level.cuda(), m, cfg.max_ancestors)
    g = torch.Generator(device="cuda").manual_seed(41)
    q, k, v = (torch.randn((cfg.batch, cfg.heads, n, d), generator=g, device="cuda", dtype=torch.float32).to(torch.float16)
               for _ in range(3))
    scale = 1.0 / math.sqrt(d)
    o, lse = fst_attention(q, k, v, *inputs, scale, BLOCK_M=m, MAX_ANCESTORS=cfg.max_ancestors, out_dtype=torch.float32,
                           return_lse=True, stream_blocks=True)
    assert STREAM in _lib.load().fsta_last_attention_kernel().decode()
    o2, lse2 = fst_attention(q, k, v, *inputs, scale, BLOCK_M=m, MAX_ANCESTORS=cfg.max_ancestors, out_dtype=torch.float32,
                             return_lse=True)
    # (float16 weights go to the matrix cores as single values, rounded relative to running maxima that differ with the
    # order of the keys: the two kernels agree to the tolerance of the type, not to float32 rounding)
    torch.testing.assert_close(o[:, :, :cfg.n_nodes], o2[:, :, :cfg.n_nodes], atol=2e-3, rtol=2e-3)
    torch.testing.assert_close(lse.view(cfg.batch, cfg.heads, n)[:, :, :cfg.n_nodes],
                               lse2.view(cfg.batch, cfg.heads, n)[:, :, :cfg.n_nodes], atol=2e-5, rtol=2e-5)
    sampled_rows_check(q, k, v, cfg.parent, o, lse, scale, 0, 64, 78, torch.float16, "reference benchmark streaming")
