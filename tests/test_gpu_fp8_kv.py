"""8-bit K/V storage (float8_e4m3fn rows + one scale per (batch, head) slice) against the dense oracle.

The oracle is the dense-masked attention on the DEQUANTISED keys and values (``k8 * k_scale``,
``v8 * v_scale``, formed in float64 on the host): the kernel widens the stored bytes exactly, so the
tolerance is the one of the 16-bit kernels (2e-3, asserted on the float32 output).
"""
import math

import numpy as np
import pytest
import torch

from fstattention_amd import fst_attention, quantize_kv_fp8, shift_for_prefix, trees
from helpers import assert_close, dense_oracle, oracle_inputs, rand_qkv

pytestmark = pytest.mark.gpu


def run_fp8(parent, block_m, z, h, d, dtype, seed, prefix=0, scales=True, spread=1.0):
    n = len(parent)
    a_idx, a_mask, l_idx, max_anc = oracle_inputs(parent, block_m)
    nq = a_idx.shape[0] * block_m
    q, k, v = rand_qkv(z, h, nq, nq + prefix, d, dtype, seed)
    if spread != 1.0:      # slices of very different magnitude: the per-slice scales must be honoured
        factor = torch.logspace(0, math.log10(spread), z * h).view(z, h, 1, 1)
        k, v = (k.float() * factor).to(dtype), (v.float() / factor).to(dtype)
    k8, v8, k_scale, v_scale = quantize_kv_fp8(k, v)
    if not scales:         # N(0,1) values rounded to the 8-bit format and used as they are
        k_scale = v_scale = None
        k8, v8 = k.to(torch.float8_e4m3fn), v.to(torch.float8_e4m3fn)
        k_deq, v_deq = k8.double(), v8.double()
    else:
        k_deq = k8.double() * k_scale.double().view(z, h, 1, 1)
        v_deq = v8.double() * v_scale.double().view(z, h, 1, 1)
    scale = 1.0 / math.sqrt(d)
    want, want_lse = dense_oracle(q.double(), k_deq, v_deq, parent, scale, prefix=prefix, nq_pad=nq - n)
    if prefix:
        a_idx, l_idx = shift_for_prefix(a_idx, l_idx, prefix)
    dev = lambda t: None if t is None else t.cuda()
    o, lse = fst_attention(q.cuda(), k8.cuda(), v8.cuda(), a_idx.cuda(), a_mask.cuda(), l_idx.cuda(), scale,
                           BLOCK_M=block_m, MAX_ANCESTORS=max_anc, out_dtype=torch.float32, return_lse=True,
                           k_scale=dev(k_scale), v_scale=dev(v_scale))
    assert_close(o, want, dtype, f"fp8 K/V n={n} m={block_m} d={d} {dtype} prefix={prefix}")
    torch.testing.assert_close(lse.cpu().double().view(z, h, nq), want_lse, atol=2e-3, rtol=2e-3)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("block_m", [32, 64, 128])
def test_shapes(block_m, d, dtype):
    parent = trees.random_recursive_parents(300, 40 + block_m + d, window=48)      # ragged last block
    run_fp8(parent, block_m, 2, 3, d, dtype, 7)


@pytest.mark.parametrize("index", [2, 3, 4])
def test_benchmark_trees_full_size(index):
    cfg = trees.config(index)
    run_fp8(cfg.parent, cfg.block_m, cfg.batch, cfg.heads, cfg.head_dim, torch.bfloat16, cfg.tensor_seed)


def test_config5_head_subset():
    cfg = trees.config(5)
    run_fp8(cfg.parent, cfg.block_m, 2, 4, cfg.head_dim, torch.bfloat16, cfg.tensor_seed)


@pytest.mark.parametrize("prefix", [100, 64, 7])
def test_shared_prefix(prefix):
    parent = trees.random_recursive_parents(200, 3, window=32)
    run_fp8(parent, 64, 1, 4, 128, torch.bfloat16, 9, prefix=prefix)


def test_per_slice_scales_and_no_scales():
    parent = trees.medusa_parents(n=256, seed=77)
    run_fp8(parent, 64, 2, 4, 128, torch.bfloat16, 11, spread=64.0)
    run_fp8(parent, 64, 2, 4, 64, torch.float16, 12, scales=False)


def test_short_and_single_tile_lists():
    bushy = np.maximum((np.arange(90) - 1) // 3, -1).astype(np.int64)
    bushy[0] = -1
    run_fp8(bushy, 32, 1, 2, 128, torch.bfloat16, 13)
    run_fp8(np.full(40, -1, dtype=np.int64), 32, 1, 2, 64, torch.bfloat16, 14)       # roots only: no ancestor tile


def test_argument_errors():
    parent = trees.random_recursive_parents(64, 5)
    a_idx, a_mask, l_idx, max_anc = oracle_inputs(parent, 32)
    q, k, v = rand_qkv(1, 2, 64, 64, 64, torch.bfloat16, 1)
    k8, v8, ks, vs = quantize_kv_fp8(k, v)
    dev = [t.cuda() for t in (q, k8, v8, a_idx, a_mask, l_idx)]
    with pytest.raises(ValueError):      # scales without 8-bit storage
        fst_attention(q.cuda(), k.cuda(), v.cuda(), *dev[3:], 0.1, BLOCK_M=32, MAX_ANCESTORS=max_anc, k_scale=ks.cuda())
    with pytest.raises(ValueError):      # mixed storage
        fst_attention(dev[0], dev[1], v.cuda(), *dev[3:], 0.1, BLOCK_M=32, MAX_ANCESTORS=max_anc)
    with pytest.raises(ValueError):      # float32 queries
        fst_attention(q.float().cuda(), dev[1], dev[2], *dev[3:], 0.1, BLOCK_M=32, MAX_ANCESTORS=max_anc)
    with pytest.raises(ValueError):      # wrong number of scales
        fst_attention(*dev, 0.1, BLOCK_M=32, MAX_ANCESTORS=max_anc, k_scale=ks[:1].cuda())
    with pytest.raises(ValueError):      # no kernel choice
        fst_attention(*dev, 0.1, BLOCK_M=32, MAX_ANCESTORS=max_anc, generic=True)
