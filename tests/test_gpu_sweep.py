"""Seeded random sweeps over shapes, types, trees and prefixes: the attention entry point against the
float64 dense oracle, the integer front-end against the oracle and the host builders (bit-exact)."""
import math
import random

import numpy as np
import pytest
import torch

from fstattention_amd import (create_fst_attention_kernel_inputs, dfs_order_gpu, fst_attention, kernel_inputs_from_parents_gpu,
                              lineage_from_parents_gpu, pack_tree_mask, renumber_parents_gpu, shift_for_prefix, trees)
from fstattention_amd import _lib
from fstattention_amd.attention import recall_packed
from helpers import TOL, dense_oracle, expected_plan, rand_qkv
from oracle import tree_precompute as tp

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("sweep_seed", [11, 12])
def test_attention_sweep_against_dense_oracle(sweep_seed):
    """Every kernel choice the launcher can make is reached by some case: head dims 16..128, all three types,
    block sizes 16..128, trees of 1..1200 nodes (chains, bushes, windows), prefixes up to the dense kernel's
    range, several (batch, head) counts, three softmax scales; O and the log-sum-exp are checked."""
    rnd = random.Random(sweep_seed)
    for case in range(60):
        dtype = rnd.choice([torch.bfloat16, torch.float16, torch.float32])
        d = rnd.choice([32, 64, 128]) if dtype != torch.float32 else rnd.choice([16, 32, 64, 128])
        m = rnd.choice([16, 32, 64, 128])
        n = rnd.choice([rnd.randint(1, 40), rnd.randint(40, 300), rnd.randint(300, 1200)])
        window = rnd.choice([None, 3, 16, 64])
        prefix = rnd.choice([0, 0, rnd.randint(1, 100), rnd.randint(100, 3000), rnd.choice([2048, 4096])])
        z, h = rnd.choice([(1, 1), (1, 3), (2, 2), (1, 8), (1, 9)])
        seed = rnd.randint(0, 10 ** 6)
        parent = trees.random_recursive_parents(n, seed, window)
        lineage, level = trees.lineage_from_parents(parent)
        max_anc = trees.required_max_ancestors(parent, m, rnd.choice([1, 16, 32]))
        what = f"case {case}: {dtype} d{d} m{m} n{n} window {window} prefix {prefix} z{z} h{h} seed {seed} A{max_anc}"
        a_idx, a_mask, l_idx = create_fst_attention_kernel_inputs(lineage.cuda(), level.cuda(), m, max_anc)
        q, k, v = rand_qkv(z, h, n, n + prefix, d, dtype, seed)
        scale = rnd.choice([1.0 / math.sqrt(d), 0.5, 2.0 / math.sqrt(d)])
        want, want_lse = dense_oracle(q, k, v, parent, scale, prefix)
        if prefix:
            a_idx, l_idx = shift_for_prefix(a_idx, l_idx, prefix)
        o, lse = fst_attention(q.cuda(), k.cuda(), v.cuda(), a_idx, a_mask, l_idx, scale, BLOCK_M=m,
                               MAX_ANCESTORS=max_anc, out_dtype=torch.float32, return_lse=True)
        assert torch.isfinite(o).all(), what
        err = (o.cpu().double() - want.double()).abs()
        bound = TOL[dtype] + TOL[dtype] * want.double().abs()       # 2e-3 / 2e-3 (1e-5 for float32)
        assert bool((err <= bound).all()), f"{what}: max err {float(err.max()):.3e}"
        lse_err = (lse.cpu().double().reshape(want_lse.shape) - want_lse.double()).abs().max()
        assert float(lse_err) < 1e-2, f"{what}: log-sum-exp off by {float(lse_err):.3e}"


def test_integer_front_end_sweep_is_bit_exact():
    """parent[] -> lineage, block inputs (with the in-place self insert), block plan, depth-first order in both
    child orders and the renumbered parents, on random forests of 1..5000 nodes and every block size."""
    rnd = random.Random(21)
    for case in range(30):
        m = rnd.choice([16, 32, 64, 128])
        n = rnd.choice([rnd.randint(1, 50), rnd.randint(50, 600), rnd.randint(600, 5000)])
        window = rnd.choice([None, 1, 3, 16, 64, 500])
        seed = rnd.randint(0, 10 ** 6)
        what = f"case {case}: m{m} n{n} window {window} seed {seed}"
        parent = trees.random_recursive_parents(n, seed, window)
        lineage, level = trees.lineage_from_parents(parent)
        pt = torch.as_tensor(np.asarray(parent), dtype=torch.int64).cuda()
        lin_d, lvl_d = lineage_from_parents_gpu(pt)
        assert torch.equal(lin_d.cpu(), lineage) and torch.equal(lvl_d.cpu(), level), what
        max_anc = trees.required_max_ancestors(parent, m, rnd.choice([1, 16, 32]))
        lin_host = lineage.numpy().copy()
        want = tp.block_inputs(lin_host, level.numpy(), m, max_anc)
        lin_dev = lineage.clone().cuda()
        got = create_fst_attention_kernel_inputs(lin_dev, level.cuda(), m, max_anc)
        for g_, w_ in zip(got, want):
            np.testing.assert_array_equal(g_.cpu().numpy(), w_, err_msg=what)
        np.testing.assert_array_equal(lin_dev.cpu().numpy(), lin_host, err_msg=what)     # utils.py:124-125
        # the same from the parent array in one launch (lineage rows built in LDS)
        packed = pack_tree_mask(got[0], got[1], got[2])
        fits = 4 * (2 * ((n + 31) // 32) + (max_anc + 31) // 32 * m + m + 4 + m * lineage.shape[1] + n) <= 160 * 1024
        if fits:
            fa, fm, fl, flin, flvl = kernel_inputs_from_parents_gpu(pt, m, max_anc, lineage.shape[1], want_bool_mask=True,
                                                                    want_lineage=True)
            for g_, w_ in zip((fa, fm, fl), want):
                np.testing.assert_array_equal(g_.cpu().numpy(), w_, err_msg="one launch, " + what)
            np.testing.assert_array_equal(flin.cpu().numpy(), lin_host, err_msg="one launch, " + what)
            np.testing.assert_array_equal(flvl.cpu().numpy(), level.numpy(), err_msg="one launch, " + what)
            fused_packed = recall_packed(fm)[1]
            np.testing.assert_array_equal(fused_packed.mask_bits.cpu().numpy(), packed.mask_bits.cpu().numpy(), err_msg=what)
            np.testing.assert_array_equal(fused_packed.anc_count.cpu().numpy(), packed.anc_count.cpu().numpy(), err_msg=what)
            if m >= 32:
                plan_want, care = expected_plan(*want)
                plan_fused = fused_packed.plan.cpu().numpy().view(np.uint32).reshape(plan_want.shape[0], -1)
                np.testing.assert_array_equal(plan_fused[care], plan_want[care], err_msg="one launch, " + what)
        else:       # tables beyond one workgroup's LDS: refused on the host
            with pytest.raises(_lib.FstaError, match="LDS"):
                kernel_inputs_from_parents_gpu(pt, m, max_anc, lineage.shape[1])
        if m >= 32:
            plan_want, care = expected_plan(*want)
            plan_got = packed.plan.cpu().numpy().view(np.uint32).reshape(plan_want.shape[0], -1)
            np.testing.assert_array_equal(plan_got[care], plan_want[care], err_msg=what)
        else:
            assert packed.plan is None, what        # blocks of 16 rows go to the scalar kernel, which reads the lists
        for children in ("index", "light_first"):
            perm_host = trees.dfs_order(parent, children)
            perm, rank = dfs_order_gpu(pt, children)
            np.testing.assert_array_equal(perm.cpu().numpy(), np.asarray(perm_host), err_msg=what)
            new_parent, rank_host = trees.renumber_parents(parent, perm_host)
            np.testing.assert_array_equal(rank.cpu().numpy(), np.asarray(rank_host), err_msg=what)
            np.testing.assert_array_equal(renumber_parents_gpu(pt, perm, rank).cpu().numpy(), np.asarray(new_parent),
                                          err_msg=what)
