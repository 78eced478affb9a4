"""Pins the CPU restatement of the block precompute (oracle/tree_precompute.py)."""
import numpy as np
import pytest
from hypothesis import given, settings, strategies as st

from conftest import golden_cases
from fstattention_amd import trees
from oracle import tree_precompute as tp


@pytest.mark.parametrize("case", golden_cases())
def test_block_inputs_match_reference_vectors(golden, case):
    """Outputs recorded from the reference's own create_fst_attention_kernel_inputs."""
    lineage = golden[f"{case}/lineage_in"].copy()
    level = golden[f"{case}/level_lookup"]
    block_m, max_anc = (int(x) for x in golden[f"{case}/params"])
    a_idx, a_mask, l_idx = tp.block_inputs(lineage, level, block_m, max_anc)
    assert a_idx.dtype == np.int64 and l_idx.dtype == np.int64 and a_mask.dtype == np.bool_
    np.testing.assert_array_equal(a_idx, golden[f"{case}/ancestor_idx"])
    np.testing.assert_array_equal(a_mask, golden[f"{case}/ancestor_mask"])
    np.testing.assert_array_equal(l_idx, golden[f"{case}/leaf_idx"])
    # the caller's lineage now holds the self entries
    np.testing.assert_array_equal(lineage, golden[f"{case}/lineage_out"])


def test_ragged_last_block_leaves_point_past_the_tree(golden):
    case = "random100_ragged"
    l_idx = golden[f"{case}/leaf_idx"]
    # 100 nodes in blocks of 32: rows 4..31 of block 3 are pad rows and are leaves
    np.testing.assert_array_equal(l_idx[3, 4:], np.arange(100, 128))
    assert not golden[f"{case}/ancestor_mask"][3, 4:].any()


def test_no_mutation_option():
    parent = trees.random_recursive_parents(40, 3)
    lineage, level = trees.lineage_from_parents(parent)
    lin = lineage.numpy().copy()
    tp.block_inputs(lin, level.numpy(), 16, 32, mutate=False)
    np.testing.assert_array_equal(lin, lineage.numpy())


def test_too_many_ancestors_raises():
    parent = np.arange(-1, 63)  # chain of 64
    lineage, level = trees.lineage_from_parents(parent)
    with pytest.raises(RuntimeError):
        tp.block_inputs(lineage.numpy().copy(), level.numpy(), 16, 16)


parents_strategy = st.integers(2, 90).flatmap(
    lambda n: st.tuples(st.just(n), st.integers(0, 2 ** 31 - 1), st.sampled_from([None, 4, 16])))


@settings(max_examples=60, deadline=None)
@given(parents_strategy, st.sampled_from([4, 16, 32]))
def test_block_inputs_equal_bruteforce_and_rebuild_dense_mask(args, block_m):
    n, seed, window = args
    parent = trees.random_recursive_parents(n, seed, window)
    # turn a few nodes into extra roots so forests are covered too
    rng = np.random.default_rng(seed)
    parent[rng.random(n) < 0.05] = -1
    lineage, level = trees.lineage_from_parents(parent)
    max_anc = trees.required_max_ancestors(parent, block_m, 8)
    got = tp.block_inputs(lineage.numpy().copy(), level.numpy(), block_m, max_anc)
    want = tp.block_inputs_bruteforce(parent, block_m, max_anc)
    for g, w in zip(got, want):
        np.testing.assert_array_equal(g, w)
    a_idx, a_mask, l_idx = got
    # structure: ascending unique ancestors, left aligned, -1 padded
    for row in a_idx:
        valid = row[row >= 0]
        assert (np.diff(valid) > 0).all()
        assert (row[: valid.size] >= 0).all() and (row[valid.size:] == -1).all()
    # ancestors and leaves partition each block's id range
    nb = a_idx.shape[0]
    for j in range(nb):
        ids = set(range(j * block_m, (j + 1) * block_m))
        leaves = set(l_idx[j][l_idx[j] >= 0].tolist())
        anc = set(a_idx[j][a_idx[j] >= 0].tolist())
        assert leaves.isdisjoint(anc)
        assert leaves | (anc & ids) == ids
    # scattering the block tensors back gives the dense ancestor-or-self mask
    dense = tp.reconstruct_dense_mask(a_idx, a_mask, l_idx, n)
    np.testing.assert_array_equal(dense[:n, :n], tp.dense_tree_mask(parent))
    assert not dense[:n, n:].any()
    # pad rows see only themselves (through the leaf path)
    for i in range(n, nb * block_m):
        assert dense[i].sum() == 1 and dense[i, i]


def test_dense_tree_mask_is_transitive_closure():
    parent = trees.random_recursive_parents(50, 11)
    mask = tp.dense_tree_mask(parent)
    adj = np.eye(50, dtype=np.int64)
    for i, p in enumerate(parent):
        if p >= 0:
            adj[i, p] = 1
    closure = np.linalg.matrix_power(adj, 50) > 0
    np.testing.assert_array_equal(mask, closure)


def test_dense_tree_mask_matches_reference_full_mask(golden):
    for case in golden_cases():
        key = f"{case}/full_mask"
        if key not in golden.files:
            continue
        full = golden[key]
        lineage = golden[f"{case}/lineage_in"]
        level = golden[f"{case}/level_lookup"]
        parent = trees.parents_from_lineage(lineage, level)
        n = parent.shape[0]
        assert full.dtype == np.float32 and full.shape == (n + 4, n + 4)
        np.testing.assert_array_equal(full[:n, :n] != 0, tp.dense_tree_mask(parent))
        assert not full[n:].any() and not full[:, n:].any()


def test_counts():
    parent = np.array([-1, 0, 0, 1, 3])
    assert tp.attended_pairs(parent) == 1 + 2 + 2 + 3 + 4
    lineage, level = trees.lineage_from_parents(parent)
    a_idx, _, l_idx = tp.block_inputs(lineage.numpy().copy(), level.numpy(), 4, 4)
    # block 0 = {0,1,2,3}: ancestors {0,1}, leaves {2,3}; block 1 = {4}+pad: ancestors {0,1,3}, leaves 4..7
    assert tp.kv_rows_loaded(a_idx, l_idx) == (2 + 2) + (3 + 4)
