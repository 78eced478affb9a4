"""Host-side generators: lineage layout, the reference's tree, the benchmark trees."""
import numpy as np
import pytest
import torch

from conftest import golden_cases
from fstattention_amd import trees
from oracle import tree_precompute as tp


@pytest.mark.parametrize("case", [c for c in golden_cases() if c.startswith("create_tree")])
def test_create_tree_matches_reference_vectors(golden, case):
    depth, topk, lwf = golden[f"{case}/tree_args"]
    lineage, level = trees.create_tree(int(depth), int(topk), float(lwf))
    assert lineage.dtype == torch.int64 and level.dtype == torch.int64
    np.testing.assert_array_equal(lineage.numpy(), golden[f"{case}/lineage_in"])
    np.testing.assert_array_equal(level.numpy(), golden[f"{case}/level_lookup"])


@pytest.mark.parametrize("case", [c for c in golden_cases() if c.startswith("create_tree")])
def test_create_full_attention_mask_matches_reference_vectors(golden, case):
    key = f"{case}/full_mask"
    if key not in golden.files:
        pytest.skip("no mask recorded for this size")
    got = trees.create_full_attention_mask(torch.from_numpy(golden[f"{case}/lineage_in"]))
    assert got.dtype == torch.float32
    np.testing.assert_array_equal(got.numpy(), golden[key])


def test_create_tree_closed_form():
    # documented sizes: depth d -> 2**(d+3) - 4 nodes, level l holds 4 * 2**l of them
    for depth in (1, 3, 7, 8):
        lineage, level = trees.create_tree(depth)
        assert lineage.shape == (2 ** (depth + 3) - 4, depth + 1)
        counts = np.bincount(level.numpy())
        np.testing.assert_array_equal(counts, 4 * 2 ** np.arange(depth + 1))
    assert trees.DEPTH_MAPPING[2048] == 8 and trees.MAX_ANCESTOR_MAPPING[2 ** 17] == 64


def test_lineage_round_trip_and_layout():
    parent = trees.random_recursive_parents(200, 5, window=8)
    lineage, level = trees.lineage_from_parents(parent)
    assert lineage.shape[1] == int(level.max()) + 1
    assert (lineage == -1).any(dim=1).all()          # every row keeps a -1
    np.testing.assert_array_equal(trees.parents_from_lineage(lineage, level), parent)
    lin = lineage.numpy()
    for i in range(200):
        chain = []
        p = parent[i]
        while p >= 0:
            chain.append(p)
            p = parent[p]
        assert sorted(chain) == sorted(lin[i][lin[i] >= 0].tolist())
        for a in chain:
            assert lin[i, level[a]] == a


def test_lineage_of_create_tree_agrees_with_parent_walk():
    lineage, level = trees.create_tree(5)
    parent = trees.parents_from_lineage(lineage, level)
    lin2, lvl2 = trees.lineage_from_parents(parent)
    np.testing.assert_array_equal(lin2.numpy(), lineage.numpy())
    np.testing.assert_array_equal(lvl2.numpy(), level.numpy())


def test_benchmark_configs_shapes():
    sizes = {1: (64, 16), 2: (256, 64), 3: (1024, 64), 4: (4096, 64), 5: (2048, 128)}
    for i, (n, m) in sizes.items():
        cfg = trees.config(i)
        assert cfg.n_nodes == n and cfg.block_m == m
        assert cfg.parent[0] == -1 and (cfg.parent[1:] < np.arange(1, n)).all()
        assert (cfg.parent[1:] >= 0).all()
        # deterministic
        np.testing.assert_array_equal(cfg.parent, trees.config(i).parent)


def test_medusa_tree_properties():
    parent = trees.medusa_parents(256, seed=1002)
    level = trees.levels_from_parents(parent)
    assert level.max() <= 4 and (np.diff(level) >= 0).all()   # numbered by depth first
    # at most 10 children per node
    assert np.bincount(parent[1:], minlength=256).max() <= 10


def test_deep_narrow_and_wide_trees():
    p3 = trees.config(3).parent
    np.testing.assert_array_equal(p3[:129], np.arange(-1, 128))
    assert trees.levels_from_parents(p3).max() <= 128 + 32
    p4 = trees.config(4).parent
    lvl = trees.levels_from_parents(p4)
    np.testing.assert_array_equal(np.bincount(lvl), [1, 8, 64, 512, 3511])
    p5 = trees.config(5).parent
    assert ((np.arange(1, 2048) - p5[1:]) <= 64).all()


def test_make_qkv_is_seeded_on_cpu():
    cfg = trees.config(1)
    q1, k1, v1 = trees.make_qkv(cfg)
    q2, _, _ = trees.make_qkv(cfg)
    assert q1.shape == (1, 8, 64, 64) and q1.dtype == torch.float32
    assert torch.equal(q1, q2)
    q3, k3, _ = trees.make_qkv(cfg, prefix=32)
    assert k3.shape[2] == 96


# --------------------------------------------------------------------------- #
# depth-first renumbering (the reference's open item, README.md:19-20)
# --------------------------------------------------------------------------- #
def _recursive_preorder(parent, light_first):
    """Textbook recursive pre-order, children in the stated order."""
    n = len(parent)
    kids = {i: [] for i in range(-1, n)}
    for i, p in enumerate(parent):
        kids[int(p)].append(i)

    def size(x):
        return 1 + sum(size(c) for c in kids[x])

    out = []

    def visit(x):
        if x >= 0:
            out.append(x)
        order = sorted(kids[x], key=(lambda c: (size(c), c)) if light_first else (lambda c: c))
        for c in order:
            visit(c)

    visit(-1)
    return np.asarray(out, dtype=np.int64)


@pytest.mark.parametrize("children", ["index", "light_first"])
def test_dfs_order_is_the_textbook_preorder(children):
    rng = np.random.default_rng(3)
    for n in (1, 2, 7, 33, 150):
        for _ in range(4):
            parent = np.array([-1] + [int(rng.integers(-1, i)) for i in range(1, n)], dtype=np.int64)  # forests too
            perm = trees.dfs_order(parent, children)
            np.testing.assert_array_equal(perm, _recursive_preorder(parent, children == "light_first"))


def test_renumbered_tree_is_the_same_tree():
    parent = trees.random_recursive_parents(200, 9)
    perm = trees.dfs_order(parent)
    new_parent, rank = trees.renumber_parents(parent, perm)
    np.testing.assert_array_equal(rank[perm], np.arange(200))
    assert (new_parent < np.arange(200)).all()                 # still a topological numbering
    old_mask = tp.dense_tree_mask(parent)
    new_mask = tp.dense_tree_mask(new_parent)
    np.testing.assert_array_equal(new_mask, old_mask[np.ix_(perm, perm)])
    # a depth-first numbered tree is a fixed point
    np.testing.assert_array_equal(trees.dfs_order(new_parent), np.arange(200))
    # in pre-order every subtree is a run of consecutive ids
    size = trees.subtree_sizes(new_parent)
    for i in range(200):
        assert new_mask[i + 1:i + size[i], i].all() and not new_mask[i + size[i]:, i].any()


def test_dfs_order_shrinks_the_ancestor_lists_of_the_benchmark_trees():
    for index, at_most in ((2, 0.75), (5, 0.60)):
        cfg = trees.config(index)
        rows = {}
        for name, parent in (("given", cfg.parent),
                             ("dfs", trees.renumber_parents(cfg.parent, trees.dfs_order(cfg.parent))[0])):
            lineage, level = trees.lineage_from_parents(parent)
            max_anc = trees.required_max_ancestors(parent, cfg.block_m)
            a_idx, _, l_idx = tp.block_inputs(lineage.numpy().copy(), level.numpy(), cfg.block_m, max_anc)
            rows[name] = tp.kv_rows_loaded(a_idx, l_idx)
        assert rows["dfs"] <= at_most * rows["given"], rows


def test_renumber_rejects_bad_orders():
    parent = np.array([-1, 0, 1, 1], dtype=np.int64)
    with pytest.raises(ValueError):
        trees.renumber_parents(parent, np.array([0, 1, 1, 3]))
    with pytest.raises(ValueError):
        trees.renumber_parents(parent, np.array([1, 0, 2, 3]))   # child before parent
    with pytest.raises(ValueError):
        trees.dfs_order(parent, children="random")


def test_medusa_builder_split_keeps_the_benchmark_tree():
    probs = trees.medusa_probs(4, 10, 0.3, 1002)
    assert probs.shape == (4, 10) and (np.diff(probs, axis=1) <= 0).all()
    np.testing.assert_allclose(probs.sum(axis=1), 1.0)
    np.testing.assert_array_equal(trees.medusa_parents_from_probs(probs, 256), trees.config(2).parent)
