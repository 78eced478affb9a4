"""GPU parity of the integer precompute kernels (bit-exact), through the C ABI."""
import numpy as np
import pytest
import torch

from conftest import golden_cases
from fstattention_amd import (create_fst_attention_kernel_inputs, dfs_order_gpu, kernel_inputs_from_parents_gpu,
                              lineage_from_parents_gpu,
                              medusa_parents_gpu, pack_tree_mask, renumber_parents_gpu, trees)
from fstattention_amd.attention import recall_packed
from oracle import tree_precompute as tp

pytestmark = pytest.mark.gpu


def _check(got, want):
    a_idx, a_mask, l_idx = got
    assert a_idx.dtype == torch.int64 and l_idx.dtype == torch.int64 and a_mask.dtype == torch.bool
    np.testing.assert_array_equal(a_idx.cpu().numpy(), want[0])
    np.testing.assert_array_equal(a_mask.cpu().numpy(), want[1])
    np.testing.assert_array_equal(l_idx.cpu().numpy(), want[2])


@pytest.mark.parametrize("case", golden_cases())
def test_reference_vectors_device_tensors(golden, case):
    lineage = torch.from_numpy(golden[f"{case}/lineage_in"].copy()).cuda()
    level = torch.from_numpy(golden[f"{case}/level_lookup"]).cuda()
    block_m, max_anc = (int(x) for x in golden[f"{case}/params"])
    got = create_fst_attention_kernel_inputs(lineage, level, block_m, max_anc)
    assert all(t.is_cuda for t in got)
    _check(got, [golden[f"{case}/{k}"] for k in ("ancestor_idx", "ancestor_mask", "leaf_idx")])
    np.testing.assert_array_equal(lineage.cpu().numpy(), golden[f"{case}/lineage_out"])


def test_reference_vectors_host_tensors_round_trip(golden):
    case = "create_tree_d5_k4_f0.5_m64_a32"
    lineage = torch.from_numpy(golden[f"{case}/lineage_in"].copy())
    level = torch.from_numpy(golden[f"{case}/level_lookup"])
    got = create_fst_attention_kernel_inputs(lineage, level, 64, 32)
    assert not any(t.is_cuda for t in got)
    _check(got, [golden[f"{case}/{k}"] for k in ("ancestor_idx", "ancestor_mask", "leaf_idx")])
    np.testing.assert_array_equal(lineage.numpy(), golden[f"{case}/lineage_out"])
    # second flavour: leave the caller's lineage alone
    lineage2 = torch.from_numpy(golden[f"{case}/lineage_in"].copy())
    create_fst_attention_kernel_inputs(lineage2, level, 64, 32, mutate_lineage=False)
    np.testing.assert_array_equal(lineage2.numpy(), golden[f"{case}/lineage_in"])


@pytest.mark.parametrize("seed", range(12))
def test_random_trees_against_oracle(seed):
    rng = np.random.default_rng(seed)
    n = int(rng.integers(1, 700))
    window = [None, 4, 32][seed % 3]
    block_m = [16, 64, 128, 8][seed % 4]
    parent = trees.random_recursive_parents(n, seed, window)
    parent[rng.random(n) < 0.03] = -1
    lineage, level = trees.lineage_from_parents(parent)
    max_anc = trees.required_max_ancestors(parent, block_m, [1, 16, 7][seed % 3])
    lin_cpu = lineage.numpy().copy()
    want = tp.block_inputs(lin_cpu, level.numpy(), block_m, max_anc)
    lin_gpu = lineage.clone().cuda()
    got = create_fst_attention_kernel_inputs(lin_gpu, level.cuda(), block_m, max_anc)
    _check(got, want)
    np.testing.assert_array_equal(lin_gpu.cpu().numpy(), lin_cpu)


@pytest.mark.parametrize("index", [3, 4, 5])
def test_benchmark_trees_full_size(index):
    cfg = trees.config(index)
    lineage, level = trees.lineage_from_parents(cfg.parent)
    max_anc = trees.required_max_ancestors(cfg.parent, cfg.block_m, 16)
    want = tp.block_inputs(lineage.numpy().copy(), level.numpy(), cfg.block_m, max_anc)
    got = create_fst_attention_kernel_inputs(lineage.cuda(), level.cuda(), cfg.block_m, max_anc)
    _check(got, want)
    # size-independent property: the three tensors rebuild the dense ancestor-or-self mask
    dense = tp.reconstruct_dense_mask(got[0].cpu().numpy(), got[1].cpu().numpy(),
                                      got[2].cpu().numpy(), cfg.n_nodes)
    np.testing.assert_array_equal(dense[:, :cfg.n_nodes], tp.dense_tree_mask(cfg.parent))


def test_reference_benchmark_tree_largest():
    # the reference's largest table entry: 2**17 tokens, depth 14, blocks of 128, 64 ancestors
    lineage, level = trees.create_tree(14)
    want = tp.block_inputs(lineage.numpy().copy(), level.numpy(), 128, 64)
    got = create_fst_attention_kernel_inputs(lineage.cuda(), level.cuda(), 128, 64)
    _check(got, want)


def test_too_many_ancestors_raises_like_the_reference():
    parent = np.arange(-1, 63)
    lineage, level = trees.lineage_from_parents(parent)
    with pytest.raises(RuntimeError):
        create_fst_attention_kernel_inputs(lineage.cuda(), level.cuda(), 16, 16)
    out = create_fst_attention_kernel_inputs(lineage.cuda(), level.cuda(), 16, 16, check=False)
    assert int(out[3].item()) & 1


def test_bad_inputs_are_flagged():
    lineage, level = trees.lineage_from_parents(np.array([-1, 0, 1, 1]))
    bad = lineage.clone()
    bad[3, 0] = 9
    with pytest.raises(ValueError):
        create_fst_attention_kernel_inputs(bad.cuda(), level.cuda(), 4, 4)
    with pytest.raises(IndexError):
        create_fst_attention_kernel_inputs(lineage.cuda(), (level + 7).cuda(), 4, 4)
    with pytest.raises(ValueError):
        create_fst_attention_kernel_inputs(lineage.int().cuda(), level.cuda(), 4, 4)


def test_block_without_padding_drops_smallest_id():
    # every row of the block is full: the reference's `[1:]` then drops the smallest node id
    lineage = torch.tensor([[0, 1], [0, 1]], dtype=torch.int64)
    level = torch.tensor([1, 1], dtype=torch.int64)
    want = tp.block_inputs(lineage.numpy().copy(), level.numpy(), 2, 4)
    got = create_fst_attention_kernel_inputs(lineage.cuda(), level.cuda(), 2, 4)
    _check(got, want)


def test_packed_mask_matches_bool_mask():
    parent = trees.random_recursive_parents(500, 42, window=40)
    lineage, level = trees.lineage_from_parents(parent)
    max_anc = trees.required_max_ancestors(parent, 64, 1)
    a_idx, a_mask, l_idx = create_fst_attention_kernel_inputs(lineage.cuda(), level.cuda(), 64, max_anc)
    from_precompute = recall_packed(a_mask)[1]
    repacked = pack_tree_mask(a_idx, a_mask)
    assert torch.equal(from_precompute.mask_bits, repacked.mask_bits)
    assert torch.equal(from_precompute.anc_count, repacked.anc_count)
    bits = repacked.mask_bits.cpu().numpy().astype(np.uint32)   # [nb, words, m]
    mask = a_mask.cpu().numpy()
    for c in range(max_anc):
        np.testing.assert_array_equal((bits[:, c // 32, :] >> (c % 32)) & 1, mask[:, :, c])
    np.testing.assert_array_equal(repacked.anc_count.cpu().numpy(), (a_idx.cpu().numpy() >= 0).sum(1))


@pytest.mark.parametrize("block_m,n,window", [(32, 200, 16), (64, 500, 40), (128, 1000, 64), (64, 70, None), (128, 100, 3)])
def test_block_plan_matches_the_lists(block_m, n, window):
    """The kernel-ready record the precompute writes beside the three reference tensors (and the one
    the packing entry point makes from them) holds exactly what they say; empty slots may repeat any
    K/V row that exists, their mask bits are clear."""
    from helpers import expected_plan
    parent = trees.random_recursive_parents(n, 11 + n, window)
    lineage, level = trees.lineage_from_parents(parent)
    max_anc = trees.required_max_ancestors(parent, block_m, 16)
    a_idx, a_mask, l_idx = create_fst_attention_kernel_inputs(lineage.cuda(), level.cuda(), block_m, max_anc)
    made = recall_packed(a_mask)[1]
    nb = a_idx.shape[0]
    want, care = expected_plan(a_idx.cpu().numpy(), a_mask.cpu().numpy(), l_idx.cpu().numpy())
    for label, packed in (("precompute", made), ("pack", pack_tree_mask(a_idx, a_mask, l_idx))):
        got = packed.plan.cpu().numpy().view(np.uint32).reshape(nb, -1)
        assert got.shape == want.shape, label
        np.testing.assert_array_equal(got[care], want[care], err_msg=label)
        assert (got[~care] < nb * block_m).all(), label      # spare keys name rows of the tree
    # ids at or past the limit count as empty slots in a plan made by the packing entry point
    limit = n // 2
    want, care = expected_plan(a_idx.cpu().numpy(), a_mask.cpu().numpy(), l_idx.cpu().numpy(), key_limit=limit)
    got = pack_tree_mask(a_idx, a_mask, l_idx, key_limit=limit).plan.cpu().numpy().view(np.uint32).reshape(nb, -1)
    np.testing.assert_array_equal(got[care], want[care])
    assert (got[~care] < limit).all()


def test_lineage_from_parents_on_gpu():
    # (up to 16384 nodes the output rows are staged in LDS; larger trees are walked row by row)
    for seed, window, n in [(1, None, 777), (2, 8, 777), (3, 64, 777), (4, 2, 3000), (5, 40, 16384),
                            (6, 300, 20000)]:
        parent = trees.random_recursive_parents(n, seed, window)
        parent[::97] = -1
        want_lin, want_lvl = trees.lineage_from_parents(parent)
        lin, lvl = lineage_from_parents_gpu(torch.from_numpy(parent).cuda())
        assert torch.equal(lin.cpu(), want_lin) and torch.equal(lvl.cpu(), want_lvl)
        wide, _ = lineage_from_parents_gpu(torch.from_numpy(parent).cuda(), width=want_lin.shape[1] + 3)
        assert torch.equal(wide.cpu()[:, :want_lin.shape[1]], want_lin)
        assert (wide.cpu()[:, want_lin.shape[1]:] == -1).all()
    with pytest.raises(ValueError):
        lineage_from_parents_gpu(torch.tensor([-1, 0, 5], dtype=torch.int64).cuda())
    with pytest.raises(ValueError):
        lineage_from_parents_gpu(torch.tensor([-1, 0, 1, 2], dtype=torch.int64).cuda(), width=2)


@pytest.mark.parametrize("children", ["index", "light_first"])
def test_dfs_order_on_gpu_matches_the_host_order(children):
    cases = [np.array([-1], dtype=np.int64), np.array([-1, -1, -1], dtype=np.int64)]
    # up to 4096 nodes one workgroup does everything, beyond that six launches over arrays in device memory do
    for seed, n, window in [(1, 2, None), (2, 300, None), (3, 1500, 8), (4, 2049, 64), (5, 4096, 200),
                            (6, 4097, 16), (7, 9000, None)]:
        parent = trees.random_recursive_parents(n, seed, window)
        parent[::101] = -1                      # forest
        cases.append(parent)
    cases += [trees.config(i).parent for i in (2, 3, 4, 5)]
    star = np.zeros(700, dtype=np.int64)        # one parent with more children than a child list is walked for
    star[0] = -1
    star[500:] = np.arange(300, 500)            # ... and a second generation below some of them
    cases.append(star)
    cases.append(np.full(100, -1, dtype=np.int64))   # 100 roots
    for parent in cases:
        want = trees.dfs_order(parent, children)
        dev_parent = torch.from_numpy(parent).cuda()
        perm, rank = dfs_order_gpu(dev_parent, children)
        np.testing.assert_array_equal(perm.cpu().numpy(), want)
        want_parent, want_rank = trees.renumber_parents(parent, want)
        np.testing.assert_array_equal(rank.cpu().numpy(), want_rank)
        np.testing.assert_array_equal(renumber_parents_gpu(dev_parent, perm, rank).cpu().numpy(), want_parent)


@pytest.mark.parametrize("children", ["index", "light_first"])
def test_dfs_order_on_gpu_at_the_reference_tree_sizes(children):
    """The reference's benchmark trees go to 2^16 tokens and its size table to 2^17 (utils.py:4-13,
    fstattention.py:246); plus a wide star, a deep chain and a large random forest."""
    cases = [trees.parents_from_lineage(*(t.numpy() for t in trees.create_tree(depth))) for depth in (13, 14)]
    cases.append(trees.random_recursive_parents(100000, 21, 500))
    cases[-1][::977] = -1
    star = np.zeros(20000, dtype=np.int64)
    star[0] = -1
    cases.append(star)
    cases.append(np.arange(-1, 29999, dtype=np.int64))          # a chain of 30000 levels
    for parent in cases:
        want = trees.dfs_order(parent, children)
        perm, rank = dfs_order_gpu(torch.from_numpy(parent).cuda(), children)
        np.testing.assert_array_equal(perm.cpu().numpy(), want)
        np.testing.assert_array_equal(rank.cpu().numpy()[want], np.arange(len(parent)))


def test_dfs_order_on_gpu_flags_bad_parents_and_sizes():
    with pytest.raises(ValueError):
        dfs_order_gpu(torch.tensor([-1, 0, 5, 1], dtype=torch.int64).cuda())
    with pytest.raises(ValueError):
        dfs_order_gpu(torch.tensor([-1, 1, 0], dtype=torch.int64).cuda())
    perm, rank = dfs_order_gpu(torch.tensor([-1, -3, 0], dtype=torch.int64).cuda(), check=False)
    assert perm.tolist() == [0, 1, 2] and rank.tolist() == [0, 1, 2]   # identity when flagged
    with pytest.raises(RuntimeError):
        dfs_order_gpu(torch.full((131073,), -1, dtype=torch.int64).cuda())
    big = torch.from_numpy(trees.random_recursive_parents(50000, 3, 100)).cuda()
    big[40000] = 45000
    perm, rank = dfs_order_gpu(big, check=False)
    assert torch.equal(perm, torch.arange(50000, device="cuda")) and torch.equal(rank, perm)
    empty, _ = dfs_order_gpu(torch.empty((0,), dtype=torch.int64).cuda())
    assert empty.numel() == 0


def test_medusa_tree_built_on_the_gpu_matches_the_host_builder():
    for seed, depths, topk, n in [(1002, 4, 10, 256), (7, 4, 10, 64), (8, 3, 5, 100), (9, 2, 4, 21), (10, 4, 10, 1)]:
        probs = trees.medusa_probs(depths, topk, 0.3, seed)
        want = trees.medusa_parents_from_probs(probs, n)
        got = medusa_parents_gpu(torch.from_numpy(probs).cuda(), n)
        np.testing.assert_array_equal(got.cpu().numpy(), want)
    with pytest.raises(ValueError):
        medusa_parents_gpu(torch.ones((2, 3)).cuda(), 14)     # only 3 + 9 paths + root exist
    # ties everywhere (the candidate order decides), every path kept, one rank per depth, float32 input
    uniform = np.full((3, 6), 0.125)
    for n in (2, 7, 8, 30, 100, 6 + 36 + 216 + 1):
        np.testing.assert_array_equal(medusa_parents_gpu(torch.from_numpy(uniform).cuda(), n).cpu().numpy(),
                                      trees.medusa_parents_from_probs(uniform, n))
    halves = np.array([[0.5, 0.25, 0.25], [0.5, 0.5, 0.0], [1.0, 0.0, 0.0]])     # products tie across depths
    for n in range(1, 3 + 9 + 27 + 2):
        np.testing.assert_array_equal(medusa_parents_gpu(torch.from_numpy(halves).cuda(), n).cpu().numpy(),
                                      trees.medusa_parents_from_probs(halves, n))
    chain = np.array([[0.9], [0.8], [0.7], [0.6], [0.5]])
    np.testing.assert_array_equal(medusa_parents_gpu(torch.from_numpy(chain).cuda(), 6).cpu().numpy(),
                                  np.array([-1, 0, 1, 2, 3, 4]))
    p32 = trees.medusa_probs(4, 10, 0.3, 11).astype(np.float32)
    np.testing.assert_array_equal(medusa_parents_gpu(torch.from_numpy(p32).cuda(), 200).cpu().numpy(),
                                  trees.medusa_parents_from_probs(p32, 200))
    big = trees.medusa_probs(4, 11, 0.3, 12)       # 16104 candidate paths: the largest the kernel takes
    np.testing.assert_array_equal(medusa_parents_gpu(torch.from_numpy(big).cuda(), 1000).cpu().numpy(),
                                  trees.medusa_parents_from_probs(big, 1000))
    # the threshold search over the short list of candidates at or above a lower bound: ties at the threshold inside
    # the short list (every path of a depth scores alike), and a short list that overflows (the last head's ranks all
    # have probability 1: every path of depth 4 ties with its prefix) so that the search walks all candidates after all
    flat = np.full((4, 10), 0.1)
    for n in (12, 111, 300, 500):
        np.testing.assert_array_equal(medusa_parents_gpu(torch.from_numpy(flat).cuda(), n).cpu().numpy(),
                                      _best_paths_host(flat, n))
    flat[3] = 1.0
    for n in (300, 513):
        np.testing.assert_array_equal(medusa_parents_gpu(torch.from_numpy(flat).cuda(), n).cpu().numpy(),
                                      _best_paths_host(flat, n))
    # many seeds through the way that never stores the last level (and its overflow into the general way)
    for seed in range(12):
        for depths, topk, n in [(4, 10, 256), (4, 10, 512), (4, 10, 1000), (3, 24, 256), (4, 8, 128), (2, 100, 90)]:
            probs = trees.medusa_probs(depths, topk, 0.3 + 0.1 * (seed % 4), 100 + seed)
            if seed % 3 == 2:
                probs = probs.astype(np.float32)
            np.testing.assert_array_equal(medusa_parents_gpu(torch.from_numpy(probs).cuda(), n).cpu().numpy(),
                                          _best_paths_host(probs, n), err_msg=f"seed {seed} {depths}x{topk} n={n}")
    # a last-level rank with a "probability" above 1: paths of depth 4 outrank their own prefixes, some kept paths have
    # no kept parent (they hang off the root, as in the host's table of ids) and the status word says so
    odd = trees.medusa_probs(4, 10, 0.3, 77)
    odd[3, 0] = 40.0
    np.testing.assert_array_equal(medusa_parents_gpu(torch.from_numpy(odd).cuda(), 256).cpu().numpy(), _best_paths_host(odd, 256))
    with pytest.raises(ValueError):
        medusa_parents_gpu(torch.from_numpy(odd).cuda(), 256, check=True)
    with pytest.raises(ValueError, match="candidate paths"):      # 8 heads of 10 ranks: more than 2**24 paths
        medusa_parents_gpu(torch.from_numpy(trees.medusa_probs(8, 10, 0.3, 13)).cuda(), 300)
    with pytest.raises(ValueError):                # a deeper path scoring above its prefix
        medusa_parents_gpu(torch.tensor([[0.5, 0.1], [3.0, 0.1]], dtype=torch.float64).cuda(), 2, check=True)



def _best_paths_host(probs, n):
    """``trees.medusa_parents_from_probs`` for candidate sets too large to enumerate in Python tuples:
    the same scores (float64 products from the first rank on), the same order (score descending,
    then depth, then ranks = candidate index), the same numbering, in numpy."""
    probs = np.asarray(probs, dtype=np.float64)
    depths, topk = probs.shape
    scores, level = [], np.ones(1)
    for d in range(depths):
        level = (level[:, None] * probs[d][None, :]).reshape(-1)      # index = ranks read as a base-topk number
        scores.append(level)
    flat = np.concatenate(scores)
    starts = np.concatenate([[0], np.cumsum([len(x) for x in scores])])
    order = np.lexsort((np.arange(len(flat)), -flat))                 # score descending, ties by index
    kept = np.sort(order[: n - 1])
    ids = np.zeros(len(flat), dtype=np.int64)
    ids[kept] = np.arange(1, n)
    parent = np.full(n, -1, dtype=np.int64)
    for c in kept:
        d = int(np.searchsorted(starts, c, side="right")) - 1
        parent[ids[c]] = 0 if d == 0 else ids[starts[d - 1] + (c - starts[d]) // topk]
    return parent


def test_medusa_tree_of_more_paths_than_one_workgroup_ranks():
    """fsta_medusa_tree_ws: scores and ids in a device workspace, a dozen launches; bit-exact against the host."""
    small = trees.medusa_probs(3, 7, 0.3, 21)       # the numpy restatement against the tuple-based builder
    np.testing.assert_array_equal(_best_paths_host(small, 120), trees.medusa_parents_from_probs(small, 120))
    for depths, topk, n, seed in [(5, 10, 1024, 31), (5, 10, 4096, 32), (2, 200, 300, 13), (6, 10, 2048, 33),
                                  (4, 12, 20000, 34), (3, 40, 64001, 35)]:
        probs = trees.medusa_probs(depths, topk, 0.3, seed)
        got = medusa_parents_gpu(torch.from_numpy(probs).cuda(), n).cpu().numpy()
        np.testing.assert_array_equal(got, _best_paths_host(probs, n), err_msg=f"depths={depths} topk={topk} n={n}")
    # ties across workgroups: equal probabilities, every path of a depth scores alike
    uniform = np.full((5, 10), 0.1)
    for n in (2, 11, 12, 1000, 11111, 50000):
        got = medusa_parents_gpu(torch.from_numpy(uniform).cuda(), n).cpu().numpy()
        np.testing.assert_array_equal(got, _best_paths_host(uniform, n), err_msg=f"uniform n={n}")
    halves = np.tile(np.array([0.5, 0.5, 0.25, 0.25, 0.125, 0.125, 0.0625, 0.0625, 0.03125, 0.03125]), (5, 1))
    for n in (100, 5000):
        got = medusa_parents_gpu(torch.from_numpy(halves).cuda(), n).cpu().numpy()
        np.testing.assert_array_equal(got, _best_paths_host(halves, n), err_msg=f"halves n={n}")
    p32 = trees.medusa_probs(5, 10, 0.3, 36).astype(np.float32)
    np.testing.assert_array_equal(medusa_parents_gpu(torch.from_numpy(p32).cuda(), 777).cpu().numpy(),
                                  _best_paths_host(p32, 777))
    # the root alone, and every path kept
    assert medusa_parents_gpu(torch.from_numpy(uniform).cuda(), 1).cpu().tolist() == [-1]
    full = medusa_parents_gpu(torch.from_numpy(trees.medusa_probs(2, 200, 0.3, 13)).cuda(), 40201).cpu().numpy()
    np.testing.assert_array_equal(full, _best_paths_host(trees.medusa_probs(2, 200, 0.3, 13), 40201))


def test_device_only_pipeline_from_probabilities_to_kernel_inputs():
    """probabilities -> tree -> depth-first order -> lineage -> kernel inputs, all on the device,
    against the host chain on the same probabilities."""
    probs = trees.medusa_probs(4, 10, 0.3, 1002)
    parent = medusa_parents_gpu(torch.from_numpy(probs).cuda(), 256)
    perm, rank = dfs_order_gpu(parent, "light_first", check=False)
    new_parent = renumber_parents_gpu(parent, perm, rank)
    lineage, level = lineage_from_parents_gpu(new_parent, width=5, check=False)
    *got, status = create_fst_attention_kernel_inputs(lineage, level, 64, 64, check=False)
    assert int(status.item()) == 0
    host_parent = trees.medusa_parents_from_probs(probs, 256)
    host_new, _ = trees.renumber_parents(host_parent, trees.dfs_order(host_parent, "light_first"))
    lin, lvl = trees.lineage_from_parents(host_new, min_width=5)
    want = tp.block_inputs(lin.numpy().copy(), lvl.numpy(), 64, 64)
    _check(got, want)


def test_kernel_inputs_from_parents_in_one_launch():
    """``fsta_precompute_from_parents`` against the two-launch chain on the benchmark trees that fit one workgroup's
    LDS (bit for bit, packed inputs and block plan included), its status bits, and its refusal of a tree too large."""
    from fstattention_amd import _lib
    for index in (2, 3, 4, 5):
        cfg = trees.config(index)
        parent = torch.from_numpy(cfg.parent).cuda()
        max_anc = trees.required_max_ancestors(cfg.parent, cfg.block_m, 16)
        lineage, level = lineage_from_parents_gpu(parent)
        want_idx, want_packed, want_leaf = create_fst_attention_kernel_inputs(lineage, level, cfg.block_m, max_anc,
                                                                              want_bool_mask=False)
        a_idx, packed, l_idx, lin, lvl = kernel_inputs_from_parents_gpu(parent, cfg.block_m, max_anc, lineage.shape[1],
                                                                        want_lineage=True)
        assert torch.equal(a_idx, want_idx) and torch.equal(l_idx, want_leaf), cfg.name
        assert torch.equal(packed.mask_bits, want_packed.mask_bits) and torch.equal(packed.anc_count, want_packed.anc_count)
        assert torch.equal(packed.plan, want_packed.plan), cfg.name
        assert torch.equal(lin, lineage) and torch.equal(lvl, level), cfg.name      # (lineage carries the self entries by now)
    # too shallow rows, a malformed parent entry, too many ancestors: flagged, no fault
    chain = torch.arange(-1, 99, dtype=torch.int64, device="cuda")
    with pytest.raises(ValueError, match="deeper"):
        kernel_inputs_from_parents_gpu(chain, 32, 128, 50)
    bad = torch.from_numpy(trees.random_recursive_parents(300, 5, 16)).cuda()
    bad[17] = 200
    with pytest.raises(ValueError, match="parent"):
        kernel_inputs_from_parents_gpu(bad, 64, 64, 64)
    with pytest.raises(RuntimeError, match="max_ancestors"):
        kernel_inputs_from_parents_gpu(chain, 32, 16, 128)
    big = torch.from_numpy(trees.random_recursive_parents(60000, 6, 64)).cuda()
    with pytest.raises(_lib.FstaError, match="LDS"):
        kernel_inputs_from_parents_gpu(big, 128, 64, 64)
