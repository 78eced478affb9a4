"""GPU parity of the fused sparse tree attention against the dense-masked oracle.

Tolerances: float32 atol=rtol=1e-5; float16/bfloat16 atol=rtol=2e-3 against the
float64 oracle evaluated on the same (already rounded) inputs, asserted on the
float32 output of the kernel.
"""
import math

import numpy as np
import pytest
import torch

from fstattention_amd import (create_fst_attention_kernel_inputs, dfs_order_gpu, fst_attention,
                              lineage_from_parents_gpu, merge_attention_states, renumber_parents_gpu, shift_for_prefix,
                              trees)
from fstattention_amd.attention import recall_packed
from helpers import TOL, assert_close, dense_oracle, oracle_inputs, rand_qkv
from oracle import tree_precompute as tp

pytestmark = pytest.mark.gpu


def run_tree(parent, block_m, z, h, d, dtype, seed, prefix=0, generic=False, fast_pv=False,
             scale=None, check_lse=True, wide_waves=False, key_splits=None, share_tiles=False, stream_blocks=None,
             native_out=False, want_kernel=None):
    n = len(parent)
    a_idx, a_mask, l_idx, max_anc = oracle_inputs(parent, block_m)
    nb = a_idx.shape[0]
    nq = nb * block_m            # the reference needs whole blocks; pad rows see themselves
    q, k, v = rand_qkv(z, h, nq, nq + prefix, d, dtype, seed)
    scale = scale if scale is not None else 1.0 / math.sqrt(d)
    want, want_lse = dense_oracle(q, k, v, parent, scale, prefix=prefix, nq_pad=nq - n)
    if prefix:
        a_idx, l_idx = shift_for_prefix(a_idx, l_idx, prefix)
    o, lse = fst_attention(q.cuda(), k.cuda(), v.cuda(), a_idx.cuda(), a_mask.cuda(), l_idx.cuda(),
                           scale, BLOCK_M=block_m, MAX_ANCESTORS=max_anc,
                           out_dtype=torch.float32, return_lse=True, generic=generic, fast_pv=fast_pv,
                           wide_waves=wide_waves, key_splits=key_splits, share_tiles=share_tiles,
                           stream_blocks=stream_blocks)
    if want_kernel is not None:
        from fstattention_amd import _lib
        assert want_kernel in _lib.load().fsta_last_attention_kernel().decode()
    if native_out:      # the output in the type of q: within one unit in the last place of the float32 result
        o_native = fst_attention(q.cuda(), k.cuda(), v.cuda(), a_idx.cuda(), a_mask.cuda(), l_idx.cuda(), scale,
                                 BLOCK_M=block_m, MAX_ANCESTORS=max_anc, generic=generic, fast_pv=fast_pv,
                                 wide_waves=wide_waves, key_splits=key_splits, share_tiles=share_tiles,
                                 stream_blocks=stream_blocks)
        assert o_native.dtype == dtype
        torch.testing.assert_close(o_native.float(), o.to(dtype).float(), atol=0, rtol=2 ** -7 if dtype == torch.bfloat16 else 2 ** -10)
    assert o.dtype == torch.float32 and o.shape == q.shape
    err = assert_close(o, want, dtype, f"n={n} m={block_m} d={d} {dtype} prefix={prefix}")
    if check_lse:
        lse_tol = 1e-4 if dtype == torch.float32 else 2e-3
        torch.testing.assert_close(lse.cpu().double().view(z, h, nq), want_lse, atol=lse_tol, rtol=lse_tol)
    return err


@pytest.mark.parametrize("generic", [False, True])
def test_config1_random64_fp32(generic):
    cfg = trees.config(1)
    run_tree(cfg.parent, cfg.block_m, cfg.batch, cfg.heads, cfg.head_dim, torch.float32,
             cfg.tensor_seed, generic=generic)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("generic", [False, True])
def test_config2_medusa256(dtype, generic):
    cfg = trees.config(2)
    run_tree(cfg.parent, cfg.block_m, cfg.batch, cfg.heads, cfg.head_dim, dtype, cfg.tensor_seed,
             generic=generic)


@pytest.mark.parametrize("wide_waves", [False, True])
@pytest.mark.parametrize("index", [3, 4])
def test_config3_4_bf16(index, wide_waves):
    cfg = trees.config(index)
    run_tree(cfg.parent, cfg.block_m, cfg.batch, cfg.heads, cfg.head_dim, torch.bfloat16,
             cfg.tensor_seed, wide_waves=wide_waves)


@pytest.mark.parametrize("wide_waves", [False, True])
def test_config5_bf16_head_subset_against_oracle(wide_waves):
    # full tree and block size, 8 of the 512 (batch, head) slices so the oracle stays small
    cfg = trees.config(5)
    run_tree(cfg.parent, cfg.block_m, 2, 4, cfg.head_dim, torch.bfloat16, cfg.tensor_seed,
             wide_waves=wide_waves)


def sampled_rows_check(q, k, v, parent, o, lse, scale, prefix, samples, seed, dtype, what):
    """Rows of a launch too large for the dense oracle: row i attends to the prefix, its ancestors
    and itself, so its output is a softmax over that handful of keys (float64 on the host)."""
    rng = np.random.default_rng(seed)
    z_, h_, nq, d = q.shape
    tol = TOL[dtype]
    for _ in range(samples):
        z, h, i = int(rng.integers(z_)), int(rng.integers(h_)), int(rng.integers(len(parent)))
        keys, a = list(range(prefix)) + [prefix + i], int(parent[i])
        while a >= 0:
            keys.append(prefix + a)
            a = int(parent[a])
        idx = torch.tensor(keys, device=q.device)
        s = (k[z, h].index_select(0, idx).double() @ q[z, h, i].double()) * scale
        w = torch.softmax(s, 0)
        want = (w[:, None] * v[z, h].index_select(0, idx).double()).sum(0)
        got = o[z, h, i].double()
        err = (got - want).abs()
        assert bool((err <= tol + tol * want.abs()).all()), f"{what}: slice ({z},{h}) row {i}: max err {float(err.max()):.3e}"
        want_lse = torch.logsumexp(s, 0) / math.log(2.0)
        assert abs(float(lse[z * h_ + h, i]) - float(want_lse)) <= 2e-3 * max(1.0, abs(float(want_lse)))


@pytest.mark.parametrize("order", [None, "light_first"])
def test_config5_full_size_sampled_rows(order):
    """All 8 x 64 slices of configuration 5 (8192 workgroups), in the given and in depth-first token
    order; checked on sampled rows, and the two kernels against each other on one whole slice."""
    cfg = trees.config(5)
    parent = cfg.parent
    if order:
        parent, _ = trees.renumber_parents(parent, trees.dfs_order(parent, order))
    m, d, n = cfg.block_m, cfg.head_dim, cfg.n_nodes
    lineage, level = trees.lineage_from_parents(parent)
    max_anc = trees.required_max_ancestors(parent, m, 16)
    inputs = create_fst_attention_kernel_inputs(lineage.cuda(), level.cuda(), m, max_anc)
    g = torch.Generator(device="cuda").manual_seed(5)
    q, k, v = (torch.randn((cfg.batch, cfg.heads, n, d), generator=g, device="cuda", dtype=torch.float32)
               .to(torch.bfloat16) for _ in range(3))
    scale = 1.0 / math.sqrt(d)
    o, lse = fst_attention(q, k, v, *inputs, scale, BLOCK_M=m, MAX_ANCESTORS=max_anc, out_dtype=torch.float32,
                           return_lse=True)
    assert bool(torch.isfinite(o).all())
    sampled_rows_check(q, k, v, parent, o, lse, scale, 0, 96, 55, torch.bfloat16, f"cfg5 order={order}")
    one = fst_attention(q[7:, 63:].contiguous(), k[7:, 63:].contiguous(), v[7:, 63:].contiguous(), *inputs, scale,
                        BLOCK_M=m, MAX_ANCESTORS=max_anc, out_dtype=torch.float32, generic=True)
    torch.testing.assert_close(o[7:, 63:], one, atol=2e-3, rtol=2e-3)


def test_config5_full_size_rows_depend_on_their_ancestors_only():
    """Size-independent property, all 8 x 64 slices of configuration 5, no oracle: a token attends to itself and
    to tokens with smaller numbers only (its ancestors), so new K/V values for all rows from r on must leave the
    outputs and log-sum-exps of the rows below r exactly as they were, and new Q rows from r on likewise."""
    cfg = trees.config(5)
    m, d, n = cfg.block_m, cfg.head_dim, cfg.n_nodes
    lineage, level = trees.lineage_from_parents(cfg.parent)
    max_anc = trees.required_max_ancestors(cfg.parent, m, 16)
    inputs = create_fst_attention_kernel_inputs(lineage.cuda(), level.cuda(), m, max_anc)
    g = torch.Generator(device="cuda").manual_seed(17)
    q, k, v = (torch.randn((cfg.batch, cfg.heads, n, d), generator=g, device="cuda", dtype=torch.float32)
               .to(torch.bfloat16) for _ in range(3))
    scale = 1.0 / math.sqrt(d)
    call = lambda: fst_attention(q, k, v, *inputs, scale, BLOCK_M=m, MAX_ANCESTORS=max_anc, return_lse=True)
    o0, lse0 = call()
    for r in (1, 777, 1280):            # inside a block, and on a block boundary
        for t in (q, k, v):
            t[:, :, r:] = torch.randn((cfg.batch, cfg.heads, n - r, d), generator=g, device="cuda",
                                      dtype=torch.float32).to(torch.bfloat16)
        o1, lse1 = call()
        assert torch.equal(o1[:, :, :r], o0[:, :, :r]), f"rows below {r} changed"
        assert torch.equal(lse1.view(cfg.batch, cfg.heads, n)[:, :, :r], lse0.view(cfg.batch, cfg.heads, n)[:, :, :r])
        assert not torch.equal(o1[:, :, r:], o0[:, :, r:])
        o0, lse0 = o1, lse1


def test_config5_layer_loop_shares_one_set_of_kernel_inputs():
    """Configuration 5 as it is timed: the kernel inputs are built ONCE on the GPU from the device-resident
    parent array and reused by every layer, each layer with fresh seeded q/k/v (seed = tensor seed + layer).
    All 32 layers, all 8 x 64 slices each; every layer is checked on sampled rows against the host (16 rows,
    48 on the first, one in the middle and the last layer)."""
    cfg = trees.config(5)
    m, d, n = cfg.block_m, cfg.head_dim, cfg.n_nodes
    max_anc = trees.required_max_ancestors(cfg.parent, m, 16)
    parent_dev = torch.from_numpy(cfg.parent).cuda()
    lineage, level = lineage_from_parents_gpu(parent_dev)
    a_idx, packed, l_idx = create_fst_attention_kernel_inputs(lineage, level, m, max_anc, want_bool_mask=False)
    scale = 1.0 / math.sqrt(d)
    assert cfg.layers == 32
    for layer in range(cfg.layers):
        g = torch.Generator(device="cuda").manual_seed(cfg.tensor_seed + layer)
        q, k, v = (torch.randn((cfg.batch, cfg.heads, n, d), generator=g, device="cuda", dtype=torch.float32)
                   .to(torch.bfloat16) for _ in range(3))
        o, lse = fst_attention(q, k, v, a_idx, packed, l_idx, scale, BLOCK_M=m, MAX_ANCESTORS=max_anc,
                               out_dtype=torch.float32, return_lse=True)
        rows = 48 if layer in (0, 13, cfg.layers - 1) else 16
        sampled_rows_check(q, k, v, cfg.parent, o, lse, scale, 0, rows, 100 + layer, torch.bfloat16, f"cfg5 layer {layer}")
        del q, k, v, o


def test_large_tree_behind_a_long_prefix_sampled_rows():
    """40000 tokens behind 5000 prefix keys, 3 heads: index arithmetic far beyond the benchmark sizes
    (key runs chosen by the library), checked on sampled rows."""
    n, prefix, m, d, h = 40000, 5000, 128, 64, 3
    parent = trees.random_recursive_parents(n, 77, window=300)
    lineage, level = trees.lineage_from_parents(parent)
    max_anc = trees.required_max_ancestors(parent, m, 16)
    a_idx, a_mask, l_idx = create_fst_attention_kernel_inputs(lineage.cuda(), level.cuda(), m, max_anc)
    a_idx, l_idx = shift_for_prefix(a_idx, l_idx, prefix)
    nq = a_idx.shape[0] * m
    g = torch.Generator(device="cuda").manual_seed(6)
    q = torch.randn((1, h, nq, d), generator=g, device="cuda").to(torch.float16)
    k, v = (torch.randn((1, h, prefix + nq, d), generator=g, device="cuda").to(torch.float16) for _ in range(2))
    scale = 1.0 / math.sqrt(d)
    for splits in (1, None):
        o, lse = fst_attention(q, k, v, a_idx, a_mask, l_idx, scale, BLOCK_M=m, MAX_ANCESTORS=max_anc,
                               out_dtype=torch.float32, return_lse=True, key_splits=splits)
        sampled_rows_check(q, k, v, parent, o, lse, scale, prefix, 48, 66, torch.float16, f"large tree splits={splits}")


def test_more_blocks_than_a_grid_axis_holds_sampled_rows():
    """65538 blocks of 32 rows: past the 65535 limit of a grid's y axis, so the kernel is launched on
    one long x axis and recovers (slice, block) by division.  The tree is a forest of 32-node trees,
    one per block, whose kernel inputs are the first block's shifted.  Checked on sampled rows, and
    every row against the vector-ALU kernel (independent code)."""
    m, d, nb = 32, 32, 65538
    one = trees.random_recursive_parents(m, 31, window=20)
    lineage, level = trees.lineage_from_parents(one)
    max_anc = trees.required_max_ancestors(one, m, 16)
    a1, mask1, l1 = create_fst_attention_kernel_inputs(lineage.cuda(), level.cuda(), m, max_anc)
    shift = torch.arange(nb, device="cuda", dtype=torch.int64)[:, None] * m
    a_idx = torch.where(a1 >= 0, a1 + shift, a1).contiguous()
    l_idx = torch.where(l1 >= 0, l1 + shift, l1).contiguous()
    a_mask = mask1.expand(nb, m, max_anc).contiguous()
    parent = np.tile(one, nb)
    parent = np.where(parent >= 0, parent + np.repeat(np.arange(nb, dtype=np.int64) * m, m), -1)
    nq = nb * m
    g = torch.Generator(device="cuda").manual_seed(8)
    q, k, v = (torch.randn((1, 1, nq, d), generator=g, device="cuda", dtype=torch.float16) for _ in range(3))
    scale = 1.0 / math.sqrt(d)
    o, lse = fst_attention(q, k, v, a_idx, a_mask, l_idx, scale, BLOCK_M=m, MAX_ANCESTORS=max_anc,
                           out_dtype=torch.float32, return_lse=True)
    sampled_rows_check(q, k, v, parent, o, lse, scale, 0, 64, 88, torch.float16, "65538 blocks")
    other = fst_attention(q, k, v, a_idx, a_mask, l_idx, scale, BLOCK_M=m, MAX_ANCESTORS=max_anc,
                          out_dtype=torch.float32, generic=True)
    torch.testing.assert_close(o, other, atol=2e-3, rtol=2e-3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("d", [16, 32, 64, 128])
@pytest.mark.parametrize("block_m", [16, 32, 64, 128])
def test_shapes_sweep(dtype, d, block_m):
    parent = trees.random_recursive_parents(200, 100 + d + block_m, window=48)
    run_tree(parent, block_m, 1, 3, d, dtype, 7)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("d", [32, 64, 128])
@pytest.mark.parametrize("block_m", [32, 64, 128])
@pytest.mark.parametrize("prefix", [0, 40])
def test_shapes_sweep_wide_wave_variant(dtype, d, block_m, prefix):
    parent = trees.random_recursive_parents(200, 200 + d + block_m, window=48)
    run_tree(parent, block_m, 1, 3, d, dtype, 7, prefix=prefix, wide_waves=True)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("prefix", [64, 100, 7])
def test_shared_prefix(dtype, prefix):
    parent = trees.random_recursive_parents(128, 5, window=32)
    run_tree(parent, 64, 2, 2, 64, dtype, 11, prefix=prefix)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("block_m,d", [(32, 64), (64, 128), (128, 128), (64, 32)])
@pytest.mark.parametrize("prefix,splits", [(300, 3), (1024, 4), (77, 2), (2048, None), (96, 3)])
def test_prefix_cut_into_key_runs(dtype, block_m, d, prefix, splits):
    """The shared prefix taken by several workgroups per block (forced counts, and the library's
    own choice for a long prefix in front of few blocks) against the oracle over all keys."""
    parent = trees.random_recursive_parents(200, 300 + d + block_m, window=48)
    run_tree(parent, block_m, 1, 3, d, dtype, 13, prefix=prefix, key_splits=splits)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("scale", [0.3, 1.0])
def test_dense_prefix_kernel_with_peaked_weights(dtype, scale):
    """A long prefix goes to the dense prefix kernel.  Scores scaled up until one or two keys carry nearly all the
    weight of a row: the rounding of the weights on their way to the matrix cores (bfloat16 weights go there as
    hi + lo pairs for this reason; single bfloat16 values fail this test) must stay inside the tolerance (2e-3 on
    the float32 output)."""
    parent = trees.random_recursive_parents(256, 77, window=32)
    run_tree(parent, 64, 1, 4, 128, dtype, 23, prefix=4096, scale=scale)
    run_tree(parent, 128, 2, 2, 64, dtype, 24, prefix=2048, scale=scale)


def test_key_runs_native_output_type_and_workspace_contract():
    """Output in the storage type through the joining kernel; the C entry point with no or too
    small a workspace runs unsplit; the workspace query is 0 where no split is planned."""
    from fstattention_amd import _lib
    from fstattention_amd.attention import _DTYPES, _packed_for
    lib = _lib.load()
    cfg = trees.config(2)
    prefix, m, d, h = 4096, cfg.block_m, cfg.head_dim, 4
    a_idx, a_mask, l_idx, max_anc = oracle_inputs(cfg.parent, m)
    nq = a_idx.shape[0] * m
    q, k, v = rand_qkv(1, h, nq, nq + prefix, d, torch.bfloat16, 21)
    scale = 1.0 / math.sqrt(d)
    want, want_lse = dense_oracle(q, k, v, cfg.parent, scale, prefix=prefix, nq_pad=nq - len(cfg.parent))
    a_idx, l_idx = shift_for_prefix(a_idx, l_idx, prefix)
    qd, kd, vd, ad, md, ld = (t.cuda() for t in (q, k, v, a_idx, a_mask, l_idx))
    o, lse = fst_attention(qd, kd, vd, ad, md, ld, scale, BLOCK_M=m, MAX_ANCESTORS=max_anc, return_lse=True)
    assert o.dtype == torch.bfloat16
    # one rounding to bfloat16 on top of the float32 tolerance
    torch.testing.assert_close(o.cpu().double(), want, atol=2e-3 + 2 ** -8, rtol=2e-3 + 2 ** -8)
    torch.testing.assert_close(lse.cpu().double().view(1, h, nq), want_lse, atol=2e-3, rtol=2e-3)

    code = _DTYPES[torch.bfloat16]
    need = lib.fsta_attention_workspace_bytes(1, h, nq, nq + prefix, d, code, m, max_anc, scale, 0)
    assert need > 0
    assert lib.fsta_attention_workspace_bytes(1, h, nq, nq, d, code, m, max_anc, scale, 0) == 0
    assert lib.fsta_attention_workspace_bytes(1, h, nq, nq + prefix, d, code, m, max_anc, scale,
                                              _lib.flag_key_splits(1)) == 0
    assert lib.fsta_attention_workspace_bytes(1, h, nq, nq + prefix, d, _DTYPES[torch.float32], m, max_anc,
                                              scale, 0) == 0
    packed = _packed_for(ad, md, ld, nq + prefix)
    outs = []
    for work_bytes in (0, need - 1, need):
        work = torch.empty((max(work_bytes, 1),), dtype=torch.uint8, device="cuda")
        o32 = torch.empty(q.shape, dtype=torch.float32, device="cuda")
        _lib.check(lib.fsta_attention_fwd_ws(
            qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), o32.data_ptr(), None, ad.data_ptr(),
            packed.mask_bits.data_ptr(), packed.anc_count.data_ptr(), ld.data_ptr(), packed.plan.data_ptr(),
            packed.key_shift, 1, h, nq, nq + prefix, d,
            code, _DTYPES[torch.float32], m, max_anc, a_idx.shape[0], scale, 0,
            work.data_ptr() if work_bytes else None, work_bytes, torch.cuda.current_stream().cuda_stream))
        assert_close(o32, want, torch.bfloat16, f"workspace of {work_bytes} bytes")
        outs.append(o32)
    unsplit = fst_attention(qd, kd, vd, ad, md, ld, scale, BLOCK_M=m, MAX_ANCESTORS=max_anc,
                            out_dtype=torch.float32, key_splits=1)
    assert torch.equal(outs[0], unsplit) and torch.equal(outs[1], unsplit)
    assert not torch.equal(outs[2], unsplit)      # the split path did run


@pytest.mark.parametrize("share_tiles", [False, True])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("block_m,d", [(32, 64), (32, 128), (64, 64), (64, 128), (128, 128), (128, 64)])
def test_short_ancestor_lists_both_wave_pairings(block_m, d, dtype, share_tiles):
    """Small launches with one or two ancestor tiles per block: the waves of a row group share the
    head dimension by default and the key tiles with the tuning flag; ragged last block included."""
    parent = trees.medusa_parents(n=230, seed=500 + d + block_m)
    run_tree(parent, block_m, 1, 5, d, dtype, 17, share_tiles=share_tiles)
    bushy = np.maximum((np.arange(90) - 1) // 3, -1).astype(np.int64)      # at most one ancestor tile
    bushy[0] = -1
    run_tree(bushy, block_m, 2, 2, d, dtype, 18, share_tiles=share_tiles)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("scale", [1.5, 6.0])
def test_two_tiles_per_step_with_peaked_weights(dtype, scale):
    """The waves that share the head dimension take two ancestor tiles in one step; scores far apart (a large
    softmax scale) send them through the full update of the running maximum over both tiles."""
    parent = trees.medusa_parents(n=256, seed=901)
    run_tree(parent, 64, 1, 6, 128, dtype, 31, scale=scale, want_kernel="-2")
    run_tree(parent, 128, 1, 3, 64, dtype, 32, scale=scale, want_kernel="-2")


def test_reference_test_shape_with_and_without_prefix():
    # the reference's own test: Z=2 H=2 N_CTX=2048 D=64 fp16, tree of 2044 nodes,
    # blocks of 128, 64 ancestors, sm_scale 0.5, inputs N(0, 0.5^2), prefix 0 or 2048
    lineage, level = trees.create_tree(trees.DEPTH_MAPPING[2048])
    parent = trees.parents_from_lineage(lineage, level)
    a_idx, a_mask, l_idx = create_fst_attention_kernel_inputs(lineage.cuda(), level.cuda(), 128,
                                                              trees.MAX_ANCESTOR_MAPPING[2048])
    for prefix in (0, 2048):
        q, k, v = rand_qkv(2, 2, 2048, 2048 + prefix, 64, torch.float16, 20)
        q, k, v = q * 0.5, k * 0.5, v * 0.5
        want, _ = dense_oracle(q, k, v, parent, 0.5, prefix=prefix, nq_pad=4)
        ai, li = shift_for_prefix(a_idx, l_idx, prefix) if prefix else (a_idx, l_idx)
        o = fst_attention(q.cuda(), k.cuda(), v.cuda(), ai, a_mask, li, 0.5)   # defaults 128 / 64
        assert o.dtype == torch.float16
        # the reference's own criterion on its own output dtype
        assert torch.allclose(o.cpu().float(), want.float(), atol=1e-2, rtol=0)
        o32 = fst_attention(q.cuda(), k.cuda(), v.cuda(), ai, a_mask, li, 0.5, out_dtype=torch.float32)
        assert_close(o32, want, torch.float16, f"reference shape prefix={prefix}")


@pytest.mark.parametrize("scale", [-0.3, 0.0])
def test_non_positive_scale(scale):
    parent = trees.random_recursive_parents(128, 77, window=32)
    for dtype in (torch.float32, torch.bfloat16):
        run_tree(parent, 64, 1, 2, 64, dtype, 13, scale=scale)


@pytest.mark.parametrize("n,block_m,heads,dtype", [(700, 64, 30, torch.bfloat16), (900, 128, 40, torch.float16),
                                                   (1000, 64, 32, torch.bfloat16)])
def test_launches_of_one_to_two_workgroups_per_cu(n, block_m, heads, dtype):
    # more than 256 and at most 512 workgroups: the late blocks of every slice are dispatched first; a ragged last
    # block, a head count that does not fill the last group of eight slices, every row against the dense oracle
    parent = trees.random_recursive_parents(n, 17, window=48)
    a_idx, a_mask, l_idx, max_anc = oracle_inputs(parent, block_m)
    q, k, v = rand_qkv(1, heads, n, n, 128, dtype, 23)
    scale = 1.0 / math.sqrt(128)
    want, _ = dense_oracle(q, k, v, parent, scale)
    o = fst_attention(q.cuda(), k.cuda(), v.cuda(), a_idx.cuda(), a_mask.cuda(), l_idx.cuda(), scale,
                      BLOCK_M=block_m, MAX_ANCESTORS=max_anc, out_dtype=torch.float32)
    from fstattention_amd import _lib
    assert "attn_mfma16_kernel" in _lib.load().fsta_last_attention_kernel().decode()
    assert_close(o, want, dtype, f"n={n} m={block_m} heads={heads}")


def test_ragged_query_count():
    # nq not a multiple of block_m: rows past nq are neither read nor written
    parent = trees.random_recursive_parents(100, 3)
    a_idx, a_mask, l_idx, max_anc = oracle_inputs(parent, 32)
    for dtype in (torch.float32, torch.bfloat16):
        q, k, v = rand_qkv(1, 2, 100, 100, 64, dtype, 5)
        want, _ = dense_oracle(q, k, v, parent, 0.125)
        o = fst_attention(q.cuda(), k.cuda(), v.cuda(), a_idx.cuda(), a_mask.cuda(), l_idx.cuda(),
                          0.125, BLOCK_M=32, MAX_ANCESTORS=max_anc, out_dtype=torch.float32)
        assert_close(o, want, dtype, "ragged")


def test_closed_forms_roots_and_equal_keys():
    parent = np.array([-1, -1, 0, 1, -1, 2, 5, 6] + [7] * 8)
    a_idx, a_mask, l_idx, max_anc = oracle_inputs(parent, 16)
    q, k, v = rand_qkv(1, 2, 16, 16, 32, torch.float16, 9)
    args = (a_idx.cuda(), a_mask.cuda(), l_idx.cuda(), 0.3)
    o = fst_attention(q.cuda(), k.cuda(), v.cuda(), *args, BLOCK_M=16, MAX_ANCESTORS=max_anc)
    for r in (0, 1, 4):    # roots attend to themselves only: o = v exactly
        assert torch.equal(o[0, :, r].cpu(), v[0, :, r])
    k_same = k[:, :, :1].expand_as(k).contiguous()
    o = fst_attention(q.cuda(), k_same.cuda(), v.cuda(), *args, BLOCK_M=16, MAX_ANCESTORS=max_anc,
                      out_dtype=torch.float32)
    m = torch.from_numpy(tp.dense_tree_mask(parent)).double()
    want = (m @ v.double()) / m.sum(-1, keepdim=True)
    assert_close(o, want, torch.float16, "equal keys -> mean of allowed values")


def test_default_output_dtype_and_bf16_rounding_report():
    cfg = trees.config(2)
    a_idx, a_mask, l_idx, max_anc = oracle_inputs(cfg.parent, cfg.block_m)
    q, k, v = trees.make_qkv(cfg)
    scale = 1 / math.sqrt(cfg.head_dim)
    want, _ = dense_oracle(q, k, v, cfg.parent, scale)
    o = fst_attention(q.cuda(), k.cuda(), v.cuda(), a_idx.cuda(), a_mask.cuda(), l_idx.cuda(), scale,
                      BLOCK_M=cfg.block_m, MAX_ANCESTORS=max_anc)
    assert o.dtype == torch.bfloat16
    # a bf16 result can be no closer than the oracle rounded to bf16: at most one ulp apart
    # (plus the error of the hi+lo bf16 weights, 2^-17 relative per term, which matters only
    # where the terms cancel to ~0)
    ulp = torch.maximum(want.abs(), torch.tensor(2.0 ** -126)).log2().floor().exp2() * 2.0 ** -7
    assert ((o.cpu().double() - want).abs() <= ulp + 1e-4).all()


@pytest.mark.parametrize("d", [32, 64, 128])
@pytest.mark.parametrize("block_m", [32, 64, 128])
def test_fast_pv_flag_stays_within_loose_bound(d, block_m):
    # single bf16 rounding of every weight (relative 2^-9 each, weights up to 2^8 before
    # normalisation): a few 1e-3 of max|v| in practice; a wrong weight would be off by O(1)
    parent = trees.random_recursive_parents(300, 5 + d + block_m, window=40)
    a_idx, a_mask, l_idx, max_anc = oracle_inputs(parent, block_m)
    nq = a_idx.shape[0] * block_m
    q, k, v = rand_qkv(1, 4, nq, nq, d, torch.bfloat16, 3)
    scale = 1 / math.sqrt(d)
    want, _ = dense_oracle(q, k, v, parent, scale, nq_pad=nq - 300)
    o = fst_attention(q.cuda(), k.cuda(), v.cuda(), a_idx.cuda(), a_mask.cuda(), l_idx.cuda(), scale,
                      BLOCK_M=block_m, MAX_ANCESTORS=max_anc, out_dtype=torch.float32, fast_pv=True)
    err = float((o.cpu().double() - want).abs().max())
    assert err < 2.5e-2, err


def test_ancestor_slots_with_holes_and_out_of_range_ids_are_skipped():
    parent = trees.random_recursive_parents(64, 8)
    a_idx, a_mask, l_idx, max_anc = oracle_inputs(parent, 32, multiple=8)
    # widen the ancestor axis and move the valid entries to odd slots; fill even slots with
    # -1 or ids past the end of K whose mask bits are set: they must be ignored
    nb = a_idx.shape[0]
    wide_idx = torch.full((nb, 2 * max_anc), -1, dtype=torch.int64)
    wide_mask = torch.zeros((nb, 32, 2 * max_anc), dtype=torch.bool)
    wide_idx[:, 1::2] = a_idx
    wide_mask[:, :, 1::2] = a_mask
    wide_idx[:, 0::4] = 10 ** 6
    wide_mask[:, :, 0::2] = True
    q, k, v = rand_qkv(1, 2, 64, 64, 64, torch.float32, 3)
    want, _ = dense_oracle(q, k, v, parent, 0.2)
    for generic in (False, True):
        o = fst_attention(q.cuda(), k.cuda(), v.cuda(), wide_idx.cuda(), wide_mask.cuda(), l_idx.cuda(),
                          0.2, BLOCK_M=32, MAX_ANCESTORS=2 * max_anc, generic=generic)
        assert_close(o, want, torch.float32, "holes")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("block_m,heads", [(32, 2), (64, 40), (128, 3)])
def test_holes_and_out_of_range_ids_in_the_block_plan(block_m, heads, dtype):
    """The same malformed lists through the matrix-core kernel, whose block plan is made from them:
    empty slots between valid ones, ids past the end of K with their mask bits set, leaf slots past
    the end of K (small and large launches)."""
    n = 3 * block_m
    parent = trees.random_recursive_parents(n, 9, window=24)
    a_idx, a_mask, l_idx, max_anc = oracle_inputs(parent, block_m, multiple=8)
    nb = a_idx.shape[0]
    wide_idx = torch.full((nb, 2 * max_anc), -1, dtype=torch.int64)
    wide_mask = torch.zeros((nb, block_m, 2 * max_anc), dtype=torch.bool)
    wide_idx[:, 1::2] = a_idx
    wide_mask[:, :, 1::2] = a_mask
    wide_idx[:, 0::4] = 10 ** 6
    wide_mask[:, :, 0::2] = True
    q, k, v = rand_qkv(1, heads, n, n, 64, dtype, 3)
    want, _ = dense_oracle(q, k, v, parent, 0.2)
    o = fst_attention(q.cuda(), k.cuda(), v.cuda(), wide_idx.cuda(), wide_mask.cuda(), l_idx.cuda(),
                      0.2, BLOCK_M=block_m, MAX_ANCESTORS=2 * max_anc, out_dtype=torch.float32)
    assert_close(o, want, dtype, "holes in the plan")
    # a leaf slot past the end of K is an empty slot: rows that are nobody's ancestor then see nothing else
    l_bad = l_idx.clone()
    l_bad[l_bad >= 0] += 10 ** 6
    o, lse = fst_attention(q.cuda(), k.cuda(), v.cuda(), a_idx.cuda(), a_mask.cuda(), l_bad.cuda(), 0.2,
                           BLOCK_M=block_m, MAX_ANCESTORS=max_anc, out_dtype=torch.float32, return_lse=True)
    mask = tp.dense_tree_mask(parent)
    mask[np.arange(n), np.arange(n)] &= (l_idx.flatten()[:n] < 0).numpy()      # leaves lose their own key
    want, _ = da_dense(q, k, v, mask, 0, 0.2)
    want = torch.nan_to_num(want, nan=0.0)                                      # roots now see nothing: 0
    assert_close(o, want, dtype, "leaf slots past the end of K")


def test_packed_inputs_follow_a_prefix_shift_and_inference_mode():
    """Kernel inputs made on the GPU as packed inputs (no bool mask), moved behind a shared prefix with
    shift_for_prefix; the same calls under torch.inference_mode(), where tensors keep no version
    counters and the bool mask is packed on every call."""
    cfg = trees.config(2)
    prefix, m, d, h = 96, cfg.block_m, 64, 3
    parent = cfg.parent
    lineage, level = trees.lineage_from_parents(parent)
    max_anc = trees.required_max_ancestors(parent, m, 16)
    n = len(parent)
    q, k, v = rand_qkv(1, h, n, n + prefix, d, torch.bfloat16, 31)
    scale = 0.125
    want, _ = dense_oracle(q, k, v, parent, scale, prefix=prefix)
    want0, _ = dense_oracle(q, k[:, :, prefix:], v[:, :, prefix:], parent, scale)
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    for inference in (False, True):
        with torch.inference_mode(inference):
            a_idx, packed, l_idx = create_fst_attention_kernel_inputs(lineage.cuda(), level.cuda(), m, max_anc,
                                                                      want_bool_mask=False)
            assert packed.plan is not None and packed.key_shift == 0
            o = fst_attention(qd, kd[:, :, prefix:].contiguous(), vd[:, :, prefix:].contiguous(), a_idx, packed, l_idx,
                              scale, BLOCK_M=m, MAX_ANCESTORS=max_anc, out_dtype=torch.float32)
            assert_close(o, want0, torch.bfloat16, f"packed inputs, inference={inference}")
            a_sh, l_sh, packed_sh = shift_for_prefix(a_idx, l_idx, prefix, packed)
            assert packed_sh.key_shift == prefix
            o = fst_attention(qd, kd, vd, a_sh, packed_sh, l_sh, scale, BLOCK_M=m, MAX_ANCESTORS=max_anc,
                              out_dtype=torch.float32)
            assert_close(o, want, torch.bfloat16, f"packed inputs behind a prefix, inference={inference}")
            # bool mask: packed by fst_attention itself (remembered for the tensor outside inference mode, and
            # never as an attribute of the caller's tensor)
            a_idx, a_mask, l_idx = create_fst_attention_kernel_inputs(lineage.cuda(), level.cuda(), m, max_anc)
            assert (recall_packed(a_mask) is not None) != inference
            assert not hasattr(a_mask, "_fsta_packed")
            a_sh, l_sh = shift_for_prefix(a_idx, l_idx, prefix)
            for _ in range(2):
                o = fst_attention(qd, kd, vd, a_sh, a_mask, l_sh, scale, BLOCK_M=m, MAX_ANCESTORS=max_anc,
                                  out_dtype=torch.float32)
                assert_close(o, want, torch.bfloat16, f"bool mask behind a prefix, inference={inference}")


def test_c_caller_without_a_block_plan_gets_the_list_reading_kernel():
    """fsta_attention_fwd with block_plan = NULL: the lists themselves are read (slower matrix-core kernel)."""
    from fstattention_amd import _lib
    from fstattention_amd.attention import _DTYPES, pack_tree_mask
    lib = _lib.load()
    cfg = trees.config(2)
    m, d, h = cfg.block_m, 128, 2
    a_idx, a_mask, l_idx, max_anc = oracle_inputs(cfg.parent, m)
    nq = a_idx.shape[0] * m
    q, k, v = rand_qkv(1, h, nq, nq, d, torch.bfloat16, 5)
    want, _ = dense_oracle(q, k, v, cfg.parent, 0.1, nq_pad=nq - len(cfg.parent))
    qd, kd, vd, ad, md, ld = (t.cuda() for t in (q, k, v, a_idx, a_mask, l_idx))
    packed = pack_tree_mask(ad, md)
    assert packed.plan is None
    o32 = torch.empty(q.shape, dtype=torch.float32, device="cuda")
    _lib.check(lib.fsta_attention_fwd(
        qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), o32.data_ptr(), None, ad.data_ptr(), packed.mask_bits.data_ptr(),
        packed.anc_count.data_ptr(), ld.data_ptr(), None, 0, 1, h, nq, nq, d, _DTYPES[torch.bfloat16],
        _DTYPES[torch.float32], m, max_anc, a_idx.shape[0], 0.1, 0, torch.cuda.current_stream().cuda_stream))
    assert_close(o32, want, torch.bfloat16, "no plan")


@pytest.mark.parametrize("block_m,prefix,variant", [(32, 0, "default"), (64, 0, "default"), (128, 0, "default"),
                                                    (64, 64, "default"), (64, 0, "wide"), (64, 0, "generic")])
def test_leaf_slots_naming_other_rows(block_m, prefix, variant):
    """A leaf slot holds a key row (reference fstattention.py:86-91 gathers K[leaf_idx]); the
    precompute always puts the row's own id there, but the kernels must honour any id.  Leaf row
    i is pointed at key i+1 (never one of its ancestors, parents come first) and the dense
    oracle's mask is edited the same way."""
    n, d, dtype = 2 * block_m, 64, torch.bfloat16
    parent = trees.random_recursive_parents(n, 11)
    a_idx, a_mask, l_idx, max_anc = oracle_inputs(parent, block_m)
    mask = tp.dense_tree_mask(parent)
    l_new = l_idx.clone()
    for j in range(l_idx.shape[0]):
        for r in range(block_m):
            i = int(l_idx[j, r])
            if i >= 0:
                other = min(i + 1, n - 1)
                l_new[j, r] = other
                mask[i, i] = False
                mask[i, other] = True
    assert not torch.equal(l_new, l_idx)
    q, k, v = rand_qkv(1, 2, n, n + prefix, d, dtype, 5)
    want, _ = da_dense(q, k, v, mask, prefix, 0.125)
    if prefix:
        a_idx, l_new = shift_for_prefix(a_idx, l_new, prefix)
    o = fst_attention(q.cuda(), k.cuda(), v.cuda(), a_idx.cuda(), a_mask.cuda(), l_new.cuda(), 0.125,
                      BLOCK_M=block_m, MAX_ANCESTORS=max_anc, out_dtype=torch.float32,
                      generic=variant == "generic", wide_waves=variant == "wide")
    assert_close(o, want, dtype, f"leaf slots naming other rows, {variant}")


def da_dense(q, k, v, tree_mask, prefix, scale):
    from oracle import dense_attention as da
    return da.dense_tree_attention(q, k, v, da.full_mask_with_prefix(tree_mask, prefix), scale, dtype=torch.float64)


@pytest.mark.parametrize("index,children", [(2, "index"), (2, "light_first"), (3, "index"), (5, "light_first")])
def test_depth_first_renumbered_tree_gives_the_same_attention(index, children):
    """Tokens laid out in depth-first order (reference README.md:19-20): the op on the renumbered
    tree and permuted q/k/v, un-permuted, is the dense oracle's result on the tree as given."""
    cfg = trees.config(index)
    n, m, d = cfg.n_nodes, cfg.block_m, cfg.head_dim
    q, k, v = rand_qkv(1, 2, n, n, d, cfg.dtype, 77)
    scale = 1.0 / math.sqrt(d)
    want, _ = dense_oracle(q, k, v, cfg.parent, scale)
    perm, rank = dfs_order_gpu(torch.from_numpy(cfg.parent).cuda(), children)
    new_parent = renumber_parents_gpu(torch.from_numpy(cfg.parent).cuda(), perm, rank)
    lineage, level = lineage_from_parents_gpu(new_parent)
    max_anc = trees.required_max_ancestors(new_parent.cpu().numpy(), m)
    a_idx, a_mask, l_idx = create_fst_attention_kernel_inputs(lineage, level, m, max_anc)
    qp, kp, vp = (t.cuda().index_select(2, perm) for t in (q, k, v))
    o = fst_attention(qp, kp, vp, a_idx, a_mask, l_idx, scale, BLOCK_M=m, MAX_ANCESTORS=max_anc,
                      out_dtype=torch.float32)
    assert_close(o.index_select(2, rank), want, cfg.dtype, f"{cfg.name} in depth-first order")


def test_very_long_ancestor_lists_take_the_kernel_with_the_smaller_lds_footprint():
    """A 4992-node chain: the last block of 128 rows has 4991 ancestors, more than the default
    kernel can keep beside its four-stage ring; the launch must still give the right answer."""
    n, m, d = 4992, 128, 128
    parent = np.arange(-1, n - 1, dtype=np.int64)
    a_idx, a_mask, l_idx, max_anc = oracle_inputs(parent, m)
    assert max_anc >= 4991
    q, k, v = rand_qkv(1, 1, n, n, d, torch.bfloat16, 3)
    want, _ = dense_oracle(q, k, v, parent, 0.05)
    o = fst_attention(q.cuda(), k.cuda(), v.cuda(), a_idx.cuda(), a_mask.cuda(), l_idx.cuda(), 0.05,
                      BLOCK_M=m, MAX_ANCESTORS=max_anc, out_dtype=torch.float32)
    assert_close(o, want, torch.bfloat16, "4992-node chain")
    # and a list no matrix-core kernel has the LDS for (falls through to the scalar kernel)
    n = 8192
    parent = np.arange(-1, n - 1, dtype=np.int64)
    a_idx, a_mask, l_idx, max_anc = oracle_inputs(parent, m)
    q, k, v = rand_qkv(1, 1, n, n, d, torch.bfloat16, 4)
    want, _ = dense_oracle(q, k, v, parent, 0.05)
    o = fst_attention(q.cuda(), k.cuda(), v.cuda(), a_idx.cuda(), a_mask.cuda(), l_idx.cuda(), 0.05,
                      BLOCK_M=m, MAX_ANCESTORS=max_anc, out_dtype=torch.float32)
    assert_close(o, want, torch.bfloat16, "8192-node chain")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_prefix_and_tree_parts_merge_into_the_full_result(dtype):
    """Attention over [prefix | tree] = the two parts computed apart and joined through their
    log-sum-exp (what exposing L of reference fstattention.py:139-141 is for).  Checked against
    the dense oracle over all keys, so the merge formula is pinned by the identity, not retyped."""
    parent = trees.random_recursive_parents(128, 21)
    m, d, prefix, scale = 64, 64, 96, 0.2
    a_idx, a_mask, l_idx, max_anc = oracle_inputs(parent, m)
    q, k, v = rand_qkv(2, 2, 128, 128 + prefix, d, dtype, 8)
    want, want_lse = dense_oracle(q, k, v, parent, scale, prefix=prefix)
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    kw = dict(BLOCK_M=m, MAX_ANCESTORS=max_anc, out_dtype=torch.float32, return_lse=True)
    # tree part: keys of the tree only
    o_t, l_t = fst_attention(qd, kd[:, :, prefix:].contiguous(), vd[:, :, prefix:].contiguous(),
                             a_idx.cuda(), a_mask.cuda(), l_idx.cuda(), scale, **kw)
    # prefix part: same call layout, tree keys switched off (empty mask, no leaf slots)
    o_p, l_p = fst_attention(qd, kd, vd, torch.full_like(a_idx, -1).cuda(), torch.zeros_like(a_mask).cuda(),
                             torch.full_like(l_idx, -1).cuda(), scale, **kw)
    o, lse = merge_attention_states(o_t, l_t, o_p, l_p)
    assert_close(o, want, dtype, "merged")
    tol = 1e-4 if dtype == torch.float32 else 2e-3
    torch.testing.assert_close(lse.cpu().double().view(2, 2, 128), want_lse, atol=tol, rtol=tol)
    # storage-type states (what a caller usually holds), an empty part, and both parts empty
    o16, lse16 = merge_attention_states(o_t.to(dtype), l_t, o_p.to(dtype), l_p)
    assert o16.dtype == dtype
    torch.testing.assert_close(o16.float().cpu().double(), want, atol=1e-2 if dtype != torch.float32 else 1e-5, rtol=1e-2)
    none = torch.full_like(l_t, float("-inf"))
    junk = torch.full_like(o_t, float("nan"))
    o_same, l_same = merge_attention_states(o_t, l_t, junk, none)
    assert torch.equal(o_same, o_t) and torch.equal(l_same, l_t)
    o_zero, l_zero = merge_attention_states(junk, none, junk, none)
    assert (o_zero == 0).all() and torch.isinf(l_zero).all() and (l_zero < 0).all()
    with pytest.raises(ValueError):
        merge_attention_states(o_t, l_t[:, :5], o_p, l_p)


@pytest.mark.parametrize("seed", range(24))
def test_random_shapes_against_oracle(seed):
    """Seeded draw over tree shape, size (ragged last blocks included), block size, head dim,
    storage type, prefix length and slice count; every fourth case has enough slices for several
    rounds of workgroups per CU (the start-up differs between small and large launches)."""
    rng = np.random.default_rng(1000 + seed)
    block_m = int(rng.choice([32, 64, 128]))
    d = int(rng.choice([32, 64, 128]))
    dtype = [torch.bfloat16, torch.float16][seed % 2]
    n = int(rng.integers(1, 5 * block_m))
    kind = seed % 3
    if kind == 0:
        parent = trees.random_recursive_parents(n, seed)
    elif kind == 1:
        parent = trees.random_recursive_parents(n, seed, window=int(rng.integers(1, 9)))   # deep
    else:
        parent = np.maximum((np.arange(n) - 1) // int(rng.integers(2, 12)), -1).astype(np.int64)   # bushy
        parent[0] = -1
    prefix = int(rng.choice([0, 0, int(rng.integers(1, 150))]))
    z, h = (2, 72) if seed % 4 == 3 else (int(rng.integers(1, 3)), int(rng.integers(1, 4)))
    run_tree(parent, block_m, z, h, d, dtype, seed, prefix=prefix, wide_waves=(seed % 8 == 5))


@pytest.mark.parametrize("seed", range(12))
def test_random_shapes_with_key_runs_against_oracle(seed):
    """The same draw with a shared prefix of up to 3000 keys, cut into a forced or library-chosen
    number of runs (ragged last runs, more runs than make sense, heads that are no multiple of 8)."""
    rng = np.random.default_rng(3000 + seed)
    block_m = int(rng.choice([32, 64, 128]))
    d = int(rng.choice([32, 64, 128]))
    dtype = [torch.bfloat16, torch.float16][seed % 2]
    n = int(rng.integers(1, 4 * block_m))
    parent = trees.random_recursive_parents(n, seed, window=[None, 4][seed % 2])
    prefix = int(rng.integers(33, 3000))
    splits = [None, 2, 3, 5, 8, 13][seed % 6]
    run_tree(parent, block_m, int(rng.integers(1, 3)), int(rng.integers(1, 6)), d, dtype, seed, prefix=prefix,
             key_splits=splits)


def test_hip_graph_replays_match_eager_calls():
    """The op captured into a HIP graph (precompute + attention, as a decoding step would), replayed
    several times with eager launches and synchronisations in between; every replay must give the
    eager result for the inputs its buffers hold at that moment."""
    cfg = trees.config(2)
    m, d = cfg.block_m, cfg.head_dim
    lineage, level = trees.lineage_from_parents(cfg.parent)
    lineage, level = lineage.cuda(), level.cuda()
    max_anc = trees.required_max_ancestors(cfg.parent, m)
    scale = 1.0 / math.sqrt(d)
    q, k, v = (t.cuda() for t in rand_qkv(1, 4, cfg.n_nodes, cfg.n_nodes, d, cfg.dtype, 31))

    def step():
        *inputs, _ = create_fst_attention_kernel_inputs(lineage, level, m, max_anc, mutate_lineage=False,
                                                        check=False, want_bool_mask=False)
        return fst_attention(q, k, v, *inputs, scale, BLOCK_M=m, MAX_ANCESTORS=max_anc, out_dtype=torch.float32)

    eager = step().clone()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        step()
        stream.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            out = step()
    for replay in range(4):
        if replay:                                   # new inputs in the same buffers, eager work in between
            g = torch.Generator().manual_seed(100 + replay)
            q.copy_(torch.randn(q.shape, generator=g).to(q.dtype))
            eager = step().clone()
            torch.cuda.synchronize()
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {replay} differs from the eager call"
    want, _ = dense_oracle(q.cpu(), k.cpu(), v.cpu(), cfg.parent, scale)
    assert_close(out, want, cfg.dtype, "last replay")


def test_hip_graph_replays_of_key_runs_match_eager_calls():
    """A long shared prefix cut into runs of keys (dense prefix kernel, then the tree part that joins: two launches
    and a workspace from torch's graph-private pool) captured into a HIP graph; replays on new q and new prefix
    rows must give the eager results."""
    cfg = trees.config(2)
    m, d, prefix = cfg.block_m, cfg.head_dim, 3000
    lineage, level = trees.lineage_from_parents(cfg.parent)
    max_anc = trees.required_max_ancestors(cfg.parent, m)
    a_idx, a_mask, l_idx = create_fst_attention_kernel_inputs(lineage.cuda(), level.cuda(), m, max_anc)
    a_idx, l_idx = shift_for_prefix(a_idx, l_idx, prefix)
    scale = 1.0 / math.sqrt(d)
    q, k, v = (t.cuda() for t in rand_qkv(1, 2, cfg.n_nodes, prefix + cfg.n_nodes, d, cfg.dtype, 41))

    def step():
        return fst_attention(q, k, v, a_idx, a_mask, l_idx, scale, BLOCK_M=m, MAX_ANCESTORS=max_anc,
                             out_dtype=torch.float32, key_splits=5)

    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        step()
        stream.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            out = step()
    for replay in range(3):
        g = torch.Generator().manual_seed(200 + replay)
        q.copy_(torch.randn(q.shape, generator=g).to(q.dtype))
        k[:, :, :prefix].copy_(torch.randn((1, 2, prefix, d), generator=g).to(k.dtype))
        eager = step().clone()
        torch.cuda.synchronize()
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {replay} differs from the eager call"
    want, _ = dense_oracle(q.cpu(), k.cpu(), v.cpu(), cfg.parent, scale, prefix=prefix)
    assert_close(out, want, cfg.dtype, "last replay")


def test_decoding_step_from_probabilities_in_one_graph():
    """Draft-head probabilities -> tree -> depth-first order -> lineage -> kernel inputs -> attention,
    captured once as one HIP graph; every replay reads new probabilities (a different tree) and new
    q/k/v from the same buffers and must match the host-built tree and the oracle."""
    from fstattention_amd import medusa_parents_gpu
    n, depths, topk, m, d, max_anc = 256, 4, 10, 64, 128, 64
    scale = 1.0 / math.sqrt(d)
    probs = torch.from_numpy(trees.medusa_probs(depths, topk, 0.3, 50)).cuda()
    q, k, v = (t.cuda() for t in rand_qkv(1, 2, n, n, d, torch.bfloat16, 50))

    def step():
        status = torch.zeros((1,), dtype=torch.int32, device="cuda")      # one status word for the whole chain
        parent = medusa_parents_gpu(probs, n, status=status)
        perm, rank = dfs_order_gpu(parent, "light_first", check=False, status=status)
        new_parent = renumber_parents_gpu(parent, perm, rank)
        lineage, level = lineage_from_parents_gpu(new_parent, width=depths + 1, check=False, status=status)
        *inputs, status = create_fst_attention_kernel_inputs(lineage, level, m, max_anc, check=False,
                                                             want_bool_mask=False, status=status)
        # tokens arrive in the builder's numbering: into depth-first order and back around the op
        o = fst_attention(q.index_select(2, perm), k.index_select(2, perm), v.index_select(2, perm), *inputs,
                          scale, BLOCK_M=m, MAX_ANCESTORS=max_anc, out_dtype=torch.float32)
        return o.index_select(2, rank), parent, status

    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        step()
        stream.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            out, parent, status = step()
    for replay in range(3):
        probs.copy_(torch.from_numpy(trees.medusa_probs(depths, topk, 0.3, 60 + replay)))
        g = torch.Generator().manual_seed(70 + replay)
        q.copy_(torch.randn(q.shape, generator=g).to(q.dtype))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want_parent = trees.medusa_parents_from_probs(probs.cpu().numpy(), n)
        np.testing.assert_array_equal(parent.cpu().numpy(), want_parent)
        assert int(status.item()) == 0
        want, _ = dense_oracle(q.cpu(), k.cpu(), v.cpu(), want_parent, scale)
        assert_close(out, want, torch.bfloat16, f"replay {replay}")


def test_two_host_threads_on_their_own_streams():
    """Entry points keep no state between calls: two threads, each with its own stream, inputs and
    tree, launching at the same time get their own results."""
    import threading
    cases, results, errors = [], {}, []
    for tid, (index, seed) in enumerate([(2, 1), (3, 2)]):
        cfg = trees.config(index)
        a_idx, a_mask, l_idx, max_anc = oracle_inputs(cfg.parent, cfg.block_m)
        q, k, v = rand_qkv(1, 2, cfg.n_nodes, cfg.n_nodes, cfg.head_dim, cfg.dtype, seed)
        want, _ = dense_oracle(q, k, v, cfg.parent, 0.1)
        cases.append((tid, cfg, [t.cuda() for t in (q, k, v, a_idx, a_mask, l_idx)], max_anc, want))
    torch.cuda.synchronize()

    def work(tid, cfg, dev, max_anc):
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                for _ in range(25):
                    o = fst_attention(*dev, 0.1, BLOCK_M=cfg.block_m, MAX_ANCESTORS=max_anc, out_dtype=torch.float32)
            stream.synchronize()
            results[tid] = o
        except Exception as exc:   # surfaced by the assertion below
            errors.append(exc)

    threads = [threading.Thread(target=work, args=c[:4]) for c in cases]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for tid, cfg, _, _, want in cases:
        assert_close(results[tid], want, cfg.dtype, f"thread {tid}")


def test_rows_without_any_key_give_zero():
    a_idx = torch.full((1, 8), -1, dtype=torch.int64)
    a_mask = torch.zeros((1, 16, 8), dtype=torch.bool)
    l_idx = torch.full((1, 16), -1, dtype=torch.int64)
    l_idx[0, 3] = 3
    q, k, v = rand_qkv(1, 1, 16, 16, 16, torch.float16, 1)
    o, lse = fst_attention(q.cuda(), k.cuda(), v.cuda(), a_idx.cuda(), a_mask.cuda(), l_idx.cuda(), 1.0,
                           BLOCK_M=16, MAX_ANCESTORS=8, return_lse=True)
    assert torch.equal(o[0, 0, 3].cpu(), v[0, 0, 3])
    rest = [r for r in range(16) if r != 3]
    assert (o[0, 0, rest] == 0).all() and torch.isinf(lse[0, rest]).all()


def test_argument_errors():
    q, k, v = (t.cuda() for t in rand_qkv(1, 1, 16, 16, 16, torch.float16, 1))
    a_idx = torch.full((1, 8), -1, dtype=torch.int64).cuda()
    a_mask = torch.zeros((1, 16, 8), dtype=torch.bool).cuda()
    l_idx = torch.arange(16).view(1, 16).cuda()
    fst_attention(q, k, v, a_idx, a_mask, l_idx, 1.0, BLOCK_M=16, MAX_ANCESTORS=8)
    with pytest.raises(AssertionError):     # the reference's assertion on the head dimension
        fst_attention(q[..., :8].contiguous(), k[..., :8].contiguous(), v[..., :8].contiguous(),
                      a_idx, a_mask, l_idx, 1.0, BLOCK_M=16, MAX_ANCESTORS=8)
    with pytest.raises(AssertionError):
        fst_attention(q, k, v[..., :8].contiguous(), a_idx, a_mask, l_idx, 1.0, BLOCK_M=16, MAX_ANCESTORS=8)
    with pytest.raises(ValueError):         # defaults 128 / 64 do not match these tensors
        fst_attention(q, k, v, a_idx, a_mask, l_idx, 1.0)
    with pytest.raises(ValueError):
        fst_attention(q.transpose(1, 2), k, v, a_idx, a_mask, l_idx, 1.0, BLOCK_M=16, MAX_ANCESTORS=8)
    with pytest.raises(ValueError):
        fst_attention(q.cpu(), k.cpu(), v.cpu(), a_idx, a_mask, l_idx, 1.0, BLOCK_M=16, MAX_ANCESTORS=8)
    with pytest.raises(ValueError):
        fst_attention(q, k.float(), v, a_idx, a_mask, l_idx, 1.0, BLOCK_M=16, MAX_ANCESTORS=8)


def test_mask_cache_follows_in_place_edits():
    parent = trees.random_recursive_parents(32, 4)
    a_idx, a_mask, l_idx, max_anc = oracle_inputs(parent, 32)
    q, k, v = (t.cuda() for t in rand_qkv(1, 1, 32, 32, 32, torch.float32, 2))
    a_idx, a_mask, l_idx = a_idx.cuda(), a_mask.cuda(), l_idx.cuda()
    o1 = fst_attention(q, k, v, a_idx, a_mask, l_idx, 0.2, BLOCK_M=32, MAX_ANCESTORS=max_anc)
    a_mask.zero_()                      # now every row only sees itself if it is a leaf
    o2 = fst_attention(q, k, v, a_idx, a_mask, l_idx, 0.2, BLOCK_M=32, MAX_ANCESTORS=max_anc)
    leaf_rows = (l_idx[0] >= 0).nonzero().flatten()
    assert torch.equal(o2[0, 0, leaf_rows], v[0, 0, leaf_rows])
    assert not torch.equal(o1, o2)


def test_non_default_stream():
    cfg = trees.config(1)
    a_idx, a_mask, l_idx, max_anc = oracle_inputs(cfg.parent, cfg.block_m)
    q, k, v = trees.make_qkv(cfg)
    want, _ = dense_oracle(q, k, v, cfg.parent, 0.125)
    dev = [t.cuda() for t in (q, k, v, a_idx, a_mask, l_idx)]
    torch.cuda.synchronize()
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        o = fst_attention(*dev, 0.125, BLOCK_M=cfg.block_m, MAX_ANCESTORS=max_anc)
    s.synchronize()
    assert_close(o, want, torch.float32, "side stream")
