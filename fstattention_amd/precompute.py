"""Block precompute on the GPU: ``create_fst_attention_kernel_inputs``.

Same signature and results as reference ``utils.py:104-129``; the per-block
Python loop is replaced by one launch of an integer HIP kernel, so a tree that
changes every decoding step can be re-chunked without leaving the device.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import _lib
from .attention import PackedTreeMask, _cache_key, _on_device, _stream_ptr, remember_packed


MEDUSA_MAX_CANDIDATES = 1 << 24    # candidate paths the tree builder takes (16384 in one launch, more over a workspace)


def _raise_for_status(status: int, max_ancestors: int):
    if status & _lib.PRE_BAD_NODE_ID:
        raise ValueError("lineage holds a node id outside [-1, n_nodes)")
    if status & _lib.PRE_BAD_LEVEL:
        raise IndexError("level_lookup holds a level outside lineage's columns")
    if status & _lib.PRE_TOO_MANY_ANCESTORS:
        # the reference fails here with a shape-mismatch RuntimeError (utils.py:120)
        raise RuntimeError(f"a block has more than max_ancestors={max_ancestors} unique ancestors")


def create_fst_attention_kernel_inputs(lineage, level_lookup, block_m=64, max_ancestors=32, *,
                                       mutate_lineage: bool = True, check: bool = True,
                                       want_bool_mask: bool = True, device=None, status=None):
    """``(ancestor_idx, ancestor_mask, leaf_idx)`` of reference ``utils.py:104-129``.

    ``ancestor_idx`` int64 ``[NB, max_ancestors]`` (ascending, ``-1`` padded),
    ``ancestor_mask`` bool ``[NB, block_m, max_ancestors]``, ``leaf_idx`` int64
    ``[NB, block_m]``, on the device of ``lineage``.  CPU inputs are staged
    through the GPU (``device`` or the current one) and come back as CPU tensors;
    GPU inputs stay there, and the returned ``ancestor_mask`` carries its packed
    form so ``fst_attention`` does not repack it.  Like the reference the
    caller's ``lineage`` receives each node's id in its own level column unless
    ``mutate_lineage=False``.  ``check`` synchronises to raise the reference's
    ``RuntimeError`` when a block has more than ``max_ancestors`` ancestors;
    with ``check=False`` a 4th value, the device status word, is returned
    instead.  ``want_bool_mask=False`` returns a :class:`PackedTreeMask` in
    place of the bool tensor.  ``status``: a zeroed int32 ``[1]`` tensor on the device to
    collect the status bits in (the stages of a front-end chain can share one, which spares
    each of them the fill of its own).
    """
    if lineage.dim() != 2 or level_lookup.dim() != 1 or level_lookup.shape[0] != lineage.shape[0]:
        raise ValueError(f"lineage {tuple(lineage.shape)} / level_lookup {tuple(level_lookup.shape)}")
    if lineage.dtype != torch.int64 or level_lookup.dtype != torch.int64:
        raise ValueError("lineage and level_lookup must be int64")
    block_m = int(block_m)
    max_ancestors = int(max_ancestors)
    on_host = not lineage.is_cuda
    if on_host:
        if not torch.cuda.is_available():
            raise RuntimeError("create_fst_attention_kernel_inputs runs on the GPU only "
                               "(no CPU fallback) and no GPU is available")
        dev = torch.device(device) if device is not None else torch.device("cuda", torch.cuda.current_device())
    else:
        dev = lineage.device
    lin = lineage.to(dev).contiguous()
    lvl = level_lookup.to(dev).contiguous()
    # one operator call (csrc/fsta_torch_binding.cpp): allocations, stream, device guard and the launch in C++
    a_idx, a_mask, l_idx, bits, count, plan, status = _lib.load_torch_ops().precompute(
        lin, lvl, block_m, max_ancestors, bool(mutate_lineage), bool(want_bool_mask), status)
    if not want_bool_mask:
        a_mask = None
    if plan is not None and plan.numel() == 0:      # (block sizes the matrix-core kernels do not take have no plan)
        plan = None
    if check:
        _raise_for_status(int(status.item()), max_ancestors)
    if mutate_lineage and lin.data_ptr() != lineage.data_ptr():
        lineage.copy_(lin)
    packed = PackedTreeMask(bits, count, block_m, max_ancestors, plan)
    if on_host:
        out = (a_idx.cpu(), a_mask.cpu() if want_bool_mask else packed, l_idx.cpu())
    else:
        key = _cache_key(a_idx, a_mask, l_idx) if want_bool_mask else None
        if key is not None:     # (tensors made in inference mode keep no edit counters: packed per call instead)
            remember_packed(a_mask, key, packed)
        out = (a_idx, a_mask if want_bool_mask else packed, l_idx)
    return out if check else out + (status,)


def kernel_inputs_from_parents_gpu(parent: torch.Tensor, block_m: int, max_ancestors: int, width: int, *,
                                   check: bool = True, want_bool_mask: bool = False, want_lineage: bool = False,
                                   status=None):
    """``parent [N]`` int64 on the GPU -> the kernel inputs of ``create_fst_attention_kernel_inputs`` in ONE launch
    (``fsta_precompute_from_parents``): what ``lineage_from_parents_gpu(parent, width)`` followed by
    ``create_fst_attention_kernel_inputs(lineage, level, block_m, max_ancestors)`` returns, bit for bit, without the
    lineage travelling through memory.  ``width``: columns of the lineage rows, at least the tree's depth + 1.
    Returns ``(ancestor_idx, ancestor_mask or PackedTreeMask, leaf_idx)`` (``want_bool_mask`` as there), followed by
    ``(lineage, level_lookup)`` with ``want_lineage`` (the lineage with the nodes' own ids entered, as the reference's
    function leaves it) and by the device status word with ``check=False``.  Trees whose tables do not fit one
    workgroup's LDS (about 16000 nodes) raise ``libfsta``'s unsupported error: use the two calls."""
    if not parent.is_cuda or parent.dtype != torch.int64 or parent.dim() != 1:
        raise ValueError("parent must be a 1-D int64 tensor on the GPU")
    lib = _lib.load()
    parent = parent.contiguous()
    dev = parent.device
    n, block_m, max_ancestors, width = parent.shape[0], int(block_m), int(max_ancestors), int(width)
    nb = -(-n // block_m)
    a_idx = torch.empty((nb, max_ancestors), dtype=torch.int64, device=dev)
    l_idx = torch.empty((nb, block_m), dtype=torch.int64, device=dev)
    a_mask = torch.empty((nb, block_m, max_ancestors), dtype=torch.bool, device=dev) if want_bool_mask else None
    bits = torch.empty((nb, lib.fsta_mask_words(max_ancestors), block_m), dtype=torch.int32, device=dev)
    count = torch.empty((nb,), dtype=torch.int32, device=dev)
    plan_bytes = lib.fsta_block_plan_bytes(nb, block_m, max_ancestors)
    plan = torch.empty((plan_bytes // 4,), dtype=torch.int32, device=dev) if plan_bytes else None
    lineage = torch.empty((n, width), dtype=torch.int64, device=dev) if want_lineage else None
    level = torch.empty((n,), dtype=torch.int64, device=dev) if want_lineage else None
    if status is None:
        status = torch.zeros((1,), dtype=torch.int32, device=dev)
    ptr = lambda t: t.data_ptr() if t is not None else None
    with _on_device(dev):
        _lib.check(lib.fsta_precompute_from_parents(parent.data_ptr(), n, width, block_m, max_ancestors, 1, ptr(lineage),
                                                    ptr(level), a_idx.data_ptr(), ptr(a_mask), l_idx.data_ptr(),
                                                    bits.data_ptr(), count.data_ptr(), ptr(plan), status.data_ptr(),
                                                    _stream_ptr(dev)))
    if check:
        st = int(status.item())
        if st & _lib.PRE_BAD_LEVEL:
            raise ValueError(f"tree is deeper than width={width}")
        if st & _lib.PRE_BAD_NODE_ID:
            raise ValueError("parent[i] must lie in [-1, i)")
        _raise_for_status(st, max_ancestors)
    packed = PackedTreeMask(bits, count, block_m, max_ancestors, plan)
    if want_bool_mask:
        key = _cache_key(a_idx, a_mask, l_idx)
        if key is not None:
            remember_packed(a_mask, key, packed)
    out = (a_idx, a_mask if want_bool_mask else packed, l_idx)
    if want_lineage:
        out += (lineage, level)
    return out if check else out + (status,)


def lineage_from_parents_gpu(parent: torch.Tensor, width: Optional[int] = None, check: bool = True, status=None):
    """``parent [N]`` int64 on the GPU -> ``(lineage [N, width], level_lookup [N])`` on the GPU.

    Layout of reference ``utils.py:66-75``.  Without ``width`` the levels are
    computed first and ``max(level) + 1`` is read back (one synchronisation).
    ``status``: optional zeroed int32 ``[1]`` device tensor to collect the status bits in.
    """
    if not parent.is_cuda or parent.dtype != torch.int64 or parent.dim() != 1:
        raise ValueError("parent must be a 1-D int64 tensor on the GPU")
    lib = _lib.load()
    parent = parent.contiguous()
    dev = parent.device
    n = parent.shape[0]
    level = torch.empty((n,), dtype=torch.int64, device=dev)
    if status is None:
        status = torch.zeros((1,), dtype=torch.int32, device=dev)
    with _on_device(dev):
        if width is None:
            _lib.check(lib.fsta_lineage_from_parents(parent.data_ptr(), n, 1, None, level.data_ptr(),
                                                     status.data_ptr(), _stream_ptr(dev)))
            width = int(level.max().item()) + 1 if n else 1
        lineage = torch.empty((n, width), dtype=torch.int64, device=dev)
        _lib.check(lib.fsta_lineage_from_parents(parent.data_ptr(), n, width, lineage.data_ptr(),
                                                 level.data_ptr(), status.data_ptr(), _stream_ptr(dev)))
    if check:
        st = int(status.item())
        if st & _lib.PRE_BAD_NODE_ID:
            raise ValueError("parent[i] must lie in [-1, i)")
        if st & _lib.PRE_BAD_LEVEL:
            raise ValueError(f"tree is deeper than width={width}")
    return lineage, level


def dfs_order_gpu(parent: torch.Tensor, children: str = "index", check: bool = True, status=None):
    """``parent [N]`` int64 on the GPU -> ``(perm, rank)`` int64 ``[N]`` on the GPU.

    Device version of ``trees.dfs_order`` (``perm[new] = old``, ``rank[old] = new``) for trees
    that are rebuilt on the GPU every decoding step; no host synchronisation with
    ``check=False``.  ``renumber_parents_gpu`` applies the order to the tree, ``index_select``
    to the token tensors.  ``status``: optional zeroed int32 ``[1]`` device tensor to collect the
    status bits in.
    """
    if not parent.is_cuda or parent.dtype != torch.int64 or parent.dim() != 1:
        raise ValueError("parent must be a 1-D int64 tensor on the GPU")
    if children not in ("index", "light_first"):
        raise ValueError(f"children={children!r}: expected 'index' or 'light_first'")
    lib = _lib.load()
    parent = parent.contiguous()
    dev = parent.device
    n = parent.shape[0]
    perm = torch.empty((n,), dtype=torch.int64, device=dev)
    rank = torch.empty((n,), dtype=torch.int64, device=dev)
    work = torch.empty((_lib.dfs_order_workspace_ints(n),), dtype=torch.int32, device=dev)
    if status is None:
        status = torch.zeros((1,), dtype=torch.int32, device=dev)
    with _on_device(dev):
        _lib.check(lib.fsta_dfs_order(parent.data_ptr(), n, 1 if children == "light_first" else 0,
                                      perm.data_ptr(), rank.data_ptr(), work.data_ptr(),
                                      status.data_ptr(), _stream_ptr(dev)))
    if check and int(status.item()) & _lib.PRE_BAD_NODE_ID:
        raise ValueError("parent[i] must lie in [-1, i)")
    return perm, rank


def renumber_parents_gpu(parent: torch.Tensor, perm: torch.Tensor, rank: torch.Tensor) -> torch.Tensor:
    """Parent array of the same forest after node ``perm[new]`` has been renamed ``new`` (one launch)."""
    if not (parent.is_cuda and rank.is_cuda) or parent.dtype != torch.int64 or rank.dtype != torch.int64 or \
            parent.shape != rank.shape or parent.dim() != 1:
        raise ValueError("parent and rank must be 1-D int64 tensors of one length on the GPU")
    lib = _lib.load()
    parent, rank = parent.contiguous(), rank.contiguous()
    new_parent = torch.empty_like(parent)
    with _on_device(parent.device):
        _lib.check(lib.fsta_renumber_parents(parent.data_ptr(), rank.data_ptr(), parent.shape[0],
                                             new_parent.data_ptr(), _stream_ptr(parent.device)))
    return new_parent


def medusa_parents_gpu(probs: torch.Tensor, n: int, check: bool = False, status=None) -> torch.Tensor:
    """``probs [depths, topk]`` on the GPU -> parent array int64 ``[n]`` on the GPU, no host round trip.

    Device version of ``trees.medusa_parents_from_probs`` (same selection, same tie-breaks, same
    numbering): a path of ranks ``(r1..rd)`` scores the product of its ranks' probabilities, the
    ``n-1`` best paths are kept (ties: shallower first, then smaller ranks) and numbered by
    ``(depth, ranks)``; node 0 is the empty path.  Scores are formed in float64 in the host
    version's multiplication order.  One launch of a HIP kernel on the current stream
    (``fsta_medusa_tree``) for up to 16384 candidate paths = sum of ``topk**d``, e.g. four heads of 10
    ranks or three of 24; larger sets (up to 2**24 paths, e.g. five or six heads of 10 ranks) go
    through ``fsta_medusa_tree_ws``: the same selection in about a dozen launches over a workspace
    of 8 bytes per path taken from torch's allocator.  With ``dfs_order_gpu``,
    ``lineage_from_parents_gpu(width=depths + 1)`` and
    ``create_fst_attention_kernel_inputs(check=False)`` a tree goes from draft-head probabilities
    to kernel inputs without touching the host.  ``check`` synchronises and raises when a kept
    path's prefix was not kept (probabilities above 1 or not numbers).  ``status``: optional zeroed
    int32 ``[1]`` device tensor to collect the status bits in.
    """
    if probs.dim() != 2 or not probs.is_cuda:
        raise ValueError("probs must be a [depths, topk] tensor on the GPU")
    depths, topk = probs.shape
    total = sum(topk ** d for d in range(1, depths + 1))
    if not 1 <= n <= total + 1:
        raise ValueError(f"n={n} outside [1, {total + 1}] for depths={depths}, topk={topk}")
    if total > MEDUSA_MAX_CANDIDATES or depths * topk > 1024:
        raise ValueError(f"depths={depths}, topk={topk} give {total} candidate paths; the tree builder takes at most "
                         f"{MEDUSA_MAX_CANDIDATES} and depths * topk <= 1024")
    if probs.dtype not in (torch.float32, torch.float64):
        probs = probs.to(torch.float64)
    probs = probs.contiguous()
    lib = _lib.load()
    dev = probs.device
    parent = torch.empty((n,), dtype=torch.int64, device=dev)
    if status is None:
        status = torch.zeros((1,), dtype=torch.int32, device=dev)
    code = _lib.F32 if probs.dtype == torch.float32 else _lib.F64
    need = lib.fsta_medusa_workspace_bytes(depths, topk)
    with _on_device(dev):
        if need:
            work = torch.empty((need,), dtype=torch.uint8, device=dev)     # (stream-ordered: free again after the launches)
            _lib.check(lib.fsta_medusa_tree_ws(probs.data_ptr(), code, depths, topk, n, parent.data_ptr(), status.data_ptr(),
                                               work.data_ptr(), need, _stream_ptr(dev)))
        else:
            _lib.check(lib.fsta_medusa_tree(probs.data_ptr(), code, depths, topk, n, parent.data_ptr(), status.data_ptr(),
                                            _stream_ptr(dev)))
    if check and int(status.item()) & _lib.TREE_NOT_PREFIX_CLOSED:
        raise ValueError("the kept paths are not closed under prefixes (probabilities above 1 or not numbers)")
    return parent
