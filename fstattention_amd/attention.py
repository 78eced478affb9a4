"""``fst_attention``: the operator of reference ``fstattention.py:153-181`` on MI355X.

Same positional signature, same tensor layouts, same two assertions.  The body
hands raw device pointers to ``libfsta.so`` (hand-written HIP for gfx950) on the
current torch stream; torch only owns the memory.
"""
from __future__ import annotations

import weakref
from typing import NamedTuple, Optional

import torch

from . import _lib

_DTYPES = {torch.float32: _lib.F32, torch.float16: _lib.F16, torch.bfloat16: _lib.BF16}


class PackedTreeMask(NamedTuple):
    """Kernel-ready form of the per-block inputs.

    ``mask_bits`` uint32-as-int32 ``[NB, ceil(A/32), M]`` (bit ``b`` of word ``w``
    of row ``r`` = ``ancestor_mask[j, r, 32*w + b]``), ``anc_count`` int32 ``[NB]``.
    ``plan`` (int32, or ``None`` for block sizes other than 32/64/128): the block plan of
    ``include/fsta.h`` -- 32-bit K/V rows of every ancestor and leaf slot, leaf validity and the
    mask words, per block, in the order the matrix-core kernel consumes them; it belongs to the
    ``ancestor_idx`` / ``leaf_idx`` it was made from.  ``key_shift``: what has been added to the
    valid entries of those tensors since (``shift_for_prefix``); the kernel adds it to the plan's
    keys.  ``key_limit``: ids at or above it were treated as empty slots when the plan was made
    (``None``: the plan comes from the tree precompute and holds tree nodes only).
    """
    mask_bits: torch.Tensor
    anc_count: torch.Tensor
    block_m: int
    max_ancestors: int
    plan: Optional[torch.Tensor] = None
    key_shift: int = 0
    key_limit: Optional[int] = None


def _stream_ptr(device) -> int:
    """Raw handle of torch's current stream on `device` (the C accessor; the Python stream object
    costs several microseconds per call)."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    try:
        return torch._C._cuda_getCurrentRawStream(index)
    except AttributeError:      # accessor missing in this torch build
        return torch.cuda.current_stream(device).cuda_stream


class _on_device:
    """``with`` block that makes `device` current only when it is not already."""

    def __init__(self, device):
        self.index = device.index
        self.prev = None

    def __enter__(self):
        if self.index is not None and self.index != torch.cuda.current_device():
            self.prev = torch.cuda.current_device()
            torch.cuda.set_device(self.index)

    def __exit__(self, *exc):
        if self.prev is not None:
            torch.cuda.set_device(self.prev)
        return False


def pack_tree_mask(ancestor_idx: torch.Tensor, ancestor_mask: torch.Tensor,
                   leaf_idx: Optional[torch.Tensor] = None, key_limit: Optional[int] = None) -> PackedTreeMask:
    """bool ``[NB, M, A]`` mask (+ ``ancestor_idx`` for the ``-1`` slots) -> packed bits; with
    ``leaf_idx`` ``[NB, M]`` (and a block size of 32, 64 or 128) also the block plan, in which
    ids outside ``[0, key_limit)`` count as empty slots (``key_limit``: rows of K/V)."""
    if not ancestor_mask.is_cuda or not ancestor_idx.is_cuda:
        raise ValueError("pack_tree_mask needs tensors on the GPU")
    if ancestor_mask.dtype != torch.bool or ancestor_idx.dtype != torch.int64:
        raise ValueError("ancestor_mask must be bool and ancestor_idx int64")
    if ancestor_mask.dim() != 3 or ancestor_idx.dim() != 2 or \
            ancestor_idx.shape != (ancestor_mask.shape[0], ancestor_mask.shape[2]):
        raise ValueError(f"shape mismatch: ancestor_idx {tuple(ancestor_idx.shape)}, "
                         f"ancestor_mask {tuple(ancestor_mask.shape)}")
    lib = _lib.load()
    nb, m, a = ancestor_mask.shape
    ancestor_mask = ancestor_mask.contiguous()
    ancestor_idx = ancestor_idx.contiguous()
    dev = ancestor_mask.device
    words = (a + 31) // 32
    bits = torch.empty((nb, words, m), dtype=torch.int32, device=dev)
    count = torch.empty((nb,), dtype=torch.int32, device=dev)
    plan, limit = None, None
    plan_bytes = lib.fsta_block_plan_bytes(nb, m, a) if leaf_idx is not None and a <= 16384 else 0
    if plan_bytes:
        if leaf_idx.dtype != torch.int64 or tuple(leaf_idx.shape) != (nb, m) or leaf_idx.device != dev:
            raise ValueError(f"leaf_idx must be int64 [{nb}, {m}] on {dev}")
        leaf_idx = leaf_idx.contiguous()
        plan = torch.empty((plan_bytes // 4,), dtype=torch.int32, device=dev)
        limit = _MAX_KEY if key_limit is None else min(int(key_limit), _MAX_KEY)
    with _on_device(dev):
        _lib.check(lib.fsta_pack_mask(ancestor_idx.data_ptr(), ancestor_mask.data_ptr(),
                                      leaf_idx.data_ptr() if plan is not None else None, nb, m, a,
                                      limit if plan is not None else 0, bits.data_ptr(), count.data_ptr(),
                                      plan.data_ptr() if plan is not None else None, _stream_ptr(dev)))
    return PackedTreeMask(bits, count, m, a, plan, 0, limit)


_MAX_KEY = 2 ** 31 - 1


def _version(t: torch.Tensor):
    """torch's in-place edit counter of `t`, or None for tensors that keep none (tensors made
    under ``torch.inference_mode()``)."""
    try:
        return t._version
    except RuntimeError:
        return None


def _cache_key(ancestor_idx, ancestor_mask, leaf_idx):
    """What a packed copy remembered for ``ancestor_mask`` was made from, or None when in-place edits of
    one of the three tensors could not be noticed."""
    versions = (_version(ancestor_mask), _version(ancestor_idx), _version(leaf_idx))
    if None in versions:
        return None
    return versions + (ancestor_idx.data_ptr(), leaf_idx.data_ptr(), tuple(ancestor_mask.shape))


# Packed copies of bool masks, by the identity of the mask tensor: id -> (weak reference, key, packed).  The
# entry goes when the tensor does (weakref.finalize), so nothing is kept alive and nothing is hung on the
# caller's objects.
_PACKED: dict = {}


def remember_packed(ancestor_mask: torch.Tensor, key, packed: PackedTreeMask) -> None:
    """Notes `packed` as the packed form of the bool tensor `ancestor_mask` in the state `key` describes."""
    ident = id(ancestor_mask)
    if ident not in _PACKED or _PACKED[ident][0]() is not ancestor_mask:
        weakref.finalize(ancestor_mask, _PACKED.pop, ident, None)
    _PACKED[ident] = (weakref.ref(ancestor_mask), key, packed)


def recall_packed(ancestor_mask: torch.Tensor):
    """(key, packed) noted for this very tensor object, or None."""
    entry = _PACKED.get(id(ancestor_mask))
    if entry is None or entry[0]() is not ancestor_mask:
        return None
    return entry[1], entry[2]


def _packed_for(ancestor_idx: torch.Tensor, ancestor_mask, leaf_idx: torch.Tensor, nk: int) -> PackedTreeMask:
    """Packed mask and block plan of a bool tensor, remembered per tensor object.

    The kernel inputs are built once per decoding step and reused by every
    layer; the packed copy is kept in a module-level table under the identity of ``ancestor_mask``
    (dropped with the tensor) and replaced when one of the three tensors has been written to since
    (torch's version counters), ``ancestor_idx`` or ``leaf_idx`` is a different tensor, or K/V have
    another number of rows than the plan was made for.  Tensors without version counters (inference
    mode) are packed on every call; pass a :class:`PackedTreeMask` to avoid that.
    """
    if isinstance(ancestor_mask, PackedTreeMask):
        return ancestor_mask
    key = _cache_key(ancestor_idx, ancestor_mask, leaf_idx)
    cached = recall_packed(ancestor_mask) if key is not None else None
    if cached is not None and cached[0] == key and cached[1].key_limit in (None, nk):
        return cached[1]
    packed = pack_tree_mask(ancestor_idx, ancestor_mask, leaf_idx, nk)
    if key is not None:
        remember_packed(ancestor_mask, key, packed)
    return packed


_FP8 = torch.float8_e4m3fn
_FP8_MAX = 448.0


def quantize_kv_fp8(k: torch.Tensor, v: torch.Tensor):
    """``k, v [Z,H,Nk,D]`` -> ``(k8, v8, k_scale, v_scale)`` for ``fst_attention``'s 8-bit K/V storage:
    ``float8_e4m3fn`` tensors and one float32 scale per (batch, head) slice (``[Z*H]``) chosen so that
    the slice's largest magnitude maps to the format's largest value (448).  ``k8 * k_scale`` is the K
    the kernel computes with.  Plain tensor operations; a model would write its KV cache this way."""
    def one(t):
        amax = t.float().abs().amax(dim=(2, 3))
        scale = torch.where(amax > 0, amax / _FP8_MAX, torch.ones_like(amax))
        t8 = (t.float() / scale[:, :, None, None]).to(_FP8)
        return t8.contiguous(), scale.reshape(-1).contiguous()
    k8, k_scale = one(k)
    v8, v_scale = one(v)
    return k8, v8, k_scale, v_scale


def fst_attention(q, k, v, ancestor_idx, ancestor_mask, leaf_idx, sm_scale,
                  BLOCK_M=128, MAX_ANCESTORS=64, *, out_dtype: Optional[torch.dtype] = None,
                  return_lse: bool = False, fast_pv: bool = False, generic: bool = False,
                  wide_waves: bool = False, key_splits: Optional[int] = None, share_tiles: bool = False,
                  k_scale: Optional[torch.Tensor] = None, v_scale: Optional[torch.Tensor] = None,
                  stream_blocks: bool = False):
    """Fused sparse tree attention forward (reference ``fstattention.py:153-181``).

    ``q [Z,H,Nq,D]``, ``k,v [Z,H,Nk,D]`` (``Nk - Nq`` leading rows are a dense
    prefix every query sees), ``ancestor_idx`` int64 ``[NB, MAX_ANCESTORS]``,
    ``ancestor_mask`` bool ``[NB, BLOCK_M, MAX_ANCESTORS]`` (or a
    :class:`PackedTreeMask`), ``leaf_idx`` int64 ``[NB, BLOCK_M]``; returns
    ``o`` shaped and typed like ``q``.

    Beyond the reference: ``out_dtype=torch.float32`` keeps the output
    unrounded, ``return_lse`` also returns the base-2 log-sum-exp ``[Z*H, Nq]``
    the reference computes and drops (``fstattention.py:139-141,181``),
    ``fast_pv`` trades accuracy of the bf16 weights for matrix-core time,
    ``generic`` forces the scalar kernel and ``wide_waves`` the matrix-core variant
    with 32 instead of 16 query rows per wave.  A long shared prefix in front of few
    query blocks is cut into runs of keys that separate workgroups take (the partial
    results live in a temporary workspace and are joined by a second kernel);
    ``key_splits`` forces the number of runs (``1``: never split); ``share_tiles`` is a tuning
    switch (wave pairs of a row group take alternate key tiles even where the library would let
    them share the head dimension); ``stream_blocks`` selects, wherever the shape allows (blocks of 64 or 128
    rows, head dim 64 or 128, no prefix), the kernel whose workgroups stay and walk a list of query blocks
    (measured slower than one workgroup per block; kept as a tested alternative).  ``k`` and ``v`` may be ``torch.float8_e4m3fn`` (8-bit K/V
    storage, half the K/V bytes; ``q`` stays float16/bfloat16) with ``k_scale`` / ``v_scale`` float32
    ``[Z*H]`` per-slice scales (``quantize_kv_fp8`` makes all four): the result is that of the 16-bit
    call on ``k * k_scale`` and ``v * v_scale``; block sizes 32/64/128 and head dims 64/128 only, and
    none of the kernel-selection switches apply.  Inputs the reference silently
    mis-handles raise ``ValueError`` here (non-contiguous tensors, index
    tensors whose shapes do not match ``BLOCK_M`` / ``MAX_ANCESTORS``).
    """
    # shape constraints (the reference's two assertions)
    Lq, Lk, Lv = q.shape[-1], k.shape[-1], v.shape[-1]
    assert Lq == Lk and Lk == Lv
    assert Lk in {16, 32, 64, 128}
    if isinstance(ancestor_mask, PackedTreeMask):
        if (ancestor_mask.block_m, ancestor_mask.max_ancestors) != (BLOCK_M, MAX_ANCESTORS):
            raise ValueError("packed mask was built for another block size / ancestor count")
        packed = ancestor_mask
        # A plan made by the tree precompute names tree nodes; with K/V laid out as [prefix | tree] the
        # only shift that makes it agree with index tensors shifted by ``shift_for_prefix`` is the
        # prefix length.  Shifted tensors passed with the unshifted packed inputs (the third return
        # value of ``shift_for_prefix`` dropped) would otherwise gather prefix rows as ancestors in
        # the kernels that read the plan and the right rows in those that read the lists.
        if packed.plan is not None and packed.key_limit is None and q.dim() == 4 and k.dim() == 4 and \
                packed.key_shift != k.shape[2] - q.shape[2]:
            raise ValueError(f"packed kernel inputs carry key_shift={packed.key_shift} but k has "
                             f"{k.shape[2] - q.shape[2]} prefix rows in front of the tree: pass the third value "
                             "returned by shift_for_prefix(ancestor_idx, leaf_idx, prefix, packed)")
    else:
        if ancestor_mask.dim() != 3 or ancestor_mask.shape[1] != BLOCK_M or ancestor_mask.shape[2] != MAX_ANCESTORS or \
                ancestor_mask.shape[0] != ancestor_idx.shape[0]:
            raise ValueError(f"ancestor_mask is {tuple(ancestor_mask.shape)}, expected "
                             f"({ancestor_idx.shape[0]}, {BLOCK_M}, {MAX_ANCESTORS})")
        if q.dim() != 4 or k.dim() != 4:
            raise ValueError("q, k, v must be [batch, heads, seq, head_dim]")
        packed = _packed_for(ancestor_idx, ancestor_mask, leaf_idx, k.shape[2])
    out_code = _DTYPES.get(out_dtype or q.dtype)
    if out_code is None:
        raise ValueError("q must be float32/float16/bfloat16 and out_dtype the input dtype or torch.float32")
    flags = 0
    if fast_pv or generic or wide_waves or key_splits or share_tiles or stream_blocks:
        flags = (_lib.FLAG_FAST_PV if fast_pv else 0) | (_lib.FLAG_GENERIC if generic else 0) | \
            (_lib.FLAG_WIDE_WAVES if wide_waves else 0) | (_lib.flag_key_splits(key_splits) if key_splits else 0) | \
            (_lib.FLAG_SHARE_TILES if share_tiles else 0) | \
            (_lib.FLAG_STREAM if stream_blocks else 0)
    # everything else (the remaining checks, o and L, the workspace of key runs, the launch on the current stream)
    # happens in the registered operator, csrc/fsta_torch_binding.cpp
    o, lse = (_OPS or _ops()).attention_fwd(q, k, v, ancestor_idx, packed.mask_bits, packed.anc_count, leaf_idx, packed.plan,
                                            packed.key_shift, float(sm_scale), BLOCK_M, MAX_ANCESTORS, out_code, return_lse, flags,
                                            k_scale, v_scale)
    return (o, lse) if return_lse else o


_OPS = None


def _ops():
    global _OPS
    _OPS = _lib.load_torch_ops()
    return _OPS


def shift_for_prefix(ancestor_idx: torch.Tensor, leaf_idx: torch.Tensor, prefix: int,
                     packed: Optional[PackedTreeMask] = None):
    """Index tensors for K/V laid out as ``[prefix | tree]``.

    The reference's caller adds the prefix length to every entry
    (``fstattention.py:211-212``), which turns the ``-1`` sentinels into the
    valid row ``prefix-1``; this shifts real entries only.  With ``packed`` (the
    :class:`PackedTreeMask` that belongs to the two tensors) a third value is returned: the same
    packed inputs with the shift noted, so that they stay valid for the shifted tensors.
    """
    shifted = (torch.where(ancestor_idx >= 0, ancestor_idx + prefix, ancestor_idx),
               torch.where(leaf_idx >= 0, leaf_idx + prefix, leaf_idx))
    if packed is None:
        return shifted
    limit = None if packed.key_limit is None else packed.key_limit + prefix
    return shifted + (packed._replace(key_shift=packed.key_shift + prefix, key_limit=limit),)


def merge_attention_states(o_a: torch.Tensor, lse_a: torch.Tensor, o_b: torch.Tensor, lse_b: torch.Tensor):
    """Joins two partial attention results of the same queries over disjoint key sets.

    ``o_*`` ``[..., Nq, D]`` (same dtype and shape), ``lse_*`` float32 with one entry per row
    of ``o_*`` in the same order: the base-2 log-sum-exp that ``fst_attention(...,
    return_lse=True)`` returns (reference ``fstattention.py:139-141``).  Returns ``(o, lse)``
    of the attention over the union of the key sets.  Typical use: the tree part from
    ``fst_attention`` with ``Nk == Nq`` and the dense shared prefix (reference
    ``fstattention.py:113-136``) from a kernel that reads a paged KV cache.
    """
    if o_a.shape != o_b.shape or o_a.dtype != o_b.dtype or o_a.dtype not in _DTYPES:
        raise ValueError("o_a and o_b must have the same shape and a dtype of float32/float16/bfloat16")
    if not (o_a.is_cuda and o_b.is_cuda and lse_a.is_cuda and lse_b.is_cuda):
        raise ValueError("merge_attention_states runs on the GPU only")
    d = o_a.shape[-1]
    rows = o_a.numel() // d if d else 0
    if lse_a.numel() != rows or lse_b.numel() != rows:
        raise ValueError(f"lse tensors need one entry per row ({rows}), got {lse_a.numel()} and {lse_b.numel()}")
    if lse_a.dtype != torch.float32 or lse_b.dtype != torch.float32:
        raise ValueError("lse tensors must be float32")
    if d % 8:
        raise ValueError(f"head dim {d} is not a multiple of 8")
    lib = _lib.load()
    o_a, o_b, lse_a, lse_b = o_a.contiguous(), o_b.contiguous(), lse_a.contiguous(), lse_b.contiguous()
    o = torch.empty_like(o_a)
    lse = torch.empty_like(lse_a)
    with _on_device(o_a.device):
        _lib.check(lib.fsta_merge_states(o_a.data_ptr(), lse_a.data_ptr(), o_b.data_ptr(), lse_b.data_ptr(),
                                         o.data_ptr(), lse.data_ptr(), rows, d, _DTYPES[o_a.dtype],
                                         _stream_ptr(o_a.device)))
    return o, lse
