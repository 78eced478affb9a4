"""Dense-masked attention oracle (test infrastructure only).

Restates the check of reference ``fstattention.py:214-219``: scores
``(q @ k^T) * sm_scale``, disallowed pairs set to ``-inf``, softmax over keys,
times ``v``.  The reference evaluates it in fp16 on the GPU; here the inputs
(already rounded to their storage dtype) are upcast and the arithmetic runs in
float64 or float32 so that the oracle carries no rounding of its own.
"""
from __future__ import annotations

import math

import numpy as np
import torch


def full_mask_with_prefix(tree_mask: np.ndarray, prefix: int) -> np.ndarray:
    """``[N, prefix + N]``: every query sees the whole shared prefix
    (reference ``fstattention.py:207-209``)."""
    n = tree_mask.shape[0]
    if prefix == 0:
        return tree_mask
    return np.concatenate([np.ones((n, prefix), dtype=np.bool_), tree_mask], axis=1)


def dense_tree_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, mask,
                         sm_scale: float, dtype=torch.float64, head_chunk: int = 8):
    """``softmax(where(mask, q k^T * scale, -inf)) v`` -> ``(o, lse2)``.

    ``q [Z,H,Nq,D]``, ``k,v [Z,H,Nk,D]``, ``mask`` bool ``[Nq,Nk]`` shared by all
    heads.  ``o`` comes back in ``dtype``; ``lse2`` is the base-2 log-sum-exp of
    the scaled scores times ``log2 e`` (reference ``fstattention.py:59,141``).
    Rows whose mask is empty give ``o = 0`` and ``lse2 = -inf``.
    """
    mask = torch.as_tensor(np.asarray(mask), dtype=torch.bool)
    z, h, nq, d = q.shape
    o = torch.empty((z, h, nq, v.shape[-1]), dtype=dtype)
    lse = torch.empty((z, h, nq), dtype=dtype)
    qf = q.reshape(z * h, nq, d)
    kf = k.reshape(z * h, k.shape[2], d)
    vf = v.reshape(z * h, v.shape[2], v.shape[-1])
    of = o.view(z * h, nq, -1)
    lf = lse.view(z * h, nq)
    for s in range(0, z * h, head_chunk):
        qq = qf[s: s + head_chunk].to(dtype)
        kk = kf[s: s + head_chunk].to(dtype)
        vv = vf[s: s + head_chunk].to(dtype)
        scores = torch.matmul(qq, kk.transpose(1, 2)) * sm_scale
        scores = scores.masked_fill(~mask, float("-inf"))
        mx = scores.max(dim=-1, keepdim=True).values
        mx = torch.where(torch.isinf(mx), torch.zeros_like(mx), mx)
        p = torch.exp(scores - mx)
        denom = p.sum(dim=-1, keepdim=True)
        out = torch.matmul(p, vv) / torch.where(denom == 0, torch.ones_like(denom), denom)
        of[s: s + head_chunk] = out
        lf[s: s + head_chunk] = ((mx + torch.log(denom)) / math.log(2.0)).squeeze(-1)
    return o, lse


def lse_base2(scores: torch.Tensor) -> torch.Tensor:
    """``log2 sum_k 2^(s_k * log2 e)`` over the last axis (``-inf`` entries ignored)."""
    return torch.logsumexp(scores, dim=-1) / math.log(2.0)


def scalar_tree_attention(q, k, v, parent, sm_scale: float, prefix: int = 0):
    """Double loop in Python floats for one head; only for tiny inputs.

    ``q [N,D]``, ``k,v [prefix+N,D]`` nested lists or arrays.  Query ``i`` sees
    keys ``0..prefix-1``, itself and its ancestors (shifted by ``prefix``).
    """
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    n, d = q.shape
    out = np.zeros((n, v.shape[1]))
    for i in range(n):
        keys = list(range(prefix)) + [prefix + i]
        p = int(parent[i])
        while p >= 0:
            keys.append(prefix + p)
            p = int(parent[p])
        s = [sum(q[i, c] * k[j, c] for c in range(d)) * sm_scale for j in keys]
        mx = max(s)
        w = [math.exp(x - mx) for x in s]
        tot = sum(w)
        for wj, j in zip(w, keys):
            out[i] += (wj / tot) * v[j]
    return out
