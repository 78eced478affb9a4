"""Fused sparse tree attention for AMD MI355X (gfx950).

Public names mirror the reference's two modules: ``fst_attention``
(``fstattention.py:153``) and ``create_fst_attention_kernel_inputs``,
``create_tree``, ``create_full_attention_mask``, ``DEPTH_MAPPING``,
``MAX_ANCESTOR_MAPPING`` (``utils.py``).  Compute runs in ``libfsta.so``
(hand-written HIP, C ABI in ``include/fsta.h``); there is no CPU fallback.
"""
from .attention import (PackedTreeMask, fst_attention, merge_attention_states, pack_tree_mask,
                        quantize_kv_fp8, shift_for_prefix)
from .precompute import (create_fst_attention_kernel_inputs, dfs_order_gpu, kernel_inputs_from_parents_gpu,
                         lineage_from_parents_gpu, medusa_parents_gpu, renumber_parents_gpu)
from .trees import (DEPTH_MAPPING, MAX_ANCESTOR_MAPPING, create_full_attention_mask, create_tree,
                    dfs_order, lineage_from_parents, renumber_parents)

__all__ = [
    "fst_attention", "create_fst_attention_kernel_inputs", "create_tree",
    "create_full_attention_mask", "DEPTH_MAPPING", "MAX_ANCESTOR_MAPPING",
    "PackedTreeMask", "pack_tree_mask", "shift_for_prefix", "lineage_from_parents",
    "lineage_from_parents_gpu", "dfs_order", "renumber_parents", "dfs_order_gpu", "renumber_parents_gpu", "merge_attention_states", "medusa_parents_gpu", "quantize_kv_fp8",
    "kernel_inputs_from_parents_gpu",
]
