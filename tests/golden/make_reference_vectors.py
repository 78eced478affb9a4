"""Writes ``reference_vectors.npz``: outputs of the reference's CPU tree helpers.

Run once, in the build container only (the reference checkout is not available
anywhere else):

    python tests/golden/make_reference_vectors.py

It imports the reference's ``utils`` module (CPU torch only; the module with the
GPU kernel is never imported) and records, for a handful of trees, what
``create_tree``, ``create_full_attention_mask`` and
``create_fst_attention_kernel_inputs`` return, plus the lineage as that last
call leaves it.  These pin behaviour no identity fixes: the exact column
placement of ``create_tree``, leaves of a ragged last block pointing past the
tree, the in-place self entries, and the padded float mask.  Inputs for the
arbitrary-tree cases come from this repository's own generators, so the file
holds data only: inputs and the reference's outputs.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
REPO = os.path.dirname(os.path.dirname(HERE))
REFERENCE = os.environ.get("FSTA_REFERENCE_DIR", "/root/reference")


def main():
    sys.path.insert(0, REFERENCE)
    import utils as ref  # the reference's CPU helpers
    sys.path.insert(0, REPO)
    from fstattention_amd import trees

    out = {}
    cases = []

    def record(name, lineage, level_lookup, block_m, max_anc, full_mask=False):
        lineage = lineage.clone()
        out[f"{name}/lineage_in"] = lineage.numpy().copy()
        out[f"{name}/level_lookup"] = level_lookup.numpy().copy()
        if full_mask:
            out[f"{name}/full_mask"] = ref.create_full_attention_mask(lineage).numpy().copy()
        a_idx, a_mask, l_idx = ref.create_fst_attention_kernel_inputs(
            lineage, level_lookup, block_m=block_m, max_ancestors=max_anc)
        out[f"{name}/ancestor_idx"] = a_idx.numpy()
        out[f"{name}/ancestor_mask"] = a_mask.numpy()
        out[f"{name}/leaf_idx"] = l_idx.numpy()
        out[f"{name}/lineage_out"] = lineage.numpy().copy()
        out[f"{name}/params"] = np.array([block_m, max_anc], dtype=np.int64)
        cases.append(name)

    # the reference's own tree generator
    for depth, topk, lwf, block_m, max_anc in [
        (3, 4, 0.5, 16, 16),     # 60 nodes, ragged last block
        (5, 4, 0.5, 64, 32),     # 252 nodes, ragged
        (5, 4, 0.5, 128, 64),
        (7, 4, 0.5, 128, 64),    # 1020 nodes
        (8, 4, 0.5, 128, 64),    # 2044 nodes: the reference test's tree
        (4, 3, 0.7, 32, 32),     # other branching / weight
    ]:
        lineage, level_lookup = ref.create_tree(depth=depth, topk=topk, left_weight_factor=lwf)
        name = f"create_tree_d{depth}_k{topk}_f{lwf}_m{block_m}_a{max_anc}"
        out[f"{name}/tree_args"] = np.array([depth, topk, lwf], dtype=np.float64)
        record(name, lineage, level_lookup, block_m, max_anc, full_mask=depth <= 5)

    # arbitrary trees from this repository's generators, through the reference precompute
    for name, parent, block_m in [
        ("cfg1_random64", trees.config(1).parent, 16),
        ("cfg2_medusa256", trees.config(2).parent, 64),
        ("cfg3_deep1024", trees.config(3).parent, 64),
        ("random100_ragged", trees.random_recursive_parents(100, 7), 32),
        ("window300_ragged", trees.random_recursive_parents(300, 8, window=16), 128),
        ("forest50", np.where(np.arange(50) < 5, -1,
                               trees.random_recursive_parents(50, 9)), 16),
    ]:
        lineage, level_lookup = trees.lineage_from_parents(parent)
        max_anc = trees.required_max_ancestors(parent, block_m, 16)
        out[f"{name}/parent"] = np.asarray(parent, dtype=np.int64)
        record(name, lineage, level_lookup, block_m, max_anc)

    out["cases"] = np.array(cases)
    path = os.path.join(HERE, "reference_vectors.npz")
    np.savez_compressed(path, **out)
    print(f"wrote {path}: {len(cases)} cases, {os.path.getsize(path)} bytes")


if __name__ == "__main__":
    main()
