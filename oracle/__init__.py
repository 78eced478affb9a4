"""CPU oracle for the fused sparse tree attention path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this; only
``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may, and only as the checker.

Contents and how each function is pinned (a check that would fail on a
plausible mistake, not a retyping of the same formula):

* ``tree_precompute.block_inputs``   restates reference ``utils.py:104-129``.
  Pinned by (a) golden fixtures written by the reference's own
  ``utils.create_fst_attention_kernel_inputs`` on CPU (``tests/golden``),
  including ragged last blocks and the in-place lineage write; (b) rebuilding
  the dense ancestor-or-self mask from its three outputs and comparing with a
  pointer-walk over the parent array; (c) a brute-force set formulation on
  random trees.
* ``tree_precompute.dense_tree_mask``  pointer walk over ``parent``; pinned by
  the transitive-closure identity and by the reference's
  ``create_full_attention_mask`` fixture.
* ``dense_attention.dense_tree_attention`` restates the dense-masked oracle of
  reference ``fstattention.py:214-219`` in float64/float32.  Pinned by
  ``torch.nn.functional.scaled_dot_product_attention`` (library routine), by the
  chain tree = causal attention special case, by roots returning their own V
  row, by equal keys giving the plain mean of the allowed V rows, and by a
  scalar double loop on tiny inputs.
* ``dense_attention.lse_base2``  base-2 log-sum-exp of reference
  ``fstattention.py:59,139-141``; pinned by ``torch.logsumexp / ln 2``.

The bit-level numerics of the reference's Triton kernel (tf32 dots, exp2
approximation, fp16 rounding of the pre-scaled Q) have no runnable oracle in
this build: the kernel needs a CUDA device and triton-nightly
2.1.0.post20240108192258, neither of which exists here.  For those bits:
parity unpinned; parity is defined, as in the reference's own test, against the
dense-masked attention.
"""
