"""Host logic of the packed-input cache that ``fst_attention`` keeps on ``ancestor_mask`` (no GPU)."""
import torch

from fstattention_amd.attention import PackedTreeMask, _cache_key, _version, shift_for_prefix


def _lists():
    idx = torch.full((2, 8), -1, dtype=torch.int64)
    idx[0, :3] = torch.tensor([0, 1, 5])
    mask = torch.zeros((2, 32, 8), dtype=torch.bool)
    leaf = torch.arange(64).view(2, 32).clone()
    leaf[0, 1] = -1
    return idx, mask, leaf


def test_key_follows_in_place_edits_and_tensor_identity():
    idx, mask, leaf = _lists()
    key = _cache_key(idx, mask, leaf)
    assert key is not None and key == _cache_key(idx, mask, leaf)
    leaf[0, 2] = -1
    assert _cache_key(idx, mask, leaf) != key          # an edited leaf list makes a new plan
    key = _cache_key(idx, mask, leaf)
    assert _cache_key(idx.clone(), mask, leaf) != key  # another tensor (e.g. shifted by a prefix)
    mask[0, 0, 0] = True
    assert _cache_key(idx, mask, leaf) != key


def test_inference_tensors_are_never_cached():
    """Tensors made under inference mode raise on ``_version``; they are packed per call."""
    with torch.inference_mode():
        idx, mask, leaf = _lists()
        assert _version(mask) is None
        assert _cache_key(idx, mask, leaf) is None
    idx2, mask2, leaf2 = _lists()
    assert _cache_key(idx2, mask, leaf2) is None and _cache_key(idx, mask2, leaf2) is None


def test_prefix_shift_travels_with_the_packed_inputs():
    idx, mask, leaf = _lists()
    packed = PackedTreeMask(torch.zeros(1), torch.zeros(1), 32, 8, torch.zeros(1), 0, 64)
    a, l, shifted = shift_for_prefix(idx, leaf, 100, packed)
    assert shifted.key_shift == 100 and shifted.key_limit == 164 and shifted.plan is packed.plan
    assert a[0, 0] == 100 and a[0, 3] == -1 and l[0, 1] == -1 and l[0, 0] == 100
    assert len(shift_for_prefix(idx, leaf, 100)) == 2
    from_tree = PackedTreeMask(torch.zeros(1), torch.zeros(1), 32, 8, torch.zeros(1))
    assert shift_for_prefix(idx, leaf, 7, from_tree)[2].key_limit is None


def test_shifted_lists_with_unshifted_packed_inputs_are_refused():
    """Index tensors moved behind a prefix must come with the packed inputs ``shift_for_prefix`` returns:
    a plan of the tree precompute whose shift is not the prefix length is refused before anything runs."""
    import pytest
    from fstattention_amd import fst_attention
    idx, _, leaf = _lists()
    from_tree = PackedTreeMask(torch.zeros(1), torch.zeros(1), 32, 8, torch.zeros(1))      # key_shift 0, tree plan
    q = torch.zeros((1, 1, 64, 64))
    kv = torch.zeros((1, 1, 64 + 100, 64))
    a_sh, l_sh = shift_for_prefix(idx, leaf, 100)
    with pytest.raises(ValueError, match="key_shift"):
        fst_attention(q, kv, kv, a_sh, from_tree, l_sh, 1.0, BLOCK_M=32, MAX_ANCESTORS=8)
    # the other way round: a shifted plan in front of K/V without the prefix
    _, _, shifted = shift_for_prefix(idx, leaf, 100, from_tree)
    with pytest.raises(ValueError, match="key_shift"):
        fst_attention(q, q, q, idx, shifted, leaf, 1.0, BLOCK_M=32, MAX_ANCESTORS=8)
