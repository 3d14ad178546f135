"""Oracle for the token-level KV pool (the reference's SGLang backend) against vectors written
by the reference's own functions (tests/golden/make_flat_pool_golden.py) and brute force."""
from __future__ import annotations

import pytest
import torch

from conftest import load_golden
from oracle import flat_pool as ofp
from oracle.selection import topk_ascending


def _lists(t):
    return [x.clone() for x in t]


def test_gather_and_compaction_equal_the_reference_bit_for_bit():
    g = load_golden("flat_pool.pt")
    idx, eff = g["req_pool_idx"], g["effective_len"]
    dense = ofp.gather_request_k_dense(_lists(g["k_before"]), g["req_to_token"], idx, eff)
    assert torch.equal(dense.view(torch.int16), g["k_dense"].view(torch.int16))
    k, v = _lists(g["k_before"]), _lists(g["v_before"])
    assert ofp.compact_shared(k, v, g["req_to_token"], idx, g["keep_shared"], eff) == g["keep_shared"].numel()
    assert torch.equal(torch.stack(k).view(torch.int16), g["k_after_shared"].view(torch.int16))
    assert torch.equal(torch.stack(v).view(torch.int16), g["v_after_shared"].view(torch.int16))
    k, v = _lists(g["k_before"]), _lists(g["v_before"])
    assert ofp.compact_per_head(k, v, g["req_to_token"], idx, g["keep_per_head"], eff) == g["keep_per_head"].shape[1]
    assert torch.equal(torch.stack(k).view(torch.int16), g["k_after_per_head"].view(torch.int16))
    assert torch.equal(torch.stack(v).view(torch.int16), g["v_after_per_head"].view(torch.int16))


def test_reclaim_equals_the_reference():
    g = load_golden("flat_pool.pt")
    r2t = g["req_to_token"].clone()
    freed = ofp.reclaim_freed_slots(r2t, g["req_pool_idx"], g["keep_shared"].numel(), g["effective_len"])
    assert torch.equal(freed, g["freed_slots"])
    assert torch.equal(r2t, g["req_to_token_after_reclaim"])
    again = ofp.reclaim_freed_slots(r2t, g["req_pool_idx"], g["keep_shared"].numel(), g["effective_len"])
    assert again.numel() == 0                       # the zeroed tail is not freed twice


def test_compaction_rejects_what_the_reference_rejects():
    g = load_golden("flat_pool.pt")
    k, v = _lists(g["k_before"]), _lists(g["v_before"])
    with pytest.raises(ValueError):
        ofp.compact_shared(k, v, g["req_to_token"], 1, torch.tensor([5, 3]), 101)
    with pytest.raises(IndexError):
        ofp.compact_shared(k, v, g["req_to_token"], 1, torch.tensor([5, 101]), 101)
    with pytest.raises(ValueError):
        ofp.compact_shared(k, v, g["req_to_token"], 1, torch.arange(102), 101)


def test_group_first_selection_uses_the_reference_normalisation_and_window_guard():
    """Reduce over the query heads first, then the reference's normalize_scores per (layer, KV
    head), mean over layers, protect_window_tokens: the oracle's final scores equal the
    reference's tensors, and the keep set is the top k of them."""
    g = load_golden("flat_pool.pt")
    raw = g["raw_scores"]                                   # [L, A, T]
    heads = g["normalized"].shape[1]
    keep, final = ofp.select_keep_group_first(raw, heads, 64, normalize=True, layer_mode="mean", window_size=17)
    assert torch.equal(final, g["window_protected"])
    assert torch.equal(keep, topk_ascending(g["window_protected"], 64))
    assert bool((keep[:, -17:] == torch.arange(300 - 17, 300)).all())
    # without normalisation and with the max over layers: brute force
    keep2, final2 = ofp.select_keep_group_first(raw, heads, 10, normalize=False, layer_mode="max")
    group = raw.shape[1] // heads
    for h in range(heads):
        want = torch.stack([raw[l, h * group:(h + 1) * group].max(dim=0).values for l in range(raw.shape[0])]).max(dim=0).values
        assert torch.equal(final2[h], want)
        assert set(keep2[h].tolist()) == set(torch.topk(want, 10).indices.tolist())
