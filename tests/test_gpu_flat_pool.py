"""The token-level KV pool (the reference's SGLang layout) on an MI355X, through the C ABI,
against the reference's own outputs (tests/golden/flat_pool.pt) and the oracle."""
from __future__ import annotations

import types

import pytest
import torch

from conftest import load_golden
from helpers import KEEP_TIE_TOL, SELECT_SCORE_TOL, assert_keep_matches
from oracle import flat_pool as ofp
from oracle import scoring as osc
from triattention_amd import flat_pool as fp
from triattention_amd import ops, synth

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _dev_lists(t):
    return [x.clone().to(DEV) for x in t]


def _same(bufs, want):
    return torch.equal(torch.stack([b.cpu() for b in bufs]).view(torch.int16), want.view(torch.int16))


def test_gather_matches_the_reference():
    g = load_golden("flat_pool.pt")
    dense = fp.gather_request_k_dense(_dev_lists(g["k_before"]), g["req_to_token"].to(DEV), g["req_pool_idx"],
                                      g["effective_len"])
    assert torch.equal(dense.cpu().view(torch.int16), g["k_dense"].view(torch.int16))


@pytest.mark.parametrize("table_on_device", [True, False])
def test_shared_compaction_matches_the_reference_bit_for_bit(table_on_device):
    """Every slot of the pool is compared: the request's prefix holds the kept rows, nothing
    outside the request's first `budget` slots is touched."""
    g = load_golden("flat_pool.pt")
    k, v = _dev_lists(g["k_before"]), _dev_lists(g["v_before"])
    r2t = g["req_to_token"].to(DEV) if table_on_device else g["req_to_token"]
    print(f"flat pool shared compaction table_on_device={table_on_device}", flush=True)
    n = fp.compact_request_kv_in_place(k, v, r2t, g["req_pool_idx"], g["keep_shared"], g["effective_len"])
    torch.cuda.synchronize()
    assert n == g["keep_shared"].numel()
    assert _same(k, g["k_after_shared"]) and _same(v, g["v_after_shared"])


def test_per_head_compaction_matches_the_reference_bit_for_bit():
    g = load_golden("flat_pool.pt")
    k, v = _dev_lists(g["k_before"]), _dev_lists(g["v_before"])
    print("flat pool per-head compaction", flush=True)
    n = fp.compact_request_kv_in_place_per_head(k, v, g["req_to_token"].to(DEV), g["req_pool_idx"],
                                                g["keep_per_head"].to(DEV), g["effective_len"])
    torch.cuda.synchronize()
    assert n == g["keep_per_head"].shape[1]
    assert _same(k, g["k_after_per_head"]) and _same(v, g["v_after_per_head"])
    # a subset of the layers: the other layer keeps its content
    k, v = _dev_lists(g["k_before"]), _dev_lists(g["v_before"])
    fp.compact_request_kv_in_place_per_head(k, v, g["req_to_token"].to(DEV), g["req_pool_idx"], g["keep_per_head"],
                                            g["effective_len"], target_layers=[1])
    torch.cuda.synchronize()
    assert torch.equal(k[0].cpu().view(torch.int16), g["k_before"][0].view(torch.int16))
    assert torch.equal(k[1].cpu().view(torch.int16), g["k_after_per_head"][1].view(torch.int16))


def test_compaction_raises_like_the_reference():
    g = load_golden("flat_pool.pt")
    k, v = _dev_lists(g["k_before"]), _dev_lists(g["v_before"])
    r2t, eff = g["req_to_token"].to(DEV), g["effective_len"]
    with pytest.raises(ValueError):
        fp.compact_request_kv_in_place(k, v, r2t, 1, torch.tensor([5, 3]), eff)
    with pytest.raises(IndexError):
        fp.compact_request_kv_in_place(k, v, r2t, 1, torch.tensor([5, eff]), eff)
    with pytest.raises(IndexError):
        fp.compact_request_kv_in_place(k, v, r2t, 1, torch.tensor([-1, 4]), eff)
    with pytest.raises(ValueError):
        fp.compact_request_kv_in_place(k, v, r2t, 1, torch.arange(eff + 1), eff)
    with pytest.raises(ValueError):
        fp.compact_request_kv_in_place_per_head(k, v, r2t, 1, torch.zeros(3, 4, dtype=torch.long), eff)
    assert fp.compact_request_kv_in_place(k, v, r2t, 1, torch.empty(0, dtype=torch.long), eff) == 0
    assert _same(k, g["k_before"])


def test_reclaim_matches_the_reference():
    g = load_golden("flat_pool.pt")
    r2t = g["req_to_token"].to(DEV)
    freed_to = []
    alloc = types.SimpleNamespace(free=lambda idx: freed_to.append(idx.clone()))
    freed = fp.reclaim_freed_slots(r2t, g["req_pool_idx"], g["keep_shared"].numel(), g["effective_len"], alloc)
    assert torch.equal(freed.cpu(), g["freed_slots"]) and torch.equal(freed_to[0].cpu(), g["freed_slots"])
    assert torch.equal(r2t.cpu(), g["req_to_token_after_reclaim"])
    assert fp.reclaim_freed_slots(r2t, g["req_pool_idx"], g["keep_shared"].numel(), g["effective_len"], alloc).numel() == 0
    assert len(freed_to) == 1


@pytest.mark.parametrize("case", [dict(), dict(layer_aggregation="max"), dict(normalize=False),
                                  dict(window_size=9, prefill_len=11, protect_prefill=True)])
def test_selection_in_the_backend_order_matches_the_oracle(case):
    """Scores straight from the pool, max over the query heads of a KV head, then the
    reference's normalisation per (layer, KV head): keep sets equal to the oracle's away from
    ties, selection scores within 1e-4 of the largest one."""
    g = torch.Generator().manual_seed(31)
    layers, hkv, group, dim, pool, eff, budget = 3, 2, 4, 128, 700, 517, 128
    hq = hkv * group
    k_pool = [(torch.randn(pool, hkv, dim, generator=g) + torch.randn(1, hkv, dim, generator=g)).to(torch.bfloat16)
              for _ in range(layers)]
    r2t = torch.zeros(2, 1024, dtype=torch.int32)
    r2t[0, :eff] = (torch.randperm(pool - 1, generator=g)[:eff] + 1).int()
    qc = torch.randn(layers, hq, dim // 2, 2, generator=g)
    qa = qc.pow(2).sum(-1).sqrt() + torch.rand(layers, hq, dim // 2, generator=g)
    omega, offs = synth.rope_inv_freq(synth.config(0)), synth.geometric_offsets()
    round_start = 900
    score = ops.ScoreConfig(ops.fold_stats(qc.to(DEV), qa.to(DEV), torch.ones_like(qa).to(DEV)), omega.to(DEV), offs.to(DEV))
    print(f"flat pool selection case={case}", flush=True)
    keep, fin = fp.select_keep_indices_per_head([b.to(DEV) for b in k_pool], r2t.to(DEV), 0, eff, score, budget,
                                                round_start, return_scores=True, **case)
    torch.cuda.synchronize()
    dense = ofp.gather_request_k_dense(k_pool, r2t, 0, eff)                       # [L, H, T, D]
    raw = torch.stack([osc.raw_scores(dense[l:l + 1].repeat_interleave(group, dim=1), qc[l], qa[l], omega, offs,
                                      torch.ones_like(qa[l]), round_start)[0] for l in range(layers)])
    want, final = ofp.select_keep_group_first(raw, hkv, budget, normalize=case.get("normalize", True),
                                              layer_mode=case.get("layer_aggregation", "mean"),
                                              window_size=case.get("window_size", 0),
                                              prefill_len=case.get("prefill_len", 0),
                                              protect_prefill=case.get("protect_prefill", False))
    got = fin.cpu()
    assert torch.equal(torch.isinf(got), torch.isinf(final))
    finite = torch.isfinite(final)
    scale = float(final[finite].abs().max())
    assert float((got[finite] - final[finite]).abs().max()) <= SELECT_SCORE_TOL * scale
    assert keep.dtype == torch.long and tuple(keep.shape) == (hkv, budget)
    assert bool((keep[:, 1:] > keep[:, :-1]).all())
    assert assert_keep_matches(keep.cpu(), want, final, budget, tie_tol=KEEP_TIE_TOL * scale) == 0
