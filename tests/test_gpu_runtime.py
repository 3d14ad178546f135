"""The reference-shaped Python API (selector, compaction functions, runner hook, dense
compressor) on an MI355X, against the reference's own outputs and the oracle."""
from __future__ import annotations

import types
from pathlib import Path

import pytest
import torch

from conftest import load_golden
from helpers import assert_keep_matches, score_tolerance, tune
from oracle import compaction as ocp
from oracle import scoring as osc
from oracle import selection as osel
from triattention_amd.core.compressor import TriAttentionCompressor
from triattention_amd.core.config import TriAttentionConfig
from triattention_amd.core.scoring import compute_scores, compute_scores_triton
from triattention_amd.runtime import (CompressionSignal, RunnerHookCompressionExecutor, TriAttentionRuntimeConfig,
                                      build_triattention_selector, compact_request_kv_in_place,
                                      compact_request_kv_in_place_per_head, gather_request_k_dense_range,
                                      install_runner_compression_hook, register_kv_layout_axis_hint)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _write_stats(path: Path, qc, qa, inv_freq, head_dim):
    layers, hq = qc.shape[:2]
    entries = {f"layer{l:02d}_head{h:02d}": {"q_mean_real": qc[l, h, :, 0].clone(), "q_mean_imag": qc[l, h, :, 1].clone(),
                                            "q_abs_mean": qa[l, h].clone()} for l in range(layers) for h in range(hq)}
    torch.save({"metadata": {"head_dim": head_dim, "rope_style": "half", "inv_freq": inv_freq.clone(),
                             "sampled_heads": [[l, h] for l in range(layers) for h in range(hq)]},
                "stats": entries}, path)


def _golden_caches(gold):
    layers, hkv, t, d = gold["keys"].shape
    bs, pool = int(gold["block_size"]), int(gold["pool_blocks"])
    ids = gold["block_ids"].tolist()
    tok = torch.arange(t)
    blk = torch.tensor(ids)[tok // bs]
    caches = []
    for l in range(layers):
        kvc = torch.zeros(2, pool, bs, hkv, d, dtype=torch.bfloat16)
        kvc[0, blk, tok % bs] = gold["keys"][l].transpose(0, 1)
        kvc[1, blk, tok % bs] = gold["values"][l].transpose(0, 1)
        caches.append(kvc)
    return caches, ids, bs


@pytest.mark.parametrize("tag,kw", [("default", {}), ("nonorm", {"sparse_normalize_scores": False}),
                                    ("aggmax", {"sparse_score_aggregation": "max"}),
                                    ("chunk64_prefill", {"score_chunk_max_tokens": 64, "protect_prefill": True})])
@pytest.mark.parametrize("fixture", ["selector_group.pt", "selector_group_d128.pt"])
def test_selector_api_matches_reference_outputs(tmp_path, tag, kw, fixture):
    gold = load_golden(fixture)
    layers, hkv, t, d = gold["keys"].shape
    _write_stats(tmp_path / "s.pt", gold["q_mean_complex"], gold["q_abs_mean"], gold["omega"], d)
    cfg = TriAttentionRuntimeConfig(kv_budget=96, divide_length=16, window_size=12, sparse_stats_path=tmp_path / "s.pt", **kw)
    layer_sel, group_sel, status = build_triattention_selector(cfg)
    assert status == "enabled"
    caches, ids, bs = _golden_caches(gold)
    caches = [c.to(DEV) for c in caches]
    common = dict(total_tokens=t, prefill_len=int(gold["prefill_len"]), protect_prefill=cfg.protect_prefill,
                  round_start=int(gold["round_start"]), budget_total=96)
    res = group_sel(layer_inputs=None, layer_input_iter=None,
                    layer_kv_iter=lambda: [(l, caches[l], ids, bs) for l in range(layers)], **common)
    assert res["mode"] == "per_head" and res["semantic"] == "hf_aligned_global_per_head"
    assert res["group_agg_mode"] == "mean" and res["debug_recent_count"] == 12
    assert res["indices"].dtype == torch.long and torch.equal(res["indices"].cpu(), gold[f"group_{tag}_keep"])
    res_l = layer_sel(keys_dense=None, kv_cache=caches[1], block_ids=torch.tensor(ids), block_size=bs, layer_idx=1, **common)
    assert res_l["mode"] == "per_head" and torch.equal(res_l["indices"].cpu(), gold[f"layer1_{tag}_keep"])
    # dense inputs give the same answer as paged ones
    dense = [(l, gather_request_k_dense_range(caches[l], ids, bs, 0, t)) for l in range(layers)]
    res_d = group_sel(layer_inputs=dense, **common)
    assert torch.equal(res_d["indices"], res["indices"])
    res_ld = layer_sel(keys_dense=dense[1][1], layer_idx=1, **common)
    assert torch.equal(res_ld["indices"], res_l["indices"])


def test_selector_modes(tmp_path):
    gold = load_golden("selector_group.pt")
    layers, hkv, t, d = gold["keys"].shape
    hq = gold["q_mean_complex"].shape[1]
    _write_stats(tmp_path / "s.pt", gold["q_mean_complex"], gold["q_abs_mean"], gold["omega"], d)
    caches, ids, bs = _golden_caches(gold)
    cache1 = caches[1].to(DEV)
    common = dict(keys_dense=None, kv_cache=cache1, block_ids=ids, block_size=bs, total_tokens=t, prefill_len=0,
                  protect_prefill=False, layer_idx=1, round_start=t, budget_total=96)
    offs = osc.geometric_offsets()
    keys = gold["keys"][1].float()
    raw_q = osc.raw_scores(keys.repeat_interleave(hq // hkv, 0), gold["q_mean_complex"][1], gold["q_abs_mean"][1],
                           gold["omega"], offs, torch.ones(hq, d // 2), t)
    # per_layer_per_head with mean over the query heads of a KV head
    cfg = TriAttentionRuntimeConfig(kv_budget=96, window_size=12, sparse_stats_path=tmp_path / "s.pt",
                                    pruning_mode="per_layer_per_head", layer_perhead_aggregation="mean")
    res = build_triattention_selector(cfg)[0](**common)
    fin = osel.layer_final_scores(raw_q, hkv, window_size=12, group_agg="mean")
    assert_keep_matches(res["indices"].cpu(), osel.topk_ascending(fin, 96), fin, 96, 1e-4)
    # legacy_layer_local: statistics mean-pooled to the KV heads
    cfg = TriAttentionRuntimeConfig(kv_budget=96, window_size=12, sparse_stats_path=tmp_path / "s.pt",
                                    per_head_selection_semantics="legacy_layer_local")
    sel_l, sel_g, _ = build_triattention_selector(cfg)
    assert sel_g(layer_inputs=[], total_tokens=t, prefill_len=0, protect_prefill=False, round_start=t, budget_total=96) is None
    qc_p = gold["q_mean_complex"][1].reshape(hkv, hq // hkv, d // 2, 2).mean(1)
    qa_p = gold["q_abs_mean"][1].reshape(hkv, hq // hkv, d // 2).mean(1)
    raw_p = osc.raw_scores(keys, qc_p, qa_p, gold["omega"], offs, torch.ones(hkv, d // 2), t)
    fin = osel.layer_final_scores(raw_p, hkv, window_size=12)
    assert_keep_matches(sel_l(**common)["indices"].cpu(), osel.topk_ascending(fin, 96), fin, 96, 1e-4)
    # per_layer: one shared list, max over heads
    cfg = TriAttentionRuntimeConfig(kv_budget=96, window_size=12, sparse_stats_path=tmp_path / "s.pt",
                                    pruning_mode="per_layer", allow_per_layer_mode=True)
    res = build_triattention_selector(cfg)[0](**common)
    fin = osel.layer_final_scores(raw_p, hkv, window_size=12, shared=True)
    assert res["mode"] == "shared" and res["indices"].ndim == 1
    assert_keep_matches(res["indices"].cpu().unsqueeze(0), osel.topk_ascending(fin, 96), fin, 96, 1e-4)


@pytest.mark.parametrize("axis", [0, 1])
def test_compaction_api_matches_reference_and_raises_like_it(axis):
    g = load_golden("compaction.pt")[f"axis{axis}"]
    bs, t = int(g["block_size"]), int(g["total_tokens"])
    pad = torch.zeros(*g["kv_before"].shape[:-1], 64, dtype=torch.bfloat16)
    pad[..., :16] = g["kv_before"]
    a = pad.to(DEV)
    n = compact_request_kv_in_place_per_head(a, g["block_ids"], bs, g["keep_per_head"].to(DEV), t)
    assert n == g["keep_per_head"].shape[1]
    assert torch.equal(a.cpu()[..., :16].view(torch.int16), g["kv_after_per_head"].view(torch.int16))
    b = pad.to(DEV)
    assert compact_request_kv_in_place(b, g["block_ids"].tolist(), bs, g["keep_shared"].tolist(), t) == g["keep_shared"].numel()
    assert torch.equal(b.cpu()[..., :16].view(torch.int16), g["kv_after_shared"].view(torch.int16))
    # prefix-only mode agrees with the reference on the kept slots
    c = pad.to(DEV)
    compact_request_kv_in_place_per_head(c, g["block_ids"], bs, g["keep_per_head"], t, preserve_dropped_tokens=False)
    k = g["keep_per_head"].shape[1]
    blk, off = ocp.token_slots(g["block_ids"], bs, torch.arange(k))
    kc, vc = ocp.split_kv(c.cpu()[..., :16].contiguous())
    kr, vr = ocp.split_kv(g["kv_after_per_head"])
    assert torch.equal(kc[blk, off].view(torch.int16), kr[blk, off].view(torch.int16))
    assert torch.equal(vc[blk, off].view(torch.int16), vr[blk, off].view(torch.int16))
    d = pad.to(DEV)
    before = d.clone()
    with pytest.raises(IndexError):
        compact_request_kv_in_place(d, g["block_ids"], bs, [0, t], t)
    with pytest.raises(ValueError):
        compact_request_kv_in_place(d, g["block_ids"], bs, [3, 3, 4], t)
    with pytest.raises(ValueError):
        compact_request_kv_in_place(d, g["block_ids"], bs, [5, 2], t)
    with pytest.raises(ValueError):
        compact_request_kv_in_place_per_head(d, g["block_ids"], bs, torch.zeros(2, 3, dtype=torch.long), t)
    with pytest.raises(ValueError):
        compact_request_kv_in_place_per_head(d, g["block_ids"], bs, torch.zeros(3, dtype=torch.long), t)
    assert compact_request_kv_in_place(d, g["block_ids"], bs, [], t) == 0
    assert compact_request_kv_in_place_per_head(d, g["block_ids"], bs, [], t) == 0
    assert compact_request_kv_in_place(d, g["block_ids"], bs, list(range(t)), t) == t
    assert torch.equal(d, before)
    from triattention_amd.runtime.kv_compaction import clear_kv_layout_axis_hints_for_tests
    clear_kv_layout_axis_hints_for_tests()       # hints are keyed by address; the allocator reuses addresses
    amb = torch.zeros(2, 2, 4, 2, 64, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(ValueError):
        compact_request_kv_in_place(amb, [0, 1], 4, [1, 2], 8)
    register_kv_layout_axis_hint(amb, 1)
    assert compact_request_kv_in_place(amb, [0, 1], 4, [1, 2], 8) == 2


@pytest.mark.parametrize("preserve", [True, False])
def test_compaction_self_check_switch(preserve, monkeypatch):
    """TRIATTN_DEBUG_VALIDATE_COMPACTION_CONTENT=1 (the reference's switch): the rows are
    gathered before the move and the compacted prefix is compared with them afterwards; a
    correct move passes, and the check itself notices a prefix that does not hold them."""
    from triattention_amd.runtime import kv_compaction as kvc
    g = load_golden("compaction.pt")["axis0"]
    bs, t = int(g["block_size"]), int(g["total_tokens"])
    pad = torch.zeros(*g["kv_before"].shape[:-1], 64, dtype=torch.bfloat16)
    pad[..., :16] = g["kv_before"]
    monkeypatch.setenv("TRIATTN_DEBUG_VALIDATE_COMPACTION_CONTENT", "1")
    a = pad.to(DEV)
    assert compact_request_kv_in_place_per_head(a, g["block_ids"], bs, g["keep_per_head"].to(DEV), t,
                                                preserve_dropped_tokens=preserve) == g["keep_per_head"].shape[1]
    b = pad.to(DEV)
    assert compact_request_kv_in_place(b, g["block_ids"], bs, g["keep_shared"].to(DEV), t,
                                       preserve_dropped_tokens=preserve) == g["keep_shared"].numel()
    # the checker against rows that are not there
    c = pad.to(DEV)
    keep = g["keep_shared"].to(DEV).long().unsqueeze(0)
    expected = [kvc._rows_of(c, g["block_ids"], bs, keep, True)]
    with pytest.raises(RuntimeError, match="TRIATTN_DEBUG_COMPACTION_KEY_MISMATCH:shared_prefix_content_mismatch"):
        kvc._validate_prefix([c], g["block_ids"], bs, int(keep.shape[1]), expected, True)      # nothing was moved


def _signal(**kw):
    base = dict(req_id="r", should_compress=True, reason="length_threshold", estimated_cache_len=301, step=1,
                kv_usage=None, protect_prefill=False, prefill_len=20, scheduled_tokens=1)
    base.update(kw)
    return CompressionSignal(**base)


def test_runner_hook_end_to_end(tmp_path):
    """Fake runner -> hook -> keep sets equal to the reference's, K/V compacted bit-exactly,
    block table truncated, result dictionary as the scheduler expects it."""
    gold = load_golden("selector_group.pt")
    layers, hkv, t, d = gold["keys"].shape
    _write_stats(tmp_path / "s.pt", gold["q_mean_complex"], gold["q_abs_mean"], gold["omega"], d)
    cfg = TriAttentionRuntimeConfig(kv_budget=96, divide_length=16, window_size=12, sparse_stats_path=tmp_path / "s.pt")
    cpu_caches, ids, bs = _golden_caches(gold)
    caches = [c.to(DEV) for c in cpu_caches]
    req = types.SimpleNamespace(num_computed_tokens=int(gold["round_start"]), block_ids=(list(ids),))
    runner = types.SimpleNamespace(requests={"r": req}, kv_caches=caches, cache_config=types.SimpleNamespace(block_size=bs))
    install_runner_compression_hook(runner, cfg)
    sched = types.SimpleNamespace(num_scheduled_tokens={"r": 1})
    # estimated length = cached tokens + the token scheduled this step
    res = RunnerHookCompressionExecutor(runner).execute("r", _signal(estimated_cache_len=t + 1), sched)
    torch.cuda.synchronize()
    assert res.applied and res.reason == "kv_compacted:per_head:hf_aligned_global_per_head"
    assert res.cache_len_after == 96 and res.details["budget_total"] == 96
    assert res.details["effective_tokens_before"] == t and res.details["selector_status"] == "enabled"
    nkeep = (96 + bs - 1) // bs
    assert req.block_ids == (ids[:nkeep],)
    grp = res.details["block_reclaim"]["groups"][0]
    assert grp["block_ids_before"] == ids and grp["block_ids_after"] == ids[:nkeep] and grp["block_ids_removed"] == ids[nkeep:]
    assert res.details["reclaimed_block_count"] == len(ids) - nkeep
    want_keep = gold["group_default_keep"]
    blk, off = ocp.token_slots(ids, bs, torch.arange(96))
    for l in range(layers):
        ref = cpu_caches[l].clone()
        ocp.compact_per_head(ref, ids, bs, want_keep, t, full_permutation=False)
        got = caches[l].cpu()
        assert torch.equal(got[:, blk, off].view(torch.int16), ref[:, blk, off].view(torch.int16))
    # second trigger right away: below budget + divide_length -> deferred
    req.num_computed_tokens += 1
    again = runner.triattention_apply_compression(req_id="r", signal=_signal(estimated_cache_len=98), scheduler_output=sched)
    assert again["applied"] is False and again["reason"] == "under_budget"


def _fake_runner(w, inp, tmp_path, **cfg_kw):
    """A runner with one request per sequence of the workload, all in one paged pool."""
    from triattention_amd import synth
    _write_stats(tmp_path / "s.pt", inp["qc"], inp["qa"], inp["omega"], w.head_dim)
    cfg = TriAttentionRuntimeConfig(kv_budget=w.budget, divide_length=16, window_size=w.window_size,
                                    sparse_stats_path=tmp_path / "s.pt", **cfg_kw)
    caches = [c.to(DEV) for c in inp["caches"]]
    reqs = {f"r{b}": types.SimpleNamespace(num_computed_tokens=t, block_ids=([int(x) for x in inp["tables"][b]],))
            for b, t in enumerate(w.seq_lens)}
    runner = types.SimpleNamespace(requests=reqs, kv_caches=caches,
                                   cache_config=types.SimpleNamespace(block_size=w.block_size))
    install_runner_compression_hook(runner, cfg)
    sched = types.SimpleNamespace(num_scheduled_tokens={rid: 1 for rid in reqs})
    signals = {f"r{b}": _signal(req_id=f"r{b}", estimated_cache_len=t + 1, prefill_len=7 + b)
               for b, t in enumerate(w.seq_lens)}
    return runner, reqs, caches, sched, signals


def test_batch_hook_equals_the_hook_called_request_by_request(tmp_path, monkeypatch):
    """All triggered requests of a step through ``triattention_apply_compression_batch``: same
    result dictionaries, same truncated block lists and bit-identical caches as the
    one-by-one hook (same kernels: the resident kernel is switched off for this comparison).
    One request is under budget and one asks for the prefill guard."""
    from helpers import build_inputs
    from triattention_amd import synth
    tune(resident_kernel="off")
    w = synth.Workload(name="t", num_layers=3, num_q_heads=8, num_kv_heads=2, head_dim=128,
                       seq_lens=(300, 1000, 97, 513, 60), budget=96, block_size=16, window_size=12, rope_theta=1e6,
                       index=31)
    inp = build_inputs(w)
    one = _fake_runner(w, inp, tmp_path)
    two = _fake_runner(w, inp, tmp_path)
    for _, _, _, _, signals in (one, two):
        signals["r3"] = _signal(req_id="r3", estimated_cache_len=514, prefill_len=40, protect_prefill=True)
    runner, reqs, caches, sched, signals = one
    from triattention_amd.runtime import hook as hook_mod
    monkeypatch.setattr(hook_mod, "SINGLE_REQUEST_IN_ONE_CALL", False)     # the reference-shaped pipeline, request by request
    want = {rid: RunnerHookCompressionExecutor(runner).execute(rid, sig, sched) for rid, sig in signals.items()}
    monkeypatch.setattr(hook_mod, "SINGLE_REQUEST_IN_ONE_CALL", True)
    three = _fake_runner(w, inp, tmp_path)
    three[4]["r3"] = signals["r3"]
    fused_single = {rid: RunnerHookCompressionExecutor(three[0]).execute(rid, sig, three[3]) for rid, sig in three[4].items()}
    assert fused_single == want                                             # ... equals the one-call path per request
    for a, b in zip(caches, three[2]):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    runner2, reqs2, caches2, sched2, signals2 = two
    got = RunnerHookCompressionExecutor(runner2).execute_batch(signals2, sched2)
    torch.cuda.synchronize()
    assert list(got) == list(want)
    for rid in want:
        assert got[rid] == want[rid], rid
        assert reqs2[rid].block_ids == reqs[rid].block_ids
    assert want["r4"].reason == "under_budget" and want["r0"].applied and want["r0"].cache_len_after == 96
    for a, b in zip(caches, caches2):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    # a second step right away: everything deferred, nothing launched
    again = RunnerHookCompressionExecutor(runner2).execute_batch(
        {rid: _signal(req_id=rid, estimated_cache_len=98) for rid in signals2}, sched2)
    assert all(not r.applied and r.reason == "under_budget" for r in again.values())


def test_batch_hook_on_the_resident_kernel(tmp_path, monkeypatch):
    """Sixteen requests of 3072 tokens fill the chip: the batch hook runs the resident kernel;
    result equal to the library calls on the same batch, and, when the resident launch is made to
    fail, to the one-by-one path (the caches were not touched by the failed step)."""
    from helpers import build_inputs
    from triattention_amd import ops, synth
    w = synth.Workload(name="t", num_layers=2, num_q_heads=8, num_kv_heads=2, head_dim=128, seq_lens=(3072,) * 16,
                       budget=256, block_size=16, window_size=12, rope_theta=1e6, index=32)
    inp = build_inputs(w)
    runner, reqs, caches, sched, signals = _fake_runner(w, inp, tmp_path)
    got = RunnerHookCompressionExecutor(runner).execute_batch(signals, sched)
    torch.cuda.synchronize()
    assert all(r.applied and r.cache_len_after == 256 for r in got.values())
    ref = [c.to(DEV) for c in inp["caches"]]
    kv = ops.PagedKV.from_kv_caches(ref)
    batch = ops.StepBatch(DEV, w.seq_lens, round_start=w.seq_lens, budgets=w.budget, block_tables=inp["tables"],
                          prefill_lens=[0] * 16)
    sc = ops.ScoreConfig(ops.fold_stats(inp["qc"].to(DEV), inp["qa"].to(DEV), inp["fs"].to(DEV)),
                         inp["omega"].to(DEV), inp["offsets"].to(DEV))
    sel = ops.SelectConfig(window_size=w.window_size)
    assert ops.select_path(kv, batch, sc, sel) == "resident_mfma"
    _, ws = ops.compress_step(kv, batch, sc, sel)
    assert ws.status() == 0
    for a, b in zip(caches, ref):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    for b in range(16):
        assert reqs[f"r{b}"].block_ids == ([int(x) for x in inp["tables"][b]][:16],)

    # forced failure of the resident launch: the hook repeats the step request by request
    runner_f, reqs_f, caches_f, sched_f, signals_f = _fake_runner(w, inp, tmp_path)
    tune(resident_wait_us=-1)
    failed = RunnerHookCompressionExecutor(runner_f).execute_batch(signals_f, sched_f)
    tune(resident_wait_us=None)
    tune(resident_kernel="off")
    runner_s, reqs_s, caches_s, sched_s, signals_s = _fake_runner(w, inp, tmp_path)
    single = {rid: RunnerHookCompressionExecutor(runner_s).execute(rid, sig, sched_s) for rid, sig in signals_s.items()}
    torch.cuda.synchronize()
    assert failed == single
    for a, b in zip(caches_f, caches_s):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))


@pytest.mark.parametrize("resident", [False, True])
def test_repeated_shape_replays_a_graph_with_the_same_results(tmp_path, monkeypatch, resident):
    """A decoding request comes back to the hook with the same lengths every ``divide_length``
    tokens: from the second visit on the selector replays a captured launch sequence.  Eight steps
    with fresh cache contents, other block lists, other round starts and a prefill guard that comes
    and goes, next to a selector that never replays: equal results, bit-identical caches after every
    step (the program's own eager work and synchronisations lie between the replays)."""
    from helpers import build_inputs
    from triattention_amd import synth
    from triattention_amd.runtime import selector as selector_mod
    if not resident:
        tune(resident_kernel="off")
    w = synth.Workload(name="t", num_layers=3, num_q_heads=8, num_kv_heads=2, head_dim=128,
                       seq_lens=(1184,) * (16 if resident else 1), budget=160, block_size=16, window_size=12,
                       rope_theta=1e6, index=41)
    inp = build_inputs(w)
    monkeypatch.setattr(selector_mod, "GRAPH_REPLAY", True)
    # (the cache is refilled by hand below; the guard against a cache that grew back is for real decoding)
    replay = _fake_runner(w, inp, tmp_path, fail_on_effective_len_regression=False)
    monkeypatch.setattr(selector_mod, "GRAPH_REPLAY", False)
    eager = _fake_runner(w, inp, tmp_path, fail_on_effective_len_regression=False)
    before = dict(selector_mod.GRAPH_COUNTS)
    gen = torch.Generator().manual_seed(5)
    pool = inp["caches"][0].shape[1]
    need = len(inp["tables"][0])
    for step in range(8):
        fresh = [torch.randn(c.shape, generator=gen).to(c.dtype) for c in inp["caches"]]
        perm = torch.randperm(pool, generator=gen).tolist()
        tables = [perm[b * need:(b + 1) * need] for b in range(w.num_seqs)]
        results = []
        for flag, (runner, reqs, caches, sched, _) in ((True, replay), (False, eager)):
            monkeypatch.setattr(selector_mod, "GRAPH_REPLAY", flag)
            for c, f in zip(caches, fresh):
                c.copy_(f)
            signals = {}
            for b, rid in enumerate(reqs):
                reqs[rid].num_computed_tokens = 1184
                reqs[rid].block_ids = (list(tables[b]),)
                guard = step in (2, 3, 4) or not resident
                signals[rid] = _signal(req_id=rid, estimated_cache_len=1185, prefill_len=30 + step + b if guard else 0,
                                       protect_prefill=guard, step=step + 1)
            ex = RunnerHookCompressionExecutor(runner)
            results.append(ex.execute_batch(signals, sched) if resident else
                           {rid: ex.execute(rid, sig, sched) for rid, sig in signals.items()})
        torch.cuda.synchronize()
        assert results[0] == results[1], f"step {step}"
        assert all(r.applied and r.cache_len_after == 160 for r in results[0].values()), f"step {step}"
        for a, b in zip(replay[2], eager[2]):
            assert torch.equal(a.view(torch.int16), b.view(torch.int16)), f"step {step}: caches differ"
        for rid in replay[1]:
            assert replay[1][rid].block_ids == eager[1][rid].block_ids
    # resident: two shapes (with and without the guard), 5 + 3 visits; otherwise one shape, 8 visits
    assert selector_mod.GRAPH_COUNTS["captured"] - before["captured"] == (2 if resident else 1)
    assert selector_mod.GRAPH_COUNTS["replayed"] - before["replayed"] == (4 if resident else 6)


def test_runner_hook_on_an_fp8_cache_kept_in_uint8_tensors(tmp_path):
    """vLLM keeps an fp8 KV cache as uint8 tensors with one scale per tensor: the hook scores
    the codes as they are and moves rows only.  Same result dictionary and the same bytes as
    the same cache handed over as float8_e4m3fn tensors."""
    from helpers import build_inputs
    from triattention_amd import synth
    w = synth.Workload(name="t", num_layers=2, num_q_heads=8, num_kv_heads=2, head_dim=128, seq_lens=(300,),
                       budget=96, block_size=16, window_size=12, rope_theta=1e6, index=33, kv_dtype="fp8")
    inp = build_inputs(w)
    results, after = [], []
    for as_uint8 in (True, False):
        runner, reqs, caches, sched, signals = _fake_runner(w, inp, tmp_path)
        if as_uint8:
            runner.kv_caches = caches = [c.view(torch.uint8) for c in caches]
        res = RunnerHookCompressionExecutor(runner).execute("r0", signals["r0"], sched)
        torch.cuda.synchronize()
        assert res.applied and res.cache_len_after == 96
        results.append(res)
        after.append([c.cpu().view(torch.uint8) for c in caches])
    assert results[0] == results[1]
    for a, b in zip(*after):
        assert torch.equal(a, b)
    assert not torch.equal(after[0][0], inp["caches"][0].view(torch.uint8))      # something moved


def test_dense_scoring_api_against_reference_scores():
    gold = load_golden("scoring_pytorch.pt")
    for name, style in (("d128_half", "half"), ("d64_inter", "interleaved")):
        case = gold[name]
        for agg in ("mean", "max"):
            for mlr, trig in ((1, 1), (0, 1), (1, 0)):
                cfg = TriAttentionConfig(device=torch.device(DEV), score_aggregation=agg, disable_mlr=not mlr,
                                         disable_trig=not trig, rope_style=style)
                got = compute_scores(key_states=case["keys"].unsqueeze(0).to(DEV), cache_positions=None,
                                     head_stats={"q_mean_complex": case["q_mean_complex"].to(DEV),
                                                 "q_abs_mean": case["q_abs_mean"].to(DEV)},
                                     omega=case["omega"].to(DEV), offsets=case["offsets"].to(DEV),
                                     freq_scale_sq=case["freq_scale_sq"].to(DEV), config=cfg,
                                     round_start=int(case["round_start"]))
                want = case[f"scores_{agg}_mlr{mlr}_trig{trig}"]
                assert got.shape == (1,) + tuple(want.shape) and got.dtype == torch.float32
                err = (got[0].cpu() - want).abs()
                assert bool((err <= score_tolerance(want) + 1e-6).all()), (name, agg, mlr, trig, float(err.max()))
    assert compute_scores_triton is compute_scores
    with pytest.raises(TypeError):
        compute_scores(key_states=torch.zeros(1, 2, 8, 64, device=DEV), cache_positions=None,
                       head_stats={"q_mean_complex": torch.zeros(2, 32, 2)}, omega=torch.zeros(32),
                       offsets=torch.ones(1), freq_scale_sq=torch.ones(2, 32),
                       config=TriAttentionConfig(device=torch.device(DEV)), round_start=1)


def test_dense_compressor_against_oracle(tmp_path):
    g = torch.Generator().manual_seed(17)
    h, t, d, budget = 4, 600, 128, 128
    omega = 1.0 / (1e6 ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
    qc = torch.randn(1, h, d // 2, 2, generator=g)
    qa = qc.pow(2).sum(-1).sqrt() + torch.randn(1, h, d // 2, generator=g).abs()
    _write_stats(tmp_path / "s.pt", qc, qa, omega, d)
    keys = (torch.randn(1, h, t, d, generator=g) + 1.0).to(torch.bfloat16)
    vals = torch.randn(1, h, t, d, generator=g).to(torch.bfloat16)
    cfg = TriAttentionConfig(device=torch.device(DEV), stats_path=tmp_path / "s.pt", kv_budget=budget, divide_length=16,
                             window_size=16, protect_prefill=False, compute_dtype=torch.float32)
    comp = TriAttentionCompressor(cfg)
    k2, v2, keep = comp.compress(keys.to(DEV), vals.to(DEV), layer_idx=0)
    assert k2.shape == (1, h, budget, d) and keep.shape == (1, h, budget)
    raw = osc.raw_scores(keys[0], qc[0], qa[0], omega, osc.geometric_offsets(), torch.ones(h, d // 2), t)
    fin = osel.protect_window(osel.znorm_two_pass(raw), 16)
    assert_keep_matches(keep[0].cpu(), osel.topk_ascending(fin, budget), fin, budget, 1e-3)
    kk = keep[0].cpu()
    for hh in range(h):
        assert torch.equal(k2[0, hh].cpu().view(torch.int16), keys[0, hh, kk[hh]].view(torch.int16))
        assert torch.equal(v2[0, hh].cpu().view(torch.int16), vals[0, hh, kk[hh]].view(torch.int16))
    assert comp.get_state()["compression_count"] == 1 and comp.get_state()["current_cache_len"] == budget
    # below budget + divide_length nothing happens
    small = TriAttentionCompressor(cfg)
    k3, v3, ident = small.compress(keys[:, :, :100].to(DEV), vals[:, :, :100].to(DEV))
    assert k3.shape[2] == 100 and ident.tolist() == list(range(100))
    with pytest.raises(ValueError):
        TriAttentionCompressor(cfg).compress(torch.zeros(2, h, 600, d, dtype=torch.bfloat16, device=DEV),
                                             torch.zeros(2, h, 600, d, dtype=torch.bfloat16, device=DEV))


def test_scheduler_and_worker_bookkeeping_around_the_hook_over_a_decode_loop(tmp_path):
    """A stand-in engine (block pool, per-group block manager, worker block table) drives the hook
    through ``engine_glue`` for 80 decode steps of two requests: the scheduler's and the worker's
    block lists stay equal, every freed block returns to the pool exactly once, the request is
    compressed again every ``divide_length`` tokens, and the lengths the attention inputs would get
    equal the scheduler's effective lengths."""
    import numpy as np
    from helpers import build_inputs
    from triattention_amd import synth
    from triattention_amd.runtime import RequestStateStore, engine_glue as eg
    NS = types.SimpleNamespace
    w = synth.Workload(name="t", num_layers=2, num_q_heads=8, num_kv_heads=2, head_dim=128, seq_lens=(300, 140),
                       budget=100, block_size=16, window_size=12, rope_theta=1e6, index=61, pool_occupancy=0.5)
    inp = build_inputs(w)
    _write_stats(tmp_path / "s.pt", inp["qc"], inp["qa"], inp["omega"], w.head_dim)
    cfg = TriAttentionRuntimeConfig(kv_budget=100, divide_length=16, window_size=12, sparse_stats_path=tmp_path / "s.pt",
                                    log_decisions=False)
    bs = w.block_size
    caches = [c.to(DEV) for c in inp["caches"]]
    used = {int(x) for tb in inp["tables"] for x in tb}
    free = [b for b in range(w.pool_blocks) if b not in used]
    freed_log = []

    class Pool:
        def free_blocks(self, blocks):
            for blk in blocks:
                assert blk.block_id not in free, "a block was freed twice"
                free.append(blk.block_id)
                freed_log.append(blk.block_id)

    rids = ["r0", "r1"]
    manager = NS(req_to_blocks={rid: [NS(block_id=int(x), block_hash=None) for x in inp["tables"][i]]
                                for i, rid in enumerate(rids)},
                 num_cached_block={rid: len(inp["tables"][i]) for i, rid in enumerate(rids)}, block_pool=Pool())
    sched_reqs = {rid: NS(num_computed_tokens=t, num_prompt_tokens=t) for rid, t in zip(rids, w.seq_lens)}
    worker_reqs = {rid: NS(num_computed_tokens=t, block_ids=([int(x) for x in inp["tables"][i]],))
                   for i, (rid, t) in enumerate(zip(rids, w.seq_lens))}
    rows = NS(num_blocks_per_row=np.array([len(tb) for tb in inp["tables"]]))
    runner = NS(requests=worker_reqs, kv_caches=caches, cache_config=NS(block_size=bs),
                input_batch=NS(block_table=rows, req_id_to_index={"r0": 0, "r1": 1}))
    install_runner_compression_hook(runner, cfg)
    store = RequestStateStore()
    runner._triattention_state_store = store
    executor = RunnerHookCompressionExecutor(runner)
    glue = eg.SchedulerCompressionGlue(cfg)
    new = [NS(req_id=rid, num_computed_tokens=0, num_prompt_tokens=t) for rid, t in zip(rids, w.seq_lens)]
    compressions = {rid: [] for rid in rids}
    true_len = dict(zip(rids, w.seq_lens))        # tokens really held in the cache
    for step in range(80):
        # -- scheduler: one token per request, a block when the cache needs one more
        for i, rid in enumerate(rids):
            if (true_len[rid] + 1 + bs - 1) // bs > len(manager.req_to_blocks[rid]):
                blk = free.pop(0)
                manager.req_to_blocks[rid].append(NS(block_id=blk, block_hash=None))
                worker_reqs[rid].block_ids[0].append(blk)
                rows.num_blocks_per_row[i] += 1
        out = NS(num_scheduled_tokens={rid: 1 for rid in rids}, scheduled_new_reqs=new if step == 0 else [],
                 finished_req_ids=set(),
                 scheduled_cached_reqs=NS(req_ids=list(rids), num_computed_tokens=[sched_reqs[r].num_computed_tokens for r in rids]))
        signals = glue.after_schedule(out, sched_reqs)
        # -- worker
        eg.register_new_requests(state_store=store, scheduler_output=out, protect_prefill=cfg.protect_prefill)
        _, signals = eg.consume_runner_signals(state_store=store, scheduler_output=out, last_step=step)
        events = eg.execute_runner_compression_actions(executor=executor, state_store=store, scheduler_output=out,
                                                       signals=signals, strict_no_downgrade=True)
        eg.apply_worker_block_reclaim_events(base_runner=runner, events=events)
        seq_bases, pos_deltas, _, _ = eg.build_effective_sparse_overrides(base_runner=runner, state_store=store,
                                                                          scheduler_output=out, compression_events=events)
        for e in events:
            if e["status"] == "applied":
                rid = e["req_id"]
                compressions[rid].append((sched_reqs[rid].num_computed_tokens, e["cache_len_after"]))
                assert e["details"]["effective_tokens_before"] == true_len[rid]
                assert e["cache_len_after"] == 100 and e["block_reclaim"]["groups"][0]["gid"] == 0
                true_len[rid] = 100
        for i, rid in enumerate(rids):
            st = store.get(rid)
            if st is not None and st.compression_count > 0:
                # the attention inputs of this step: cached length before its token, and the shift of
                # the slot positions against the absolute ones
                assert seq_bases[i] == true_len[rid], (step, rid)
                assert pos_deltas[i] == true_len[rid] - sched_reqs[rid].num_computed_tokens
            else:
                assert not seq_bases or i not in seq_bases
            worker_reqs[rid].num_computed_tokens += 1
            sched_reqs[rid].num_computed_tokens += 1
            true_len[rid] += 1
        # -- scheduler again: the events of this step
        glue.apply_compression_events(events, sched_reqs, [manager], bs)
        for i, rid in enumerate(rids):
            assert [b.block_id for b in manager.req_to_blocks[rid]] == worker_reqs[rid].block_ids[0], (step, rid)
            assert rows.num_blocks_per_row[i] == len(worker_reqs[rid].block_ids[0])
            assert len(worker_reqs[rid].block_ids[0]) * bs >= true_len[rid]
    torch.cuda.synchronize()
    # r0 (300 tokens) is due at once and then every 16 tokens; r1 (140) likewise
    for rid, t in zip(rids, w.seq_lens):
        ncts = [n for n, _ in compressions[rid]]
        assert ncts[0] == t and len(ncts) >= 4, (rid, ncts)
        assert all(15 <= b - a <= 17 for a, b in zip(ncts, ncts[1:])), (rid, ncts)      # every divide_length tokens
    assert freed_log
    live = [b.block_id for rid in rids for b in manager.req_to_blocks[rid]]
    assert len(live) == len(set(live)) and not set(live) & set(free)
    assert len(live) + len(free) == w.pool_blocks
