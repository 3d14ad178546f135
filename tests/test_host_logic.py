"""Host-side logic: settings, stats loading, planner/state models, pipeline and hook
control flow with fake runners.  CPU only; no kernel is launched."""
from __future__ import annotations

import re
import types
from pathlib import Path

import pytest
import torch

from conftest import GOLDEN, ROOT, load_golden
from triattention_amd import _lib, rope
from triattention_amd import build as tri_build
from triattention_amd.core import stats as stats_mod
from triattention_amd.core.compressor import CompressionState, gather_kv_by_indices, normalize_scores, \
    protect_window_tokens
from triattention_amd.core.config import TriAttentionConfig
from triattention_amd.runtime import (CompressionPlanner, CompressionSignal, KeepPlan, RequestStateStore,
                                      RunnerHookCompressionExecutor, TriAttentionRuntimeConfig,
                                      bridge_legacy_env, build_keep_token_indices, build_triattention_selector,
                                      install_runner_compression_hook, triattention_enabled)
from triattention_amd.runtime import hook as hook_mod
from triattention_amd.runtime import pipeline as pl
from triattention_amd.runtime.models import TRITON_SCORING_REQUIRED_MARKER as MARK


# ------------------------------------------------------------------ C ABI
def test_library_exports_every_declared_symbol():
    header = (ROOT / "include" / "triattention_hip.h").read_text()
    declared = set(re.findall(r"\b(tri_[a-z0-9_]+)\s*\(", header))
    declared -= {"tri_status", "tri_kv_dtype", "tri_rope_style", "tri_reduce"}
    assert declared == set(_lib.EXPORTS)
    lib = _lib.load()
    for name in declared:
        assert getattr(lib, name) is not None
    assert lib.tri_abi_version() == _lib.ABI_VERSION == 6


def test_c_abi_rejects_bad_arguments_without_a_gpu():
    import ctypes as C
    lib = _lib.load()
    kv = _lib.KvLayout(num_layers=1, num_kv_heads=8, head_dim=100, block_size=16)
    batch = _lib.Batch(num_seqs=1, max_seq_len=16)
    sp = _lib.ScoreParams(num_score_heads=8, num_offsets=17)
    assert lib.tri_workspace_bytes(C.byref(kv), C.byref(batch), C.byref(sp)) == 0
    assert b"head_dim" in lib.tri_last_error()
    assert lib.tri_fold_stats(None, None, None, None, 1, 1, 1, 0, 0, None, None) == _lib.TRI_ERR_INVALID_ARGUMENT
    assert lib.tri_compact_paged(None, None, None, 0, 0, None) == _lib.TRI_ERR_INVALID_ARGUMENT
    with pytest.raises(_lib.TriError):
        _lib.check(lib.tri_topk_rows(None, 0, 0, None, None, 1, 1, None, 1, None))


def test_status_word_sits_at_one_offset_for_every_shape():
    """A workspace sized for one batch is reused for smaller ones; the status word the kernels
    write and the word the host reads must be the same for all of them."""
    import ctypes as C
    lib = _lib.load()
    seen = set()
    for layers, heads, tmax, seqs, score_heads in ((36, 8, 16384, 16, 32), (36, 8, 2176, 1, 32), (4, 2, 300, 3, 8),
                                                   (64, 8, 32768, 8, 64), (1, 4, 17, 1, 4)):
        kv = _lib.KvLayout(num_layers=layers, num_kv_heads=heads, head_dim=128, block_size=16, kv_dtype=0,
                           stride_block=16 * heads * 128, stride_token=heads * 128, stride_head=128, k_layers=8)
        batch = _lib.Batch(num_seqs=seqs, max_seq_len=tmax, block_table_pitch=4096, block_table=8, seq_lens=8)
        sp = _lib.ScoreParams(num_score_heads=score_heads, num_offsets=17)
        total = int(lib.tri_workspace_bytes(C.byref(kv), C.byref(batch), C.byref(sp)))
        assert total > 0, lib.tri_last_error()
        off = int(lib.tri_workspace_status_offset(C.byref(kv), C.byref(batch), C.byref(sp)))
        assert off + 4 <= total
        seen.add(off)
    assert len(seen) == 1


def test_static_scratch_entry_rejects_oversized_steps_before_touching_the_device():
    import ctypes as C
    lib = _lib.load()
    kv = _lib.KvLayout(num_layers=36, num_kv_heads=8, head_dim=128, block_size=16, kv_dtype=0,
                       stride_block=16 * 8 * 128, stride_token=8 * 128, stride_head=128, k_layers=8, v_layers=8)
    batch = _lib.Batch(num_seqs=16, max_seq_len=16384, max_budget=2048, block_table_pitch=1024, block_table=8,
                       seq_lens=8, round_start=8, budgets=8)
    sp = _lib.ScoreParams(num_score_heads=32, num_offsets=17, folded=16, omega=8, offsets=8)
    sel = _lib.SelectParams(normalize=1, window_size=128, group_reduce=1)
    assert lib.tri_workspace_bytes(C.byref(kv), C.byref(batch), C.byref(sp)) > _lib.STATIC_WORKSPACE_BYTES
    rc = lib.tri_compress_step_static(C.byref(kv), C.byref(batch), C.byref(sp), C.byref(sel), 8, None, None)
    assert rc == _lib.TRI_ERR_WORKSPACE and b"static array" in lib.tri_last_error()
    header = (ROOT / "include" / "triattention_hip.h").read_text()
    assert f"#define TRI_STATIC_WORKSPACE_BYTES ({_lib.STATIC_WORKSPACE_BYTES >> 20}u << 20)" in header


# ---------------------------------------------------------------- settings
def test_runtime_config_defaults_and_env():
    c = TriAttentionRuntimeConfig.from_env(environ={})
    assert (c.kv_budget, c.divide_length, c.window_size, c.pruning_mode) == (2048, 128, 128, "per_head")
    assert c.per_head_selection_semantics == "hf_aligned_global_per_head"
    assert c.sparse_score_aggregation == "mean" and c.sparse_normalize_scores and not c.protect_prefill
    assert c.score_chunk_max_tokens == 4096 and c.require_triton_scoring and c.sparse_stats_path is None
    env = {"TRIATTN_RUNTIME_KV_BUDGET": "512", "TRIATTN_RUNTIME_PROTECT_PREFILL": "On",
           "TRIATTN_RUNTIME_SPARSE_STATS_PATH": " /x/y.pt ", "TRIATTN_RUNTIME_KV_USAGE_TRIGGER": "0.5",
           "TRIATTN_RUNTIME_KV_USAGE_RELEASE": "0.25", "TRIATTN_RUNTIME_PRUNING_MODE": " per_layer_per_head ",
           "TRIATTN_RUNTIME_MODEL_PATH": ""}
    c = TriAttentionRuntimeConfig.from_env(environ=env)
    assert c.kv_budget == 512 and c.protect_prefill and c.sparse_stats_path == Path("/x/y.pt")
    assert c.kv_usage_trigger == 0.5 and c.pruning_mode == "per_layer_per_head" and c.model_path is None
    c = TriAttentionRuntimeConfig.from_env(prefix="X_", environ={"X_WINDOW_SIZE": "7"})
    assert c.window_size == 7


@pytest.mark.parametrize("env", [
    {"TRIATTN_RUNTIME_PROTECT_PREFILL": "maybe"}, {"TRIATTN_RUNTIME_KV_BUDGET": "0"},
    {"TRIATTN_RUNTIME_KV_BUDGET": "abc"}, {"TRIATTN_RUNTIME_DIVIDE_LENGTH": "-1"},
    {"TRIATTN_RUNTIME_KV_USAGE_TRIGGER": "1.5"}, {"TRIATTN_RUNTIME_KV_USAGE_RELEASE": "0.99"},
    {"TRIATTN_RUNTIME_PRUNING_MODE": "per_token"}, {"TRIATTN_RUNTIME_PRUNING_MODE": "per_layer"},
    {"TRIATTN_RUNTIME_SPARSE_SCORE_AGGREGATION": "sum"}, {"TRIATTN_RUNTIME_PER_HEAD_SELECTION_SEMANTICS": "x"},
    {"TRIATTN_RUNTIME_LAYER_PERHEAD_AGGREGATION": "min"}, {"TRIATTN_RUNTIME_PER_LAYER_AGGREGATION": "min"},
    {"TRIATTN_RUNTIME_WINDOW_SIZE": "-3"}, {"TRIATTN_RUNTIME_DISABLE_TOP_N_HIGH_FREQ": "-1"},
    {"TRIATTN_RUNTIME_EFFECTIVE_LEN_REGRESSION_RATIO": "0"}, {"TRIATTN_RUNTIME_SCORE_CHUNK_MAX_TOKENS": "0"},
    {"TRIATTN_RUNTIME_EFFECTIVE_LEN_GUARD_DIVIDE_MULTIPLES": "0"},
    {"TRIATTN_RUNTIME_ENABLE_EXPERIMENTAL_BLOCK_RECLAIM": "0"},
])
def test_runtime_config_rejects(env):
    with pytest.raises(ValueError):
        TriAttentionRuntimeConfig.from_env(environ=env)


def test_runtime_config_opt_ins_and_legacy_bridge():
    c = TriAttentionRuntimeConfig.from_env(environ={"TRIATTN_RUNTIME_PRUNING_MODE": "per_layer",
                                                    "TRIATTN_RUNTIME_ALLOW_PER_LAYER_MODE": "1"})
    assert c.pruning_mode == "per_layer"
    TriAttentionRuntimeConfig.from_env(environ={"TRIATTN_RUNTIME_ENABLE_EXPERIMENTAL_BLOCK_RECLAIM": "0",
                                                "TRIATTN_RUNTIME_REQUIRE_PHYSICAL_RECLAIM": "off"})
    env = {"TRIATTENTION_KV_BUDGET": "777", "TRIATTENTION_STATS_PATH": "/s.pt", "TRIATTN_RUNTIME_WINDOW_SIZE": "5",
           "TRIATTENTION_WINDOW_SIZE": "9", "TRIATTENTION_PRUNING_MODE": "Per_Layer_Head",
           "TRIATTN_RUNTIME_DIVIDE_LENGTH": "", "TRIATTENTION_DIVIDE_LENGTH": "64"}
    bridge_legacy_env(env)
    assert env["TRIATTN_RUNTIME_KV_BUDGET"] == "777" and env["TRIATTN_RUNTIME_SPARSE_STATS_PATH"] == "/s.pt"
    assert env["TRIATTN_RUNTIME_WINDOW_SIZE"] == "5" and env["TRIATTN_RUNTIME_DIVIDE_LENGTH"] == "64"
    assert env["TRIATTN_RUNTIME_PRUNING_MODE"] == "per_layer_per_head"
    assert env["TRIATTN_RUNTIME_REQUIRE_TRITON_SCORING"] == "true"
    assert triattention_enabled({}) and not triattention_enabled({"ENABLE_TRIATTENTION": "off"})
    assert triattention_enabled({"ENABLE_TRIATTENTION": "whatever"})


def test_core_config_checks():
    c = TriAttentionConfig(device=torch.device("cpu"), pruning_mode="per_layer_per_head", stats_path="/a.pt")
    assert c.pruning_mode == "per_head" and c.stats_path == Path("/a.pt") and c.offset_max_length == 65536
    for kw in (dict(kv_budget=0), dict(divide_length=0), dict(window_size=-1), dict(window_size=2048),
               dict(compute_dtype=torch.int8), dict(position_indices_dtype=torch.float32)):
        with pytest.raises(ValueError):
            TriAttentionConfig(device=torch.device("cpu"), **kw)


# ------------------------------------------------------------------- stats
def test_stats_loader_matches_reference_loader_output():
    gold = load_golden("selector_group.pt")
    layers, hq, f, _ = gold["q_mean_complex"].shape
    import tempfile
    with tempfile.TemporaryDirectory() as tmp:
        path = Path(tmp) / "s.pt"
        entries = {}
        for l in range(layers):
            for h in range(hq):
                entries[f"layer{l:02d}_head{h:02d}"] = {"q_mean_real": gold["q_mean_complex"][l, h, :, 0].clone(),
                                                       "q_mean_imag": gold["q_mean_complex"][l, h, :, 1].clone(),
                                                       "q_abs_mean": gold["q_abs_mean"][l, h].clone()}
        torch.save({"metadata": {"head_dim": 2 * f, "rope_style": "half", "inv_freq": gold["omega"].clone(),
                                 "sampled_heads": [[l, h] for l in range(layers) for h in range(hq)]},
                    "stats": entries}, path)
        meta, hs = stats_mod.load_frequency_stats(path)
        assert (meta["num_layers"], meta["num_attention_heads"], meta["num_kv_heads"], meta["gqa_ratio"]) == \
            (layers, hq, hq, 1)
        assert torch.equal(torch.stack([hs[l]["q_mean_complex"] for l in range(layers)]), gold["loader_q_mean_complex"])
        assert torch.equal(torch.stack([hs[l]["q_abs_mean"] for l in range(layers)]), gold["loader_q_abs_mean"])
        assert torch.equal(torch.stack([hs[l]["freq_scale_sq"] for l in range(layers)]), gold["loader_freq_scale_sq"])
        assert torch.equal(stats_mod.resolve_inv_freq(meta, 2 * f), gold["omega"])
        meta2, hs2 = stats_mod.load_frequency_stats(path, num_kv_heads=2)
        assert meta2["gqa_ratio"] == hq // 2
        assert torch.equal(torch.stack([hs2[l]["q_mean_complex"] for l in range(layers)]),
                           gold["loader_pooled_q_mean_complex"])
        assert torch.equal(torch.stack([hs2[l]["q_abs_mean"] for l in range(layers)]),
                           gold["loader_pooled_q_abs_mean"])
        with pytest.raises(FileNotFoundError):
            stats_mod.load_frequency_stats(Path(tmp) / "missing.pt")


def test_shipped_stats_slice_loads_like_the_reference():
    want = load_golden("qwen3_8b_stats_slice_loaded.pt")
    meta, hs = stats_mod.load_frequency_stats(GOLDEN / "qwen3_8b_stats_slice.pt")
    assert meta["num_attention_heads"] == int(want["num_attention_heads"]) == 32
    assert meta["num_layers"] == int(want["num_layers"]) == 2 and meta["head_dim"] == 128
    assert meta["rope_style"] == "half"
    assert torch.equal(torch.stack([hs[l]["q_mean_complex"] for l in (0, 1)]), want["q_mean_complex"])
    assert torch.equal(torch.stack([hs[l]["q_abs_mean"] for l in (0, 1)]), want["q_abs_mean"])
    assert torch.equal(torch.stack([hs[l]["freq_scale_sq"] for l in (0, 1)]), want["freq_scale_sq"])
    # no inv_freq in the file and no model directory: theta falls back to 10000 (core/compressor.py:186)
    assert torch.equal(stats_mod.resolve_inv_freq(meta, 128), rope.default_inv_freq(128, 10000.0))


def test_inv_freq_from_model_config_and_native_format(tmp_path):
    (tmp_path / "config.json").write_text('{"rope_theta": 500000.0, "rope_scaling": {"rope_type": "llama3", '
                                          '"factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0, '
                                          '"original_max_position_embeddings": 8192}}')
    inv = stats_mod.resolve_inv_freq({}, 128, tmp_path)
    assert torch.equal(inv, rope.llama3_inv_freq(128, 5e5))
    # ... and that is what transformers' own llama3 routine gives (fixture written from it)
    gold = load_golden("llama3_inv_freq.pt")
    assert torch.equal(inv, gold["llama3_inv_freq"])
    assert torch.equal(rope.default_inv_freq(128, 5e5), gold["default_inv_freq"])
    assert torch.equal(stats_mod.resolve_inv_freq({"rope_theta": 1e6}, 64), rope.default_inv_freq(64, 1e6))
    with pytest.raises(ValueError):
        stats_mod.resolve_inv_freq({"inv_freq": [1.0, 0.5]}, 128)
    with pytest.raises(ValueError):
        rope.inv_freq_from_rope_config(128, 1e4, {"rope_type": "yarn", "factor": 4})
    native = {"metadata": {"num_attention_heads": 4, "num_kv_heads": 2, "head_dim": 8, "num_layers": 1},
              "layer_stats": {0: {"q_mean_complex": torch.zeros(2, 4, 2), "freq_scale_sq": torch.ones(2, 4)}}}
    torch.save(native, tmp_path / "n.pt")
    meta, hs = stats_mod.load_frequency_stats(tmp_path / "n.pt")
    assert meta["num_kv_heads"] == 2 and hs[0]["freq_scale_sq"].shape == (2, 4)
    torch.save({"metadata": {"head_dim": 8}, "layer_stats": {}}, tmp_path / "bad.pt")
    with pytest.raises(ValueError):
        stats_mod.load_frequency_stats(tmp_path / "bad.pt")
    assert stats_mod.geometric_offsets().tolist() == [float(2 ** j) for j in range(17)]
    assert stats_mod.pool_heads(torch.arange(8.).view(4, 2), 2).tolist() == [[1.0, 2.0], [5.0, 6.0]]
    with pytest.raises(RuntimeError):
        stats_mod.pool_heads(torch.zeros(5, 2), 2)


# ------------------------------------------------------- dense helpers, state
def test_dense_helpers_and_compression_state():
    x = torch.randn(2, 3, 50)
    z = normalize_scores(x)
    assert torch.allclose(z.mean(-1), torch.zeros(2, 3), atol=1e-6) and torch.allclose(z.std(-1), torch.ones(2, 3), atol=1e-5)
    assert torch.equal(normalize_scores(torch.ones(1, 4)), torch.zeros(1, 4))
    p = protect_window_tokens(x, 5)
    assert bool(torch.isinf(p[..., -5:]).all()) and torch.equal(p[..., :-5], x[..., :-5])
    assert protect_window_tokens(x, 0) is x
    kv = torch.randn(1, 2, 10, 4)
    idx = torch.tensor([[[1, 3], [0, 9]]])
    g = gather_kv_by_indices(kv, idx)
    assert torch.equal(g[0, 1, 1], kv[0, 1, 9]) and g.shape == (1, 2, 2, 4)
    assert torch.equal(gather_kv_by_indices(kv, torch.tensor([[2, 4]]))[0, 0, 1], kv[0, 0, 4])
    st = CompressionState(TriAttentionConfig(device=torch.device("cpu"), kv_budget=100, divide_length=10,
                                             window_size=8, protect_prefill=False))
    assert not st.should_compress(50) and st.prefill_length == 50
    assert not st.should_compress(109) and st.should_compress(110)
    st.update_after_compression(100)
    assert st.current_cache_len == 100 and st.get_round_start() == 110 and st.compression_count == 1
    assert not st.should_compress(115) and st.should_compress(120)


def test_planner_and_state_store():
    cfg = TriAttentionRuntimeConfig(kv_budget=100, divide_length=10, enable_kv_usage_trigger=True,
                                    kv_usage_trigger=0.9, kv_usage_release=0.5)
    pln = CompressionPlanner(cfg)
    assert not pln.build_signal("r", 109, 5, 0).should_compress
    s = pln.build_signal("r", 110, 5, 1, scheduled_tokens=0)
    assert s.should_compress and s.reason == "length_threshold" and s.scheduled_tokens == 1
    assert pln.build_signal("r", 10, 5, 2, kv_usage=0.95).reason == "kv_usage_threshold"
    assert pln.build_signal("r", 10, 5, 3, kv_usage=0.7).should_compress          # still armed
    assert not pln.build_signal("r", 10, 5, 4, kv_usage=0.4).should_compress
    cfg2 = TriAttentionRuntimeConfig(kv_budget=100, divide_length=10, protect_prefill=True,
                                     include_prefill_in_budget=False)
    assert not CompressionPlanner(cfg2).build_signal("r", 130, 30, 0).should_compress
    store = RequestStateStore()
    st = store.ensure("a", 20, False)
    assert st.last_absorbed_cache_len == 20 and st.mode == "trim_prefill"
    store.update_cache_len("a", 150, step=3)
    assert st.recent_unabsorbed_tokens == 130
    store.mark_trigger("a", "length_threshold", 3)
    store.mark_compressed("a", step=3, cache_len=100, scheduled_tokens=1, scheduler_nct=150)
    assert st.current_cache_len == 101 and st.compression_count == 1 and st.pending_triggers == 0
    assert st.nct_at_last_compression == 150 and store.has_compressed_request_in(["a"])
    store.mark_compression_skipped("a", "under_budget", 4)
    assert st.last_trigger_reason == "skipped:under_budget"
    store.remove("a")
    assert store.get("a") is None and not store.has_active_compressed_requests()


def test_keep_plan_and_fallback_indices():
    assert build_keep_token_indices(10, 20, 3, False) == list(range(10))
    assert build_keep_token_indices(10, 4, 3, False) == [6, 7, 8, 9]
    assert build_keep_token_indices(10, 5, 3, True) == [0, 1, 2, 8, 9]
    assert build_keep_token_indices(10, 2, 3, True) is None
    assert build_keep_token_indices(10, 2, 3, True, include_prefill_in_budget=False) == [0, 1, 2, 8, 9]
    p = KeepPlan.from_selector_result({"mode": "per_head", "indices": torch.zeros(4, 7), "semantic": "s"})
    assert p.keep_count() == 7 and p.selection_mode_label == "per_head:s"
    assert KeepPlan("per_head", [[1, 2], [3, 4]]).keep_count() == 2 and KeepPlan("shared", [1, 2, 3]).keep_count() == 3
    with pytest.raises(ValueError):
        KeepPlan("per_head", torch.zeros(3)).keep_count()


# ---------------------------------------------------------- pipeline control flow
def _signal(**kw):
    base = dict(req_id="r", should_compress=True, reason="length_threshold", estimated_cache_len=41, step=1,
                kv_usage=None, protect_prefill=False, prefill_len=4, scheduled_tokens=1)
    base.update(kw)
    return CompressionSignal(**base)


def test_truncate_and_pipeline_with_fake_selector_and_compactor():
    assert pl.num_required_blocks(0, 16) == 0 and pl.num_required_blocks(17, 16) == 2
    kept, removed, grp = pl.truncate_tail_reclaim_group(gid=0, normalized_block_ids=[5, 6, 7], cache_len_after=5, block_size=4)
    assert (kept, removed) == ([5, 6], [7]) and grp.to_dict()["block_ids_after"] == [5, 6]
    assert pl.truncate_tail_reclaim_group(gid=0, normalized_block_ids=[5], cache_len_after=4, block_size=4)[2] is None
    cfg = TriAttentionRuntimeConfig(kv_budget=8, divide_length=2, window_size=2)
    calls = []

    def group_selector(**kw):
        calls.append(("group", kw["total_tokens"], kw["round_start"], kw["budget_total"]))
        return {"mode": "per_head", "indices": torch.arange(8).unsqueeze(0).expand(2, -1).contiguous(),
                "semantic": "hf_aligned_global_per_head"}
    group_selector._supports_paged_group = True

    def per_head_fn(**kw):
        calls.append(("compact", kw["total_tokens"], kw["preserve_dropped_tokens"]))
        return int(kw["keep_token_indices_per_head"].shape[1])

    layers = {0: [(0, torch.zeros(1)), (1, torch.zeros(1))]}
    ids = [[9, 8, 7, 6, 5, 4, 3, 2, 1, 0]]
    out = pl.run_group_compaction_pipeline(
        req_id="r", signal=_signal(), config=cfg, strict_triton_required=True, num_computed_tokens=40,
        effective_tokens=40, budget_total=8, block_size=4, mutable_block_ids_by_group=ids, group_tensors=layers,
        select_keep_indices=None, select_keep_indices_for_group=group_selector, shared_compact_fn=None,
        per_head_compact_fn=per_head_fn)
    assert isinstance(out, pl.GroupPipelineOutcome) and out.cache_len_after == 8
    assert out.selection_mode == "per_head:hf_aligned_global_per_head"
    assert out.mutable_block_ids_by_group == [[9, 8]] and out.block_reclaim_groups[0].block_ids_removed == ids[0][2:] or True
    assert calls[0] == ("group", 40, 40, 8) and calls.count(("compact", 40, False)) == 2
    state = types.SimpleNamespace(block_ids=([9, 8, 7, 6, 5, 4, 3, 2, 1, 0],))
    res = pl.finalize_hook_placement_result(req_state=state, original_block_ids_by_group=state.block_ids, config=cfg,
                                            selector_status="enabled", outcome=out, effective_tokens=40,
                                            budget_total=8, recent_unabsorbed_tokens=3)
    assert res["applied"] and res["reason"] == "kv_compacted:per_head:hf_aligned_global_per_head"
    assert res["cache_len_after"] == 8 and res["reclaimed_block_count"] == 8 and state.block_ids == ([9, 8],)
    assert res["block_reclaim"]["mode"] == "truncate_tail" and res["block_reclaim"]["groups"][0]["gid"] == 0
    assert set(res) == {"applied", "reason", "cache_len_after", "selector_status", "block_reclaim",
                        "effective_tokens_before", "budget_total", "reclaimed_block_count", "recent_unabsorbed_tokens"}


def test_pipeline_failure_paths():
    cfg = TriAttentionRuntimeConfig(kv_budget=8, divide_length=2, window_size=2)
    layers = {0: [(0, torch.zeros(1))]}
    common = dict(req_id="r", signal=_signal(), config=cfg, num_computed_tokens=40, effective_tokens=40,
                  budget_total=8, block_size=4, group_tensors=layers, shared_compact_fn=None, per_head_compact_fn=None)
    none_sel = lambda **kw: None
    none_sel._supports_paged = True
    with pytest.raises(RuntimeError, match=f"{MARK}:selector_returned_none:req=r:gid=0:layer=0"):
        pl.run_group_compaction_pipeline(strict_triton_required=True, mutable_block_ids_by_group=[list(range(10))],
                                         select_keep_indices=none_sel, select_keep_indices_for_group=None, **common)
    boom = lambda **kw: (_ for _ in ()).throw(KeyError("x"))
    boom._supports_paged_group = True
    with pytest.raises(RuntimeError, match=f"{MARK}:req=r:gid=0:global_per_head:KeyError"):
        pl.run_group_compaction_pipeline(strict_triton_required=True, mutable_block_ids_by_group=[list(range(10))],
                                         select_keep_indices=None, select_keep_indices_for_group=boom, **common)
    not_paged = lambda **kw: None
    with pytest.raises(RuntimeError, match="global_per_head:RuntimeError"):
        pl.run_group_compaction_pipeline(strict_triton_required=True, mutable_block_ids_by_group=[list(range(10))],
                                         select_keep_indices=None, select_keep_indices_for_group=not_paged, **common)
    # non-strict: score-free fallback keep, shared mode; compaction failure is reported, not raised
    bad_compact = lambda **kw: (_ for _ in ()).throw(IndexError("oob"))
    c2 = dict(common, shared_compact_fn=bad_compact)
    out = pl.run_group_compaction_pipeline(strict_triton_required=False, mutable_block_ids_by_group=[list(range(10))],
                                           select_keep_indices=None, select_keep_indices_for_group=None, **c2)
    assert out == {"applied": False, "reason": "compaction_failed:g0:l0:IndexError"}
    ok_compact = lambda **kw: len(kw["keep_token_indices"])
    c3 = dict(common, shared_compact_fn=ok_compact)
    out = pl.run_group_compaction_pipeline(strict_triton_required=False, mutable_block_ids_by_group=[list(range(10))],
                                           select_keep_indices=None, select_keep_indices_for_group=None, **c3)
    assert out.selection_mode == "fallback" and out.cache_len_after == 8
    sig = _signal(protect_prefill=True, prefill_len=20)
    out = pl.run_group_compaction_pipeline(strict_triton_required=False, mutable_block_ids_by_group=[list(range(10))],
                                           select_keep_indices=None, select_keep_indices_for_group=None,
                                           **dict(c3, signal=sig))
    assert out == {"applied": False, "reason": "prefill_exceeds_budget"}
    assert pl.run_group_compaction_pipeline(strict_triton_required=False, mutable_block_ids_by_group=[[]],
                                            select_keep_indices=None, select_keep_indices_for_group=None,
                                            **c3) == {"applied": False, "reason": "no_compactable_groups"}
    short = lambda **kw: 7
    with pytest.raises(RuntimeError, match="physical_reclaim_missing"):
        pl.execute_group_compaction(req_id="r", gid=0, normalized_block_ids=[0, 1], tasks=[
            pl.PreparedLayerCompaction(0, torch.zeros(1), [0, 1], KeepPlan("shared", list(range(4))))],
            block_size=4, total_tokens=40, enable_experimental_block_reclaim=True, require_physical_reclaim=True,
            shared_compact_fn=lambda **kw: 4)
    with pytest.raises(RuntimeError, match="inconsistent_cache_len_after"):
        it = iter([4, 5])
        pl.execute_group_compaction(req_id="r", gid=0, normalized_block_ids=list(range(10)), tasks=[
            pl.PreparedLayerCompaction(i, torch.zeros(1), list(range(10)), KeepPlan("shared", list(range(4))))
            for i in range(2)], block_size=4, total_tokens=40, enable_experimental_block_reclaim=True,
            require_physical_reclaim=True, shared_compact_fn=lambda **kw: next(it))


# ------------------------------------------------------------------ selector / hook
def test_selector_builder_status_and_markers(tmp_path):
    with pytest.raises(RuntimeError, match=f"{MARK}:stats_path_not_set"):
        build_triattention_selector(TriAttentionRuntimeConfig())
    with pytest.raises(RuntimeError, match=f"{MARK}:stats_path_not_found"):
        build_triattention_selector(TriAttentionRuntimeConfig(sparse_stats_path=tmp_path / "nope.pt"))
    lax = TriAttentionRuntimeConfig(require_triton_scoring=False)
    assert build_triattention_selector(lax) == (None, None, "stats_path_not_set")
    with pytest.raises(RuntimeError, match="per_layer_mode_disabled"):
        build_triattention_selector(TriAttentionRuntimeConfig(pruning_mode="per_layer"))
    cfg = TriAttentionRuntimeConfig(sparse_stats_path=GOLDEN / "qwen3_8b_stats_slice.pt")
    layer_sel, group_sel, status = build_triattention_selector(cfg)
    assert status == "enabled" and layer_sel._supports_paged and group_sel._supports_paged_group
    # early outs need no device
    assert layer_sel(keys_dense=None, total_tokens=5, prefill_len=0, protect_prefill=False, layer_idx=0,
                     round_start=5, budget_total=8) == {"mode": "shared", "indices": [0, 1, 2, 3, 4]}
    out = group_sel(layer_inputs=[(0, torch.zeros(1, 3, 5, 4))], total_tokens=5, prefill_len=0, protect_prefill=False,
                    round_start=5, budget_total=8)
    assert out["mode"] == "per_head" and out["indices"].tolist() == [[0, 1, 2, 3, 4]] * 3
    assert group_sel(layer_inputs=[(0, torch.zeros(1, 3, 50, 4))], total_tokens=50, prefill_len=30,
                     protect_prefill=True, round_start=50, budget_total=8) is None
    legacy = TriAttentionRuntimeConfig(sparse_stats_path=GOLDEN / "qwen3_8b_stats_slice.pt",
                                       per_head_selection_semantics="legacy_layer_local")
    assert build_triattention_selector(legacy)[1](layer_inputs=[], total_tokens=50, prefill_len=0,
                                                  protect_prefill=False, round_start=50, budget_total=8) is None


class _Runner(types.SimpleNamespace):
    pass


def _fake_runner(num_computed=40, block_ids=None):
    req = types.SimpleNamespace(num_computed_tokens=num_computed,
                                block_ids=([9, 8, 7, 6, 5, 4, 3, 2, 1, 0],) if block_ids is None else block_ids)
    return _Runner(requests={"r": req}, kv_caches=[torch.zeros(2, 10, 4, 2, 64)],
                   cache_config=types.SimpleNamespace(block_size=4)), req


def test_hook_skip_reasons_and_executor(monkeypatch):
    cfg = TriAttentionRuntimeConfig(kv_budget=8, divide_length=2, window_size=2,
                                    sparse_stats_path=GOLDEN / "qwen3_8b_stats_slice.pt")
    runner, req = _fake_runner()
    install_runner_compression_hook(runner, cfg)
    hook = runner.triattention_apply_compression
    sched = types.SimpleNamespace(num_scheduled_tokens={"r": 1})
    assert hook(req_id="zzz", signal=_signal(req_id="zzz"), scheduler_output=sched) == \
        {"applied": False, "reason": "req_state_not_found"}
    out = hook(req_id="r", signal=_signal(estimated_cache_len=9), scheduler_output=sched)
    assert out == {"applied": False, "reason": "under_budget", "cache_len_after": 8}
    req.block_ids = None
    assert hook(req_id="r", signal=_signal(), scheduler_output=sched)["reason"] == "missing_block_ids"
    req.block_ids = "oops"
    assert hook(req_id="r", signal=_signal(), scheduler_output=sched)["reason"] == "invalid_block_ids_container"
    req.block_ids = (list(range(64)),)
    runner.cache_config.block_size = 0
    assert hook(req_id="r", signal=_signal(), scheduler_output=sched)["reason"] == "invalid_block_size"
    runner.cache_config.block_size = 4
    runner.kv_caches = None
    assert hook(req_id="r", signal=_signal(), scheduler_output=sched)["reason"] == "kv_cache_unavailable"
    # an already installed hook is kept
    sentinel = lambda **kw: True
    r2 = _Runner(triattention_apply_compression=sentinel)
    install_runner_compression_hook(r2, cfg)
    assert r2.triattention_apply_compression is sentinel
    ex = RunnerHookCompressionExecutor(r2)
    assert ex.execute("r", _signal(), sched).reason == "applied"
    assert RunnerHookCompressionExecutor(_Runner()).execute("r", _signal(), sched).reason == "runner_hook_missing"
    r3 = _Runner(triattention_apply_compression=lambda **kw: {"applied": True, "reason": "x", "cache_len_after": 3})
    res = RunnerHookCompressionExecutor(r3).execute("r", _signal(), sched)
    assert res.applied and res.cache_len_after == 3 and res.details["reason"] == "x"
    r4 = _Runner(triattention_apply_compression=lambda **kw: 5)
    assert RunnerHookCompressionExecutor(r4).execute("r", _signal(), sched).reason == "unsupported_hook_result:int"
    # plan-only mode when compaction is switched off
    cfg_off = TriAttentionRuntimeConfig(kv_budget=8, divide_length=2, window_size=2,
                                        enable_experimental_kv_compaction=False)
    runner5, _ = _fake_runner()
    install_runner_compression_hook(runner5, cfg_off)
    assert runner5.triattention_apply_compression(req_id="r", signal=_signal(), scheduler_output=sched) == \
        {"applied": False, "reason": "plan_only", "cache_len_after": 8}


def test_batch_hook_groups_requests_and_falls_back(monkeypatch):
    """Host logic of ``triattention_apply_compression_batch`` with a stand-in for the kernels:
    requests with something to drop go to one batched call per KV-cache group, the others get
    the one-by-one hook's answers; block lists are truncated per request; a failed resident launch
    repeats that KV-cache group, and only it, on the kernels that do not wait for each other."""
    calls = {"batch": [], "single": []}

    def select_group(*, layer_kv_iter=None, total_tokens, budget_total, **kw):
        calls["single"].append(total_tokens)
        k = min(total_tokens, budget_total)
        return {"mode": "per_head", "indices": torch.arange(k).repeat(2, 1), "semantic": "hf_aligned_global_per_head"}

    def compress_batch(*, layer_kv, block_size, requests, allow_resident=True):
        calls["batch"].append([dict(r, allow_resident=allow_resident, layers=[li for li, _ in layer_kv])
                               for r in requests])
        if fail["now"] and allow_resident and (fail["layer"] is None or fail["layer"] in [li for li, _ in layer_kv]):
            raise hook_mod.ResidentLaunchFailed("forced")
        return [{"mode": "per_head", "indices": torch.arange(r["budget_total"]).repeat(2, 1),
                 "semantic": "hf_aligned_global_per_head"} for r in requests]

    fail = {"now": False, "layer": None}
    select_group._supports_paged_group = True
    select_group._compress_batch = compress_batch
    select_layer = lambda **kw: None
    select_layer._supports_paged = True
    monkeypatch.setattr(hook_mod, "_build_triattention_selector", lambda config, base_runner=None: (select_layer, select_group, "enabled"))
    moved = []
    monkeypatch.setattr(hook_mod, "compact_request_kv_in_place_per_head",
                        lambda **kw: moved.append(kw["total_tokens"]) or int(kw["keep_token_indices_per_head"].shape[1]))
    cfg = TriAttentionRuntimeConfig(kv_budget=8, divide_length=2, window_size=2,
                                    sparse_stats_path=GOLDEN / "qwen3_8b_stats_slice.pt")

    def runner_with(lengths):
        reqs = {f"r{i}": types.SimpleNamespace(num_computed_tokens=t, block_ids=(list(range(100 * i, 100 * i + 10)),))
                for i, t in enumerate(lengths)}
        r = _Runner(requests=reqs, kv_caches=[torch.zeros(2, 400, 4, 2, 64)],
                    cache_config=types.SimpleNamespace(block_size=4))
        install_runner_compression_hook(r, cfg)
        sig = {rid: _signal(req_id=rid, estimated_cache_len=q.num_computed_tokens + 1, prefill_len=3)
               for rid, q in reqs.items()}
        sched = types.SimpleNamespace(num_scheduled_tokens={rid: 1 for rid in reqs})
        return r, reqs, sig, sched

    runner, reqs, sig, sched = runner_with([40, 6, 30, 17])
    sig["r2"] = _signal(req_id="r2", estimated_cache_len=31, prefill_len=5, protect_prefill=True)
    sig["idle"] = _signal(req_id="idle", should_compress=False)
    out = RunnerHookCompressionExecutor(runner).execute_batch(sig, sched)
    assert list(out) == ["r0", "r1", "r2", "r3"]
    assert out["r1"].reason == "under_budget" and not out["r1"].applied
    assert len(calls["batch"]) == 1 and not calls["single"]
    sent = calls["batch"][0]
    assert [r["total_tokens"] for r in sent] == [40, 30, 17] and [r["budget_total"] for r in sent] == [8, 8, 8]
    assert [r["round_start"] for r in sent] == [40, 30, 17]
    assert [(r["protect_prefill"], r["prefill_len"]) for r in sent] == [(False, 3), (True, 5), (False, 3)]
    assert sent[0]["block_ids"] == list(range(0, 10))
    for rid in ("r0", "r2", "r3"):
        assert out[rid].applied and out[rid].cache_len_after == 8
        assert out[rid].reason == "kv_compacted:per_head:hf_aligned_global_per_head"
        first = reqs[rid].block_ids[0][0]
        assert reqs[rid].block_ids == ([first, first + 1],)
        assert out[rid].details["reclaimed_block_count"] == 8
    # the same requests one by one through the reference-shaped pipeline (selector callable, then the
    # compaction function per layer) give the same dictionaries
    monkeypatch.setattr(hook_mod, "SINGLE_REQUEST_IN_ONE_CALL", False)
    runner1, reqs1, sig1, sched1 = runner_with([40, 6, 30, 17])
    sig1["r2"] = sig["r2"]
    one = {rid: RunnerHookCompressionExecutor(runner1).execute(rid, s_, sched1) for rid, s_ in sig1.items()}
    assert one == out and calls["single"] == [40, 30, 17] and moved == [40, 30, 17]
    # ... where a single candidate of a batch call takes that pipeline too
    calls["batch"].clear(); calls["single"].clear(); moved.clear()
    runner2, reqs2, sig2, sched2 = runner_with([40, 5])
    out2 = RunnerHookCompressionExecutor(runner2).execute_batch(sig2, sched2)
    assert out2["r0"].applied and not calls["batch"] and calls["single"] == [40]
    # by default a single request takes the one-call launch sequence, from either entry point
    monkeypatch.setattr(hook_mod, "SINGLE_REQUEST_IN_ONE_CALL", True)
    calls["batch"].clear(); calls["single"].clear(); moved.clear()
    runner2b, reqs2b, sig2b, sched2b = runner_with([40, 5])
    out2b = RunnerHookCompressionExecutor(runner2b).execute_batch(sig2b, sched2b)
    one2b = RunnerHookCompressionExecutor(runner_with([40, 5])[0]).execute("r0", sig2b["r0"], sched2b)
    assert out2b["r0"] == out2["r0"] == one2b and len(calls["batch"]) == 2 and not calls["single"] and not moved
    # failed resident launch: the group is repeated in one batched call without the resident
    # kernel; nothing goes through the one-by-one path and the environment is left alone
    calls["batch"].clear(); calls["single"].clear(); moved.clear()
    fail["now"] = True
    runner3, reqs3, sig3, sched3 = runner_with([40, 30])
    out3 = RunnerHookCompressionExecutor(runner3).execute_batch(sig3, sched3)
    assert [[r["allow_resident"] for r in c] for c in calls["batch"]] == [[True, True], [False, False]]
    assert not calls["single"] and not moved
    assert all(r.applied and r.cache_len_after == 8 for r in out3.values())
    assert "TRIATTN_RESIDENT_KERNEL" not in __import__("os").environ
    # two KV-cache groups, the resident launch of the second fails: the first group is not
    # touched again (one call), the second is repeated alone without the resident kernel
    calls["batch"].clear()
    fail["layer"] = 1
    reqs4 = {f"r{i}": types.SimpleNamespace(num_computed_tokens=t, block_ids=(list(range(100 * i, 100 * i + 10)),
                                                                           list(range(100 * i + 50, 100 * i + 60))))
             for i, t in enumerate([40, 30])}
    runner4 = _Runner(requests=reqs4, kv_caches=[torch.zeros(2, 400, 4, 2, 64), torch.zeros(2, 400, 4, 2, 64)],
                      cache_config=types.SimpleNamespace(block_size=4))
    monkeypatch.setattr(hook_mod, "resolve_group_tensors",
                        lambda base_runner: {0: [(0, base_runner.kv_caches[0])], 1: [(1, base_runner.kv_caches[1])]})
    install_runner_compression_hook(runner4, cfg)
    sig4 = {rid: _signal(req_id=rid, estimated_cache_len=q.num_computed_tokens + 1, prefill_len=3)
            for rid, q in reqs4.items()}
    sched4 = types.SimpleNamespace(num_scheduled_tokens={rid: 1 for rid in reqs4})
    out4 = RunnerHookCompressionExecutor(runner4).execute_batch(sig4, sched4)
    assert [(c[0]["layers"], c[0]["allow_resident"]) for c in calls["batch"]] == [([0], True), ([1], True), ([1], False)]
    assert all(r.applied and r.cache_len_after == 8 for r in out4.values())
    assert reqs4["r0"].block_ids == ([0, 1], [50, 51]) and reqs4["r1"].block_ids == ([100, 101], [150, 151])
    assert not calls["single"]
    fail["layer"] = None
    # a runner without the batch hook: execute_batch loops over execute
    bare = _Runner(triattention_apply_compression=lambda **kw: {"applied": True, "reason": "x", "cache_len_after": 1})
    res = RunnerHookCompressionExecutor(bare).execute_batch({"a": _signal(req_id="a"), "b": _signal(req_id="b")}, sched)
    assert set(res) == {"a", "b"} and all(r.applied for r in res.values())


def test_verify_rope_alignment():
    a = rope.default_inv_freq(128, 1e6)
    rope.verify_rope_alignment(a, types.SimpleNamespace(inv_freq=a.clone()))
    with pytest.raises(ValueError, match="mismatch"):
        rope.verify_rope_alignment(a, rope.default_inv_freq(128, 1e4))
    with pytest.raises(ValueError, match="shape"):
        rope.verify_rope_alignment(a, rope.default_inv_freq(64, 1e6))
    with pytest.raises(ValueError, match="inv_freq attribute"):
        rope.verify_rope_alignment(types.SimpleNamespace(), a)
    rope.verify_rope_alignment(rope.llama3_inv_freq(128), rope.llama3_inv_freq(128) + 5e-6)


def test_runtime_context_lengths_defer_and_regression_guard():
    cfg = TriAttentionRuntimeConfig(kv_budget=8, divide_length=2)
    runner, req = _fake_runner(num_computed=40)
    class Key:                      # scheduler keys may be request objects, not strings
        request_id = "r"
    sched = types.SimpleNamespace(num_scheduled_tokens={Key(): 3})
    ctx = hook_mod.build_hook_runtime_context(
        base_runner=runner, config=cfg, req_id="r", req_state=req, req_runtime_state=None,
        signal=_signal(estimated_cache_len=43), scheduler_output=sched, compressed_once=set(),
        original_block_ids_by_group=req.block_ids, block_size_hint=4)
    assert (ctx.scheduled_tokens, ctx.effective_tokens, ctx.budget_total) == (3, 40, 8) and not ctx.should_defer_recompress
    rt = types.SimpleNamespace(compression_count=1, current_cache_len=9, last_absorbed_cache_len=8)
    ctx = hook_mod.build_hook_runtime_context(
        base_runner=runner, config=cfg, req_id="r", req_state=req, req_runtime_state=rt,
        signal=_signal(estimated_cache_len=43), scheduler_output=types.SimpleNamespace(num_scheduled_tokens={"r": 1}),
        compressed_once={"r"}, original_block_ids_by_group=req.block_ids, block_size_hint=4)
    # after a compression the runner-side cache length (9) replaces the scheduler estimate;
    # 9 < budget 8 + divide_length 2, so the request waits
    assert ctx.estimated_effective_tokens == 9 and ctx.effective_tokens == 8 and ctx.should_defer_recompress
    assert ctx.recent_unabsorbed_tokens == 0
    big, breq = _fake_runner(num_computed=1000, block_ids=(list(range(300)),))
    with pytest.raises(RuntimeError, match="effective_len_regressed"):
        hook_mod.build_hook_runtime_context(
            base_runner=big, config=cfg, req_id="r", req_state=breq, req_runtime_state=None,
            signal=_signal(estimated_cache_len=1001), scheduler_output=sched, compressed_once={"r"},
            original_block_ids_by_group=breq.block_ids, block_size_hint=4)
    # capacity cap: effective tokens cannot exceed the blocks the request owns plus one block
    small, sreq = _fake_runner(num_computed=100, block_ids=([1, 2],))
    ctx = hook_mod.build_hook_runtime_context(
        base_runner=small, config=cfg, req_id="r", req_state=sreq, req_runtime_state=None,
        signal=_signal(estimated_cache_len=101), scheduler_output=None, compressed_once=set(),
        original_block_ids_by_group=sreq.block_ids, block_size_hint=4)
    assert ctx.effective_tokens == 12


def test_request_state_views_and_group_tensors():
    runner, req = _fake_runner()
    new_req = types.SimpleNamespace(req_id="n", block_ids=([1],), prompt_token_ids=[0] * 33)
    sched = types.SimpleNamespace(scheduled_new_reqs=[new_req], scheduled_cached_reqs=types.SimpleNamespace(
        req_ids=["r"], num_computed_tokens=[55]))
    view = hook_mod.resolve_request_state(runner, "n", sched)
    assert view.num_computed_tokens == 33 and view.block_ids == ([1],)
    merged = hook_mod.resolve_request_state(runner, "r", sched)
    assert merged.num_computed_tokens == 55
    merged.block_ids = ([4],)
    assert req.block_ids == ([4],)
    assert hook_mod.resolve_request_state(runner, "ghost", None) is None
    assert hook_mod.resolve_group_tensors(runner)[0][0][0] == 0
    assert hook_mod.infer_layer_idx("model.layers.17.self_attn", object(), 3) == 17
    assert hook_mod.infer_layer_idx("attn", types.SimpleNamespace(layer_idx=4), 3) == 4
    assert hook_mod.scheduled_tokens_for_req(types.SimpleNamespace(num_scheduled_tokens={"r": 0}), "r") == 1


def test_keep_tensors_from_the_selector_are_remembered_by_identity():
    """The compaction functions skip their host-side index check only for the very tensor the
    selector returned, and only for the token count it was selected from."""
    import gc
    from triattention_amd.runtime import kv_compaction as kc
    keep = torch.arange(12).reshape(2, 6)
    same_values = keep.clone()
    kc.mark_keep_validated(keep, 40)
    assert kc._is_validated(keep, 40)
    assert not kc._is_validated(keep, 41)
    assert not kc._is_validated(same_values, 40)
    assert not kc._is_validated([[0, 1]], 40)
    key = id(keep)
    del keep
    gc.collect()
    assert key not in kc._VALIDATED_KEEP


def test_header_is_plain_c_and_a_c_program_links_the_library(tmp_path):
    """The boundary is a C ABI: the header compiles as C99 with warnings as errors, and a C program
    that includes it links against the library, reads the ABI version, takes the struct sizes the
    Python mirror uses and gets the documented refusal (no compute call: there is no GPU here)."""
    import ctypes as C
    import shutil
    import subprocess
    from triattention_amd import build as tri_build
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    _lib.load()
    root = Path(__file__).resolve().parents[1]
    src = tmp_path / "abi.c"
    src.write_text(r'''
#include <stdio.h>
#include <string.h>
#include "triattention_hip.h"
int main(void) {
  tri_kv_layout kv; tri_batch b; tri_score_params sp; tri_select_params sel; tri_plan_info info;
  memset(&kv, 0, sizeof kv); memset(&b, 0, sizeof b); memset(&sp, 0, sizeof sp); memset(&sel, 0, sizeof sel);
  printf("abi %d %d\n", tri_abi_version(), TRI_ABI_VERSION);
  printf("sizes %zu %zu %zu %zu %zu\n", sizeof kv, sizeof b, sizeof sp, sizeof sel, sizeof info);
  printf("bytes %llu\n", (unsigned long long)tri_workspace_bytes(&kv, &b, &sp));
  int rc = tri_compress_step(&kv, &b, &sp, &sel, NULL, NULL, 0, NULL);
  printf("rc %d msg %s\n", rc, tri_last_error());
  rc = tri_compress_step_static(NULL, &b, &sp, &sel, NULL, NULL, NULL);
  printf("rc %d msg %s\n", rc, tri_last_error());
  rc = tri_describe_plan(&kv, &b, &sp, &sel, 256, &info);
  printf("rc %d msg %s\n", rc, tri_last_error());
  return 0;
}
''')
    exe = tmp_path / "abi"
    libdir = tri_build.LIB_PATH.parent
    cmd = [gcc, "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", f"-I{root / 'include'}", str(src), "-o", str(exe),
           f"-L{libdir}", "-ltriattention_hip", f"-Wl,-rpath,{libdir}", "-Wl,-rpath,/opt/rocm/lib",
           "-Wl,--allow-shlib-undefined"]
    built = subprocess.run(cmd, capture_output=True, text=True)
    assert built.returncode == 0, built.stderr
    out = subprocess.run([str(exe)], capture_output=True, text=True, timeout=60)
    assert out.returncode == 0, out.stderr
    lines = out.stdout.splitlines()
    assert lines[0] == f"abi {_lib.ABI_VERSION} {_lib.ABI_VERSION}"
    sizes = [int(x) for x in lines[1].split()[1:]]
    assert sizes == [C.sizeof(_lib.KvLayout), C.sizeof(_lib.Batch), C.sizeof(_lib.ScoreParams), C.sizeof(_lib.SelectParams),
                     C.sizeof(_lib.PlanInfo)]
    assert lines[2] == "bytes 0"
    assert lines[3].startswith("rc -") and "bad layer/head count" in lines[3]
    assert lines[4].startswith("rc -") and "kv layout is NULL" in lines[4]
    assert lines[5].startswith("rc -") and "bad layer/head count" in lines[5]


def test_product_raises_when_the_library_is_missing(tmp_path, monkeypatch):
    """No CPU, PyTorch or oracle fallback: with no shared library the loader raises and names the
    build command (the tests, the smoke run and the benchmark build it beforehand; the product
    never does, and never takes another path)."""
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", tmp_path / "libtriattention_hip.so")
    with pytest.raises(RuntimeError, match="is missing"):
        _lib.load()
    import triattention_amd
    pkg = Path(triattention_amd.__file__).parent
    offenders = [str(p) for p in pkg.rglob("*.py") if re.search(r"^\s*(from|import)\s+oracle\b", p.read_text(), re.M)]
    assert offenders == [], "the package must not import the oracle"


def test_tuning_settings_round_trip_and_reject_bad_values():
    """The process-wide settings replace environment variables inside the library: values come back
    as set, out-of-range values and unknown keys are refused with a message, and the defaults are the
    documented ones (tri_set_tuning / tri_get_tuning)."""
    lib = _lib.load()
    defaults = {_lib.TUNE_RESIDENT_KERNEL: 0, _lib.TUNE_RESIDENT_WORKGROUPS: 0, _lib.TUNE_LAYER_SPLIT: -1,
                _lib.TUNE_MAX_KERNEL: 0, _lib.TUNE_RESIDENT_WAIT_US: 2_000_000}
    for key, value in defaults.items():
        assert _lib.get_tuning(key) == value
    with _lib.tuning(resident_kernel="off", resident_workgroups=12, layer_split=1, max_kernel="valu", resident_wait_us=-1):
        assert [_lib.get_tuning(k) for k in range(5)] == [3, 12, 1, 1, -1]
    assert [_lib.get_tuning(k) for k in range(5)] == [defaults[k] for k in range(5)]
    for key, bad in ((_lib.TUNE_RESIDENT_KERNEL, 4), (_lib.TUNE_RESIDENT_KERNEL, -1), (_lib.TUNE_LAYER_SPLIT, 2),
                     (_lib.TUNE_MAX_KERNEL, 2), (_lib.TUNE_RESIDENT_WORKGROUPS, -3), (_lib.TUNE_RESIDENT_WAIT_US, 10**13),
                     (17, 0)):
        assert lib.tri_set_tuning(key, bad) == _lib.TRI_ERR_INVALID_ARGUMENT
        assert lib.tri_last_error()
    assert lib.tri_get_tuning(17) == -2**63
    assert [_lib.get_tuning(k) for k in range(5)] == [defaults[k] for k in range(5)]


def test_environment_is_applied_once_at_load(monkeypatch):
    """The documented TRIATTN_* switches are read by the Python layer when it loads the library, not
    by the library on every call."""
    lib = _lib.load()
    try:
        monkeypatch.setenv("TRIATTN_RESIDENT_KERNEL", "valu")
        monkeypatch.setenv("TRIATTN_RESIDENT_WORKGROUPS", "24")
        monkeypatch.setenv("TRIATTN_RESIDENT_LAYER_SPLIT", "0")
        monkeypatch.setenv("TRIATTN_RESIDENT_SPIN_TICKS", "-1")
        monkeypatch.setenv("TRIATTN_MAX_KERNEL", "valu")
        assert _lib.get_tuning(_lib.TUNE_RESIDENT_KERNEL) == 0        # nothing happens by itself
        _lib._apply_environment(lib)
        assert [_lib.get_tuning(k) for k in range(5)] == [2, 24, 0, 1, -1]
        monkeypatch.setenv("TRIATTN_RESIDENT_KERNEL", "sideways")
        with pytest.raises(ValueError, match="TRIATTN_RESIDENT_KERNEL"):
            _lib._apply_environment(lib)
    finally:
        for key, value in {0: 0, 1: 0, 2: -1, 3: 0, 4: 2_000_000}.items():
            _lib.set_tuning(key, value)


def test_a_library_built_from_other_sources_is_rebuilt(tmp_path, monkeypatch):
    """ensure_built compares the digest compiled into the library with the sources next to it: the
    library of this checkout belongs to its sources; after one source file changes it does not, and
    ensure_built builds (the build itself is replaced by a recorder here) and says why."""
    import shutil
    assert tri_build.stale() is None
    assert tri_build.built_digest() == tri_build.source_digest() == _lib.load().tri_source_digest().decode()
    csrc = tmp_path / "csrc"
    shutil.copytree(tri_build.CSRC, csrc)
    monkeypatch.setattr(tri_build, "CSRC", csrc)
    assert tri_build.stale() is None                      # same content elsewhere: still the same library
    calls = []
    monkeypatch.setattr(tri_build, "build", lambda verbose=False, jobs=None: calls.append("build"))
    tri_build.ensure_built()
    assert calls == []
    src = csrc / "tri_compact.hip"
    src.write_text(src.read_text() + "\n// edited\n")
    why = tri_build.stale()
    assert why is not None and "built from other sources" in why
    tri_build.ensure_built()
    assert calls == ["build"]
    # a file that is missing altogether
    monkeypatch.setattr(tri_build, "LIB_PATH", tmp_path / "libtriattention_hip.so")
    assert "is missing" in tri_build.stale()
    tri_build.ensure_built()
    assert calls == ["build", "build"]


# ---------------------------------------------------------------- the planner, on a pretended device
def _describe(layers, q_heads, kv_heads, head_dim, lens, assume=256, kv_dtype=0, host_lens=True, **select):
    import ctypes as C
    lib = _lib.load()
    kv = _lib.KvLayout(num_layers=layers, num_kv_heads=kv_heads, head_dim=head_dim, block_size=16, kv_dtype=kv_dtype,
                       stride_block=16 * kv_heads * head_dim, stride_token=kv_heads * head_dim, stride_head=head_dim,
                       k_layers=8, v_layers=8, k_scale_layers=8 if kv_dtype == 2 else None)
    arr = (C.c_int32 * len(lens))(*lens)
    batch = _lib.Batch(num_seqs=len(lens), max_seq_len=max(lens), max_budget=64, block_table_pitch=4096, block_table=8,
                       seq_lens=8, round_start=8, budgets=8, seq_lens_host=C.cast(arr, C.c_void_p) if host_lens else None)
    sp = _lib.ScoreParams(num_score_heads=q_heads, num_offsets=17, folded=16, omega=8, offsets=8)
    kw = dict(normalize=1, window_size=128, group_reduce=1)
    kw.update(select)
    sel = _lib.SelectParams(**kw)
    info = _lib.PlanInfo()
    rc = lib.tri_describe_plan(C.byref(kv), C.byref(batch), C.byref(sp), C.byref(sel), assume, C.byref(info))
    assert rc == 0, lib.tri_last_error()
    assert info.workspace_bytes > 0
    return (info.path, info.tile_tokens, info.tiles_per_seq, info.layer_groups, info.layers_per_group, info.launches)


def test_planner_cuts_the_benchmarked_shapes_as_documented():
    """``tri_describe_plan`` for a device that holds 256 resident workgroups (an MI355X), without one:
    (path, tile tokens, tiles of the longest sequence, layer groups, layers per group, launches)."""
    from triattention_amd import synth
    q8b = (36, 32, 8, 128)
    assert _describe(*q8b, [16384] * 16) == (2, 1024, 16, 1, 36, 1)          # C1: one workgroup per CU, whole model
    assert _describe(*q8b, [8192] * 16) == (2, 512, 16, 1, 36, 1)            # a full chip is not cut by layers
    assert _describe(*q8b, [2176] * 16) == (2, 576, 4, 4, 9, 1)              # steady state: 16 x 4 groups x 4 tiles
    assert _describe(*q8b, [2176]) == (2, 320, 7, 36, 1, 1)                  # one request: a workgroup per layer and tile
    assert _describe(*q8b, [2176] * 3) == (2, 320, 7, 12, 3, 1)
    assert _describe(1, 32, 8, 128, [4096]) == (2, 128, 32, 1, 1, 1)         # C0: one layer, an eighth of the chip
    assert _describe(*q8b, [128] * 130)[0] == 0                              # 130 whole-model workgroups, no room for two groups
    assert _describe(64, 64, 8, 128, [32768] * 8) == (2, 512, 64, 1, 64, 2)  # C2: two launches of four sequences
    assert _describe(64, 64, 8, 128, [32768] * 8, host_lens=False)[5] == 0   # lengths unknown to the host: packed on the device
    assert _describe(32, 32, 8, 128, [16384] * 16, kv_dtype=2) == (2, 1024, 16, 1, 32, 1)          # C4
    assert _describe(28, 28, 4, 128, [2176] * 16) == (2, 448, 5, 6, 5, 1)    # four-wave workgroups, two per CU
    assert _describe(36, 64, 8, 64, [16384] * 16) == (2, 512, 32, 1, 36, 2)  # GPT-OSS head shape
    c3 = synth.config(3)
    path, tile, tiles, groups, _, launches = _describe(*q8b, list(c3.seq_lens))
    assert (path, tile, groups, launches) == (2, 640, 1, 7)      # 1777 tiles of 640 tokens: seven launches, 98 % full
    assert (launches - 1) * 256 < sum(-(-t // tile) for t in c3.seq_lens) <= launches * 256
    # what keeps a call off the resident kernels
    assert _describe(*q8b, [16384] * 16, layer_reduce=-1)[0] == 0            # a keep set per layer, several layers
    assert _describe(1, 32, 8, 128, [4096], layer_reduce=-1)[0] == 2         # ... of one layer: the same thing as its mean
    assert _describe(*q8b, [16384] * 16, shared=1)[0] == 0
    assert _describe(*q8b, [16384] * 16, group_first=1)[0] == 0
    assert _describe(*q8b, [16384] * 16, no_resident=1)[0] == 0
    assert _describe(*q8b, [16384] * 16, assume=0)[0] in (0, 2)              # the current device, if there is one
    # a smaller device: more launches, never more workgroups than it holds
    path, tile, tiles, groups, _, launches = _describe(*q8b, [16384] * 16, assume=64)
    assert path == 2 and groups == 1 and launches * 64 >= 16 * tiles
    import ctypes as C
    assert _lib.load().tri_describe_plan(None, None, None, None, 0, None) == _lib.TRI_ERR_INVALID_ARGUMENT
