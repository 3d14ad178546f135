"""Host-integer logic of the hot path against what the REFERENCE returns for the same scenarios.

``tests/golden/host_scenarios.py`` drives both: ``tests/golden/make_hook_golden.py`` ran it with the
reference's functions and stored the outcome in ``tests/golden/host_logic.json``; here it runs with this
package's functions (``runtime/hook.py``, ``runtime/pipeline.py``, ``runtime/models.py``,
``runtime/engine_glue.py``) and every recorded value -- result dictionaries, block lists, the arguments
the selector and the compaction functions were called with, exception types and messages, tracker and
state-store snapshots, event lists, override tuples -- must be equal."""
from __future__ import annotations

import json
import logging
import sys
import types

import pytest

from conftest import GOLDEN

sys.path.insert(0, str(GOLDEN))
import host_scenarios  # noqa: E402

from triattention_amd.runtime import (CompressionPlanner, CompressionSignal, RequestStateStore,  # noqa: E402
                                      TriAttentionRuntimeConfig)
from triattention_amd.runtime import engine_glue  # noqa: E402
from triattention_amd.runtime import hook as hook_mod  # noqa: E402


@pytest.fixture(scope="module")
def golden():
    return json.loads((GOLDEN / "host_logic.json").read_text())


@pytest.fixture()
def api(monkeypatch):
    def make_hook(runner, config, select_layer, select_group, compact_shared, compact_per_head, gather):
        monkeypatch.setattr(hook_mod, "_build_triattention_selector",
                            lambda cfg, base_runner=None: (select_layer, select_group, "enabled"))
        monkeypatch.setattr(hook_mod, "compact_request_kv_in_place", compact_shared)
        monkeypatch.setattr(hook_mod, "compact_request_kv_in_place_per_head", compact_per_head)
        monkeypatch.setattr(hook_mod, "gather_request_k_dense", gather)
        return hook_mod.make_runner_compression_hook(base_runner=runner, config=config)

    logging.disable(logging.CRITICAL)
    yield types.SimpleNamespace(
        Config=TriAttentionRuntimeConfig, Signal=CompressionSignal, Planner=CompressionPlanner,
        Tracker=engine_glue.EffectiveCacheLenTracker, StateStore=RequestStateStore,
        Executor=hook_mod.RunnerHookCompressionExecutor,
        runtime_context=hook_mod.build_hook_runtime_context, make_hook=make_hook,
        worker_reclaim=lambda runner, events: engine_glue.apply_worker_block_reclaim_events(base_runner=runner,
                                                                                            events=events),
        sparse_overrides=lambda runner, store, sched, events: engine_glue.build_effective_sparse_overrides(
            base_runner=runner, state_store=store, scheduler_output=sched, compression_events=events),
        # (one request at a time, as the reference's loop does; the batched route has tests of its own)
        runner_actions=lambda executor, store, sched, signals, strict, allowed: engine_glue.execute_runner_compression_actions(
            executor=executor, state_store=store, scheduler_output=sched, signals=signals, strict_no_downgrade=strict,
            allowed_strict_skip_reasons=set(allowed), log_decisions=False, batched=False),
    )
    logging.disable(logging.NOTSET)


def _same(got, want, where=""):
    """Deep equality with a path in the failure message."""
    if isinstance(want, dict):
        assert isinstance(got, dict), f"{where}: {got!r} is not a dict"
        assert sorted(got) == sorted(want), f"{where}: keys {sorted(got)} != {sorted(want)}"
        for k in want:
            _same(got[k], want[k], f"{where}.{k}")
    elif isinstance(want, list):
        assert isinstance(got, list) and len(got) == len(want), f"{where}: {got!r} != {want!r}"
        for i, (g, w) in enumerate(zip(got, want)):
            _same(g, w, f"{where}[{i}]")
    else:
        assert got == want and type(got) is type(want), f"{where}: {got!r} != {want!r}"


def _through_json(value):
    return json.loads(json.dumps(value, sort_keys=True))


def test_runtime_context_matches_the_reference(api, golden):
    """569 combinations of settings, request progress, scheduler estimates, runtime state, block lists,
    prefill lengths and trigger reasons: effective tokens, budget, deferral, the attribute left on the
    runner, and the regression guard's error text (runtime/hook_runtime_context.py:106-209)."""
    got = _through_json(host_scenarios.runtime_context_cases(api))
    want = golden["runtime_context"]
    assert len(got) == len(want) == 569
    raised = sum("raises" in c["result"] for c in want)
    deferred = sum(bool(c["result"].get("ok", {}).get("should_defer_recompress")) for c in want)
    assert raised >= 5 and deferred >= 20, "the grid must keep exercising the guard and the deferral"
    for i, (g, w) in enumerate(zip(got, want)):
        _same(g, w, f"case {i} {({k: v for k, v in w.items() if k != 'result'})}")


@pytest.mark.parametrize("name", list(host_scenarios.HOOK_SCENARIOS))
def test_hook_results_and_block_lists_match_the_reference(api, golden, name):
    """The hook end to end with stand-ins for the scorer and the row moves: result dictionary (or the
    exception), ``req_state.block_ids`` before and after and its container type, what the selector
    callables and the compaction functions were called with, for one and two KV-cache groups, first and
    repeated compressions (runtime/hook_impl.py:59-165, hook_group_pipeline.py:42-200,
    selection_planner.py:94-275, layout_engine.py:57-227)."""
    got = _through_json(host_scenarios.hook_scenario(api, name))
    _same(got, golden["hook"][name], name)


def test_planner_and_tracker_over_decode_loops_match_the_reference(api, golden):
    """Scheduler side of a generation: the signal of every step and the tracker's effective base, over
    80 steps with a compression every ``divide_length`` tokens, with the prefill outside the budget, and
    with the usage trigger's hysteresis (runtime/planner.py:27-62, effective_len_tracker.py:25-52)."""
    want = golden["decode_loop"]
    got = {
        "default_80_steps": host_scenarios.decode_loop(api, dict(kv_budget=32, divide_length=8), prompt=50, steps=80),
        "protect_prefill_outside_budget": host_scenarios.decode_loop(
            api, dict(kv_budget=32, divide_length=8, protect_prefill=True, include_prefill_in_budget=False),
            prompt=20, steps=60),
        "kv_usage_trigger": host_scenarios.decode_loop(
            api, dict(kv_budget=64, divide_length=16, enable_kv_usage_trigger=True, kv_usage_trigger=0.9,
                      kv_usage_release=0.5), prompt=10, steps=40, kv_usages=[0.1, 0.95, 0.7, 0.7, 0.4, 0.6, 0.91, 0.2]),
    }
    assert sorted(got) == sorted(want)
    assert sum(bool(r.get("signal", {}).get("should_compress")) for r in want["default_80_steps"]) == 10
    _same(_through_json(got), want, "decode_loop")


def test_worker_block_tables_shrink_like_the_reference(api, golden):
    """runtime/worker_reclaim_sync.py:15-128: rows of one table and of a table per KV-cache group, list
    and tuple block lists, events that are not applied, unknown requests."""
    _same(_through_json(host_scenarios.worker_reclaim_cases(api)), golden["worker_reclaim"], "worker_reclaim")


@pytest.mark.parametrize("mode", ["strict", "lenient"])
def test_runner_actions_state_store_and_overrides_match_the_reference(api, golden, mode):
    """The worker's action loop over four steps with a scripted executor: events, which requests reached
    the executor (back-to-back signals are de-duplicated), the state store after every step, the
    effective-length override tuples with and without the scheduler's own progress counters, and in
    strict mode the fatal error for an unexpected skip (runtime/runner_compression_actions.py:11-237,
    state.py:46-153, effective_overrides.py:209-359, executor.py:30-84)."""
    got = _through_json(host_scenarios.runner_action_loop(api, mode == "strict"))
    _same(got, golden["runner_actions"][mode], mode)
