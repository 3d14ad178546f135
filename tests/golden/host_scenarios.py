"""Scenarios for the host-integer half of the hot path: effective lengths, budgets, deferral, the
regression guard, the hook's result dictionary and block-list truncation, the scheduler-side trigger
with the effective-length tracker, the worker's block-table shrink, the runner's action loop and the
effective-length overrides.

One driver, two callers.  ``run_all(api)`` builds every input from plain Python objects and pushes it
through the functions ``api`` names; it returns a JSON-serialisable dictionary.
``make_hook_golden.py`` calls it with the REFERENCE's functions (in the build container, where the
reference checkout is mounted) and stores the result as ``host_logic.json``; the tests call it with this
package's functions and compare with the stored dictionary, key by key.  Nothing here imports either.

``api`` is a namespace with:

* ``Config`` (TriAttentionRuntimeConfig), ``Signal`` (CompressionSignal), ``Planner``, ``Tracker``,
  ``StateStore``, ``Executor`` (RunnerHookCompressionExecutor)
* ``runtime_context(**kw)``            -> build_hook_runtime_context
* ``make_hook(runner, config, select_layer, select_group, compact_shared, compact_per_head, gather)``
                                       -> the runner hook with the given selector / compaction stand-ins
* ``worker_reclaim(base_runner, events)``, ``sparse_overrides(base_runner, state_store, scheduler_output,
  compression_events)``, ``runner_actions(executor, state_store, scheduler_output, signals, strict,
  allowed)``
"""
from __future__ import annotations

import itertools
import types
from dataclasses import asdict, is_dataclass

import numpy as np
import torch

NS = types.SimpleNamespace


def plain(value):
    """JSON-serialisable form of results (tuples -> lists, dataclasses -> dicts, tensors -> lists)."""
    if is_dataclass(value) and not isinstance(value, type):
        return plain(asdict(value))
    if isinstance(value, dict):
        return {str(k): plain(v) for k, v in value.items()}
    if isinstance(value, (list, tuple)):
        return [plain(v) for v in value]
    if isinstance(value, (set, frozenset)):
        return sorted(plain(v) for v in value)
    if isinstance(value, torch.Tensor):
        return value.tolist()
    if isinstance(value, np.ndarray):
        return value.tolist()
    if isinstance(value, (np.integer,)):
        return int(value)
    if isinstance(value, (np.floating,)):
        return float(value)
    if hasattr(value, "to_dict") and callable(value.to_dict):
        return plain(value.to_dict())
    return value


def _outcome(fn):
    """Result of ``fn()`` or the exception it raises, both as data."""
    try:
        return {"ok": plain(fn())}
    except Exception as exc:      # noqa: BLE001 - the exception is the recorded outcome
        return {"raises": type(exc).__name__, "message": str(exc)}


def signal_of(api, **kw):
    base = dict(req_id="r", should_compress=True, reason="length_threshold", estimated_cache_len=0, step=1,
                kv_usage=None, protect_prefill=False, prefill_len=0, scheduled_tokens=1)
    base.update(kw)
    return api.Signal(**base)


# ----------------------------------------------------------------- 1. runtime context
CONTEXT_CONFIGS = {
    "default": dict(kv_budget=64, divide_length=16),
    "protect_in_budget": dict(kv_budget=64, divide_length=16, protect_prefill=True, include_prefill_in_budget=True),
    "protect_outside_budget": dict(kv_budget=64, divide_length=16, protect_prefill=True, include_prefill_in_budget=False),
    "no_guard": dict(kv_budget=64, divide_length=16, fail_on_effective_len_regression=False),
    "tight_guard": dict(kv_budget=64, divide_length=16, effective_len_regression_ratio=0.5,
                        effective_len_guard_divide_multiples=1),
    "no_compaction": dict(kv_budget=64, divide_length=16, enable_experimental_kv_compaction=False,
                          enable_experimental_block_reclaim=False, require_physical_reclaim=False),
}
RUNTIME_STATES = {
    "none": None,
    "fresh": dict(compression_count=0, current_cache_len=0, last_absorbed_cache_len=30),
    "once": dict(compression_count=1, current_cache_len=70, last_absorbed_cache_len=64),
    "once_long": dict(compression_count=2, current_cache_len=300, last_absorbed_cache_len=64),
}


def runtime_context_cases(api):
    out = []
    grid = itertools.product(
        CONTEXT_CONFIGS, RUNTIME_STATES,
        (50, 81, 200, 1000),                 # num_computed_tokens
        (1, 8),                              # tokens scheduled in this step
        ("plus_scheduled", "small", "huge"),  # what the scheduler estimated
        (False, True),                       # compressed before
        ((6,), (100,), (100, 4)),            # blocks per KV-cache group
        (0, 30, 500),                        # prefill length
        ("length_threshold", "kv_usage_threshold"),
    )
    for n, (cfg_name, rt_name, nct, sched_n, est_kind, before, blocks, prefill, reason) in enumerate(grid):
        if n % 37 != 5:                      # a fixed subset: every 37th of the 20736 combinations
            continue
        out.append(_one_context_case(api, cfg_name, rt_name, nct, sched_n, est_kind, before, blocks, prefill, reason,
                                     post_forward=False))
    # the post-forward (prefill chunk) convention, on the signal as an extra attribute
    for cfg_name, nct, sched_n in itertools.product(("default", "protect_outside_budget"), (81, 200), (1, 64)):
        out.append(_one_context_case(api, cfg_name, "none", nct, sched_n, "plus_scheduled", False, (100,), 30,
                                     "length_threshold", post_forward=True))
    return out


def _one_context_case(api, cfg_name, rt_name, nct, sched_n, est_kind, before, blocks, prefill, reason, post_forward):
    cfg = api.Config(**CONTEXT_CONFIGS[cfg_name])
    estimated = {"plus_scheduled": nct + sched_n, "small": 70, "huge": 2000}[est_kind]
    sig = signal_of(api, estimated_cache_len=estimated, protect_prefill=bool(cfg.protect_prefill), prefill_len=prefill,
                    reason=reason, scheduled_tokens=sched_n)
    if post_forward:
        object.__setattr__(sig, "_post_forward", True)
    rt = RUNTIME_STATES[rt_name]
    runner = NS()
    block_ids = tuple(list(range(100 * g, 100 * g + n)) for g, n in enumerate(blocks))
    case = dict(config=cfg_name, runtime_state=rt_name, num_computed_tokens=nct, scheduled=sched_n, estimated=estimated,
                compressed_before=before, blocks=list(blocks), prefill_len=prefill, reason=reason,
                post_forward=post_forward)
    res = _outcome(lambda: api.runtime_context(
        base_runner=runner, config=cfg, req_id="r", req_state=NS(num_computed_tokens=nct),
        req_runtime_state=NS(**rt) if rt is not None else None, signal=sig,
        scheduler_output=NS(num_scheduled_tokens={"r": sched_n}), compressed_once={"r"} if before else set(),
        original_block_ids_by_group=block_ids, block_size_hint=16))
    case["result"] = res
    case["runner_recent_unabsorbed"] = getattr(runner, "_triattention_active_recent_unabsorbed_tokens", "unset")
    return case


# ----------------------------------------------------------------- 2. the hook
def _fake_selectors(calls, heads, always_none=False):
    """A deterministic stand-in for the scorer: keeps the guarded prefix, every other token after
    it, and the tail, per head shifted by the head index where there is room.  Like the real selector
    it has no answer (None) when a protected prefill alone exceeds the budget; ``always_none``: never
    an answer (an unavailable scorer)."""

    def keep_rows(total_tokens, prefill_len, protect_prefill, budget_total):
        k = min(budget_total, total_tokens)
        rows = []
        for h in range(heads):
            must = list(range(min(prefill_len, k))) if protect_prefill else []
            tail = [t for t in range(total_tokens - 1, -1, -1) if t not in must][: max(0, (k - len(must)) // 2)]
            rest = [t for t in range(h % 3, total_tokens, 2) if t not in must and t not in tail]
            fill = [t for t in range(total_tokens) if t not in must and t not in tail and t not in rest]
            chosen = (must + tail + rest + fill)[:k]
            rows.append(sorted(chosen))
        return torch.tensor(rows, dtype=torch.long)

    def select_group(*, layer_inputs=None, layer_input_iter=None, layer_kv_iter=None, total_tokens, prefill_len,
                     protect_prefill, round_start, budget_total):
        layers = [e[0] for e in layer_kv_iter()] if layer_kv_iter is not None else None
        calls.append(dict(fn="select_group", layers=layers, total_tokens=total_tokens, prefill_len=prefill_len,
                          protect_prefill=bool(protect_prefill), round_start=round_start, budget_total=budget_total))
        if always_none or (protect_prefill and prefill_len > budget_total):
            return None
        if total_tokens <= budget_total:
            return {"mode": "per_head", "indices": torch.arange(total_tokens).repeat(heads, 1)}
        return {"mode": "per_head", "indices": keep_rows(total_tokens, prefill_len, protect_prefill, budget_total),
                "semantic": "hf_aligned_global_per_head"}

    def select_layer(**kw):
        calls.append(dict(fn="select_layer", layer_idx=kw.get("layer_idx"), total_tokens=kw.get("total_tokens"),
                          budget_total=kw.get("budget_total"), round_start=kw.get("round_start")))
        return None

    select_group._supports_paged_group = True
    select_layer._supports_paged = True
    return select_layer, select_group


def _fake_compactors(calls):
    def per_head(*, kv_cache, block_ids, block_size, keep_token_indices_per_head, total_tokens,
                 preserve_dropped_tokens=True, **kw):
        keep = keep_token_indices_per_head
        calls.append(dict(fn="compact_per_head", blocks=len(block_ids), block_size=block_size, total_tokens=total_tokens,
                          keep_shape=list(keep.shape), first_row=keep[0].tolist()[:6]))
        return int(keep.shape[1])

    def shared(*, kv_cache, block_ids, block_size, keep_token_indices, total_tokens, preserve_dropped_tokens=True, **kw):
        keep = keep_token_indices
        n = int(keep.numel()) if isinstance(keep, torch.Tensor) else len(keep)
        calls.append(dict(fn="compact_shared", blocks=len(block_ids), block_size=block_size, total_tokens=total_tokens,
                          keep_count=n))
        return n

    def gather(**kw):
        raise AssertionError("the paged selectors of these scenarios never ask for dense keys")

    return shared, per_head, gather


HOOK_SCENARIOS = {
    # name: (config kwargs, block counts per KV-cache group, request facts, signal facts, what came before)
    "first_compression": (dict(kv_budget=32, divide_length=8), (12,), dict(nct=150), dict(est=151), ()),
    "two_groups": (dict(kv_budget=32, divide_length=8), (12, 7), dict(nct=150), dict(est=151), ()),
    "second_group_holds_no_more_than_the_budget": (dict(kv_budget=32, divide_length=8), (12, 2), dict(nct=150),
                                                   dict(est=151), ()),
    "under_budget": (dict(kv_budget=32, divide_length=8), (12,), dict(nct=20), dict(est=21), ()),
    "protect_prefill_in_budget": (dict(kv_budget=32, divide_length=8, protect_prefill=True), (12,), dict(nct=150),
                                  dict(est=151, prefill=10), ()),
    "protect_prefill_outside_budget": (dict(kv_budget=32, divide_length=8, protect_prefill=True,
                                            include_prefill_in_budget=False), (12,), dict(nct=150),
                                       dict(est=151, prefill=10), ()),
    "prefill_exceeds_budget": (dict(kv_budget=32, divide_length=8, protect_prefill=True), (12,), dict(nct=150),
                               dict(est=151, prefill=40), ()),
    "no_reclaim": (dict(kv_budget=32, divide_length=8, enable_experimental_block_reclaim=False,
                        require_physical_reclaim=False), (12,), dict(nct=150), dict(est=151), ()),
    "fallback_keep_when_not_strict": (dict(kv_budget=32, divide_length=8, require_triton_scoring=False), (12,),
                                      dict(nct=150), dict(est=151, selector_none=True), ()),
    "fallback_keep_with_protected_prefill": (dict(kv_budget=32, divide_length=8, require_triton_scoring=False,
                                                  protect_prefill=True), (12,), dict(nct=150),
                                             dict(est=151, prefill=10, selector_none=True), ()),
    "no_selector_answer_in_strict_mode": (dict(kv_budget=32, divide_length=8), (12,), dict(nct=150),
                                          dict(est=151, selector_none=True), ()),
    "plan_only": (dict(kv_budget=32, divide_length=8, enable_experimental_kv_compaction=False,
                       enable_experimental_block_reclaim=False, require_physical_reclaim=False), (12,), dict(nct=150),
                  dict(est=151), ()),
    "chunked_prefill_step": (dict(kv_budget=32, divide_length=8), (12,), dict(nct=100), dict(est=164, scheduled=64), ()),
    "kv_usage_reason": (dict(kv_budget=32, divide_length=8), (12,), dict(nct=150), dict(est=151, reason="kv_usage_threshold"), ()),
    # second calls on the same hook (same request): deferral until budget + divide_length, then again
    "recompress_deferred": (dict(kv_budget=32, divide_length=8), (12,), dict(nct=150), dict(est=151),
                            (dict(nct=153, est=36, state=dict(compression_count=1, current_cache_len=36,
                                                              last_absorbed_cache_len=32)),)),
    "recompress_due": (dict(kv_budget=32, divide_length=8), (12,), dict(nct=150), dict(est=151),
                       (dict(nct=158, est=41, blocks=3, state=dict(compression_count=1, current_cache_len=41,
                                                                   last_absorbed_cache_len=32)),)),
    "regression_guard": (dict(kv_budget=32, divide_length=8), (40,), dict(nct=150), dict(est=151),
                         (dict(nct=600, est=601, blocks=40, state=None),)),
}


def hook_scenario(api, name):
    cfg_kw, blocks, req_kw, sig_kw, followups = HOOK_SCENARIOS[name]
    cfg = api.Config(**cfg_kw)
    heads, bs = 2, 16
    calls: list = []
    select_layer, select_group = _fake_selectors(calls, heads, always_none=bool(sig_kw.get("selector_none")))
    shared, per_head, gather = _fake_compactors(calls)
    # one tensor per layer, two layers per KV-cache group; never read by the stand-ins
    layers_per_group = 2
    kv_caches = [torch.zeros(2, 64, bs, heads, 8) for _ in range(layers_per_group * len(blocks))]
    block_ids = tuple(list(range(1000 * g + 7, 1000 * g + 7 + n)) for g, n in enumerate(blocks))
    req = NS(num_computed_tokens=req_kw["nct"], block_ids=block_ids)
    store = NS(states={}, get=lambda rid: store.states.get(rid))
    runner = NS(requests={"r": req}, kv_caches=kv_caches, cache_config=NS(block_size=bs),
                _triattention_state_store=store)
    if len(blocks) > 1:
        names = [[f"model.layers.{g * layers_per_group + i}.attn" for i in range(layers_per_group)]
                 for g in range(len(blocks))]
        runner.kv_cache_config = NS(kv_cache_groups=[NS(layer_names=n) for n in names])
        runner.compilation_config = NS(static_forward_context={
            nm: NS(kv_cache=[kv_caches[g * layers_per_group + i]]) for g, group in enumerate(names)
            for i, nm in enumerate(group)})
    hook = api.make_hook(runner, cfg, select_layer, select_group, shared, per_head, gather)
    steps = []

    def one_call(nct, est, scheduled=1, prefill=0, reason="length_threshold", state=None, blocks_now=None):
        req.num_computed_tokens = nct
        if blocks_now is not None:
            req.block_ids = tuple(list(range(1000 * g + 7, 1000 * g + 7 + blocks_now)) for g in range(len(blocks)))
        store.states.clear()
        if state is not None:
            store.states["r"] = NS(**state)
        sig = signal_of(api, estimated_cache_len=est, protect_prefill=bool(cfg.protect_prefill), prefill_len=prefill,
                        reason=reason, scheduled_tokens=scheduled)
        del calls[:]
        before = plain(req.block_ids)
        res = _outcome(lambda: hook(req_id="r", signal=sig, scheduler_output=NS(num_scheduled_tokens={"r": scheduled})))
        steps.append(dict(result=res, block_ids_before=before, block_ids_after=plain(req.block_ids),
                          block_ids_type=type(req.block_ids).__name__, calls=plain(list(calls)),
                          active_req_id=getattr(runner, "_triattention_active_req_id", None)))

    one_call(req_kw["nct"], sig_kw["est"], sig_kw.get("scheduled", 1), sig_kw.get("prefill", 0),
             sig_kw.get("reason", "length_threshold"))
    for f in followups:
        one_call(f["nct"], f["est"], state=f.get("state"), blocks_now=f.get("blocks"))
    return steps


# ----------------------------------------------------------------- 3. planner + tracker over a decode loop
def decode_loop(api, cfg_kw, prompt, steps, kv_usages=None):
    """The scheduler's side of a generation: estimated length = effective base + scheduled tokens
    (scheduler.py:203-213); a compression is applied whenever the signal asks for one, down to the
    budget, as the runner would report it."""
    cfg = api.Config(**cfg_kw)
    planner, tracker = api.Planner(cfg), api.Tracker()
    tracker.reset_request("r", 0)
    rows = []
    nct = 0
    for step in range(steps):
        scheduled = prompt if step == 0 else 1
        base = tracker.observe_num_computed("r", nct)
        usage = kv_usages[step % len(kv_usages)] if kv_usages else None
        sig = planner.build_signal(req_id="r", estimated_cache_len=base + scheduled, prefill_len=prompt, step=step,
                                   kv_usage=usage, scheduled_tokens=scheduled)
        row = dict(step=step, nct=nct, base=base, signal=plain(sig), override=tracker.has_effective_len_override("r"))
        nct += scheduled
        if sig.should_compress:
            budget = cfg.kv_budget + (prompt if cfg.protect_prefill and not cfg.include_prefill_in_budget else 0)
            after = min(base + scheduled, budget)
            tracker.apply_compression("r", cache_len_after=after, num_computed_tokens=nct)
            row["applied_after"] = after
        row["snapshot"] = plain(tracker.snapshot())
        rows.append(row)
    tracker.remove_request("r")
    rows.append(dict(final_snapshot=plain(tracker.snapshot()), any_override=tracker.has_any_effective_len_overrides()))
    return rows


# ----------------------------------------------------------------- 4. worker block tables
def worker_reclaim_cases(api):
    out = []
    for name, multi in (("single_table", False), ("multi_group", True)):
        tables = [NS(num_blocks_per_row=np.array([10, 7, 3, 12], dtype=np.int32)) for _ in range(2 if multi else 1)]
        block_table = NS(block_tables=tables) if multi else tables[0]
        reqs = {"a": NS(block_ids=([1, 2, 3, 4, 5, 6, 7, 8, 9, 10],)), "b": NS(block_ids=([11, 12, 13, 14, 15, 16, 17],)),
                "c": NS(block_ids=([21, 22, 23], [31, 32, 33, 34])), "d": NS(block_ids=(tuple(range(40, 52)),))}
        runner = NS(input_batch=NS(block_table=block_table, req_id_to_index={"a": 0, "b": 1, "c": 2, "d": 3}),
                    requests=reqs, cache_config=NS(block_size=16))
        events = [
            {"req_id": "a", "status": "applied", "cache_len_after": 33},          # 3 blocks
            {"req_id": "b", "status": "skipped", "cache_len_after": 16},          # not applied: untouched
            {"req_id": "c", "status": "applied", "cache_len_after": 16},          # 1 block, both groups
            {"req_id": "d", "status": "applied", "cache_len_after": 64},          # a tuple of ids is left alone
            {"req_id": "zz", "status": "applied", "cache_len_after": 16},         # unknown request
            {"req_id": "a", "status": "applied", "cache_len_after": 0},           # no length: ignored
            "not an event",
        ]
        res = _outcome(lambda: api.worker_reclaim(runner, events))
        out.append(dict(name=name, result=res, rows=[t.num_blocks_per_row.tolist() for t in tables],
                        block_ids={k: plain(v.block_ids) for k, v in reqs.items()}))
    # a runner that keeps its block tables itself, and one with nothing to shrink
    runner2 = NS(block_tables=object(), input_batch=None, requests={}, cache_config=NS(block_size=16))
    out.append(dict(name="runner_owns_tables", result=_outcome(
        lambda: api.worker_reclaim(runner2, [{"req_id": "a", "status": "applied", "cache_len_after": 16}]))))
    out.append(dict(name="no_events", result=_outcome(lambda: api.worker_reclaim(runner2, None))))
    return out


# ----------------------------------------------------------------- 5. runner actions + state store + overrides
def runner_action_loop(api, strict):
    """A worker's steps for two requests: registration, triggers, hook results of every kind through
    a scripted executor, the de-duplication of back-to-back signals, and the overrides the next
    step's inputs are built from."""
    store = api.StateStore()
    script = {
        ("a", 3): {"applied": True, "reason": "kv_compacted:per_head", "cache_len_after": 32,
                   "effective_tokens_before": 48, "budget_total": 32, "reclaimed_block_count": 1,
                   "recent_unabsorbed_tokens": 8,
                   "block_reclaim": {"mode": "truncate_tail", "groups": [{"gid": 0, "block_ids_before": [1, 2, 3],
                                                                          "block_ids_after": [1, 2],
                                                                          "block_ids_removed": [3]}]}},
        ("b", 3): {"applied": False, "reason": "under_budget", "cache_len_after": 20},
        ("a", 4): {"applied": True, "reason": "kv_compacted:per_head", "cache_len_after": 32},
        ("b", 5): True,
        ("a", 9): {"applied": True, "reason": "kv_compacted:per_head", "cache_len_after": None},
        ("b", 9): {"applied": False, "reason": "something_else"},
    }
    seen = []

    class Scripted:
        def execute(self, req_id, signal, scheduler_output):
            seen.append([req_id, signal.step])
            return api.Executor(NS(triattention_apply_compression=lambda **kw: script[(req_id, signal.step)])).execute(
                req_id, signal, scheduler_output)

    store.ensure("a", 40, False)
    store.ensure("b", 10, False)
    rows = []
    for step, sigs, ncts in (
        (3, {"a": dict(est=49), "b": dict(est=21), "c": dict(est=5, should=False)}, {"a": 48, "b": 20}),
        (4, {"a": dict(est=34)}, {"a": 49}),                      # right after a compression, one token: de-duplicated
        (5, {"b": dict(est=23)}, {"b": 22}),
        (9, {"a": dict(est=41, scheduled=4), "b": dict(est=27)}, {"a": 54, "b": 26}),
    ):
        signals = {rid: signal_of(api, req_id=rid, estimated_cache_len=kw["est"], step=step,
                                  should_compress=kw.get("should", True), scheduled_tokens=kw.get("scheduled", 1),
                                  prefill_len=40 if rid == "a" else 10) for rid, kw in sigs.items()}
        for rid, sig in signals.items():
            if rid in ("a", "b"):
                store.update_cache_len(rid, sig.estimated_cache_len, step)
                if sig.should_compress:
                    store.mark_trigger(rid, sig.reason, step)
        sched = NS(num_scheduled_tokens={rid: s.scheduled_tokens for rid, s in signals.items()},
                   scheduled_cached_reqs=NS(req_ids=list(ncts), num_computed_tokens=list(ncts.values())),
                   triattention_step=step)
        del seen[:]
        res = _outcome(lambda: api.runner_actions(Scripted(), store, sched, signals, strict,
                                                  {"under_budget", "req_state_not_found"}))
        runner = NS(requests={rid: NS(num_computed_tokens=n) for rid, n in ncts.items()},
                    input_batch=NS(req_id_to_index={"a": 0, "b": 1}))
        events = res.get("ok") if isinstance(res.get("ok"), list) else None
        over = _outcome(lambda: api.sparse_overrides(runner, store, sched, events))
        # ... and without the scheduler's own progress counters (the older derivation from the state)
        bare = NS(num_scheduled_tokens=dict(sched.num_scheduled_tokens), triattention_step=step)
        over_bare = _outcome(lambda: api.sparse_overrides(runner, store, bare, events))
        rows.append(dict(step=step, executed=list(seen), events=res, overrides=over, overrides_without_counters=over_bare,
                         states={rid: plain(st) for rid, st in sorted(store.snapshot().items())},
                         any_compressed=store.has_active_compressed_requests(),
                         compressed_in=store.has_compressed_request_in(["b", "zz"])))
        if "raises" in res:
            break
    store.mark_preempted("a")
    store.mark_resumed("a")
    store.remove("b")
    rows.append(dict(final_states={rid: plain(st) for rid, st in sorted(store.snapshot().items())},
                     any_compressed=store.has_active_compressed_requests()))
    return rows


def run_all(api) -> dict:
    return {
        "runtime_context": runtime_context_cases(api),
        "hook": {name: hook_scenario(api, name) for name in HOOK_SCENARIOS},
        "decode_loop": {
            "default_80_steps": decode_loop(api, dict(kv_budget=32, divide_length=8), prompt=50, steps=80),
            "protect_prefill_outside_budget": decode_loop(
                api, dict(kv_budget=32, divide_length=8, protect_prefill=True, include_prefill_in_budget=False),
                prompt=20, steps=60),
            "kv_usage_trigger": decode_loop(
                api, dict(kv_budget=64, divide_length=16, enable_kv_usage_trigger=True, kv_usage_trigger=0.9,
                          kv_usage_release=0.5), prompt=10, steps=40,
                kv_usages=[0.1, 0.95, 0.7, 0.7, 0.4, 0.6, 0.91, 0.2]),
        },
        "worker_reclaim": worker_reclaim_cases(api),
        "runner_actions": {"strict": runner_action_loop(api, True), "lenient": runner_action_loop(api, False)},
    }
