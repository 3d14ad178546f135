"""Scheduler / worker bookkeeping around the compression hook (triattention_amd.runtime.engine_glue)
with stand-ins for the engine's objects; hand-derived cases.  CPU only."""
from __future__ import annotations

import types

import numpy as np
import pytest

from triattention_amd.runtime import (CompressionSignal, RequestStateStore, TriAttentionRuntimeConfig)
from triattention_amd.runtime import engine_glue as eg
from triattention_amd.runtime.hook import CompressionExecutionResult
from triattention_amd.runtime.models import TRITON_SCORING_REQUIRED_MARKER as MARK

NS = types.SimpleNamespace


def _cfg(**kw):
    base = dict(kv_budget=2048, divide_length=128, window_size=128)
    base.update(kw)
    return TriAttentionRuntimeConfig(**base)


def _sched(tokens: dict, new=(), finished=(), cached=None):
    return NS(num_scheduled_tokens=dict(tokens), scheduled_new_reqs=list(new), finished_req_ids=set(finished),
              scheduled_cached_reqs=cached)


# ------------------------------------------------------------------ small pieces
def test_scheduled_token_items_accept_ids_and_request_objects():
    class Key:                      # hashable by identity, as a request object is
        def __init__(self, **kw):
            self.__dict__.update(kw)

    key_obj = Key(request_id="b")
    out = NS(num_scheduled_tokens={"a": 1, key_obj: "3", 7: 2, Key(): 1, "bad": "x"})
    assert [(rid, n) for _k, rid, n in eg.iter_scheduled_token_items(out)] == [("a", 1), ("b", 3), (7, 2)]
    items = eg.get_scheduled_token_items(out)
    assert eg.get_scheduled_token_items(out) is items            # cached on the output
    assert eg.get_scheduled_token_items(None) == [] and list(eg.iter_scheduled_token_items(NS())) == []


def test_effective_length_tracker():
    t = eg.EffectiveCacheLenTracker()
    assert t.observe_num_computed("r", 100) == 100 and not t.has_effective_len_override("r")
    t.apply_compression("r", cache_len_after=2048, num_computed_tokens=2176)
    assert t.has_effective_len_override("r") and t.has_any_effective_len_overrides()
    assert t.observe_num_computed("r", 2177) == 2049          # cache_len_after + tokens computed since
    assert t.observe_num_computed("r", 2300) == 2172
    assert t.observe_num_computed("r", 2000) == 2000          # a rollback never grows the length
    assert t.snapshot()["r"] == (2000, 2000)
    t.reset_request("r", 5)
    assert not t.has_effective_len_override("r") and t.snapshot()["r"] == (-1, 5)
    t.remove_request("r")
    assert t.snapshot() == {}


def test_allocation_offset_on_the_request():
    req = NS(num_computed_tokens=2176)
    assert eg.update_request_effective_kv_offset(request=req, cache_len_after=2048) == 128
    assert getattr(req, eg.EFFECTIVE_KV_OFFSET_ATTR) == 128
    req.num_computed_tokens = 2200
    assert eg.prepare_request_effective_num_computed(req) == 2072
    assert eg.resolve_request_effective_num_computed(req) == 2072
    req.num_computed_tokens = 100                 # started over below the offset: everything is forgotten
    assert eg.prepare_request_effective_num_computed(req) is None
    assert not hasattr(req, eg.EFFECTIVE_KV_OFFSET_ATTR) and eg.resolve_request_effective_num_computed(req) is None
    req.num_computed_tokens = 500
    assert eg.update_request_effective_kv_offset(request=req, cache_len_after=900) == 0      # nothing to offset
    assert eg.update_request_effective_kv_offset(request=None, cache_len_after=1) is None
    assert eg.update_request_effective_kv_offset(request=NS(num_computed_tokens="x"), cache_len_after=1) is None


# ------------------------------------------------------------------ trigger
def test_signals_follow_the_effective_length():
    glue = eg.SchedulerCompressionGlue(_cfg())
    req = NS(num_computed_tokens=0, num_prompt_tokens=300)
    requests = {"r": req}
    new = NS(req_id="r", num_computed_tokens=0, prompt_token_ids=list(range(300)))
    out = _sched({"r": 300}, new=[new])
    assert glue.after_schedule(out, requests) == {} and out.triattention_step == 1
    assert glue.prefill_lens["r"] == 300 and glue.length_thresholds["r"] == 2176
    req.num_computed_tokens = 2174
    assert glue.after_schedule(_sched({"r": 1}), requests) == {}                 # 2175 < 2048 + 128
    req.num_computed_tokens = 2175
    sig = glue.after_schedule(_sched({"r": 1}), requests)["r"]                   # 2176: due
    assert sig.should_compress and sig.reason == "length_threshold" and sig.estimated_cache_len == 2176
    assert sig.prefill_len == 300 and sig.scheduled_tokens == 1 and sig.step == 3
    # the runner compressed to 2048 when 2175 tokens were computed; the event comes back
    glue.apply_compression_events([{"status": "applied", "req_id": "r", "cache_len_after": 2048}], requests, None, 16)
    req.num_computed_tokens = 2176
    sig = glue.after_schedule(_sched({"r": 1}), requests)["r"]                   # reported, not due: 2048 + 1 + 1
    assert not sig.should_compress and sig.estimated_cache_len == 2050
    req.num_computed_tokens = 2175 + 127
    sig = glue.after_schedule(_sched({"r": 1}), requests)["r"]                   # 2048 + 127 + 1 = 2176: due again
    assert sig.should_compress and sig.estimated_cache_len == 2176
    # chunked prefill: a 512-token step crosses the threshold at once
    glue2 = eg.SchedulerCompressionGlue(_cfg())
    r2 = NS(num_computed_tokens=2000, num_prompt_tokens=4000)
    sig = glue2.after_schedule(_sched({"q": 512}), {"q": r2})["q"]
    assert sig.should_compress and sig.estimated_cache_len == 2512 and sig.scheduled_tokens == 512
    assert glue2.prefill_lens["q"] == 4000
    # finished requests are forgotten
    glue.after_schedule(_sched({}, finished=["r"]), requests)
    assert "r" not in glue.prefill_lens and not glue.tracker.has_any_effective_len_overrides()


def test_prefill_outside_the_budget_moves_the_threshold():
    glue = eg.SchedulerCompressionGlue(_cfg(protect_prefill=True, include_prefill_in_budget=False))
    assert glue.compute_length_threshold(500) == 2048 + 128 + 500
    req = NS(num_computed_tokens=2400, num_prompt_tokens=500)
    assert glue.after_schedule(_sched({"r": 1}), {"r": req}) == {}
    req.num_computed_tokens = 2675
    sig = glue.after_schedule(_sched({"r": 1}), {"r": req})["r"]
    assert sig.should_compress and sig.protect_prefill and sig.prefill_len == 500


def test_usage_trigger_and_disabled_compression():
    glue = eg.SchedulerCompressionGlue(_cfg(enable_kv_usage_trigger=True, kv_usage_trigger=0.9, kv_usage_release=0.5))
    req = NS(num_computed_tokens=10, num_prompt_tokens=5)
    sig = glue.after_schedule(_sched({"r": 1}), {"r": req}, kv_usage=0.95)["r"]
    assert sig.should_compress and sig.reason == "kv_usage_threshold" and sig.kv_usage == 0.95
    assert glue.after_schedule(_sched({"r": 1}), {"r": req}, kv_usage=0.7)["r"].should_compress     # still armed
    assert glue.after_schedule(_sched({"r": 1}), {"r": req}, kv_usage=0.4) == {}                    # released
    off = eg.SchedulerCompressionGlue(_cfg(disable_compression=True))
    big = NS(num_computed_tokens=9000, num_prompt_tokens=5)
    assert off.after_schedule(_sched({"r": 1}), {"r": big}) == {}
    assert off.max_chunk_for_compression(1000, 16) is None
    on = eg.SchedulerCompressionGlue(_cfg())
    assert on.max_chunk_for_compression(1000, 16) == 1000 * 16 - 2048 - 16
    assert on.max_chunk_for_compression(128, 16) is None and on.max_chunk_for_compression(0, 16) is None
    assert on.max_chunk_for_compression(129, 16) == 1


# ------------------------------------------------------------------ freeing blocks
class _Pool:
    def __init__(self):
        self.freed, self.evicted = [], []

    def free_blocks(self, blocks):
        self.freed.append([b.block_id for b in blocks])

    def _maybe_evict_cached_block(self, block):
        self.evicted.append(block.block_id)


def _manager(req_id, ids, hashed=()):
    return NS(req_to_blocks={req_id: [NS(block_id=i, block_hash=("h" if i in hashed else None)) for i in ids]},
              num_cached_block={req_id: len(ids)}, block_pool=_Pool())


def _event(groups, after=32, scheduled=1, **kw):
    e = {"status": "applied", "req_id": "r", "step": 4, "cache_len_after": after, "scheduled_tokens": scheduled,
         "block_reclaim": None if groups is None else {"mode": "truncate_tail", "groups": groups}}
    e.update(kw)
    return e


def test_events_free_the_old_tail_and_keep_blocks_appended_since():
    glue = eg.SchedulerCompressionGlue(_cfg(kv_budget=32, divide_length=8, window_size=4))
    req = NS(num_computed_tokens=40)
    m = _manager("r", [5, 9, 2, 7, 11], hashed={7})         # the hook saw [5, 9, 2, 7]; 11 was appended after it ran
    group = {"gid": 0, "block_ids_before": [5, 9, 2, 7], "block_ids_after": [5, 9], "block_ids_removed": [2, 7]}
    glue.apply_compression_events([_event([group])], {"r": req}, [m], 16)
    assert [b.block_id for b in m.req_to_blocks["r"]] == [5, 9, 11] and m.num_cached_block["r"] == 3
    assert m.block_pool.freed == [[7, 2]] and m.block_pool.evicted == [7]       # last block first; hashed one evicted
    assert getattr(req, eg.EFFECTIVE_KV_OFFSET_ATTR) == 8 and glue.tracker.snapshot()["r"] == (32, 40)
    # events that are not "applied", or about unknown requests, change nothing
    glue.apply_compression_events([{"status": "skipped", "req_id": "r"}, _event([group], req_id="zz")], {"r": req}, [m], 16)
    assert m.block_pool.freed == [[7, 2]]


@pytest.mark.parametrize("after_ids,match", [
    ([5, 2], "prefix mismatch"), ([5, 5], "duplicate block ids"), ([5, 9, 2, 7, 1, 3], "invalid length"),
    ([5, 9, 2], "insufficient shrink"),
])
def test_events_that_do_not_fit_the_managers_blocks_raise(after_ids, match):
    glue = eg.SchedulerCompressionGlue(_cfg(kv_budget=32, divide_length=8, window_size=4))
    m = _manager("r", [5, 9, 2, 7])
    group = {"gid": 0, "block_ids_before": [5, 9, 2, 7], "block_ids_after": after_ids}
    with pytest.raises(RuntimeError, match=match):
        glue.apply_compression_events([_event([group])], {"r": NS(num_computed_tokens=40)}, [m], 16)
    assert m.block_pool.freed == []


def test_groups_missing_from_an_event_are_truncated_except_during_prefill():
    glue = eg.SchedulerCompressionGlue(_cfg(kv_budget=32, divide_length=8, window_size=4))
    req = NS(num_computed_tokens=40)
    m0, m1 = _manager("r", [1, 2, 3]), _manager("r", [4, 5, 6, 8])
    group0 = {"gid": 0, "block_ids_before": [1, 2, 3], "block_ids_after": [1, 2]}
    glue.apply_compression_events([_event([group0])], {"r": req}, [m0, m1], 16)          # group 1 not listed
    assert [b.block_id for b in m1.req_to_blocks["r"]] == [4, 5] and m1.block_pool.freed == [[8, 6]]
    # no reclaim payload at all (the worker truncated in an earlier step): same synthesis ...
    m2 = _manager("r", [1, 2, 3])
    glue.apply_compression_events([_event(None)], {"r": req}, [m2], 16)
    assert [b.block_id for b in m2.req_to_blocks["r"]] == [1, 2] and m2.num_cached_block["r"] == 2
    # ... but never in a multi-token step, where appended blocks cannot be told from old ones
    m3 = _manager("r", [1, 2, 3])
    glue.apply_compression_events([_event(None, scheduled=512)], {"r": req}, [m3], 16)
    assert len(m3.req_to_blocks["r"]) == 3 and m3.block_pool.freed == []
    # block reclaim switched off: only the tracker moves
    off = eg.SchedulerCompressionGlue(_cfg(kv_budget=32, divide_length=8, window_size=4,
                                           enable_experimental_block_reclaim=False, require_physical_reclaim=False))
    m4 = _manager("r", [1, 2, 3])
    off.apply_compression_events([_event([group0])], {"r": req}, [m4], 16)
    assert len(m4.req_to_blocks["r"]) == 3 and off.tracker.has_effective_len_override("r")


# ------------------------------------------------------------------ worker side
def test_worker_block_tables_shrink_to_the_compacted_length(monkeypatch):
    t0, t1 = NS(num_blocks_per_row=np.array([9, 140, 3])), NS(num_blocks_per_row=np.array([9, 130, 3]))
    state = NS(block_ids=(list(range(140)), list(range(130))))
    runner = NS(input_batch=NS(block_table=NS(block_tables=[t0, t1]), req_id_to_index={"a": 0, "r": 1}),
                cache_config=NS(block_size=16), requests={"r": state})
    events = [{"status": "applied", "req_id": "r", "cache_len_after": 2048},
              {"status": "skipped", "req_id": "a", "cache_len_after": 16}, {"status": "applied", "req_id": "gone",
                                                                            "cache_len_after": 16}]
    eg.apply_worker_block_reclaim_events(base_runner=runner, events=events)
    assert t0.num_blocks_per_row.tolist() == [9, 128, 3] and t1.num_blocks_per_row.tolist() == [9, 128, 3]
    assert [len(g) for g in state.block_ids] == [128, 128]
    single = NS(num_blocks_per_row=np.array([200]))
    runner2 = NS(input_batch=NS(block_table=single, req_id_to_index={"r": 0}), cache_config=NS(block_size=16), requests={})
    eg.apply_worker_block_reclaim_events(base_runner=runner2, events=[{"status": "applied", "req_id": "r",
                                                                      "cache_len_after": 2049}])
    assert single.num_blocks_per_row.tolist() == [129]
    monkeypatch.setenv("TRIATTN_DEBUG_DISABLE_WORKER_RECLAIM_SYNC", "1")
    single.num_blocks_per_row[0] = 200
    eg.apply_worker_block_reclaim_events(base_runner=runner2, events=[{"status": "applied", "req_id": "r",
                                                                      "cache_len_after": 2049}])
    assert single.num_blocks_per_row.tolist() == [200]
    monkeypatch.delenv("TRIATTN_DEBUG_DISABLE_WORKER_RECLAIM_SYNC")
    eg.apply_worker_block_reclaim_events(base_runner=NS(block_tables=object()), events=events)     # nothing to do
    eg.apply_worker_block_reclaim_events(base_runner=NS(), events=None)


def test_runner_actions_emit_events_and_keep_the_state_store_in_step():
    store = RequestStateStore()
    store.ensure("a", 10, False); store.ensure("b", 10, False); store.ensure("c", 10, False)
    sig = lambda rid, step=5, due=True, scheduled=1: CompressionSignal(rid, due, "length_threshold" if due else "none",
                                                                       2176, step, None, False, 10, scheduled)
    calls = []

    class Executor:
        def execute(self, req_id, signal, scheduler_output):
            calls.append(("one", req_id))
            if req_id == "c":
                return CompressionExecutionResult(False, "under_budget", 2000, {"applied": False})
            return CompressionExecutionResult(True, "kv_compacted:per_head", 2048,
                                              {"block_reclaim": {"mode": "truncate_tail", "groups": []}})

        def execute_batch(self, signals, scheduler_output):
            calls.append(("batch", sorted(signals)))
            return {rid: self.execute(rid, s, scheduler_output) for rid, s in signals.items()}

    out = NS(scheduled_cached_reqs=NS(req_ids=["a", "b"], num_computed_tokens=[2175, 2300]))
    signals = {"a": sig("a"), "b": sig("b"), "c": sig("c"), "idle": sig("idle", due=False)}
    events = eg.execute_runner_compression_actions(executor=Executor(), state_store=store, scheduler_output=out,
                                                   signals=signals, strict_no_downgrade=True)
    assert calls[0] == ("batch", ["a", "b", "c"])
    assert [(e["req_id"], e["status"], e["reason"], e["cache_len_after"]) for e in events] == [
        ("a", "applied", "kv_compacted:per_head", 2048), ("b", "applied", "kv_compacted:per_head", 2048),
        ("c", "skipped", "under_budget", 2000)]
    assert events[0]["block_reclaim"] == {"mode": "truncate_tail", "groups": []} and events[0]["scheduled_tokens"] == 1
    assert set(events[0]) == {"req_id", "step", "status", "reason", "cache_len_after", "details", "scheduled_tokens",
                              "estimated_cache_len", "prefill_len", "block_reclaim"}
    a = store.get("a")
    assert (a.compression_count, a.current_cache_len, a.nct_at_last_compression, a.cache_len_after_last_compression) == \
        (1, 2049, 2175, 2048)
    assert store.get("c").last_trigger_reason == "skipped:under_budget" and store.has_active_compressed_requests()
    # the step after a compression: a single-token trigger is not executed again
    calls.clear()
    events = eg.execute_runner_compression_actions(executor=Executor(), state_store=store, scheduler_output=out,
                                                   signals={"a": sig("a", step=6)}, strict_no_downgrade=True)
    assert not calls and events[0]["status"] == "skipped" and events[0]["reason"] == "batch_queue_dedup"
    events = eg.execute_runner_compression_actions(executor=Executor(), state_store=store, scheduler_output=out,
                                                   signals={"a": sig("a", step=6, scheduled=512)},
                                                   strict_no_downgrade=True)
    assert calls == [("one", "a")] and events[0]["status"] == "applied"      # (a prefill chunk is)

    class Broken:
        def execute(self, req_id, signal, scheduler_output):
            raise ValueError("boom")

    with pytest.raises(RuntimeError, match=f"{MARK}:executor_exception:req=b:step=9:type=ValueError"):
        eg.execute_runner_compression_actions(executor=Broken(), state_store=store, scheduler_output=out,
                                              signals={"b": sig("b", step=9)}, strict_no_downgrade=True)
    events = eg.execute_runner_compression_actions(executor=Broken(), state_store=store, scheduler_output=out,
                                                   signals={"b": sig("b", step=9)}, strict_no_downgrade=False)
    assert events[0]["status"] == "error" and events[0]["reason"] == "executor_exception:ValueError"

    class Odd:
        def execute(self, req_id, signal, scheduler_output):
            return CompressionExecutionResult(False, "kv_cache_unavailable")

    with pytest.raises(RuntimeError, match=f"{MARK}:unexpected_skip:req=b:step=9:reason=kv_cache_unavailable"):
        eg.execute_runner_compression_actions(executor=Odd(), state_store=store, scheduler_output=out,
                                              signals={"b": sig("b", step=9)}, strict_no_downgrade=True)


def test_worker_lifecycle_and_its_own_length_recurrence(monkeypatch):
    store = RequestStateStore()
    out = NS(scheduled_new_reqs=[NS(req_id="r", prompt_token_ids=[0] * 300)], finished_req_ids=[], preempted_req_ids=["r"],
             scheduled_cached_reqs=NS(req_ids=["r"]), triattention_step=4,
             triattention_signals={"r": CompressionSignal("r", True, "length_threshold", 2176, 4, None, False, 300, 1)})
    eg.register_new_requests(state_store=store, scheduler_output=out, protect_prefill=False)
    assert store.get("r").prefill_len == 300
    eg.mark_preemptions(state_store=store, scheduler_output=out)
    assert store.get("r").is_preempted
    eg.mark_resumed(state_store=store, scheduler_output=out)
    assert not store.get("r").is_preempted
    step, signals = eg.consume_runner_signals(state_store=store, scheduler_output=out, last_step=3)
    st = store.get("r")
    assert step == 4 and st.current_cache_len == 2176 and st.pending_triggers == 1 and st.current_cache_len_step == 4
    store.mark_compressed("r", step=4, cache_len=2048, scheduled_tokens=1, scheduler_nct=2175)
    assert st.current_cache_len == 2049
    # once compressed, the worker counts on from its own value whatever the scheduler's estimate says
    out.triattention_signals = {"r": CompressionSignal("r", False, "none", 2050, 5, None, False, 300, 1)}
    out.triattention_step = 5
    eg.consume_runner_signals(state_store=store, scheduler_output=out, last_step=4)
    assert st.current_cache_len == 2050
    out.triattention_signals = {"r": CompressionSignal("r", False, "none", 9999, 6, None, False, 300, 1)}
    eg.consume_runner_signals(state_store=store, scheduler_output=out, last_step=5)
    assert st.current_cache_len == 2051
    monkeypatch.setenv("TRIATTN_RUNTIME_LEGACY_COMPRESSED_ESTIMATE", "1")
    eg.consume_runner_signals(state_store=store, scheduler_output=out, last_step=6)
    assert st.current_cache_len == 9999
    out.finished_req_ids = ["r"]
    eg.cleanup_finished_requests(state_store=store, scheduler_output=out)
    assert store.get("r") is None


# ------------------------------------------------------------------ lengths the attention inputs need
def test_sparse_overrides_after_a_compression():
    store = RequestStateStore()
    store.ensure("a", 100, False); store.ensure("b", 100, False); store.ensure("c", 100, False)
    store.mark_compressed("a", step=7, cache_len=2048, scheduled_tokens=1, scheduler_nct=2175)
    runner = NS(requests={"a": NS(num_computed_tokens=2180), "b": NS(num_computed_tokens=500),
                          "c": NS(num_computed_tokens=900)},
                input_batch=NS(req_id_to_index={"a": 2, "b": 0, "c": 1}))
    out = NS(num_scheduled_tokens={"a": 1, "b": 1, "c": 1}, triattention_step=12,
             scheduled_cached_reqs=NS(req_ids=["a", "b", "c"], num_computed_tokens=[2180, 500, 900]))
    seq, pos, one_seq, one_pos = eg.build_effective_sparse_overrides(base_runner=runner, state_store=store,
                                                                     scheduler_output=out)
    # a: 2048 kept when 2175 were computed, 5 computed since: 2053 cached, positions shifted by 2048 - 2175
    assert seq == {2: 2053} and pos == {2: -127} and (one_seq, one_pos) == (2053, -127)
    assert eg.build_effective_sparse_overrides(base_runner=runner, state_store=store, scheduler_output=out) \
        is out._triattention_cached_sparse_overrides[(id(runner), id(store))]
    # without the scheduler's view of num_computed_tokens: the state's own length, which includes this step's tokens
    out2 = NS(num_scheduled_tokens={"a": 1, "b": 1}, triattention_step=12, scheduled_cached_reqs=None)
    store.update_cache_len("a", 2054, step=12)
    seq, pos, _, _ = eg.build_effective_sparse_overrides(base_runner=runner, state_store=store, scheduler_output=out2)
    assert seq == {2: 2053} and pos == {2: 2053 - 2180}
    st = store.get("a")
    st.current_cache_len_semantics, st.current_cache_len_step, st.current_cache_len = "effective_pre_step", 12, 2053
    out3 = NS(num_scheduled_tokens={"a": 1}, triattention_step=12, scheduled_cached_reqs=None)
    assert eg.build_effective_sparse_overrides(base_runner=runner, state_store=store, scheduler_output=out3)[0] == {2: 2053}
    # a compressed request whose state does not say what its length means is an error, not a guess
    st.current_cache_len_semantics = None
    out4 = NS(num_scheduled_tokens={"a": 1}, triattention_step=12, scheduled_cached_reqs=None)
    with pytest.raises(RuntimeError, match="TRIATTN_EFFECTIVE_BASE_STATE_SEMANTICS_MISSING"):
        eg.build_effective_sparse_overrides(base_runner=runner, state_store=store, scheduler_output=out4)
    # nothing compressed yet: no overrides; applied events without a compressed request are a mismatch
    fresh = RequestStateStore()
    out5 = NS(num_scheduled_tokens={"a": 1})
    assert eg.build_effective_sparse_overrides(base_runner=runner, state_store=fresh, scheduler_output=out5) == \
        (None, None, None, 0)
    with pytest.raises(RuntimeError, match="TRIATTN_COMPRESSION_EVENT_STATE_MISMATCH"):
        eg.build_effective_sparse_overrides(base_runner=runner, state_store=fresh, scheduler_output=NS(num_scheduled_tokens={"a": 1}),
                                            compression_events=[{"status": "applied", "req_id": "a"}])
    assert eg.resolve_req_id_to_index(NS(input_batch=NS(req_ids=["x", None, "y"]))) == ({"x": 0, "y": 2}, "input_batch_req_ids")
    assert eg.resolve_req_id_to_index(NS()) == (None, "none")


def test_first_decode_step_after_a_compressed_prefill_uses_the_full_prompt_length():
    """runtime/effective_overrides.py:160-167: the progress counter may still be one prefill chunk behind."""
    st = NS(compression_count=1, prefill_len=4000, current_cache_len=2048, current_cache_len_semantics="effective_pre_step",
            current_cache_len_step=3, nct_at_last_compression=None, cache_len_after_last_compression=None)
    store = NS(get=lambda rid: st, has_active_compressed_requests=lambda: True)
    runner = NS(requests={"r": NS(num_computed_tokens=3488)}, input_batch=NS(req_id_to_index={"r": 0}))
    out = NS(num_scheduled_tokens={"r": 1}, triattention_step=3, scheduled_cached_reqs=None)
    seq, pos, _, _ = eg.build_effective_sparse_overrides(base_runner=runner, state_store=store, scheduler_output=out)
    assert seq == {0: 2048} and pos == {0: 2048 - 4000}
