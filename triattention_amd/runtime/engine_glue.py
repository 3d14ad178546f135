"""Host-side bookkeeping between a serving engine's scheduler / worker and the compression hook:
when a request is due (length estimate after earlier compressions), what the scheduler frees
once a compression event comes back, how the worker's block tables shrink, and which sequence
length / position offsets the attention inputs need afterwards.

The reference implements these as methods of a vLLM ``Scheduler`` subclass and as helpers that
reach into vLLM's runner (triattention/vllm/runtime/scheduler.py, worker_reclaim_sync.py,
effective_overrides.py, effective_len_tracker.py, kv_allocation_sync.py,
request_key_compat.py).  Here they are plain functions and one small class over duck-typed
objects — a dict of requests with ``num_computed_tokens``, per-group block managers with
``req_to_blocks`` / ``num_cached_block`` / ``block_pool``, an input batch with
``req_id_to_index`` and block tables with ``num_blocks_per_row`` — so an engine binds them
where its scheduler and worker own those objects, and they are testable without the engine.
Names, arguments, result shapes and error strings follow the reference.
"""
from __future__ import annotations

import logging
import os
from typing import Any, Iterator

import numpy as np

from .config import TriAttentionRuntimeConfig
from .models import TRITON_SCORING_REQUIRED_MARKER as MARK
from .models import CompressionPlanner, CompressionSignal

logger = logging.getLogger(__name__)

EFFECTIVE_KV_OFFSET_ATTR = "_triattention_effective_kv_offset"
EFFECTIVE_NUM_COMPUTED_ATTR = "_triattention_effective_num_computed_tokens"


# ------------------------------------------------------------ scheduled-token keys
def req_id_from_scheduled_key(key: Any) -> Any:
    """``num_scheduled_tokens`` may be keyed by request id or by an object carrying one
    (runtime/request_key_compat.py:17-27)."""
    if isinstance(key, (str, int)):
        return key
    for attr in ("request_id", "req_id"):
        rid = getattr(key, attr, None)
        if isinstance(rid, (str, int)):
            return rid
    return None


def iter_scheduled_token_items(scheduler_output: Any) -> Iterator[tuple]:
    """``(raw_key, req_id, scheduled_tokens)`` in mapping order (runtime/request_key_compat.py:30-45)."""
    scheduled = getattr(scheduler_output, "num_scheduled_tokens", None)
    if not isinstance(scheduled, dict):
        return
    for raw_key, raw_value in scheduled.items():
        rid = req_id_from_scheduled_key(raw_key)
        if rid is None:
            continue
        try:
            tokens = int(raw_value)
        except (TypeError, ValueError):
            continue
        yield raw_key, rid, tokens


def get_scheduled_token_items(scheduler_output: Any) -> list:
    """The same as a list, cached on the scheduler output when it allows attributes
    (runtime/request_key_compat.py:48-69)."""
    if scheduler_output is None:
        return []
    cached = getattr(scheduler_output, "_triattention_cached_scheduled_token_items", None)
    if isinstance(cached, list):
        return cached
    items = list(iter_scheduled_token_items(scheduler_output))
    try:
        setattr(scheduler_output, "_triattention_cached_scheduled_token_items", items)
    except Exception:
        pass
    return items


# ------------------------------------------------------------ effective length per request
class EffectiveCacheLenTracker:
    """``num_computed_tokens`` only grows; the cached length shrinks at every compression.
    After the first compression of a request its effective length is ``cache_len_after`` plus
    what has been computed since (runtime/effective_len_tracker.py:6-68)."""

    def __init__(self) -> None:
        self._effective_len: dict = {}
        self._last_num_computed: dict = {}

    def reset_request(self, req_id, num_computed_tokens: int) -> None:
        self._effective_len.pop(req_id, None)
        self._last_num_computed[req_id] = max(0, int(num_computed_tokens))

    def remove_request(self, req_id) -> None:
        self._effective_len.pop(req_id, None)
        self._last_num_computed.pop(req_id, None)

    def observe_num_computed(self, req_id, num_computed_tokens: int) -> int:
        now = max(0, int(num_computed_tokens))
        if req_id not in self._effective_len:
            self._last_num_computed[req_id] = now
            return now
        before = self._last_num_computed.get(req_id, now)
        eff = self._effective_len[req_id]
        eff = eff + (now - before) if now >= before else min(eff, now)      # (a rollback never grows it)
        self._effective_len[req_id] = max(0, eff)
        self._last_num_computed[req_id] = now
        return self._effective_len[req_id]

    def apply_compression(self, req_id, cache_len_after: int, num_computed_tokens: int) -> None:
        self._effective_len[req_id] = max(0, int(cache_len_after))
        self._last_num_computed[req_id] = max(0, int(num_computed_tokens))

    def snapshot(self) -> dict:
        keys = set(self._effective_len) | set(self._last_num_computed)
        return {k: (self._effective_len.get(k, -1), self._last_num_computed.get(k)) for k in keys}

    def has_effective_len_override(self, req_id) -> bool:
        return req_id in self._effective_len

    def has_any_effective_len_overrides(self) -> bool:
        return bool(self._effective_len)


# ------------------------------------------------------------ allocation offset on the request
def _non_negative_int(value: Any):
    try:
        return max(0, int(value))
    except (TypeError, ValueError):
        return None


def _drop_attr(obj: Any, name: str) -> None:
    if hasattr(obj, name):
        try:
            delattr(obj, name)
        except Exception:
            try:
                setattr(obj, name, None)
            except Exception:
                pass


def clear_request_allocation_sync_state(request: Any) -> None:
    """runtime/kv_allocation_sync.py:22-35."""
    if request is None:
        return
    _drop_attr(request, EFFECTIVE_KV_OFFSET_ATTR)
    _drop_attr(request, EFFECTIVE_NUM_COMPUTED_ATTR)


def update_request_effective_kv_offset(*, request: Any, cache_len_after: int):
    """After blocks were freed: remember ``num_computed_tokens - cache_len_after`` on the request, so
    the allocator sizes the next step from the effective length (runtime/kv_allocation_sync.py:38-61)."""
    if request is None:
        return None
    logical = _non_negative_int(getattr(request, "num_computed_tokens", None))
    effective = _non_negative_int(cache_len_after)
    if logical is None or effective is None:
        return None
    offset = logical - min(effective, logical)
    if offset <= 0:
        _drop_attr(request, EFFECTIVE_KV_OFFSET_ATTR)
        return 0
    setattr(request, EFFECTIVE_KV_OFFSET_ATTR, offset)
    return offset


def prepare_request_effective_num_computed(request: Any):
    """Before a schedule step: ``num_computed_tokens - offset`` as the marker the allocation patch
    reads (runtime/kv_allocation_sync.py:64-84)."""
    if request is None:
        return None
    logical = _non_negative_int(getattr(request, "num_computed_tokens", None))
    if logical is None:
        return None
    offset = _non_negative_int(getattr(request, EFFECTIVE_KV_OFFSET_ATTR, None))
    if offset is None or offset <= 0:
        _drop_attr(request, EFFECTIVE_NUM_COMPUTED_ATTR)
        return None
    if logical == 0 or logical < offset:      # the request started over (preemption): forget the offset
        clear_request_allocation_sync_state(request)
        return None
    setattr(request, EFFECTIVE_NUM_COMPUTED_ATTR, logical - offset)
    return logical - offset


def resolve_request_effective_num_computed(request: Any):
    """runtime/kv_allocation_sync.py:87-94."""
    if request is None:
        return None
    logical = _non_negative_int(getattr(request, "num_computed_tokens", None))
    effective = _non_negative_int(getattr(request, EFFECTIVE_NUM_COMPUTED_ATTR, None))
    if logical is None or effective is None or effective > logical:
        return None
    return effective


# ------------------------------------------------------------ scheduler side
def resolve_full_prefill_len(request_like: Any) -> int:
    """Longest of the prompt-length views a request object offers (runtime/scheduler.py:54-82)."""
    found = []
    for attr in ("prompt_token_ids", "prefill_token_ids"):
        ids = getattr(request_like, attr, None)
        if ids is not None:
            try:
                found.append(len(ids))
            except Exception:
                pass
    for attr in ("prompt_token_ids_len", "num_prompt_tokens"):
        raw = getattr(request_like, attr, None)
        if raw is not None:
            try:
                found.append(int(raw))
            except (TypeError, ValueError):
                pass
    return max(found, default=0)


def _free_reclaimed_blocks(manager: Any, removed_blocks: list) -> bool:
    """Tail blocks go back to the pool, last block first, after their prefix-cache identity is
    dropped (runtime/scheduler.py:29-51)."""
    if not removed_blocks:
        return False
    pool = getattr(manager, "block_pool", None)
    evict = getattr(pool, "_maybe_evict_cached_block", None) if pool is not None else None
    for block in removed_blocks:
        if block is not None and getattr(block, "block_hash", None) is not None and callable(evict):
            evict(block)
    if pool is None:
        return False
    pool.free_blocks(reversed(removed_blocks))
    return True


class SchedulerCompressionGlue:
    """What the reference's ``TriAttentionScheduler`` adds to vLLM's scheduler, without the base
    class (runtime/scheduler.py:85-595).  The engine's scheduler calls

    * ``before_schedule(running)`` ahead of its own scheduling pass and caps its token budget with
      ``max_chunk_for_compression``;
    * ``after_schedule(scheduler_output, requests, kv_usage)``, which attaches ``triattention_step``
      and ``triattention_signals`` to the output;
    * ``apply_compression_events(events, requests, managers, block_size)`` when the runner's events
      come back, and ``forget_finished(req_ids)``.
    """

    def __init__(self, config: TriAttentionRuntimeConfig | None = None) -> None:
        self.config = config if config is not None else TriAttentionRuntimeConfig.from_env()
        self.planner = CompressionPlanner(self.config)
        self.tracker = EffectiveCacheLenTracker()
        self.prefill_lens: dict = {}
        self.length_thresholds: dict = {}
        self.step = 0

    # -- trigger ------------------------------------------------------------------
    def compute_length_threshold(self, prefill_len: int) -> int:
        """runtime/scheduler.py:132-136."""
        threshold = self.config.kv_budget + self.config.divide_length
        if self.config.protect_prefill and not self.config.include_prefill_in_budget:
            threshold += max(0, int(prefill_len))
        return threshold

    def _resolve_prefill_len(self, req_id, requests: dict) -> int:
        if req_id in self.prefill_lens:
            return self.prefill_lens[req_id]
        req = requests.get(req_id)
        return 0 if req is None else int(getattr(req, "num_prompt_tokens", 0))

    def _remember_prefill(self, req_id, prefill_len: int) -> None:
        self.prefill_lens[req_id] = prefill_len
        self.length_thresholds[req_id] = self.compute_length_threshold(prefill_len)

    def sync_prefill_lens(self, scheduler_output: Any, requests: dict) -> None:
        """New, finished and resumed requests of this step (runtime/scheduler.py:138-175).  A request
        that shows up again in ``scheduled_new_reqs`` (chunked prefill) keeps its tracker state."""
        for new_req in getattr(scheduler_output, "scheduled_new_reqs", None) or []:
            rid = new_req.req_id
            if rid not in self.prefill_lens:
                self.tracker.reset_request(rid, getattr(new_req, "num_computed_tokens", 0))
            self._remember_prefill(rid, resolve_full_prefill_len(new_req))
        for rid in getattr(scheduler_output, "finished_req_ids", None) or []:
            clear_request_allocation_sync_state(requests.get(rid))
            self.forget_finished([rid])
        cached = getattr(scheduler_output, "scheduled_cached_reqs", None)
        resumed = []
        if cached is not None:
            resumed = getattr(cached, "resumed_req_ids", None)
            if resumed is None:
                resumed = getattr(cached, "req_ids", []) or []
        for rid in resumed:
            if rid not in self.prefill_lens:
                self._remember_prefill(rid, self._resolve_prefill_len(rid, requests))

    def forget_finished(self, req_ids) -> None:
        for rid in req_ids:
            self.prefill_lens.pop(rid, None)
            self.length_thresholds.pop(rid, None)
            self.tracker.remove_request(rid)

    def build_signals(self, scheduler_output: Any, requests: dict, kv_usage: float | None = None) -> dict:
        """``{req_id: CompressionSignal}`` for the requests of this step that are due or that were
        compressed before and therefore need effective-length updates (runtime/scheduler.py:184-264).
        ``estimated_cache_len = effective base + scheduled tokens``; the base is
        ``num_computed_tokens`` until the first compression."""
        usage_on = bool(self.config.enable_kv_usage_trigger)
        usage = kv_usage if usage_on else None
        disabled = bool(self.config.disable_compression)
        signals: dict = {}
        for _raw, rid, scheduled in iter_scheduled_token_items(scheduler_output):
            req = requests.get(rid)
            if req is None:
                continue
            overridden = self.tracker.has_effective_len_override(rid)
            nct = int(getattr(req, "num_computed_tokens", 0))
            base = self.tracker.observe_num_computed(req_id=rid, num_computed_tokens=nct) if overridden else nct
            estimated = base + scheduled
            if not overridden:
                if disabled and not usage_on:
                    continue
                if not usage_on and not disabled:
                    threshold = self.length_thresholds.get(rid)
                    if threshold is None:
                        self._remember_prefill(rid, self._resolve_prefill_len(rid, requests))
                        threshold = self.length_thresholds[rid]
                    if estimated < threshold:
                        continue
            if rid not in self.prefill_lens:
                self._remember_prefill(rid, self._resolve_prefill_len(rid, requests))
            signal = self.planner.build_signal(req_id=rid, estimated_cache_len=estimated,
                                               prefill_len=self.prefill_lens[rid], step=self.step,
                                               kv_usage=usage, scheduled_tokens=scheduled)
            if signal.should_compress or overridden:
                signals[rid] = signal
        return signals

    def before_schedule(self, running) -> None:
        """runtime/scheduler.py:266-271."""
        if isinstance(running, list):
            for req in running:
                prepare_request_effective_num_computed(req)

    def max_chunk_for_compression(self, num_gpu_blocks: int, block_size: int):
        """Most tokens a step may schedule so that budget + chunk still fits the physical cache, one
        block held back; ``None``: no cap (runtime/scheduler.py:273-289)."""
        if self.config.disable_compression or num_gpu_blocks is None or num_gpu_blocks <= 0:
            return None
        bs = int(block_size or 16)
        headroom = int(num_gpu_blocks) * bs - self.config.kv_budget
        if headroom <= 0:
            return None
        return max(1, headroom - bs)

    def after_schedule(self, scheduler_output: Any, requests: dict, kv_usage: float | None = None) -> dict:
        """runtime/scheduler.py:305-321."""
        self.step += 1
        self.sync_prefill_lens(scheduler_output, requests)
        if (self.config.disable_compression and not self.config.enable_kv_usage_trigger
                and not self.tracker.has_any_effective_len_overrides()):
            signals = {}
        else:
            signals = self.build_signals(scheduler_output, requests, kv_usage)
        setattr(scheduler_output, "triattention_step", self.step)
        setattr(scheduler_output, "triattention_signals", signals)
        return signals

    # -- events -------------------------------------------------------------------
    def apply_compression_events(self, compression_events, requests: dict, managers, block_size: int) -> None:
        """Per applied event: the tracker takes ``cache_len_after``; with block reclaim on, every
        group's ``block_ids_after`` must be a duplicate-free prefix of what the manager holds (and, with
        ``require_physical_reclaim``, exactly ``ceil(cache_len_after / block_size)`` long where a
        shrink was due); the manager keeps that prefix plus the blocks appended since the hook ran
        (those beyond ``block_ids_before``), the old tail is freed last block first.  Groups the
        event does not list (the worker truncated them in an earlier step whose event is still
        under way) are truncated to the required length, but never during a multi-token (prefill)
        step, where new blocks cannot be told from old ones (runtime/scheduler.py:338-564)."""
        bs = int(block_size) if int(block_size) > 0 else 1
        many = isinstance(managers, (list, tuple))

        def truncate_to_required(gids, req_id, required) -> bool:
            freed = False
            for gid in sorted(gids):
                manager = managers[gid]
                blocks = manager.req_to_blocks.get(req_id)
                if not blocks or required >= len(blocks):
                    continue
                kept, removed = blocks[:required], blocks[required:]
                manager.req_to_blocks[req_id] = kept
                if req_id in manager.num_cached_block:
                    manager.num_cached_block[req_id] = min(manager.num_cached_block[req_id], len(kept))
                freed = _free_reclaimed_blocks(manager, removed) or freed
            return freed

        for event in compression_events or []:
            if event.get("status") != "applied":
                continue
            rid = event.get("req_id")
            after = event.get("cache_len_after")
            if rid is None or not isinstance(after, int):
                continue
            req = requests.get(rid)
            if req is None:
                continue
            self.tracker.apply_compression(req_id=rid, cache_len_after=after,
                                           num_computed_tokens=req.num_computed_tokens)
            if not self.config.enable_experimental_block_reclaim:
                continue
            required = 0 if after <= 0 else (after + bs - 1) // bs
            scheduled = int(event.get("scheduled_tokens", 1))
            due = set()
            if many:
                for gid, manager in enumerate(managers):
                    blocks = manager.req_to_blocks.get(rid)
                    if blocks and required < len(blocks):
                        due.add(gid)
            reclaim = event.get("block_reclaim")
            groups = reclaim.get("groups") if isinstance(reclaim, dict) else None
            freed_any = False
            if not isinstance(groups, list):
                if scheduled <= 1 and due and many:
                    freed_any = truncate_to_required(due, rid, required)
                if freed_any:
                    update_request_effective_kv_offset(request=req, cache_len_after=after)
                continue
            if not many:
                continue
            seen = set()
            for group in groups:
                if not isinstance(group, dict):
                    continue
                gid, ids_after = group.get("gid"), group.get("block_ids_after")
                if not isinstance(gid, int) or gid < 0 or gid >= len(managers):
                    continue
                if not isinstance(ids_after, list) or not all(isinstance(x, int) for x in ids_after):
                    continue
                manager = managers[gid]
                blocks = manager.req_to_blocks.get(rid)
                if not blocks:
                    continue
                seen.add(gid)
                current = [blk.block_id for blk in blocks]
                kept_len = len(ids_after)
                if kept_len > len(current):
                    raise RuntimeError("TriAttention block reclaim invalid length: "
                                       f"req={rid} gid={gid} kept_len={kept_len} curr_len={len(current)}")
                if len(set(ids_after)) != kept_len:
                    raise RuntimeError("TriAttention block reclaim contains duplicate block ids: "
                                       f"req={rid} gid={gid} block_ids_after={ids_after}")
                if current[:kept_len] != ids_after:
                    raise RuntimeError("TriAttention block reclaim prefix mismatch: "
                                       f"req={rid} gid={gid} expected_prefix={current[:kept_len]} "
                                       f"actual_after={ids_after}")
                if (getattr(self.config, "require_physical_reclaim", False) and gid in due
                        and kept_len != required):
                    raise RuntimeError("TriAttention block reclaim insufficient shrink: "
                                       f"req={rid} gid={gid} kept_len={kept_len} required_blocks={required}")
                ids_before = group.get("block_ids_before")
                original = len(ids_before) if isinstance(ids_before, list) else len(blocks)
                kept_old, removed_old, appended = list(blocks[:kept_len]), list(blocks[kept_len:original]), \
                    list(blocks[original:])
                manager.req_to_blocks[rid] = kept_old + appended
                if rid in manager.num_cached_block:
                    manager.num_cached_block[rid] = min(manager.num_cached_block[rid], len(kept_old) + len(appended))
                if removed_old:
                    freed_any = _free_reclaimed_blocks(manager, removed_old) or freed_any
            missing = due - seen
            if missing and scheduled <= 1:
                freed_any = truncate_to_required(missing, rid, required) or freed_any
            if freed_any:
                update_request_effective_kv_offset(request=req, cache_len_after=after)


# ------------------------------------------------------------ worker side
ALLOWED_STRICT_SKIP_REASONS = frozenset({"under_budget", "prefill_exceeds_budget", "req_state_not_found",
                                         "batch_queue_dedup"})


def register_new_requests(*, state_store: Any, scheduler_output: Any, protect_prefill: bool) -> None:
    """runtime/runner_state_updates.py:47-54."""
    for new_req in getattr(scheduler_output, "scheduled_new_reqs", None) or []:
        state_store.ensure(req_id=new_req.req_id, prefill_len=resolve_full_prefill_len(new_req),
                           protect_prefill=protect_prefill)


def cleanup_finished_requests(*, state_store: Any, scheduler_output: Any) -> None:
    for rid in getattr(scheduler_output, "finished_req_ids", None) or []:
        state_store.remove(rid)


def mark_preemptions(*, state_store: Any, scheduler_output: Any) -> None:
    for rid in getattr(scheduler_output, "preempted_req_ids", None) or []:
        state_store.mark_preempted(rid)


def mark_resumed(*, state_store: Any, scheduler_output: Any) -> None:
    cached = getattr(scheduler_output, "scheduled_cached_reqs", None)
    if cached is None:
        return
    resumed = getattr(cached, "resumed_req_ids", None)
    if resumed is None:
        resumed = getattr(cached, "req_ids", []) or []
    for rid in resumed:
        state_store.mark_resumed(rid)


def consume_runner_signals(*, state_store: Any, scheduler_output: Any, last_step: int, log_decisions: bool = False):
    """The worker's view of the step's signals: every signalled request gets its state and its
    cached length with this step's tokens.  Until a request's first compression that length is the
    scheduler's estimate; afterwards the worker counts on from its own last value (the scheduler's
    snapshots can lag under asynchronous scheduling), unless
    ``TRIATTN_RUNTIME_LEGACY_COMPRESSED_ESTIMATE`` is set (runtime/runner_state_updates.py:82-128).
    Returns ``(step, signals)``."""
    step = getattr(scheduler_output, "triattention_step", last_step + 1)
    signals = getattr(scheduler_output, "triattention_signals", {})
    legacy = os.environ.get("TRIATTN_RUNTIME_LEGACY_COMPRESSED_ESTIMATE", "0").strip().lower() in {"1", "true", "yes", "on"}
    for rid, signal in signals.items():
        state = state_store.ensure(req_id=rid, prefill_len=signal.prefill_len, protect_prefill=signal.protect_prefill)
        scheduled = max(0, int(getattr(signal, "scheduled_tokens", 1)))
        estimate = max(0, int(signal.estimated_cache_len))
        if int(getattr(state, "compression_count", 0)) > 0 and not legacy:
            estimate = max(0, int(getattr(state, "current_cache_len", 0))) + scheduled
        state_store.update_cache_len(rid, estimate, step=signal.step)
        if signal.should_compress:
            state_store.mark_trigger(rid, signal.reason, signal.step)
            if log_decisions:
                logger.debug("TriAttention trigger req=%s step=%d reason=%s len=%d mode=%s", rid, signal.step,
                             signal.reason, signal.estimated_cache_len, state.mode)
    return step, signals


def _scheduler_nct(scheduler_output: Any, req_id):
    cached = getattr(scheduler_output, "scheduled_cached_reqs", None)
    ids = getattr(cached, "req_ids", None) if cached is not None else None
    ncts = getattr(cached, "num_computed_tokens", None) if cached is not None else None
    if isinstance(ids, list) and isinstance(ncts, list):
        try:
            return int(ncts[ids.index(req_id)])
        except (ValueError, IndexError):
            return None
    return None


def execute_runner_compression_actions(*, executor: Any, state_store: Any, scheduler_output: Any, signals: dict,
                                       strict_no_downgrade: bool,
                                       allowed_strict_skip_reasons=ALLOWED_STRICT_SKIP_REASONS,
                                       log_decisions: bool = False, batched: bool = True) -> list:
    """The worker's part of a step: run the hook for every triggered request, keep the request state
    store in step, and return the event dictionaries the scheduler consumes
    (runtime/runner_compression_actions.py:11-237; event keys ``req_id, step, status, reason,
    cache_len_after, details, scheduled_tokens, estimated_cache_len, prefill_len, block_reclaim``).
    A request compressed in the previous step is not compressed again in a single-token step (the
    scheduler may not have seen that event yet).  In strict mode an exception or a skip for any
    reason outside ``allowed_strict_skip_reasons`` raises with the fatal marker.

    ``batched``: requests that are due in the same step go through ``executor.execute_batch`` when the
    executor has it (one launch sequence for all of them; the reference calls ``execute`` per
    request), with identical events."""
    events: list = []

    def base_event(rid, signal, status, reason, after):
        return {"req_id": rid, "step": signal.step, "status": status, "reason": reason, "cache_len_after": after,
                "scheduled_tokens": int(getattr(signal, "scheduled_tokens", 1)),
                "estimated_cache_len": int(getattr(signal, "estimated_cache_len", 0)),
                "prefill_len": int(getattr(signal, "prefill_len", 0))}

    due = {}
    for rid, signal in signals.items():
        if not signal.should_compress:
            continue
        st = state_store.get(rid) if hasattr(state_store, "get") else None
        if st is not None:
            last = getattr(st, "last_compression_step", -1)
            count = int(getattr(st, "compression_count", 0) or 0)
            if count > 0 and last >= 0 and signal.step - last <= 1 and int(getattr(signal, "scheduled_tokens", 1)) <= 1:
                if hasattr(state_store, "mark_compression_skipped"):
                    state_store.mark_compression_skipped(req_id=rid, reason="batch_queue_dedup", step=signal.step)
                events.append(base_event(rid, signal, "skipped", "batch_queue_dedup",
                                         getattr(st, "current_cache_len", None)))
                continue
        due[rid] = signal

    results, failures = {}, {}
    run_batch = getattr(executor, "execute_batch", None) if batched and len(due) > 1 else None
    if callable(run_batch):
        try:
            results = dict(run_batch(due, scheduler_output))
        except Exception as exc:
            failures = {rid: exc for rid in due}
    for rid, signal in due.items():
        if rid in results or rid in failures:
            continue
        try:
            results[rid] = executor.execute(req_id=rid, signal=signal, scheduler_output=scheduler_output)
        except Exception as exc:
            failures[rid] = exc

    for rid, signal in due.items():
        if rid in failures:
            exc = failures[rid]
            if strict_no_downgrade:
                raise RuntimeError(f"{MARK}:executor_exception:req={rid}:step={signal.step}:"
                                   f"type={type(exc).__name__}") from exc
            if MARK in str(exc):
                raise exc
            state_store.mark_compression_skipped(req_id=rid, reason=f"executor_exception:{type(exc).__name__}",
                                                 step=signal.step)
            logger.error("TriAttention compression executor failed req=%s step=%d: %r", rid, signal.step, exc)
            events.append(base_event(rid, signal, "error", f"executor_exception:{type(exc).__name__}", None))
            continue
        result = results[rid]
        if strict_no_downgrade and not result.applied and result.reason not in allowed_strict_skip_reasons:
            raise RuntimeError(f"{MARK}:unexpected_skip:req={rid}:step={signal.step}:reason={result.reason}")
        details = result.details if isinstance(result.details, dict) else None
        reclaim = details.get("block_reclaim") if details is not None else None
        if result.applied:
            after = signal.estimated_cache_len if result.cache_len_after is None else result.cache_len_after
            state_store.mark_compressed(req_id=rid, step=signal.step, cache_len=after,
                                        scheduled_tokens=int(getattr(signal, "scheduled_tokens", 1)),
                                        scheduler_nct=_scheduler_nct(scheduler_output, rid))
            if log_decisions:
                logger.debug("TriAttention compression applied req=%s step=%d reason=%s after=%d", rid, signal.step,
                             result.reason, after)
            event = base_event(rid, signal, "applied", result.reason, after)
        else:
            state_store.mark_compression_skipped(req_id=rid, reason=result.reason, step=signal.step)
            event = base_event(rid, signal, "skipped", result.reason, result.cache_len_after)
        event["details"] = result.details
        event["block_reclaim"] = reclaim
        events.append(event)
    return events


def apply_worker_block_reclaim_events(*, base_runner: Any, events) -> None:
    """After a compression the worker's own block tables must start appending at the shortened
    length: ``num_blocks_per_row[row]`` of every (group) table drops to
    ``ceil(cache_len_after / block_size)`` and the request state's block id lists are cut to
    that length (runtime/worker_reclaim_sync.py:15-128).  Runners that keep ``block_tables`` on
    themselves are already up to date after the hook."""
    if os.environ.get("TRIATTN_DEBUG_DISABLE_WORKER_RECLAIM_SYNC", "0").strip().lower() in {"1", "true", "yes", "on"}:
        return
    if not isinstance(events, list) or not events:
        return
    batch = getattr(base_runner, "input_batch", None)
    table_obj = getattr(batch, "block_table", None) if batch else None
    if table_obj is None:
        if getattr(base_runner, "block_tables", None) is None:
            logger.warning("TriAttention worker reclaim: block table not found")
        return
    row_of = getattr(batch, "req_id_to_index", None)
    if not isinstance(row_of, dict):
        logger.warning("TriAttention worker reclaim: req_id_to_index not found on input_batch")
        return
    inner = getattr(table_obj, "block_tables", None)
    tables = inner if isinstance(inner, list) else [table_obj]
    bs = int(getattr(getattr(base_runner, "cache_config", None), "block_size", 16))
    if bs <= 0:
        bs = 16
    requests = getattr(base_runner, "requests", None)
    for event in events:
        if not isinstance(event, dict) or event.get("status") != "applied":
            continue
        rid = event.get("req_id")
        row = row_of.get(rid) if rid is not None else None
        after = event.get("cache_len_after")
        if not isinstance(row, int) or not isinstance(after, int) or after <= 0:
            continue
        required = (after + bs - 1) // bs
        for table in tables:
            rows = getattr(table, "num_blocks_per_row", None)
            if not isinstance(rows, np.ndarray):
                continue
            if int(rows[row]) > required:
                rows[row] = required
        if isinstance(requests, dict):
            state = requests.get(rid)
            ids = getattr(state, "block_ids", None) if state is not None else None
            if isinstance(ids, (list, tuple)):
                for group in ids:
                    if isinstance(group, list) and len(group) > required:
                        del group[required:]


def resolve_req_id_to_index(base_runner: Any):
    """``(req_id -> row, where it was found)`` (runtime/runner_struct_compat.py:40-55)."""
    for owner, label in ((getattr(base_runner, "req_states", None), "req_states"),
                         (getattr(base_runner, "input_batch", None), "input_batch")):
        mapping = getattr(owner, "req_id_to_index", None) if owner is not None else None
        if isinstance(mapping, dict) and mapping:
            return mapping, label
    ids = getattr(getattr(base_runner, "input_batch", None), "req_ids", None)
    if isinstance(ids, (list, tuple)):
        rebuilt = {rid: i for i, rid in enumerate(ids) if rid is not None}
        if rebuilt:
            return rebuilt, "input_batch_req_ids"
    return None, "none"


def _marks_effective_pre_step(state: Any, scheduler_step):
    """True / False when the request state says what ``current_cache_len`` means, None when it does
    not say (runtime/effective_overrides.py:48-70)."""
    if state is None:
        return None
    semantics = getattr(state, "current_cache_len_semantics", None)
    if not isinstance(semantics, str):
        return None
    if semantics != "effective_pre_step":
        return False
    at = getattr(state, "current_cache_len_step", None)
    if isinstance(scheduler_step, int) and isinstance(at, int):
        return at == scheduler_step
    return True


def effective_base_before_step(*, state: Any, abs_progress: int, scheduled_tokens: int, scheduler_step) -> int:
    """Cached tokens of a request before this step's tokens are appended
    (runtime/effective_overrides.py:73-98)."""
    current = int(getattr(state, "current_cache_len", abs_progress)) if state is not None else abs_progress
    marked = _marks_effective_pre_step(state, scheduler_step)
    if marked is True:
        return current
    if marked is None and state is not None:
        count = getattr(state, "compression_count", None)
        if isinstance(count, int) and count > 0:
            raise RuntimeError("TRIATTN_EFFECTIVE_BASE_STATE_SEMANTICS_MISSING:"
                               "compressed_request_state_missing_current_cache_len_semantics")
    return max(0, current - max(0, int(scheduled_tokens)))


def _abs_progress_for_override(*, req_state, state, scheduled_tokens, scheduler_step, scheduler_nct):
    """runtime/effective_overrides.py:124-168."""
    progress = int(scheduler_nct) if scheduler_nct is not None else \
        (int(getattr(req_state, "num_computed_tokens", 0)) if req_state is not None else 0)
    if state is None:
        return progress
    count, prefill = getattr(state, "compression_count", None), getattr(state, "prefill_len", None)
    if not isinstance(count, int) or count <= 0 or not isinstance(prefill, int) or prefill <= 0:
        return progress
    if progress >= prefill:
        return progress
    # first decode step after the last prefill chunk: the counter may still be one chunk behind
    if int(scheduled_tokens) == 1 and _marks_effective_pre_step(state, scheduler_step) is True:
        return int(prefill)
    return progress


def build_effective_sparse_overrides(*, base_runner: Any, state_store: Any, scheduler_output: Any,
                                     compression_events=None):
    """``(seq_bases, pos_deltas, single_seq_base, single_pos_delta)``: per request row, the cached
    length before this step and ``effective base - num_computed_tokens`` for the slot mapping, only
    for rows where the two differ; the last two are a one-row fast path
    (runtime/effective_overrides.py:209-359).  Between compressions the delta is the constant
    ``cache_len_after_last_compression - nct_at_last_compression`` when the request state has both
    and the scheduler output carries the request's ``num_computed_tokens``."""
    key = (id(base_runner), id(state_store))
    cache = getattr(scheduler_output, "_triattention_cached_sparse_overrides", None) \
        if scheduler_output is not None else None
    if isinstance(cache, dict) and isinstance(cache.get(key), tuple) and len(cache[key]) == 4:
        return cache[key]

    def done(value):
        if scheduler_output is not None:
            try:
                store = getattr(scheduler_output, "_triattention_cached_sparse_overrides", None)
                if not isinstance(store, dict):
                    store = {}
                    setattr(scheduler_output, "_triattention_cached_sparse_overrides", store)
                store[key] = value
            except Exception:
                pass
        return value

    requests = getattr(base_runner, "requests", None)
    if not isinstance(requests, dict):
        return done((None, None, None, 0))
    row_of, _ = resolve_req_id_to_index(base_runner)
    if not isinstance(row_of, dict):
        return done((None, None, None, 0))
    active = None
    checker = getattr(state_store, "has_active_compressed_requests", None) if state_store is not None else None
    if callable(checker):
        try:
            active = bool(checker())
        except Exception:
            active = None
    applied = {e["req_id"] for e in (compression_events or []) if isinstance(e, dict)
               and e.get("status") == "applied" and e.get("req_id") is not None} \
        if isinstance(compression_events, list) else set()
    if active is False and applied:
        raise RuntimeError("TRIATTN_COMPRESSION_EVENT_STATE_MISMATCH:"
                           "applied_compression_events_present_but_state_store_reports_no_compressed_requests")
    if active is False:
        return done((None, None, None, 0))
    items = get_scheduled_token_items(scheduler_output)
    if not items:
        return done((None, None, None, 0))
    step = getattr(scheduler_output, "triattention_step", None)
    step = int(step) if isinstance(step, int) else None
    nct_map = None
    cached_reqs = getattr(scheduler_output, "scheduled_cached_reqs", None)
    if cached_reqs is not None:
        ids, ncts = getattr(cached_reqs, "req_ids", None), getattr(cached_reqs, "num_computed_tokens", None)
        if isinstance(ids, list) and isinstance(ncts, list) and len(ids) == len(ncts):
            nct_map = dict(zip(ids, ncts))
    state_get = getattr(state_store, "get", None)
    state_get = state_get if callable(state_get) else None
    seq_bases, pos_deltas = {}, {}
    for _raw, rid, scheduled in items:
        row = row_of.get(rid)
        if not isinstance(row, int):
            continue
        state = state_get(rid) if state_get is not None else None
        if state is not None:
            count = getattr(state, "compression_count", None)
            if isinstance(count, int) and count <= 0:
                continue          # never compressed: the engine's own lengths are right
        nct_then = getattr(state, "nct_at_last_compression", None) if state is not None else None
        len_then = getattr(state, "cache_len_after_last_compression", None) if state is not None else None
        nct_now = nct_map.get(rid) if nct_map is not None else None
        if isinstance(nct_then, int) and isinstance(len_then, int) and isinstance(nct_now, int):
            before_step = len_then + (nct_now - nct_then)
            delta = int(len_then - nct_then)
        else:
            progress = _abs_progress_for_override(req_state=requests.get(rid), state=state,
                                                  scheduled_tokens=scheduled, scheduler_step=step,
                                                  scheduler_nct=nct_now)
            before_step = effective_base_before_step(state=state, abs_progress=progress,
                                                     scheduled_tokens=scheduled, scheduler_step=step)
            delta = int(before_step - progress)
        if delta == 0:
            continue
        seq_bases[row] = before_step
        pos_deltas[row] = delta
    single_base, single_delta = None, 0
    if len(seq_bases) == 1:
        single_base = next(iter(seq_bases.values()))
        single_delta = int(next(iter(pos_deltas.values())))
    return done((seq_bases or None, pos_deltas or None, single_base, single_delta))
