"""The runner hook ``triattention_apply_compression(req_id, signal, scheduler_output)``.

This is the plug-in seam of the reference (runtime/executor.py:31-85,
runtime/hook_impl.py:30-185): ``install_runner_compression_hook`` puts a callable of
that name on the base runner unless one is already there, and the executor calls it
once per triggered request.  Request-state lookup follows runtime/hook_preflight.py and
runtime/runner_struct_compat.py, the length bookkeeping runtime/hook_runtime_context.py,
the KV tensors per cache group runtime/kv_group_resolver.py.  Only plain attribute
access is used on the runner, so any object with ``requests``, ``kv_caches`` and
``cache_config.block_size`` works.
"""
from __future__ import annotations

import os
import re
from dataclasses import dataclass
from typing import Any, Callable

import torch

from .config import TriAttentionRuntimeConfig
from .kv_compaction import (build_keep_token_indices, compact_request_kv_in_place,
                            compact_request_kv_in_place_per_head, gather_request_k_dense,
                            register_kv_layout_axis_hint)
from .models import TRITON_SCORING_REQUIRED_MARKER as MARK, CompressionSignal
from .pipeline import (GroupPipelineOutcome, finalize_hook_placement_result, normalize_mutable_block_ids_by_group,
                       num_required_blocks, run_group_compaction_pipeline, truncate_tail_reclaim_group)
from .selector import ResidentLaunchFailed, build_triattention_selector as _build_triattention_selector


# --------------------------------------------------------------- executor side
@dataclass(frozen=True)
class CompressionExecutionResult:
    applied: bool
    reason: str
    cache_len_after: int | None = None
    details: dict | None = None


class CompressionExecutor:
    def execute(self, req_id: str, signal: CompressionSignal, scheduler_output: Any) -> CompressionExecutionResult:
        raise NotImplementedError


class RunnerHookCompressionExecutor(CompressionExecutor):
    """Delegates to the hook on the base runner (runtime/executor.py:31-85)."""

    hook_name = "triattention_apply_compression"

    def __init__(self, base_runner: Any):
        self._base_runner = base_runner

    def execute(self, req_id, signal, scheduler_output) -> CompressionExecutionResult:
        hook = getattr(self._base_runner, self.hook_name, None)
        if not callable(hook):
            return CompressionExecutionResult(False, "runner_hook_missing")
        out = hook(req_id=req_id, signal=signal, scheduler_output=scheduler_output)
        if isinstance(out, bool):
            return CompressionExecutionResult(out, "applied" if out else "runner_hook_rejected")
        if isinstance(out, dict):
            d = dict(out)
            return CompressionExecutionResult(bool(d.get("applied", False)), str(d.get("reason", "runner_hook_result")),
                                              d.get("cache_len_after"), d)
        return CompressionExecutionResult(False, f"unsupported_hook_result:{type(out).__name__}")

    batch_hook_name = "triattention_apply_compression_batch"

    def execute_batch(self, signals: dict, scheduler_output) -> dict:
        """All triggered requests of a step in one call (no counterpart in the reference, whose
        runner walks them one by one, runtime/runner_compression_actions.py:24-70):
        ``{req_id: CompressionExecutionResult}``.  Falls back to ``execute`` per request when
        the runner carries no batch hook."""
        hook = getattr(self._base_runner, self.batch_hook_name, None)
        todo = {rid: sig for rid, sig in signals.items() if getattr(sig, "should_compress", True)}
        if not callable(hook):
            return {rid: self.execute(rid, sig, scheduler_output) for rid, sig in todo.items()}
        out = hook(signals=todo, scheduler_output=scheduler_output)
        results = {}
        for rid in todo:
            d = dict(out.get(rid) or {"applied": False, "reason": "runner_hook_result_missing"})
            results[rid] = CompressionExecutionResult(bool(d.get("applied", False)),
                                                      str(d.get("reason", "runner_hook_result")),
                                                      d.get("cache_len_after"), d)
        return results


# ------------------------------------------------------------- request lookup
def req_id_from_scheduled_key(key: Any):
    if isinstance(key, (str, int)):
        return key
    for attr in ("request_id", "req_id"):
        v = getattr(key, attr, None)
        if isinstance(v, (str, int)):
            return v
    return None


def scheduled_tokens_for_req(scheduler_output: Any, req_id: str) -> int:
    """Tokens scheduled for the request this step, at least 1
    (runtime/hook_runtime_context.py:57-76, runtime/request_key_compat.py)."""
    table = getattr(scheduler_output, "num_scheduled_tokens", None)
    if not isinstance(table, dict):
        return 1
    for raw_key, raw_val in table.items():
        if req_id_from_scheduled_key(raw_key) == req_id:
            try:
                return max(1, int(raw_val))
            except (TypeError, ValueError):
                return 1
    return 1


@dataclass
class _SchedulerRequestView:
    req_id: str
    num_computed_tokens: int
    block_ids: Any


class _MergedRequestView:
    """Runner-side state whose num_computed_tokens lags the scheduler's
    (runtime/hook_preflight.py:40-61)."""

    def __init__(self, base, num_computed_tokens: int, fallback_block_ids):
        self._base, self._nct, self._fallback = base, int(num_computed_tokens), fallback_block_ids

    @property
    def num_computed_tokens(self) -> int:
        return self._nct

    @property
    def block_ids(self):
        ids = getattr(self._base, "block_ids", None)
        return ids if ids is not None else self._fallback

    @block_ids.setter
    def block_ids(self, value) -> None:
        setattr(self._base, "block_ids", value)


class _IndexedRequestView:
    """Request addressed by its row in the runner's batch tables
    (runtime/runner_struct_compat.py:61-141)."""

    def __init__(self, runner, req_id, index, requests_state):
        self._runner, self.req_id, self._index, self._requests_state = runner, req_id, index, requests_state

    @property
    def num_computed_tokens(self) -> int:
        gpu = getattr(getattr(getattr(self._runner, "req_states", None), "num_computed_tokens", None), "gpu", None)
        if torch.is_tensor(gpu):
            return int(gpu[self._index].item())
        cpu = getattr(getattr(self._runner, "input_batch", None), "num_computed_tokens_cpu", None)
        try:
            return int(cpu[self._index]) if cpu is not None else 0
        except Exception:
            return 0

    @property
    def block_ids(self):
        tables = getattr(self._runner, "block_tables", None)
        rows = getattr(tables, "block_tables", None)
        counts = getattr(getattr(tables, "num_blocks", None), "np", None)
        if isinstance(rows, list) and counts is not None:
            out, ok = [], True
            for gid, table in enumerate(rows):
                try:
                    n = int(counts[gid, self._index])
                except Exception:
                    ok = False
                    break
                gpu = getattr(table, "gpu", None)
                if n <= 0:
                    out.append([])
                elif torch.is_tensor(gpu):
                    out.append([int(x) for x in gpu[self._index, :n].tolist()])
                else:
                    ok = False
                    break
            if ok and any(out):
                return tuple(out)
        ids = getattr(self._requests_state, "block_ids", None)
        if isinstance(ids, (list, tuple)):
            return tuple([int(b) for b in g] if isinstance(g, (list, tuple)) else [] for g in ids)
        return None

    @block_ids.setter
    def block_ids(self, new_ids) -> None:
        if not isinstance(new_ids, (list, tuple)):
            raise TypeError("block_ids must be a list/tuple by group")
        norm = tuple([int(b) for b in g] if isinstance(g, (list, tuple)) else [] for g in new_ids)
        tables = getattr(self._runner, "block_tables", None)
        if tables is not None:
            tables.append_block_ids(self._index, norm, overwrite=True)
            tables.apply_staged_writes()
        if self._requests_state is not None:
            setattr(self._requests_state, "block_ids", norm)


def _scheduler_view(scheduler_output, req_id):
    for new_req in getattr(scheduler_output, "scheduled_new_reqs", None) or []:
        if getattr(new_req, "req_id", None) != req_id or getattr(new_req, "block_ids", None) is None:
            continue
        lens = []
        for attr in ("prompt_token_ids", "prefill_token_ids"):
            v = getattr(new_req, attr, None)
            if v is not None:
                try:
                    lens.append(len(v))
                except Exception:
                    pass
        for attr in ("prompt_token_ids_len", "num_prompt_tokens"):
            v = getattr(new_req, attr, None)
            try:
                if v is not None:
                    lens.append(int(v))
            except (TypeError, ValueError):
                pass
        return _SchedulerRequestView(req_id, max(lens, default=0), new_req.block_ids)
    cached = getattr(scheduler_output, "scheduled_cached_reqs", None)
    ids, ncts = getattr(cached, "req_ids", None), getattr(cached, "num_computed_tokens", None)
    if isinstance(ids, list) and isinstance(ncts, list):
        for i, rid in enumerate(ids):
            if rid == req_id and i < len(ncts):
                try:
                    return _SchedulerRequestView(req_id, int(ncts[i]), None)
                except Exception:
                    return None
    return None


def resolve_request_state(base_runner: Any, req_id: str, scheduler_output: Any = None):
    """The request's state object (has ``num_computed_tokens`` and settable
    ``block_ids``), or None (runtime/hook_preflight.py:124-219)."""
    requests = getattr(base_runner, "requests", None)
    requests_state = requests.get(req_id) if isinstance(requests, dict) else None
    state = None
    for owner_name in ("req_states", "input_batch"):
        index_map = getattr(getattr(base_runner, owner_name, None), "req_id_to_index", None)
        if isinstance(index_map, dict) and isinstance(index_map.get(req_id), int):
            state = _IndexedRequestView(base_runner, req_id, index_map[req_id], requests_state)
            break
    if state is None:
        batch = getattr(base_runner, "input_batch", None)
        ids = getattr(batch, "req_ids", None)
        try:
            ids = ids() if callable(ids) else ids
        except Exception:
            ids = None
        if not isinstance(ids, list):
            ids = getattr(batch, "_req_ids", None)
        if isinstance(ids, list) and req_id in ids:
            state = _IndexedRequestView(base_runner, req_id, ids.index(req_id), requests_state)
    if state is None:
        state = requests_state
    sched = _scheduler_view(scheduler_output, req_id) if scheduler_output is not None else None
    if state is None:
        return sched
    if sched is not None:
        try:
            mine = int(getattr(state, "num_computed_tokens", 0) or 0)
            if int(sched.num_computed_tokens) > mine:
                return _MergedRequestView(state, sched.num_computed_tokens, sched.block_ids)
        except Exception:
            pass
    return state


# ------------------------------------------------------------- KV tensors by group
def infer_layer_idx(layer_name: str, layer_obj: Any, fallback_idx: int) -> int:
    for attr in ("layer_idx", "layer_id", "idx"):
        v = getattr(layer_obj, attr, None)
        if isinstance(v, int):
            return v
    digits = re.findall(r"\d+", layer_name)
    return int(digits[-1]) if digits else fallback_idx


def _kv_axis_of_backend(base_runner: Any, gid: int):
    """0 for [2, nb, ...] backends, 1 for [nb, 2, ...] (runtime/kv_group_resolver.py:24-66)."""
    groups = getattr(base_runner, "attn_groups", None)
    if not isinstance(groups, (list, tuple)) or not 0 <= gid < len(groups):
        return None
    backend = getattr(groups[gid], "backend", None)
    if backend is None:
        return None
    cls = backend if isinstance(backend, type) else backend.__class__
    shape_fn = getattr(cls, "get_kv_cache_shape", None)
    if callable(shape_fn):
        try:
            shape = tuple(int(x) for x in shape_fn(3, 16, 1, 1))
            if len(shape) >= 2 and (shape[0] == 2) != (shape[1] == 2):
                return 0 if shape[0] == 2 else 1
        except Exception:
            pass
    ident = f"{getattr(cls, '__module__', '')}.{getattr(cls, '__name__', '')}".lower()
    if "flash_attn" in ident:
        return 0
    if "triton_attn" in ident:
        return 1
    return None


def resolve_group_tensors(base_runner: Any) -> dict:
    """gid -> [(layer_idx, kv_cache tensor)] (runtime/kv_group_resolver.py:69-141)."""
    out: dict = {}
    kv_cfg = getattr(base_runner, "kv_cache_config", None)
    ctx = getattr(getattr(base_runner, "compilation_config", None), "static_forward_context", None)
    if kv_cfg is None or not isinstance(ctx, dict):
        caches = getattr(base_runner, "kv_caches", None)
        if isinstance(caches, list):
            pairs = [(i, t) for i, t in enumerate(caches) if isinstance(t, torch.Tensor)]
            if pairs:
                out[0] = pairs
        return out
    for gid, group in enumerate(getattr(kv_cfg, "kv_cache_groups", None) or []):
        names = getattr(group, "layer_names", None)
        if not isinstance(names, (list, tuple)):
            continue
        pairs, seen = [], set()
        for local_idx, name in enumerate(names):
            layer = ctx.get(name)
            caches = getattr(layer, "kv_cache", None)
            if not isinstance(caches, list) or not caches or not isinstance(caches[0], torch.Tensor):
                continue
            if caches[0].data_ptr() in seen:
                continue
            seen.add(caches[0].data_ptr())
            pairs.append((infer_layer_idx(name, layer, local_idx), caches[0]))
        if pairs:
            axis = _kv_axis_of_backend(base_runner, gid)
            if axis is not None:
                for _, t in pairs:
                    try:
                        register_kv_layout_axis_hint(t, axis)
                    except ValueError:
                        pass
            out[gid] = pairs
    return out


# ------------------------------------------------------------- length bookkeeping
@dataclass(frozen=True)
class HookRuntimeContext:
    scheduled_tokens: int
    num_computed_tokens: int
    estimated_effective_tokens: int
    effective_tokens: int
    budget_total: int
    recent_unabsorbed_tokens: int | None
    should_defer_recompress: bool


def effective_budget_for_signal(config, signal, total_tokens: int) -> int:
    budget = config.kv_budget
    if signal.protect_prefill and not config.include_prefill_in_budget:
        budget += max(signal.prefill_len, 0)
    return min(total_tokens, budget)


def build_hook_runtime_context(*, base_runner: Any, config: TriAttentionRuntimeConfig, req_id: str, req_state: Any,
                               req_runtime_state: Any, signal: CompressionSignal, scheduler_output: Any,
                               compressed_once: set, original_block_ids_by_group: Any,
                               block_size_hint: int) -> HookRuntimeContext:
    """Effective cached tokens, budget and the re-compression gate
    (runtime/hook_runtime_context.py:106-209)."""
    capacities = [len(g) * block_size_hint for g in (original_block_ids_by_group or ())
                  if isinstance(g, (list, tuple))] if isinstance(original_block_ids_by_group, (list, tuple)) else []
    capacity = min(capacities) if capacities and block_size_hint > 0 else None

    scheduled = scheduled_tokens_for_req(scheduler_output, req_id)
    nct = int(getattr(req_state, "num_computed_tokens", 0))
    estimated = max(0, int(getattr(signal, "estimated_cache_len", 0)))
    if req_runtime_state is not None:
        cnt = getattr(req_runtime_state, "compression_count", None)
        cur = getattr(req_runtime_state, "current_cache_len", None)
        if isinstance(cnt, int) and cnt > 0 and isinstance(cur, int) and cur > 0:
            estimated = max(0, cur)

    post_forward = getattr(signal, "_post_forward", False)
    effective = max(0, estimated) if post_forward else max(0, estimated - max(0, scheduled))
    effective = min(effective, nct + (scheduled if post_forward else 0))
    if isinstance(capacity, int):
        effective = min(effective, capacity + block_size_hint)

    recent = None
    if req_runtime_state is not None:
        recent = max(0, effective - int(getattr(req_runtime_state, "last_absorbed_cache_len", 0)))
    setattr(base_runner, "_triattention_active_recent_unabsorbed_tokens", recent)

    prefill_len = int(getattr(signal, "prefill_len", 0) or 0)
    if (config.fail_on_effective_len_regression and config.enable_experimental_block_reclaim
            and req_id in compressed_once and not (prefill_len > 0 and nct < prefill_len)):
        upper = config.kv_budget + (max(signal.prefill_len, 0) if signal.protect_prefill
                                    and not config.include_prefill_in_budget else 0)
        upper += max(1, config.effective_len_guard_divide_multiples) * max(1, config.divide_length)
        slack = block_size_hint + max(1, int(getattr(signal, "estimated_cache_len", 0)) - nct) + max(1, scheduled)
        if (effective > upper + slack and nct > upper + slack
                and effective >= int(config.effective_len_regression_ratio * nct)):
            raise RuntimeError(f"{MARK}:effective_len_regressed:req={req_id}:effective_tokens={effective}:"
                               f"num_computed_tokens={nct}:guard_upper={upper}")

    budget_total = effective_budget_for_signal(config, signal, effective)
    gate_hit = estimated >= budget_total + max(1, config.divide_length)
    defer = (config.enable_experimental_kv_compaction and req_id in compressed_once
             and str(getattr(signal, "reason", "")) != "kv_usage_threshold" and not gate_hit)
    return HookRuntimeContext(int(scheduled), int(nct), int(estimated), int(effective), int(budget_total),
                              int(recent) if isinstance(recent, int) else None, bool(defer))


# A single request in the default mode goes through the same one-call launch sequence as a batch
# of requests; False sends it through the reference-shaped pipeline (selector callable, then the
# per-head compaction function), which gives the same result dictionaries and cache contents.
SINGLE_REQUEST_IN_ONE_CALL = True


@dataclass
class _Ready:
    """A triggered request that passed every check in front of the kernels."""
    req_id: str
    signal: CompressionSignal
    req_state: Any
    ctx: HookRuntimeContext
    original_ids: Any
    mutable_ids: list
    block_size: int
    strict: bool


def _debug_env_active() -> bool:
    """Debug switches that only the one-by-one path implements."""
    on = {"1", "true", "yes", "on"}
    return bool(os.environ.get("TRIATTN_DEBUG_OVERRIDE_FIRST_KEEP_JSON", "").strip()) or \
        os.environ.get("TRIATTN_DEBUG_FORCE_PRESERVE_DROPPED", "0").strip().lower() in on


# ------------------------------------------------------------------- the hook
def make_runner_compression_hook(base_runner: Any, config: TriAttentionRuntimeConfig) -> Callable[..., dict]:
    """runtime/hook_impl.py:30-165."""
    try:
        select_layer, select_group, selector_status = _build_triattention_selector(config, base_runner=base_runner)
    except TypeError:
        select_layer, select_group, selector_status = _build_triattention_selector(config)
    group_tensors: dict | None = None
    compressed_once: set = set()
    compress_batch = getattr(select_group, "_compress_batch", None) if select_group is not None else None

    def _prepare(req_id: str, signal: CompressionSignal, scheduler_output: Any):
        """Everything before the kernels: a result dictionary when the request is skipped,
        else the facts the compaction needs."""
        nonlocal group_tensors
        setattr(base_runner, "_triattention_active_req_id", req_id)
        strict = bool(config.enable_experimental_kv_compaction and config.require_triton_scoring)
        req_state = resolve_request_state(base_runner, req_id, scheduler_output)
        if req_state is None:
            return {"applied": False, "reason": "req_state_not_found"}
        store = getattr(base_runner, "_triattention_state_store", None)
        runtime_state = store.get(req_id) if store is not None and hasattr(store, "get") else None
        block_size_hint = int(getattr(getattr(base_runner, "cache_config", None), "block_size", 0))
        if block_size_hint <= 0:
            block_size_hint = 1
        original_ids = getattr(req_state, "block_ids", None)
        ctx = build_hook_runtime_context(
            base_runner=base_runner, config=config, req_id=req_id, req_state=req_state,
            req_runtime_state=runtime_state, signal=signal, scheduler_output=scheduler_output,
            compressed_once=compressed_once, original_block_ids_by_group=original_ids,
            block_size_hint=block_size_hint)
        if ctx.effective_tokens <= ctx.budget_total or ctx.should_defer_recompress:
            return {"applied": False, "reason": "under_budget", "cache_len_after": ctx.effective_tokens}

        if not config.enable_experimental_kv_compaction:
            plan = build_keep_token_indices(total_tokens=ctx.effective_tokens, kv_budget=config.kv_budget,
                                            prefill_len=signal.prefill_len, protect_prefill=signal.protect_prefill,
                                            include_prefill_in_budget=config.include_prefill_in_budget)
            if plan is None:
                return {"applied": False, "reason": "prefill_exceeds_budget"}
            return {"applied": False, "reason": "plan_only", "cache_len_after": len(plan)}
        if strict and select_layer is None:
            raise RuntimeError(f"{MARK}:selector_unavailable:{selector_status}")

        kv_caches = getattr(base_runner, "kv_caches", None)
        cache_config = getattr(base_runner, "cache_config", None)
        if not isinstance(kv_caches, list) or cache_config is None:
            return {"applied": False, "reason": "kv_cache_unavailable"}
        block_size = int(getattr(cache_config, "block_size", 0))
        if block_size <= 0:
            return {"applied": False, "reason": "invalid_block_size"}
        if not original_ids:
            return {"applied": False, "reason": "missing_block_ids"}
        mutable_ids = normalize_mutable_block_ids_by_group(original_ids)
        if mutable_ids is None:
            return {"applied": False, "reason": "invalid_block_ids_container"}
        if group_tensors is None:
            group_tensors = resolve_group_tensors(base_runner)
        return _Ready(req_id, signal, req_state, ctx, original_ids, mutable_ids, block_size, strict)

    def _finish(r: "_Ready", out) -> dict:
        if isinstance(out, dict):
            return out
        compressed_once.add(r.req_id)
        return finalize_hook_placement_result(
            req_state=r.req_state, original_block_ids_by_group=r.original_ids, config=config,
            selector_status=str(selector_status), outcome=out, effective_tokens=r.ctx.effective_tokens,
            budget_total=r.ctx.budget_total, recent_unabsorbed_tokens=r.ctx.recent_unabsorbed_tokens)

    def _run_single(r: "_Ready") -> dict:
        setattr(base_runner, "_triattention_active_req_id", r.req_id)
        out = run_group_compaction_pipeline(
            req_id=r.req_id, signal=r.signal, config=config, strict_triton_required=r.strict,
            num_computed_tokens=r.ctx.num_computed_tokens, effective_tokens=r.ctx.effective_tokens,
            budget_total=r.ctx.budget_total, block_size=r.block_size, mutable_block_ids_by_group=r.mutable_ids,
            group_tensors=group_tensors, select_keep_indices=select_layer,
            select_keep_indices_for_group=select_group, shared_compact_fn=compact_request_kv_in_place,
            per_head_compact_fn=compact_request_kv_in_place_per_head, gather_dense_fn=gather_request_k_dense)
        return _finish(r, out)

    def _hook(req_id: str, signal: CompressionSignal, scheduler_output: Any) -> dict:
        ready = _prepare(req_id, signal, scheduler_output)
        if isinstance(ready, dict):
            return ready
        if SINGLE_REQUEST_IN_ONE_CALL and _batchable(ready):
            # Default mode, something to drop: score, select and compact in one library call with one
            # host synchronisation at its end (the layer-by-layer pipeline below waits for the keep
            # indices on the host before the compaction is launched).
            return _run_batch([ready])[req_id]
        return _run_single(ready)

    def _batchable(r: "_Ready") -> bool:
        """True when the one-by-one path would take the group selector and the ordered
        per-head compaction for every KV-cache group of this request, with nothing that only
        that path knows how to do (debug overrides, the keep-everything and prefill early outs)."""
        if compress_batch is None or _debug_env_active():
            return False
        sig = r.signal
        groups = 0
        for gid, ids in enumerate(r.mutable_ids):
            if not ids or not group_tensors.get(gid):
                continue
            total = min(r.ctx.effective_tokens, len(ids) * r.block_size)
            if total <= 0:
                continue
            budget = min(r.ctx.budget_total, total)
            if budget <= 0 or total <= budget:
                return False
            if sig.protect_prefill and config.include_prefill_in_budget and min(int(sig.prefill_len), total) > budget:
                return False
            groups += 1
        return groups > 0

    def _run_batch(batch: list) -> dict:
        """One launch sequence per KV-cache group for all requests of ``batch``."""
        cache_len = {r.req_id: None for r in batch}
        reclaim = {r.req_id: [] for r in batch}
        gids = sorted({gid for r in batch for gid, ids in enumerate(r.mutable_ids) if ids and group_tensors.get(gid)})
        for gid in gids:
            members, requests = [], []
            for r in batch:
                ids = r.mutable_ids[gid] if gid < len(r.mutable_ids) else None
                if not ids:
                    continue
                total = min(r.ctx.effective_tokens, len(ids) * r.block_size)
                if total <= 0:
                    continue
                members.append((r, ids, total))
                requests.append(dict(block_ids=ids, total_tokens=total,
                                     prefill_len=min(int(r.signal.prefill_len), total),
                                     protect_prefill=bool(r.signal.protect_prefill),
                                     round_start=int(max(0, r.ctx.num_computed_tokens)),
                                     budget_total=min(r.ctx.budget_total, total)))
            if not members:
                continue
            try:
                try:
                    selected = compress_batch(layer_kv=group_tensors[gid], block_size=batch[0].block_size,
                                              requests=requests)
                except ResidentLaunchFailed:
                    # The guarded compaction moved nothing of THIS group; groups handled before it
                    # are compacted and truncated already and stay as they are.  Repeat this
                    # group alone on the kernels that do not wait for each other.
                    selected = compress_batch(layer_kv=group_tensors[gid], block_size=batch[0].block_size,
                                              requests=requests, allow_resident=False)
            except Exception as exc:
                raise RuntimeError(f"{MARK}:batch:gid={gid}:global_per_head:{type(exc).__name__}") from exc
            for (r, ids, total), res in zip(members, selected):
                after = int(res["indices"].shape[1])
                if cache_len[r.req_id] is not None and cache_len[r.req_id] != after:
                    raise RuntimeError(f"{MARK}:inconsistent_cache_len_after:req={r.req_id}:gid={gid}:"
                                       f"expected={cache_len[r.req_id]}:actual={after}")
                cache_len[r.req_id] = after
                if config.enable_experimental_block_reclaim:
                    kept, removed, group = truncate_tail_reclaim_group(gid=gid, normalized_block_ids=ids,
                                                                       cache_len_after=after,
                                                                       block_size=r.block_size)
                    if config.require_physical_reclaim:
                        expected = max(0, num_required_blocks(total, r.block_size)
                                       - num_required_blocks(after, r.block_size))
                        if expected > 0 and len(removed) < expected:
                            raise RuntimeError(f"{MARK}:physical_reclaim_missing:req={r.req_id}:gid={gid}:"
                                               f"expected_removed>={expected}:actual_removed={len(removed)}:"
                                               f"effective_tokens={total}:cache_len_after={after}")
                    r.mutable_ids[gid] = list(kept)
                    if group is not None:
                        reclaim[r.req_id].append(group)
        out = {}
        for r in batch:
            # (what the one-by-one path leaves on the runner while it works on a request, hook_impl.py:60)
            setattr(base_runner, "_triattention_active_req_id", r.req_id)
            if cache_len[r.req_id] is None:
                out[r.req_id] = {"applied": False, "reason": "no_compactable_groups"}
                continue
            out[r.req_id] = _finish(r, GroupPipelineOutcome(
                cache_len_after=int(cache_len[r.req_id]), selection_mode="per_head:hf_aligned_global_per_head",
                block_reclaim_groups=reclaim[r.req_id], mutable_block_ids_by_group=r.mutable_ids))
        return out

    def _batch_hook(signals: dict, scheduler_output: Any) -> dict:
        """All triggered requests of a scheduler step at once: ``{req_id: result}`` with the
        result dictionaries the one-by-one hook returns.  Requests that qualify (the default
        per-head mode, something to drop) are scored, selected and compacted together, one
        launch sequence per KV-cache group; the others go through the one-by-one path."""
        results, together = {}, []
        for req_id, signal in signals.items():
            if not getattr(signal, "should_compress", True):
                continue
            ready = _prepare(req_id, signal, scheduler_output)
            if isinstance(ready, dict):
                results[req_id] = ready
            elif _batchable(ready):
                together.append(ready)
            else:
                results[req_id] = _run_single(ready)
        if len(together) == 1 and not SINGLE_REQUEST_IN_ONE_CALL:
            results[together[0].req_id] = _run_single(together[0])
        elif together:
            results.update(_run_batch(together))
        return {req_id: results[req_id] for req_id in signals if req_id in results}

    _hook.batch = _batch_hook
    return _hook


def install_runner_compression_hook(base_runner: Any, config: TriAttentionRuntimeConfig) -> None:
    """Install the hook unless the runner already has one (runtime/hook_impl.py:174-185)."""
    if hasattr(base_runner, "triattention_apply_compression"):
        return
    hook = make_runner_compression_hook(base_runner=base_runner, config=config)
    setattr(base_runner, "triattention_apply_compression", hook)
    setattr(base_runner, RunnerHookCompressionExecutor.batch_hook_name, hook.batch)
