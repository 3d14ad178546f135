"""Per-request compaction pipeline: selection -> in-place compaction of every layer of a
KV-cache group -> tail-block truncation.

Covers the reference's ``selection_planner.py`` (prepare_group_layer_compactions),
``layout_engine.py`` (compact_layer_with_keep_plan, execute_group_compaction,
truncate_tail_reclaim_group) and ``hook_group_pipeline.py`` (run_group_compaction_pipeline,
finalize_hook_placement_result): same inputs, outcome objects, result dictionaries and
error strings.  Where the reference loops over layers and calls one compaction per
layer, a group whose layers share one keep plan is compacted by a single kernel launch
over all layers.

Only the kept prefix is written (slots ``0..k-1`` in ascending token order): the
reference rewrites all T slots as ``[kept..., dropped...]`` (layout_engine.py:71-80)
but slots >= k are never read again once the effective length is k.  Setting
``TRIATTN_DEBUG_FORCE_PRESERVE_DROPPED=1`` restores the full permutation.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from pathlib import Path
from typing import Any, Callable

import torch

from .config import TriAttentionRuntimeConfig
from .kv_compaction import (build_keep_token_indices, compact_request_kv_in_place,
                            compact_request_kv_in_place_per_head)
from .models import (TRITON_SCORING_REQUIRED_MARKER as MARK, CompressionSignal, KeepPlan, PlacementPlan,
                     ReclaimEvent, ReclaimGroup)

_ON = {"1", "true", "yes", "on"}


def _env_on(name: str) -> bool:
    return os.environ.get(name, "0").strip().lower() in _ON


def num_required_blocks(total_tokens: int, block_size: int) -> int:
    """layout_engine.py:25-28."""
    return 0 if total_tokens <= 0 else (total_tokens + block_size - 1) // block_size


def truncate_tail_reclaim_group(*, gid: int, normalized_block_ids: list, cache_len_after: int, block_size: int):
    """Keep the first ceil(k / block_size) ids, report the rest (layout_engine.py:209-227)."""
    n = num_required_blocks(cache_len_after, block_size)
    kept, removed = list(normalized_block_ids[:n]), list(normalized_block_ids[n:])
    group = ReclaimGroup(gid=gid, block_ids_before=list(normalized_block_ids), block_ids_after=kept,
                         block_ids_removed=removed) if removed else None
    return kept, removed, group


def count_reclaimed_blocks(groups: list) -> int:
    return sum(len(g.block_ids_removed) for g in groups)


@dataclass(frozen=True)
class LayerCompactionResult:
    cache_len_after: int
    keep_count: int
    before_required_blocks: int
    after_required_blocks: int
    preserve_dropped_tokens: bool


@dataclass(frozen=True)
class PreparedLayerCompaction:
    layer_idx: int
    kv_cache: torch.Tensor
    block_ids: Any
    keep_plan: KeepPlan


@dataclass(frozen=True)
class PreparedGroupSelection:
    tasks: list
    selection_mode: str
    shared_plan: bool = False     # every task carries the same KeepPlan object


@dataclass(frozen=True)
class GroupCompactionOutcome:
    layer_results: list
    cache_len_after: int | None
    kept_block_ids: list
    removed_block_ids: list
    reclaim_group: ReclaimGroup | None


@dataclass(frozen=True)
class GroupPipelineOutcome:
    cache_len_after: int
    selection_mode: str
    block_reclaim_groups: list
    mutable_block_ids_by_group: list


def normalize_mutable_block_ids_by_group(original):
    """hook_group_pipeline.py:26-39."""
    if not original or not isinstance(original, (list, tuple)):
        return None
    return [[int(b) for b in g] if isinstance(g, (list, tuple)) else None for g in original]


_override_state = {"used": False, "tensor": None}


def _maybe_override_first_keep(plan: KeepPlan, round_start: int, total_tokens: int) -> KeepPlan:
    """TRIATTN_DEBUG_OVERRIDE_FIRST_KEEP_JSON: replace the first per-head keep set of a
    fresh request by indices read from a file (selection_planner.py:36-91)."""
    path = os.environ.get("TRIATTN_DEBUG_OVERRIDE_FIRST_KEEP_JSON", "").strip()
    if not path or _override_state["used"] or plan.mode != "per_head" or int(round_start) != int(total_tokens):
        return plan
    if _override_state["tensor"] is None:
        payload = json.loads(Path(path).read_text(encoding="utf-8"))
        t = torch.as_tensor(payload.get("indices") if isinstance(payload, dict) else payload, dtype=torch.long)
        if t.ndim != 2:
            raise RuntimeError(f"override_keep_ndim_{int(t.ndim)}")
        _override_state["tensor"] = t.contiguous()
    cur = plan.indices if isinstance(plan.indices, torch.Tensor) else torch.as_tensor(plan.indices, dtype=torch.long)
    ov = _override_state["tensor"]
    if tuple(cur.shape) != tuple(ov.shape):
        raise RuntimeError(f"override_keep_shape_mismatch:current={tuple(cur.shape)}:override={tuple(ov.shape)}")
    _override_state["used"] = True
    new = ov.to(cur.device) if isinstance(plan.indices, torch.Tensor) else ov.tolist()
    return KeepPlan(mode=plan.mode, indices=new, semantic=plan.semantic)


def prepare_group_layer_compactions(*, req_id: str, gid: int, layer_tensors: list, normalized_block_ids: list,
                                    block_size: int, group_total_tokens: int, group_prefill_len: int,
                                    protect_prefill: bool, round_start: int, group_budget_total: int,
                                    config: TriAttentionRuntimeConfig, strict_triton_required: bool,
                                    select_keep_indices: Callable | None,
                                    select_keep_indices_for_group: Callable | None,
                                    gather_dense_fn: Callable | None = None) -> PreparedGroupSelection:
    """Selector output -> one task per layer (selection_planner.py:94-275)."""
    group_result = None
    use_group = (select_keep_indices_for_group is not None and config.pruning_mode == "per_head"
                 and config.per_head_selection_semantics == "hf_aligned_global_per_head"
                 and not _env_on("TRIATTN_RUNTIME_DEBUG_DISABLE_GROUP_SELECTOR"))
    if use_group:
        try:
            paged = getattr(select_keep_indices_for_group, "_supports_paged_group", False)
            if strict_triton_required and not paged:
                raise RuntimeError("paged_group_selector_required")
            common = dict(total_tokens=group_total_tokens, prefill_len=group_prefill_len,
                          protect_prefill=protect_prefill, round_start=round_start,
                          budget_total=group_budget_total)
            if paged:
                group_result = select_keep_indices_for_group(
                    layer_inputs=None, layer_input_iter=None,
                    layer_kv_iter=lambda: [(li, kv, normalized_block_ids, block_size) for li, kv in layer_tensors],
                    **common)
            else:
                from .kv_compaction import gather_request_k_dense
                gather = gather_dense_fn or gather_request_k_dense
                group_result = select_keep_indices_for_group(
                    layer_inputs=None, layer_kv_iter=None,
                    layer_input_iter=lambda: [(li, gather(kv_cache=kv, block_ids=normalized_block_ids,
                                                          block_size=block_size, total_tokens=group_total_tokens))
                                              for li, kv in layer_tensors],
                    **common)
        except Exception as exc:
            raise RuntimeError(f"{MARK}:req={req_id}:gid={gid}:global_per_head:{type(exc).__name__}") from exc

    tasks, mode_label = [], "fallback"
    shared_plan_obj = None
    for layer_idx, kv_cache in layer_tensors:
        selected = group_result
        if selected is None and select_keep_indices is not None:
            try:
                paged = getattr(select_keep_indices, "_supports_paged", False)
                if strict_triton_required and not paged:
                    raise RuntimeError("paged_selector_required")
                common = dict(total_tokens=group_total_tokens, prefill_len=group_prefill_len,
                              protect_prefill=protect_prefill, layer_idx=layer_idx, round_start=round_start,
                              budget_total=group_budget_total)
                if paged:
                    selected = select_keep_indices(keys_dense=None, kv_cache=kv_cache,
                                                   block_ids=normalized_block_ids, block_size=block_size, **common)
                else:
                    from .kv_compaction import gather_request_k_dense
                    gather = gather_dense_fn or gather_request_k_dense
                    selected = select_keep_indices(
                        keys_dense=gather(kv_cache=kv_cache, block_ids=normalized_block_ids,
                                          block_size=block_size, total_tokens=group_total_tokens), **common)
            except Exception as exc:
                raise RuntimeError(f"{MARK}:req={req_id}:gid={gid}:layer={layer_idx}:{type(exc).__name__}") from exc
        from_fallback = False
        if selected is None:
            keep = build_keep_token_indices(total_tokens=group_total_tokens, kv_budget=config.kv_budget,
                                            prefill_len=group_prefill_len, protect_prefill=protect_prefill,
                                            include_prefill_in_budget=config.include_prefill_in_budget)
            if keep is None:
                raise ValueError("prefill_exceeds_budget")
            if strict_triton_required:
                raise RuntimeError(f"{MARK}:selector_returned_none:req={req_id}:gid={gid}:layer={layer_idx}")
            selected = {"mode": "shared", "indices": keep}
            from_fallback = True
        if selected is group_result and shared_plan_obj is not None:
            plan = shared_plan_obj
        else:
            plan = _maybe_override_first_keep(KeepPlan.from_selector_result(selected), round_start,
                                              group_total_tokens)
            if selected is group_result:
                shared_plan_obj = plan
        mode_label = "fallback" if from_fallback else plan.selection_mode_label
        tasks.append(PreparedLayerCompaction(layer_idx=layer_idx, kv_cache=kv_cache,
                                             block_ids=normalized_block_ids, keep_plan=plan))
    return PreparedGroupSelection(tasks=tasks, selection_mode=str(mode_label),
                                  shared_plan=group_result is not None and len(tasks) > 0)


def compact_layer_with_keep_plan(*, kv_cache, block_ids, block_size: int, keep_plan: KeepPlan, total_tokens: int,
                                 enable_experimental_block_reclaim: bool, shared_compact_fn: Callable | None = None,
                                 per_head_compact_fn: Callable | None = None) -> LayerCompactionResult:
    """Compact one layer (or, given a list of caches, several layers at once) with one
    keep plan (layout_engine.py:57-109)."""
    keep_count = keep_plan.keep_count()
    preserve = _env_on("TRIATTN_DEBUG_FORCE_PRESERVE_DROPPED")
    if keep_plan.mode == "per_head":
        fn = per_head_compact_fn or compact_request_kv_in_place_per_head
        after = fn(kv_cache=kv_cache, block_ids=block_ids, block_size=block_size,
                   keep_token_indices_per_head=keep_plan.indices, total_tokens=total_tokens,
                   preserve_dropped_tokens=preserve)
    else:
        fn = shared_compact_fn or compact_request_kv_in_place
        after = fn(kv_cache=kv_cache, block_ids=block_ids, block_size=block_size,
                   keep_token_indices=keep_plan.indices, total_tokens=total_tokens,
                   preserve_dropped_tokens=preserve)
    return LayerCompactionResult(cache_len_after=int(after), keep_count=int(keep_count),
                                 before_required_blocks=num_required_blocks(total_tokens, block_size),
                                 after_required_blocks=num_required_blocks(keep_count, block_size),
                                 preserve_dropped_tokens=bool(preserve))


def execute_group_compaction(*, req_id: str, gid: int, normalized_block_ids: list, tasks: list, block_size: int,
                             total_tokens: int, enable_experimental_block_reclaim: bool,
                             require_physical_reclaim: bool, shared_compact_fn: Callable | None = None,
                             per_head_compact_fn: Callable | None = None,
                             shared_plan: bool = False) -> GroupCompactionOutcome:
    """Compaction and reclaim derivation for one KV-cache group (layout_engine.py:141-206)."""
    results = []
    native = shared_compact_fn in (None, compact_request_kv_in_place) and \
        per_head_compact_fn in (None, compact_request_kv_in_place_per_head)
    if shared_plan and native and len(tasks) > 1:
        res = compact_layer_with_keep_plan(kv_cache=[t.kv_cache for t in tasks], block_ids=normalized_block_ids,
                                           block_size=block_size, keep_plan=tasks[0].keep_plan,
                                           total_tokens=total_tokens,
                                           enable_experimental_block_reclaim=enable_experimental_block_reclaim)
        results = [(t.layer_idx, res) for t in tasks]
    else:
        for t in tasks:
            results.append((t.layer_idx, compact_layer_with_keep_plan(
                kv_cache=t.kv_cache, block_ids=t.block_ids, block_size=block_size, keep_plan=t.keep_plan,
                total_tokens=total_tokens, enable_experimental_block_reclaim=enable_experimental_block_reclaim,
                shared_compact_fn=shared_compact_fn, per_head_compact_fn=per_head_compact_fn)))
    after = None
    for layer_idx, res in results:
        if after is not None and res.cache_len_after != after:
            raise RuntimeError(f"{MARK}:inconsistent_cache_len_after:req={req_id}:gid={gid}:layer={layer_idx}:"
                               f"expected={after}:actual={res.cache_len_after}")
        after = int(res.cache_len_after)
    kept, removed, group = list(normalized_block_ids), [], None
    if enable_experimental_block_reclaim and after is not None:
        kept, removed, group = truncate_tail_reclaim_group(gid=gid, normalized_block_ids=normalized_block_ids,
                                                           cache_len_after=after, block_size=block_size)
        if require_physical_reclaim:
            expected = max(0, num_required_blocks(total_tokens, block_size) - num_required_blocks(after, block_size))
            if expected > 0 and len(removed) < expected:
                raise RuntimeError(f"{MARK}:physical_reclaim_missing:req={req_id}:gid={gid}:"
                                   f"expected_removed>={expected}:actual_removed={len(removed)}:"
                                   f"effective_tokens={total_tokens}:cache_len_after={after}")
    return GroupCompactionOutcome(layer_results=results, cache_len_after=after, kept_block_ids=kept,
                                  removed_block_ids=removed, reclaim_group=group)


def run_group_compaction_pipeline(*, req_id: str, signal: CompressionSignal, config: TriAttentionRuntimeConfig,
                                  strict_triton_required: bool, num_computed_tokens: int, effective_tokens: int,
                                  budget_total: int, block_size: int, mutable_block_ids_by_group: list,
                                  group_tensors: dict, select_keep_indices: Callable | None,
                                  select_keep_indices_for_group: Callable | None,
                                  shared_compact_fn: Callable | None = None,
                                  per_head_compact_fn: Callable | None = None,
                                  gather_dense_fn: Callable | None = None):
    """hook_group_pipeline.py:42-155."""
    after_all, mode_label, reclaim_groups = None, "fallback", []
    for gid, block_ids in enumerate(mutable_block_ids_by_group):
        layers = group_tensors.get(gid)
        if not block_ids or not layers:
            continue
        total = min(effective_tokens, len(block_ids) * block_size)
        if total <= 0:
            continue
        try:
            sel = prepare_group_layer_compactions(
                req_id=req_id, gid=gid, layer_tensors=layers, normalized_block_ids=block_ids,
                block_size=block_size, group_total_tokens=total,
                group_prefill_len=min(int(signal.prefill_len), total), protect_prefill=signal.protect_prefill,
                round_start=int(max(0, num_computed_tokens)), group_budget_total=min(budget_total, total),
                config=config, strict_triton_required=strict_triton_required,
                select_keep_indices=select_keep_indices,
                select_keep_indices_for_group=select_keep_indices_for_group, gather_dense_fn=gather_dense_fn)
        except ValueError as exc:
            if str(exc) == "prefill_exceeds_budget":
                return {"applied": False, "reason": "prefill_exceeds_budget"}
            raise
        mode_label = sel.selection_mode
        try:
            outcome = execute_group_compaction(
                req_id=req_id, gid=gid, normalized_block_ids=block_ids, tasks=sel.tasks, block_size=block_size,
                total_tokens=total, enable_experimental_block_reclaim=config.enable_experimental_block_reclaim,
                require_physical_reclaim=config.require_physical_reclaim, shared_compact_fn=shared_compact_fn,
                per_head_compact_fn=per_head_compact_fn, shared_plan=sel.shared_plan)
        except Exception as exc:
            first = sel.tasks[0].layer_idx if sel.tasks else -1
            return {"applied": False, "reason": f"compaction_failed:g{gid}:l{first}:{type(exc).__name__}"}
        if outcome.cache_len_after is None:
            continue
        if after_all is not None and outcome.cache_len_after != after_all:
            raise RuntimeError(f"{MARK}:inconsistent_cache_len_after:req={req_id}:gid={gid}:"
                               f"layer={outcome.layer_results[0][0]}:expected={after_all}:"
                               f"actual={outcome.cache_len_after}")
        after_all = int(outcome.cache_len_after)
        if config.enable_experimental_block_reclaim:
            mutable_block_ids_by_group[gid] = list(outcome.kept_block_ids)
            if outcome.reclaim_group is not None:
                reclaim_groups.append(outcome.reclaim_group)
    if after_all is None:
        return {"applied": False, "reason": "no_compactable_groups"}
    return GroupPipelineOutcome(cache_len_after=after_all, selection_mode=str(mode_label),
                                block_reclaim_groups=reclaim_groups,
                                mutable_block_ids_by_group=mutable_block_ids_by_group)


def finalize_hook_placement_result(*, req_state: Any, original_block_ids_by_group: Any,
                                   config: TriAttentionRuntimeConfig, selector_status: str,
                                   outcome: GroupPipelineOutcome, effective_tokens: int, budget_total: int,
                                   recent_unabsorbed_tokens: int | None) -> dict:
    """Write the truncated block lists back and build the hook's result dictionary
    (hook_group_pipeline.py:158-200)."""
    event = None
    if config.enable_experimental_block_reclaim and outcome.block_reclaim_groups:
        new_ids = [original_block_ids_by_group[i] if g is None else g
                   for i, g in enumerate(outcome.mutable_block_ids_by_group)]
        req_state.block_ids = tuple(new_ids) if isinstance(original_block_ids_by_group, tuple) else new_ids
        event = ReclaimEvent(mode="truncate_tail", groups=outcome.block_reclaim_groups)
    return PlacementPlan(cache_len_after=int(outcome.cache_len_after), selector_status=str(selector_status),
                         selection_mode=str(outcome.selection_mode), effective_tokens_before=int(effective_tokens),
                         budget_total=int(budget_total),
                         recent_unabsorbed_tokens=(int(recent_unabsorbed_tokens)
                                                   if isinstance(recent_unabsorbed_tokens, int) else None),
                         block_reclaim=event).to_hook_result_dict()
