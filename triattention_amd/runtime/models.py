"""Plain data carried between the scheduler, the hook and the layout code.

``CompressionSignal`` (runtime/signals.py:12-26), ``KeepPlan`` / ``ReclaimGroup`` /
``ReclaimEvent`` / ``PlacementPlan`` (runtime/plan_models.py:13-134), per-request
``RequestCompressionState`` with its store (runtime/state.py:9-153) and
``CompressionPlanner`` (runtime/planner.py:9-62): same fields and the same result
dictionaries, since the scheduler side consumes them by key.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Iterable

from .config import TriAttentionRuntimeConfig

TRITON_SCORING_REQUIRED_MARKER = "TRIATTN_FATAL_TRITON_SCORING_REQUIRED"


@dataclass(frozen=True)
class CompressionSignal:
    req_id: str
    should_compress: bool
    reason: str                      # "none" | "length_threshold" | "kv_usage_threshold"
    estimated_cache_len: int
    step: int
    kv_usage: float | None
    protect_prefill: bool
    prefill_len: int
    scheduled_tokens: int = 1


class CompressionPlanner:
    """Length / KV-usage trigger with hysteresis (runtime/planner.py:9-62)."""

    def __init__(self, config: TriAttentionRuntimeConfig) -> None:
        self.config = config
        self._armed = False

    def _usage_triggered(self, kv_usage: float | None) -> bool:
        if not self.config.enable_kv_usage_trigger or kv_usage is None:
            return False
        if kv_usage >= self.config.kv_usage_trigger:
            self._armed = True
        elif kv_usage <= self.config.kv_usage_release:
            self._armed = False
        return self._armed

    def build_signal(self, req_id: str, estimated_cache_len: int, prefill_len: int, step: int,
                     kv_usage: float | None = None, scheduled_tokens: int = 1) -> CompressionSignal:
        threshold = self.config.kv_budget + self.config.divide_length
        if self.config.protect_prefill and not self.config.include_prefill_in_budget:
            threshold += max(prefill_len, 0)
        by_length = estimated_cache_len >= threshold
        by_usage = self._usage_triggered(kv_usage)
        reason = "kv_usage_threshold" if by_usage else ("length_threshold" if by_length else "none")
        return CompressionSignal(req_id=req_id, should_compress=by_length or by_usage, reason=reason,
                                 estimated_cache_len=estimated_cache_len, step=step, kv_usage=kv_usage,
                                 protect_prefill=self.config.protect_prefill, prefill_len=prefill_len,
                                 scheduled_tokens=max(1, int(scheduled_tokens)))


@dataclass(frozen=True)
class KeepPlan:
    """What a selector returned: ``mode`` "shared" (one index list) or "per_head"."""
    mode: str
    indices: Any
    semantic: str | None = None

    @classmethod
    def from_selector_result(cls, result: dict) -> "KeepPlan":
        sem = result.get("semantic")
        return cls(mode=str(result.get("mode", "shared")), indices=result.get("indices"),
                   semantic=None if sem is None else str(sem))

    @property
    def selection_mode_label(self) -> str:
        return f"{self.mode}:{self.semantic}" if self.semantic else self.mode

    def keep_count(self) -> int:
        idx = self.indices
        if self.mode == "per_head":
            if hasattr(idx, "ndim") and hasattr(idx, "shape"):
                if int(idx.ndim) != 2:
                    raise ValueError(f"per_head indices tensor must be 2D, got ndim={idx.ndim}")
                return int(idx.shape[1])
            if isinstance(idx, list):
                return len(idx[0]) if idx and isinstance(idx[0], list) else 0
            raise ValueError(f"unsupported per_head indices type: {type(idx).__name__}")
        if hasattr(idx, "numel"):
            return int(idx.numel())
        if isinstance(idx, list):
            return len(idx)
        raise ValueError(f"unsupported shared indices type: {type(idx).__name__}")

    def to_selector_result(self) -> dict:
        out = {"mode": self.mode, "indices": self.indices}
        if self.semantic is not None:
            out["semantic"] = self.semantic
        return out


@dataclass(frozen=True)
class ReclaimGroup:
    gid: int
    block_ids_before: list
    block_ids_after: list
    block_ids_removed: list

    def to_dict(self) -> dict:
        return {"gid": self.gid, "block_ids_before": list(self.block_ids_before),
                "block_ids_after": list(self.block_ids_after),
                "block_ids_removed": list(self.block_ids_removed)}


@dataclass(frozen=True)
class ReclaimEvent:
    mode: str
    groups: list

    def reclaimed_block_count(self) -> int:
        return sum(len(g.block_ids_removed) for g in self.groups)

    def to_dict(self) -> dict:
        return {"mode": self.mode, "groups": [g.to_dict() for g in self.groups]}


@dataclass(frozen=True)
class PlacementPlan:
    cache_len_after: int
    selector_status: str
    selection_mode: str
    effective_tokens_before: int
    budget_total: int
    recent_unabsorbed_tokens: int | None
    block_reclaim: ReclaimEvent | None = None

    @property
    def reclaimed_block_count(self) -> int:
        return 0 if self.block_reclaim is None else self.block_reclaim.reclaimed_block_count()

    def to_hook_result_dict(self) -> dict:
        return {
            "applied": True,
            "reason": f"kv_compacted:{self.selection_mode}",
            "cache_len_after": self.cache_len_after,
            "selector_status": self.selector_status,
            "block_reclaim": None if self.block_reclaim is None else self.block_reclaim.to_dict(),
            "effective_tokens_before": self.effective_tokens_before,
            "budget_total": self.budget_total,
            "reclaimed_block_count": self.reclaimed_block_count,
            "recent_unabsorbed_tokens": self.recent_unabsorbed_tokens,
        }


@dataclass
class RequestCompressionState:
    req_id: str
    prefill_len: int
    protect_prefill: bool
    current_cache_len: int = 0
    last_absorbed_cache_len: int = 0
    recent_unabsorbed_tokens: int = 0
    compression_count: int = 0
    last_compression_step: int = -1
    pending_triggers: int = 0
    last_trigger_reason: str = "none"
    is_preempted: bool = False
    current_cache_len_semantics: str = "unknown"
    current_cache_len_step: int = -1
    nct_at_last_compression: int | None = None
    cache_len_after_last_compression: int | None = None

    @property
    def mode(self) -> str:
        return "protect_prefill" if self.protect_prefill else "trim_prefill"


class RequestStateStore:
    """Per-request bookkeeping keyed by req_id (runtime/state.py:38-153)."""

    def __init__(self) -> None:
        self._states: dict[str, RequestCompressionState] = {}
        self._compressed: set[str] = set()

    def ensure(self, req_id: str, prefill_len: int, protect_prefill: bool) -> RequestCompressionState:
        st = self._states.get(req_id)
        if st is None:
            st = RequestCompressionState(req_id=req_id, prefill_len=prefill_len, protect_prefill=protect_prefill,
                                         last_absorbed_cache_len=max(0, prefill_len))
            self._states[req_id] = st
            return st
        st.prefill_len = max(st.prefill_len, prefill_len)
        st.protect_prefill = protect_prefill
        if st.compression_count <= 0:
            st.last_absorbed_cache_len = max(st.last_absorbed_cache_len, st.prefill_len)
        return st

    def get(self, req_id: str):
        return self._states.get(req_id)

    def remove(self, req_id: str) -> None:
        self._states.pop(req_id, None)
        self._compressed.discard(req_id)

    def snapshot(self) -> dict:
        return dict(self._states)

    def mark_preempted(self, req_id: str) -> None:
        if req_id in self._states:
            self._states[req_id].is_preempted = True

    def mark_resumed(self, req_id: str) -> None:
        if req_id in self._states:
            self._states[req_id].is_preempted = False

    def update_cache_len(self, req_id: str, cache_len: int, step: int | None = None) -> None:
        st = self._states.get(req_id)
        if st is None:
            return
        st.current_cache_len = max(0, int(cache_len))
        st.current_cache_len_semantics = "estimated_with_scheduled"
        if isinstance(step, int):
            st.current_cache_len_step = step
        st.recent_unabsorbed_tokens = max(0, st.current_cache_len - max(0, int(st.last_absorbed_cache_len)))

    def mark_trigger(self, req_id: str, reason: str, step: int) -> None:
        st = self._states.get(req_id)
        if st is not None:
            st.pending_triggers += 1
            st.last_trigger_reason = reason

    def mark_compressed(self, req_id: str, step: int, cache_len: int, scheduled_tokens: int = 0,
                        scheduler_nct: int | None = None) -> None:
        st = self._states.get(req_id)
        if st is None:
            return
        self._compressed.add(req_id)
        st.compression_count += 1
        st.pending_triggers = max(st.pending_triggers - 1, 0)
        st.last_compression_step = step
        st.current_cache_len = cache_len + max(0, scheduled_tokens)
        st.current_cache_len_semantics = "estimated_with_scheduled"
        st.current_cache_len_step = int(step)
        st.last_absorbed_cache_len = max(0, int(cache_len))
        st.recent_unabsorbed_tokens = 0
        st.last_trigger_reason = "applied"
        st.cache_len_after_last_compression = int(cache_len)
        if scheduler_nct is not None:
            st.nct_at_last_compression = int(scheduler_nct)

    def mark_compression_skipped(self, req_id: str, reason: str, step: int) -> None:
        st = self._states.get(req_id)
        if st is not None:
            st.pending_triggers = max(st.pending_triggers - 1, 0)
            st.last_trigger_reason = f"skipped:{reason}"

    def has_active_compressed_requests(self) -> bool:
        return bool(self._compressed)

    def has_compressed_request_in(self, req_ids: Iterable[str]) -> bool:
        return any(r in self._compressed for r in req_ids)
