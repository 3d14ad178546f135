"""Keep-set selection for the runtime hook: the callable pair the reference builds in
``build_triattention_selector`` (triattention/vllm/runtime/selector_hf.py:15-1083), same
keyword signatures, result dictionaries and failure markers, executed by the HIP scorer,
the combine kernel and the radix top-k.

Nothing is chunked and K is neither gathered nor repeated per query head: the scorer
reads the paged blocks of every layer once and, for shapes that have a resident kernel,
keeps the raw scores on chip (``ops.select_paged``).  Ties at the budget keep the lowest token
index (the reference's ``torch.topk`` leaves them undefined).
"""
from __future__ import annotations

import os
from pathlib import Path
from typing import Any, Callable, Iterable

import torch

from .. import ops
from ..core import stats as stats_mod
from .config import TriAttentionRuntimeConfig
from .kv_compaction import kv_axis_hint, mark_keep_validated
from .models import TRITON_SCORING_REQUIRED_MARKER as MARK


class _DeviceStats:
    """Statistics of one stats file resident on one device, folded once per head layout."""

    def __init__(self, config: TriAttentionRuntimeConfig, stats_path: Path, model_path):
        self.config = config
        self.metadata, self.head_stats = stats_mod.load_frequency_stats(
            stats_path, device="cpu", dtype=torch.float32, num_kv_heads=None, model_path=model_path)
        if not self.head_stats:
            raise RuntimeError("empty_head_stats")
        self.layers = tuple(sorted(self.head_stats.keys()))
        self.head_dim = int(self.metadata["head_dim"])
        self.rope_style = str(self.metadata.get("rope_style", "half"))
        self.inv_freq = stats_mod.resolve_inv_freq(self.metadata, self.head_dim, model_path)
        self.offsets = stats_mod.geometric_offsets(65536)
        self.stats_heads = int(self.head_stats[self.layers[0]]["freq_scale_sq"].shape[0])
        self._folded: dict = {}
        self._vectors: dict = {}

    def resolve_layer(self, layer_idx: int) -> int:
        """Layer index modulo the layers the file has (selector_hf.py:132-143)."""
        if layer_idx in self.head_stats:
            return layer_idx
        return self.layers[layer_idx % len(self.layers)]

    def vectors(self, device):
        v = self._vectors.get(device)
        if v is None:
            v = (self.inv_freq.to(device).contiguous(), self.offsets.to(device).contiguous())
            self._vectors[device] = v
        return v

    def folded(self, layer_ids: tuple, score_heads: int, device) -> torch.Tensor:
        """[L, score_heads, 3, F] for the given runtime layers; heads mean-pooled when the
        caller scores fewer heads than the file holds (selector_hf.py:147-203)."""
        key = (layer_ids, score_heads, str(device))
        hit = self._folded.get(key)
        if hit is not None:
            return hit
        qc, qa, fs = [], [], []
        for layer in layer_ids:
            entry = self.head_stats[self.resolve_layer(layer)]
            if "q_mean_complex" not in entry:
                raise RuntimeError("stats file has no q_mean_real/q_mean_imag entries")
            qc.append(stats_mod.pool_heads(entry["q_mean_complex"], score_heads))
            qa.append(stats_mod.pool_heads(entry["q_abs_mean"], score_heads))
            fs.append(stats_mod.pool_heads(entry["freq_scale_sq"], score_heads))
        out = ops.fold_stats(torch.stack(qc).to(device), torch.stack(qa).to(device), torch.stack(fs).to(device),
                             disable_mlr=self.config.disable_mlr, disable_trig=self.config.disable_trig)
        self._folded[key] = out
        return out


# Steady-state steps (a shape seen before) replay their launch sequence from a HIP graph.
GRAPH_REPLAY = True
# ... for steps whose scratch stays below this many bytes: every captured shape keeps scratch and keep
# rows of its own, and the steps that repeat are the small ones (budget + divide_length tokens a
# request).  A selector keeps at most GRAPH_MAX_SHAPES captured shapes and at most
# GRAPH_MAX_TOTAL_BYTES of their scratch, the least recently replayed one goes first; shapes seen once
# are only remembered by their key (GRAPH_MAX_SEEN of them), so one-off batches never push a captured
# shape out.
GRAPH_MAX_SCRATCH_BYTES = 64 << 20
GRAPH_MAX_SHAPES = 8
GRAPH_MAX_TOTAL_BYTES = 256 << 20
GRAPH_MAX_SEEN = 64
GRAPH_COUNTS = {"captured": 0, "replayed": 0}     # process-wide, for tests and diagnostics


class ResidentLaunchFailed(RuntimeError):
    """The resident kernel gave up waiting for its other workgroups (the GPU was shared with
    another workload for seconds); nothing was compacted, the step can be repeated."""


def build_triattention_selector(config: TriAttentionRuntimeConfig, base_runner: Any | None = None):
    """(select_keep_indices, select_keep_indices_for_group, status)."""
    mode = config.pruning_mode
    if mode == "per_layer" and not bool(getattr(config, "allow_per_layer_mode", False)):
        raise RuntimeError(f"{MARK}:per_layer_mode_disabled:set allow_per_layer_mode=True for explicit opt-in")
    strict = bool(config.enable_experimental_kv_compaction and config.require_triton_scoring)

    def _unavailable(reason: str):
        if strict:
            raise RuntimeError(f"{MARK}:{reason}")
        return None, None, reason

    if config.sparse_stats_path is None:
        return _unavailable("stats_path_not_set")
    stats_path = Path(config.sparse_stats_path).expanduser()
    if not stats_path.exists():
        return _unavailable("stats_path_not_found")
    if mode not in {"per_layer", "per_head", "per_layer_per_head"}:
        return _unavailable(f"unsupported_pruning_mode:{mode}")
    try:
        from .. import _lib
        _lib.load()
    except Exception as exc:
        raise RuntimeError(f"{MARK}:import_failed:{type(exc).__name__}") from exc

    semantics = config.per_head_selection_semantics
    model_path = getattr(config, "model_path", None)
    if model_path is None and base_runner is not None:
        for owner in (getattr(base_runner, "model_config", None),
                      getattr(getattr(base_runner, "vllm_config", None), "model_config", None)):
            cand = getattr(owner, "model", None)
            if isinstance(cand, Path) or (isinstance(cand, str) and cand.strip()):
                model_path = Path(cand)
                break

    holder: dict = {}

    def _stats() -> _DeviceStats:
        if "s" not in holder:
            holder["s"] = _DeviceStats(config, stats_path, model_path)
        return holder["s"]

    def _recent_count(total_tokens: int) -> int:
        if total_tokens <= 0 or config.window_size <= 0:
            return 0
        return min(config.window_size, total_tokens)

    def _head_layout(runtime_heads: int):
        """(heads scored per layer, group reduce): all file heads with a max (or the
        configured per-layer reduce) when the file is per query head, else stats pooled
        down to the runtime heads (selector_hf.py:242-297)."""
        st = _stats()
        group_max = st.stats_heads != runtime_heads and (
            (mode == "per_head" and semantics == "hf_aligned_global_per_head") or mode == "per_layer_per_head")
        if group_max:
            if runtime_heads <= 0 or st.stats_heads % runtime_heads:
                raise RuntimeError(f"{MARK}:incompatible_head_mapping:source={st.stats_heads},target={runtime_heads}")
            return st.stats_heads, (config.layer_perhead_aggregation if mode == "per_layer_per_head" else "max")
        return runtime_heads, "max"

    def _paged_kv(caches):
        hints = {kv_axis_hint(c) for c in caches}
        return ops.PagedKV.for_kv_caches(caches, rope_style=_stats().rope_style,
                                          kv_axis=hints.pop() if len(hints) == 1 else None)

    def _resident_failed(status: int) -> bool:
        """Book-keeping after a resident launch.  An expired wait (1) means the launch was starved
        of CUs (a shared or masked GPU): that is still so at the next step and every such launch costs
        its full wait limit, so the selector stays on the two-pass kernels from then on.  A value
        outside fp16's range (2) ends a launch at once; it may be this model's statistics (every
        step) or one odd key (this step), so the selector gives up on the resident kernels after
        three such steps in a row.  A disagreement between host and device lengths (3) concerns one
        step."""
        if status == 0:
            holder["range_failures"] = 0
            return False
        if status == 1:
            holder["resident_ok"] = False
        elif status == 2:
            holder["range_failures"] = holder.get("range_failures", 0) + 1
            if holder["range_failures"] >= 3:
                holder["resident_ok"] = False
        return True

    def _score_and_select(kv: ops.PagedKV, layer_ids: tuple, block_ids, total_tokens: int, prefill_len: int,
                          protect_prefill: bool, round_start: int, k: int, layer_reduce, group_reduce: str,
                          score_heads: int, shared: bool, allow_resident: bool = True) -> torch.Tensor:
        st = _stats()
        omega, offsets = st.vectors(kv.device)
        sc = ops.ScoreConfig(st.folded(layer_ids, score_heads, kv.device), omega, offsets,
                             config.sparse_score_aggregation)
        if block_ids is None:
            batch = ops.StepBatch(kv.device, [total_tokens], round_start=[round_start], budgets=[k],
                                  prefill_lens=[prefill_len])
        else:
            ids = block_ids.flatten().tolist() if isinstance(block_ids, torch.Tensor) else block_ids
            batch = ops.StepBatch.for_request(kv.device, total_tokens, ids, round_start=int(round_start), budget=int(k),
                                              prefill_len=int(prefill_len))
        sel = ops.SelectConfig(normalize=config.sparse_normalize_scores, window_size=config.window_size,
                               protect_prefill=bool(protect_prefill and prefill_len > 0),
                               group_reduce=group_reduce, layer_reduce=layer_reduce, shared=shared,
                               allow_resident=allow_resident and holder.get("resident_ok", True))
        try:
            resident = ops.select_path(kv, batch, sc, sel) != "two_pass"
            keep, _, ws = ops.select_paged(kv, batch, sc, sel)
            if resident and _resident_failed(ws.status()):
                # The keep lists mean nothing.  Nothing has been moved yet; score again on the
                # kernels that do not wait for each other.
                sel.allow_resident = False
                keep, _, ws = ops.select_paged(kv, batch, sc, sel, ws)
        except Exception as exc:
            raise RuntimeError(f"{MARK}:score_failed:{type(exc).__name__}") from exc
        return mark_keep_validated(keep.to(torch.long), total_tokens)

    def _select_keep_indices(*, keys_dense: torch.Tensor | None = None, kv_cache: torch.Tensor | None = None,
                             block_ids=None, block_size: int | None = None, total_tokens: int, prefill_len: int,
                             protect_prefill: bool, layer_idx: int, round_start: int, budget_total: int):
        """One layer (selector_hf.py:679-747, paged streaming :473-677)."""
        if total_tokens <= budget_total:
            return {"mode": "shared", "indices": list(range(total_tokens))}
        if protect_prefill and config.include_prefill_in_budget and prefill_len > budget_total:
            return None
        if keys_dense is not None:
            if keys_dense.shape[0] != 1:
                raise RuntimeError("selector expects keys_dense of shape [1, H, T, D]")
            kv = ops.PagedKV.from_dense_keys(keys_dense[..., :total_tokens, :], rope_style=_stats().rope_style)
            tables = None
        elif kv_cache is not None and block_ids is not None and block_size is not None:
            kv = _paged_kv([kv_cache])
            tables = block_ids
        else:
            raise RuntimeError("missing scoring inputs for selector")
        k = min(int(budget_total), int(total_tokens))
        if k <= 0:
            return {"mode": "shared", "indices": []}
        score_heads, group_reduce = _head_layout(kv.num_kv_heads)
        per_head = mode in {"per_head", "per_layer_per_head"}
        # One call per layer and request: on the resident kernel every one of them would end in a read
        # of the status word, where the two-pass launches queue up behind each other unwatched (one
        # request of 2176 tokens x 36 layers through the hook: 15 % slower on the resident kernel).
        keep = _score_and_select(kv, (int(layer_idx),), tables, total_tokens, prefill_len, protect_prefill,
                                 round_start, k, None, group_reduce, score_heads, shared=not per_head,
                                 allow_resident=False)
        if per_head:
            return {"mode": "per_head", "indices": keep.contiguous()}
        return {"mode": "shared", "indices": keep[0].contiguous()}

    def _select_keep_indices_for_group_per_head(*, layer_inputs=None,
                                                layer_input_iter: Callable[[], Iterable] | None = None,
                                                layer_kv_iter: Callable[[], Iterable] | None = None,
                                                total_tokens: int, prefill_len: int, protect_prefill: bool,
                                                round_start: int, budget_total: int):
        """One keep set for every layer of a KV-cache group (selector_hf.py:749-1079)."""
        if mode != "per_head" or semantics != "hf_aligned_global_per_head":
            return None
        if layer_kv_iter is not None:
            entries = list(layer_kv_iter())
            paged = True
        else:
            entries = list(layer_input_iter()) if layer_input_iter is not None else list(layer_inputs or [])
            paged = False
        if total_tokens <= budget_total:
            if not entries:
                return {"mode": "per_head", "indices": []}
            first = entries[0][1]
            heads = int(first.shape[3] if paged else first.shape[1])
            ident = torch.arange(total_tokens, dtype=torch.long, device=first.device)
            return {"mode": "per_head", "indices": ident.unsqueeze(0).expand(heads, -1).contiguous()}
        if protect_prefill and config.include_prefill_in_budget and prefill_len > budget_total:
            return None
        if not entries:
            return None
        k = min(budget_total, total_tokens)
        if k <= 0:
            return {"mode": "per_head", "indices": []}
        layer_ids = tuple(int(e[0]) for e in entries)
        if paged:
            agg = os.environ.get("TRIATTN_RUNTIME_DEBUG_GROUP_PERHEAD_AGG_MODE", "mean").strip().lower()
            if agg not in {"mean", "max"}:
                agg = "mean"
            if len({int(e[3]) for e in entries}) != 1:
                raise RuntimeError("layers of one KV-cache group must share one block size")
            kv = _paged_kv([e[1] for e in entries])
            tables = entries[0][2]
        else:
            agg = "mean"
            kv = ops.PagedKV([e[1][..., :total_tokens, :].permute(0, 2, 1, 3) for e in entries], None,
                             _stats().rope_style)
            tables = None
        score_heads, group_reduce = _head_layout(kv.num_kv_heads)
        keep = _score_and_select(kv, layer_ids, tables, total_tokens, prefill_len, protect_prefill, round_start,
                                 k, agg, "max", score_heads, shared=False)
        return {"mode": "per_head", "indices": keep.contiguous(), "semantic": "hf_aligned_global_per_head",
                "group_agg_mode": agg, "debug_group_layer_indices": list(layer_ids),
                "debug_recent_count": _recent_count(total_tokens)}

    def _compress_group_batch(*, layer_kv: list, block_size: int, requests: list,
                              allow_resident: bool = True) -> list:
        """Selection **and** compaction of several requests of one KV-cache group in one launch
        sequence (no counterpart in the reference, which walks the requests one by one,
        runner_compression_actions.py:24; per request the result equals what
        ``_select_keep_indices_for_group_per_head`` followed by the per-head compaction gives).

        ``layer_kv``: [(layer_idx, kv_cache)] of the group; ``requests``: one dict per request
        with ``block_ids, total_tokens, prefill_len, protect_prefill, round_start, budget_total``
        and ``total_tokens > budget_total > 0``.  Returns the selector result dictionaries in
        request order (``indices``: int32, valid until this selector's next step); the caches then hold
        the kept rows in slots ``0..k-1``.  Raises
        ``ResidentLaunchFailed`` with the caches of this group untouched when a wait inside the
        resident kernel expired; the caller repeats the call with ``allow_resident=False``, which
        takes the kernels that do not wait for each other."""
        if mode != "per_head" or semantics != "hf_aligned_global_per_head":
            raise RuntimeError("batched compression serves the per_head / hf_aligned_global_per_head mode only")
        agg = os.environ.get("TRIATTN_RUNTIME_DEBUG_GROUP_PERHEAD_AGG_MODE", "mean").strip().lower()
        if agg not in {"mean", "max"}:
            agg = "mean"
        layer_ids = tuple(int(li) for li, _ in layer_kv)
        kv = _paged_kv([c for _, c in layer_kv])
        if int(kv.block_size) != int(block_size):
            raise RuntimeError("layers of one KV-cache group must share one block size")
        score_heads, _ = _head_layout(kv.num_kv_heads)
        st = _stats()
        omega, offsets = st.vectors(kv.device)
        sc = ops.ScoreConfig(st.folded(layer_ids, score_heads, kv.device), omega, offsets,
                             config.sparse_score_aggregation)
        totals = [int(r["total_tokens"]) for r in requests]
        ks = [min(int(r["budget_total"]), t) for r, t in zip(requests, totals)]
        if any(k <= 0 or k >= t for k, t in zip(ks, totals)):
            raise RuntimeError("batched compression expects total_tokens > budget_total > 0")
        guards = [int(r["prefill_len"]) if r["protect_prefill"] and int(r["prefill_len"]) > 0 else 0 for r in requests]
        rounds = [int(r["round_start"]) for r in requests]
        tables = [[int(x) for x in r["block_ids"]] for r in requests]
        use_resident = bool(allow_resident) and holder.get("resident_ok", True)
        rows = len(requests) * kv.num_kv_heads
        # A long generation repeats one shape (budget + divide_length tokens down to budget) every
        # divide_length tokens.  The second time a shape is seen its launch sequence is captured into
        # a HIP graph over device arrays that stay put; from then on a step is one small pinned copy
        # of the step's integers and one graph launch.  (The first time runs eagerly: most shapes,
        # e.g. the first compression after a long prompt, never come back.)
        key = (id(kv), layer_ids, tuple(totals), tuple(ks), tuple(len(t) for t in tables), any(g > 0 for g in guards),
               agg, use_resident)
        graphs = holder.setdefault("graphs", {})       # captured shapes, least recently used first
        seen = holder.setdefault("seen", {})           # keys of shapes that ran once, oldest first
        entry = graphs.get(key) if GRAPH_REPLAY else None
        try:
            if entry is not None:
                graphs[key] = graphs.pop(key)          # most recently used
                batch, ws, keep, resident = entry["batch"], entry["ws"], entry["keep"], entry["resident"]
                batch.refill(rounds, tables, guards)
                if resident:
                    # A graph holds neither the wait on the process's previous resident launch nor the
                    # record of this one; the library's own gate is put around the replay.
                    with ops.resident_gate():
                        entry["graph"].replay()
                else:
                    entry["graph"].replay()
                GRAPH_COUNTS["replayed"] += 1
            else:
                batch = ops.StepBatch(kv.device, totals, round_start=rounds, budgets=ks, block_tables=tables,
                                      prefill_lens=guards)
                sel = ops.SelectConfig(normalize=config.sparse_normalize_scores, window_size=config.window_size,
                                       protect_prefill=any(g > 0 for g in guards), group_reduce="max", layer_reduce=agg,
                                       allow_resident=use_resident)
                resident = ops.select_path(kv, batch, sc, sel) != "two_pass"
                if not (GRAPH_REPLAY and key in seen):
                    # Scratch and keep rows of the previous step are reused when they fit; the results
                    # handed out below are fresh tensors.
                    keep_buf = holder.get("keep")
                    if keep_buf is None or keep_buf.device != kv.device or keep_buf.numel() < rows * batch.max_budget:
                        keep_buf = holder["keep"] = torch.empty(rows * batch.max_budget, dtype=torch.int32,
                                                                device=kv.device)
                    keep, ws = ops.compress_step(kv, batch, sc, sel, holder.get("ws"),
                                                 keep_buf[:rows * batch.max_budget].view(rows, batch.max_budget))
                    holder["ws"] = ws
                    if GRAPH_REPLAY and ws.bytes <= GRAPH_MAX_SCRATCH_BYTES:
                        if len(seen) >= GRAPH_MAX_SEEN:
                            seen.pop(next(iter(seen)))
                        seen[key] = True
                else:
                    # Second visit: buffers of the entry's own, capture (nothing runs), then replay.
                    seen.pop(key, None)
                    ws = ops.Workspace(kv, batch, sc)
                    while graphs and (len(graphs) >= GRAPH_MAX_SHAPES or
                                      sum(e["ws"].bytes for e in graphs.values()) + ws.bytes > GRAPH_MAX_TOTAL_BYTES):
                        graphs.pop(next(iter(graphs)))
                    keep = torch.empty(rows, batch.max_budget, dtype=torch.int32, device=kv.device)
                    graph = torch.cuda.CUDAGraph()
                    # (thread-local error mode: another thread of the engine may use the GPU meanwhile)
                    with torch.cuda.graph(graph, capture_error_mode="thread_local"):
                        ops.compress_step(kv, batch, sc, sel, ws, keep)
                    graphs[key] = dict(graph=graph, batch=batch, ws=ws, keep=keep, resident=resident, kv=kv, sc=sc)
                    if resident:
                        with ops.resident_gate():
                            graph.replay()
                    else:
                        graph.replay()
                    GRAPH_COUNTS["captured"] += 1
        except Exception as exc:
            raise RuntimeError(f"{MARK}:score_failed:{type(exc).__name__}") from exc
        if resident and _resident_failed(ws.status()):
            raise ResidentLaunchFailed("a wait inside the resident kernel expired; the caches were left untouched")
        h = kv.num_kv_heads
        # The per-request indices are int32 views of a buffer this selector writes again at its next
        # step (the hook reads their shape only; a caller that keeps them copies them).
        return [{"mode": "per_head", "indices": keep[b * h:(b + 1) * h, :k],
                 "semantic": "hf_aligned_global_per_head", "group_agg_mode": agg,
                 "debug_group_layer_indices": list(layer_ids), "debug_recent_count": _recent_count(t)}
                for b, (k, t) in enumerate(zip(ks, totals))]

    setattr(_select_keep_indices, "_supports_paged", True)
    setattr(_select_keep_indices_for_group_per_head, "_supports_paged_group", True)
    if mode == "per_head" and semantics == "hf_aligned_global_per_head":
        setattr(_select_keep_indices_for_group_per_head, "_compress_batch", _compress_group_batch)
    return _select_keep_indices, _select_keep_indices_for_group_per_head, "enabled"
