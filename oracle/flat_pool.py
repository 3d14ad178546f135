"""Oracle: the token-level (flat) KV pool of the reference's SGLang backend (test
infrastructure, CPU only).

Restates ``triattention/sglang/kv_compaction.py`` (gather :56-137, shared compaction
:146-270, per-head compaction :283-420, slot reclaim :423-470) and the selection order of
``triattention/sglang/scheduler_hooks.py:655-745``: per layer the raw scores of the query heads
of a KV head are reduced by max first (``sglang/scoring_utils.py:160-166``), then normalised
per (layer, KV head) with ``core/utils.py:466-480``, then aggregated over layers, guarded,
and the top ``k`` kept per KV head in ascending order.  Ties: lowest token index wins (the
reference's ``torch.topk(sorted=False)`` leaves them undefined).
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch

from .selection import topk_ascending, znorm_two_pass


def request_slots(req_to_token: torch.Tensor, req_pool_idx: int, effective_len: int) -> torch.Tensor:
    """Physical slot of every valid token of a request (kv_compaction.py:89)."""
    if effective_len > req_to_token.shape[1]:
        raise ValueError(f"effective_len ({effective_len}) exceeds req_to_token column count ({req_to_token.shape[1]})")
    return req_to_token[req_pool_idx, :effective_len].long()


def gather_request_k_dense(k_buffers: Sequence[torch.Tensor], req_to_token: torch.Tensor, req_pool_idx: int,
                           effective_len: int, target_layers: Optional[List[int]] = None) -> torch.Tensor:
    """[layers, H, effective_len, D] (kv_compaction.py:56-137)."""
    slots = request_slots(req_to_token, req_pool_idx, effective_len)
    layers = target_layers if target_layers is not None else list(range(len(k_buffers)))
    return torch.stack([k_buffers[l][slots].permute(1, 0, 2) for l in layers])


def _check_keep(keep: torch.Tensor, effective_len: int) -> None:
    if keep.shape[-1] > effective_len:
        raise ValueError(f"budget ({keep.shape[-1]}) exceeds effective_len ({effective_len})")
    if keep.shape[-1] > 1 and not torch.equal(keep, torch.sort(keep, dim=-1).values):
        raise ValueError("keep indices must be sorted in ascending order")
    if int(keep.min()) < 0:
        raise IndexError("keep indices contain negative values")
    if int(keep.max()) >= effective_len:
        raise IndexError(f"keep indices max ({int(keep.max())}) >= effective_len ({effective_len})")


def compact_shared(k_buffers, v_buffers, req_to_token, req_pool_idx: int, keep: torch.Tensor, effective_len: int,
                   target_layers: Optional[List[int]] = None) -> int:
    """One index list for all heads: slot ``req_to_token[i]`` receives the row of token
    ``keep[i]`` (kv_compaction.py:146-270; read everything, then write)."""
    keep = keep.long()
    budget = int(keep.shape[0])
    if budget <= 0:
        return 0
    _check_keep(keep, effective_len)
    slots = request_slots(req_to_token, req_pool_idx, effective_len)
    layers = target_layers if target_layers is not None else list(range(len(k_buffers)))
    for l in layers:
        for buf in (k_buffers[l], v_buffers[l]):
            rows = buf[slots[keep]].clone()
            for i in range(budget):
                buf[slots[i]] = rows[i]
    return budget


def compact_per_head(k_buffers, v_buffers, req_to_token, req_pool_idx: int, keep: torch.Tensor, effective_len: int,
                     target_layers: Optional[List[int]] = None) -> int:
    """``keep`` [H, budget]: head h of slot ``req_to_token[i]`` receives head h of token
    ``keep[h, i]`` (kv_compaction.py:283-420)."""
    keep = keep.long()
    heads, budget = int(keep.shape[0]), int(keep.shape[1])
    if budget <= 0:
        return 0
    _check_keep(keep, effective_len)
    slots = request_slots(req_to_token, req_pool_idx, effective_len)
    layers = target_layers if target_layers is not None else list(range(len(k_buffers)))
    for l in layers:
        for buf in (k_buffers[l], v_buffers[l]):
            before = buf.clone()
            for h in range(heads):
                for i in range(budget):
                    buf[slots[i], h] = before[slots[keep[h, i]], h]
    return budget


def reclaim_freed_slots(req_to_token: torch.Tensor, req_pool_idx: int, budget: int, effective_len: int) -> torch.Tensor:
    """Slots handed back to the allocator: the tail of the row without zeros, and the tail is
    zeroed (kv_compaction.py:423-470)."""
    if budget >= effective_len:
        return torch.empty(0, dtype=torch.int64)
    freed = req_to_token[req_pool_idx, budget:effective_len].long()
    freed = freed[freed != 0]
    if freed.numel():
        req_to_token[req_pool_idx, budget:effective_len] = 0
    return freed


def select_keep_group_first(raw: torch.Tensor, num_kv_heads: int, k: int, normalize: bool = True,
                            layer_mode: str = "mean", window_size: int = 0, prefill_len: int = 0,
                            protect_prefill: bool = False):
    """raw [L, A, T] fp32 per-query-head scores -> (keep [H, k] ascending, final [H, T]).

    scheduler_hooks.py:655-745 with scoring_utils.py:160-166 for the group reduction.
    """
    layers, heads, tokens = raw.shape
    group = heads // num_kv_heads
    agg = None
    for l in range(layers):
        s = raw[l].view(num_kv_heads, group, tokens).max(dim=1).values
        if normalize:
            s = znorm_two_pass(s)
        if agg is None:
            agg = s.clone()
        elif layer_mode == "max":
            agg = torch.maximum(agg, s)
        else:
            agg = agg + s
    if layer_mode != "max" and layers > 1:
        agg = agg / float(layers)
    if window_size > 0:
        agg = agg.clone()
        agg[..., -window_size:] = float("inf")
    if protect_prefill and prefill_len > 0:
        agg[..., :prefill_len] = float("inf")
    kk = min(k, tokens)
    return topk_ascending(agg, kk), agg
