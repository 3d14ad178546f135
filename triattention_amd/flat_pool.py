"""The token-level (flat) KV pool of the reference's SGLang backend on the HIP kernels.

SGLang keeps K and V of a layer as ``[total_slots, H, D]`` buffers and a ``req_to_token``
table that maps (request, position) to a slot (``triattention/sglang/kv_compaction.py``).
To the kernels that is a paged cache with one token per block and the request's row of
``req_to_token`` as its block table, so scoring, selection and compaction run on the same
kernels as the vLLM layout; the functions below have the reference's names, arguments, return
values and exception types.

The backend's selection differs from the vLLM runtime in the order of operations
(``sglang/scheduler_hooks.py:655-745``): the raw scores of the query heads of a KV head are
reduced by max first, each (layer, KV head) row is then normalised with torch mean / unbiased
std (``core/utils.py:466-480``), layers are averaged (or maxed), the window and prefill guards
come last.  ``select_keep_indices_per_head`` does that in one batched launch sequence straight
from the pool (no dense gather, no per-layer Python loop).
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch

from . import ops
from .runtime.kv_compaction import _is_validated, mark_keep_validated

_POOLS: dict = {}


def _pool_kv(k_buffers: Sequence[torch.Tensor], v_buffers: Optional[Sequence[torch.Tensor]],
             layers: Sequence[int], rope_style: str = "half") -> ops.PagedKV:
    """The chosen layers of a pool as one-token-per-block paged storage (built once per set
    of buffer addresses; holds no reference to the buffers)."""
    sample = k_buffers[layers[0]]
    if sample.ndim != 3:
        raise ValueError(f"expected [total_slots, H, D] buffers, got {tuple(sample.shape)}")
    key = (tuple(int(k_buffers[l].data_ptr()) for l in layers),
           None if v_buffers is None else tuple(int(v_buffers[l].data_ptr()) for l in layers),
           tuple(sample.shape), tuple(sample.stride()), sample.dtype, str(sample.device), rope_style)
    hit = _POOLS.get(key)
    if hit is None:
        k_views = [k_buffers[l].unsqueeze(1) for l in layers]
        v_views = None if v_buffers is None else [v_buffers[l].unsqueeze(1) for l in layers]
        hit = ops.PagedKV(k_views, v_views, rope_style)
        hit._keep = None
        if len(_POOLS) >= 16:
            _POOLS.pop(next(iter(_POOLS)))
        _POOLS[key] = hit
    return hit


def _request_row(req_to_token: torch.Tensor, req_pool_idx: int, effective_len: int, device) -> torch.Tensor:
    if effective_len > int(req_to_token.shape[1]):
        raise ValueError(f"effective_len ({effective_len}) exceeds req_to_token column count "
                         f"({int(req_to_token.shape[1])})")
    return req_to_token[req_pool_idx, :effective_len].to(device=device, dtype=torch.int32).unsqueeze(0).contiguous()


def gather_request_k_dense(k_buffers: List[torch.Tensor], req_to_token: torch.Tensor, req_pool_idx: int,
                           effective_len: int, target_layers: Optional[List[int]] = None) -> torch.Tensor:
    """Dense keys ``[layers, H, effective_len, D]`` of one request (kv_compaction.py:56-137).
    API only: the scorer reads the pool in place."""
    layers = target_layers if target_layers is not None else list(range(len(k_buffers)))
    slots = _request_row(req_to_token, req_pool_idx, effective_len, k_buffers[layers[0]].device)[0].long()
    pool_size = int(k_buffers[layers[0]].shape[0])
    lo, hi = int(slots.min().item()), int(slots.max().item())
    if lo < 0 or hi >= pool_size:
        raise ValueError(f"slot_indices out of bounds: min={lo}, max={hi}, k_buffer pool size={pool_size}")
    return torch.stack([k_buffers[l].index_select(0, slots).permute(1, 0, 2) for l in layers])


def _checked_keep(keep, rows: int, effective_len: int, device) -> Optional[torch.Tensor]:
    """[rows, budget] int64 on the device after the reference's checks
    (kv_compaction.py:196-222, 336-372); None when there is nothing to move.  The very tensor
    ``select_keep_indices_per_head`` returned for the same effective length is what the top-k kernel
    wrote -- ascending, in range, without duplicates by construction -- and skips the checks on the
    device (a sort and four device-to-host reads, 0.3 ms where the compaction itself takes 0.1 ms)."""
    trusted = _is_validated(keep, effective_len)
    keep = keep.to(device=device, dtype=torch.long)
    budget = int(keep.shape[-1])
    if budget <= 0:
        return None
    if budget > effective_len:
        raise ValueError(f"budget ({budget}) exceeds effective_len ({effective_len})")
    if trusted:
        return keep.reshape(rows, budget)
    if budget > 1 and not torch.equal(keep, torch.sort(keep, dim=-1).values):
        raise ValueError("keep indices must be sorted in ascending order to preserve original token order")
    lo, hi = int(keep.min().item()), int(keep.max().item())
    if lo < 0:
        raise IndexError("keep indices contain negative values")
    if hi >= effective_len:
        raise IndexError(f"keep indices max ({hi}) >= effective_len ({effective_len})")
    if budget > 1 and bool((keep[..., 1:] == keep[..., :-1]).any().item()):
        raise ValueError("keep indices must not contain duplicates")
    return keep.reshape(rows, budget)


def _compact(k_buffers, v_buffers, req_to_token, req_pool_idx, keep_rows, effective_len, target_layers, shared):
    layers = target_layers if target_layers is not None else list(range(len(k_buffers)))
    kv = _pool_kv(k_buffers, v_buffers, layers)
    budget = int(keep_rows.shape[1])
    batch = ops.StepBatch(kv.device, [effective_len], budgets=[budget],
                          block_tables=_request_row(req_to_token, req_pool_idx, effective_len, kv.device))
    ops.compact(kv, batch, keep_rows.to(torch.int32).contiguous(), shared=shared)
    return budget


def compact_request_kv_in_place(k_buffers: List[torch.Tensor], v_buffers: List[torch.Tensor],
                                req_to_token: torch.Tensor, req_pool_idx: int, keep_indices: torch.Tensor,
                                effective_len: int, target_layers: Optional[List[int]] = None) -> int:
    """One index list for all heads (kv_compaction.py:146-270): afterwards slot
    ``req_to_token[i]`` holds the row of token ``keep_indices[i]``, every layer in one launch."""
    keep = _checked_keep(keep_indices.reshape(1, -1), 1, effective_len, k_buffers[0].device)
    if keep is None:
        return 0
    return _compact(k_buffers, v_buffers, req_to_token, req_pool_idx, keep, effective_len, target_layers, True)


def compact_request_kv_in_place_per_head(k_buffers: List[torch.Tensor], v_buffers: List[torch.Tensor],
                                         req_to_token: torch.Tensor, req_pool_idx: int,
                                         keep_indices_per_head: torch.Tensor, effective_len: int,
                                         target_layers: Optional[List[int]] = None) -> int:
    """``keep_indices_per_head`` [H, budget] (kv_compaction.py:283-420): head h of slot
    ``req_to_token[i]`` receives head h of token ``keep_indices_per_head[h, i]``."""
    heads = int(k_buffers[0].shape[1])
    if keep_indices_per_head.ndim != 2 or int(keep_indices_per_head.shape[0]) != heads:
        raise ValueError(f"keep_indices_per_head must be [{heads}, budget], got {tuple(keep_indices_per_head.shape)}")
    keep = _checked_keep(keep_indices_per_head, heads, effective_len, k_buffers[0].device)
    if keep is None:
        return 0
    return _compact(k_buffers, v_buffers, req_to_token, req_pool_idx, keep, effective_len, target_layers, False)


def reclaim_freed_slots(req_to_token: torch.Tensor, req_pool_idx: int, budget: int, effective_len: int,
                        allocator: object) -> torch.Tensor:
    """Hand the slots behind the kept prefix back to the allocator and zero them in the table
    (kv_compaction.py:423-470).  Host logic on the table; no kernel of this package is involved."""
    if budget >= effective_len:
        return torch.empty(0, dtype=torch.int64, device=req_to_token.device)
    freed = req_to_token[req_pool_idx, budget:effective_len].long()
    freed = freed[freed != 0]                 # slot 0 is the allocator's dummy slot; zeros were freed before
    if freed.numel() == 0:
        return freed
    allocator.free(freed)
    req_to_token[req_pool_idx, budget:effective_len] = 0
    return freed


def select_keep_indices_per_head(k_buffers: List[torch.Tensor], req_to_token: torch.Tensor, req_pool_idx: int,
                                 effective_len: int, score: ops.ScoreConfig, budget: int, round_start: int, *,
                                 normalize: bool = True, layer_aggregation: str = "mean", window_size: int = 0,
                                 prefill_len: int = 0, protect_prefill: bool = False,
                                 target_layers: Optional[List[int]] = None, rope_style: str = "half",
                                 return_scores: bool = False):
    """Keep indices ``[H, min(budget, effective_len)]`` (int64, ascending) of one request, in the
    SGLang backend's order of operations (scheduler_hooks.py:655-745).

    ``score.folded`` holds the folded statistics of the chosen layers in order, per query head
    (``ops.fold_stats``); ``round_start`` is the request's logical length
    (scheduler_hooks.py:655-657).  ``window_size`` is 0 in the backend's configuration
    (sglang/config.py:147) but honoured when given.
    """
    layers = target_layers if target_layers is not None else list(range(len(k_buffers)))
    kv = _pool_kv(k_buffers, None, layers, rope_style)
    k = min(int(budget), int(effective_len))
    if k <= 0:
        raise ValueError("nothing to select")
    batch = ops.StepBatch(kv.device, [effective_len], round_start=[round_start], budgets=[k],
                          block_tables=_request_row(req_to_token, req_pool_idx, effective_len, kv.device),
                          prefill_lens=[prefill_len])
    sel = ops.SelectConfig(normalize=normalize, window_size=window_size,
                           protect_prefill=bool(protect_prefill and prefill_len > 0), group_reduce="max",
                           layer_reduce="max" if layer_aggregation == "max" else "mean", group_first=True)
    keep, fin, _ = ops.select_paged(kv, batch, score, sel, want_scores=return_scores)
    keep = mark_keep_validated(keep[:, :k].to(torch.long), effective_len)
    return (keep, fin[:, :effective_len]) if return_scores else keep
