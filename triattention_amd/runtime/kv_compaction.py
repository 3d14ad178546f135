"""Paged-KV helpers with the reference's names and call shapes
(triattention/vllm/runtime/kv_compaction.py).  The moves run in the HIP compaction
kernels; argument checks raise the same exception types as the reference.

Differences, all on purpose:

* keep indices must be ascending (every selector returns them so,
  runtime/selector_hf.py:1025); the in-place kernels rely on ``keep[j] >= j``.
* ``preserve_dropped_tokens=True`` reproduces the reference's full ``[kept...,
  dropped...]`` permutation of all ``total_tokens`` slots through a staging buffer
  (kv_compaction.py:512-546).  ``False`` writes only the kept prefix, in ascending
  order; the reference's unordered fill-hole placement (kv_compaction.py:602-678) is
  not reproduced.
"""
from __future__ import annotations

import os
import weakref
from typing import Iterable

import torch

from .. import ops

_KV_AXIS_HINTS: dict = {}

# Keep-index tensors that came out of this package's own top-k kernel: ascending, unique and
# inside [0, T) by construction (whatever the scores were), so the host-side check of the
# compaction functions (two device-to-host reads, each a stream synchronisation in the middle
# of a compression) is skipped for them.  Anything else is checked as the reference does.
_VALIDATED_KEEP: dict = {}     # id(tensor) -> (weak reference, number of tokens it was selected from)


def mark_keep_validated(keep: torch.Tensor, total_tokens: int) -> torch.Tensor:
    key = id(keep)
    _VALIDATED_KEEP[key] = (weakref.ref(keep, lambda _ref, key=key: _VALIDATED_KEEP.pop(key, None)), int(total_tokens))
    return keep


def _is_validated(keep, total_tokens: int) -> bool:
    entry = _VALIDATED_KEEP.get(id(keep))
    return entry is not None and entry[0]() is keep and entry[1] == int(total_tokens)


def _hint_key(kv_cache: torch.Tensor):
    return (int(kv_cache.data_ptr()), int(kv_cache.storage_offset()), tuple(int(x) for x in kv_cache.shape),
            tuple(int(x) for x in kv_cache.stride()), str(kv_cache.device))


def register_kv_layout_axis_hint(kv_cache: torch.Tensor, kv_axis: int) -> None:
    """Say which of two size-2 leading dims is the K/V axis (kv_compaction.py:38-53)."""
    if kv_cache.ndim != 5:
        raise ValueError(f"Expected 5D kv_cache for layout hint, got ndim={kv_cache.ndim}")
    if kv_axis not in (0, 1):
        raise ValueError(f"kv_axis must be 0 or 1, got {kv_axis}")
    if int(kv_cache.shape[kv_axis]) != 2:
        raise ValueError(f"kv_axis={kv_axis} does not point to K/V dimension (shape={tuple(kv_cache.shape)})")
    _KV_AXIS_HINTS[_hint_key(kv_cache)] = kv_axis


def clear_kv_layout_axis_hints_for_tests() -> None:
    _KV_AXIS_HINTS.clear()


def kv_axis_hint(kv_cache: torch.Tensor):
    if not _KV_AXIS_HINTS:          # the usual case: nothing registered, no key to build
        return None
    return _KV_AXIS_HINTS.get(_hint_key(kv_cache))


def _split_kv_axes(kv_cache: torch.Tensor):
    return ops.split_kv_axes(kv_cache, kv_axis_hint(kv_cache))


def build_keep_token_indices(total_tokens: int, kv_budget: int, prefill_len: int, protect_prefill: bool,
                             include_prefill_in_budget: bool = True):
    """Score-free keep list: prefill (if protected) plus the most recent tokens
    (kv_compaction.py:60-91).  None when the prefill alone exceeds the budget."""
    budget = kv_budget + (max(prefill_len, 0) if protect_prefill and not include_prefill_in_budget else 0)
    budget = min(total_tokens, budget)
    if total_tokens <= budget:
        return list(range(total_tokens))
    if protect_prefill:
        if include_prefill_in_budget and prefill_len > budget:
            return None
        tail_start = max(prefill_len, total_tokens - max(0, budget - prefill_len))
        return list(range(prefill_len)) + list(range(tail_start, total_tokens))
    return list(range(max(0, total_tokens - budget), total_tokens))


def _block_ids_list(block_ids) -> list:
    if isinstance(block_ids, torch.Tensor):
        return [int(x) for x in block_ids.flatten().tolist()]
    return [int(x) for x in block_ids]


def _token_slots(block_ids, block_size: int, tokens: torch.Tensor, device):
    ids = torch.as_tensor(_block_ids_list(block_ids), device=device, dtype=torch.long)
    logical = torch.div(tokens, block_size, rounding_mode="floor")
    if logical.numel() > 0 and int(logical.max().item()) >= int(ids.numel()):
        raise IndexError(f"token indices require block_idx={int(logical.max().item())}, "
                         f"but only {int(ids.numel())} blocks exist")
    return ids[logical], torch.remainder(tokens, block_size)


def gather_request_k_dense_range(kv_cache: torch.Tensor, block_ids, block_size: int, start_token: int,
                                 num_tokens: int) -> torch.Tensor:
    """Dense [1, H, num_tokens, D] copy of a request's keys (kv_compaction.py:322-352).
    The HIP scorer reads the paged blocks directly and never calls this; it exists for
    callers that want the dense tensor."""
    if start_token < 0:
        raise ValueError(f"start_token must be >= 0, got {start_token}")
    if num_tokens <= 0:
        raise ValueError(f"num_tokens must be > 0, got {num_tokens}")
    key_cache, _ = _split_kv_axes(kv_cache)
    tok = torch.arange(start_token, start_token + num_tokens, device=key_cache.device, dtype=torch.long)
    blk, off = _token_slots(block_ids, block_size, tok, key_cache.device)
    return key_cache[blk, off].transpose(0, 1).unsqueeze(0)


def gather_request_k_dense(kv_cache, block_ids, block_size: int, total_tokens: int) -> torch.Tensor:
    if total_tokens <= 0:
        raise ValueError(f"total_tokens must be > 0, got {total_tokens}")
    return gather_request_k_dense_range(kv_cache, block_ids, block_size, 0, total_tokens)


def gather_request_kv_dense(kv_cache, block_ids, block_size: int, total_tokens: int):
    if total_tokens <= 0:
        raise ValueError(f"total_tokens must be > 0, got {total_tokens}")
    key_cache, value_cache = _split_kv_axes(kv_cache)
    tok = torch.arange(total_tokens, device=key_cache.device, dtype=torch.long)
    blk, off = _token_slots(block_ids, block_size, tok, key_cache.device)
    return (key_cache[blk, off].transpose(0, 1).unsqueeze(0),
            value_cache[blk, off].transpose(0, 1).unsqueeze(0))


def _check_rows(keep: torch.Tensor, total_tokens: int, what: str) -> None:
    """Range, duplicate and order checks on [rows, k] keep indices (one host sync)."""
    lo, hi = int(keep.min().item()), int(keep.max().item())
    if lo < 0 or hi >= total_tokens:
        raise IndexError(f"keep token index out of range: min={lo}, max={hi}, expected [0, {total_tokens})")
    if keep.shape[1] > 1:
        diff = keep[:, 1:] - keep[:, :-1]
        if bool((diff <= 0).any().item()):
            srt = torch.sort(keep, dim=1).values
            if bool((srt[:, 1:] == srt[:, :-1]).any().item()):
                raise ValueError(f"{what} must not contain duplicates")
            raise ValueError(f"{what} must be ascending for in-place compaction")


def _debug_validate_compaction_content() -> bool:
    """The reference's self-check switch (kv_compaction.py:24-25)."""
    return os.environ.get("TRIATTN_DEBUG_VALIDATE_COMPACTION_CONTENT", "0") == "1"


def _rows_of(cache, block_ids, block_size: int, keep_rows: torch.Tensor, shared: bool):
    """K and V rows ``[k, H, D]`` (as bytes) that the slots 0..k-1 must hold after compaction."""
    out = []
    for side in _split_kv_axes(cache):
        if shared:
            blk, off = _token_slots(block_ids, block_size, keep_rows[0], side.device)
            rows = side[blk, off]
        else:
            per_head = []
            for h in range(int(side.shape[2])):
                blk, off = _token_slots(block_ids, block_size, keep_rows[h], side.device)
                per_head.append(side[blk, off, h])
            rows = torch.stack(per_head, dim=1)
        out.append(rows.contiguous().view(torch.uint8).clone())
    return out


def _validate_prefix(kv_caches, block_ids, block_size: int, k: int, expected: list, shared: bool) -> None:
    """Re-read the compacted prefix and compare it bit for bit with the rows gathered before
    the move (kv_compaction.py:441-456,548-563; same exception texts)."""
    label = "shared" if shared else "per_head"
    for cache, (want_k, want_v) in zip(kv_caches, expected):
        key_cache, value_cache = _split_kv_axes(cache)
        tok = torch.arange(k, device=key_cache.device, dtype=torch.long)
        blk, off = _token_slots(block_ids, block_size, tok, key_cache.device)
        if not torch.equal(key_cache[blk, off].contiguous().view(torch.uint8), want_k):
            raise RuntimeError(f"TRIATTN_DEBUG_COMPACTION_KEY_MISMATCH:{label}_prefix_content_mismatch")
        if not torch.equal(value_cache[blk, off].contiguous().view(torch.uint8), want_v):
            raise RuntimeError(f"TRIATTN_DEBUG_COMPACTION_VALUE_MISMATCH:{label}_prefix_content_mismatch")


def _run_compaction(kv_caches, block_ids, block_size: int, keep_rows: torch.Tensor, total_tokens: int,
                    shared: bool, full_permutation: bool) -> None:
    expected = None
    if _debug_validate_compaction_content():
        expected = [_rows_of(c, block_ids, block_size, keep_rows, shared) for c in kv_caches]
    hints = {kv_axis_hint(c) for c in kv_caches}
    if len(hints) != 1:
        raise ValueError("layers of one group disagree on the K/V axis hint")
    kv = ops.PagedKV.for_kv_caches(kv_caches, kv_axis=hints.pop())
    if kv.block_size != block_size:
        raise ValueError(f"block_size={block_size} does not match the cache's {kv.block_size}")
    k = int(keep_rows.shape[1])
    batch = ops.StepBatch.for_request(kv.device, total_tokens, _block_ids_list(block_ids), budget=k)
    ops.compact(kv, batch, keep_rows.to(device=kv.device, dtype=torch.int32).contiguous(),
                shared=shared, full_permutation=full_permutation)
    if expected is not None:
        _validate_prefix(kv_caches, block_ids, block_size, k, expected, shared)


def compact_request_kv_in_place(kv_cache, block_ids, block_size: int, keep_token_indices,
                                total_tokens: int, preserve_dropped_tokens: bool = True) -> int:
    """One index list for all heads (kv_compaction.py:355-458).  ``kv_cache`` may be a
    list of per-layer tensors: all layers are then compacted by one launch."""
    caches = list(kv_cache) if isinstance(kv_cache, (list, tuple)) else [kv_cache]
    device = caches[0].device
    if isinstance(keep_token_indices, torch.Tensor):
        keep = keep_token_indices.to(device=device, dtype=torch.long).flatten()
    else:
        keep = torch.as_tensor(list(keep_token_indices), device=device, dtype=torch.long)
    if keep.numel() == 0:
        return 0
    _split_kv_axes(caches[0])      # layout check, raises like the reference
    _check_rows(keep.unsqueeze(0), total_tokens, "keep_token_indices")
    k = int(keep.numel())
    if k >= total_tokens:
        return k
    _run_compaction(caches, block_ids, block_size, keep.unsqueeze(0), total_tokens, shared=True,
                    full_permutation=bool(preserve_dropped_tokens))
    return k


def compact_request_kv_in_place_per_head(kv_cache, block_ids, block_size: int, keep_token_indices_per_head,
                                         total_tokens: int, preserve_dropped_tokens: bool = True) -> int:
    """Independent index list per KV head, [H, k] (kv_compaction.py:461-599)."""
    caches = list(kv_cache) if isinstance(kv_cache, (list, tuple)) else [kv_cache]
    key_cache, _ = _split_kv_axes(caches[0])
    device, heads = key_cache.device, int(key_cache.shape[2])
    trusted = _is_validated(keep_token_indices_per_head, total_tokens)
    if isinstance(keep_token_indices_per_head, torch.Tensor):
        keep = keep_token_indices_per_head.to(device=device, dtype=torch.long)
    else:
        if not keep_token_indices_per_head:
            return 0
        keep = torch.as_tensor(keep_token_indices_per_head, device=device, dtype=torch.long)
    if keep.ndim != 2:
        raise ValueError(f"keep_token_indices_per_head must be 2D, got shape={tuple(keep.shape)}")
    if int(keep.shape[0]) != heads:
        raise ValueError("keep_token_indices_per_head head count mismatch: "
                         f"expected {heads}, got {int(keep.shape[0])}")
    k = int(keep.shape[1])
    if k <= 0:
        return 0
    if not trusted:
        _check_rows(keep, total_tokens, "per-head keep indices")
    if k >= total_tokens:
        return k
    _run_compaction(caches, block_ids, block_size, keep, total_tokens, shared=False,
                    full_permutation=bool(preserve_dropped_tokens))
    return k
