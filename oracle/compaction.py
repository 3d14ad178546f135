"""Oracle: paged-KV gather, in-place compaction, block-table truncation (test
infrastructure, CPU only).

Restates ``triattention/vllm/runtime/kv_compaction.py`` (layout split ``:94-117``,
slot resolution ``:139-187``, dense gathers ``:254-352``, shared compaction
``:355-458``, per-head compaction ``:461-599``) and
``triattention/vllm/runtime/layout_engine.py:25-28,209-227``.
"""
from __future__ import annotations

import torch


def split_kv(kv_cache: torch.Tensor, kv_axis: int | None = None):
    """K and V views [num_blocks, block_size, H, D] of a 5-D cache (kv_compaction.py:94-117)."""
    if kv_cache.ndim != 5:
        raise ValueError(f"Unsupported kv_cache ndim={kv_cache.ndim}, expect 5")
    d0, d1 = int(kv_cache.shape[0]) == 2, int(kv_cache.shape[1]) == 2
    if d0 and d1:
        if kv_axis is None:
            raise ValueError("Ambiguous KV layout: both dim0 and dim1 have size 2")
        d0, d1 = kv_axis == 0, kv_axis == 1
    if d0:
        return kv_cache[0], kv_cache[1]
    if d1:
        return kv_cache[:, 0], kv_cache[:, 1]
    raise ValueError("Unsupported KV layout: expected a dimension with size 2")


def token_slots(block_ids: torch.Tensor, block_size: int, token_indices: torch.Tensor):
    """(physical block, in-block offset) of logical tokens (kv_compaction.py:139-157)."""
    block_ids = torch.as_tensor(block_ids, dtype=torch.long)
    logical = torch.div(token_indices, block_size, rounding_mode="floor")
    if logical.numel() > 0 and int(logical.max()) >= block_ids.numel():
        raise IndexError("token indices require more blocks than the request owns")
    return block_ids[logical], torch.remainder(token_indices, block_size)


def gather_dense(cache_bthd: torch.Tensor, block_ids, block_size: int, start: int, count: int):
    """[1, H, count, D] dense copy of logical tokens [start, start+count) (kv_compaction.py:322-352)."""
    tok = torch.arange(start, start + count, dtype=torch.long)
    blk, off = token_slots(block_ids, block_size, tok)
    return cache_bthd[blk, off].transpose(0, 1).unsqueeze(0)


def _validate_keep(keep: torch.Tensor, total_tokens: int):
    if keep.numel() == 0:
        return
    lo, hi = int(keep.min()), int(keep.max())
    if lo < 0 or hi >= total_tokens:
        raise IndexError(f"keep token index out of range: min={lo}, max={hi}, expected [0, {total_tokens})")


def compact_per_head(kv_cache, block_ids, block_size: int, keep: torch.Tensor, total_tokens: int,
                     *, kv_axis: int | None = None, full_permutation: bool = True) -> int:
    """Per-head in-place compaction (kv_compaction.py:461-599).

    ``full_permutation=True`` is the reference behaviour: every head's T rows are
    rewritten as [kept..., dropped...] (dropped in ascending order,
    kv_compaction.py:518-546).  ``False`` writes only the kept prefix, which is
    what survives block-table truncation.
    """
    key_cache, value_cache = split_kv(kv_cache, kv_axis)
    h = key_cache.shape[2]
    keep = torch.as_tensor(keep, dtype=torch.long)
    if keep.ndim != 2:
        raise ValueError(f"keep_token_indices_per_head must be 2D, got shape={tuple(keep.shape)}")
    if keep.shape[0] != h:
        raise ValueError(f"head count mismatch: expected {h}, got {keep.shape[0]}")
    k = int(keep.shape[1])
    if k <= 0:
        return 0
    _validate_keep(keep, total_tokens)
    srt = torch.sort(keep, dim=1).values
    if k > 1 and bool((srt[:, 1:] == srt[:, :-1]).any()):
        raise ValueError("per-head keep indices must not contain duplicates")
    if torch.equal(keep, torch.arange(k).unsqueeze(0).expand(h, -1)):
        return k
    if full_permutation:
        mask = torch.ones((h, total_tokens), dtype=torch.bool)
        mask.scatter_(1, keep, False)
        tail = torch.arange(total_tokens).unsqueeze(0).expand(h, -1)[mask].view(h, total_tokens - k)
        perm = torch.cat([keep, tail], dim=1)
        dst = torch.arange(total_tokens)
    else:
        perm = keep
        dst = torch.arange(k)
    sb, so = token_slots(block_ids, block_size, perm)
    hidx = torch.arange(h).unsqueeze(1)
    gk = key_cache[sb, so, hidx].clone()       # [H, n, D]
    gv = value_cache[sb, so, hidx].clone()
    db, do = token_slots(block_ids, block_size, dst)
    key_cache[db, do] = gk.permute(1, 0, 2).contiguous()
    value_cache[db, do] = gv.permute(1, 0, 2).contiguous()
    return k


def compact_shared(kv_cache, block_ids, block_size: int, keep: torch.Tensor, total_tokens: int,
                   *, kv_axis: int | None = None, full_permutation: bool = True) -> int:
    """Shared-index in-place compaction (kv_compaction.py:355-458)."""
    keep = torch.as_tensor(keep, dtype=torch.long).flatten()
    if keep.numel() == 0:
        return 0
    key_cache, value_cache = split_kv(kv_cache, kv_axis)
    _validate_keep(keep, total_tokens)
    if torch.unique(keep).numel() != keep.numel():
        raise ValueError("keep_token_indices must not contain duplicates")
    k = int(keep.numel())
    if k >= total_tokens or torch.equal(keep, torch.arange(k)):
        return k
    if full_permutation:
        mask = torch.ones(total_tokens, dtype=torch.bool)
        mask[keep] = False
        perm = torch.cat([keep, torch.arange(total_tokens)[mask]])
        dst = torch.arange(total_tokens)
    else:
        perm, dst = keep, torch.arange(k)
    sb, so = token_slots(block_ids, block_size, perm)
    gk = key_cache[sb, so].clone()
    gv = value_cache[sb, so].clone()
    db, do = token_slots(block_ids, block_size, dst)
    key_cache[db, do] = gk
    value_cache[db, do] = gv
    return k


def required_blocks(tokens: int, block_size: int) -> int:
    """layout_engine.py:25-28."""
    return 0 if tokens <= 0 else (tokens + block_size - 1) // block_size


def truncate_tail(block_ids, cache_len_after: int, block_size: int):
    """(kept ids, removed ids) after compaction (layout_engine.py:209-227)."""
    n = required_blocks(cache_len_after, block_size)
    ids = [int(x) for x in block_ids]
    return ids[:n], ids[n:]
