"""Oracle: score normalisation, guards, head/layer aggregation, top-k (test
infrastructure, CPU only).

Restates ``triattention/vllm/runtime/selector_hf.py`` (group selection
``:813-1033``, per-layer streaming selection ``:473-677``, dense selection
``:679-747``) and ``triattention/vllm/core/utils.py:466-502``.

Tie rule.  ``torch.topk(sorted=False)`` leaves the order among equal scores
undefined and the reference's chunked merge (selector_hf.py:1004-1019) changes it
again, so the oracle fixes one: among equal scores the LOWEST token index wins.
Everything else is the reference's arithmetic in the reference's order.
"""
from __future__ import annotations

from typing import Sequence

import torch


def znorm_two_pass(scores: torch.Tensor, eps: float = 1e-8) -> torch.Tensor:
    """core/utils.py:466-480: (x - mean) / std, unbiased std, std < eps -> 1."""
    mean = scores.mean(dim=-1, keepdim=True)
    std = scores.std(dim=-1, keepdim=True)
    std_safe = torch.where(std < eps, torch.ones_like(std), std)
    return (scores - mean) / std_safe


def score_chunk_tokens(block_size: int, total_tokens: int, score_chunk_max_tokens: int = 4096) -> int:
    """selector_hf.py:465-471."""
    upper = max(block_size, int(score_chunk_max_tokens))
    if total_tokens <= upper:
        return max(block_size, total_tokens)
    return upper


def znorm_stats_streaming(raw: torch.Tensor, chunk_tokens: int, eps: float = 1e-8, exact: bool = False):
    """Per-row mean and safe std from chunked sums (selector_hf.py:884-913).

    mean = sum/N; var = (sumsq - N*mean^2)/(N-1) clamped at 0; std < eps -> 1.
    ``exact``: the same formula with every sum and operation in double precision (what the
    reference's fp32 arithmetic approximates; used to bound how far two correct fp32 evaluations
    may disagree).
    """
    ft = torch.float64 if exact else torch.float32
    total = raw.shape[-1]
    sum_vec = None
    sumsq_vec = None
    count = 0
    start = 0
    while start < total:
        cur = min(chunk_tokens, total - start)
        chunk = raw[..., start:start + cur].to(ft)
        cs = chunk.sum(dim=-1)
        cq = (chunk * chunk).sum(dim=-1)
        sum_vec = cs if sum_vec is None else sum_vec + cs
        sumsq_vec = cq if sumsq_vec is None else sumsq_vec + cq
        count += cur
        start += cur
    mean = sum_vec / float(count)
    if count > 1:
        var = (sumsq_vec - float(count) * (mean * mean)) / float(count - 1)
    else:
        var = torch.zeros_like(mean)
    var = torch.clamp(var, min=0.0)
    std = torch.sqrt(var)
    std_safe = torch.where(std < eps, torch.ones_like(std), std)
    return mean, std_safe


def guard_mask(total_tokens: int, window_size: int, prefill_len: int, protect_prefill: bool, device="cpu"):
    """Bool [T]: True where a token is always kept (selector_hf.py:417-441,121-130)."""
    pos = torch.arange(total_tokens, device=device)
    mask = torch.zeros(total_tokens, dtype=torch.bool, device=device)
    if window_size > 0 and total_tokens > 0:
        recent = min(window_size, total_tokens)
        mask |= pos >= max(0, total_tokens - recent)
    if protect_prefill and prefill_len > 0:
        mask |= pos < prefill_len
    return mask


def reduce_group(scores: torch.Tensor, num_kv_heads: int, mode: str = "max") -> torch.Tensor:
    """[Hq, T] -> [Hkv, T] over consecutive groups (selector_hf.py:277-292)."""
    hq, t = scores.shape
    grouped = scores.view(num_kv_heads, hq // num_kv_heads, t)
    return grouped.mean(dim=1) if mode == "mean" else grouped.max(dim=1).values


def topk_ascending(scores: torch.Tensor, k: int) -> torch.Tensor:
    """Indices of the k largest per row, ascending; ties -> lowest index first."""
    order = torch.sort(scores, dim=-1, descending=True, stable=True).indices[..., :k]
    return torch.sort(order, dim=-1).values.contiguous()


def group_final_scores(
    raw_by_layer: Sequence[torch.Tensor],   # L tensors [Hq, T] fp32 raw scores
    num_kv_heads: int,
    *,
    normalize: bool = True,
    window_size: int = 128,
    prefill_len: int = 0,
    protect_prefill: bool = False,
    chunk_tokens: int | None = None,
    layer_agg: str = "mean",
    exact: bool = False,
) -> torch.Tensor:
    """Fin[Hkv, T]: z-norm -> guards(+inf) -> GQA max -> mean (or max) over layers.

    selector_hf.py:916-989.  The reference walks chunks in the outer loop and
    layers in the inner loop; per element that is the same sequence of fp32
    operations as below (subtract, divide, fill, max, running add in layer
    order, one division by the layer count).  ``exact``: the same formula on the
    same fp32 raw scores with every operation in double precision (returns fp64).
    """
    ft = torch.float64 if exact else torch.float32
    total = raw_by_layer[0].shape[-1]
    chunk = total if chunk_tokens is None else chunk_tokens
    guard = guard_mask(total, window_size, prefill_len, protect_prefill, raw_by_layer[0].device)
    agg = None
    for raw in raw_by_layer:
        x = raw.to(ft)
        if normalize:
            mean, std_safe = znorm_stats_streaming(x, chunk, exact=exact)
            x = (x - mean.view(-1, 1)) / std_safe.view(-1, 1)
        if bool(guard.any()):
            x = x.masked_fill(guard.view(1, -1), float("inf"))
        if x.shape[0] != num_kv_heads:
            x = reduce_group(x, num_kv_heads, "max")
        if agg is None:
            agg = x.clone()
        elif layer_agg == "max":
            agg = torch.maximum(agg, x)
        else:
            agg.add_(x)
    if layer_agg == "max":
        return agg
    return agg.div(float(len(raw_by_layer)))


def group_keep_per_head(raw_by_layer, num_kv_heads: int, budget_total: int, **kw):
    """keep[Hkv, k] int64 ascending for a whole KV-cache group, plus Fin.

    selector_hf.py:813-1033 (paged branch).  ``T <= budget`` keeps everything
    (selector_hf.py:768-798).
    """
    total = raw_by_layer[0].shape[-1]
    if total <= budget_total:
        idx = torch.arange(total, dtype=torch.long).unsqueeze(0).expand(num_kv_heads, -1).contiguous()
        return idx, None
    k = min(budget_total, total)
    fin = group_final_scores(raw_by_layer, num_kv_heads, **kw)
    return topk_ascending(fin, k), fin


def layer_final_scores(
    raw: torch.Tensor,                      # [Hs, T] raw scores of one layer
    num_kv_heads: int,
    *,
    normalize: bool = True,
    window_size: int = 128,
    prefill_len: int = 0,
    protect_prefill: bool = False,
    chunk_tokens: int | None = None,
    group_agg: str = "max",
    shared: bool = False,
) -> torch.Tensor:
    """Per-layer selection scores (selector_hf.py:584-602,636-637).

    z-norm, group reduce (max or mean) when the score heads outnumber the KV
    heads, guards, and for the shared (per_layer) mode a max over heads.
    """
    total = raw.shape[-1]
    x = raw.to(torch.float32)
    if normalize:
        mean, std_safe = znorm_stats_streaming(x, total if chunk_tokens is None else chunk_tokens)
        x = (x - mean.view(-1, 1)) / std_safe.view(-1, 1)
    if x.shape[0] != num_kv_heads:
        x = reduce_group(x, num_kv_heads, group_agg)
    guard = guard_mask(total, window_size, prefill_len, protect_prefill)
    if bool(guard.any()):
        x = x.masked_fill(guard.view(1, -1), float("inf"))
    if shared:
        x = x.max(dim=0, keepdim=True).values
    return x


def hf_final_scores(raw_by_layer: Sequence[torch.Tensor], num_kv_heads: int, decode_start: int,
                    normalize: bool = True) -> torch.Tensor:
    """Selection scores of the research path, over the decode tokens only
    (triattention/methods/triattention.py:250-258 and :368-425): every (layer, head) row of
    raw scores from token ``decode_start`` on is z-scored with the POPULATION standard deviation
    clamped from below at 1e-6 (not the runtime's unbiased std with ``< 1e-8 -> 1``), then
    per KV head the maximum over its query heads per layer and the mean over layers.
    The 1e-6 uniform noise of :260-267 exists only when the object carries a generator and is
    not part of this.  Returns [Hkv, T - decode_start]."""
    rows = torch.stack([r[:, decode_start:].to(torch.float32) for r in raw_by_layer])       # [L, Hq, Td]
    if normalize and rows.numel() > 0:
        mean = rows.mean(dim=-1, keepdim=True)
        std = rows.std(dim=-1, unbiased=False, keepdim=True).clamp_min(1e-6)
        rows = (rows - mean) / std
    layers, hq, td = rows.shape
    grouped = rows.view(layers, num_kv_heads, hq // num_kv_heads, td)
    return grouped.max(dim=2).values.mean(dim=0)


def hf_keep_per_head(raw_by_layer, num_kv_heads: int, decode_start: int, keep_count: int, normalize: bool = True):
    """[Hkv, decode_start + k] absolute indices, ascending: the prefill, then the top ``keep_count``
    decode tokens per KV head (methods/triattention.py:427-448; the reference leaves the decode part
    in top-k order, the oracle sorts it and breaks ties by the lowest index).  Also returns the
    selection scores."""
    fin = hf_final_scores(raw_by_layer, num_kv_heads, decode_start, normalize)
    k = min(keep_count, fin.shape[-1])
    dec = topk_ascending(fin, k) + decode_start
    pre = torch.arange(decode_start, dtype=torch.long).unsqueeze(0).expand(num_kv_heads, -1)
    return torch.cat([pre, dec], dim=1).contiguous(), fin


def protect_window(scores: torch.Tensor, window_size: int) -> torch.Tensor:
    """core/utils.py:483-502."""
    if window_size <= 0:
        return scores
    out = scores.clone()
    out[..., -window_size:] = float("inf")
    return out
