"""Per-KV-head selection with the research path's semantics (the reference's Hugging Face
integration, triattention/methods/triattention.py:168-304 and :368-450), on the same kernels as
the serving runtime.

It differs from the runtime's selection (runtime/selector_hf.py:813-1033) in three ways: only the
tokens from ``decode_start`` on are scored and ranked (the prefill is always kept); every
(layer, query head) row is z-scored with the population standard deviation clamped at 1e-6
(``:255-258``) instead of the streaming unbiased one with ``< 1e-8 -> 1``; and there is no recent
window.  The reference can add uniform noise of 1e-6 to break ties (``:260-267``, only when it
was built with a generator); here ties keep the lowest token index, so kept sets agree with a
noise-free run of the reference except between scores closer than that noise.
"""
from __future__ import annotations

from typing import Sequence

import torch

from . import ops


def select_keep_indices_per_head(key_states_by_layer: Sequence[torch.Tensor], *, decode_start: int, keep_count: int,
                                 folded_stats: torch.Tensor, inv_freq: torch.Tensor, offsets: torch.Tensor,
                                 round_start: int, normalize: bool = True, rope_style: str = "half",
                                 aggregation: str = "mean") -> torch.Tensor:
    """``key_states_by_layer``: one post-RoPE ``[1, Hkv, T, D]`` bf16 / fp16 device tensor per layer (a
    Hugging Face cache's key tensors); ``folded_stats``: ``ops.fold_stats`` of the per-query-head
    statistics of those layers.  Returns int64 ``[Hkv, decode_start + k]``, ``k = min(keep_count,
    T - decode_start)``: the prefill indices followed by the kept decode tokens, ascending
    (the reference returns the decode part in top-k order, methods/triattention.py:427-448)."""
    if not key_states_by_layer:
        raise ValueError("no layers")
    k0 = key_states_by_layer[0]
    if k0.ndim != 4 or k0.shape[0] != 1:
        raise ValueError(f"expected [1, Hkv, T, D] key states, got {tuple(k0.shape)}")
    hkv, total = int(k0.shape[1]), int(k0.shape[2])
    decode_start = max(0, min(int(decode_start), total))
    prefill = torch.arange(decode_start, dtype=torch.long, device=k0.device).unsqueeze(0).expand(hkv, -1)
    k = min(int(keep_count), total - decode_start)
    if k <= 0:
        return prefill.contiguous()
    views = [ks[..., decode_start:, :].permute(0, 2, 1, 3) for ks in key_states_by_layer]      # [1, Td, Hkv, D], no copy
    kv = ops.PagedKV(views, None, rope_style)
    batch = ops.StepBatch(kv.device, [total - decode_start], round_start=[int(round_start)], budgets=[k])
    sc = ops.ScoreConfig(folded_stats, inv_freq, offsets, aggregation)
    sel = ops.SelectConfig(normalize="population" if normalize else False, window_size=0, group_reduce="max",
                           layer_reduce="mean")
    keep, _, _ = ops.select_paged(kv, batch, sc, sel)
    return torch.cat([prefill, keep.to(torch.long) + decode_start], dim=1).contiguous()
