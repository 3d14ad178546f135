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


def score_keys_for_round(key_states: torch.Tensor, q_mean_complex: torch.Tensor, q_abs_mean: torch.Tensor,
                         inv_freq: torch.Tensor, offsets: torch.Tensor, freq_scale_sq: torch.Tensor, round_start: int,
                         aggregation: str = "mean", rope_style: str = "half", attention_scale: float = 1.0,
                         disable_mlr: bool = False, disable_trig: bool = False) -> torch.Tensor:
    """Raw scores ``[Hq, T]`` (fp32, on the device) of the cached keys of one layer for the round that
    starts at ``round_start``: what the research path computes per sampled head by un-rotating the
    keys, forming amplitude / phase / extra against the head's query statistics and summing
    ``amp * cos((round_start - p + offset) * omega + phi) + extra`` over the frequency pairs
    (triattention/methods/pruning_utils.py:51-82, 245-309, called from methods/triattention.py:627-660).

    ``key_states``: the cache's POST-RoPE keys ``[1, Hkv, T, D]`` in bf16 / fp16, as they lie.  A rotated
    key carries its position in its phase, ``k_rot = scale * k * exp(i p omega)``, so
    ``q conj(k_rot) exp(i (round_start + offset) omega)`` is the reference's term at ``round_start - p + offset``
    times ``scale``: nothing is un-rotated and no position table is needed (positions that have gaps after
    earlier pruning included); the result is divided by ``attention_scale``.  ``q_mean_complex``
    ``[Hq, F, 2]`` (or complex ``[Hq, F]``) and ``q_abs_mean`` ``[Hq, F]`` are the statistics of the layer's
    query heads; one read of a KV head's keys serves its whole group of query heads."""
    if key_states.ndim != 4 or key_states.shape[0] != 1:
        raise ValueError(f"expected [1, Hkv, T, D] key states, got {tuple(key_states.shape)}")
    if attention_scale == 0:
        raise ValueError("attention scaling factor must be non-zero")
    dev = key_states.device
    if q_mean_complex.is_complex():
        q_mean_complex = torch.view_as_real(q_mean_complex)
    qc = q_mean_complex.to(device=dev, dtype=torch.float32)
    qa = q_abs_mean.to(device=dev, dtype=torch.float32)
    fs = freq_scale_sq.to(device=dev, dtype=torch.float32)
    if fs.ndim == 1:
        fs = fs.unsqueeze(0).expand(qa.shape[0], -1)
    total = int(key_states.shape[2])
    kv = ops.PagedKV([key_states.permute(0, 2, 1, 3)], None, rope_style)                   # [1, T, Hkv, D] view, no copy
    batch = ops.StepBatch(dev, [total], round_start=[int(round_start)])
    folded = ops.fold_stats(qc.unsqueeze(0), qa.unsqueeze(0), fs.contiguous().unsqueeze(0),
                            disable_mlr=disable_mlr, disable_trig=disable_trig)
    sc = ops.ScoreConfig(folded, inv_freq.to(device=dev, dtype=torch.float32).contiguous(),
                         offsets.to(device=dev, dtype=torch.float32).contiguous(), aggregation)
    raw, _ = ops.score_paged(kv, batch, sc, head_major=True)                               # [1, 1, Hq, T]
    scores = raw[0, 0]
    return scores if attention_scale == 1.0 else scores / float(attention_scale)


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
