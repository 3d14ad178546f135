"""Dense-key scoring entry points with the reference's call shape
(triattention/vllm/core/scoring.py:18-204), executed by the HIP scorer.

``compute_scores_triton`` keeps its name so call sites that import it (the reference's
selector does, runtime/selector_hf.py:59) bind to the HIP kernel unchanged; there is no
Triton and no PyTorch scorer here, and a missing library raises.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from .config import TriAttentionConfig


def _round_start(round_start, cache_positions, seq_len: int) -> int:
    """core/scoring.py:126-132."""
    if round_start is not None:
        return int(round_start)
    if cache_positions is not None:
        return int(cache_positions.max().item())
    return seq_len - 1


def compute_scores_hip(key_states: torch.Tensor, cache_positions: Optional[torch.Tensor],
                       head_stats: Dict[str, torch.Tensor], omega: torch.Tensor, offsets: torch.Tensor,
                       freq_scale_sq: torch.Tensor, config: TriAttentionConfig,
                       round_start: Optional[int] = None, trig_cache=None) -> torch.Tensor:
    """Scores [batch, heads, seq_len] (or [batch, seq_len] in per_layer mode) for
    post-RoPE keys [batch, heads, seq_len, head_dim] in the cache dtype.

    ``head_stats['q_mean_complex']`` is [heads, F, 2]; ``'q_abs_mean'`` [heads, F] is
    optional and defaults to |q_mean| (no magnitude term), as in core/scoring.py:120-124.
    ``trig_cache`` is accepted and ignored: the offset tables are rebuilt on the device
    from the fp32 phase ``(round_start + offset) * omega`` for every call, which is what
    the reference's PyTorch path evaluates (core/scoring.py:313-324).
    """
    if key_states.ndim != 4:
        raise ValueError(f"key_states must be [batch, heads, seq_len, head_dim], got {tuple(key_states.shape)}")
    if key_states.dtype not in (torch.bfloat16, torch.float16):
        raise TypeError(f"key_states must be in the cache dtype (bf16 or fp16), got {key_states.dtype}")
    if key_states.stride(3) != 1:
        key_states = key_states.contiguous()
    b, h, t, d = (int(x) for x in key_states.shape)
    dev = key_states.device
    qc = head_stats["q_mean_complex"].to(device=dev, dtype=torch.float32)
    if "q_abs_mean" in head_stats:
        qa = head_stats["q_abs_mean"].to(device=dev, dtype=torch.float32)
    else:
        qa = torch.sqrt(qc[..., 0] ** 2 + qc[..., 1] ** 2 + 1e-8)
    fs = freq_scale_sq.to(device=dev, dtype=torch.float32)
    if int(qc.shape[0]) != h:
        raise ValueError(f"stats have {int(qc.shape[0])} heads, keys have {h}")
    rs = _round_start(round_start, cache_positions, t)

    kv = ops.PagedKV.from_dense_keys(key_states, rope_style=config.rope_style)
    batch = ops.StepBatch(dev, [t] * b, round_start=[rs] * b)
    folded = ops.fold_stats(qc.unsqueeze(0), qa.unsqueeze(0), fs.unsqueeze(0),
                            disable_mlr=config.disable_mlr, disable_trig=config.disable_trig)
    sc = ops.ScoreConfig(folded, omega.to(device=dev, dtype=torch.float32).contiguous(),
                         offsets.to(device=dev, dtype=torch.float32).contiguous(), config.score_aggregation)
    raw, _ = ops.score_paged(kv, batch, sc, head_major=True)      # [B, 1, H, T]
    scores = raw[:, 0]
    if config.pruning_mode == "per_layer":
        scores = scores.mean(dim=1)
    return scores.to(dtype=config.topk_dtype)


# The names the reference exports.  All three run the same kernel.
compute_scores_triton = compute_scores_hip
compute_scores = compute_scores_hip
