"""Dense KV compression: score -> normalise -> protect window -> top-k -> gather.

The reference's ``TriAttentionCompressor`` (triattention/vllm/core/compressor.py:27-421)
with ``CompressionState`` (core/state.py:23-196) and the dense helpers of
core/utils.py:433-502.  Scoring, normalisation, window guard and top-k run in the HIP
kernels; only the final gather into NEW dense tensors uses ``torch.gather`` (this API
returns fresh tensors, it does not touch a paged cache).
"""
from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch

from .. import ops
from . import stats as stats_mod
from .config import TriAttentionConfig
from .scoring import compute_scores


def normalize_scores(scores: torch.Tensor, eps: float = 1e-8) -> torch.Tensor:
    """z-score along the last axis, unbiased std, std < eps -> 1 (core/utils.py:466-480)."""
    mean = scores.mean(dim=-1, keepdim=True)
    std = scores.std(dim=-1, keepdim=True)
    return (scores - mean) / torch.where(std < eps, torch.ones_like(std), std)


def protect_window_tokens(scores: torch.Tensor, window_size: int) -> torch.Tensor:
    """Last ``window_size`` tokens -> +inf (core/utils.py:483-502)."""
    if window_size <= 0:
        return scores
    out = scores.clone()
    out[..., -window_size:] = float("inf")
    return out


def gather_kv_by_indices(kv_tensor: torch.Tensor, indices: torch.Tensor, dim: int = 2) -> torch.Tensor:
    """[B, H, T, D] gathered along T by [B, k] or [B, H, k] indices (core/utils.py:433-463)."""
    if indices.ndim == 2:
        b, k = indices.shape
        idx = indices.view(b, 1, k, 1).expand(b, kv_tensor.shape[1], k, kv_tensor.shape[3])
    elif indices.ndim == 3:
        idx = indices.unsqueeze(-1).expand(*indices.shape, kv_tensor.shape[3])
    else:
        raise ValueError(f"Unsupported indices shape: {indices.shape}")
    return torch.gather(kv_tensor, dim=dim, index=idx)


class CompressionState:
    """Per-request counters that decide when to compress (core/state.py:23-196):
    trigger at budget + divide_length, compress down to budget."""

    def __init__(self, config: TriAttentionConfig):
        self.config = config
        self.reset()

    def reset(self) -> None:
        self.absolute_position = 0
        self.compression_count = 0
        self.prefill_length = 0
        self.tokens_in_round = 0
        self.current_cache_len = 0
        self.last_prune_step = 0

    def initialize(self, seq_len: int) -> None:
        self.current_cache_len = self.prefill_length = self.absolute_position = seq_len

    def append_tokens(self, n: int) -> None:
        self.current_cache_len += n
        self.absolute_position += n
        self.tokens_in_round += n

    def should_compress(self, current_len: int) -> bool:
        if self.absolute_position == 0:
            self.initialize(current_len)
            effective = current_len
        else:
            new_tokens = current_len - self.absolute_position
            if new_tokens > 0:
                self.append_tokens(new_tokens)
            effective = self.current_cache_len
        if self.config.protect_prefill:
            effective = max(0, effective - self.prefill_length)
        return effective >= self.config.kv_budget + self.config.divide_length

    def update_after_compression(self, new_cache_len: int) -> None:
        self.current_cache_len = new_cache_len
        self.last_prune_step = self.absolute_position
        self.tokens_in_round = 0
        self.compression_count += 1

    def get_effective_budget(self) -> int:
        if self.config.protect_prefill:
            return max(0, self.config.kv_budget - self.prefill_length)
        return self.config.kv_budget

    def get_round_start(self) -> int:
        return self.absolute_position

    def to_dict(self) -> dict:
        return {k: getattr(self, k) for k in ("absolute_position", "compression_count", "prefill_length",
                                              "tokens_in_round", "current_cache_len", "last_prune_step")}


class TriAttentionCompressor:
    def __init__(self, config: TriAttentionConfig):
        self.config = config
        self.state = CompressionState(config)
        self.metadata: Optional[Dict] = None
        self.head_stats: Optional[Dict] = None
        self.inv_freq = self.omega = self.freq_scale_sq = self.offsets = None
        self.trig_cache = None      # kept for attribute compatibility; the HIP scorer needs no table cache
        self._initialized = False

    def _lazy_init(self) -> None:
        """core/compressor.py:70-117."""
        if self._initialized:
            return
        cfg = self.config
        if cfg.stats_path is None:
            raise ValueError("stats_path must be specified in TriAttentionConfig.")
        self.metadata, self.head_stats = stats_mod.load_frequency_stats(
            cfg.stats_path, device=cfg.device, dtype=cfg.compute_dtype, num_kv_heads=cfg.num_kv_heads,
            model_path=cfg.model_path)
        if cfg.head_dim is None:
            cfg.head_dim = self.metadata["head_dim"]
        if cfg.num_kv_heads is None:
            cfg.num_kv_heads = self.metadata["num_kv_heads"]
        if cfg.num_layers is None:
            cfg.num_layers = self.metadata["num_layers"]
        if "rope_style" in self.metadata:
            cfg.rope_style = str(self.metadata["rope_style"])
        self.inv_freq = stats_mod.resolve_inv_freq(self.metadata, cfg.head_dim, cfg.model_path).to(cfg.device)
        self.omega = self.inv_freq
        f = cfg.head_dim // 2
        self.freq_scale_sq = torch.zeros(cfg.num_layers, cfg.num_kv_heads, f, device=cfg.device,
                                         dtype=cfg.compute_dtype)
        for layer in range(cfg.num_layers):
            entry = self.head_stats.get(layer)
            if entry is not None and "freq_scale_sq" in entry:
                self.freq_scale_sq[layer] = entry["freq_scale_sq"]
        self.offsets = stats_mod.geometric_offsets(cfg.offset_max_length).to(cfg.device)
        self._initialized = True

    def _compute_scores(self, key_states: torch.Tensor, layer_idx: int) -> torch.Tensor:
        if layer_idx not in self.head_stats:
            raise ValueError(f"No stats found for layer {layer_idx}")
        return compute_scores(key_states=key_states, cache_positions=None, head_stats=self.head_stats[layer_idx],
                              omega=self.omega, offsets=self.offsets, freq_scale_sq=self.freq_scale_sq[layer_idx],
                              config=self.config, round_start=self.state.get_round_start(),
                              trig_cache=self.trig_cache)

    def _select_topk(self, scores: torch.Tensor, k: int) -> torch.Tensor:
        """Indices of the k largest along the last axis, ascending (core/compressor.py:388-409
        leaves their order undefined)."""
        flat = scores.reshape(-1, scores.shape[-1]).to(torch.float32).contiguous()
        keep = ops.topk_rows(flat, k)[:, :k].to(torch.long)
        return keep.reshape(*scores.shape[:-1], k)

    def compress(self, key_states: torch.Tensor, value_states: torch.Tensor,
                 cache_positions: Optional[torch.Tensor] = None, layer_idx: int = 0
                 ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        """core/compressor.py:279-346; batch size 1 only, as in the reference."""
        self._lazy_init()
        b, h, t, d = key_states.shape
        if b > 1:
            raise ValueError(f"TriAttention currently only supports batch_size=1 for compression. Got batch_size={b}.")
        if not self.state.should_compress(t):
            return key_states, value_states, torch.arange(t, device=key_states.device)
        scores = self._compute_scores(key_states, layer_idx)
        if self.config.sparse_normalize_scores:
            scores = normalize_scores(scores)
        if self.config.window_size > 0:
            scores = protect_window_tokens(scores, self.config.window_size)
        keep = self._select_topk(scores, self.config.kv_budget)
        keys = gather_kv_by_indices(key_states, keep, dim=2)
        values = gather_kv_by_indices(value_states, keep, dim=2)
        self.state.update_after_compression(keys.shape[2])
        return keys, values, keep

    def reset(self) -> None:
        self.state.reset()

    def get_state(self) -> Dict:
        return self.state.to_dict()
