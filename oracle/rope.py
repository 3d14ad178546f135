"""Oracle: RoPE inverse frequencies (test infrastructure, CPU only).

``default_inv_freq`` follows ``triattention/vllm/core/utils.py:520-542``.
``llama3_inv_freq`` restates the published llama-3.1 frequency scaling that the
reference obtains from ``transformers`` (``LlamaRotaryEmbedding`` through
``triattention/common/rope_utils.py:30-56``; transformers is a third-party
dependency, unpinned in the reference's setup.py as ``transformers>=4.48.1``):
wavelengths above ``orig_ctx/low`` are divided by ``factor``, those below
``orig_ctx/high`` are kept, the band in between is interpolated linearly in
``orig_ctx/wavelen``.
"""
from __future__ import annotations

import math

import torch


def default_inv_freq(head_dim: int, rope_theta: float = 10000.0) -> torch.Tensor:
    if head_dim % 2 != 0:
        raise ValueError(f"head_dim must be even, got {head_dim}")
    return 1.0 / (rope_theta ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))


def llama3_inv_freq(head_dim: int, rope_theta: float = 500000.0, factor: float = 8.0,
                    low_freq_factor: float = 1.0, high_freq_factor: float = 4.0,
                    original_max_position_embeddings: int = 8192) -> torch.Tensor:
    inv_freq = 1.0 / (rope_theta ** (torch.arange(0, head_dim, 2, dtype=torch.int64).float() / head_dim))
    low_freq_wavelen = original_max_position_embeddings / low_freq_factor
    high_freq_wavelen = original_max_position_embeddings / high_freq_factor
    wavelen = 2 * math.pi / inv_freq
    scaled = torch.where(wavelen > low_freq_wavelen, inv_freq / factor, inv_freq)
    smooth = (original_max_position_embeddings / wavelen - low_freq_factor) / (
        high_freq_factor - low_freq_factor)
    smoothed = (1 - smooth) * scaled / factor + smooth * scaled
    medium = ~(wavelen < high_freq_wavelen) & ~(wavelen > low_freq_wavelen)
    return torch.where(medium, smoothed, scaled)
