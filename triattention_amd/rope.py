"""Rotary inverse frequencies for the scorer (omega of the cosine series).

The reference takes ``inv_freq`` from, in order: the stats file's metadata, the
model's rotary embedding (through transformers), or ``rope_theta`` alone
(core/compressor.py:119-194).  Here the model's rope parameters are read from a plain
dict (the ``rope_scaling`` / ``rope_parameters`` entry of a HF config.json), so no
model code is imported.
"""
from __future__ import annotations

import math
from typing import Any, Mapping

import torch


def default_inv_freq(head_dim: int, rope_theta: float = 10000.0) -> torch.Tensor:
    """theta^(-2i/D), i = 0..D/2-1 (core/utils.py:520-542)."""
    if head_dim % 2 != 0:
        raise ValueError(f"head_dim must be even, got {head_dim}")
    exponent = torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim
    return 1.0 / (rope_theta ** exponent)


def llama3_inv_freq(head_dim: int, rope_theta: float = 500000.0, factor: float = 8.0,
                    low_freq_factor: float = 1.0, high_freq_factor: float = 4.0,
                    original_max_position_embeddings: int = 8192) -> torch.Tensor:
    """Llama-3.1 frequency scaling: long wavelengths divided by ``factor``, short ones
    kept, the band between ``orig/high`` and ``orig/low`` blended linearly."""
    base = default_inv_freq(head_dim, rope_theta)
    wavelen = 2.0 * math.pi / base
    lo_wl = original_max_position_embeddings / low_freq_factor
    hi_wl = original_max_position_embeddings / high_freq_factor
    out = torch.where(wavelen > lo_wl, base / factor, base)
    blend = (original_max_position_embeddings / wavelen - low_freq_factor) / (high_freq_factor - low_freq_factor)
    mixed = (1.0 - blend) * out / factor + blend * out
    band = (wavelen >= hi_wl) & (wavelen <= lo_wl)
    return torch.where(band, mixed, out)


def linear_inv_freq(head_dim: int, rope_theta: float, factor: float) -> torch.Tensor:
    return default_inv_freq(head_dim, rope_theta) / factor


def inv_freq_from_rope_config(head_dim: int, rope_theta: float | None,
                              rope_scaling: Mapping[str, Any] | None) -> torch.Tensor:
    """inv_freq for a HF-style rope description; unknown types raise."""
    rs = dict(rope_scaling or {})
    kind = rs.get("rope_type", rs.get("type", "default")) or "default"
    theta = float(rs.get("rope_theta", rope_theta if rope_theta is not None else 10000.0))
    if kind == "default":
        return default_inv_freq(head_dim, theta)
    if kind == "linear":
        return linear_inv_freq(head_dim, theta, float(rs["factor"]))
    if kind == "llama3":
        return llama3_inv_freq(head_dim, theta, float(rs["factor"]), float(rs["low_freq_factor"]),
                               float(rs["high_freq_factor"]), int(rs["original_max_position_embeddings"]))
    raise ValueError(f"unsupported rope_type {kind!r}: put inv_freq into the stats file's metadata")
