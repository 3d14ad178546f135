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


def verify_rope_alignment(pruner_rotary: Any, model_rotary: Any, tolerance: float = 1e-5) -> None:
    """Raise ``ValueError`` unless both objects carry the same ``inv_freq`` (shape, and values
    within ``tolerance``): statistics scored with other frequencies than the model's rotate to
    meaningless scores without any error (core/utils.py:364-405).  Tensors are taken as they are."""
    def freqs(obj, name):
        f = obj if isinstance(obj, torch.Tensor) else getattr(obj, "inv_freq", None)
        if f is None:
            raise ValueError(f"{name} does not have inv_freq attribute")
        return f
    a, b = freqs(pruner_rotary, "pruner_rotary"), freqs(model_rotary, "model_rotary")
    if a.shape != b.shape:
        raise ValueError(f"RoPE inv_freq shape mismatch: pruner={tuple(a.shape)}, model={tuple(b.shape)}")
    worst = float((a.detach().double().cpu() - b.detach().double().cpu()).abs().max())
    if worst > tolerance:
        raise ValueError(f"RoPE inv_freq mismatch (max diff={worst:.2e} > tolerance={tolerance:.2e}): the "
                         "statistics and the model disagree on the rotary frequencies (rope_theta or scaling)")
