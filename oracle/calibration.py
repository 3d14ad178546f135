"""Oracle: per-query-head frequency statistics from captured query states (test
infrastructure, CPU only).

Restates the arithmetic of the reference's calibration pass, ``scripts/calibrate.py``:
RoPE inversion (:47-82, same as ``triattention/methods/pruning_utils.py:51-86``), complex
pairing (:85-98) and the per-head means (:199-224).  Everything up to the pairing runs in
the dtype of the captured queries (bf16 in the reference, :125), so every elementwise
operation rounds to that dtype; the statistics are fp32.
"""
from __future__ import annotations

import torch


def rotate_half(x: torch.Tensor, style: str = "half") -> torch.Tensor:
    """scripts/calibrate.py:38-44."""
    if style == "interleaved":
        return torch.stack((-x[..., 1::2], x[..., ::2]), dim=-1).flatten(-2)
    d = x.shape[-1] // 2
    return torch.cat((-x[..., d:], x[..., :d]), dim=-1)


def apply_rope(q: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, scale: float, style: str = "half") -> torch.Tensor:
    """What the capture hook stores: ``(q*cos + rotate_half(q)*sin) * scale`` in q's dtype
    (scripts/calibrate.py:185-186)."""
    return (q * cos + rotate_half(q, style) * sin) * scale


def invert_rope(rotated: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, scale: float,
                style: str = "half") -> torch.Tensor:
    """scripts/calibrate.py:47-82: divide queries and tables by the attention scale, then
    rotate back.  ``cos`` / ``sin`` broadcast against ``rotated`` ([T, D] against [H, T, D])."""
    if scale == 0:
        raise ValueError("attention scaling factor must be non-zero")
    scale_t = torch.tensor(scale, dtype=rotated.dtype)
    base = rotated / scale_t
    cos_unit = cos / scale_t
    sin_unit = sin / scale_t
    if style == "interleaved":
        even, odd = base[..., ::2], base[..., 1::2]
        cos_even, cos_odd = cos_unit[..., ::2], cos_unit[..., 1::2]
        sin_even, sin_odd = sin_unit[..., ::2], sin_unit[..., 1::2]
        det = (cos_even * cos_odd + sin_even * sin_odd).clamp_min(1e-12)
        restored = torch.empty_like(base)
        restored[..., ::2] = (even * cos_odd + odd * sin_even) / det
        restored[..., 1::2] = (odd * cos_even - even * sin_odd) / det
        return restored
    return base * cos_unit - rotate_half(base, style) * sin_unit


def to_complex_pairs(x: torch.Tensor, style: str = "half") -> torch.Tensor:
    """scripts/calibrate.py:85-98: fp32 complex, pair f = (x[f], x[f + D/2]) or (x[2f], x[2f+1])."""
    real_dtype = torch.float32 if x.dtype in (torch.bfloat16, torch.float16) else x.dtype
    xr = x.to(real_dtype)
    if style == "interleaved":
        return torch.complex(xr[..., ::2].contiguous(), xr[..., 1::2].contiguous())
    f = x.shape[-1] // 2
    return torch.complex(xr[..., :f].contiguous(), xr[..., f:].contiguous())


def head_frequency_stats(q_rot: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, scale: float,
                         style: str = "half"):
    """Per head: mean over tokens of the un-rotated query as a complex number per frequency
    pair, and the mean of its modulus (scripts/calibrate.py:199-224).

    q_rot [H, T, D], cos / sin [T, D] in the capture dtype.  Returns three fp32 [H, D/2]
    tensors: q_mean_real, q_mean_imag, q_abs_mean.
    """
    q_base = invert_rope(q_rot, cos.unsqueeze(0), sin.unsqueeze(0), scale, style)
    real, imag, mod = [], [], []
    for h in range(q_rot.shape[0]):
        z = to_complex_pairs(q_base[h], style)          # [T, F]
        m = z.mean(dim=0)
        real.append(m.real)
        imag.append(m.imag)
        mod.append(z.abs().mean(dim=0))
    return torch.stack(real), torch.stack(imag), torch.stack(mod)


def rope_tables(num_tokens: int, inv_freq: torch.Tensor, scale: float, dtype: torch.dtype, style: str = "half"):
    """cos / sin [T, D] as a Hugging Face rotary module hands them out: fp32 angles
    ``position * inv_freq`` laid out per pairing style, times the attention scale, cast to the
    model dtype (transformers ``modeling_rope_utils`` / ``*RotaryEmbedding.forward``)."""
    pos = torch.arange(num_tokens, dtype=torch.float32)
    ang = pos[:, None] * inv_freq.to(torch.float32)[None, :]
    emb = torch.repeat_interleave(ang, 2, dim=-1) if style == "interleaved" else torch.cat((ang, ang), dim=-1)
    return (emb.cos() * scale).to(dtype), (emb.sin() * scale).to(dtype)
