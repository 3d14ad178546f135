"""Oracle: trigonometric key scores (test infrastructure, CPU only).

Restates ``triattention/vllm/core/scoring.py:207-362`` (``compute_scores_pytorch``)
for post-RoPE keys, and ``triattention/methods/pruning_utils.py:245-309`` for the
same score on un-rotated keys with explicit positions.
"""
from __future__ import annotations

import torch


def split_pairs(keys: torch.Tensor, rope_style: str):
    """Real / imaginary halves of every frequency pair.

    ``half``: pair f = (K[..., f], K[..., f + D/2]); ``interleaved``: (K[..., 2f],
    K[..., 2f+1]).  Follows scoring.py:275-282.
    """
    d = keys.shape[-1]
    if rope_style == "interleaved":
        pairs = keys.reshape(*keys.shape[:-1], d // 2, 2)
        return pairs[..., 0], pairs[..., 1]
    return keys[..., : d // 2], keys[..., d // 2:]


def geometric_offsets(max_length: int = 65536) -> torch.Tensor:
    """[1, 2, 4, ..., <= max_length] as fp32 (compressor.py:222-242)."""
    vals = []
    v = 1
    while v <= max_length:
        vals.append(float(v))
        v *= 2
    return torch.tensor(vals, dtype=torch.float32)


def raw_scores(
    keys: torch.Tensor,            # [..., H, T, D] post-RoPE keys, any float dtype
    q_mean_complex: torch.Tensor,  # [H, F, 2] fp32
    q_abs_mean: torch.Tensor,      # [H, F] fp32
    omega: torch.Tensor,           # [F] fp32
    offsets: torch.Tensor,         # [NO] fp32
    freq_scale_sq: torch.Tensor,   # [H, F] fp32
    round_start: int,
    aggregation: str = "mean",
    rope_style: str = "half",
    disable_mlr: bool = False,
    disable_trig: bool = False,
    k_abs_eps: float = 0.0,
) -> torch.Tensor:
    """Raw score per (head, token); fp32 accumulation (keys promoted first).

    scoring.py:255-362 with the keys promoted to fp32 up front (the runtime
    selector runs with compute_dtype=float32, selector_hf.py:115).  ``k_abs_eps``
    is 0 for the PyTorch path (scoring.py:283) and 1e-8 for the Triton kernel
    (kernels/triton_scoring.py:277).
    """
    keys = keys.to(torch.float32)
    q_r = q_mean_complex[..., 0].to(torch.float32)
    q_i = q_mean_complex[..., 1].to(torch.float32)
    q_abs_mean = q_abs_mean.to(torch.float32)
    omega = omega.to(torch.float32)
    s = freq_scale_sq.to(torch.float32).unsqueeze(-2)           # [H, 1, F]

    q_mean_abs = torch.sqrt(q_r ** 2 + q_i ** 2 + 1e-8)          # scoring.py:264
    k_r, k_i = split_pairs(keys, rope_style)
    if k_abs_eps:
        k_abs = torch.sqrt(k_r ** 2 + k_i ** 2 + k_abs_eps)
    else:
        k_abs = torch.sqrt(k_r ** 2 + k_i ** 2)                  # scoring.py:283

    qr_e = q_r.unsqueeze(-2)                                     # [H, 1, F]
    qi_e = q_i.unsqueeze(-2)
    prod_real = qr_e * k_r + qi_e * k_i                          # scoring.py:290
    prod_imag = qi_e * k_r - qr_e * k_i                          # scoring.py:291

    per_offset = []
    for off in offsets:
        t = round_start + off.item()                             # scoring.py:313
        if not disable_trig:
            phase = t * omega                                    # fp32 product
            term = s * (prod_real * torch.cos(phase) - prod_imag * torch.sin(phase))
        else:
            term = torch.zeros_like(prod_real)
        per_offset.append(term.sum(dim=-1))                      # scoring.py:332
    stacked = torch.stack(per_offset, dim=0)
    if aggregation == "mean":
        scores = stacked.mean(dim=0)
    elif aggregation == "max":
        scores = stacked.max(dim=0).values
    else:
        raise ValueError(f"Unsupported score_aggregation: {aggregation}")

    extra_coef = q_abs_mean if disable_mlr else (q_abs_mean - q_mean_abs)
    extra = (k_abs * extra_coef.unsqueeze(-2) * s).sum(dim=-1)   # scoring.py:355
    return scores + extra


def rope_rotate(x: torch.Tensor, positions: torch.Tensor, omega: torch.Tensor,
                rope_style: str = "half", scale: float = 1.0) -> torch.Tensor:
    """Apply RoPE at ``positions`` to ``x[..., T, D]`` in fp32.

    Rotation by angle p*omega_f of the complex pair (x_r + i x_i): the forward
    counterpart of ``invert_rope`` (pruning_utils.py:51-82).
    """
    x = x.to(torch.float32)
    ang = positions.to(torch.float32).unsqueeze(-1) * omega.to(torch.float32)   # [T, F]
    c, s_ = torch.cos(ang) * scale, torch.sin(ang) * scale
    x_r, x_i = split_pairs(x, rope_style)
    y_r = x_r * c - x_i * s_
    y_i = x_i * c + x_r * s_
    if rope_style == "interleaved":
        return torch.stack((y_r, y_i), dim=-1).flatten(-2)
    return torch.cat((y_r, y_i), dim=-1)


def raw_scores_unrotated(
    keys_unrot: torch.Tensor,      # [H, T, D] keys before RoPE
    positions: torch.Tensor,       # [T] key positions
    q_mean_complex: torch.Tensor,
    q_abs_mean: torch.Tensor,
    omega: torch.Tensor,
    offsets: torch.Tensor,
    freq_scale_sq: torch.Tensor,
    round_start: int,
    aggregation: str = "mean",
    rope_style: str = "half",
    disable_mlr: bool = False,
    disable_trig: bool = False,
) -> torch.Tensor:
    """The HF-path form: amp*cos((round_start - p + o)*omega + phi) + extra.

    pruning_utils.py:245-263 (amp, phi, extra; |q| without epsilon) and
    pruning_utils.py:266-309 (phase grid, aggregation).
    """
    k = keys_unrot.to(torch.float32)
    k_r, k_i = split_pairs(k, rope_style)
    kc = torch.complex(k_r.contiguous(), k_i.contiguous())                     # [H, T, F]
    qc = torch.complex(q_mean_complex[..., 0].float().contiguous(),
                       q_mean_complex[..., 1].float().contiguous())            # [H, F]
    q_mean_abs = torch.abs(qc)
    k_abs = torch.abs(kc)
    rel = qc.unsqueeze(-2) * torch.conj(kc)
    phi = torch.atan2(rel.imag, rel.real)
    amp = q_mean_abs.unsqueeze(-2) * k_abs
    coef = q_abs_mean.float() if disable_mlr else (q_abs_mean.float() - q_mean_abs)
    extra = coef.unsqueeze(-2) * k_abs                                         # [H, T, F]

    s = freq_scale_sq.to(torch.float32)
    base_delta = round_start - positions.to(torch.float32)                     # [T]
    delta = base_delta.unsqueeze(-1) + offsets.to(torch.float32).unsqueeze(0)  # [T, NO]
    phase = delta.unsqueeze(-1) * omega.float().view(1, 1, -1)                 # [T, NO, F]
    phase = phase.unsqueeze(0) + phi.unsqueeze(2)                              # [H, T, NO, F]
    base = (amp.unsqueeze(2) * s.view(s.shape[0], 1, 1, -1) * torch.cos(phase)).sum(dim=-1)
    additive = (extra * s.unsqueeze(-2)).sum(dim=-1, keepdim=True)             # [H, T, 1]
    combined = additive.expand_as(base) if disable_trig else base + additive
    if aggregation == "mean":
        return combined.mean(dim=-1)
    return combined.max(dim=-1).values


def dequant_fp8(codes: torch.Tensor, scales: torch.Tensor) -> torch.Tensor:
    """e4m3 codes [..., H, D] times per-(token, head) fp32 scale [..., H] -> fp32.

    No counterpart in the reference (it has no fp8 code); parity unpinned beyond
    this closed form.
    """
    return codes.to(torch.float32) * scales.to(torch.float32).unsqueeze(-1)
