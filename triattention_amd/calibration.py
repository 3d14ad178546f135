"""Producer of the frequency-statistics file the scorer loads.

What the reference's calibration pass does (``scripts/calibrate.py``): one forward pass over
a text; before every attention module runs, the query states it is about to use are
reconstructed (``q_proj`` of the incoming hidden states, RoPE with the model's rotary module,
times the attention scale, :170-188); per query head the un-rotated queries are then averaged
per frequency pair into ``q_mean_real``, ``q_mean_imag`` and ``q_abs_mean`` (:196-224) and
written as ``{"metadata": ..., "stats": {"layerLL_headHH": {...}}}`` (:252-271).

Here the arithmetic on a layer's captured queries is one HIP kernel (``ops.query_stats``),
run as soon as that layer has been captured, so only one layer's queries are alive at a
time (the reference holds all layers until the forward pass ends).  The file additionally
records ``metadata["inv_freq"]`` — the rotary frequencies the statistics belong to, which the
loader otherwise has to recover from the model's configuration (``core/utils.py:81-92``) —
and the head / layer counts; the reference's loader accepts both.
"""
from __future__ import annotations

from pathlib import Path
from typing import Callable, Dict, Tuple

import torch

from . import ops


def _rotate(x: torch.Tensor, style: str) -> torch.Tensor:
    # (-second half, first half), or (-odd, even) interleaved: scripts/calibrate.py:38-44
    if style == "interleaved":
        return torch.stack((-x[..., 1::2], x[..., ::2]), dim=-1).flatten(-2)
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


class StatsCollector:
    """Statistics of the layers seen so far, and the file they go into."""

    def __init__(self, head_dim: int, rope_style: str = "half", metadata: dict | None = None):
        if rope_style not in ("half", "interleaved"):
            raise ValueError(f"rope_style must be 'half' or 'interleaved', got {rope_style!r}")
        self.head_dim = int(head_dim)
        self.rope_style = rope_style
        self.metadata = dict(metadata or {})
        self._layers: Dict[int, Tuple[torch.Tensor, torch.Tensor, torch.Tensor]] = {}

    def add_layer(self, layer_idx: int, q_rot: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
                  scale: float = 1.0) -> None:
        """Captured queries of one layer, [H, T, D] or [1, H, T, D], with the rotary tables
        [T, D] they were rotated by and the attention scale they were multiplied with."""
        if q_rot.ndim == 4:
            if q_rot.shape[0] != 1:
                raise ValueError("one sequence at a time")
            q_rot = q_rot[0]
        if int(q_rot.shape[-1]) != self.head_dim:
            raise ValueError(f"head_dim {int(q_rot.shape[-1])} != {self.head_dim}")
        real, imag, mod = ops.query_stats(q_rot, cos, sin, scale, self.rope_style)
        self._layers[int(layer_idx)] = (real.cpu(), imag.cpu(), mod.cpu())

    def payload(self) -> dict:
        stats, sampled = {}, []
        for layer_idx in sorted(self._layers):
            real, imag, mod = self._layers[layer_idx]
            for head_idx in range(int(real.shape[0])):
                stats[f"layer{layer_idx:02d}_head{head_idx:02d}"] = {
                    "q_mean_real": real[head_idx].clone(),
                    "q_mean_imag": imag[head_idx].clone(),
                    "q_abs_mean": mod[head_idx].clone(),
                }
                sampled.append([layer_idx, head_idx])
        meta = {"num_traces": 1, "head_dim": self.head_dim, "rope_style": self.rope_style,
                "sampled_heads": sampled}
        meta.update(self.metadata)
        return {"metadata": meta, "stats": stats}

    def save(self, path) -> Path:
        out = Path(path)
        out.parent.mkdir(parents=True, exist_ok=True)
        torch.save(self.payload(), out)
        return out


def collect_model_stats(model: torch.nn.Module, input_ids: torch.Tensor, *, num_heads: int, head_dim: int,
                        rope_style: str = "half", rotary: Callable | None = None,
                        metadata: dict | None = None) -> StatsCollector:
    """One forward pass of a Hugging Face style decoder (``model.model.layers[i].self_attn``
    with a ``q_proj``; a rotary module on the backbone or on the attention modules that maps
    ``(probe [1, T, D], position_ids [1, T])`` to ``(cos, sin)`` and may carry
    ``attention_scaling`` and ``inv_freq``), collecting every layer's statistics."""
    backbone = getattr(model, "model", model)
    blocks = getattr(backbone, "layers", None)
    if blocks is None:
        raise RuntimeError("expected the decoder blocks under model.model.layers")
    attention = [getattr(block, "self_attn", None) for block in blocks]
    if any(a is None for a in attention):
        raise RuntimeError("a decoder block has no self_attn")
    if rotary is None:
        rotary = getattr(backbone, "rotary_emb", None) or attention[0].rotary_emb
    scale = float(getattr(rotary, "attention_scaling", 1.0))
    collector = StatsCollector(head_dim, rope_style, metadata)

    def capture(layer_idx: int):
        def pre_hook(module, args, kwargs):
            hidden = args[0] if args else kwargs.get("hidden_states")
            if hidden is None:
                return
            batch, tokens, _ = hidden.shape
            q = module.q_proj(hidden).view(batch, tokens, num_heads, head_dim).transpose(1, 2)
            positions = torch.arange(tokens, device=hidden.device).unsqueeze(0)
            probe = torch.zeros(1, tokens, head_dim, device=hidden.device, dtype=hidden.dtype)
            cos, sin = rotary(probe, positions)
            q_rot = (q * cos.unsqueeze(1) + _rotate(q, rope_style) * sin.unsqueeze(1)) * scale
            collector.add_layer(layer_idx, q_rot.detach(), cos[0], sin[0], scale)
        return pre_hook

    handles = [a.register_forward_pre_hook(capture(i), with_kwargs=True) for i, a in enumerate(attention)]
    try:
        with torch.no_grad():
            model(input_ids)
    finally:
        for handle in handles:
            handle.remove()
    inv_freq = getattr(rotary, "inv_freq", None)
    if isinstance(inv_freq, torch.Tensor):
        collector.metadata.setdefault("inv_freq", inv_freq.detach().to(torch.float32).cpu().flatten().clone())
    collector.metadata.setdefault("num_attention_heads", int(num_heads))
    collector.metadata.setdefault("num_layers", len(attention))
    return collector
