"""Frequency-statistics files and what the scorer derives from them.

File format (written by the reference's calibration, scripts/calibrate.py:252-271 and
methods/pruning_utils.py:312-333): ``{"metadata": {...}, "stats": {"layerLL_headHH":
{"q_mean_real", "q_mean_imag", "q_abs_mean"}}}`` with one entry per QUERY head; a
second format carries stacked per-layer tensors under ``"layer_stats"``.  Loading
follows core/utils.py:18-361; the rotary frequencies follow the priority of
core/compressor.py:119-194: ``metadata["inv_freq"]``, then the model's rope description
(read from ``config.json`` under ``model_path``, no model code is imported), then
``rope_theta`` alone (default 10000).
"""
from __future__ import annotations

import json
import re
from pathlib import Path
from typing import Any, Dict, Optional, Tuple

import torch

from .. import rope as rope_mod

_KEY = re.compile(r"^layer(\d+)_head(\d+)$")


def _read_model_config(model_path) -> dict | None:
    if model_path is None:
        return None
    cfg = Path(model_path) / "config.json"
    if not cfg.is_file():
        return None
    try:
        return json.loads(cfg.read_text(encoding="utf-8"))
    except (OSError, ValueError):
        return None


def _as_inv_freq(raw, freq_count: int) -> torch.Tensor | None:
    if isinstance(raw, torch.Tensor):
        inv = raw.to(torch.float32)
    elif isinstance(raw, (list, tuple)):
        inv = torch.tensor(raw, dtype=torch.float32)
    else:
        return None
    if inv.numel() < freq_count:
        raise ValueError("metadata.inv_freq has fewer elements than required by "
                         f"head_dim={2 * freq_count}: got {inv.numel()}, expected at least {freq_count}")
    return inv.flatten()[:freq_count].contiguous()


def resolve_inv_freq(metadata: dict, head_dim: int, model_path=None) -> torch.Tensor:
    """core/compressor.py:119-194."""
    f = head_dim // 2
    inv = _as_inv_freq(metadata.get("inv_freq"), f)
    if inv is not None:
        return inv
    cfg = _read_model_config(model_path)
    if cfg is not None:
        try:
            scaling = cfg.get("rope_scaling") or cfg.get("rope_parameters")
            return rope_mod.inv_freq_from_rope_config(head_dim, cfg.get("rope_theta"), scaling)[:f].contiguous()
        except (KeyError, ValueError, TypeError):
            pass
    return rope_mod.default_inv_freq(head_dim, float(metadata.get("rope_theta", 10000.0)))


def _attention_scaling_sq(metadata: dict, model_path) -> float:
    """freq_scale_sq = (cos0^2 + sin0^2) at position 0 = attention_scaling^2 of the
    model's rotary embedding (common/rope_utils.py:78-90); 1 for default, linear and
    llama3 scaling.  Without a readable model config the reference falls back to ones
    (core/utils.py:286-295), and so does this."""
    cfg = _read_model_config(model_path) or {}
    scaling = cfg.get("rope_scaling") or cfg.get("rope_parameters") or {}
    factor = scaling.get("attention_factor", scaling.get("attn_factor"))
    return float(factor) ** 2 if isinstance(factor, (int, float)) and factor > 0 else 1.0


def load_frequency_stats(stats_path, device="cpu", dtype: torch.dtype = torch.float32,
                         num_kv_heads: Optional[int] = None, model_path=None) -> Tuple[Dict, Dict]:
    """(metadata, head_stats): ``head_stats[layer] = {"q_mean_complex" [H, F, 2],
    "q_abs_mean" [H, F], "freq_scale_sq" [H, F]}``.

    H is the number of query heads in the file unless ``num_kv_heads`` is given, in
    which case consecutive groups are mean-pooled (core/utils.py:328-356).  The file
    is read with ``weights_only=True``: nothing in it is executed.
    """
    stats_path = Path(stats_path)
    if not stats_path.exists():
        raise FileNotFoundError(f"Stats file not found: {stats_path}")
    payload = torch.load(stats_path, map_location="cpu", weights_only=True)
    metadata = dict(payload.get("metadata", {}) or {})
    per_head = payload.get("stats") or {}
    if per_head and any(_KEY.match(str(k)) for k in per_head):
        return _from_per_head_entries(metadata, per_head, device, dtype, num_kv_heads, model_path)

    missing = [k for k in ("num_attention_heads", "num_kv_heads", "head_dim", "num_layers") if k not in metadata]
    if missing:
        raise ValueError(f"Stats file missing required metadata keys: {missing}. Found keys: {list(metadata.keys())}")
    layer_stats = payload.get("layer_stats") or {}
    if not layer_stats:
        raise ValueError("Stats file does not contain 'layer_stats'")
    inv = _as_inv_freq(metadata.get("inv_freq"), int(metadata["head_dim"]) // 2)
    if inv is not None:
        metadata["inv_freq"] = inv.to(device)
    head_stats = {}
    for layer_idx, entry in layer_stats.items():
        head_stats[layer_idx] = {k: (v.to(device=device, dtype=dtype) if isinstance(v, torch.Tensor) else v)
                                 for k, v in entry.items()}
    return metadata, head_stats


def _from_per_head_entries(file_meta, entries, device, dtype, num_kv_heads, model_path):
    layers, heads = set(), set()
    for key in entries:
        m = _KEY.match(str(key))
        if m:
            layers.add(int(m.group(1)))
            heads.add(int(m.group(2)))
    num_layers, num_q = len(layers), len(heads)
    head_dim = int(file_meta.get("head_dim", 128))
    f = head_dim // 2
    if num_kv_heads is None:
        num_kv_heads = num_q
    group = num_q // num_kv_heads if num_kv_heads > 0 else 1

    metadata = {
        "num_attention_heads": num_q, "num_kv_heads": num_kv_heads, "head_dim": head_dim,
        "num_layers": num_layers, "rope_style": file_meta.get("rope_style", "half"),
        "rope_type": file_meta.get("rope_type"), "rope_theta": file_meta.get("rope_theta", 10000.0),
        "gqa_ratio": group, "rkv_metadata": file_meta,
    }
    inv = _as_inv_freq(file_meta.get("inv_freq"), f)
    if inv is None and model_path is not None and _read_model_config(model_path) is not None:
        inv = resolve_inv_freq({}, head_dim, model_path)
    if inv is not None:
        metadata["inv_freq"] = inv.to(device)

    scale_sq = _attention_scaling_sq(file_meta, model_path)
    head_stats = {}
    for layer in sorted(layers):
        abs_rows, re_rows, im_rows = [], [], []
        for head in sorted(heads):
            entry = entries.get(f"layer{layer:02d}_head{head:02d}")
            if entry is None:
                continue
            qa = entry.get("q_abs_mean")
            abs_rows.append(qa.to(dtype) if qa is not None else torch.ones(f, dtype=dtype))
            if "q_mean_real" in entry and "q_mean_imag" in entry:
                re_rows.append(entry["q_mean_real"].to(dtype))
                im_rows.append(entry["q_mean_imag"].to(dtype))
        q_abs = torch.stack(abs_rows, dim=0)
        if group > 1:
            q_abs = q_abs.reshape(num_kv_heads, group, f).mean(dim=1)
        out = {"freq_scale_sq": torch.full((num_kv_heads, f), scale_sq, dtype=dtype, device=device),
               "q_abs_mean": q_abs.to(device)}
        if re_rows and im_rows:
            q_re, q_im = torch.stack(re_rows, dim=0), torch.stack(im_rows, dim=0)
            if group > 1:
                q_re = q_re.reshape(num_kv_heads, group, f).mean(dim=1)
                q_im = q_im.reshape(num_kv_heads, group, f).mean(dim=1)
            out["q_mean_complex"] = torch.stack([q_re, q_im], dim=-1).to(device)
        head_stats[layer] = out
    return metadata, head_stats


def geometric_offsets(max_length: int = 65536) -> torch.Tensor:
    """[1, 2, 4, ... <= max_length] fp32 (core/compressor.py:222-242)."""
    if int(max_length) < 1:
        raise ValueError(f"offset_max_length must be >= 1, got {max_length}")
    vals, v = [], 1
    while v <= int(max_length):
        vals.append(float(v))
        v *= 2
    return torch.tensor(vals, dtype=torch.float32)


def pool_heads(t: torch.Tensor, target_heads: int) -> torch.Tensor:
    """Mean over consecutive groups of heads (runtime/selector_hf.py:147-203)."""
    src = int(t.shape[0])
    if src == target_heads:
        return t
    if target_heads <= 0 or src % target_heads:
        raise RuntimeError(f"incompatible_head_mapping:source={src},target={target_heads}")
    return t.reshape(target_heads, src // target_heads, *t.shape[1:]).mean(dim=1).contiguous()
