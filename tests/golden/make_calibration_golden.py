"""Writes tests/golden/calibration_stats.pt: inputs and outputs of the reference's calibration
arithmetic (scripts/calibrate.py: _invert_rope, _to_complex_pairs and the per-head means of
lines 199-224), run on CPU in this container.  The op order and the bf16 rounding after every
elementwise operation are what this fixture pins; nothing else in the repository reads the
reference.

    python tests/golden/make_calibration_golden.py /root/reference
"""
from __future__ import annotations

import importlib.util
import sys
from pathlib import Path

import torch


def main() -> None:
    ref = Path(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
    spec = importlib.util.spec_from_file_location("ref_calibrate", ref / "scripts" / "calibrate.py")
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)

    cases = {}
    for name, (heads, tokens, dim, style, scale, dtype, theta) in {
        "half_bf16": (4, 120, 128, "half", 1.0, torch.bfloat16, 1e6),
        "half_bf16_scaled": (3, 77, 128, "half", 1.25, torch.bfloat16, 5e5),
        "interleaved_bf16": (2, 130, 64, "interleaved", 1.0, torch.bfloat16, 1e4),
        "half_fp16": (2, 96, 128, "half", 0.5, torch.float16, 1e6),
    }.items():
        g = torch.Generator().manual_seed(len(name) * 1000 + tokens)
        inv_freq = theta ** (-torch.arange(0, dim, 2, dtype=torch.float32) / dim)
        pos = torch.arange(tokens, dtype=torch.float32)
        ang = pos[:, None] * inv_freq[None, :]
        emb = torch.repeat_interleave(ang, 2, dim=-1) if style == "interleaved" else torch.cat((ang, ang), dim=-1)
        cos = (emb.cos() * scale).to(dtype)
        sin = (emb.sin() * scale).to(dtype)
        q = (torch.randn(heads, tokens, dim, generator=g) + 2.0 * torch.randn(heads, 1, dim, generator=g)).to(dtype)
        # what the reference's capture hook stores (calibrate.py:185-186)
        q_rot = (q * cos.unsqueeze(0)) + (mod._rotate_half(q, style=style) * sin.unsqueeze(0))
        q_rot = q_rot * scale
        q_base = mod._invert_rope(q_rot, cos.unsqueeze(0), sin.unsqueeze(0), scale, style=style)
        real, imag, absm = [], [], []
        for h in range(heads):
            z = mod._to_complex_pairs(q_base[h], style=style)
            m = z.mean(dim=0)
            real.append(m.real.clone())
            imag.append(m.imag.clone())
            absm.append(z.abs().mean(dim=0))
        cases[name] = {"q_rot": q_rot, "cos": cos, "sin": sin, "scale": float(scale), "style": style,
                       "inv_freq": inv_freq, "q_base": q_base, "q_mean_real": torch.stack(real),
                       "q_mean_imag": torch.stack(imag), "q_abs_mean": torch.stack(absm)}
    out = Path(__file__).resolve().parent / "calibration_stats.pt"
    torch.save(cases, out)
    print("wrote", out, out.stat().st_size, "bytes")


if __name__ == "__main__":
    main()
