#!/usr/bin/env python3
"""Write tests/golden/hf_score.pt: outputs of the research path's scoring helpers
(triattention/methods/pruning_utils.py: ``invert_rope`` :51-82, ``compute_frequency_statistics_from_means``
:245-263, ``score_keys_for_round`` :266-309, ``build_geometric_offsets`` :231-242) on rotated bf16
keys as a Hugging Face cache holds them: the keys are cast to fp32 and un-rotated with the rotary
tables at their positions (methods/triattention.py:627-638), turned into (amplitude, phase, extra) against the per-head query statistics, and scored
for one round -- mean and max over the offsets, half and interleaved pairing, with and without the
``disable_mlr`` switch.

Runs ONLY in the build container, where the reference checkout is mounted read-only.

Usage:  python tests/golden/make_hf_score_golden.py [/root/reference]
"""
from __future__ import annotations

import sys
from pathlib import Path

import torch

HERE = Path(__file__).resolve().parent
REF = Path(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")


def rope_tables(positions: torch.Tensor, inv_freq: torch.Tensor, style: str, scale: float):
    """cos / sin [T, D] as a Hugging Face rotary embedding returns them (times the attention scale)."""
    ang = positions.float().unsqueeze(-1) * inv_freq.float().unsqueeze(0)                 # [T, F]
    emb = torch.cat((ang, ang), dim=-1) if style == "half" else ang.repeat_interleave(2, dim=-1)
    return emb.cos() * scale, emb.sin() * scale


def main() -> int:
    sys.path.insert(0, str(REF))
    from triattention.methods import pruning_utils as pu

    out = {}
    cases = {
        # name: (Hq, Hkv, T, D, style, scale, theta, round_start, seed)
        "half_d128": (8, 2, 192, 128, "half", 1.0, 1.0e6, 1000, 81),
        "interleaved_d64": (4, 4, 130, 64, "interleaved", 1.0, 1.0e4, 130, 82),
        "half_scaled": (6, 2, 97, 128, "half", 1.25, 5.0e5, 4096, 83),
    }
    for name, (hq, hkv, t, d, style, scale, theta, round_start, seed) in cases.items():
        g = torch.Generator().manual_seed(seed)
        f = d // 2
        inv_freq = theta ** (-torch.arange(0, f, dtype=torch.float32) / f)
        positions = torch.arange(t, dtype=torch.long) + 3                                  # key positions (not 0-based)
        cos, sin = rope_tables(positions, inv_freq, style, scale)
        k_pre = (torch.randn(hkv, t, d, generator=g) + torch.randn(hkv, 1, d, generator=g) * 1.4)
        rot = pu.rotate_half(k_pre, style=style)
        k_rot = (k_pre * cos.unsqueeze(0) + rot * sin.unsqueeze(0)).to(torch.bfloat16)     # what the cache holds
        q_mean = torch.complex(torch.randn(hq, f, generator=g), torch.randn(hq, f, generator=g))
        q_abs = q_mean.abs() + torch.randn(hq, f, generator=g).abs()
        offsets = pu.build_geometric_offsets(65536, torch.device("cpu"))
        freq_scale_sq = torch.full((f,), scale * scale)
        # fp32, as the research path runs it (methods/triattention.py:627,638,715: keys cast to config.dtype = float32)
        k_unrot = torch.stack([pu.invert_rope(k_rot[h].to(torch.float32), cos, sin, scale, style=style) for h in range(hkv)])
        case = {"k_rot": k_rot, "positions": positions, "cos": cos, "sin": sin, "inv_freq": inv_freq,
                "q_mean_real": q_mean.real.clone(), "q_mean_imag": q_mean.imag.clone(), "q_abs_mean": q_abs,
                "offsets": offsets, "freq_scale_sq": freq_scale_sq, "round_start": torch.tensor(round_start),
                "scale": torch.tensor(scale), "k_unrot": k_unrot, "style": style}
        group = hq // hkv
        for tag, mlr in (("", False), ("_nomlr", True)):
            for agg in ("mean", "max"):
                rows = []
                for a in range(hq):
                    amp, phi, extra = pu.compute_frequency_statistics_from_means(
                        q_mean[a], q_abs[a], k_unrot[a // group], style=style, disable_mlr=mlr)
                    rows.append(pu.score_keys_for_round(positions, round_start, amp, phi, inv_freq, extra, offsets,
                                                        agg, freq_scale_sq))
                case[f"scores_{agg}{tag}"] = torch.stack(rows)                             # [Hq, T]
        out[name] = case
        print(name, tuple(case["scores_mean"].shape), float(case["scores_mean"].abs().max()))
    torch.save(out, HERE / "hf_score.pt")
    print("written", HERE / "hf_score.pt", (HERE / "hf_score.pt").stat().st_size, "bytes")
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
