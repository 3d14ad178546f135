#!/usr/bin/env python3
"""Write tests/golden/hf_select.pt: keep indices of the research path's per-KV-head selection
(``TriAttention._select_per_head_independent``, triattention/methods/triattention.py:368-450) for
a head matrix normalised as ``compute_keep_indices`` does (:255-258: population std clamped at
1e-6; the tie-breaking noise of :260-267 is only added when the object carries a generator and is
left out, so the fixture is deterministic).

Runs ONLY in the build container, where the reference checkout is mounted read-only.  The method is
called unbound on a stand-in object that carries the four attributes it reads.

Usage:  python tests/golden/make_hf_select_golden.py [/root/reference]
"""
from __future__ import annotations

import sys
import types
from pathlib import Path

import torch

HERE = Path(__file__).resolve().parent
REF = Path(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")


def main() -> int:
    sys.path.insert(0, str(REF))
    from triattention.methods.triattention import TriAttention

    out = {}
    for name, (layers, hq, hkv, t, decode_start, keep, seed) in {
        "gqa4": (3, 8, 2, 300, 40, 96, 71), "gqa7_no_prefill": (2, 14, 2, 257, 0, 64, 72), "mha": (4, 4, 4, 130, 17, 100, 73),
    }.items():
        g = torch.Generator().manual_seed(seed)
        raw = torch.randn(layers, hq, t, generator=g) * (1.0 + torch.rand(layers, hq, 1, generator=g)) \
            + torch.randn(layers, hq, 1, generator=g) * 3.0
        raw[0, 1] = 0.25                                   # a constant row: its std is clamped, not replaced by 1
        head_matrix = raw[:, :, decode_start:].reshape(layers * hq, t - decode_start).clone()
        mean = head_matrix.mean(dim=1, keepdim=True)
        std = head_matrix.std(dim=1, unbiased=False, keepdim=True).clamp_min(1e-6)
        normalised = (head_matrix - mean) / std
        fake = types.SimpleNamespace(sampled_heads=[(l, h) for l in range(layers) for h in range(hq)],
                                     num_key_value_groups=hq // hkv, num_key_value_heads=hkv,
                                     config=types.SimpleNamespace(device=torch.device("cpu")))
        keep_idx = TriAttention._select_per_head_independent(fake, normalised, keep, decode_start)
        assert tuple(keep_idx.shape) == (hkv, decode_start + keep)
        out[name] = {"raw": raw, "decode_start": torch.tensor(decode_start), "keep_count": torch.tensor(keep),
                     "num_kv_heads": torch.tensor(hkv), "keep": keep_idx.clone()}
        print(name, tuple(keep_idx.shape))
    torch.save(out, HERE / "hf_select.pt")
    print("written", HERE / "hf_select.pt")
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
