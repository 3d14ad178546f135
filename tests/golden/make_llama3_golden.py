#!/usr/bin/env python3
"""Write tests/golden/llama3_inv_freq.pt: the 64 rotary frequencies of a Llama-3.1-8B-shaped head
(head_dim 128, rope_theta 5e5, llama3 scaling: factor 8, low / high frequency factors 1 / 4,
original context 8192) as `transformers` computes them
(``transformers.modeling_rope_utils.ROPE_INIT_FUNCTIONS["llama3"]``, the routine the reference
reaches through its rotary builders, triattention/common/rope_utils.py:30-90), plus the unscaled
frequencies of the same head.  Runs in the build container (transformers is importable there);
the fixture is 128 floats.

Usage:  python tests/golden/make_llama3_golden.py
"""
from __future__ import annotations

from pathlib import Path
from types import SimpleNamespace

import torch

HERE = Path(__file__).resolve().parent


def main() -> int:
    import transformers
    from transformers.modeling_rope_utils import ROPE_INIT_FUNCTIONS

    scaling = {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
               "original_max_position_embeddings": 8192, "rope_theta": 500000.0}

    class Cfg(SimpleNamespace):
        def standardize_rope_params(self):      # newer transformers call this on the config
            return None

    cfg = Cfg(rope_theta=500000.0, head_dim=128, hidden_size=4096, num_attention_heads=32,
              max_position_embeddings=131072, partial_rotary_factor=1.0, rope_scaling=dict(scaling),
              rope_parameters=dict(scaling))
    inv_freq, attention_scaling = ROPE_INIT_FUNCTIONS["llama3"](cfg, torch.device("cpu"))
    plain = 1.0 / (500000.0 ** (torch.arange(0, 128, 2, dtype=torch.int64).to(torch.float32) / 128))
    assert inv_freq.dtype == torch.float32 and tuple(inv_freq.shape) == (64,)
    torch.save({"llama3_inv_freq": inv_freq.clone(), "default_inv_freq": plain, "attention_scaling": torch.tensor(float(attention_scaling)),
                "rope_theta": torch.tensor(500000.0), "factor": torch.tensor(8.0), "low_freq_factor": torch.tensor(1.0),
                "high_freq_factor": torch.tensor(4.0), "original_max_position_embeddings": torch.tensor(8192),
                "head_dim": torch.tensor(128)}, HERE / "llama3_inv_freq.pt")
    print("transformers", transformers.__version__, "->", HERE / "llama3_inv_freq.pt")
    print("scaled pairs:", int((inv_freq != plain).sum()), "of 64; attention_scaling", float(attention_scaling))
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
