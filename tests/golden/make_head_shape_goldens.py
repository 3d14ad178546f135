#!/usr/bin/env python3
"""Write tests/golden/selector_c2_shape.pt and selector_gpt_oss_shape.pt: keep sets of the
reference's group selector (triattention/vllm/runtime/selector_hf.py:813-1033) at two more head
shapes the benchmark and the shipped statistics name, for one request of 5000 cached tokens that
crosses the reference's 4096-token scoring chunk:

* ``c2``: 64 query / 8 KV heads of 128 (Qwen3-32B attention; eight query heads per KV head), budget
  1850 of 5000 (the 37 % keep ratio of the benchmark's 12000 of 32768), synthetic statistics;
* ``gpt_oss``: 64 query / 8 KV heads of 64 with layers 0 and 1 of the statistics the reference ships
  for GPT-OSS-120B (``triattention/vllm/stats/gpt_oss_120b_stats.pt``) and the rotary frequencies
  that file's own metadata describes (YaRN: theta 150000, factor 32, beta_fast 32, beta_slow 1,
  original context 4096), computed by ``transformers.modeling_rope_utils.ROPE_INIT_FUNCTIONS["yarn"]``
  and handed to the reference through ``metadata["inv_freq"]`` (its loader's first choice,
  core/utils.py:81-92; the model name is left out so that nothing is fetched).

Runs ONLY in the build container, where the reference checkout is mounted read-only.  Keys are not
stored: ``hashed_inputs.hashed_rows`` rebuilds them bit for bit from the seed.  As in make_golden.py the
selector's hard-wired Triton scorer is rebound to the reference's own PyTorch scorer.

Usage:  python tests/golden/make_head_shape_goldens.py [/root/reference]
"""
from __future__ import annotations

import functools
import os
import sys
import tempfile
from pathlib import Path
from types import SimpleNamespace

import torch

HERE = Path(__file__).resolve().parent
REF = Path(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
sys.path.insert(0, str(HERE))

from hashed_inputs import checksum, hashed_rows          # noqa: E402
from make_golden import synth_stats, write_stats_file     # noqa: E402

T, BS, WINDOW, PREFILL = 5000, 16, 128, 300
SHAPES = {
    # name: layers, query heads, KV heads, head_dim, budget, seeds (keys, stats, table)
    "c2": dict(layers=3, hq=64, hkv=8, d=128, budget=1850, seeds=(511, 512, 513)),
    "gpt_oss": dict(layers=2, hq=64, hkv=8, d=64, budget=2048, seeds=(521, 0, 523)),
}


def yarn_inv_freq(meta: dict) -> torch.Tensor:
    from transformers.modeling_rope_utils import ROPE_INIT_FUNCTIONS
    scaling = dict(meta["rope_scaling"])
    scaling["rope_theta"] = float(meta["rope_theta"])

    class Cfg(SimpleNamespace):
        def standardize_rope_params(self):
            return None

    cfg = Cfg(rope_theta=float(meta["rope_theta"]), head_dim=int(meta["head_dim"]),
              hidden_size=int(meta["head_dim"]) * int(meta["num_attention_heads"]),
              num_attention_heads=int(meta["num_attention_heads"]), max_position_embeddings=131072,
              partial_rotary_factor=1.0, rope_scaling=dict(scaling), rope_parameters=dict(scaling))
    inv_freq, attention_scaling = ROPE_INIT_FUNCTIONS["yarn"](cfg, torch.device("cpu"))
    assert inv_freq.dtype == torch.float32 and tuple(inv_freq.shape) == (int(meta["head_dim"]) // 2,)
    return inv_freq.clone(), float(attention_scaling)


def main() -> int:
    sys.path.insert(0, str(REF))
    from triattention.vllm.core import config as ref_core_config
    from triattention.vllm.core import scoring as ref_scoring
    from triattention.vllm.core.config import TriAttentionConfig
    from triattention.vllm.runtime import selector_hf as ref_sel
    from triattention.vllm.runtime.config import TriAttentionRuntimeConfig

    cpu = torch.device("cpu")

    def _torch_scorer(key_states, cache_positions, head_stats, omega, offsets, freq_scale_sq, config,
                      round_start=None, trig_cache=None):
        return ref_scoring.compute_scores_pytorch(
            key_states=key_states.float(), cache_positions=cache_positions, head_stats=head_stats, omega=omega,
            offsets=offsets, freq_scale_sq=freq_scale_sq, config=config, round_start=round_start)
    ref_scoring.compute_scores_triton = _torch_scorer
    ref_core_config.TriAttentionConfig = functools.partial(TriAttentionConfig, device=cpu)

    for name, shp in SHAPES.items():
        layers, hq, hkv, d, budget = shp["layers"], shp["hq"], shp["hkv"], shp["d"], shp["budget"]
        key_seed, stats_seed, table_seed = shp["seeds"]
        extra = {}
        if name == "gpt_oss":
            shipped = torch.load(REF / "triattention" / "vllm" / "stats" / "gpt_oss_120b_stats.pt", map_location="cpu",
                                 weights_only=True)
            meta = shipped["metadata"]
            assert int(meta["head_dim"]) == d and int(meta["num_attention_heads"]) == hq and int(meta["num_kv_heads"]) == hkv
            omega, attention_scaling = yarn_inv_freq(meta)
            qc = torch.stack([torch.stack([torch.stack((shipped["stats"][f"layer{l:02d}_head{h:02d}"]["q_mean_real"],
                                                        shipped["stats"][f"layer{l:02d}_head{h:02d}"]["q_mean_imag"]), -1)
                                           for h in range(hq)]) for l in range(layers)]).float()
            qa = torch.stack([torch.stack([shipped["stats"][f"layer{l:02d}_head{h:02d}"]["q_abs_mean"] for h in range(hq)])
                              for l in range(layers)]).float()
            extra = {"attention_scaling": torch.tensor(attention_scaling), "rope_theta": torch.tensor(float(meta["rope_theta"])),
                     "yarn_factor": torch.tensor(float(meta["rope_scaling"]["factor"]))}
        else:
            omega = 1.0 / (1e6 ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
            qc, qa = synth_stats(stats_seed, layers, hq, d // 2)
        keys = hashed_rows(key_seed, layers, hkv, T, d)
        nblk = (T + BS - 1) // BS
        pool = nblk + 37
        block_ids = torch.randperm(pool, generator=torch.Generator().manual_seed(table_seed))[:nblk]
        slot_block = block_ids[torch.arange(T) // BS]
        slot_off = torch.arange(T) % BS
        kv_caches = []
        for l in range(layers):
            kv = torch.zeros(2, pool, BS, hkv, d, dtype=torch.bfloat16)
            kv[0, slot_block, slot_off] = keys[l].transpose(0, 1)
            kv_caches.append(kv)
        out = {"q_mean_complex": qc, "q_abs_mean": qa, "omega": omega, "block_ids": block_ids,
               "key_seed": torch.tensor(key_seed), "key_checksum": torch.tensor(checksum(keys)),
               "shape": torch.tensor([layers, hq, hkv, d, T, BS]), "pool_blocks": torch.tensor(pool),
               "budget": torch.tensor(budget), "window": torch.tensor(WINDOW), "prefill_len": torch.tensor(PREFILL),
               "round_start": torch.tensor(T), **extra}
        with tempfile.TemporaryDirectory() as tmp:
            sp = Path(tmp) / "stats.pt"
            write_stats_file(sp, qc, qa, omega, d)
            for tag, kw in {"default": dict(), "chunk64_prefill": dict(score_chunk_max_tokens=64, protect_prefill=True)}.items():
                rc = TriAttentionRuntimeConfig(kv_budget=budget, divide_length=128, window_size=WINDOW,
                                               sparse_stats_path=sp, **kw)
                os.environ.pop("TRIATTN_RUNTIME_DEBUG_GROUP_PERHEAD_AGG_MODE", None)
                _, sel_group, status = ref_sel.build_triattention_selector(rc, base_runner=None)
                assert status == "enabled"
                res = sel_group(layer_inputs=None, layer_input_iter=None,
                                layer_kv_iter=lambda: [(l, kv_caches[l], block_ids.tolist(), BS) for l in range(layers)],
                                total_tokens=T, prefill_len=PREFILL, protect_prefill=rc.protect_prefill,
                                round_start=T, budget_total=budget)
                keep = res["indices"]
                assert tuple(keep.shape) == (hkv, budget) and bool((keep[:, 1:] > keep[:, :-1]).all())
                out[f"group_{tag}_keep"] = keep.to(torch.int32).clone()
                print(name, tag, "kept", tuple(keep.shape), "tokens beyond the first chunk:", int((keep >= 4096).sum()))
        torch.save(out, HERE / f"selector_{name}_shape.pt")
        print("written", HERE / f"selector_{name}_shape.pt")
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
