#!/usr/bin/env python3
"""Write tests/golden/selector_c1_shape.pt: keep sets of the reference's group selector at the
head shape of the benchmarked step (32 query / 8 KV heads of 128, block size 16, budget 2048,
window 128) for one request whose 5000 cached tokens cross the reference's 4096-token scoring
chunk, so its streaming variance spans two chunks and its chunked top-k merge
(triattention/vllm/runtime/selector_hf.py:990-1019) actually merges.

Runs ONLY in the build container, where the reference checkout is mounted read-only.  The keys are
not stored: ``hashed_inputs.hashed_rows`` rebuilds them bit for bit from the seed (the fixture
holds a checksum), so the file stays small.  As in make_golden.py the selector's hard-wired Triton
scorer is rebound to the reference's own PyTorch scorer, which needs no GPU.

Usage:  python tests/golden/make_c1_shape_golden.py [/root/reference]
"""
from __future__ import annotations

import functools
import os
import sys
import tempfile
from pathlib import Path

import torch

HERE = Path(__file__).resolve().parent
REF = Path(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
sys.path.insert(0, str(HERE))

from hashed_inputs import checksum, hashed_rows          # noqa: E402
from make_golden import synth_stats, write_stats_file     # noqa: E402

LAYERS, HQ, HKV, D, T, BS, BUDGET, WINDOW, PREFILL = 4, 32, 8, 128, 5000, 16, 2048, 128, 300
KEY_SEED, STATS_SEED, TABLE_SEED = 501, 502, 503


def main() -> int:
    sys.path.insert(0, str(REF))
    from triattention.vllm.core import config as ref_core_config
    from triattention.vllm.core import scoring as ref_scoring
    from triattention.vllm.core.config import TriAttentionConfig
    from triattention.vllm.runtime import selector_hf as ref_sel
    from triattention.vllm.runtime.config import TriAttentionRuntimeConfig

    cpu = torch.device("cpu")
    omega = 1.0 / (1e6 ** (torch.arange(0, D, 2, dtype=torch.float32) / D))
    qc, qa = synth_stats(STATS_SEED, LAYERS, HQ, D // 2)
    keys = hashed_rows(KEY_SEED, LAYERS, HKV, T, D)
    nblk = (T + BS - 1) // BS
    pool = nblk + 37
    block_ids = torch.randperm(pool, generator=torch.Generator().manual_seed(TABLE_SEED))[:nblk]
    slot_block = block_ids[torch.arange(T) // BS]
    slot_off = torch.arange(T) % BS
    kv_caches = []
    for l in range(LAYERS):
        kv = torch.zeros(2, pool, BS, HKV, D, dtype=torch.bfloat16)
        kv[0, slot_block, slot_off] = keys[l].transpose(0, 1)
        kv_caches.append(kv)

    def _torch_scorer(key_states, cache_positions, head_stats, omega, offsets, freq_scale_sq, config,
                      round_start=None, trig_cache=None):
        return ref_scoring.compute_scores_pytorch(
            key_states=key_states.float(), cache_positions=cache_positions, head_stats=head_stats, omega=omega,
            offsets=offsets, freq_scale_sq=freq_scale_sq, config=config, round_start=round_start)
    ref_scoring.compute_scores_triton = _torch_scorer
    ref_core_config.TriAttentionConfig = functools.partial(TriAttentionConfig, device=cpu)

    out = {"q_mean_complex": qc, "q_abs_mean": qa, "omega": omega, "block_ids": block_ids,
           "key_seed": torch.tensor(KEY_SEED), "key_checksum": torch.tensor(checksum(keys)),
           "shape": torch.tensor([LAYERS, HQ, HKV, D, T, BS]), "pool_blocks": torch.tensor(pool),
           "budget": torch.tensor(BUDGET), "window": torch.tensor(WINDOW), "prefill_len": torch.tensor(PREFILL),
           "round_start": torch.tensor(T)}
    with tempfile.TemporaryDirectory() as tmp:
        sp = Path(tmp) / "stats.pt"
        write_stats_file(sp, qc, qa, omega, D)
        for tag, kw in {"default": dict(), "chunk64_prefill": dict(score_chunk_max_tokens=64, protect_prefill=True)}.items():
            rc = TriAttentionRuntimeConfig(kv_budget=BUDGET, divide_length=128, window_size=WINDOW,
                                           sparse_stats_path=sp, **kw)
            os.environ.pop("TRIATTN_RUNTIME_DEBUG_GROUP_PERHEAD_AGG_MODE", None)
            _, sel_group, status = ref_sel.build_triattention_selector(rc, base_runner=None)
            assert status == "enabled"
            res = sel_group(layer_inputs=None, layer_input_iter=None,
                            layer_kv_iter=lambda: [(l, kv_caches[l], block_ids.tolist(), BS) for l in range(LAYERS)],
                            total_tokens=T, prefill_len=PREFILL, protect_prefill=rc.protect_prefill,
                            round_start=T, budget_total=BUDGET)
            keep = res["indices"]
            assert tuple(keep.shape) == (HKV, BUDGET) and bool((keep[:, 1:] > keep[:, :-1]).all())
            out[f"group_{tag}_keep"] = keep.to(torch.int32).clone()
            print(tag, "kept", tuple(keep.shape), "tokens beyond the first chunk:", int((keep >= 4096).sum()))
    torch.save(out, HERE / "selector_c1_shape.pt")
    print("written", HERE / "selector_c1_shape.pt")
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
