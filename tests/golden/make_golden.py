#!/usr/bin/env python3
"""Write the golden input/output vectors under tests/golden/.

Runs ONLY in the build container, where the reference checkout is mounted
read-only; the fixtures it writes are plain tensors and travel, the reference
does not.  It imports four reference functions whose exact op order, epsilon
placement and index conventions cannot be fixed by closed forms alone:

* ``triattention.vllm.core.scoring.compute_scores_pytorch``
* ``triattention.vllm.runtime.selector_hf.build_triattention_selector`` (paged
  group branch and per-layer streaming branch; its hard-wired Triton scorer is
  rebound to the reference's own PyTorch scorer, which needs no GPU)
* ``triattention.vllm.runtime.kv_compaction.compact_request_kv_in_place(_per_head)``
* ``triattention.vllm.core.utils.load_frequency_stats`` (per-head key ordering)

Usage:  python tests/golden/make_golden.py [/root/reference]
"""
from __future__ import annotations

import os
import sys
import tempfile
from pathlib import Path

import torch

HERE = Path(__file__).resolve().parent
REF = Path(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")


def synth_stats(seed: int, layers: int, hq: int, f: int):
    g = torch.Generator().manual_seed(seed)
    qc = torch.randn(layers, hq, f, 2, generator=g)
    qa = qc.pow(2).sum(-1).sqrt() + torch.randn(layers, hq, f, generator=g).abs()
    return qc, qa


def synth_keys(seed: int, layers: int, hkv: int, t: int, d: int, omega: torch.Tensor):
    """Post-RoPE bf16 keys: N(0,1) + per-(layer, head, dim) centre, rotated at 0..T-1."""
    g = torch.Generator().manual_seed(seed)
    k = torch.randn(layers, hkv, t, d, generator=g)
    c = torch.randn(layers, hkv, 1, d, generator=g) * (2.0 ** 0.5)
    k = k + c
    ang = torch.arange(t, dtype=torch.float32).unsqueeze(-1) * omega
    cos, sin = torch.cos(ang), torch.sin(ang)
    kr, ki = k[..., : d // 2], k[..., d // 2:]
    rot = torch.cat((kr * cos - ki * sin, ki * cos + kr * sin), dim=-1)
    v = torch.randn(layers, hkv, t, d, generator=g)
    return rot.to(torch.bfloat16), v.to(torch.bfloat16)


def write_stats_file(path: Path, qc, qa, inv_freq, head_dim: int):
    layers, hq, f, _ = qc.shape
    stats = {}
    sampled = []
    for l in range(layers):
        for h in range(hq):
            stats[f"layer{l:02d}_head{h:02d}"] = {
                "q_mean_real": qc[l, h, :, 0].clone(),
                "q_mean_imag": qc[l, h, :, 1].clone(),
                "q_abs_mean": qa[l, h].clone(),
            }
            sampled.append([l, h])
    torch.save({"metadata": {"head_dim": head_dim, "rope_style": "half", "sampled_heads": sampled,
                             "inv_freq": inv_freq.clone()},
                "stats": stats}, path)


def main() -> int:
    sys.path.insert(0, str(REF))
    from triattention.vllm.core.config import TriAttentionConfig
    from triattention.vllm.core import scoring as ref_scoring
    from triattention.vllm.core.utils import load_frequency_stats
    from triattention.vllm.runtime import kv_compaction as ref_kvc
    from triattention.vllm.runtime.config import TriAttentionRuntimeConfig
    from triattention.vllm.runtime import selector_hf as ref_sel

    cpu = torch.device("cpu")

    # ------------------------------------------------------------------ scoring
    out = {}
    for name, (h, t, d, theta, rs, style) in {
        "d128_half": (4, 96, 128, 1e6, 4096, "half"),
        "d64_inter": (3, 50, 64, 1e4, 777, "interleaved"),
    }.items():
        f = d // 2
        omega = 1.0 / (theta ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
        qc, qa = synth_stats(11, 1, h, f)
        keys, _ = synth_keys(12, 1, h, t, d, omega)
        g = torch.Generator().manual_seed(13)
        fs = 0.5 + torch.rand(h, f, generator=g)
        offsets = torch.tensor([float(2 ** j) for j in range(17)])
        case = {"keys": keys[0], "q_mean_complex": qc[0], "q_abs_mean": qa[0], "omega": omega,
                "offsets": offsets, "freq_scale_sq": fs, "round_start": torch.tensor(rs)}
        for agg in ("mean", "max"):
            for dm, dt in ((False, False), (True, False), (False, True)):
                cfg = TriAttentionConfig(device=cpu, compute_dtype=torch.float32, score_aggregation=agg,
                                         disable_mlr=dm, disable_trig=dt, rope_style=style,
                                         use_triton_scoring=False)
                sc = ref_scoring.compute_scores_pytorch(
                    key_states=keys[0].float().unsqueeze(0), cache_positions=None,
                    head_stats={"q_mean_complex": qc[0], "q_abs_mean": qa[0]},
                    omega=omega, offsets=offsets, freq_scale_sq=fs, config=cfg, round_start=rs)
                case[f"scores_{agg}_mlr{int(not dm)}_trig{int(not dt)}"] = sc[0].clone()
        out[name] = case
    torch.save(out, HERE / "scoring_pytorch.pt")

    # ------------------------------------------------------ selector (paged)
    def selector_case(out_name, layers, hq, hkv, d, t, bs, seed):
        f = d // 2
        omega = 1.0 / (1e6 ** (torch.arange(0, d, 2, dtype=torch.float32) / d))
        qc, qa = synth_stats(seed, layers, hq, f)
        keys, vals = synth_keys(seed + 1, layers, hkv, t, d, omega)
        nblk_req = (t + bs - 1) // bs
        pool = nblk_req + 5
        g = torch.Generator().manual_seed(seed + 2)
        block_ids = torch.randperm(pool, generator=g)[:nblk_req].tolist()
        kv_caches = []
        for l in range(layers):
            kv = torch.zeros(2, pool, bs, hkv, d, dtype=torch.bfloat16)
            for n in range(t):
                kv[0, block_ids[n // bs], n % bs] = keys[l, :, n]
                kv[1, block_ids[n // bs], n % bs] = vals[l, :, n]
            kv_caches.append(kv)

        # The selector calls compute_scores_triton; bind it to the PyTorch scorer.
        def _torch_scorer(key_states, cache_positions, head_stats, omega, offsets, freq_scale_sq,
                          config, round_start=None, trig_cache=None):
            return ref_scoring.compute_scores_pytorch(
                key_states=key_states.float(), cache_positions=cache_positions, head_stats=head_stats,
                omega=omega, offsets=offsets, freq_scale_sq=freq_scale_sq, config=config,
                round_start=round_start)
        ref_scoring.compute_scores_triton = _torch_scorer
        # The selector builds its TriAttentionConfig with the default device ("cuda");
        # there is no GPU here, so pin the device argument to CPU.
        import functools
        from triattention.vllm.core import config as ref_core_config
        ref_core_config.TriAttentionConfig = functools.partial(TriAttentionConfig, device=cpu)

        sel_out = {"keys": keys, "values": vals, "q_mean_complex": qc, "q_abs_mean": qa, "omega": omega,
                   "block_ids": torch.tensor(block_ids), "block_size": torch.tensor(bs),
                   "pool_blocks": torch.tensor(pool)}
        with tempfile.TemporaryDirectory() as tmp:
            sp = Path(tmp) / "stats.pt"
            write_stats_file(sp, qc, qa, omega, d)
            meta, head_stats = load_frequency_stats(sp, device=cpu, dtype=torch.float32, num_kv_heads=None)
            sel_out["loader_q_mean_complex"] = torch.stack([head_stats[l]["q_mean_complex"] for l in range(layers)])
            sel_out["loader_q_abs_mean"] = torch.stack([head_stats[l]["q_abs_mean"] for l in range(layers)])
            sel_out["loader_freq_scale_sq"] = torch.stack([head_stats[l]["freq_scale_sq"] for l in range(layers)])
            meta8, hs8 = load_frequency_stats(sp, device=cpu, dtype=torch.float32, num_kv_heads=hkv)
            sel_out["loader_pooled_q_mean_complex"] = torch.stack([hs8[l]["q_mean_complex"] for l in range(layers)])
            sel_out["loader_pooled_q_abs_mean"] = torch.stack([hs8[l]["q_abs_mean"] for l in range(layers)])

            for tag, kw in {
                "default": dict(),
                "chunk64_prefill": dict(score_chunk_max_tokens=64, protect_prefill=True),
                "nonorm": dict(sparse_normalize_scores=False),
                "aggmax": dict(sparse_score_aggregation="max"),
            }.items():
                rc = TriAttentionRuntimeConfig(kv_budget=96, divide_length=16, window_size=12,
                                               sparse_stats_path=sp, **kw)
                os.environ.pop("TRIATTN_RUNTIME_DEBUG_GROUP_PERHEAD_AGG_MODE", None)
                sel_layer, sel_group, status = ref_sel.build_triattention_selector(rc, base_runner=None)
                assert status == "enabled"
                prefill = 20
                res = sel_group(layer_inputs=None, layer_input_iter=None,
                                layer_kv_iter=lambda: [(l, kv_caches[l], block_ids, bs) for l in range(layers)],
                                total_tokens=t, prefill_len=prefill, protect_prefill=rc.protect_prefill,
                                round_start=t + 3, budget_total=96)
                sel_out[f"group_{tag}_keep"] = res["indices"].clone()
                res_l = sel_layer(keys_dense=None, kv_cache=kv_caches[1], block_ids=torch.tensor(block_ids),
                                  block_size=bs, total_tokens=t, prefill_len=prefill,
                                  protect_prefill=rc.protect_prefill, layer_idx=1, round_start=t + 3,
                                  budget_total=96)
                assert res_l["mode"] == "per_head"
                sel_out[f"layer1_{tag}_keep"] = res_l["indices"].clone()
            sel_out["prefill_len"] = torch.tensor(20)
            sel_out["round_start"] = torch.tensor(t + 3)
            sel_out["budget"] = torch.tensor(96)
            sel_out["window"] = torch.tensor(12)
        torch.save(sel_out, HERE / out_name)

    selector_case("selector_group.pt", 3, 8, 2, 64, 300, 16, 21)
    # head_dim 128: the shape the resident kernels of the HIP path take
    selector_case("selector_group_d128.pt", 3, 8, 2, 128, 700, 16, 41)

    # ------------------------------------------------------------ compaction
    comp = {}
    g = torch.Generator().manual_seed(31)
    hkv, d, bs, t, k = 3, 16, 4, 37, 11
    nb = (t + bs - 1) // bs
    pool = nb + 3
    ids = torch.randperm(pool, generator=g)[:nb]
    for axis in (0, 1):
        shape = (2, pool, bs, hkv, d) if axis == 0 else (pool, 2, bs, hkv, d)
        kv = torch.randn(shape, generator=g).to(torch.bfloat16)
        keep_ph = torch.stack([torch.sort(torch.randperm(t, generator=g)[:k]).values for _ in range(hkv)])
        keep_sh = torch.sort(torch.randperm(t, generator=g)[:k]).values
        a = kv.clone()
        n1 = ref_kvc.compact_request_kv_in_place_per_head(a, ids, bs, keep_ph, t, preserve_dropped_tokens=True)
        b = kv.clone()
        n2 = ref_kvc.compact_request_kv_in_place(b, ids, bs, keep_sh, t, preserve_dropped_tokens=True)
        assert n1 == k and n2 == k
        comp[f"axis{axis}"] = {"kv_before": kv, "block_ids": ids, "keep_per_head": keep_ph,
                               "keep_shared": keep_sh, "kv_after_per_head": a, "kv_after_shared": b,
                               "block_size": torch.tensor(bs), "total_tokens": torch.tensor(t)}
    torch.save(comp, HERE / "compaction.pt")

    # ------------------------------------- slice of a shipped calibration file
    # Two layers of the reference's Qwen3-8B statistics (a data file, loaded with
    # weights_only=True), plus what the reference's loader makes of the slice.
    shipped = REF / "triattention" / "calibration" / "for_aime24_experiment" / "qwen3_8b.pt"
    full = torch.load(shipped, map_location="cpu", weights_only=True)
    keep_keys = [k for k in full["stats"] if k.startswith("layer00_") or k.startswith("layer01_")]
    meta = {k: v for k, v in full["metadata"].items() if k != "sampled_heads"}
    meta["sampled_heads"] = [p for p in full["metadata"]["sampled_heads"] if p[0] in (0, 1)]
    sl = {"metadata": meta, "stats": {k: {n: t.clone() for n, t in full["stats"][k].items()} for k in keep_keys}}
    torch.save(sl, HERE / "qwen3_8b_stats_slice.pt")
    sl_noname = {"metadata": {k: v for k, v in meta.items() if k not in ("model_name", "model_path")},
                 "stats": sl["stats"]}
    with tempfile.TemporaryDirectory() as tmp:
        sp = Path(tmp) / "slice.pt"
        torch.save(sl_noname, sp)
        m, hs = load_frequency_stats(sp, device=cpu, dtype=torch.float32, num_kv_heads=None)
        torch.save({"num_attention_heads": torch.tensor(m["num_attention_heads"]),
                    "num_layers": torch.tensor(m["num_layers"]), "head_dim": torch.tensor(m["head_dim"]),
                    "q_mean_complex": torch.stack([hs[l]["q_mean_complex"] for l in (0, 1)]),
                    "q_abs_mean": torch.stack([hs[l]["q_abs_mean"] for l in (0, 1)]),
                    "freq_scale_sq": torch.stack([hs[l]["freq_scale_sq"] for l in (0, 1)])},
                   HERE / "qwen3_8b_stats_slice_loaded.pt")
    print("golden fixtures written to", HERE)
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
