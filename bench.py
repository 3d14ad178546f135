#!/usr/bin/env python3
"""Benchmark of the KV compression step (score + select + compact) on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 1] [--no-cpu-baseline]

A step is one pass of the hot path over one batch of synthetic paged KV: every layer
of every sequence is scored, the budget is selected per KV head, K and V are compacted
in place.  Inputs are resident in HBM before the timed region; compaction is
destructive, so the blocks it overwrites are restored between steps outside the timed
region (each step is timed with HIP events on the stream the kernels run on).
Prints one JSON line.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0   # MI355X HBM3E, published

# HBM bytes one launch of the dominant kernel moves on the C1 workload, from two rocprofv3
# --pmc runs of this script (FETCH_SIZE x 2.0 + WRITE_SIZE x 1.0 KiB; the factors are what
# the same counters read for the 1 GiB copies of --copy-calibration).  Keyed by
# (workload, path); absent = not measured.
MEASURED_TRAFFIC_BYTES = {
    ("c1_qwen3_8b_36l_b16_16k", "resident_mfma"): (9_472_453 * 1024 * 2 + 12_800 * 1024,     # fused_mfma_kernel
                                                    "profiles/c1_step_hbm_counters.txt"),
}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", type=int, default=1, help="workload index 0..4 (default 1: 36 layers, 16 x 16384 tokens)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--sustained-steps", type=int, default=400,
                    help="back-to-back steps of the sustained (warm clocks) measurement after the timed region; 0: skip")
    ap.add_argument("--no-parity-check", action="store_true",
                    help="skip the keep-set comparison of the timed path with the two-pass kernels (and, with the CPU "
                         "baseline, with the oracle on sequence 0)")
    ap.add_argument("--cpu-layers", type=int, default=36, help="layers of one sequence the CPU baseline scores")
    ap.add_argument("--seq-len", type=int, default=0,
                    help="override every sequence's cached length (e.g. budget + 128 for the steady-state step)")
    ap.add_argument("--sequences", type=int, default=0, help="override the number of sequences (with --seq-len)")
    ap.add_argument("--no-scattered-pool", "--no-exact-pool", dest="no_scattered_pool", action="store_true",
                    help="skip the second leg: the same step with the live blocks scattered over a pool four times "
                         "their number (at most 160 GiB)")
    ap.add_argument("--pool-occupancy", type=float, default=0.0,
                    help="live blocks / blocks of the shared pool.  Default: the workload's own where it names one "
                         "(config 3: 0.8), otherwise 1 (a pool of exactly the live blocks)")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="skip the brief legs over the other benchmark configurations (default invocation only)")
    ap.add_argument("--other-steps", type=int, default=10, help="timed steps of each of the other configurations")
    ap.add_argument("--graph-steps", type=int, default=20,
                    help="replays of the step captured into a HIP graph (resident path; 0: skip)")
    ap.add_argument("--kv-dtype", choices=["bf16", "fp16"], default="",
                    help="key/value dtype of the synthetic cache (default: the workload's own)")
    ap.add_argument("--layers", type=int, default=0, help="override the number of layers")
    ap.add_argument("--q-heads", type=int, default=0, help="override the number of query heads")
    ap.add_argument("--kv-heads", type=int, default=0, help="override the number of KV heads")
    ap.add_argument("--head-dim", type=int, default=0, help="override the head dimension")
    ap.add_argument("--aggregation", choices=["mean", "max"], default="mean",
                    help="aggregation of the score over the position offsets (the reference's default: mean)")
    ap.add_argument("--two-pass", action="store_true",
                    help="time the score_paged + select pair (raw scores through HBM) instead of select_paged")
    ap.add_argument("--hook-latency", action="store_true",
                    help="also time the runner hook for one request and the batch hook for a batch of requests of "
                         "budget + 128 tokens, host side included")
    ap.add_argument("--flat-pool", action="store_true",
                    help="also time one request on a token-level pool (the SGLang backend's cache) through flat_pool")
    ap.add_argument("--query-stats", action="store_true",
                    help="also time the calibration statistics kernel on one layer's captured queries "
                         "(32 heads x 32768 tokens x 128, bf16)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run three plain 1 GiB device copies (reference point for HBM byte counters)")
    return ap.parse_args()


def cpu_baseline(w, layers: int, seq0=None):
    """The CPU oracle (a port of the reference's PyTorch path) on a bounded sample: one sequence,
    `layers` layers.  With ``seq0`` (the blocks of sequence 0 of the GPU run, copied to the host:
    ``{"caches": [L x [2, nblk, bs, H, D]], "qc", "qa"}``) the oracle scores exactly what the GPU
    scored, and its keep set is returned for comparison; otherwise same shapes and seeded
    distributions."""
    from oracle import compaction as ocp
    from oracle import scoring as osc
    from oracle import selection as osel
    from triattention_amd import synth

    torch.set_num_threads(os.cpu_count() or 1)
    layers = min(layers, w.num_layers)
    sample = w.scaled(seq_lens=(w.seq_lens[0],), num_layers=layers, kv_dtype="bf16" if w.kv_dtype == "fp8" else w.kv_dtype)
    if seq0 is not None and layers == w.num_layers:
        caches, qc, qa = seq0["caches"], seq0["qc"], seq0["qa"]
        tables = [list(range(int(caches[0].shape[1])))]
    else:
        seq0 = None
        tables = synth.make_block_tables(sample)
        caches = synth.make_kv_pool(sample, tables, "cpu")
        qc, qa = synth.make_stats(sample, "cpu")
    omega, offsets = synth.rope_inv_freq(sample), synth.geometric_offsets()
    fs = torch.ones(layers, sample.num_q_heads, sample.head_dim // 2)
    t = sample.seq_lens[0]
    g = sample.num_q_heads // sample.num_kv_heads
    t0 = time.perf_counter()
    raw = []
    for l in range(layers):
        kc, _ = ocp.split_kv(caches[l])
        keys = ocp.gather_dense(kc, tables[0], sample.block_size, 0, t)[0].float().repeat_interleave(g, dim=0)
        raw.append(osc.raw_scores(keys, qc[l], qa[l], omega, offsets, fs[l], t))
    keep, fin = osel.group_keep_per_head(raw, sample.num_kv_heads, sample.budget, window_size=sample.window_size,
                                         chunk_tokens=osel.score_chunk_tokens(sample.block_size, t))
    for l in range(layers):
        ocp.compact_per_head(caches[l], tables[0], sample.block_size, keep, t, full_permutation=True)
    dt = time.perf_counter() - t0
    # one "key" is one cached token across ALL layers of the model: scale the sample's layer count up
    keys_per_s = t / (dt * w.num_layers / layers)
    what = "sequence 0 of the GPU run (its own keys and statistics)" if seq0 is not None else "1 sequence"
    out = {"value": keys_per_s, "unit": "keys/s", "cores": torch.get_num_threads(), "kind": "port",
           "sample": f"{what} x {t} tokens x {layers} of {w.num_layers} layers, {dt:.2f} s on the host; "
                     f"rate scaled to all {w.num_layers} layers"}
    return out, (keep, fin) if seq0 is not None else None


def keep_differences(got: torch.Tensor, want: torch.Tensor, fin: torch.Tensor, ks, heads: int, tie: float = 1e-5,
                     lens=None):
    """Kept indices of ``got`` that ``want`` does not hold (rows = sequences x heads, CPU tensors), and
    how many of them are near-ties: selection score within ``tie`` x the largest finite score of the
    row's sequence of the row's threshold (the k-th largest of ``fin``).  ``lens``: the sequences' own
    lengths (rows of a ragged batch hold nothing meaningful beyond them)."""
    diff = near = 0
    for r in range(got.shape[0]):
        k = ks[r // heads]
        a, b = set(got[r, :k].tolist()), set(want[r, :k].tolist())
        if a == b:
            continue
        row = fin[r] if lens is None else fin[r, :lens[r // heads]]
        finite = row[torch.isfinite(row)]
        scale = float(finite.abs().max()) if finite.numel() else 1.0
        thr = float(torch.sort(row, descending=True).values[k - 1])
        for idx in a - b:
            diff += 1
            near += abs(float(row[idx]) - thr) <= tie * scale
    return diff, near


def hook_latency(w, dev, calls: int = 30, requests: int = 1):
    """Wall time of the runner hook for requests of budget + 128 tokens (the steady state of a
    long generation): host logic, launches and host reads, synchronised before and after.
    One request: one call of ``triattention_apply_compression``.  Several: the same requests
    through one call of ``triattention_apply_compression_batch`` and, for comparison, through
    the one-by-one hook in a loop."""
    import tempfile
    import types
    from triattention_amd import synth
    from triattention_amd.runtime import CompressionSignal, TriAttentionRuntimeConfig, install_runner_compression_hook

    t = w.budget + 128
    qc, qa = synth.make_stats(w)
    entries = {f"layer{l:02d}_head{h:02d}": {"q_mean_real": qc[l, h, :, 0].clone(), "q_mean_imag": qc[l, h, :, 1].clone(),
                                            "q_abs_mean": qa[l, h].clone()}
               for l in range(w.num_layers) for h in range(w.num_q_heads)}
    with tempfile.TemporaryDirectory() as tmp:
        path = os.path.join(tmp, "stats.pt")
        torch.save({"metadata": {"head_dim": w.head_dim, "rope_style": w.rope_style,
                                 "inv_freq": synth.rope_inv_freq(w).clone(),
                                 "sampled_heads": [[l, h] for l in range(w.num_layers) for h in range(w.num_q_heads)]},
                    "stats": entries}, path)
        cfg = TriAttentionRuntimeConfig(kv_budget=w.budget, divide_length=128, window_size=w.window_size,
                                        sparse_stats_path=path, log_decisions=False)
        per_req = (t + w.block_size - 1) // w.block_size + 8
        nblk = per_req * requests
        perm = torch.randperm(nblk + 64, generator=torch.Generator().manual_seed(1))[:nblk].tolist()
        ids = {f"r{i}": perm[i * per_req:(i + 1) * per_req] for i in range(requests)}
        caches = [torch.randn(2, nblk + 64, w.block_size, w.num_kv_heads, w.head_dim, device=dev).to(torch.bfloat16)
                  for _ in range(w.num_layers)]
        reqs = {rid: types.SimpleNamespace(num_computed_tokens=t, block_ids=(list(b),)) for rid, b in ids.items()}
        runner = types.SimpleNamespace(requests=reqs, kv_caches=caches,
                                       cache_config=types.SimpleNamespace(block_size=w.block_size))
        install_runner_compression_hook(runner, cfg)
        sched = types.SimpleNamespace(num_scheduled_tokens={rid: 1 for rid in reqs})

        def signals():
            for rid, req in reqs.items():
                req.num_computed_tokens = t
                req.block_ids = (list(ids[rid]),)
            return {rid: CompressionSignal(req_id=rid, should_compress=True, reason="length_threshold",
                                           estimated_cache_len=t + 1, step=1, kv_usage=None, protect_prefill=False,
                                           prefill_len=0, scheduled_tokens=1) for rid in reqs}

        def one_by_one():
            return [runner.triattention_apply_compression(req_id=rid, signal=sig, scheduler_output=sched)
                    for rid, sig in signals().items()]

        def together():
            return list(runner.triattention_apply_compression_batch(signals=signals(), scheduler_output=sched).values())

        def timed(fn):
            for _ in range(3):
                res = fn()
            if not all(r["applied"] for r in res):
                raise RuntimeError(f"hook did not compress: {res}")
            times = []
            for _ in range(calls):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                fn()
                torch.cuda.synchronize()
                times.append((time.perf_counter() - t0) * 1e3)
            times.sort()
            return {"ms_median": times[len(times) // 2], "ms_min": times[0], "ms_max": times[-1]}

        out = {"requests": requests, "tokens": t, "budget": w.budget, "layers": w.num_layers, "calls": calls}
        if requests == 1:
            out.update(timed(one_by_one))
        else:
            out["batch_hook"] = timed(together)
            out["one_by_one"] = timed(one_by_one)
    return out


def query_stats_leg(dev, heads: int = 32, tokens: int = 32768, dim: int = 128, calls: int = 20):
    """ops.query_stats on one layer of captured query states in the layout a Hugging Face
    attention module produces them ([1, T, H, D] viewed as [H, T, D]).  The operand that has
    to come from HBM is q_rot: heads * tokens * dim * 2 bytes."""
    from triattention_amd import ops

    q = torch.randn(1, tokens, heads, dim, device=dev).to(torch.bfloat16).transpose(1, 2)[0]
    inv = 1e6 ** (-torch.arange(0, dim, 2, device=dev, dtype=torch.float32) / dim)
    ang = torch.arange(tokens, device=dev, dtype=torch.float32)[:, None] * inv[None]
    emb = torch.cat((ang, ang), -1)
    cos, sin = emb.cos().to(torch.bfloat16), emb.sin().to(torch.bfloat16)
    for _ in range(3):
        ops.query_stats(q, cos, sin)
    torch.cuda.synchronize()
    times = []
    for _ in range(calls):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        ops.query_stats(q, cos, sin)
        e1.record()
        torch.cuda.synchronize()
        times.append(e0.elapsed_time(e1))
    times.sort()
    nbytes = heads * tokens * dim * 2
    med = times[len(times) // 2]
    return {"heads": heads, "tokens": tokens, "head_dim": dim, "dtype": "bf16", "ms_median": med,
            "query_bytes": nbytes, "gbs": nbytes / (med * 1e-3) / 1e9, "frac_of_hbm_peak": nbytes / (med * 1e-3) / 1e9 / HBM_PEAK_GBS}


def flat_pool_leg(dev, layers: int = 36, heads: int = 8, q_heads: int = 32, dim: int = 128, tokens: int = 16384,
                  budget: int = 2048, calls: int = 10):
    """One request on a token-level pool (the SGLang backend's cache: per-layer [slots, H, D] buffers, a
    req_to_token table with one slot per token): selection in the backend's order of operations, then
    per-head compaction, through ``triattention_amd.flat_pool``.  One token per block, so the scorer is
    the two-pass vector-unit kernel.  Bytes as for the paged step: every key row once, kept rows of K
    and V read and written."""
    from triattention_amd import flat_pool, ops
    g = torch.Generator(device=dev).manual_seed(77)
    slots = tokens + 64
    k_buffers = [torch.randn(slots, heads, dim, generator=g, device=dev).to(torch.bfloat16) for _ in range(layers)]
    v_buffers = [torch.randn(slots, heads, dim, generator=g, device=dev).to(torch.bfloat16) for _ in range(layers)]
    perm = (torch.randperm(slots - 1, generator=g, device=dev) + 1)[:tokens].to(torch.int32)       # slot 0 is the dummy slot
    req_to_token = torch.zeros(2, tokens + 8, dtype=torch.int32, device=dev)
    req_to_token[1, :tokens] = perm
    f = dim // 2
    qc = torch.randn(layers, q_heads, f, 2, generator=g, device=dev)
    qa = qc.pow(2).sum(-1).sqrt() + torch.randn(layers, q_heads, f, generator=g, device=dev).abs()
    folded = ops.fold_stats(qc, qa, torch.ones(layers, q_heads, f, device=dev))
    inv = 1e6 ** (-torch.arange(0, dim, 2, device=dev, dtype=torch.float32) / dim)
    offsets = torch.tensor([float(2 ** j) for j in range(17)], device=dev)
    score = ops.ScoreConfig(folded, inv, offsets)
    saved_k = [b[perm[:budget].long()].clone() for b in k_buffers]
    saved_v = [b[perm[:budget].long()].clone() for b in v_buffers]
    sel_ms, cmp_ms = [], []
    for i in range(calls + 2):
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
        ev[0].record()
        keep = flat_pool.select_keep_indices_per_head(k_buffers, req_to_token, 1, tokens, score, budget=budget,
                                                      round_start=tokens)
        ev[1].record()
        flat_pool.compact_request_kv_in_place_per_head(k_buffers, v_buffers, req_to_token, 1, keep, tokens)
        ev[2].record()
        torch.cuda.synchronize()
        for b, sk, sv, vb in zip(k_buffers, saved_k, saved_v, v_buffers):              # put the overwritten prefix back
            b[perm[:budget].long()] = sk
            vb[perm[:budget].long()] = sv
        if i >= 2:
            sel_ms.append(ev[0].elapsed_time(ev[1]))
            cmp_ms.append(ev[1].elapsed_time(ev[2]))
    sel_ms.sort()
    cmp_ms.sort()
    row = heads * dim * 2
    score_bytes = layers * tokens * row
    compact_bytes = layers * budget * row * 4
    sm, cm = sel_ms[len(sel_ms) // 2], cmp_ms[len(cmp_ms) // 2]
    total = (score_bytes + compact_bytes) / ((sm + cm) * 1e-3) / 1e9
    return {"layers": layers, "kv_heads": heads, "q_heads": q_heads, "head_dim": dim, "tokens": tokens, "budget": budget,
            "calls": calls, "select_ms_median": sm, "compact_ms_median": cm, "host_included": True,
            "algorithmic_bytes": {"score": score_bytes, "compact": compact_bytes},
            "achieved_gbs": total, "frac_of_hbm_peak": total / HBM_PEAK_GBS}


def pool_bytes_per_block(w) -> int:
    return 2 * w.block_size * w.num_kv_heads * w.head_dim * (1 if w.kv_dtype == "fp8" else 2) * w.num_layers


def default_pool_blocks(w) -> int:
    """Four times the live blocks, at most 160 GiB over all layers."""
    live = sum(w.blocks_per_seq)
    return max(live, min(4 * live, (160 << 30) // pool_bytes_per_block(w)))


class StepRun:
    """One workload resident on the device, and the step that is timed on it.

    Stage boundaries (events): 0 | scores of every key -> selection scores | 1 | top-k | 2 |
    compaction | 3.  Default path: ``select_paged`` (one resident kernel when the shape has one,
    raw scores stay in LDS); ``two_pass``: ``score_paged`` writes the raw scores, ``select``
    normalises and reduces.  Compaction is destructive, so the blocks it overwrites (the first
    ceil(k / block_size) of every sequence) are saved once and restored between steps."""

    def __init__(self, w, dev, sc, sel, force_two_pass: bool):
        from triattention_amd import ops, synth
        self.ops, self.w, self.sc, self.sel = ops, w, sc, sel
        self.tables = synth.make_block_tables(w)
        pool = synth.make_kv_pool(w, self.tables, dev)
        self.k_scales = self.v_scales = None
        if w.kv_dtype == "fp8":
            self.caches, self.k_scales, self.v_scales = pool
            self.kv = ops.PagedKV([c[0] for c in self.caches], [c[1] for c in self.caches], w.rope_style,
                                  self.k_scales, self.v_scales)
        else:
            self.caches = pool
            self.kv = ops.PagedKV.from_kv_caches(self.caches, w.rope_style)
        self.batch = ops.StepBatch(dev, w.seq_lens, round_start=w.seq_lens, budgets=w.budget, block_tables=self.tables)
        self.ws = ops.Workspace(self.kv, self.batch, sc)
        rows = w.num_seqs * w.num_kv_heads
        self.keep = torch.empty(rows, self.batch.max_budget, dtype=torch.int32, device=dev)
        self.fin_buf = torch.empty(rows, self.batch.max_seq_len, dtype=torch.float32, device=dev)
        self.path = "two_pass" if force_two_pass else ops.select_path(self.kv, self.batch, sc, sel)
        self.two_pass = self.path == "two_pass"
        # How the library cuts this step into workgroups (tile length, layer groups, launches).
        self.plan = None if force_two_pass else {k: v for k, v in ops.describe_plan(self.kv, self.batch, sc, sel).items()
                                                 if k != "path"}
        self.raw_buf = None
        if self.two_pass:
            self.raw_buf = torch.empty(w.num_seqs, w.num_layers, self.batch.max_seq_len, w.num_q_heads,
                                       dtype=torch.float32, device=dev)
        nkeep_blocks = (w.budget + w.block_size - 1) // w.block_size
        self.ids = torch.tensor([b for tbl in self.tables for b in tbl[:nkeep_blocks]], device=dev, dtype=torch.long)
        self.saved = [c[:, self.ids].clone() for c in self.caches]
        self.saved_scales = None
        if self.k_scales is not None:
            self.slot = (self.ids.unsqueeze(1) * w.block_size + torch.arange(w.block_size, device=dev)).flatten()
            self.saved_scales = [(ks[self.slot].clone(), vs[self.slot].clone())
                                 for ks, vs in zip(self.k_scales, self.v_scales)]
        torch.cuda.synchronize()

    def restore(self):
        for i, c in enumerate(self.caches):
            c[:, self.ids] = self.saved[i]
            if self.saved_scales is not None:
                self.k_scales[i][self.slot] = self.saved_scales[i][0]
                self.v_scales[i][self.slot] = self.saved_scales[i][1]

    def step(self, events=None):
        """The step as a serving engine issues it: ONE call of the C ABI's ``tri_compress_step`` (score +
        select + compact, one launch sequence); ``events``: a pair recorded around the call."""
        if self.two_pass:
            return self.staged_step(events if events is None else [events[0], None, None, events[1]])
        if events is not None:
            events[0].record()
        self.ops.compress_step(self.kv, self.batch, self.sc, self.sel, self.ws, self.keep)
        if events is not None:
            events[1].record()

    def staged_step(self, events=None):
        """The same kernels issued stage by stage (three calls of the C ABI), with an event at every stage
        boundary: where the step's time goes.  The event records and the separate calls cost some 20 us a
        step, which is why the step itself is timed by ``step``."""
        ops = self.ops
        record = lambda i: events is not None and events[i] is not None and events[i].record()
        if events is not None:
            events[0].record()
        if self.two_pass:
            raw, _ = ops.score_paged(self.kv, self.batch, self.sc, self.ws, out=self.raw_buf)
            record(1)
            ops.select(self.kv, self.batch, self.sc, self.sel, raw, self.ws, keep=self.keep)
        else:
            ops.select_paged(self.kv, self.batch, self.sc, self.sel, self.ws, scores_out=self.fin_buf, want_keep=False)
            record(1)
            ops.topk_batch(self.fin_buf, self.batch, self.w.num_kv_heads, self.keep)
        record(2)
        ops.compact(self.kv, self.batch, self.keep)
        record(3)

    def timed(self, warmup: int, steps: int, staged: bool = False):
        """``warmup`` untimed steps, then ``steps`` timed ones.  Everything is enqueued asynchronously
        on one stream: restore(i-1), then the events and kernels of step i.  The host runs ahead while
        the restore copies execute, so the event pairs bracket GPU time only and restores stay outside
        every timed interval.  Returns (events per step, wall seconds of the timed region): two events
        per step, or four with ``staged`` (stage boundaries)."""
        fn = self.staged_step if staged else self.step
        for _ in range(warmup):
            fn()
            self.restore()
        torch.cuda.synchronize()
        evs = [[torch.cuda.Event(enable_timing=True) for _ in range(4 if staged else 2)] for _ in range(steps)]
        wall0 = time.perf_counter()
        for i in range(steps):
            fn(evs[i])
            if i + 1 < steps:
                self.restore()
        torch.cuda.synchronize()
        return evs, time.perf_counter() - wall0

    def graph_timed(self, warmup: int, steps: int):
        """The same one-call step captured once into a HIP graph and replayed (how the runtime's selector
        issues a step whose shape it has seen before).  Returns the mean milliseconds per replay."""
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            self.step()
        torch.cuda.current_stream().wait_stream(side)
        self.restore()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, capture_error_mode="thread_local"):
            self.step()
        self.restore()
        for _ in range(warmup):
            graph.replay()
            self.restore()
        torch.cuda.synchronize()
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
        for a, b in evs:
            a.record()
            graph.replay()
            b.record()
            self.restore()
        torch.cuda.synchronize()
        return sum(a.elapsed_time(b) for a, b in evs) / steps

    def status_raised(self) -> bool:
        return not self.two_pass and self.ws.status() != 0


def percentile(xs, q: float):
    xs = sorted(xs)
    return xs[min(len(xs) - 1, int(q * len(xs)))]


def measure(run: "StepRun", warmup: int, steps: int) -> dict:
    """Times ``steps`` one-call steps (two events each) and then ``steps`` staged ones (an event at every
    stage boundary) on a resident workload.  ``ms_per_step`` and everything derived from it come from
    the one-call steps; ``stage_ms`` from the staged ones."""
    w = run.w
    mean = lambda xs: sum(xs) / len(xs)
    evs, wall_s = run.timed(warmup, steps)
    step_ms = [e[0].elapsed_time(e[1]) for e in evs]
    if run.status_raised():
        return {"error": "status word raised during the timed steps"}
    run.restore()
    sev, _ = run.timed(1, steps, staged=True)
    if run.status_raised():
        return {"error": "status word raised during the staged steps"}
    run.restore()
    score_ms = [e[0].elapsed_time(e[1]) for e in sev]
    select_ms = [e[1].elapsed_time(e[2]) for e in sev]
    compact_ms = [e[2].elapsed_time(e[3]) for e in sev]
    ms = mean(step_ms)
    algo = w.algorithmic_bytes()
    gbs = algo["total"] / (ms * 1e-3) / 1e9
    return {
        "steps": steps, "ms_per_step": ms, "value": sum(w.seq_lens) / (ms * 1e-3), "achieved_gbs": gbs,
        "frac_of_hbm_peak": gbs / HBM_PEAK_GBS, "path": run.path, "plan": run.plan,
        "stage_ms": {"score": mean(score_ms), "select" if run.two_pass else "topk": mean(select_ms),
                     "compact": mean(compact_ms)},
        "staged_ms_per_step": mean([e[0].elapsed_time(e[3]) for e in sev]),
        "stage_gbs": {"score": algo["score"] / (mean(score_ms) * 1e-3) / 1e9,
                      "compact": algo["compact"] / (mean(compact_ms) * 1e-3) / 1e9},
        "step_ms_p50": percentile(step_ms, 0.5), "step_ms_p99": percentile(step_ms, 0.99),
        "compact_ms_p50": percentile(compact_ms, 0.5), "compact_ms_p99": percentile(compact_ms, 0.99),
        "timed_region_wall_s": wall_s,
    }


def pool_description(w) -> dict:
    return {"pool_blocks_per_layer": w.pool_blocks, "pool_occupancy": round(sum(w.blocks_per_seq) / w.pool_blocks, 4),
            "pool_gib": round(w.pool_blocks * pool_bytes_per_block(w) / 2**30, 1)}


def score_config(w, dev, aggregation: str = "mean"):
    from triattention_amd import ops, synth
    qc, qa = synth.make_stats(w, dev)
    fs = torch.ones(w.num_layers, w.num_q_heads, w.head_dim // 2, device=dev)
    sc = ops.ScoreConfig(ops.fold_stats(qc, qa, fs), synth.rope_inv_freq(w, dev), synth.geometric_offsets(device=dev),
                         aggregation)
    return sc, qc, qa


def gpu_parity(run: "StepRun", keep_timed: torch.Tensor) -> dict:
    """On the pristine cache: the timed path's keep rows again (must reproduce what the timed steps left)
    and against the two-pass kernels' rows, with the near-tie count."""
    ops, w = run.ops, run.w
    heads = w.num_kv_heads
    ks = [min(w.budget, t) for t in w.seq_lens]
    two = ops.SelectConfig(window_size=w.window_size, allow_resident=False)
    ops.select_paged(run.kv, run.batch, run.sc, two if run.two_pass else run.sel, run.ws, scores_out=run.fin_buf,
                     want_keep=False)
    keep_again = ops.topk_batch(run.fin_buf, run.batch, heads)
    keep_tp, fin_tp, _ = ops.select_paged(run.kv, run.batch, run.sc, two, run.ws, want_scores=True)
    torch.cuda.synchronize()
    same = all(torch.equal(keep_again[b * heads:(b + 1) * heads, :k], keep_timed[b * heads:(b + 1) * heads, :k])
               for b, k in enumerate(ks))
    diff, near = keep_differences(keep_again.cpu(), keep_tp.cpu(), fin_tp.cpu(), ks, heads, lens=list(w.seq_lens))
    return {"timed_path": run.path, "kept_indices_compared": sum(ks) * heads, "timed_keep_reproduced": same,
            "vs_two_pass_diff": diff, "vs_two_pass_near_tie_swaps": near, "near_tie_bound": "1e-5 of the largest score",
            "_rows0": keep_again[:heads, :ks[0]].cpu()}


def oracle_seq0(run: "StepRun", qc, qa, rows0: torch.Tensor) -> dict:
    """Sequence 0 of a resident workload through the CPU oracle (its own blocks copied to the host), and
    the GPU's keep rows of that sequence against the oracle's."""
    w = run.w
    blocks0 = torch.tensor(run.tables[0], device=run.caches[0].device, dtype=torch.long)
    seq0 = {"caches": [c[:, blocks0].cpu() for c in run.caches], "qc": qc.cpu(), "qa": qa.cpu()}
    base, (okeep, ofin) = cpu_baseline(w, w.num_layers, seq0)
    diff, near = keep_differences(rows0, okeep, ofin, [int(okeep.shape[1])], w.num_kv_heads)
    return base, {"vs_oracle_seq0_diff": diff, "vs_oracle_seq0_near_tie_swaps": near,
                  "vs_oracle_seq0_compared": int(okeep.numel())}


def other_config(name: str, w, dev, steps: int, oracle: bool) -> dict:
    """One of the other benchmark configurations, briefly: the same measurement as the headline leg, the
    status word checked, the timed path's rows against the two-pass kernels' and (small ones) sequence 0
    against the CPU oracle."""
    t0 = time.perf_counter()
    from triattention_amd import ops
    sc, qc, qa = score_config(w, dev)
    sel = ops.SelectConfig(window_size=w.window_size)
    run = StepRun(w, dev, sc, sel, False)
    out = {"workload": w.name, "layers": w.num_layers, "sequences": w.num_seqs, "tokens_per_sequence": max(w.seq_lens),
           "budget": w.budget, "kv_dtype": w.kv_dtype, **pool_description(w)}
    out.update(measure(run, 2, steps))
    if "error" not in out:
        keep_timed = run.keep.clone()
        run.restore()
        par = gpu_parity(run, keep_timed)
        rows0 = par.pop("_rows0")
        if oracle and w.kv_dtype != "fp8":
            _, vs = oracle_seq0(run, qc, qa, rows0)
            par.update(vs)
        out["parity_check"] = par
    out["algorithmic_bytes"] = w.algorithmic_bytes()
    out["wall_s"] = round(time.perf_counter() - t0, 2)
    del run
    torch.cuda.empty_cache()
    return out


def main() -> int:
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: the path shards by sequence and KV head with no exchange, "
              f"and this build has no multi-GPU leg (got --gpus {args.gpus}).", file=sys.stderr)
        return 2
    if not torch.cuda.is_available():
        print("bench.py needs an MI355X (torch.cuda.is_available() is False)", file=sys.stderr)
        return 2

    from triattention_amd import build as tri_build
    tri_build.ensure_built()          # loads what is built; builds only when there is no library at all
    from triattention_amd import _lib, ops, synth

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    w = synth.config(args.config)
    plain = args.config == 1 and not (args.seq_len or args.layers or args.q_heads or args.kv_heads or args.head_dim
                                      or args.kv_dtype or args.two_pass or args.aggregation != "mean")
    if args.seq_len > 0:
        nseq = args.sequences if args.sequences > 0 else w.num_seqs
        w = w.scaled(name=f"{w.name}_b{nseq}_len{args.seq_len}", seq_lens=(args.seq_len,) * nseq)
    shape = {k: v for k, v in (("num_layers", args.layers), ("num_q_heads", args.q_heads),
                               ("num_kv_heads", args.kv_heads), ("head_dim", args.head_dim)) if v > 0}
    if shape:
        tags = {"num_layers": "layers", "num_q_heads": "q", "num_kv_heads": "kv", "head_dim": "dim"}
        w = w.scaled(name=w.name + "_" + "_".join(f"{tags[k]}{v}" for k, v in shape.items()), **shape)
    if args.kv_dtype and args.kv_dtype != w.kv_dtype:
        if "fp8" in (args.kv_dtype, w.kv_dtype):
            raise SystemExit("--kv-dtype switches between bf16 and fp16; the fp8 workload is --config 4")
        w = w.scaled(name=f"{w.name}_{args.kv_dtype}", kv_dtype=args.kv_dtype)
    # The shared pool.  A workload that names its own occupancy keeps it.  Otherwise the first leg, whose
    # figures are the line's top-level ones, runs on a pool of exactly the live blocks (every block of
    # the pool belongs to a sequence of the batch), and a second leg runs the same step with the live
    # blocks scattered over a pool four times their number (a serving engine's cache spans most of
    # the HBM and a batch's blocks lie scattered over it).
    w_scattered = None
    if args.pool_occupancy > 0:
        if not 0.0 < args.pool_occupancy <= 1.0:
            raise SystemExit("--pool-occupancy is a fraction in (0, 1]")
        w = w.scaled(pool_occupancy=args.pool_occupancy)
    elif w.pool_occupancy == 1.0:
        live = sum(w.blocks_per_seq)
        blocks = default_pool_blocks(w)
        if blocks > live:
            w_scattered = w.scaled(pool_occupancy=live / blocks)
    t_setup = time.perf_counter()
    sc, qc, qa = score_config(w, dev, args.aggregation)
    sel = ops.SelectConfig(window_size=w.window_size)
    run = StepRun(w, dev, sc, sel, args.two_pass)
    setup_s = time.perf_counter() - t_setup
    path, two_pass = run.path, run.two_pass

    m = measure(run, args.warmup, args.steps)
    if "error" in m:
        print("bench.py: the resident kernel raised its status word; the step did not do its work and the "
              "timing is void", file=sys.stderr)
        return 3
    ms_per_step = m["ms_per_step"]
    total_keys = sum(w.seq_lens)
    algo = w.algorithmic_bytes()
    run.step()
    torch.cuda.synchronize()
    keep_timed = run.keep.clone()
    run.restore()

    graph_ms = None
    if not two_pass and args.graph_steps > 0:
        graph_ms = run.graph_timed(2, args.graph_steps)
        if run.status_raised():
            print("bench.py: status word raised during the graph replays", file=sys.stderr)
            return 3

    # Sustained figure: the same step back to back (with the restore copies between, which keep the
    # memory system just as busy) for a few seconds, so the GPU sits at the clocks it holds under
    # this load; the last quarter of the steps is what is reported.
    sustained = None
    if args.sustained_steps > 0:
        n = args.sustained_steps
        tail = max(1, min(100, n // 4))
        sev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(tail)]
        run.restore()
        torch.cuda.synchronize()
        s0 = time.perf_counter()
        for i in range(n):
            j = i - (n - tail)
            run.step(sev[j] if j >= 0 else None)
            run.restore()
        torch.cuda.synchronize()
        s_wall = time.perf_counter() - s0
        if run.status_raised():
            print("bench.py: status word raised during the sustained steps", file=sys.stderr)
            return 3
        tail_ms = sorted(a.elapsed_time(b) for a, b in sev)
        s_ms = sum(tail_ms) / len(tail_ms)
        sustained = {"steps": n, "wall_s": s_wall, "ms_per_step": s_ms, "ms_per_step_of": f"last {tail} steps",
                     "step_ms_p50": tail_ms[len(tail_ms) // 2], "step_ms_max": tail_ms[-1],
                     "value": total_keys / (s_ms * 1e-3), "achieved_gbs": algo["total"] / (s_ms * 1e-3) / 1e9,
                     "frac_of_hbm_peak": algo["total"] / (s_ms * 1e-3) / 1e9 / HBM_PEAK_GBS}

    # Parity of what was timed, outside every timed region: on the pristine cache the timed path's
    # keep rows against the two-pass kernels' and against the CPU oracle on sequence 0.
    parity = None
    cpu = None
    if not args.no_parity_check and args.aggregation == "mean":
        run.restore()
        parity = gpu_parity(run, keep_timed)
        rows0 = parity.pop("_rows0")
        if not args.no_cpu_baseline and w.kv_dtype != "fp8" and args.cpu_layers >= w.num_layers:
            cpu, vs = oracle_seq0(run, qc, qa, rows0)
            parity.update(vs)
    if cpu is None and not args.no_cpu_baseline:
        cpu, _ = cpu_baseline(w, args.cpu_layers)

    if args.aggregation == "mean":
        two_pass_kernel = "score_mean_kernel"
    elif w.kv_dtype == "bf16" and w.head_dim == 128 and _lib.get_tuning(_lib.TUNE_MAX_KERNEL) != 1:
        two_pass_kernel = "score_max_mfma_kernel"
    else:
        two_pass_kernel = "score_max_kernel"
    traffic = MEASURED_TRAFFIC_BYTES.get((w.name, path)) if args.aggregation == "mean" else None
    score_gbs = m["stage_gbs"]["score"]
    out = {
        "metric": "keys scored+compacted/sec & achieved HBM GB/s (% peak), Qwen3-8B 16k ctx",
        "value": m["value"],
        "unit": "keys/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "dtype_note": f"arithmetic in fp32 (accumulation, statistics, selection scores); keys and values stored as {w.kv_dtype}",
        "data": "synthetic",
        "config": {"workload": w.name, "layers": w.num_layers, "sequences": w.num_seqs,
                   "tokens_per_sequence": max(w.seq_lens), "budget": w.budget, "kv_heads": w.num_kv_heads,
                   "q_heads": w.num_q_heads, "head_dim": w.head_dim, "block_size": w.block_size,
                   "kv_dtype": w.kv_dtype, **pool_description(w),
                   "pool_note": ("block tables are a random permutation of a shared pool of pool_blocks_per_layer blocks; "
                                 "scattered_pool (when present) is the same step with the live blocks scattered over a "
                                 "pool four times their number"),
                   "step": "one call of tri_compress_step (score + select + compact), HIP events around the call"},
        "achieved_gbs": m["achieved_gbs"],
        "frac_of_hbm_peak": m["frac_of_hbm_peak"],
        "algorithmic_bytes": algo,
        "stage_ms": m["stage_ms"],
        "staged_ms_per_step": m["staged_ms_per_step"],
        "stage_note": "stage_ms: a second pass of the same steps issued stage by stage with an event at every boundary",
        "stage_gbs": m["stage_gbs"],
        "key_vectors_per_s": total_keys * w.num_layers * w.num_kv_heads / (ms_per_step * 1e-3),
        "compact_ms_p50": m["compact_ms_p50"], "compact_ms_p99": m["compact_ms_p99"],
        "step_ms_p50": m["step_ms_p50"], "step_ms_p99": m["step_ms_p99"],
        "timed_region_wall_s": m["timed_region_wall_s"],
        "setup_s": setup_s,
        "path": path,
        "plan": m["plan"],
        "roofline": {"kernel": {"two_pass": two_pass_kernel, "resident_valu": "fused_select_kernel",
                                "resident_mfma": "fused_mfma_kernel"}[path], "bound": "hbm",
                     "achieved": score_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": score_gbs / HBM_PEAK_GBS,
                     "traffic": traffic[0] if traffic else None,
                     "traffic_source": (traffic[1] + " (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this command, scaled by "
                                        "the same counters on a 1 GiB copy; not measured by this run)") if traffic else None},
    }
    if graph_ms is not None:
        out["graph_replay"] = {"steps": args.graph_steps, "ms_per_step": graph_ms,
                               "frac_of_hbm_peak": algo["total"] / (graph_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                               "what": "the same one-call step captured once into a HIP graph and replayed"}
    if sustained is not None:
        out["sustained"] = sustained
    if parity is not None:
        out["parity_check"] = parity
    # A plain device-to-device copy of 1 GiB on the same box, for scale: bytes read + bytes
    # written per second (outside every timed region of the step).
    src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
    dst = torch.empty_like(src)
    dst.copy_(src)
    c0, c1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    c0.record()
    for _ in range(5):
        dst.copy_(src)
    c1.record()
    torch.cuda.synchronize()
    out["device_copy_gbs"] = 5 * 2 * (1 << 30) / (c0.elapsed_time(c1) * 1e-3) / 1e9
    out["frac_of_device_copy"] = m["achieved_gbs"] / out["device_copy_gbs"]
    del src, dst
    if args.copy_calibration:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        out["copy_calibration_bytes"] = 1 << 30
        del src, dst
    if args.query_stats:
        out["query_stats"] = query_stats_leg(dev)
    if args.flat_pool:
        out["flat_pool"] = flat_pool_leg(dev)
    if args.hook_latency and w.kv_dtype != "fp8":
        out["hook_call"] = hook_latency(w, dev)
        out["hook_batch_call"] = hook_latency(w, dev, calls=20, requests=len(w.seq_lens))
    del run
    torch.cuda.empty_cache()
    if w_scattered is not None and not args.no_scattered_pool:
        run2 = StepRun(w_scattered, dev, sc, sel, args.two_pass)
        leg = {**pool_description(w_scattered), **measure(run2, args.warmup, args.steps)}
        del run2
        torch.cuda.empty_cache()
        out["scattered_pool"] = leg
    if cpu is not None:
        out["cpu_baseline"] = cpu
    # The other benchmark configurations, briefly (the default invocation only).
    if plain and not args.no_other_configs:
        others = {}
        steady = synth.config(1)
        steady = steady.scaled(name=f"{steady.name}_len{steady.budget + 128}",
                               seq_lens=(steady.budget + 128,) * steady.num_seqs)
        for name, wo, oracle in (("c0", synth.config(0), True), ("steady_2176", steady, True),
                                 ("c4", synth.config(4), False), ("c2", synth.config(2), False),
                                 ("c3", synth.config(3), False)):
            try:
                others[name] = other_config(name, wo, dev, args.other_steps, oracle)
            except Exception as exc:      # a leg that fails must not take the headline with it
                others[name] = {"error": f"{type(exc).__name__}: {exc}"}
                torch.cuda.empty_cache()
        out["other_configs"] = others
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
