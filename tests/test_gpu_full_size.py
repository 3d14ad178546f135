"""The benchmark configurations at their full sizes, one step each, checked through properties that
do not need the CPU oracle at that size: the step the benchmark times (resident matrix-core kernel)
against the two-pass kernels on the same cache, the guards, the shape of the keep rows, and the
compacted prefix against a torch gather of the rows taken before the step ran.

Oracle-backed parity at sizes the oracle finishes in seconds lives in test_gpu_parity.py; the
chain is oracle = reference goldens, two-pass kernels = oracle, resident = two-pass (there at small
sizes, here at the sizes bench.py runs)."""
from __future__ import annotations

import pytest
import torch

from helpers import assert_keep_within_exact_bound, device_exact_gate, record_swaps
from triattention_amd import ops, synth

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _slots(tables: torch.Tensor, block_size: int, tokens: torch.Tensor) -> torch.Tensor:
    """Flat pool slot of logical token positions; tables [B, pitch], tokens [B, ...] -> [B, ...]."""
    b = torch.arange(tables.shape[0], device=tables.device).view(-1, *([1] * (tokens.ndim - 1)))
    return tables[b, tokens // block_size].long() * block_size + tokens % block_size


def _check_config(index: int, want_path: str = "resident_mfma"):
    w = synth.config(index)
    print(f"config {index}: {w.name}, {w.num_layers} layers, {w.num_seqs} sequences of up to {max(w.seq_lens)} tokens, "
          f"budget {w.budget}, {w.kv_dtype}", flush=True)
    dev = torch.device(DEV)
    tables = synth.make_block_tables(w)
    pool = synth.make_kv_pool(w, tables, dev)
    fp8 = w.kv_dtype == "fp8"
    if fp8:
        caches, k_scales, v_scales = pool
        kv = ops.PagedKV([c[0] for c in caches], [c[1] for c in caches], w.rope_style, k_scales, v_scales)
    else:
        caches, k_scales, v_scales = pool, None, None
        kv = ops.PagedKV.from_kv_caches(caches, w.rope_style)
    qc, qa = synth.make_stats(w, dev)
    fs = torch.ones(w.num_layers, w.num_q_heads, w.head_dim // 2, device=dev)
    sc = ops.ScoreConfig(ops.fold_stats(qc, qa, fs), synth.rope_inv_freq(w, dev), synth.geometric_offsets(device=dev))
    sel = ops.SelectConfig(window_size=w.window_size)
    batch = ops.StepBatch(dev, w.seq_lens, round_start=w.seq_lens, budgets=w.budget, block_tables=tables)
    assert ops.select_path(kv, batch, sc, sel) == want_path
    B, H, L, D, bs = w.num_seqs, w.num_kv_heads, w.num_layers, w.head_dim, w.block_size
    kmax = batch.max_budget
    ks = [min(w.budget, t) for t in w.seq_lens]

    # 1. selection on the two-pass kernels and on the path the benchmark takes; nothing moves yet
    keep_t, fin_t, _ = ops.select_paged(kv, batch, sc, ops.SelectConfig(window_size=w.window_size, allow_resident=False),
                                        want_scores=True)
    keep_r = torch.full((B * H, kmax), -1, dtype=torch.int32, device=dev)
    _, _, ws = ops.select_paged(kv, batch, sc, sel, keep=keep_r)
    assert ws.status() == 0
    kt, kr, fin = keep_t.cpu().long(), keep_r.cpu().long(), fin_t.cpu()
    del keep_t, fin_t
    # The oracle's selection formula on the device, on the raw scores of the two-pass scorer (which small
    # sizes check against the CPU oracle): its fp32 rows, and the double-precision scores that bound where
    # an fp32 evaluation may fall on the other side of the threshold.
    raw, _ = ops.score_paged(kv, batch, sc, ws)
    swapped = swapped_oracle = compared = 0
    for b, (t, k) in enumerate(zip(w.seq_lens, ks)):
        rows = kr[b * H:(b + 1) * H]
        assert bool((rows[:, k:] == -1).all()), f"sequence {b}: entries beyond its own budget were written"
        rows = rows[:, :k]
        assert bool((rows[:, 1:] > rows[:, :-1]).all()) and int(rows.min()) >= 0 and int(rows.max()) < t
        recent = min(w.window_size, t, k)
        assert torch.equal(rows[:, k - recent:], torch.arange(t - recent, t).expand(H, -1)), f"sequence {b}: window"
        want, fin64, bound = device_exact_gate(raw, b, t, H, k, bs, window_size=w.window_size)
        f = fin[b * H:(b + 1) * H, :t]
        scale = float(f[torch.isfinite(f)].abs().max())
        assert bound <= 1e-4 * scale, (b, bound, scale)
        swapped += assert_keep_within_exact_bound(rows, kt[b * H:(b + 1) * H, :k], fin64, k, bound)
        swapped_oracle += assert_keep_within_exact_bound(rows, want, fin64, k, bound)
        compared += H * k
    del raw
    record_swaps(f"full_size_resident_vs_two_pass:{w.name}", swapped, compared)
    record_swaps(f"full_size_resident_vs_device_oracle:{w.name}", swapped_oracle, compared)
    print(f"  resident vs two-pass: {swapped} of {compared} kept indices differ, vs the oracle's formula on the device: "
          f"{swapped_oracle} (all where the fp32 evaluation itself is undecided)", flush=True)

    # 2. what the kept prefix must hold afterwards, gathered from the cache as it is now
    pitch = max(len(tb) for tb in tables)
    tab = torch.tensor([list(tb) + [0] * (pitch - len(tb)) for tb in tables], dtype=torch.int32, device=dev)
    keep3 = keep_r.view(B, H, kmax).long().clamp_min(0)                      # [B, H, kmax]; padding reads token 0
    src = _slots(tab, bs, keep3)                                              # [B, H, kmax]
    dst = _slots(tab, bs, torch.arange(kmax, device=dev).expand(B, kmax))    # [B, kmax]
    live = torch.tensor([[j < k for j in range(kmax)] for k in ks], device=dev)      # [B, kmax]
    head = torch.arange(H, device=dev).view(1, H, 1)

    def rows_of(view, slot_bhk):        # view [nb, bs, H, D] -> [B, H, kmax, D]
        return view.reshape(-1, H, view.shape[-1])[slot_bhk, head]

    def kv_views(l):
        return (kv._keep[0][l], kv._keep[1][l])

    expected = []
    for l in range(L):
        kview, vview = kv_views(l)
        item = [rows_of(kview, src), rows_of(vview, src)]
        if fp8:
            item += [k_scales[l].view(-1, H)[src, head], v_scales[l].view(-1, H)[src, head]]
        expected.append(item)

    # 3. the step the benchmark times: score + select + compact
    keep_s = torch.full((B * H, kmax), -1, dtype=torch.int32, device=dev)
    ops.compress_step(kv, batch, sc, sel, ws, keep_s)
    assert ws.status() == 0
    assert torch.equal(keep_s, keep_r), "the step selected other rows than the selection alone"

    # 4. slots 0..k-1 of every sequence, layer and head hold exactly those rows (and scales)
    dst_bhk = dst.view(B, 1, kmax).expand(B, H, kmax)
    mask = live.view(B, 1, kmax, 1)
    for l in range(L):
        kview, vview = kv_views(l)
        for name, view, want in (("K", kview, expected[l][0]), ("V", vview, expected[l][1])):
            got = rows_of(view, dst_bhk)
            same = (got.view(torch.uint8) == want.view(torch.uint8)) | ~mask
            assert bool(same.all()), f"layer {l} {name}: compacted prefix differs from the gathered rows"
        if fp8:
            for name, arr, want in (("K", k_scales[l], expected[l][2]), ("V", v_scales[l], expected[l][3])):
                got = arr.view(-1, H)[dst_bhk, head]
                assert bool(((got == want) | ~live.view(B, 1, kmax)).all()), f"layer {l} {name} scales"
        expected[l] = None
    print("  compacted prefix bit-equal to the gathered rows in every layer", flush=True)


def test_c1_qwen3_8b_16_sequences_of_16384():
    _check_config(1)


def test_c2_qwen3_32b_8_sequences_of_32768_budget_12000():
    _check_config(2)


def test_c3_ragged_64_sequences():
    _check_config(3)


def test_c4_llama31_fp8_16_sequences_of_16384():
    _check_config(4)
