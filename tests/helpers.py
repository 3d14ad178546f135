"""Test helpers: run the oracle end to end on a synthetic workload (CPU) and push the
same inputs through the HIP path."""
from __future__ import annotations

import torch

from oracle import compaction as ocp
from oracle import scoring as osc
from oracle import selection as osel
from triattention_amd import ops, synth


def build_inputs(w: synth.Workload, kv_axis: int = 0):
    """CPU-generated, seeded inputs of a workload."""
    tables = synth.make_block_tables(w)
    pool = synth.make_kv_pool(w, tables, "cpu", kv_axis)
    caches, k_scales, v_scales = pool if w.kv_dtype == "fp8" else (pool, None, None)
    qc, qa = synth.make_stats(w, "cpu")
    omega = synth.rope_inv_freq(w)
    offsets = synth.geometric_offsets()
    fs = torch.ones(w.num_layers, w.num_q_heads, w.head_dim // 2)
    return dict(tables=tables, caches=caches, qc=qc, qa=qa, omega=omega, offsets=offsets, fs=fs, kv_axis=kv_axis,
                k_scales=k_scales, v_scales=v_scales)


def oracle_raw(w, inp, b, round_start, aggregation="mean", disable_mlr=False, disable_trig=False):
    """Raw scores [L][Hq, T_b] of sequence b from the oracle."""
    g = w.num_q_heads // w.num_kv_heads
    out = []
    for l in range(w.num_layers):
        kc, _ = ocp.split_kv(inp["caches"][l], inp["kv_axis"])
        if inp.get("k_scales") is not None:      # fp8: dequantise the pool, then proceed as for bf16
            nb, bs, h, d = kc.shape
            kc = osc.dequant_fp8(kc.reshape(nb * bs, h, d), inp["k_scales"][l]).view(nb, bs, h, d)
        keys = ocp.gather_dense(kc, inp["tables"][b], w.block_size, 0, w.seq_lens[b])[0]      # [Hkv, T, D]
        keys = keys.float().repeat_interleave(g, dim=0)
        out.append(osc.raw_scores(keys, inp["qc"][l], inp["qa"][l], inp["omega"], inp["offsets"], inp["fs"][l],
                                  round_start, aggregation, w.rope_style, disable_mlr, disable_trig))
    return out


def device_objects(w, inp, device, round_start=None, budgets=None, prefill_lens=None, aggregation="mean",
                   disable_mlr=False, disable_trig=False):
    caches = [c.to(device) for c in inp["caches"]]
    if inp.get("k_scales") is not None:
        ks = [t.to(device) for t in inp["k_scales"]]
        vs = [t.to(device) for t in inp["v_scales"]]
        ax = inp["kv_axis"]
        kv = ops.PagedKV([c[0] if ax == 0 else c[:, 0] for c in caches],
                         [c[1] if ax == 0 else c[:, 1] for c in caches], w.rope_style, ks, vs)
    else:
        kv = ops.PagedKV.from_kv_caches(caches, w.rope_style, kv_axis=inp["kv_axis"])
    batch = ops.StepBatch(device, w.seq_lens, round_start=round_start,
                          budgets=budgets if budgets is not None else w.budget,
                          block_tables=inp["tables"], prefill_lens=prefill_lens)
    folded = ops.fold_stats(inp["qc"].to(device), inp["qa"].to(device), inp["fs"].to(device),
                            disable_mlr, disable_trig)
    sc = ops.ScoreConfig(folded, inp["omega"].to(device), inp["offsets"].to(device), aggregation)
    return caches, kv, batch, sc


def score_tolerance(ref: torch.Tensor):
    """1e-3 relative, taken against the per-head RMS of the score (raw scores cross zero)."""
    return 1e-3 * ref.pow(2).mean(dim=-1, keepdim=True).sqrt()


# The contract is "identical kept-index sets except at exact score ties".  fp32 sums taken in
# another order move a selection score by ~1e-6 of the largest one (measured), so an index may
# legitimately differ only when its score lies within KEEP_TIE_TOL (ten times that) of the
# threshold score; selection scores themselves must agree to SELECT_SCORE_TOL.  Both are
# fractions of the largest finite selection score of the rows compared.
KEEP_TIE_TOL = 1e-5
SELECT_SCORE_TOL = 5e-5



def selection_score_tol(raw_rows) -> float:
    """Tolerance for selection scores, as a fraction of the largest one.  The reference's streaming
    variance, sum(x^2) - n * mean^2 in fp32 (runtime/selector_hf.py:902-909), cancels
    kappa = mean(x^2) / var(x) leading digits, so two correct fp32 evaluations that group their sums
    differently disagree by a few eps * kappa in the z-scores: 1.5e-5 at kappa = 130 (head_dim 128
    with the benchmark's key distribution), 9e-5 at kappa = 430 (head_dim 256, measured).
    ``raw_rows``: raw scores with tokens along the last dimension (a tensor or a list of tensors);
    rows of fewer than two tokens have no variance and are left out."""
    rows = raw_rows if isinstance(raw_rows, (list, tuple)) else [raw_rows]
    kappa = 1.0
    for r in rows:
        if r.shape[-1] < 2:
            continue
        r = r.double()
        var = r.var(-1)
        ok = var > 0
        if bool(ok.any()):
            kappa = max(kappa, float((r.pow(2).mean(-1)[ok] / var[ok]).max()))
    return max(SELECT_SCORE_TOL, 8 * 2.0 ** -24 * kappa)


# test id -> (indices swapped at near-ties, indices compared); reported in one line at the end of a run
SWAPS: dict = {}


def record_swaps(case: str, swapped: int, compared: int) -> None:
    have = SWAPS.get(case, (0, 0))
    SWAPS[case] = (have[0] + int(swapped), have[1] + int(compared))


def assert_keep_matches(keep: torch.Tensor, want: torch.Tensor, fin: torch.Tensor, k: int, tie_tol: float):
    """Kept sets equal, except indices whose oracle score is within tie_tol of the
    k-th largest oracle score (fp32 rounding of a different summation order can swap
    those).  Returns the number of swapped indices."""
    swapped = 0
    for h in range(want.shape[0]):
        a, b = set(keep[h].tolist()), set(want[h].tolist())
        if a == b:
            continue
        thr = torch.sort(fin[h], descending=True).values[k - 1]
        for idx in a ^ b:
            assert abs(float(fin[h, idx]) - float(thr)) <= tie_tol, (h, idx, float(fin[h, idx]), float(thr))
            swapped += 1
    return swapped


def exact_gate(raw_by_layer, num_kv_heads: int, **kw):
    """The kept-set gate of one fixture, derived from the fixture itself.  ``raw_by_layer``: the fp32
    raw scores the selection starts from; ``kw``: the selection settings (as for
    ``oracle.selection.group_final_scores``).  Returns (fin64, bound): the selection scores of the
    same formula evaluated in double precision, and the largest distance of the reference's own fp32
    selection scores (the oracle restates its arithmetic operation for operation) from them -- how far
    the reference itself sits from exact arithmetic on this fixture (its streaming variance
    sum(x^2) - n * mean^2 cancels leading digits, runtime/selector_hf.py:902-909)."""
    fin32 = osel.group_final_scores(raw_by_layer, num_kv_heads, **kw)
    fin64 = osel.group_final_scores(raw_by_layer, num_kv_heads, exact=True, **kw)
    finite = torch.isfinite(fin32)
    bound = float((fin32[finite].double() - fin64[finite]).abs().max()) if bool(finite.any()) else 0.0
    return fin64, bound


def device_exact_gate(raw: torch.Tensor, b: int, t: int, num_kv_heads: int, k: int, block_size: int = 16, **kw):
    """The same gate for sizes the CPU oracle does not finish in seconds: the oracle's selection formula
    run on the device on the raw scores the two-pass scorer wrote (``raw``: [B, L, Tmax, A] fp32 from
    ``ops.score_paged``), for sequence ``b`` of ``t`` tokens.  Returns (want, fin64, bound) on the CPU:
    the keep rows of the fp32 evaluation with the reference's chunked sums, the double-precision selection
    scores, and the largest distance between the two evaluations."""
    rows = [raw[b, l, :t].t() for l in range(raw.shape[1])]
    kw.setdefault("chunk_tokens", osel.score_chunk_tokens(block_size, t))
    fin32 = osel.group_final_scores(rows, num_kv_heads, **kw)
    fin64 = osel.group_final_scores(rows, num_kv_heads, exact=True, **kw)
    finite = torch.isfinite(fin32)
    bound = float((fin32[finite].double() - fin64[finite]).abs().max()) if bool(finite.any()) else 0.0
    return osel.topk_ascending(fin32, k).cpu(), fin64.cpu(), bound


def assert_keep_within_exact_bound(keep: torch.Tensor, want: torch.Tensor, fin64: torch.Tensor, k: int, bound: float):
    """Kept sets equal to the reference's, except indices whose exact (double precision) selection score
    lies no further from the exact threshold score (the k-th largest) than ``bound``, the reference's own
    distance from exact arithmetic on this fixture: there the reference's fp32 rounding, not the formula,
    decides which side of the threshold an index falls on.  Returns the number of such indices."""
    swapped = 0
    for h in range(want.shape[0]):
        a, b = set(keep[h].tolist()), set(want[h].tolist())
        if a == b:
            continue
        thr = float(torch.sort(fin64[h], descending=True).values[k - 1])
        for idx in a ^ b:
            gap = abs(float(fin64[h, idx]) - thr)
            assert gap <= bound, (h, idx, float(fin64[h, idx]), thr, gap, bound)
            swapped += 1
    return swapped


_TUNE_ENV = {"TRIATTN_RESIDENT_KERNEL": "resident_kernel", "TRIATTN_RESIDENT_WORKGROUPS": "resident_workgroups",
             "TRIATTN_RESIDENT_LAYER_SPLIT": "layer_split", "TRIATTN_MAX_KERNEL": "max_kernel"}


def tune(**settings):
    """Process-wide settings of the library for the rest of the test (``tri_set_tuning``; an autouse
    fixture puts the defaults back after every test): ``resident_kernel`` ("auto" / "mfma" / "valu" /
    "off"), ``resident_workgroups``, ``layer_split``, ``max_kernel`` ("auto" / "valu", "mfma" = auto),
    ``resident_wait_us`` (None: the default of two seconds).  Keys may also be given by the names of the
    environment variables the Python layer reads at load time."""
    from triattention_amd import _lib
    for name, value in settings.items():
        name = _TUNE_ENV.get(name, name)
        key = _lib.tuning._KEYS[name]
        if name == "resident_kernel":
            value = _lib.RESIDENT_KERNEL_CHOICES[value] if isinstance(value, str) else int(value)
        elif name == "max_kernel":
            value = {"auto": 0, "mfma": 0, "valu": 1}[value] if isinstance(value, str) else int(value)
        elif name == "resident_wait_us" and value is None:
            value = TUNING_DEFAULTS[key]
        _lib.set_tuning(key, int(value))


TUNING_DEFAULTS = {0: 0, 1: 0, 2: -1, 3: 0, 4: 2_000_000}


def reset_tuning():
    from triattention_amd import _lib
    for key, value in TUNING_DEFAULTS.items():
        _lib.set_tuning(key, value)
