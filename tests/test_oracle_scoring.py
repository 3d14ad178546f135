"""Pins oracle.scoring: reference-written golden vectors, fp64 brute force, closed
forms and the un-rotated (HF) formulation.  CPU only."""
from __future__ import annotations

import math

import pytest
import torch

from conftest import load_golden
from oracle import rope as orope
from oracle import scoring as osc


def _case_args(case):
    return dict(keys=case["keys"], q_mean_complex=case["q_mean_complex"], q_abs_mean=case["q_abs_mean"],
                omega=case["omega"], offsets=case["offsets"], freq_scale_sq=case["freq_scale_sq"],
                round_start=int(case["round_start"]))


@pytest.mark.parametrize("name,style", [("d128_half", "half"), ("d64_inter", "interleaved")])
@pytest.mark.parametrize("agg", ["mean", "max"])
@pytest.mark.parametrize("mlr,trig", [(1, 1), (0, 1), (1, 0)])
def test_matches_reference_compute_scores_pytorch(name, style, agg, mlr, trig):
    case = load_golden("scoring_pytorch.pt")[name]
    got = osc.raw_scores(**_case_args(case), aggregation=agg, rope_style=style,
                         disable_mlr=not mlr, disable_trig=not trig)
    want = case[f"scores_{agg}_mlr{mlr}_trig{trig}"]
    # Same torch ops in the same order on the same machine: bit-identical.
    assert torch.equal(got, want)


def _brute_force(keys, qc, qa, omega, offsets, fs, round_start, agg, style):
    """fp64 python loops straight from the definition; phase rounded like fp32 t*omega."""
    h, t, d = keys.shape
    f = d // 2
    out = torch.zeros(h, t, dtype=torch.float64)
    kd = keys.double()
    for a in range(h):
        for n in range(t):
            extra = 0.0
            base = [0.0] * len(offsets)
            for i in range(f):
                if style == "half":
                    kr, ki = float(kd[a, n, i]), float(kd[a, n, i + f])
                else:
                    kr, ki = float(kd[a, n, 2 * i]), float(kd[a, n, 2 * i + 1])
                qr, qi = float(qc[a, i, 0]), float(qc[a, i, 1])
                s = float(fs[a, i])
                amp_a = qr * kr + qi * ki
                amp_b = qi * kr - qr * ki
                qabs = math.sqrt(qr * qr + qi * qi + 1e-8)
                extra += (float(qa[a, i]) - qabs) * math.hypot(kr, ki) * s
                for j, o in enumerate(offsets):
                    ph = float((torch.tensor(float(round_start + float(o)), dtype=torch.float32)
                                * omega[i]).item())
                    base[j] += s * (amp_a * math.cos(ph) - amp_b * math.sin(ph))
            agg_v = sum(base) / len(base) if agg == "mean" else max(base)
            out[a, n] = agg_v + extra
    return out


@pytest.mark.parametrize("style", ["half", "interleaved"])
@pytest.mark.parametrize("agg", ["mean", "max"])
def test_brute_force_fp64(style, agg):
    g = torch.Generator().manual_seed(5)
    h, t, d = 2, 5, 16
    keys = torch.randn(h, t, d, generator=g).to(torch.bfloat16)
    qc = torch.randn(h, d // 2, 2, generator=g)
    qa = qc.pow(2).sum(-1).sqrt() + torch.rand(h, d // 2, generator=g)
    omega = orope.default_inv_freq(d, 1e4)
    offsets = osc.geometric_offsets(64)
    fs = 0.5 + torch.rand(h, d // 2, generator=g)
    got = osc.raw_scores(keys, qc, qa, omega, offsets, fs, 100, agg, style)
    want = _brute_force(keys, qc, qa, omega, offsets, fs, 100, agg, style)
    assert torch.allclose(got.double(), want, rtol=0, atol=2e-5)


def test_single_frequency_closed_form():
    # D=2, one offset: s|q||k|cos(t*w + arg q - arg k) + (q_abs - |q|)|k| s
    qr, qi, kr, ki, w, s, qabs, rs, off = 0.7, -1.1, 1.5, 0.25, 0.37, 1.3, 2.0, 10, 4.0
    keys = torch.tensor([[[kr, ki]]])
    got = osc.raw_scores(keys, torch.tensor([[[qr, qi]]]), torch.tensor([[qabs]]), torch.tensor([w]),
                         torch.tensor([off]), torch.tensor([[s]]), rs)
    qm = math.sqrt(qr * qr + qi * qi + 1e-8)
    km = math.hypot(kr, ki)
    want = s * math.hypot(qr, qi) * km * math.cos((rs + off) * w + math.atan2(qi, qr) - math.atan2(ki, kr)) \
        + (qabs - qm) * km * s
    assert abs(float(got) - want) < 1e-5


def test_zero_omega_and_zero_centre():
    g = torch.Generator().manual_seed(6)
    h, t, d = 2, 7, 8
    f = d // 2
    keys = torch.randn(h, t, d, generator=g)
    qc = torch.randn(h, f, 2, generator=g)
    qa = qc.pow(2).sum(-1).sqrt() + 0.5
    fs = torch.ones(h, f)
    offs = osc.geometric_offsets(16)
    # omega = 0: sum_f s Re(q conj k) + extra
    got = osc.raw_scores(keys, qc, qa, torch.zeros(f), offs, fs, 33)
    kr, ki = keys[..., :f], keys[..., f:]
    re = (qc[..., 0].unsqueeze(1) * kr + qc[..., 1].unsqueeze(1) * ki).sum(-1)
    extra = ((qa - torch.sqrt(qc.pow(2).sum(-1) + 1e-8)).unsqueeze(1) * torch.sqrt(kr ** 2 + ki ** 2)).sum(-1)
    assert torch.allclose(got, re + extra, atol=1e-5)
    # zero Q centre: pure norm term with coefficient q_abs - 1e-4
    got0 = osc.raw_scores(keys, torch.zeros(h, f, 2), qa, orope.default_inv_freq(d), offs, fs, 33)
    want0 = ((qa - 1e-4).unsqueeze(1) * torch.sqrt(kr ** 2 + ki ** 2)).sum(-1)
    assert torch.allclose(got0, want0, atol=1e-5)


def test_rotation_invariance():
    # Rotating key pair f by theta and shifting the query phase by -theta/omega_f
    # leaves the score unchanged; with one frequency this is a shift of round_start.
    w = 0.125
    keys = torch.tensor([[[0.8, -0.3]]])
    qc = torch.tensor([[[0.4, 0.9]]])
    qa = torch.tensor([[1.7]])
    base = osc.raw_scores(keys, qc, qa, torch.tensor([w]), torch.tensor([2.0]), torch.ones(1, 1), 16)
    rot = osc.rope_rotate(keys, torch.tensor([8]), torch.tensor([w]))      # theta = 8 w
    moved = osc.raw_scores(rot, qc, qa, torch.tensor([w]), torch.tensor([2.0]), torch.ones(1, 1), 24)
    assert torch.allclose(base, moved, atol=1e-6)


@pytest.mark.parametrize("style", ["half", "interleaved"])
@pytest.mark.parametrize("agg", ["mean", "max"])
def test_rotated_and_unrotated_forms_agree(style, agg):
    g = torch.Generator().manual_seed(7)
    h, t, d = 3, 40, 32
    f = d // 2
    omega = orope.default_inv_freq(d, 1e4)
    k_un = torch.randn(h, t, d, generator=g)
    pos = torch.arange(t)
    k_rot = osc.rope_rotate(k_un, pos, omega, style)
    qc = torch.randn(h, f, 2, generator=g)
    qa = qc.pow(2).sum(-1).sqrt() + torch.rand(h, f, generator=g)
    fs = 0.5 + torch.rand(h, f, generator=g)
    offs = osc.geometric_offsets(256)
    a = osc.raw_scores(k_rot, qc, qa, omega, offs, fs, t, agg, style)
    b = osc.raw_scores_unrotated(k_un, pos, qc, qa, omega, offs, fs, t, agg, style)
    assert torch.allclose(a, b, rtol=1e-4, atol=2e-3)


def test_offsets_and_inv_freq():
    offs = osc.geometric_offsets(65536)
    assert offs.tolist() == [float(2 ** j) for j in range(17)]
    inv = orope.default_inv_freq(128, 1e6)
    assert inv.shape == (64,)
    assert abs(float(inv[0]) - 1.0) < 1e-7
    assert abs(float(inv[32]) - 1e6 ** -0.5) / 1e-3 < 1e-5
    assert abs(float(inv[63]) - 1e6 ** (-126 / 128)) / float(inv[63]) < 1e-5


def test_llama3_inv_freq_regimes():
    base = orope.default_inv_freq(128, 5e5)
    got = orope.llama3_inv_freq(128, 5e5, 8.0, 1.0, 4.0, 8192)
    wl = 2 * math.pi / base
    hi = wl < 8192 / 4
    lo = wl > 8192 / 1
    assert torch.equal(got[hi], base[hi])                       # short wavelengths untouched
    assert torch.allclose(got[lo], base[lo] / 8.0, rtol=1e-6)   # long wavelengths / factor
    mid = ~hi & ~lo
    assert int(mid.sum()) > 0
    sm = (8192 / wl[mid] - 1.0) / 3.0
    assert torch.allclose(got[mid], (1 - sm) * base[mid] / 8 + sm * base[mid], rtol=1e-5)
    assert bool((got[mid] < base[mid]).all()) and bool((got[mid] > base[mid] / 8).all())


def test_llama3_inv_freq_equals_transformers_golden():
    """64 frequencies written by transformers' own llama3 routine (tests/golden/make_llama3_golden.py):
    bit for bit, all three bands."""
    from conftest import load_golden
    gold = load_golden("llama3_inv_freq.pt")
    got = orope.llama3_inv_freq(int(gold["head_dim"]), float(gold["rope_theta"]), float(gold["factor"]),
                                float(gold["low_freq_factor"]), float(gold["high_freq_factor"]),
                                int(gold["original_max_position_embeddings"]))
    assert torch.equal(got, gold["llama3_inv_freq"])
    assert torch.equal(orope.default_inv_freq(128, 5e5), gold["default_inv_freq"])
    changed = gold["llama3_inv_freq"] != gold["default_inv_freq"]
    assert 0 < int(changed.sum()) < 64 and float(gold["attention_scaling"]) == 1.0


def test_fp8_dequant_closed_form():
    codes = torch.tensor([[[0.5, -1.5, 448.0, 0.0]]]).to(torch.float8_e4m3fn)
    scales = torch.tensor([[0.25]])
    assert osc.dequant_fp8(codes, scales).flatten().tolist() == [0.125, -0.375, 112.0, 0.0]


@pytest.mark.parametrize("case", ["half_d128", "interleaved_d64", "half_scaled"])
def test_unrotated_form_matches_the_research_paths_own_scores(case):
    """``oracle.scoring.raw_scores_unrotated`` (and ``oracle.calibration.invert_rope``, the same inverse
    rotation) against outputs of the reference's own helpers on the keys of a Hugging Face cache
    (fixture written by tests/golden/make_hf_score_golden.py from methods/pruning_utils.py:
    ``invert_rope`` -> ``compute_frequency_statistics_from_means`` -> ``score_keys_for_round``): mean
    and max over the offsets, with and without the MLR term.  Then the form the kernels evaluate --
    rotated keys, no positions -- against the same reference scores: a rotated key carries its
    position in its phase, and one factor of the attention scale."""
    from oracle import calibration as ocal
    gold = load_golden("hf_score.pt")[case]
    style, scale = gold["style"], float(gold["scale"])
    k_rot = gold["k_rot"]
    hkv = k_rot.shape[0]
    hq = gold["q_abs_mean"].shape[0]
    k_un = ocal.invert_rope(k_rot.float(), gold["cos"], gold["sin"], scale, style)
    assert torch.equal(k_un, gold["k_unrot"])
    qc = torch.stack([gold["q_mean_real"], gold["q_mean_imag"]], dim=-1)
    fs = gold["freq_scale_sq"].unsqueeze(0).expand(hq, -1)
    rs = int(gold["round_start"])
    for tag, mlr in (("", False), ("_nomlr", True)):
        for agg in ("mean", "max"):
            want = gold[f"scores_{agg}{tag}"]
            got = osc.raw_scores_unrotated(k_un.repeat_interleave(hq // hkv, dim=0), gold["positions"], qc,
                                           gold["q_abs_mean"], gold["inv_freq"], gold["offsets"], fs, rs, agg, style,
                                           disable_mlr=mlr)
            scale_of = float(want.abs().max())
            assert float((got - want).abs().max()) <= 2e-6 * scale_of, (case, agg, tag)
            rotated = osc.raw_scores(k_rot.float().repeat_interleave(hq // hkv, dim=0), qc, gold["q_abs_mean"],
                                     gold["inv_freq"], gold["offsets"], fs, rs, agg, style, disable_mlr=mlr) / scale
            # (fp32 phases of up to 65536 rad carry errors of 4e-3 rad, different ones in the two forms)
            assert float((rotated - want).abs().max()) <= 5e-4 * scale_of, (case, agg, tag)
