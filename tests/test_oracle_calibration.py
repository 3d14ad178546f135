"""Oracle for the calibration arithmetic against vectors written by the reference's own
helpers (tests/golden/make_calibration_golden.py), and against what the mathematics fixes."""
from __future__ import annotations

import math

import pytest
import torch

from conftest import load_golden
from oracle import calibration as ocal

CASES = ["half_bf16", "half_bf16_scaled", "interleaved_bf16", "half_fp16"]


@pytest.mark.parametrize("name", CASES)
def test_invert_rope_and_means_equal_the_reference_bit_for_bit(name):
    g = load_golden("calibration_stats.pt")[name]
    q_base = ocal.invert_rope(g["q_rot"], g["cos"].unsqueeze(0), g["sin"].unsqueeze(0), g["scale"], g["style"])
    assert torch.equal(q_base.view(torch.int16), g["q_base"].view(torch.int16))
    real, imag, mod = ocal.head_frequency_stats(g["q_rot"], g["cos"], g["sin"], g["scale"], g["style"])
    assert torch.equal(real, g["q_mean_real"])
    assert torch.equal(imag, g["q_mean_imag"])
    assert torch.equal(mod, g["q_abs_mean"])


@pytest.mark.parametrize("name", CASES)
def test_rope_tables_reproduce_the_fixture_tables(name):
    g = load_golden("calibration_stats.pt")[name]
    cos, sin = ocal.rope_tables(g["q_rot"].shape[1], g["inv_freq"], g["scale"], g["q_rot"].dtype, g["style"])
    assert torch.equal(cos.view(torch.int16), g["cos"].view(torch.int16))
    assert torch.equal(sin.view(torch.int16), g["sin"].view(torch.int16))


@pytest.mark.parametrize("style", ["half", "interleaved"])
def test_inversion_undoes_the_rotation_in_exact_arithmetic(style):
    """In fp64 there is no rounding to speak of: rotating by the tables and inverting must
    return the input, for both pairings (a wrong sign or a swapped cos / sin in either branch
    fails this).  With an attention scale s the capture hook multiplies by s on top of tables
    that already carry s (scripts/calibrate.py:185-186), and the inversion divides both by s
    once: the reference's statistics are those of s*q, and so are these."""
    g = torch.Generator().manual_seed(5)
    t, d, scale = 40, 32, 1.7
    inv_freq = 10000.0 ** (-torch.arange(0, d, 2, dtype=torch.float64) / d)
    q = torch.randn(3, t, d, generator=g, dtype=torch.float64)
    ang = torch.arange(t, dtype=torch.float64)[:, None] * inv_freq[None, :]
    emb = torch.repeat_interleave(ang, 2, dim=-1) if style == "interleaved" else torch.cat((ang, ang), dim=-1)
    cos, sin = emb.cos() * scale, emb.sin() * scale
    back = ocal.invert_rope(ocal.apply_rope(q, cos, sin, scale, style), cos, sin, scale, style)
    assert float((back - scale * q).abs().max()) < 1e-12


def test_statistics_of_a_constant_rotating_query():
    """q_t = r * exp(i*phi) for every token: the complex mean is the value itself and the mean
    modulus is r, whatever the positions."""
    t, d = 64, 16
    f = d // 2
    r = torch.linspace(0.5, 2.0, f, dtype=torch.float64)
    phi = torch.linspace(-3.0, 3.0, f, dtype=torch.float64)
    q = torch.cat((r * phi.cos(), r * phi.sin())).expand(1, t, d).clone()
    inv_freq = 10000.0 ** (-torch.arange(0, d, 2, dtype=torch.float64) / d)
    ang = torch.arange(t, dtype=torch.float64)[:, None] * inv_freq[None, :]
    emb = torch.cat((ang, ang), dim=-1)
    cos, sin = emb.cos(), emb.sin()
    real, imag, mod = ocal.head_frequency_stats(ocal.apply_rope(q, cos, sin, 1.0), cos, sin, 1.0)
    assert float((real[0] - r * phi.cos()).abs().max()) < 1e-12
    assert float((imag[0] - r * phi.sin()).abs().max()) < 1e-12
    assert float((mod[0] - r).abs().max()) < 1e-12
    assert math.isclose(float(mod[0, 0]), 0.5)
