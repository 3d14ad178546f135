"""Calibration statistics on an MI355X (through the C ABI) against the reference's own
outputs (tests/golden/calibration_stats.pt) and the oracle."""
from __future__ import annotations

import types

import pytest
import torch

from conftest import load_golden
from oracle import calibration as ocal
from triattention_amd import ops
from triattention_amd.calibration import StatsCollector, collect_model_stats
from triattention_amd.core.stats import load_frequency_stats

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

# The un-rotated queries are bit-identical to the reference's (every elementwise step rounds
# to the 16-bit dtype exactly as a tensor op does); the means differ only by the order of the
# fp32 summation over tokens and by sqrt(re^2 + im^2) against torch's hypot: 1e-5 of the
# head's largest statistic.
TOL = 1e-5


def _close(got: torch.Tensor, want: torch.Tensor) -> bool:
    scale = want.abs().amax(dim=-1, keepdim=True).clamp_min(1e-6)
    return bool(((got.cpu() - want).abs() <= TOL * scale).all())


@pytest.mark.parametrize("name", ["half_bf16", "half_bf16_scaled", "interleaved_bf16", "half_fp16"])
def test_query_stats_match_the_reference_outputs(name):
    g = load_golden("calibration_stats.pt")[name]
    print(f"calibration case={name}", flush=True)
    real, imag, mod = ops.query_stats(g["q_rot"].to(DEV), g["cos"].to(DEV), g["sin"].to(DEV), g["scale"], g["style"])
    torch.cuda.synchronize()
    assert _close(real, g["q_mean_real"]) and _close(imag, g["q_mean_imag"]) and _close(mod, g["q_abs_mean"])


@pytest.mark.parametrize("style,dim", [("half", 128), ("interleaved", 128), ("half", 64), ("half", 256)])
def test_query_stats_match_the_oracle_on_a_strided_capture(style, dim):
    """[1, H, T, D] as a transposed view of [1, T, H, D] (what q_proj().view().transpose()
    hands the hook), several token chunks with a ragged last one."""
    g = torch.Generator().manual_seed(dim + len(style))
    heads, tokens, scale = 5, 1337, 1.0
    inv_freq = 1e6 ** (-torch.arange(0, dim, 2, dtype=torch.float32) / dim)
    cos, sin = ocal.rope_tables(tokens, inv_freq, scale, torch.bfloat16, style)
    q = (torch.randn(1, tokens, heads, dim, generator=g) + torch.randn(1, 1, heads, dim, generator=g)).to(torch.bfloat16)
    q_rot = ocal.apply_rope(q.transpose(1, 2), cos, sin, scale, style)          # [1, H, T, D], computed on CPU
    want = ocal.head_frequency_stats(q_rot[0], cos, sin, scale, style)
    dev_q = q_rot.transpose(1, 2).contiguous().to(DEV).transpose(1, 2)[0]       # strided [H, T, D]
    assert not dev_q.is_contiguous()
    print(f"calibration strided style={style} dim={dim}", flush=True)
    got = ops.query_stats(dev_q, cos.to(DEV), sin.to(DEV), scale, style)
    torch.cuda.synchronize()
    for a, b in zip(got, want):
        assert _close(a, b)


def test_query_stats_reject_what_the_kernel_does_not_take():
    q = torch.zeros(2, 8, 128, dtype=torch.bfloat16, device=DEV)
    t = torch.zeros(8, 128, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError):
        ops.query_stats(q.cpu(), t.cpu(), t.cpu())
    with pytest.raises(ValueError):
        ops.query_stats(q.float(), t.float(), t.float())
    with pytest.raises(ValueError):
        ops.query_stats(q, t[:4], t)
    with pytest.raises(ValueError):
        ops.query_stats(q[..., :48], t[:, :48], t[:, :48])
    with pytest.raises(Exception):
        ops.query_stats(q, t, t, scale=0.0)


class _Rotary(torch.nn.Module):
    def __init__(self, dim, theta, scaling):
        super().__init__()
        self.register_buffer("inv_freq", theta ** (-torch.arange(0, dim, 2, dtype=torch.float32) / dim))
        self.attention_scaling = scaling

    def forward(self, x, position_ids):
        ang = position_ids[0].to(torch.float32)[:, None] * self.inv_freq[None, :]
        emb = torch.cat((ang, ang), dim=-1)[None]
        return (emb.cos() * self.attention_scaling).to(x.dtype), (emb.sin() * self.attention_scaling).to(x.dtype)


class _Attention(torch.nn.Module):
    def __init__(self, hidden, heads, dim):
        super().__init__()
        self.q_proj = torch.nn.Linear(hidden, heads * dim, bias=False)

    def forward(self, hidden_states):
        return hidden_states


class _Block(torch.nn.Module):
    def __init__(self, hidden, heads, dim):
        super().__init__()
        self.self_attn = _Attention(hidden, heads, dim)
        self.mix = torch.nn.Linear(hidden, hidden, bias=False)

    def forward(self, hidden_states):
        return hidden_states + 0.1 * self.mix(self.self_attn(hidden_states=hidden_states))


class _Decoder(torch.nn.Module):
    def __init__(self, vocab, hidden, heads, dim, layers):
        super().__init__()
        self.model = torch.nn.Module()
        self.model.embed = torch.nn.Embedding(vocab, hidden)
        self.model.layers = torch.nn.ModuleList(_Block(hidden, heads, dim) for _ in range(layers))
        self.model.rotary_emb = _Rotary(dim, 1e4, 1.0)

    def forward(self, input_ids):
        h = self.model.embed(input_ids)
        for block in self.model.layers:
            h = block(h)
        return h


def test_collected_file_loads_and_matches_the_oracle(tmp_path):
    """A small decoder with the attribute layout of a Hugging Face model: the pre-hooks capture
    every layer, the written file goes through the stats loader, and its numbers equal the
    oracle's on queries recomputed independently from the model's weights."""
    torch.manual_seed(7)
    heads, dim, layers, tokens = 3, 64, 2, 300
    model = _Decoder(50, 96, heads, dim, layers).to(DEV).to(torch.bfloat16).eval()
    ids = torch.randint(0, 50, (1, tokens), device=DEV)
    col = collect_model_stats(model, ids, num_heads=heads, head_dim=dim)
    path = col.save(tmp_path / "stats.pt")
    payload = torch.load(path, weights_only=True)
    assert payload["metadata"]["sampled_heads"] == [[l, h] for l in range(layers) for h in range(heads)]
    assert payload["metadata"]["head_dim"] == dim and payload["metadata"]["rope_style"] == "half"
    assert torch.equal(payload["metadata"]["inv_freq"], model.model.rotary_emb.inv_freq.cpu())
    # independent recomputation of what each layer's attention saw
    with torch.no_grad():
        h = model.model.embed(ids)
        pos = torch.arange(tokens, device=DEV).unsqueeze(0)
        cos, sin = model.model.rotary_emb(torch.zeros(1, tokens, dim, device=DEV, dtype=torch.bfloat16), pos)
        for l, block in enumerate(model.model.layers):
            q = block.self_attn.q_proj(h).view(1, tokens, heads, dim).transpose(1, 2)
            q_rot = ocal.apply_rope(q.cpu(), cos.cpu(), sin.cpu(), 1.0)
            want = ocal.head_frequency_stats(q_rot[0], cos[0].cpu(), sin[0].cpu(), 1.0)
            for hd in range(heads):
                entry = payload["stats"][f"layer{l:02d}_head{hd:02d}"]
                assert _close(entry["q_mean_real"][None], want[0][hd][None])
                assert _close(entry["q_mean_imag"][None], want[1][hd][None])
                assert _close(entry["q_abs_mean"][None], want[2][hd][None])
            h = block(h)
    meta, head_stats = load_frequency_stats(path)
    assert sorted(head_stats) == list(range(layers))
    assert tuple(head_stats[0]["q_mean_complex"].shape) == (heads, dim // 2, 2)
    assert torch.equal(head_stats[1]["q_abs_mean"][2], payload["stats"]["layer01_head02"]["q_abs_mean"])
