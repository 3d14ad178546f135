"""Seeded synthetic workloads: paged KV pools, block tables and per-head Q statistics
of the shapes the benchmark configurations name.  Used by the tests (small sizes, CPU
generator, copied to the device) and by bench.py (full sizes, generated on the device).

Measurement and test infrastructure, not part of the product path: nothing under
``triattention_amd.core`` or ``triattention_amd.runtime`` imports this module.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field, replace

import torch


@dataclass(frozen=True)
class Workload:
    name: str
    num_layers: int
    num_q_heads: int
    num_kv_heads: int
    head_dim: int
    seq_lens: tuple
    budget: int
    block_size: int = 16
    window_size: int = 128
    rope_theta: float = 1e6
    rope_scaling: str = "default"       # or "llama3"
    rope_style: str = "half"
    kv_dtype: str = "bf16"              # "bf16", "fp16", "fp8"
    pool_occupancy: float = 1.0         # live blocks / pool blocks
    index: int = 0                      # seeds: 1000+index keys, 2000+index stats, 3000+index tables

    @property
    def num_seqs(self) -> int:
        return len(self.seq_lens)

    @property
    def blocks_per_seq(self):
        return [(t + self.block_size - 1) // self.block_size for t in self.seq_lens]

    @property
    def pool_blocks(self) -> int:
        live = sum(self.blocks_per_seq)
        return max(live, int(math.ceil(live / self.pool_occupancy)))

    def algorithmic_bytes(self) -> dict:
        """Bytes the step must move: every cached key once, kept K and V rows read
        and written once.  Block tables, statistics and score scratch are overhead."""
        e = 1 if self.kv_dtype == "fp8" else 2
        scale = 4 if self.kv_dtype == "fp8" else 0
        row = self.num_kv_heads * (self.head_dim * e + scale)
        score = sum(self.seq_lens) * self.num_layers * row
        kept = sum(min(self.budget, t) for t in self.seq_lens)
        comp = 2 * 2 * kept * self.num_layers * row
        return {"score": score, "compact": comp, "total": score + comp}

    def scaled(self, **kw) -> "Workload":
        return replace(self, **kw)


def _ragged_lengths(n: int, lo: int, hi: int, seed: int) -> tuple:
    g = torch.Generator().manual_seed(seed)
    return tuple(int(x) for x in torch.randint(lo, hi + 1, (n,), generator=g))


def config(i: int) -> Workload:
    """The five benchmark configurations."""
    if i == 0:
        return Workload("c0_qwen3_8b_1layer_4k", 1, 32, 8, 128, (4096,), 2048, index=0)
    if i == 1:
        return Workload("c1_qwen3_8b_36l_b16_16k", 36, 32, 8, 128, (16384,) * 16, 2048, index=1)
    if i == 2:
        return Workload("c2_qwen3_32b_64l_b8_32k", 64, 64, 8, 128, (32768,) * 8, 12000, index=2)
    if i == 3:
        return Workload("c3_qwen3_8b_ragged64", 36, 32, 8, 128, _ragged_lengths(64, 2048, 32768, 4000), 2048,
                        pool_occupancy=0.8, index=3)
    if i == 4:
        return Workload("c4_llama31_8b_fp8_b16_16k", 32, 32, 8, 128, (16384,) * 16, 2048, rope_theta=5e5,
                        rope_scaling="llama3", kv_dtype="fp8", index=4)
    raise ValueError(f"no config {i}")


def rope_inv_freq(w: Workload, device="cpu") -> torch.Tensor:
    from .rope import default_inv_freq, llama3_inv_freq
    if w.rope_scaling == "llama3":
        return llama3_inv_freq(w.head_dim, w.rope_theta).to(device)
    return default_inv_freq(w.head_dim, w.rope_theta).to(device)


def geometric_offsets(max_length: int = 65536, device="cpu") -> torch.Tensor:
    vals, v = [], 1
    while v <= max_length:
        vals.append(float(v))
        v *= 2
    return torch.tensor(vals, dtype=torch.float32, device=device)


def make_stats(w: Workload, device="cpu"):
    """Per-(layer, query head) Q centre N(0,1)+iN(0,1) and q_abs = |centre| + |N(0,1)|."""
    g = torch.Generator(device=device).manual_seed(2000 + w.index)
    f = w.head_dim // 2
    qc = torch.randn(w.num_layers, w.num_q_heads, f, 2, generator=g, device=device)
    qa = qc.pow(2).sum(-1).sqrt() + torch.randn(w.num_layers, w.num_q_heads, f, generator=g, device=device).abs()
    return qc, qa


def make_block_tables(w: Workload):
    """Each sequence's table is a slice of one random permutation of the pool."""
    g = torch.Generator().manual_seed(3000 + w.index)
    perm = torch.randperm(w.pool_blocks, generator=g).tolist()
    tables, pos = [], 0
    for n in w.blocks_per_seq:
        tables.append(perm[pos:pos + n])
        pos += n
    return tables


_TORCH_DTYPE = {"bf16": torch.bfloat16, "fp16": torch.float16}


def make_kv_pool(w: Workload, block_tables, device="cpu", kv_axis: int = 0):
    """One [2, nb, bs, H, D] (kv_axis 0) or [nb, 2, bs, H, D] (kv_axis 1) tensor per layer.

    Keys are N(0,1) plus a per-(layer, head, dim) centre of variance 2, rotated by
    RoPE at positions 0..T-1 in fp32, then stored in the cache dtype; values N(0,1).
    For fp8 returns (caches, k_scales, v_scales) with per-(token, head) fp32 scales.
    """
    g = torch.Generator(device=device).manual_seed(1000 + w.index)
    bs, h, d, f = w.block_size, w.num_kv_heads, w.head_dim, w.head_dim // 2
    nb = w.pool_blocks
    omega = rope_inv_freq(w, device)
    fp8 = w.kv_dtype == "fp8"
    dt = torch.float8_e4m3fn if fp8 else _TORCH_DTYPE[w.kv_dtype]
    slots = []
    for tbl, t in zip(block_tables, w.seq_lens):
        tok = torch.arange(t, device=device)
        blk = torch.tensor(tbl, device=device, dtype=torch.long)[tok // bs]
        slots.append(blk * bs + tok % bs)
    slot_idx = torch.cat(slots)                                          # flat pool slot of every token
    pos = torch.cat([torch.arange(t, device=device, dtype=torch.float32) for t in w.seq_lens])
    ang = pos.unsqueeze(-1) * omega                                      # [N, F]
    cos, sin = torch.cos(ang).unsqueeze(1), torch.sin(ang).unsqueeze(1)  # [N, 1, F]
    n_tok = int(slot_idx.numel())
    caches, k_scales, v_scales = [], [], []
    for _ in range(w.num_layers):
        k = torch.randn(n_tok, h, d, generator=g, device=device)
        c = torch.randn(1, h, d, generator=g, device=device) * math.sqrt(2.0)
        v = torch.randn(n_tok, h, d, generator=g, device=device)
        k = k + c
        if w.rope_style == "interleaved":
            kr, ki = k[..., 0::2], k[..., 1::2]
            k = torch.stack((kr * cos - ki * sin, ki * cos + kr * sin), dim=-1).flatten(-2)
        else:
            kr, ki = k[..., :f], k[..., f:]
            k = torch.cat((kr * cos - ki * sin, ki * cos + kr * sin), dim=-1)
        shape = (2, nb, bs, h, d) if kv_axis == 0 else (nb, 2, bs, h, d)
        cache = torch.zeros(shape, dtype=dt, device=device)
        kview = cache[0] if kv_axis == 0 else cache[:, 0]
        vview = cache[1] if kv_axis == 0 else cache[:, 1]
        if fp8:
            ks = k.abs().amax(dim=-1).clamp_min(1e-6) / 448.0
            vs = v.abs().amax(dim=-1).clamp_min(1e-6) / 448.0
            ksc = torch.ones(nb * bs, h, dtype=torch.float32, device=device)
            vsc = torch.ones(nb * bs, h, dtype=torch.float32, device=device)
            ksc[slot_idx] = ks
            vsc[slot_idx] = vs
            kview.view(nb * bs, h, d)[slot_idx] = (k / ks.unsqueeze(-1)).to(dt)
            vview.view(nb * bs, h, d)[slot_idx] = (v / vs.unsqueeze(-1)).to(dt)
            k_scales.append(ksc)
            v_scales.append(vsc)
        else:
            if kv_axis == 0:
                kview.view(nb * bs, h, d)[slot_idx] = k.to(dt)
                vview.view(nb * bs, h, d)[slot_idx] = v.to(dt)
            else:
                kview[slot_idx // bs, slot_idx % bs] = k.to(dt)
                vview[slot_idx // bs, slot_idx % bs] = v.to(dt)
        caches.append(cache)
    if fp8:
        return caches, k_scales, v_scales
    return caches
