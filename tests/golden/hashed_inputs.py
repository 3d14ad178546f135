"""Key/value tensors that are bit-identical on every machine: integer hashing and exact fp32
arithmetic only (no random-number generator, no transcendental function), so a golden fixture
can name a seed instead of carrying tens of megabytes of keys.  Used by the script that writes
``selector_c1_shape.pt`` from the reference and by the tests that read it."""
from __future__ import annotations

import torch

_M32 = 0xFFFFFFFF


def _mix(x: torch.Tensor) -> torch.Tensor:
    """A 32-bit integer finaliser on int64 tensors (every intermediate stays below 2^63)."""
    x = x & _M32
    x = ((x ^ (x >> 16)) * 0x45D9F3B) & _M32
    x = ((x ^ (x >> 16)) * 0x45D9F3B) & _M32
    return (x ^ (x >> 16)) & _M32


def hashed_rows(seed: int, layers: int, heads: int, tokens: int, dim: int) -> torch.Tensor:
    """bf16 [layers, heads, tokens, dim]: a sum of three hashed uniforms per element (close to
    N(0, 1)) plus a per-(layer, head, dim) centre in [-2, 2); all values are multiples of 1/512
    below 8 in magnitude, so every fp32 step is exact and the bf16 rounding is the only rounding."""
    n = layers * heads * tokens * dim
    idx = torch.arange(n, dtype=torch.int64)
    acc = torch.zeros(n, dtype=torch.int64)
    for j in range(3):
        acc += _mix(idx * 3 + j + (seed * 0x9E3779B1 & _M32)) & 1023
    body = (acc - 1536).to(torch.float32) / 512.0
    cidx = torch.arange(layers * heads * dim, dtype=torch.int64)
    centre = ((_mix(cidx + ((seed + 7) * 0x85EBCA6B & _M32)) & 1023) - 512).to(torch.float32) / 256.0
    out = body.view(layers, heads, tokens, dim) + centre.view(layers, heads, 1, dim)
    return out.to(torch.bfloat16)


def checksum(t: torch.Tensor) -> int:
    """Order-sensitive 62-bit checksum of a bf16 tensor's bit patterns."""
    bits = t.contiguous().view(torch.int16).to(torch.int64).flatten() & 0xFFFF
    weights = (torch.arange(bits.numel(), dtype=torch.int64) % 8191) + 1
    return int((bits * weights).sum().item() & 0x3FFFFFFFFFFFFFFF)
