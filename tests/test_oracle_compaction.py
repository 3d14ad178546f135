"""Pins oracle.compaction against the reference's own compaction outputs (golden)
and brute-force row loops.  CPU only."""
from __future__ import annotations

import pytest
import torch

from conftest import load_golden
from oracle import compaction as ocp


@pytest.mark.parametrize("axis", [0, 1])
def test_full_permutation_matches_reference(axis):
    g = load_golden("compaction.pt")[f"axis{axis}"]
    bs, t = int(g["block_size"]), int(g["total_tokens"])
    a = g["kv_before"].clone()
    n = ocp.compact_per_head(a, g["block_ids"], bs, g["keep_per_head"], t, full_permutation=True)
    assert n == g["keep_per_head"].shape[1]
    assert torch.equal(a.view(torch.int16), g["kv_after_per_head"].view(torch.int16))
    b = g["kv_before"].clone()
    ocp.compact_shared(b, g["block_ids"], bs, g["keep_shared"], t, full_permutation=True)
    assert torch.equal(b.view(torch.int16), g["kv_after_shared"].view(torch.int16))


@pytest.mark.parametrize("axis", [0, 1])
def test_prefix_only_agrees_on_kept_slots(axis):
    g = load_golden("compaction.pt")[f"axis{axis}"]
    bs, t = int(g["block_size"]), int(g["total_tokens"])
    a = g["kv_before"].clone()
    k = ocp.compact_per_head(a, g["block_ids"], bs, g["keep_per_head"], t, full_permutation=False)
    ka, va = ocp.split_kv(a)
    kr, vr = ocp.split_kv(g["kv_after_per_head"])
    blk, off = ocp.token_slots(g["block_ids"], bs, torch.arange(k))
    assert torch.equal(ka[blk, off].view(torch.int16), kr[blk, off].view(torch.int16))
    assert torch.equal(va[blk, off].view(torch.int16), vr[blk, off].view(torch.int16))


def test_bruteforce_rows_and_multiset():
    g = torch.Generator().manual_seed(9)
    h, d, bs, t, k = 2, 4, 4, 19, 6
    nb = 5
    ids = torch.tensor([7, 2, 5, 0, 3])
    kv = torch.randn(2, 9, bs, h, d, generator=g)
    keep = torch.stack([torch.sort(torch.randperm(t, generator=g)[:k]).values for _ in range(h)])
    before = kv.clone()
    ocp.compact_per_head(kv, ids, bs, keep, t)
    for which in (0, 1):
        for hh in range(h):
            dropped = [n for n in range(t) if n not in set(keep[hh].tolist())]
            order = keep[hh].tolist() + dropped
            for j, src in enumerate(order):
                want = before[which, ids[src // bs], src % bs, hh]
                got = kv[which, ids[j // bs], j % bs, hh]
                assert torch.equal(got, want)
    # blocks the request does not own are untouched
    other = [b for b in range(9) if b not in ids.tolist()]
    assert torch.equal(kv[:, other], before[:, other])
    # slot t (beyond the logical length, inside the last block) untouched
    assert torch.equal(kv[:, ids[4], 3], before[:, ids[4], 3])


def test_identity_and_errors():
    kv = torch.randn(2, 4, 4, 2, 4)
    before = kv.clone()
    ident = torch.arange(5).unsqueeze(0).expand(2, -1)
    assert ocp.compact_per_head(kv, [0, 1, 2], 4, ident, 10) == 5
    assert torch.equal(kv, before)
    with pytest.raises(IndexError):
        ocp.compact_per_head(kv, [0, 1, 2], 4, torch.tensor([[0, 12], [1, 2]]), 12 - 1)
    with pytest.raises(ValueError):
        ocp.compact_per_head(kv, [0, 1, 2], 4, torch.tensor([[3, 3], [1, 2]]), 10)
    with pytest.raises(ValueError):
        ocp.compact_per_head(kv, [0, 1, 2], 4, torch.tensor([[1, 2]]), 10)
    with pytest.raises(ValueError):
        ocp.split_kv(torch.zeros(2, 2, 4, 1, 4))
    assert ocp.compact_shared(kv, [0, 1, 2], 4, torch.tensor([], dtype=torch.long), 10) == 0


def test_gather_and_truncate():
    kv = torch.arange(2 * 6 * 4 * 1 * 2, dtype=torch.float32).view(2, 6, 4, 1, 2)
    kc, _ = ocp.split_kv(kv)
    ids = [4, 1, 3]
    dense = ocp.gather_dense(kc, ids, 4, 2, 7)
    assert dense.shape == (1, 1, 7, 2)
    for i, n in enumerate(range(2, 9)):
        assert torch.equal(dense[0, 0, i], kc[ids[n // 4], n % 4, 0])
    assert ocp.required_blocks(0, 16) == 0 and ocp.required_blocks(2048, 16) == 128
    assert ocp.required_blocks(2049, 16) == 129
    assert ocp.truncate_tail([9, 8, 7, 6], 5, 4) == ([9, 8], [7, 6])
