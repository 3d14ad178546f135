"""Writes tests/golden/flat_pool.pt: a small token-level KV pool before and after the
reference's SGLang compaction functions (triattention/sglang/kv_compaction.py, loaded by file
so that the sglang package itself is not needed), its dense gather, its slot reclaim, and the
reference's normalize_scores / protect_window_tokens (triattention/vllm/core/utils.py) on
group-max scores.  Run on CPU in this container:

    python tests/golden/make_flat_pool_golden.py /root/reference
"""
from __future__ import annotations

import importlib.util
import sys
from pathlib import Path

import torch


def _load(path: Path, name: str):
    spec = importlib.util.spec_from_file_location(name, path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


class _Allocator:
    def __init__(self):
        self.freed = []

    def free(self, idx):
        self.freed.append(idx.clone())


def main() -> None:
    ref = Path(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
    kvc = _load(ref / "triattention" / "sglang" / "kv_compaction.py", "ref_sglang_kvc")
    sys.path.insert(0, str(ref))
    from triattention.vllm.core.utils import normalize_scores, protect_window_tokens

    g = torch.Generator().manual_seed(77)
    layers, heads, dim, pool, eff, budget = 2, 2, 64, 128, 101, 40
    k0 = [torch.randn(pool, heads, dim, generator=g).to(torch.bfloat16) for _ in range(layers)]
    v0 = [torch.randn(pool, heads, dim, generator=g).to(torch.bfloat16) for _ in range(layers)]
    req_to_token = torch.zeros(3, 128, dtype=torch.int32)
    perm = torch.randperm(pool - 1, generator=g)[:eff] + 1            # slot 0 is the allocator's dummy slot
    req_to_token[1, :eff] = perm.int()
    keep_shared = torch.sort(torch.randperm(eff, generator=g)[:budget]).values
    keep_heads = torch.stack([torch.sort(torch.randperm(eff, generator=g)[:budget]).values for _ in range(heads)])

    out = {"k_before": torch.stack(k0), "v_before": torch.stack(v0), "req_to_token": req_to_token.clone(),
           "req_pool_idx": 1, "effective_len": eff, "keep_shared": keep_shared, "keep_per_head": keep_heads}
    out["k_dense"] = kvc.gather_request_k_dense(k0, req_to_token, 1, eff)

    ks, vs = [t.clone() for t in k0], [t.clone() for t in v0]
    assert kvc.compact_request_kv_in_place(ks, vs, req_to_token, 1, keep_shared, eff) == budget
    out["k_after_shared"], out["v_after_shared"] = torch.stack(ks), torch.stack(vs)

    kp, vp = [t.clone() for t in k0], [t.clone() for t in v0]
    assert kvc.compact_request_kv_in_place_per_head(kp, vp, req_to_token, 1, keep_heads, eff) == budget
    out["k_after_per_head"], out["v_after_per_head"] = torch.stack(kp), torch.stack(vp)

    r2t = req_to_token.clone()
    alloc = _Allocator()
    freed = kvc.reclaim_freed_slots(r2t, 1, budget, eff, alloc)
    out["freed_slots"], out["req_to_token_after_reclaim"] = freed.clone(), r2t

    # normalisation and window guard on group-max scores [1, H, T]
    raw = torch.randn(3, heads * 2, 300, generator=g) * 3.0 + torch.randn(3, heads * 2, 1, generator=g)
    grouped = raw.view(3, heads, 2, 300).max(dim=2).values
    out["raw_scores"] = raw
    out["normalized"] = torch.stack([normalize_scores(grouped[l:l + 1])[0] for l in range(3)])
    out["window_protected"] = protect_window_tokens(out["normalized"].mean(dim=0, keepdim=True), 17)[0]

    path = Path(__file__).resolve().parent / "flat_pool.pt"
    torch.save(out, path)
    print("wrote", path, path.stat().st_size, "bytes")


if __name__ == "__main__":
    main()
