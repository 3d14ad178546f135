"""Tensor-level wrappers over the C ABI: device pointers, strides and the current
HIP stream are taken from torch tensors; every byte of arithmetic on the hot path
runs in the gfx950 kernels of libtriattention_hip.so.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Sequence

import torch

from . import _lib
from ._lib import (KV_BF16, KV_FP16, KV_FP8_E4M3, REDUCE_MAX, REDUCE_MEAN, REDUCE_NONE, ROPE_HALF,
                   ROPE_INTERLEAVED, Batch, KvLayout, ScoreParams, SelectParams)

_DTYPES = {torch.bfloat16: KV_BF16, torch.float16: KV_FP16}
_UNIT_SCALES: dict = {}


def _unit_scales(device, count: int) -> torch.Tensor:
    """An array of ones standing in for the per-(token, head) scales of an fp8 cache that has none."""
    key = (str(device), int(count))
    hit = _UNIT_SCALES.get(key)
    if hit is None:
        if len(_UNIT_SCALES) >= 4:
            _UNIT_SCALES.pop(next(iter(_UNIT_SCALES)))
        hit = _UNIT_SCALES[key] = torch.ones(count, dtype=torch.float32, device=device)
    return hit


if hasattr(torch, "float8_e4m3fn"):
    _DTYPES[torch.float8_e4m3fn] = KV_FP8_E4M3
    _DTYPES[torch.uint8] = KV_FP8_E4M3      # vLLM keeps the codes of an fp8 cache in uint8 tensors


def _stream() -> int:
    return int(torch.cuda.current_stream().cuda_stream)


def _ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else int(t.data_ptr())


def _i32(values, device) -> torch.Tensor:
    if isinstance(values, torch.Tensor):
        return values.to(device=device, dtype=torch.int32).contiguous()
    return torch.tensor([int(v) for v in values], dtype=torch.int32, device=device)


def split_kv_axes(kv_cache: torch.Tensor, kv_axis: int | None = None):
    """K and V views [num_blocks, block_size, H, D] of a 5-D vLLM cache tensor.

    Accepts [2, nb, bs, H, D] and [nb, 2, bs, H, D]; when both leading dims are 2 the
    caller must say which one is the K/V axis (runtime/kv_compaction.py:94-117).
    """
    if kv_cache.ndim != 5:
        raise ValueError(f"Unsupported kv_cache ndim={kv_cache.ndim}, expect 5")
    d0, d1 = int(kv_cache.shape[0]) == 2, int(kv_cache.shape[1]) == 2
    if d0 and d1:
        if kv_axis not in (0, 1):
            raise ValueError(
                "Ambiguous KV layout for compaction: both dim0 and dim1 have size 2. "
                "Register an explicit layout hint via register_kv_layout_axis_hint(...).")
        d0, d1 = kv_axis == 0, kv_axis == 1
    if d0:
        return kv_cache[0], kv_cache[1]
    if d1:
        return kv_cache[:, 0], kv_cache[:, 1]
    raise ValueError("Unsupported KV layout for compaction: expected a dimension with size 2")


class PagedKV:
    """Key/value storage of the layers of one KV-cache group, as the kernels see it."""

    def __init__(self, k_views: Sequence[torch.Tensor], v_views: Sequence[torch.Tensor] | None = None,
                 rope_style: str = "half", k_scales: Sequence[torch.Tensor] | None = None,
                 v_scales: Sequence[torch.Tensor] | None = None):
        if not k_views:
            raise ValueError("no layers")
        k0 = k_views[0]
        if k0.ndim != 4:
            raise ValueError(f"expected [num_blocks, block_size, H, D] views, got {tuple(k0.shape)}")
        if not k0.is_cuda:
            raise RuntimeError("the scoring/compaction kernels need device memory; got a CPU tensor "
                               "(there is no CPU fallback)")
        if k0.dtype not in _DTYPES:
            raise TypeError(f"unsupported KV dtype {k0.dtype}")
        if k0.stride(3) != 1:
            raise ValueError("head_dim must be contiguous")
        views = list(k_views) + (list(v_views) if v_views is not None else [])
        for t in views:
            if t.shape != k0.shape or t.stride() != k0.stride() or t.dtype != k0.dtype or t.device != k0.device:
                raise ValueError("all layers must share shape, strides, dtype and device")
            if t.data_ptr() % 16:
                raise ValueError("KV base pointers must be 16-byte aligned")
        if rope_style not in ("half", "interleaved"):
            raise ValueError(f"rope_style must be 'half' or 'interleaved', got {rope_style!r}")
        self.device = k0.device
        self.dtype = k0.dtype
        self.num_layers = len(k_views)
        self.num_blocks, self.block_size, self.num_kv_heads, self.head_dim = (int(x) for x in k0.shape)
        self.rope_style = rope_style
        self._keep = (list(k_views), list(v_views) if v_views is not None else None, k_scales, v_scales)
        self.k_ptrs = torch.tensor([t.data_ptr() for t in k_views], dtype=torch.int64, device=self.device)
        self.v_ptrs = (torch.tensor([t.data_ptr() for t in v_views], dtype=torch.int64, device=self.device)
                       if v_views is not None else None)
        self.ks_ptrs = self.vs_ptrs = None
        if _DTYPES[self.dtype] == KV_FP8_E4M3:
            if k_scales is None:
                # A cache with one scale per tensor (vLLM's fp8 KV cache): the codes are scored as
                # they are (a factor common to a layer cancels in the normalised scores; callers
                # that do not normalise fold it into freq_scale_sq), and rows move without scales.
                if v_scales is not None:
                    raise ValueError("v_scales without k_scales")
                unit = _unit_scales(self.device, self.num_blocks * self.block_size * self.num_kv_heads)
                k_scales = [unit] * self.num_layers
                self._unit = unit           # ours, so kept alive here whatever becomes of _keep
            self.ks_ptrs = torch.tensor([t.data_ptr() for t in k_scales], dtype=torch.int64, device=self.device)
            if v_scales is not None:
                self.vs_ptrs = torch.tensor([t.data_ptr() for t in v_scales], dtype=torch.int64, device=self.device)
        self.struct = KvLayout(
            num_layers=self.num_layers, num_kv_heads=self.num_kv_heads, head_dim=self.head_dim,
            block_size=self.block_size, kv_dtype=_DTYPES[self.dtype],
            rope_style=ROPE_INTERLEAVED if rope_style == "interleaved" else ROPE_HALF,
            stride_block=int(k0.stride(0)), stride_token=int(k0.stride(1)), stride_head=int(k0.stride(2)),
            k_layers=_ptr(self.k_ptrs), v_layers=_ptr(self.v_ptrs),
            k_scale_layers=_ptr(self.ks_ptrs), v_scale_layers=_ptr(self.vs_ptrs))

    @classmethod
    def from_kv_caches(cls, kv_caches: Sequence[torch.Tensor], rope_style: str = "half",
                       kv_axis: int | None = None) -> "PagedKV":
        ks, vs = zip(*(split_kv_axes(t, kv_axis) for t in kv_caches))
        return cls(ks, vs, rope_style)

    _recent: "dict[tuple, PagedKV]" = {}

    @classmethod
    def for_kv_caches(cls, kv_caches: Sequence[torch.Tensor], rope_style: str = "half",
                      kv_axis: int | None = None) -> "PagedKV":
        """``from_kv_caches`` for callers that come back with the same cache tensors on every
        call (a serving loop): the description of a set of layer tensors, pointer tables on
        the device included, is built once per (addresses, geometry) and reused.  The cached
        object holds no reference to the cache tensors; it is only ever handed to a caller
        who holds tensors of that geometry at those addresses."""
        c0 = kv_caches[0]
        key = (tuple(int(t.data_ptr()) for t in kv_caches), tuple(c0.shape), tuple(c0.stride()), c0.dtype,
               str(c0.device), rope_style, kv_axis)
        hit = cls._recent.get(key)
        if hit is None:
            for t in kv_caches:
                if t.shape != c0.shape or t.stride() != c0.stride() or t.dtype != c0.dtype:
                    raise ValueError("all layers must share shape, strides, dtype and device")
            hit = cls.from_kv_caches(kv_caches, rope_style, kv_axis)
            hit._keep = None
            if len(cls._recent) >= 256:         # (the per-layer modes come with one tensor at a time: 2 x layers keys)
                cls._recent.pop(next(iter(cls._recent)))
            cls._recent[key] = hit
        return hit

    @classmethod
    def from_dense_keys(cls, key_states: torch.Tensor, rope_style: str = "half") -> "PagedKV":
        """[B, H, T, D] keys as one 'block' per sequence (score-only)."""
        if key_states.ndim != 4:
            raise ValueError(f"expected [B, H, T, D], got {tuple(key_states.shape)}")
        view = key_states.permute(0, 2, 1, 3)          # [B, T, H, D], no copy
        return cls([view], None, rope_style)


class StepBatch:
    """The sequences of one compression step, on the device."""

    def __init__(self, device, seq_lens, round_start=None, budgets=None, block_tables=None,
                 prefill_lens=None):
        self.device = device
        self.seq_lens_host = [int(x) for x in (seq_lens.tolist() if isinstance(seq_lens, torch.Tensor) else seq_lens)]
        self.num_seqs = len(self.seq_lens_host)
        if self.num_seqs == 0:
            raise ValueError("empty batch")
        n = self.num_seqs

        def host_list(values, what):
            if values is None:
                return None
            v = values.tolist() if isinstance(values, torch.Tensor) else values
            if isinstance(v, int):
                v = [v] * n
            v = [int(x) for x in v]
            if len(v) != n:
                raise ValueError(f"{what} has {len(v)} entries for {n} sequences")
            return v

        rs = host_list(round_start, "round_start") or self.seq_lens_host
        pf = host_list(prefill_lens, "prefill_lens")
        self.budgets_host = None
        bud = host_list(budgets, "budgets")
        if bud is not None:
            self.budgets_host = [min(x, t) for x, t in zip(bud, self.seq_lens_host)]
        rows, pitch = None, 0
        if block_tables is not None and not isinstance(block_tables, torch.Tensor):
            if len(block_tables) != n:
                raise ValueError("block table rows != number of sequences")
            pitch = max(len(r) for r in block_tables)
            rows = [int(x) for r in block_tables for x in (list(r) + [0] * (pitch - len(r)))]
        # One host-to-device copy for all the small integer arrays of the step.
        parts = [self.seq_lens_host, rs, pf or [], self.budgets_host or [], rows or []]
        flat = torch.tensor([x for part in parts for x in part], dtype=torch.int32,
                            pin_memory=True).to(device, non_blocking=True)
        cuts, pos = [], 0
        for part in parts:
            cuts.append(flat[pos:pos + len(part)])
            pos += len(part)
        self._flat, self._sizes, self._table_in_flat = flat, [len(part) for part in parts], rows is not None
        self.seq_lens, self.round_start = cuts[0], cuts[1]
        self.prefill_lens = cuts[2] if pf is not None else None
        self.budgets = cuts[3] if self.budgets_host is not None else None
        self.block_table = None
        if rows is not None:
            self.block_table = cuts[4].view(n, pitch)
        elif block_tables is not None:
            bt = block_tables.to(device=device, dtype=torch.int32)
            if bt.ndim == 1:
                bt = bt.unsqueeze(0)
            self.block_table = bt.contiguous()
            pitch = int(self.block_table.shape[1])
            if int(self.block_table.shape[0]) != n:
                raise ValueError("block table rows != number of sequences")
        self.max_seq_len = max(self.seq_lens_host)
        self.max_budget = max(self.budgets_host) if self.budgets_host else 0
        self._lens_host = (C.c_int32 * n)(*self.seq_lens_host)     # kept alive with the batch
        self.struct = Batch(
            num_seqs=self.num_seqs, max_seq_len=self.max_seq_len, max_budget=self.max_budget,
            block_table_pitch=pitch, block_table=_ptr(self.block_table), seq_lens=_ptr(self.seq_lens),
            round_start=_ptr(self.round_start), prefill_lens=_ptr(self.prefill_lens),
            budgets=_ptr(self.budgets), seq_lens_host=C.cast(self._lens_host, C.c_void_p))

    _recent: "dict[tuple, StepBatch]" = {}

    @classmethod
    def for_request(cls, device, total_tokens: int, block_ids, round_start: int | None = None,
                    budget: int | None = None, prefill_len: int | None = None) -> "StepBatch":
        """The batch of a single request, for callers that come back with the same request several
        times in a row (the per-layer selection modes: one selection and one compaction per layer,
        all with the same lengths and block ids): built once per set of values and reused.  The
        device arrays of a batch are only ever read, so sharing one between launches is safe."""
        ids = tuple(int(x) for x in block_ids)
        key = (str(device), int(total_tokens), ids, round_start, budget, prefill_len)
        hit = cls._recent.get(key)
        if hit is None:
            hit = cls(device, [int(total_tokens)], round_start=None if round_start is None else [int(round_start)],
                      budgets=None if budget is None else [int(budget)], block_tables=[list(ids)],
                      prefill_lens=None if prefill_len is None else [int(prefill_len)])
            if len(cls._recent) >= 8:
                cls._recent.pop(next(iter(cls._recent)))
            cls._recent[key] = hit
        return hit

    def refill(self, round_start, block_tables, prefill_lens=None) -> None:
        """New round starts, block tables and prefill lengths for the SAME sequence lengths and
        budgets, written into the device arrays this batch already owns (their addresses do not
        change: a launch sequence captured into a HIP graph with this batch can be replayed).
        One pinned host-to-device copy, stream ordered."""
        n = self.num_seqs
        if not self._table_in_flat:
            raise ValueError("this batch was not built from host lists with block tables")
        pitch = int(self.block_table.shape[1])
        if len(block_tables) != n or len(round_start) != n or (prefill_lens is not None and len(prefill_lens) != n):
            raise ValueError("refill needs the shapes the batch was built with")
        staging = getattr(self, "_staging", None)
        if staging is None:
            # Pinned mirror of the device array; the lengths and budgets in it never change.
            staging = self._staging = torch.empty(self._flat.numel(), dtype=torch.int32, pin_memory=True)
            self._host = staging.numpy()
            self._host[:n] = self.seq_lens_host
            o = 2 * n + self._sizes[2]
            self._host[o:o + self._sizes[3]] = self.budgets_host or []
            self._staged = torch.cuda.Event()
        else:
            self._staged.synchronize()          # the previous copy out of the staging buffer has finished
        host = self._host
        host[n:2 * n] = round_start
        if self.prefill_lens is not None:
            host[2 * n:3 * n] = prefill_lens if prefill_lens is not None else 0
        o = 2 * n + self._sizes[2] + self._sizes[3]
        for r in block_tables:
            m = len(r)
            if m > pitch:
                raise ValueError(f"a block table of {m} entries does not fit the batch's pitch of {pitch}")
            host[o:o + m] = r
            host[o + m:o + pitch] = 0
            o += pitch
        self._flat.copy_(staging, non_blocking=True)
        self._staged.record()

    def check_capacity(self, block_size: int) -> None:
        """Host-side bounds check: every sequence owns enough blocks for its tokens."""
        if self.block_table is None:
            return
        pitch = int(self.block_table.shape[1])
        for t in self.seq_lens_host:
            if (t + block_size - 1) // block_size > pitch:
                raise IndexError(f"sequence of {t} tokens needs more than {pitch} blocks of {block_size}")


@dataclass
class ScoreConfig:
    folded: torch.Tensor        # [L, A, 3, F] fp32 from fold_stats
    omega: torch.Tensor         # [F] fp32
    offsets: torch.Tensor       # [NO] fp32
    aggregation: str = "mean"

    @property
    def num_score_heads(self) -> int:
        return int(self.folded.shape[1])

    def struct(self) -> ScoreParams:
        return ScoreParams(num_score_heads=self.num_score_heads, num_offsets=int(self.offsets.numel()),
                           aggregation=REDUCE_MAX if self.aggregation == "max" else REDUCE_MEAN,
                           folded=_ptr(self.folded), omega=_ptr(self.omega), offsets=_ptr(self.offsets))


@dataclass
class SelectConfig:
    normalize: bool | str = True         # True / False, or "population": population std clamped at 1e-6 (research path)
    window_size: int = 128
    protect_prefill: bool = False
    group_reduce: str = "max"
    layer_reduce: str | None = "mean"    # None: one keep set per layer
    shared: bool = False
    group_first: bool = False            # reduce over the query heads of a KV head before normalising
    allow_resident: bool = True          # False: never a resident kernel (repeat of a step whose resident launch failed)

    def struct(self) -> SelectParams:
        lr = REDUCE_NONE if self.layer_reduce is None else (REDUCE_MAX if self.layer_reduce == "max" else REDUCE_MEAN)
        return SelectParams(normalize=2 if self.normalize == "population" else int(bool(self.normalize)),
                            window_size=int(self.window_size),
                            protect_prefill=int(self.protect_prefill),
                            group_reduce=REDUCE_MAX if self.group_reduce == "max" else REDUCE_MEAN,
                            layer_reduce=lr, shared=int(self.shared), group_first=int(self.group_first),
                            no_resident=int(not self.allow_resident))


def fold_stats(q_mean_complex: torch.Tensor, q_abs_mean: torch.Tensor, freq_scale_sq: torch.Tensor,
               disable_mlr: bool = False, disable_trig: bool = False) -> torch.Tensor:
    """[L, A, F, 2], [L, A, F], [L, A, F] device fp32 -> folded [L, A, 3, F]."""
    lib = _lib.load()
    if not q_mean_complex.is_cuda:
        raise RuntimeError("fold_stats needs device tensors (there is no CPU fallback)")
    qr = q_mean_complex[..., 0].to(torch.float32).contiguous()
    qi = q_mean_complex[..., 1].to(torch.float32).contiguous()
    qa = q_abs_mean.to(torch.float32).contiguous()
    fs = freq_scale_sq.to(torch.float32).contiguous()
    if qr.ndim != 3 or qa.shape != qr.shape or fs.shape != qr.shape:
        raise ValueError("stats must be [L, A, F]")
    L, A, F = (int(x) for x in qr.shape)
    out = torch.empty(L, A, 3, F, dtype=torch.float32, device=qr.device)
    _lib.check(lib.tri_fold_stats(_ptr(qr), _ptr(qi), _ptr(qa), _ptr(fs), L, A, F, int(disable_mlr),
                                  int(disable_trig), _ptr(out), _stream()))
    return out


class Workspace:
    """Device scratch for one (layout, batch, score config); reusable across steps."""

    def __init__(self, kv: PagedKV, batch: StepBatch, sc: ScoreConfig):
        lib = _lib.load()
        sp = sc.struct()
        self.bytes = int(lib.tri_workspace_bytes(C.byref(kv.struct), C.byref(batch.struct), C.byref(sp)))
        if self.bytes == 0:
            raise ValueError("invalid layout / batch / score parameters: " +
                             lib.tri_last_error().decode("utf-8", "replace"))
        self.buf = torch.empty(self.bytes + 256, dtype=torch.uint8, device=kv.device)
        off = (-self.buf.data_ptr()) % 256
        self.ptr = self.buf.data_ptr() + off
        # The library keeps the status word at one offset for every shape, so a workspace reused
        # for another batch (fits()) still reads the word the kernels of that batch write.
        self._status_at = off + int(lib.tri_workspace_status_offset(C.byref(kv.struct), C.byref(batch.struct),
                                                                    C.byref(sp)))

    def status(self) -> int:
        """Synchronises the device, then returns the resident kernel's status word (0 = fine).
        The word travels to pinned host memory with a copy queued on the current stream before
        that wait, so the host waits once."""
        if getattr(self, "_status_host", None) is None:
            self._status_host = torch.empty(1, dtype=torch.int32, pin_memory=True)
        self._status_host.copy_(self.buf[self._status_at:self._status_at + 4].view(torch.int32), non_blocking=True)
        torch.cuda.synchronize(self.buf.device)
        return int(self._status_host[0])

    def fits(self, kv, batch, sc) -> bool:
        if self.buf.device != kv.device:
            return False
        sp = sc.struct()
        need = int(_lib.load().tri_workspace_bytes(C.byref(kv.struct), C.byref(batch.struct), C.byref(sp)))
        return 0 < need <= self.bytes


def _check_devices(kv: PagedKV, sc: ScoreConfig):
    for t in (sc.folded, sc.omega, sc.offsets):
        if t.device != kv.device or t.dtype != torch.float32 or not t.is_contiguous():
            raise ValueError("score parameters must be contiguous fp32 tensors on the cache's device")
    if int(sc.folded.shape[0]) != kv.num_layers or int(sc.folded.shape[3]) != kv.head_dim // 2:
        raise ValueError(f"folded stats {tuple(sc.folded.shape)} do not match {kv.num_layers} layers / "
                         f"head_dim {kv.head_dim}")


def score_paged(kv: PagedKV, batch: StepBatch, sc: ScoreConfig, ws: Workspace | None = None,
                head_major: bool = False, out: torch.Tensor | None = None):
    """Raw scores of every key.  Returns (raw, ws); raw is [B, L, Tmax, A] fp32, or
    [B, L, A, Tmax] when head_major (the reference's [batch, heads, seq] order)."""
    lib = _lib.load()
    _check_devices(kv, sc)
    batch.check_capacity(kv.block_size)
    ws = ws if ws is not None and ws.fits(kv, batch, sc) else Workspace(kv, batch, sc)
    B, L, T, A = batch.num_seqs, kv.num_layers, batch.max_seq_len, sc.num_score_heads
    shape = (B, L, A, T) if head_major else (B, L, T, A)
    strides = (A * T, 1, T) if head_major else (T * A, A, 1)
    if out is not None:
        if tuple(out.shape) != shape or out.dtype != torch.float32 or not out.is_contiguous() or out.device != kv.device:
            raise ValueError(f"out must be a contiguous fp32 tensor of shape {shape} on the cache's device")
        raw = out
    else:
        raw = torch.empty(shape, dtype=torch.float32, device=kv.device)
    sp = sc.struct()
    _lib.check(lib.tri_score_paged(C.byref(kv.struct), C.byref(batch.struct), C.byref(sp), _ptr(raw),
                                   strides[0], strides[1], strides[2], ws.ptr, ws.bytes, _stream()))
    return raw, ws


def select(kv: PagedKV, batch: StepBatch, sc: ScoreConfig, sel: SelectConfig, raw: torch.Tensor,
           ws: Workspace, head_major: bool = False, want_scores: bool = False,
           keep: torch.Tensor | None = None):
    """keep int32 [rows, max_budget] (ascending) and optionally the selection scores."""
    lib = _lib.load()
    if batch.budgets is None:
        raise ValueError("batch has no budgets")
    B, L, T, A = batch.num_seqs, kv.num_layers, batch.max_seq_len, sc.num_score_heads
    strides = (A * T, 1, T) if head_major else (T * A, A, 1)
    rows = B * (L if sel.layer_reduce is None else 1) * (1 if sel.shared else kv.num_kv_heads)
    if keep is None:
        keep = torch.empty(rows, batch.max_budget, dtype=torch.int32, device=kv.device)
    elif (keep.numel() != rows * batch.max_budget or keep.dtype != torch.int32 or not keep.is_contiguous()
          or keep.device != kv.device):
        raise ValueError(f"keep must be a contiguous int32 tensor with {rows} x {batch.max_budget} entries")
    if raw.numel() != B * L * T * A or raw.dtype != torch.float32 or not raw.is_contiguous():
        raise ValueError("raw must be the contiguous fp32 tensor returned by score_paged for this batch")
    fin = torch.empty(rows, T, dtype=torch.float32, device=kv.device) if want_scores else None
    sp, ss = sc.struct(), sel.struct()
    _lib.check(lib.tri_select(C.byref(kv.struct), C.byref(batch.struct), C.byref(sp), C.byref(ss), _ptr(raw),
                              strides[0], strides[1], strides[2], _ptr(fin), _ptr(keep), ws.ptr, ws.bytes,
                              _stream()))
    return keep, fin


def select_paged(kv: PagedKV, batch: StepBatch, sc: ScoreConfig, sel: SelectConfig,
                 ws: Workspace | None = None, want_scores: bool = False, keep: torch.Tensor | None = None,
                 scores_out: torch.Tensor | None = None, want_keep: bool = True):
    """Score and select in one call; the raw scores stay on the device side (in LDS when
    the shape has a resident kernel).  Returns (keep, selection scores or None, ws);
    with want_keep=False only the selection scores are produced (see topk_batch)."""
    lib = _lib.load()
    _check_devices(kv, sc)
    if batch.budgets is None:
        raise ValueError("batch has no budgets")
    batch.check_capacity(kv.block_size)
    ws = ws if ws is not None and ws.fits(kv, batch, sc) else Workspace(kv, batch, sc)
    rows = batch.num_seqs * (kv.num_layers if sel.layer_reduce is None else 1) * (1 if sel.shared else kv.num_kv_heads)
    if not want_keep:
        keep, want_scores = None, True
    elif keep is None:
        keep = torch.empty(rows, batch.max_budget, dtype=torch.int32, device=kv.device)
    elif (keep.numel() != rows * batch.max_budget or keep.dtype != torch.int32 or not keep.is_contiguous()
          or keep.device != kv.device):
        raise ValueError(f"keep must be a contiguous int32 tensor with {rows} x {batch.max_budget} entries")
    fin = None
    if scores_out is not None:
        if (tuple(scores_out.shape) != (rows, batch.max_seq_len) or scores_out.dtype != torch.float32
                or not scores_out.is_contiguous() or scores_out.device != kv.device):
            raise ValueError(f"scores_out must be a contiguous fp32 [{rows}, {batch.max_seq_len}] device tensor")
        fin = scores_out
    elif want_scores:
        fin = torch.empty(rows, batch.max_seq_len, dtype=torch.float32, device=kv.device)
    sp, ss = sc.struct(), sel.struct()
    _lib.check(lib.tri_select_paged(C.byref(kv.struct), C.byref(batch.struct), C.byref(sp), C.byref(ss),
                                    _ptr(fin), _ptr(keep), ws.ptr, ws.bytes, _stream()))
    return keep, fin, ws


def select_path(kv: PagedKV, batch: StepBatch, sc: ScoreConfig, sel: SelectConfig) -> str:
    """'resident_mfma' / 'resident_valu' when select_paged / compress_step run the single
    resident kernel (scoring on the matrix cores / on the vector unit) for these arguments
    on the current device, else 'two_pass'."""
    sp, ss = sc.struct(), sel.struct()
    rc = int(_lib.load().tri_select_path(C.byref(kv.struct), C.byref(batch.struct), C.byref(sp), C.byref(ss)))
    if rc < 0:
        raise ValueError("invalid arguments: " + _lib.load().tri_last_error().decode("utf-8", "replace"))
    return {2: "resident_mfma", 1: "resident_valu"}.get(rc, "two_pass")


def describe_plan(kv: PagedKV, batch: StepBatch, sc: ScoreConfig, sel: SelectConfig,
                  assume_resident_workgroups: int = 0) -> dict:
    """How select_paged / compress_step would cut these arguments into workgroups (``tri_describe_plan``):
    path, tile length, tiles of the longest sequence, layer groups, launches, workspace bytes --
    for the current device, or for one that holds ``assume_resident_workgroups`` at once."""
    sp, ss, info = sc.struct(), sel.struct(), _lib.PlanInfo()
    _lib.check(_lib.load().tri_describe_plan(C.byref(kv.struct), C.byref(batch.struct), C.byref(sp), C.byref(ss),
                                             int(assume_resident_workgroups), C.byref(info)))
    out = {name: int(getattr(info, name)) for name, _ in _lib.PlanInfo._fields_}
    out["path"] = {2: "resident_mfma", 1: "resident_valu"}.get(out["path"], "two_pass")
    return out


def topk_rows(scores: torch.Tensor, k: int | Sequence[int], lens: Sequence[int] | None = None) -> torch.Tensor:
    """Ascending int32 indices of the k largest entries of every row of a 2-D fp32 tensor."""
    lib = _lib.load()
    if not scores.is_cuda:
        raise RuntimeError("topk_rows needs a device tensor (there is no CPU fallback)")
    if scores.ndim != 2 or scores.dtype != torch.float32 or scores.stride(1) != 1:
        raise ValueError("scores must be a 2-D fp32 tensor with contiguous rows")
    R, T = (int(x) for x in scores.shape)
    ks = [int(k)] * R if isinstance(k, int) else [int(x) for x in k]
    ls = [T] * R if lens is None else [int(x) for x in lens]
    kmax = max(max(ks), 1)
    keep = torch.empty(R, kmax, dtype=torch.int32, device=scores.device)
    lens_t, ks_t = _i32(ls, scores.device), _i32(ks, scores.device)
    _lib.check(lib.tri_topk_rows(_ptr(scores), int(scores.stride(0)), R, _ptr(lens_t), _ptr(ks_t), 1, T,
                                 _ptr(keep), kmax, _stream()))
    return keep


def query_stats(q_rot: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, scale: float = 1.0,
                rope_style: str = "half"):
    """Frequency statistics of one layer's captured query states (scripts/calibrate.py:196-224).

    q_rot [H, T, D] (any strides with contiguous D), cos / sin [T, D], all bf16 or all fp16 on
    the device.  Returns fp32 [H, D/2] tensors (q_mean_real, q_mean_imag, q_abs_mean).
    """
    lib = _lib.load()
    if not q_rot.is_cuda:
        raise RuntimeError("query_stats needs device tensors (there is no CPU fallback)")
    if q_rot.ndim != 3 or q_rot.dtype not in (torch.bfloat16, torch.float16) or q_rot.stride(2) != 1:
        raise ValueError("q_rot must be a [H, T, D] bf16/fp16 tensor with contiguous head_dim")
    H, T, D = (int(x) for x in q_rot.shape)
    if T == 0:
        raise ValueError("no tokens")
    tables = []
    for name, t in (("cos", cos), ("sin", sin)):
        if t.ndim == 3 and t.shape[0] == 1:
            t = t[0]
        if tuple(t.shape) != (T, D) or t.dtype != q_rot.dtype or t.device != q_rot.device:
            raise ValueError(f"{name} must be a [{T}, {D}] tensor of q_rot's dtype on its device")
        tables.append(t.contiguous())
    if rope_style not in ("half", "interleaved"):
        raise ValueError(f"rope_style must be 'half' or 'interleaved', got {rope_style!r}")
    nbytes = int(lib.tri_qstats_workspace_bytes(H, T, D))
    if nbytes == 0:
        raise ValueError(f"unsupported head_dim {D} (64, 128 or 256)")
    ws = torch.empty(nbytes, dtype=torch.uint8, device=q_rot.device)
    out = torch.empty(3, H, D // 2, dtype=torch.float32, device=q_rot.device)
    _lib.check(lib.tri_qstats(_ptr(q_rot), int(q_rot.stride(0)), int(q_rot.stride(1)), _ptr(tables[0]), _ptr(tables[1]),
                              H, T, D, _DTYPES[q_rot.dtype], ROPE_INTERLEAVED if rope_style == "interleaved" else ROPE_HALF,
                              float(scale), _ptr(out[0]), _ptr(out[1]), _ptr(out[2]), _ptr(ws), nbytes, _stream()))
    return out[0], out[1], out[2]


def topk_batch(scores: torch.Tensor, batch: StepBatch, rows_per_seq: int, keep: torch.Tensor | None = None):
    """keep rows (ascending int32 [rows, max_budget]) from selection scores [rows, Tmax] with
    the batch's own device-side lengths and budgets; rows_per_seq rows belong to a sequence."""
    lib = _lib.load()
    if batch.budgets is None:
        raise ValueError("batch has no budgets")
    rows, T = (int(x) for x in scores.shape)
    if (rows != batch.num_seqs * rows_per_seq or T != batch.max_seq_len or scores.dtype != torch.float32
            or not scores.is_contiguous()):
        raise ValueError("scores must be the contiguous fp32 [rows, max_seq_len] tensor of select_paged")
    if keep is None:
        keep = torch.empty(rows, batch.max_budget, dtype=torch.int32, device=scores.device)
    _lib.check(lib.tri_topk_rows(_ptr(scores), T, rows, _ptr(batch.seq_lens), _ptr(batch.budgets), rows_per_seq, T,
                                 _ptr(keep), batch.max_budget, _stream()))
    return keep


def compact(kv: PagedKV, batch: StepBatch, keep: torch.Tensor, keep_per_layer: bool = False,
            shared: bool = False, full_permutation: bool = False) -> None:
    """In-place compaction of K and V of every layer.  keep: ascending int32 rows."""
    lib = _lib.load()
    if batch.budgets is None or batch.block_table is None:
        raise ValueError("compaction needs budgets and block tables")
    batch.check_capacity(kv.block_size)
    rows = batch.num_seqs * (kv.num_layers if keep_per_layer else 1) * (1 if shared else kv.num_kv_heads)
    if keep.dtype != torch.int32 or not keep.is_contiguous() or keep.device != kv.device:
        raise ValueError("keep must be a contiguous int32 tensor on the cache's device")
    if keep.numel() != rows * batch.max_budget:
        raise ValueError(f"keep has {keep.numel()} entries, expected {rows} x {batch.max_budget}")
    if full_permutation:
        need = int(lib.tri_compact_full_staging_bytes(C.byref(kv.struct), C.byref(batch.struct)))
        staging = torch.empty(need + 16, dtype=torch.uint8, device=kv.device)
        _lib.check(lib.tri_compact_paged_full(C.byref(kv.struct), C.byref(batch.struct), _ptr(keep),
                                              int(keep_per_layer), int(shared), _ptr(staging), need, _stream()))
        # The staging tensor is released to torch's caching allocator, which keeps it
        # alive until work already queued on this stream has finished with it.
        return
    _lib.check(lib.tri_compact_paged(C.byref(kv.struct), C.byref(batch.struct), _ptr(keep),
                                     int(keep_per_layer), int(shared), _stream()))


def compress_step(kv: PagedKV, batch: StepBatch, sc: ScoreConfig, sel: SelectConfig,
                  ws: Workspace | None = None, keep: torch.Tensor | None = None):
    """score + select + compact for every layer of every sequence.  Returns (keep, ws)."""
    lib = _lib.load()
    _check_devices(kv, sc)
    if batch.budgets is None or batch.block_table is None:
        raise ValueError("compress_step needs budgets and block tables")
    batch.check_capacity(kv.block_size)
    ws = ws if ws is not None and ws.fits(kv, batch, sc) else Workspace(kv, batch, sc)
    rows = batch.num_seqs * (kv.num_layers if sel.layer_reduce is None else 1) * (1 if sel.shared else kv.num_kv_heads)
    if keep is None:
        keep = torch.empty(rows, batch.max_budget, dtype=torch.int32, device=kv.device)
    sp, ss = sc.struct(), sel.struct()
    _lib.check(lib.tri_compress_step(C.byref(kv.struct), C.byref(batch.struct), C.byref(sp), C.byref(ss),
                                     _ptr(keep), ws.ptr, ws.bytes, _stream()))
    return keep, ws


class resident_gate:
    """Brackets the replay of a captured launch sequence that contains a resident kernel: on entry the
    current stream waits (on the device) for the process's previous resident launch, on exit the replay
    is recorded as the latest one (``tri_resident_gate_enter`` / ``_leave``).  Launches the library issues
    outside graph capture chain themselves; a graph holds no such wait or record."""

    def __enter__(self):
        _lib.check(_lib.load().tri_resident_gate_enter(_stream()))
        return self

    def __exit__(self, *exc):
        _lib.check(_lib.load().tri_resident_gate_leave(_stream()))
        return False


def compress_step_static(kv: PagedKV, batch: StepBatch, sc: ScoreConfig, sel: SelectConfig, keep: torch.Tensor):
    """``compress_step`` on the library's own static scratch: the call allocates nothing (``keep``
    is the caller's, int32 [rows, max_budget]), always takes the score-then-select kernels, and
    rejects steps whose scratch exceeds ``_lib.STATIC_WORKSPACE_BYTES``.  Calls that overlap
    in time on one GPU share that scratch and race.  Returns the device address of the status word."""
    lib = _lib.load()
    _check_devices(kv, sc)
    if batch.budgets is None or batch.block_table is None:
        raise ValueError("compress_step_static needs budgets and block tables")
    batch.check_capacity(kv.block_size)
    rows = batch.num_seqs * (kv.num_layers if sel.layer_reduce is None else 1) * (1 if sel.shared else kv.num_kv_heads)
    if (keep.numel() != rows * batch.max_budget or keep.dtype != torch.int32 or not keep.is_contiguous()
            or keep.device != kv.device):
        raise ValueError(f"keep must be a contiguous int32 tensor with {rows} x {batch.max_budget} entries")
    sp, ss = sc.struct(), sel.struct()
    status = C.c_void_p()
    _lib.check(lib.tri_compress_step_static(C.byref(kv.struct), C.byref(batch.struct), C.byref(sp), C.byref(ss),
                                            _ptr(keep), C.byref(status), _stream()))
    return int(status.value or 0)
