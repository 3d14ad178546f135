"""tri_compress_step_static: the entry point that allocates nothing (scratch in a device array
of the library) against tri_compress_step on a caller-provided workspace, through the C ABI."""
from __future__ import annotations

import ctypes as C

import pytest
import torch

from helpers import build_inputs, device_objects, tune
from triattention_amd import _lib, ops, synth

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _read_device_word(address: int) -> int:
    """Four bytes at a raw device address (the status word lives in the library's own array)."""
    hip = C.CDLL("libamdhip64.so")
    hip.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
    word = C.c_uint32(0xdeadbeef)
    torch.cuda.synchronize()
    assert hip.hipMemcpy(C.byref(word), C.c_void_p(address), 4, 2) == 0      # 2 = device to host
    return int(word.value)


def _both_ways(w, kv_axis=0):
    """One step through tri_compress_step (two-pass kernels, torch workspace) and one through
    tri_compress_step_static on identical caches; returns what each left behind."""
    inp = build_inputs(w, kv_axis)
    sel = ops.SelectConfig(window_size=w.window_size, allow_resident=False)
    caches_a, kv_a, batch_a, sc_a = device_objects(w, inp, DEV)
    keep_a, ws = ops.compress_step(kv_a, batch_a, sc_a, sel)
    assert ws.status() == 0
    caches_b, kv_b, batch_b, sc_b = device_objects(w, inp, DEV)
    keep_b = torch.full_like(keep_a, -7)
    sel_b = ops.SelectConfig(window_size=w.window_size)       # the entry point takes the two-pass kernels by itself
    status_at = ops.compress_step_static(kv_b, batch_b, sc_b, sel_b, keep_b)
    assert status_at != 0 and status_at % 256 == 0
    assert _read_device_word(status_at) == 0
    for b, t in enumerate(w.seq_lens):
        k = min(w.budget, t)
        rows = slice(b * w.num_kv_heads, (b + 1) * w.num_kv_heads)
        assert torch.equal(keep_a[rows, :k], keep_b[rows, :k]), (w.name, b)
    for l, (a, b) in enumerate(zip(caches_a, caches_b)):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16)), (w.name, l)
    if w.kv_dtype == "fp8":
        for a, b in zip(kv_a._keep[2] + kv_a._keep[3], kv_b._keep[2] + kv_b._keep[3]):
            assert torch.equal(a, b)
    return status_at


def test_static_scratch_step_equals_the_workspace_step_twice_in_a_row():
    """Two calls in a row share the one static array; the second is smaller, so whatever the first
    left beyond the second's regions must not matter."""
    big = synth.Workload("static_a", 3, 16, 4, 128, (1500, 700, 333), 256, index=31)
    small = synth.Workload("static_b", 2, 16, 4, 128, (600,), 128, index=32)
    first = _both_ways(big)
    second = _both_ways(small, kv_axis=1)
    assert first == second          # one array per GPU, one status word in it
    _both_ways(big)                 # and growing again after the small call


def test_static_scratch_step_at_the_steady_state_shape():
    """One request of budget + 128 tokens of a Qwen3-8B-shaped cache (4 of its layers)."""
    w = synth.Workload("static_steady", 4, 32, 8, 128, (2176,), 2048, index=33)
    _both_ways(w)


def test_static_scratch_step_moves_fp8_scales():
    w = synth.Workload("static_fp8", 2, 16, 4, 128, (900, 400), 200, kv_dtype="fp8", index=34)
    _both_ways(w)


def test_static_scratch_rejects_steps_beyond_its_array():
    w = synth.Workload("static_big", 2, 32, 8, 128, (16,), 8, index=35)
    inp = build_inputs(w)
    caches, kv, batch, sc = device_objects(w, inp, DEV)
    # claim a batch whose raw scores alone (64 x 36... here 2 layers x 400000 tokens x 32 heads x 4 B) exceed the array
    huge = ops.StepBatch(DEV, [400000], budgets=8, block_tables=[list(range(25000))])
    sp, ss = sc.struct(), ops.SelectConfig().struct()
    lib = _lib.load()
    need = int(lib.tri_workspace_bytes(C.byref(kv.struct), C.byref(huge.struct), C.byref(sp)))
    assert need > _lib.STATIC_WORKSPACE_BYTES
    keep = torch.empty(w.num_kv_heads, 8, dtype=torch.int32, device=DEV)
    rc = lib.tri_compress_step_static(C.byref(kv.struct), C.byref(huge.struct), C.byref(sp), C.byref(ss),
                                      keep.data_ptr(), None, None)
    assert rc == _lib.TRI_ERR_WORKSPACE and b"static array" in lib.tri_last_error()


def test_static_scratch_limits_are_the_documented_ones():
    """Qwen3-8B shapes: four requests of 2176 tokens or one of 11400 fit the array, five or 11500 do not
    (the scratch is sized for the score-then-select kernels the call runs, not for a resident plan).
    The refusals come from the host-side check; the accepted shapes are not launched here (the
    steady-state test above runs one)."""
    w = synth.Workload("static_limits", 36, 32, 8, 128, (16,), 8, index=36)
    inp = build_inputs(w)
    caches, kv, batch, sc = device_objects(w, inp, DEV)
    sp, ss = sc.struct(), ops.SelectConfig(window_size=128).struct()
    lib = _lib.load()
    keep = torch.empty(5 * w.num_kv_heads, 2048, dtype=torch.int32, device=DEV)
    for lens, fits in (((2176,) * 5, False), ((11500,), False)):
        claim = ops.StepBatch(DEV, list(lens), budgets=2048, block_tables=[list(range(800))] * len(lens))
        rc = lib.tri_compress_step_static(C.byref(kv.struct), C.byref(claim.struct), C.byref(sp), C.byref(ss),
                                          keep.data_ptr(), None, None)
        assert rc == _lib.TRI_ERR_WORKSPACE and b"static array" in lib.tri_last_error(), lens
    # the accepted side of the limit, through the planner's own answer for a device without resident kernels
    tune(resident_kernel="off")
    for lens in ((2176,) * 4, (11400,)):
        claim = ops.StepBatch(DEV, list(lens), budgets=2048, block_tables=[list(range(800))] * len(lens))
        need = int(lib.tri_workspace_bytes(C.byref(kv.struct), C.byref(claim.struct), C.byref(sp)))
        assert 0 < need <= _lib.STATIC_WORKSPACE_BYTES, (lens, need)


def _free_device_bytes() -> int:
    hip = C.CDLL("libamdhip64.so")
    free, total = C.c_size_t(0), C.c_size_t(0)
    assert hip.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
    return int(free.value)


def test_static_scratch_step_allocates_nothing_and_runs_under_graph_capture():
    """What the entry point is for.  After one warm-up call on the device (the first call looks up the
    array's address and asks the occupancy calculator once), a call leaves the device's free memory
    and torch's allocator exactly as they were, and the same call recorded into a HIP graph (where
    an allocation would abort the capture) replays with the eager call's results."""
    w = synth.Workload("static_graph", 3, 16, 4, 128, (1100, 640), 192, index=36)
    inp = build_inputs(w)
    sel = ops.SelectConfig(window_size=w.window_size)
    caches, kv, batch, sc = device_objects(w, inp, DEV)
    pristine = [c.clone() for c in caches]
    keep = torch.empty(w.num_seqs * w.num_kv_heads, batch.max_budget, dtype=torch.int32, device=DEV)
    status_at = ops.compress_step_static(kv, batch, sc, sel, keep)            # warm-up, and the eager result
    assert _read_device_word(status_at) == 0
    want_keep, want_caches = keep.clone(), [c.clone() for c in caches]

    def restore():
        for c, p in zip(caches, pristine):
            c.copy_(p)

    restore()
    torch.cuda.synchronize()
    before = (_free_device_bytes(), torch.cuda.memory_allocated(), torch.cuda.memory_reserved())
    ops.compress_step_static(kv, batch, sc, sel, keep)
    torch.cuda.synchronize()
    after = (_free_device_bytes(), torch.cuda.memory_allocated(), torch.cuda.memory_reserved())
    assert before == after
    assert torch.equal(keep, want_keep)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        restore()
        ops.compress_step_static(kv, batch, sc, sel, keep)                    # once on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    restore()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        ops.compress_step_static(kv, batch, sc, sel, keep)
    for rep in range(3):
        restore()
        keep.fill_(-3)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert _read_device_word(status_at) == 0
        assert torch.equal(keep, want_keep), rep
        for c, x in zip(caches, want_caches):
            assert torch.equal(c.view(torch.int16), x.view(torch.int16)), rep
