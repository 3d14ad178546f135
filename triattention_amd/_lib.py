"""ctypes binding of libtriattention_hip.so (the C ABI in include/triattention_hip.h).

There is no fallback: if the shared library is missing, ``load()`` raises, and so
does every operator that needs it.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

import os

# TRIATTN_HIP_LIBRARY points at another build of the same ABI (e.g. an instrumented one).
LIB_PATH = Path(os.environ.get("TRIATTN_HIP_LIBRARY") or Path(__file__).resolve().parent / "libtriattention_hip.so")

ABI_VERSION = 6
STATIC_WORKSPACE_BYTES = 64 << 20
TRI_OK = 0
TRI_ERR_INVALID_ARGUMENT = -1
TRI_ERR_UNSUPPORTED = -2
TRI_ERR_WORKSPACE = -3
TRI_ERR_LAUNCH = -4

KV_BF16, KV_FP16, KV_FP8_E4M3 = 0, 1, 2
ROPE_HALF, ROPE_INTERLEAVED = 0, 1
REDUCE_MEAN, REDUCE_MAX, REDUCE_NONE = 0, 1, -1

# tri_tuning keys
TUNE_RESIDENT_KERNEL, TUNE_RESIDENT_WORKGROUPS, TUNE_LAYER_SPLIT, TUNE_MAX_KERNEL, TUNE_RESIDENT_WAIT_US = range(5)
RESIDENT_KERNEL_CHOICES = {"auto": 0, "mfma": 1, "valu": 2, "off": 3}

EXPORTS = (
    "tri_abi_version", "tri_last_error", "tri_source_digest", "tri_set_tuning", "tri_get_tuning", "tri_resident_gate_enter",
    "tri_resident_gate_leave", "tri_fold_stats", "tri_workspace_bytes", "tri_workspace_status_offset",
    "tri_score_paged",
    "tri_select", "tri_select_paged", "tri_select_path", "tri_describe_plan", "tri_topk_rows", "tri_compact_paged", "tri_compact_full_staging_bytes",
    "tri_compact_paged_full", "tri_compress_step", "tri_compress_step_static", "tri_qstats_workspace_bytes", "tri_qstats",
)


class KvLayout(C.Structure):
    _fields_ = [
        ("num_layers", C.c_int32), ("num_kv_heads", C.c_int32), ("head_dim", C.c_int32),
        ("block_size", C.c_int32), ("kv_dtype", C.c_int32), ("rope_style", C.c_int32),
        ("stride_block", C.c_int64), ("stride_token", C.c_int64), ("stride_head", C.c_int64),
        ("k_layers", C.c_void_p), ("v_layers", C.c_void_p),
        ("k_scale_layers", C.c_void_p), ("v_scale_layers", C.c_void_p),
    ]


class Batch(C.Structure):
    _fields_ = [
        ("num_seqs", C.c_int32), ("max_seq_len", C.c_int32), ("max_budget", C.c_int32),
        ("block_table_pitch", C.c_int32),
        ("block_table", C.c_void_p), ("seq_lens", C.c_void_p), ("round_start", C.c_void_p),
        ("prefill_lens", C.c_void_p), ("budgets", C.c_void_p), ("seq_lens_host", C.c_void_p),
    ]


class PlanInfo(C.Structure):
    _fields_ = [
        ("path", C.c_int32), ("tile_tokens", C.c_int32), ("tiles_per_seq", C.c_int32), ("layer_groups", C.c_int32),
        ("layers_per_group", C.c_int32), ("launches", C.c_int32), ("waves_per_workgroup", C.c_int32),
        ("resident_workgroups", C.c_int32), ("workspace_bytes", C.c_int64),
    ]


class ScoreParams(C.Structure):
    _fields_ = [
        ("num_score_heads", C.c_int32), ("num_offsets", C.c_int32), ("aggregation", C.c_int32),
        ("folded", C.c_void_p), ("omega", C.c_void_p), ("offsets", C.c_void_p),
    ]


class SelectParams(C.Structure):
    _fields_ = [
        ("normalize", C.c_int32), ("window_size", C.c_int32), ("protect_prefill", C.c_int32),
        ("group_reduce", C.c_int32), ("layer_reduce", C.c_int32), ("shared", C.c_int32),
        ("group_first", C.c_int32), ("no_resident", C.c_int32),
    ]


class TriError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"libtriattention_hip error {code}: {message}")
        self.code = code


_lib = None


def load() -> C.CDLL:
    """Load the library once; raise if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m triattention_amd.build` "
            "(hipcc, gfx950). There is no CPU or PyTorch fallback for this path.")
    lib = C.CDLL(str(LIB_PATH))
    P, I32, I64, U64 = C.c_void_p, C.c_int32, C.c_int64, C.c_uint64
    lib.tri_abi_version.restype = C.c_int
    lib.tri_last_error.restype = C.c_char_p
    lib.tri_source_digest.restype = C.c_char_p
    lib.tri_set_tuning.argtypes = [I32, I64]
    lib.tri_get_tuning.argtypes = [I32]
    lib.tri_get_tuning.restype = I64
    lib.tri_resident_gate_enter.argtypes = [P]
    lib.tri_resident_gate_leave.argtypes = [P]
    lib.tri_fold_stats.argtypes = [P, P, P, P, I32, I32, I32, I32, I32, P, P]
    lib.tri_workspace_bytes.argtypes = [C.POINTER(KvLayout), C.POINTER(Batch), C.POINTER(ScoreParams)]
    lib.tri_workspace_bytes.restype = U64
    lib.tri_workspace_status_offset.argtypes = [C.POINTER(KvLayout), C.POINTER(Batch), C.POINTER(ScoreParams)]
    lib.tri_workspace_status_offset.restype = U64
    lib.tri_score_paged.argtypes = [C.POINTER(KvLayout), C.POINTER(Batch), C.POINTER(ScoreParams),
                                    P, I64, I64, I64, P, U64, P]
    lib.tri_select.argtypes = [C.POINTER(KvLayout), C.POINTER(Batch), C.POINTER(ScoreParams),
                               C.POINTER(SelectParams), P, I64, I64, I64, P, P, P, U64, P]
    lib.tri_select_paged.argtypes = [C.POINTER(KvLayout), C.POINTER(Batch), C.POINTER(ScoreParams),
                                     C.POINTER(SelectParams), P, P, P, U64, P]
    lib.tri_select_path.argtypes = [C.POINTER(KvLayout), C.POINTER(Batch), C.POINTER(ScoreParams),
                                    C.POINTER(SelectParams)]
    lib.tri_describe_plan.argtypes = [C.POINTER(KvLayout), C.POINTER(Batch), C.POINTER(ScoreParams),
                                      C.POINTER(SelectParams), I32, C.POINTER(PlanInfo)]
    lib.tri_topk_rows.argtypes = [P, I64, I32, P, P, I32, I32, P, I32, P]
    lib.tri_compact_paged.argtypes = [C.POINTER(KvLayout), C.POINTER(Batch), P, I32, I32, P]
    lib.tri_compact_full_staging_bytes.argtypes = [C.POINTER(KvLayout), C.POINTER(Batch)]
    lib.tri_compact_full_staging_bytes.restype = U64
    lib.tri_compact_paged_full.argtypes = [C.POINTER(KvLayout), C.POINTER(Batch), P, I32, I32, P, U64, P]
    lib.tri_compress_step.argtypes = [C.POINTER(KvLayout), C.POINTER(Batch), C.POINTER(ScoreParams),
                                      C.POINTER(SelectParams), P, P, U64, P]
    lib.tri_compress_step_static.argtypes = [C.POINTER(KvLayout), C.POINTER(Batch), C.POINTER(ScoreParams),
                                             C.POINTER(SelectParams), P, C.POINTER(C.c_void_p), P]
    lib.tri_qstats_workspace_bytes.argtypes = [I32, I32, I32]
    lib.tri_qstats_workspace_bytes.restype = U64
    lib.tri_qstats.argtypes = [P, I64, I64, P, P, I32, I32, I32, I32, I32, C.c_float, P, P, P, P, U64, P]
    for name in EXPORTS:
        fn = getattr(lib, name)
        if fn.restype is C.c_int and name not in ("tri_abi_version",):
            fn.restype = C.c_int
    if lib.tri_abi_version() != ABI_VERSION:
        raise RuntimeError(f"{LIB_PATH}: ABI version {lib.tri_abi_version()} != {ABI_VERSION}; rebuild the library")
    _lib = lib
    _apply_environment(lib)
    return lib


def _apply_environment(lib) -> None:
    """The library reads no environment variable; the ones documented for comparison runs are
    applied here, once, when the library is loaded (later changes of the environment have no
    effect: use ``set_tuning``)."""
    env = os.environ
    v = env.get("TRIATTN_RESIDENT_KERNEL", "").strip().lower()
    if v:
        if v not in RESIDENT_KERNEL_CHOICES:
            raise ValueError(f"TRIATTN_RESIDENT_KERNEL={v!r}: one of {sorted(RESIDENT_KERNEL_CHOICES)}")
        lib.tri_set_tuning(TUNE_RESIDENT_KERNEL, RESIDENT_KERNEL_CHOICES[v])
    for name, key in (("TRIATTN_RESIDENT_WORKGROUPS", TUNE_RESIDENT_WORKGROUPS),
                      ("TRIATTN_RESIDENT_LAYER_SPLIT", TUNE_LAYER_SPLIT)):
        v = env.get(name, "").strip()
        if v:
            lib.tri_set_tuning(key, int(v))
    v = env.get("TRIATTN_RESIDENT_SPIN_TICKS", "").strip()      # ticks of the 100 MHz wall clock
    if v:
        lib.tri_set_tuning(TUNE_RESIDENT_WAIT_US, -1 if int(v) < 0 else max(1, int(v) // 100))
    if env.get("TRIATTN_MAX_KERNEL", "").strip().lower() == "valu":
        lib.tri_set_tuning(TUNE_MAX_KERNEL, 1)


def set_tuning(key: int, value: int) -> int:
    """Set one process-wide setting of the library (``tri_set_tuning``); returns the previous value."""
    lib = load()
    old = int(lib.tri_get_tuning(key))
    check(lib.tri_set_tuning(key, int(value)))
    return old


def get_tuning(key: int) -> int:
    return int(load().tri_get_tuning(key))


class tuning:
    """Context manager: settings of the library for the duration of a block (tests, comparison runs).

        with tuning(resident_kernel="mfma", resident_workgroups=16): ...
    """

    _KEYS = {"resident_kernel": TUNE_RESIDENT_KERNEL, "resident_workgroups": TUNE_RESIDENT_WORKGROUPS,
             "layer_split": TUNE_LAYER_SPLIT, "max_kernel": TUNE_MAX_KERNEL, "resident_wait_us": TUNE_RESIDENT_WAIT_US}

    def __init__(self, **settings):
        self.settings, self.saved = {}, {}
        for name, value in settings.items():
            if name not in self._KEYS:
                raise KeyError(name)
            if name == "resident_kernel" and isinstance(value, str):
                value = RESIDENT_KERNEL_CHOICES[value]
            if name == "max_kernel" and isinstance(value, str):
                value = {"auto": 0, "valu": 1}[value]
            self.settings[self._KEYS[name]] = int(value)

    def __enter__(self):
        for key, value in self.settings.items():
            self.saved[key] = set_tuning(key, value)
        return self

    def __exit__(self, *exc):
        for key, value in self.saved.items():
            set_tuning(key, value)
        return False


def check(code: int) -> None:
    """Map a tri_status to a Python exception."""
    if code == TRI_OK:
        return
    msg = load().tri_last_error().decode("utf-8", "replace")
    raise TriError(code, msg)
