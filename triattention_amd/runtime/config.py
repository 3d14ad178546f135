"""Runtime settings: the TRIATTN_RUNTIME_* contract.

Same names, defaults, parsing and validation rules as the reference's
``TriAttentionRuntimeConfig`` (triattention/vllm/runtime/config.py:19-276), driven here
by one table instead of one call per field.  ``REQUIRE_TRITON_SCORING`` keeps its name
and now reads "require the accelerated (HIP) scorer"; ``SCORE_CHUNK_MAX_TOKENS`` is
accepted and validated but the fused scorer does not chunk.
"""
from __future__ import annotations

import os
from dataclasses import dataclass, fields
from pathlib import Path
from typing import Mapping

_TRUE = {"1", "true", "yes", "on"}
_FALSE = {"0", "false", "no", "off"}


def parse_bool(raw: str) -> bool:
    """1/true/yes/on, 0/false/no/off (any case); anything else is an error
    (runtime/config.py:10-16)."""
    token = raw.strip().lower()
    if token in _TRUE:
        return True
    if token in _FALSE:
        return False
    raise ValueError(f"Invalid boolean value: {raw!r}")


def _opt_str(raw: str, default):
    raw = raw.strip()
    return raw if raw else default


@dataclass
class TriAttentionRuntimeConfig:
    kv_budget: int = 2048
    divide_length: int = 128
    protect_prefill: bool = False
    disable_compression: bool = False

    enable_kv_usage_trigger: bool = False
    kv_usage_trigger: float = 0.98
    kv_usage_release: float = 0.90

    enable_experimental_kv_compaction: bool = True
    enable_experimental_block_reclaim: bool = True
    require_triton_scoring: bool = True
    require_physical_reclaim: bool = True
    log_decisions: bool = True
    fail_on_effective_len_regression: bool = True
    effective_len_regression_ratio: float = 0.9
    effective_len_guard_divide_multiples: int = 2
    score_chunk_max_tokens: int = 4096

    sparse_stats_path: Path | None = None
    model_path: Path | None = None
    pruning_mode: str = "per_head"
    sparse_score_aggregation: str = "mean"
    sparse_normalize_scores: bool = True
    window_size: int = 128
    include_prefill_in_budget: bool = True
    per_head_selection_semantics: str = "hf_aligned_global_per_head"
    layer_perhead_aggregation: str = "max"
    per_layer_aggregation: str = "max"
    allow_per_layer_mode: bool = False
    disable_mlr: bool = False
    disable_trig: bool = False
    disable_top_n_high_freq: int = 0

    @classmethod
    def from_env(cls, prefix: str = "TRIATTN_RUNTIME_",
                 environ: Mapping[str, str] | None = None) -> "TriAttentionRuntimeConfig":
        """Every field FOO is read from ``<prefix>FOO``; unset keeps the default."""
        env = os.environ if environ is None else environ
        values = {}
        for f in fields(cls):
            raw = env.get(prefix + f.name.upper())
            if raw is None:
                continue
            default = f.default
            if f.name in ("sparse_stats_path", "model_path"):
                text = _opt_str(raw, None)
                values[f.name] = Path(text) if text else None
            elif isinstance(default, bool):
                values[f.name] = parse_bool(raw)
            elif isinstance(default, int):
                values[f.name] = int(raw)
            elif isinstance(default, float):
                values[f.name] = float(raw)
            else:
                values[f.name] = _opt_str(raw, default) or default
        cfg = cls(**values)
        cfg.validate()
        return cfg

    def validate(self) -> None:
        """runtime/config.py:183-276."""
        def need(ok: bool, msg: str):
            if not ok:
                raise ValueError(msg)

        need(self.kv_budget > 0, f"kv_budget must be > 0, got {self.kv_budget}")
        need(self.divide_length > 0, f"divide_length must be > 0, got {self.divide_length}")
        need(0.0 < self.kv_usage_trigger <= 1.0,
             f"kv_usage_trigger must be in (0, 1], got {self.kv_usage_trigger}")
        need(0.0 <= self.kv_usage_release <= 1.0,
             f"kv_usage_release must be in [0, 1], got {self.kv_usage_release}")
        need(self.kv_usage_release <= self.kv_usage_trigger,
             "kv_usage_release should be <= kv_usage_trigger to avoid hysteresis inversion")
        need(self.pruning_mode in {"per_layer", "per_head", "per_layer_per_head"},
             "pruning_mode must be one of {'per_layer','per_head','per_layer_per_head'}, "
             f"got {self.pruning_mode!r}")
        need(self.pruning_mode != "per_layer" or self.allow_per_layer_mode,
             "pruning_mode='per_layer' is disabled by default in the runtime to prevent accidental use. "
             "Set allow_per_layer_mode=True (env TRIATTN_RUNTIME_ALLOW_PER_LAYER_MODE=1) for explicit opt-in.")
        need(self.sparse_score_aggregation in {"mean", "max"},
             f"sparse_score_aggregation must be 'mean' or 'max', got {self.sparse_score_aggregation!r}")
        need(self.per_head_selection_semantics in {"legacy_layer_local", "hf_aligned_global_per_head"},
             "per_head_selection_semantics must be one of "
             "{'legacy_layer_local','hf_aligned_global_per_head'}, "
             f"got {self.per_head_selection_semantics!r}")
        need(self.layer_perhead_aggregation in {"max", "mean"},
             f"layer_perhead_aggregation must be 'max' or 'mean', got {self.layer_perhead_aggregation!r}")
        need(self.per_layer_aggregation in {"max", "mean", "pure_mean"},
             "per_layer_aggregation must be one of {'max','mean','pure_mean'}, "
             f"got {self.per_layer_aggregation!r}")
        need(self.window_size >= 0, f"window_size must be >= 0, got {self.window_size}")
        need(self.disable_top_n_high_freq >= 0,
             f"disable_top_n_high_freq must be >= 0, got {self.disable_top_n_high_freq}")
        need(0.0 < self.effective_len_regression_ratio <= 1.0,
             f"effective_len_regression_ratio must be in (0, 1], got {self.effective_len_regression_ratio}")
        need(self.effective_len_guard_divide_multiples >= 1,
             f"effective_len_guard_divide_multiples must be >= 1, got {self.effective_len_guard_divide_multiples}")
        need(self.score_chunk_max_tokens >= 1,
             f"score_chunk_max_tokens must be >= 1, got {self.score_chunk_max_tokens}")
        need(not (self.enable_experimental_kv_compaction and self.require_physical_reclaim
                  and not self.enable_experimental_block_reclaim),
             "enable_experimental_kv_compaction requires enable_experimental_block_reclaim=True "
             "when require_physical_reclaim=True")


# Legacy TRIATTENTION_* names the plugin entry point maps onto the runtime prefix
# (triattention/vllm/plugin.py:29-58).
LEGACY_ENV_BRIDGE = {
    "TRIATTENTION_KV_BUDGET": "TRIATTN_RUNTIME_KV_BUDGET",
    "TRIATTENTION_DIVIDE_LENGTH": "TRIATTN_RUNTIME_DIVIDE_LENGTH",
    "TRIATTENTION_WINDOW_SIZE": "TRIATTN_RUNTIME_WINDOW_SIZE",
    "TRIATTENTION_LOG_DECISIONS": "TRIATTN_RUNTIME_LOG_DECISIONS",
    "TRIATTENTION_STATS_PATH": "TRIATTN_RUNTIME_SPARSE_STATS_PATH",
}
STRICT_DEFAULTS = (
    "TRIATTN_RUNTIME_ENABLE_EXPERIMENTAL_KV_COMPACTION",
    "TRIATTN_RUNTIME_ENABLE_EXPERIMENTAL_BLOCK_RECLAIM",
    "TRIATTN_RUNTIME_REQUIRE_TRITON_SCORING",
    "TRIATTN_RUNTIME_REQUIRE_PHYSICAL_RECLAIM",
)


def bridge_legacy_env(environ=None) -> None:
    """Legacy names fill runtime names that are unset or empty; the four strict switches
    default to "true"; TRIATTENTION_PRUNING_MODE maps with the per_layer_head alias."""
    env = os.environ if environ is None else environ
    for old, new in LEGACY_ENV_BRIDGE.items():
        if not env.get(new) and env.get(old):
            env[new] = env[old]
    for name in STRICT_DEFAULTS:
        env.setdefault(name, "true")
    if not env.get("TRIATTN_RUNTIME_PRUNING_MODE") and env.get("TRIATTENTION_PRUNING_MODE"):
        mode = env["TRIATTENTION_PRUNING_MODE"].strip().lower()
        env["TRIATTN_RUNTIME_PRUNING_MODE"] = "per_layer_per_head" if mode == "per_layer_head" else mode


def triattention_enabled(environ=None) -> bool:
    """ENABLE_TRIATTENTION (default on; unknown spellings keep the default), plugin.py:18-27,63-65."""
    env = os.environ if environ is None else environ
    raw = env.get("ENABLE_TRIATTENTION")
    if raw is None:
        return True
    token = raw.strip().lower()
    return False if token in _FALSE else True
