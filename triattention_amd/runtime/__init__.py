"""Runtime plug-in surface: settings, signals, selector, paged-KV compaction and the
runner hook (the reference's triattention/vllm/runtime package, hot-path part)."""
from .config import TriAttentionRuntimeConfig, bridge_legacy_env, triattention_enabled
from .hook import (CompressionExecutionResult, CompressionExecutor, RunnerHookCompressionExecutor,
                   install_runner_compression_hook, make_runner_compression_hook)
from .kv_compaction import (build_keep_token_indices, compact_request_kv_in_place,
                            compact_request_kv_in_place_per_head, gather_request_k_dense,
                            gather_request_k_dense_range, gather_request_kv_dense,
                            register_kv_layout_axis_hint)
from .models import (TRITON_SCORING_REQUIRED_MARKER, CompressionPlanner, CompressionSignal, KeepPlan,
                     PlacementPlan, ReclaimEvent, ReclaimGroup, RequestCompressionState, RequestStateStore)
from .selector import build_triattention_selector
from .engine_glue import (EffectiveCacheLenTracker, SchedulerCompressionGlue, apply_worker_block_reclaim_events,
                          build_effective_sparse_overrides, consume_runner_signals,
                          execute_runner_compression_actions)

# Public alias, as in the reference's runtime package.
TriAttentionConfig = TriAttentionRuntimeConfig

__all__ = [
    "TriAttentionRuntimeConfig", "TriAttentionConfig", "bridge_legacy_env", "triattention_enabled",
    "CompressionExecutionResult", "CompressionExecutor", "RunnerHookCompressionExecutor",
    "install_runner_compression_hook", "make_runner_compression_hook", "build_keep_token_indices",
    "compact_request_kv_in_place", "compact_request_kv_in_place_per_head", "gather_request_k_dense",
    "gather_request_k_dense_range", "gather_request_kv_dense", "register_kv_layout_axis_hint",
    "TRITON_SCORING_REQUIRED_MARKER", "CompressionPlanner", "CompressionSignal", "KeepPlan", "PlacementPlan",
    "ReclaimEvent", "ReclaimGroup", "RequestCompressionState", "RequestStateStore",
    "build_triattention_selector", "EffectiveCacheLenTracker", "SchedulerCompressionGlue",
    "apply_worker_block_reclaim_events", "build_effective_sparse_overrides", "consume_runner_signals",
    "execute_runner_compression_actions",
]
