#!/usr/bin/env python3
"""Write tests/golden/host_logic.json: what the REFERENCE's host-side functions return for the
scenarios of host_scenarios.py (effective lengths, budgets, deferral, regression guard, the hook's
result dictionary and block-list truncation, planner + effective-length tracker over decode loops,
worker block-table shrink, runner actions with the request state store, effective-length overrides).

Runs ONLY in the build container, where the reference checkout is mounted read-only.  It imports the
reference's pure-Python runtime modules (torch / numpy / stdlib only; nothing of them needs vLLM or a
GPU):

* ``triattention.vllm.runtime.hook_runtime_context.build_hook_runtime_context``
* ``triattention.vllm.runtime.hook_impl.make_runner_compression_hook`` (its module-level selector
  builder and compaction functions are rebound to the scenario's stand-ins, the way the reference's
  own unit tests rebind them)
* ``triattention.vllm.runtime.planner.CompressionPlanner``, ``effective_len_tracker.EffectiveCacheLenTracker``,
  ``state.RequestStateStore``, ``executor.RunnerHookCompressionExecutor``
* ``triattention.vllm.runtime.worker_reclaim_sync.apply_worker_block_reclaim_events``
* ``triattention.vllm.runtime.runner_compression_actions.execute_runner_compression_actions``
* ``triattention.vllm.runtime.effective_overrides.build_effective_sparse_overrides``

The fixture is data (inputs are rebuilt by host_scenarios.py, outputs are stored); the reference does
not travel.

Usage:  python tests/golden/make_hook_golden.py [/root/reference]
"""
from __future__ import annotations

import json
import logging
import sys
import types
from pathlib import Path

HERE = Path(__file__).resolve().parent
REF = Path(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")


def reference_api():
    sys.path.insert(0, str(REF))
    from triattention.vllm.runtime import hook_impl
    from triattention.vllm.runtime.config import TriAttentionRuntimeConfig
    from triattention.vllm.runtime.effective_len_tracker import EffectiveCacheLenTracker
    from triattention.vllm.runtime.effective_overrides import build_effective_sparse_overrides
    from triattention.vllm.runtime.executor import RunnerHookCompressionExecutor
    from triattention.vllm.runtime.hook_runtime_context import build_hook_runtime_context
    from triattention.vllm.runtime.planner import CompressionPlanner
    from triattention.vllm.runtime.runner_compression_actions import execute_runner_compression_actions
    from triattention.vllm.runtime.signals import CompressionSignal
    from triattention.vllm.runtime.state import RequestStateStore
    from triattention.vllm.runtime.worker_reclaim_sync import apply_worker_block_reclaim_events

    quiet = logging.getLogger("host_logic_golden")
    quiet.addHandler(logging.NullHandler())
    quiet.propagate = False

    def make_hook(runner, config, select_layer, select_group, compact_shared, compact_per_head, gather):
        hook_impl._build_triattention_selector = lambda cfg, base_runner=None: (select_layer, select_group, "enabled")
        hook_impl.compact_request_kv_in_place = compact_shared
        hook_impl.compact_request_kv_in_place_per_head = compact_per_head
        hook_impl.gather_request_k_dense = gather
        return hook_impl.make_runner_compression_hook(base_runner=runner, config=config)

    return types.SimpleNamespace(
        Config=TriAttentionRuntimeConfig, Signal=CompressionSignal, Planner=CompressionPlanner,
        Tracker=EffectiveCacheLenTracker, StateStore=RequestStateStore, Executor=RunnerHookCompressionExecutor,
        runtime_context=build_hook_runtime_context, make_hook=make_hook,
        worker_reclaim=lambda runner, events: apply_worker_block_reclaim_events(base_runner=runner, events=events),
        sparse_overrides=lambda runner, store, sched, events: build_effective_sparse_overrides(
            base_runner=runner, state_store=store, scheduler_output=sched, compression_events=events),
        runner_actions=lambda executor, store, sched, signals, strict, allowed: execute_runner_compression_actions(
            executor=executor, state_store=store, scheduler_output=sched, signals=signals, strict_no_downgrade=strict,
            allowed_strict_skip_reasons=set(allowed), logger=quiet, log_decisions=False),
    )


def main() -> int:
    logging.disable(logging.CRITICAL)
    sys.path.insert(0, str(HERE))
    import host_scenarios
    out = host_scenarios.run_all(reference_api())
    text = json.dumps(out, indent=None, separators=(",", ":"), sort_keys=True)
    (HERE / "host_logic.json").write_text(text + "\n")
    print(f"wrote {HERE / 'host_logic.json'}: {len(text)} bytes, "
          f"{len(out['runtime_context'])} runtime-context cases, {len(out['hook'])} hook scenarios")
    return 0


if __name__ == "__main__":
    sys.exit(main())
