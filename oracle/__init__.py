"""CPU restatement of the reference's KV scoring / selection / compaction math.

THIS PACKAGE IS TEST INFRASTRUCTURE.  It is the checker the HIP path is compared
against, never the thing that ships or is measured: only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import it.  Nothing under ``triattention_amd/`` imports it, and the product path
raises when the HIP library is missing instead of falling back to this code.

Everything here is plain ``torch`` on CPU tensors (the reference is Python /
PyTorch, so the restatement uses the same tensor ops in the same order), each
function citing the reference file:line it follows.  Paths are relative to the
reference checkout root.

How each function is pinned (see tests/test_oracle_*.py):

===========================  ==================================================
function                     pinned by
===========================  ==================================================
scoring.raw_scores           golden vectors written by the reference's own
                             ``compute_scores_pytorch`` (tests/golden), fp64
                             brute-force loops, closed forms (single frequency,
                             omega=0, zero Q centre), rotation invariance, and
                             equality with the un-rotated HF formulation
scoring.raw_scores_unrotated closed forms + equality with raw_scores
rope.*                       closed form theta^(-2i/D); llama3 piecewise formula
                             checked at the three regimes and against the
                             golden 64-float vector
selection.znorm_*            torch.mean / torch.std (unbiased) on the same data
selection.group_keep_*       golden vectors from the reference selector's paged
                             group branch; brute-force python loops on tiny
                             inputs; guard invariants
selection.topk_ascending     full sort on tiny inputs
compaction.*                 golden vectors from the reference's
                             ``compact_request_kv_in_place(_per_head)``;
                             brute-force row loops; multiset preservation
===========================  ==================================================

fp8 (e4m3 + per-token-head scale) keys have no counterpart in the reference;
``scoring.dequant_fp8`` is pinned by closed form only: **parity unpinned** beyond
"dequantise, then score as fp32".
"""
