/*
 * triattention_hip.h -- C ABI of the MI355X (gfx950) KV scoring / selection /
 * compaction library (libtriattention_hip.so).
 *
 * Every entry point is stream ordered: it enqueues kernels on `stream`
 * (a hipStream_t passed as void*, NULL = the null stream), never synchronises the
 * device and never allocates device memory.  (Once per device and process the library
 * creates an event to chain its resident launches and, for fp8 caches with per-row scales,
 * a side stream with two events on which the scales move next to the rows; neither is
 * used while `stream` is under graph capture.)  All pointers are DEVICE pointers unless a comment
 * says "host".  Return value: TRI_OK or a negative tri_status; a message for the
 * last failure on the calling thread is available from tri_last_error().
 * Nothing is thrown and no torch type crosses this boundary.
 *
 * Reference citations are paths inside the TriAttention checkout
 * (triattention/vllm/...).
 */
#ifndef TRIATTENTION_HIP_H
#define TRIATTENTION_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TRI_ABI_VERSION 6

typedef enum tri_status {
  TRI_OK = 0,
  TRI_ERR_INVALID_ARGUMENT = -1, /* shape / flag / null-pointer check failed on the host */
  TRI_ERR_UNSUPPORTED = -2,      /* valid request this build has no kernel for */
  TRI_ERR_WORKSPACE = -3,        /* workspace too small */
  TRI_ERR_LAUNCH = -4            /* hipLaunchKernel reported an error */
} tri_status;

typedef enum tri_kv_dtype { TRI_KV_BF16 = 0, TRI_KV_FP16 = 1, TRI_KV_FP8_E4M3 = 2 } tri_kv_dtype;
typedef enum tri_rope_style { TRI_ROPE_HALF = 0, TRI_ROPE_INTERLEAVED = 1 } tri_rope_style;
typedef enum tri_reduce { TRI_REDUCE_MEAN = 0, TRI_REDUCE_MAX = 1 } tri_reduce;

/* Paged (or dense) key/value storage of every layer of one KV-cache group.
 * Element (layer l, physical block p, in-block token o, head h, dim d) of K lives at
 *   k_layers[l] + p*stride_block + o*stride_token + h*stride_head + d   (in elements)
 * which covers both vLLM layouts, [2, nb, bs, H, D] and [nb, 2, bs, H, D]
 * (runtime/kv_compaction.py:38-53,94-117), by passing separate K and V bases.
 * A dense [B, H, T, D] tensor (core/scoring.py:93) is the same thing with
 * block_size = T, one block per sequence and an identity block table; a token-level
 * pool [total_slots, H, D] with a (request, position) -> slot table
 * (sglang/kv_compaction.py:56-137) is the same thing with block_size = 1. */
typedef struct tri_kv_layout {
  int32_t num_layers;
  int32_t num_kv_heads;
  int32_t head_dim;           /* 64, 128 or 256 */
  int32_t block_size;         /* tokens per block */
  int32_t kv_dtype;           /* tri_kv_dtype */
  int32_t rope_style;         /* tri_rope_style */
  int64_t stride_block;
  int64_t stride_token;
  int64_t stride_head;
  const void* const* k_layers; /* device array [num_layers] of device pointers */
  const void* const* v_layers; /* device array [num_layers]; may be NULL for score-only calls */
  /* fp8 only: per-(token, head) fp32 dequantisation scales, element
   * (l, p, o, h) at k_scale_layers[l] + (p*block_size + o)*num_kv_heads + h.
   * v_scale_layers == NULL: the rows carry no scales of their own (a cache with one scale
   * per tensor, as vLLM's fp8 KV cache); compaction then moves rows only, and
   * k_scale_layers must still point to readable scales for the scorer (all ones; the
   * entries of every layer may point to the same array). */
  const float* const* k_scale_layers;
  const float* const* v_scale_layers;
} tri_kv_layout;

/* The sequences of one compression step (the reference handles one request per
 * call, runtime/runner_compression_actions.py:24; a batch is a loop of those). */
typedef struct tri_batch {
  int32_t num_seqs;
  int32_t max_seq_len;          /* host copy of max(seq_lens): sizes grids and scratch rows */
  int32_t max_budget;           /* host copy of max(budgets) */
  int32_t block_table_pitch;    /* int32 elements between rows of block_table */
  const int32_t* block_table;   /* [num_seqs][pitch] physical block ids (runtime/kv_compaction.py:139-157) */
  const int32_t* seq_lens;      /* [num_seqs] cached tokens T (group_total_tokens, runtime/hook_group_pipeline.py:72-73) */
  const int32_t* round_start;   /* [num_seqs] num_computed_tokens (runtime/hook_group_pipeline.py:78) */
  const int32_t* prefill_lens;  /* [num_seqs] or NULL (=0) */
  const int32_t* budgets;       /* [num_seqs] k = min(budget_total, T) (runtime/selector_hf.py:823) */
  const int32_t* seq_lens_host; /* HOST copy of seq_lens, or NULL.  With it a batch that needs several resident
                                 * launches gets the tile size that fills them best and exactly as many
                                 * launches as it needs (without: the worst case for max_seq_len). */
} tri_batch;

/* Scoring statistics, already resolved per runtime layer (layer index modulo the
 * available stats layers, runtime/selector_hf.py:132-143) and folded by
 * tri_fold_stats. */
typedef struct tri_score_params {
  int32_t num_score_heads;      /* heads scored per layer: Hq when stats are per query head, else Hkv */
  int32_t num_offsets;          /* <= 32 */
  int32_t aggregation;          /* tri_reduce over offsets (core/scoring.py:336-341) */
  const float* folded;          /* [L][num_score_heads][3][F] from tri_fold_stats */
  const float* omega;           /* [F] rotary inv_freq (core/compressor.py:192-194) */
  const float* offsets;         /* [num_offsets] (core/compressor.py:222-242) */
} tri_score_params;

/* Selection semantics (runtime/selector_hf.py:813-1033 and :473-677). */
typedef struct tri_select_params {
  int32_t normalize;            /* 0: raw scores; 1: sparse_normalize_scores (streaming unbiased std, std < 1e-8 -> 1,
                                   runtime/selector_hf.py:902-909); 2: the research path's z-score (population std
                                   clamped at 1e-6, methods/triattention.py:255-258) */
  int32_t window_size;          /* recent tokens forced to +inf (runtime/selector_hf.py:121-130) */
  int32_t protect_prefill;      /* tokens < prefill_len forced to +inf */
  int32_t group_reduce;         /* tri_reduce over the query heads of a KV head (runtime/selector_hf.py:277-297) */
  int32_t layer_reduce;         /* tri_reduce over layers; -1 = none (one keep set per layer) */
  int32_t shared;               /* 1: max over KV heads, one index list per (seq[, layer]) (runtime/selector_hf.py:636-637) */
  int32_t group_first;          /* 0: normalise every score head, then reduce over the query heads of a KV head (vLLM
                                   runtime, runtime/selector_hf.py:916-989).  1: reduce first, then normalise per
                                   (layer, KV head) with torch mean / unbiased std (SGLang backend,
                                   sglang/scheduler_hooks.py:655-690, core/utils.py:466-480) */
  int32_t no_resident;          /* 1: never take a resident kernel for this call, whatever the shape and the
                                   TRI_TUNE_RESIDENT_KERNEL setting say (a caller repeating a step whose resident
                                   launch raised the status word).  No counterpart in the reference. */
} tri_select_params;

int tri_abi_version(void);
const char* tri_last_error(void);
/* SHA-256 (hex) of the sources and compiler flags this library was built from ("unknown" for a
 * build outside the package's build script); the build script compares it with the sources next to
 * the library and rebuilds a library that does not belong to them.  No counterpart in the reference. */
const char* tri_source_digest(void);

/* Process-wide settings of the library (no counterpart in the reference, whose Triton kernels have
 * none of these choices).  The library itself reads no environment variable for them; the Python
 * layer applies TRIATTN_RESIDENT_KERNEL / _WORKGROUPS / _LAYER_SPLIT / _SPIN_TICKS and
 * TRIATTN_MAX_KERNEL once, when it loads the library.  tri_set_tuning returns TRI_OK or
 * TRI_ERR_INVALID_ARGUMENT; tri_get_tuning returns the value in force (INT64_MIN for an unknown key).
 * Settings are read when a call plans its launches; changing one while another thread is inside a
 * call affects that call or the next. */
typedef enum tri_tuning {
  TRI_TUNE_RESIDENT_KERNEL = 0,     /* 0 (default): the library chooses by shape and batch; 1: the matrix-core
                                       resident kernel whenever the shape has one, however small the launch;
                                       2: the vector-unit resident kernel; 3: never a resident kernel */
  TRI_TUNE_RESIDENT_WORKGROUPS = 1, /* 0 (default): the device's own capacity; n > 0: plan as if the device held
                                       n resident workgroups (never more than it does): small inputs then need
                                       several launches (tests) */
  TRI_TUNE_LAYER_SPLIT = 2,         /* -1 (default): single-launch batches are cut by layers where that shortens the
                                       longest workgroup, unless the kernel was forced
                                       with TRI_TUNE_RESIDENT_KERNEL = 1; 0: never; 1: always allowed */
  TRI_TUNE_MAX_KERNEL = 3,          /* 0 (default): max aggregation on the matrix cores where a kernel exists;
                                       1: always the vector-unit kernel (comparison runs) */
  TRI_TUNE_RESIDENT_WAIT_US = 4     /* how long a resident workgroup waits for the other workgroups of its launch
                                       before it raises status word 1, in microseconds: default 2,000,000; a serving
                                       engine that shares the GPU may lower it (a starved launch costs this much
                                       once, after which the selector stays on the other kernels); negative: every
                                       wait gives up at once (exercises the failure path from the host) */
} tri_tuning;
int tri_set_tuning(int32_t key, int64_t value);
int64_t tri_get_tuning(int32_t key);

/* Resident launches of one process are chained on the device with an event (two of them running at
 * the same time would each hold part of the CUs and wait for the other's workgroups).  The library
 * does that itself for every launch it issues outside graph capture.  A launch sequence captured
 * into a HIP graph contains no such wait or record (event nodes of a replay would refer to the
 * capture-time record), so a caller that replays a captured tri_compress_step / tri_select_paged
 * whose path is a resident kernel brackets the replay with these two calls on the stream it
 * replays on: enter makes `stream` wait (on the device) for the previous resident launch of the
 * process, leave records the replay as the latest one.  No counterpart in the reference. */
int tri_resident_gate_enter(void* stream);
int tri_resident_gate_leave(void* stream);

/* Replaces the per-call stat preparation of core/scoring.py:259-271,346-351:
 * folded[l][a][0][f] = s*q_r, [1] = s*q_i, [2] = s*(q_abs - sqrt(q_r^2+q_i^2+1e-8))
 * (s*q_abs when disable_mlr; [0]=[1]=0 when disable_trig).  Inputs [L][A][F] fp32. */
int tri_fold_stats(const float* q_mean_real, const float* q_mean_imag, const float* q_abs_mean,
                   const float* freq_scale_sq, int32_t num_layers, int32_t num_score_heads,
                   int32_t num_pairs, int32_t disable_mlr, int32_t disable_trig, float* folded,
                   void* stream);

/* Bytes of device scratch the calls below need for (layout, batch, score params);
 * 0 on invalid input.  Host-only, launches nothing. */
uint64_t tri_workspace_bytes(const tri_kv_layout* kv, const tri_batch* batch,
                             const tri_score_params* sp);

/* Byte offset inside the workspace of a 32-bit status word (the same for every layout, batch and
 * score parameters of one library build, so one workspace reused for steps of different shapes
 * keeps its word in one place): tri_select_paged and
 * tri_compress_step clear it and the resident kernel sets it to non-zero if one of its
 * bounded waits on another workgroup expired (1), or if a magnitude coefficient (with fp16
 * keys: any coefficient) or a key's magnitude does not fit the fp16 pieces the matrix-core
 * kernel holds it in, i.e. exceeds 65504, or if the keys of a layer are so small throughout
 * (no magnitude of 2^-9 among those looked at) that the pieces would be subnormals (2)
 * (results are then invalid; the compaction
 * inside tri_compress_step sees the word and moves nothing, so the cache is intact and
 * the caller can repeat the step with tri_select_params.no_resident = 1).  The caller may read
 * it after synchronising the stream.  Host-only; no counterpart in the reference. */
uint64_t tri_workspace_status_offset(const tri_kv_layout* kv, const tri_batch* batch,
                                     const tri_score_params* sp);

/* Raw scores of every cached key of every sequence and layer, straight from the
 * paged blocks; replaces gather_request_k_dense_range + repeat_interleave +
 * compute_scores_triton per (layer, chunk) (runtime/selector_hf.py:860-894,
 * runtime/kv_compaction.py:322-352, core/scoring.py:79-204; math of
 * core/scoring.py:207-362).  raw[(b*L + l)*raw_stride_layer + n*raw_stride_token
 * + a*raw_stride_head], fp32.  Also leaves per-(seq, layer, head) sum / sum of
 * squares partials in the workspace for tri_select. */
int tri_score_paged(const tri_kv_layout* kv, const tri_batch* batch, const tri_score_params* sp,
                    float* raw, int64_t raw_stride_layer, int64_t raw_stride_token,
                    int64_t raw_stride_head, void* workspace, uint64_t workspace_bytes,
                    void* stream);

/* z-normalise, guard, reduce over the GQA group and over layers, then keep the
 * top budget per row, ascending; replaces runtime/selector_hf.py:896-1025 (group
 * mode) and :538-677 (per-layer modes).  `raw` and the workspace come from
 * tri_score_paged on the same stream.  final_scores (may be NULL) receives the
 * selection scores [rows][max_seq_len]; keep receives int32
 * [rows][max_budget], rows = B * (layer_reduce<0 ? L : 1) * (shared ? 1 : Hkv).
 * Ties at the threshold keep the lowest token index. */
int tri_select(const tri_kv_layout* kv, const tri_batch* batch, const tri_score_params* sp,
               const tri_select_params* sel, const float* raw, int64_t raw_stride_layer,
               int64_t raw_stride_token, int64_t raw_stride_head, float* final_scores,
               int32_t* keep, void* workspace, uint64_t workspace_bytes, void* stream);

/* tri_score_paged + tri_select in one call, without the raw scores ever being handed to
 * the caller: the device side of _select_keep_indices_for_group_per_head's paged branch
 * (runtime/selector_hf.py:813-1033) and of the per-layer selector (:473-677).  When the
 * shape allows (head_dim 128, or 64 / 256 with two-byte keys; at most eight query heads
 * per KV head; mean aggregation over offsets; power-of-two block size; layer_reduce >= 0,
 * or a single layer, where a keep set per layer is the same thing; not shared; workgroups
 * that run one layer each, or a batch that fills most of the GPU; sequences that fit its
 * LDS in tiles) one resident kernel keeps each layer's raw scores in LDS
 * and they never reach memory; otherwise the two calls above run back to back on the
 * workspace.  Outputs as tri_select; keep may be NULL when only final_scores is wanted
 * (tri_topk_rows then turns them into keep rows). */
int tri_select_paged(const tri_kv_layout* kv, const tri_batch* batch, const tri_score_params* sp,
                     const tri_select_params* sel, float* final_scores, int32_t* keep, void* workspace,
                     uint64_t workspace_bytes, void* stream);

/* Which path tri_select_paged / tri_compress_step take for these arguments on the
 * current device: 2 = resident kernel scoring on the matrix cores (bf16, fp16 and fp8 keys), 1 = resident
 * kernel scoring on the vector unit, 0 = score then select, -1 = invalid arguments.
 * Host-only.  No counterpart in the reference (it has a single path). */
int tri_select_path(const tri_kv_layout* kv, const tri_batch* batch, const tri_score_params* sp,
                    const tri_select_params* sel);

/* How tri_select_paged / tri_compress_step would cut these arguments into workgroups: the path
 * as tri_select_path reports it and, for the resident kernels, the tile length, the tiles of the
 * longest sequence, the groups the layers are cut into (1: every workgroup runs the whole model)
 * and the number of launches (0: as many as the device-side packing of the ragged lengths needs,
 * at most ceil(num_seqs / sequences per launch)).  assume_resident_workgroups > 0 answers for a
 * device that holds that many resident workgroups at once (a dry run that touches no device:
 * capacity planning, tests of the planner on a host without a GPU; 256 is an MI355X with 8-wave
 * workgroups); 0 answers for the current device.  Host-only.  No counterpart in the reference. */
typedef struct tri_plan_info {
  int32_t path;                 /* 0 two-pass, 1 resident on the vector unit, 2 resident on the matrix cores */
  int32_t tile_tokens;          /* tokens a workgroup scores per layer (0 on the two-pass path) */
  int32_t tiles_per_seq;        /* by max_seq_len */
  int32_t layer_groups;
  int32_t layers_per_group;
  int32_t launches;
  int32_t waves_per_workgroup;
  int32_t resident_workgroups;  /* capacity the plan was made for, in workgroups of eight waves (two of four waves take the place of one) */
  int64_t workspace_bytes;      /* what tri_workspace_bytes returns for that plan */
} tri_plan_info;
int tri_describe_plan(const tri_kv_layout* kv, const tri_batch* batch, const tri_score_params* sp,
                      const tri_select_params* sel, int32_t assume_resident_workgroups, tri_plan_info* out);

/* Top-k of arbitrary fp32 rows (core/compressor.py:388-409): keep[r][0..k_r) =
 * ascending indices of the k_r largest of scores[r][0..len_r). */
int tri_topk_rows(const float* scores, int64_t row_pitch, int32_t num_rows, const int32_t* row_lens,
                  const int32_t* row_ks, int32_t rows_per_entry, int32_t max_len, int32_t* keep,
                  int32_t keep_pitch, void* stream);

/* In-place, order-preserving compaction of K and V of every layer: slot j of
 * (seq b, head h) receives the row of token keep[...][j], for j < budget_b;
 * replaces compact_request_kv_in_place(_per_head) per layer
 * (runtime/kv_compaction.py:355-599, runtime/layout_engine.py:112-138) for the
 * slots that survive truncate_tail_reclaim_group (runtime/layout_engine.py:209-227).
 * keep rows must be strictly ascending.  keep_per_layer: keep is
 * [B][L][rows][max_budget] instead of [B][rows][max_budget]; shared: rows = 1. */
int tri_compact_paged(const tri_kv_layout* kv, const tri_batch* batch, const int32_t* keep,
                      int32_t keep_per_layer, int32_t shared, void* stream);

/* The reference's full permutation [kept..., dropped...] over all T slots
 * (runtime/kv_compaction.py:512-546), through a caller-provided staging buffer of
 * tri_compact_full_staging_bytes(). */
uint64_t tri_compact_full_staging_bytes(const tri_kv_layout* kv, const tri_batch* batch);
int tri_compact_paged_full(const tri_kv_layout* kv, const tri_batch* batch, const int32_t* keep,
                           int32_t keep_per_layer, int32_t shared, void* staging,
                           uint64_t staging_bytes, void* stream);

/* score + select + compact for every layer of every sequence in one call: the
 * device side of run_group_compaction_pipeline (runtime/hook_group_pipeline.py:42-155)
 * in the default per_head / hf_aligned_global_per_head mode. */
int tri_compress_step(const tri_kv_layout* kv, const tri_batch* batch, const tri_score_params* sp,
                      const tri_select_params* sel, int32_t* keep, void* workspace,
                      uint64_t workspace_bytes, void* stream);

/* tri_compress_step for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): no counterpart in the
 * reference.  The scratch the kernels need (coefficients, trig tables, per-tile sums, raw
 * scores, selection scores, status word) lives in a device array inside the library,
 * TRI_STATIC_WORKSPACE_BYTES per GPU from the moment the library is loaded until the process
 * ends; the call allocates nothing, frees nothing, creates no stream or event, and always takes
 * the score-then-select kernels (never a resident kernel; for fp8 caches the scales follow the
 * rows on `stream`).  A step whose scratch for those kernels exceeds the array is rejected
 * with TRI_ERR_WORKSPACE (tri_workspace_bytes is an upper bound of it: on a device with resident
 * kernels it also covers their regions, which this call does not use): Qwen3-8B shapes (36 layers)
 * fit up to 4 sequences of budget + 128 = 2176 tokens, or one sequence of 11400.  Every call on a GPU uses that GPU's one array, which keeps the
 * previous call's contents (nothing in it needs to start at zero except the status word, which
 * the call clears): calls that overlap in time on one GPU, from any streams or threads, race.
 * Results are those of tri_compress_step with no_resident = 1.  status_out (may be NULL)
 * receives the device address of the status word for callers that want to read it.
 * The first call on a device also looks up the array's address (hipGetSymbolAddress) and asks the
 * occupancy calculator once; a caller that records the call into a graph makes one call on that
 * device outside capture first. */
#define TRI_STATIC_WORKSPACE_BYTES (64u << 20)
int tri_compress_step_static(const tri_kv_layout* kv, const tri_batch* batch, const tri_score_params* sp,
                             const tri_select_params* sel, int32_t* keep, const uint32_t** status_out,
                             void* stream);

/* Calibration: per-query-head frequency statistics of one layer's captured query states;
 * replaces the RoPE inversion and the per-head means of scripts/calibrate.py:196-224
 * (helpers :38-98; same arithmetic as triattention/methods/pruning_utils.py:40-98).
 * q_rot[h*stride_head + t*stride_token + d] are the queries after RoPE times the attention
 * scale, cos / sin are [num_tokens][head_dim] rotary tables, all in `dtype` (TRI_KV_BF16 or
 * TRI_KV_FP16); every elementwise step of the inversion rounds to that dtype, as the
 * reference's tensors do.  out_real / out_imag / out_abs: fp32 [num_heads][head_dim/2], the
 * mean over tokens of the un-rotated query per frequency pair (real, imaginary) and of its
 * modulus: the "q_mean_real" / "q_mean_imag" / "q_abs_mean" entries of the stats file.
 * workspace: tri_qstats_workspace_bytes() bytes of device memory, 16-byte aligned. */
uint64_t tri_qstats_workspace_bytes(int32_t num_heads, int32_t num_tokens, int32_t head_dim);
int tri_qstats(const void* q_rot, int64_t stride_head, int64_t stride_token, const void* cos,
               const void* sin, int32_t num_heads, int32_t num_tokens, int32_t head_dim,
               int32_t dtype, int32_t rope_style, float scale, float* out_real, float* out_imag,
               float* out_abs, void* workspace, uint64_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TRIATTENTION_HIP_H */
