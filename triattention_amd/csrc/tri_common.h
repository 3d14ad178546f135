// Shared declarations of the gfx950 kernels behind include/triattention_hip.h.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "triattention_hip.h"

namespace tri {

constexpr int kWave = 64;
constexpr int kScoreThreads = 256;      // 4 waves per scorer workgroup
constexpr int kScoreTileTokens = 512;   // tokens of one (sequence, layer) per scorer workgroup
constexpr int kQPerPass = 4;            // query heads scored per wave pass
constexpr int kPairsPerLane = 8;        // frequency pairs held by one lane
constexpr int kMaxOffsets = 32;
constexpr int kFusedWaves = 8;          // waves of a resident-scorer workgroup
constexpr int kFusedThreads = kFusedWaves * kWave;

inline __host__ __device__ int64_t align_up(int64_t x, int64_t a) { return (x + a - 1) / a * a; }
inline __host__ __device__ int ceil_div(int a, int b) { return (a + b - 1) / b; }
inline __host__ __device__ int64_t ceil_div64(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Geometry of the resident (single-kernel) score + reduce path; eligible == 0 when the
// shape has no such kernel and the two-kernel path is used.
struct FusedPlan {
  int eligible;         // 0: none, 1: vector-unit kernel, 2: matrix-core kernel
  int tw;               // tokens per wave
  int HC;               // chunks of 8 KV heads; waves of a workgroup are split over them
  int tile_tokens;      // tokens per workgroup
  int tiles_per_seq;    // workgroups per sequence (by max_seq_len)
  int seqs_per_launch;  // whole sequences of maximum length per launch
  int resident;         // workgroups the device holds at once
  int bs_shift;
  int waves;            // matrix-core kernel: waves per workgroup (8, or 4 with two workgroups per CU)
  int launches;         // matrix-core kernel, several launches: how many (0: the worst case for the longest sequence)
  int layer_groups;     // matrix-core kernel, a batch too small to fill the chip with whole-model workgroups: the
                        // layers are cut into this many groups, one workgroup per (sequence, group, tile)
  int layers_per_group;
};
// Workgroups of the resident kernel the current device can hold at once (0: none).
int fused_resident_workgroups();
// The occupancy calculator's answer for the largest resident instance on the current device.
bool fused_mfma_fits_device();
// any_fill: plan the resident kernel even for a launch that would leave most CUs idle.
FusedPlan plan_fused(int B, int Hkv, int D, int G, int block_size, bool paged, int aggregation, int Tmax,
                     int resident, bool any_fill);
// L > 0 and split_layers: a single launch that would leave most of the chip idle is cut by layers too.
FusedPlan plan_fused_mfma(int B, int Hkv, int D, int G, int block_size, bool paged, int aggregation, int Tmax,
                          int resident, bool any_fill, int kv_dtype, const int32_t* host_lens = nullptr,
                          int L = 0, bool split_layers = false);

// Scratch carved out of the caller's workspace.  All offsets in bytes, 256-aligned.
struct Workspace {
  int64_t coef;      // [B][L][A][3][F] fp32: P, R, E for mean aggregation; A1, A2, E for max
  int64_t trig;      // [B][2][F] offset means of cos / sin, then [B][NO][2][F] tables (max aggregation)
  int64_t partial;   // [B][L][NT][A][2] fp32 per-tile sum / sum of squares
  int64_t mustd;     // [B][L][A][2] fp32 mean / safe std
  int64_t raw;       // [B][L][Tmax][A] fp32 raw scores (tri_compress_step)
  int64_t fin;       // [B*L*Hkv][Tmax] fp32 selection scores (worst case: per-layer selection)
  int64_t xchg;      // [B][L][tiles_per_seq][A][2] tagged sums exchanged by the resident kernel
  int64_t status;    // one word: non-zero when a bounded wait of the resident kernel expired
  int64_t pack;      // [2][B] int32: launch of every sequence and its first workgroup there (several launches)
  int64_t bmat;      // [B][L][Hkv][groups of 4 query heads][slabs][64][8] bf16 coefficient slabs (matrix-core kernel)
  int64_t total;
  int32_t num_tiles; // NT
  FusedPlan fused;
};

inline Workspace plan_workspace(int B, int L, int A, int F, int NO, int Hkv, int Tmax, const FusedPlan& fused) {
  Workspace w{};
  w.fused = fused;
  int64_t off = 0;
  auto take = [&](int64_t bytes) { int64_t o = off; off = align_up(off + bytes, 256); return o; };
  w.num_tiles = ceil_div(Tmax > 0 ? Tmax : 1, kScoreTileTokens);
  // The status word comes first, so its place does not depend on the batch: a caller that
  // reuses one workspace for steps of different shapes always reads the same word.
  w.status = take(256);
  w.coef = take((int64_t)B * L * A * 3 * F * 4);
  w.trig = take((int64_t)B * (NO + 1) * 2 * F * 4);
  w.partial = take((int64_t)B * L * w.num_tiles * A * 2 * 4);
  w.mustd = take((int64_t)B * L * A * 2 * 4);
  w.raw = take((int64_t)B * L * Tmax * A * 4);
  w.fin = take((int64_t)B * L * Hkv * Tmax * 4);
  w.xchg = take(fused.eligible ? (int64_t)B * L * fused.tiles_per_seq * A * 2 * 8 : 0);
  w.pack = take(fused.eligible ? (int64_t)B * 8 : 0);
  // key slabs (head_dim / 32) and magnitude slabs (half as many) per group of four query heads
  const int slabs = max(F / 16 + F / 32, 6);
  w.bmat = take(fused.eligible == 2 ? (int64_t)B * L * Hkv * (A / Hkv > 4 ? 2 : 1) * slabs * 64 * 16 : 0);
  w.total = off;
  return w;
}

// ---- launchers (defined in the .hip files; all validate nothing: tri_capi.hip does) ----

struct ScoreLaunch {
  // geometry
  int B, L, Hkv, D, block_size, kv_dtype, rope_style, A, G, NO, aggregation;
  int Tmax, num_tiles;
  int64_t stride_block, stride_token, stride_head;
  const void* const* k_layers;
  const float* const* k_scale_layers;
  const int32_t* block_table;
  int block_table_pitch;
  const int32_t* seq_lens;
  const float* coef;     // workspace
  const float* trig;     // workspace
  float* partial;        // workspace
  float* raw;
  int64_t raw_stride_layer, raw_stride_token, raw_stride_head;
};

hipError_t launch_fold_stats(const float* qr, const float* qi, const float* qabs, const float* fs,
                             int L, int A, int F, int disable_mlr, int disable_trig, float* folded,
                             hipStream_t s);
hipError_t launch_prepare(const float* folded, const float* omega, const float* offsets, int NO,
                          const int32_t* round_start, int B, int L, int A, int F, int aggregation,
                          float* coef, float* trig, hipStream_t s);
hipError_t launch_score(const ScoreLaunch& a, hipStream_t s);

struct SelectLaunch {
  int B, L, Hkv, A, G, Tmax, num_tiles, max_budget;
  int normalize, window_size, protect_prefill, group_reduce, layer_reduce, shared, group_first;
  const int32_t* seq_lens;
  const int32_t* prefill_lens;
  const int32_t* budgets;
  const float* partial;
  float* mustd;
  const float* raw;
  int64_t raw_stride_layer, raw_stride_token, raw_stride_head;
  float* fin;          // [rows][Tmax]
  int32_t* keep;       // [rows][max_budget]
  // Scratch for the chunk sums of the reduce-first statistics (group_first): any part of the workspace
  // that no later launch of the call reads (the scorer's coefficient tables: every score call rebuilds them).
  double* group_scratch;
  int64_t group_scratch_bytes;
};
hipError_t launch_select(const SelectLaunch& a, hipStream_t s);
hipError_t launch_clear_status(uint32_t* status, hipStream_t s);
// groups > 1: row r is the sum (group_max: maximum) of `groups` partial rows group_stride floats apart,
// added while loading (rows of at most topk_register_row_limit() elements).
hipError_t launch_topk_rows(const float* scores, int64_t row_pitch, int num_rows,
                            const int32_t* row_lens, const int32_t* row_ks, int rows_per_entry, int max_len,
                            int32_t* keep, int keep_pitch, hipStream_t s, int groups = 1, int64_t group_stride = 0,
                            int group_max = 0);
int topk_register_row_limit();

struct FusedLaunch {
  int B, L, Hkv, D, block_size, kv_dtype, rope_style, A, G, Tmax;
  int normalize, window_size, protect_prefill, group_reduce, layer_reduce;
  int64_t stride_block, stride_token, stride_head;
  const void* const* k_layers;
  const float* const* k_scale_layers;
  const int32_t* block_table;
  int block_table_pitch;
  const int32_t* seq_lens;
  const int32_t* prefill_lens;
  const float* coef;             // workspace (vector-unit kernel: written by launch_prepare)
  // matrix-core kernel: it prepares its own coefficients from these
  const float* folded; const float* omega; const float* offsets; int NO; const int32_t* round_start;
  unsigned long long* xchg;      // workspace
  uint32_t* status;              // workspace
  int32_t* pack;                 // workspace
  void* bmat;                    // workspace (matrix-core kernel)
  float* fin;                    // [B*Hkv][Tmax]
  float* fin_part;               // workspace: [layer groups][B*Hkv][Tmax] (layer-split launches of the matrix-core kernel)
  int skip_layer_reduce;         // 1: leave the groups' partial rows in fin_part (the top-k adds them while loading)
  FusedPlan plan;
};
// Process-wide settings (tri_set_tuning); defined in tri_capi.hip.
int64_t tuning(int key);
// Limit of the resident kernels' waits on other workgroups, in ticks of the 100 MHz wall
// clock, from TRI_TUNE_RESIDENT_WAIT_US (default 2 s; a negative value makes every wait give
// up at once, which raises the status word while every workgroup still runs to its end).
long long resident_spin_ticks();
hipError_t launch_fused_select(const FusedLaunch& a, hipStream_t s);
hipError_t launch_fused_mfma(const FusedLaunch& a, hipStream_t s);

struct CompactLaunch {
  int B, L, Hkv, D, block_size, elem_bytes, max_budget;
  int keep_per_layer, shared, has_scales;
  int64_t stride_block, stride_token, stride_head;   // elements
  const void* const* k_layers;
  const void* const* v_layers;
  const float* const* k_scale_layers;
  const float* const* v_scale_layers;
  const int32_t* block_table;
  int block_table_pitch;
  const int32_t* seq_lens;
  const int32_t* budgets;
  const int32_t* keep;
  int Tmax;
  void* staging;       // full-permutation mode only
  const uint32_t* guard;   // optional: a device word; the kernels move nothing when it is non-zero
  int no_side_stream;      // 1: fp8 scales follow the rows on the caller's stream (nothing is created)
};
hipError_t launch_compact(const CompactLaunch& a, hipStream_t s);

// Calibration statistics of one layer's captured queries (tri_calib.hip).
struct QStatsLaunch {
  const void* q_rot;      // [H][T][D] through (stride_head, stride_token), 16-bit elements
  const void* cos;        // [T][D]
  const void* sin;        // [T][D]
  int64_t stride_head, stride_token;
  int H, T, D, dtype, rope_style;
  float scale;
  float* out_real;        // [H][D/2]
  float* out_imag;
  float* out_abs;
  void* workspace;
};
int64_t qstats_workspace_bytes(int H, int T, int D);
hipError_t launch_qstats(const QStatsLaunch& q, hipStream_t s);
hipError_t launch_compact_full(const CompactLaunch& a, hipStream_t s);

}  // namespace tri
