// extern "C" boundary of libtriattention_hip.so: argument validation on the host,
// then kernel launches on the caller's stream.  Nothing here allocates or waits.
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <atomic>
#include <climits>
#include <mutex>

#include "tri_common.h"

// Scratch of tri_compress_step_static: one copy per GPU, loaded with the code object.  In host
// code this name is only a handle for hipGetSymbolAddress; the address kernels are given is
// the one that call returns on the device in question.
static __device__ __align__(256) unsigned char scratch[TRI_STATIC_WORKSPACE_BYTES];

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int launch_status(hipError_t e, const char* what) {
  if (e == hipSuccess) return TRI_OK;
  return fail(TRI_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
}

bool is_aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

int elem_bytes(int dt) { return dt == TRI_KV_FP8_E4M3 ? 1 : 2; }

int check_layout(const tri_kv_layout* kv, bool need_v) {
  if (!kv) return fail(TRI_ERR_INVALID_ARGUMENT, "kv layout is NULL");
  if (kv->num_layers <= 0 || kv->num_kv_heads <= 0 || kv->num_kv_heads > 256)
    return fail(TRI_ERR_INVALID_ARGUMENT, "bad layer/head count (%d, %d)", kv->num_layers, kv->num_kv_heads);
  if (kv->head_dim != 64 && kv->head_dim != 128 && kv->head_dim != 256)
    return fail(TRI_ERR_UNSUPPORTED, "head_dim %d not in {64,128,256}", kv->head_dim);
  if (kv->block_size <= 0) return fail(TRI_ERR_INVALID_ARGUMENT, "block_size %d", kv->block_size);
  if (kv->kv_dtype != TRI_KV_BF16 && kv->kv_dtype != TRI_KV_FP16 && kv->kv_dtype != TRI_KV_FP8_E4M3)
    return fail(TRI_ERR_INVALID_ARGUMENT, "kv_dtype %d", kv->kv_dtype);
  if (kv->rope_style != TRI_ROPE_HALF && kv->rope_style != TRI_ROPE_INTERLEAVED)
    return fail(TRI_ERR_INVALID_ARGUMENT, "rope_style %d", kv->rope_style);
  const int eb = elem_bytes(kv->kv_dtype);
  const int64_t per16 = 16 / eb;   // elements per 16-byte access
  if (kv->stride_block % per16 || kv->stride_token % per16 || kv->stride_head % per16)
    return fail(TRI_ERR_INVALID_ARGUMENT, "strides must be multiples of %lld elements (16 bytes)", (long long)per16);
  if (kv->stride_head < kv->head_dim && kv->num_kv_heads > 1)
    return fail(TRI_ERR_INVALID_ARGUMENT, "stride_head %lld < head_dim", (long long)kv->stride_head);
  if (!kv->k_layers) return fail(TRI_ERR_INVALID_ARGUMENT, "k_layers is NULL");
  if (need_v && !kv->v_layers) return fail(TRI_ERR_INVALID_ARGUMENT, "v_layers is NULL");
  if (kv->kv_dtype == TRI_KV_FP8_E4M3 && !kv->k_scale_layers)
    return fail(TRI_ERR_INVALID_ARGUMENT, "fp8 cache without k_scale_layers");
  // v_scale_layers may be NULL: the rows then carry no scales of their own (a cache with one
  // scale per tensor) and compaction moves rows only.
  return TRI_OK;
}

int check_batch(const tri_batch* b, bool need_budget) {
  if (!b) return fail(TRI_ERR_INVALID_ARGUMENT, "batch is NULL");
  if (b->num_seqs <= 0) return fail(TRI_ERR_INVALID_ARGUMENT, "num_seqs %d", b->num_seqs);
  if (b->max_seq_len <= 0) return fail(TRI_ERR_INVALID_ARGUMENT, "max_seq_len %d", b->max_seq_len);
  if (!b->seq_lens) return fail(TRI_ERR_INVALID_ARGUMENT, "seq_lens is NULL");
  if (b->block_table && b->block_table_pitch <= 0)
    return fail(TRI_ERR_INVALID_ARGUMENT, "block_table_pitch %d", b->block_table_pitch);
  if (b->seq_lens_host)
    for (int i = 0; i < b->num_seqs; ++i)
      if (b->seq_lens_host[i] < 0 || b->seq_lens_host[i] > b->max_seq_len)
        return fail(TRI_ERR_INVALID_ARGUMENT, "seq_lens_host[%d] = %d not in [0, max_seq_len = %d]", i,
                    b->seq_lens_host[i], b->max_seq_len);
  if (need_budget) {
    if (!b->budgets) return fail(TRI_ERR_INVALID_ARGUMENT, "budgets is NULL");
    if (b->max_budget <= 0) return fail(TRI_ERR_INVALID_ARGUMENT, "max_budget %d", b->max_budget);
  }
  return TRI_OK;
}

int check_score(const tri_kv_layout* kv, const tri_score_params* sp) {
  if (!sp) return fail(TRI_ERR_INVALID_ARGUMENT, "score params are NULL");
  if (sp->num_score_heads <= 0 || sp->num_score_heads % kv->num_kv_heads)
    return fail(TRI_ERR_INVALID_ARGUMENT, "num_score_heads %d is not a multiple of num_kv_heads %d",
                sp->num_score_heads, kv->num_kv_heads);
  if (sp->num_offsets <= 0 || sp->num_offsets > tri::kMaxOffsets)
    return fail(TRI_ERR_INVALID_ARGUMENT, "num_offsets %d not in [1, %d]", sp->num_offsets, tri::kMaxOffsets);
  if (sp->aggregation != TRI_REDUCE_MEAN && sp->aggregation != TRI_REDUCE_MAX)
    return fail(TRI_ERR_INVALID_ARGUMENT, "aggregation %d", sp->aggregation);
  if (!sp->folded || !sp->omega || !sp->offsets)
    return fail(TRI_ERR_INVALID_ARGUMENT, "folded / omega / offsets is NULL");
  if (!is_aligned(sp->folded, 16)) return fail(TRI_ERR_INVALID_ARGUMENT, "folded must be 16-byte aligned");
  return TRI_OK;
}

tri::Workspace plan(const tri_kv_layout* kv, const tri_batch* b, const tri_score_params* sp, int assume_resident = 0,
                    bool allow_resident = true) {
  // Resident kernels: two-byte and fp8 keys go to the matrix-core kernel where the shape has one,
  // and only launches that fill most of the chip take them.  TRI_TUNE_RESIDENT_KERNEL overrides
  // the choice: 1 / 2 take the matrix-core / vector-unit kernel whenever the shape has it (however
  // small the launch), 3 never takes a resident kernel.
  const int64_t force = tri::tuning(TRI_TUNE_RESIDENT_KERNEL);
  const bool f_valu = force == 2;
  const bool f_mfma = force == 1;
  const bool f_off = force == 3;
  // The matrix-core kernel addresses the 16 rows of a step with 32-bit offsets from a scalar base.
  const bool want_mfma = (kv->kv_dtype == TRI_KV_BF16 || kv->kv_dtype == TRI_KV_FP16 || kv->kv_dtype == TRI_KV_FP8_E4M3) &&
                         !f_valu &&
                         kv->stride_token > 0 && kv->stride_token < (1 << 25);
  const int G = sp->num_score_heads / kv->num_kv_heads;
  const bool paged = b->block_table != nullptr;
  // assume_resident > 0: a dry run for a device of that size (tri_describe_plan); no device is asked.
  const int resident = (f_off || !allow_resident) ? 0
                       : (assume_resident > 0 ? assume_resident : tri::fused_resident_workgroups());
  tri::FusedPlan fused{};
  // Small batches are cut by layers as well (TRI_TUNE_LAYER_SPLIT = 0 switches that off, 1 switches
  // it on where the kernel was forced, which otherwise keeps whole-model workgroups).
  const int64_t split_set = tri::tuning(TRI_TUNE_LAYER_SPLIT);
  const bool split = split_set >= 0 ? split_set != 0 : !f_mfma;
  if (want_mfma)
    fused = tri::plan_fused_mfma(b->num_seqs, kv->num_kv_heads, kv->head_dim, G, kv->block_size, paged,
                                 sp->aggregation, b->max_seq_len, resident, f_mfma, kv->kv_dtype, b->seq_lens_host,
                                 kv->num_layers, split);
  if (!fused.eligible && !f_mfma)
    fused = tri::plan_fused(b->num_seqs, kv->num_kv_heads, kv->head_dim, G, kv->block_size, paged, sp->aggregation,
                            b->max_seq_len, resident, f_valu);
  return tri::plan_workspace(b->num_seqs, kv->num_layers, sp->num_score_heads, kv->head_dim / 2, sp->num_offsets,
                             kv->num_kv_heads, b->max_seq_len, fused);
}

int check_workspace(const tri::Workspace& w, void* ws, uint64_t bytes) {
  if (!ws) return fail(TRI_ERR_WORKSPACE, "workspace is NULL");
  if (!is_aligned(ws, 256)) return fail(TRI_ERR_WORKSPACE, "workspace must be 256-byte aligned");
  if (bytes < (uint64_t)w.total)
    return fail(TRI_ERR_WORKSPACE, "workspace has %llu bytes, %lld needed", (unsigned long long)bytes, (long long)w.total);
  return TRI_OK;
}

struct ResidentGate {
  static constexpr int kMaxDevices = 64;
  std::mutex mutex;
  hipEvent_t event[kMaxDevices] = {};
};
ResidentGate& resident_gate() {
  static ResidentGate gate;
  return gate;
}

// Both with the gate's mutex held.  A stream under capture is left alone.
bool gate_applies(hipStream_t s, int& dev) {
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  return hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < ResidentGate::kMaxDevices &&
         hipStreamIsCapturing(s, &cap) == hipSuccess && cap == hipStreamCaptureStatusNone;
}
int gate_enter(ResidentGate& gate, hipStream_t s) {
  int dev = 0;
  if (!gate_applies(s, dev) || !gate.event[dev]) return TRI_OK;
  return launch_status(hipStreamWaitEvent(s, gate.event[dev], 0), "resident chain wait");
}
int gate_leave(ResidentGate& gate, hipStream_t s) {
  int dev = 0;
  if (!gate_applies(s, dev)) return TRI_OK;
  if (!gate.event[dev]) {
    const hipError_t e = hipEventCreateWithFlags(&gate.event[dev], hipEventDisableTiming);
    if (e != hipSuccess) return launch_status(e, "resident chain event");
  }
  return launch_status(hipEventRecord(gate.event[dev], s), "resident chain record");
}

// Process-wide settings (tri_set_tuning).
constexpr int kTunings = 5;
std::atomic<int64_t> g_tuning[kTunings] = {{0}, {0}, {-1}, {0}, {2000000}};

// Device address of `scratch` on the current device, looked up once per device.
struct StaticScratch {
  static constexpr int kMaxDevices = 64;
  std::mutex mutex;
  void* ptr[kMaxDevices] = {};
};
int static_scratch(void** out) {
  static StaticScratch st;
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return launch_status(e, "hipGetDevice");
  if (dev < 0 || dev >= StaticScratch::kMaxDevices) return fail(TRI_ERR_UNSUPPORTED, "device %d out of range", dev);
  std::lock_guard<std::mutex> lock(st.mutex);
  if (!st.ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return launch_status(e, "hipGetSymbolAddress(scratch)");
    if (!p || !is_aligned(p, 256)) return fail(TRI_ERR_WORKSPACE, "static scratch at %p is not 256-byte aligned", p);
    st.ptr[dev] = p;
  }
  *out = st.ptr[dev];
  return TRI_OK;
}

template <typename T>
T* at(void* ws, int64_t off) { return reinterpret_cast<T*>(reinterpret_cast<char*>(ws) + off); }

int do_score(const tri_kv_layout* kv, const tri_batch* batch, const tri_score_params* sp, float* raw,
             int64_t rs_layer, int64_t rs_token, int64_t rs_head, void* ws, const tri::Workspace& w,
             hipStream_t s) {
  const int F = kv->head_dim / 2;
  hipError_t e = tri::launch_prepare(sp->folded, sp->omega, sp->offsets, sp->num_offsets, batch->round_start,
                                     batch->num_seqs, kv->num_layers, sp->num_score_heads, F, sp->aggregation,
                                     at<float>(ws, w.coef), at<float>(ws, w.trig), s);
  if (e != hipSuccess) return launch_status(e, "prepare");
  tri::ScoreLaunch a{};
  a.B = batch->num_seqs; a.L = kv->num_layers; a.Hkv = kv->num_kv_heads; a.D = kv->head_dim;
  a.block_size = kv->block_size; a.kv_dtype = kv->kv_dtype; a.rope_style = kv->rope_style;
  a.A = sp->num_score_heads; a.G = sp->num_score_heads / kv->num_kv_heads; a.NO = sp->num_offsets;
  a.aggregation = sp->aggregation;
  a.Tmax = batch->max_seq_len; a.num_tiles = w.num_tiles;
  a.stride_block = kv->stride_block; a.stride_token = kv->stride_token; a.stride_head = kv->stride_head;
  a.k_layers = kv->k_layers; a.k_scale_layers = kv->k_scale_layers;
  a.block_table = batch->block_table; a.block_table_pitch = batch->block_table_pitch;
  a.seq_lens = batch->seq_lens;
  a.coef = at<float>(ws, w.coef); a.trig = at<float>(ws, w.trig); a.partial = at<float>(ws, w.partial);
  a.raw = raw; a.raw_stride_layer = rs_layer; a.raw_stride_token = rs_token; a.raw_stride_head = rs_head;
  return launch_status(tri::launch_score(a, s), "score");
}

int check_select(const tri_select_params* sel) {
  if (!sel) return fail(TRI_ERR_INVALID_ARGUMENT, "select params are NULL");
  if (sel->group_reduce != TRI_REDUCE_MEAN && sel->group_reduce != TRI_REDUCE_MAX)
    return fail(TRI_ERR_INVALID_ARGUMENT, "group_reduce %d", sel->group_reduce);
  if (sel->layer_reduce != TRI_REDUCE_MEAN && sel->layer_reduce != TRI_REDUCE_MAX && sel->layer_reduce != -1)
    return fail(TRI_ERR_INVALID_ARGUMENT, "layer_reduce %d", sel->layer_reduce);
  if (sel->window_size < 0) return fail(TRI_ERR_INVALID_ARGUMENT, "window_size %d", sel->window_size);
  if (sel->normalize < 0 || sel->normalize > 2) return fail(TRI_ERR_INVALID_ARGUMENT, "normalize %d", sel->normalize);
  if (sel->normalize == 2 && sel->group_first)
    return fail(TRI_ERR_UNSUPPORTED, "the population-std normalisation is built for the normalise-then-reduce order only");
  return TRI_OK;
}

int do_select(const tri_kv_layout* kv, const tri_batch* batch, const tri_score_params* sp,
              const tri_select_params* sel, const float* raw, int64_t rs_layer, int64_t rs_token,
              int64_t rs_head, float* fin, int32_t* keep, void* ws, const tri::Workspace& w, hipStream_t s) {
  tri::SelectLaunch a{};
  a.B = batch->num_seqs; a.L = kv->num_layers; a.Hkv = kv->num_kv_heads; a.A = sp->num_score_heads;
  a.G = sp->num_score_heads / kv->num_kv_heads; a.Tmax = batch->max_seq_len; a.num_tiles = w.num_tiles;
  a.max_budget = batch->max_budget;
  a.normalize = sel->normalize; a.window_size = sel->window_size; a.protect_prefill = sel->protect_prefill;
  a.group_reduce = sel->group_reduce; a.layer_reduce = sel->layer_reduce; a.shared = sel->shared;
  a.group_first = sel->group_first ? 1 : 0;
  a.seq_lens = batch->seq_lens; a.prefill_lens = batch->prefill_lens; a.budgets = batch->budgets;
  a.partial = at<float>(ws, w.partial); a.mustd = at<float>(ws, w.mustd);
  a.raw = raw; a.raw_stride_layer = rs_layer; a.raw_stride_token = rs_token; a.raw_stride_head = rs_head;
  a.fin = fin ? fin : at<float>(ws, w.fin);
  a.keep = keep;
  a.group_scratch = at<double>(ws, w.coef);
  a.group_scratch_bytes = w.trig - w.coef;
  return launch_status(tri::launch_select(a, s), "select");
}

// A keep set per layer (layer_reduce -1) of a single layer is the mean over that one layer: same
// rows, same scores (x / 1).  The reference's per-layer modes call their selector once per layer
// (runtime/selector_hf.py:473-747 from the layer loop), so those calls may take a resident kernel.
int layer_reduce_of(const tri_kv_layout* kv, const tri_select_params* sel) {
  return (sel->layer_reduce < 0 && kv->num_layers == 1) ? TRI_REDUCE_MEAN : sel->layer_reduce;
}

bool takes_resident(const tri::Workspace& w, const tri_kv_layout* kv, const tri_select_params* sel) {
  return w.fused.eligible && layer_reduce_of(kv, sel) >= 0 && !sel->shared && !sel->group_first && !sel->no_resident;
}

// Selection straight from the paged keys: the resident kernel when the shape has one,
// else score into the workspace and select from there.
int do_select_paged(const tri_kv_layout* kv, const tri_batch* batch, const tri_score_params* sp,
                    const tri_select_params* sel, float* fin, int32_t* keep, void* ws, const tri::Workspace& w,
                    hipStream_t s) {
  const bool fused = takes_resident(w, kv, sel);
  if (!fused) {
    // The status word belongs to the resident kernel; on this path it just reads "fine".
    const hipError_t ce = tri::launch_clear_status(at<uint32_t>(ws, w.status), s);
    if (ce != hipSuccess) return launch_status(ce, "clear_status");
    float* raw = at<float>(ws, w.raw);
    const int64_t A = sp->num_score_heads;
    const int64_t rs_layer = (int64_t)batch->max_seq_len * A;
    const int rc = do_score(kv, batch, sp, raw, rs_layer, A, 1, ws, w, s);
    if (rc) return rc;
    return do_select(kv, batch, sp, sel, raw, rs_layer, A, 1, fin, keep, ws, w, s);
  }
  const int F = kv->head_dim / 2;
  hipError_t e = hipSuccess;
  if (w.fused.eligible != 2) {   // the matrix-core kernel has a preparation launch of its own
    e = tri::launch_prepare(sp->folded, sp->omega, sp->offsets, sp->num_offsets, batch->round_start,
                            batch->num_seqs, kv->num_layers, sp->num_score_heads, F, sp->aggregation,
                            at<float>(ws, w.coef), at<float>(ws, w.trig), s);
    if (e != hipSuccess) return launch_status(e, "prepare");
  }
  tri::FusedLaunch a{};
  a.B = batch->num_seqs; a.L = kv->num_layers; a.Hkv = kv->num_kv_heads; a.D = kv->head_dim;
  a.block_size = kv->block_size; a.kv_dtype = kv->kv_dtype; a.rope_style = kv->rope_style;
  a.A = sp->num_score_heads; a.G = sp->num_score_heads / kv->num_kv_heads; a.Tmax = batch->max_seq_len;
  a.normalize = sel->normalize; a.window_size = sel->window_size; a.protect_prefill = sel->protect_prefill;
  a.group_reduce = sel->group_reduce; a.layer_reduce = layer_reduce_of(kv, sel);
  a.stride_block = kv->stride_block; a.stride_token = kv->stride_token; a.stride_head = kv->stride_head;
  a.k_layers = kv->k_layers; a.k_scale_layers = kv->k_scale_layers;
  a.block_table = batch->block_table; a.block_table_pitch = batch->block_table_pitch;
  a.seq_lens = batch->seq_lens; a.prefill_lens = batch->prefill_lens;
  a.coef = at<float>(ws, w.coef);
  a.folded = sp->folded; a.omega = sp->omega; a.offsets = sp->offsets; a.NO = sp->num_offsets;
  a.round_start = batch->round_start;
  a.xchg = at<unsigned long long>(ws, w.xchg);
  a.status = at<uint32_t>(ws, w.status);
  a.pack = at<int32_t>(ws, w.pack);
  a.fin = fin ? fin : at<float>(ws, w.fin);
  // Partial results of a layer-split launch live where the two-pass path keeps its raw scores
  // ([B][L][Tmax][A] floats, never smaller than [groups][B][Hkv][Tmax]).
  a.fin_part = at<float>(ws, w.raw);
  a.plan = w.fused;
  // Nobody asked for the selection scores themselves: the groups' partial rows go straight to the
  // top-k, which adds them while it loads (one launch less).
  const bool split = w.fused.eligible == 2 && w.fused.layer_groups > 1;
  a.skip_layer_reduce = split && !fin && keep && batch->max_seq_len <= tri::topk_register_row_limit();
  a.bmat = at<char>(ws, w.bmat);
  if (w.fused.eligible == 2) {
    // The preparation launch writes one 16-byte entry per (sequence, layer, KV head, group of four
    // query heads, slab, lane); the region planned for them must hold that.
    const int64_t groups = a.G > 4 ? 2 : 1, slabs = a.D / 32 + a.D / 64;
    const int64_t need = (int64_t)a.B * a.L * a.Hkv * groups * slabs * 64 * 16;
    if (need > w.total - w.bmat)
      return fail(TRI_ERR_WORKSPACE, "coefficient slabs need %lld bytes, %lld planned", (long long)need,
                  (long long)(w.total - w.bmat));
  }
  {
    // Two resident launches that run at the same time on one device would each hold part of
    // the CUs and wait for the other's workgroups until their waits expire.  Launches of this
    // process are therefore chained: each waits (on the device, not on the host) for the
    // previous one on whatever stream that was.  Streams under graph capture are left alone
    // (whoever replays the graph brackets the replay with tri_resident_gate_enter / _leave).
    ResidentGate& gate = resident_gate();
    std::lock_guard<std::mutex> lock(gate.mutex);
    int rc = gate_enter(gate, s);
    if (rc) return rc;
    e = w.fused.eligible == 2 ? tri::launch_fused_mfma(a, s) : tri::launch_fused_select(a, s);
    if (e != hipSuccess) return launch_status(e, "fused_select");
    rc = gate_leave(gate, s);
    if (rc) return rc;
  }
  if (!keep) return TRI_OK;   // selection scores only
  if (a.skip_layer_reduce)
    return launch_status(tri::launch_topk_rows(a.fin_part, a.Tmax, a.B * a.Hkv, a.seq_lens, batch->budgets, a.Hkv, a.Tmax,
                                               keep, batch->max_budget, s, w.fused.layer_groups,
                                               (int64_t)a.B * a.Hkv * a.Tmax, a.layer_reduce == TRI_REDUCE_MAX),
                         "topk_rows");
  return launch_status(tri::launch_topk_rows(a.fin, a.Tmax, a.B * a.Hkv, a.seq_lens, batch->budgets, a.Hkv, a.Tmax, keep,
                                             batch->max_budget, s),
                       "topk_rows");
}

int fill_compact(const tri_kv_layout* kv, const tri_batch* batch, const int32_t* keep, int keep_per_layer,
                 int shared, tri::CompactLaunch& a) {
  int rc = check_layout(kv, true);
  if (rc) return rc;
  rc = check_batch(batch, true);
  if (rc) return rc;
  if (!batch->block_table) return fail(TRI_ERR_INVALID_ARGUMENT, "compaction needs a block table");
  if (!keep) return fail(TRI_ERR_INVALID_ARGUMENT, "keep is NULL");
  const int eb = elem_bytes(kv->kv_dtype);
  a.B = batch->num_seqs; a.L = kv->num_layers; a.Hkv = kv->num_kv_heads; a.D = kv->head_dim;
  a.block_size = kv->block_size; a.elem_bytes = eb; a.max_budget = batch->max_budget;
  a.keep_per_layer = keep_per_layer ? 1 : 0; a.shared = shared ? 1 : 0;
  a.has_scales = kv->kv_dtype == TRI_KV_FP8_E4M3 && kv->v_scale_layers != nullptr;
  a.stride_block = kv->stride_block; a.stride_token = kv->stride_token; a.stride_head = kv->stride_head;
  a.k_layers = kv->k_layers; a.v_layers = kv->v_layers;
  a.k_scale_layers = kv->k_scale_layers; a.v_scale_layers = kv->v_scale_layers;
  a.block_table = batch->block_table; a.block_table_pitch = batch->block_table_pitch;
  a.seq_lens = batch->seq_lens; a.budgets = batch->budgets; a.keep = keep; a.Tmax = batch->max_seq_len;
  a.staging = nullptr;
  return TRI_OK;
}

}  // namespace

namespace tri {
int64_t tuning(int key) { return key >= 0 && key < kTunings ? g_tuning[key].load(std::memory_order_relaxed) : 0; }
}  // namespace tri

extern "C" {

int tri_abi_version(void) { return TRI_ABI_VERSION; }

const char* tri_last_error(void) { return g_err; }

#ifndef TRI_SOURCE_DIGEST
#define TRI_SOURCE_DIGEST "unknown"
#endif
const char* tri_source_digest(void) {
  static const char digest[] = "TRI_SOURCE_DIGEST=" TRI_SOURCE_DIGEST;
  return digest + sizeof("TRI_SOURCE_DIGEST=") - 1;
}

int tri_set_tuning(int32_t key, int64_t value) {
  switch (key) {
    case TRI_TUNE_RESIDENT_KERNEL:
      if (value < 0 || value > 3) return fail(TRI_ERR_INVALID_ARGUMENT, "TRI_TUNE_RESIDENT_KERNEL takes 0..3, got %lld", (long long)value);
      break;
    case TRI_TUNE_RESIDENT_WORKGROUPS:
      if (value < 0 || value > INT_MAX) return fail(TRI_ERR_INVALID_ARGUMENT, "TRI_TUNE_RESIDENT_WORKGROUPS %lld", (long long)value);
      break;
    case TRI_TUNE_LAYER_SPLIT:
      if (value < -1 || value > 1) return fail(TRI_ERR_INVALID_ARGUMENT, "TRI_TUNE_LAYER_SPLIT takes -1, 0 or 1, got %lld", (long long)value);
      break;
    case TRI_TUNE_MAX_KERNEL:
      if (value < 0 || value > 1) return fail(TRI_ERR_INVALID_ARGUMENT, "TRI_TUNE_MAX_KERNEL takes 0 or 1, got %lld", (long long)value);
      break;
    case TRI_TUNE_RESIDENT_WAIT_US:
      // (the kernels count ticks of a 100 MHz clock in 64 bits)
      if (value > (int64_t)3600 * 1000000) return fail(TRI_ERR_INVALID_ARGUMENT, "TRI_TUNE_RESIDENT_WAIT_US beyond one hour");
      break;
    default:
      return fail(TRI_ERR_INVALID_ARGUMENT, "unknown tuning key %d", key);
  }
  g_tuning[key].store(value, std::memory_order_relaxed);
  return TRI_OK;
}

int64_t tri_get_tuning(int32_t key) {
  if (key < 0 || key >= kTunings) return INT64_MIN;
  return g_tuning[key].load(std::memory_order_relaxed);
}

int tri_resident_gate_enter(void* stream) {
  ResidentGate& gate = resident_gate();
  std::lock_guard<std::mutex> lock(gate.mutex);
  return gate_enter(gate, (hipStream_t)stream);
}

int tri_resident_gate_leave(void* stream) {
  ResidentGate& gate = resident_gate();
  std::lock_guard<std::mutex> lock(gate.mutex);
  return gate_leave(gate, (hipStream_t)stream);
}

int tri_fold_stats(const float* q_mean_real, const float* q_mean_imag, const float* q_abs_mean,
                   const float* freq_scale_sq, int32_t num_layers, int32_t num_score_heads,
                   int32_t num_pairs, int32_t disable_mlr, int32_t disable_trig, float* folded,
                   void* stream) {
  if (!q_mean_real || !q_mean_imag || !q_abs_mean || !freq_scale_sq || !folded)
    return fail(TRI_ERR_INVALID_ARGUMENT, "tri_fold_stats: NULL pointer");
  if (num_layers <= 0 || num_score_heads <= 0 || num_pairs <= 0)
    return fail(TRI_ERR_INVALID_ARGUMENT, "tri_fold_stats: bad sizes (%d, %d, %d)", num_layers, num_score_heads, num_pairs);
  return launch_status(tri::launch_fold_stats(q_mean_real, q_mean_imag, q_abs_mean, freq_scale_sq, num_layers,
                                              num_score_heads, num_pairs, disable_mlr, disable_trig, folded,
                                              (hipStream_t)stream),
                       "fold_stats");
}

uint64_t tri_workspace_bytes(const tri_kv_layout* kv, const tri_batch* batch, const tri_score_params* sp) {
  if (check_layout(kv, false) || check_batch(batch, false) || !sp || sp->num_score_heads <= 0 ||
      sp->num_offsets <= 0)
    return 0;
  return (uint64_t)plan(kv, batch, sp).total;
}

uint64_t tri_workspace_status_offset(const tri_kv_layout* kv, const tri_batch* batch,
                                     const tri_score_params* sp) {
  if (check_layout(kv, false) || check_batch(batch, false) || !sp || sp->num_score_heads <= 0 ||
      sp->num_offsets <= 0)
    return 0;
  return (uint64_t)plan(kv, batch, sp).status;
}

int tri_score_paged(const tri_kv_layout* kv, const tri_batch* batch, const tri_score_params* sp,
                    float* raw, int64_t raw_stride_layer, int64_t raw_stride_token,
                    int64_t raw_stride_head, void* workspace, uint64_t workspace_bytes, void* stream) {
  int rc = check_layout(kv, false);
  if (rc) return rc;
  rc = check_batch(batch, false);
  if (rc) return rc;
  rc = check_score(kv, sp);
  if (rc) return rc;
  if (!batch->round_start) return fail(TRI_ERR_INVALID_ARGUMENT, "round_start is NULL");
  if (!raw) return fail(TRI_ERR_INVALID_ARGUMENT, "raw is NULL");
  const tri::Workspace w = plan(kv, batch, sp);
  rc = check_workspace(w, workspace, workspace_bytes);
  if (rc) return rc;
  return do_score(kv, batch, sp, raw, raw_stride_layer, raw_stride_token, raw_stride_head, workspace, w,
                  (hipStream_t)stream);
}

int tri_select(const tri_kv_layout* kv, const tri_batch* batch, const tri_score_params* sp,
               const tri_select_params* sel, const float* raw, int64_t raw_stride_layer,
               int64_t raw_stride_token, int64_t raw_stride_head, float* final_scores, int32_t* keep,
               void* workspace, uint64_t workspace_bytes, void* stream) {
  int rc = check_layout(kv, false);
  if (rc) return rc;
  rc = check_batch(batch, true);
  if (rc) return rc;
  if (!sp || sp->num_score_heads <= 0 || sp->num_score_heads % kv->num_kv_heads || sp->num_offsets <= 0)
    return fail(TRI_ERR_INVALID_ARGUMENT, "tri_select: bad score params");
  rc = check_select(sel);
  if (rc) return rc;
  if (!raw || !keep) return fail(TRI_ERR_INVALID_ARGUMENT, "raw / keep is NULL");
  const tri::Workspace w = plan(kv, batch, sp);
  rc = check_workspace(w, workspace, workspace_bytes);
  if (rc) return rc;
  return do_select(kv, batch, sp, sel, raw, raw_stride_layer, raw_stride_token, raw_stride_head, final_scores,
                   keep, workspace, w, (hipStream_t)stream);
}

int tri_select_paged(const tri_kv_layout* kv, const tri_batch* batch, const tri_score_params* sp,
                     const tri_select_params* sel, float* final_scores, int32_t* keep, void* workspace,
                     uint64_t workspace_bytes, void* stream) {
  int rc = check_layout(kv, false);
  if (rc) return rc;
  rc = check_batch(batch, true);
  if (rc) return rc;
  rc = check_score(kv, sp);
  if (rc) return rc;
  rc = check_select(sel);
  if (rc) return rc;
  if (!batch->round_start) return fail(TRI_ERR_INVALID_ARGUMENT, "round_start is NULL");
  if (!keep && !final_scores) return fail(TRI_ERR_INVALID_ARGUMENT, "keep and final_scores are both NULL");
  const tri::Workspace w = plan(kv, batch, sp);
  rc = check_workspace(w, workspace, workspace_bytes);
  if (rc) return rc;
  return do_select_paged(kv, batch, sp, sel, final_scores, keep, workspace, w, (hipStream_t)stream);
}

int tri_select_path(const tri_kv_layout* kv, const tri_batch* batch, const tri_score_params* sp,
                    const tri_select_params* sel) {
  if (check_layout(kv, false) || check_batch(batch, false) || check_score(kv, sp) || check_select(sel)) return -1;
  const tri::Workspace w = plan(kv, batch, sp);
  return takes_resident(w, kv, sel) ? w.fused.eligible : 0;
}

int tri_describe_plan(const tri_kv_layout* kv, const tri_batch* batch, const tri_score_params* sp,
                      const tri_select_params* sel, int32_t assume_resident_workgroups, tri_plan_info* out) {
  if (!out) return fail(TRI_ERR_INVALID_ARGUMENT, "tri_describe_plan: out is NULL");
  if (assume_resident_workgroups < 0)
    return fail(TRI_ERR_INVALID_ARGUMENT, "assume_resident_workgroups %d", assume_resident_workgroups);
  int rc = check_layout(kv, false);
  if (!rc) rc = check_batch(batch, false);
  if (!rc) rc = check_score(kv, sp);
  if (!rc) rc = check_select(sel);
  if (rc) return rc;
  const tri::Workspace w = plan(kv, batch, sp, assume_resident_workgroups);
  *out = tri_plan_info{};
  out->workspace_bytes = w.total;
  out->layer_groups = 1;
  out->layers_per_group = kv->num_layers;
  if (!takes_resident(w, kv, sel)) return TRI_OK;
  const tri::FusedPlan& f = w.fused;
  out->path = f.eligible;
  out->tile_tokens = f.tile_tokens;
  out->tiles_per_seq = f.tiles_per_seq;
  out->resident_workgroups = (f.eligible == 2 && f.waves == 4) ? f.resident / 2 : f.resident;
  out->waves_per_workgroup = f.eligible == 2 ? f.waves : 8;
  if (f.eligible == 2 && f.layer_groups > 1) {
    out->layer_groups = f.layer_groups;
    out->layers_per_group = f.layers_per_group;
  }
  if (batch->num_seqs <= f.seqs_per_launch) out->launches = 1;
  else out->launches = f.launches;      // > 0: the planner replayed the packing of the host's lengths
  return TRI_OK;
}

int tri_topk_rows(const float* scores, int64_t row_pitch, int32_t num_rows, const int32_t* row_lens,
                  const int32_t* row_ks, int32_t rows_per_entry, int32_t max_len, int32_t* keep,
                  int32_t keep_pitch, void* stream) {
  if (!scores || !row_lens || !row_ks || !keep) return fail(TRI_ERR_INVALID_ARGUMENT, "tri_topk_rows: NULL pointer");
  if (num_rows < 0 || rows_per_entry <= 0 || row_pitch < max_len || keep_pitch <= 0 || max_len <= 0)
    return fail(TRI_ERR_INVALID_ARGUMENT, "tri_topk_rows: bad sizes");
  return launch_status(tri::launch_topk_rows(scores, row_pitch, num_rows, row_lens, row_ks, rows_per_entry, max_len, keep,
                                             keep_pitch, (hipStream_t)stream),
                       "topk_rows");
}

int tri_compact_paged(const tri_kv_layout* kv, const tri_batch* batch, const int32_t* keep,
                      int32_t keep_per_layer, int32_t shared, void* stream) {
  tri::CompactLaunch a{};
  const int rc = fill_compact(kv, batch, keep, keep_per_layer, shared, a);
  if (rc) return rc;
  return launch_status(tri::launch_compact(a, (hipStream_t)stream), "compact");
}

uint64_t tri_compact_full_staging_bytes(const tri_kv_layout* kv, const tri_batch* batch) {
  if (check_layout(kv, true) || check_batch(batch, false)) return 0;
  // one layer: K and V of every head row of every logical slot of every sequence
  return (uint64_t)batch->num_seqs * 2 * kv->num_kv_heads * (uint64_t)batch->max_seq_len * kv->head_dim *
         elem_bytes(kv->kv_dtype);
}

int tri_compact_paged_full(const tri_kv_layout* kv, const tri_batch* batch, const int32_t* keep,
                           int32_t keep_per_layer, int32_t shared, void* staging, uint64_t staging_bytes,
                           void* stream) {
  tri::CompactLaunch a{};
  const int rc = fill_compact(kv, batch, keep, keep_per_layer, shared, a);
  if (rc) return rc;
  if (a.has_scales) return fail(TRI_ERR_UNSUPPORTED, "full-permutation compaction of fp8 caches is not built");
  if (!staging || !is_aligned(staging, 16)) return fail(TRI_ERR_WORKSPACE, "staging is NULL or unaligned");
  if (staging_bytes < tri_compact_full_staging_bytes(kv, batch))
    return fail(TRI_ERR_WORKSPACE, "staging has %llu bytes, %llu needed", (unsigned long long)staging_bytes,
                (unsigned long long)tri_compact_full_staging_bytes(kv, batch));
  a.staging = staging;
  return launch_status(tri::launch_compact_full(a, (hipStream_t)stream), "compact_full");
}

int tri_compress_step(const tri_kv_layout* kv, const tri_batch* batch, const tri_score_params* sp,
                      const tri_select_params* sel, int32_t* keep, void* workspace,
                      uint64_t workspace_bytes, void* stream) {
  int rc = check_layout(kv, true);
  if (rc) return rc;
  rc = check_batch(batch, true);
  if (rc) return rc;
  rc = check_score(kv, sp);
  if (rc) return rc;
  rc = check_select(sel);
  if (rc) return rc;
  if (!batch->round_start) return fail(TRI_ERR_INVALID_ARGUMENT, "round_start is NULL");
  if (!batch->block_table) return fail(TRI_ERR_INVALID_ARGUMENT, "tri_compress_step needs a block table");
  if (!keep) return fail(TRI_ERR_INVALID_ARGUMENT, "keep is NULL");
  const tri::Workspace w = plan(kv, batch, sp);
  rc = check_workspace(w, workspace, workspace_bytes);
  if (rc) return rc;
  hipStream_t s = (hipStream_t)stream;
  rc = do_select_paged(kv, batch, sp, sel, nullptr, keep, workspace, w, s);
  if (rc) return rc;
  tri::CompactLaunch c{};
  rc = fill_compact(kv, batch, keep, sel->layer_reduce < 0, sel->shared, c);
  if (rc) return rc;
  // A resident kernel whose bounded wait expired leaves meaningless keep lists and a raised
  // status word: the compaction kernels look at that word and then leave the cache alone.
  c.guard = at<uint32_t>(workspace, w.status);
  return launch_status(tri::launch_compact(c, s), "compact");
}

int tri_compress_step_static(const tri_kv_layout* kv, const tri_batch* batch, const tri_score_params* sp,
                             const tri_select_params* sel, int32_t* keep, const uint32_t** status_out,
                             void* stream) {
  int rc = check_layout(kv, true);
  if (rc) return rc;
  rc = check_batch(batch, true);
  if (rc) return rc;
  rc = check_score(kv, sp);
  if (rc) return rc;
  rc = check_select(sel);
  if (rc) return rc;
  if (!batch->round_start) return fail(TRI_ERR_INVALID_ARGUMENT, "round_start is NULL");
  if (!batch->block_table) return fail(TRI_ERR_INVALID_ARGUMENT, "tri_compress_step_static needs a block table");
  if (!keep) return fail(TRI_ERR_INVALID_ARGUMENT, "keep is NULL");
  // Always the score-then-select kernels, so the scratch is sized for them alone (a resident plan
  // would add its coefficient slabs and exchange words; the status word sits at the same offset).
  const tri::Workspace w = plan(kv, batch, sp, 0, false);
  if ((uint64_t)w.total > (uint64_t)TRI_STATIC_WORKSPACE_BYTES)
    return fail(TRI_ERR_WORKSPACE, "this step needs %lld bytes of scratch, the library's static array holds %llu; "
                "use tri_compress_step with a workspace of the caller's", (long long)w.total,
                (unsigned long long)TRI_STATIC_WORKSPACE_BYTES);
  void* ws = nullptr;
  rc = static_scratch(&ws);
  if (rc) return rc;
  if (status_out) *status_out = at<uint32_t>(ws, w.status);
  tri_select_params two_pass = *sel;
  two_pass.no_resident = 1;   // the resident path chains its launches with an event it creates
  hipStream_t s = (hipStream_t)stream;
  rc = do_select_paged(kv, batch, sp, &two_pass, nullptr, keep, ws, w, s);
  if (rc) return rc;
  tri::CompactLaunch c{};
  rc = fill_compact(kv, batch, keep, sel->layer_reduce < 0, sel->shared, c);
  if (rc) return rc;
  c.guard = at<uint32_t>(ws, w.status);
  c.no_side_stream = 1;
  return launch_status(tri::launch_compact(c, s), "compact");
}

uint64_t tri_qstats_workspace_bytes(int32_t num_heads, int32_t num_tokens, int32_t head_dim) {
  if (num_heads <= 0 || num_tokens <= 0 || (head_dim != 64 && head_dim != 128 && head_dim != 256)) return 0;
  return (uint64_t)tri::qstats_workspace_bytes(num_heads, num_tokens, head_dim);
}

int tri_qstats(const void* q_rot, int64_t stride_head, int64_t stride_token, const void* cos, const void* sin,
               int32_t num_heads, int32_t num_tokens, int32_t head_dim, int32_t dtype, int32_t rope_style,
               float scale, float* out_real, float* out_imag, float* out_abs, void* workspace,
               uint64_t workspace_bytes, void* stream) {
  if (!q_rot || !cos || !sin || !out_real || !out_imag || !out_abs)
    return fail(TRI_ERR_INVALID_ARGUMENT, "tri_qstats: NULL pointer");
  if (num_heads <= 0 || num_tokens <= 0) return fail(TRI_ERR_INVALID_ARGUMENT, "tri_qstats: bad sizes");
  if (head_dim != 64 && head_dim != 128 && head_dim != 256)
    return fail(TRI_ERR_UNSUPPORTED, "head_dim %d not in {64,128,256}", head_dim);
  if (dtype != TRI_KV_BF16 && dtype != TRI_KV_FP16)
    return fail(TRI_ERR_UNSUPPORTED, "tri_qstats: dtype %d (bf16 or fp16 query states)", dtype);
  if (rope_style != TRI_ROPE_HALF && rope_style != TRI_ROPE_INTERLEAVED)
    return fail(TRI_ERR_INVALID_ARGUMENT, "rope_style %d", rope_style);
  if (scale == 0.f) return fail(TRI_ERR_INVALID_ARGUMENT, "attention scaling factor must be non-zero");
  if (stride_token < head_dim || stride_token % 2 || stride_head % 2 || !is_aligned(q_rot, 4) || !is_aligned(cos, 4) ||
      !is_aligned(sin, 4))
    return fail(TRI_ERR_INVALID_ARGUMENT, "tri_qstats: rows must be 4-byte aligned and head_dim contiguous");
  const uint64_t need = tri_qstats_workspace_bytes(num_heads, num_tokens, head_dim);
  if (!workspace || workspace_bytes < need || !is_aligned(workspace, 16))
    return fail(TRI_ERR_WORKSPACE, "tri_qstats: workspace of %llu bytes needed", (unsigned long long)need);
  tri::QStatsLaunch q{};
  q.q_rot = q_rot; q.cos = cos; q.sin = sin;
  q.stride_head = stride_head; q.stride_token = stride_token;
  q.H = num_heads; q.T = num_tokens; q.D = head_dim; q.dtype = dtype; q.rope_style = rope_style;
  q.scale = scale;
  q.out_real = out_real; q.out_imag = out_imag; q.out_abs = out_abs;
  q.workspace = workspace;
  return launch_status(tri::launch_qstats(q, (hipStream_t)stream), "qstats");
}

}  // extern "C"
