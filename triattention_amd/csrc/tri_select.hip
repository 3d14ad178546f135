// Score normalisation, guards, head / layer reduction and per-row top-k for gfx950.
//
//  finalize_stats_kernel : per-(sequence, layer, score head) mean and safe std from the
//                          scorer's per-tile sums (runtime/selector_hf.py:896-913).
//  combine_kernel        : z-score, +inf guards, reduce over the query heads of a KV
//                          head, reduce over layers (runtime/selector_hf.py:916-989).
//  group_stats_kernel    : the other order of operations (the reference's SGLang backend,
//                          sglang/scheduler_hooks.py:655-690): reduce over the query heads of
//                          a KV head first, then normalise per (layer, KV head) with
//                          core/utils.py:466-480 (torch mean / unbiased std).
//  topk_rows_kernel      : order-preserving radix select on the monotone integer
//                          image of the float, then an ordered compaction that emits
//                          the kept token indices ascending; ties at the threshold
//                          keep the lowest index (replaces torch.topk + chunk merge +
//                          torch.sort, runtime/selector_hf.py:990-1025).
#include "tri_common.h"

namespace tri {
namespace {

__global__ void finalize_stats_kernel(const float* partial, const int32_t* seq_lens, int B, int L, int A,
                                      int num_tiles, int normalize, float* mustd) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= B * L * A) return;
  const int a = idx % A, bl = idx / A, b = bl / L;
  float mean = 0.f, sd = 1.f;
  if (normalize) {
    const int T = seq_lens[b];
    const int nt = ceil_div(T, kScoreTileTokens);
    double s = 0.0, q = 0.0;
    for (int t = 0; t < nt; ++t) {
      const float* p = partial + (((int64_t)bl * num_tiles + t) * A + a) * 2;
      s += (double)p[0];
      q += (double)p[1];
    }
    // The reference's formula on fp32 sums (runtime/selector_hf.py:902-909).
    const float sum = (float)s, sumsq = (float)q, cnt = (float)T;
    mean = __fdiv_rn(sum, cnt);
    float var = 0.f;
    if (T > 1) var = __fdiv_rn(__fsub_rn(sumsq, __fmul_rn(cnt, __fmul_rn(mean, mean))), (float)(T - 1));
    var = fmaxf(var, 0.f);
    sd = __fsqrt_rn(var);
    if (sd < 1e-8f) sd = 1.f;
    if (normalize == 2) {
      // The research path's normalisation (methods/triattention.py:255-258): population standard
      // deviation, clamped from below at 1e-6; from the double-precision sums.
      const double m = s / (double)T;
      const double v = q / (double)T - m * m;
      mean = (float)m;
      sd = fmaxf((float)sqrt(v > 0.0 ? v : 0.0), 1e-6f);
    }
  }
  mustd[(int64_t)idx * 2] = mean;
  mustd[(int64_t)idx * 2 + 1] = sd;
}

// Reduce-first order: mean and std over the tokens of m[n] = reduce over the query heads of
// raw[n][h*G .. h*G+G), per (sequence, layer, KV head), with torch's definitions
// (core/utils.py:476-479: mean, unbiased std, std < 1e-8 -> 1).  Sums in double; one
// workgroup per (sequence, layer, KV head).  mustd[(b*L + l)*A*2 + h*2] = (mean, std).
__global__ __launch_bounds__(256) void group_stats_kernel(const float* raw, int64_t stride_layer, int64_t stride_token,
                                                          int64_t stride_head, const int32_t* seq_lens, int L, int Hkv,
                                                          int A, int G, int group_reduce, int normalize, float* mustd) {
  __shared__ double red[256][2];
  const int h = blockIdx.x % Hkv;
  const int bl = blockIdx.x / Hkv, b = bl / L;
  float* out = mustd + ((int64_t)bl * A + h) * 2;
  if (!normalize) {
    if (threadIdx.x == 0) { out[0] = 0.f; out[1] = 1.f; }
    return;
  }
  const int T = seq_lens[b];
  const float* base = raw + (int64_t)bl * stride_layer + (int64_t)h * G * stride_head;
  double s = 0.0, q = 0.0;
  for (int n = threadIdx.x; n < T; n += 256) {
    const float* p = base + (int64_t)n * stride_token;
    float m = (group_reduce == TRI_REDUCE_MAX) ? -INFINITY : 0.f;
    for (int g = 0; g < G; ++g) {
      const float x = p[(int64_t)g * stride_head];
      m = (group_reduce == TRI_REDUCE_MAX) ? fmaxf(m, x) : __fadd_rn(m, x);
    }
    if (group_reduce != TRI_REDUCE_MAX) m = __fdiv_rn(m, (float)G);
    s += (double)m;
    q += (double)m * (double)m;
  }
  red[threadIdx.x][0] = s;
  red[threadIdx.x][1] = q;
  __syncthreads();
  for (int off = 128; off > 0; off >>= 1) {
    if (threadIdx.x < off) {
      red[threadIdx.x][0] += red[threadIdx.x + off][0];
      red[threadIdx.x][1] += red[threadIdx.x + off][1];
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    const double mean = red[0][0] / (double)T;
    double var = T > 1 ? (red[0][1] - (double)T * mean * mean) / (double)(T - 1) : 0.0;
    if (var < 0.0) var = 0.0;
    float sd = (float)sqrt(var);
    if (sd < 1e-8f) sd = 1.f;     // also a single token, where torch's unbiased std is undefined
    out[0] = (float)mean;
    out[1] = sd;
  }
}

// The same statistics for the usual layout -- four query heads per KV head, raw scores head-contiguous
// ([token][head], 16-byte aligned), a power-of-two number of KV heads -- in two launches that read whole
// token rows: a workgroup takes a chunk of 2048 tokens of one (sequence, layer) with thread = (token,
// KV head), so a wave reads 1 KB of consecutive memory per load where the kernel above reads 16 bytes
// of every 128-byte row eight times over (one request of 16384 tokens x 36 layers: 117 -> 30 us), and
// leaves the chunk's sums in double; the second launch adds the chunks in order.
constexpr int kGroupStatsChunk = 2048;
__global__ __launch_bounds__(256) void group_stats_partial_kernel(const float* raw, int64_t stride_layer,
                                                                  int64_t stride_token, const int32_t* seq_lens, int L,
                                                                  int Hkv, int chunks, int group_reduce,
                                                                  double* partial) {
  __shared__ double red[256][2];
  const int c = blockIdx.x, bl = blockIdx.y, b = bl / L;
  const int T = seq_lens[b];
  const int h = threadIdx.x % Hkv, tn = threadIdx.x / Hkv, tstep = 256 / Hkv;
  const int n_end = min(T, (c + 1) * kGroupStatsChunk);
  const float* base = raw + (int64_t)bl * stride_layer + h * 4;
  double s = 0.0, q = 0.0;
  for (int n = c * kGroupStatsChunk + tn; n < n_end; n += tstep) {
    const float4 x = *reinterpret_cast<const float4*>(base + (int64_t)n * stride_token);
    float m;
    if (group_reduce == TRI_REDUCE_MAX) m = fmaxf(fmaxf(x.x, x.y), fmaxf(x.z, x.w));
    else m = __fdiv_rn(__fadd_rn(__fadd_rn(__fadd_rn(x.x, x.y), x.z), x.w), 4.f);
    s += (double)m;
    q += (double)m * (double)m;
  }
  red[threadIdx.x][0] = s;
  red[threadIdx.x][1] = q;
  __syncthreads();
  for (int off = 128; off >= Hkv; off >>= 1) {       // threads `off` apart hold the same KV head
    if ((int)threadIdx.x < off) {
      red[threadIdx.x][0] += red[threadIdx.x + off][0];
      red[threadIdx.x][1] += red[threadIdx.x + off][1];
    }
    __syncthreads();
  }
  if ((int)threadIdx.x < Hkv) {
    double* out = partial + (((int64_t)bl * chunks + c) * Hkv + threadIdx.x) * 2;
    out[0] = red[threadIdx.x][0];
    out[1] = red[threadIdx.x][1];
  }
}

__global__ void group_stats_finish_kernel(const double* partial, const int32_t* seq_lens, int BL, int L, int Hkv, int A,
                                          int chunks, float* mustd) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= BL * Hkv) return;
  const int h = idx % Hkv, bl = idx / Hkv, b = bl / L;
  const int T = seq_lens[b];
  const int nc = ceil_div(T, kGroupStatsChunk);
  double s = 0.0, q = 0.0;
  for (int c = 0; c < nc; ++c) {
    const double* p = partial + (((int64_t)bl * chunks + c) * Hkv + h) * 2;
    s += p[0];
    q += p[1];
  }
  const double mean = s / (double)T;
  double var = T > 1 ? (q - (double)T * mean * mean) / (double)(T - 1) : 0.0;
  if (var < 0.0) var = 0.0;
  float sd = (float)sqrt(var);
  if (sd < 1e-8f) sd = 1.f;
  float* out = mustd + ((int64_t)bl * A + h) * 2;
  out[0] = (float)mean;
  out[1] = sd;
}

struct CombineArgs {
  const float* raw;
  const float* mustd;
  const int32_t* seq_lens;
  const int32_t* prefill_lens;
  float* fin;
  int64_t raw_stride_layer, raw_stride_token, raw_stride_head;
  int B, L, Hkv, A, G, Tmax;
  int window_size, protect_prefill, group_reduce, layer_reduce, shared;
  int group_first;    // 1: reduce over the query heads of a KV head before normalising (mustd is per KV head)
  int rows_per_seq;   // rows per (sequence[, layer]): shared ? 1 : Hkv
  int tokens_per_wg;  // 256 / rows_per_seq
};

// z-score of one raw value with the reference's operation order: (x - mean) / std.
__device__ __forceinline__ float zscore(float x, float mean, float sd) {
  return __fdiv_rn(__fsub_rn(x, mean), sd);
}

// One thread per (token, output row).  Grid: (token tiles, layers or 1, B).
// NV > 0: groups of 4 * NV query heads (4 or 8), raw scores head-contiguous and 16-byte aligned, read as
// NV 16-byte loads per layer; NV = 0: any layout, one score at a time.
template <int NV>
__global__ __launch_bounds__(256) void combine_kernel(CombineArgs a) {
  extern __shared__ float tile[];  // [rows_per_seq][tokens_per_wg]
  const int b = blockIdx.z;
  const int T = a.seq_lens[b];
  const int n0 = blockIdx.x * a.tokens_per_wg;
  if (n0 >= T) return;
  const int R = a.rows_per_seq;
  const int tn = threadIdx.x / R, r = threadIdx.x % R;
  const int n = n0 + tn;
  const bool per_layer = a.layer_reduce < 0;
  const int l_begin = per_layer ? blockIdx.y : 0;
  const int l_end = per_layer ? blockIdx.y + 1 : a.L;

  if (tn < a.tokens_per_wg && n < T) {
    bool guard = false;
    if (a.window_size > 0) guard = n >= T - min(a.window_size, T);
    if (a.protect_prefill && a.prefill_lens) guard = guard || (n < a.prefill_lens[b]);
    const int h_begin = a.shared ? 0 : r;
    const int h_end = a.shared ? a.Hkv : r + 1;
    float acc = 0.f;
    if (NV > 0 && !a.shared) {
      // Default shapes: one KV head per thread, its query heads in NV 16-byte loads; several layers in
      // flight per thread.
      constexpr int NVV = NV > 0 ? NV : 1;
      constexpr int GQ = 4 * NVV;                  // query heads per KV head
      constexpr int U = NVV == 1 ? 4 : 2;          // layers in flight
      const float* raw0 = a.raw + (int64_t)b * a.L * a.raw_stride_layer + (int64_t)n * a.raw_stride_token + r * GQ;
      // Reduce-first order (group_first): the statistics are those of the KV head's reduced score and
      // sit in entry r of the layer's table; they arrive in m[0].x / m[0].y (the rest unused).
      const float* ms0 = a.mustd + ((int64_t)b * a.L * a.A + (a.group_first ? r : r * GQ)) * 2;
      struct LayerIn { float4 x[NVV]; float4 m[2 * NVV]; };
      auto load_layer = [&](int l, LayerIn& in) {
        const float* rl = raw0 + (int64_t)l * a.raw_stride_layer;
        const float* ms = ms0 + (int64_t)l * a.A * 2;
#pragma unroll
        for (int i = 0; i < NVV; ++i) in.x[i] = *reinterpret_cast<const float4*>(rl + 4 * i);
        if (a.group_first) {
          const float2 m = *reinterpret_cast<const float2*>(ms);
#pragma unroll
          for (int i = 0; i < 2 * NVV; ++i) in.m[i] = float4{m.x, m.y, 0.f, 0.f};
        } else {
          // mustd is [head][mean, std]: m[2 i] = (mean, std) of query heads 4 i and 4 i + 1, m[2 i + 1] of the next two.
#pragma unroll
          for (int i = 0; i < 2 * NVV; ++i) in.m[i] = *reinterpret_cast<const float4*>(ms + 4 * i);
        }
      };
      auto layer_value = [&](const LayerIn& in) {
        float xs[GQ];
#pragma unroll
        for (int i = 0; i < NVV; ++i) { xs[4 * i] = in.x[i].x; xs[4 * i + 1] = in.x[i].y; xs[4 * i + 2] = in.x[i].z; xs[4 * i + 3] = in.x[i].w; }
        float v;
        if (a.group_first) {
          // (the order of the scalar path below: query heads one after the other)
          float m = xs[0];
#pragma unroll
          for (int q = 1; q < GQ; ++q) m = (a.group_reduce == TRI_REDUCE_MAX) ? fmaxf(m, xs[q]) : __fadd_rn(m, xs[q]);
          if (a.group_reduce != TRI_REDUCE_MAX) m = __fdiv_rn(m, (float)GQ);
          v = zscore(m, in.m[0].x, in.m[0].y);
        } else {
          float z[GQ];
#pragma unroll
          for (int i = 0; i < 2 * NVV; ++i) {
            z[2 * i] = zscore(xs[2 * i], in.m[i].x, in.m[i].y);
            z[2 * i + 1] = zscore(xs[2 * i + 1], in.m[i].z, in.m[i].w);
          }
          v = z[0];
#pragma unroll
          for (int q = 1; q < GQ; ++q) v = (a.group_reduce == TRI_REDUCE_MAX) ? fmaxf(v, z[q]) : __fadd_rn(v, z[q]);
          if (a.group_reduce != TRI_REDUCE_MAX) v = __fdiv_rn(v, (float)GQ);
        }
        return guard ? INFINITY : v;
      };
      int l = l_begin;
      for (; l + U <= l_end; l += U) {
        LayerIn in[U];
#pragma unroll
        for (int u = 0; u < U; ++u) load_layer(l + u, in[u]);
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const float v = layer_value(in[u]);
          if (l + u == l_begin) acc = v;
          else acc = (a.layer_reduce == TRI_REDUCE_MAX) ? fmaxf(acc, v) : __fadd_rn(acc, v);
        }
      }
      for (; l < l_end; ++l) {
        LayerIn in;
        load_layer(l, in);
        const float v = layer_value(in);
        if (l == l_begin) acc = v;
        else acc = (a.layer_reduce == TRI_REDUCE_MAX) ? fmaxf(acc, v) : __fadd_rn(acc, v);
      }
    } else {
      for (int l = l_begin; l < l_end; ++l) {
        const float* raw_l = a.raw + (int64_t)(b * a.L + l) * a.raw_stride_layer + (int64_t)n * a.raw_stride_token;
        const float* ms = a.mustd + (int64_t)(b * a.L + l) * a.A * 2;
        float v = -INFINITY;
        for (int h = h_begin; h < h_end; ++h) {
          float gv = (a.group_reduce == TRI_REDUCE_MAX) ? -INFINITY : 0.f;
          for (int q = 0; q < a.G; ++q) {
            const int ah = h * a.G + q;
            const float x = raw_l[(int64_t)ah * a.raw_stride_head];
            const float z = a.group_first ? x : zscore(x, ms[ah * 2], ms[ah * 2 + 1]);
            gv = (a.group_reduce == TRI_REDUCE_MAX) ? fmaxf(gv, z) : __fadd_rn(gv, z);
          }
          if (a.group_reduce != TRI_REDUCE_MAX) gv = __fdiv_rn(gv, (float)a.G);
          if (a.group_first) gv = zscore(gv, ms[h * 2], ms[h * 2 + 1]);
          v = fmaxf(v, gv);
        }
        if (guard) v = INFINITY;
        if (l == l_begin) acc = v;
        else acc = (a.layer_reduce == TRI_REDUCE_MAX) ? fmaxf(acc, v) : __fadd_rn(acc, v);
      }
    }
    if (a.layer_reduce == TRI_REDUCE_MEAN) acc = __fdiv_rn(acc, (float)a.L);
    tile[r * a.tokens_per_wg + tn] = acc;
  }
  __syncthreads();
  // Coalesced write of the [rows][tokens] tile.
  const int nvalid = min(a.tokens_per_wg, T - n0);
  const int64_t row0 = per_layer ? ((int64_t)(b * a.L + blockIdx.y) * R) : ((int64_t)b * R);
  for (int i = threadIdx.x; i < R * a.tokens_per_wg; i += 256) {
    const int rr = i / a.tokens_per_wg, tt = i % a.tokens_per_wg;
    if (tt < nvalid) a.fin[(row0 + rr) * a.Tmax + n0 + tt] = tile[i];
  }
}

// Monotone map float -> uint32: a < b  <=>  key(a) < key(b).
__device__ __forceinline__ uint32_t float_key(float f) {
  const uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

constexpr int kTopkThreads = 1024;

// One workgroup per row.
__global__ __launch_bounds__(kTopkThreads) void topk_rows_kernel(const float* scores, int64_t row_pitch,
                                                                const int32_t* row_lens,
                                                                const int32_t* row_ks, int rows_per_entry,
                                                                int32_t* keep, int keep_pitch, int max_len) {
  __shared__ uint32_t hist[256];
  __shared__ uint32_t scan[256];
  __shared__ uint32_t sh_prefix, sh_remaining;
  __shared__ uint32_t cnt_gt[kTopkThreads];
  __shared__ uint32_t cnt_eq[kTopkThreads];

  const int row = blockIdx.x;
  const int entry = row / rows_per_entry;
  // Lengths and budgets live on the device; the host sized rows for max_len scores and
  // keep_pitch indices, and neither is ever exceeded whatever the device arrays say.
  const int T = min(row_lens[entry], max_len);
  int k = min(row_ks[entry], keep_pitch);
  if (k > T) k = T;
  if (k <= 0 || T <= 0) return;
  const float* x = scores + (int64_t)row * row_pitch;
  int32_t* out = keep + (int64_t)row * keep_pitch;
  const int tid = threadIdx.x;

  if (k >= T) {
    for (int i = tid; i < T; i += kTopkThreads) out[i] = i;
    return;
  }

  // ---- radix select of the k-th largest key, 8 bits per pass from the top.
  uint32_t prefix = 0, mask = 0, remaining = (uint32_t)k;
  for (int shift = 24; shift >= 0; shift -= 8) {
    if (tid < 256) hist[tid] = 0;
    __syncthreads();
    for (int i = tid; i < T; i += kTopkThreads) {
      const uint32_t key = float_key(x[i]);
      if ((key & mask) == prefix) atomicAdd(&hist[(key >> shift) & 255u], 1u);
    }
    __syncthreads();
    // suffix[d] = number of candidates with digit >= d (Hillis-Steele over 256 bins).
    if (tid < 256) scan[tid] = hist[tid];
    __syncthreads();
    for (int off = 1; off < 256; off <<= 1) {
      uint32_t v = 0;
      if (tid < 256 && tid + off < 256) v = scan[tid + off];
      __syncthreads();
      if (tid < 256) scan[tid] += v;
      __syncthreads();
    }
    if (tid < 256) {
      const uint32_t ge = scan[tid];
      const uint32_t gt = (tid < 255) ? scan[tid + 1] : 0u;
      if (gt < remaining && remaining <= ge) {   // exactly one digit satisfies this
        sh_prefix = prefix | ((uint32_t)tid << shift);
        sh_remaining = remaining - gt;
      }
    }
    __syncthreads();
    prefix = sh_prefix;
    remaining = sh_remaining;
    mask |= 255u << shift;
    __syncthreads();
  }
  const uint32_t thr = prefix;        // key of the k-th largest element
  const uint32_t need_eq = remaining; // how many elements equal to it are kept (lowest index first)

  // ---- ordered compaction: every thread owns a contiguous chunk of the row.
  const int chunk = ceil_div(T, kTopkThreads);
  const int c0 = min(tid * chunk, T), c1 = min(c0 + chunk, T);
  uint32_t g = 0, e = 0;
  for (int i = c0; i < c1; ++i) {
    const uint32_t key = float_key(x[i]);
    g += key > thr;
    e += key == thr;
  }
  cnt_gt[tid] = g;
  cnt_eq[tid] = e;
  __syncthreads();
  // Exclusive scan of both counters over threads (Hillis-Steele, inclusive then shift).
  for (int off = 1; off < kTopkThreads; off <<= 1) {
    uint32_t vg = 0, ve = 0;
    if (tid >= off) { vg = cnt_gt[tid - off]; ve = cnt_eq[tid - off]; }
    __syncthreads();
    cnt_gt[tid] += vg;
    cnt_eq[tid] += ve;
    __syncthreads();
  }
  uint32_t gt_before = cnt_gt[tid] - g;
  uint32_t eq_before = cnt_eq[tid] - e;
  uint32_t pos = gt_before + min(eq_before, need_eq);
  for (int i = c0; i < c1; ++i) {
    const uint32_t key = float_key(x[i]);
    if (key > thr) {
      out[pos++] = i;
    } else if (key == thr) {
      if (eq_before < need_eq) out[pos++] = i;
      ++eq_before;
    }
  }
}

// The same selection for rows of at most VPT * 1024 elements: the row is read once into
// registers (thread t owns the contiguous elements [t*VPT, (t+1)*VPT), so the ordered
// emission needs no second pass over memory), the 256-bin suffix sums of a radix pass are
// taken by one wave with shuffles, and the final scan over threads is a wave scan plus 16
// wave totals: 3 barriers per radix pass instead of 19.
template <int VPT>
__global__ __launch_bounds__(kTopkThreads) void topk_rows_reg_kernel(const float* scores, int64_t row_pitch,
                                                                    const int32_t* row_lens,
                                                                    const int32_t* row_ks, int rows_per_entry,
                                                                    int32_t* keep, int keep_pitch, int max_len,
                                                                    int groups, int64_t group_stride, int group_max) {
  __shared__ uint32_t hist[256];
  __shared__ uint32_t sh_prefix, sh_remaining;
  __shared__ uint32_t wave_tot[kTopkThreads / 64];

  const int row = blockIdx.x;
  const int entry = row / rows_per_entry;
  // Lengths and budgets live on the device; the host sized rows for max_len scores and
  // keep_pitch indices, and neither is ever exceeded whatever the device arrays say.
  const int T = min(row_lens[entry], max_len);
  int k = min(row_ks[entry], keep_pitch);
  if (k > T) k = T;
  if (k <= 0 || T <= 0) return;
  const float* x = scores + (int64_t)row * row_pitch;
  int32_t* out = keep + (int64_t)row * keep_pitch;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

  if (k >= T) {
    for (int i = tid; i < T; i += kTopkThreads) out[i] = i;
    return;
  }

  const int c0 = tid * VPT;
  const int nvalid = min(max(T - c0, 0), VPT);
  uint32_t key[VPT];
  if (groups > 1) {
    // The row arrives as `groups` partial rows `group_stride` floats apart (a resident launch cut
    // by layers): they are added (or maximised) in group order, exactly as
    // fused_layer_reduce_kernel does; the division by the layer count that turns the sum into a
    // mean does not change the order of the scores and is left out.
    // The rows of several groups are requested before the first is added (a thread's loads of one
    // group after the other, each waited for, made 36 groups of a single request take 30 us).
    constexpr int U = VPT >= 32 ? 1 : (VPT >= 16 ? 2 : 4);            // groups in flight per round
    const bool vec = nvalid == VPT && (reinterpret_cast<uintptr_t>(x + c0) & 15) == 0 && (group_stride & 3) == 0;
    auto load_row = [&](int g, float (&y)[VPT]) __attribute__((always_inline)) {
      const float* p = x + (int64_t)g * group_stride + c0;
      if (vec) {
#pragma unroll
        for (int i = 0; i < VPT; i += 4) {
          const float4 q = *reinterpret_cast<const float4*>(p + i);
          y[i] = q.x; y[i + 1] = q.y; y[i + 2] = q.z; y[i + 3] = q.w;
        }
      } else {
#pragma unroll
        for (int i = 0; i < VPT; ++i) y[i] = i < nvalid ? p[i] : 0.f;
      }
    };
    float v[VPT];
    load_row(0, v);
    int g = 1;
    for (; g + U <= groups; g += U) {
      float y[U][VPT];
#pragma unroll
      for (int u = 0; u < U; ++u) load_row(g + u, y[u]);
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int i = 0; i < VPT; ++i) v[i] = group_max ? fmaxf(v[i], y[u][i]) : __fadd_rn(v[i], y[u][i]);
    }
    for (; g < groups; ++g) {
      float y[VPT];
      load_row(g, y);
#pragma unroll
      for (int i = 0; i < VPT; ++i) v[i] = group_max ? fmaxf(v[i], y[i]) : __fadd_rn(v[i], y[i]);
    }
#pragma unroll
    for (int i = 0; i < VPT; ++i) key[i] = i < nvalid ? float_key(v[i]) : 0u;
  } else if (nvalid == VPT && (reinterpret_cast<uintptr_t>(x + c0) & 15) == 0) {
#pragma unroll
    for (int i = 0; i < VPT; i += 4) {
      const float4 v = *reinterpret_cast<const float4*>(x + c0 + i);
      key[i] = float_key(v.x); key[i + 1] = float_key(v.y); key[i + 2] = float_key(v.z); key[i + 3] = float_key(v.w);
    }
  } else {
#pragma unroll
    for (int i = 0; i < VPT; ++i) key[i] = i < nvalid ? float_key(x[c0 + i]) : 0u;
  }

  // ---- radix select of the k-th largest key, 8 bits per pass from the top.
  uint32_t prefix = 0, mask = 0, remaining = (uint32_t)k;
  for (int shift = 24; shift >= 0; shift -= 8) {
    if (tid < 256) hist[tid] = 0;
    __syncthreads();
    // Selection scores are sums of z-scores of similar size, so the leading digit (sign and the top
    // exponent bits) takes three or four values in a whole row and the first pass would send all 64
    // lanes of every atomic to the same few counters, one after the other.  The lanes of a wave that
    // hold the same digit are counted with a ballot and added once (up to four distinct digits per
    // round; what is left, and the later passes, whose digits are spread, take the plain atomics).
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const bool part = i < nvalid && (key[i] & mask) == prefix;
      const uint32_t digit = (key[i] >> shift) & 255u;
      unsigned long long todo = __ballot(part);
      if (shift == 24) {
        for (int it = 0; it < 4 && todo; ++it) {
          const int leader = __builtin_amdgcn_readfirstlane(__ffsll((long long)todo) - 1);
          const uint32_t dl = (uint32_t)__builtin_amdgcn_readlane((int)digit, leader);
          const unsigned long long same = __ballot(part && digit == dl) & todo;
          if (lane == leader) atomicAdd(&hist[dl], (uint32_t)__popcll(same));
          todo &= ~same;
        }
      }
      if ((todo >> lane) & 1ull) atomicAdd(&hist[digit], 1u);
    }
    __syncthreads();
    if (wave == 0) {
      // lane owns bins 4*lane .. 4*lane+3; ge[j] = candidates whose digit is >= that bin
      uint32_t h[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) h[j] = hist[4 * lane + j];
      const uint32_t own = h[0] + h[1] + h[2] + h[3];
      uint32_t suffix = own;                         // sum over lanes >= lane
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const uint32_t v = __shfl_down(suffix, off);
        if (lane + off < 64) suffix += v;
      }
      uint32_t gt = suffix - own;                    // digits above this lane's bins
#pragma unroll
      for (int j = 3; j >= 0; --j) {
        const uint32_t ge = gt + h[j];
        if (gt < remaining && remaining <= ge) {     // exactly one bin satisfies this
          sh_prefix = prefix | ((uint32_t)(4 * lane + j) << shift);
          sh_remaining = remaining - gt;
        }
        gt = ge;
      }
    }
    __syncthreads();
    prefix = sh_prefix;
    remaining = sh_remaining;
    mask |= 255u << shift;
  }
  const uint32_t thr = prefix;        // key of the k-th largest element
  const uint32_t need_eq = remaining; // how many elements equal to it are kept (lowest index first)

  // ---- ordered compaction.  Counts of (greater, equal) packed as (g << 16) | e: a row has
  // at most 32768 elements, so neither half overflows.
  uint32_t g = 0, e = 0;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    if (i < nvalid) {
      g += key[i] > thr;
      e += key[i] == thr;
    }
  }
  const uint32_t mine = (g << 16) | e;
  uint32_t incl = mine;                              // inclusive scan inside the wave
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const uint32_t v = __shfl_up(incl, off);
    if (lane >= off) incl += v;
  }
  if (lane == 63) wave_tot[wave] = incl;
  __syncthreads();
  uint32_t before = incl - mine;
  for (int w = 0; w < wave; ++w) before += wave_tot[w];
  const uint32_t gt_before = before >> 16;
  uint32_t eq_before = before & 0xffffu;
  uint32_t pos = gt_before + min(eq_before, need_eq);
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    if (i < nvalid) {
      if (key[i] > thr) {
        out[pos++] = c0 + i;
      } else if (key[i] == thr) {
        if (eq_before < need_eq) out[pos++] = c0 + i;
        ++eq_before;
      }
    }
  }
}

}  // namespace

hipError_t launch_topk_rows(const float* scores, int64_t row_pitch, int num_rows,
                            const int32_t* row_lens, const int32_t* row_ks, int rows_per_entry, int max_len,
                            int32_t* keep, int keep_pitch, hipStream_t s, int groups, int64_t group_stride,
                            int group_max) {
  if (num_rows <= 0) return hipSuccess;
  if (max_len > 0 && max_len <= 8 * kTopkThreads)
    hipLaunchKernelGGL(topk_rows_reg_kernel<8>, dim3(num_rows), dim3(kTopkThreads), 0, s, scores, row_pitch, row_lens,
                       row_ks, rows_per_entry, keep, keep_pitch, max_len, groups, group_stride, group_max);
  else if (max_len > 0 && max_len <= 16 * kTopkThreads)
    hipLaunchKernelGGL(topk_rows_reg_kernel<16>, dim3(num_rows), dim3(kTopkThreads), 0, s, scores, row_pitch, row_lens,
                       row_ks, rows_per_entry, keep, keep_pitch, max_len, groups, group_stride, group_max);
  else if (max_len > 0 && max_len <= 32 * kTopkThreads)
    hipLaunchKernelGGL(topk_rows_reg_kernel<32>, dim3(num_rows), dim3(kTopkThreads), 0, s, scores, row_pitch, row_lens,
                       row_ks, rows_per_entry, keep, keep_pitch, max_len, groups, group_stride, group_max);
  else if (groups > 1)
    return hipErrorInvalidValue;      // rows beyond the register kernels are reduced by the caller first
  else
    hipLaunchKernelGGL(topk_rows_kernel, dim3(num_rows), dim3(kTopkThreads), 0, s, scores, row_pitch, row_lens,
                       row_ks, rows_per_entry, keep, keep_pitch, max_len);
  return hipGetLastError();
}

// Longest row the register top-k kernels take (they can also add partial rows while loading).
int topk_register_row_limit() { return 32 * kTopkThreads; }

__global__ void clear_word_kernel(uint32_t* word) { *word = 0u; }

hipError_t launch_clear_status(uint32_t* status, hipStream_t s) {
  hipLaunchKernelGGL(clear_word_kernel, dim3(1), dim3(1), 0, s, status);
  return hipGetLastError();
}

hipError_t launch_select(const SelectLaunch& a, hipStream_t s) {
  const int n = a.B * a.L * a.A;
  // Whole token rows for the usual layout; the chunk sums ([B][L][chunks of 2048][Hkv][2] doubles) go
  // into scratch the caller names.
  const int chunks = ceil_div(a.Tmax, kGroupStatsChunk);
  const bool rows = a.group_first && a.normalize && a.G == 4 && a.A == a.Hkv * 4 && a.raw_stride_head == 1 &&
                    a.raw_stride_token % 4 == 0 && a.raw_stride_layer % 4 == 0 &&
                    (reinterpret_cast<uintptr_t>(a.raw) % 16) == 0 && a.Hkv <= 128 && (a.Hkv & (a.Hkv - 1)) == 0 &&
                    a.group_scratch != nullptr &&
                    (int64_t)a.B * a.L * chunks * a.Hkv * 16 <= a.group_scratch_bytes;
  if (rows) {
    double* part = a.group_scratch;
    hipLaunchKernelGGL(group_stats_partial_kernel, dim3(chunks, a.B * a.L), dim3(256), 0, s, a.raw, a.raw_stride_layer,
                       a.raw_stride_token, a.seq_lens, a.L, a.Hkv, chunks, a.group_reduce, part);
    hipLaunchKernelGGL(group_stats_finish_kernel, dim3(ceil_div(a.B * a.L * a.Hkv, 256)), dim3(256), 0, s, part,
                       a.seq_lens, a.B * a.L, a.L, a.Hkv, a.A, chunks, a.mustd);
  } else if (a.group_first)
    hipLaunchKernelGGL(group_stats_kernel, dim3(a.B * a.L * a.Hkv), dim3(256), 0, s, a.raw, a.raw_stride_layer,
                       a.raw_stride_token, a.raw_stride_head, a.seq_lens, a.L, a.Hkv, a.A, a.G, a.group_reduce,
                       a.normalize, a.mustd);
  else
    hipLaunchKernelGGL(finalize_stats_kernel, dim3(ceil_div(n, 256)), dim3(256), 0, s, a.partial, a.seq_lens,
                       a.B, a.L, a.A, a.num_tiles, a.normalize, a.mustd);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;

  CombineArgs c{};
  c.raw = a.raw;
  c.mustd = a.mustd;
  c.seq_lens = a.seq_lens;
  c.prefill_lens = a.prefill_lens;
  c.fin = a.fin;
  c.raw_stride_layer = a.raw_stride_layer;
  c.raw_stride_token = a.raw_stride_token;
  c.raw_stride_head = a.raw_stride_head;
  c.B = a.B; c.L = a.L; c.Hkv = a.Hkv; c.A = a.A; c.G = a.G; c.Tmax = a.Tmax;
  c.window_size = a.window_size;
  c.protect_prefill = a.protect_prefill;
  c.group_reduce = a.group_reduce;
  c.layer_reduce = a.layer_reduce;
  c.shared = a.shared;
  c.group_first = a.group_first;
  c.rows_per_seq = a.shared ? 1 : a.Hkv;
  c.tokens_per_wg = 256 / c.rows_per_seq;
  const bool per_layer = a.layer_reduce < 0;
  dim3 grid(ceil_div(a.Tmax, c.tokens_per_wg), per_layer ? a.L : 1, a.B);
  const size_t smem = (size_t)c.rows_per_seq * c.tokens_per_wg * sizeof(float);
  const bool vec = (a.G == 4 || a.G == 8) && a.raw_stride_head == 1 && a.raw_stride_token % 4 == 0 &&
                   a.raw_stride_layer % 4 == 0 && (reinterpret_cast<uintptr_t>(a.raw) % 16) == 0 &&
                   (reinterpret_cast<uintptr_t>(a.mustd) % 16) == 0;
  if (vec && a.G == 4)
    hipLaunchKernelGGL(combine_kernel<1>, grid, dim3(256), smem, s, c);
  else if (vec)
    hipLaunchKernelGGL(combine_kernel<2>, grid, dim3(256), smem, s, c);
  else
    hipLaunchKernelGGL(combine_kernel<0>, grid, dim3(256), smem, s, c);
  e = hipGetLastError();
  if (e != hipSuccess) return e;

  if (!a.keep) return hipSuccess;   // selection scores only
  const int rows_per_entry = c.rows_per_seq * (per_layer ? a.L : 1);
  return launch_topk_rows(a.fin, a.Tmax, a.B * rows_per_entry, a.seq_lens, a.budgets, rows_per_entry, a.Tmax, a.keep,
                          a.max_budget, s);
}

}  // namespace tri
