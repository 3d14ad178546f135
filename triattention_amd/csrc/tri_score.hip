// Fused paged key scorer for gfx950 (wave64).
//
// One key row (D elements of one KV head of one token) is shared by LPH = D/16
// lanes; every lane holds 8 frequency pairs: it loads 16 bytes of real parts and
// 16 bytes of imaginary parts ("half" RoPE layout) or 32 contiguous bytes
// ("interleaved").  The per-pair coefficients of the four query heads a wave pass
// scores live in registers (3 x 8 x 4 floats per lane), so one read of a key
// serves the whole GQA group; the reference instead expands K G-fold and reads it
// per query head (runtime/selector_hf.py:308-312).
//
// Mean aggregation over offsets is linear in cos/sin, so the 17 offsets collapse
// into per-pair coefficients before the kernel runs (launch_prepare):
//   raw = sum_f  k_r*P_f + k_i*R_f + |k_f|*E_f
//   P = s*(q_r*C - q_i*S), R = s*(q_i*C + q_r*S), E = s*(q_abs - |q|),
//   C = mean_j cos(t_j*w_f), S = mean_j sin(t_j*w_f)          (core/scoring.py:290-355)
// Max aggregation keeps the per-offset sums and takes cos/sin tables from LDS.
//
// The sum over a row's pairs is a transposed butterfly on DPP lane permutes: after
// two exchange steps each lane of a quad owns one query head, a half-row mirror
// adds the two quads, so lanes 0-3 / 4-7 of a row hold duplicates; those two quads
// store two different tokens with a single instruction.
#include "tri_common.h"
#include "tri_score_device.h"
#include <cstdlib>
#include <cstring>

namespace tri {
namespace {

struct ScoreArgs {
  const void* const* k_layers;
  const float* const* k_scale_layers;   // fp8 only
  const int32_t* block_table;
  const int32_t* seq_lens;
  const float* coef;
  const float* trig;
  float* partial;
  float* raw;
  int64_t stride_block, stride_token, stride_head;
  int64_t raw_stride_layer, raw_stride_token, raw_stride_head;
  int L, Hkv, A, G, NO;
  int block_size, bs_shift;     // bs_shift >= 0 when block_size is a power of two
  int block_table_pitch;        // < 0: dense, physical block = sequence index
  int num_tiles, QC, Hpad;
};

// Lane geometry shared by the mean and max kernels.
template <int LPH>
struct LaneMap {
  int m, g, head, tsub, tpi, q0, nq, qsel;
  bool b0, b1, store_lane, slot_b;
  __device__ LaneMap(const ScoreArgs& a, int lane, int sib) {
    constexpr int UPW = kWave / LPH;
    m = lane % LPH;
    g = lane / LPH;
    const int hc = sib / a.QC, qc = sib % a.QC;
    if (a.Hpad >= UPW) {
      tpi = 1; tsub = 0; head = hc * UPW + g;
    } else {
      tpi = UPW / a.Hpad; head = g % a.Hpad; tsub = g / a.Hpad;
    }
    const int flip = (LPH >= 8) ? ((m >> 2) & 1) : 0;
    b0 = ((m & 1) ^ flip) != 0;
    b1 = (((m >> 1) & 1) ^ flip) != 0;
    qsel = 2 * (int)b0 + (int)b1;
    q0 = qc * kQPerPass;
    nq = min(kQPerPass, a.G - q0);
    store_lane = (LPH >= 8) ? (m < 8) : true;
    slot_b = (LPH >= 8) && (m >= 4);
  }
};

template <int LPH, int DT, bool IL>
__device__ __forceinline__ RowData load_row(const ScoreArgs& a, const char* kbase, const float* kscale,
                                            int head, int b, int tok, int last_tok, const int* lds_blk,
                                            int lb0, int64_t lane_off_elems) {
  // Rows past the tile are clamped to its last token (loaded, never stored), so
  // every address stays inside the blocks whose ids were staged in LDS.
  const int t = min(tok, last_tok);
  int64_t phys, in_off;
  if (a.block_table_pitch < 0) {
    phys = b; in_off = t;
  } else {
    const int lb = a.bs_shift >= 0 ? (t >> a.bs_shift) : (t / a.block_size);
    phys = lds_blk[lb - lb0];
    in_off = t - lb * a.block_size;
  }
  const int64_t e = phys * a.stride_block + in_off * a.stride_token + lane_off_elems;
  GlobalBytes p = (GlobalBytes)(uintptr_t)kbase + e * elem_size<DT>();
  RowData d;
  d.scale = 1.f;
  if constexpr (DT == TRI_KV_FP8_E4M3) {
    if (IL) {
      const u32x4 lo = *(GlobalU4)(p);
      d.lo = uint4{lo.x, lo.y, lo.z, lo.w};
      d.hi = uint4{0, 0, 0, 0};
    } else {
      const u32x2 lo = *(GlobalU2)(p);
      const u32x2 hi = *(GlobalU2)(p + LPH * 8);
      d.lo = uint4{lo.x, lo.y, 0, 0};
      d.hi = uint4{hi.x, hi.y, 0, 0};
    }
    d.scale = ((GlobalF32)(uintptr_t)kscale)[(phys * a.block_size + in_off) * a.Hkv + head];
  } else {
    const u32x4 lo = *(GlobalU4)(p);
    const u32x4 hi = *(GlobalU4)(p + (IL ? 16 : LPH * 16));
    d.lo = uint4{lo.x, lo.y, lo.z, lo.w};
    d.hi = uint4{hi.x, hi.y, hi.z, hi.w};
  }
  return d;
}

// ------------------------------------------------------------------ mean
// UNI: one token per wave iteration (the KV heads fill the wave's rows) and the tokens
// of a stage share a block (or the keys are dense): scalar addressing, buffer loads.
template <int LPH, int DT, bool IL, int SP, bool UNI>
__global__ __launch_bounds__(kScoreThreads) void score_mean_kernel(ScoreArgs a) {
  constexpr int F = LPH * kPairsPerLane;
  __shared__ int lds_blk[kScoreTileTokens + 2];
  __shared__ float lds_s1[kScoreThreads];
  __shared__ float lds_s2[kScoreThreads];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int tile = blockIdx.x, sib = blockIdx.y;
  const int b = blockIdx.z / a.L, l = blockIdx.z % a.L;
  const int seq_len = a.seq_lens[b];
  const int n0 = tile * kScoreTileTokens;
  if (n0 >= seq_len) return;
  const int n1 = min(n0 + kScoreTileTokens, seq_len);

  int lb0 = 0;
  if (a.block_table_pitch >= 0) {
    lb0 = n0 / a.block_size;
    const int lb1 = (n1 - 1) / a.block_size;
    for (int i = threadIdx.x; i <= lb1 - lb0; i += kScoreThreads)
      lds_blk[i] = a.block_table[(int64_t)b * a.block_table_pitch + lb0 + i];
  }
  __syncthreads();

  const LaneMap<LPH> lm(a, lane, sib);
  const bool head_ok = lm.head < a.Hkv;
  const int head_c = head_ok ? lm.head : 0;

  // Coefficients of the (up to) four query heads of this pass.
  float P[4][8], R[4][8], E[4][8];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const bool ok = head_ok && q < lm.nq;
    const int ah = head_c * a.G + lm.q0 + (q < lm.nq ? q : 0);
    const float* c = a.coef + (((int64_t)(b * a.L + l) * a.A + ah) * 3) * F + lm.m * kPairsPerLane;
#pragma unroll
    for (int v = 0; v < 2; ++v) {
      float4 p4 = ok ? *reinterpret_cast<const float4*>(c + v * 4) : float4{0, 0, 0, 0};
      float4 r4 = ok ? *reinterpret_cast<const float4*>(c + F + v * 4) : float4{0, 0, 0, 0};
      float4 e4 = ok ? *reinterpret_cast<const float4*>(c + 2 * F + v * 4) : float4{0, 0, 0, 0};
      P[q][v * 4 + 0] = p4.x; P[q][v * 4 + 1] = p4.y; P[q][v * 4 + 2] = p4.z; P[q][v * 4 + 3] = p4.w;
      R[q][v * 4 + 0] = r4.x; R[q][v * 4 + 1] = r4.y; R[q][v * 4 + 2] = r4.z; R[q][v * 4 + 3] = r4.w;
      E[q][v * 4 + 0] = e4.x; E[q][v * 4 + 1] = e4.y; E[q][v * 4 + 2] = e4.z; E[q][v * 4 + 3] = e4.w;
    }
  }

  constexpr bool FP8 = DT == TRI_KV_FP8_E4M3;
  constexpr int ES = elem_size<DT>();
  const char* kbase = reinterpret_cast<const char*>(a.k_layers[l]);
  const float* kscale = FP8 ? a.k_scale_layers[l] : nullptr;
  const int64_t lane_off = (int64_t)head_c * a.stride_head + (IL ? lm.m * 16 : lm.m * 8);
  const uint32_t lane_off_bytes = (uint32_t)(lane_off * ES);

  // This wave's tokens: a quarter of the tile, walked in stages of SP token pairs.
  constexpr int TW = kScoreTileTokens / 4;
  const int wstart = n0 + wave * TW;
  const int wend = min(wstart + TW, n1);
  const int tok_per_pair = UNI ? 2 : 2 * lm.tpi;
  const int tok_per_stage = SP * tok_per_pair;

  const int a_out = head_c * a.G + lm.q0 + lm.qsel;
  const bool out_ok = head_ok && lm.store_lane && lm.qsel < lm.nq;
  float* raw_bl = a.raw + (int64_t)(b * a.L + l) * a.raw_stride_layer;
  float* raw_row = raw_bl + (int64_t)a_out * a.raw_stride_head;
  // UNI: per-lane element offset from the (scalar) address of token A's row.
  const uint32_t store_off = (uint32_t)((int64_t)a_out * a.raw_stride_head + (lm.slot_b ? a.raw_stride_token : 0));
  const bool out_ok_a = out_ok && !lm.slot_b;   // lanes that store when token B is out of range

  float s1 = 0.f, s2 = 0.f;

  const int last_tok = n1 - 1;
  const uint32_t tok_bytes = (uint32_t)(a.stride_token * ES);
  const uint32_t scale_tok_bytes = (uint32_t)a.Hkv * 4u;
  auto load_stage = [&](RowData (&buf)[SP][2], int base) {
    if (UNI) {
      // Rows past the tile are clamped to its last token (loaded, never stored).
      const int t0 = min(base, last_tok);
      int64_t row_elems, slot;
      if (a.block_table_pitch < 0) {
        row_elems = (int64_t)b * a.stride_block + (int64_t)t0 * a.stride_token;
        slot = (int64_t)b * a.block_size + t0;
      } else {
        const int lb = t0 >> a.bs_shift;
        const int64_t phys = __builtin_amdgcn_readfirstlane(lds_blk[lb - lb0]);
        row_elems = phys * a.stride_block + (int64_t)(t0 - (lb << a.bs_shift)) * a.stride_token;
        slot = phys * a.block_size + (t0 - (lb << a.bs_shift));
      }
      const __amdgpu_buffer_rsrc_t rsrc =
          __builtin_amdgcn_make_buffer_rsrc((void*)(kbase + row_elems * ES), 0, 0x7fffffff, 0x00020000);
      __amdgpu_buffer_rsrc_t srsrc = rsrc;
      if constexpr (FP8)
        srsrc = __builtin_amdgcn_make_buffer_rsrc((void*)(kscale + slot * a.Hkv), 0, 0x7fffffff, 0x00020000);
#pragma unroll
      for (int p = 0; p < SP; ++p) {
#pragma unroll
        for (int r = 0; r < 2; ++r) {
          const uint32_t dt = (uint32_t)(min(base + p * 2 + r, last_tok) - t0);
          const uint32_t soff = dt * tok_bytes;
          if constexpr (FP8) {
            if (IL) {
              buf[p][r].lo = buffer_load16(rsrc, lane_off_bytes, soff);
              buf[p][r].hi = uint4{0, 0, 0, 0};
            } else {
              buf[p][r].lo = buffer_load8(rsrc, lane_off_bytes, soff);
              buf[p][r].hi = buffer_load8(rsrc, lane_off_bytes + LPH * 8, soff);
            }
            buf[p][r].scale = buffer_load_f32(srsrc, (uint32_t)head_c * 4u, dt * scale_tok_bytes);
          } else {
            buf[p][r].lo = buffer_load16(rsrc, lane_off_bytes, soff);
            buf[p][r].hi = buffer_load16(rsrc, lane_off_bytes + (IL ? 16 : LPH * 16), soff);
          }
        }
      }
    } else {
#pragma unroll
      for (int p = 0; p < SP; ++p) {
        const int ta = base + p * tok_per_pair + lm.tsub;
        buf[p][0] = load_row<LPH, DT, IL>(a, kbase, kscale, head_c, b, ta, last_tok, lds_blk, lb0, lane_off);
        buf[p][1] = load_row<LPH, DT, IL>(a, kbase, kscale, head_c, b, ta + lm.tpi, last_tok, lds_blk, lb0, lane_off);
      }
    }
  };

  auto score_row = [&](const RowData& d) -> float {
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int p = 0; p < 8; ++p) {
      float kr, ki;
      unpack_pair<DT, IL>(d, p, kr, ki);
      const float mag = __builtin_amdgcn_sqrtf(fmaf(ki, ki, kr * kr));
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        acc[q] = fmaf(kr, P[q][p], acc[q]);
        acc[q] = fmaf(ki, R[q][p], acc[q]);
        acc[q] = fmaf(mag, E[q][p], acc[q]);
      }
    }
    const float r = reduce_row<LPH>(acc, lm.b0, lm.b1);
    return FP8 ? r * d.scale : r;
  };

  auto compute_stage = [&](const RowData (&buf)[SP][2], int base) {
#pragma unroll
    for (int p = 0; p < SP; ++p) {
      const float ra = score_row(buf[p][0]);
      const float rb = score_row(buf[p][1]);
      if (UNI && LPH >= 8) {
        // Token A = base + 2p (uniform), token B the next one: quad 0 stores A, quad 1 stores B.
        const int ta = base + p * 2;
        if (ta < wend) {
          const float v = lm.slot_b ? rb : ra;
          float* row = raw_bl + (int64_t)ta * a.raw_stride_token;
          const bool ok = (ta + 1 < wend) ? out_ok : out_ok_a;
          if (ok) {
            row[store_off] = v;
            s1 += v;
            s2 = fmaf(v, v, s2);
          }
        }
        continue;
      }
      const int ta = base + p * tok_per_pair + lm.tsub;
      const int tb = ta + lm.tpi;
      if (LPH >= 8) {
        const float v = lm.slot_b ? rb : ra;
        const int t = lm.slot_b ? tb : ta;
        if (out_ok && t < wend) {
          raw_row[(int64_t)t * a.raw_stride_token] = v;
          s1 += v;
          s2 = fmaf(v, v, s2);
        }
      } else {
        if (out_ok && ta < wend) {
          raw_row[(int64_t)ta * a.raw_stride_token] = ra;
          s1 += ra;
          s2 = fmaf(ra, ra, s2);
        }
        if (out_ok && tb < wend) {
          raw_row[(int64_t)tb * a.raw_stride_token] = rb;
          s1 += rb;
          s2 = fmaf(rb, rb, s2);
        }
      }
    }
  };

  if (wstart < wend) {
    RowData buf_a[SP][2], buf_b[SP][2];
    int base = wstart;
    load_stage(buf_a, base);
    while (base < wend) {
      load_stage(buf_b, base + tok_per_stage);
      compute_stage(buf_a, base);
      base += tok_per_stage;
      if (base >= wend) break;
      load_stage(buf_a, base + tok_per_stage);
      compute_stage(buf_b, base);
      base += tok_per_stage;
    }
  }

  // Per-tile sum and sum of squares of every (head, query head) of this pass, in
  // a fixed order so that the statistics are reproducible run to run.
  lds_s1[threadIdx.x] = s1;
  lds_s2[threadIdx.x] = s2;
  __syncthreads();
  constexpr int UPW = kWave / LPH;
  const int heads_here = (a.Hpad >= UPW) ? UPW : a.Hpad;
  const int tpi = (a.Hpad >= UPW) ? 1 : UPW / a.Hpad;
  if ((int)threadIdx.x < heads_here * kQPerPass) {
    const int hl = threadIdx.x / kQPerPass, q = threadIdx.x % kQPerPass;
    const int hc = sib / a.QC, qc = sib % a.QC;
    const int head = (a.Hpad >= UPW) ? hc * UPW + hl : hl;
    const int qq = qc * kQPerPass + q;
    if (head < a.Hkv && qq < a.G) {
      const int ma = (q >> 1) | ((q & 1) << 1);                           // token-A lane of q
      const int mb = 4 + (1 - (q >> 1)) + 2 * (1 - (q & 1));              // token-B lane of q
      float t1 = 0.f, t2 = 0.f;
      for (int w = 0; w < 4; ++w)
        for (int ts = 0; ts < tpi; ++ts) {
          const int g = ts * heads_here + hl;
          const int la = w * kWave + g * LPH + ma;
          t1 += lds_s1[la];
          t2 += lds_s2[la];
          if (LPH >= 8) {
            const int lb = w * kWave + g * LPH + mb;
            t1 += lds_s1[lb];
            t2 += lds_s2[lb];
          }
        }
      float* out = a.partial + (((int64_t)(b * a.L + l) * a.num_tiles + tile) * a.A + head * a.G + qq) * 2;
      out[0] = t1;
      out[1] = t2;
    }
  }
}

// ------------------------------------------------------------------- max
// Per-offset sums, max over offsets (core/scoring.py:338-339).  Not the default
// setting; written for correctness, not tuned.
template <int LPH, int DT, bool IL>
__global__ __launch_bounds__(kScoreThreads) void score_max_kernel(ScoreArgs a) {
  constexpr int F = LPH * kPairsPerLane;
  __shared__ int lds_blk[kScoreTileTokens + 2];
  __shared__ float lds_s1[kScoreThreads];
  __shared__ float lds_s2[kScoreThreads];
  __shared__ float lds_cos[kMaxOffsets * F];
  __shared__ float lds_sin[kMaxOffsets * F];

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int tile = blockIdx.x, sib = blockIdx.y;
  const int b = blockIdx.z / a.L, l = blockIdx.z % a.L;
  const int seq_len = a.seq_lens[b];
  const int n0 = tile * kScoreTileTokens;
  if (n0 >= seq_len) return;
  const int n1 = min(n0 + kScoreTileTokens, seq_len);

  int lb0 = 0;
  if (a.block_table_pitch >= 0) {
    lb0 = n0 / a.block_size;
    const int lb1 = (n1 - 1) / a.block_size;
    for (int i = threadIdx.x; i <= lb1 - lb0; i += kScoreThreads)
      lds_blk[i] = a.block_table[(int64_t)b * a.block_table_pitch + lb0 + i];
  }
  for (int i = threadIdx.x; i < a.NO * F; i += kScoreThreads) {
    const int j = i / F, f = i % F;
    lds_cos[i] = a.trig[((int64_t)(b * a.NO + j) * 2 + 0) * F + f];
    lds_sin[i] = a.trig[((int64_t)(b * a.NO + j) * 2 + 1) * F + f];
  }
  __syncthreads();

  const LaneMap<LPH> lm(a, lane, sib);
  const bool head_ok = lm.head < a.Hkv;
  const int head_c = head_ok ? lm.head : 0;

  float A1[4][8], A2[4][8], E[4][8];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const bool ok = head_ok && q < lm.nq;
    const int ah = head_c * a.G + lm.q0 + (q < lm.nq ? q : 0);
    const float* c = a.coef + (((int64_t)(b * a.L + l) * a.A + ah) * 3) * F + lm.m * kPairsPerLane;
#pragma unroll
    for (int p = 0; p < 8; ++p) {
      A1[q][p] = ok ? c[p] : 0.f;
      A2[q][p] = ok ? c[F + p] : 0.f;
      E[q][p] = ok ? c[2 * F + p] : 0.f;
    }
  }

  constexpr bool FP8 = DT == TRI_KV_FP8_E4M3;
  const char* kbase = reinterpret_cast<const char*>(a.k_layers[l]);
  const float* kscale = FP8 ? a.k_scale_layers[l] : nullptr;
  const int64_t lane_off = (int64_t)head_c * a.stride_head + (IL ? lm.m * 16 : lm.m * 8);
  constexpr int TW = kScoreTileTokens / 4;
  const int wstart = n0 + wave * TW;
  const int wend = min(wstart + TW, n1);
  const int a_out = head_c * a.G + lm.q0 + lm.qsel;
  const bool out_ok = head_ok && lm.store_lane && lm.qsel < lm.nq;
  float* raw_row = a.raw + (int64_t)(b * a.L + l) * a.raw_stride_layer + (int64_t)a_out * a.raw_stride_head;
  float s1 = 0.f, s2 = 0.f;

  auto score_row = [&](const RowData& d) -> float {
    float kr[8], ki[8], ext[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int p = 0; p < 8; ++p) {
      unpack_pair<DT, IL>(d, p, kr[p], ki[p]);
      const float mag = __builtin_amdgcn_sqrtf(fmaf(ki[p], ki[p], kr[p] * kr[p]));
#pragma unroll
      for (int q = 0; q < 4; ++q) ext[q] = fmaf(mag, E[q][p], ext[q]);
    }
    const float extra = reduce_row<LPH>(ext, lm.b0, lm.b1);
    float best = -INFINITY;
    for (int j = 0; j < a.NO; ++j) {
      float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int p = 0; p < 8; ++p) {
        const float c = lds_cos[j * F + lm.m * kPairsPerLane + p];
        const float s = lds_sin[j * F + lm.m * kPairsPerLane + p];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float pa = fmaf(A1[q][p], kr[p], A2[q][p] * ki[p]);   // s*Re(q conj k)
          const float pb = fmaf(A2[q][p], kr[p], -A1[q][p] * ki[p]);  // s*Im(q conj k)
          acc[q] = fmaf(pa, c, acc[q]);
          acc[q] = fmaf(-pb, s, acc[q]);
        }
      }
      best = fmaxf(best, reduce_row<LPH>(acc, lm.b0, lm.b1));
    }
    return FP8 ? (best + extra) * d.scale : best + extra;
  };

  const int step = 2 * lm.tpi;
  for (int base = wstart; base < wend; base += step) {
    const int ta = base + lm.tsub, tb = ta + lm.tpi;
    const RowData da = load_row<LPH, DT, IL>(a, kbase, kscale, head_c, b, ta, n1 - 1, lds_blk, lb0, lane_off);
    const RowData db = load_row<LPH, DT, IL>(a, kbase, kscale, head_c, b, tb, n1 - 1, lds_blk, lb0, lane_off);
    const float ra = score_row(da);
    const float rb = score_row(db);
    if (LPH >= 8) {
      const float v = lm.slot_b ? rb : ra;
      const int t = lm.slot_b ? tb : ta;
      if (out_ok && t < wend) {
        raw_row[(int64_t)t * a.raw_stride_token] = v;
        s1 += v; s2 = fmaf(v, v, s2);
      }
    } else {
      if (out_ok && ta < wend) { raw_row[(int64_t)ta * a.raw_stride_token] = ra; s1 += ra; s2 = fmaf(ra, ra, s2); }
      if (out_ok && tb < wend) { raw_row[(int64_t)tb * a.raw_stride_token] = rb; s1 += rb; s2 = fmaf(rb, rb, s2); }
    }
  }

  lds_s1[threadIdx.x] = s1;
  lds_s2[threadIdx.x] = s2;
  __syncthreads();
  constexpr int UPW = kWave / LPH;
  const int heads_here = (a.Hpad >= UPW) ? UPW : a.Hpad;
  const int tpi = (a.Hpad >= UPW) ? 1 : UPW / a.Hpad;
  if ((int)threadIdx.x < heads_here * kQPerPass) {
    const int hl = threadIdx.x / kQPerPass, q = threadIdx.x % kQPerPass;
    const int hc = sib / a.QC, qc = sib % a.QC;
    const int head = (a.Hpad >= UPW) ? hc * UPW + hl : hl;
    const int qq = qc * kQPerPass + q;
    if (head < a.Hkv && qq < a.G) {
      const int ma = (q >> 1) | ((q & 1) << 1);
      const int mb = 4 + (1 - (q >> 1)) + 2 * (1 - (q & 1));
      float t1 = 0.f, t2 = 0.f;
      for (int w = 0; w < 4; ++w)
        for (int ts = 0; ts < tpi; ++ts) {
          const int g = ts * heads_here + hl;
          t1 += lds_s1[w * kWave + g * LPH + ma];
          t2 += lds_s2[w * kWave + g * LPH + ma];
          if (LPH >= 8) {
            t1 += lds_s1[w * kWave + g * LPH + mb];
            t2 += lds_s2[w * kWave + g * LPH + mb];
          }
        }
      float* out = a.partial + (((int64_t)(b * a.L + l) * a.num_tiles + tile) * a.A + head * a.G + qq) * 2;
      out[0] = t1;
      out[1] = t2;
    }
  }
}

// ------------------------------------------------------- max, matrix cores
// The same scores as score_max_kernel for two-byte bf16 keys with a head dimension of 128, as
// a matrix product: per offset j the sum over the pairs is linear in the key,
//   raw_j = sum_f kr_f (A1_f cos_jf - A2_f sin_jf) + ki_f (A2_f cos_jf + A1_f sin_jf),
// so 16 tokens x 128 key elements times 128 x (query heads x offsets) coefficients gives every
// per-offset sum of a step (v_mfma_f32_16x16x32_bf16; the keys are exact in bf16, a
// coefficient enters as three bf16 pieces accumulated into the same column).  Column tile q
// (of four) holds offsets 0..15 of the workgroup's query head q, so the maximum over them is
// a maximum over the 16 lanes of a row group; offsets from 16 on sit in NX further tiles as
// column 4 (j - 16) + q, four lanes apart per head.  The magnitude term goes through the
// matrix cores too: |k_f| in two bf16 pieces times E in three pieces, one piece per column
// group.  A workgroup builds its operand slabs in LDS from the per-sequence tables (60 KB
// for 17 offsets), then each wave takes 16 tokens a step.  Outputs as score_max_kernel: raw
// rows and per-tile sums.
typedef __bf16 mx_bf16x8 __attribute__((ext_vector_type(8)));
typedef float mx_f32x4 __attribute__((ext_vector_type(4)));
constexpr int kDppRor4 = 0x124;        // row_ror:4

__device__ __forceinline__ mx_f32x4 mx_mfma(const uint4& a, const uint4& b, mx_f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(mx_bf16x8, a), __builtin_bit_cast(mx_bf16x8, b), c, 0, 0, 0);
}
__device__ __forceinline__ uint32_t bf16_bits(float x) {
  return (uint32_t)__builtin_bit_cast(unsigned short, (__bf16)x);
}
// x = p[0] + p[1] + p[2] up to 24 bits: each piece is what bf16 holds of the remainder.
__device__ __forceinline__ void bf16_pieces(float x, uint32_t (&p)[3]) {
#pragma unroll
  for (int i = 0; i < 3; ++i) {
    p[i] = bf16_bits(x);
    x -= __uint_as_float(p[i] << 16);
  }
}
__device__ __forceinline__ float bf16_elem(const uint4& v, int e) {   // e: compile-time
  const uint32_t w = e < 2 ? v.x : e < 4 ? v.y : e < 6 ? v.z : v.w;
  return (e & 1) ? __uint_as_float(w & 0xffff0000u) : __uint_as_float(w << 16);
}

// max(keep, send of the lane `lane ^ 1` / `^ 2` / `^ 4` / `^ 8` of the row of 16): one instruction (two
// for ^ 4, which no single lane pattern of this chip expresses).  Written out because the compiler puts a
// quieting v_max in front of every operand of fmaxf and moves the other lane's value into a register
// first; the idle cycles cover the distance this chip requires between a vector instruction's write and a
// lane-crossing read of that register.
__device__ __forceinline__ float max_xor1(float keep, float send) {
  float r;
  asm("s_nop 1\n\tv_max_f32_dpp %0, %1, %2 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf" : "=v"(r) : "v"(send), "v"(keep));
  return r;
}
__device__ __forceinline__ float max_xor2(float keep, float send) {
  float r;
  asm("s_nop 1\n\tv_max_f32_dpp %0, %1, %2 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf" : "=v"(r) : "v"(send), "v"(keep));
  return r;
}
__device__ __forceinline__ float max_xor4(float keep, float send) {
  float r = keep;      // lanes 0..3 and 8..11 of a row take lane + 4, the others lane - 4
  asm("s_nop 1\n\tv_max_f32_dpp %0, %1, %0 row_ror:12 row_mask:0xf bank_mask:0x5\n\t"
      "v_max_f32_dpp %0, %1, %0 row_ror:4 row_mask:0xf bank_mask:0xa" : "+v"(r) : "v"(send));
  return r;
}
__device__ __forceinline__ float max_xor8(float keep, float send) {
  float r;
  asm("s_nop 1\n\tv_max_f32_dpp %0, %1, %2 row_ror:8 row_mask:0xf bank_mask:0xf" : "=v"(r) : "v"(send), "v"(keep));
  return r;
}
__device__ __forceinline__ float max_plain(float a, float b) {
  float r;
  asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}
// m[i] = sqrt(x[i].lo^2 + x[i].hi^2) for four packed bf16 pairs (see magnitudes4 of the resident kernel:
// the spacing this chip requires after a dot product's and a transcendental's write is provided here).
__device__ __forceinline__ void pair_magnitudes4(const uint32_t (&x)[4], float* m) {
  asm("v_dot2_f32_bf16 %0, %4, %4, 0\n\t"
      "v_dot2_f32_bf16 %1, %5, %5, 0\n\t"
      "v_dot2_f32_bf16 %2, %6, %6, 0\n\t"
      "v_dot2_f32_bf16 %3, %7, %7, 0\n\t"
      "v_sqrt_f32 %0, %0\n\t"
      "v_sqrt_f32 %1, %1\n\t"
      "v_sqrt_f32 %2, %2\n\t"
      "v_sqrt_f32 %3, %3\n\t"
      "s_nop 0"
      : "=&v"(m[0]), "=&v"(m[1]), "=&v"(m[2]), "=&v"(m[3])
      : "v"(x[0]), "v"(x[1]), "v"(x[2]), "v"(x[3]));
}
typedef __bf16 mx_bf16x2 __attribute__((ext_vector_type(2)));
typedef float mx_f32x2 __attribute__((ext_vector_type(2)));
// Two fp32 values as packed bf16 and what is left of them as packed bf16 (16 bits of each value).
__device__ __forceinline__ void split_pair_bf16(float x0, float x1, uint32_t& hi, uint32_t& lo) {
  const mx_f32x2 x = {x0, x1};
  hi = __builtin_bit_cast(uint32_t, __builtin_convertvector(x, mx_bf16x2));
  const mx_f32x2 r = {x0 - __uint_as_float(hi << 16), x1 - __uint_as_float(hi & 0xffff0000u)};
  lo = __builtin_bit_cast(uint32_t, __builtin_convertvector(r, mx_bf16x2));
}

constexpr int kMaxMfmaHeads = 4;   // query heads of one KV head per workgroup
constexpr int kMaxMfmaTilesPerGroup = 8;   // consecutive 512-token tiles per workgroup
// Waves of a workgroup (they share the operand slabs in LDS; two workgroups fit a CU).  Eight waves, four
// per SIMD in 128 registers, run no faster (6.84 against 6.85 ms on 16 x 16384 tokens x 36 layers).
constexpr int kMaxMfmaWaves = 4;
constexpr int kMaxMfmaThreads = kMaxMfmaWaves * 64;
constexpr int kTrigPitch = 65;     // floats per offset in LDS (odd: 16 offsets read at once fall into 16 banks)
__host__ __device__ constexpr size_t max_mfma_lds_bytes(int nx, int no) {
  return (size_t)(kMaxMfmaHeads + nx) * 12 * 64 * 16 + 2 * 64 * 16 + 3 * kMaxMfmaHeads * 64 * 4 +
         (size_t)2 * no * kTrigPitch * 4 + (kScoreTileTokens + 2) * 4 + kMaxMfmaWaves * kMaxMfmaHeads * 2 * 4;
}

template <int NX, bool IL>
__global__ __launch_bounds__(kMaxMfmaThreads) __attribute__((amdgpu_waves_per_eu(kMaxMfmaWaves / 2, kMaxMfmaWaves / 2)))
void score_max_mfma_kernel(ScoreArgs a) {
  constexpr int F = 64;
  constexpr int NT = kMaxMfmaHeads + NX;
  extern __shared__ __align__(16) char max_mfma_lds[];
  uint4* Bk = reinterpret_cast<uint4*>(max_mfma_lds);          // [NT][4 key slabs][3 pieces][64 lanes]
  uint4* Bm = Bk + NT * 12 * 64;                               // [2 magnitude slabs][64 lanes]
  float* cf = reinterpret_cast<float*>(Bm + 2 * 64);           // [A1 | A2 | E][4 query heads][F]
  float* tcos = cf + 3 * kMaxMfmaHeads * F;                    // [NO][kTrigPitch]
  float* tsin = tcos + a.NO * kTrigPitch;                      // [NO][kTrigPitch]
  int* lds_blk = reinterpret_cast<int*>(tsin + a.NO * kTrigPitch);   // [kScoreTileTokens + 2]
  float* red = reinterpret_cast<float*>(lds_blk + kScoreTileTokens + 2);   // [waves][4 heads][2]

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int head = blockIdx.y / a.QC, qc = blockIdx.y % a.QC;
  const int tile_group = blockIdx.x;
  const int q0 = qc * kMaxMfmaHeads, nq = min(kMaxMfmaHeads, a.G - q0);
  const int b = blockIdx.z / a.L, l = blockIdx.z % a.L;
  const int seq_len = a.seq_lens[b];
  // The operand slabs depend on (sequence, layer, KV head, group of query heads) only: a workgroup
  // builds them once (as many vector instructions as scoring 400 tokens) and then takes
  // kMaxMfmaTilesPerGroup consecutive tiles of 512 tokens.
  if (tile_group * kMaxMfmaTilesPerGroup * kScoreTileTokens >= seq_len) return;

  for (int i = threadIdx.x; i < 3 * kMaxMfmaHeads * F; i += kMaxMfmaThreads) {
    const int which = i / (kMaxMfmaHeads * F), q = (i / F) % kMaxMfmaHeads, f = i % F;
    const int ah = head * a.G + q0 + min(q, nq - 1);
    cf[i] = q < nq ? a.coef[(((int64_t)(b * a.L + l) * a.A + ah) * 3 + which) * F + f] : 0.f;
  }
  for (int i = threadIdx.x; i < a.NO * F; i += kMaxMfmaThreads) {
    const int j = i / F, f = i % F;
    tcos[j * kTrigPitch + f] = a.trig[((int64_t)(b * a.NO + j) * 2 + 0) * F + f];
    tsin[j * kTrigPitch + f] = a.trig[((int64_t)(b * a.NO + j) * 2 + 1) * F + f];
  }
  __syncthreads();

  // Operand slabs.  Lane (c16 = lane % 16, kb = lane / 16) of slab (t, s) holds one column
  // and key elements 32 s + 8 kb + 0..7; the column is (head t, offset c16) in the first
  // four tiles and (head c16 % 4, offset 16 + 4 (t - 4) + c16 / 4) in the others.
  for (int i = threadIdx.x; i < NT * 4 * 64; i += kMaxMfmaThreads) {
    const int ln = i & 63, sl = (i >> 6) & 3, t = i >> 8;
    const int c16 = ln & 15, kb = ln >> 4;
    const int q = t < kMaxMfmaHeads ? t : (c16 & 3);
    const int j = t < kMaxMfmaHeads ? c16 : 16 + 4 * (t - kMaxMfmaHeads) + (c16 >> 2);
    // A column beyond the last offset repeats a live one of the same head (the first, or in the
    // further tiles the last), so that the maxima below need no masks.
    const bool live = q < nq;
    const int jc = j < a.NO ? j : (t < kMaxMfmaHeads ? 0 : a.NO - 1);
    uint32_t w[3][4];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int d = 32 * sl + 8 * kb + e;
      const int f = IL ? (d >> 1) : (d & 63);
      const bool im = IL ? (d & 1) != 0 : d >= 64;
      const float a1 = cf[(0 * kMaxMfmaHeads + q) * F + f], a2 = cf[(1 * kMaxMfmaHeads + q) * F + f];
      const float cs = tcos[jc * kTrigPitch + f], sn = tsin[jc * kTrigPitch + f];
      float x = im ? fmaf(a2, cs, a1 * sn) : fmaf(a1, cs, -(a2 * sn));
      if (!live) x = 0.f;
      uint32_t pc[3];
      bf16_pieces(x, pc);
#pragma unroll
      for (int p = 0; p < 3; ++p) {
        if (e & 1) w[p][e >> 1] |= pc[p] << 16;
        else w[p][e >> 1] = pc[p];
      }
    }
#pragma unroll
    for (int p = 0; p < 3; ++p) Bk[((t * 4 + sl) * 3 + p) * 64 + ln] = uint4{w[p][0], w[p][1], w[p][2], w[p][3]};
  }
  // Magnitude slabs: column c16 = query head (c16 % 4), piece (c16 / 4) of E; element e of slab
  // m is the pair whose magnitude the same lane forms from its key registers below.
  for (int i = threadIdx.x; i < 2 * 64; i += kMaxMfmaThreads) {
    const int ln = i & 63, m = i >> 6;
    const int c16 = ln & 15, kb = ln >> 4;
    const int q = c16 & 3, piece = c16 >> 2;
    const bool live = piece < 3 && q < nq;
    uint32_t w[4];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int f = IL ? 16 * (2 * m + (e >> 2)) + 4 * kb + (e & 3) : 32 * m + 8 * kb + e;
      uint32_t pc[3];
      bf16_pieces(live ? cf[(2 * kMaxMfmaHeads + q) * F + f] : 0.f, pc);
      const uint32_t v = piece == 0 ? pc[0] : piece == 1 ? pc[1] : pc[2];
      if (e & 1) w[e >> 1] |= v << 16;
      else w[e >> 1] = v;
    }
    Bm[m * 64 + ln] = uint4{w[0], w[1], w[2], w[3]};
  }

  const int r16 = lane & 15, kb = lane >> 4;
  const bool b0 = (r16 & 1) != 0, b1 = (r16 & 2) != 0, b2 = (r16 & 4) != 0, b3 = (r16 & 8) != 0;
  // After the maxima lane r16 of a row group holds the score of query head r16 % 4 and of the group's
  // token r16 / 4: every lane stores one score.
  const int out_q = r16 & 3, out_i = r16 >> 2;
  const bool far_spread = a.NO > 17;            // more than one offset beyond the first 16: they sit in different lanes
  const char* kbase = reinterpret_cast<const char*>(a.k_layers[l]);
  const int64_t lane_off = (int64_t)head * a.stride_head + 8 * kb;
  constexpr int TW = kScoreTileTokens / kMaxMfmaWaves;
  const bool out_lane = out_q < nq;
  float* raw_row = a.raw + (int64_t)(b * a.L + l) * a.raw_stride_layer +
                   (int64_t)(head * a.G + q0 + (out_lane ? out_q : 0)) * a.raw_stride_head;

  for (int tile = tile_group * kMaxMfmaTilesPerGroup; tile < (tile_group + 1) * kMaxMfmaTilesPerGroup; ++tile) {
  const int n0 = tile * kScoreTileTokens;
  if (n0 >= seq_len) break;                     // (the same for every thread of the workgroup)
  const int n1 = min(n0 + kScoreTileTokens, seq_len);
  __syncthreads();                              // slabs built; the previous tile's block ids and sums read
  int lb0 = 0;
  if (a.block_table_pitch >= 0) {
    lb0 = n0 / a.block_size;
    const int lb1 = (n1 - 1) / a.block_size;
    for (int i = threadIdx.x; i <= lb1 - lb0; i += kMaxMfmaThreads)
      lds_blk[i] = a.block_table[(int64_t)b * a.block_table_pitch + lb0 + i];
    __syncthreads();
  }
  const int wstart = n0 + wave * TW;
  const int wend = min(wstart + TW, n1);
  float s1 = 0.f, s2 = 0.f;

  // Row lane % 16 of the step that starts at token t0: four 16-byte pieces, one per key slab.
  // Rows past the tile are clamped to its last token (loaded, never stored).
  auto load_step = [&](int t0, uint4 (&A)[4]) __attribute__((always_inline)) {
    const int t = min(t0 + r16, n1 - 1);
    int64_t phys, in_off;
    if (a.block_table_pitch < 0) {
      phys = b; in_off = t;
    } else {
      const int lb = a.bs_shift >= 0 ? (t >> a.bs_shift) : (t / a.block_size);
      phys = lds_blk[lb - lb0];
      in_off = t - lb * a.block_size;
    }
    const int64_t e = phys * a.stride_block + in_off * a.stride_token + lane_off;
    GlobalBytes p = (GlobalBytes)(uintptr_t)kbase + e * 2;
#pragma unroll
    for (int sl = 0; sl < 4; ++sl) {
      const u32x4 v = *(GlobalU4)(p + sl * 64);
      A[sl] = uint4{v.x, v.y, v.z, v.w};
    }
  };

  // What follows the key products of one 16-token step: magnitude term, maxima, stores.
  auto finish = [&](const uint4 (&A)[4], mx_f32x4 (&acc)[NT], int t0) __attribute__((always_inline)) {
    // Magnitudes of this lane's 16 pairs (dot product of the bf16 pair with itself, square root) as
    // two bf16 pieces each.
    mx_f32x4 accm = mx_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int m = 0; m < 2; ++m) {
      float mag[8];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        uint32_t x[4];
        if (IL) {
          const uint4& v = A[2 * m + h];
          x[0] = v.x; x[1] = v.y; x[2] = v.z; x[3] = v.w;
        } else {
          const uint32_t re[2] = {h ? A[m].z : A[m].x, h ? A[m].w : A[m].y};
          const uint32_t im[2] = {h ? A[m + 2].z : A[m + 2].x, h ? A[m + 2].w : A[m + 2].y};
#pragma unroll
          for (int i = 0; i < 2; ++i) {
            x[2 * i] = __builtin_amdgcn_perm(im[i], re[i], 0x05040100u);
            x[2 * i + 1] = __builtin_amdgcn_perm(im[i], re[i], 0x07060302u);
          }
        }
        pair_magnitudes4(x, &mag[4 * h]);
      }
      uint32_t hi[4], lo[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) split_pair_bf16(mag[2 * i], mag[2 * i + 1], hi[i], lo[i]);
      const uint4 bm = Bm[m * 64 + lane];
      accm = mx_mfma(uint4{lo[0], lo[1], lo[2], lo[3]}, bm, accm);
      accm = mx_mfma(uint4{hi[0], hi[1], hi[2], hi[3]}, bm, accm);
    }

    // Offsets 0..15 of head q are the 16 lanes of a row group in tile q: 16 values per lane (4 heads x 4
    // tokens), each to be maximised over the 16 lanes.  A transposed butterfly: at every stage a lane
    // keeps half of its values and hands the other half to the lane one bit away, so the 16 + 8 + 4 + 2
    // values shrink to the one of (head r16 % 4, token r16 / 4) in 15 exchanges.
    float u[2][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int p = 0; p < 2; ++p) {
        const float x = acc[2 * p][i], y = acc[2 * p + 1][i];
        u[p][i] = max_xor1(b0 ? y : x, b0 ? x : y);
      }
    float v4[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) v4[i] = max_xor2(b1 ? u[1][i] : u[0][i], b1 ? u[0][i] : u[1][i]);
    float w2[2];
#pragma unroll
    for (int p = 0; p < 2; ++p) w2[p] = max_xor4(b2 ? v4[2 * p + 1] : v4[2 * p], b2 ? v4[2 * p] : v4[2 * p + 1]);
    float best = max_xor8(b3 ? w2[1] : w2[0], b3 ? w2[0] : w2[1]);

    // Offsets from 16 on: the further tiles hold them as column 4 (j - 16) + head, i.e. this lane's head
    // already; the maximum over the tiles, then (more than one such offset) over the four lanes of the head.
    if constexpr (NX > 0) {
      float f[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float v = acc[kMaxMfmaHeads][i];
#pragma unroll
        for (int x = 1; x < NX; ++x) v = max_plain(v, acc[kMaxMfmaHeads + x][i]);
        f[i] = v;
      }
      float v = b3 ? (b2 ? f[3] : f[2]) : (b2 ? f[1] : f[0]);
      if (far_spread) {
        // every lane of the head needs the maximum of token out_i over the head's four lanes, which
        // hold different tokens' selections: reduce all four tokens, then select
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          f[i] = max_xor4(f[i], f[i]);
          f[i] = max_xor8(f[i], f[i]);
        }
        v = b3 ? (b2 ? f[3] : f[2]) : (b2 ? f[1] : f[0]);
      }
      best = max_plain(best, v);
    }
    // Magnitude term: the three pieces of E sit four lanes apart (column group 3 is zero).
    float ex[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float x = accm[i];
      x += dpp<kDppRor4>(x);
      x += dpp<kDppRor8>(x);
      ex[i] = x;
    }
    const float v = best + (b3 ? (b2 ? ex[3] : ex[2]) : (b2 ? ex[1] : ex[0]));
    const int tk = t0 + 4 * kb + out_i;
    if (out_lane && tk < wend) {
      raw_row[(int64_t)tk * a.raw_stride_token] = v;
      s1 += v;
      s2 = fmaf(v, v, s2);
    }
  };

  // Two steps (32 tokens) share every read of an operand slab from LDS — those reads, 60 KB a
  // step, are what the CU runs out of first; the keys of the next two steps are in flight
  // meanwhile.  (A second step that lies beyond the wave's tokens works on clamped rows and
  // stores nothing.)
  uint4 A0[4] = {}, A1[4] = {}, N0[4] = {}, N1[4] = {};
  if (wstart < wend) { load_step(wstart, A0); load_step(wstart + 16, A1); }
  for (int t0 = wstart; t0 < wend; t0 += 32) {
    if (t0 + 32 < wend) { load_step(t0 + 32, N0); load_step(t0 + 48, N1); }

    mx_f32x4 acc0[NT], acc1[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      acc0[t] = mx_f32x4{0.f, 0.f, 0.f, 0.f};
      acc1[t] = mx_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int sl = 0; sl < 4; ++sl)
#pragma unroll
        for (int p = 2; p >= 0; --p) {
          const uint4 bk = Bk[((t * 4 + sl) * 3 + p) * 64 + lane];
          acc0[t] = mx_mfma(A0[sl], bk, acc0[t]);
          acc1[t] = mx_mfma(A1[sl], bk, acc1[t]);
        }
      // One tile's operands at a time: left to itself the scheduler requests the slabs of all
      // tiles up front and spills the keys to make room for them.  (Requesting a tile's twelve slabs
      // one tile ahead, into a second set of registers, changes nothing: 6.84 -> 6.86 ms.)
      __builtin_amdgcn_sched_barrier(0);
    }
    finish(A0, acc0, t0);
    __builtin_amdgcn_sched_barrier(0);
    finish(A1, acc1, t0 + 16);
#pragma unroll
    for (int sl = 0; sl < 4; ++sl) { A0[sl] = N0[sl]; A1[sl] = N1[sl]; }
  }

  // Per-tile sums of every query head: over the four row groups of a wave, then the waves.
  // (lane r16 of every row group holds the sums of head r16 % 4 over its token r16 / 4)
  s1 += __shfl_xor(s1, 4); s1 += __shfl_xor(s1, 8); s1 += __shfl_xor(s1, 16); s1 += __shfl_xor(s1, 32);
  s2 += __shfl_xor(s2, 4); s2 += __shfl_xor(s2, 8); s2 += __shfl_xor(s2, 16); s2 += __shfl_xor(s2, 32);
  if (lane < kMaxMfmaHeads) {
    red[(wave * kMaxMfmaHeads + lane) * 2 + 0] = s1;
    red[(wave * kMaxMfmaHeads + lane) * 2 + 1] = s2;
  }
  __syncthreads();
  if ((int)threadIdx.x < nq) {
    float t1 = 0.f, t2 = 0.f;
    for (int w = 0; w < kMaxMfmaWaves; ++w) {
      t1 += red[(w * kMaxMfmaHeads + threadIdx.x) * 2 + 0];
      t2 += red[(w * kMaxMfmaHeads + threadIdx.x) * 2 + 1];
    }
    float* out = a.partial + (((int64_t)(b * a.L + l) * a.num_tiles + tile) * a.A + head * a.G + q0 + threadIdx.x) * 2;
    out[0] = t1;
    out[1] = t2;
  }
  }   // tiles of this workgroup
}

template <int NX>
hipError_t launch_max_mfma_nx(const ScoreArgs& k, dim3 grid, int il, size_t lds, hipStream_t s) {
  const void* fn = il ? reinterpret_cast<const void*>(&score_max_mfma_kernel<NX, true>)
                      : reinterpret_cast<const void*>(&score_max_mfma_kernel<NX, false>);
  hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return e;
  if (il) hipLaunchKernelGGL((score_max_mfma_kernel<NX, true>), grid, dim3(kMaxMfmaThreads), lds, s, k);
  else hipLaunchKernelGGL((score_max_mfma_kernel<NX, false>), grid, dim3(kMaxMfmaThreads), lds, s, k);
  return hipGetLastError();
}

hipError_t launch_max_mfma(const ScoreArgs& k, int B, int il, hipStream_t s) {
  const int nx = k.NO > 16 ? ceil_div(k.NO - 16, 4) : 0;
  const size_t lds = max_mfma_lds_bytes(nx, k.NO);
  dim3 grid(ceil_div(k.num_tiles, kMaxMfmaTilesPerGroup), k.Hkv * k.QC, B * k.L);
  switch (nx) {
    case 0: return launch_max_mfma_nx<0>(k, grid, il, lds, s);
    case 1: return launch_max_mfma_nx<1>(k, grid, il, lds, s);
    case 2: return launch_max_mfma_nx<2>(k, grid, il, lds, s);
    case 3: return launch_max_mfma_nx<3>(k, grid, il, lds, s);
    case 4: return launch_max_mfma_nx<4>(k, grid, il, lds, s);
    default: return hipErrorInvalidValue;
  }
}

// -------------------------------------------------------------- prologues
__global__ void fold_stats_kernel(const float* qr, const float* qi, const float* qabs, const float* fs,
                                  int n_heads_total, int F, int disable_mlr, int disable_trig,
                                  float* folded) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= n_heads_total * F) return;
  const int la = idx / F, f = idx % F;
  const float r = qr[idx], i = qi[idx], s = fs[idx];
  const float qmag = __fsqrt_rn(__fadd_rn(__fadd_rn(__fmul_rn(r, r), __fmul_rn(i, i)), 1e-8f));
  const float coef = disable_mlr ? qabs[idx] : __fsub_rn(qabs[idx], qmag);
  float* o = folded + (int64_t)la * 3 * F;
  o[f] = disable_trig ? 0.f : s * r;
  o[F + f] = disable_trig ? 0.f : s * i;
  o[2 * F + f] = s * coef;
}

// cos/sin of the fp32-rounded phase t*w per offset (phase_cos_sin) and their means over the offsets.
__global__ void trig_kernel(const float* omega, const float* offsets, int NO, const int32_t* round_start,
                            int F, float* trig, float* mean_cs) {
  const int b = blockIdx.x, f = threadIdx.x;
  if (f >= F) return;
  const float w = omega[f];
  const float rs = (float)round_start[b];
  double sc = 0.0, ss = 0.0;
  for (int j = 0; j < NO; ++j) {
    const float t = __fadd_rn(rs, offsets[j]);
    float c, s;
    phase_cos_sin(__fmul_rn(t, w), c, s);
    if (trig) {
      trig[((int64_t)(b * NO + j) * 2 + 0) * F + f] = c;
      trig[((int64_t)(b * NO + j) * 2 + 1) * F + f] = s;
    }
    sc += c;
    ss += s;
  }
  mean_cs[(int64_t)b * 2 * F + f] = (float)(sc / NO);
  mean_cs[(int64_t)b * 2 * F + F + f] = (float)(ss / NO);
}

__global__ void coef_kernel(const float* folded, const float* mean_cs, int LA, int F, int mean_mode,
                            float* coef) {
  const int b = blockIdx.y;
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= LA * F) return;
  const int la = idx / F, f = idx % F;
  const float* in = folded + (int64_t)la * 3 * F;
  float* o = coef + ((int64_t)b * LA + la) * 3 * F;
  const float a1 = in[f], a2 = in[F + f], e = in[2 * F + f];
  if (mean_mode) {
    const float c = mean_cs[(int64_t)b * 2 * F + f], s = mean_cs[(int64_t)b * 2 * F + F + f];
    o[f] = fmaf(a1, c, -a2 * s);
    o[F + f] = fmaf(a2, c, a1 * s);
  } else {
    o[f] = a1;
    o[F + f] = a2;
  }
  o[2 * F + f] = e;
}

template <int LPH, int DT, bool IL>
hipError_t launch_score_t(const ScoreArgs& args, dim3 grid, int aggregation, hipStream_t s) {
  // Scalar addressing needs one token per wave iteration (the padded KV heads fill the
  // wave's rows) and a stage of 4 tokens inside one block (or dense keys).
  const bool uni = args.Hpad >= kWave / LPH &&
                   (args.block_table_pitch < 0 || (args.bs_shift >= 2));
  if (aggregation == TRI_REDUCE_MEAN) {
    if (uni)
      hipLaunchKernelGGL((score_mean_kernel<LPH, DT, IL, 2, true>), grid, dim3(kScoreThreads), 0, s, args);
    else
      hipLaunchKernelGGL((score_mean_kernel<LPH, DT, IL, 2, false>), grid, dim3(kScoreThreads), 0, s, args);
  } else
    hipLaunchKernelGGL((score_max_kernel<LPH, DT, IL>), grid, dim3(kScoreThreads), 0, s, args);
  return hipGetLastError();
}

template <int LPH>
hipError_t launch_score_lph(const ScoreArgs& args, dim3 grid, int dt, int il, int aggregation, hipStream_t s) {
  if (dt == TRI_KV_BF16)
    return il ? launch_score_t<LPH, TRI_KV_BF16, true>(args, grid, aggregation, s)
              : launch_score_t<LPH, TRI_KV_BF16, false>(args, grid, aggregation, s);
  if (dt == TRI_KV_FP16)
    return il ? launch_score_t<LPH, TRI_KV_FP16, true>(args, grid, aggregation, s)
              : launch_score_t<LPH, TRI_KV_FP16, false>(args, grid, aggregation, s);
  if (dt == TRI_KV_FP8_E4M3)
    return il ? launch_score_t<LPH, TRI_KV_FP8_E4M3, true>(args, grid, aggregation, s)
              : launch_score_t<LPH, TRI_KV_FP8_E4M3, false>(args, grid, aggregation, s);
  return hipErrorInvalidValue;
}

}  // namespace

hipError_t launch_fold_stats(const float* qr, const float* qi, const float* qabs, const float* fs,
                             int L, int A, int F, int disable_mlr, int disable_trig, float* folded,
                             hipStream_t s) {
  const int n = L * A * F;
  hipLaunchKernelGGL(fold_stats_kernel, dim3(ceil_div(n, 256)), dim3(256), 0, s, qr, qi, qabs, fs, L * A, F,
                     disable_mlr, disable_trig, folded);
  return hipGetLastError();
}

hipError_t launch_prepare(const float* folded, const float* omega, const float* offsets, int NO,
                          const int32_t* round_start, int B, int L, int A, int F, int aggregation,
                          float* coef, float* trig, hipStream_t s) {
  // The first 2*F floats per sequence of the trig area hold the offset means; the
  // per-offset tables (max aggregation) follow the means of all sequences.
  float* mean_cs = trig;
  float* tables = (aggregation == TRI_REDUCE_MAX) ? trig + (int64_t)B * 2 * F : nullptr;
  hipLaunchKernelGGL(trig_kernel, dim3(B), dim3(F), 0, s, omega, offsets, NO, round_start, F, tables, mean_cs);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(coef_kernel, dim3(ceil_div(L * A * F, 256), B), dim3(256), 0, s, folded, mean_cs, L * A, F,
                     aggregation == TRI_REDUCE_MEAN ? 1 : 0, coef);
  return hipGetLastError();
}

// TRI_TUNE_MAX_KERNEL = 1 keeps max aggregation on the vector-unit kernel (comparison runs).
static bool max_on_vector_unit() { return tuning(TRI_TUNE_MAX_KERNEL) == 1; }

hipError_t launch_score(const ScoreLaunch& a, hipStream_t s) {
  ScoreArgs k{};
  k.k_layers = a.k_layers;
  k.k_scale_layers = a.k_scale_layers;
  k.block_table = a.block_table;
  k.seq_lens = a.seq_lens;
  k.coef = a.coef;
  k.trig = (a.aggregation == TRI_REDUCE_MAX) ? a.trig + (int64_t)a.B * 2 * (a.D / 2) : nullptr;
  k.partial = a.partial;
  k.raw = a.raw;
  k.stride_block = a.stride_block;
  k.stride_token = a.stride_token;
  k.stride_head = a.stride_head;
  k.raw_stride_layer = a.raw_stride_layer;
  k.raw_stride_token = a.raw_stride_token;
  k.raw_stride_head = a.raw_stride_head;
  k.L = a.L; k.Hkv = a.Hkv; k.A = a.A; k.G = a.G; k.NO = a.NO;
  k.block_size = a.block_size;
  k.bs_shift = -1;
  for (int sft = 0; sft < 31; ++sft)
    if ((1 << sft) == a.block_size) k.bs_shift = sft;
  k.block_table_pitch = a.block_table ? a.block_table_pitch : -1;
  k.num_tiles = a.num_tiles;
  k.QC = ceil_div(a.G, kQPerPass);
  int hpad = 1;
  while (hpad < a.Hkv) hpad <<= 1;
  k.Hpad = hpad;
  const int il_max = a.rope_style == TRI_ROPE_INTERLEAVED;
  if (a.aggregation == TRI_REDUCE_MAX && a.kv_dtype == TRI_KV_BF16 && a.D == 128 && a.NO <= kMaxOffsets &&
      !max_on_vector_unit())
    return launch_max_mfma(k, a.B, il_max, s);
  const int lph = a.D / 16;
  const int upw = kWave / lph;
  const int HC = hpad >= upw ? hpad / upw : 1;
  dim3 grid(a.num_tiles, HC * k.QC, a.B * a.L);
  const int il = a.rope_style == TRI_ROPE_INTERLEAVED;
  switch (lph) {
    case 4: return launch_score_lph<4>(k, grid, a.kv_dtype, il, a.aggregation, s);
    case 8: return launch_score_lph<8>(k, grid, a.kv_dtype, il, a.aggregation, s);
    case 16: return launch_score_lph<16>(k, grid, a.kv_dtype, il, a.aggregation, s);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace tri
