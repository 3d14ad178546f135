// Resident score + normalise + reduce kernel for gfx950: selection scores straight from
// the paged keys, without writing the raw per-query-head scores to memory.
//
// The selection score of token n for KV head h is a reduction over layers of
//   max_q (raw[l][h,q][n] - mean[l][h,q]) / std[l][h,q]           (runtime/selector_hf.py:896-989)
// and mean/std run over ALL tokens of the sequence, so a layer's raw scores can only be
// consumed once every token of that layer has been scored.  The two-kernel path writes
// them to memory (128 bytes per token and layer); here they stay in LDS instead:
//
//  * one workgroup per tile of a sequence and at most one workgroup per CU in a launch, so
//    all tiles of the launch are resident at once; a wave owns TW tokens and keeps their
//    raw scores of one layer in a ring of TW + SL slots in LDS;
//  * after a layer, each workgroup publishes its per-head sum / sum of squares as 8-byte
//    words (value, layer tag) with device-scope atomic stores; consumers poll the tagged
//    words with device-scope atomic loads, so no fence and no cache write-back is
//    needed and a word is either absent or complete;
//  * a wave keeps scoring the first SL tokens of the next layer before it needs the
//    statistics of the previous one, which hides the exchange latency; then it turns the
//    previous layer's ring entries into z-scores, reduces over the query heads of each KV
//    head and accumulates over layers in registers;
//  * the key loads are one continuous double-buffered stream across layer boundaries.
//
// Each wave waits only on data other workgroups publish unconditionally, so progress
// needs nothing but every workgroup of the launch getting a CU, which holds because a
// launch never has more workgroups than the device has CUs (workgroups that must queue
// behind another stream's kernels start late, they are never starved).  Every wait is
// also bounded in time and raises a status word instead of spinning forever.
#include <cstdlib>

#include "tri_common.h"
#include "tri_score_device.h"
#include "tri_fused_device.h"

namespace tri {
namespace {

template <int DT, bool IL, int TW, int SL>
__global__ __launch_bounds__(kFusedThreads) void fused_select_kernel(FusedArgs a) {
  constexpr int LPH = 8, F = LPH * kPairsPerLane, RING = TW + SL;
  constexpr bool FP8 = DT == TRI_KV_FP8_E4M3;
  constexpr int ES = elem_size<DT>();
  extern __shared__ __align__(16) float lds[];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  int b, tile;
  if (!locate_workgroup(a, a.tiles_per_seq, 1, reinterpret_cast<int*>(lds), b, tile)) return;
  const int T = checked_seq_len(a.seq_lens, b, a.Tmax, a.status);
  const int n0 = tile * a.tile_tokens;
  if (n0 >= T) return;
  const int n1 = min(n0 + a.tile_tokens, T);
  const int seq_tiles = ceil_div(T, a.tile_tokens);

  float* ring = lds + wave * (RING * 32);
  float* part = lds + kFusedWaves * (RING * 32);              // [waves][64][2]
  float* stats = part + kFusedWaves * 128;                    // [2][A][2]
  uint32_t* ctl = reinterpret_cast<uint32_t*>(stats + 4 * a.A);  // arrive count, claimed, ready
  int* lds_blk = reinterpret_cast<int*>(ctl + 8);

  for (int i = threadIdx.x; i < kFusedWaves * 128; i += kFusedThreads) part[i] = 0.f;
  if (threadIdx.x < 8) ctl[threadIdx.x] = 0;
  int lb0 = 0;
  if (a.block_table_pitch >= 0) {
    lb0 = n0 >> a.bs_shift;
    const int lb1 = (n1 - 1) >> a.bs_shift;
    for (int i = threadIdx.x; i <= lb1 - lb0; i += kFusedThreads)
      lds_blk[i] = a.block_table[(int64_t)b * a.block_table_pitch + lb0 + i];
  }
  __syncthreads();
  // From here on the waves of the workgroup run independently.

  const int hc = wave % a.HC, wsub = wave / a.HC;
  const int wstart = n0 + wsub * TW;
  if (wstart >= n1) return;
  const int wend = min(wstart + TW, n1);
  const int ntok = wend - wstart;
  const int active_waves = ceil_div(n1 - n0, TW) * a.HC;
  const int last_tok = n1 - 1;

  const int m = lane & 7, g = lane >> 3;
  const int head = hc * 8 + g;
  const bool head_ok = head < a.Hkv;
  const int head_c = head_ok ? head : 0;
  const int flip = (m >> 2) & 1;
  const bool b0 = ((m & 1) ^ flip) != 0;
  const bool b1 = (((m >> 1) & 1) ^ flip) != 0;
  const int qsel = 2 * (int)b0 + (int)b1;
  const bool slot_b = m >= 4;
  const bool out_ok = head_ok && qsel < a.G;
  const int ring_col = g * 4 + qsel;

  float P[4][8], R[4][8], E[4][8];
  auto load_coefs = [&](int l) __attribute__((always_inline)) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const bool ok = head_ok && q < a.G;
      const int ah = head_c * a.G + (q < a.G ? q : 0);
      const float* c = a.coef + (((int64_t)(b * a.L + l) * a.A + ah) * 3) * F + m * kPairsPerLane;
#pragma unroll
      for (int v = 0; v < 2; ++v) {
        const float4 p4 = ok ? *reinterpret_cast<const float4*>(c + v * 4) : float4{0, 0, 0, 0};
        const float4 r4 = ok ? *reinterpret_cast<const float4*>(c + F + v * 4) : float4{0, 0, 0, 0};
        const float4 e4 = ok ? *reinterpret_cast<const float4*>(c + 2 * F + v * 4) : float4{0, 0, 0, 0};
        P[q][v * 4 + 0] = p4.x; P[q][v * 4 + 1] = p4.y; P[q][v * 4 + 2] = p4.z; P[q][v * 4 + 3] = p4.w;
        R[q][v * 4 + 0] = r4.x; R[q][v * 4 + 1] = r4.y; R[q][v * 4 + 2] = r4.z; R[q][v * 4 + 3] = r4.w;
        E[q][v * 4 + 0] = e4.x; E[q][v * 4 + 1] = e4.y; E[q][v * 4 + 2] = e4.z; E[q][v * 4 + 3] = e4.w;
      }
    }
  };

  // Physical block ids of this wave's tokens, one per lane (TW / block_size <= 64), so the
  // per-pair address needs a lane read instead of an LDS round trip.
  int blk_of_lane = 0;
  const int wlb0 = wstart >> (a.block_table_pitch >= 0 ? a.bs_shift : 0);
  if (a.block_table_pitch >= 0) blk_of_lane = lds_blk[min(wlb0 + lane, last_tok >> a.bs_shift) - lb0];

  const uint32_t lane_off_bytes =
      (uint32_t)(((int64_t)head_c * a.stride_head + (IL ? m * 16 : m * 8)) * ES);
  const uint32_t tok_bytes = (uint32_t)(a.stride_token * ES);
  const uint32_t scale_tok_bytes = (uint32_t)a.Hkv * 4u;

  // The two tokens of layer l starting at local token t (t even).
  auto load_pair = [&](RowData (&buf)[2], int l, int t) __attribute__((always_inline)) {
    const char* kbase = table_entry(a.k_layers, l);
    const int t0 = min(wstart + t, last_tok);
    int64_t row_elems, slot;
    if (a.block_table_pitch < 0) {
      row_elems = (int64_t)b * a.stride_block + (int64_t)t0 * a.stride_token;
      slot = (int64_t)b * a.block_size + t0;
    } else {
      const int lb = t0 >> a.bs_shift;
      const int64_t phys = __builtin_amdgcn_readlane(blk_of_lane, lb - wlb0);
      const int in_off = t0 - (lb << a.bs_shift);
      row_elems = phys * a.stride_block + (int64_t)in_off * a.stride_token;
      slot = phys * a.block_size + in_off;
    }
    const __amdgpu_buffer_rsrc_t rsrc =
        __builtin_amdgcn_make_buffer_rsrc(uniform_ptr(kbase + row_elems * ES), 0, 0x7fffffff, 0x00020000);
    __amdgpu_buffer_rsrc_t srsrc = rsrc;
    if constexpr (FP8)
      srsrc = __builtin_amdgcn_make_buffer_rsrc(uniform_ptr(reinterpret_cast<const float*>(table_entry(reinterpret_cast<const void* const*>(a.k_scale_layers), l)) + slot * a.Hkv), 0, 0x7fffffff,
                                                0x00020000);
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      const uint32_t dt = (uint32_t)(min(wstart + t + r, last_tok) - t0);
      const uint32_t soff = dt * tok_bytes;
      buf[r].scale = 1.f;
      if constexpr (FP8) {
        if (IL) {
          buf[r].lo = buffer_load16(rsrc, lane_off_bytes, soff);
          buf[r].hi = uint4{0, 0, 0, 0};
        } else {
          buf[r].lo = buffer_load8(rsrc, lane_off_bytes, soff);
          buf[r].hi = buffer_load8(rsrc, lane_off_bytes + LPH * 8, soff);
        }
        buf[r].scale = buffer_load_f32(srsrc, (uint32_t)head_c * 4u, dt * scale_tok_bytes);
      } else {
        buf[r].lo = buffer_load16(rsrc, lane_off_bytes, soff);
        buf[r].hi = buffer_load16(rsrc, lane_off_bytes + (IL ? 16 : LPH * 16), soff);
      }
    }
  };

  auto score_row = [&](const RowData& d) __attribute__((always_inline)) -> float {
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
    const float r = reduce_row<LPH>(acc, b0, b1);
    return FP8 ? r * d.scale : r;
  };

  float s1 = 0.f, s2 = 0.f;
  auto compute_pair = [&](const RowData (&buf)[2], int l, int t) __attribute__((always_inline)) {
    const float ra = score_row(buf[0]);
    const float rb = score_row(buf[1]);
    const float v = slot_b ? rb : ra;
    const int tl = t + (slot_b ? 1 : 0);
    if (out_ok && tl < ntok) {
      ring[((uint32_t)(l * TW + tl) % RING) * 32 + ring_col] = v;
      s1 += v;
      s2 = fmaf(v, v, s2);
    }
  };

  bool aborted = false;
  uint32_t* arrive_cnt = ctl;
  uint32_t* claimed = ctl + 1;
  uint32_t* ready = ctl + 2;

  // Deposit this wave's sums of layer l; the last wave of the workgroup to do so adds
  // the waves in a fixed order and publishes the tile's sums.  Every wave deposits
  // layer l before any wave deposits layer l + 1 (a wave consumes layer l, which needs
  // every deposit of layer l, before it finishes layer l + 1), so the counter never
  // mixes layers and never needs a reset.
  auto arrive = [&](int l) __attribute__((always_inline)) {
    part[(wave * 64 + lane) * 2] = s1;
    part[(wave * 64 + lane) * 2 + 1] = s2;
    s1 = 0.f;
    s2 = 0.f;
    uint32_t prev = 0;
    if (lane == 0) prev = __hip_atomic_fetch_add(arrive_cnt, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_WORKGROUP);
    prev = __builtin_amdgcn_readfirstlane(prev);
    if (prev + 1 != (uint32_t)(l + 1) * (uint32_t)active_waves) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    unsigned long long* out = a.xchg + ((int64_t)(b * a.L + l) * a.tiles_per_seq + tile) * a.A * 2;
    const unsigned long long tag = (unsigned long long)(uint32_t)(l + 1) << 32;
    const int waves_per_chunk = kFusedWaves / a.HC;
    for (int item = lane; item < a.A * 2; item += 64) {
      const int ah = item >> 1, which = item & 1;
      const int hd = ah / a.G, q = ah - hd * a.G;
      const int chunk = hd >> 3, hl = hd & 7;
      const int ma = (q >> 1) | ((q & 1) << 1);                  // token-A lane of query head q
      const int mb = 4 + (1 - (q >> 1)) + 2 * (1 - (q & 1));     // token-B lane
      float t = 0.f;
      for (int ws = 0; ws < waves_per_chunk; ++ws) {
        const int w = ws * a.HC + chunk;
        t += part[(w * 64 + hl * 8 + ma) * 2 + which];
        t += part[(w * 64 + hl * 8 + mb) * 2 + which];
      }
      xchg_store(out + item, tag | __float_as_uint(t));
    }
  };

  float fin[TW / 8];
#pragma unroll
  for (int k = 0; k < TW / 8; ++k) fin[k] = 0.f;
  const int ch = lane & 7;                 // head within the chunk this lane consumes
  const int chead = hc * 8 + ch;
  const bool chead_ok = chead < a.Hkv;
  const int prefill = (a.protect_prefill && a.prefill_lens) ? a.prefill_lens[b] : 0;
  const int window_from = a.window_size > 0 ? T - min(a.window_size, T) : T;

  // Turn layer l's ring entries into selection-score contributions.
  auto consume = [&](int l) __attribute__((always_inline)) {
    float mean[4] = {0.f, 0.f, 0.f, 0.f}, sd[4] = {1.f, 1.f, 1.f, 1.f};
    if (a.normalize) {
      // The first wave to get here fetches the layer's statistics for the workgroup:
      // `claimed` moves from l to l + 1 exactly once; `ready` only ever grows.
      uint32_t won = 0;
      if (lane == 0) {
        uint32_t expect = (uint32_t)l;
        won = __hip_atomic_compare_exchange_strong(claimed, &expect, (uint32_t)(l + 1), __ATOMIC_ACQ_REL,
                                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) ? 1u : 0u;
      }
      won = __builtin_amdgcn_readfirstlane(won);
      if (won) {
        gather_layer_stats(a, b, l, seq_tiles, T, 0, a.A * 2, stats + (l & 1) * a.A * 2, lane, aborted);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        if (lane == 0) __hip_atomic_store(ready, (uint32_t)(l + 1), __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
      } else {
        // The claiming wave always finishes (its own waits are bounded).
        while (__hip_atomic_load(ready, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) < (uint32_t)(l + 1))
          __builtin_amdgcn_s_sleep(2);
      }
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
      const float* st = stats + (l & 1) * a.A * 2;
#pragma unroll
      for (int q = 0; q < 4; ++q)
        if (chead_ok && q < a.G) {
          mean[q] = st[(chead * a.G + q) * 2];
          sd[q] = __fdiv_rn(1.f, st[(chead * a.G + q) * 2 + 1]);   // the tokens multiply by the reciprocal
        }
    }
#pragma unroll
    for (int k = 0; k < TW / 8; ++k) {
      const int tl = (lane >> 3) + 8 * k;
      if (tl >= ntok) continue;
      const float4 x = *reinterpret_cast<const float4*>(&ring[((uint32_t)(l * TW + tl) % RING) * 32 + ch * 4]);
      const float xs[4] = {x.x, x.y, x.z, x.w};
      float v;
      if (a.group_reduce == TRI_REDUCE_MAX) {
        v = -INFINITY;
#pragma unroll
        for (int q = 0; q < 4; ++q)
          if (q < a.G) v = fmaxf(v, __fmul_rn(__fsub_rn(xs[q], mean[q]), sd[q]));
      } else {
        v = 0.f;
#pragma unroll
        for (int q = 0; q < 4; ++q)
          if (q < a.G) v = __fadd_rn(v, __fmul_rn(__fsub_rn(xs[q], mean[q]), sd[q]));
        v = __fdiv_rn(v, (float)a.G);
      }
      const int n = wstart + tl;
      if (n >= window_from || n < prefill) v = INFINITY;
      if (l == 0) fin[k] = v;
      else fin[k] = (a.layer_reduce == TRI_REDUCE_MAX) ? fmaxf(fin[k], v) : __fadd_rn(fin[k], v);
    }
  };

  // ---- one continuous stream of key rows over (layer, token pair).  Four pair buffers
  // rotate; a buffer is refilled as soon as it has been scored, so three pairs of loads
  // are in flight while one pair is being scored.  A layer is padded to whole rotations
  // (padding slots re-read the last row and are not scored), and the rotations form
  // inner loops that contain nothing but key loads and scoring, so that the waits the
  // compiler places in them are for exactly the buffer about to be scored; the work at
  // layer boundaries sits between the inner loops.
  const int npairs = (ntok + 1) >> 1;
  const int rotations = (npairs + 3) >> 2;                  // per layer
  const int rot_before_consume = min(SL / 8, rotations);    // SL tokens = SL/8 rotations
  int ld_l = 0, ld_slot = 0;                                // next pair slot to fetch
  auto fetch = [&](RowData (&buf)[2]) __attribute__((always_inline)) {
    // Always issued, so the number of loads in flight is the same at every point of a loop.
    const int l = __builtin_amdgcn_readfirstlane(min(ld_l, a.L - 1));
    const int t = __builtin_amdgcn_readfirstlane(min(ld_slot, npairs - 1) * 2);
    load_pair(buf, l, t);
    if (++ld_slot >= rotations * 4) { ld_slot = 0; ++ld_l; }
  };
  auto score = [&](const RowData (&buf)[2], int l, int slot) __attribute__((always_inline)) {
    if (slot < npairs) compute_pair(buf, l, slot * 2);
  };
  RowData buf0[2], buf1[2], buf2[2], buf3[2];
  auto rotate = [&](int l, int r0, int r1) __attribute__((always_inline)) {
    for (int r = r0; r < r1; ++r) {
      score(buf0, l, r * 4 + 0);
      fetch(buf0);
      score(buf1, l, r * 4 + 1);
      fetch(buf1);
      score(buf2, l, r * 4 + 2);
      fetch(buf2);
      score(buf3, l, r * 4 + 3);
      fetch(buf3);
    }
  };
  // Everything outstanding has arrived: the inner loops start from a known state.
  auto settle = [&]() __attribute__((always_inline)) { __builtin_amdgcn_s_waitcnt(0x0F70); };

  load_coefs(0);
  fetch(buf0);
  fetch(buf1);
  fetch(buf2);
  fetch(buf3);
  for (int l = 0; l < a.L; ++l) {
    settle();
    rotate(l, 0, rot_before_consume);
    if (l > 0) consume(l - 1);
    rotate(l, rot_before_consume, rotations);
    if (a.normalize) arrive(l);
    if (l + 1 < a.L) load_coefs(l + 1);
  }
  consume(a.L - 1);

  if (chead_ok) {
    float* out = a.fin + ((int64_t)b * a.Hkv + chead) * a.Tmax + wstart;
#pragma unroll
    for (int k = 0; k < TW / 8; ++k) {
      const int tl = (lane >> 3) + 8 * k;
      if (tl < ntok) out[tl] = (a.layer_reduce == TRI_REDUCE_MEAN) ? __fdiv_rn(fin[k], (float)a.L) : fin[k];
    }
  }
}

template <int TW, int SL>
size_t fused_lds_bytes(int A, int tile_tokens, int bs_shift, bool paged) {
  const int blocks = paged ? (tile_tokens >> bs_shift) + 2 : 0;
  return ((size_t)kFusedWaves * (TW + SL) * 32 + kFusedWaves * 128 + 4 * (size_t)A + 8 + blocks) * 4;
}

template <int DT, bool IL, int TW, int SL>
hipError_t launch_fused_t(FusedArgs& k, int seqs_per_launch, int resident, int B, hipStream_t s) {
  const size_t lds = fused_lds_bytes<TW, SL>(k.A, k.tile_tokens, k.bs_shift, k.block_table_pitch >= 0);
  if (lds > (size_t)kFusedLdsLimit) return hipErrorInvalidValue;
  const void* fn = reinterpret_cast<const void*>(&fused_select_kernel<DT, IL, TW, SL>);
  hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return e;
  if (B <= seqs_per_launch) {
    k.packed = 0;
    k.seq_base = 0;
    const int n = B;
    hipLaunchKernelGGL((fused_select_kernel<DT, IL, TW, SL>), dim3(n * k.tiles_per_seq), dim3(kFusedThreads), lds, s, k);
    return hipGetLastError();
  }
  // More workgroups than the device holds at once: whole sequences are packed into
  // launches on the device (the host does not know the individual lengths); the host
  // issues as many launches as the worst case needs, surplus ones find no work.
  k.packed = 1;
  const int launches = ceil_div(B, seqs_per_launch);
  hipLaunchKernelGGL(fused_pack_kernel, dim3(1), dim3(256), 0, s, k.seq_lens, B, k.tile_tokens, 1, resident,
                     const_cast<int32_t*>(k.seq_launch), const_cast<int32_t*>(k.seq_wg_base), launches, k.Tmax,
                     k.status);
  e = hipGetLastError();
  if (e != hipSuccess) return e;
  for (int i = 0; i < launches; ++i) {
    k.launch_idx = i;
    hipLaunchKernelGGL((fused_select_kernel<DT, IL, TW, SL>), dim3(resident), dim3(kFusedThreads), lds, s, k);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

template <int DT, bool IL>
hipError_t launch_fused_tw(FusedArgs& k, int tw, int seqs_per_launch, int resident, int B, hipStream_t s) {
  switch (tw) {
    case 128: return launch_fused_t<DT, IL, 128, 16>(k, seqs_per_launch, resident, B, s);
    case 64: return launch_fused_t<DT, IL, 64, 16>(k, seqs_per_launch, resident, B, s);
    case 32: return launch_fused_t<DT, IL, 32, 8>(k, seqs_per_launch, resident, B, s);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace

int fused_resident_workgroups() {
  // One workgroup per CU (the kernel's LDS and register use allow no more); cached per device.
  static int cached[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
  if (cached[dev] == 0) {
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) cus = 0;
    // The workgroups of a launch wait for each other, so all of them must be on the chip at once.
    // That is assumed only where it can be checked: the occupancy calculator must place one
    // workgroup of the largest instance on a CU, and no CU mask may be in force for the process
    // (the CU count above does not show one); otherwise the two-pass kernels are used.
    const bool masked = std::getenv("HSA_CU_MASK") || std::getenv("ROC_GLOBAL_CU_MASK");
    if (masked || !fused_mfma_fits_device()) cus = 0;
    cached[dev] = cus > 0 ? cus : -1;
  }
  int n = cached[dev] > 0 ? cached[dev] : 0;
  // Tests: pretend the device is smaller, so that small inputs need several launches.
  const int64_t want = tuning(TRI_TUNE_RESIDENT_WORKGROUPS);
  if (want > 0 && want < n) n = (int)want;
  return n;
}

FusedPlan plan_fused(int B, int Hkv, int D, int G, int block_size, bool paged, int aggregation, int Tmax,
                     int resident, bool any_fill) {
  FusedPlan p{};
  if (resident <= 0 || D != 128 || G < 1 || G > 4 || aggregation != TRI_REDUCE_MEAN || Tmax <= 0 || B <= 0)
    return p;
  int bs_shift = -1;
  for (int sft = 0; sft < 31; ++sft)
    if ((1 << sft) == block_size) bs_shift = sft;
  if (paged && bs_shift < 1) return p;
  int hpad = 8;
  while (hpad < Hkv) hpad <<= 1;
  const int HC = hpad / 8;
  if (HC > kFusedWaves) return p;
  const int tws[3] = {32, 64, 128};
  int tw = 128;
  for (int i = 0; i < 3; ++i) {
    const int tile = tws[i] * (kFusedWaves / HC);
    if ((int64_t)B * ceil_div(Tmax, tile) <= resident) { tw = tws[i]; break; }
  }
  const int tile = tw * (kFusedWaves / HC);
  const int tiles = ceil_div(Tmax, tile);
  if (tiles > resident) return p;
  // A launch that fills fewer than ~70 % of the CUs loses to the two-pass kernels.
  if (!any_fill && (int64_t)B * tiles * 10 < (int64_t)resident * 7) return p;
  p.eligible = 1;
  p.tw = tw;
  p.HC = HC;
  p.tile_tokens = tile;
  p.tiles_per_seq = tiles;
  p.seqs_per_launch = resident / tiles;
  p.resident = resident;
  p.bs_shift = bs_shift;
  return p;
}

long long resident_spin_ticks() {
  const int64_t us = tuning(TRI_TUNE_RESIDENT_WAIT_US);
  return us < 0 ? -1LL : (long long)us * 100LL;     // the wall clock ticks at 100 MHz
}

hipError_t launch_fused_select(const FusedLaunch& a, hipStream_t s) {
  FusedArgs k{};
  k.k_layers = a.k_layers;
  k.k_scale_layers = a.k_scale_layers;
  k.block_table = a.block_table;
  k.seq_lens = a.seq_lens;
  k.prefill_lens = a.prefill_lens;
  k.coef = a.coef;
  k.xchg = a.xchg;
  k.fin = a.fin;
  k.status = a.status;
  k.stride_block = a.stride_block; k.stride_token = a.stride_token; k.stride_head = a.stride_head;
  k.L = a.L; k.Hkv = a.Hkv; k.A = a.A; k.G = a.G; k.HC = a.plan.HC;
  k.block_size = a.block_size; k.bs_shift = a.plan.bs_shift;
  k.block_table_pitch = a.block_table ? a.block_table_pitch : -1;
  k.tiles_per_seq = a.plan.tiles_per_seq; k.tile_tokens = a.plan.tile_tokens;
  k.seq_base = 0; k.num_seqs = a.B; k.Tmax = a.Tmax;
  k.normalize = a.normalize; k.window_size = a.window_size; k.protect_prefill = a.protect_prefill;
  k.group_reduce = a.group_reduce; k.layer_reduce = a.layer_reduce;
  k.spin_ticks = resident_spin_ticks();
  k.seq_launch = a.pack;
  k.seq_wg_base = a.pack + a.B;
  const int64_t words = (int64_t)a.B * a.L * k.tiles_per_seq * a.A * 2;
  hipLaunchKernelGGL(fused_clear_kernel, dim3((unsigned)ceil_div64(words, 256)), dim3(256), 0, s, a.xchg, words,
                     a.status);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  const bool il = a.rope_style == TRI_ROPE_INTERLEAVED;
  switch (a.kv_dtype) {
    case TRI_KV_BF16:
      return il ? launch_fused_tw<TRI_KV_BF16, true>(k, a.plan.tw, a.plan.seqs_per_launch, a.plan.resident, a.B, s)
                : launch_fused_tw<TRI_KV_BF16, false>(k, a.plan.tw, a.plan.seqs_per_launch, a.plan.resident, a.B, s);
    case TRI_KV_FP16:
      return il ? launch_fused_tw<TRI_KV_FP16, true>(k, a.plan.tw, a.plan.seqs_per_launch, a.plan.resident, a.B, s)
                : launch_fused_tw<TRI_KV_FP16, false>(k, a.plan.tw, a.plan.seqs_per_launch, a.plan.resident, a.B, s);
    case TRI_KV_FP8_E4M3:
      return il ? launch_fused_tw<TRI_KV_FP8_E4M3, true>(k, a.plan.tw, a.plan.seqs_per_launch, a.plan.resident, a.B, s)
                : launch_fused_tw<TRI_KV_FP8_E4M3, false>(k, a.plan.tw, a.plan.seqs_per_launch, a.plan.resident, a.B, s);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace tri
