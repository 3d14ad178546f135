// Pieces shared by the two resident score + reduce kernels (tri_fused.hip: vector-unit
// scoring; tri_fused_mfma.hip: matrix-core scoring): kernel arguments, the tagged-word
// exchange between workgroups, and scalar-register helpers.
#pragma once

#include "tri_common.h"

namespace tri {
namespace {

constexpr int kFusedLdsLimit = 160 * 1024;

struct FusedArgs {
  const void* const* k_layers;
  const float* const* k_scale_layers;
  const int32_t* block_table;
  const int32_t* seq_lens;
  const int32_t* prefill_lens;
  const float* coef;              // [B][L][A][3][F]
  unsigned long long* xchg;       // [B][L][tiles_per_seq][A][2]: (tag << 32) | float bits
  float* fin;                     // [B * Hkv][Tmax]
  uint32_t* status;
  int64_t stride_block, stride_token, stride_head;
  int L, Hkv, A, G, HC;
  int block_size, bs_shift, block_table_pitch;
  int tiles_per_seq, tile_tokens, seq_base, num_seqs, Tmax;
  int normalize, window_size, protect_prefill, group_reduce, layer_reduce;
  long long spin_ticks;
  // Several launches (more workgroups than the device holds at once): which launch a
  // sequence belongs to and its first workgroup there, written by fused_pack_kernel.
  const int32_t* seq_launch;
  const int32_t* seq_wg_base;
  int packed, launch_idx;
  // Layers cut into groups (one launch only): num_seqs counts (sequence, group) pairs, a workgroup
  // runs the layers of its group and leaves its sum (or maximum) over them in fin_part
  // [group][num sequences * Hkv][Tmax]; fused_layer_reduce_kernel combines the groups.
  int layer_groups, layers_per_group;
  float* fin_part;
};

// Which (sequence, workgroup within the sequence) this workgroup serves; false: none.
// One launch: sequences in order, wgs_per_seq workgroups each.  Several launches: looked up
// in the packing tables.  `slot` is one int of LDS; contains a __syncthreads().
// Position of this workgroup in the launch's linear order of (sequence, tile, head chunk).
// The hardware hands workgroup i to XCD i % 8; the order is permuted so that every XCD owns
// a contiguous range of it, i.e. the workgroups of a sequence share an XCD.  The XCDs do not
// stream at the same pace, and the workgroups of a sequence advance in lockstep (per-layer
// statistics): spread over all XCDs every sequence moves at the pace of the slowest one and
// the others wait (3.44 ms on 16 x 16384 tokens x 36 layers); with sequences confined to an
// XCD nobody waits (3.32 ms, faster than the same kernel without the exchange).
__device__ __forceinline__ int linear_workgroup() {
  const int n = gridDim.x, i = blockIdx.x;
  const int x = i & 7, q = n >> 3, r = n & 7;
  return x * q + min(x, r) + (i >> 3);
}

__device__ __forceinline__ bool locate_workgroup(const FusedArgs& a, int wgs_per_seq, int wg_mult, int* slot,
                                                 int& b, int& within) {
  const int idx = linear_workgroup();
  if (!a.packed) {
    b = a.seq_base + idx / wgs_per_seq;
    within = idx % wgs_per_seq;
    return b < a.num_seqs;
  }
  if (threadIdx.x == 0) *slot = -1;
  __syncthreads();
  for (int s = threadIdx.x; s < a.num_seqs; s += blockDim.x) {
    if (a.seq_launch[s] != a.launch_idx) continue;
    const int n = ceil_div(a.seq_lens[s], a.tile_tokens) * wg_mult;
    const int base = a.seq_wg_base[s];
    if (idx >= base && idx < base + n) *slot = s;
  }
  __syncthreads();
  b = *slot;
  if (b < 0) return false;
  within = idx - a.seq_wg_base[b];
  return true;
}

// Packs whole sequences into launches of at most `capacity` workgroups: longest first, each
// into the first of the eight most recently opened launches that still has room.  No
// launch holds fewer sequences than capacity / (largest sequence) allows, so the number of
// launches never exceeds what the host provides for.  One workgroup.
// `launches` is how many launches the host will issue and `Tmax` the length it sized everything
// for: a sequence that lands in a later launch (the host planned with other lengths than the
// device holds) or is longer than Tmax would never be scored, so the status word is raised (3)
// and the step's compaction, which looks at that word, leaves the cache alone.
__global__ __launch_bounds__(256) void fused_pack_kernel(const int32_t* seq_lens, int B, int tile_tokens,
                                                         int wg_mult, int capacity, int32_t* seq_launch,
                                                         int32_t* seq_wg_base, int launches, int Tmax,
                                                         uint32_t* status) {
  constexpr int kMaxSorted = 4096;
  __shared__ int order[kMaxSorted];
  const bool sorted = B <= kMaxSorted;
  if (sorted) {
    for (int s = threadIdx.x; s < B; s += blockDim.x) {
      const int n = ceil_div(seq_lens[s], tile_tokens);
      int rank = 0;
      for (int c = 0; c < B; ++c) {
        const int m = ceil_div(seq_lens[c], tile_tokens);
        rank += (m > n) || (m == n && c < s);
      }
      order[rank] = s;
    }
  }
  __syncthreads();
  if (threadIdx.x != 0) return;
  int used[8];
  int first = 0, open = 1;          // launches [first, first + open) are candidates
  for (int i = 0; i < 8; ++i) used[i] = 0;
  for (int i = 0; i < B; ++i) {
    const int s = sorted ? order[i] : i;
    const int n = ceil_div(seq_lens[s], tile_tokens) * wg_mult;
    int pick = -1;
    for (int c = 0; c < open; ++c)
      if (used[c] + n <= capacity) { pick = c; break; }
    if (pick < 0) {
      if (open == 8) {               // forget the oldest candidate
        for (int c = 0; c < 7; ++c) used[c] = used[c + 1];
        ++first;
        --open;
      }
      pick = open++;
      used[pick] = 0;
    }
    seq_launch[s] = first + pick;
    seq_wg_base[s] = used[pick];
    used[pick] += n;
    if (first + pick >= launches || seq_lens[s] > Tmax) atomicExch(status, 3u);
  }
}

// Length of sequence b as the kernels use it.  The host sized grids, rings and output rows for
// Tmax; a device length beyond it (a caller whose host copy was stale) is cut there and raises
// the status word (3), so nothing is read or written out of range and the results are flagged.
__device__ __forceinline__ int checked_seq_len(const int32_t* seq_lens, int b, int Tmax, uint32_t* status) {
  int T = seq_lens[b];
  if (T > Tmax) {
    if (threadIdx.x == 0) atomicExch(status, 3u);
    T = Tmax;
  }
  return T;
}

__device__ __forceinline__ unsigned long long xchg_load(const unsigned long long* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void xchg_store(unsigned long long* p, unsigned long long v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Entry l of a device-resident table of pointers, read through the constant address space:
// a scalar load (tracked by its own counter), where a vector load would make the wave
// wait for every key load issued before it.  The tables are never written by a kernel.
__device__ __forceinline__ const char* table_entry(const void* const* table, int l) {
  typedef const __attribute__((address_space(4))) uint64_t* ConstU64;
  return reinterpret_cast<const char*>(((ConstU64)(uintptr_t)table)[l]);
}

// A wave-uniform address, pinned to scalar registers: 64-bit address arithmetic may be
// done on the vector unit, and a buffer descriptor built from vector registers costs a
// readfirstlane loop around every load that uses it.
__device__ __forceinline__ void* uniform_ptr(const void* p) {
  const uint64_t v = reinterpret_cast<uint64_t>(p);
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return reinterpret_cast<void*>(((uint64_t)hi << 32) | lo);
}

// Selection scores from the per-layer-group partial results of a layer-split launch: groups
// combined in group order, then the division by the layer count of a mean over layers.
__global__ __launch_bounds__(256) void fused_layer_reduce_kernel(const float* part, float* fin, int64_t count,
                                                                 int groups, int layer_reduce, int L) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= count) return;
  float v = part[i];
  for (int g = 1; g < groups; ++g) {
    const float x = part[(int64_t)g * count + i];
    v = (layer_reduce == TRI_REDUCE_MAX) ? fmaxf(v, x) : __fadd_rn(v, x);
  }
  fin[i] = (layer_reduce == TRI_REDUCE_MEAN) ? __fdiv_rn(v, (float)L) : v;
}

// Clears the exchange words and the status word before a launch sequence.
__global__ void fused_clear_kernel(unsigned long long* xchg, int64_t words, uint32_t* status) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < words) xchg[i] = 0ull;
  if (i == 0) *status = 0u;
}

// The research path's normalisation (methods/triattention.py:255-258; tri_select_params.normalize = 2):
// population standard deviation clamped from below at 1e-6, from the double-precision sums, as the
// two-pass path's finalize_stats_kernel evaluates it.  `mine` / `other`: this lane's total and its
// neighbour's; `odd`: this lane holds the sum of squares.
__device__ __forceinline__ void population_mean_std(double mine, double other, bool odd, int T, float& mean, float& sd) {
  const double sum = odd ? other : mine, sumsq = odd ? mine : other;
  const double m = sum / (double)T;
  const double v = sumsq / (double)T - m * m;
  mean = (float)m;
  sd = fmaxf((float)sqrt(v > 0.0 ? v : 0.0), 1e-6f);
}

// Mean and safe standard deviation, over all tokens of sequence b, of layer l's raw scores
// for `items / 2` consecutive score heads starting at head ah0: waits (bounded) until every
// tile of the sequence has published its tagged sums, adds them in tile order in double,
// then applies the reference's streaming formula on the fp32 sums
// (runtime/selector_hf.py:902-909).  st[2*i] = mean, st[2*i + 1] = std of head ah0 + i.
// Called by one whole wave.
__device__ __forceinline__ void gather_layer_stats(const FusedArgs& a, int b, int l, int seq_tiles, int T, int ah0,
                                                   int items, float* st, int lane, bool& aborted) {
  const unsigned long long* in = a.xchg + ((int64_t)(b * a.L + l) * a.tiles_per_seq * a.A + ah0) * 2;
  const uint32_t want = (uint32_t)(l + 1);
  const long long t_begin = wall_clock64();
  if (a.spin_ticks < 0 && !aborted) {   // set by the host to exercise the failure path: give up without waiting
    aborted = true;
    if (lane == 0) atomicCAS(a.status, 0u, 1u);
  }
  for (int base = 0; base < items; base += 64) {
    const int item = base + lane;
    const bool live = item < items;
    double acc = 0.0;
    for (int t0 = 0; t0 < seq_tiles; t0 += 8) {
      unsigned long long w[8];
      for (;;) {
        bool ok = true;
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int t = min(t0 + u, seq_tiles - 1);
          w[u] = live ? xchg_load(in + (int64_t)t * a.A * 2 + item) : ((unsigned long long)want << 32);
          ok = ok && (uint32_t)(w[u] >> 32) == want;
        }
        if (__all(ok) || aborted) break;
        if (wall_clock64() - t_begin > a.spin_ticks ||
            __hip_atomic_load(a.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) {
          aborted = true;
          if (lane == 0) atomicCAS(a.status, 0u, 1u);   // keeps the reason another workgroup gave (2, 3)
        }
        __builtin_amdgcn_s_sleep(4);
      }
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (t0 + u < seq_tiles) acc += (double)__uint_as_float((uint32_t)w[u]);
    }
    // Lanes 2i / 2i+1 hold the sum and the sum of squares of head ah0 + base/2 + i.
    float mean, sd;
    if (a.normalize == 2) {
      population_mean_std(acc, __shfl_xor(acc, 1), (lane & 1) != 0, T, mean, sd);
    } else {
      const float mine = (float)acc;
      const float other = __shfl_xor(mine, 1);
      const float sum = (lane & 1) ? other : mine;
      const float sumsq = (lane & 1) ? mine : other;
      const float cnt = (float)T;
      mean = __fdiv_rn(sum, cnt);
      float var = 0.f;
      if (T > 1) var = __fdiv_rn(__fsub_rn(sumsq, __fmul_rn(cnt, __fmul_rn(mean, mean))), (float)(T - 1));
      var = fmaxf(var, 0.f);
      sd = __fsqrt_rn(var);
      if (sd < 1e-8f) sd = 1.f;
    }
    if (live) st[item] = (lane & 1) ? sd : mean;
  }
}

// The same statistics for the score heads of ONE KV head (`heads` of them, at most 8, starting at
// score head ah_first), gathered by the wave that scores that KV head, with no other wave
// involved: the 64 lanes are (item, part) pairs -- item = (head, sum | sum of squares), 16 slots of
// which 2 * heads are used; part = a quarter of the sequence's tiles -- so the tagged words of all
// tiles are requested in ceil(tiles / 32) rounds of eight loads per lane, where one wave gathering
// for all eight KV heads of the workgroup needs tiles / 4 rounds (16 of them, on the critical
// path of every layer, for 64 tiles of eight query heads per KV head).  Tile order inside a
// part, parts in order: a fixed summation order.  mean[i] / sd[i] of head ah_first + i come back in
// every lane.  Called by one whole wave.  (Fetching a head's two neighbouring words with one 16-byte
// load, lanes = 8 head slots x 8 parts, i.e. one round for up to 64 tiles, is no faster: 6.74 .. 6.87
// against 6.6 .. 6.8 ms for 8 x 32768 tokens x 64 layers.  The second round is not what the layer waits for.)
__device__ __forceinline__ void gather_head_stats(const FusedArgs& a, int b, int l, int seq_tiles, int T, int ah_first,
                                                  int heads, float* mean, float* sd, int lane, bool& aborted) {
  const int item = lane & 15, part = lane >> 4;
  const bool live = item < 2 * heads;
  const int per_part = ceil_div(seq_tiles, 4);
  const int t_lo = part * per_part, t_hi = min(t_lo + per_part, seq_tiles);
  const unsigned long long* in =
      a.xchg + ((int64_t)(b * a.L + l) * a.tiles_per_seq * a.A + ah_first) * 2 + (live ? item : 0);
  const uint32_t want = (uint32_t)(l + 1);
  const long long t_begin = wall_clock64();
  if (a.spin_ticks < 0 && !aborted) {
    aborted = true;
    if (lane == 0) atomicCAS(a.status, 0u, 1u);
  }
  double acc = 0.0;
  for (int t0 = 0; t0 < per_part; t0 += 8) {       // (wave-uniform trip count; lanes past their part's end idle)
    unsigned long long w[8];
    for (;;) {
      bool ok = true;
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int t = t_lo + t0 + u;
        const bool mine = live && t < t_hi;
        w[u] = mine ? xchg_load(in + (int64_t)t * a.A * 2) : ((unsigned long long)want << 32);
        ok = ok && (uint32_t)(w[u] >> 32) == want;
      }
      if (__all(ok) || aborted) break;
      if (wall_clock64() - t_begin > a.spin_ticks ||
          __hip_atomic_load(a.status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) {
        aborted = true;
        if (lane == 0) atomicCAS(a.status, 0u, 1u);
      }
      __builtin_amdgcn_s_sleep(4);
    }
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (t_lo + t0 + u < t_hi) acc += (double)__uint_as_float((uint32_t)w[u]);
  }
  // parts in order: ((p0 + p1) + p2) + p3, in lanes 0..15
  double total = acc;
  total += __shfl(acc, item + 16);
  total += __shfl(acc, item + 32);
  total += __shfl(acc, item + 48);
  const float mine = (float)total;
  const float cnt = (float)T;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    float m, s;
    if (a.normalize == 2) {
      population_mean_std(__shfl(total, 2 * i), __shfl(total, 2 * i + 1), false, T, m, s);
    } else {
      const float sum = __shfl(mine, 2 * i), sumsq = __shfl(mine, 2 * i + 1);
      m = __fdiv_rn(sum, cnt);
      float var = 0.f;
      if (T > 1) var = __fdiv_rn(__fsub_rn(sumsq, __fmul_rn(cnt, __fmul_rn(m, m))), (float)(T - 1));
      var = fmaxf(var, 0.f);
      s = __fsqrt_rn(var);
      if (s < 1e-8f) s = 1.f;
    }
    if (i < heads) { mean[i] = m; sd[i] = s; }
  }
}

}  // namespace
}  // namespace tri
