// In-place, order-preserving paged K/V compaction for gfx950.
//
// keep[] is strictly ascending, so keep[j] >= j: destination slot j always lies at
// or below its source.  One workgroup owns one (sequence, layer, K or V, head) and walks the
// destination slots in ascending tiles.  Every tile is read completely
// into registers, the workgroup synchronises, then the tile is written: a tile's writes
// land below the next tile's first slot while every later source lies at or above
// it, so nothing that is still to be read is ever overwritten and no staging copy
// of the cache is needed.  The reference gathers all T rows of K and V into
// temporaries and scatters them back (runtime/kv_compaction.py:529-546).
#include "tri_common.h"
#include <cstdlib>
#include <mutex>

namespace tri {
namespace {

constexpr int kCompactThreads = 256;
constexpr int kChunksPerThread = 4;                                  // 16-byte chunks held per thread
static_assert(kChunksPerThread == 4, "compact_kernel spells out four chunk registers");
constexpr int kTileChunks = kCompactThreads * kChunksPerThread;      // 16 KiB per tile
constexpr int kOrderedThreads = 256;                                 // ordered pass: 4 waves, 16 KiB per tile; a whole batch of streams fits the chip at once
constexpr int kOrderedTileChunks = kOrderedThreads * kChunksPerThread;
constexpr int kSegEntries = 2048;                                    // (slot, list) addresses staged in LDS at a time

// The per-layer pointers come out of a device-side table and are generic to the compiler;
// these casts tell it they are global memory, so it emits global (not flat) loads and
// stores, which complete in issue order and can be waited for individually.
typedef unsigned int cu32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(1))) cu32x4* GlobalChunk;
typedef const __attribute__((address_space(1))) cu32x4* GlobalChunkIn;
__device__ __forceinline__ uint4 load_chunk(const char* p) {
  const cu32x4 v = *(GlobalChunkIn)(uintptr_t)p;
  return uint4{v.x, v.y, v.z, v.w};
}
// (Non-temporal stores here are slower: 1.84 against 1.74 ms for the 16 x 16384-token step's
// compaction; non-temporal loads change nothing.)
__device__ __forceinline__ void store_chunk(char* p, const uint4& v) {
  *(GlobalChunk)(uintptr_t)p = cu32x4{v.x, v.y, v.z, v.w};
}

struct CompactArgs {
  const void* const* k_layers;
  const void* const* v_layers;
  const float* const* k_scale_layers;
  const float* const* v_scale_layers;
  const int32_t* block_table;
  const int32_t* seq_lens;
  const int32_t* budgets;
  const int32_t* keep;
  const uint32_t* guard;   // optional; non-zero word: move nothing
  int64_t stride_block_b, stride_token_b, stride_head_b;   // bytes
  uint32_t block_units, token_units, head_units;           // the same strides in 16-byte units
  int B, L, Hkv, block_size, bs_shift, block_table_pitch, max_budget;
  int keep_per_layer, shared;
  int lists_per_wg;        // keep lists (heads) one workgroup of the ordered pass moves together
  int split_bulk;          // 1: the ordered kernel stops at the first source >= budget
  int chunks_per_row;      // 16-byte chunks of one head row (D * elem_bytes / 16)
  int heads_per_slot;      // shared ? Hkv : 1
  int streams_per_layer;   // 2 * (shared ? 1 : Hkv)
  int layer_stride;        // coprime to L: consecutive units take layers this far apart (unit_of)
};

__device__ __forceinline__ int64_t slot_offset(const CompactArgs& a, const int32_t* bt, int tok) {
  const int lb = a.bs_shift >= 0 ? (tok >> a.bs_shift) : (tok / a.block_size);
  const int in_off = tok - lb * a.block_size;
  return (int64_t)bt[lb] * a.stride_block_b + (int64_t)in_off * a.stride_token_b;
}

// Offsets are kept in 16-byte units so the per-row index arithmetic stays 32-bit.
__device__ __forceinline__ uint32_t slot_units(const CompactArgs& a, const int32_t* bt, int tok) {
  const int lb = a.bs_shift >= 0 ? (tok >> a.bs_shift) : (tok / a.block_size);
  const int in_off = tok - lb * a.block_size;
  return (uint32_t)bt[lb] * a.block_units + (uint32_t)in_off * a.token_units;
}

constexpr uint32_t kNoSource = 0xffffffffu;

// Which (sequence, layer, K or V) the unit with this index is.  Units that run at the same time
// (neighbouring indices) are spread over the whole cache: the layer runs fastest, in steps of
// `layer_stride` (coprime to L, about a third of it), then K | V, then the sequence.  With the
// layers of one sequence side by side (layer, layer + 1, ... and K next to V) the rows in flight
// at any moment lie within a few GiB of address space; spread over all of it the same
// compaction of 16 x 16384 tokens x 36 layers takes 1.68 ms instead of 1.75 when the cache spans
// 144 GiB (alternated inside one process: 1.75 / 1.70 / 1.69 / 1.69 ms for strides 1 / 7 / 11 / 13
// with K | V fastest, 1.73 / 1.69 / 1.68 with the layer fastest), and the same 1.97 ms when
// the whole cache is one piece of 36 GiB.
struct Unit { int b, l, kv; };
__device__ __forceinline__ Unit unit_of(const CompactArgs& a, int idx) {
  Unit u;
  u.l = (int)(((int64_t)(idx % a.L) * a.layer_stride) % a.L);
  idx /= a.L;
  u.kv = idx % 2;
  u.b = idx / 2;
  return u;
}

// The keep lists of a step come from a resident kernel whose waits are bounded; when one
// expired the lists are meaningless, and the step's compaction must not touch the cache.
__device__ __forceinline__ bool guard_raised(const uint32_t* guard) {
  return guard && __hip_atomic_load(guard, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0;
}

// Ordered pass: the slots whose source token lies inside the kept prefix [0, k).  With keep
// ascending they form a prefix of every list, and only they can be overwritten before they
// are read.  One workgroup owns one (sequence, layer, K or V, group of keep lists) and moves
// a tile of destination slots of its lists together.  A tile is read completely, the
// workgroup synchronises, the tile is written: a tile's writes land below the next tile's
// first slot while every later source lies at or above it, for every list, so nothing that
// is still to be read is overwritten.  Slots whose source lies at or beyond k are left to
// compact_bulk_kernel.
__global__ __launch_bounds__(kOrderedThreads) void compact_kernel(CompactArgs a) {
  __shared__ uint32_t src_units[kSegEntries];   // [slot][list], kNoSource: not this pass's
  __shared__ uint32_t dst_units[kSegEntries];   // [slot]
  __shared__ int prefix_len[256];
  if (guard_raised(a.guard)) return;

  // workgroup -> (sequence, layer, K or V, group of lists)
  const int all_lists = a.shared ? 1 : a.Hkv;
  const int lists = a.lists_per_wg;
  const int groups = all_lists / lists;
  int sidx = blockIdx.x;
  const int list0 = (sidx % groups) * lists; sidx /= groups;
  const Unit unit = unit_of(a, sidx);
  const int kv = unit.kv, l = unit.l, b = unit.b;

  int k = a.budgets[b];
  const int T = a.seq_lens[b];
  if (k > T) k = T;
  if (k > a.max_budget) k = a.max_budget;   // keep rows hold max_budget entries, whatever the device array says
  if (k <= 0) return;
  const int32_t* keep =
      a.keep + ((int64_t)(a.keep_per_layer ? (b * a.L + l) : b) * all_lists + list0) * a.max_budget;
  const int32_t* bt = a.block_table + (int64_t)b * a.block_table_pitch;
  char* base = reinterpret_cast<char*>(const_cast<void*>(kv ? a.v_layers[l] : a.k_layers[l]));

  // Length of the prefix of every list (entries below k), and the longest one.
  for (int h = threadIdx.x; h < lists; h += kOrderedThreads) prefix_len[h] = 0;
  __syncthreads();
  for (int h = 0; h < lists; ++h) {
    int below = 0;
    for (int j = threadIdx.x; j < k; j += kOrderedThreads) below += keep[(int64_t)h * a.max_budget + j] < k;
    if (below) atomicAdd(&prefix_len[h], below);
  }
  __syncthreads();
  int J = 0;
  for (int h = 0; h < lists; ++h) J = max(J, prefix_len[h]);
  if (J <= 0) return;

  const int row_chunks = a.heads_per_slot * a.chunks_per_row;       // chunks one list moves per slot
  const int slot_chunks = lists * row_chunks;                       // chunks of a whole token row
  const int slots_per_tile = max(kOrderedTileChunks / slot_chunks, 1);
  const int seg_slots = max(kSegEntries / lists / slots_per_tile, 1) * slots_per_tile;

  for (int seg = 0; seg < J; seg += seg_slots) {
    const int nseg = min(seg_slots, J - seg);
    __syncthreads();   // previous segment's LDS no longer in use
    for (int i = threadIdx.x; i < nseg * lists; i += kOrderedThreads) {
      const int sl = i / lists, h = i - sl * lists;
      const int j = seg + sl;
      const int src = keep[(int64_t)h * a.max_budget + j];
      const bool mine = j < prefix_len[h] && src != j;             // source below k, row not already in place
      src_units[i] = mine ? slot_units(a, bt, src) : kNoSource;
      if (h == 0) dst_units[sl] = slot_units(a, bt, j);
    }
    __syncthreads();

    // Units of work: tiles of slots, or, when a token row is wider than a tile, the passes
    // over one row.  The loads of unit u+1 are issued before the stores of unit u (their
    // sources lie at or above the first slot of unit u+1, beyond everything unit u writes;
    // passes of one row touch disjoint chunks), so a load batch and a store batch are
    // always in flight together; a barrier between the loads of a unit and its stores
    // orders them across the workgroup.
    const int passes = max(ceil_div(slot_chunks, kOrderedTileChunks), 1);
    const int tiles = ceil_div(nseg, slots_per_tile);
    const int units = tiles * passes;
    uint32_t dsto[kChunksPerThread];
    bool live[kChunksPerThread];
    uint4 r0, r1, r2, r3;
    auto issue = [&](int u) __attribute__((always_inline)) {
      const int t0 = (u / passes) * slots_per_tile, c0 = (u % passes) * kOrderedTileChunks;
      const int nchunks = min(slots_per_tile, nseg - t0) * slot_chunks;
      uint32_t so[kChunksPerThread];
#pragma unroll
      for (int c = 0; c < kChunksPerThread; ++c) {
        // Branch-free: a chunk index beyond the tile (a token row whose chunk count does not
        // divide the tile) repeats the pass's first chunk, load and store alike, so what it
        // writes is what that chunk writes.
        const int ci = c0 + c * kOrderedThreads + threadIdx.x;
        const bool in = ci < nchunks;
        const int cic = in ? ci : c0;
        const int sl = t0 + cic / slot_chunks;
        const int within = cic % slot_chunks;
        const int h = within / row_chunks, rem = within - h * row_chunks;
        const int hh = rem / a.chunks_per_row, cc = rem - hh * a.chunks_per_row;
        const uint32_t inner = (uint32_t)((a.shared ? 0 : list0 + h) + hh) * a.head_units + (uint32_t)cc;
        const uint32_t su = src_units[sl * lists + h];
        dsto[c] = dst_units[sl] + inner;
        live[c] = su != kNoSource;
        so[c] = live[c] ? su + inner : dsto[c];
      }
      r0 = load_chunk(base + ((uint64_t)so[0] << 4));
      r1 = load_chunk(base + ((uint64_t)so[1] << 4));
      r2 = load_chunk(base + ((uint64_t)so[2] << 4));
      r3 = load_chunk(base + ((uint64_t)so[3] << 4));
    };
    issue(0);
    __builtin_amdgcn_s_waitcnt(0x0070);   // vmcnt(0) lgkmcnt(0): this thread's loads of unit 0 have arrived
    __syncthreads();                       // ... and every other thread's
    uint4 w0 = r0, w1 = r1, w2 = r2, w3 = r3;
    uint32_t d0 = dsto[0], d1 = dsto[1], d2 = dsto[2], d3 = dsto[3];
    bool l0 = live[0], l1 = live[1], l2 = live[2], l3 = live[3];
    for (int u = 0; u + 1 < units; ++u) {
      // Unit u is a full tile (only the last unit of a segment can be partial): every chunk
      // stores, a chunk that is not this pass's writes back what it read from its own
      // destination.  Exactly four stores follow the four loads of unit u+1, and vector
      // memory operations complete in issue order, so "at most four outstanding" means the
      // loads of unit u+1 have arrived; the wave does not wait for its stores to be
      // acknowledged.  The loaded registers are copied right after that wait, so nothing at
      // the top of the loop depends on a load.
      issue(u + 1);
      store_chunk(base + ((uint64_t)d0 << 4), w0);
      store_chunk(base + ((uint64_t)d1 << 4), w1);
      store_chunk(base + ((uint64_t)d2 << 4), w2);
      store_chunk(base + ((uint64_t)d3 << 4), w3);
      asm volatile("" ::: "memory");            // keep the compiler from moving memory operations across
      __builtin_amdgcn_s_waitcnt(0x0074);       // vmcnt(4) lgkmcnt(0)
      w0 = r0; w1 = r1; w2 = r2; w3 = r3;
      d0 = dsto[0]; d1 = dsto[1]; d2 = dsto[2]; d3 = dsto[3];
      l0 = live[0]; l1 = live[1]; l2 = live[2]; l3 = live[3];
      __builtin_amdgcn_s_barrier();             // ... in every thread of the workgroup
      asm volatile("" ::: "memory");
    }
    // Last unit of the segment: its loads have arrived in every thread.
    if (l0) store_chunk(base + ((uint64_t)d0 << 4), w0);
    if (l1) store_chunk(base + ((uint64_t)d1 << 4), w1);
    if (l2) store_chunk(base + ((uint64_t)d2 << 4), w2);
    if (l3) store_chunk(base + ((uint64_t)d3 << 4), w3);
  }
}

// Slots whose source token lies at or beyond the budget: sources (>= k) and
// destinations (< k) cannot overlap, so this is a flat gather copy.  One workgroup
// moves a tile of destination slots for all heads, i.e. whole contiguous token rows.
// With keep ascending these slots are a suffix of every list, at most T - k long, so the
// tiles are counted from the end of the lists and a workgroup stops at the first tile in
// which no list has such a slot: when a step drops few tokens (T = k + 128) only a few
// tiles per (sequence, layer) do anything, and the host sizes the grid for that
// (workgroups stride over the tiles, so a grid smaller than the number of tiles is
// still complete).
__global__ __launch_bounds__(kCompactThreads) void compact_bulk_kernel(CompactArgs a) {
  if (guard_raised(a.guard)) return;
  const Unit unit = unit_of(a, blockIdx.y);
  const int kv = unit.kv, l = unit.l, b = unit.b;
  int k = a.budgets[b];
  const int T = a.seq_lens[b];
  if (k > T) k = T;
  if (k > a.max_budget) k = a.max_budget;   // keep rows hold max_budget entries, whatever the device array says
  if (k <= 0) return;
  const int lists = a.shared ? 1 : a.Hkv;
  const int chunks_per_entry = a.heads_per_slot * a.chunks_per_row;
  const int slots_per_tile = max(kTileChunks / (lists * chunks_per_entry), 1);
  const int32_t* keep = a.keep + (int64_t)(a.keep_per_layer ? (b * a.L + l) : b) * lists * a.max_budget;
  const int32_t* bt = a.block_table + (int64_t)b * a.block_table_pitch;
  char* base = reinterpret_cast<char*>(const_cast<void*>(kv ? a.v_layers[l] : a.k_layers[l]));
  const int tiles = ceil_div(k, slots_per_tile);

  for (int t = blockIdx.x; t < tiles; t += gridDim.x) {
    const int j1 = k - t * slots_per_tile;              // tile t from the end: slots [j0, j1)
    const int j0 = max(j1 - slots_per_tile, 0);
    bool any = false;
    for (int h = 0; h < lists; ++h) any = any || keep[(int64_t)h * a.max_budget + j1 - 1] >= k;
    if (!any) break;                                    // nor has any tile below this one
    const int nchunks = (j1 - j0) * lists * chunks_per_entry;

    // Three dependent lookups per chunk (keep -> block table -> row).  Each level is
    // issued for all of a thread's chunks before the next one, without branches: idle
    // chunks are clamped onto valid entries and only their final store is masked.
    for (int c0 = 0; c0 < nchunks; c0 += kTileChunks) {
      bool live[kChunksPerThread];
      int jj[kChunksPerThread], src[kChunksPerThread];
      uint32_t inner[kChunksPerThread];
#pragma unroll
      for (int c = 0; c < kChunksPerThread; ++c) {
        const int ci = c0 + c * kCompactThreads + threadIdx.x;
        live[c] = ci < nchunks;
        const int cic = live[c] ? ci : 0;
        const int e = cic / chunks_per_entry, within = cic % chunks_per_entry;
        const int h = e % lists;
        jj[c] = j0 + e / lists;
        const int hh = within / a.chunks_per_row, cc = within % a.chunks_per_row;
        inner[c] = (uint32_t)((a.shared ? 0 : h) + hh) * a.head_units + (uint32_t)cc;
        src[c] = keep[(int64_t)h * a.max_budget + jj[c]];
      }
      uint32_t so[kChunksPerThread], dsto[kChunksPerThread];
#pragma unroll
      for (int c = 0; c < kChunksPerThread; ++c) {
        live[c] = live[c] && src[c] >= k;
        const int sc = live[c] ? src[c] : j0;              // idle chunk: re-read one row of the tile (cache hit)
        so[c] = slot_units(a, bt, sc) + inner[c];
        dsto[c] = slot_units(a, bt, jj[c]) + inner[c];
      }
      uint4 regs[kChunksPerThread];
#pragma unroll
      for (int c = 0; c < kChunksPerThread; ++c)
        regs[c] = load_chunk(base + ((uint64_t)so[c] << 4));
#pragma unroll
      for (int c = 0; c < kChunksPerThread; ++c)
        if (live[c]) store_chunk(base + ((uint64_t)dsto[c] << 4), regs[c]);
    }
  }
}

// fp8 caches carry one fp32 scale per (token, head); they move with the rows.
// Same ascending-tile argument, one thread per (slot, head).
struct ScaleArgs {
  const float* const* k_scale_layers;
  const float* const* v_scale_layers;
  const int32_t* block_table;
  const int32_t* seq_lens;
  const int32_t* budgets;
  const int32_t* keep;
  const uint32_t* guard;
  int B, L, Hkv, block_size, block_table_pitch, max_budget, keep_per_layer, shared;
};

__global__ __launch_bounds__(256) void compact_scales_kernel(ScaleArgs a) {
  // One workgroup per (sequence, layer, K or V) moves the scales of all heads: a thread owns
  // (slot, head) pairs with the head fastest, so the eight heads of a destination slot are
  // written by neighbouring threads as one 32-byte piece (one workgroup per head wrote it
  // as eight separate 4-byte pieces at different times).  Tiles of 256 * kScalesPerThread
  // pairs; every level of the dependent lookups (keep -> block table -> scale) is issued
  // for all of a thread's pairs before the next one.  Within a tile all reads precede all
  // writes (barrier); a later tile reads sources at or beyond its own first slot, which
  // earlier tiles (writing below that slot) never touch.
  constexpr int kScalesPerThread = 8;
  if (guard_raised(a.guard)) return;
  int sidx = blockIdx.x;
  const int kv = sidx % 2; sidx /= 2;
  const int l = sidx % a.L;
  const int b = sidx / a.L;
  int k = a.budgets[b];
  const int T = a.seq_lens[b];
  if (k > T) k = T;
  if (k > a.max_budget) k = a.max_budget;   // keep rows hold max_budget entries, whatever the device array says
  if (k <= 0) return;
  const int rows = a.shared ? 1 : a.Hkv;
  const int32_t* keep = a.keep + (int64_t)(a.keep_per_layer ? (b * a.L + l) : b) * rows * a.max_budget;
  const int32_t* bt = a.block_table + (int64_t)b * a.block_table_pitch;
  float* sc = const_cast<float*>(kv ? a.v_scale_layers[l] : a.k_scale_layers[l]);
  const int slots_per_tile = max(256 * kScalesPerThread / a.Hkv, 1);
  for (int t0 = 0; t0 < k; t0 += slots_per_tile) {
    int src[kScalesPerThread], jj[kScalesPerThread], hh[kScalesPerThread];
    bool live[kScalesPerThread];
#pragma unroll
    for (int i = 0; i < kScalesPerThread; ++i) {
      const int p = i * 256 + threadIdx.x;
      const int sl = p / a.Hkv;
      hh[i] = p - sl * a.Hkv;
      live[i] = sl < slots_per_tile && t0 + sl < k;
      jj[i] = live[i] ? t0 + sl : 0;
      src[i] = keep[(int64_t)(a.shared ? 0 : hh[i]) * a.max_budget + jj[i]];
    }
    int sblk[kScalesPerThread], dblk[kScalesPerThread];
#pragma unroll
    for (int i = 0; i < kScalesPerThread; ++i) {
      sblk[i] = bt[src[i] / a.block_size];
      dblk[i] = bt[jj[i] / a.block_size];
    }
    float v[kScalesPerThread];
    int64_t d[kScalesPerThread];
#pragma unroll
    for (int i = 0; i < kScalesPerThread; ++i) {
      const int64_t from = ((int64_t)sblk[i] * a.block_size + src[i] % a.block_size) * a.Hkv + hh[i];
      d[i] = ((int64_t)dblk[i] * a.block_size + jj[i] % a.block_size) * a.Hkv + hh[i];
      v[i] = sc[from];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < kScalesPerThread; ++i)
      if (live[i]) sc[d[i]] = v[i];
  }
}

// ---- full permutation [kept..., dropped...] through a staging buffer ----------
// Phase 1 copies every head row of the T logical slots into staging in permuted
// order; phase 2 copies staging back over slots 0..T-1.  Two kernels on one stream,
// so phase 2 starts only after phase 1 has read everything.
struct FullArgs {
  CompactArgs c;
  char* staging;   // one layer's worth: [B][2][rows][Tmax] slots
  int Tmax;
  int layer;       // the two phases run layer by layer so the staging stays small
};

// rank[j] for dropped tokens is derived on the fly: dropped token n lands at slot
// k + (n - number of kept tokens below n).  One thread block per (stream, tile of
// 256 source tokens); a kept token n = keep[j] goes to slot j.
__global__ __launch_bounds__(256) void permute_to_staging_kernel(FullArgs f) {
  const CompactArgs& a = f.c;
  int sidx = blockIdx.y;
  const int row = sidx % (a.streams_per_layer / 2); sidx /= (a.streams_per_layer / 2);
  const int kv = sidx % 2;
  const int b = sidx / 2;
  const int l = f.layer;
  const int T = a.seq_lens[b];
  int k = a.budgets[b];
  if (k > T) k = T;
  if (k > a.max_budget) k = a.max_budget;   // keep rows hold max_budget entries, whatever the device array says
  const int n0 = blockIdx.x * 256;
  if (n0 >= T || k <= 0 || k >= T) return;
  const int rows = a.shared ? 1 : a.Hkv;
  const int32_t* keep = a.keep + ((int64_t)(a.keep_per_layer ? (b * a.L + l) : b) * rows + row) * a.max_budget;
  const int32_t* bt = a.block_table + (int64_t)b * a.block_table_pitch;
  const char* base = reinterpret_cast<const char*>(kv ? a.v_layers[l] : a.k_layers[l]);
  const int head0 = a.shared ? 0 : row;
  const int chunks_per_slot = a.heads_per_slot * a.chunks_per_row;

  __shared__ int dest[256];
  const int n = n0 + threadIdx.x;
  if (n < T) {
    // lower_bound(keep, n): number of kept tokens < n, and whether n itself is kept.
    int lo = 0, hi = k;
    while (lo < hi) {
      const int mid = (lo + hi) >> 1;
      if (keep[mid] < n) lo = mid + 1; else hi = mid;
    }
    const bool kept = lo < k && keep[lo] == n;
    dest[threadIdx.x] = kept ? lo : k + (n - lo);
  }
  __syncthreads();
  const int nvalid = min(256, T - n0);
  char* stage = f.staging + (int64_t)blockIdx.y * f.Tmax * chunks_per_slot * 16;
  for (int ci = threadIdx.x; ci < nvalid * chunks_per_slot; ci += 256) {
    const int sl = ci / chunks_per_slot, within = ci % chunks_per_slot;
    const int hh = within / a.chunks_per_row, cc = within % a.chunks_per_row;
    const int64_t so = slot_offset(a, bt, n0 + sl) + (int64_t)(head0 + hh) * a.stride_head_b + cc * 16;
    const uint4 v = load_chunk(base + so);
    store_chunk(stage + ((int64_t)dest[sl] * chunks_per_slot + within) * 16, v);
  }
}

__global__ __launch_bounds__(256) void staging_to_cache_kernel(FullArgs f) {
  const CompactArgs& a = f.c;
  int sidx = blockIdx.y;
  const int row = sidx % (a.streams_per_layer / 2); sidx /= (a.streams_per_layer / 2);
  const int kv = sidx % 2;
  const int b = sidx / 2;
  const int l = f.layer;
  const int T = a.seq_lens[b];
  int k = a.budgets[b];
  if (k > T) k = T;
  if (k > a.max_budget) k = a.max_budget;   // keep rows hold max_budget entries, whatever the device array says
  const int n0 = blockIdx.x * 256;
  if (n0 >= T || k <= 0 || k >= T) return;
  const int32_t* bt = a.block_table + (int64_t)b * a.block_table_pitch;
  char* base = reinterpret_cast<char*>(const_cast<void*>(kv ? a.v_layers[l] : a.k_layers[l]));
  const int head0 = a.shared ? 0 : row;
  const int chunks_per_slot = a.heads_per_slot * a.chunks_per_row;
  const int nvalid = min(256, T - n0);
  const char* stage = f.staging + (int64_t)blockIdx.y * f.Tmax * chunks_per_slot * 16;
  for (int ci = threadIdx.x; ci < nvalid * chunks_per_slot; ci += 256) {
    const int sl = ci / chunks_per_slot, within = ci % chunks_per_slot;
    const int hh = within / a.chunks_per_row, cc = within % a.chunks_per_row;
    const int64_t d = slot_offset(a, bt, n0 + sl) + (int64_t)(head0 + hh) * a.stride_head_b + cc * 16;
    store_chunk(base + d, load_chunk(stage + ((int64_t)(n0 + sl) * chunks_per_slot + within) * 16));
  }
}

CompactArgs make_args(const CompactLaunch& a) {
  CompactArgs c{};
  c.k_layers = a.k_layers;
  c.v_layers = a.v_layers;
  c.k_scale_layers = a.k_scale_layers;
  c.v_scale_layers = a.v_scale_layers;
  c.block_table = a.block_table;
  c.seq_lens = a.seq_lens;
  c.budgets = a.budgets;
  c.keep = a.keep;
  c.guard = a.guard;
  c.stride_block_b = a.stride_block * a.elem_bytes;
  c.stride_token_b = a.stride_token * a.elem_bytes;
  c.stride_head_b = a.stride_head * a.elem_bytes;
  c.block_units = (uint32_t)(c.stride_block_b / 16);
  c.token_units = (uint32_t)(c.stride_token_b / 16);
  c.head_units = (uint32_t)(c.stride_head_b / 16);
  c.B = a.B; c.L = a.L; c.Hkv = a.Hkv;
  c.block_size = a.block_size;
  c.bs_shift = -1;
  for (int s = 0; s < 31; ++s)
    if ((1 << s) == a.block_size) c.bs_shift = s;
  c.block_table_pitch = a.block_table_pitch;
  c.max_budget = a.max_budget;
  c.keep_per_layer = a.keep_per_layer;
  c.shared = a.shared;
  c.split_bulk = 1;
  // One list per workgroup: the ordered pass is a chain of dependent tiles per workgroup, so
  // with few sequences its run time is the chain length, and a chain over one head is
  // Hkv times shorter than one over whole token rows; with many sequences it is bound by
  // the memory system either way (16 x 16384 tokens x 36 layers, compaction alone, one process:
  // 1.965 ms with one list, 2.02 with all eight).
  // Tried and not kept, measured the same way (ordered + bulk, budget 2048 of 16384 tokens / 12000
  // of 32768 / fp8 rows):
  //  - the ordered pass cut into levels: with t0 = k and t(i+1) = entries below t(i), the
  //    positions [t(i+1), t(i)) take their rows from [t(i), t(i-1)), disjoint ranges, so each level
  //    is a flat gather without barriers between its tiles and only the last remainder needs the
  //    tile order (levels deepest first, a workgroup barrier between them): 1.966 / 10.12 / 0.955
  //    ms against 1.965 / 10.01 / 0.952.  The tile-by-tile order is not what bounds the pass.
  //  - workgroups ordered so that all sequences of one layer's K (or V) tensor run next to each
  //    other (a smaller set of pages in use at any time): 1.97 / 10.19 / 1.017 against
  //    1.96 / 9.96 / 0.98, and 1.89 against 1.74 in a second process.
  // What does move these figures is where the cache lies physically: the same virtual range freed
  // and allocated again runs the same compaction in 1.69 to 1.98 ms (one box, one process), and
  // physically contiguous allocations (hipDeviceMallocContiguous) show the same spread.
  c.lists_per_wg = 1;
  // Smallest stride of at least 0.3 L that is coprime to L (a permutation of the layers): 11 of 36, 11 of 32, 21 of 64.
  c.layer_stride = 1;
  for (int st = (3 * a.L + 9) / 10; st < a.L; ++st) {
    int x = st, y = a.L;
    while (y) { const int r = x % y; x = y; y = r; }
    if (x == 1) { c.layer_stride = st; break; }
  }
  c.chunks_per_row = a.D * a.elem_bytes / 16;
  c.heads_per_slot = a.shared ? a.Hkv : 1;
  c.streams_per_layer = 2 * (a.shared ? 1 : a.Hkv);
  return c;
}

hipError_t launch_scales(const CompactLaunch& a, hipStream_t s) {
  ScaleArgs sa{};
  sa.k_scale_layers = a.k_scale_layers;
  sa.v_scale_layers = a.v_scale_layers;
  sa.block_table = a.block_table;
  sa.seq_lens = a.seq_lens;
  sa.budgets = a.budgets;
  sa.keep = a.keep;
  sa.guard = a.guard;
  sa.B = a.B; sa.L = a.L; sa.Hkv = a.Hkv;
  sa.block_size = a.block_size;
  sa.block_table_pitch = a.block_table_pitch;
  sa.max_budget = a.max_budget;
  sa.keep_per_layer = a.keep_per_layer;
  sa.shared = a.shared;
  hipLaunchKernelGGL(compact_scales_kernel, dim3(a.B * a.L * 2), dim3(256), 0, s, sa);
  return hipGetLastError();
}

// The scales of a one-byte cache live in arrays of their own, so their kernel (small dependent
// accesses, bound by latency: 0.19 ms beside 0.93 ms of row moves on 16 x 16384 tokens x 32
// layers) runs on a side stream of the library next to the row kernels: forked from the
// caller's stream with an event, joined back with another.  One side stream and one pair of
// events per device, used under a lock (an event wait refers to the record before it, so a
// fork / join pair must not interleave with another thread's).  A stream under graph capture
// is left alone: there the scales follow the rows on the caller's stream.
struct SideStream {
  std::mutex mutex;
  static constexpr int kMaxDevices = 16;
  hipStream_t stream[kMaxDevices] = {};
  hipEvent_t fork[kMaxDevices] = {}, join[kMaxDevices] = {};
};
SideStream& side_stream() {
  static SideStream s;
  return s;
}

}  // namespace

hipError_t launch_compact(const CompactLaunch& a, hipStream_t s) {
  const CompactArgs c = make_args(a);
  const int streams = a.B * a.L * c.streams_per_layer;
  if (streams <= 0 || a.max_budget <= 0) return hipSuccess;
  int dev = -1;
  bool forked = false;
  SideStream& side = side_stream();
  std::unique_lock<std::mutex> lock(side.mutex, std::defer_lock);
  if (a.has_scales && !a.no_side_stream) {
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < SideStream::kMaxDevices &&
        hipStreamIsCapturing(s, &cap) == hipSuccess && cap == hipStreamCaptureStatusNone) {
      lock.lock();
      hipError_t e = hipSuccess;
      if (!side.stream[dev]) {
        e = hipStreamCreateWithFlags(&side.stream[dev], hipStreamNonBlocking);
        if (e == hipSuccess) e = hipEventCreateWithFlags(&side.fork[dev], hipEventDisableTiming);
        if (e == hipSuccess) e = hipEventCreateWithFlags(&side.join[dev], hipEventDisableTiming);
        if (e != hipSuccess) return e;
      }
      e = hipEventRecord(side.fork[dev], s);
      if (e == hipSuccess) e = hipStreamWaitEvent(side.stream[dev], side.fork[dev], 0);
      if (e == hipSuccess) e = launch_scales(a, side.stream[dev]);
      if (e == hipSuccess) e = hipEventRecord(side.join[dev], side.stream[dev]);
      if (e != hipSuccess) return e;
      forked = true;
    }
  }
  // Ordered pass over the slots whose sources lie inside the kept prefix, then the
  // unordered bulk pass over the rest; the first must finish reading before the second
  // writes, which stream order guarantees.
  const int ordered_groups = (a.shared ? 1 : a.Hkv) / c.lists_per_wg;
  hipLaunchKernelGGL(compact_kernel, dim3(a.B * a.L * 2 * ordered_groups), dim3(kOrderedThreads), 0, s, c);
  if (c.split_bulk) {
    hipError_t e0 = hipGetLastError();
    if (e0 != hipSuccess) return e0;
    const int lists = a.shared ? 1 : a.Hkv;
    const int slots_per_tile = max(kTileChunks / (lists * c.heads_per_slot * c.chunks_per_row), 1);
    // At most T - k slots of a list take their row from beyond the budget; one more tile
    // for the misalignment of that suffix against the tile grid.  (A sequence whose own
    // budget is smaller than max_budget may have a longer suffix: its workgroups take
    // several tiles each.)
    const int suffix = max(a.Tmax - a.max_budget, 0);
    const int tiles = min(ceil_div(suffix, slots_per_tile) + 1, ceil_div(a.max_budget, slots_per_tile));
    // (Four tiles per workgroup, every level of the lookups issued for all of them before the next,
    // i.e. 64 KiB of rows in flight behind one round of lookups, is slower: 1.95 against 1.79 ms
    // on 16 x 16384 tokens x 36 layers, 10.5 against 9.8 ms at budget 12000.  Block tables in
    // ascending order instead of a random permutation change nothing either, 1.93 against 1.98 ms:
    // the pass is bound by 256-byte rows read at one-eighth density, not by where the blocks lie.)
    dim3 grid(max(tiles, 1), a.B * a.L * 2);
    // (Fewer resident workgroups are slower as well: 8 / 5 / 4 / 2 per CU give 1.99 / 2.10 / 2.20 / 2.97 ms.)
    hipLaunchKernelGGL(compact_bulk_kernel, grid, dim3(kCompactThreads), 0, s, c);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess || !a.has_scales) return e;
  if (forked) return hipStreamWaitEvent(s, side.join[dev], 0);
  return launch_scales(a, s);
}

hipError_t launch_compact_full(const CompactLaunch& a, hipStream_t s) {
  FullArgs f{};
  f.c = make_args(a);
  f.staging = reinterpret_cast<char*>(a.staging);
  f.Tmax = a.Tmax;
  const int streams = a.B * f.c.streams_per_layer;
  if (streams <= 0 || a.Tmax <= 0) return hipSuccess;
  dim3 grid(ceil_div(a.Tmax, 256), streams);
  for (int l = 0; l < a.L; ++l) {
    f.layer = l;
    hipLaunchKernelGGL(permute_to_staging_kernel, grid, dim3(256), 0, s, f);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(staging_to_cache_kernel, grid, dim3(256), 0, s, f);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

}  // namespace tri
