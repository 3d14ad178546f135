// Resident score + normalise + reduce kernel with the contraction on the matrix cores
// (gfx950, v_mfma_f32_16x16x32_bf16).  Same structure as tri_fused.hip (raw scores of a
// layer stay in LDS, per-layer statistics exchanged through tagged words, one continuous
// stream of key loads), different mapping of the arithmetic:
//
//   raw[n][q] = sum_e k[n][e] * C[e][q]  +  sum_f |k_f[n]| * E[f][q]
//
// with k[n][.] the 128 cached elements of one KV head of token n (bf16, exact), C the P / R
// coefficients laid out per element, E the magnitude coefficients.  One wave owns one KV
// head.  An MFMA multiplies a 16-token x 32-element slab of keys, taken straight from the
// 16-byte loads (no unpacking), with a 32 x 16 coefficient slab whose columns are
// (query head, split): every fp32 coefficient is carried as three bf16 pieces
// c = c1 + c2 + c3, so the products are exact and the sum is an fp32 accumulation of the
// same terms the vector-unit kernel adds.  The magnitudes are evaluated on the vector unit
// in fp32 (sqrt(k_r^2 + k_i^2)), cut into two fp16 pieces and contracted the same way
// (v_mfma_f32_16x16x32_f16 against fp16 pieces of the magnitude coefficients).
// The three column groups of a query head are added with row rotations, which leaves every
// token's four scores spread over the lanes exactly as the ring in LDS wants them.
//
// Per 16 tokens of a head: 8 MFMAs, and vector work only for the magnitudes (about a third
// of the vector-unit kernel's instruction count), so bf16 keys run at the key stream's pace.
// fp8 e4m3 keys are widened to bf16 (exact) in registers and take the same route; the
// per-(token, head) scale multiplies the finished score.
#include <algorithm>
#include <vector>

#include "tri_common.h"
#include "tri_score_device.h"
#include "tri_fused_device.h"

namespace tri {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

constexpr int kDppRor4 = 0x124;   // row_ror:4
constexpr int kDppRor8m = 0x128;  // row_ror:8

// What a lane loads of one (token, head) row per step; the token is lane % 16 of the step,
// kb = lane / 16.  Two-byte keys: the 16-byte chunks 4*s + kb, s = 0..3 (8 elements each,
// MFMA s takes chunk s).  fp8 keys: the 16-byte chunks kb and 4 + kb (16 elements each;
// MFMA s takes half s % 2 of chunk s / 2) and the dequantisation scale of the token this
// lane will store.
// HD: head dimension, 128 or (two-byte keys only) 64: half the chunks, MFMAs and pairs.
template <int DT, int HD>
struct StepData {
  uint4 c[DT == TRI_KV_FP8_E4M3 ? 2 : HD / 32];
  float scale;
};

// Index, inside the 128 elements of a head row, of element e of lane block kb in MFMA s.
template <int DT>
__host__ __device__ constexpr int slab_elem(int s, int kb, int e) {
  return DT == TRI_KV_FP8_E4M3 ? (kb + 4 * (s >> 1)) * 16 + (s & 1) * 8 + e : (4 * s + kb) * 8 + e;
}

__device__ __forceinline__ bf16x8 as_bf16x8(const uint4& v) { return __builtin_bit_cast(bf16x8, v); }

// Largest of three (the instruction returns the other operands' maximum when one is a NaN, as
// fmaxf does; written out because the compiler canonicalises every operand of fmaxf first).
__device__ __forceinline__ float max3(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}

__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

// m[i] = sqrt(x[i].lo^2 + x[i].hi^2) for four packed bf16 pairs, in fp32.  Written out for
// two reasons: the compiler only selects the accumulating two-operand dot product
// (v_dot2c_f32_bf16) and spends a v_mov per value on zeroing its destination, and it does
// not see the opcodes inside an asm statement, so the spacing gfx950 requires between a dot
// product's write and another vector instruction's read of that register (three
// instructions) and after a transcendental's write (one) is provided here: four dot
// products, then the four square roots in the same order, then one idle cycle.
template <int DT>
__device__ __forceinline__ void magnitudes4(const uint32_t (&x)[4], float* m) {
  if constexpr (DT == TRI_KV_FP16) {
    asm("v_dot2_f32_f16 %0, %4, %4, 0\n\t"
        "v_dot2_f32_f16 %1, %5, %5, 0\n\t"
        "v_dot2_f32_f16 %2, %6, %6, 0\n\t"
        "v_dot2_f32_f16 %3, %7, %7, 0\n\t"
        "v_sqrt_f32 %0, %0\n\t"
        "v_sqrt_f32 %1, %1\n\t"
        "v_sqrt_f32 %2, %2\n\t"
        "v_sqrt_f32 %3, %3\n\t"
        "s_nop 0"
        : "=&v"(m[0]), "=&v"(m[1]), "=&v"(m[2]), "=&v"(m[3])
        : "v"(x[0]), "v"(x[1]), "v"(x[2]), "v"(x[3]));
  } else {
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
}

// Two fp32 values -> packed fp16 and the fp32 remainders, the remainders by the
// mixed-precision fused multiply-add, which reads the halves of the packed register as they
// are (x - half is exact): four instructions per two values where a bf16 split needs six.
__device__ __forceinline__ uint32_t split_pair_f16(float x0, float x1, float& r0, float& r1) {
  const f32x2 x = {x0, x1};
  const uint32_t packed = __builtin_bit_cast(uint32_t, __builtin_convertvector(x, f16x2));
  asm("v_fma_mix_f32 %0, %1, -1.0, %2 op_sel:[0,0,0] op_sel_hi:[1,0,0]" : "=v"(r0) : "v"(packed), "v"(x0));
  asm("v_fma_mix_f32 %0, %1, -1.0, %2 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(r1) : "v"(packed), "v"(x1));
  return packed;
}

// One 16x16x32 matrix-core step in the operand type of the keys (fp8 keys are converted to bf16).
template <int DT>
__device__ __forceinline__ f32x4 mfma_step(const uint4& a, const uint4& b, f32x4 c) {
  if constexpr (DT == TRI_KV_FP16)
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(a), as_bf16x8(b), c, 0, 0, 0);
}

// Piece `pieces` of x in the operand type: what is left of x after `pieces` roundings.
template <int DT>
__device__ __forceinline__ float coefficient_piece(float x, int pieces) {
  for (int s = 0; s < pieces; ++s) {
    if constexpr (DT == TRI_KV_FP16)
      x = x - (float)(_Float16)x;
    else
      x = x - __uint_as_float((uint32_t)__builtin_bit_cast(unsigned short, (__bf16)x) << 16);
  }
  return x;
}

// Everything the resident kernel needs before it starts, in one launch: workgroup (l, b)
//  - clears its share of the exchange words (and workgroup (0, 0) the status word);
//  - evaluates cos / sin of (round_start[b] + offset_j) * omega_f for all offsets and their
//    means over the offsets, the way trig_kernel does (phase_cos_sin, means summed in offset
//    order in double);
//  - combines the means with the folded statistics of layer l into P = a1*C - a2*S,
//    R = a2*C + a1*S, E (as coef_kernel) and writes them as MFMA B operands:
// bmat[(((b*L + l)*Hkv + head)*QG + g)*6 + o][lane][8] bf16.  Group g holds query heads
// 4g..4g+3 of the KV head.  Operand o: 0..3 the key slabs of MFMA o, 4 and 5 the magnitudes
// of pair sets 0 and 1.  Lane (j = lane % 16, kb): column j = (query head 4g + j % 4, split
// j / 4); element e = k index kb*8 + e of the slab.  Piece `split` of a coefficient x is
// what is left of x after `split` roundings to bf16 (x = x1 + x2 + x3).
constexpr int kPrepThreads = 1024;
// Query heads whose coefficients are staged at a time, and the pitch of a staged head
// [P | R | E][F] in floats (odd: the four query heads and four k blocks a wave reads at once
// then fall into 16 different banks).
template <int HD> constexpr int prep_heads() { return HD > 128 ? 32 : 64; }
template <int HD> constexpr int prep_pitch() { return 3 * (HD / 2) + 1; }

template <int DT, bool IL, int HD>
__global__ __launch_bounds__(kPrepThreads) void prep_mfma_kernel(const float* folded, const float* omega,
                                                                 const float* offsets, int NO,
                                                                 const int32_t* round_start, int L, int Hkv, int G,
                                                                 int A, int QG, uint4* bmat,
                                                                 unsigned long long* xchg, int64_t words,
                                                                 uint32_t* status) {
  // One buffer, used twice: the per-offset cos / sin values, then the coefficients of up to
  // kPrepHeads query heads as [head][P | R | E][F] with a row pitch of 3F + 1 floats.
  constexpr int F = HD / 2;              // frequency pairs
  constexpr int NS = HD / 32;            // key slabs (MFMAs) per step
  constexpr int NSO = NS + NS / 2;       // operands per query-head group: key slabs, magnitude slabs
  constexpr int kPrepHeads = prep_heads<HD>(), kPrepPitch = prep_pitch<HD>();
  __shared__ float buf[kPrepHeads * kPrepPitch];
  __shared__ float mean_cs[2][F];
  static_assert(kPrepHeads * kPrepPitch >= 2 * kMaxOffsets * F, "the trig values must fit the buffer");
  float (*part)[kMaxOffsets][F] = reinterpret_cast<float (*)[kMaxOffsets][F]>(buf);
  const int l = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
  const int64_t wg = (int64_t)b * gridDim.x + l, nwg = (int64_t)gridDim.x * gridDim.y;
  for (int64_t i = wg * kPrepThreads + tid; i < words; i += nwg * kPrepThreads) xchg[i] = 0ull;
  if (wg == 0 && tid == 0) *status = 0u;

  const float rs = (float)round_start[b];
  for (int i = tid; i < NO * F; i += kPrepThreads) {
    const int j = i / F, f = i % F;
    phase_cos_sin(__fmul_rn(__fadd_rn(rs, offsets[j]), omega[f]), part[0][j][f], part[1][j][f]);
  }
  __syncthreads();
  if (tid < 2 * F) {
    const int which = tid / F, f = tid % F;
    double sum = 0.0;
    for (int j = 0; j < NO; ++j) sum += part[which][j][f];
    mean_cs[which][f] = (float)(sum / NO);
  }

  const int heads_per_pass = max(1, kPrepHeads / G);        // whole KV heads
  for (int head0 = 0; head0 < Hkv; head0 += heads_per_pass) {
    const int nh = min(heads_per_pass, Hkv - head0);
    __syncthreads();                                        // means written; buffer free
    // P = a1*C - a2*S, R = a2*C + a1*S, E, of query heads head0*G .. (head0 + nh)*G - 1
    const float* in = folded + ((int64_t)l * A + (int64_t)head0 * G) * 3 * F;   // [head][a1 | a2 | e][F]
    for (int i = tid; i < nh * G * F; i += kPrepThreads) {
      const int q = i / F, f = i % F;
      const float a1 = in[q * 3 * F + f], a2 = in[q * 3 * F + F + f], e = in[q * 3 * F + 2 * F + f];
      const float c = mean_cs[0][f], sn = mean_cs[1][f];
      buf[q * kPrepPitch + f] = fmaf(a1, c, -a2 * sn);
      buf[q * kPrepPitch + F + f] = fmaf(a2, c, a1 * sn);
      buf[q * kPrepPitch + 2 * F + f] = e;
    }
    __syncthreads();
    const int items = nh * QG * NSO * 64;                   // (head, group, operand, lane)
    uint4* out_base = bmat + (((int64_t)b * L + l) * Hkv + head0) * QG * NSO * 64;
    for (int idx = tid; idx < items; idx += kPrepThreads) {
      const int lane = idx & 63;
      const int o = (idx >> 6) % NSO;
      const int g = (idx / (64 * NSO)) % QG;
      const int head = idx / (64 * NSO * QG);
      const int j = lane & 15, kb = lane >> 4;
      const int q = 4 * g + (j & 3), sp = j >> 2;
      uint32_t out[4] = {0, 0, 0, 0};
      if (q < G && sp < 3) {
        const float* c = buf + (head * G + q) * kPrepPitch;
        float v[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          int which, pair;   // which: 0 = P, 1 = R, 2 = E
          constexpr bool kRegrouped = DT == TRI_KV_FP8_E4M3 && !IL;   // see compute_step
          if (o < NS) {
            const int el = slab_elem<DT>(o, kb, e);
            if (kRegrouped) { which = e & 1; pair = kb * 16 + 4 * o + (e >> 1); }
            else if (IL) { which = el & 1; pair = el >> 1; }
            else { which = el >= F ? 1 : 0; pair = el & (F - 1); }
          } else {
            which = 2;
            const int set = o - NS;
            // interleaved: pairs of MFMAs 2*set and 2*set + 1; half: real parts of MFMA `set`
            if (kRegrouped) pair = kb * 16 + 4 * (2 * set + (e >> 2)) + (e & 3);
            else if (IL) pair = slab_elem<DT>(2 * set + (e >> 2), kb, 2 * (e & 3)) >> 1;
            else pair = slab_elem<DT>(set, kb, e) & (F - 1);
          }
          // The magnitudes go through the fp16 matrix-core instruction whatever the key type (see
          // compute_step), so the magnitude slabs are fp16 pieces.
          const bool half_slab = DT == TRI_KV_FP16 || o >= NS;
          v[e] = half_slab ? coefficient_piece<TRI_KV_FP16>(c[which * F + pair], sp)
                           : coefficient_piece<TRI_KV_BF16>(c[which * F + pair], sp);
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const f32x2 x = {v[2 * e], v[2 * e + 1]};
          if (DT == TRI_KV_FP16 || o >= NS)
            out[e] = __builtin_bit_cast(uint32_t, __builtin_convertvector(x, f16x2));
          else
            out[e] = __builtin_bit_cast(uint32_t, __builtin_convertvector(x, bf16x2));
        }
      }
      out_base[idx] = uint4{out[0], out[1], out[2], out[3]};
    }
  }
}

// QG: groups of four query heads per KV head (1 or 2).
__device__ __forceinline__ int nsteps_of(int ntok) { return (ntok + 15) >> 4; }

// W: waves per workgroup.  Eight (one workgroup per CU), or four for models with at most four
// KV heads: a workgroup of eight would leave half its waves without a head and the CU with half
// the loads in flight, so two workgroups of four share a CU (half the LDS each; two waves per
// SIMD either way, which the register budget of 256 is for).
template <int DT, bool IL, int TW, int SL, int QG, int NB, int W, int HD>
__global__ __launch_bounds__(W * kWave) __attribute__((amdgpu_waves_per_eu(2, 2)))
void fused_mfma_kernel(FusedArgs a, const uint4* bmat) {
  static_assert(HD == 128 || ((HD == 64 || HD == 256) && DT != TRI_KV_FP8_E4M3), "head dimensions with a kernel");
  constexpr int NS = HD / 32;            // key slabs (MFMAs) per step
  constexpr int NSO = NS + NS / 2;       // operands per query-head group
  static_assert(SL % (16 * NB) == 0, "the slack must hold whole rotations of the step buffers");
  constexpr int RING = TW + SL;
  constexpr int RQ = 4 * QG;                                   // ring floats per token
  extern __shared__ __align__(16) float lds[];

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  int b, within;
  if (!locate_workgroup(a, a.HC * a.tiles_per_seq, a.HC, reinterpret_cast<int*>(lds), b, within)) return;
  // Layers of this workgroup: all of them, or one group of a layer-split launch, where `b` so far
  // counts (sequence, group) pairs.
  const int lgroup = b % a.layer_groups;
  b /= a.layer_groups;
  const int l_begin = lgroup * a.layers_per_group;
  const int l_end = min(a.L, l_begin + a.layers_per_group);
  const int chunk = within % a.HC;
  const int tile = within / a.HC;
  const int T = checked_seq_len(a.seq_lens, b, a.Tmax, a.status);
  const int n0 = tile * a.tile_tokens;
  if (n0 >= T) return;
  const int n1 = min(n0 + a.tile_tokens, T);
  const int ntok = n1 - n0;
  const int last_tok = n1 - 1;
  const int seq_tiles = ceil_div(T, a.tile_tokens);
  const int heads_here = min(8, a.Hkv - chunk * 8);

  float* ring = lds + wave * (RING * RQ);                      // [QG][RING][4 query heads]
  float* part = lds + W * (RING * RQ);                         // [waves][64][QG][2]
  float* stats = part + W * 128 * QG;                          // [2][32*QG score heads][2]
  uint32_t* ctl = reinterpret_cast<uint32_t*>(stats + 128 * QG);  // arrive count, claimed, ready; [8..15]: how far each wave is
  for (int i = threadIdx.x; i < W * 128 * QG; i += W * kWave) part[i] = 0.f;
  if (threadIdx.x < 16) ctl[threadIdx.x] = 0;
  __syncthreads();
  // From here on the waves of the workgroup run independently.
  if (wave >= heads_here) return;
  const int head = chunk * 8 + wave;

  const int j = lane & 15, kb = lane >> 4;       // MFMA column / k block; also output row block
  const int q = j & 3, rsel = j >> 2;

  // Coefficient slabs of the current layer.
  uint4 B[QG][NSO];
  auto load_coefs = [&](int l) __attribute__((always_inline)) {
    const uint4* p = bmat + (((int64_t)(b * a.L + l) * a.Hkv + head) * QG * NSO) * 64 + lane;
#pragma unroll
    for (int g = 0; g < QG; ++g)
#pragma unroll
      for (int o = 0; o < NSO; ++o) B[g][o] = p[(g * NSO + o) * 64];
    {
      // A coefficient beyond fp16's range (65504) arrives as an infinity: the scores of this
      // launch would be meaningless, so the status word is raised (the caller repeats the
      // step on the vector-unit kernels) and every wait of the launch gives up.  fp16 keys:
      // all slabs; otherwise the magnitude slabs.
      uint32_t bad = 0;
#pragma unroll
      for (int g = 0; g < QG; ++g)
#pragma unroll
        for (int o = (DT == TRI_KV_FP16 ? 0 : NS); o < NSO; ++o) {
          const uint32_t w4[4] = {B[g][o].x, B[g][o].y, B[g][o].z, B[g][o].w};
#pragma unroll
          for (int i = 0; i < 4; ++i)
            bad |= (uint32_t)((w4[i] & 0x7c00u) == 0x7c00u) | (uint32_t)((w4[i] & 0x7c000000u) == 0x7c000000u);
        }
      if (__any(bad != 0) && lane == 0) atomicExch(a.status, 2u);
    }
  };

  // A step is 16 consecutive tokens starting at a multiple of 16, so with blocks of at
  // least 16 tokens it lies inside one block: lane i keeps the block of step i of the tile
  // (a tile has at most 64 steps), and a step's block is one v_readlane away.  Dense keys:
  // the "block" is the sequence.
  const bool paged = a.block_table_pitch >= 0;
  int step_blk = b;
  if (paged) {
    const int n = min(n0 + 16 * lane, last_tok);
    step_blk = a.block_table[(int64_t)b * a.block_table_pitch + (n >> a.bs_shift)];
  }
  const int bs_mask = paged ? (1 << a.bs_shift) - 1 : -1;

  // Sixteen tokens of layer l starting at local token t (t % 16 == 0).  The address splits
  // into a wave-uniform base (layer, block, first token of the step, head: scalar unit) and
  // a 32-bit lane offset (row lane % 16 of the step, 16-byte chunk lane / 16); rows past the
  // tile's last token re-read that token (loaded, never stored).
  constexpr bool FP8 = DT == TRI_KV_FP8_E4M3;
  constexpr int ES = FP8 ? 1 : 2;
  const uint32_t tok_bytes = (uint32_t)(a.stride_token * ES);
  const uint32_t lane_row = (uint32_t)j * tok_bytes;
  const uint32_t lane_col = (uint32_t)kb * 16u;
  const uint32_t lane_scale_row = (uint32_t)(4 * kb + rsel) * (uint32_t)a.Hkv * 4u;   // fp8: token this lane stores
  struct LayerBase { const char* k; const char* scale; };   // of this wave's head (scalar registers)
  auto layer_base = [&](int l) __attribute__((always_inline)) {
    LayerBase lb;
    lb.k = table_entry(a.k_layers, l) + (int64_t)head * a.stride_head * ES;
    lb.scale = nullptr;
    if constexpr (FP8)
      lb.scale = table_entry(reinterpret_cast<const void* const*>(a.k_scale_layers), l) + head * 4;
    return lb;
  };
  // One-byte keys: with eight step buffers and a scale per row the scalar registers do not
  // hold the strides, masks and sizes of the address arithmetic any more (the compiler kept
  // them in lanes of a vector register and fetched 16 of them back per step with v_readlane,
  // a tenth of the step's vector instructions).  For them the arithmetic is done once per
  // tile instead: lane i keeps the byte offset of step i's first row from the head's base
  // (the same in every layer) and the index of its first token slot.
  uint32_t step_off_lo = 0, step_off_hi = 0;
  int step_slot = 0;
  if constexpr (FP8) {
    const int nt = min(n0 + 16 * lane, (nsteps_of(ntok) - 1) * 16 + n0);
    const int in_blk = nt & bs_mask;
    const int64_t off = ((int64_t)step_blk * a.stride_block + (int64_t)in_blk * a.stride_token) * ES;
    step_off_lo = (uint32_t)off;
    step_off_hi = (uint32_t)((uint64_t)off >> 32);
    step_slot = step_blk * a.block_size + in_blk;
  }
  auto load_step = [&](StepData<DT, HD>& d, const LayerBase& lb, int t) __attribute__((always_inline)) {
    if constexpr (FP8) {
      const int step = t >> 4;
      const uint32_t rows_left = (uint32_t)(last_tok - (n0 + t));
      const uint64_t row_off = ((uint64_t)(uint32_t)__builtin_amdgcn_readlane((int)step_off_hi, step) << 32) |
                               (uint32_t)__builtin_amdgcn_readlane((int)step_off_lo, step);
      const char* base = reinterpret_cast<const char*>(uniform_ptr(lb.k + row_off));
      const uint32_t off = min(lane_row, rows_left * tok_bytes) + lane_col;
      GlobalBytes p = (GlobalBytes)(uintptr_t)base + off;
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const u32x4 v = *(GlobalU4)(p + s * 64);
        d.c[s] = uint4{v.x, v.y, v.z, v.w};
      }
      const uint32_t hkv4 = (uint32_t)a.Hkv * 4u;
      const uint64_t slot_off = (uint64_t)(uint32_t)__builtin_amdgcn_readlane(step_slot, step) * hkv4;
      const char* sc = reinterpret_cast<const char*>(uniform_ptr(lb.scale + slot_off));
      const uint32_t soff = min(lane_scale_row, rows_left * hkv4);
      d.scale = *(GlobalF32)((GlobalBytes)(uintptr_t)sc + soff);
      return;
    }
    const int blk = __builtin_amdgcn_readlane(step_blk, t >> 4);
    const int nt = n0 + t;
    const int in_blk = nt & bs_mask;
    const uint32_t rows_left = (uint32_t)(last_tok - nt);
    const int64_t row0 = (int64_t)blk * a.stride_block + (int64_t)in_blk * a.stride_token;
    const char* base = reinterpret_cast<const char*>(uniform_ptr(lb.k + row0 * ES));
    const uint32_t off = min(lane_row, rows_left * tok_bytes) + lane_col;
    GlobalBytes p = (GlobalBytes)(uintptr_t)base + off;
    d.scale = 1.f;
#pragma unroll
    for (int s = 0; s < (FP8 ? 2 : NS); ++s) {
      const u32x4 v = *(GlobalU4)(p + s * 64);
      d.c[s] = uint4{v.x, v.y, v.z, v.w};
    }
    if constexpr (FP8) {
      const int64_t slot0 = (int64_t)blk * a.block_size + in_blk;
      const char* sc = reinterpret_cast<const char*>(uniform_ptr(lb.scale + slot0 * a.Hkv * 4));
      const uint32_t soff = min(lane_scale_row, rows_left * (uint32_t)a.Hkv * 4u);
      d.scale = *(GlobalF32)((GlobalBytes)(uintptr_t)sc + soff);
    }
  };

  // Ring of this wave: [group of four query heads][RING tokens][4], so that the 64 lanes of a store
  // (16 tokens x 4 heads of one group) cover 64 consecutive words and the 16-byte reads of
  // consecutive tokens are 16 bytes apart, whatever the number of groups (with [RING][8] the stores of
  // one group fell on half the banks; it does not show in the kernel's time).
  const uint32_t lane_ring = (uint32_t)(4 * kb + rsel) * 4 + q;
  float s1[QG], s2[QG];
#pragma unroll
  for (int g = 0; g < QG; ++g) { s1[g] = 0.f; s2[g] = 0.f; }
  // Largest of a sample of the layer's magnitudes (their first fp16 pieces), per lane; see the check
  // after every layer.
  f16x2 mag_seen = {(_Float16)0.f, (_Float16)0.f};
  // Scores of the 16 tokens of a step: MFMAs over keys and magnitudes, split columns added
  // by row rotations; lane (j, kb) ends up with the score of token 4*kb + j/4, query head j%4.
  auto compute_step = [&](const StepData<DT, HD>& raw, int l, int t, int which) __attribute__((always_inline)) {
    // The four bf16 A operands of the step as dwords (two elements each): the loaded
    // registers for bf16 keys, one conversion per dword (exact) for fp8 keys.
    uint32_t w[NS][4];
    // One-byte keys in the half-split layout: lane block kb holds the real parts of pairs
    // 16*kb .. 16*kb + 15 in c[0] and their imaginary parts in c[1].  Two byte permutes per
    // dword pair put (real, imaginary) next to each other before the conversion, so every
    // converted dword is a pair: operand s holds pairs 16*kb + 4*s .. + 3, the magnitudes need
    // no regrouping (8 permutes per step instead of 16 after the conversion), and the
    // coefficient slabs are laid out to match.
    constexpr bool kRegrouped = FP8 && !IL;
    if constexpr (kRegrouped) {
      const uint32_t re[4] = {raw.c[0].x, raw.c[0].y, raw.c[0].z, raw.c[0].w};
      const uint32_t im[4] = {raw.c[1].x, raw.c[1].y, raw.c[1].z, raw.c[1].w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t lo = __builtin_amdgcn_perm(im[i], re[i], 0x05010400u);   // (re0, im0, re1, im1)
        const uint32_t hi = __builtin_amdgcn_perm(im[i], re[i], 0x07030602u);   // (re2, im2, re3, im3)
        w[i][0] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo, 1.0f, false));
        w[i][1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(lo, 1.0f, true));
        w[i][2] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi, 1.0f, false));
        w[i][3] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(hi, 1.0f, true));
      }
    } else if constexpr (FP8) {
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const uint32_t r[4] = {raw.c[s].x, raw.c[s].y, raw.c[s].z, raw.c[s].w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          uint32_t* o = &w[2 * s + (i >> 1)][(i & 1) * 2];
          o[0] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(r[i], 1.0f, false));
          o[1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(r[i], 1.0f, true));
        }
      }
    } else {
#pragma unroll
      for (int s = 0; s < NS; ++s) {
        w[s][0] = raw.c[s].x; w[s][1] = raw.c[s].y; w[s][2] = raw.c[s].z; w[s][3] = raw.c[s].w;
      }
    }
    struct { uint4 c[NS]; } d;
#pragma unroll
    for (int s = 0; s < NS; ++s) d.c[s] = uint4{w[s][0], w[s][1], w[s][2], w[s][3]};
    f32x4 acc[QG], acc_e[QG];
#pragma unroll
    for (int g = 0; g < QG; ++g) {
      acc[g] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < NS; ++s)
        acc[g] = mfma_step<DT>(d.c[s], B[g][s], acc[g]);
      acc_e[g] = acc[g];   // the magnitude MFMAs continue the sum (the key MFMAs are long done by then)
    }
#pragma unroll
    for (int set = 0; set < NS / 2; ++set) {
      // |k_f|^2 = k_r^2 + k_i^2 straight from the bf16 pairs (v_dot2_f32_bf16).
      // interleaved: dword e % 4 of operand 2*set + e/4 is the (real, imaginary) pair;
      // half: real parts in operand `set`, imaginary parts in operand `set + 2`, regrouped
      // into (real, imaginary) dwords by two byte permutes per dword.
      float mag[8];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        uint32_t x[4];
        if constexpr (IL || kRegrouped) {
#pragma unroll
          for (int i = 0; i < 4; ++i) x[i] = w[2 * set + h][i];
        } else {
#pragma unroll
          for (int i = 0; i < 2; ++i) {
            const uint32_t re = w[set][2 * h + i], im = w[set + NS / 2][2 * h + i];
            x[2 * i] = __builtin_amdgcn_perm(im, re, 0x05040100u);
            x[2 * i + 1] = __builtin_amdgcn_perm(im, re, 0x07060302u);
          }
        }
        magnitudes4<DT>(x, &mag[4 * h]);
      }
      uint4 hi, lo;
      float r[8];
      // The magnitudes are cut into two fp16 pieces (22 bits; two bf16 pieces would carry 16) and
      // go through the fp16 matrix-core instruction whatever the key type: the fp16 split is two
      // instructions per pair cheaper than the bf16 one.  Magnitudes of one-byte codes lie in
      // [2^-9, 634]; a two-byte key beyond fp16's range turns its scores into infinities or NaNs,
      // which the check after every layer finds (status word 2: the caller repeats the step on the
      // vector-unit kernels).
      hi.x = split_pair_f16(mag[0], mag[1], r[0], r[1]);
      hi.y = split_pair_f16(mag[2], mag[3], r[2], r[3]);
      hi.z = split_pair_f16(mag[4], mag[5], r[4], r[5]);
      hi.w = split_pair_f16(mag[6], mag[7], r[6], r[7]);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const f32x2 x = {r[2 * i], r[2 * i + 1]};
        (&lo.x)[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(x, f16x2));
      }
      if constexpr (!FP8)   // `which` is the step buffer's number: a constant after unrolling
        mag_seen = __builtin_elementwise_max(mag_seen, __builtin_bit_cast(f16x2, (&hi.x)[which & 3]));
      constexpr int MT = TRI_KV_FP16;                // operand type of the magnitude MFMAs
#pragma unroll
      for (int g = 0; g < QG; ++g) {
        acc_e[g] = mfma_step<MT>(hi, B[g][NS + set], acc_e[g]);
        acc_e[g] = mfma_step<MT>(lo, B[g][NS + set], acc_e[g]);
      }
    }
    const int tl = t + 4 * kb + rsel;
    // first ring slot of the step (scalar; a step never straddles the wrap: t and RING are
    // multiples of 16)
    const uint32_t slot0 = (uint32_t)(l * TW + t) % RING;
#pragma unroll
    for (int g = 0; g < QG; ++g) {
      float v = 0.f;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float x = acc_e[g][r];
        x += dpp<kDppRor8m>(x);
        x += dpp<kDppRor4>(x);
        v = (rsel == r) ? x : v;
      }
      if (FP8) v *= raw.scale;
      if (4 * g + q < a.G && tl < ntok) {
        ring[(uint32_t)g * (RING * 4) + slot0 * 4 + lane_ring] = v;
        s1[g] += v;
        s2[g] = fmaf(v, v, s2[g]);
      }
    }
  };

  bool aborted = false;
  uint32_t* arrive_cnt = ctl;
  uint32_t* claimed = ctl + 1;
  uint32_t* ready = ctl + 2;
  const int items = heads_here * a.G * 2;        // (score head, sum | sum of squares) of this workgroup
  const int ah0 = chunk * 8 * a.G;

  // Deposit this wave's sums of layer l; the last wave of the workgroup to do so adds the
  // lanes in a fixed order and publishes the tile's sums.  Every wave deposits layer l
  // before any wave deposits layer l + 1 (a wave consumes layer l, which needs every
  // deposit of layer l, before it finishes layer l + 1), so the counter never mixes layers.
  auto arrive = [&](int l) __attribute__((always_inline)) {
#pragma unroll
    for (int g = 0; g < QG; ++g) {
      part[((wave * 64 + lane) * QG + g) * 2] = s1[g];
      part[((wave * 64 + lane) * QG + g) * 2 + 1] = s2[g];
      s1[g] = 0.f;
      s2[g] = 0.f;
    }
    uint32_t prev = 0;
    if (lane == 0) prev = __hip_atomic_fetch_add(arrive_cnt, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_WORKGROUP);
    prev = __builtin_amdgcn_readfirstlane(prev);
    if (prev + 1 != (uint32_t)(l - l_begin + 1) * (uint32_t)heads_here) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    unsigned long long* out = a.xchg + (((int64_t)(b * a.L + l) * a.tiles_per_seq + tile) * a.A + ah0) * 2;
    for (int item = lane; item < items; item += 64) {
      const int ahl = item >> 1, which = item & 1;
      const int w = ahl / a.G, qq = ahl - w * a.G;
      const int g = qq >> 2, q4 = qq & 3;
      float t = 0.f;
      for (int i = 0; i < 16; ++i)
        t += part[((w * 64 + (i >> 2) * 16 + (i & 3) * 4 + q4) * QG + g) * 2 + which];
      xchg_store(out + item, ((unsigned long long)(uint32_t)(l + 1) << 32) | __float_as_uint(t));
    }
  };

  float fin[TW / 64];
#pragma unroll
  for (int k = 0; k < TW / 64; ++k) fin[k] = 0.f;
  const int prefill = (a.protect_prefill && a.prefill_lens) ? a.prefill_lens[b] : 0;
  const int window_from = a.window_size > 0 ? T - min(a.window_size, T) : T;

  // Turn layer l's ring entries into selection-score contributions (lane = token).
  auto consume = [&](int l) __attribute__((always_inline)) {
    float mean[RQ], sd[RQ];
#pragma unroll
    for (int qq = 0; qq < RQ; ++qq) { mean[qq] = 0.f; sd[qq] = 1.f; }
    if (a.normalize) {
      if constexpr (QG == 2) {
        // More than four query heads per KV head: twice the words per tile and tiles half as long,
        // so the gather is four times the work; every wave fetches the words of its own KV head
        // (8 x 32768 tokens x 64 layers, 64 query heads: 7.55 -> 6.82 ms).  With up to four query
        // heads the one wave's gather below hides behind the slack and this form is slower (16 x 16384
        // tokens x 36 layers: 3.29 -> 3.30 ms; fp8 keys 1.72 -> 1.80; 16 x 2176 tokens 0.54 -> 0.62).
        float m8[8], s8[8];
        gather_head_stats(a, b, l, seq_tiles, T, (chunk * 8 + wave) * a.G, a.G, m8, s8, lane, aborted);
#pragma unroll
        for (int qq = 0; qq < RQ; ++qq)
          if (qq < a.G) {
            mean[qq] = m8[qq];
            sd[qq] = __fdiv_rn(1.f, s8[qq]);
          }
      } else {
      uint32_t won = 0;
      if (lane == 0) {
        uint32_t expect = (uint32_t)(l - l_begin);
        won = __hip_atomic_compare_exchange_strong(claimed, &expect, (uint32_t)(l - l_begin + 1), __ATOMIC_ACQ_REL,
                                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) ? 1u : 0u;
      }
      won = __builtin_amdgcn_readfirstlane(won);
      if (won) {
        gather_layer_stats(a, b, l, seq_tiles, T, ah0, items, stats + (l & 1) * 64 * QG, lane, aborted);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        if (lane == 0)
          __hip_atomic_store(ready, (uint32_t)(l - l_begin + 1), __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
      } else {
        // The claiming wave always finishes (its own waits are bounded).
        while (__hip_atomic_load(ready, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) < (uint32_t)(l - l_begin + 1))
          __builtin_amdgcn_s_sleep(2);
      }
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
      const float* st = stats + (l & 1) * 64 * QG;
#pragma unroll
      for (int qq = 0; qq < RQ; ++qq)
        if (qq < a.G) {
          mean[qq] = st[(wave * a.G + qq) * 2];
          // One division per head and layer; the tokens multiply by the reciprocal (a
          // division per score costs ten vector instructions, 7 % of the kernel's total).
          sd[qq] = __fdiv_rn(1.f, st[(wave * a.G + qq) * 2 + 1]);
        }
      }
    }
    // The usual mode -- every query-head slot of the group in use, maximum over the group, running sum
    // over layers, whole chunks of 64 tokens, not the first layer -- without the per-head predicates, the
    // two reduction variants, the lane masks and the modulo per token of the general loop below: a third
    // of its instructions.  The guards need no attention here: the first layer of a workgroup goes
    // through the general loop, which sets the guarded tokens to +inf, and a finite contribution leaves
    // them there.  This piece of work sits on every wave's path once per layer (removed altogether, for
    // timing only, it is worth 3.4 % of the kernel on 16 x 16384 tokens x 36 layers, 4.2 % with eight
    // query heads per KV head).
    if (a.G == RQ && a.group_reduce == TRI_REDUCE_MAX && a.layer_reduce == TRI_REDUCE_MEAN && l != l_begin &&
        (ntok & 63) == 0) {
      // This lane's entry of chunk 0 inside the wave's ring; chunk k lies 64 k entries further on, or
      // RING entries back once that passes the ring's end (one compare and one select per chunk, the
      // distance itself goes into the LDS instruction's offset field).
      const uint32_t lane_pos = (uint32_t)(l * TW) % RING + (uint32_t)lane;          // below 2 * RING
      uint32_t at = lane_pos * 4, at_wrapped = (lane_pos - RING) * 4;               // in floats
      asm volatile("" : "+v"(at), "+v"(at_wrapped));     // (keeps both in vector registers)
      struct Entry { float4 x[QG]; };
      auto entry = [&](int k) __attribute__((always_inline)) {
        const uint32_t p = (lane_pos >= (uint32_t)(RING - 64 * k)) ? at_wrapped : at;
        Entry e;
#pragma unroll
        for (int g = 0; g < QG; ++g)
          e.x[g] = *reinterpret_cast<const float4*>(ring + p + (64 * 4 * k + g * (RING * 4)));
        return e;
      };
      auto contribution = [&](const Entry& e) __attribute__((always_inline)) {
        float z[RQ];
#pragma unroll
        for (int g = 0; g < QG; ++g) {
          z[4 * g] = __fmul_rn(__fsub_rn(e.x[g].x, mean[4 * g]), sd[4 * g]);
          z[4 * g + 1] = __fmul_rn(__fsub_rn(e.x[g].y, mean[4 * g + 1]), sd[4 * g + 1]);
          z[4 * g + 2] = __fmul_rn(__fsub_rn(e.x[g].z, mean[4 * g + 2]), sd[4 * g + 2]);
          z[4 * g + 3] = __fmul_rn(__fsub_rn(e.x[g].w, mean[4 * g + 3]), sd[4 * g + 3]);
        }
        float v = max3(z[0], z[1], z[2]);
#pragma unroll
        for (int qq = 3; qq + 1 < RQ; qq += 2) v = max3(v, z[qq], z[qq + 1]);
        return max3(v, z[RQ - 1], z[RQ - 1]);
      };
      if (ntok == TW) {
        // a whole tile: straight-line code, the ring entries of four chunks requested before the first is used
        constexpr int kAhead = QG == 1 ? 4 : 2;
#pragma unroll
        for (int k0 = 0; k0 < TW / 64; k0 += kAhead) {
          Entry e[kAhead];
#pragma unroll
          for (int i = 0; i < kAhead; ++i) e[i] = entry(k0 + i);
#pragma unroll
          for (int i = 0; i < kAhead; ++i) fin[k0 + i] = __fadd_rn(fin[k0 + i], contribution(e[i]));
        }
      } else {
#pragma unroll
        for (int k = 0; k < TW / 64; ++k)
          if (64 * k < ntok) fin[k] = __fadd_rn(fin[k], contribution(entry(k)));            // (wave-uniform)
      }
      return;
    }
#pragma unroll
    for (int k = 0; k < TW / 64; ++k) {
      const int tl = lane + 64 * k;
      if (tl >= ntok) continue;
      float xs[RQ];
#pragma unroll
      for (int g = 0; g < QG; ++g) {
        const float4 x = *reinterpret_cast<const float4*>(&ring[(uint32_t)g * (RING * 4) + ((uint32_t)(l * TW + tl) % RING) * 4]);
        xs[4 * g] = x.x; xs[4 * g + 1] = x.y; xs[4 * g + 2] = x.z; xs[4 * g + 3] = x.w;
      }
      float v;
      if (a.group_reduce == TRI_REDUCE_MAX) {
        v = -INFINITY;
#pragma unroll
        for (int qq = 0; qq < RQ; ++qq)
          if (qq < a.G) v = fmaxf(v, __fmul_rn(__fsub_rn(xs[qq], mean[qq]), sd[qq]));
      } else {
        v = 0.f;
#pragma unroll
        for (int qq = 0; qq < RQ; ++qq)
          if (qq < a.G) v = __fadd_rn(v, __fmul_rn(__fsub_rn(xs[qq], mean[qq]), sd[qq]));
        v = __fdiv_rn(v, (float)a.G);
      }
      const int n = n0 + tl;
      if (n >= window_from || n < prefill) v = INFINITY;
      if (l == l_begin) fin[k] = v;
      else fin[k] = (a.layer_reduce == TRI_REDUCE_MAX) ? fmaxf(fin[k], v) : __fadd_rn(fin[k], v);
    }
  };

  // ---- one continuous stream of key rows over (layer, step of 16 tokens).  NB step
  // buffers rotate (four of 64 bytes per lane, or eight of 36 for one-byte keys, which keeps
  // the same number of bytes in flight); a buffer is refilled as soon as it has been scored,
  // with the step NB ahead.  A layer is padded to whole rotations (padding steps re-read the
  // last row and are not scored), so the loads of a layer's last rotation are exactly the
  // first NB steps of the next layer; the rotations form inner loops that contain nothing
  // but key loads and scoring, and the work at layer boundaries sits between them.
  const int nsteps = (ntok + 15) >> 4;
  const int rotations = (nsteps + NB - 1) / NB;
  const int rot_before_consume = min(SL / (16 * NB), rotations);
  auto score = [&](const StepData<DT, HD>& d, int l, int slot, int which) __attribute__((always_inline)) {
    if (slot < nsteps) compute_step(d, l, slot * 16, which);
  };
  StepData<DT, HD> buf[NB];
  LayerBase base_cur = layer_base(l_begin), base_next = base_cur;
  // The two waves of a SIMD (waves i and i + 4 of a workgroup of eight) compete for its issue slots and
  // the arbiter prefers the older one: left alone, waves 0..3 of every workgroup run ahead, then wait at
  // the next layer's statistics for waves 4..7 of every tile, and the SIMD is half empty meanwhile (with
  // eight query heads per KV head waves 0..3 spent 18 % of their time in that wait, waves 4..7 11 %).
  // So each wave posts how far it is at every rotation and takes the higher priority while it is behind
  // its neighbour (8 x 32768 tokens x 64 layers 6.55 -> 6.48 ms, one-byte keys 1.70 -> 1.63 ms).
  uint32_t* progress = ctl + 8;
  auto rotate = [&](int l, int r0, int r1) __attribute__((always_inline)) {
    for (int r = r0; r < r1; ++r) {
      if constexpr (W == 8) {
        const uint32_t mine = (uint32_t)((l - l_begin) * rotations + r);
        if (lane == 0) __hip_atomic_store(progress + wave, mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        const uint32_t other = (uint32_t)__builtin_amdgcn_readfirstlane(
            (int)__hip_atomic_load(progress + (wave ^ 4), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP));
        if (mine < other) __builtin_amdgcn_s_setprio(2);
        else __builtin_amdgcn_s_setprio(0);
      }
      const bool wrap = r + 1 >= rotations;
      const LayerBase lb = {wrap ? base_next.k : base_cur.k, wrap ? base_next.scale : base_cur.scale};
      const int s0 = wrap ? 0 : (r + 1) * NB;
#pragma unroll
      for (int i = 0; i < NB; ++i) {
        score(buf[i], l, r * NB + i, i);
        load_step(buf[i], lb, min(s0 + i, nsteps - 1) * 16);
      }
    }
  };
  auto settle = [&]() __attribute__((always_inline)) { __builtin_amdgcn_s_waitcnt(0x0F70); };

  load_coefs(l_begin);
#pragma unroll
  for (int i = 0; i < NB; ++i) load_step(buf[i], base_cur, min(i, nsteps - 1) * 16);
  for (int l = l_begin; l < l_end; ++l) {
    base_cur = base_next;
    base_next = layer_base(min(l + 1, l_end - 1));
    settle();
    rotate(l, 0, rot_before_consume);
    if (l > l_begin) consume(l - 1);
    rotate(l, rot_before_consume, rotations);
    if constexpr (!FP8) {
      // A magnitude beyond fp16's range (or a key that is not finite) has left an infinity or a NaN
      // in this layer's sums.
      bool bad = false;
#pragma unroll
      for (int g = 0; g < QG; ++g) bad = bad || !(s2[g] < INFINITY);
      // The other end of fp16's range: below 2^-14 the first piece is a subnormal and below 2^-3 the
      // second one is, so magnitudes carry an absolute error of up to 2^-25 whatever their size.
      // Against keys of ordinary size that is nothing (scaled by 2^-10, magnitudes around 2^-9, the
      // selection scores are as close to the fp64 ones as unscaled); keys that are all tiny (scaled by
      // 2^-14: errors of 2e-4 of the largest score) are left to the other kernels: no lane of the
      // wave has seen a magnitude of 2^-9 in this layer (of every step one pair in four is looked at,
      // another one in each of the step buffers, so every frequency pair is among them).
      const bool seen = (float)mag_seen[0] >= 0x1p-9f || (float)mag_seen[1] >= 0x1p-9f;
      mag_seen = f16x2{(_Float16)0.f, (_Float16)0.f};
      if ((__any(bad) || !__any(seen)) && lane == 0) atomicExch(a.status, 2u);
    }
    if (a.normalize) arrive(l);
    if (l + 1 < l_end) load_coefs(l + 1);
  }
  consume(l_end - 1);

  if (a.layer_groups > 1) {
    // This group's sum (or maximum) over its layers; fused_layer_reduce_kernel combines the groups.
    const int64_t rows = (int64_t)(a.num_seqs / a.layer_groups) * a.Hkv;
    float* out = a.fin_part + (((int64_t)lgroup * rows + (int64_t)b * a.Hkv + head) * a.Tmax) + n0;
#pragma unroll
    for (int k = 0; k < TW / 64; ++k) {
      const int tl = lane + 64 * k;
      if (tl < ntok) out[tl] = fin[k];
    }
    return;
  }
  float* out = a.fin + ((int64_t)b * a.Hkv + head) * a.Tmax + n0;
#pragma unroll
  for (int k = 0; k < TW / 64; ++k) {
    const int tl = lane + 64 * k;
    if (tl < ntok) out[tl] = (a.layer_reduce == TRI_REDUCE_MEAN) ? __fdiv_rn(fin[k], (float)a.L) : fin[k];
  }
}

// How a batch is cut into launches (from the plan).
struct LaunchShape {
  int seqs_per_launch;   // whole sequences of maximum length one launch holds
  int resident;          // workgroups the device holds at once
  int num_seqs;
  int launches;          // > 0: exactly this many (the planner replayed the device's packing); 0: the worst case
};

template <int TW, int SL, int QG, int W>
constexpr size_t mfma_lds_bytes() {
  return ((size_t)W * (TW + SL) * 4 * QG + W * 128 * QG + 128 * QG + 16) * 4;
}

template <int DT, bool IL, int TW, int SL, int QG, int NB, int W = kFusedWaves, int HD = 128>
hipError_t launch_mfma_t(FusedArgs& k, const uint4* bmat, const LaunchShape& shape, hipStream_t s) {
  const int seqs_per_launch = shape.seqs_per_launch, resident = shape.resident, B = shape.num_seqs;
  const int known_launches = shape.launches;
  constexpr size_t lds = mfma_lds_bytes<TW, SL, QG, W>();
  // 8 waves: one workgroup per CU; 4 waves: two (LDS is handed out in blocks of 1280 bytes).
  static_assert(((lds + 1279) / 1280 * 1280) * (kFusedWaves / W) <= (size_t)kFusedLdsLimit, "LDS of a CU");
  const void* fn = reinterpret_cast<const void*>(&fused_mfma_kernel<DT, IL, TW, SL, QG, NB, W, HD>);
  hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return e;
  if (B <= seqs_per_launch) {
    k.packed = 0;
    k.seq_base = 0;
    const int n = B * k.layer_groups;      // (sequence, layer group) pairs; k.num_seqs counts the same
    hipLaunchKernelGGL((fused_mfma_kernel<DT, IL, TW, SL, QG, NB, W, HD>), dim3(n * k.tiles_per_seq * k.HC), dim3(W * kWave), lds, s, k, bmat);
    return hipGetLastError();
  }
  if (k.layer_groups != 1) return hipErrorInvalidValue;   // layer groups exist in single launches only
  // More workgroups than the device holds at once: whole sequences are packed into
  // launches on the device (the host does not know the individual lengths); the host
  // issues as many launches as the worst case needs, surplus ones find no work.
  k.packed = 1;
  const int launches = known_launches > 0 ? known_launches : ceil_div(B, seqs_per_launch);
  hipLaunchKernelGGL(fused_pack_kernel, dim3(1), dim3(256), 0, s, k.seq_lens, B, k.tile_tokens, k.HC, resident,
                     const_cast<int32_t*>(k.seq_launch), const_cast<int32_t*>(k.seq_wg_base), launches, k.Tmax,
                     k.status);
  e = hipGetLastError();
  if (e != hipSuccess) return e;
  for (int i = 0; i < launches; ++i) {
    k.launch_idx = i;
    hipLaunchKernelGGL((fused_mfma_kernel<DT, IL, TW, SL, QG, NB, W, HD>), dim3(resident), dim3(W * kWave), lds, s, k, bmat);
    e = hipGetLastError();
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

}  // namespace

// Does the current device hold one resident workgroup per CU?  Asked once per device of the
// runtime's occupancy calculator, for the instance with the largest ring (1024 + 192 tokens, eight
// waves, 256 registers a lane): a part with less LDS per CU, or a runtime that gives the kernel
// fewer resources than this file assumes, then takes the two-pass kernels instead of launching
// workgroups that would wait for others that cannot start.
bool fused_mfma_fits_device() {
  const void* fn = reinterpret_cast<const void*>(&fused_mfma_kernel<TRI_KV_BF16, false, 1024, 192, 1, 4, kFusedWaves, 128>);
  constexpr size_t lds = mfma_lds_bytes<1024, 192, 1, kFusedWaves>();
  if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  int per_cu = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, fn, kFusedWaves * kWave, lds) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return per_cu >= 1;
}

namespace {

template <int DT, bool IL>
hipError_t launch_mfma_tw(FusedArgs& k, const uint4* bmat, int tw, int waves, int head_dim, const LaunchShape& shape,
                          hipStream_t s) {
  if (head_dim == 256) {
    // Twice the bytes per row: two step buffers hold as many bytes as four do for 128.
    if constexpr (DT != TRI_KV_FP8_E4M3) {
      if (k.G > 4) {
        if (tw != 512) return hipErrorInvalidValue;
        return waves == 4 ? launch_mfma_t<DT, IL, 512, 64, 2, 2, 4, 256>(k, bmat, shape, s)
                          : launch_mfma_t<DT, IL, 512, 64, 2, 2, 8, 256>(k, bmat, shape, s);
      }
      if (tw != 1024) return hipErrorInvalidValue;
      return waves == 4 ? launch_mfma_t<DT, IL, 1024, 128, 1, 2, 4, 256>(k, bmat, shape, s)
                        : launch_mfma_t<DT, IL, 1024, 192, 1, 2, 8, 256>(k, bmat, shape, s);
    }
    return hipErrorInvalidValue;
  }
  if (head_dim == 64) {
    // Half the bytes per row: eight step buffers keep as many bytes in flight (four query heads
    // per KV head; with eight the LDS has no room for the slack that eight buffers need).  One
    // instance per shape, with the largest ring.
    if constexpr (DT != TRI_KV_FP8_E4M3) {
      if (k.G > 4) {
        if (tw != 512) return hipErrorInvalidValue;
        return waves == 4 ? launch_mfma_t<DT, IL, 512, 64, 2, 4, 4, 64>(k, bmat, shape, s)
                          : launch_mfma_t<DT, IL, 512, 64, 2, 4, 8, 64>(k, bmat, shape, s);
      }
      if (tw != 1024) return hipErrorInvalidValue;
      return waves == 4 ? launch_mfma_t<DT, IL, 1024, 128, 1, 8, 4, 64>(k, bmat, shape, s)
                        : launch_mfma_t<DT, IL, 1024, 128, 1, 8, 8, 64>(k, bmat, shape, s);
    }
    return hipErrorInvalidValue;
  }
  if (waves == 4) {
    // Two workgroups per CU: the ring of the largest tile with one rotation of slack less
    // (a smaller tile is a run-time argument inside it).
    constexpr int NB4 = DT == TRI_KV_FP8_E4M3 ? 8 : 4;
    if (k.G > 4) return tw == 512 ? launch_mfma_t<DT, IL, 512, 64, 2, 4, 4>(k, bmat, shape, s)
                                  : hipErrorInvalidValue;
    return tw == 1024 ? launch_mfma_t<DT, IL, 1024, 128, 1, NB4, 4>(k, bmat, shape, s)
                      : hipErrorInvalidValue;
  }
  if (k.G > 4) {
    switch (tw) {   // eight query heads per KV head: 32 bytes of ring per token
      case 512: return launch_mfma_t<DT, IL, 512, 64, 2, 4>(k, bmat, shape, s);
      case 256: return launch_mfma_t<DT, IL, 256, 64, 2, 4>(k, bmat, shape, s);
      default: return hipErrorInvalidValue;
    }
  }
  // One-byte keys: eight step buffers.
  constexpr int NB = DT == TRI_KV_FP8_E4M3 ? 8 : 4;
  // Slack: as much as LDS allows beside the ring of a 1024-token tile, in whole rotations
  // (16 x 16384 tokens x 36 layers, bf16, warm GPU: 3.54 ms with 64, 3.49 with 128, 3.45 with 192).
  constexpr int SL = DT == TRI_KV_FP8_E4M3 ? 128 : 192;
  switch (tw) {
    case 1024: return launch_mfma_t<DT, IL, 1024, SL, 1, NB>(k, bmat, shape, s);
    case 512: return launch_mfma_t<DT, IL, 512, SL, 1, NB>(k, bmat, shape, s);
    case 256: return launch_mfma_t<DT, IL, 256, SL, 1, NB>(k, bmat, shape, s);
    default: return hipErrorInvalidValue;
  }
}

// What fused_pack_kernel will do with these lengths, on the host: sequences by falling tile
// count, each into the first of the eight most recently opened launches with room.  Returns the
// number of launches.
int host_pack_launches(const int32_t* lens, int B, int tile, int wg_mult, int capacity) {
  std::vector<int> tiles(B);
  for (int i = 0; i < B; ++i) tiles[i] = ceil_div(lens[i], tile);
  std::vector<int> order(B);
  for (int i = 0; i < B; ++i) order[i] = i;
  if (B <= 4096)   // (the kernel sorts up to that many)
    std::stable_sort(order.begin(), order.end(), [&](int x, int y) { return tiles[x] > tiles[y]; });
  int used[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  int first = 0, open = 1;
  for (int i = 0; i < B; ++i) {
    const int n = tiles[order[i]] * wg_mult;
    int pick = -1;
    for (int c = 0; c < open; ++c)
      if (used[c] + n <= capacity) { pick = c; break; }
    if (pick < 0) {
      if (open == 8) {
        for (int c = 0; c < 7; ++c) used[c] = used[c + 1];
        ++first;
        --open;
      }
      pick = open++;
      used[pick] = 0;
    }
    used[pick] += n;
  }
  return first + open;
}

}  // namespace

FusedPlan plan_fused_mfma(int B, int Hkv, int D, int G, int block_size, bool paged, int aggregation, int Tmax,
                          int resident, bool any_fill, int kv_dtype, const int32_t* host_lens, int L,
                          bool split_layers) {
  FusedPlan p{};
  const bool dim_ok = D == 128 || ((D == 64 || D == 256) && kv_dtype != TRI_KV_FP8_E4M3);
  if (resident <= 0 || !dim_ok || G < 1 || G > 8 || aggregation != TRI_REDUCE_MEAN || Tmax <= 0 || B <= 0)
    return p;
  int bs_shift = -1;
  for (int sft = 0; sft < 31; ++sft)
    if ((1 << sft) == block_size) bs_shift = sft;
  if (paged && bs_shift < 4) return p;    // a 16-token step must lie inside one block
  const int HC = ceil_div(Hkv, 8);
  // At most four KV heads: workgroups of four waves, two per CU.
  const int waves = Hkv <= 4 ? 4 : kFusedWaves;
  if (waves == 4) resident *= 2;
  const int tws[3] = {256, 512, 1024};
  const int ntw = G > 4 ? 2 : 3;          // the ring of a 1024-token tile fits LDS for four query heads only
  int tw = tws[ntw - 1];
  if (waves == kFusedWaves && D == 128)   // (four waves, head dimensions 64 and 256: one kernel instance, with the largest ring)
    for (int i = 0; i < ntw; ++i)
      if ((int64_t)B * ceil_div(Tmax, tws[i]) * HC <= resident) { tw = tws[i]; break; }
  int tile = tw, tiles = ceil_div(Tmax, tw);
  if ((int64_t)tiles * HC > resident) return p;
  if ((int64_t)B * tiles * HC <= resident) {
    // The whole batch is one launch: cut the sequences into as many tiles as the chip has
    // room for, in whole rotations of the step buffers (64 tokens, 128 for one-byte keys), so
    // that e.g. 16 sequences of 3072 tokens run as 16 x 16 tiles of 192 instead of 16 x 12 of
    // 256.  Not below 128 tokens and not more than 64 tiles per sequence: smaller tiles pay the
    // per-layer work of a workgroup too often, and every workgroup gathers the statistics of
    // all tiles of its sequence (one sequence of 16384 tokens as 256 tiles of 64 fills the
    // chip and takes 1.14 ms; the two-pass kernels take 0.38).
    const int granule = (kv_dtype == TRI_KV_FP8_E4M3 || (D == 64 && G <= 4)) ? 128 : 64;   // a rotation of the step buffers
    const int tiles_max = min(resident / (B * HC), 64);
    tile = ceil_div(ceil_div(Tmax, tiles_max), granule) * granule;
    tile = min(tw, max(128, tile));
    tiles = ceil_div(Tmax, tile);
  }
  // A launch that fills fewer than ~60 % of the CUs loses to the two-pass kernels, which
  // spread a small problem over the whole chip (16 sequences: even at 2176 tokens = 56 % of
  // the CUs, 10 % ahead at 2560 = 62 %, 21 % ahead at 3072 = 75 %).
  // (Workgroups of four waves: 45 %.  28 query / 4 KV heads, 16 x 2176 tokens, 272 of 512
  // workgroups: 0.40 ms against 0.48 ms on the two-pass kernels.)
  const int64_t need = waves == 4 ? 45 : 60;
  int layer_groups = 1, layers_per_group = L;
  if (split_layers && L > 1 && (int64_t)B * tiles * HC <= resident) {
    // A batch that is one launch: the layers are independent until the reduction over them, so
    // they can be cut into groups, a workgroup running one (sequence, group, tile).  A launch takes
    // as long as its longest workgroup: layers x (tile tokens + the fixed work of a layer, worth
    // ~32 tokens: the exchange of the statistics, the coefficient loads).  Whole-model workgroups
    // of a few requests (the reference's runner compresses one at a time,
    // runtime/runner_compression_actions.py:24) would use a fraction of the chip, 17 of 256 CUs
    // for one request of 2176 tokens x 36 layers: that becomes 36 groups x 7 tiles of 320 tokens
    // = 252 workgroups.  Mid-size batches gain as well: 16 requests of 2176 tokens are 16 x 12
    // tiles of 192 tokens x 36 layers (75 % of the CUs) or, with four groups of nine layers,
    // 16 x 4 x 4 tiles of 576 tokens on every CU, a quarter less per workgroup.  A cut must
    // win 5 % to be taken: the groups' partial sums cost a pass of their own, and a launch that
    // fills the chip already is bound by HBM as much as by its longest workgroup (16 x 8192 tokens
    // as two groups of 1024-token tiles: 1 % slower than whole-model tiles of 512).
    const int granule = (kv_dtype == TRI_KV_FP8_E4M3 || (D == 64 && G <= 4)) ? 128 : 64;
    const int tw_max = tws[ntw - 1];                       // the longest tile any instance of this shape holds
    const bool one_instance = !(waves == kFusedWaves && D == 128);
    constexpr int kLayerFixed = 32;
    int64_t best = (int64_t)L * (tile + kLayerFixed) * 95 / 100;
    for (int lpg = L - 1; lpg >= 1; --lpg) {
      const int groups = ceil_div(L, lpg);
      const int64_t units = (int64_t)B * groups * HC;
      if (units > resident) break;                         // fewer layers per group: more groups still
      const int tiles_max = (int)min((int64_t)64, resident / units);
      int t = ceil_div(ceil_div(Tmax, tiles_max), granule) * granule;
      t = min(tw_max, max(128, t));
      const int nt = ceil_div(Tmax, t);
      if (units * nt > resident) continue;
      const int64_t cost = (int64_t)lpg * (t + kLayerFixed) + groups;
      if (cost >= best) continue;
      best = cost;
      layer_groups = groups;
      layers_per_group = lpg;
      tile = t;
      tiles = nt;
      if (!one_instance)
        for (int i = 0; i < ntw; ++i)
          if (tws[i] >= t) { tw = tws[i]; break; }           // the instance with the smallest ring that holds the tile
    }
  }
  // The rule above is about workgroups that run layer after layer on a chip they do not fill.  With
  // one layer per workgroup the launch is short however few workgroups it has, and the two-pass
  // kernels pay five launches before their first byte: one layer of 1 x 4096 tokens as 32 tiles of
  // 128 takes 0.049 ms (score + select) against 0.079 ms.
  if (!any_fill && layers_per_group > 1 &&
      (int64_t)B * layer_groups * tiles * HC * 100 < (int64_t)resident * need)
    return p;
  p.eligible = 2;
  p.tw = tw;
  p.HC = HC;
  p.tile_tokens = tile;
  p.tiles_per_seq = tiles;
  p.seqs_per_launch = resident / (tiles * HC);
  p.resident = resident;
  p.bs_shift = bs_shift;
  p.waves = waves;
  p.launches = 0;
  p.layer_groups = layer_groups;
  p.layers_per_group = layers_per_group;
  if (layer_groups > 1) p.seqs_per_launch = B;      // one launch by construction
  if (host_lens && (int64_t)B * tiles * HC > resident) {
    // Several launches, and the lengths are known: a launch takes as long as its tiles are
    // long, however many of its workgroups have work, so the tile size that packs the
    // sequences into the fewest tile-lengths wins (64 sequences of 2k-32k tokens, 1.12 M in all:
    // 1124 tiles of 1024 tokens are 4.4 launches' worth and take five, 5 x 1024 tile-lengths;
    // 1777 tiles of 640 fill seven launches to 98 %, 7 x 640).
    const int granule = (kv_dtype == TRI_KV_FP8_E4M3 || (D == 64 && G <= 4)) ? 128 : 64;
    int64_t best_cost = -1;
    for (int cand = tw; cand >= tw / 2 && cand >= 128; cand -= granule) {
      const int per_seq = ceil_div(Tmax, cand) * HC;
      if (per_seq > resident) break;
      const int n = host_pack_launches(host_lens, B, cand, HC, resident);
      const int64_t cost = (int64_t)n * (cand + 32);      // 32 tokens' worth of fixed work per launch and layer
      if (best_cost < 0 || cost < best_cost) {
        best_cost = cost;
        p.tile_tokens = cand;
        p.tiles_per_seq = ceil_div(Tmax, cand);
        p.seqs_per_launch = resident / per_seq;
        p.launches = n;
      }
    }
  }
  return p;
}

hipError_t launch_fused_mfma(const FusedLaunch& a, hipStream_t s) {
  FusedArgs k{};
  k.k_layers = a.k_layers;
  k.k_scale_layers = a.k_scale_layers;
  k.block_table = a.block_table;
  k.seq_lens = a.seq_lens;
  k.prefill_lens = a.prefill_lens;
  k.coef = nullptr;   // this kernel takes its coefficients from bmat
  k.xchg = a.xchg;
  k.fin = a.fin;
  k.status = a.status;
  k.stride_block = a.stride_block; k.stride_token = a.stride_token; k.stride_head = a.stride_head;
  k.L = a.L; k.Hkv = a.Hkv; k.A = a.A; k.G = a.G; k.HC = a.plan.HC;
  k.block_size = a.block_size; k.bs_shift = a.plan.bs_shift;
  k.block_table_pitch = a.block_table ? a.block_table_pitch : -1;
  k.tiles_per_seq = a.plan.tiles_per_seq; k.tile_tokens = a.plan.tile_tokens;
  k.layer_groups = a.plan.layer_groups > 1 ? a.plan.layer_groups : 1;
  k.layers_per_group = k.layer_groups > 1 ? a.plan.layers_per_group : a.L;
  k.fin_part = a.fin_part;
  if (k.layer_groups > 1 && (!a.fin_part || (int64_t)k.layer_groups * k.layers_per_group < a.L)) return hipErrorInvalidValue;
  k.seq_base = 0; k.num_seqs = a.B * k.layer_groups; k.Tmax = a.Tmax;
  k.normalize = a.normalize; k.window_size = a.window_size; k.protect_prefill = a.protect_prefill;
  k.group_reduce = a.group_reduce; k.layer_reduce = a.layer_reduce;
  k.spin_ticks = resident_spin_ticks();
  k.seq_launch = a.pack;
  k.seq_wg_base = a.pack + a.B;
  const LaunchShape shape{a.plan.seqs_per_launch, a.plan.resident, a.B, a.plan.launches};
  const int64_t words = (int64_t)a.B * a.L * k.tiles_per_seq * a.A * 2;
  const bool il = a.rope_style == TRI_ROPE_INTERLEAVED;
  uint4* bmat = reinterpret_cast<uint4*>(a.bmat);
  const int QG = a.G > 4 ? 2 : 1;
  const bool fp8 = a.kv_dtype == TRI_KV_FP8_E4M3;
  const bool fp16 = a.kv_dtype == TRI_KV_FP16;
  if (a.kv_dtype != TRI_KV_BF16 && !fp8 && !fp16) return hipErrorInvalidValue;
  if (a.NO <= 0 || a.NO > kMaxOffsets || (a.D != 128 && a.D != 64 && a.D != 256)) return hipErrorInvalidValue;
  if (a.D != 128 && fp8) return hipErrorInvalidValue;
  auto prep_launch = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3((unsigned)a.L, (unsigned)a.B), dim3(kPrepThreads), 0, s, a.folded, a.omega,
                       a.offsets, a.NO, a.round_start, a.L, a.Hkv, a.G, a.A, QG, bmat, a.xchg, words, a.status);
  };
  if (fp8) {
    if (il) prep_launch(prep_mfma_kernel<TRI_KV_FP8_E4M3, true, 128>);
    else prep_launch(prep_mfma_kernel<TRI_KV_FP8_E4M3, false, 128>);
  } else if (fp16) {
    if (a.D == 64) {
      if (il) prep_launch(prep_mfma_kernel<TRI_KV_FP16, true, 64>);
      else prep_launch(prep_mfma_kernel<TRI_KV_FP16, false, 64>);
    } else if (a.D == 256) {
      if (il) prep_launch(prep_mfma_kernel<TRI_KV_FP16, true, 256>);
      else prep_launch(prep_mfma_kernel<TRI_KV_FP16, false, 256>);
    } else {
      if (il) prep_launch(prep_mfma_kernel<TRI_KV_FP16, true, 128>);
      else prep_launch(prep_mfma_kernel<TRI_KV_FP16, false, 128>);
    }
  } else {
    if (a.D == 64) {
      if (il) prep_launch(prep_mfma_kernel<TRI_KV_BF16, true, 64>);
      else prep_launch(prep_mfma_kernel<TRI_KV_BF16, false, 64>);
    } else if (a.D == 256) {
      if (il) prep_launch(prep_mfma_kernel<TRI_KV_BF16, true, 256>);
      else prep_launch(prep_mfma_kernel<TRI_KV_BF16, false, 256>);
    } else {
      if (il) prep_launch(prep_mfma_kernel<TRI_KV_BF16, true, 128>);
      else prep_launch(prep_mfma_kernel<TRI_KV_BF16, false, 128>);
    }
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  if (fp8)
    e = il ? launch_mfma_tw<TRI_KV_FP8_E4M3, true>(k, bmat, a.plan.tw, a.plan.waves, a.D, shape, s)
           : launch_mfma_tw<TRI_KV_FP8_E4M3, false>(k, bmat, a.plan.tw, a.plan.waves, a.D, shape, s);
  else if (fp16)
    e = il ? launch_mfma_tw<TRI_KV_FP16, true>(k, bmat, a.plan.tw, a.plan.waves, a.D, shape, s)
           : launch_mfma_tw<TRI_KV_FP16, false>(k, bmat, a.plan.tw, a.plan.waves, a.D, shape, s);
  else
    e = il ? launch_mfma_tw<TRI_KV_BF16, true>(k, bmat, a.plan.tw, a.plan.waves, a.D, shape, s)
           : launch_mfma_tw<TRI_KV_BF16, false>(k, bmat, a.plan.tw, a.plan.waves, a.D, shape, s);
  if (e != hipSuccess || k.layer_groups <= 1 || a.skip_layer_reduce) return e;
  const int64_t count = (int64_t)a.B * a.Hkv * a.Tmax;
  hipLaunchKernelGGL(fused_layer_reduce_kernel, dim3((unsigned)ceil_div64(count, 256)), dim3(256), 0, s, a.fin_part, a.fin,
                     count, k.layer_groups, a.layer_reduce, a.L);
  return hipGetLastError();
}

}  // namespace tri
