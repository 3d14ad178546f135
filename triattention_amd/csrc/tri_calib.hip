// Calibration: per-query-head frequency statistics from captured query states (gfx950).
//
// For one layer's captured queries q_rot[H][T][D] (after RoPE, times the attention scale) and
// the rotary tables cos / sin [T][D], all in the model's 16-bit dtype:
//
//   q_base = invert_rope(q_rot, cos, sin, scale)        scripts/calibrate.py:47-82
//   z[t][f] = complex pair f of q_base[t]               scripts/calibrate.py:85-98
//   mean_f z, mean_f |z| over the T tokens, per head    scripts/calibrate.py:199-224
//
// The reference does the inversion with tensors of the model dtype, so every elementwise
// operation rounds to that dtype; the kernel evaluates the same operations in fp32 and rounds
// after each one (`rnd`), which is what a 16-bit elementwise op is.  Means are fp32.
//
// One pass over q_rot (the only large operand: H*T*D*2 bytes): a workgroup takes a chunk of
// tokens of one head, a thread two adjacent frequency pairs (4-byte loads), token lanes are
// folded through LDS, chunk partials are summed in double by a second small kernel.
#include <cstring>

#include "tri_common.h"

namespace tri {
namespace {

constexpr int kCalibThreads = 256;
constexpr int kCalibChunk = 256;      // tokens per workgroup

// Round an fp32 value to the 16-bit dtype (nearest even) and widen it again.  Written with the
// conversion instructions themselves: expressed as casts, (float)(__bf16)(a * b) - ... had its
// inner rounding dropped by the compiler (the product went into an fma unrounded), and the
// rounding after every operation is the whole point here.
template <int DT>
__device__ __forceinline__ float rnd(float x) {
  if constexpr (DT == TRI_KV_BF16) {
    uint32_t packed;
    asm("v_cvt_pk_bf16_f32 %0, %1, %1" : "=v"(packed) : "v"(x));
    return __uint_as_float(packed << 16);
  } else {
    float half_bits, out;
    asm("v_cvt_f16_f32 %0, %1" : "=v"(half_bits) : "v"(x));
    asm("v_cvt_f32_f16 %0, %1" : "=v"(out) : "v"(half_bits));
    return out;
  }
}
template <int DT>
__device__ __forceinline__ float widen(uint32_t half_bits) {
  if constexpr (DT == TRI_KV_BF16) return __uint_as_float(half_bits << 16);
  else return (float)__builtin_bit_cast(_Float16, (unsigned short)half_bits);
}
template <int DT>
__device__ __forceinline__ void widen2(uint32_t w, float& lo, float& hi) {
  lo = widen<DT>(w & 0xffffu);
  hi = widen<DT>(w >> 16);
}

// One complex pair of the un-rotated query from the scaled-down operands: (b0, b1) the pair's
// two elements of q_rot / scale, (cu0, cu1) / (su0, su1) the entries of cos / scale and
// sin / scale at the same two positions; half style: elements f and f + D/2, interleaved: 2f
// and 2f + 1.
template <int DT, bool IL>
__device__ __forceinline__ void unrotate_pair(float b0, float b1, float cu0, float cu1, float su0, float su1,
                                              float& re, float& im) {
  if constexpr (IL) {
    // scripts/calibrate.py:62-77
    float det = rnd<DT>(rnd<DT>(cu0 * cu1) + rnd<DT>(su0 * su1));
    det = fmaxf(det, rnd<DT>(1e-12f));
    re = rnd<DT>(__fdiv_rn(rnd<DT>(rnd<DT>(b0 * cu1) + rnd<DT>(b1 * su0)), det));
    im = rnd<DT>(__fdiv_rn(rnd<DT>(rnd<DT>(b1 * cu0) - rnd<DT>(b0 * su1)), det));
  } else {
    // base*cos - rotate_half(base)*sin with rotate_half = (-second half, first half)  (:38-44, :82)
    re = rnd<DT>(rnd<DT>(b0 * cu0) - rnd<DT>(-b1 * su0));
    im = rnd<DT>(rnd<DT>(b1 * cu1) - rnd<DT>(b0 * su1));
  }
}

struct CalibArgs {
  const unsigned short* q;
  const unsigned short* cos;      // cos / scale and sin / scale when the scale is not 1 (unit_tables_kernel)
  const unsigned short* sin;
  int64_t stride_head, stride_token;
  int H, T, D, chunks;
  float scale;            // already rounded to the 16-bit dtype
  float* partial;         // [H][chunks][D/2][3]
};

// cos / scale and sin / scale, once per table entry instead of once per head.
template <int DT>
__global__ void unit_tables_kernel(const unsigned short* cos, const unsigned short* sin, int64_t n, float scale,
                                   unsigned short* cos_unit, unsigned short* sin_unit) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const float c = rnd<DT>(__fdiv_rn(widen<DT>(cos[i]), scale)), sn = rnd<DT>(__fdiv_rn(widen<DT>(sin[i]), scale));
  if constexpr (DT == TRI_KV_BF16) {
    cos_unit[i] = (unsigned short)(__float_as_uint(c) >> 16);
    sin_unit[i] = (unsigned short)(__float_as_uint(sn) >> 16);
  } else {
    cos_unit[i] = __builtin_bit_cast(unsigned short, (_Float16)c);     // exact: c is an fp16 value
    sin_unit[i] = __builtin_bit_cast(unsigned short, (_Float16)sn);
  }
}

// UNIT: the scale is 1, q_rot / scale is q_rot.  HG heads per thread share the table entries.
template <int DT, bool IL, bool UNIT, int HG>
__global__ __launch_bounds__(kCalibThreads) void qstats_partial_kernel(CalibArgs a) {
  __shared__ float red[kCalibThreads][6];
  const int h0 = blockIdx.y * HG, chunk = blockIdx.x;
  const int F = a.D / 2;
  const int tpp = F / 2;                          // threads per token: two pairs each
  const int p = threadIdx.x % tpp;                // pairs 2p, 2p+1
  const int tl = threadIdx.x / tpp, lanes = kCalibThreads / tpp;
  const int t0 = chunk * kCalibChunk, t1 = min(t0 + kCalibChunk, a.T);
  // element offsets of the two 4-byte words this thread reads from a row of D elements
  const int e0 = IL ? 4 * p : 2 * p;
  const int e1 = IL ? 4 * p + 2 : F + 2 * p;
  float acc[HG][6];                               // (re, im, |z|) of pair 2p, then of pair 2p+1
#pragma unroll
  for (int g = 0; g < HG; ++g)
#pragma unroll
    for (int i = 0; i < 6; ++i) acc[g][i] = 0.f;
  for (int t = t0 + tl; t < t1; t += lanes) {
    const unsigned short* cr = a.cos + (int64_t)t * a.D;
    const unsigned short* sr = a.sin + (int64_t)t * a.D;
    const uint32_t ca = *reinterpret_cast<const uint32_t*>(cr + e0), cb = *reinterpret_cast<const uint32_t*>(cr + e1);
    const uint32_t sa = *reinterpret_cast<const uint32_t*>(sr + e0), sb = *reinterpret_cast<const uint32_t*>(sr + e1);
    float c0, c1, c2, c3, s0, s1, s2, s3;
    widen2<DT>(ca, c0, c1); widen2<DT>(cb, c2, c3);
    widen2<DT>(sa, s0, s1); widen2<DT>(sb, s2, s3);
    uint32_t qa[HG], qb[HG];
#pragma unroll
    for (int g = 0; g < HG; ++g) {
      const unsigned short* qr = a.q + (int64_t)min(h0 + g, a.H - 1) * a.stride_head + (int64_t)t * a.stride_token;
      qa[g] = *reinterpret_cast<const uint32_t*>(qr + e0);
      qb[g] = *reinterpret_cast<const uint32_t*>(qr + e1);
    }
#pragma unroll
    for (int g = 0; g < HG; ++g) {
      float q0, q1, q2, q3;
      widen2<DT>(qa[g], q0, q1); widen2<DT>(qb[g], q2, q3);
      if constexpr (!UNIT) {
        q0 = rnd<DT>(__fdiv_rn(q0, a.scale)); q1 = rnd<DT>(__fdiv_rn(q1, a.scale));
        q2 = rnd<DT>(__fdiv_rn(q2, a.scale)); q3 = rnd<DT>(__fdiv_rn(q3, a.scale));
      }
      float re0, im0, re1, im1;
      if constexpr (IL) {     // word a = pair 2p (re, im), word b = pair 2p+1
        unrotate_pair<DT, IL>(q0, q1, c0, c1, s0, s1, re0, im0);
        unrotate_pair<DT, IL>(q2, q3, c2, c3, s2, s3, re1, im1);
      } else {                // word a = first-half elements 2p, 2p+1; word b = their partners
        unrotate_pair<DT, IL>(q0, q2, c0, c2, s0, s2, re0, im0);
        unrotate_pair<DT, IL>(q1, q3, c1, c3, s1, s3, re1, im1);
      }
      acc[g][0] += re0; acc[g][1] += im0; acc[g][2] += __fsqrt_rn(fmaf(im0, im0, re0 * re0));
      acc[g][3] += re1; acc[g][4] += im1; acc[g][5] += __fsqrt_rn(fmaf(im1, im1, re1 * re1));
    }
  }
#pragma unroll
  for (int g = 0; g < HG; ++g) {
    if (g > 0) __syncthreads();
#pragma unroll
    for (int i = 0; i < 6; ++i) red[threadIdx.x][i] = acc[g][i];
    __syncthreads();
    if (threadIdx.x < tpp && h0 + g < a.H) {
      float sum[6] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      for (int l = 0; l < lanes; ++l)
#pragma unroll
        for (int i = 0; i < 6; ++i) sum[i] += red[l * tpp + p][i];
      float* out = a.partial + (((int64_t)(h0 + g) * a.chunks + chunk) * F + 2 * p) * 3;
#pragma unroll
      for (int i = 0; i < 6; ++i) out[i] = sum[i];
    }
  }
}

// Sum of the chunk partials in double, divided by the token count.  A workgroup takes 32
// (head, pair) entries; its eight lanes per entry walk the chunks and meet in LDS.
__global__ __launch_bounds__(256) void qstats_finalize_kernel(const float* partial, int H, int chunks, int F, int T,
                                                              float* out_real, float* out_imag, float* out_abs) {
  __shared__ double red[8][32][3];
  const int e = threadIdx.x & 31, cl = threadIdx.x >> 5;
  const int idx = blockIdx.x * 32 + e;                         // (head, pair)
  double s[3] = {0.0, 0.0, 0.0};
  if (idx < H * F) {
    const int h = idx / F, f = idx - h * F;
    for (int c = cl; c < chunks; c += 8) {
      const float* p = partial + (((int64_t)h * chunks + c) * F + f) * 3;
      s[0] += (double)p[0];
      s[1] += (double)p[1];
      s[2] += (double)p[2];
    }
  }
  red[cl][e][0] = s[0]; red[cl][e][1] = s[1]; red[cl][e][2] = s[2];
  __syncthreads();
  if (cl == 0 && idx < H * F) {
    for (int l = 1; l < 8; ++l) { s[0] += red[l][e][0]; s[1] += red[l][e][1]; s[2] += red[l][e][2]; }
    out_real[idx] = (float)(s[0] / (double)T);
    out_imag[idx] = (float)(s[1] / (double)T);
    out_abs[idx] = (float)(s[2] / (double)T);
  }
}

// torch.tensor(scale, dtype=...) on the host: round to nearest even into the 16-bit type.
float round_scale(float scale, int dtype) {
  if (dtype == TRI_KV_FP16) return (float)(_Float16)scale;
  uint32_t u;
  memcpy(&u, &scale, 4);
  u += 0x7fffu + ((u >> 16) & 1u);
  u &= 0xffff0000u;
  float r;
  memcpy(&r, &u, 4);
  return r;
}

}  // namespace

constexpr int kCalibHeads = 4;     // heads per thread

int64_t qstats_partial_bytes(int H, int T, int D) {
  return (int64_t)H * ceil_div(T, kCalibChunk) * (D / 2) * 3 * (int64_t)sizeof(float);
}

int64_t qstats_workspace_bytes(int H, int T, int D) {
  // chunk partials, then room for cos / scale and sin / scale
  return ceil_div64(qstats_partial_bytes(H, T, D), 16) * 16 + 2 * (int64_t)T * D * 2;
}

namespace {

template <int DT, bool IL, bool UNIT>
void launch_partial(const CalibArgs& a, hipStream_t s) {
  const dim3 grid(a.chunks, ceil_div(a.H, kCalibHeads));
  hipLaunchKernelGGL((qstats_partial_kernel<DT, IL, UNIT, kCalibHeads>), grid, dim3(kCalibThreads), 0, s, a);
}

template <int DT>
hipError_t launch_typed(CalibArgs a, const QStatsLaunch& q, hipStream_t s) {
  const bool il = q.rope_style == TRI_ROPE_INTERLEAVED;
  if (a.scale == 1.f) {
    if (il) launch_partial<DT, true, true>(a, s); else launch_partial<DT, false, true>(a, s);
    return hipGetLastError();
  }
  char* tables = static_cast<char*>(q.workspace) + ceil_div64(qstats_partial_bytes(q.H, q.T, q.D), 16) * 16;
  unsigned short* cos_unit = reinterpret_cast<unsigned short*>(tables);
  unsigned short* sin_unit = cos_unit + (int64_t)q.T * q.D;
  const int64_t n = (int64_t)q.T * q.D;
  hipLaunchKernelGGL(unit_tables_kernel<DT>, dim3((unsigned)ceil_div64(n, 256)), dim3(256), 0, s, a.cos, a.sin, n,
                     a.scale, cos_unit, sin_unit);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  a.cos = cos_unit;
  a.sin = sin_unit;
  if (il) launch_partial<DT, true, false>(a, s); else launch_partial<DT, false, false>(a, s);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_qstats(const QStatsLaunch& q, hipStream_t s) {
  CalibArgs a{};
  a.q = static_cast<const unsigned short*>(q.q_rot);
  a.cos = static_cast<const unsigned short*>(q.cos);
  a.sin = static_cast<const unsigned short*>(q.sin);
  a.stride_head = q.stride_head; a.stride_token = q.stride_token;
  a.H = q.H; a.T = q.T; a.D = q.D;
  a.chunks = ceil_div(q.T, kCalibChunk);
  a.scale = round_scale(q.scale, q.dtype);
  a.partial = static_cast<float*>(q.workspace);
  hipError_t e = q.dtype == TRI_KV_BF16 ? launch_typed<TRI_KV_BF16>(a, q, s) : launch_typed<TRI_KV_FP16>(a, q, s);
  if (e != hipSuccess) return e;
  const int n = q.H * (q.D / 2);
  hipLaunchKernelGGL(qstats_finalize_kernel, dim3(ceil_div(n, 32)), dim3(256), 0, s, a.partial, q.H, a.chunks, q.D / 2,
                     q.T, q.out_real, q.out_imag, q.out_abs);
  return hipGetLastError();
}

}  // namespace tri
