// Device-side building blocks shared by the scoring kernels (gfx950, wave64): DPP row
// reduction, element decoding, row loads.
#pragma once

#include "tri_common.h"

namespace tri {
namespace {

// cos and sin of a phase that is an fp32 value, evaluated in double and rounded to fp32 once:
// the correctly rounded value of what torch.cos(t * omega) approximates in fp32
// (core/scoring.py:322-324).  Four-term Cody-Waite reduction by pi/2 (33-bit pieces: n * piece
// is exact inside an fma for n < 2^20, and the error stays far below an fp32 half-ulp up to
// phases of 2^30), then the classic minimax polynomials of degree 13 / 14 on [-pi/4, pi/4].
// About 40 fp64 instructions; the library's cos() and sin() each run a full-range reduction of
// several hundred.  Compared on the host with libm over 77 million phases of all magnitudes
// and next to multiples of pi/2: no fp32 result differs.
__device__ __forceinline__ void phase_cos_sin(float phase, float& c_out, float& s_out) {
  const double x = (double)phase;
  const double n = __builtin_rint(x * 6.36619772367581382433e-01);
  double r = __builtin_fma(-n, 1.57079632673412561417e+00, x);
  r = __builtin_fma(-n, 6.07710050630396597660e-11, r);
  r = __builtin_fma(-n, 2.02226624871116645580e-21, r);
  r = __builtin_fma(-n, 8.47842766036889956997e-32, r);
  const double z = r * r;
  const double ps = -1.66666666666666324348e-01 + z * (8.33333333332248946124e-03 + z * (-1.98412698298579493134e-04 +
                    z * (2.75573137070700676789e-06 + z * (-2.50507602534068634195e-08 + z * 1.58969099521155010221e-10))));
  const double pc = 4.16666666666666019037e-02 + z * (-1.38888888888741095749e-03 + z * (2.48015872894767294178e-05 +
                    z * (-2.75573143513906633035e-07 + z * (2.08757232129817482790e-09 + z * -1.13596475577881948265e-11))));
  const double sr = r + r * z * ps;
  const double cr = 1.0 - 0.5 * z + z * z * pc;
  const int q = (int)(long long)n & 3;
  const double c = q == 0 ? cr : q == 1 ? -sr : q == 2 ? -cr : sr;
  const double s = q == 0 ? sr : q == 1 ? cr : q == 2 ? -sr : -cr;
  c_out = (float)c;
  s_out = (float)s;
}

template <int CTRL>
__device__ __forceinline__ float dpp(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
constexpr int kDppXor1 = 0xB1;        // quad_perm:[1,0,3,2]
constexpr int kDppXor2 = 0x4E;        // quad_perm:[2,3,0,1]
constexpr int kDppHalfMirror = 0x141; // row_half_mirror
constexpr int kDppRor8 = 0x128;       // row_ror:8

// Sum four per-lane partials over the LPH lanes of a row.  Returns the total of
// query head (2*b0 + b1) of this lane.
template <int LPH>
__device__ __forceinline__ float reduce_row(const float (&a)[4], bool b0, bool b1) {
  const float keep_a = b0 ? a[2] : a[0];
  const float keep_b = b0 ? a[3] : a[1];
  const float send_a = b0 ? a[0] : a[2];
  const float send_b = b0 ? a[1] : a[3];
  const float ra = keep_a + dpp<kDppXor1>(send_a);
  const float rb = keep_b + dpp<kDppXor1>(send_b);
  const float keep = b1 ? rb : ra;
  const float send = b1 ? ra : rb;
  float r = keep + dpp<kDppXor2>(send);
  if (LPH >= 8) r += dpp<kDppHalfMirror>(r);
  if (LPH >= 16) r += dpp<kDppRor8>(r);
  return r;
}

template <int DT>
__device__ __forceinline__ float elem_lo(uint32_t w);
template <int DT>
__device__ __forceinline__ float elem_hi(uint32_t w);
template <>
__device__ __forceinline__ float elem_lo<TRI_KV_BF16>(uint32_t w) { return __uint_as_float(w << 16); }
template <>
__device__ __forceinline__ float elem_hi<TRI_KV_BF16>(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
template <>
__device__ __forceinline__ float elem_lo<TRI_KV_FP16>(uint32_t w) {
  return (float)__builtin_bit_cast(_Float16, (unsigned short)(w & 0xffffu));
}
template <>
__device__ __forceinline__ float elem_hi<TRI_KV_FP16>(uint32_t w) {
  return (float)__builtin_bit_cast(_Float16, (unsigned short)(w >> 16));
}

// fp8 e4m3 (OCP encoding on gfx950): byte SEL of a 32-bit word.
template <int SEL>
__device__ __forceinline__ float fp8_byte(uint32_t w) {
  return __builtin_amdgcn_cvt_f32_fp8((int)w, SEL);
}

template <int DT>
constexpr int elem_size() { return DT == TRI_KV_FP8_E4M3 ? 1 : 2; }

// Pointers fetched from the per-layer pointer table are generic to the compiler;
// the casts below tell it they are global memory, so it emits global (not flat) loads
// and can keep a wave-uniform base in scalar registers.
typedef const __attribute__((address_space(1))) char* GlobalBytes;
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef const __attribute__((address_space(1))) u32x4* GlobalU4;

typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef const __attribute__((address_space(1))) u32x2* GlobalU2;
typedef const __attribute__((address_space(1))) float* GlobalF32;

// 2-byte elements: lo/hi are 16 bytes each.  fp8: "half" uses lo.xy (8 real parts) and
// hi.xy (8 imaginary parts), "interleaved" uses the 16 bytes of lo; `scale` is the
// row's dequantisation scale (the score is homogeneous of degree one in the key, so
// the scale multiplies the reduced score once).
struct RowData {
  uint4 lo;  // half: 8 real parts          interleaved: pairs 0-3
  uint4 hi;  // half: 8 imaginary parts     interleaved: pairs 4-7
  float scale;
};

// Real and imaginary part of this lane's pair p (0..7).
template <int DT, bool IL>
__device__ __forceinline__ void unpack_pair(const RowData& d, int p, float& kr, float& ki) {
  const uint32_t* lo = reinterpret_cast<const uint32_t*>(&d.lo);
  const uint32_t* hi = reinterpret_cast<const uint32_t*>(&d.hi);
  if constexpr (DT == TRI_KV_FP8_E4M3) {
    if (IL) {
      const uint32_t w = lo[p >> 1];
      kr = (p & 1) ? fp8_byte<2>(w) : fp8_byte<0>(w);
      ki = (p & 1) ? fp8_byte<3>(w) : fp8_byte<1>(w);
    } else {
      const uint32_t wr = lo[p >> 2], wi = hi[p >> 2];
      switch (p & 3) {
        case 0: kr = fp8_byte<0>(wr); ki = fp8_byte<0>(wi); break;
        case 1: kr = fp8_byte<1>(wr); ki = fp8_byte<1>(wi); break;
        case 2: kr = fp8_byte<2>(wr); ki = fp8_byte<2>(wi); break;
        default: kr = fp8_byte<3>(wr); ki = fp8_byte<3>(wi); break;
      }
    }
  } else if (IL) {
    const uint32_t w = (p < 4) ? lo[p] : hi[p - 4];
    kr = elem_lo<DT>(w);
    ki = elem_hi<DT>(w);
  } else {
    const uint32_t wr = lo[p >> 1], wi = hi[p >> 1];
    kr = (p & 1) ? elem_hi<DT>(wr) : elem_lo<DT>(wr);
    ki = (p & 1) ? elem_hi<DT>(wi) : elem_lo<DT>(wi);
  }
}

// 16-byte buffer load: scalar descriptor (row base) + scalar byte offset + per-lane
// byte offset, so a wave-uniform row costs no vector instruction for addressing.
__device__ __forceinline__ uint4 buffer_load16(__amdgpu_buffer_rsrc_t rsrc, uint32_t lane_off, uint32_t sgpr_off) {
  const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)lane_off, (int)sgpr_off, 0);
  return uint4{v.x, v.y, v.z, v.w};
}

__device__ __forceinline__ uint4 buffer_load8(__amdgpu_buffer_rsrc_t rsrc, uint32_t lane_off, uint32_t sgpr_off) {
  const u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(rsrc, (int)lane_off, (int)sgpr_off, 0);
  return uint4{v.x, v.y, 0, 0};
}
__device__ __forceinline__ float buffer_load_f32(__amdgpu_buffer_rsrc_t rsrc, uint32_t lane_off, uint32_t sgpr_off) {
  return __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)lane_off, (int)sgpr_off, 0));
}

}  // namespace
}  // namespace tri
