// Device-side building blocks shared by every GroupNorm kernel: element types and 128-bit lane
// vectors, conversions, activations and their derivatives, and fixed-order reductions.
// gfx950 (CDNA4) only: wave64, 256 CUs in 8 XCDs.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "gn_plan.h"

namespace gn {

// ---------------------------------------------------------------------------------------------
// Element types.  Storage types are plain bit containers; all arithmetic is done in the
// accumulation type (float for f32/f16/bf16, double for f64), with one rounding on store.
// The reference instead evaluates the half/bfloat16 forward in 16-bit arithmetic
// (src/gnnhwc/csrc/gn_kernel.cu:294-303); torch's GroupNorm, which defines the expected results,
// computes in fp32, and so does this code.
// ---------------------------------------------------------------------------------------------
struct bf16_t { uint16_t bits; };
typedef _Float16 f16_t;

template <typename T> struct acc_of { typedef float type; };
template <> struct acc_of<double> { typedef double type; };

template <typename T> struct vec_of { static constexpr int value = 16 / (int)sizeof(T); };

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef double f64x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float bf16_bits_to_float(uint32_t hi16_in_place) {
  return __builtin_bit_cast(float, hi16_in_place);
}
// Round-to-nearest-even float -> bfloat16 pair; clang lowers the fptrunc to v_cvt_pk_bf16_f32 on gfx950.
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  f32x2 f = {lo, hi};
  bf16x2 b = __builtin_convertvector(f, bf16x2);
  return __builtin_bit_cast(uint32_t, b);
}
__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {
  __bf16 b = (__bf16)f;
  return __builtin_bit_cast(uint16_t, b);
}

// ---- lane vectors: VEC elements of T moved by one (ideally 128-bit) access ----
// raw_t is what travels (and what a lane keeps in registers while more loads are in flight);
// unpack / pack convert to and from the accumulation type.
template <typename T, int VEC> struct LaneVec;

// Keeps the memory operations written before it ahead of those written after it in the instruction stream
// (the scheduler is otherwise free to issue independent loads in any order, and loads return in issue order).
__device__ __forceinline__ void issue_order_fence() { asm volatile("" ::: "memory"); }

// Makes a register value opaque to the optimiser.  A kernel that keeps packed rows in registers across
// several passes unpacks them again in every pass; without this the unpacked copies of one pass are
// kept alive for the next, which doubles or triples the registers a 16-bit tile needs.
template <typename R> __device__ __forceinline__ void pin(R &r) { asm volatile("" : "+v"(r)); }

template <> struct LaneVec<float, 4> {
  typedef f32x4 raw_t;
  static __device__ __forceinline__ raw_t load(const float *p) { return *(const raw_t *)p; }
  static __device__ __forceinline__ void store(float *p, raw_t r) { *(raw_t *)p = r; }
  static __device__ __forceinline__ void unpack(raw_t r, float (&v)[4]) { v[0] = r.x; v[1] = r.y; v[2] = r.z; v[3] = r.w; }
  static __device__ __forceinline__ raw_t pack(const float (&v)[4]) { return raw_t{v[0], v[1], v[2], v[3]}; }
};
template <> struct LaneVec<double, 2> {
  typedef f64x2 raw_t;
  static __device__ __forceinline__ raw_t load(const double *p) { return *(const raw_t *)p; }
  static __device__ __forceinline__ void store(double *p, raw_t r) { *(raw_t *)p = r; }
  static __device__ __forceinline__ void unpack(raw_t r, double (&v)[2]) { v[0] = r.x; v[1] = r.y; }
  static __device__ __forceinline__ raw_t pack(const double (&v)[2]) { return raw_t{v[0], v[1]}; }
};
template <> struct LaneVec<f16_t, 8> {
  typedef f16x8 raw_t;
  static __device__ __forceinline__ raw_t load(const f16_t *p) { return *(const raw_t *)p; }
  static __device__ __forceinline__ void store(f16_t *p, raw_t r) { *(raw_t *)p = r; }
  static __device__ __forceinline__ void unpack(raw_t r, float (&v)[8]) {
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = (float)r[j];
  }
  static __device__ __forceinline__ raw_t pack(const float (&v)[8]) {
    raw_t r;
#pragma unroll
    for (int j = 0; j < 8; ++j) r[j] = (_Float16)v[j];  // v_cvt_f16_f32, round to nearest even
    return r;
  }
};
template <> struct LaneVec<bf16_t, 8> {
  typedef u32x4 raw_t;
  static __device__ __forceinline__ raw_t load(const bf16_t *p) { return *(const raw_t *)p; }
  static __device__ __forceinline__ void store(bf16_t *p, raw_t r) { *(raw_t *)p = r; }
  static __device__ __forceinline__ void unpack(raw_t r, float (&v)[8]) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      v[2 * j] = bf16_bits_to_float(r[j] << 16);
      v[2 * j + 1] = bf16_bits_to_float(r[j] & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ raw_t pack(const float (&v)[8]) {
    raw_t r;
#pragma unroll
    for (int j = 0; j < 4; ++j) r[j] = pack_bf16x2(v[2 * j], v[2 * j + 1]);
    return r;
  }
};
// scalar fall-back: any C, any alignment
template <> struct LaneVec<float, 1> {
  typedef float raw_t;
  static __device__ __forceinline__ raw_t load(const float *p) { return *p; }
  static __device__ __forceinline__ void store(float *p, raw_t r) { *p = r; }
  static __device__ __forceinline__ void unpack(raw_t r, float (&v)[1]) { v[0] = r; }
  static __device__ __forceinline__ raw_t pack(const float (&v)[1]) { return v[0]; }
};
template <> struct LaneVec<double, 1> {
  typedef double raw_t;
  static __device__ __forceinline__ raw_t load(const double *p) { return *p; }
  static __device__ __forceinline__ void store(double *p, raw_t r) { *p = r; }
  static __device__ __forceinline__ void unpack(raw_t r, double (&v)[1]) { v[0] = r; }
  static __device__ __forceinline__ raw_t pack(const double (&v)[1]) { return v[0]; }
};
template <> struct LaneVec<f16_t, 1> {
  typedef f16_t raw_t;
  static __device__ __forceinline__ raw_t load(const f16_t *p) { return *p; }
  static __device__ __forceinline__ void store(f16_t *p, raw_t r) { *p = r; }
  static __device__ __forceinline__ void unpack(raw_t r, float (&v)[1]) { v[0] = (float)r; }
  static __device__ __forceinline__ raw_t pack(const float (&v)[1]) { return (_Float16)v[0]; }
};
template <> struct LaneVec<bf16_t, 1> {
  typedef uint16_t raw_t;
  static __device__ __forceinline__ raw_t load(const bf16_t *p) { return p->bits; }
  static __device__ __forceinline__ void store(bf16_t *p, raw_t r) { p->bits = r; }
  static __device__ __forceinline__ void unpack(raw_t r, float (&v)[1]) { v[0] = bf16_bits_to_float((uint32_t)r << 16); }
  static __device__ __forceinline__ raw_t pack(const float (&v)[1]) { return float_to_bf16_bits(v[0]); }
};

// Streaming forms of the lane-vector accesses (non-temporal hint).  A result row is written once and not read again
// by the kernel that writes it: stored this way it does not wait in the L2 cache for the write-back at the end of
// the kernel (measured on the single-launch kernels: 9 - 13 % shorter launches and shorter gaps between them).
template <typename LV, typename T> __device__ __forceinline__ void store_streaming(T *p, typename LV::raw_t r) {
  __builtin_nontemporal_store(r, (typename LV::raw_t *)p);
}
template <typename LV, typename T> __device__ __forceinline__ typename LV::raw_t load_streaming(const T *p) {
  return __builtin_nontemporal_load((const typename LV::raw_t *)p);
}
// One lane vector of forward results, stored at element `e` of y.  y normally has the data type; float data may also be
// written as a 16-bit type (ydtype GN_F16 / GN_BF16; the host admits nothing else), each value rounded once from the
// fp32 result: the layer that consumes y in half precision then reads half the bytes and no cast kernel runs between.
template <typename T, int VEC, typename A>
__device__ __forceinline__ void store_result(T *y, int64_t e, const A (&v)[VEC], int ydtype) {
  using LV = LaneVec<T, VEC>;
  if constexpr (sizeof(T) == 4) {
    if (ydtype != GN_F32) {
      uint16_t *yp = (uint16_t *)y + e;
      if constexpr (VEC == 4) {
        u32x2 r;
        if (ydtype == GN_BF16) {
          r.x = pack_bf16x2(v[0], v[1]);
          r.y = pack_bf16x2(v[2], v[3]);
        } else {
          const f16x2 lo = {(_Float16)v[0], (_Float16)v[1]}, hi = {(_Float16)v[2], (_Float16)v[3]};
          r.x = __builtin_bit_cast(uint32_t, lo);
          r.y = __builtin_bit_cast(uint32_t, hi);
        }
        __builtin_nontemporal_store(r, (u32x2 *)yp);
      } else {
        const _Float16 h = (_Float16)v[0];
        *yp = ydtype == GN_BF16 ? float_to_bf16_bits(v[0]) : __builtin_bit_cast(uint16_t, h);
      }
      return;
    }
  }
  store_streaming<LV>(y + e, LV::pack(v));
}

// ---- runtime-typed scalar access to parameters / statistics (read once per workgroup) ----
template <typename ACC> __device__ __forceinline__ ACC load_scalar(const void *p, int64_t i, int dtype) {
  switch (dtype) {
    case GN_F32: return (ACC)((const float *)p)[i];
    case GN_F64: return (ACC)((const double *)p)[i];
    case GN_F16: return (ACC)(float)((const _Float16 *)p)[i];
    default: return (ACC)bf16_bits_to_float((uint32_t)((const uint16_t *)p)[i] << 16);
  }
}
// The same read without control flow: the candidate loads of every width are all issued (from `safe`, any
// readable 8-byte-aligned address, when the width does not apply) and the result is selected.  A load under a
// branch makes the compiler drain every outstanding load at the join; this form can sit next to bulk loads.
template <typename ACC> __device__ __forceinline__ ACC load_scalar_flat(const void *p, int64_t i, int dtype, const void *safe) {
  const bool half = dtype == GN_F16 || dtype == GN_BF16;
  const float *pf = dtype == GN_F32 ? (const float *)p + i : (const float *)safe;
  const uint16_t *ph = half ? (const uint16_t *)p + i : (const uint16_t *)safe;
  const float vf = *pf;
  const uint16_t vh = *ph;
  ACC r;
  if constexpr (sizeof(ACC) == 8) {
    const double *pd = dtype == GN_F64 ? (const double *)p + i : (const double *)safe;
    r = (ACC)*pd;
  } else {
    r = (ACC)0;
  }
  const float h16 = (float)__builtin_bit_cast(_Float16, vh);
  const float b16 = bf16_bits_to_float((uint32_t)vh << 16);
  if (dtype == GN_F32) r = (ACC)vf;
  if (dtype == GN_F16) r = (ACC)h16;
  if (dtype == GN_BF16) r = (ACC)b16;
  return r;
}
template <typename ACC> __device__ __forceinline__ void store_scalar(void *p, int64_t i, int dtype, ACC v) {
  switch (dtype) {
    case GN_F32: ((float *)p)[i] = (float)v; break;
    case GN_F64: ((double *)p)[i] = (double)v; break;
    case GN_F16: ((_Float16 *)p)[i] = (_Float16)(float)v; break;
    default: ((uint16_t *)p)[i] = float_to_bf16_bits((float)v); break;
  }
}

// ---------------------------------------------------------------------------------------------
// Activations and derivatives, evaluated in the accumulation type.
// Definitions follow src/gnnhwc/csrc/gn_kernel.cu:62-106 (identity, relu, silu = x/(1+e^-x),
// gelu = x/2 (1+erf(x/sqrt2)), gelu_tanh = x/2 (1+tanh(sqrt(2/pi)(x+0.044715x^3)))), which are also
// the torch definitions (F.relu / F.silu / F.gelu / F.gelu(approximate='tanh')).
// fp32 forms use the hardware exp2 / rcp (1 ulp each), never a fast-math libm.
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }
__device__ __forceinline__ double fast_rcp(double x) { return 1.0 / x; }
// 1 / sqrt(v): hardware estimate (1 ulp) refined by one Newton step; a few instructions where the division
// sequence takes a dozen, and these sit in the serial section every workgroup of a group waits for.
__device__ __forceinline__ float fast_rsqrt(float v) {
  const float r = __builtin_amdgcn_rsqf(v);
  return r * (1.5f - 0.5f * v * r * r);
}
__device__ __forceinline__ double fast_rsqrt(double v) { return 1.0 / sqrt(v); }
// logistic sigmoid 1/(1+e^-x); exp2 overflow to +inf gives rcp(inf) = 0, underflow gives 1.
__device__ __forceinline__ float sigmoid(float x) {
  return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * -1.44269504088896340736f));
}
__device__ __forceinline__ double sigmoid(double x) { return 1.0 / (1.0 + exp(-x)); }
// Standard normal CDF Phi(z) = (1 + erf(z / sqrt 2)) / 2.  fp32: erfc(t / sqrt 2) = exp2(t P(t)) for t = min(|z|, 6),
// P a degree-10 least-squares fit of log2(erfc(t / sqrt 2)) / t on [0, 6] (result: absolute error 8e-8, relative
// error 4e-6, so the left tail of Phi keeps its relative accuracy); straight-line code, no branches.
__device__ __forceinline__ float normal_cdf(float z) {
  const float t = fminf(fabsf(z), 6.0f);
  float p = 2.729510037e-09f;
  p = p * t + -1.013394950e-07f;
  p = p * t + 1.666771318e-06f;
  p = p * t + -1.587480181e-05f;
  p = p * t + 9.414357042e-05f;
  p = p * t + -3.183018466e-04f;
  p = p * t + 5.031143559e-05f;
  p = p * t + 6.909817011e-03f;
  p = p * t + -5.242731270e-02f;
  p = p * t + -4.592229807e-01f;
  p = p * t + -1.151104130e+00f;
  const float h = 0.5f * __builtin_amdgcn_exp2f(t * p);  // Phi(-|z|)
  return z < 0.0f ? h : 1.0f - h;
}
__device__ __forceinline__ double normal_cdf(double z) { return 0.5 * erfc(z * -0.70710678118654752440); }
__device__ __forceinline__ float exp_acc(float x) { return __builtin_amdgcn_exp2f(x * 1.44269504088896340736f); }
__device__ __forceinline__ double exp_acc(double x) { return exp(x); }

// sigmoid(2u) for u = sqrt(2/pi) (z + 0.044715 z^3), with the constants of the exponent folded
__device__ __forceinline__ float sigmoid_2u(float z, float z2) {
  constexpr float k1 = (float)(-2.0 * 0.79788456080286535588 * 1.44269504088896340736);
  constexpr float k3 = (float)(-2.0 * 0.79788456080286535588 * 1.44269504088896340736 * 0.044715);
  return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(z * (z2 * k3 + k1)));
}
__device__ __forceinline__ double sigmoid_2u(double z, double z2) {
  return sigmoid(2.0 * 0.79788456080286535588 * (z + 0.044715 * z2 * z));
}

template <int ACT, typename A> __device__ __forceinline__ A act_fwd(A z) {
  if constexpr (ACT == GN_ACT_IDENTITY) {
    return z;
  } else if constexpr (ACT == GN_ACT_RELU) {
    return z <= (A)0 ? (A)0 : z;  // NaN propagates, like torch.relu
  } else if constexpr (ACT == GN_ACT_SILU) {
    return z * sigmoid(z);
  } else if constexpr (ACT == GN_ACT_GELU) {
    return z * normal_cdf(z);
  } else {
    // 1 + tanh(u) == 2 sigmoid(2u): the same function without the cancellation at u << 0
    return z * sigmoid_2u(z, z * z);
  }
}
template <int ACT, typename A> __device__ __forceinline__ A act_bwd(A z) {
  if constexpr (ACT == GN_ACT_IDENTITY) {
    return (A)1;
  } else if constexpr (ACT == GN_ACT_RELU) {
    return z <= (A)0 ? (A)0 : (A)1;
  } else if constexpr (ACT == GN_ACT_SILU) {
    const A s = sigmoid(z);
    return s * ((A)1 + z * ((A)1 - s));
  } else if constexpr (ACT == GN_ACT_GELU) {
    const A cdf = normal_cdf(z);
    const A pdf = exp_acc((A)-0.5 * z * z) * (A)0.39894228040143267794;
    return cdf + z * pdf;
  } else {
    const A z2 = z * z;
    const A s = sigmoid_2u(z, z2);  // (1 + tanh u) / 2
    const A du2 = z2 * (A)(2.0 * 0.79788456080286535588 * 0.134145) + (A)(2.0 * 0.79788456080286535588);  // 2 du/dz
    // d/dz [z s] = s + z * 2 s (1 - s) * du/dz
    return (z * s * du2) * ((A)1 - s) + s;
  }
}

// ---------------------------------------------------------------------------------------------
// Statistics are carried as (count, mean, M2) triples, the quantities of WelfordData
// (src/gnnhwc/csrc/Welford.h:8-21); the variance is the biased one, M2 / n (Welford.h:66-72 with
// correction 0, gn_kernel.cu:175,254).  Where the reference merges triples pairwise with
// WelfordOps::combine (Welford.h:44-65), sets of triples are merged here with the equivalent exact
// two-pass form, which is a pair of plain sums and therefore reduces with fixed butterfly trees:
//   n = sum n_i,  mean = sum n_i mean_i / n,  M2 = sum (M2_i + n_i (mean_i - mean)^2),
// or, where one pass must do, with the same sums taken about a pivot K that is itself the mean of one of
// the parts (so |K - mean| is a small fraction of the spread and nothing cancels):
//   s1 = sum n_i (mean_i - K),  s2 = sum (M2_i + n_i (mean_i - K)^2),  mean = K + s1 / n,  M2 = s2 - s1^2 / n.
// ---------------------------------------------------------------------------------------------
template <typename A> struct Moments {
  A n, mean, m2;
};
template <typename A> __device__ __forceinline__ A shfl_xor_acc(A v, int mask, int width) {
  return __shfl_xor(v, mask, width);
}
// Cross-lane exchange inside a row of 16 lanes with a DPP modifier (VALU latency, no LDS traffic).
template <int CTRL> __device__ __forceinline__ float dpp_move(float v) {
  const int i = __builtin_bit_cast(int, v);
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(i, i, CTRL, 0xF, 0xF, false));
}
template <int CTRL> __device__ __forceinline__ double dpp_move(double v) {
  const unsigned long long u = __builtin_bit_cast(unsigned long long, v);
  const int lo = (int)(unsigned)u, hi = (int)(unsigned)(u >> 32);
  const unsigned rlo = (unsigned)__builtin_amdgcn_update_dpp(lo, lo, CTRL, 0xF, 0xF, false);
  const unsigned rhi = (unsigned)__builtin_amdgcn_update_dpp(hi, hi, CTRL, 0xF, 0xF, false);
  return __builtin_bit_cast(double, (unsigned long long)rlo | ((unsigned long long)rhi << 32));
}
constexpr int kDppQuadXor1 = 0xB1;       // quad_perm:[1,0,3,2]
constexpr int kDppQuadXor2 = 0x4E;       // quad_perm:[2,3,0,1]
constexpr int kDppRowHalfMirror = 0x141; // lane i <-> 7 - i inside each 8
constexpr int kDppRowMirror = 0x140;     // lane i <-> 15 - i inside each 16
// Sum over `width` consecutive lanes (power of two <= 64, aligned).  Every lane of the segment ends with
// the same bits: each step adds the value of a lane from the other half of the growing group, whose
// members already agree, and floating-point addition is commutative.  The first four steps are DPP
// moves; only widths 32 and 64 need a trip through the LDS crossbar.
template <typename A> __device__ __forceinline__ A segment_sum(A v, int width) {
  if (width >= 2) v += dpp_move<kDppQuadXor1>(v);
  if (width >= 4) v += dpp_move<kDppQuadXor2>(v);
  if (width >= 8) v += dpp_move<kDppRowHalfMirror>(v);
  if (width >= 16) v += dpp_move<kDppRowMirror>(v);
  if (width >= 32) v += shfl_xor_acc(v, 16, 64);
  if (width >= 64) v += shfl_xor_acc(v, 32, 64);
  return v;
}
// Two independent sums at once (their latencies overlap).
template <typename A> __device__ __forceinline__ void segment_sum2(A &a, A &b, int width) {
  if (width >= 2) { a += dpp_move<kDppQuadXor1>(a); b += dpp_move<kDppQuadXor1>(b); }
  if (width >= 4) { a += dpp_move<kDppQuadXor2>(a); b += dpp_move<kDppQuadXor2>(b); }
  if (width >= 8) { a += dpp_move<kDppRowHalfMirror>(a); b += dpp_move<kDppRowHalfMirror>(b); }
  if (width >= 16) { a += dpp_move<kDppRowMirror>(a); b += dpp_move<kDppRowMirror>(b); }
  if (width >= 32) {
    const A oa = shfl_xor_acc(a, 16, 64), ob = shfl_xor_acc(b, 16, 64);
    a += oa;
    b += ob;
  }
  if (width >= 64) {
    const A oa = shfl_xor_acc(a, 32, 64), ob = shfl_xor_acc(b, 32, 64);
    a += oa;
    b += ob;
  }
}
// The same for callers that need the totals in ONE lane of the segment only: segment_leader(width).  Up to a row of 16
// lanes this is the butterfly above; the steps across rows are DPP row broadcasts (lane 15 of a row into the next
// row, lane 31 into the upper half of the wavefront), which cost one addition each where the butterfly's cross-row
// exchanges go through the LDS crossbar (an address computation, a permute and a wait per value and step).
constexpr int kDppRowBcast15 = 0x142, kDppRowBcast31 = 0x143;
template <int CTRL, int ROW_MASK> __device__ __forceinline__ float dpp_rows_add(float v) {
  const int i = __builtin_bit_cast(int, v);
  return v + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, i, CTRL, ROW_MASK, 0xF, false));
}
__device__ __forceinline__ void segment_reduce2(float &a, float &b, int width) {
  if (width >= 2) { a += dpp_move<kDppQuadXor1>(a); b += dpp_move<kDppQuadXor1>(b); }
  if (width >= 4) { a += dpp_move<kDppQuadXor2>(a); b += dpp_move<kDppQuadXor2>(b); }
  if (width >= 8) { a += dpp_move<kDppRowHalfMirror>(a); b += dpp_move<kDppRowHalfMirror>(b); }
  if (width >= 16) { a += dpp_move<kDppRowMirror>(a); b += dpp_move<kDppRowMirror>(b); }
  if (width >= 32) { a = dpp_rows_add<kDppRowBcast15, 0xA>(a); b = dpp_rows_add<kDppRowBcast15, 0xA>(b); }
  if (width >= 64) { a = dpp_rows_add<kDppRowBcast31, 0xC>(a); b = dpp_rows_add<kDppRowBcast31, 0xC>(b); }
}
__device__ __forceinline__ void segment_reduce2(double &a, double &b, int width) { segment_sum2(a, b, width); }
// Lane (inside its segment) that holds the totals after segment_reduce2.
template <typename A> __device__ __forceinline__ int segment_leader(int width) {
  return sizeof(A) == 4 && width >= 32 ? width - 1 : 0;
}
// Segment index of a thread when the workgroup is cut into segments of L lanes (a power of two <= 64), numbered so that
// consecutive segments sit in DIFFERENT wavefronts: the first few groups of a chunk then keep all four SIMDs of the CU
// busy instead of queueing in the first wavefront.
__device__ __forceinline__ int spread_segment(int L) {
  const int wave = threadIdx.x >> 6, sub = (threadIdx.x & 63) >> __builtin_ctz(L);
  return sub * (kBlock / 64) + wave;
}
__device__ __forceinline__ int pow2_ceil_clamped(int v, int hi) {
  int p = 1;
  while (p < v && p < hi) p <<= 1;
  return p;
}

}  // namespace gn
