// Device-side helpers shared by the gfx950 kernels: storage-type traits,
// 16-byte vector access, activation functions, wavefront reductions.
#ifndef ODLA_HIP_DEVICE_UTILS_H_
#define ODLA_HIP_DEVICE_UTILS_H_

#include <hip/hip_runtime.h>
#include <type_traits>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "kernels.h"

namespace ohip {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef int intx4 __attribute__((ext_vector_type(4)));
typedef int intx16 __attribute__((ext_vector_type(16)));
typedef _Float16 halfx8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int uintx4 __attribute__((ext_vector_type(4)));
typedef unsigned int uintx2 __attribute__((ext_vector_type(2)));

struct bf16_t { uint16_t bits; };
struct f16_t { uint16_t bits; };

__device__ __forceinline__ float bf16_to_f32(uint16_t b) {
  return __uint_as_float(((uint32_t)b) << 16);
}
// Round to nearest even; NaN stays NaN.
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
__device__ __forceinline__ float f16_to_f32(uint16_t h) {
  _Float16 v;
  __builtin_memcpy(&v, &h, 2);
  return (float)v;
}
__device__ __forceinline__ uint16_t f32_to_f16(float f) {
  _Float16 v = (_Float16)f;  // v_cvt_f16_f32: round to nearest even
  uint16_t h;
  __builtin_memcpy(&h, &v, 2);
  return h;
}

// Storage traits: load/store one element as float.
template <typename T> struct Store;
template <> struct Store<float> {
  static constexpr DType dt = DT_F32;
  __device__ static __forceinline__ float ld(const float* p) { return *p; }
  __device__ static __forceinline__ void st(float* p, float v) { *p = v; }
};
template <> struct Store<f16_t> {
  static constexpr DType dt = DT_F16;
  __device__ static __forceinline__ float ld(const f16_t* p) { return f16_to_f32(p->bits); }
  __device__ static __forceinline__ void st(f16_t* p, float v) { p->bits = f32_to_f16(v); }
};
template <> struct Store<bf16_t> {
  static constexpr DType dt = DT_BF16;
  __device__ static __forceinline__ float ld(const bf16_t* p) { return bf16_to_f32(p->bits); }
  __device__ static __forceinline__ void st(bf16_t* p, float v) { p->bits = f32_to_bf16(v); }
};

// 16-byte vector of T viewed as floats.
template <typename T> struct Vec16 {
  static constexpr int N = 16 / sizeof(T);
  uintx4 raw;
  __device__ __forceinline__ void load(const T* p) { raw = *reinterpret_cast<const uintx4*>(p); }
  __device__ __forceinline__ void store(T* p) const { *reinterpret_cast<uintx4*>(p) = raw; }
  __device__ __forceinline__ float get(int i) const {
    const T* e = reinterpret_cast<const T*>(&raw);
    return Store<T>::ld(e + i);
  }
  __device__ __forceinline__ void set(int i, float v) {
    T* e = reinterpret_cast<T*>(&raw);
    Store<T>::st(e + i, v);
  }
};

// Eight fp32 values to eight 2-byte values, round to nearest even.  bf16 goes
// through v_cvt_pk_bf16_f32 (the integer formulation of the same rounding costs
// five to six instructions per value, a quarter of a bf16 GEMM epilogue).
template <typename T>
__device__ __forceinline__ uintx4 pack8_rne(const float (&v)[8]) {
  if constexpr (std::is_same<T, bf16_t>::value) {
    typedef float floatx2 __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    uintx4 o;
    o.x = __builtin_bit_cast(unsigned, __builtin_convertvector((floatx2){v[0], v[1]}, bf16x2));
    o.y = __builtin_bit_cast(unsigned, __builtin_convertvector((floatx2){v[2], v[3]}, bf16x2));
    o.z = __builtin_bit_cast(unsigned, __builtin_convertvector((floatx2){v[4], v[5]}, bf16x2));
    o.w = __builtin_bit_cast(unsigned, __builtin_convertvector((floatx2){v[6], v[7]}, bf16x2));
    return o;
  } else {
    Vec16<T> o;
#pragma unroll
    for (int e = 0; e < 8; ++e) o.set(e, v[e]);
    return o.raw;
  }
}

// x * Phi(x) with Phi from erfc(|x| / sqrt 2) = 2^(t * q(t)), q a polynomial of degree 9 fitted
// to log2(erfc(t)) / t on [0, 4] (beyond 4 erfc is below 2e-8: Phi is 0 or 1 there, as in the
// float formula 0.5 x (1 + erff(x / sqrt 2))).  No branch, one v_exp_f32, twelve multiply-adds -
// a third of erff's instructions, which matters where this runs in a GEMM epilogue - and no
// cancellation for negative x: against the exact function, absolute error below 4e-7 and
// relative error below 4e-6 for every x (the float formula loses all relative accuracy in the
// negative tail, where 1 + erff cancels).
__device__ __forceinline__ float gelu_erf(float x) {
  const float tz = fabsf(x) * 0.70710678118654752440f;
  const float t = fminf(tz, 4.0f);
  float q = -7.638809052e-07f;
  q = __builtin_fmaf(q, t, 1.656449240e-05f);
  q = __builtin_fmaf(q, t, -1.540622325e-04f);
  q = __builtin_fmaf(q, t, 7.796748541e-04f);
  q = __builtin_fmaf(q, t, -2.041657222e-03f);
  q = __builtin_fmaf(q, t, -2.589797077e-04f);
  q = __builtin_fmaf(q, t, 2.797562815e-02f);
  q = __builtin_fmaf(q, t, -1.483925730e-01f);
  q = __builtin_fmaf(q, t, -9.184330702e-01f);
  q = __builtin_fmaf(q, t, -1.627907276e+00f);
  float h = 0.5f * __builtin_amdgcn_exp2f(q * t);   // erfc(|x| / sqrt 2) / 2 (the argument is >= -28: no denormals)
  h = tz < 4.0f ? h : 0.f;                           // (a NaN falls through to x * 0 = NaN)
  return x * (x >= 0.f ? 1.0f - h : h);
}
__device__ __forceinline__ float gelu_tanh(float x) {
  const float k = 0.79788456080286535588f;  // sqrt(2/pi)
  return 0.5f * x * (1.0f + tanhf(k * (x + 0.044715f * x * x * x)));
}

__device__ __forceinline__ float apply_act(float v, ActKind act, float a, float b) {
  switch (act) {
    case ACT_NONE: return v;
    case ACT_RELU: return v > 0.f ? v : 0.f;
    case ACT_LEAKY: return v > 0.f ? v : a * v;
    case ACT_CLAMP: return fminf(fmaxf(v, a), b);
    case ACT_SIGMOID: return 1.0f / (1.0f + expf(-v));
    case ACT_TANH: return tanhf(v);
    case ACT_GELU_ERF: return gelu_erf(v);
    case ACT_GELU_TANH: return gelu_tanh(v);
    case ACT_EXP: return expf(v);
    case ACT_LOG: return logf(v);
    case ACT_SQRT: return sqrtf(v);
    case ACT_RSQRT: return 1.0f / sqrtf(v);
    case ACT_ERF: return erff(v);
    case ACT_ABS: return fabsf(v);
    case ACT_NEG: return -v;
    case ACT_ROUND: return rintf(v);
    case ACT_RECIP: return 1.0f / v;
    case ACT_CEIL: return ceilf(v);
    case ACT_FLOOR: return floorf(v);
    case ACT_SIGN: return v > 0.f ? 1.f : (v < 0.f ? -1.f : v);
    case ACT_SIN: return sinf(v);
    case ACT_COS: return cosf(v);
    case ACT_TAN: return tanf(v);
    case ACT_ASIN: return asinf(v);
    case ACT_ACOS: return acosf(v);
    case ACT_ATAN: return atanf(v);
    case ACT_SINH: return sinhf(v);
    case ACT_COSH: return coshf(v);
    case ACT_ASINH: return asinhf(v);
    case ACT_ACOSH: return acoshf(v);
    case ACT_ATANH: return atanhf(v);
    case ACT_ELU: return v > 0.f ? v : a * expm1f(v);
    case ACT_SELU: return b * (v > 0.f ? v : a * expm1f(v));
    case ACT_CELU: return fmaxf(v, 0.f) + fminf(0.f, a * expm1f(v / a));
    case ACT_HARDSIGMOID: return fminf(fmaxf(a * v + b, 0.f), 1.f);
    case ACT_SOFTPLUS: return logf(expf(v) + 1.0f);
    case ACT_SOFTSIGN: return v / (fabsf(v) + 1.0f);
    case ACT_THRESHOLDED: return v > a ? v : 0.f;
    case ACT_SHRINK: return v > b ? v - a : (v < -b ? v + a : 0.f);
    case ACT_DIV_CONST: return v / a;
  }
  return v;
}

// n / d for 0 <= n < 2^31 with the divisor's magic pair (div_magic on the host
// side): three instructions instead of the ~35 of a 32-bit division.
__device__ __forceinline__ int fast_div(int n, unsigned magic, int shift) {
  return (int)(__umulhi((unsigned)n << 1, magic) >> shift);
}

// Cross-lane reductions.  Inside a row of 16 lanes the partner values arrive
// through DPP operands of the arithmetic instruction itself (quad permutes,
// then the half-row and row mirrors: once a quad / half row is uniform, its
// mirror image is the other quad / half row), which costs no LDS crossbar trip
// like ds_bpermute does; the four row totals are then read as scalars.
// Every lane of a group of LPR lanes (a power of two, groups aligned) receives
// op over the group.  Call from wavefront-uniform control flow only: DPP and
// v_readlane read lanes whatever their EXEC bit.
template <int CTRL>
__device__ __forceinline__ float dpp_move(const float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
template <int LPR, typename Op>
__device__ __forceinline__ float group_allreduce(float v, Op op) {
  static_assert(LPR >= 1 && LPR <= 64 && (LPR & (LPR - 1)) == 0, "groups are powers of two up to the wavefront");
  if constexpr (LPR >= 2) v = op(v, dpp_move<0xB1>(v));    // quad_perm:[1,0,3,2]
  if constexpr (LPR >= 4) v = op(v, dpp_move<0x4E>(v));    // quad_perm:[2,3,0,1]
  if constexpr (LPR >= 8) v = op(v, dpp_move<0x141>(v));   // row_half_mirror
  if constexpr (LPR >= 16) v = op(v, dpp_move<0x140>(v));  // row_mirror
  if constexpr (LPR >= 32) {
    const int bits = __builtin_bit_cast(int, v);
    const float t0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 0));
    const float t1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 16));
    const float t2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 32));
    const float t3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(bits, 48));
    if constexpr (LPR == 64) v = op(op(t0, t1), op(t2, t3));
    else v = (threadIdx.x & 32) ? op(t2, t3) : op(t0, t1);
  }
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
  return group_allreduce<64>(v, [](float a, float b) { return a + b; });
}
__device__ __forceinline__ float wave_max(float v) {
  return group_allreduce<64>(v, [](float a, float b) { return fmaxf(a, b); });
}

// Block-wide reductions for blocks of NT threads (NT multiple of 64, <= 1024).
// `smem` must hold NT/64 floats; every thread receives the result.
template <int NT>
__device__ __forceinline__ float block_sum(float v, float* smem) {
  v = wave_sum(v);
  if (NT == 64) return v;
  const int w = threadIdx.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) smem[w] = v;
  __syncthreads();
  float r = 0.f;
#pragma unroll
  for (int i = 0; i < NT / 64; ++i) r += smem[i];
  return r;
}
template <int NT>
__device__ __forceinline__ float block_max(float v, float* smem) {
  v = wave_max(v);
  if (NT == 64) return v;
  const int w = threadIdx.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) smem[w] = v;
  __syncthreads();
  float r = smem[0];
#pragma unroll
  for (int i = 1; i < NT / 64; ++i) r = fmaxf(r, smem[i]);
  return r;
}

// Quantised 8-bit activations are stored as q-128 (int8); these convert
// between the stored byte and the unsigned level q in [0,255].
__device__ __forceinline__ int q_from_stored(int8_t s) { return (int)s + 128; }
__device__ __forceinline__ int8_t q_to_stored(int q) { return (int8_t)(q - 128); }

inline int grid_for(int64_t work_items, int per_block, int max_blocks = 256 * 32) {
  int64_t g = (work_items + per_block - 1) / per_block;
  if (g < 1) g = 1;
  if (g > max_blocks) g = max_blocks;
  return (int)g;
}

}  // namespace ohip
#endif
