// Typed element-wise kernels with broadcast for the operators the streaming
// float kernels do not cover: integer arithmetic, comparisons and logic with
// boolean results, Select and the predicates IsNaN / IsInf / Not.  One thread
// per output element; consecutive lanes write consecutive elements.  Float
// types compute in fp32, integer types in int64.
#include <math.h>

#include "device_utils.h"

namespace ohip {

namespace {
constexpr int kThreads = 256;

template <typename T> struct Elem;
template <> struct Elem<float> {
  using C = float;
  __device__ static __forceinline__ C ld(const float* p) { return *p; }
  __device__ static __forceinline__ void st(float* p, C v) { *p = v; }
};
template <> struct Elem<f16_t> {
  using C = float;
  __device__ static __forceinline__ C ld(const f16_t* p) { return Store<f16_t>::ld(p); }
  __device__ static __forceinline__ void st(f16_t* p, C v) { Store<f16_t>::st(p, v); }
};
template <> struct Elem<bf16_t> {
  using C = float;
  __device__ static __forceinline__ C ld(const bf16_t* p) { return Store<bf16_t>::ld(p); }
  __device__ static __forceinline__ void st(bf16_t* p, C v) { Store<bf16_t>::st(p, v); }
};
template <> struct Elem<int32_t> {
  using C = int64_t;
  __device__ static __forceinline__ C ld(const int32_t* p) { return *p; }
  __device__ static __forceinline__ void st(int32_t* p, C v) { *p = (int32_t)v; }
};
template <> struct Elem<int64_t> {
  using C = int64_t;
  __device__ static __forceinline__ C ld(const int64_t* p) { return *p; }
  __device__ static __forceinline__ void st(int64_t* p, C v) { *p = v; }
};
template <> struct Elem<int8_t> {
  using C = int64_t;
  __device__ static __forceinline__ C ld(const int8_t* p) { return *p; }
  __device__ static __forceinline__ void st(int8_t* p, C v) { *p = (int8_t)v; }
};
template <> struct Elem<uint8_t> {  // also bool: stored 0 / 1
  using C = int64_t;
  __device__ static __forceinline__ C ld(const uint8_t* p) { return *p; }
  __device__ static __forceinline__ void st(uint8_t* p, C v) { *p = (uint8_t)v; }
};

__device__ __forceinline__ float arith(float a, float b, EwiseOp op) {
  switch (op) {
    case EW_ADD: return a + b;
    case EW_SUB: return a - b;
    case EW_MUL: return a * b;
    case EW_DIV: return a / b;
    case EW_MAX: return fmaxf(a, b);
    case EW_MIN: return fminf(a, b);
    case EW_POW: return powf(a, b);
    case EW_MOD: {  // the sign follows the divisor
      const float q = (float)floor((double)a / (double)b);
      return a - b * q;
    }
    case EW_FMOD: {  // the sign follows the dividend; the quotient passes through int32
      const double t = (double)a / (double)b;
      const float q = (float)(int)(t > 0.0 ? floor(t) : ceil(t));
      return a - b * q;
    }
    case EW_PRELU: return a < 0.f ? a * b : a;
    case EW_SQDIFF: return (a - b) * (a - b);
    default: return a;
  }
}
__device__ __forceinline__ int64_t ipow(int64_t a, int64_t b) {
  if (b < 0) return a == 1 ? 1 : (a == -1 ? ((b & 1) ? -1 : 1) : 0);
  int64_t r = 1;
  while (b) {
    if (b & 1) r *= a;
    a *= a;
    b >>= 1;
  }
  return r;
}
__device__ __forceinline__ int64_t arith(int64_t a, int64_t b, EwiseOp op) {
  switch (op) {
    case EW_ADD: return a + b;
    case EW_SUB: return a - b;
    case EW_MUL: return a * b;
    case EW_DIV: return b == 0 ? 0 : a / b;
    case EW_MAX: return a > b ? a : b;
    case EW_MIN: return a < b ? a : b;
    case EW_POW: return ipow(a, b);
    case EW_MOD: {
      if (b == 0) return 0;
      const int64_t q = (int64_t)floor((double)a / (double)b);
      return a - b * q;
    }
    case EW_FMOD: {
      if (b == 0) return 0;
      const double t = (double)a / (double)b;
      const int64_t q = (int64_t)(int)(t > 0.0 ? floor(t) : ceil(t));
      return a - b * q;
    }
    case EW_PRELU: return a < 0 ? a * b : a;
    case EW_SQDIFF: return (a - b) * (a - b);
    default: return a;
  }
}
template <typename C>
__device__ __forceinline__ bool compare(C a, C b, EwiseOp op) {
  switch (op) {
    case EW_EQ: return a == b;
    case EW_NE: return a != b;
    case EW_LT: return a < b;
    case EW_LE: return a <= b;
    case EW_GT: return a > b;
    case EW_GE: return a >= b;
    case EW_AND: return (a != 0) && (b != 0);
    case EW_OR: return (a != 0) || (b != 0);
    case EW_XOR: return (a != 0) != (b != 0);
    case EW_NOT: return a == 0;
    default: return false;
  }
}
__device__ __forceinline__ bool predicate(float a, EwiseOp op) {
  switch (op) {
    case EW_ISNAN: return isnan(a);
    case EW_ISINF: return isinf(a);
    case EW_ISINF_POS: return isinf(a) && a > 0.f;
    case EW_ISINF_NEG: return isinf(a) && a < 0.f;
    default: return false;
  }
}
__device__ __forceinline__ bool predicate(int64_t, EwiseOp) { return false; }

template <int ES> struct BytesOf;
template <> struct BytesOf<1> { using type = uint8_t; };
template <> struct BytesOf<2> { using type = uint16_t; };
template <> struct BytesOf<4> { using type = uint32_t; };
template <> struct BytesOf<8> { using type = uint64_t; };

struct Offsets { int64_t a, b, c; };
__device__ __forceinline__ Offsets decompose(const EwiseParams& p, int64_t i) {
  Offsets o = {0, 0, 0};
  int64_t rem = i;
#pragma unroll
  for (int d = 5; d >= 0; --d) {
    if (d < p.rank) {
      const int64_t q = rem / p.dims[d];
      const int64_t idx = rem - q * p.dims[d];
      rem = q;
      o.a += idx * p.sa[d];
      o.b += idx * p.sb[d];
      o.c += idx * p.sc[d];
    }
  }
  return o;
}

// y = a op b, operands and result of type T
template <typename T>
__global__ void __launch_bounds__(kThreads) ewise_arith_kernel(EwiseParams p, int64_t n) {
  const T* a = reinterpret_cast<const T*>(p.a);
  const T* b = reinterpret_cast<const T*>(p.b);
  T* y = reinterpret_cast<T*>(p.y);
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += stride) {
    const Offsets o = decompose(p, i);
    Elem<T>::st(y + i, arith(Elem<T>::ld(a + o.a), Elem<T>::ld(b + o.b), p.op));
  }
}

// y (bool) = a op b or predicate(a)
template <typename T>
__global__ void __launch_bounds__(kThreads) ewise_bool_kernel(EwiseParams p, int64_t n) {
  const T* a = reinterpret_cast<const T*>(p.a);
  const T* b = reinterpret_cast<const T*>(p.b);
  uint8_t* y = reinterpret_cast<uint8_t*>(p.y);
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  const bool pred = p.op >= EW_ISNAN;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += stride) {
    const Offsets o = decompose(p, i);
    const typename Elem<T>::C va = Elem<T>::ld(a + o.a);
    bool r;
    if (pred) r = predicate(va, p.op);
    else r = compare(va, Elem<T>::ld(b + o.b), p.op);
    y[i] = r ? 1 : 0;
  }
}

// y = a (bool) ? b : c; moves raw elements of ES bytes
template <int ES>
__global__ void __launch_bounds__(kThreads) ewise_select_kernel(EwiseParams p, int64_t n) {
  using W = typename BytesOf<ES>::type;
  const uint8_t* a = reinterpret_cast<const uint8_t*>(p.a);
  const W* b = reinterpret_cast<const W*>(p.b);
  const W* c = reinterpret_cast<const W*>(p.c);
  W* y = reinterpret_cast<W*>(p.y);
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += stride) {
    const Offsets o = decompose(p, i);
    y[i] = a[o.a] != 0 ? b[o.b] : c[o.c];
  }
}

// y = a << b or a >> b on unsigned words of ES bytes
template <int ES>
__global__ void __launch_bounds__(kThreads) ewise_shift_kernel(EwiseParams p, int64_t n, bool left) {
  using W = typename BytesOf<ES>::type;
  const W* a = reinterpret_cast<const W*>(p.a);
  const W* b = reinterpret_cast<const W*>(p.b);
  W* y = reinterpret_cast<W*>(p.y);
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += stride) {
    const Offsets o = decompose(p, i);
    const W v = a[o.a], s = b[o.b];
    y[i] = s >= (W)(ES * 8) ? (W)0 : (left ? (W)(v << s) : (W)(v >> s));
  }
}

#define EWISE_TYPE_DISPATCH(dt, EXPR)                                 \
  switch (dt) {                                                       \
    case DT_F32: { using T = float; EXPR; break; }                    \
    case DT_F16: { using T = f16_t; EXPR; break; }                    \
    case DT_BF16: { using T = bf16_t; EXPR; break; }                  \
    case DT_I32: { using T = int32_t; EXPR; break; }                  \
    case DT_I64: { using T = int64_t; EXPR; break; }                  \
    case DT_I8: { using T = int8_t; EXPR; break; }                    \
    case DT_U8: case DT_BOOL: { using T = uint8_t; EXPR; break; }     \
    default: return hipErrorInvalidValue;                             \
  }

}  // namespace

hipError_t launch_ewise(const EwiseParams& p, hipStream_t stream) {
  if (!p.a || !p.y || p.rank < 1 || p.rank > 6) return hipErrorInvalidValue;
  int64_t n = 1;
  for (int d = 0; d < p.rank; ++d) {
    if (p.dims[d] <= 0) return hipErrorInvalidValue;
    n *= p.dims[d];
  }
  const bool shift = p.op == EW_SHL || p.op == EW_SHR;
  const bool unary = p.op == EW_NOT || (p.op >= EW_ISNAN && !shift);
  EwiseParams q = p;
  if (unary) { q.b = p.a; for (int d = 0; d < 6; ++d) q.sb[d] = p.sa[d]; }
  if (!q.b) return hipErrorInvalidValue;
  const int grid = grid_for(n, kThreads * 4);
  if (p.op == EW_SELECT) {
    if (!p.c) return hipErrorInvalidValue;
    switch (dtype_size(p.dt)) {
      case 1: hipLaunchKernelGGL(ewise_select_kernel<1>, dim3(grid), dim3(kThreads), 0, stream, q, n); break;
      case 2: hipLaunchKernelGGL(ewise_select_kernel<2>, dim3(grid), dim3(kThreads), 0, stream, q, n); break;
      case 4: hipLaunchKernelGGL(ewise_select_kernel<4>, dim3(grid), dim3(kThreads), 0, stream, q, n); break;
      case 8: hipLaunchKernelGGL(ewise_select_kernel<8>, dim3(grid), dim3(kThreads), 0, stream, q, n); break;
      default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
  }
  if (shift) {
    if (p.dt != DT_U8 && p.dt != DT_I32 && p.dt != DT_I64) return hipErrorInvalidValue;
    const bool left = p.op == EW_SHL;
    switch (dtype_size(p.dt)) {
      case 1: hipLaunchKernelGGL(ewise_shift_kernel<1>, dim3(grid), dim3(kThreads), 0, stream, q, n, left); break;
      case 4: hipLaunchKernelGGL(ewise_shift_kernel<4>, dim3(grid), dim3(kThreads), 0, stream, q, n, left); break;
      default: hipLaunchKernelGGL(ewise_shift_kernel<8>, dim3(grid), dim3(kThreads), 0, stream, q, n, left); break;
    }
    return hipGetLastError();
  }
  if (p.op >= EW_EQ) {
    if ((p.op >= EW_AND && p.op <= EW_NOT) && p.dt != DT_BOOL && p.dt != DT_U8) return hipErrorInvalidValue;
    if (p.op >= EW_ISNAN && !dtype_is_float(p.dt)) return hipErrorInvalidValue;
    EWISE_TYPE_DISPATCH(p.dt, hipLaunchKernelGGL(ewise_bool_kernel<T>, dim3(grid), dim3(kThreads), 0, stream, q, n));
    return hipGetLastError();
  }
  if (p.dt == DT_BOOL) return hipErrorInvalidValue;
  EWISE_TYPE_DISPATCH(p.dt, hipLaunchKernelGGL(ewise_arith_kernel<T>, dim3(grid), dim3(kThreads), 0, stream, q, n));
  return hipGetLastError();
}

}  // namespace ohip
