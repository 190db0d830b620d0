// Streaming element-wise kernels for gfx950: unary activations, per-channel
// affine (folded BatchNorm), broadcasting binary ops, casts and affine
// (de)quantisation.  All are HBM-bound: each thread moves 16-byte vectors,
// consecutive lanes touch consecutive vectors, and the grid is a grid-stride
// loop sized to a few workgroups per CU.
#include "device_utils.h"

namespace ohip {

namespace {
constexpr int kThreads = 256;

// Streaming loop shape shared by the flat kernels: every thread keeps U 16-byte
// loads in flight before it touches the data.  Results leave with plain stores:
// measured on [256,256,56,56] fp16, non-temporal stores were slower here (ReLU
// 168 -> 269 us, residual Add 238 -> 252 us), unlike in the convolution epilogue.
constexpr int kUnroll = 4;

template <typename T>
__device__ __forceinline__ void out_store(Vec16<T>& v, T* p) {
  v.store(p);
}

// A workgroup owns one contiguous tile of kThreads * U 16-byte vectors: load u of
// a thread is vector tile * kThreads * U + u * kThreads + thread, so that every
// load instruction of a wavefront covers one contiguous KiB and a workgroup's U
// loads cover one contiguous U * 4 KiB, all in flight before the first use.
// KIND >= 0 fixes the activation at compile time (the switch folds away; per
// element it would cost more than the arithmetic); KIND < 0 takes it from `act`.
template <typename T, int KIND, int U>
__global__ void __launch_bounds__(kThreads)
unary_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t n, ActKind act, float a, float b) {
  constexpr int V = Vec16<T>::N;
  const ActKind kind = KIND >= 0 ? (ActKind)KIND : act;
  const int64_t nvec = n / V;
  const int64_t base = (int64_t)blockIdx.x * (kThreads * U) + threadIdx.x;
  Vec16<T> v[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int64_t i = base + u * kThreads;
    if (i < nvec) v[u].raw = __builtin_nontemporal_load(reinterpret_cast<const uintx4*>(x + i * V));
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int64_t i = base + u * kThreads;
    if (i < nvec) {
#pragma unroll
      for (int e = 0; e < V; ++e) v[u].set(e, apply_act(v[u].get(e), kind, a, b));
      out_store(v[u], y + i * V);
    }
  }
  // tail (fewer than V elements), by the first workgroup
  if (blockIdx.x == 0) {
    for (int64_t i = nvec * V + threadIdx.x; i < n; i += kThreads)
      Store<T>::st(y + i, apply_act(Store<T>::ld(x + i), kind, a, b));
  }
}

// y = x * scale[c] + shift[c].  inner == 1: channel is the innermost index
// (channels-last), so a vector spans V consecutive channels; when the grid
// stride is a multiple of the channel count every thread meets the same V
// channels in every iteration and keeps their parameters in registers.
// inner > 1 (row-major N,C,HW): the channel is constant across a vector when
// inner % V == 0.
template <typename T, int U>
__global__ void __launch_bounds__(kThreads)
channel_affine_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t n, int64_t inner,
                      int channels, const float* __restrict__ scale,
                      const float* __restrict__ shift) {
  constexpr int V = Vec16<T>::N;
  const bool vec_ok = (inner == 1) ? (channels % V == 0) : (inner % V == 0);
  if (vec_ok) {
    // tiled like unary_kernel: a workgroup owns kThreads * U consecutive vectors
    const int64_t nvec = n / V;
    const int64_t tile0 = (int64_t)blockIdx.x * (kThreads * U);
    const int64_t base = tile0 + threadIdx.x;
    // channel of the tile's first element (wavefront-uniform), then 32-bit arithmetic per vector
    const unsigned c_tile = inner == 1 ? (unsigned)((tile0 * V) % channels) : 0u;
    Vec16<T> v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t i = base + u * kThreads;
      if (i < nvec) v[u].raw = __builtin_nontemporal_load(reinterpret_cast<const uintx4*>(x + i * V));
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t i = base + u * kThreads;
      if (i >= nvec) continue;
      if (inner == 1) {
        const unsigned c0 = (c_tile + (unsigned)(u * kThreads + threadIdx.x) * V) % (unsigned)channels;
        float sc[V], sh[V];
        if constexpr (V == 8) {
          const floatx4 s0 = *reinterpret_cast<const floatx4*>(scale + c0), s1 = *reinterpret_cast<const floatx4*>(scale + c0 + 4);
          const floatx4 t0 = *reinterpret_cast<const floatx4*>(shift + c0), t1 = *reinterpret_cast<const floatx4*>(shift + c0 + 4);
          sc[0] = s0.x; sc[1] = s0.y; sc[2] = s0.z; sc[3] = s0.w; sc[4] = s1.x; sc[5] = s1.y; sc[6] = s1.z; sc[7] = s1.w;
          sh[0] = t0.x; sh[1] = t0.y; sh[2] = t0.z; sh[3] = t0.w; sh[4] = t1.x; sh[5] = t1.y; sh[6] = t1.z; sh[7] = t1.w;
        } else {
#pragma unroll
          for (int e = 0; e < V; ++e) { sc[e] = scale[c0 + e]; sh[e] = shift[c0 + e]; }
        }
#pragma unroll
        for (int e = 0; e < V; ++e) v[u].set(e, v[u].get(e) * sc[e] + sh[e]);
      } else {
        const int c = (int)(((i * V) / inner) % channels);
        const float sc = scale[c], sh = shift[c];
#pragma unroll
        for (int e = 0; e < V; ++e) v[u].set(e, v[u].get(e) * sc + sh);
      }
      out_store(v[u], y + i * V);
    }
  } else {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x * U;
    for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += stride / U) {
      const int c = (int)((i / inner) % channels);
      Store<T>::st(y + i, Store<T>::ld(x + i) * scale[c] + shift[c]);
    }
  }
}

__global__ void bn_fold_kernel(const float* mean, const float* var, const float* gamma,
                               const float* beta, float sgamma, float sbeta, float eps,
                               int channels, float* scale, float* shift) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const float g = gamma ? gamma[c] : sgamma;
  const float b = beta ? beta[c] : sbeta;
  const float m = g / sqrtf(var[c] + eps);
  scale[c] = m;
  shift[c] = b - mean[c] * m;
}

__device__ __forceinline__ float bin_op(float a, float b, BinKind op) {
  switch (op) {
    case BIN_ADD: return a + b;
    case BIN_SUB: return a - b;
    case BIN_MUL: return a * b;
    case BIN_DIV: return a / b;
    case BIN_MAX: return fmaxf(a, b);
    case BIN_MIN: return fminf(a, b);
  }
  return a;
}

// Same-shape, contiguous operands; tiled like unary_kernel.  OP / KIND >= 0 fix the
// operator / the fused activation at compile time.
template <typename T, int OP, int KIND, int U>
__global__ void __launch_bounds__(kThreads)
binary_flat_kernel(const T* __restrict__ a, const T* __restrict__ b, T* __restrict__ y, int64_t n,
                   BinKind op_rt, ActKind act, float aa, float ab) {
  constexpr int V = Vec16<T>::N;
  const BinKind op = OP >= 0 ? (BinKind)OP : op_rt;
  const ActKind kind = KIND >= 0 ? (ActKind)KIND : act;
  const int64_t nvec = n / V;
  const int64_t base = (int64_t)blockIdx.x * (kThreads * U) + threadIdx.x;
  Vec16<T> va[U], vb[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int64_t i = base + u * kThreads;
    if (i < nvec) {
      va[u].raw = __builtin_nontemporal_load(reinterpret_cast<const uintx4*>(a + i * V));
      vb[u].raw = __builtin_nontemporal_load(reinterpret_cast<const uintx4*>(b + i * V));
    }
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int64_t i = base + u * kThreads;
    if (i < nvec) {
#pragma unroll
      for (int e = 0; e < V; ++e) va[u].set(e, apply_act(bin_op(va[u].get(e), vb[u].get(e), op), kind, aa, ab));
      out_store(va[u], y + i * V);
    }
  }
  if (blockIdx.x == 0) {
    for (int64_t i = nvec * V + threadIdx.x; i < n; i += kThreads)
      Store<T>::st(y + i, apply_act(bin_op(Store<T>::ld(a + i), Store<T>::ld(b + i), op), kind, aa, ab));
  }
}

// One operand is a vector indexed by the innermost output dim (bias rows,
// channels-last per-channel constants): b index = i % period.
template <typename T>
__global__ void __launch_bounds__(kThreads)
binary_rowvec_kernel(const T* __restrict__ a, const T* __restrict__ b, T* __restrict__ y,
                     int64_t n, int period, bool b_is_lhs, BinKind op, ActKind act, float aa,
                     float ab) {
  constexpr int V = Vec16<T>::N;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  if (period % V == 0) {
    const int64_t nvec = n / V;
    for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < nvec; i += stride) {
      Vec16<T> va, vb;
      va.load(a + i * V);
      vb.load(b + (i * V) % period);
#pragma unroll
      for (int e = 0; e < V; ++e) {
        const float l = b_is_lhs ? vb.get(e) : va.get(e);
        const float r = b_is_lhs ? va.get(e) : vb.get(e);
        va.set(e, apply_act(bin_op(l, r, op), act, aa, ab));
      }
      va.store(y + i * V);
    }
  } else {
    for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += stride) {
      const float av = Store<T>::ld(a + i), bv = Store<T>::ld(b + i % period);
      Store<T>::st(y + i, apply_act(b_is_lhs ? bin_op(bv, av, op) : bin_op(av, bv, op), act, aa, ab));
    }
  }
}

// General broadcast: decompose the flat output index over `rank` dims.
template <typename T>
__global__ void __launch_bounds__(kThreads)
binary_bcast_kernel(BinaryParams p, int64_t n) {
  const T* a = reinterpret_cast<const T*>(p.a);
  const T* b = reinterpret_cast<const T*>(p.b);
  T* y = reinterpret_cast<T*>(p.y);
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += stride) {
    int64_t rem = i, oa = 0, ob = 0;
#pragma unroll
    for (int d = 5; d >= 0; --d) {
      if (d < p.rank) {
        const int64_t q = rem / p.dims[d];
        const int64_t idx = rem - q * p.dims[d];
        rem = q;
        oa += idx * p.sa[d];
        ob += idx * p.sb[d];
      }
    }
    Store<T>::st(y + i, apply_act(bin_op(Store<T>::ld(a + oa), Store<T>::ld(b + ob), p.op), p.act,
                                  p.act_a, p.act_b));
  }
}

// Quantised add (8-bit levels stored as q-128), same shape, contiguous:
// the float sequence dequantise, op, requantise of the unfused graph.
__global__ void __launch_bounds__(kThreads)
binary_q8_kernel(BinaryParams p, int64_t n) {
  const int8_t* a = reinterpret_cast<const int8_t*>(p.a);
  const int8_t* b = reinterpret_cast<const int8_t*>(p.b);
  int8_t* y = reinterpret_cast<int8_t*>(p.y);
  const int64_t nvec = n / 16;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  auto one = [&](int8_t sa, int8_t sb) -> int8_t {
    const float fa = (float)(q_from_stored(sa) - p.a_zp) * p.a_scale;
    const float fb = (float)(q_from_stored(sb) - p.b_zp) * p.b_scale;
    const float f = bin_op(fa, fb, p.op);
    int q = (int)rintf(f * p.y_inv) + p.y_zp;
    q = q < p.y_lo ? p.y_lo : q;
    q = q > 255 ? 255 : q;
    return q_to_stored(q);
  };
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < nvec; i += stride) {
    uintx4 va = *reinterpret_cast<const uintx4*>(a + i * 16);
    uintx4 vb = *reinterpret_cast<const uintx4*>(b + i * 16);
    const int8_t* ea = reinterpret_cast<const int8_t*>(&va);
    const int8_t* eb = reinterpret_cast<const int8_t*>(&vb);
    uintx4 vo;
    int8_t* eo = reinterpret_cast<int8_t*>(&vo);
#pragma unroll
    for (int e = 0; e < 16; ++e) eo[e] = one(ea[e], eb[e]);
    *reinterpret_cast<uintx4*>(y + i * 16) = vo;
  }
  for (int64_t i = nvec * 16 + blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += stride)
    y[i] = one(a[i], b[i]);
}

template <typename TS, typename TD>
__global__ void __launch_bounds__(kThreads)
cast_kernel(const TS* __restrict__ x, TD* __restrict__ y, int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  // 4 elements per thread step keeps loads/stores >= 8 bytes for 16-bit types.
  const int64_t n4 = n / 4;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n4; i += stride) {
    float v[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = Store<TS>::ld(x + i * 4 + e);
#pragma unroll
    for (int e = 0; e < 4; ++e) Store<TD>::st(y + i * 4 + e, v[e]);
  }
  for (int64_t i = n4 * 4 + blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += stride)
    Store<TD>::st(y + i, Store<TS>::ld(x + i));
}

// Conversions that involve an integer type, one element per thread step.
// Rules, following the reference's cast (a oneDNN reorder): a floating-point
// value that becomes an integer is rounded to the nearest integer, ties to
// even, and saturates at the ends of the target range; an integer that becomes
// a narrower integer saturates; an integer that becomes a floating-point value
// is rounded to nearest even; anything that becomes a bool is "!= 0".
// [ref: ODLA/platforms/dnnl/odla_dnnl_cast.cc:232-258]
template <typename T> struct CastElem;
template <> struct CastElem<float> { static constexpr bool is_float = true; };
template <> struct CastElem<f16_t> { static constexpr bool is_float = true; };
template <> struct CastElem<bf16_t> { static constexpr bool is_float = true; };
template <> struct CastElem<int8_t> { static constexpr bool is_float = false; static constexpr long long lo = -128, hi = 127; };
template <> struct CastElem<uint8_t> { static constexpr bool is_float = false; static constexpr long long lo = 0, hi = 255; };
template <> struct CastElem<int32_t> { static constexpr bool is_float = false; static constexpr long long lo = -2147483648ll, hi = 2147483647ll; };
template <> struct CastElem<int64_t> { static constexpr bool is_float = false; static constexpr long long lo = INT64_MIN, hi = INT64_MAX; };

// float -> integer type TD: clamp in float to the representable ends of the
// target (2147483520 is the largest float below 2^31, 2^63 - 2^39 the largest
// below 2^63), then round to nearest even.  NaN becomes 0.
template <typename TD>
__device__ __forceinline__ TD float_to_int_sat(float v) {
  if (v != v) return (TD)0;
  float lo, hi;
  if constexpr (sizeof(TD) == 8) { lo = -9223372036854775808.f; hi = 9223371487098961920.f; }
  else if constexpr (sizeof(TD) == 4) { lo = -2147483648.f; hi = 2147483520.f; }
  else { lo = (float)CastElem<TD>::lo; hi = (float)CastElem<TD>::hi; }
  const float c = fminf(fmaxf(v, lo), hi);
  if constexpr (sizeof(TD) == 8) return (TD)__float2ll_rn(c);
  else return (TD)__float2int_rn(c);
}

template <typename TS, typename TD, bool kDstBool>
__global__ void __launch_bounds__(kThreads)
cast_int_kernel(const TS* __restrict__ x, TD* __restrict__ y, int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += stride) {
    if constexpr (CastElem<TS>::is_float) {
      const float v = Store<TS>::ld(x + i);
      if constexpr (kDstBool) y[i] = (TD)(v != 0.f);
      else y[i] = float_to_int_sat<TD>(v);
    } else {
      const long long v = (long long)x[i];
      if constexpr (kDstBool) {
        y[i] = (TD)(v != 0);
      } else if constexpr (CastElem<TD>::is_float) {
        Store<TD>::st(y + i, (float)v);
      } else {
        const long long lo = CastElem<TD>::lo, hi = CastElem<TD>::hi;
        y[i] = (TD)(v < lo ? lo : (v > hi ? hi : v));
      }
    }
  }
}

// q = sat(rne(x / scale) + zp)
template <typename TS>
__device__ __forceinline__ int quant_one(float x, float scale, float zf, bool sgn) {
  const float t = rintf(x / scale) + zf;  // the reference adds the zero point in float before the saturating cast
  return sgn ? (int)fminf(fmaxf(t, -128.f), 127.f) : (int)fminf(fmaxf(t, 0.f), 255.f);
}

// rne(x / scale) without the division where that is certain: x * (1 / scale) is within 1.5
// units of the last place of the quotient, so unless it lies that close to a rounding boundary
// (k + 0.5) both round to the same integer; the rare lanes near a boundary divide.
__device__ __forceinline__ float rne_quotient(float x, float scale, float inv) {
  const float m = x * inv;
  float q = rintf(m);
  if (fabsf(fabsf(m - q) - 0.5f) <= 4e-7f * fabsf(m) + 1e-30f) q = rintf(x / scale);
  return q;
}

template <typename TS>
__global__ void __launch_bounds__(kThreads)
quantize_kernel(QuantParams p) {
  const TS* x = reinterpret_cast<const TS*>(p.src);
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  const int64_t t0 = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  int64_t done = 0;
  if (p.channels == 1 && (reinterpret_cast<uintptr_t>(p.src) & 15u) == 0 && (reinterpret_cast<uintptr_t>(p.dst) & 15u) == 0) {
    // per-tensor parameters: a workgroup takes contiguous tiles of 256 threads x 2 x 16 elements;
    // a thread's loads are issued back to back and each of its two results is one 16-byte store
    const float sc = p.scale[0], zf = p.zp ? (float)p.zp[0] : 0.f;
    const float inv = 1.0f / sc;
    constexpr int LV = 16 * (int)sizeof(TS) / 16;   // 16-byte loads per 16 elements
    constexpr int PER = 16 / LV;                     // elements per load
    const int64_t tile = (int64_t)kThreads * 32;
    const int64_t ntiles = p.n / tile;
    for (int64_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
      Vec16<TS> in[2][LV];
#pragma unroll
      for (int g = 0; g < 2; ++g)
#pragma unroll
        for (int l = 0; l < LV; ++l) in[g][l].load(x + t * tile + ((int64_t)g * kThreads + threadIdx.x) * 16 + l * PER);
#pragma unroll
      for (int g = 0; g < 2; ++g) {
        uintx4 ov;
        if (!p.dst_signed) {
          // unsigned levels: the packing conversion rounds (an integer already) and saturates to [0, 255]
          unsigned w[4] = {0u, 0u, 0u, 0u};
#pragma unroll
          for (int l = 0; l < LV; ++l)
#pragma unroll
            for (int e = 0; e < PER; ++e) {
              const int k = l * PER + e;
              w[k >> 2] = __builtin_amdgcn_cvt_pk_u8_f32(rne_quotient(in[g][l].get(e), sc, inv) + zf, k & 3, w[k >> 2]);
            }
          const unsigned flip = p.dst_dt == DT_I8 ? 0x80808080u : 0u;   // stored as level - 128
          ov = uintx4{w[0] ^ flip, w[1] ^ flip, w[2] ^ flip, w[3] ^ flip};
        } else {
          unsigned char o[16];
#pragma unroll
          for (int l = 0; l < LV; ++l)
#pragma unroll
            for (int e = 0; e < PER; ++e) o[l * PER + e] = (unsigned char)quant_one<TS>(in[g][l].get(e), sc, zf, true);
          __builtin_memcpy(&ov, o, 16);
        }
        *reinterpret_cast<uintx4*>(reinterpret_cast<unsigned char*>(p.dst) + t * tile + ((int64_t)g * kThreads + threadIdx.x) * 16) = ov;
      }
    }
    done = ntiles * tile;
  }
  for (int64_t i = done + t0; i < p.n; i += stride) {
    const int c = (p.channels > 1) ? (int)((i / p.inner) % p.channels) : 0;
    const int q = quant_one<TS>(Store<TS>::ld(x + i), p.scale[c], p.zp ? (float)p.zp[c] : 0.f, p.dst_signed);
    if (p.dst_signed) reinterpret_cast<int8_t*>(p.dst)[i] = (int8_t)q;
    else if (p.dst_dt == DT_I8) reinterpret_cast<int8_t*>(p.dst)[i] = q_to_stored(q);
    else reinterpret_cast<uint8_t*>(p.dst)[i] = (uint8_t)q;
  }
}

// x = (q - zp) * scale
template <typename TD>
__global__ void __launch_bounds__(kThreads)
dequantize_kernel(QuantParams p) {
  TD* y = reinterpret_cast<TD*>(p.dst);
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  const int64_t t0 = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
  auto level = [&](unsigned char raw) -> float {
    if (p.src_dt == DT_U8) return (float)raw;
    if (p.dst_signed) return (float)(int8_t)raw;
    return (float)q_from_stored((int8_t)raw);
  };
  int64_t done = 0;
  if (p.channels == 1 && (reinterpret_cast<uintptr_t>(p.src) & 7u) == 0 && (reinterpret_cast<uintptr_t>(p.dst) & 15u) == 0) {
    const float sc = p.scale[0], zf = p.zp ? (float)p.zp[0] : 0.f;
    const int64_t n8 = p.n / 8;
    for (int64_t i = t0; i < n8; i += stride) {
      const uintx2 rv = *reinterpret_cast<const uintx2*>(reinterpret_cast<const unsigned char*>(p.src) + i * 8);
      unsigned char r[8];
      __builtin_memcpy(r, &rv, 8);
      float v[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = (level(r[e]) - zf) * sc;
      if constexpr (sizeof(TD) == 2) {
        Vec16<TD> o;
#pragma unroll
        for (int e = 0; e < 8; ++e) o.set(e, v[e]);
        o.store(y + i * 8);
      } else {
        *reinterpret_cast<floatx4*>(reinterpret_cast<float*>(y) + i * 8) = (floatx4){v[0], v[1], v[2], v[3]};
        *reinterpret_cast<floatx4*>(reinterpret_cast<float*>(y) + i * 8 + 4) = (floatx4){v[4], v[5], v[6], v[7]};
      }
    }
    done = n8 * 8;
  }
  for (int64_t i = done + t0; i < p.n; i += stride) {
    const int c = (p.channels > 1) ? (int)((i / p.inner) % p.channels) : 0;
    const float zf = p.zp ? (float)p.zp[c] : 0.f;
    Store<TD>::st(y + i, (level(reinterpret_cast<const unsigned char*>(p.src)[i]) - zf) * p.scale[c]);
  }
}

__global__ void fill_i32_kernel(int32_t* p, int64_t n, int32_t v) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += stride) p[i] = v;
}

bool al16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// One launch for a group of unary / binary operators (see FusedParams).  The
// registers of the program live in LDS, one column per thread, because the
// program addresses them at run time.  A thread runs every instruction for E
// consecutive points of its walk at once (register q, point e at
// regs[(q * E + e) * kThreads + thread]): the E loads of an instruction are in
// flight together and the decoding of the instruction is shared.
// Activation inside a group.  With 16-bit storage the result keeps 8 or 11
// significant bits, so the hardware exponential and reciprocal (1 ulp each)
// stand in for the library's exp and the IEEE division.
template <typename T>
__device__ __forceinline__ float fused_act(const float v, const ActKind act, const float a, const float b) {
  if constexpr (sizeof(T) == 2) {
    if (act == ACT_SIGMOID) return __builtin_amdgcn_rcpf(1.0f + __expf(-v));
    if (act == ACT_EXP) return __expf(v);
  }
  return apply_act(v, act, a, b);
}

// I is the type of the index arithmetic: 32-bit when the walk and every view fit
// (integer division and multiplication in 64 bits cost several times as much).
template <typename T, int E, typename I>
__global__ void __launch_bounds__(kThreads) fused_eltwise_kernel(const FusedParams p) {
  extern __shared__ float fused_regs[];
  float* r = fused_regs + threadIdx.x;
  const I d1 = (I)p.dims[1], d2 = (I)p.dims[2], d3 = (I)p.dims[3];
  const I walk = p.walk > 0 ? (I)p.walk : d2;
  const I pieces = (d2 + walk - 1) / walk;
  const int64_t total = p.dims[0] * p.dims[1] * (int64_t)pieces * p.dims[3];
  for (int64_t t64 = blockIdx.x * (int64_t)kThreads + threadIdx.x; t64 < total; t64 += (int64_t)gridDim.x * kThreads) {
    const I t = (I)t64;
    I q = t / d3;
    const I i3 = t - q * d3;
    const I q1 = q / pieces;
    const I piece = q - q1 * pieces;
    const I i0 = q1 / d1;
    const I i1 = q1 - i0 * d1;
    const I i2_end = piece * walk + walk < d2 ? piece * walk + walk : d2;
    for (I i2 = piece * walk; i2 < i2_end; i2 += E) {
      const int live = i2_end - i2 < (I)E ? (int)(i2_end - i2) : E;
      for (int k = 0; k < p.n_instr; ++k) {
        const FusedInstr& in = p.prog[k];
        switch (in.op) {
          case FOP_LOAD: {
            const FusedView& v = p.view[in.a];
            const I st2 = (I)v.st[2];
            const T* src = reinterpret_cast<const T*>(v.base) +
                           (I)((I)v.off + i0 * (I)v.st[0] + i1 * (I)v.st[1] + i2 * st2 + i3 * (I)v.st[3]);
            float val[E];
#pragma unroll
            for (int e = 0; e < E; ++e) val[e] = e < live ? Store<T>::ld(src + (I)e * st2) : 0.f;
#pragma unroll
            for (int e = 0; e < E; ++e) r[(in.dst * E + e) * kThreads] = val[e];
            break;
          }
          case FOP_UNARY:
#pragma unroll
            for (int e = 0; e < E; ++e)
              r[(in.dst * E + e) * kThreads] = fused_act<T>(r[(in.a * E + e) * kThreads], (ActKind)in.kind, in.fa, in.fb);
            break;
          case FOP_BINARY:   // a negative register number selects the immediate
#pragma unroll
            for (int e = 0; e < E; ++e) {
              const float lhs = in.a < 0 ? in.fa : r[(in.a * E + e) * kThreads];
              const float rhs = in.b < 0 ? in.fa : r[(in.b * E + e) * kThreads];
              r[(in.dst * E + e) * kThreads] = bin_op(lhs, rhs, (BinKind)in.kind);
            }
            break;
          default: {
            const FusedView& v = p.view[in.dst];
            const I st2 = (I)v.st[2];
            T* dst = const_cast<T*>(reinterpret_cast<const T*>(v.base)) +
                     (I)((I)v.off + i0 * (I)v.st[0] + i1 * (I)v.st[1] + i2 * st2 + i3 * (I)v.st[3]);
#pragma unroll
            for (int e = 0; e < E; ++e)
              if (e < live) Store<T>::st(dst + (I)e * st2, r[(in.a * E + e) * kThreads]);
            break;
          }
        }
      }
    }
  }
}

}  // namespace

#define FLOAT_DISPATCH(dt, EXPR)                         \
  switch (dt) {                                          \
    case DT_F32: { using T = float; EXPR; break; }       \
    case DT_F16: { using T = f16_t; EXPR; break; }       \
    case DT_BF16: { using T = bf16_t; EXPR; break; }     \
    default: return hipErrorInvalidValue;                \
  }

hipError_t launch_unary(const void* x, void* y, DType dt, int64_t n, ActKind act, float a, float b,
                        hipStream_t stream) {
  if (n <= 0) return n == 0 ? hipSuccess : hipErrorInvalidValue;
  if (!x || !y || !al16(x) || !al16(y)) return hipErrorInvalidValue;
  constexpr int U = 4;
  const int64_t tiles = (n / (16 / dtype_size(dt)) + kThreads * U - 1) / (kThreads * U);
  if (tiles > 0x7fffffff) return hipErrorInvalidValue;
  const dim3 grid((unsigned)(tiles > 0 ? tiles : 1));
#define UNARY_CASE(K_)                                                                                  \
  case K_:                                                                                              \
    FLOAT_DISPATCH(dt, hipLaunchKernelGGL((unary_kernel<T, (int)K_, U>), grid, dim3(kThreads), 0, stream, \
                                          (const T*)x, (T*)y, n, act, a, b));                           \
    break;
  switch (act) {
    UNARY_CASE(ACT_RELU)
    UNARY_CASE(ACT_LEAKY)
    UNARY_CASE(ACT_CLAMP)
    UNARY_CASE(ACT_NEG)
    UNARY_CASE(ACT_SIGMOID)
    UNARY_CASE(ACT_TANH)
    UNARY_CASE(ACT_GELU_ERF)
    UNARY_CASE(ACT_GELU_TANH)
    UNARY_CASE(ACT_EXP)
    default:
      FLOAT_DISPATCH(dt, hipLaunchKernelGGL((unary_kernel<T, -1, U>), grid, dim3(kThreads), 0, stream, (const T*)x,
                                            (T*)y, n, act, a, b));
  }
#undef UNARY_CASE
  return hipGetLastError();
}

hipError_t launch_channel_affine(const void* x, void* y, DType dt, int64_t n, int64_t inner,
                                 int channels, const float* scale, const float* shift,
                                 hipStream_t stream) {
  if (n <= 0) return n == 0 ? hipSuccess : hipErrorInvalidValue;
  if (!x || !y || !scale || !shift || !al16(x) || !al16(y) || inner <= 0 || channels <= 0)
    return hipErrorInvalidValue;
  if (n % (inner * channels) != 0) return hipErrorInvalidValue;
  constexpr int U = 4;
  const int64_t tiles = (n / (16 / dtype_size(dt)) + kThreads * U - 1) / (kThreads * U);
  if (tiles > 0x7fffffff) return hipErrorInvalidValue;
  const unsigned grid = (unsigned)(tiles > 0 ? tiles : 1);
  FLOAT_DISPATCH(dt, hipLaunchKernelGGL((channel_affine_kernel<T, U>), dim3(grid), dim3(kThreads), 0,
                                        stream, (const T*)x, (T*)y, n, inner, channels, scale, shift));
  return hipGetLastError();
}

hipError_t launch_bn_fold(const float* mean, const float* var, const float* gamma,
                          const float* beta, float sgamma, float sbeta, float eps, int channels,
                          float* scale, float* shift, hipStream_t stream) {
  if (!mean || !var || !scale || !shift || channels <= 0) return hipErrorInvalidValue;
  hipLaunchKernelGGL(bn_fold_kernel, dim3((channels + 255) / 256), dim3(256), 0, stream, mean, var,
                     gamma, beta, sgamma, sbeta, eps, channels, scale, shift);
  return hipGetLastError();
}

hipError_t launch_binary(const BinaryParams& p, hipStream_t stream) {
  if (!p.a || !p.b || !p.y || p.rank < 1 || p.rank > 6) return hipErrorInvalidValue;
  int64_t n = 1;
  for (int d = 0; d < p.rank; ++d) {
    if (p.dims[d] <= 0) return hipErrorInvalidValue;
    n *= p.dims[d];
  }
  // contiguous strides of the output
  int64_t cs[6];
  {
    int64_t s = 1;
    for (int d = p.rank - 1; d >= 0; --d) { cs[d] = s; s *= p.dims[d]; }
  }
  auto is_full = [&](const int64_t* st) {
    for (int d = 0; d < p.rank; ++d)
      if (p.dims[d] != 1 && st[d] != cs[d]) return false;
    return true;
  };
  // operand indexed only by a trailing block of dims (contiguous there), 0 elsewhere
  auto rowvec_period = [&](const int64_t* st) -> int64_t {
    int d = p.rank - 1;
    int64_t period = 1;
    while (d >= 0 && (p.dims[d] == 1 || st[d] == cs[d])) { period *= p.dims[d]; --d; }
    for (; d >= 0; --d)
      if (p.dims[d] != 1 && st[d] != 0) return -1;
    return period;
  };
  const int grid = grid_for(n, kThreads * 8);
  if (p.dt == DT_I8) {
    if (!is_full(p.sa) || !is_full(p.sb) || !al16(p.a) || !al16(p.b) || !al16(p.y))
      return hipErrorInvalidValue;
    hipLaunchKernelGGL(binary_q8_kernel, dim3(grid_for(n, kThreads * 16)), dim3(kThreads), 0, stream, p, n);
    return hipGetLastError();
  }
  const bool aligned = al16(p.a) && al16(p.b) && al16(p.y);
  if (aligned && is_full(p.sa) && is_full(p.sb)) {
    constexpr int U = 4;
    const int64_t tiles = (n / (16 / dtype_size(p.dt)) + kThreads * U - 1) / (kThreads * U);
    if (tiles > 0x7fffffff) return hipErrorInvalidValue;
    const dim3 fgrid((unsigned)(tiles > 0 ? tiles : 1));
#define BIN_FLAT(OP_, K_)                                                                                           \
  FLOAT_DISPATCH(p.dt, hipLaunchKernelGGL((binary_flat_kernel<T, OP_, K_, U>), fgrid, dim3(kThreads), 0, stream,     \
                                          (const T*)p.a, (const T*)p.b, (T*)p.y, n, p.op, p.act, p.act_a, p.act_b))
    if (p.op == BIN_ADD && p.act == ACT_NONE) { BIN_FLAT((int)BIN_ADD, (int)ACT_NONE); }
    else if (p.op == BIN_ADD && p.act == ACT_RELU) { BIN_FLAT((int)BIN_ADD, (int)ACT_RELU); }
    else if (p.op == BIN_MUL && p.act == ACT_NONE) { BIN_FLAT((int)BIN_MUL, (int)ACT_NONE); }
    else if (p.op == BIN_SUB && p.act == ACT_NONE) { BIN_FLAT((int)BIN_SUB, (int)ACT_NONE); }
    else { BIN_FLAT(-1, -1); }
#undef BIN_FLAT
    return hipGetLastError();
  }
  if (aligned && is_full(p.sa)) {
    const int64_t per = rowvec_period(p.sb);
    if (per > 0 && per < (1ll << 30)) {
      FLOAT_DISPATCH(p.dt, hipLaunchKernelGGL(binary_rowvec_kernel<T>, dim3(grid), dim3(kThreads), 0,
                                              stream, (const T*)p.a, (const T*)p.b, (T*)p.y, n, (int)per,
                                              false, p.op, p.act, p.act_a, p.act_b));
      return hipGetLastError();
    }
  }
  if (aligned && is_full(p.sb)) {
    const int64_t per = rowvec_period(p.sa);
    if (per > 0 && per < (1ll << 30)) {
      FLOAT_DISPATCH(p.dt, hipLaunchKernelGGL(binary_rowvec_kernel<T>, dim3(grid), dim3(kThreads), 0,
                                              stream, (const T*)p.b, (const T*)p.a, (T*)p.y, n, (int)per,
                                              true, p.op, p.act, p.act_a, p.act_b));
      return hipGetLastError();
    }
  }
  FLOAT_DISPATCH(p.dt, hipLaunchKernelGGL(binary_bcast_kernel<T>, dim3(grid_for(n, kThreads * 2)),
                                          dim3(kThreads), 0, stream, p, n));
  return hipGetLastError();
}

hipError_t launch_cast(const void* src, DType sdt, void* dst, DType ddt, int64_t n, hipStream_t stream) {
  if (n <= 0) return n == 0 ? hipSuccess : hipErrorInvalidValue;
  if (!src || !dst) return hipErrorInvalidValue;
  const int grid = grid_for(n, kThreads * 4);
#define CAST_CASE(S_, D_, TS_, TD_, K_)                                                   \
  if (sdt == S_ && ddt == D_) {                                                           \
    hipLaunchKernelGGL((K_<TS_, TD_>), dim3(grid), dim3(kThreads), 0, stream, (const TS_*)src, \
                       (TD_*)dst, n);                                                     \
    return hipGetLastError();                                                             \
  }
  CAST_CASE(DT_F32, DT_F16, float, f16_t, cast_kernel)
  CAST_CASE(DT_F32, DT_BF16, float, bf16_t, cast_kernel)
  CAST_CASE(DT_F16, DT_F32, f16_t, float, cast_kernel)
  CAST_CASE(DT_BF16, DT_F32, bf16_t, float, cast_kernel)
  CAST_CASE(DT_F32, DT_F32, float, float, cast_kernel)
  CAST_CASE(DT_F16, DT_F16, f16_t, f16_t, cast_kernel)
  CAST_CASE(DT_BF16, DT_BF16, bf16_t, bf16_t, cast_kernel)
  CAST_CASE(DT_F16, DT_BF16, f16_t, bf16_t, cast_kernel)
  CAST_CASE(DT_BF16, DT_F16, bf16_t, f16_t, cast_kernel)
#define CAST_INT_CASE(S_, D_, TS_, TD_, B_)                                                  \
  if (sdt == S_ && ddt == D_) {                                                              \
    hipLaunchKernelGGL((cast_int_kernel<TS_, TD_, B_>), dim3(grid), dim3(kThreads), 0, stream, \
                       (const TS_*)src, (TD_*)dst, n);                                       \
    return hipGetLastError();                                                                \
  }
  // every source type to every integer type and bool ...
#define CAST_TO_INTS(S_, TS_)                        \
  CAST_INT_CASE(S_, DT_I8, TS_, int8_t, false)       \
  CAST_INT_CASE(S_, DT_U8, TS_, uint8_t, false)      \
  CAST_INT_CASE(S_, DT_I32, TS_, int32_t, false)     \
  CAST_INT_CASE(S_, DT_I64, TS_, int64_t, false)     \
  CAST_INT_CASE(S_, DT_BOOL, TS_, uint8_t, true)
  CAST_TO_INTS(DT_F32, float)
  CAST_TO_INTS(DT_F16, f16_t)
  CAST_TO_INTS(DT_BF16, bf16_t)
  CAST_TO_INTS(DT_I8, int8_t)
  CAST_TO_INTS(DT_U8, uint8_t)
  CAST_TO_INTS(DT_I32, int32_t)
  CAST_TO_INTS(DT_I64, int64_t)
  CAST_TO_INTS(DT_BOOL, uint8_t)
  // ... and every integer type and bool to every floating-point type
#define CAST_TO_FLOATS(S_, TS_)                      \
  CAST_INT_CASE(S_, DT_F32, TS_, float, false)       \
  CAST_INT_CASE(S_, DT_F16, TS_, f16_t, false)       \
  CAST_INT_CASE(S_, DT_BF16, TS_, bf16_t, false)
  CAST_TO_FLOATS(DT_I8, int8_t)
  CAST_TO_FLOATS(DT_U8, uint8_t)
  CAST_TO_FLOATS(DT_I32, int32_t)
  CAST_TO_FLOATS(DT_I64, int64_t)
  CAST_TO_FLOATS(DT_BOOL, uint8_t)
#undef CAST_TO_FLOATS
#undef CAST_TO_INTS
#undef CAST_INT_CASE
#undef CAST_CASE
  return hipErrorInvalidValue;
}

hipError_t launch_quantize(const QuantParams& p, hipStream_t stream) {
  if (p.n <= 0) return p.n == 0 ? hipSuccess : hipErrorInvalidValue;
  if (!p.src || !p.dst || !p.scale || p.channels <= 0 || p.inner <= 0) return hipErrorInvalidValue;
  if (p.dst_dt != DT_U8 && p.dst_dt != DT_I8) return hipErrorInvalidValue;
  const int grid = grid_for(p.n, kThreads * 16);
  FLOAT_DISPATCH(p.src_dt, hipLaunchKernelGGL(quantize_kernel<T>, dim3(grid), dim3(kThreads), 0, stream, p));
  return hipGetLastError();
}

hipError_t launch_dequantize(const QuantParams& p, hipStream_t stream) {
  if (p.n <= 0) return p.n == 0 ? hipSuccess : hipErrorInvalidValue;
  if (!p.src || !p.dst || !p.scale || p.channels <= 0 || p.inner <= 0) return hipErrorInvalidValue;
  if (p.src_dt != DT_U8 && p.src_dt != DT_I8) return hipErrorInvalidValue;
  const int grid = grid_for(p.n, kThreads * 16);
  FLOAT_DISPATCH(p.dst_dt, hipLaunchKernelGGL(dequantize_kernel<T>, dim3(grid), dim3(kThreads), 0, stream, p));
  return hipGetLastError();
}

hipError_t launch_fill_i32(int32_t* p, int64_t n, int32_t v, hipStream_t stream) {
  if (n <= 0) return n == 0 ? hipSuccess : hipErrorInvalidValue;
  if (!p) return hipErrorInvalidValue;
  hipLaunchKernelGGL(fill_i32_kernel, dim3(grid_for(n, 256)), dim3(256), 0, stream, p, n, v);
  return hipGetLastError();
}

hipError_t launch_fused_eltwise(const FusedParams& p, hipStream_t stream) {
  if (p.n_instr <= 0 || p.n_instr > kFusedMaxInstr) return hipErrorInvalidValue;
  int64_t threads = 1;
  for (int i = 0; i < 4; ++i) {
    if (p.dims[i] <= 0) return hipErrorInvalidValue;
    if (i != 2) threads *= p.dims[i];
  }
  if (p.walk < 0) return hipErrorInvalidValue;
  const int64_t walk = p.walk > 0 ? p.walk : p.dims[2];
  threads *= (p.dims[2] + walk - 1) / walk;
  for (int k = 0; k < p.n_instr; ++k) {
    const FusedInstr& in = p.prog[k];
    const bool is_store = in.op == FOP_STORE, is_load = in.op == FOP_LOAD;
    const int view = is_store ? in.dst : in.a;
    if ((is_store || is_load) && (view < 0 || view >= kFusedMaxViews || p.view[view].base == nullptr)) return hipErrorInvalidValue;
    if (!is_store && (in.dst < 0 || in.dst >= kFusedMaxRegs)) return hipErrorInvalidValue;
    const bool is_bin = in.op == FOP_BINARY;
    if (!is_load && (in.a >= kFusedMaxRegs || (in.a < 0 && !is_bin))) return hipErrorInvalidValue;
    if (is_bin && (in.b >= kFusedMaxRegs || (in.a < 0 && in.b < 0))) return hipErrorInvalidValue;
    if (in.op < FOP_LOAD || in.op > FOP_STORE) return hipErrorInvalidValue;
  }
  int n_regs = 1;
  for (int k = 0; k < p.n_instr; ++k)
    if (p.prog[k].op != FOP_STORE && p.prog[k].dst + 1 > n_regs) n_regs = p.prog[k].dst + 1;
  // points of the walk per instruction: as many as 32 KiB of LDS registers allow
  const int e = (walk >= 4 && n_regs * 4 <= 32) ? 4 : ((walk >= 2 && n_regs * 2 <= 32) ? 2 : 1);
  const size_t lds = (size_t)n_regs * e * kThreads * sizeof(float);
  const int grid = grid_for(threads, kThreads);
  // 32-bit index arithmetic when the thread count and every view's furthest element fit
  bool small = threads < ((int64_t)1 << 31);
  for (int v = 0; v < kFusedMaxViews && small; ++v) {
    if (p.view[v].base == nullptr) continue;
    int64_t far = p.view[v].off;
    if (far < 0) small = false;
    for (int q = 0; q < 4 && small; ++q) {
      if (p.view[v].st[q] < 0) small = false;
      else far += (p.dims[q] - 1 + (q == 2 ? e : 0)) * p.view[v].st[q];
    }
    if (far >= ((int64_t)1 << 31)) small = false;
  }
#define FUSED_LAUNCH(E_)                                                                                                  \
  do {                                                                                                                    \
    if (small) { FLOAT_DISPATCH(p.dt, hipLaunchKernelGGL((fused_eltwise_kernel<T, E_, uint32_t>), dim3(grid), dim3(kThreads), lds, stream, p)); } \
    else { FLOAT_DISPATCH(p.dt, hipLaunchKernelGGL((fused_eltwise_kernel<T, E_, int64_t>), dim3(grid), dim3(kThreads), lds, stream, p)); }        \
  } while (0)
  if (e == 4) FUSED_LAUNCH(4);
  else if (e == 2) FUSED_LAUNCH(2);
  else FUSED_LAUNCH(1);
#undef FUSED_LAUNCH
  return hipGetLastError();
}

}  // namespace ohip
