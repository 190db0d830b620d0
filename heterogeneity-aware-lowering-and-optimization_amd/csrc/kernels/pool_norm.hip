// Pooling, axis reductions, softmax and layer normalisation for gfx950.
// All are HBM-bound streaming kernels: channels-last pooling moves 16-byte
// channel vectors, row kernels keep the row in registers between the
// statistics pass and the normalising pass so every element is read once.
#include "device_utils.h"

namespace ohip {
namespace {

constexpr int kThreads = 256;

// --------------------------------------------------------------------------
// Pooling, channels-last.  One thread per (n, ho, wo, channel vector).
template <typename T, bool IS_MAX>
__global__ void __launch_bounds__(kThreads) pool2d_vec_kernel(PoolParams p) {
  constexpr int V = Vec16<T>::N;
  const int cv = p.C / V;  // C % V == 0 checked by the launcher
  const int64_t total = (int64_t)p.N * p.Ho * p.Wo * cv;
  const T* x = reinterpret_cast<const T*>(p.x);
  T* y = reinterpret_cast<T*>(p.y);
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int c = (int)(i % cv) * V;
    int64_t t = i / cv;
    const int wo = (int)(t % p.Wo); t /= p.Wo;
    const int ho = (int)(t % p.Ho);
    const int n = (int)(t / p.Ho);
    const int h0 = ho * p.sh - p.ph, w0 = wo * p.sw - p.pw;
    float acc[V];
#pragma unroll
    for (int e = 0; e < V; ++e) acc[e] = IS_MAX ? -INFINITY : 0.f;
    int cnt = 0;
    for (int r = 0; r < p.kh; ++r) {
      const int hi = h0 + r;
      if ((unsigned)hi >= (unsigned)p.H) continue;
      for (int s = 0; s < p.kw; ++s) {
        const int wi = w0 + s;
        if ((unsigned)wi >= (unsigned)p.W) continue;
        Vec16<T> v;
        v.load(x + (((int64_t)n * p.H + hi) * p.W + wi) * p.cs + c);
#pragma unroll
        for (int e = 0; e < V; ++e) acc[e] = IS_MAX ? fmaxf(acc[e], v.get(e)) : acc[e] + v.get(e);
        ++cnt;
      }
    }
    Vec16<T> o;
    if (IS_MAX) {
#pragma unroll
      for (int e = 0; e < V; ++e) o.set(e, acc[e]);
    } else {
      const float div = (float)(p.count_include_pad ? p.kh * p.kw : (cnt > 0 ? cnt : 1));
#pragma unroll
      for (int e = 0; e < V; ++e) o.set(e, acc[e] / div);
    }
    o.store(y + (((int64_t)n * p.Ho + ho) * p.Wo + wo) * p.ycs + c);
  }
}

// Scalar-channel fallback (C not a multiple of the vector width).
template <typename T, bool IS_MAX>
__global__ void __launch_bounds__(kThreads) pool2d_scalar_kernel(PoolParams p) {
  const int64_t total = (int64_t)p.N * p.Ho * p.Wo * p.C;
  const T* x = reinterpret_cast<const T*>(p.x);
  T* y = reinterpret_cast<T*>(p.y);
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int c = (int)(i % p.C);
    int64_t t = i / p.C;
    const int wo = (int)(t % p.Wo); t /= p.Wo;
    const int ho = (int)(t % p.Ho);
    const int n = (int)(t / p.Ho);
    const int h0 = ho * p.sh - p.ph, w0 = wo * p.sw - p.pw;
    float acc = IS_MAX ? -INFINITY : 0.f;
    int cnt = 0;
    for (int r = 0; r < p.kh; ++r) {
      const int hi = h0 + r;
      if ((unsigned)hi >= (unsigned)p.H) continue;
      for (int s = 0; s < p.kw; ++s) {
        const int wi = w0 + s;
        if ((unsigned)wi >= (unsigned)p.W) continue;
        const float v = Store<T>::ld(x + (((int64_t)n * p.H + hi) * p.W + wi) * p.cs + c);
        acc = IS_MAX ? fmaxf(acc, v) : acc + v;
        ++cnt;
      }
    }
    if (!IS_MAX) acc /= (float)(p.count_include_pad ? p.kh * p.kw : (cnt > 0 ? cnt : 1));
    Store<T>::st(y + (((int64_t)n * p.Ho + ho) * p.Wo + wo) * p.ycs + c, acc);
  }
}

// 8-bit levels stored as q-128.  Max keeps levels; average requantises:
// q = clamp(rne(((sum - cnt*zp_in) / cnt) * q_mul) + zp_out, 0, 255).
template <bool IS_MAX>
__global__ void __launch_bounds__(kThreads) pool2d_q8_kernel(PoolParams p) {
  const int cv = p.C / 16;
  const int64_t total = (int64_t)p.N * p.Ho * p.Wo * cv;
  const int8_t* x = reinterpret_cast<const int8_t*>(p.x);
  int8_t* y = reinterpret_cast<int8_t*>(p.y);
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int c = (int)(i % cv) * 16;
    int64_t t = i / cv;
    const int wo = (int)(t % p.Wo); t /= p.Wo;
    const int ho = (int)(t % p.Ho);
    const int n = (int)(t / p.Ho);
    const int h0 = ho * p.sh - p.ph, w0 = wo * p.sw - p.pw;
    int acc[16];
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = IS_MAX ? -1000 : 0;
    int cnt = 0;
    for (int r = 0; r < p.kh; ++r) {
      const int hi = h0 + r;
      if ((unsigned)hi >= (unsigned)p.H) continue;
      for (int s = 0; s < p.kw; ++s) {
        const int wi = w0 + s;
        if ((unsigned)wi >= (unsigned)p.W) continue;
        const uintx4 v = *reinterpret_cast<const uintx4*>(x + (((int64_t)n * p.H + hi) * p.W + wi) * p.cs + c);
        const int8_t* ev = reinterpret_cast<const int8_t*>(&v);
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int q = q_from_stored(ev[e]);
          acc[e] = IS_MAX ? (q > acc[e] ? q : acc[e]) : acc[e] + q;
        }
        ++cnt;
      }
    }
    uintx4 o;
    int8_t* eo = reinterpret_cast<int8_t*>(&o);
    const int div = p.count_include_pad ? p.kh * p.kw : (cnt > 0 ? cnt : 1);
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      int q;
      if (IS_MAX) {
        q = acc[e];
      } else {
        const float f = (float)(acc[e] - cnt * p.zp_in) / (float)div;
        q = (int)rintf(f * p.q_mul) + p.zp_out;
        q = q < 0 ? 0 : (q > 255 ? 255 : q);
      }
      eo[e] = q_to_stored(q);
    }
    *reinterpret_cast<uintx4*>(y + (((int64_t)n * p.Ho + ho) * p.Wo + wo) * p.ycs + c) = o;
  }
}

// --------------------------------------------------------------------------
// Reduction over the middle axis of [outer][len][inner].
// inner == 1: one wavefront per row, lanes stride the row.
template <typename TI, typename TO>
__global__ void __launch_bounds__(kThreads)
reduce_rows_kernel(const TI* __restrict__ x, TO* __restrict__ y, int64_t rows, int64_t len,
                   ReduceKind kind) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = (blockIdx.x * (int64_t)blockDim.x + threadIdx.x) >> 6;
  const int64_t nwaves = ((int64_t)gridDim.x * blockDim.x) >> 6;
  for (int64_t r = wave; r < rows; r += nwaves) {
    const TI* row = x + r * len;
    float acc = kind == RED_MAX ? -INFINITY : 0.f;
    for (int64_t i = lane; i < len; i += 64) {
      const float v = Store<TI>::ld(row + i);
      acc = kind == RED_MAX ? fmaxf(acc, v) : acc + v;
    }
    acc = kind == RED_MAX ? wave_max(acc) : wave_sum(acc);
    if (kind == RED_MEAN) acc /= (float)len;
    if (lane == 0) Store<TO>::st(y + r, acc);
  }
}
// inner > 1: one thread per (outer, inner) column; consecutive threads read
// consecutive inner positions, so each step over `len` is a coalesced row.
template <typename TI, typename TO>
__global__ void __launch_bounds__(kThreads)
reduce_cols_kernel(const TI* __restrict__ x, TO* __restrict__ y, int64_t outer, int64_t len,
                   int64_t inner, ReduceKind kind) {
  const int64_t total = outer * inner;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t o = i / inner, in = i - o * inner;
    const TI* col = x + o * len * inner + in;
    float acc = kind == RED_MAX ? -INFINITY : 0.f;
    for (int64_t k = 0; k < len; ++k) {
      const float v = Store<TI>::ld(col + k * inner);
      acc = kind == RED_MAX ? fmaxf(acc, v) : acc + v;
    }
    if (kind == RED_MEAN) acc /= (float)len;
    Store<TO>::st(y + i, acc);
  }
}
// Quantised mean over the middle axis: y = ((sum - len*zp) / len) * scale (fp32).
__global__ void __launch_bounds__(kThreads)
reduce_cols_q8_kernel(const int8_t* __restrict__ x, float* __restrict__ y, int64_t outer,
                      int64_t len, int64_t inner, float scale, int zp) {
  const int64_t total = outer * inner;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t o = i / inner, in = i - o * inner;
    const int8_t* col = x + o * len * inner + in;
    int acc = 0;
    for (int64_t k = 0; k < len; ++k) acc += q_from_stored(col[k * inner]);
    y[i] = ((float)(acc - (int)len * zp) / (float)len) * scale;
  }
}

// --------------------------------------------------------------------------
// Softmax over a contiguous row (inner == 1).  A workgroup of NT threads
// owns one row at a time; each thread keeps up to PER elements in registers.
template <typename TI, typename TO, int NT, int PER>
__global__ void __launch_bounds__(NT)
softmax_row_kernel(const TI* __restrict__ x, TO* __restrict__ y, int64_t rows, int len, bool logsm) {
  __shared__ float red[NT / 64];
  for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
    const TI* row = x + r * (int64_t)len;
    float v[PER];
    float mx = -INFINITY;
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int i = threadIdx.x + k * NT;
      v[k] = i < len ? Store<TI>::ld(row + i) : -INFINITY;
      mx = fmaxf(mx, v[k]);
    }
    mx = block_max<NT>(mx, red);
    float sum = 0.f;
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int i = threadIdx.x + k * NT;
      const float e = i < len ? expf(v[k] - mx) : 0.f;
      sum += e;
      if (!logsm) v[k] = e;
    }
    sum = block_sum<NT>(sum, red);
    TO* out = y + r * (int64_t)len;
    const float lsum = logf(sum);
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int i = threadIdx.x + k * NT;
      if (i < len) Store<TO>::st(out + i, logsm ? (v[k] - mx - lsum) : v[k] / sum);
    }
    __syncthreads();
  }
}
// Short rows: one wavefront per row, whole row in registers (len <= 64*PER).
template <typename TI, typename TO, int PER>
__global__ void __launch_bounds__(kThreads)
softmax_wave_kernel(const TI* __restrict__ x, TO* __restrict__ y, int64_t rows, int len, bool logsm) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = (blockIdx.x * (int64_t)blockDim.x + threadIdx.x) >> 6;
  const int64_t nwaves = ((int64_t)gridDim.x * blockDim.x) >> 6;
  for (int64_t r = wave; r < rows; r += nwaves) {
    const TI* row = x + r * (int64_t)len;
    float v[PER];
    float mx = -INFINITY;
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int i = lane + k * 64;
      v[k] = i < len ? Store<TI>::ld(row + i) : -INFINITY;
      mx = fmaxf(mx, v[k]);
    }
    mx = wave_max(mx);
    float sum = 0.f;
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int i = lane + k * 64;
      const float e = i < len ? expf(v[k] - mx) : 0.f;
      sum += e;
      if (!logsm) v[k] = e;
    }
    sum = wave_sum(sum);
    const float lsum = logf(sum);
    TO* out = y + r * (int64_t)len;
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int i = lane + k * 64;
      if (i < len) Store<TO>::st(out + i, logsm ? (v[k] - mx - lsum) : v[k] / sum);
    }
  }
}
// Generic: strided axis or very long rows; three passes over the column.
template <typename TI, typename TO>
__global__ void __launch_bounds__(kThreads)
softmax_generic_kernel(const TI* __restrict__ x, TO* __restrict__ y, int64_t outer, int64_t len,
                       int64_t inner, bool logsm) {
  const int64_t total = outer * inner;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t o = i / inner, in = i - o * inner;
    const TI* col = x + o * len * inner + in;
    TO* out = y + o * len * inner + in;
    float mx = -INFINITY;
    for (int64_t k = 0; k < len; ++k) mx = fmaxf(mx, Store<TI>::ld(col + k * inner));
    float sum = 0.f;
    for (int64_t k = 0; k < len; ++k) sum += expf(Store<TI>::ld(col + k * inner) - mx);
    const float lsum = logf(sum);
    for (int64_t k = 0; k < len; ++k) {
      const float d = Store<TI>::ld(col + k * inner) - mx;
      Store<TO>::st(out + k * inner, logsm ? d - lsum : expf(d) / sum);
    }
  }
}

// --------------------------------------------------------------------------
// LayerNorm over contiguous rows: biased variance, eps inside the root.
template <typename T, int NT, int PER>
__global__ void __launch_bounds__(NT)
layernorm_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t rows, int len,
                 const float* __restrict__ gamma, const float* __restrict__ beta, float eps) {
  __shared__ float red[NT / 64];
  for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
    const T* row = x + r * (int64_t)len;
    float v[PER];
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int i = threadIdx.x + k * NT;
      v[k] = i < len ? Store<T>::ld(row + i) : 0.f;
      s += v[k];
    }
    const float mean = block_sum<NT>(s, red) / (float)len;
    float q = 0.f;
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int i = threadIdx.x + k * NT;
      const float d = i < len ? v[k] - mean : 0.f;
      q += d * d;
    }
    const float var = block_sum<NT>(q, red) / (float)len;
    const float rstd = 1.0f / sqrtf(var + eps);
    T* out = y + r * (int64_t)len;
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int i = threadIdx.x + k * NT;
      if (i < len) {
        const float g = gamma ? gamma[i] : 1.f, b = beta ? beta[i] : 0.f;
        Store<T>::st(out + i, (v[k] - mean) * rstd * g + b);
      }
    }
    __syncthreads();
  }
}

bool al16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace

#define FLOAT_DISPATCH(dt, EXPR)                         \
  switch (dt) {                                          \
    case DT_F32: { using T = float; EXPR; break; }       \
    case DT_F16: { using T = f16_t; EXPR; break; }       \
    case DT_BF16: { using T = bf16_t; EXPR; break; }     \
    default: return hipErrorInvalidValue;                \
  }

hipError_t launch_pool2d(const PoolParams& p, hipStream_t stream) {
  if (!p.x || !p.y || p.N <= 0 || p.H <= 0 || p.W <= 0 || p.C <= 0 || p.Ho <= 0 || p.Wo <= 0)
    return hipErrorInvalidValue;
  if (p.cs < p.C || p.ycs < p.C || p.kh <= 0 || p.kw <= 0 || p.sh <= 0 || p.sw <= 0)
    return hipErrorInvalidValue;
  const int es = dtype_size(p.dt);
  if (es == 0) return hipErrorInvalidValue;
  const int V = 16 / es;
  const bool vec = (p.C % V == 0) && (p.cs % V == 0) && (p.ycs % V == 0) && al16(p.x) && al16(p.y);
  if (p.dt == DT_I8) {
    if (!vec) return hipErrorInvalidValue;
    const int64_t total = (int64_t)p.N * p.Ho * p.Wo * (p.C / 16);
    const int grid = grid_for(total, kThreads);
    if (p.is_max) hipLaunchKernelGGL(pool2d_q8_kernel<true>, dim3(grid), dim3(kThreads), 0, stream, p);
    else hipLaunchKernelGGL(pool2d_q8_kernel<false>, dim3(grid), dim3(kThreads), 0, stream, p);
    return hipGetLastError();
  }
  if (vec) {
    const int64_t total = (int64_t)p.N * p.Ho * p.Wo * (p.C / V);
    const int grid = grid_for(total, kThreads);
    if (p.is_max) { FLOAT_DISPATCH(p.dt, hipLaunchKernelGGL((pool2d_vec_kernel<T, true>), dim3(grid), dim3(kThreads), 0, stream, p)); }
    else { FLOAT_DISPATCH(p.dt, hipLaunchKernelGGL((pool2d_vec_kernel<T, false>), dim3(grid), dim3(kThreads), 0, stream, p)); }
  } else {
    const int64_t total = (int64_t)p.N * p.Ho * p.Wo * p.C;
    const int grid = grid_for(total, kThreads);
    if (p.is_max) { FLOAT_DISPATCH(p.dt, hipLaunchKernelGGL((pool2d_scalar_kernel<T, true>), dim3(grid), dim3(kThreads), 0, stream, p)); }
    else { FLOAT_DISPATCH(p.dt, hipLaunchKernelGGL((pool2d_scalar_kernel<T, false>), dim3(grid), dim3(kThreads), 0, stream, p)); }
  }
  return hipGetLastError();
}

hipError_t launch_reduce_q8_mean(const void* x, float* y, int64_t outer, int64_t len, int64_t inner,
                                 float scale, int zp, hipStream_t stream) {
  if (!x || !y || outer <= 0 || len <= 0 || inner <= 0 || len > (1 << 23)) return hipErrorInvalidValue;
  hipLaunchKernelGGL(reduce_cols_q8_kernel, dim3(grid_for(outer * inner, kThreads)), dim3(kThreads), 0,
                     stream, (const int8_t*)x, y, outer, len, inner, scale, zp);
  return hipGetLastError();
}

template <typename TI>
static hipError_t reduce_out(const void* x, void* y, DType out_dt, int64_t outer, int64_t len,
                             int64_t inner, ReduceKind kind, hipStream_t stream) {
  auto go = [&](auto tag) -> hipError_t {
    using TO = decltype(tag);
    if (inner == 1) {
      const int grid = grid_for(outer * 64, kThreads);
      hipLaunchKernelGGL((reduce_rows_kernel<TI, TO>), dim3(grid), dim3(kThreads), 0, stream,
                         (const TI*)x, (TO*)y, outer, len, kind);
    } else {
      const int grid = grid_for(outer * inner, kThreads);
      hipLaunchKernelGGL((reduce_cols_kernel<TI, TO>), dim3(grid), dim3(kThreads), 0, stream,
                         (const TI*)x, (TO*)y, outer, len, inner, kind);
    }
    return hipGetLastError();
  };
  if (out_dt == DT_F32) return go(float{});
  if (out_dt == DT_F16) return go(f16_t{});
  if (out_dt == DT_BF16) return go(bf16_t{});
  return hipErrorInvalidValue;
}

hipError_t launch_reduce(const void* x, void* y, DType in_dt, DType out_dt, int64_t outer,
                         int64_t len, int64_t inner, ReduceKind kind, hipStream_t stream) {
  if (!x || !y || outer <= 0 || len <= 0 || inner <= 0) return hipErrorInvalidValue;
  switch (in_dt) {
    case DT_F32: return reduce_out<float>(x, y, out_dt, outer, len, inner, kind, stream);
    case DT_F16: return reduce_out<f16_t>(x, y, out_dt, outer, len, inner, kind, stream);
    case DT_BF16: return reduce_out<bf16_t>(x, y, out_dt, outer, len, inner, kind, stream);
    default: return hipErrorInvalidValue;
  }
}

template <typename TI, typename TO>
static hipError_t softmax_typed(const void* x, void* y, int64_t outer, int64_t len, int64_t inner,
                                bool logsm, hipStream_t stream) {
  if (inner == 1 && len <= 64 * 4) {
    const int grid = grid_for(outer * 64, kThreads);
    if (len <= 64) hipLaunchKernelGGL((softmax_wave_kernel<TI, TO, 1>), dim3(grid), dim3(kThreads), 0, stream, (const TI*)x, (TO*)y, outer, (int)len, logsm);
    else if (len <= 128) hipLaunchKernelGGL((softmax_wave_kernel<TI, TO, 2>), dim3(grid), dim3(kThreads), 0, stream, (const TI*)x, (TO*)y, outer, (int)len, logsm);
    else hipLaunchKernelGGL((softmax_wave_kernel<TI, TO, 4>), dim3(grid), dim3(kThreads), 0, stream, (const TI*)x, (TO*)y, outer, (int)len, logsm);
  } else if (inner == 1 && len <= 256 * 16) {
    const int grid = (int)(outer < 8192 ? outer : 8192);
    if (len <= 256 * 4) hipLaunchKernelGGL((softmax_row_kernel<TI, TO, 256, 4>), dim3(grid), dim3(256), 0, stream, (const TI*)x, (TO*)y, outer, (int)len, logsm);
    else hipLaunchKernelGGL((softmax_row_kernel<TI, TO, 256, 16>), dim3(grid), dim3(256), 0, stream, (const TI*)x, (TO*)y, outer, (int)len, logsm);
  } else {
    const int grid = grid_for(outer * inner, kThreads);
    hipLaunchKernelGGL((softmax_generic_kernel<TI, TO>), dim3(grid), dim3(kThreads), 0, stream,
                       (const TI*)x, (TO*)y, outer, len, inner, logsm);
  }
  return hipGetLastError();
}

hipError_t launch_softmax(const void* x, void* y, DType in_dt, DType out_dt, int64_t outer,
                          int64_t len, int64_t inner, bool log_softmax, hipStream_t stream) {
  if (!x || !y || outer <= 0 || len <= 0 || inner <= 0 || len >= (1ll << 31)) return hipErrorInvalidValue;
#define SM_CASE(I_, O_, TI_, TO_) \
  if (in_dt == I_ && out_dt == O_) return softmax_typed<TI_, TO_>(x, y, outer, len, inner, log_softmax, stream);
  SM_CASE(DT_F32, DT_F32, float, float)
  SM_CASE(DT_F16, DT_F16, f16_t, f16_t)
  SM_CASE(DT_BF16, DT_BF16, bf16_t, bf16_t)
  SM_CASE(DT_F16, DT_F32, f16_t, float)
  SM_CASE(DT_BF16, DT_F32, bf16_t, float)
#undef SM_CASE
  return hipErrorInvalidValue;
}

hipError_t launch_layernorm(const void* x, void* y, DType dt, int64_t rows, int64_t len,
                            const float* gamma, const float* beta, float eps, hipStream_t stream) {
  if (!x || !y || rows <= 0 || len <= 0) return hipErrorInvalidValue;
  if (len > 256 * 16) return hipErrorInvalidValue;
  const int grid = (int)(rows < 16384 ? rows : 16384);
  if (len <= 256 * 4) {
    FLOAT_DISPATCH(dt, hipLaunchKernelGGL((layernorm_kernel<T, 256, 4>), dim3(grid), dim3(256), 0, stream,
                                          (const T*)x, (T*)y, rows, (int)len, gamma, beta, eps));
  } else {
    FLOAT_DISPATCH(dt, hipLaunchKernelGGL((layernorm_kernel<T, 256, 16>), dim3(grid), dim3(256), 0, stream,
                                          (const T*)x, (T*)y, rows, (int)len, gamma, beta, eps));
  }
  return hipGetLastError();
}

}  // namespace ohip
