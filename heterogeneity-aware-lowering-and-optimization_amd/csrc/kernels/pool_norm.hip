// Pooling, axis reductions, softmax and layer normalisation for gfx950.
// All are HBM-bound streaming kernels: channels-last pooling moves 16-byte
// channel vectors, row kernels keep the row in registers between the
// statistics pass and the normalising pass so every element is read once.
#include <type_traits>

#include "device_utils.h"

namespace ohip {
namespace {

constexpr int kThreads = 256;

inline bool al16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// --------------------------------------------------------------------------
// Pooling, channels-last.  One thread per (n, ho, wo, channel vector).
// KH, KW > 0: compile-time window; all taps are loaded unconditionally from a
// clamped (always valid) address so that the loads issue back to back, and
// out-of-range taps are masked afterwards.  KH == 0: run-time window.
template <typename T, bool IS_MAX, int KH, int KW>
__global__ void __launch_bounds__(kThreads) pool2d_vec_kernel(PoolParams p) {
  constexpr int V = Vec16<T>::N;
  const int cv = p.C / V;  // C % V == 0 checked by the launcher
  const T* x = reinterpret_cast<const T*>(p.x);
  T* y = reinterpret_cast<T*>(p.y);
  // blockIdx.x walks the (ho, wo, channel vector) positions of one image, blockIdx.y the
  // images: 32-bit index arithmetic with magic divisions (a 64-bit division per thread
  // costs as much as the thread's memory traffic)
  const int per_image = p.Ho * p.Wo * cv, row = p.Wo * cv;
  const int i = blockIdx.x * kThreads + threadIdx.x;
  if (i >= per_image) return;
  const int ho = fast_div(i, p.row_magic, p.row_shift);
  const int rem = i - ho * row;
  const int wo = fast_div(rem, p.cv_magic, p.cv_shift);
  const int c = (rem - wo * cv) * V;
  for (int n = blockIdx.y; n < p.N; n += gridDim.y) {
    const int h0 = ho * p.sh - p.ph, w0 = wo * p.sw - p.pw;
    float acc[V];
#pragma unroll
    for (int e = 0; e < V; ++e) acc[e] = IS_MAX ? -INFINITY : 0.f;
    int cnt = 0;
    if constexpr (KH > 0) {
      Vec16<T> v[KH * KW];
      bool ok[KH * KW];
#pragma unroll
      for (int r = 0; r < KH; ++r)
#pragma unroll
        for (int s = 0; s < KW; ++s) {
          const int hi = h0 + r, wi = w0 + s;
          ok[r * KW + s] = ((unsigned)hi < (unsigned)p.H) && ((unsigned)wi < (unsigned)p.W);
          const int hc = hi < 0 ? 0 : (hi >= p.H ? p.H - 1 : hi);
          const int wc = wi < 0 ? 0 : (wi >= p.W ? p.W - 1 : wi);
          v[r * KW + s].load(x + (((int64_t)n * p.H + hc) * p.W + wc) * p.cs + c);
        }
#pragma unroll
      for (int k = 0; k < KH * KW; ++k) {
        if (ok[k]) {
#pragma unroll
          for (int e = 0; e < V; ++e) acc[e] = IS_MAX ? fmaxf(acc[e], v[k].get(e)) : acc[e] + v[k].get(e);
          ++cnt;
        }
      }
    } else {
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
    __builtin_nontemporal_store(o.raw, reinterpret_cast<uintx4*>(y + (((int64_t)n * p.Ho + ho) * p.Wo + wo) * p.ycs + c));
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
// KH, KW > 0 (maximum only): a window of that size with all its loads in flight at once.
// A tap outside the image is read at the nearest position inside, which belongs to the
// same window (every window overlaps the image), so the maximum is unchanged.
template <bool IS_MAX, int KH = 0, int KW = 0>
__global__ void __launch_bounds__(kThreads) pool2d_q8_kernel(PoolParams p) {
  const int cv = p.C / 16;
  const int8_t* x = reinterpret_cast<const int8_t*>(p.x);
  int8_t* y = reinterpret_cast<int8_t*>(p.y);
  const int per_image = p.Ho * p.Wo * cv, row = p.Wo * cv;
  const int i = blockIdx.x * kThreads + threadIdx.x;
  if (i >= per_image) return;
  const int ho = fast_div(i, p.row_magic, p.row_shift);
  const int rem = i - ho * row;
  const int wo = fast_div(rem, p.cv_magic, p.cv_shift);
  const int c = (rem - wo * cv) * 16;
  for (int n = blockIdx.y; n < p.N; n += gridDim.y) {
    const int h0 = ho * p.sh - p.ph, w0 = wo * p.sw - p.pw;
    if constexpr (IS_MAX) {
      // Stored bytes are signed (level - 128) and keep their order as the high byte of a signed
      // 16-bit lane: the even bytes of a dword move there with one byte permute, the odd ones
      // with one mask, and one packed 16-bit maximum handles two of them.
      typedef short shortx2 __attribute__((ext_vector_type(2)));
      unsigned ev[4] = {0x80008000u, 0x80008000u, 0x80008000u, 0x80008000u};
      unsigned od[4] = {0x80008000u, 0x80008000u, 0x80008000u, 0x80008000u};
      auto take = [&](const uintx4 v) {
        const unsigned w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const shortx2 a0 = __builtin_bit_cast(shortx2, ev[k]);
          const shortx2 b0 = __builtin_bit_cast(shortx2, __builtin_amdgcn_perm(0u, w[k], 0x020c000cu));   // [b2, 0, b0, 0]
          const shortx2 a1 = __builtin_bit_cast(shortx2, od[k]), b1 = __builtin_bit_cast(shortx2, w[k] & 0xff00ff00u);
          ev[k] = __builtin_bit_cast(unsigned, __builtin_elementwise_max(a0, b0));
          od[k] = __builtin_bit_cast(unsigned, __builtin_elementwise_max(a1, b1));
        }
      };
      if constexpr (KH > 0) {
        uintx4 v[KH * KW];
#pragma unroll
        for (int r = 0; r < KH; ++r) {
          const int hi = h0 + r, hc = hi < 0 ? 0 : (hi < p.H ? hi : p.H - 1);
#pragma unroll
          for (int s = 0; s < KW; ++s) {
            const int wi = w0 + s, wc = wi < 0 ? 0 : (wi < p.W ? wi : p.W - 1);
            // (read by at most a few neighbouring windows, all of them close in time)
            v[r * KW + s] = *reinterpret_cast<const uintx4*>(x + (((int64_t)n * p.H + hc) * p.W + wc) * p.cs + c);
          }
        }
#pragma unroll
        for (int t = 0; t < KH * KW; ++t) take(v[t]);
      } else {
        for (int r = 0; r < p.kh; ++r) {
          const int hi = h0 + r;
          if ((unsigned)hi >= (unsigned)p.H) continue;
          for (int s = 0; s < p.kw; ++s) {
            const int wi = w0 + s;
            if ((unsigned)wi >= (unsigned)p.W) continue;
            take(*reinterpret_cast<const uintx4*>(x + (((int64_t)n * p.H + hi) * p.W + wi) * p.cs + c));
          }
        }
      }
      uintx4 o;
      o.x = (ev[0] >> 8) | od[0];   // (the low byte of every lane stayed 0)
      o.y = (ev[1] >> 8) | od[1];
      o.z = (ev[2] >> 8) | od[2];
      o.w = (ev[3] >> 8) | od[3];
      // (a window without a valid tap cannot occur: the planner derives Ho, Wo from the padding)
      *reinterpret_cast<uintx4*>(y + (((int64_t)n * p.Ho + ho) * p.Wo + wo) * p.ycs + c) = o;
    } else {
      int acc[16];
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[e] = 0;
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
          for (int e = 0; e < 16; ++e) acc[e] += q_from_stored(ev[e]);
          ++cnt;
        }
      }
      uintx4 o;
      int8_t* eo = reinterpret_cast<int8_t*>(&o);
      const int div = p.count_include_pad ? p.kh * p.kw : (cnt > 0 ? cnt : 1);
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const float f = (float)(acc[e] - cnt * p.zp_in) / (float)div;
        int q = (int)rintf(f * p.q_mul) + p.zp_out;
        q = q < 0 ? 0 : (q > 255 ? 255 : q);
        eo[e] = q_to_stored(q);
      }
      *reinterpret_cast<uintx4*>(y + (((int64_t)n * p.Ho + ho) * p.Wo + wo) * p.ycs + c) = o;
    }
  }
}

// --------------------------------------------------------------------------
// Reduction over the middle axis of [outer][len][inner].
// The accumulation rule is a compile-time choice (a run-time switch inside the
// inner loops costs more than the loads): 0 sum, 1 max, 2 min, 3 product,
// 4 sum of magnitudes, 5 sum of squares.
enum { ACC_SUM = 0, ACC_MAX, ACC_MIN, ACC_PROD, ACC_ABS, ACC_SQ };
template <int A> __device__ __forceinline__ float red_init() {
  return A == ACC_MAX ? -INFINITY : (A == ACC_MIN ? INFINITY : (A == ACC_PROD ? 1.f : 0.f));
}
template <int A> __device__ __forceinline__ float red_step(float acc, float v) {
  if (A == ACC_MAX) return fmaxf(acc, v);
  if (A == ACC_MIN) return fminf(acc, v);
  if (A == ACC_PROD) return acc * v;
  if (A == ACC_ABS) return acc + fabsf(v);
  if (A == ACC_SQ) return acc + v * v;
  return acc + v;
}
template <int A> __device__ __forceinline__ float red_merge(float a, float b) {
  if (A == ACC_MAX) return fmaxf(a, b);
  if (A == ACC_MIN) return fminf(a, b);
  if (A == ACC_PROD) return a * b;
  return a + b;
}
__device__ __forceinline__ float red_final(float acc, int64_t len, ReduceKind k, float eps) {
  switch (k) {
    case RED_MEAN: return acc / (float)len;
    case RED_L1: return acc + eps;
    case RED_L2: return sqrtf(acc + eps);
    case RED_LOGSUM: return logf(acc);
    default: return acc;
  }
}
// inner == 1: one wavefront per row, lanes stride the row.
template <typename TI, typename TO, int A>
__global__ void __launch_bounds__(kThreads)
reduce_rows_kernel(const TI* __restrict__ x, TO* __restrict__ y, int64_t rows, int64_t len,
                   ReduceKind kind, float eps) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = (blockIdx.x * (int64_t)blockDim.x + threadIdx.x) >> 6;
  const int64_t nwaves = ((int64_t)gridDim.x * blockDim.x) >> 6;
  for (int64_t r = wave; r < rows; r += nwaves) {
    const TI* row = x + r * len;
    float acc = red_init<A>();
    for (int64_t i = lane; i < len; i += 64) acc = red_step<A>(acc, Store<TI>::ld(row + i));
    acc = group_allreduce<64>(acc, [](float a, float b) { return red_merge<A>(a, b); });
    if (lane == 0) Store<TO>::st(y + r, red_final(acc, len, kind, eps));
  }
}
// inner > 1: one thread per (outer, inner) column; consecutive threads read
// consecutive inner positions, so each step over `len` is a coalesced row.
template <typename TI, typename TO, int A>
__global__ void __launch_bounds__(kThreads)
reduce_cols_kernel(const TI* __restrict__ x, TO* __restrict__ y, int64_t outer, int64_t len,
                   int64_t inner, ReduceKind kind, float eps) {
  const int64_t total = outer * inner;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t o = i / inner, in = i - o * inner;
    const TI* col = x + o * len * inner + in;
    float acc = red_init<A>();
    for (int64_t k = 0; k < len; ++k) acc = red_step<A>(acc, Store<TI>::ld(col + k * inner));
    Store<TO>::st(y + i, red_final(acc, len, kind, eps));
  }
}
// inner % V == 0: one thread per (outer, 16-byte group of inner positions); every
// step over `len` is a coalesced row of vectors.
template <typename TI, typename TO, int A>
__global__ void __launch_bounds__(kThreads)
reduce_cols_vec_kernel(const TI* __restrict__ x, TO* __restrict__ y, int64_t outer, int64_t len,
                       int64_t inner, ReduceKind kind, float eps) {
  constexpr int V = Vec16<TI>::N;
  const int64_t iv = inner / V;
  const int64_t total = outer * iv;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t o = i / iv, in = (i - o * iv) * V;
    const TI* col = x + o * len * inner + in;
    float acc[V];
#pragma unroll
    for (int e = 0; e < V; ++e) acc[e] = red_init<A>();
    int64_t k = 0;
    for (; k + 4 <= len; k += 4) {
      Vec16<TI> v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) v[u].load(col + (k + u) * inner);
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int e = 0; e < V; ++e) acc[e] = red_step<A>(acc[e], v[u].get(e));
    }
    for (; k < len; ++k) {
      Vec16<TI> v;
      v.load(col + k * inner);
#pragma unroll
      for (int e = 0; e < V; ++e) acc[e] = red_step<A>(acc[e], v.get(e));
    }
#pragma unroll
    for (int e = 0; e < V; ++e) Store<TO>::st(y + o * inner + in + e, red_final(acc[e], len, kind, eps));
  }
}
// Few columns and many rows (a global pool over a large image, a mean over a
// long sequence): one thread per column leaves most of the chip idle.  Here a
// workgroup owns `cl` 16-byte column groups of one outer index, its NT / cl
// thread rows stride the reduced axis, and the partial results meet in LDS.
template <typename TI, typename TO, int A, int NT>
__global__ void __launch_bounds__(NT)
reduce_cols_split_kernel(const TI* __restrict__ x, TO* __restrict__ y, int64_t len, int64_t inner,
                         int cl, ReduceKind kind, float eps) {
  constexpr int V = Vec16<TI>::N;
  __shared__ float part[NT * V];
  const int c = threadIdx.x % cl, s = threadIdx.x / cl, S = NT / cl;
  const int64_t iv = inner / V;
  const int64_t cv = blockIdx.x * (int64_t)cl + c;
  const int64_t o = blockIdx.y;
  float acc[V];
#pragma unroll
  for (int e = 0; e < V; ++e) acc[e] = red_init<A>();
  if (cv < iv) {
    const TI* col = x + o * len * inner + cv * V;
    int64_t k = s;
    for (; k + 3 * (int64_t)S < len; k += 4 * (int64_t)S) {
      Vec16<TI> v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) v[u].load(col + (k + u * (int64_t)S) * inner);
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int e = 0; e < V; ++e) acc[e] = red_step<A>(acc[e], v[u].get(e));
    }
    for (; k < len; k += S) {
      Vec16<TI> v;
      v.load(col + k * inner);
#pragma unroll
      for (int e = 0; e < V; ++e) acc[e] = red_step<A>(acc[e], v.get(e));
    }
  }
  const int width = cl * V;
#pragma unroll
  for (int e = 0; e < V; ++e) part[s * width + c * V + e] = acc[e];
  __syncthreads();
  for (int j = threadIdx.x; j < width; j += NT) {
    const int64_t col = blockIdx.x * (int64_t)width + j;
    if (col >= inner) break;
    float r = part[j];
    for (int t = 1; t < S; ++t) r = red_merge<A>(r, part[t * width + j]);
    Store<TO>::st(y + o * inner + col, red_final(r, len, kind, eps));
  }
}
// Few long rows (inner == 1): a workgroup per row, 16-byte loads.
template <typename TI, typename TO, int A>
__global__ void __launch_bounds__(kThreads)
reduce_row_block_kernel(const TI* __restrict__ x, TO* __restrict__ y, int64_t len, ReduceKind kind, float eps) {
  constexpr int V = Vec16<TI>::N;
  __shared__ float part[kThreads / 64];
  const TI* row = x + blockIdx.x * len;
  const int64_t nv = len / V;
  float acc = red_init<A>();
  int64_t i = threadIdx.x;
  for (; i + 3 * kThreads < nv; i += 4 * kThreads) {
    Vec16<TI> v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) v[u].load(row + (i + u * kThreads) * V);
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int e = 0; e < V; ++e) acc = red_step<A>(acc, v[u].get(e));
  }
  for (; i < nv; i += kThreads) {
    Vec16<TI> v;
    v.load(row + i * V);
#pragma unroll
    for (int e = 0; e < V; ++e) acc = red_step<A>(acc, v.get(e));
  }
  acc = group_allreduce<64>(acc, [](float a, float b) { return red_merge<A>(a, b); });
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    float r = part[0];
    for (int w = 1; w < kThreads / 64; ++w) r = red_merge<A>(r, part[w]);
    Store<TO>::st(y + blockIdx.x, red_final(r, len, kind, eps));
  }
}
// Index of the extreme value along the middle axis; one thread per (outer,
// inner) column.  Ties keep the first index, or the last when `last` is set.
template <typename TI, typename TO>
__global__ void __launch_bounds__(kThreads)
arg_extreme_kernel(const TI* __restrict__ x, TO* __restrict__ y, int64_t outer, int64_t len,
                   int64_t inner, bool is_max, bool last) {
  const int64_t total = outer * inner;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t o = i / inner, in = i - o * inner;
    const TI* col = x + o * len * inner + in;
    float val = Store<TI>::ld(col);
    int64_t idx = 0;
    for (int64_t k = 1; k < len; ++k) {
      const float cur = Store<TI>::ld(col + k * inner);
      if ((is_max && cur > val) || (!is_max && cur < val) || (cur == val && last)) { val = cur; idx = k; }
    }
    y[i] = (TO)idx;
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

// The same with 16 columns per thread and the rows of one outer index split
// over the workgroup (the global pool behind a quantised backbone: 49 rows).
__global__ void __launch_bounds__(kThreads)
reduce_cols_q8_split_kernel(const int8_t* __restrict__ x, float* __restrict__ y, int64_t len,
                            int64_t inner, int cl, float scale, int zp) {
  __shared__ int part[kThreads * 16];
  const int c = threadIdx.x % cl, s = threadIdx.x / cl, S = kThreads / cl;
  const int64_t iv = inner / 16;
  const int64_t cv = blockIdx.x * (int64_t)cl + c;
  const int64_t o = blockIdx.y;
  int acc[16];
#pragma unroll
  for (int e = 0; e < 16; ++e) acc[e] = 0;
  if (cv < iv) {
    const int8_t* col = x + o * len * inner + cv * 16;
    for (int64_t k = s; k < len; k += S) {
      const uintx4 v = *reinterpret_cast<const uintx4*>(col + k * inner);
      const int8_t* b = reinterpret_cast<const int8_t*>(&v);
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[e] += q_from_stored(b[e]);
    }
  }
  const int width = cl * 16;
#pragma unroll
  for (int e = 0; e < 16; ++e) part[s * width + c * 16 + e] = acc[e];
  __syncthreads();
  for (int j = threadIdx.x; j < width; j += kThreads) {
    const int64_t col = blockIdx.x * (int64_t)width + j;
    if (col >= inner) break;
    int r = part[j];
    for (int t = 1; t < S; ++t) r += part[t * width + j];
    y[o * inner + col] = ((float)(r - (int)len * zp) / (float)len) * scale;
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
// Rows of 16-byte vectors (len % V == 0, row start 16-byte aligned): LPR lanes
// share one row, each lane holds PER vectors; several short rows fit in one
// wavefront.  Reductions stay inside the LPR-lane group (group_allreduce).
template <int LPR>
__device__ __forceinline__ float group_max(float v) {
  return group_allreduce<LPR>(v, [](float a, float b) { return fmaxf(a, b); });
}
template <int LPR>
__device__ __forceinline__ float group_sum(float v) {
  return group_allreduce<LPR>(v, [](float a, float b) { return a + b; });
}

template <typename TO, int V>
__device__ __forceinline__ void store_row_vec(TO* dst, const float* v) {
  if constexpr (sizeof(TO) == 2 && V == 8) {
    Vec16<TO> o;
    const float (&v8)[8] = *reinterpret_cast<const float (*)[8]>(v);
    o.raw = pack8_rne<TO>(v8);
    o.store(dst);
  } else if constexpr (sizeof(TO) * V == 16) {
    Vec16<TO> o;
#pragma unroll
    for (int e = 0; e < V; ++e) o.set(e, v[e]);
    o.store(dst);
  } else if constexpr (sizeof(TO) == 4 && V % 4 == 0) {
#pragma unroll
    for (int e = 0; e < V; e += 4)
      *reinterpret_cast<floatx4*>(reinterpret_cast<float*>(dst) + e) = (floatx4){v[e], v[e + 1], v[e + 2], v[e + 3]};
  } else {
#pragma unroll
    for (int e = 0; e < V; ++e) Store<TO>::st(dst + e, v[e]);
  }
}

template <typename TI, typename TO, int LPR, int PER>
__global__ void __launch_bounds__(kThreads)
softmax_vec_kernel(const TI* __restrict__ x, TO* __restrict__ y, int64_t rows, int len, bool logsm,
                   const TI* __restrict__ add, int64_t add_div) {
  // add: optional term added to the input first (attention masks), one row of
  // `len` values shared by add_div consecutive rows of x
  constexpr int V = Vec16<TI>::N;
  constexpr int RPW = 64 / LPR;
  const int lane = threadIdx.x & 63;
  const int sub = lane % LPR;
  const int nv = len / V;
  const int64_t wave = (blockIdx.x * (int64_t)blockDim.x + threadIdx.x) >> 6;
  const int64_t nwaves = ((int64_t)gridDim.x * blockDim.x) >> 6;
  for (int64_t r0 = wave * RPW; r0 < rows; r0 += nwaves * RPW) {
    const int64_t r = r0 + lane / LPR;
    const bool row_ok = r < rows;
    const TI* row = x + (row_ok ? r : 0) * (int64_t)len;
    const TI* arow = add ? add + ((row_ok ? r : 0) / add_div) * (int64_t)len : nullptr;
    float v[PER][V];
    float mx = -INFINITY;
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int vi = sub + k * LPR;
      if (vi < nv && row_ok) {
        Vec16<TI> t;
        t.load(row + vi * V);
        if (arow != nullptr) {
          Vec16<TI> ta;
          ta.load(arow + vi * V);
#pragma unroll
          for (int e = 0; e < V; ++e) { v[k][e] = t.get(e) + ta.get(e); mx = fmaxf(mx, v[k][e]); }
        } else {
#pragma unroll
          for (int e = 0; e < V; ++e) { v[k][e] = t.get(e); mx = fmaxf(mx, v[k][e]); }
        }
      } else {
#pragma unroll
        for (int e = 0; e < V; ++e) v[k][e] = -INFINITY;
      }
    }
    mx = group_max<LPR>(mx);
    float sum = 0.f;
#pragma unroll
    for (int k = 0; k < PER; ++k)
#pragma unroll
      for (int e = 0; e < V; ++e) {
        // exp(-inf) = 0 for the padding slots.  A 16-bit result keeps 8 or 11 significant bits:
        // the hardware exponential (1 ulp) stands in for the library's.
        const float ex = sizeof(TO) == 2 ? __expf(v[k][e] - mx) : expf(v[k][e] - mx);
        sum += ex;
        if (!logsm) v[k][e] = ex;
      }
    sum = group_sum<LPR>(sum);
    const float lsum = logf(sum), inv = 1.0f / sum;
    if (row_ok) {
      TO* out = y + r * (int64_t)len;
#pragma unroll
      for (int k = 0; k < PER; ++k) {
        const int vi = sub + k * LPR;
        if (vi < nv) {
          float o[V];
#pragma unroll
          for (int e = 0; e < V; ++e) o[e] = logsm ? (v[k][e] - mx - lsum) : v[k][e] * inv;
          store_row_vec<TO, V>(out + vi * V, o);
        }
      }
    }
  }
}

template <typename T, int LPR, int PER>
__global__ void __launch_bounds__(kThreads)
layernorm_vec_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t rows, int len,
                     const float* __restrict__ gamma, const float* __restrict__ beta, float eps,
                     void* __restrict__ y2 = nullptr, const int y2_kind = 0) {
  constexpr int V = Vec16<T>::N;
  constexpr int RPW = 64 / LPR;
  const int lane = threadIdx.x & 63;
  const int sub = lane % LPR;
  const int nv = len / V;
  const int64_t wave = (blockIdx.x * (int64_t)blockDim.x + threadIdx.x) >> 6;
  const int64_t nwaves = ((int64_t)gridDim.x * blockDim.x) >> 6;
  for (int64_t r0 = wave * RPW; r0 < rows; r0 += nwaves * RPW) {
    const int64_t r = r0 + lane / LPR;
    const bool row_ok = r < rows;
    const T* row = x + (row_ok ? r : 0) * (int64_t)len;
    float v[PER][V];
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int vi = sub + k * LPR;
      if (vi < nv && row_ok) {
        Vec16<T> t;
        t.load(row + vi * V);
#pragma unroll
        for (int e = 0; e < V; ++e) { v[k][e] = t.get(e); s += v[k][e]; }
      } else {
#pragma unroll
        for (int e = 0; e < V; ++e) v[k][e] = 0.f;
      }
    }
    const float mean = group_sum<LPR>(s) / (float)len;
    float q = 0.f;
#pragma unroll
    for (int k = 0; k < PER; ++k) {
      const int vi = sub + k * LPR;
      if (vi < nv) {
#pragma unroll
        for (int e = 0; e < V; ++e) { const float d = v[k][e] - mean; q += d * d; }
      }
    }
    const float var = group_sum<LPR>(q) / (float)len;
    const float rstd = 1.0f / sqrtf(var + eps);
    if (row_ok) {
      T* out = y + r * (int64_t)len;
#pragma unroll
      for (int k = 0; k < PER; ++k) {
        const int vi = sub + k * LPR;
        if (vi < nv) {
          float o[V], g[V], b[V];
          // gamma / beta are fp32 vectors, 16-byte aligned (V is a multiple of 4)
#pragma unroll
          for (int e = 0; e < V; e += 4) {
            const floatx4 gv = gamma ? *reinterpret_cast<const floatx4*>(gamma + vi * V + e) : (floatx4){1.f, 1.f, 1.f, 1.f};
            const floatx4 bv = beta ? *reinterpret_cast<const floatx4*>(beta + vi * V + e) : (floatx4){0.f, 0.f, 0.f, 0.f};
            g[e] = gv.x; g[e + 1] = gv.y; g[e + 2] = gv.z; g[e + 3] = gv.w;
            b[e] = bv.x; b[e + 1] = bv.y; b[e + 2] = bv.z; b[e + 3] = bv.w;
          }
#pragma unroll
          for (int e = 0; e < V; ++e) o[e] = (v[k][e] - mean) * rstd * g[e] + b[e];
          store_row_vec<T, V>(out + vi * V, o);
          // a second copy of the row in a 2-byte type (y2_kind 1: f16, 2: bf16; fp32 rows only):
          // the matrix products that read this result take it as their operand, no conversion
          // launch in between
          if constexpr (V == 4) {
            if (y2 != nullptr) {
              const float o8[8] = {o[0], o[1], o[2], o[3], 0.f, 0.f, 0.f, 0.f};
              const uintx4 h = y2_kind == 1 ? pack8_rne<f16_t>(o8) : pack8_rne<bf16_t>(o8);
              typedef unsigned uintx2 __attribute__((ext_vector_type(2)));
              *reinterpret_cast<uintx2*>(reinterpret_cast<unsigned short*>(y2) + r * (int64_t)len + vi * V) = (uintx2){h.x, h.y};
            }
          }
        }
      }
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

// Rows longer than a workgroup can hold in registers: the same three steps, each
// a strided walk over the row in memory (the second and third walk hit in cache).
template <typename T, int NT>
__global__ void __launch_bounds__(NT)
layernorm_long_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t rows, int64_t len,
                      const float* __restrict__ gamma, const float* __restrict__ beta, float eps) {
  __shared__ float red[NT / 64];
  for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
    const T* row = x + r * len;
    float s = 0.f;
    for (int64_t i = threadIdx.x; i < len; i += NT) s += Store<T>::ld(row + i);
    const float mean = block_sum<NT>(s, red) / (float)len;
    float q = 0.f;
    for (int64_t i = threadIdx.x; i < len; i += NT) {
      const float d = Store<T>::ld(row + i) - mean;
      q += d * d;
    }
    const float var = block_sum<NT>(q, red) / (float)len;
    const float rstd = 1.0f / sqrtf(var + eps);
    T* out = y + r * len;
    for (int64_t i = threadIdx.x; i < len; i += NT) {
      const float g = gamma ? gamma[i] : 1.f, b = beta ? beta[i] : 0.f;
      Store<T>::st(out + i, (Store<T>::ld(row + i) - mean) * rstd * g + b);
    }
    __syncthreads();
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

hipError_t launch_pool2d(const PoolParams& p_in, hipStream_t stream) {
  PoolParams p = p_in;
  if (!p.x || !p.y || p.N <= 0 || p.H <= 0 || p.W <= 0 || p.C <= 0 || p.Ho <= 0 || p.Wo <= 0)
    return hipErrorInvalidValue;
  if (p.cs < p.C || p.ycs < p.C || p.kh <= 0 || p.kw <= 0 || p.sh <= 0 || p.sw <= 0)
    return hipErrorInvalidValue;
  const int es = dtype_size(p.dt);
  if (es == 0) return hipErrorInvalidValue;
  const int V = 16 / es;
  const bool vec = (p.C % V == 0) && (p.cs % V == 0) && (p.ycs % V == 0) && al16(p.x) && al16(p.y);
  if (p.dt == DT_I8 && !vec) return hipErrorInvalidValue;
  if (vec) {
    // one image per blockIdx.y (folded beyond the grid limit), positions of an image along x
    const int cv = p.C / V;
    const int64_t per_image = (int64_t)p.Ho * p.Wo * cv;
    if (per_image >= (1ll << 31)) return hipErrorInvalidValue;
    div_magic(p.Wo * cv, &p.row_magic, &p.row_shift);
    div_magic(cv, &p.cv_magic, &p.cv_shift);
    const dim3 grid((unsigned)((per_image + kThreads - 1) / kThreads), (unsigned)(p.N < 65535 ? p.N : 65535));
    if (p.dt == DT_I8) {
      // (the clamped taps of the unrolled windows need every window to overlap the image)
      const bool overlap = p.ph < p.kh && p.pw < p.kw && (int64_t)(p.Ho - 1) * p.sh - p.ph < p.H &&
                           (int64_t)(p.Wo - 1) * p.sw - p.pw < p.W;
      if (p.is_max && p.kh == 3 && p.kw == 3 && overlap) hipLaunchKernelGGL((pool2d_q8_kernel<true, 3, 3>), grid, dim3(kThreads), 0, stream, p);
      else if (p.is_max && p.kh == 2 && p.kw == 2 && overlap) hipLaunchKernelGGL((pool2d_q8_kernel<true, 2, 2>), grid, dim3(kThreads), 0, stream, p);
      else if (p.is_max) hipLaunchKernelGGL(pool2d_q8_kernel<true>, grid, dim3(kThreads), 0, stream, p);
      else hipLaunchKernelGGL(pool2d_q8_kernel<false>, grid, dim3(kThreads), 0, stream, p);
      return hipGetLastError();
    }
#define POOL_LAUNCH(MAX_, KH_, KW_) \
  FLOAT_DISPATCH(p.dt, hipLaunchKernelGGL((pool2d_vec_kernel<T, MAX_, KH_, KW_>), grid, dim3(kThreads), 0, stream, p))
    if (p.kh == 3 && p.kw == 3) { if (p.is_max) { POOL_LAUNCH(true, 3, 3); } else { POOL_LAUNCH(false, 3, 3); } }
    else if (p.kh == 2 && p.kw == 2) { if (p.is_max) { POOL_LAUNCH(true, 2, 2); } else { POOL_LAUNCH(false, 2, 2); } }
    else if (p.kh == 1 && p.kw == 1) { if (p.is_max) { POOL_LAUNCH(true, 1, 1); } else { POOL_LAUNCH(false, 1, 1); } }
    else { if (p.is_max) { POOL_LAUNCH(true, 0, 0); } else { POOL_LAUNCH(false, 0, 0); } }
#undef POOL_LAUNCH
  } else {
    const int64_t total = (int64_t)p.N * p.Ho * p.Wo * p.C;
    const int grid = grid_for(total, kThreads);
    if (p.is_max) { FLOAT_DISPATCH(p.dt, hipLaunchKernelGGL((pool2d_scalar_kernel<T, true>), dim3(grid), dim3(kThreads), 0, stream, p)); }
    else { FLOAT_DISPATCH(p.dt, hipLaunchKernelGGL((pool2d_scalar_kernel<T, false>), dim3(grid), dim3(kThreads), 0, stream, p)); }
  }
  return hipGetLastError();
}

// Below this many column threads (half the chip's resident threads at 512 per
// CU) the reductions split the reduced axis over the workgroup as well.
static constexpr int64_t kSplitBelow = 256 * 512;
static int split_columns(int64_t groups) {
  int cl = 64;
  while (cl > 1 && cl > groups) cl >>= 1;
  return cl;
}

hipError_t launch_reduce_q8_mean(const void* x, float* y, int64_t outer, int64_t len, int64_t inner,
                                 float scale, int zp, hipStream_t stream) {
  if (!x || !y || outer <= 0 || len <= 0 || inner <= 0 || len > (1 << 23)) return hipErrorInvalidValue;
  if (inner % 16 == 0 && al16(x) && outer * (inner / 16) < kSplitBelow && len >= 8 && outer <= 65535) {
    const int cl = split_columns(inner / 16);
    hipLaunchKernelGGL(reduce_cols_q8_split_kernel, dim3((unsigned)((inner / 16 + cl - 1) / cl), (unsigned)outer),
                       dim3(kThreads), 0, stream, (const int8_t*)x, y, len, inner, cl, scale, zp);
    return hipGetLastError();
  }
  hipLaunchKernelGGL(reduce_cols_q8_kernel, dim3(grid_for(outer * inner, kThreads)), dim3(kThreads), 0,
                     stream, (const int8_t*)x, y, outer, len, inner, scale, zp);
  return hipGetLastError();
}

template <typename TI>
static hipError_t reduce_out(const void* x, void* y, DType out_dt, int64_t outer, int64_t len,
                             int64_t inner, ReduceKind kind, float eps, hipStream_t stream) {
  auto go = [&](auto tag, auto rule) -> hipError_t {
    using TO = decltype(tag);
    constexpr int A = decltype(rule)::value;
    constexpr int V = 16 / (int)sizeof(TI);
    if (inner == 1 && outer <= 2048 && len >= 16384 && len % V == 0 && al16(x)) {
      hipLaunchKernelGGL((reduce_row_block_kernel<TI, TO, A>), dim3((unsigned)outer), dim3(kThreads), 0, stream,
                         (const TI*)x, (TO*)y, len, kind, eps);
    } else if (inner > 1 && inner % V == 0 && al16(x) && outer * (inner / V) < kSplitBelow && len >= 32 &&
               outer <= 65535) {
      const int cl = split_columns(inner / V);
      const dim3 grid((unsigned)((inner / V + cl - 1) / cl), (unsigned)outer);
      if (len >= 1024)
        hipLaunchKernelGGL((reduce_cols_split_kernel<TI, TO, A, 1024>), grid, dim3(1024), 0, stream,
                           (const TI*)x, (TO*)y, len, inner, cl, kind, eps);
      else
        hipLaunchKernelGGL((reduce_cols_split_kernel<TI, TO, A, kThreads>), grid, dim3(kThreads), 0, stream,
                           (const TI*)x, (TO*)y, len, inner, cl, kind, eps);
    } else if (inner == 1) {
      const int grid = grid_for(outer * 64, kThreads);
      hipLaunchKernelGGL((reduce_rows_kernel<TI, TO, A>), dim3(grid), dim3(kThreads), 0, stream,
                         (const TI*)x, (TO*)y, outer, len, kind, eps);
    } else if (inner % (16 / (int)sizeof(TI)) == 0 && al16(x)) {
      const int grid = grid_for(outer * (inner / (16 / (int)sizeof(TI))), kThreads);
      hipLaunchKernelGGL((reduce_cols_vec_kernel<TI, TO, A>), dim3(grid), dim3(kThreads), 0, stream,
                         (const TI*)x, (TO*)y, outer, len, inner, kind, eps);
    } else {
      const int grid = grid_for(outer * inner, kThreads);
      hipLaunchKernelGGL((reduce_cols_kernel<TI, TO, A>), dim3(grid), dim3(kThreads), 0, stream,
                         (const TI*)x, (TO*)y, outer, len, inner, kind, eps);
    }
    return hipGetLastError();
  };
  auto with_rule = [&](auto tag) -> hipError_t {
    switch (kind) {
      case RED_MAX: return go(tag, std::integral_constant<int, ACC_MAX>{});
      case RED_MIN: return go(tag, std::integral_constant<int, ACC_MIN>{});
      case RED_PROD: return go(tag, std::integral_constant<int, ACC_PROD>{});
      case RED_L1: return go(tag, std::integral_constant<int, ACC_ABS>{});
      case RED_L2: case RED_SUMSQ: return go(tag, std::integral_constant<int, ACC_SQ>{});
      default: return go(tag, std::integral_constant<int, ACC_SUM>{});
    }
  };
  if (out_dt == DT_F32) return with_rule(float{});
  if (out_dt == DT_F16) return with_rule(f16_t{});
  if (out_dt == DT_BF16) return with_rule(bf16_t{});
  return hipErrorInvalidValue;
}

hipError_t launch_reduce(const void* x, void* y, DType in_dt, DType out_dt, int64_t outer,
                         int64_t len, int64_t inner, ReduceKind kind, hipStream_t stream, float eps) {
  if (!x || !y || outer <= 0 || len <= 0 || inner <= 0) return hipErrorInvalidValue;
  switch (in_dt) {
    case DT_F32: return reduce_out<float>(x, y, out_dt, outer, len, inner, kind, eps, stream);
    case DT_F16: return reduce_out<f16_t>(x, y, out_dt, outer, len, inner, kind, eps, stream);
    case DT_BF16: return reduce_out<bf16_t>(x, y, out_dt, outer, len, inner, kind, eps, stream);
    default: return hipErrorInvalidValue;
  }
}

hipError_t launch_arg_extreme(const void* x, void* y, DType in_dt, DType out_dt, int64_t outer,
                              int64_t len, int64_t inner, bool is_max, bool last, hipStream_t stream) {
  if (!x || !y || outer <= 0 || len <= 0 || inner <= 0) return hipErrorInvalidValue;
  if (out_dt != DT_I32 && out_dt != DT_I64) return hipErrorInvalidValue;
  const int grid = grid_for(outer * inner, kThreads);
  if (out_dt == DT_I32) {
    FLOAT_DISPATCH(in_dt, hipLaunchKernelGGL((arg_extreme_kernel<T, int32_t>), dim3(grid), dim3(kThreads), 0, stream,
                                             (const T*)x, (int32_t*)y, outer, len, inner, is_max, last));
  } else {
    FLOAT_DISPATCH(in_dt, hipLaunchKernelGGL((arg_extreme_kernel<T, int64_t>), dim3(grid), dim3(kThreads), 0, stream,
                                             (const T*)x, (int64_t*)y, outer, len, inner, is_max, last));
  }
  return hipGetLastError();
}

template <typename TI, typename TO>
static hipError_t softmax_typed(const void* x, void* y, int64_t outer, int64_t len, int64_t inner,
                                bool logsm, hipStream_t stream, const void* add = nullptr, int64_t add_div = 1) {
  constexpr int V = 16 / (int)sizeof(TI);
  const bool vec_ok = inner == 1 && len % V == 0 && len / V <= 256 && al16(x) && (sizeof(TO) != sizeof(TI) || al16(y));
  if (add != nullptr && (!vec_ok || !al16(add) || add_div <= 0)) return hipErrorInvalidValue;
  if (vec_ok) {
    const int nv = (int)(len / V);
    int lpr = 1;
    while (lpr < nv && lpr < 64) lpr <<= 1;
    const int per = (nv + lpr - 1) / lpr;
    const int rpw = 64 / lpr;
    const int grid = grid_for((outer + rpw - 1) / rpw * 64, kThreads);
#define SMV(LPR_, PER_) hipLaunchKernelGGL((softmax_vec_kernel<TI, TO, LPR_, PER_>), dim3(grid), dim3(kThreads), 0, stream, (const TI*)x, (TO*)y, outer, (int)len, logsm, (const TI*)add, add_div)
    if (lpr <= 8) SMV(8, 1);
    else if (lpr == 16) SMV(16, 1);
    else if (lpr == 32) SMV(32, 1);
    else if (per == 1) SMV(64, 1);
    else if (per == 2) SMV(64, 2);
    else SMV(64, 4);
#undef SMV
    return hipGetLastError();
  }
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
                          int64_t len, int64_t inner, bool log_softmax, hipStream_t stream,
                          const void* add, int64_t add_div) {
  if (!x || !y || outer <= 0 || len <= 0 || inner <= 0 || len >= (1ll << 31)) return hipErrorInvalidValue;
#define SM_CASE(I_, O_, TI_, TO_) \
  if (in_dt == I_ && out_dt == O_)  \
    return softmax_typed<TI_, TO_>(x, y, outer, len, inner, log_softmax, stream, add, add_div);
  SM_CASE(DT_F32, DT_F32, float, float)
  SM_CASE(DT_F16, DT_F16, f16_t, f16_t)
  SM_CASE(DT_BF16, DT_BF16, bf16_t, bf16_t)
  SM_CASE(DT_F16, DT_F32, f16_t, float)
  SM_CASE(DT_BF16, DT_F32, bf16_t, float)
  // fp32 scores, probabilities in the operand type of the matrix product that reads them
  SM_CASE(DT_F32, DT_BF16, float, bf16_t)
  SM_CASE(DT_F32, DT_F16, float, f16_t)
#undef SM_CASE
  return hipErrorInvalidValue;
}

bool layernorm_dual_ok(DType dt, int64_t len) { return dt == DT_F32 && len % 4 == 0 && len / 4 <= 256; }

hipError_t launch_layernorm(const void* x, void* y, DType dt, int64_t rows, int64_t len,
                            const float* gamma, const float* beta, float eps, hipStream_t stream,
                            void* y2, DType y2_dt) {
  if (!x || !y || rows <= 0 || len <= 0) return hipErrorInvalidValue;
  const int y2_kind = y2 == nullptr ? 0 : (y2_dt == DT_F16 ? 1 : (y2_dt == DT_BF16 ? 2 : -1));
  // (the second, 2-byte copy: fp32 rows on the vector path only - layernorm_dual_ok)
  if (y2_kind < 0 || (y2_kind > 0 && !(layernorm_dual_ok(dt, len) && al16(x) && al16(y) && (reinterpret_cast<uintptr_t>(y2) & 7u) == 0 &&
                                      (!gamma || al16(gamma)) && (!beta || al16(beta)))))
    return hipErrorInvalidValue;
  if (len > 256 * 16) {
    const int grid = (int)(rows < 16384 ? rows : 16384);
    FLOAT_DISPATCH(dt, hipLaunchKernelGGL((layernorm_long_kernel<T, 256>), dim3(grid), dim3(256), 0, stream,
                                          (const T*)x, (T*)y, rows, len, gamma, beta, eps));
    return hipGetLastError();
  }
  {
    const int es = dtype_size(dt);
    const int V = es ? 16 / es : 1;
    if (es && len % V == 0 && len / V <= 256 && al16(x) && al16(y) && (!gamma || al16(gamma)) && (!beta || al16(beta))) {
      const int nv = (int)(len / V);
      int lpr = 1;
      while (lpr < nv && lpr < 64) lpr <<= 1;
      const int per = (nv + lpr - 1) / lpr;
      const int rpw = 64 / lpr;
      const int grid = grid_for((rows + rpw - 1) / rpw * 64, kThreads);
#define LNV(LPR_, PER_) FLOAT_DISPATCH(dt, hipLaunchKernelGGL((layernorm_vec_kernel<T, LPR_, PER_>), dim3(grid), dim3(kThreads), 0, stream, (const T*)x, (T*)y, rows, (int)len, gamma, beta, eps, y2, y2_kind))
      if (lpr <= 16) { LNV(16, 1); }
      else if (lpr == 32) { LNV(32, 1); }
      else if (per == 1) { LNV(64, 1); }
      else if (per == 2) { LNV(64, 2); }
      else { LNV(64, 4); }
#undef LNV
      return hipGetLastError();
    }
  }
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
