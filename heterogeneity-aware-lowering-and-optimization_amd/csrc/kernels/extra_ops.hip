// Kernels for the wider operator surface: constant fill, TopK, cross-channel
// LRN and per-row normalisation with per-channel parameters (instance norm).
// All work on row-major tensors; float types compute in fp32.
#include <math.h>

#include "device_utils.h"

namespace ohip {

namespace {
constexpr int kThreads = 256;

__global__ void __launch_bounds__(kThreads) fill_u32_kernel(uint32_t* __restrict__ p, int64_t n, uint32_t v) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
    p[i] = v;
}

// --------------------------------------------------------------------------
// TopK along the middle axis of [outer][len][inner]: one wavefront per (outer,
// inner) column.  Results come out in order (best first); equal values are
// ordered by ascending index.  Round j selects the best element that comes
// strictly after the winner of round j-1 in that order, so no element is
// marked and the column is only read.
template <typename T, typename TI>
__global__ void __launch_bounds__(kThreads)
topk_kernel(const T* __restrict__ x, T* __restrict__ vals, TI* __restrict__ idxs, int64_t outer,
            int64_t len, int64_t inner, int K, bool largest) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = (blockIdx.x * (int64_t)blockDim.x + threadIdx.x) >> 6;
  const int64_t nwaves = ((int64_t)gridDim.x * blockDim.x) >> 6;
  const int64_t cols = outer * inner;
  for (int64_t c = wave; c < cols; c += nwaves) {
    const int64_t o = c / inner, in = c - o * inner;
    const T* col = x + o * len * inner + in;
    // keys are negated for "smallest" so that both modes pick maxima
    float prev_v = INFINITY;
    int64_t prev_i = -1;
    for (int j = 0; j < K; ++j) {
      float best_v = -INFINITY;
      int64_t best_i = -1;
      for (int64_t i = lane; i < len; i += 64) {
        float v = Store<T>::ld(col + i * inner);
        if (!largest) v = -v;
        const bool after = v < prev_v || (v == prev_v && i > prev_i);
        if (after && (best_i < 0 || v > best_v)) { best_v = v; best_i = i; }
      }
#pragma unroll
      for (int s = 32; s > 0; s >>= 1) {
        const float ov = __shfl_xor(best_v, s, 64);
        const int64_t oi = (int64_t)__shfl_xor((long long)best_i, s, 64);
        const bool take = oi >= 0 && (best_i < 0 || ov > best_v || (ov == best_v && oi < best_i));
        if (take) { best_v = ov; best_i = oi; }
      }
      if (lane == 0) {
        const int64_t dst = (o * K + j) * inner + in;
        Store<T>::st(vals + dst, best_i >= 0 ? (largest ? best_v : -best_v) : 0.f);
        idxs[dst] = (TI)(best_i >= 0 ? best_i : 0);
      }
      prev_v = best_v;
      prev_i = best_i;
    }
  }
}

// --------------------------------------------------------------------------
// LRN across channels of x[N][C][inner]:
// y = x / (bias + alpha / size * sum_{|c' - c| <= half} x[c']^2) ^ beta, size = 2 half + 1
template <typename T>
__global__ void __launch_bounds__(kThreads)
lrn_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t N, int C, int64_t inner, int half,
           float alpha, float beta, float bias) {
  const int64_t total = N * C * inner;
  const float k = alpha / (float)(2 * half + 1);
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t in = i % inner;
    const int64_t nc = i / inner;
    const int c = (int)(nc % C);
    const int64_t n = nc / C;
    const int lo = c - half < 0 ? 0 : c - half, hi = c + half >= C ? C - 1 : c + half;
    float s = 0.f;
    for (int cc = lo; cc <= hi; ++cc) {
      const float v = Store<T>::ld(x + (n * C + cc) * inner + in);
      s += v * v;
    }
    Store<T>::st(y + i, Store<T>::ld(x + i) / powf(bias + k * s, beta));
  }
}

// --------------------------------------------------------------------------
// Per-row normalisation, rows of any length: y = (x - mean) / sqrt(var + eps)
// * gamma[r % channels] + beta[r % channels]; biased variance computed from
// the deviations (second pass), one workgroup per row.
template <typename T>
__global__ void __launch_bounds__(kThreads)
rownorm_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t rows, int64_t len, int channels,
               const float* __restrict__ gamma, const float* __restrict__ beta, float sgamma, float sbeta,
               float eps) {
  __shared__ float red[kThreads / 64];
  for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
    const T* row = x + r * len;
    float s = 0.f;
    for (int64_t i = threadIdx.x; i < len; i += kThreads) s += Store<T>::ld(row + i);
    const float mean = block_sum<kThreads>(s, red) / (float)len;
    float q = 0.f;
    for (int64_t i = threadIdx.x; i < len; i += kThreads) {
      const float d = Store<T>::ld(row + i) - mean;
      q += d * d;
    }
    const float var = block_sum<kThreads>(q, red) / (float)len;
    const float sd = sqrtf(var + eps);
    const int c = (int)(r % channels);
    const float g = gamma ? gamma[c] : sgamma, b = beta ? beta[c] : sbeta;
    T* out = y + r * len;
    for (int64_t i = threadIdx.x; i < len; i += kThreads)
      Store<T>::st(out + i, (Store<T>::ld(row + i) - mean) / sd * g + b);
    __syncthreads();
  }
}

// --------------------------------------------------------------------------
// Range statistics for calibration: x fp32 [outer][C][inner] -> partial minima
// and maxima part[c][s] = {min, max} over the s-th interleaved share of
// channel c.  grid = (splits, C); the few partials are combined on the host.
__global__ void __launch_bounds__(kThreads)
minmax_partial_kernel(const float* __restrict__ x, float* __restrict__ part, int64_t outer, int C, int64_t inner) {
  __shared__ float red[kThreads / 64];
  const int c = blockIdx.y, s = blockIdx.x, S = gridDim.x;
  const int64_t per = outer * inner;
  float lo = INFINITY, hi = -INFINITY;
  for (int64_t e = (int64_t)s * kThreads + threadIdx.x; e < per; e += (int64_t)S * kThreads) {
    const int64_t o = e / inner, i = e - o * inner;
    const float v = x[(o * C + c) * inner + i];
    lo = fminf(lo, v);
    hi = fmaxf(hi, v);
  }
  hi = block_max<kThreads>(hi, red);
  lo = -block_max<kThreads>(-lo, red);
  if (threadIdx.x == 0) {
    part[((int64_t)c * S + s) * 2 + 0] = lo;
    part[((int64_t)c * S + s) * 2 + 1] = hi;
  }
}

#define FLOAT_DISPATCH(dt, EXPR)                         \
  switch (dt) {                                          \
    case DT_F32: { using T = float; EXPR; break; }       \
    case DT_F16: { using T = f16_t; EXPR; break; }       \
    case DT_BF16: { using T = bf16_t; EXPR; break; }     \
    default: return hipErrorInvalidValue;                \
  }

}  // namespace

hipError_t launch_fill_bytes(void* p, size_t bytes, uint32_t pattern, hipStream_t stream) {
  if (!p || (bytes & 3) || (reinterpret_cast<uintptr_t>(p) & 3)) return hipErrorInvalidValue;
  const int64_t n = (int64_t)(bytes / 4);
  if (n == 0) return hipSuccess;
  hipLaunchKernelGGL(fill_u32_kernel, dim3(grid_for(n, kThreads * 4)), dim3(kThreads), 0, stream, (uint32_t*)p, n, pattern);
  return hipGetLastError();
}

hipError_t launch_minmax_partial(const float* x, float* part, int64_t outer, int C, int64_t inner, int splits,
                                 hipStream_t stream) {
  if (!x || !part || outer <= 0 || C <= 0 || C > 65535 || inner <= 0 || splits <= 0) return hipErrorInvalidValue;
  hipLaunchKernelGGL(minmax_partial_kernel, dim3(splits, C), dim3(kThreads), 0, stream, x, part, outer, C, inner);
  return hipGetLastError();
}

hipError_t launch_topk(const void* x, void* vals, void* idxs, DType dt, DType idx_dt, int64_t outer,
                       int64_t len, int64_t inner, int K, bool largest, hipStream_t stream) {
  if (!x || !vals || !idxs || outer <= 0 || len <= 0 || inner <= 0 || K <= 0 || K > len) return hipErrorInvalidValue;
  if (idx_dt != DT_I32 && idx_dt != DT_I64) return hipErrorInvalidValue;
  const int grid = grid_for(outer * inner * 64, kThreads);
  if (idx_dt == DT_I32) {
    FLOAT_DISPATCH(dt, hipLaunchKernelGGL((topk_kernel<T, int32_t>), dim3(grid), dim3(kThreads), 0, stream, (const T*)x,
                                          (T*)vals, (int32_t*)idxs, outer, len, inner, K, largest));
  } else {
    FLOAT_DISPATCH(dt, hipLaunchKernelGGL((topk_kernel<T, int64_t>), dim3(grid), dim3(kThreads), 0, stream, (const T*)x,
                                          (T*)vals, (int64_t*)idxs, outer, len, inner, K, largest));
  }
  return hipGetLastError();
}

hipError_t launch_lrn(const void* x, void* y, DType dt, int64_t N, int C, int64_t inner, int half, float alpha,
                      float beta, float bias, hipStream_t stream) {
  if (!x || !y || N <= 0 || C <= 0 || inner <= 0 || half < 0) return hipErrorInvalidValue;
  const int grid = grid_for(N * C * inner, kThreads * 2);
  FLOAT_DISPATCH(dt, hipLaunchKernelGGL(lrn_kernel<T>, dim3(grid), dim3(kThreads), 0, stream, (const T*)x, (T*)y, N, C,
                                        inner, half, alpha, beta, bias));
  return hipGetLastError();
}

hipError_t launch_rownorm(const void* x, void* y, DType dt, int64_t rows, int64_t len, int channels,
                          const float* gamma, const float* beta, float sgamma, float sbeta, float eps,
                          hipStream_t stream) {
  if (!x || !y || rows <= 0 || len <= 0 || channels <= 0) return hipErrorInvalidValue;
  const int grid = (int)(rows < 16384 ? rows : 16384);
  FLOAT_DISPATCH(dt, hipLaunchKernelGGL(rownorm_kernel<T>, dim3(grid), dim3(kThreads), 0, stream, (const T*)x, (T*)y,
                                        rows, len, channels, gamma, beta, sgamma, sbeta, eps));
  return hipGetLastError();
}

}  // namespace ohip
