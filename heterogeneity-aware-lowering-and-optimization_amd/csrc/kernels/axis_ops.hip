// Operators that walk one axis of a row-major tensor seen as [outer][len][inner]:
// GatherElements, CumSum, Hardmax (the one-hot half; the index comes from the
// arg-extreme kernel) and Compress.  Element moves are done on raw words of the
// element size; CumSum accumulates in fp32.
#include "device_utils.h"

namespace ohip {

namespace {
constexpr int kThreads = 256;

template <int ES> struct Word;
template <> struct Word<1> { using type = uint8_t; };
template <> struct Word<2> { using type = uint16_t; };
template <> struct Word<4> { using type = uint32_t; };
template <> struct Word<8> { using type = uint64_t; };

// y[i][j][k] = x[i][idx[i][j][k]][k]; idx is [ii][ij][ik], x is [..][dj][dk].  A negative
// index counts from the end of the axis; an index outside the axis is clamped into it.
template <int ES, typename TI>
__global__ void __launch_bounds__(kThreads)
gather_elements_kernel(const typename Word<ES>::type* __restrict__ x, const TI* __restrict__ idx,
                       typename Word<ES>::type* __restrict__ y, int64_t n, int64_t ij, int64_t ik, int64_t dj, int64_t dk) {
  for (int64_t e = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; e < n; e += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = e / ik, k = e - t * ik;
    const int64_t i = t / ij;
    int64_t v = (int64_t)idx[e];
    if (v < 0) v += dj;
    v = v < 0 ? 0 : (v >= dj ? dj - 1 : v);
    y[e] = x[(i * dj + v) * dk + k];
  }
}

// One thread per (outer, inner) line, elements added in order (the order of a scalar loop).
template <typename T>
__global__ void __launch_bounds__(kThreads)
cumsum_lines_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t outer, int64_t len, int64_t inner,
                    bool exclusive, bool reverse) {
  const int64_t lines = outer * inner;
  for (int64_t l = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; l < lines; l += (int64_t)gridDim.x * blockDim.x) {
    const int64_t o = l / inner, in = l - o * inner;
    const int64_t base = o * len * inner + in;
    float acc = 0.f;
    for (int64_t q = 0; q < len; ++q) {
      const int64_t off = base + (reverse ? len - 1 - q : q) * inner;
      const float v = Store<T>::ld(x + off);
      Store<T>::st(y + off, exclusive ? acc : acc + v);
      acc += v;
    }
  }
}

// One wavefront per line of a contiguous axis (inner == 1): 64 consecutive elements per
// step, a shuffle scan across the lanes plus the running total of the steps before.
template <typename T>
__global__ void __launch_bounds__(kThreads)
cumsum_wave_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t lines, int64_t len, bool exclusive, bool reverse) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = (blockIdx.x * (int64_t)blockDim.x + threadIdx.x) >> 6;
  const int64_t nwaves = ((int64_t)gridDim.x * blockDim.x) >> 6;
  for (int64_t l = wave; l < lines; l += nwaves) {
    const int64_t base = l * len;
    float carry = 0.f;
    for (int64_t q0 = 0; q0 < len; q0 += 64) {
      const int64_t q = q0 + lane;
      const bool ok = q < len;
      const int64_t off = base + (reverse ? len - 1 - q : q);
      const float v = ok ? Store<T>::ld(x + off) : 0.f;
      float s = v;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const float t = __shfl_up(s, d, 64);
        if (lane >= d) s += t;
      }
      if (ok) Store<T>::st(y + off, carry + (exclusive ? s - v : s));
      carry += __shfl(s, 63, 64);
    }
  }
}

// y[o][i][in] = (i == amax[o][in]) ? 1 : 0
template <typename T, typename TI>
__global__ void __launch_bounds__(kThreads)
onehot_axis_kernel(const TI* __restrict__ amax, T* __restrict__ y, int64_t n, int64_t len, int64_t inner) {
  for (int64_t e = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; e < n; e += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = e / inner, in = e - t * inner;
    const int64_t o = t / len, i = t - o * len;
    Store<T>::st(y + e, (int64_t)amax[o * inner + in] == i ? 1.f : 0.f);
  }
}

// sel[0] = number of non-zero conditions, sel[1 + r] = position of the r-th of them.
// One workgroup: every thread counts a contiguous share, thread 0 turns the counts into
// offsets, every thread writes its share's positions.
__global__ void __launch_bounds__(kThreads)
compress_select_kernel(const uint8_t* __restrict__ cond, int n, int32_t* __restrict__ sel) {
  __shared__ int cnt[kThreads + 1];
  const int tid = threadIdx.x;
  const int per = (n + kThreads - 1) / kThreads;
  const int lo = tid * per < n ? tid * per : n;
  const int hi = lo + per < n ? lo + per : n;
  int c = 0;
  for (int j = lo; j < hi; ++j) c += cond[j] != 0;
  cnt[tid + 1] = c;
  __syncthreads();
  if (tid == 0) {
    cnt[0] = 0;
    for (int t = 0; t < kThreads; ++t) cnt[t + 1] += cnt[t];
    sel[0] = cnt[kThreads];
  }
  __syncthreads();
  int r = cnt[tid];
  for (int j = lo; j < hi; ++j)
    if (cond[j] != 0) sel[1 + r++] = j;
}

// The selected slices of every outer index, one behind the other from the start of y
// ([outer][selected][inner], dense); zeros behind them up to the declared size.
template <int ES>
__global__ void __launch_bounds__(kThreads)
compress_copy_kernel(const typename Word<ES>::type* __restrict__ x, const int32_t* __restrict__ sel,
                     typename Word<ES>::type* __restrict__ y, int64_t outer, int64_t len, int64_t inner, int64_t n_out) {
  const int64_t per = (int64_t)sel[0] * inner;
  const int64_t filled = outer * per;
  for (int64_t e = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; e < n_out; e += (int64_t)gridDim.x * blockDim.x) {
    typename Word<ES>::type v = 0;
    if (e < filled) {
      const int64_t o = e / per, r = e - o * per;
      const int64_t jo = r / inner, k = r - jo * inner;
      v = x[(o * len + sel[1 + jo]) * inner + k];
    }
    y[e] = v;
  }
}

#define AXIS_WORD_DISPATCH(es, EXPR)          \
  switch (es) {                               \
    case 1: { constexpr int ES = 1; EXPR; break; } \
    case 2: { constexpr int ES = 2; EXPR; break; } \
    case 4: { constexpr int ES = 4; EXPR; break; } \
    case 8: { constexpr int ES = 8; EXPR; break; } \
    default: return hipErrorInvalidValue;     \
  }
#define AXIS_FLOAT_DISPATCH(dt, EXPR)                  \
  switch (dt) {                                        \
    case DT_F32: { using T = float; EXPR; break; }     \
    case DT_F16: { using T = f16_t; EXPR; break; }     \
    case DT_BF16: { using T = bf16_t; EXPR; break; }   \
    default: return hipErrorInvalidValue;              \
  }

}  // namespace

hipError_t launch_gather_elements(const void* x, const void* idx, DType idx_dt, void* y, int elem_size, int64_t ii,
                                  int64_t ij, int64_t ik, int64_t di, int64_t dj, int64_t dk, hipStream_t stream) {
  if (!x || !idx || !y || ii <= 0 || ij <= 0 || ik <= 0 || dj <= 0 || ii > di || ik > dk) return hipErrorInvalidValue;
  if (idx_dt != DT_I32 && idx_dt != DT_I64) return hipErrorInvalidValue;
  const int64_t n = ii * ij * ik;
  const int grid = grid_for(n, kThreads);
  using W1 = int32_t; using W2 = int64_t;
  if (idx_dt == DT_I32) {
    AXIS_WORD_DISPATCH(elem_size, hipLaunchKernelGGL((gather_elements_kernel<ES, W1>), dim3(grid), dim3(kThreads), 0, stream,
                       reinterpret_cast<const typename Word<ES>::type*>(x), reinterpret_cast<const W1*>(idx),
                       reinterpret_cast<typename Word<ES>::type*>(y), n, ij, ik, dj, dk));
  } else {
    AXIS_WORD_DISPATCH(elem_size, hipLaunchKernelGGL((gather_elements_kernel<ES, W2>), dim3(grid), dim3(kThreads), 0, stream,
                       reinterpret_cast<const typename Word<ES>::type*>(x), reinterpret_cast<const W2*>(idx),
                       reinterpret_cast<typename Word<ES>::type*>(y), n, ij, ik, dj, dk));
  }
  return hipGetLastError();
}

hipError_t launch_cumsum(const void* x, void* y, DType dt, int64_t outer, int64_t len, int64_t inner, bool exclusive,
                         bool reverse, hipStream_t stream) {
  if (!x || !y || outer <= 0 || len <= 0 || inner <= 0) return hipErrorInvalidValue;
  const int64_t lines = outer * inner;
  // few long contiguous lines: a wavefront each (the additions then form a tree per 64
  // elements instead of one chain); otherwise a thread each, neighbours on neighbouring lines
  if (inner == 1 && len >= 128 && lines < 64 * 1024) {
    const int grid = grid_for(lines * 64, kThreads);
    AXIS_FLOAT_DISPATCH(dt, hipLaunchKernelGGL(cumsum_wave_kernel<T>, dim3(grid), dim3(kThreads), 0, stream,
                        reinterpret_cast<const T*>(x), reinterpret_cast<T*>(y), lines, len, exclusive, reverse));
  } else {
    const int grid = grid_for(lines, kThreads);
    AXIS_FLOAT_DISPATCH(dt, hipLaunchKernelGGL(cumsum_lines_kernel<T>, dim3(grid), dim3(kThreads), 0, stream,
                        reinterpret_cast<const T*>(x), reinterpret_cast<T*>(y), outer, len, inner, exclusive, reverse));
  }
  return hipGetLastError();
}

hipError_t launch_onehot_axis(const void* amax, DType idx_dt, void* y, DType dt, int64_t outer, int64_t len, int64_t inner,
                              hipStream_t stream) {
  if (!amax || !y || outer <= 0 || len <= 0 || inner <= 0) return hipErrorInvalidValue;
  if (idx_dt != DT_I32 && idx_dt != DT_I64) return hipErrorInvalidValue;
  const int64_t n = outer * len * inner;
  const int grid = grid_for(n, kThreads);
  if (idx_dt == DT_I32) {
    AXIS_FLOAT_DISPATCH(dt, hipLaunchKernelGGL((onehot_axis_kernel<T, int32_t>), dim3(grid), dim3(kThreads), 0, stream,
                        reinterpret_cast<const int32_t*>(amax), reinterpret_cast<T*>(y), n, len, inner));
  } else {
    AXIS_FLOAT_DISPATCH(dt, hipLaunchKernelGGL((onehot_axis_kernel<T, int64_t>), dim3(grid), dim3(kThreads), 0, stream,
                        reinterpret_cast<const int64_t*>(amax), reinterpret_cast<T*>(y), n, len, inner));
  }
  return hipGetLastError();
}

hipError_t launch_compress(const void* x, const void* cond, int n_cond, int32_t* sel, void* y, int elem_size,
                           int64_t outer, int64_t len, int64_t inner, int64_t n_out, hipStream_t stream) {
  if (!x || !cond || !sel || !y || n_cond < 0 || n_cond > len || outer <= 0 || len <= 0 || inner <= 0 || n_out <= 0)
    return hipErrorInvalidValue;
  hipLaunchKernelGGL(compress_select_kernel, dim3(1), dim3(kThreads), 0, stream, reinterpret_cast<const uint8_t*>(cond),
                     n_cond, sel);
  const int grid = grid_for(n_out, kThreads);
  AXIS_WORD_DISPATCH(elem_size, hipLaunchKernelGGL(compress_copy_kernel<ES>, dim3(grid), dim3(kThreads), 0, stream,
                     reinterpret_cast<const typename Word<ES>::type*>(x), sel,
                     reinterpret_cast<typename Word<ES>::type*>(y), outer, len, inner, n_out));
  return hipGetLastError();
}

}  // namespace ohip
