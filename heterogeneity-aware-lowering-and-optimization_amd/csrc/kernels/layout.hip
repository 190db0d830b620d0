// Data-movement kernels for gfx950: N,C,HW <-> channels-last conversion with
// type conversion (LDS-tiled so both sides stay coalesced), generic strided
// copy (transpose / concat / slice), nearest resize and row gather.
#include "device_utils.h"

namespace ohip {
namespace {

constexpr int kThreads = 256;
constexpr int TC = 32;   // channels per tile
constexpr int THW = 64;  // positions per tile

template <typename T> __device__ __forceinline__ float ld_as_float(const T* p, float, int) {
  return Store<T>::ld(p);
}
// dequantise a stored 8-bit level
template <> __device__ __forceinline__ float ld_as_float<int8_t>(const int8_t* p, float scale, int zp) {
  return (float)(q_from_stored(*p) - zp) * scale;
}
template <typename T> __device__ __forceinline__ void st_from_float(T* p, float v, float, int) {
  Store<T>::st(p, v);
}
// quantise to a stored 8-bit level: q = clamp(rne(v / scale) + zp, 0, 255)
template <> __device__ __forceinline__ void st_from_float<int8_t>(int8_t* p, float v, float scale, int zp) {
  float t = rintf(v / scale) + (float)zp;
  t = fminf(fmaxf(t, 0.f), 255.f);
  *p = q_to_stored((int)t);
}

// src [N][C][HW] -> dst [N][HW][cs]; channels C..cs-1 are written as `fill`.
template <typename TS, typename TD>
__global__ void __launch_bounds__(kThreads) nchw_to_nhwc_tiled(LayoutParams p, float fill) {
  __shared__ float tile[TC][THW + 1];
  const TS* src = reinterpret_cast<const TS*>(p.src);
  TD* dst = reinterpret_cast<TD*>(p.dst);
  const int tiles_hw = (p.HW + THW - 1) / THW;
  const int tiles_c = (p.cs + TC - 1) / TC;
  const int64_t ntiles = (int64_t)p.N * tiles_hw * tiles_c;
  for (int64_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
    const int tc = (int)(t % tiles_c);
    const int thw = (int)((t / tiles_c) % tiles_hw);
    const int n = (int)(t / ((int64_t)tiles_c * tiles_hw));
    const int c0 = tc * TC, hw0 = thw * THW;
    {
      const int tx = threadIdx.x % THW, ty = threadIdx.x / THW;
      for (int cc = ty; cc < TC; cc += kThreads / THW) {
        const int c = c0 + cc, hw = hw0 + tx;
        float v = fill;
        if (c < p.C && hw < p.HW) v = ld_as_float<TS>(src + ((int64_t)n * p.C + c) * p.HW + hw, p.scale, p.zp);
        tile[cc][tx] = v;
      }
    }
    __syncthreads();
    {
      const int tx = threadIdx.x % TC, ty = threadIdx.x / TC;
      for (int hh = ty; hh < THW; hh += kThreads / TC) {
        const int c = c0 + tx, hw = hw0 + hh;
        if (c < p.cs && hw < p.HW)
          st_from_float<TD>(dst + ((int64_t)n * p.HW + hw) * p.cs + c, tile[tx][hh], p.scale, p.zp);
      }
    }
    __syncthreads();
  }
}

// Few channels (cs <= 16): one thread per PX consecutive pixels; each channel
// plane is read with one PX-wide load per thread (coalesced across the
// wavefront) and PX contiguous pixels are written per thread.
template <typename TS, typename TD, int PX>
__global__ void __launch_bounds__(kThreads) nchw_to_nhwc_smallc(LayoutParams p, float fill) {
  const TS* src = reinterpret_cast<const TS*>(p.src);
  TD* dst = reinterpret_cast<TD*>(p.dst);
  const int64_t hwg = p.HW / PX;  // HW % PX == 0 checked by the launcher
  const int64_t total = (int64_t)p.N * hwg;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t n = i / hwg, hw = (i - n * hwg) * PX;
    float in[16][PX];
#pragma unroll
    for (int c = 0; c < 16; ++c) {
      if (c < p.C) {
        const TS* s = src + (n * p.C + c) * p.HW + hw;
        if constexpr (PX == 4 && sizeof(TS) == 4) {
          const floatx4 t = *reinterpret_cast<const floatx4*>(s);
          in[c][0] = t.x; in[c][1] = t.y; in[c][2] = t.z; in[c][3] = t.w;
        } else {
#pragma unroll
          for (int k = 0; k < PX; ++k) in[c][k] = ld_as_float<TS>(s + k, p.scale, p.zp);
        }
      }
    }
#pragma unroll
    for (int k = 0; k < PX; ++k) {
      // (every index into `out` below is a constant once the loops are unrolled: an array read
      //  back through a vector pointer at a run-time index is not split into registers, and the
      //  compiler then keeps it in LDS)
      alignas(16) TD out[16];
#pragma unroll
      for (int c = 0; c < 16; ++c) st_from_float<TD>(&out[c], c < p.C ? in[c][k] : fill, p.scale, p.zp);
      TD* o = dst + (n * p.HW + hw + k) * p.cs;
      if ((p.cs * sizeof(TD)) % 16 == 0) {
        constexpr int NV = 16 * (int)sizeof(TD) / 16;
#pragma unroll
        for (int v = 0; v < NV; ++v)
          if (v * 16 < p.cs * (int)sizeof(TD)) reinterpret_cast<uintx4*>(o)[v] = reinterpret_cast<const uintx4*>(out)[v];
      } else {
#pragma unroll
        for (int c = 0; c < 16; ++c)
          if (c < p.cs) o[c] = out[c];
      }
    }
  }
}

// The same for results of exactly 16 bytes per pixel (cs * sizeof(TD) == 16) and HW a multiple of
// 1024: a workgroup takes 1024 consecutive pixels and a thread the four pixels tid, tid + 256,
// ... of them, so that every store instruction of a wavefront writes 1 KiB of contiguous
// memory (with four consecutive pixels per thread its lanes are 64 bytes apart and every
// instruction touches 64 cache lines a quarter each).  The loads are one element per lane per
// channel plane, 256 contiguous bytes per instruction.
template <typename TS, typename TD>
__global__ void __launch_bounds__(kThreads) nchw_to_nhwc_rows16(LayoutParams p, float fill) {
  const TS* src = reinterpret_cast<const TS*>(p.src);
  TD* dst = reinterpret_cast<TD*>(p.dst);
  constexpr int CS = 16 / (int)sizeof(TD);
  const int64_t blocks_per_image = p.HW / 1024;
  const int64_t total = (int64_t)p.N * blocks_per_image;
  for (int64_t b = blockIdx.x; b < total; b += gridDim.x) {
    const int64_t n = b / blocks_per_image;
    const int64_t hw0 = (b - n * blocks_per_image) * 1024 + threadIdx.x;
    float in[CS][4];
#pragma unroll
    for (int c = 0; c < CS; ++c) {
#pragma unroll
      for (int k = 0; k < 4; ++k) in[c][k] = fill;
      if (c < p.C) {   // (uniform: p.C is a kernel argument)
        const TS* s = src + (n * p.C + c) * p.HW + hw0;
#pragma unroll
        for (int k = 0; k < 4; ++k) in[c][k] = ld_as_float<TS>(s + k * 256, p.scale, p.zp);
      }
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      TD out[CS];
#pragma unroll
      for (int c = 0; c < CS; ++c) st_from_float<TD>(&out[c], in[c][k], p.scale, p.zp);
      uintx4* o = reinterpret_cast<uintx4*>(dst + (n * p.HW + hw0 + k * 256) * p.cs);
      __builtin_nontemporal_store(*reinterpret_cast<const uintx4*>(out), o);
    }
  }
}

// src [N][HW][cs] -> dst [N][C][HW]
template <typename TS, typename TD>
__global__ void __launch_bounds__(kThreads) nhwc_to_nchw_tiled(LayoutParams p) {
  __shared__ float tile[TC][THW + 1];
  const TS* src = reinterpret_cast<const TS*>(p.src);
  TD* dst = reinterpret_cast<TD*>(p.dst);
  const int tiles_hw = (p.HW + THW - 1) / THW;
  const int tiles_c = (p.C + TC - 1) / TC;
  const int64_t ntiles = (int64_t)p.N * tiles_hw * tiles_c;
  for (int64_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
    const int tc = (int)(t % tiles_c);
    const int thw = (int)((t / tiles_c) % tiles_hw);
    const int n = (int)(t / ((int64_t)tiles_c * tiles_hw));
    const int c0 = tc * TC, hw0 = thw * THW;
    {
      const int tx = threadIdx.x % TC, ty = threadIdx.x / TC;
      for (int hh = ty; hh < THW; hh += kThreads / TC) {
        const int c = c0 + tx, hw = hw0 + hh;
        float v = 0.f;
        if (c < p.C && hw < p.HW) v = ld_as_float<TS>(src + ((int64_t)n * p.HW + hw) * p.cs + c, p.scale, p.zp);
        tile[tx][hh] = v;
      }
    }
    __syncthreads();
    {
      const int tx = threadIdx.x % THW, ty = threadIdx.x / THW;
      for (int cc = ty; cc < TC; cc += kThreads / THW) {
        const int c = c0 + cc, hw = hw0 + tx;
        if (c < p.C && hw < p.HW)
          st_from_float<TD>(dst + ((int64_t)n * p.C + c) * p.HW + hw, tile[cc][tx], p.scale, p.zp);
      }
    }
    __syncthreads();
  }
}

// Generic strided copy of `ES`-byte elements; the innermost dim is walked by
// consecutive threads.  I is the type the flat index is decomposed in: 32-bit
// division costs a fifth of the 64-bit one.
template <typename E, typename I>
__global__ void __launch_bounds__(kThreads) strided_copy_kernel(StridedCopyParams p, int64_t n) {
  const E* x = reinterpret_cast<const E*>(p.x) + p.x_off;
  E* y = reinterpret_cast<E*>(p.y) + p.y_off;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x) {
    I rem = (I)i;
    int64_t ox = 0, oy = 0;
#pragma unroll
    for (int d = 7; d >= 0; --d) {
      if (d < p.rank) {
        const I dim = (I)p.dims[d];
        const I q = rem / dim;
        const int64_t idx = (int64_t)(rem - q * dim);
        rem = q;
        ox += idx * p.sx[d];
        oy += idx * p.sy[d];
      }
    }
    y[oy] = x[ox];
  }
}

// Strided copy whose source is contiguous along one dim (`a`) and whose
// destination is contiguous along another (`b`): 64 x 64 tiles of the (a, b)
// plane go through LDS, so that both sides move whole runs.  The remaining
// dims index the tiles' origins.
struct TileCopyParams {
  const void* x; void* y;
  int64_t x_off, y_off;
  int Da, Db;          // extents of the two dims
  int64_t sxb, sya;    // source stride along b, destination stride along a
  int n_outer;
  int64_t odims[6], osx[6], osy[6];
};

template <typename E>
__global__ void __launch_bounds__(kThreads) strided_tile_copy_kernel(TileCopyParams p, int64_t ntiles) {
  constexpr int TS = 64;
  __shared__ E tile[TS][TS + 2];
  const E* x = reinterpret_cast<const E*>(p.x) + p.x_off;
  E* y = reinterpret_cast<E*>(p.y) + p.y_off;
  const int ta_n = (p.Da + TS - 1) / TS, tb_n = (p.Db + TS - 1) / TS;
  const int tx = threadIdx.x % TS, ty = threadIdx.x / TS;
  for (int64_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
    const int a0 = (int)(t % ta_n) * TS;
    const int b0 = (int)((t / ta_n) % tb_n) * TS;
    int64_t o = t / ((int64_t)ta_n * tb_n), ox = 0, oy = 0;
    for (int d = p.n_outer - 1; d >= 0; --d) {
      const int64_t q = o / p.odims[d], idx = o - q * p.odims[d];
      o = q;
      ox += idx * p.osx[d];
      oy += idx * p.osy[d];
    }
    for (int rr = ty; rr < TS; rr += kThreads / TS) {
      const int b = b0 + rr, a = a0 + tx;
      if (b < p.Db && a < p.Da) tile[rr][tx] = x[ox + b * p.sxb + a];
    }
    __syncthreads();
    for (int cc = ty; cc < TS; cc += kThreads / TS) {
      const int a = a0 + cc, b = b0 + tx;
      if (a < p.Da && b < p.Db) y[oy + a * p.sya + b] = tile[tx][cc];
    }
    __syncthreads();
  }
}

// The same for 2-byte elements, moving eight of them per request on the side(s) whose
// strides and base keep 16-byte alignment (VL: the source runs, VS: the destination runs);
// the other side moves single elements as above.  Tile [b][a], 66 elements per row.
template <bool VL, bool VS>
__global__ void __launch_bounds__(kThreads) strided_tile_copy16_kernel(TileCopyParams p, int64_t ntiles) {
  constexpr int TS = 64, PITCH = 66;
  __shared__ __attribute__((aligned(16))) uint16_t tile[TS * PITCH];
  const uint16_t* x = reinterpret_cast<const uint16_t*>(p.x) + p.x_off;
  uint16_t* y = reinterpret_cast<uint16_t*>(p.y) + p.y_off;
  const int ta_n = (p.Da + TS - 1) / TS, tb_n = (p.Db + TS - 1) / TS;
  const int tid = threadIdx.x;
  for (int64_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
    const int a0 = (int)(t % ta_n) * TS;
    const int b0 = (int)((t / ta_n) % tb_n) * TS;
    int64_t o = t / ((int64_t)ta_n * tb_n), ox = 0, oy = 0;
    for (int d = p.n_outer - 1; d >= 0; --d) {
      const int64_t q = o / p.odims[d], idx = o - q * p.odims[d];
      o = q;
      ox += idx * p.osx[d];
      oy += idx * p.osy[d];
    }
    if constexpr (VL) {
      const int v = tid & 7;
#pragma unroll
      for (int pass = 0; pass < 2; ++pass) {
        const int bb = (tid >> 3) + pass * 32;
        const int a = a0 + v * 8, b = b0 + bb;
        if (b < p.Db && a < p.Da) {
          const uint16_t* src = x + ox + (int64_t)b * p.sxb + a;
          uint16_t* dst = tile + bb * PITCH + v * 8;
          if (a + 8 <= p.Da) {
            const uintx4 q = *reinterpret_cast<const uintx4*>(src);
            uint32_t* d32 = reinterpret_cast<uint32_t*>(dst);   // (PITCH and 8 v are even)
            d32[0] = q.x; d32[1] = q.y; d32[2] = q.z; d32[3] = q.w;
          } else {
            for (int e = 0; a + e < p.Da; ++e) dst[e] = src[e];
          }
        }
      }
    } else {
      const int tx = tid % TS, ty = tid / TS;
      for (int rr = ty; rr < TS; rr += kThreads / TS) {
        const int b = b0 + rr, a = a0 + tx;
        if (b < p.Db && a < p.Da) tile[rr * PITCH + tx] = x[ox + (int64_t)b * p.sxb + a];
      }
    }
    __syncthreads();
    if constexpr (VS) {
      const int v = tid & 7;
#pragma unroll
      for (int pass = 0; pass < 2; ++pass) {
        const int aa = (tid >> 3) + pass * 32;
        const int a = a0 + aa, b = b0 + v * 8;
        if (a < p.Da && b < p.Db) {
          uint16_t* dst = y + oy + (int64_t)a * p.sya + b;
          const uint16_t* src = tile + (v * 8) * PITCH + aa;
          if (b + 8 <= p.Db) {
            uint32_t w[4];
#pragma unroll
            for (int e = 0; e < 4; ++e)
              w[e] = (uint32_t)src[(2 * e) * PITCH] | ((uint32_t)src[(2 * e + 1) * PITCH] << 16);
            *reinterpret_cast<uintx4*>(dst) = uintx4{w[0], w[1], w[2], w[3]};
          } else {
            for (int e = 0; b + e < p.Db; ++e) dst[e] = src[e * PITCH];
          }
        }
      }
    } else {
      const int tx = tid % TS, ty = tid / TS;
      for (int cc = ty; cc < TS; cc += kThreads / TS) {
        const int a = a0 + cc, b = b0 + tx;
        if (a < p.Da && b < p.Db) y[oy + (int64_t)a * p.sya + b] = tile[tx * PITCH + cc];
      }
    }
    __syncthreads();
  }
}

// Batched 2-D transpose through an LDS tile: y[b][c][r] = x[b][r][c]; the
// destination row pitch may exceed `rows` (zero padding is the caller's job).
template <typename E>
__global__ void __launch_bounds__(kThreads)
transpose2d_kernel(const E* __restrict__ x, E* __restrict__ y, int batch, int rows, int cols,
                   int dst_pitch) {
  constexpr int TS = 64;
  __shared__ E tile[TS][TS + 2];
  const int tr = (rows + TS - 1) / TS, tc = (cols + TS - 1) / TS;
  const int64_t ntiles = (int64_t)batch * tr * tc;
  for (int64_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
    const int ct = (int)(t % tc);
    const int rt = (int)((t / tc) % tr);
    const int b = (int)(t / ((int64_t)tc * tr));
    const int r0 = rt * TS, c0 = ct * TS;
    const int tx = threadIdx.x % TS, ty = threadIdx.x / TS;
    for (int rr = ty; rr < TS; rr += kThreads / TS) {
      const int r = r0 + rr, c = c0 + tx;
      if (r < rows && c < cols) tile[rr][tx] = x[((int64_t)b * rows + r) * cols + c];
    }
    __syncthreads();
    for (int cc = ty; cc < TS; cc += kThreads / TS) {
      const int c = c0 + cc, r = r0 + tx;
      if (r < rows && c < cols) y[((int64_t)b * cols + c) * dst_pitch + r] = tile[tx][cc];
    }
    __syncthreads();
  }
}

template <typename E>
__global__ void __launch_bounds__(kThreads)
resize_nearest_kernel(const E* __restrict__ x, E* __restrict__ y, int N, int H, int W, int cv,
                      int Ho, int Wo) {
  const int64_t total = (int64_t)N * Ho * Wo * cv;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int c = (int)(i % cv);
    int64_t t = i / cv;
    const int wo = (int)(t % Wo); t /= Wo;
    const int ho = (int)(t % Ho);
    const int n = (int)(t / Ho);
    const int hi = (int)(((int64_t)ho * H) / Ho), wi = (int)(((int64_t)wo * W) / Wo);
    y[i] = x[(((int64_t)n * H + hi) * W + wi) * cv + c];
  }
}

// Nearest resize by whole factors (Ho = fh * H, Wo = fw * W): workgroups walk source rows
// (grid.x) in pieces of 256 vectors (grid.y); every source vector is read once and written fh * fw times; no division per element
// but the one by the vectors per pixel.
template <typename E>
__global__ void __launch_bounds__(kThreads)
resize_nearest_whole_kernel(const E* __restrict__ x, E* __restrict__ y, int rows, int H, int W, int cv, int fh, int fw) {
  const int row_vecs = W * cv;
  const int Wo = W * fw;
  for (int row = blockIdx.x; row < rows; row += gridDim.x) {
    const int n = row / H, hi = row - n * H;
    const E* src = x + (int64_t)row * row_vecs;
    E* dst = y + ((int64_t)n * H * fh + (int64_t)hi * fh) * Wo * cv;
    for (int j = blockIdx.y * kThreads + threadIdx.x; j < row_vecs; j += gridDim.y * kThreads) {
      const int wi = j / cv, c = j - wi * cv;
      const E v = src[j];
      for (int a = 0; a < fh; ++a)
        for (int b = 0; b < fw; ++b) dst[((int64_t)a * Wo + wi * fw + b) * cv + c] = v;
    }
  }
}

// Bilinear resize, channels-last, pixel centres at half-integers and edge
// clamping: source coordinate s = (o + 0.5) * in / out - 0.5, neighbours
// floor(s) and floor(s) + 1 clamped into the image, weights 1 - frac and frac
// (oneDNN's resampling_linear, which is what the reference calls for
// ODLA_LINEAR whatever coordinate mode is passed).  One thread per group of V
// channels of one output pixel.
template <typename T, int V>
__global__ void __launch_bounds__(kThreads)
resize_linear_kernel(const T* __restrict__ x, T* __restrict__ y, int N, int H, int W, int cs,
                     int Ho, int Wo, float fh, float fw) {
  const int cv = cs / V;
  const int64_t total = (int64_t)N * Ho * Wo * cv;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int c = (int)(i % cv) * V;
    int64_t t = i / cv;
    const int wo = (int)(t % Wo); t /= Wo;
    const int ho = (int)(t % Ho);
    const int n = (int)(t / Ho);
    float sh = ((float)ho + 0.5f) * fh - 0.5f, sw = ((float)wo + 0.5f) * fw - 0.5f;
    sh = sh < 0.f ? 0.f : sh;
    sw = sw < 0.f ? 0.f : sw;
    int h0 = (int)sh, w0 = (int)sw;
    h0 = h0 > H - 1 ? H - 1 : h0;
    w0 = w0 > W - 1 ? W - 1 : w0;
    const int h1 = h0 < H - 1 ? h0 + 1 : h0, w1 = w0 < W - 1 ? w0 + 1 : w0;
    const float ah = sh - (float)h0, aw = sw - (float)w0;
    const float k00 = (1.f - ah) * (1.f - aw), k01 = (1.f - ah) * aw, k10 = ah * (1.f - aw), k11 = ah * aw;
    const T* base = x + (int64_t)n * H * W * cs + c;
    const T* p00 = base + ((int64_t)h0 * W + w0) * cs;
    const T* p01 = base + ((int64_t)h0 * W + w1) * cs;
    const T* p10 = base + ((int64_t)h1 * W + w0) * cs;
    const T* p11 = base + ((int64_t)h1 * W + w1) * cs;
    T* out = y + (((int64_t)n * Ho + ho) * Wo + wo) * cs + c;
    if constexpr (V > 1) {
      Vec16<T> a, b, d, e, o;
      a.load(p00); b.load(p01); d.load(p10); e.load(p11);
#pragma unroll
      for (int k = 0; k < V; ++k) o.set(k, k00 * a.get(k) + k01 * b.get(k) + k10 * d.get(k) + k11 * e.get(k));
      o.store(out);
    } else {
      Store<T>::st(out, k00 * Store<T>::ld(p00) + k01 * Store<T>::ld(p01) + k10 * Store<T>::ld(p10) + k11 * Store<T>::ld(p11));
    }
  }
}

template <typename IDX>
__global__ void __launch_bounds__(kThreads)
gather_rows_kernel(const unsigned char* __restrict__ x, const IDX* __restrict__ idx,
                   unsigned char* __restrict__ y, int64_t outer, int64_t n_src, int64_t n_idx,
                   int64_t row_bytes, int vec) {
  // vec = bytes moved per thread step (16, 4, 2 or 1; row_bytes % vec == 0)
  const int64_t per_row = row_bytes / vec;
  const int64_t total = outer * n_idx * per_row;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t v = i % per_row;
    const int64_t rj = i / per_row;
    const int64_t j = rj % n_idx, o = rj / n_idx;
    int64_t s = (int64_t)idx[j];
    if (s < 0) s += n_src;
    s = s < 0 ? 0 : (s >= n_src ? n_src - 1 : s);  // clamp: never read outside the table
    const unsigned char* src = x + (o * n_src + s) * row_bytes + v * vec;
    unsigned char* dst = y + rj * row_bytes + v * vec;
    if (vec == 16) *reinterpret_cast<uintx4*>(dst) = *reinterpret_cast<const uintx4*>(src);
    else if (vec == 4) *reinterpret_cast<uint32_t*>(dst) = *reinterpret_cast<const uint32_t*>(src);
    else if (vec == 2) *reinterpret_cast<uint16_t*>(dst) = *reinterpret_cast<const uint16_t*>(src);
    else *dst = *src;
  }
}

struct b16 { uintx4 v; };

}  // namespace

#define LAYOUT_PAIR_DISPATCH(KERNEL, ...)                                                      \
  do {                                                                                         \
    if (p.src_dt == DT_F32 && p.dst_dt == DT_F32) { KERNEL(float, float, __VA_ARGS__); }       \
    else if (p.src_dt == DT_F32 && p.dst_dt == DT_F16) { KERNEL(float, f16_t, __VA_ARGS__); }  \
    else if (p.src_dt == DT_F32 && p.dst_dt == DT_BF16) { KERNEL(float, bf16_t, __VA_ARGS__); }\
    else if (p.src_dt == DT_F16 && p.dst_dt == DT_F32) { KERNEL(f16_t, float, __VA_ARGS__); }  \
    else if (p.src_dt == DT_BF16 && p.dst_dt == DT_F32) { KERNEL(bf16_t, float, __VA_ARGS__); }\
    else if (p.src_dt == DT_F16 && p.dst_dt == DT_F16) { KERNEL(f16_t, f16_t, __VA_ARGS__); }  \
    else if (p.src_dt == DT_BF16 && p.dst_dt == DT_BF16) { KERNEL(bf16_t, bf16_t, __VA_ARGS__); }\
    else if (p.src_dt == DT_F32 && p.dst_dt == DT_I8) { KERNEL(float, int8_t, __VA_ARGS__); }  \
    else if (p.src_dt == DT_I8 && p.dst_dt == DT_F32) { KERNEL(int8_t, float, __VA_ARGS__); }  \
    else return hipErrorInvalidValue;                                                          \
  } while (0)

static bool layout_ok(const LayoutParams& p) {
  return p.src && p.dst && p.N > 0 && p.C > 0 && p.HW > 0 && p.cs >= p.C;
}

hipError_t launch_nchw_to_nhwc(const LayoutParams& p, hipStream_t stream) {
  if (!layout_ok(p)) return hipErrorInvalidValue;
  // padding lanes hold the real value 0 (its quantised level for 8-bit data)
  const float fill = 0.f;
  if (p.cs * dtype_size(p.dst_dt) == 16 && p.HW % 1024 == 0 && (reinterpret_cast<uintptr_t>(p.dst) & 15u) == 0 &&
      (p.dst_dt == DT_F16 || p.dst_dt == DT_BF16 || p.dst_dt == DT_I8)) {
    const int64_t blocks = (int64_t)p.N * (p.HW / 1024);
    const int grid = (int)(blocks < 65536 ? blocks : 65536);
#define K0(TS, TD, ...) hipLaunchKernelGGL((nchw_to_nhwc_rows16<TS, TD>), dim3(grid), dim3(kThreads), 0, stream, p, fill)
    LAYOUT_PAIR_DISPATCH(K0, 0);
#undef K0
    return hipGetLastError();
  }
  if (p.cs <= 16) {
    const bool px4 = p.HW % 4 == 0 && (reinterpret_cast<uintptr_t>(p.src) & 15u) == 0 && p.src_dt == DT_F32;
    if (px4) {
      const int grid = grid_for((int64_t)p.N * p.HW / 4, kThreads);
#define K1(TS, TD, ...) hipLaunchKernelGGL((nchw_to_nhwc_smallc<TS, TD, 4>), dim3(grid), dim3(kThreads), 0, stream, p, fill)
      LAYOUT_PAIR_DISPATCH(K1, 0);
#undef K1
    } else {
      const int grid = grid_for((int64_t)p.N * p.HW, kThreads);
#define K1(TS, TD, ...) hipLaunchKernelGGL((nchw_to_nhwc_smallc<TS, TD, 1>), dim3(grid), dim3(kThreads), 0, stream, p, fill)
      LAYOUT_PAIR_DISPATCH(K1, 0);
#undef K1
    }
  } else {
    const int64_t ntiles = (int64_t)p.N * ((p.HW + THW - 1) / THW) * ((p.cs + TC - 1) / TC);
    const int grid = (int)(ntiles < 65536 ? ntiles : 65536);
#define K2(TS, TD, ...) hipLaunchKernelGGL((nchw_to_nhwc_tiled<TS, TD>), dim3(grid), dim3(kThreads), 0, stream, p, fill)
    LAYOUT_PAIR_DISPATCH(K2, 0);
#undef K2
  }
  return hipGetLastError();
}

// NCHW -> channels-last space-to-depth: dst pixel (hh, ww) of the half-size
// image holds the 2x2 source block at (2hh, 2ww), channel (py*2 + px)*C + c =
// src[n][c][2hh+py][2ww+px]; source positions beyond an odd H / W and the
// channel padding up to cs hold the real value 0.  A stride-2 convolution over
// the source is a stride-1 convolution over this tensor with a quarter of the
// filter taps and four times the channels: few-channel network inputs then fill
// their 16-byte vectors instead of being padded 3 -> 8.
// CC = number of source channels (a template parameter so that the channel
// index of every value is a constant and `out` stays in registers).
template <typename TS, typename TD, int CC>
__global__ void __launch_bounds__(kThreads) nchw_to_s2d_kernel(S2dParams p) {
  const TS* src = reinterpret_cast<const TS*>(p.src);
  TD* dst = reinterpret_cast<TD*>(p.dst);
  const int Hs = (p.H + 1) >> 1, Ws = (p.W + 1) >> 1;
  const int64_t total = (int64_t)p.N * Hs * Ws;
  // an even row length keeps every 2-pixel pair of a float source 8-byte aligned
  const bool pairs = std::is_same<TS, float>::value && (p.W & 1) == 0 && (reinterpret_cast<uintptr_t>(src) & 7u) == 0;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int ww = (int)(i % Ws);
    const int64_t t = i / Ws;
    const int hh = (int)(t % Hs);
    const int64_t n = t / Hs;
    float in[2][CC][2];
#pragma unroll
    for (int py = 0; py < 2; ++py) {
      const int h = 2 * hh + py;
#pragma unroll
      for (int c = 0; c < CC; ++c) {
        in[py][c][0] = in[py][c][1] = 0.f;
        if (h < p.H) {
          const TS* row = src + ((n * CC + c) * p.H + h) * (int64_t)p.W + 2 * ww;
          if (pairs) {
            typedef float floatx2 __attribute__((ext_vector_type(2)));
            const floatx2 v = __builtin_nontemporal_load(reinterpret_cast<const floatx2*>(row));
            in[py][c][0] = v.x;
            in[py][c][1] = v.y;
          } else {
            in[py][c][0] = ld_as_float<TS>(row, p.scale, p.zp);
            if (2 * ww + 1 < p.W) in[py][c][1] = ld_as_float<TS>(row + 1, p.scale, p.zp);
          }
        }
      }
    }
    TD* o = dst + i * p.cs;
    if constexpr (sizeof(TD) <= 2) {
      // The pixel's 16 stored values, packed into registers word by word.  (An array of TD read
      // back through a vector pointer at a run-time index is not split into registers: the
      // compiler moved it to LDS - two-byte writes, half of its LDS cycles bank conflicts.)
      constexpr int PW = 4 / (int)sizeof(TD);   // values per 32-bit word
      unsigned word[16 / PW];
#pragma unroll
      for (int w = 0; w < 16 / PW; ++w) {
        word[w] = 0;
#pragma unroll
        for (int e = 0; e < PW; ++e) {
          const int c = w * PW + e;   // (py * 2 + px) * CC + cc, zeros from 4 * CC on
          const float val = c < 4 * CC ? in[(c / CC) >> 1][c % CC][(c / CC) & 1] : 0.f;
          TD t;
          st_from_float<TD>(&t, val, p.scale, p.zp);
          unsigned bits;
          if constexpr (sizeof(TD) == 2) bits = __builtin_bit_cast(unsigned short, t);
          else bits = __builtin_bit_cast(unsigned char, t);
          word[w] |= bits << (e * 8 * (int)sizeof(TD));
        }
      }
      if ((p.cs * sizeof(TD)) % 16 == 0) {
        reinterpret_cast<uintx4*>(o)[0] = (uintx4){word[0], word[1], word[2], word[3]};
        if constexpr (sizeof(TD) == 2) {
          if (p.cs == 16) reinterpret_cast<uintx4*>(o)[1] = (uintx4){word[4], word[5], word[6], word[7]};
        }
      } else {
#pragma unroll
        for (int c = 0; c < 16; ++c)
          if (c < p.cs) {
            const unsigned b = word[c / PW] >> ((c % PW) * 8 * (int)sizeof(TD));
            if constexpr (sizeof(TD) == 2) o[c] = __builtin_bit_cast(TD, (unsigned short)b);
            else o[c] = __builtin_bit_cast(TD, (unsigned char)b);
          }
      }
    } else {
      TD out[16];
#pragma unroll
      for (int c = 4 * CC; c < 16; ++c) st_from_float<TD>(&out[c], 0.f, p.scale, p.zp);
#pragma unroll
      for (int py = 0; py < 2; ++py)
#pragma unroll
        for (int px = 0; px < 2; ++px)
#pragma unroll
          for (int c = 0; c < CC; ++c) st_from_float<TD>(&out[(py * 2 + px) * CC + c], in[py][c][px], p.scale, p.zp);
      if ((p.cs * sizeof(TD)) % 16 == 0) {
        const int nv = p.cs * (int)sizeof(TD) / 16;
        for (int v = 0; v < nv; ++v) reinterpret_cast<uintx4*>(o)[v] = reinterpret_cast<const uintx4*>(out)[v];
      } else {
        for (int c = 0; c < p.cs; ++c) o[c] = out[c];
      }
    }
  }
}

hipError_t launch_nchw_to_s2d(const S2dParams& p, hipStream_t stream) {
  if (!p.src || !p.dst || p.N <= 0 || p.C <= 0 || p.C > 4 || p.H <= 0 || p.W <= 0 || p.cs < 4 * p.C || p.cs > 16)
    return hipErrorInvalidValue;
  const int64_t total = (int64_t)p.N * ((p.H + 1) / 2) * ((p.W + 1) / 2);
  const int grid = grid_for(total, kThreads);
#define K4(TS, TD, CC_) hipLaunchKernelGGL((nchw_to_s2d_kernel<TS, TD, CC_>), dim3(grid), dim3(kThreads), 0, stream, p)
  switch (p.C) {
    case 1: LAYOUT_PAIR_DISPATCH(K4, 1); break;
    case 2: LAYOUT_PAIR_DISPATCH(K4, 2); break;
    case 3: LAYOUT_PAIR_DISPATCH(K4, 3); break;
    default: LAYOUT_PAIR_DISPATCH(K4, 4); break;
  }
#undef K4
  return hipGetLastError();
}

hipError_t launch_nhwc_to_nchw(const LayoutParams& p, hipStream_t stream) {
  if (!layout_ok(p)) return hipErrorInvalidValue;
  const int64_t ntiles = (int64_t)p.N * ((p.HW + THW - 1) / THW) * ((p.C + TC - 1) / TC);
  const int grid = (int)(ntiles < 65536 ? ntiles : 65536);
#define K3(TS, TD, ...) hipLaunchKernelGGL((nhwc_to_nchw_tiled<TS, TD>), dim3(grid), dim3(kThreads), 0, stream, p)
  LAYOUT_PAIR_DISPATCH(K3, 0);
#undef K3
  return hipGetLastError();
}

hipError_t launch_strided_copy(const StridedCopyParams& p_in, hipStream_t stream) {
  if (!p_in.x || !p_in.y || p_in.rank < 1 || p_in.rank > 8) return hipErrorInvalidValue;
  int64_t n = 1;
  for (int d = 0; d < p_in.rank; ++d) {
    if (p_in.dims[d] <= 0) return hipErrorInvalidValue;
    n *= p_in.dims[d];
  }
  // Drop dims of extent 1 and merge neighbours that both sides walk as one run.
  StridedCopyParams p = p_in;
  int r = 0;
  for (int d = 0; d < p_in.rank; ++d) {
    if (p_in.dims[d] == 1) continue;
    if (r > 0 && p.sx[r - 1] == p_in.sx[d] * p_in.dims[d] && p.sy[r - 1] == p_in.sy[d] * p_in.dims[d]) {
      p.dims[r - 1] *= p_in.dims[d];
      p.sx[r - 1] = p_in.sx[d];
      p.sy[r - 1] = p_in.sy[d];
    } else {
      p.dims[r] = p_in.dims[d]; p.sx[r] = p_in.sx[d]; p.sy[r] = p_in.sy[d];
      ++r;
    }
  }
  if (r == 0) { p.dims[0] = 1; p.sx[0] = p.sy[0] = 0; r = 1; }
  for (int d = r; d < 8; ++d) { p.dims[d] = 1; p.sx[d] = p.sy[d] = 0; }
  p.rank = r;

  // A dim the source runs along and another the destination runs along: tiles.
  int a = -1, b = -1;
  for (int d = 0; d < r; ++d) {
    if (p.sx[d] == 1 && (a < 0 || p.dims[d] > p.dims[a])) a = d;
    if (p.sy[d] == 1 && (b < 0 || p.dims[d] > p.dims[b])) b = d;
  }
  const bool tiles = a >= 0 && b >= 0 && a != b && p.sy[a] != 1 && p.sx[b] != 1 && p.dims[a] >= 16 &&
                     p.dims[b] >= 16 && p.dims[a] < (1 << 30) && p.dims[b] < (1 << 30) && r <= 8 &&
                     p.elem_size <= 8;
  if (tiles) {
    TileCopyParams tp;
    tp.x = p.x; tp.y = p.y; tp.x_off = p.x_off; tp.y_off = p.y_off;
    tp.Da = (int)p.dims[a]; tp.Db = (int)p.dims[b];
    tp.sxb = p.sx[b]; tp.sya = p.sy[a];
    tp.n_outer = 0;
    int64_t outer = 1;
    for (int d = 0; d < r; ++d) {
      if (d == a || d == b) continue;
      tp.odims[tp.n_outer] = p.dims[d]; tp.osx[tp.n_outer] = p.sx[d]; tp.osy[tp.n_outer] = p.sy[d];
      ++tp.n_outer;
      outer *= p.dims[d];
    }
    for (int d = tp.n_outer; d < 6; ++d) { tp.odims[d] = 1; tp.osx[d] = tp.osy[d] = 0; }
    const int64_t ntiles = outer * ((tp.Da + 63) / 64) * ((tp.Db + 63) / 64);
    const int grid = (int)(ntiles < 65536 ? ntiles : 65536);
    if (p.elem_size == 2) {
      // eight elements per request on the sides that stay 16-byte aligned
      bool vl = tp.sxb % 8 == 0 && tp.x_off % 8 == 0 && (reinterpret_cast<uintptr_t>(tp.x) & 15u) == 0;
      bool vs = tp.sya % 8 == 0 && tp.y_off % 8 == 0 && (reinterpret_cast<uintptr_t>(tp.y) & 15u) == 0;
      for (int d = 0; d < tp.n_outer; ++d) {
        vl = vl && tp.osx[d] % 8 == 0;
        vs = vs && tp.osy[d] % 8 == 0;
      }
      if (vl && vs) hipLaunchKernelGGL((strided_tile_copy16_kernel<true, true>), dim3(grid), dim3(kThreads), 0, stream, tp, ntiles);
      else if (vl) hipLaunchKernelGGL((strided_tile_copy16_kernel<true, false>), dim3(grid), dim3(kThreads), 0, stream, tp, ntiles);
      else if (vs) hipLaunchKernelGGL((strided_tile_copy16_kernel<false, true>), dim3(grid), dim3(kThreads), 0, stream, tp, ntiles);
      if (vl || vs) return hipGetLastError();
    }
    switch (p.elem_size) {
      case 1: hipLaunchKernelGGL(strided_tile_copy_kernel<uint8_t>, dim3(grid), dim3(kThreads), 0, stream, tp, ntiles); break;
      case 2: hipLaunchKernelGGL(strided_tile_copy_kernel<uint16_t>, dim3(grid), dim3(kThreads), 0, stream, tp, ntiles); break;
      case 4: hipLaunchKernelGGL(strided_tile_copy_kernel<uint32_t>, dim3(grid), dim3(kThreads), 0, stream, tp, ntiles); break;
      case 8: hipLaunchKernelGGL(strided_tile_copy_kernel<uint64_t>, dim3(grid), dim3(kThreads), 0, stream, tp, ntiles); break;
      default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
  }

  const int grid = grid_for(n, kThreads * 2);
#define SC(E) do { \
    if (n < (int64_t)1 << 31) hipLaunchKernelGGL((strided_copy_kernel<E, uint32_t>), dim3(grid), dim3(kThreads), 0, stream, p, n); \
    else hipLaunchKernelGGL((strided_copy_kernel<E, int64_t>), dim3(grid), dim3(kThreads), 0, stream, p, n); \
  } while (0)
  switch (p.elem_size) {
    case 1: SC(uint8_t); break;
    case 2: SC(uint16_t); break;
    case 4: SC(uint32_t); break;
    case 8: SC(uint64_t); break;
    case 16: SC(b16); break;
    default: return hipErrorInvalidValue;
  }
#undef SC
  return hipGetLastError();
}

hipError_t launch_transpose2d(const void* x, void* y, int elem_size, int batch, int rows, int cols,
                              int dst_pitch, hipStream_t stream) {
  if (!x || !y || batch <= 0 || rows <= 0 || cols <= 0 || dst_pitch < rows) return hipErrorInvalidValue;
  if (elem_size == 2 && rows >= 16 && cols >= 16) {   // (the tiled strided copy has vector requests for this size)
    StridedCopyParams cp;
    cp.x = x; cp.y = y; cp.elem_size = 2; cp.rank = 3;
    cp.dims[0] = batch; cp.dims[1] = cols; cp.dims[2] = rows;
    cp.sy[0] = (int64_t)cols * dst_pitch; cp.sy[1] = dst_pitch; cp.sy[2] = 1;
    cp.sx[0] = (int64_t)rows * cols; cp.sx[1] = 1; cp.sx[2] = cols;
    return launch_strided_copy(cp, stream);
  }
  const int64_t ntiles = (int64_t)batch * ((rows + 63) / 64) * ((cols + 63) / 64);
  const int grid = (int)(ntiles < 65536 ? ntiles : 65536);
  switch (elem_size) {
    case 1: hipLaunchKernelGGL(transpose2d_kernel<uint8_t>, dim3(grid), dim3(kThreads), 0, stream, (const uint8_t*)x, (uint8_t*)y, batch, rows, cols, dst_pitch); break;
    case 2: hipLaunchKernelGGL(transpose2d_kernel<uint16_t>, dim3(grid), dim3(kThreads), 0, stream, (const uint16_t*)x, (uint16_t*)y, batch, rows, cols, dst_pitch); break;
    case 4: hipLaunchKernelGGL(transpose2d_kernel<uint32_t>, dim3(grid), dim3(kThreads), 0, stream, (const uint32_t*)x, (uint32_t*)y, batch, rows, cols, dst_pitch); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

hipError_t launch_resize_nearest_nhwc(const void* x, void* y, int elem_size, int N, int H, int W,
                                      int cs, int Ho, int Wo, hipStream_t stream) {
  if (!x || !y || N <= 0 || H <= 0 || W <= 0 || cs <= 0 || Ho <= 0 || Wo <= 0) return hipErrorInvalidValue;
  const int64_t row_bytes = (int64_t)cs * elem_size;
  const bool v16 = row_bytes % 16 == 0 && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15u) == 0;
  if (v16 && Ho % H == 0 && Wo % W == 0 && (int64_t)N * H < (1ll << 31) && (int64_t)W * (row_bytes / 16) < (1ll << 31)) {
    // (nearest: source index floor(o * in / out) = o / factor)
    const int cv = (int)(row_bytes / 16);
    const int64_t rows = (int64_t)N * H;
    const int64_t pieces = ((int64_t)W * cv + kThreads - 1) / kThreads;   // workgroups per source row
    hipLaunchKernelGGL(resize_nearest_whole_kernel<b16>,
                       dim3((unsigned)(rows < 65536 * 16 ? rows : 65536 * 16), (unsigned)(pieces < 64 ? pieces : 64)), dim3(kThreads), 0,
                       stream, (const b16*)x, (b16*)y, (int)rows, H, W, cv, Ho / H, Wo / W);
  } else if (v16) {
    const int cv = (int)(row_bytes / 16);
    const int grid = grid_for((int64_t)N * Ho * Wo * cv, kThreads * 2);
    hipLaunchKernelGGL(resize_nearest_kernel<b16>, dim3(grid), dim3(kThreads), 0, stream,
                       (const b16*)x, (b16*)y, N, H, W, cv, Ho, Wo);
  } else {
    const int grid = grid_for((int64_t)N * Ho * Wo * cs, kThreads * 2);
    switch (elem_size) {
      case 1: hipLaunchKernelGGL(resize_nearest_kernel<uint8_t>, dim3(grid), dim3(kThreads), 0, stream, (const uint8_t*)x, (uint8_t*)y, N, H, W, cs, Ho, Wo); break;
      case 2: hipLaunchKernelGGL(resize_nearest_kernel<uint16_t>, dim3(grid), dim3(kThreads), 0, stream, (const uint16_t*)x, (uint16_t*)y, N, H, W, cs, Ho, Wo); break;
      case 4: hipLaunchKernelGGL(resize_nearest_kernel<uint32_t>, dim3(grid), dim3(kThreads), 0, stream, (const uint32_t*)x, (uint32_t*)y, N, H, W, cs, Ho, Wo); break;
      default: return hipErrorInvalidValue;
    }
  }
  return hipGetLastError();
}

hipError_t launch_resize_linear_nhwc(const void* x, void* y, DType dt, int N, int H, int W, int cs,
                                     int Ho, int Wo, hipStream_t stream) {
  if (!x || !y || N <= 0 || H <= 0 || W <= 0 || cs <= 0 || Ho <= 0 || Wo <= 0) return hipErrorInvalidValue;
  const float fh = (float)H / (float)Ho, fw = (float)W / (float)Wo;
  const int es = dtype_size(dt);
  if (es == 0) return hipErrorInvalidValue;
  const int v = 16 / es;
  const bool vec = cs % v == 0 && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15u) == 0;
  const int grid = grid_for((int64_t)N * Ho * Wo * (vec ? cs / v : cs), kThreads);
#define RESIZE_LINEAR(T_)                                                                                          \
  do {                                                                                                             \
    if (vec)                                                                                                       \
      hipLaunchKernelGGL((resize_linear_kernel<T_, 16 / (int)sizeof(T_)>), dim3(grid), dim3(kThreads), 0, stream,  \
                         (const T_*)x, (T_*)y, N, H, W, cs, Ho, Wo, fh, fw);                                      \
    else                                                                                                           \
      hipLaunchKernelGGL((resize_linear_kernel<T_, 1>), dim3(grid), dim3(kThreads), 0, stream, (const T_*)x,       \
                         (T_*)y, N, H, W, cs, Ho, Wo, fh, fw);                                                     \
  } while (0)
  switch (dt) {
    case DT_F32: RESIZE_LINEAR(float); break;
    case DT_F16: RESIZE_LINEAR(f16_t); break;
    case DT_BF16: RESIZE_LINEAR(bf16_t); break;
    default: return hipErrorInvalidValue;
  }
#undef RESIZE_LINEAR
  return hipGetLastError();
}

hipError_t launch_gather_rows(const void* x, const void* idx, DType idx_dt, void* y, int64_t outer,
                              int64_t n_src_rows, int64_t n_idx, int64_t row_bytes,
                              hipStream_t stream) {
  if (!x || !idx || !y || outer <= 0 || n_src_rows <= 0 || n_idx <= 0 || row_bytes <= 0)
    return hipErrorInvalidValue;
  const uintptr_t al = reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y) | (uintptr_t)row_bytes;
  const int vec = (al % 16 == 0) ? 16 : (al % 4 == 0) ? 4 : (al % 2 == 0) ? 2 : 1;
  const int64_t total = outer * n_idx * (row_bytes / vec);
  const int grid = grid_for(total, kThreads * 2);
  if (idx_dt == DT_I32)
    hipLaunchKernelGGL(gather_rows_kernel<int32_t>, dim3(grid), dim3(kThreads), 0, stream,
                       (const unsigned char*)x, (const int32_t*)idx, (unsigned char*)y, outer,
                       n_src_rows, n_idx, row_bytes, vec);
  else if (idx_dt == DT_I64)
    hipLaunchKernelGGL(gather_rows_kernel<int64_t>, dim3(grid), dim3(kThreads), 0, stream,
                       (const unsigned char*)x, (const int64_t*)idx, (unsigned char*)y, outer,
                       n_src_rows, n_idx, row_bytes, vec);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}

}  // namespace ohip
