/*
 * CPU oracle kernels for the ODLA hot path -- TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C restatement of the arithmetic the reference CPU backend
 * (ODLA/platforms/dnnl) performs for the heavy operators, used to check the
 * GPU library and as the timed CPU baseline.  Nothing in the shipped library
 * links or calls this file.
 *
 * Layouts follow the ODLA ABI: activations N,C,H,W, kernels O,I/g,R,S, all
 * row-major.  OpenMP parallelises over (image, output channel).
 *
 *   odla_ref_conv2d_f32   [ref: ODLA/platforms/dnnl/odla_dnnl.cc:1014-1129]
 *       direct cross-correlation with groups, strides, dilations, asymmetric
 *       zero padding and optional bias; fp32 multiply-add accumulated in fp32.
 *   odla_ref_pool2d_f32   [ref: odla_dnnl.cc:1360-1446]
 *       max / average pooling; the average divides by the number of in-bounds
 *       elements unless count_include_pad is set.
 *   odla_ref_conv2d_q8    parity unpinned by the reference (it has no int8
 *       convolution of its own; oneDNN would supply it).  Defines the int8
 *       plan: u8 activations with zero point, s8 weights, exact int32
 *       accumulation of (x - zp_x) * w, plus int32 bias.
 *   odla_ref_requant_q8   the requantisation: one fused multiply-add of the
 *       int32 accumulator with a per-channel multiplier and the zero point (or
 *       the rescaled residual), lower clamp, round-half-even, saturate.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#if defined(_OPENMP)
#include <omp.h>
#endif

int odla_ref_num_threads(void) {
#if defined(_OPENMP)
  return omp_get_max_threads();
#else
  return 1;
#endif
}

void odla_ref_conv2d_f32(const float* x, const float* w, const float* bias, float* y, int N, int C,
                         int H, int W, int O, int R, int S, int group, int sh, int sw, int dh, int dw,
                         int pt, int pl, int Ho, int Wo) {
  const int Cg = C / group, Og = O / group;
#pragma omp parallel for collapse(2) schedule(static)
  for (int n = 0; n < N; ++n) {
    for (int o = 0; o < O; ++o) {
      const int g = o / Og;
      float* yo = y + ((size_t)n * O + o) * Ho * Wo;
      const float b = bias ? bias[o] : 0.f;
      for (int i = 0; i < Ho * Wo; ++i) yo[i] = 0.f;
      for (int c = 0; c < Cg; ++c) {
        const float* xc = x + ((size_t)n * C + g * Cg + c) * H * W;
        const float* wc = w + (((size_t)o * Cg + c) * R) * S;
        for (int r = 0; r < R; ++r) {
          for (int s = 0; s < S; ++s) {
            const float wv = wc[r * S + s];
            /* output columns whose input column is in range */
            for (int ho = 0; ho < Ho; ++ho) {
              const int hi = ho * sh - pt + r * dh;
              if (hi < 0 || hi >= H) continue;
              const float* xr = xc + (size_t)hi * W;
              float* yr = yo + (size_t)ho * Wo;
              const int off = s * dw - pl;
              int wo0 = 0;
              while (wo0 < Wo && wo0 * sw + off < 0) ++wo0;
              int wo1 = Wo;
              while (wo1 > wo0 && (wo1 - 1) * sw + off >= W) --wo1;
              if (sw == 1) {
                for (int wo = wo0; wo < wo1; ++wo) yr[wo] += wv * xr[wo + off];
              } else {
                for (int wo = wo0; wo < wo1; ++wo) yr[wo] += wv * xr[wo * sw + off];
              }
            }
          }
        }
      }
      if (bias)
        for (int i = 0; i < Ho * Wo; ++i) yo[i] += b;
    }
  }
}

void odla_ref_pool2d_f32(const float* x, float* y, int N, int C, int H, int W, int kh, int kw, int sh,
                         int sw, int pt, int pl, int Ho, int Wo, int is_max, int count_include_pad) {
#pragma omp parallel for collapse(2) schedule(static)
  for (int n = 0; n < N; ++n) {
    for (int c = 0; c < C; ++c) {
      const float* xc = x + ((size_t)n * C + c) * H * W;
      float* yc = y + ((size_t)n * C + c) * Ho * Wo;
      for (int ho = 0; ho < Ho; ++ho) {
        for (int wo = 0; wo < Wo; ++wo) {
          float acc = is_max ? -INFINITY : 0.f;
          int cnt = 0;
          for (int r = 0; r < kh; ++r) {
            const int hi = ho * sh - pt + r;
            if (hi < 0 || hi >= H) continue;
            for (int s = 0; s < kw; ++s) {
              const int wi = wo * sw - pl + s;
              if (wi < 0 || wi >= W) continue;
              const float v = xc[(size_t)hi * W + wi];
              if (is_max) acc = v > acc ? v : acc; else acc += v;
              ++cnt;
            }
          }
          if (!is_max) acc /= (float)(count_include_pad ? kh * kw : (cnt > 0 ? cnt : 1));
          yc[(size_t)ho * Wo + wo] = acc;
        }
      }
    }
  }
}

/* acc[n][o][ho][wo] = bias[o] + sum (x[n][c][hi][wi] - zp_x) * w[o][c][r][s], out-of-bounds taps
 * contribute 0.  Exact in int32 as long as |acc| < 2^31 (K * 255 * 127 < 2^31 for K < 66k). */
void odla_ref_conv2d_q8(const uint8_t* x, int zp_x, const int8_t* w, const int32_t* bias, int32_t* acc,
                        int N, int C, int H, int W, int O, int R, int S, int sh, int sw, int pt, int pl,
                        int Ho, int Wo) {
  /* (x - zp_x) once, as int16: the loops below then run on plain multiply-adds */
  const size_t nx = (size_t)N * C * H * W;
  int16_t* xs = (int16_t*)malloc(nx * sizeof(int16_t) + 64);
  if (xs == NULL) return;
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < nx; ++i) xs[i] = (int16_t)((int)x[i] - zp_x);
#pragma omp parallel for collapse(2) schedule(static)
  for (int n = 0; n < N; ++n) {
    for (int o = 0; o < O; ++o) {
      int32_t* yo = acc + ((size_t)n * O + o) * Ho * Wo;
      const int32_t b = bias ? bias[o] : 0;
      for (int i = 0; i < Ho * Wo; ++i) yo[i] = b;
      if (R == 1 && S == 1 && sh == 1 && sw == 1 && pt == 0 && pl == 0 && Ho == H && Wo == W) {
        /* 1x1 filters: the whole image is one contiguous run */
        const int hw = H * W;
        for (int c = 0; c < C; ++c) {
          const int16_t* xc = xs + ((size_t)n * C + c) * hw;
          const int32_t wv = w[(size_t)o * C + c];
          if (wv == 0) continue;
          for (int i = 0; i < hw; ++i) yo[i] += wv * (int32_t)xc[i];
        }
        continue;
      }
      for (int c = 0; c < C; ++c) {
        const int16_t* xc = xs + ((size_t)n * C + c) * H * W;
        const int8_t* wc = w + (((size_t)o * C + c) * R) * S;
        for (int r = 0; r < R; ++r) {
          for (int s = 0; s < S; ++s) {
            const int32_t wv = wc[r * S + s];
            if (wv == 0) continue;
            for (int ho = 0; ho < Ho; ++ho) {
              const int hi = ho * sh - pt + r;
              if (hi < 0 || hi >= H) continue;
              const int16_t* xr = xc + (size_t)hi * W;
              int32_t* yr = yo + (size_t)ho * Wo;
              const int off = s - pl;
              int wo0 = 0;
              while (wo0 < Wo && wo0 * sw + off < 0) ++wo0;
              int wo1 = Wo;
              while (wo1 > wo0 && (wo1 - 1) * sw + off >= W) --wo1;
              if (sw == 1) {
                for (int wo = wo0; wo < wo1; ++wo) yr[wo] += wv * (int32_t)xr[wo + off];
              } else {
                for (int wo = wo0; wo < wo1; ++wo) yr[wo] += wv * (int32_t)xr[wo * sw + off];
              }
            }
          }
        }
      }
    }
  }
  free(xs);
}

/* Requantisation of the int8 plan, per channel o; acc (int32 accumulator plus
 * int32 bias) is [N][O][HW]:
 *   q = sat8(max(fma((float)acc, mul[o], add), lo))
 * where `add` is the zero point of the result, or, with a residual r (levels of
 * an 8-bit tensor of the same shape), add = fma((float)r, r_mul, r_add) per
 * element.  fma is ONE fused multiply-add in binary32 (a single rounding: fmaf);
 * sat8 rounds to the nearest integer, ties to even, and saturates to [0, 255]. */
void odla_ref_requant_q8(const int32_t* acc, const float* mul, float add, float lo, const uint8_t* res,
                         float r_mul, float r_add, uint8_t* q, int N, int O, int HW) {
#pragma omp parallel for collapse(2) schedule(static)
  for (int n = 0; n < N; ++n) {
    for (int o = 0; o < O; ++o) {
      const size_t base = ((size_t)n * O + o) * HW;
      const float m = mul[o];
      for (int i = 0; i < HW; ++i) {
        const float a = res ? fmaf((float)res[base + i], r_mul, r_add) : add;
        float f = fmaf((float)acc[base + i], m, a);
        f = f > lo ? f : lo;
        float r = nearbyintf(f);
        r = r < 0.f ? 0.f : (r > 255.f ? 255.f : r);
        q[base + i] = (uint8_t)r;
      }
    }
  }
}
