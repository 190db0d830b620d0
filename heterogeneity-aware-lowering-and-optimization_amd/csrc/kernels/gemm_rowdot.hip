// Matrix products with very few output columns and a long reduction (a softmax-regression
// or classifier head over a handful of rows: [64, 784] x [784, 10]): an MFMA tile would be
// nine tenths padding and ONE workgroup would walk the whole K dimension stage by stage
// (25 stages of fp32, one memory round trip each).  Here every output row is one wavefront:
// lane l takes the 16-byte pieces l, l + 64, .. of the row and of every weight row, all of
// a lane's requests are in flight together, and the partial sums meet in a wavefront
// reduction.  fp32 only (the summation order differs from the tiled kernels': within the
// fp32 bound, as theirs differ among themselves).  With every column of a row in one wavefront
// a Softmax / LogSoftmax over the columns is a few more instructions (IgemmParams::row_softmax).
#include <hip/hip_runtime.h>

#include <cstdlib>
#include <cstring>

#include "device_utils.h"
#include "kernels.h"

namespace ohip {
namespace {

template <int NB>
__global__ __launch_bounds__(64) void gemm_rowdot_kernel(const IgemmParams p) {
  const int m = blockIdx.x, lane = threadIdx.x;
  const float* x = reinterpret_cast<const float*>(p.x) + (int64_t)m * p.xcs;
  const float* w = reinterpret_cast<const float*>(p.w);
  float acc[NB];
#pragma unroll
  for (int n = 0; n < NB; ++n) acc[n] = 0.f;
  const int pieces = p.C >> 2;
  for (int k4 = lane; k4 < pieces; k4 += 64) {
    const floatx4 a = *reinterpret_cast<const floatx4*>(x + k4 * 4);
#pragma unroll
    for (int n = 0; n < NB; ++n) {
      // (columns past the last read the last one's weights: no branch around a request)
      const int nn = n < p.Kout ? n : p.Kout - 1;
      const floatx4 b = *reinterpret_cast<const floatx4*>(w + (int64_t)nn * p.w_rs + k4 * 4);
      acc[n] = __builtin_fmaf(a.x, b.x, acc[n]);
      acc[n] = __builtin_fmaf(a.y, b.y, acc[n]);
      acc[n] = __builtin_fmaf(a.z, b.z, acc[n]);
      acc[n] = __builtin_fmaf(a.w, b.w, acc[n]);
    }
  }
  // every lane receives every sum; lane n keeps column n
  float mine = 0.f;
#pragma unroll
  for (int n = 0; n < NB; ++n) {
    const float s = wave_sum(acc[n]);
    mine = lane == n ? s : mine;
  }
  const bool col = lane < p.Kout;
  const float b = col && p.bias ? reinterpret_cast<const float*>(p.bias)[lane] : 0.f;
  float v = __builtin_fmaf(mine, p.alpha, b);
  v = apply_act(v, p.act, p.act_a, p.act_b);
  if (p.row_softmax != 0) {
    // (wavefront-uniform)  the row's columns sit in lanes 0 .. Kout-1: maximum, exponentials and
    // their sum across the wavefront, the arithmetic of the stand-alone Softmax launch
    const float mx = wave_max(col ? v : -INFINITY);
    const float e = col ? expf(v - mx) : 0.f;
    const float sum = wave_sum(e);
    v = p.row_softmax == 2 ? (v - mx) - logf(sum) : e * (1.0f / sum);
  }
  if (col) reinterpret_cast<float*>(p.y)[(int64_t)m * p.ycs + lane] = v;
}

}  // namespace

bool gemm_rowdot_shape(const IgemmParams& p) {
  if (const char* e = getenv("ODLA_HIP_ROWDOT")) {  // tuning aid: 0 keeps these products on the tiled kernels
    if (e[0] == '0') return false;
  }
  if (const char* force = getenv("ODLA_HIP_IGEMM_TILE")) {
    if (force[0] != 0) return false;
  }
  if (p.in_dt != DT_F32 || p.out_dt != DT_F32) return false;
  if (p.R != 1 || p.S != 1 || p.sh != 1 || p.sw != 1 || p.ph != 0 || p.pw != 0 || p.batch != 1) return false;
  if (p.Ho != p.H || p.Wo != p.W) return false;
  if (p.residual != nullptr || p.y_rdiv > 0 || p.y_zdiv > 0 || p.qmul != nullptr) return false;
  const int64_t M = (int64_t)p.N * p.Ho * p.Wo;
  // few columns, a reduction of at least eight 128-byte stages, and no more rows than keep the
  // weights' re-reads (once per row, out of L2) below the tiled kernel's single pass
  if (p.Kout < 1 || p.Kout > 16 || p.C < 256 || M < 1 || M > 4096) return false;
  if (p.C % 4 != 0 || p.xcs % 4 != 0 || p.w_rs % 4 != 0 || p.w_rs < p.C || p.xcs < p.C || p.ycs < p.Kout) return false;
  return true;
}

hipError_t launch_gemm_rowdot(const IgemmParams& p, hipStream_t stream) {
  auto al16 = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15u) == 0; };
  if (!gemm_rowdot_shape(p) || p.x == nullptr || p.w == nullptr || p.y == nullptr || !al16(p.x) || !al16(p.w))
    return hipErrorInvalidValue;
  const dim3 grid((unsigned)((int64_t)p.N * p.Ho * p.Wo)), block(64);
  if (p.Kout <= 4) hipLaunchKernelGGL(gemm_rowdot_kernel<4>, grid, block, 0, stream, p);
  else if (p.Kout <= 8) hipLaunchKernelGGL(gemm_rowdot_kernel<8>, grid, block, 0, stream, p);
  else hipLaunchKernelGGL(gemm_rowdot_kernel<16>, grid, block, 0, stream, p);
  return hipGetLastError();
}

}  // namespace ohip
