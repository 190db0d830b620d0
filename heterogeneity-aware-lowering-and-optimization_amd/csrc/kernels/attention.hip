// One-launch attention for short sequences on gfx950:
//
//   out[b, h] = softmax(scale * q[b, h] . k[b, h]^T + mask[b]) . v[b, h]
//
// for 16-bit operands (bf16 / fp16), head size 64 and up to 128 keys - the block
// that an encoder layer otherwise runs as matrix product, Softmax, transposition
// of v and matrix product, each with its own pass over a [B, heads, S, S] tensor
// [ref: the reference compiler matches the same block as one instruction,
//  lib/transforms/fusion.cc:315-348].
//
// One workgroup per (batch, head), one wavefront per 32 queries.  k goes through
// LDS once (rows padded to 144 bytes), v is transposed on its way into LDS, q
// comes straight from global memory into MFMA operand registers.
//   scores  C[key][query] = k . q^T  (v_mfma_f32_32x32x16): a lane then holds, for
//           ITS query, 16 keys of every 32-key block, so the Softmax over the keys
//           is a reduction inside the lane plus one exchange with lane + 32;
//           scores, mask and exponentials stay fp32 in registers;
//   context C[dv][query] = v^T . p^T: the probabilities a lane holds are packed to
//           the operand type as they are - the order of the keys inside one MFMA
//           is free as long as v^T is stored in the same order, which the
//           transposing LDS write takes care of (slot_of_key);
//   result  rows of 64 values leave as 16-byte vectors formed by exchanging
//           dwords between lanes l and l + 32 (v_permlane32_swap).
#include "igemm_common.h"

#include <cstdlib>

namespace ohip {

namespace {

constexpr int kAttnD = 64;            // head size
constexpr int kKPitch = 144;          // bytes per staged k row (128 + 16: conflict-free 16-byte fragment reads)
constexpr int kVPitch = 272;          // bytes per staged v^T row (128 keys x 2 + 16)

__device__ __forceinline__ void swap32f(float& x, float& y) {
#if defined(__HIP_DEVICE_COMPILE__)
  const uintx2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(y), false, false);
  x = __uint_as_float(r.x);
  y = __uint_as_float(r.y);
#endif
}
__device__ __forceinline__ void swap32u(unsigned& x, unsigned& y) {
#if defined(__HIP_DEVICE_COMPILE__)
  const uintx2 r = __builtin_amdgcn_permlane32_swap(x, y, false, false);
  x = r.x;
  y = r.y;
#endif
}
// the value of the partner lane (l ^ 32) combined with the own one
__device__ __forceinline__ float pair_max(float v) {
  float x = v, y = v;
  swap32f(x, y);   // x = [v.lo | v.lo], y = [v.hi | v.hi]
  return fmaxf(x, y);
}
__device__ __forceinline__ float pair_sum(float v) {
  float x = v, y = v;
  swap32f(x, y);
  return x + y;
}

// Position of key (0 .. 127) inside a staged v^T row.  In the score layout a lane of half
// s holds keys kb*32 + q*8 + s*4 + r; the context product consumes, per step (kb, h), the
// lane's groups q = 2h and 2h + 1, so those eight keys sit next to each other:
// slot = kb*32 + h*16 + s*8 + (q & 1)*4 + r.
__device__ __forceinline__ int slot_of_key(const int key) {
  const int kb = key >> 5, q = (key >> 3) & 3, s = (key >> 2) & 1, r = key & 3;
  return kb * 32 + (q >> 1) * 16 + s * 8 + (q & 1) * 4 + r;
}

template <typename T, int NKB>   // NKB: 32-key blocks (S = 32 NKB); NKB wavefronts
__global__ void __launch_bounds__(NKB * 64, 2)
attention_kernel(const AttentionParams p) {
  constexpr int S = NKB * 32, NT = NKB * 64;
  __shared__ __attribute__((aligned(16))) unsigned char smem[S * kKPitch + kAttnD * kVPitch + S * 4];
  unsigned char* ks = smem;
  unsigned char* vts = smem + S * kKPitch;
  float* ms = reinterpret_cast<float*>(smem + S * kKPitch + kAttnD * kVPitch);

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int l32 = lane & 31, lg = lane >> 5;
  const int b = blockIdx.x / p.heads, h = blockIdx.x % p.heads;
  const T* q = reinterpret_cast<const T*>(p.q) + (int64_t)b * p.q_bs + (int64_t)h * p.q_hs;
  const T* k = reinterpret_cast<const T*>(p.k) + (int64_t)b * p.k_bs + (int64_t)h * p.k_hs;
  const T* v = reinterpret_cast<const T*>(p.v) + (int64_t)b * p.v_bs + (int64_t)h * p.v_hs;

  // ---- this lane's piece of the query operand: d values [16 kk + 8 lg, +8) of its query
  uintx4 qf[4];
  {
    const uintx4* row = reinterpret_cast<const uintx4*>(q + (int64_t)(wave * 32 + l32) * p.q_rs) + lg;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) qf[kk] = row[2 * kk];
  }
  // ---- stage k (rows of 128 bytes, padded) and v^T (keys in slot order), the mask as fp32
  {
    const int c = tid & 7;   // 16-byte chunk of the row
#pragma unroll
    for (int i = 0; i < S * 8 / NT; ++i) {
      const int row = (tid >> 3) + i * (NT / 8);
      const uintx4 kv = *(reinterpret_cast<const uintx4*>(k + (int64_t)row * p.k_rs) + c);
      *reinterpret_cast<uintx4*>(ks + row * kKPitch + c * 16) = kv;
      const uintx4 vv = *(reinterpret_cast<const uintx4*>(v + (int64_t)row * p.v_rs) + c);
      const unsigned w[4] = {vv.x, vv.y, vv.z, vv.w};
      unsigned char* dst = vts + slot_of_key(row) * 2;
#pragma unroll
      for (int e = 0; e < 8; ++e)
        *reinterpret_cast<unsigned short*>(dst + (c * 8 + e) * kVPitch) = (unsigned short)(w[e >> 1] >> (16 * (e & 1)));
    }
    for (int j = tid; j < S; j += NT) {
      float m = 0.f;
      if (p.mask != nullptr) {
        if (p.mask_dt == DT_F32) m = reinterpret_cast<const float*>(p.mask)[(int64_t)b * p.mask_bs + j];
        else m = Store<T>::ld(reinterpret_cast<const T*>(p.mask) + (int64_t)b * p.mask_bs + j);
      }
      ms[j] = m;
    }
  }
  __syncthreads();

  // ---- scores: acc[kb][q*4 + r] = k[kb*32 + q*8 + lg*4 + r] . q[query]
  floatx16 acc[NKB];
#pragma unroll
  for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[kb][e] = 0.f;
#pragma unroll
  for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      const uintx4 a = *reinterpret_cast<const uintx4*>(ks + (kb * 32 + l32) * kKPitch + kk * 32 + lg * 16);
      acc[kb] = Mma<T>::run(a, qf[kk], acc[kb]);
    }
  // ---- Softmax over the keys of this lane's query (fp32)
  float mx = -INFINITY;
#pragma unroll
  for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
    for (int qq = 0; qq < 4; ++qq) {
      const floatx4 m4 = *reinterpret_cast<const floatx4*>(ms + kb * 32 + qq * 8 + lg * 4);
      acc[kb][qq * 4 + 0] = __builtin_fmaf(acc[kb][qq * 4 + 0], p.scale, m4.x);
      acc[kb][qq * 4 + 1] = __builtin_fmaf(acc[kb][qq * 4 + 1], p.scale, m4.y);
      acc[kb][qq * 4 + 2] = __builtin_fmaf(acc[kb][qq * 4 + 2], p.scale, m4.z);
      acc[kb][qq * 4 + 3] = __builtin_fmaf(acc[kb][qq * 4 + 3], p.scale, m4.w);
#pragma unroll
      for (int r = 0; r < 4; ++r) mx = fmaxf(mx, acc[kb][qq * 4 + r]);
    }
  mx = pair_max(mx);
  float sum = 0.f;
#pragma unroll
  for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      // (the result keeps 8 or 11 significant bits: the hardware exponential, 1 ulp, stands in for the library's)
      const float ex = __expf(acc[kb][e] - mx);
      acc[kb][e] = ex;
      sum += ex;
    }
  sum = pair_sum(sum);
  const float inv = 1.0f / sum;

  // ---- context: o[dvb][q*4 + r] = sum over keys p[key] * v[key][dvb*32 + q*8 + lg*4 + r]
  floatx16 o[2];
#pragma unroll
  for (int dvb = 0; dvb < 2; ++dvb)
#pragma unroll
    for (int e = 0; e < 16; ++e) o[dvb][e] = 0.f;
#pragma unroll
  for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) {
      float pv[8];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        pv[r] = acc[kb][(2 * hh) * 4 + r] * inv;
        pv[4 + r] = acc[kb][(2 * hh + 1) * 4 + r] * inv;
      }
      const uintx4 pf = pack8_rne<T>(pv);
#pragma unroll
      for (int dvb = 0; dvb < 2; ++dvb) {
        const uintx4 a = *reinterpret_cast<const uintx4*>(vts + (dvb * 32 + l32) * kVPitch + (kb * 32 + hh * 16 + lg * 8) * 2);
        o[dvb] = Mma<T>::run(a, pf, o[dvb]);
      }
    }

  // ---- result rows: lane (query, lg) holds, per 32-value block, the groups (q, lg) of four
  // values; after the exchange lg = 0 holds values 0 .. 15 of the block and lg = 1 16 .. 31.
  T* orow = reinterpret_cast<T*>(p.out) + (int64_t)b * p.o_bs + (int64_t)h * p.o_hs + (int64_t)(wave * 32 + l32) * p.o_rs;
#pragma unroll
  for (int dvb = 0; dvb < 2; ++dvb) {
    unsigned g[4][2];   // group q as two dwords (four 16-bit values)
#pragma unroll
    for (int qq = 0; qq < 4; ++qq) {
      float f[8] = {o[dvb][qq * 4 + 0], o[dvb][qq * 4 + 1], o[dvb][qq * 4 + 2], o[dvb][qq * 4 + 3], 0.f, 0.f, 0.f, 0.f};
      const uintx4 pk = pack8_rne<T>(f);
      g[qq][0] = pk.x;
      g[qq][1] = pk.y;
    }
    // swap32(x = group q0, y = group q2): x' = [(q0, 0) | (q2, 0)], y' = [(q0, 1) | (q2, 1)]
#pragma unroll
    for (int w = 0; w < 2; ++w) {
      swap32u(g[0][w], g[2][w]);
      swap32u(g[1][w], g[3][w]);
    }
    // now, for lg = 0: g[0] = (q0,0), g[2] = (q0,1), g[1] = (q1,0), g[3] = (q1,1): values 0 .. 15;
    // for lg = 1 the same registers hold q2 and q3: values 16 .. 31
    uintx4* dst = reinterpret_cast<uintx4*>(orow + dvb * 32 + lg * 16);
    dst[0] = uintx4{g[0][0], g[0][1], g[2][0], g[2][1]};
    dst[1] = uintx4{g[1][0], g[1][1], g[3][0], g[3][1]};
  }
}

}  // namespace

bool attention_supported(const AttentionParams& p) {
  if (const char* off = getenv("ODLA_HIP_FUSED_ATTENTION")) {   // tuning / test aid: "0" turns the kernel off
    if (off[0] == '0') return false;
  }
  if (p.dt != DT_BF16 && p.dt != DT_F16) return false;
  if (p.d != kAttnD || p.S < 32 || p.S > 128 || p.S % 32 != 0) return false;
  if (p.B <= 0 || p.heads <= 0 || (int64_t)p.B * p.heads > 0x7fffffff) return false;
  if (p.mask_dt != p.dt && p.mask_dt != DT_F32) return false;
  // rows and bases allow 16-byte accesses
  auto ok8 = [](int64_t s) { return s % 8 == 0; };
  if (!ok8(p.q_bs) || !ok8(p.q_hs) || !ok8(p.q_rs) || !ok8(p.k_bs) || !ok8(p.k_hs) || !ok8(p.k_rs) || !ok8(p.v_bs) ||
      !ok8(p.v_hs) || !ok8(p.v_rs) || !ok8(p.o_bs) || !ok8(p.o_hs) || !ok8(p.o_rs))
    return false;
  return true;
}

hipError_t launch_attention(const AttentionParams& p, hipStream_t stream) {
  if (!attention_supported(p) || p.q == nullptr || p.k == nullptr || p.v == nullptr || p.out == nullptr)
    return hipErrorInvalidValue;
  auto al16 = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15u) == 0; };
  if (!al16(p.q) || !al16(p.k) || !al16(p.v) || !al16(p.out)) return hipErrorInvalidValue;
  const dim3 grid((unsigned)(p.B * p.heads));
  const int nkb = p.S / 32;
#define ATTN_CASE(T_, NKB_)                                                                                \
  if (nkb == NKB_) {                                                                                       \
    hipLaunchKernelGGL((attention_kernel<T_, NKB_>), grid, dim3(NKB_ * 64), 0, stream, p);                 \
    return hipGetLastError();                                                                              \
  }
  if (p.dt == DT_BF16) {
    ATTN_CASE(bf16_t, 1) ATTN_CASE(bf16_t, 2) ATTN_CASE(bf16_t, 3) ATTN_CASE(bf16_t, 4)
  } else {
    ATTN_CASE(f16_t, 1) ATTN_CASE(f16_t, 2) ATTN_CASE(f16_t, 3) ATTN_CASE(f16_t, 4)
  }
#undef ATTN_CASE
  return hipErrorInvalidValue;
}

}  // namespace ohip
