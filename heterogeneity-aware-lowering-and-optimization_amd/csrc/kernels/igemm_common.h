// Device code shared by the implicit-GEMM kernels (igemm.hip, igemm_big.hip):
// the MFMA wrappers per operand type, the fused epilogues and the per-wavefront
// epilogue that stages accumulators through LDS for vector stores.
#ifndef ODLA_HIP_IGEMM_COMMON_H_
#define ODLA_HIP_IGEMM_COMMON_H_

#include "device_utils.h"

#include <type_traits>

namespace ohip {

// Element offset of result row m / column n / problem z (see IgemmParams::y_rdiv, y_zdiv).
__device__ __forceinline__ int64_t y_row_off(const IgemmParams& p, const int m) {
  if (p.y_rdiv > 0) {
    const int a = fast_div(m, p.yr_magic, p.yr_shift);
    return (int64_t)a * p.y_rhi + (int64_t)(m - a * p.y_rdiv) * p.y_rlo;
  }
  return (int64_t)m * p.ycs;
}
__device__ __forceinline__ int64_t y_col_off(const IgemmParams& p, const int n) {
  if (p.y_rdiv > 0) {
    const int c = fast_div(n, p.yc_magic, p.yc_shift);
    return (int64_t)c * p.y_chi + (int64_t)(n - c * p.y_cdiv);
  }
  return n;
}
__device__ __forceinline__ int64_t y_batch_off(const IgemmParams& p, const int z) {
  if (p.y_zdiv > 0) return (int64_t)(z / p.y_zdiv) * p.y_bs_hi + (int64_t)(z % p.y_zdiv) * p.y_bs;
  return (int64_t)z * p.y_bs;
}

template <typename T> struct Mma;
template <> struct Mma<float> {
  using Acc = floatx16;
  __device__ static __forceinline__ Acc run(uintx4 a, uintx4 b, Acc c) {
    // 16 bytes = 4 k values per lane; 32x32x2 consumes one per lane group.
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.x), __uint_as_float(b.x), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.y), __uint_as_float(b.y), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.z), __uint_as_float(b.z), c, 0, 0, 0);
    c = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.w), __uint_as_float(b.w), c, 0, 0, 0);
    return c;
  }
};
template <> struct Mma<f16_t> {
  using Acc = floatx16;
  __device__ static __forceinline__ Acc run(uintx4 a, uintx4 b, Acc c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(halfx8, a),
                                                  __builtin_bit_cast(halfx8, b), c, 0, 0, 0);
  }
};
template <> struct Mma<bf16_t> {
  using Acc = floatx16;
  __device__ static __forceinline__ Acc run(uintx4 a, uintx4 b, Acc c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  }
};
template <> struct Mma<int8_t> {
  using Acc = intx16;
  __device__ static __forceinline__ Acc run(uintx4 a, uintx4 b, Acc c) {
    return __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(intx4, a),
                                                 __builtin_bit_cast(intx4, b), c, 0, 0, 0);
  }
};

// ---------------------------------------------------------------------------
// Epilogues.  Each handles eight consecutive output channels n..n+7 of one
// output row; yrow / rrow / bias already point at channel n.  `vec` says all
// eight are valid and the row pointers allow one vector access.

// Only the cheap activations are fused (a full transcendental switch inlined
// per element bloats the epilogue until the compiler stops unrolling it and
// the accumulators fall out of registers); the planner keeps the others as a
// separate streaming kernel.
__device__ __forceinline__ float epi_act(float v, ActKind act, float a, float b) {
  switch (act) {
    case ACT_RELU: return v > 0.f ? v : 0.f;
    case ACT_LEAKY: return v > 0.f ? v : a * v;
    case ACT_CLAMP: return fminf(fmaxf(v, a), b);
    default: return v;
  }
}
// Eight values at once: the (wavefront-uniform) switch is taken once, not per
// element - per element it compiles to a tree of scalar branches that costs
// more than the arithmetic of the whole epilogue.
template <bool kRich = false>
__device__ __forceinline__ void epi_act8(float (&v)[8], ActKind act, float a, float b) {
  if constexpr (kRich) {
    // Variant with the transcendental activations (GELU behind a feed-forward
    // GEMM, Sigmoid / Tanh gates): a separate instantiation, so that the common
    // epilogue stays small.
    // (one element after the other: interleaving eight polynomial evaluations
    // would take the registers the accumulators of the other slices live in)
    switch (act) {
      case ACT_GELU_ERF:
#pragma unroll
        for (int e = 0; e < 8; ++e) { v[e] = gelu_erf(v[e]); __builtin_amdgcn_sched_barrier(0); }
        return;
      case ACT_GELU_TANH:
#pragma unroll
        for (int e = 0; e < 8; ++e) { v[e] = gelu_tanh(v[e]); __builtin_amdgcn_sched_barrier(0); }
        return;
      case ACT_SIGMOID:
#pragma unroll
        for (int e = 0; e < 8; ++e) { v[e] = 1.0f / (1.0f + expf(-v[e])); __builtin_amdgcn_sched_barrier(0); }
        return;
      case ACT_TANH:
#pragma unroll
        for (int e = 0; e < 8; ++e) { v[e] = tanhf(v[e]); __builtin_amdgcn_sched_barrier(0); }
        return;
      default: break;
    }
  }
  switch (act) {
    case ACT_RELU:
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = v[e] > 0.f ? v[e] : 0.f;
      break;
    case ACT_LEAKY:
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = v[e] > 0.f ? v[e] : a * v[e];
      break;
    case ACT_CLAMP:
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = fminf(fmaxf(v[e], a), b);
      break;
    default: break;
  }
}

template <typename TOut, bool kRich = false>
struct EpiFloat {
  using AccE = float;
  using RVec = uintx4;  // eight 2-byte residual elements fetched ahead of use
  static constexpr bool kPrefetchResidual = sizeof(TOut) == 2;
  // b8: this lane's eight bias values (zero when absent); rpre: residual vector
  // fetched ahead (valid when have_rpre), otherwise r points at the residual row.
  __device__ static __forceinline__ void store8(const IgemmParams& p, const float* acc, int nvalid, bool vec,
                                                const float* b8, const float*, TOut* y, const TOut* r,
                                                bool have_rpre, RVec rpre) {
    float v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = __builtin_fmaf(acc[e], p.alpha, b8[e]);
    // the activation comes before the residual in networks whose shortcut joins
    // an already activated branch, behind it in the ResNet order
    if (p.res_after_act) epi_act8<kRich>(v, p.act, p.act_a, p.act_b);
    if (vec) {
      if (r != nullptr) {
        if constexpr (sizeof(TOut) == 4) {
          const floatx4 r0 = *reinterpret_cast<const floatx4*>(r);
          const floatx4 r1 = *reinterpret_cast<const floatx4*>(r + 4);
          v[0] += r0.x; v[1] += r0.y; v[2] += r0.z; v[3] += r0.w;
          v[4] += r1.x; v[5] += r1.y; v[6] += r1.z; v[7] += r1.w;
        } else {
          // (both callers request the vector ahead whenever this branch is taken: vec, a
          //  residual and a 2-byte result.  A load here, even on a path never taken, would make
          //  the compiler wait for every store in flight where the paths join.)
          Vec16<TOut> rv;
          (void)have_rpre;
          rv.raw = rpre;
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] += rv.get(e);
        }
      }
      if (!p.res_after_act) epi_act8<kRich>(v, p.act, p.act_a, p.act_b);
      if constexpr (sizeof(TOut) == 4) {
        *reinterpret_cast<floatx4*>(y) = (floatx4){v[0], v[1], v[2], v[3]};
        *reinterpret_cast<floatx4*>(y + 4) = (floatx4){v[4], v[5], v[6], v[7]};
      } else {
        Vec16<TOut> o;
        o.raw = pack8_rne<TOut>(v);
        // (not in the instantiations with the wider activation set: they have no registers to spare)
        if (!kRich && p.stream_out) {
          // The pointer passes through an empty asm so that the optimizer cannot
          // fold this store and the plain one below into one plain store.
          uintx4* yv = reinterpret_cast<uintx4*>(y);
          asm volatile("" : "+v"(yv));
          __builtin_nontemporal_store(o.raw, (__attribute__((address_space(1))) uintx4*)yv);
        } else {
          o.store(y);
        }
      }
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (e < nvalid && r != nullptr) v[e] += Store<TOut>::ld(r + e);
      if (!p.res_after_act) epi_act8<kRich>(v, p.act, p.act_a, p.act_b);
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (e < nvalid) Store<TOut>::st(y + e, v[e]);
    }
  }
};

// int8 operands, int32 accumulators.  MODE 0: requantised 8-bit output (stored
// q-128), MODE 1: dequantised fp32 output, MODE 2: raw int32 accumulators.
template <int MODE> struct QuantOut;
template <> struct QuantOut<0> { using T = int8_t; };
template <> struct QuantOut<1> { using T = float; };
template <> struct QuantOut<2> { using T = int; };

template <int MODE>
struct EpiQuant {
  using AccE = int;
  using TOut = typename QuantOut<MODE>::T;
  using RVec = uintx2;
  static constexpr bool kPrefetchResidual = false;
  // MODE 1 / 2 only (the accumulators already hold the int32 bias); requantised
  // 8-bit output goes through igemm_epilogue_q8 / igemm_epilogue_rows128_q8.
  __device__ static __forceinline__ void store8(const IgemmParams& p, const int* acc, int nvalid, bool,
                                                const int*, const float* m8, TOut* y, const TOut* r,
                                                bool, RVec) {
    if constexpr (MODE == 2) {
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (e < nvalid) y[e] = acc[e];
    } else if constexpr (MODE == 1) {
      float f[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        f[e] = (float)acc[e] * m8[e];
        if (e < nvalid && r != nullptr) f[e] += r[e];
      }
      epi_act8(f, p.act, p.act_a, p.act_b);
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (e < nvalid) y[e] = f[e];
    }
  }
};

template <typename Epi> struct EpiTraits;
template <typename T, bool R> struct EpiTraits<EpiFloat<T, R>> { using TOut = T; static constexpr bool quant = false; static constexpr bool rich = R; };
template <int M> struct EpiTraits<EpiQuant<M>> { using TOut = typename QuantOut<M>::T; static constexpr bool quant = true; static constexpr bool rich = false; };

// ---------------------------------------------------------------------------
// 8-bit layers keep their int32 bias in the accumulators from the start: element
// q*4 + r of a lane's 32 x 32 block is channel q*8 + (lane/32)*4 + r.  n0 is the
// first channel of the wavefront's blocks (wavefront-uniform, so these are
// scalar loads and no vector-memory operation is left in flight).
template <int TM, int TN>
__device__ __forceinline__ void acc_init_bias(const IgemmParams& p, const int z, const int n0, const int lg,
                                              intx16 (&acc)[TM][TN]) {
  if (p.bias == nullptr) return;
  const int* bias = reinterpret_cast<const int*>(p.bias) + (int64_t)z * p.bias_bs;
  const int last = p.Kout - 1;  // channels past the end are computed but never stored
#pragma unroll
  for (int j = 0; j < TN; ++j)
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int c0 = n0 + j * 32 + q * 8 + r, c1 = c0 + 4;
        const int b0 = bias[c0 < last ? c0 : last], b1 = bias[c1 < last ? c1 : last];
        const int b = lg ? b1 : b0;
#pragma unroll
        for (int i = 0; i < TM; ++i) acc[i][j][q * 4 + r] = b;
      }
}

// The same through 16-byte vector loads (a lane's four channels of a block are
// consecutive): for kernels whose vector-memory waits the compiler manages.
template <int TM, int TN>
__device__ __forceinline__ void acc_init_bias_vec(const IgemmParams& p, const int z, const int n0, const int lg,
                                                  intx16 (&acc)[TM][TN]) {
  if (p.bias == nullptr) return;
  const int* bias = reinterpret_cast<const int*>(p.bias) + (int64_t)z * p.bias_bs;
  const int last = p.Kout - 1;  // channels past the end are computed but never stored
  const bool al = (reinterpret_cast<uintptr_t>(bias) & 15u) == 0;
#pragma unroll
  for (int j = 0; j < TN; ++j)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int c = n0 + j * 32 + q * 8 + lg * 4;
      intx4 b;
      if (al && c + 3 <= last) {
        b = *reinterpret_cast<const intx4*>(bias + c);
      } else {
        b.x = bias[c < last ? c : last];
        b.y = bias[c + 1 < last ? c + 1 : last];
        b.z = bias[c + 2 < last ? c + 2 : last];
        b.w = bias[c + 3 < last ? c + 3 : last];
      }
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        acc[i][j][q * 4 + 0] = b.x;
        acc[i][j][q * 4 + 1] = b.y;
        acc[i][j][q * 4 + 2] = b.z;
        acc[i][j][q * 4 + 3] = b.w;
      }
    }
}

// Requantisation of four consecutive channels of one pixel (one dword of the
// 8-bit result):  q = sat8(max(fma(float(acc), m, add), lo)), where `add` is the
// result's zero point or, with a residual, fma(float(r), r_mul, r_add) per
// channel.  v_cvt_pk_u8_f32 rounds to nearest even and saturates to [0, 255];
// stored bytes are level - 128, i.e. level ^ 0x80.
// kClamp = false: the lower bound is 0 (no ReLU, or a ReLU whose result has zero point 0, the
// usual case), which the saturating conversion applies by itself - same bits, one operation less.
template <bool kRes, bool kClamp = true>
__device__ __forceinline__ unsigned requant4(const int a0, const int a1, const int a2, const int a3, const floatx4 m,
                                             const unsigned res_stored, const IgemmParams& p) {
  float add0 = p.q_add, add1 = p.q_add, add2 = p.q_add, add3 = p.q_add;
  if constexpr (kRes) {
    const unsigned r = res_stored ^ 0x80808080u;  // stored -> levels
    add0 = __builtin_fmaf((float)(r & 0xffu), p.r_mul, p.r_add);
    add1 = __builtin_fmaf((float)((r >> 8) & 0xffu), p.r_mul, p.r_add);
    add2 = __builtin_fmaf((float)((r >> 16) & 0xffu), p.r_mul, p.r_add);
    add3 = __builtin_fmaf((float)(r >> 24), p.r_mul, p.r_add);
  }
  float f0 = __builtin_fmaf((float)a0, m.x, add0);
  float f1 = __builtin_fmaf((float)a1, m.y, add1);
  float f2 = __builtin_fmaf((float)a2, m.z, add2);
  float f3 = __builtin_fmaf((float)a3, m.w, add3);
  if constexpr (kClamp) {
    f0 = fmaxf(f0, p.q_lo); f1 = fmaxf(f1, p.q_lo); f2 = fmaxf(f2, p.q_lo); f3 = fmaxf(f3, p.q_lo);
  }
  unsigned w = 0u;
  w = __builtin_amdgcn_cvt_pk_u8_f32(f0, 0, w);
  w = __builtin_amdgcn_cvt_pk_u8_f32(f1, 1, w);
  w = __builtin_amdgcn_cvt_pk_u8_f32(f2, 2, w);
  w = __builtin_amdgcn_cvt_pk_u8_f32(f3, 3, w);
  return w ^ 0x80808080u;  // levels -> stored
}

// The multipliers of a lane's four channels of block (j, q): one 16-byte load
// when the channels exist and the table is aligned, clamped scalars otherwise.
__device__ __forceinline__ floatx4 load_qmul4(const float* qmul, const int c, const int Kout) {
  if (c + 3 < Kout && (reinterpret_cast<uintptr_t>(qmul + c) & 15u) == 0) return *reinterpret_cast<const floatx4*>(qmul + c);
  const int last = Kout - 1;
  floatx4 m;
  m.x = qmul[c < last ? c : last];
  m.y = qmul[c + 1 < last ? c + 1 : last];
  m.z = qmul[c + 2 < last ? c + 2 : last];
  m.w = qmul[c + 3 < last ? c + 3 : last];
  return m;
}

// 16 consecutive bytes of an 8-bit row: one vector access when `vec`, bytes otherwise.
__device__ __forceinline__ uintx4 load_row16(const int8_t* row, const bool vec, const int nvalid) {
  if (vec) return __builtin_nontemporal_load(reinterpret_cast<const uintx4*>(row));  // read once by the whole launch
  unsigned w[4] = {0u, 0u, 0u, 0u};
  for (int e = 0; e < nvalid; ++e) w[e >> 2] |= (unsigned)(uint8_t)row[e] << (8 * (e & 3));
  return (uintx4){w[0], w[1], w[2], w[3]};
}
__device__ __forceinline__ void store_row16(int8_t* row, const uintx4 v, const bool vec, const int nvalid,
                                            const bool stream) {
  if (vec) {
    if (stream) {
      uintx4* yv = reinterpret_cast<uintx4*>(row);
      asm volatile("" : "+v"(yv));  // keeps this store apart from the plain one (see EpiFloat::store8)
      __builtin_nontemporal_store(v, (__attribute__((address_space(1))) uintx4*)yv);
    } else {
      *reinterpret_cast<uintx4*>(row) = v;
    }
    return;
  }
  const unsigned w[4] = {v.x, v.y, v.z, v.w};
  for (int e = 0; e < nvalid; ++e) row[e] = (int8_t)(w[e >> 2] >> (8 * (e & 3)));
}

// Bank swizzle of the staged byte tiles.  Row pitches are a multiple of 16 bytes
// (the 16-byte row accesses need that), i.e. 4 banks modulo 8, so the dword that
// 32 lanes hold for 32 pixel rows would land in 8 banks, four rows each.  Dword d
// of row r therefore lives at d ^ ((r >> 3) & 3): the four rows that share a bank
// group take its four banks.  A 16-byte chunk stays a chunk; its dwords are
// exchanged on the way in and out (the exchange is its own inverse).
__device__ __forceinline__ int q8_swz(const int row) { return ((row >> 3) & 3) << 2; }
__device__ __forceinline__ uintx4 q8_swz_chunk(const uintx4 v, const int row) {
  const uintx4 t = (row & 8) ? uintx4{v.y, v.x, v.w, v.z} : v;
  return (row & 16) ? uintx4{t.z, t.w, t.x, t.y} : t;
}

// f(integral_constant<int, 0>{}) ... f(integral_constant<int, N - 1>{}), in order: a loop whose
// index is a constant in every iteration (a loop the optimizer declines to unroll would index
// the accumulators dynamically and move them to scratch memory).
template <int N, int I = 0, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<N, I + 1>(f);
  }
}

// Position of a lane in the order in which the LDS serves a 16-byte access of a wavefront:
// four passes of sixteen lanes, and within each half of the wavefront lanes {0-3, 12-15, 20-27}
// form one pass and lanes {4-11, 16-19, 28-31} the other (measured: two lanes that trade their
// 16-byte slots cost an extra pass exactly when they are of different sets).  Two lanes of a
// pass conflict when their slots are equal modulo 16.  Returns pass * 16 + place in the pass.
__device__ __forceinline__ int lds_pass_order(const int lane) {
  const int l = lane & 31;
  const bool second = (l >= 4 && l < 12) || (l >= 16 && l < 20) || l >= 28;
  const int k = second ? (l < 12 ? l - 4 : (l < 20 ? l - 8 : l - 16)) : (l < 4 ? l : (l < 16 ? l - 8 : l - 12));
  return (lane & 32) + (second ? 16 : 0) + k;
}

// Makes the compiler wait HERE for a value that was requested from memory in conditional code.
// The epilogues below request bias and residual vectors inside branches (per-lane validity) and
// consume them in later branches, between which they store results.  For a value whose request
// or first use sits in a branch the compiler cannot count the operations in flight behind it and
// waits for all of them at every later use - stores included, which share the counter: one store
// round trip per pass of an epilogue.  Naming the value as an operand of an (empty) statement in
// straight-line code settles it once, before the first store; the passes then issue their stores
// back to back.
template <typename T>
__device__ __forceinline__ void epi_settle(T& v) {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("" : "+v"(v));
#else
  (void)v;
#endif
}

// Output pixel (row of the GEMM) behind pixel `local` of a workgroup's tile: consecutive
// rows from `first` on, or - for kernels whose tile is a patch of the image rather than a
// run of rows - the entry of the tile's table in LDS (-1: no such pixel).
__device__ __forceinline__ int epi_pixel(const int* mtab, const int first, const int local) {
  return mtab != nullptr ? mtab[local] : first + local;
}

// ---------------------------------------------------------------------------
// Epilogue of the 8-bit layers, per wavefront.  The requantisation runs in the
// accumulator layout (a lane's four consecutive channels become one dword), so
// that only BYTES pass through LDS on their way to 16-byte row stores - a
// quarter of the LDS traffic of parking int32 accumulators, and the arithmetic
// per element is cvt, fma, max, cvt_pk.  A residual tile takes the same road in
// the other direction: 16-byte row loads, through LDS, read back as the dword of
// the lane's four channels.
// LDS per wavefront: two [32 pixels][WN + 16] byte tiles (result, residual; dwords
// swizzled by q8_swz) and the WN multipliers of its channels.
// kMulReady: the caller has parked the wavefront's multipliers already (a kernel that
// runs the epilogue for many pixel tiles of the same channels does that once, and
// keeps a vector-memory wait out of every epilogue).
template <int BM, int BN, int WM, int WN, bool kEnterBarrier = true, bool kMulReady = false>
__device__ __forceinline__ void igemm_epilogue_q8(const IgemmParams& p, const int epi_vec, intx16 (&acc)[WM / 32][WN / 32],
                                                  unsigned char* smem, const int tile_m, const int tile_n, const int z,
                                                  const int M, const int wave, const int lane, const int n_off = 0,
                                                  const int* mtab = nullptr) {
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int PITCH = WN + 16;          // bytes per staged pixel row
  constexpr int TILE = 32 * PITCH;
  constexpr int LPP = WN / 16;            // lanes per pixel row in the 16-byte passes
  constexpr int PPP = 64 / LPP;           // pixels per pass
  constexpr int NPASS = 32 / PPP;
  static_assert(NPASS >= 1, "a wavefront covers at most 32 pixels x 128 channels per pass set");
  const int wm = wave % (BM / WM), wn = wave / (BM / WM);
  const int l32 = lane & 31, lg = lane >> 5;
  const int n0 = tile_n * BN + wn * WN + n_off;  // first channel of this wavefront

  int8_t* ybase = reinterpret_cast<int8_t*>(p.y) + (int64_t)z * p.y_bs;
  const int8_t* rbase = p.residual ? reinterpret_cast<const int8_t*>(p.residual) + (int64_t)z * p.r_bs : nullptr;
  const bool has_res = rbase != nullptr;

  unsigned char* otile = smem + wave * (2 * TILE + WN * 4);
  unsigned char* rtile = otile + TILE;
  float* mtile = reinterpret_cast<float*>(rtile + TILE);  // the wavefront's WN multipliers

  // row-pass mapping: lane handles 16 channels c16 .. c16+15 of pixel rp (+ PPP per pass)
  const int rp = lane / LPP;
  const int c16 = (lane % LPP) * 16;
  int nvalid = p.Kout - (n0 + c16);
  nvalid = nvalid < 0 ? 0 : (nvalid > 16 ? 16 : nvalid);
  const bool vec = (epi_vec & 2) && nvalid == 16;

  // residual rows of slice i (one register set: the next slice is requested right
  // after the current one has been handed to LDS)
  uintx4 rcur[NPASS];
  auto rfetch = [&](const int i) {
#pragma unroll
    for (int ps = 0; ps < NPASS; ++ps) {
      const int m = epi_pixel(mtab, tile_m * BM, wm * WM + i * 32 + ps * PPP + rp);
      const int mc = (unsigned)m < (unsigned)M ? m : M - 1;
      rcur[ps] = nvalid > 0 ? load_row16(rbase + (int64_t)mc * p.rcs + n0 + c16, vec, nvalid) : uintx4{0u, 0u, 0u, 0u};
    }
  };
#pragma unroll
  for (int ps = 0; ps < NPASS; ++ps) rcur[ps] = uintx4{0u, 0u, 0u, 0u};
  if (has_res) rfetch(0);
  // the multipliers of the wavefront's channels, four per lane, parked in LDS below
  floatx4 mload = {0.f, 0.f, 0.f, 0.f};
  if constexpr (!kMulReady) {
    if (lane < WN / 4) mload = load_qmul4(p.qmul, n0 + lane * 4, p.Kout);
  }

  auto wave_fence = [&]() {
    // each wavefront only touches its own tiles and its LDS operations complete in issue order
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };

  if constexpr (kEnterBarrier) __syncthreads();  // the K loop's LDS traffic is done; the buffer becomes the staging area
  if constexpr (!kMulReady) {
    if (lane < WN / 4) *reinterpret_cast<floatx4*>(mtile + lane * 4) = mload;
  }
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    if (has_res) {
#pragma unroll
      for (int ps = 0; ps < NPASS; ++ps)
        *reinterpret_cast<uintx4*>(rtile + (ps * PPP + rp) * PITCH + c16) = q8_swz_chunk(rcur[ps], ps * PPP + rp);
    }
    wave_fence();
    if (has_res && i + 1 < TM) rfetch(i + 1);
    // requantise in the accumulator layout: lane holds, for pixel l32, channels j*32 + q*8 + lg*4 + (0..3)
    // (the residual case is a wavefront-uniform branch around the whole block: as a
    // per-element condition it costs a select per value)
    auto requant_block = [&](auto with_res, auto with_clamp) {
      constexpr bool kRes = decltype(with_res)::value;
      constexpr bool kClamp = decltype(with_clamp)::value;
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int ch = j * 32 + q * 8 + lg * 4;
          const int off = (l32 * PITCH + ch) ^ q8_swz(l32);
          const floatx4 m = *reinterpret_cast<const floatx4*>(mtile + ch);
          const unsigned rs = kRes ? *reinterpret_cast<const unsigned*>(rtile + off) : 0u;
          const unsigned w = requant4<kRes, kClamp>(acc[i][j][q * 4 + 0], acc[i][j][q * 4 + 1], acc[i][j][q * 4 + 2],
                                            acc[i][j][q * 4 + 3], m, rs, p);
          *reinterpret_cast<unsigned*>(otile + off) = w;
        }
    };
    const bool clamp = p.q_lo > 0.f;   // (wavefront-uniform, like has_res)
    if (has_res) { if (clamp) requant_block(std::true_type{}, std::true_type{}); else requant_block(std::true_type{}, std::false_type{}); }
    else { if (clamp) requant_block(std::false_type{}, std::true_type{}); else requant_block(std::false_type{}, std::false_type{}); }
    wave_fence();
#pragma unroll
    for (int ps = 0; ps < NPASS; ++ps) {
      const int pix = ps * PPP + rp;
      const int m = epi_pixel(mtab, tile_m * BM, wm * WM + i * 32 + pix);
      const uintx4 v = q8_swz_chunk(*reinterpret_cast<const uintx4*>(otile + pix * PITCH + c16), pix);
      if ((unsigned)m < (unsigned)M && nvalid > 0) store_row16(ybase + (int64_t)m * p.ycs + n0 + c16, v, vec, nvalid, p.stream_out);
    }
  }
}

// ---------------------------------------------------------------------------
// Epilogue shared by the kernels below: each wavefront parks one 32-pixel slice
// of its accumulators in LDS (pixel-major, fp32 / int32), then every lane picks
// eight consecutive output channels of one pixel, so that global stores and
// residual loads are 16-byte vectors and consecutive lanes cover contiguous
// memory.  `smem` is the K loop's buffer; it is reused once every wavefront of
// the workgroup has left the loop.
// kEnterBarrier = false: the caller's wavefronts never shared `smem` before
// (each only ever touches its own staging slice); n_off shifts the channels
// this call covers within the tile.
template <typename TIn, typename Epi, int BM, int BN, int WM, int WN, bool kEnterBarrier = true, bool kMulReady = false>
__device__ __forceinline__ void igemm_epilogue(const IgemmParams& p, const int epi_vec,
                                               typename Mma<TIn>::Acc (&acc)[WM / 32][WN / 32],
                                               unsigned char* smem, const int tile_m, const int tile_n,
                                               const int z, const int M, const int wave, const int lane,
                                               const int n_off = 0, const int* mtab = nullptr) {
  if constexpr (std::is_same<Epi, EpiQuant<0>>::value) {
    igemm_epilogue_q8<BM, BN, WM, WN, kEnterBarrier, kMulReady>(p, epi_vec, acc, smem, tile_m, tile_n, z, M, wave, lane, n_off, mtab);
    return;
  }
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int EPI_PITCH = WN + 4;  // 4-byte words per staged pixel row
  using AccE = typename Epi::AccE;
  using TOut = typename EpiTraits<Epi>::TOut;
  const int wm = wave % (BM / WM), wn = wave / (BM / WM);
  const int l32 = lane & 31, lg = lane >> 5;

  TOut* ybase = reinterpret_cast<TOut*>(p.y) + y_batch_off(p, z);
  const TOut* rbase = p.residual ? reinterpret_cast<const TOut*>(p.residual) + (int64_t)z * p.r_bs : nullptr;
  const AccE* bias = p.bias ? reinterpret_cast<const AccE*>(p.bias) + (int64_t)z * p.bias_bs : nullptr;

  AccE* stage = reinterpret_cast<AccE*>(smem) + wave * (32 * EPI_PITCH);
  constexpr int LPP = WN / 8;    // lanes per pixel row in the read-back
  constexpr int PPP = 64 / LPP;  // pixels per read-back pass
  // Which (pixel, eight channels) of a pass a lane moves: any assignment covers the same full
  // rows per store instruction, so it is chosen for the read-back from LDS - the sixteen lanes
  // of an LDS pass (lds_pass_order) take pixel rows an odd number of 16-byte slots apart,
  // consecutive pairs of slots each, i.e. sixteen different banks (lanes in their natural
  // order put slots of equal bank into one pass: 25 % of the LDS cycles of the streaming 2-byte
  // kernel were conflicts).
  const int vl = lds_pass_order(lane), vp = vl >> 4, vw = vl & 15;
  int rp, c8;                    // pixel within a pass, first channel
  if constexpr (LPP == 8) { rp = vl >> 3; c8 = (vl & 7) * 8; }
  else if constexpr (LPP == 16) { rp = (vp >> 1) * 2 + (vw >> 3); c8 = ((vp & 1) * 8 + (vw & 7)) * 8; }
  else if constexpr (LPP == 4) { rp = (vw >> 3) * 8 + vp * 2 + ((vw >> 2) & 1); c8 = (vw & 3) * 8; }
  else { rp = lane / LPP; c8 = (lane % LPP) * 8; }
  (void)vp; (void)vw;
  const int n = tile_n * BN + wn * WN + c8 + n_off;
  int nvalid = p.Kout - n;
  nvalid = nvalid < 0 ? 0 : (nvalid > 8 ? 8 : nvalid);
  const bool vec = (epi_vec & 1) && nvalid == 8;
  const int64_t ycol = y_col_off(p, n);

  // lane-constant epilogue operands: the lane's eight channels are the same in every pass
  AccE b8[8];
  float m8[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) { b8[e] = 0; m8[e] = 0.f; }
  if (nvalid > 0) {
    // (8-bit layers carry their bias in the accumulators already)
    if (bias != nullptr && !EpiTraits<Epi>::quant) {
      if (vec) {
        const intx4 t0 = *reinterpret_cast<const intx4*>(bias + n);
        const intx4 t1 = *reinterpret_cast<const intx4*>(bias + n + 4);
        __builtin_memcpy(&b8[0], &t0, 16);
        __builtin_memcpy(&b8[4], &t1, 16);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (e < nvalid) b8[e] = bias[n + e];
      }
    }
    if constexpr (EpiTraits<Epi>::quant) {
      if (p.qmul != nullptr) {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (e < nvalid) m8[e] = p.qmul[n + e];
      }
    }
  }

  // Residual vectors are requested one 32-pixel slice ahead of their use, so
  // that their latency overlaps with the staging of the previous slice.
  constexpr int NPASS = 32 / PPP;
  using RVec = typename Epi::RVec;
  const bool have_rpre = Epi::kPrefetchResidual && vec && rbase != nullptr;
  auto rfetch = [&](const int i, RVec (&dst)[NPASS]) {
#pragma unroll
    for (int ps = 0; ps < NPASS; ++ps) {
      const int m = epi_pixel(mtab, tile_m * BM, wm * WM + i * 32 + ps * PPP + rp);
      const int mc = (unsigned)m < (unsigned)M ? m : M - 1;
      // read once by the whole launch: a non-temporal load leaves the cache lines to the operands that are re-read
      dst[ps] = __builtin_nontemporal_load(reinterpret_cast<const RVec*>(rbase + (int64_t)mc * p.rcs + n));
    }
  };
  RVec rcur[NPASS], rnxt[NPASS];
#pragma unroll
  for (int ps = 0; ps < NPASS; ++ps) { rcur[ps] = RVec{}; rnxt[ps] = RVec{}; }
  if constexpr (Epi::kPrefetchResidual) {
    if (have_rpre) rfetch(0, rcur);
  }

  if constexpr (kEnterBarrier) __syncthreads();  // the K loop's LDS reads are done; the buffer becomes the staging area
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    // park: lane holds, for pixel l32, channels j*32 + q*8 + lg*4 + (0..3)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        AccE* dst = stage + l32 * EPI_PITCH + j * 32 + q * 8 + lg * 4;
        if constexpr (sizeof(AccE) == 4 && !EpiTraits<Epi>::quant) {
          *reinterpret_cast<floatx4*>(dst) =
              (floatx4){acc[i][j][q * 4 + 0], acc[i][j][q * 4 + 1], acc[i][j][q * 4 + 2], acc[i][j][q * 4 + 3]};
        } else {
          *reinterpret_cast<intx4*>(dst) =
              (intx4){(int)acc[i][j][q * 4 + 0], (int)acc[i][j][q * 4 + 1], (int)acc[i][j][q * 4 + 2], (int)acc[i][j][q * 4 + 3]};
        }
      }
    }
    // Each wavefront only touches its own staging slice and its LDS operations
    // complete in issue order, so a wavefront-scope fence (no workgroup barrier)
    // orders the parking writes before the read-back.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    // this slice's operands from memory are complete before its first store (see epi_settle;
    // not in the instantiations with the wider activation set, which have no registers to spare)
    if (i == 0 && !EpiTraits<Epi>::rich) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        if constexpr (EpiTraits<Epi>::quant) epi_settle(m8[e]);
        else epi_settle(b8[e]);
      }
    }
    if constexpr (Epi::kPrefetchResidual && !EpiTraits<Epi>::rich) {
#pragma unroll
      for (int ps = 0; ps < NPASS; ++ps) epi_settle(rcur[ps]);
    }
    if constexpr (Epi::kPrefetchResidual && TM > 1) {
      if (have_rpre && i + 1 < TM) rfetch(i + 1, rnxt);
    }
#pragma unroll
    for (int ps = 0; ps < NPASS; ++ps) {
      const int pix = ps * PPP + rp;
      const int m = epi_pixel(mtab, tile_m * BM, wm * WM + i * 32 + pix);
      AccE a8[8];
      const AccE* src = stage + pix * EPI_PITCH + c8;
      if constexpr (!EpiTraits<Epi>::quant) {
        const floatx4 v0 = *reinterpret_cast<const floatx4*>(src);
        const floatx4 v1 = *reinterpret_cast<const floatx4*>(src + 4);
        a8[0] = v0.x; a8[1] = v0.y; a8[2] = v0.z; a8[3] = v0.w;
        a8[4] = v1.x; a8[5] = v1.y; a8[6] = v1.z; a8[7] = v1.w;
      } else {
        const intx4 v0 = *reinterpret_cast<const intx4*>(src);
        const intx4 v1 = *reinterpret_cast<const intx4*>(src + 4);
        a8[0] = v0.x; a8[1] = v0.y; a8[2] = v0.z; a8[3] = v0.w;
        a8[4] = v1.x; a8[5] = v1.y; a8[6] = v1.z; a8[7] = v1.w;
      }
      if ((unsigned)m < (unsigned)M && nvalid > 0) {
        TOut* yrow = ybase + y_row_off(p, m) + ycol;
        const TOut* rrow = rbase ? rbase + (int64_t)m * p.rcs + n : nullptr;
        Epi::store8(p, a8, nvalid, vec, b8, m8, yrow, rrow, have_rpre, rcur[ps]);
      }
    }
#pragma unroll
    for (int ps = 0; ps < NPASS; ++ps) rcur[ps] = rnxt[ps];
    if (i + 1 < TM) {
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
  }
}

// ---------------------------------------------------------------------------
// The 8-bit form of the epilogue below (four wavefronts, each with all 128 pixels
// of the tile and a 32-channel slice): every wavefront requantises its slice in
// the accumulator layout and writes the dwords of its 32 channels into one
// [32 pixels][128 channels] BYTE tile, side by side with the others; then each
// of the 256 threads moves 16 consecutive channels of one pixel, i.e. one pass
// covers the 32 x 128 tile with full 128-byte rows.  The residual tile takes the
// same road in the other direction.  Two tile pairs alternate, so that a slice
// needs one barrier between its phases and one before its tiles are reused.
// mtile: the tile's 128 multipliers in LDS (parked there by the caller ahead of its K
// loop: the epilogue then starts without a round trip to memory), or nullptr.
template <int TM = 4>
__device__ __forceinline__ void igemm_epilogue_rows128_q8(const IgemmParams& p, const int epi_vec, intx16 (&acc)[TM][1],
                                                          unsigned char* smem, const int tile_m, const int tile_n,
                                                          const int z, const int M, const int wave, const int lane,
                                                          const float* mtile = nullptr, const int* mtab = nullptr) {
  constexpr int BM = TM * 32, BN = 128;
  constexpr int PITCH = BN + 16;  // bytes per staged pixel row
  constexpr int TILE = 32 * PITCH;
  const int tid = wave * 64 + lane;
  const int l32 = lane & 31, lg = lane >> 5;
  const int n0 = tile_n * BN;

  int8_t* ybase = reinterpret_cast<int8_t*>(p.y) + (int64_t)z * p.y_bs;
  const int8_t* rbase = p.residual ? reinterpret_cast<const int8_t*>(p.residual) + (int64_t)z * p.r_bs : nullptr;
  const bool has_res = rbase != nullptr;

  const int rp = tid >> 3;         // pixel of the slice this thread moves
  const int c16 = (tid & 7) * 16;  // ... and its 16 channels
  int nvalid = p.Kout - (n0 + c16);
  nvalid = nvalid < 0 ? 0 : (nvalid > 16 ? 16 : nvalid);
  const bool vec = (epi_vec & 2) && nvalid == 16;

  floatx4 mq[4];
#pragma unroll
  for (int q = 0; q < 4; ++q)
    mq[q] = mtile != nullptr ? *reinterpret_cast<const floatx4*>(mtile + wave * 32 + q * 8 + lg * 4)
                             : load_qmul4(p.qmul, n0 + wave * 32 + q * 8 + lg * 4, p.Kout);

  // The residual rows of all four slices are requested ahead of the first barrier:
  // one memory round trip per tile.
  uintx4 rall[TM];
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    rall[i] = uintx4{0u, 0u, 0u, 0u};
    if (has_res && nvalid > 0) {
      const int m = epi_pixel(mtab, tile_m * BM, i * 32 + rp);
      const int mc = (unsigned)m < (unsigned)M ? m : M - 1;
      rall[i] = load_row16(rbase + (int64_t)mc * p.rcs + n0 + c16, vec, nvalid);
    }
  }

  // Workgroup barrier for LDS traffic only: the fence of __syncthreads would
  // also wait for the global stores of the slices before.
  auto lds_barrier = [&]() {
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0), other counters at their maxima
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
  };
  lds_barrier();  // the K loop's LDS reads are done; the ring becomes the staging area
  // (with or without a residual: two straight-line copies of the slice chosen by one
  // workgroup-uniform branch; as a condition inside, every value pays a move or a select)
  auto slice = [&](auto slice_no, auto with_res, auto with_clamp) __attribute__((always_inline)) {
    constexpr int i = decltype(slice_no)::value;
    constexpr bool kRes = decltype(with_res)::value;
    constexpr bool kClamp = decltype(with_clamp)::value;
    unsigned char* otile = smem + (i & 1) * (2 * TILE);
    unsigned char* rtile = otile + TILE;
    if constexpr (kRes) {
      *reinterpret_cast<uintx4*>(rtile + rp * PITCH + c16) = q8_swz_chunk(rall[i], rp);
      lds_barrier();
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int off = (l32 * PITCH + wave * 32 + q * 8 + lg * 4) ^ q8_swz(l32);
      const unsigned rs = kRes ? *reinterpret_cast<const unsigned*>(rtile + off) : 0u;
      *reinterpret_cast<unsigned*>(otile + off) =
          requant4<kRes, kClamp>(acc[i][0][q * 4 + 0], acc[i][0][q * 4 + 1], acc[i][0][q * 4 + 2], acc[i][0][q * 4 + 3], mq[q], rs, p);
    }
    // Nobody passes this barrier before every wavefront has written slice i; a wavefront
    // writes slice i+1 into the other tile pair, and slice i+2 into this one only after
    // the barrier(s) of slice i+1, which every wavefront reaches after its reads here.
    lds_barrier();
    const int m = epi_pixel(mtab, tile_m * BM, i * 32 + rp);
    const uintx4 v = q8_swz_chunk(*reinterpret_cast<const uintx4*>(otile + rp * PITCH + c16), rp);
    if ((unsigned)m < (unsigned)M && nvalid > 0) store_row16(ybase + (int64_t)m * p.ycs + n0 + c16, v, vec, nvalid, p.stream_out);
  };
  auto slices = [&](auto with_res, auto with_clamp) __attribute__((always_inline)) {
    static_for<TM>([&](auto slice_no) __attribute__((always_inline)) { slice(slice_no, with_res, with_clamp); });
  };
  const bool clamp = p.q_lo > 0.f;   // (a lower bound of 0 is what the saturating conversion applies anyway)
  if (has_res) { if (clamp) slices(std::true_type{}, std::true_type{}); else slices(std::true_type{}, std::false_type{}); }
  else { if (clamp) slices(std::false_type{}, std::true_type{}); else slices(std::false_type{}, std::false_type{}); }
}

// ---------------------------------------------------------------------------
// Epilogue for workgroups whose four wavefronts each own all 128 pixels of the
// tile and a 32-channel slice: per 32-pixel slice the four wavefronts park
// their channels side by side in one [32 pixels][128 channels] LDS tile (two
// tiles, alternating, one workgroup barrier per slice), and every thread then
// handles eight consecutive channels of one pixel, so that 16 consecutive lanes
// write one full 128-channel output row and no cache line is written in halves
// by different wavefronts.
// kSettleRes = false leaves the residual vectors unsettled (a kernel at its register limit whose
// layers carry no residual: settling holds all of them in registers at once, zeros included).
template <typename TIn, typename Epi, int TM = 4, bool kSettleRes = true>
__device__ __forceinline__ void igemm_epilogue_rows128(const IgemmParams& p, const int epi_vec,
                                                       typename Mma<TIn>::Acc (&acc)[TM][1], unsigned char* smem,
                                                       const int tile_m, const int tile_n, const int z, const int M,
                                                       const int wave, const int lane, const float* mtile = nullptr,
                                                       const int* mtab = nullptr) {
  if constexpr (std::is_same<Epi, EpiQuant<0>>::value) {
    igemm_epilogue_rows128_q8<TM>(p, epi_vec, acc, smem, tile_m, tile_n, z, M, wave, lane, mtile, mtab);
    return;
  }
  constexpr int BM = TM * 32, BN = 128;
  constexpr int PITCH = BN + 4;  // 4-byte words per staged pixel row
  constexpr int TILE_WORDS = 32 * PITCH;
  using AccE = typename Epi::AccE;
  using TOut = typename EpiTraits<Epi>::TOut;
  const int tid = wave * 64 + lane;
  const int l32 = lane & 31, lg = lane >> 5;

  TOut* ybase = reinterpret_cast<TOut*>(p.y) + y_batch_off(p, z);
  const TOut* rbase = p.residual ? reinterpret_cast<const TOut*>(p.residual) + (int64_t)z * p.r_bs : nullptr;
  const AccE* bias = p.bias ? reinterpret_cast<const AccE*>(p.bias) + (int64_t)z * p.bias_bs : nullptr;

  const int rp = tid >> 4;          // pixel within a pass of 16
  const int c8 = (tid & 15) * 8;    // this thread's eight channels
  const int n = tile_n * BN + c8;
  int nvalid = p.Kout - n;
  nvalid = nvalid < 0 ? 0 : (nvalid > 8 ? 8 : nvalid);
  const bool vec = (epi_vec & 1) && nvalid == 8;

  AccE b8[8];
  float m8[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) { b8[e] = 0; m8[e] = 0.f; }
  if (nvalid > 0) {
    // (8-bit layers carry their bias in the accumulators already)
    if (bias != nullptr && !EpiTraits<Epi>::quant) {
      if (vec) {
        const intx4 t0 = *reinterpret_cast<const intx4*>(bias + n);
        const intx4 t1 = *reinterpret_cast<const intx4*>(bias + n + 4);
        __builtin_memcpy(&b8[0], &t0, 16);
        __builtin_memcpy(&b8[4], &t1, 16);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (e < nvalid) b8[e] = bias[n + e];
      }
    }
    if constexpr (EpiTraits<Epi>::quant) {
      if (p.qmul != nullptr) {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (e < nvalid) m8[e] = p.qmul[n + e];
      }
    }
  }

  TOut* const ythr = ybase + y_col_off(p, n);  // + the row's offset
  const TOut* const rthr = rbase ? rbase + (int64_t)(tile_m * BM + rp) * p.rcs + n : nullptr;

  using RVec = typename Epi::RVec;
  const bool have_rpre = Epi::kPrefetchResidual && vec && rbase != nullptr;
  auto rfetch = [&](const int i, RVec (&dst)[2]) {
#pragma unroll
    for (int ps = 0; ps < 2; ++ps) {
      const int m = epi_pixel(mtab, tile_m * BM, i * 32 + ps * 16 + rp);
      const int mc = (unsigned)m < (unsigned)M ? m : M - 1;
      // read once by the whole launch: a non-temporal load leaves the cache lines to the operands that are re-read
      dst[ps] = __builtin_nontemporal_load(reinterpret_cast<const RVec*>(rbase + (int64_t)mc * p.rcs + n));
    }
  };
  // The residual vectors of all four slices are requested here, ahead of the
  // parking and the barriers of the first slice: one memory round trip per tile.
  // (Fetched a slice ahead instead, each slice would wait for its own request:
  // behind the stores of the slice before, the compiler waits for every
  // vector-memory operation in flight.)
  RVec rall[TM][2];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int ps = 0; ps < 2; ++ps) rall[i][ps] = RVec{};
  if constexpr (Epi::kPrefetchResidual) {
    if (have_rpre) {
#pragma unroll
      for (int i = 0; i < TM; ++i) rfetch(i, rall[i]);
    }
  }

  // Workgroup barrier for LDS traffic only: the fence of __syncthreads would
  // also wait for the global stores of the slices before, one store round trip
  // per slice.
  auto lds_barrier = [&]() {
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0), other counters at their maxima
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
  };
  lds_barrier();  // the K loop's LDS reads are done; the ring becomes the staging area
  // every operand requested from memory above is complete before the first store (see epi_settle)
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    if constexpr (EpiTraits<Epi>::quant) epi_settle(m8[e]);
    else epi_settle(b8[e]);
  }
  if constexpr (Epi::kPrefetchResidual && kSettleRes) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int ps = 0; ps < 2; ++ps) epi_settle(rall[i][ps]);
  }
  // One call per 32-pixel slice with the slice number as a constant: a loop the
  // optimizer declines to unroll would index the accumulators dynamically and
  // move them to scratch memory.
  auto slice = [&](auto slice_no) __attribute__((always_inline)) {
    constexpr int i = decltype(slice_no)::value;
    AccE* tile = reinterpret_cast<AccE*>(smem) + (i & 1) * TILE_WORDS;
    // park: lane holds, for pixel l32, channels wave*32 + q*8 + lg*4 + (0..3)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      AccE* dst = tile + l32 * PITCH + wave * 32 + q * 8 + lg * 4;
      if constexpr (sizeof(AccE) == 4 && !EpiTraits<Epi>::quant) {
        *reinterpret_cast<floatx4*>(dst) =
            (floatx4){acc[i][0][q * 4 + 0], acc[i][0][q * 4 + 1], acc[i][0][q * 4 + 2], acc[i][0][q * 4 + 3]};
      } else {
        *reinterpret_cast<intx4*>(dst) =
            (intx4){(int)acc[i][0][q * 4 + 0], (int)acc[i][0][q * 4 + 1], (int)acc[i][0][q * 4 + 2], (int)acc[i][0][q * 4 + 3]};
      }
    }
    // One barrier per slice is enough: a wavefront parks slice i+1 into the
    // other tile only after its own read-back of slice i, and nobody passes
    // this barrier before every wavefront has finished reading slice i-1.
    lds_barrier();
#pragma unroll
    for (int ps = 0; ps < 2; ++ps) {
      const int pix = ps * 16 + rp;
      const int m = epi_pixel(mtab, tile_m * BM, i * 32 + pix);
      AccE a8[8];
      const AccE* src = tile + pix * PITCH + c8;
      if constexpr (!EpiTraits<Epi>::quant) {
        const floatx4 v0 = *reinterpret_cast<const floatx4*>(src);
        const floatx4 v1 = *reinterpret_cast<const floatx4*>(src + 4);
        a8[0] = v0.x; a8[1] = v0.y; a8[2] = v0.z; a8[3] = v0.w;
        a8[4] = v1.x; a8[5] = v1.y; a8[6] = v1.z; a8[7] = v1.w;
      } else {
        const intx4 v0 = *reinterpret_cast<const intx4*>(src);
        const intx4 v1 = *reinterpret_cast<const intx4*>(src + 4);
        a8[0] = v0.x; a8[1] = v0.y; a8[2] = v0.z; a8[3] = v0.w;
        a8[4] = v1.x; a8[5] = v1.y; a8[6] = v1.z; a8[7] = v1.w;
      }
      if ((unsigned)m < (unsigned)M && nvalid > 0) {
        // thread row pointer + a wavefront-uniform offset
        TOut* yrow = ythr + y_row_off(p, m);
        const TOut* rrow = !rbase ? nullptr : mtab ? rbase + (int64_t)m * p.rcs + n : rthr + (int64_t)(i * 32 + ps * 16) * p.rcs;
        Epi::store8(p, a8, nvalid, vec, b8, m8, yrow, rrow, have_rpre, rall[i][ps]);
      }
    }
  };
  static_for<TM>(slice);
}

}  // namespace ohip
#endif
