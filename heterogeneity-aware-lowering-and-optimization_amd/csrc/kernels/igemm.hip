// Implicit-GEMM convolution / GEMM for gfx950 (CDNA4) matrix cores.
//
// One kernel template covers odla_Conv and odla_Gemm for fp32, fp16, bf16 and
// int8 operands.  Activations are channels-last, so the reduction index
// k = (r, s, c) is contiguous in c and every global load is a 16-byte vector.
// A workgroup owns a BM (pixels) x BN (output channels) tile; each 64-lane
// wavefront owns a WM x WN sub-tile built from 32x32 MFMA blocks.  Per K stage
// the workgroup stages 64 bytes of K per row for both operands in LDS (rows
// padded to 80 bytes so that the 16-byte fragment reads of 16 consecutive lanes
// fall into distinct banks), double buffered, with the next stage's global
// loads in flight while the current stage feeds the MFMAs.
//
// The weight rows are the MFMA "A" operand and the pixel rows the "B" operand:
// in the 32x32 accumulator layout lane l then holds, for pixel (l % 32), groups
// of four consecutive output channels, which is what a channels-last store
// wants.  Both operands use the same k -> (lane group, element) assignment, so
// the exact k permutation inside one MFMA is irrelevant to the result.
#include "device_utils.h"

namespace ohip {

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

template <typename TOut>
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
    for (int e = 0; e < 8; ++e) v[e] = acc[e] * p.alpha + b8[e];
    if (vec) {
      if (r != nullptr) {
        if constexpr (sizeof(TOut) == 4) {
          const floatx4 r0 = *reinterpret_cast<const floatx4*>(r);
          const floatx4 r1 = *reinterpret_cast<const floatx4*>(r + 4);
          v[0] += r0.x; v[1] += r0.y; v[2] += r0.z; v[3] += r0.w;
          v[4] += r1.x; v[5] += r1.y; v[6] += r1.z; v[7] += r1.w;
        } else {
          Vec16<TOut> rv;
          if (have_rpre) rv.raw = rpre; else rv.load(r);
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] += rv.get(e);
        }
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = epi_act(v[e], p.act, p.act_a, p.act_b);
      if constexpr (sizeof(TOut) == 4) {
        *reinterpret_cast<floatx4*>(y) = (floatx4){v[0], v[1], v[2], v[3]};
        *reinterpret_cast<floatx4*>(y + 4) = (floatx4){v[4], v[5], v[6], v[7]};
      } else {
        Vec16<TOut> o;
#pragma unroll
        for (int e = 0; e < 8; ++e) o.set(e, v[e]);
        o.store(y);
      }
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        if (e < nvalid) {
          float t = v[e];
          if (r != nullptr) t += Store<TOut>::ld(r + e);
          Store<TOut>::st(y + e, epi_act(t, p.act, p.act_a, p.act_b));
        }
      }
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
  using RVec = uintx2;  // eight 1-byte residual levels fetched ahead of use
  static constexpr bool kPrefetchResidual = MODE == 0;
  __device__ static __forceinline__ void store8(const IgemmParams& p, const int* acc, int nvalid, bool vec,
                                                const int* b8, const float* m8, TOut* y, const TOut* r,
                                                bool have_rpre, RVec rpre) {
    if constexpr (MODE == 0) {
      int8_t rs[8] = {0, 0, 0, 0, 0, 0, 0, 0};
      if (r != nullptr) {
        if (vec) {
          const uintx2 rv = have_rpre ? rpre : *reinterpret_cast<const uintx2*>(r);
          __builtin_memcpy(rs, &rv, 8);
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (e < nvalid) rs[e] = r[e];
        }
      }
      int8_t out[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int a = acc[e] + b8[e];
        const float f0 = (float)a * m8[e];   // v_cvt_f32_i32 (RNE), then one v_mul_f32
        int q = (int)rintf(f0) + p.q_zp;      // v_rndne_f32
        q = q < p.q_lo ? p.q_lo : q;
        q = q > 255 ? 255 : q;
        if (r != nullptr) {
          const float fa = (float)(q - p.q_zp) * p.q_scale;
          const float fb = (float)(q_from_stored(rs[e]) - p.r_zp) * p.r_scale;
          const float f = fa + fb;
          q = (int)rintf(f * p.s_inv) + p.s_zp;
          q = q < p.s_lo ? p.s_lo : q;
          q = q > 255 ? 255 : q;
        }
        out[e] = q_to_stored(q);
      }
      if (vec) {
        uintx2 ov;
        __builtin_memcpy(&ov, out, 8);
        *reinterpret_cast<uintx2*>(y) = ov;
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (e < nvalid) y[e] = out[e];
      }
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        if (e < nvalid) {
          const int a = acc[e] + b8[e];
          if constexpr (MODE == 2) {
            y[e] = a;
          } else {
            float f = (float)a * m8[e];
            if (r != nullptr) f += r[e];
            y[e] = epi_act(f, p.act, p.act_a, p.act_b);
          }
        }
      }
    }
  }
};

template <typename Epi> struct EpiTraits;
template <typename T> struct EpiTraits<EpiFloat<T>> { using TOut = T; static constexpr bool quant = false; };
template <int M> struct EpiTraits<EpiQuant<M>> { using TOut = typename QuantOut<M>::T; static constexpr bool quant = true; };

// ---------------------------------------------------------------------------
// Main kernel.
//
// K pipeline: per stage the workgroup holds 128 bytes of K per row for both
// operands in one LDS buffer; the next stage's global loads are issued right
// after the buffer is published and stay in flight, in registers, while the
// MFMAs of the current stage run.  Other resident workgroups of the CU cover
// the two barriers per stage.
//
// Epilogue: each wavefront parks one 32-pixel slice of its accumulators in LDS
// (pixel-major, fp32 / int32), then every lane picks eight consecutive output
// channels of one pixel, so that global stores and residual loads are 16-byte
// vectors and consecutive lanes cover contiguous memory.
template <typename TIn, typename Epi, int BM, int BN, int WM, int WN>
__global__ void __launch_bounds__((BM / WM) * (BN / WN) * 64)
igemm_kernel(const IgemmParams p, const int epi_vec) {
  constexpr int NW = (BM / WM) * (BN / WN);
  constexpr int NT = NW * 64;
  constexpr int ES = sizeof(TIn);
  constexpr int VEC = 16 / ES;    // elements per 16-byte vector
  constexpr int BKB = 128;        // bytes of K per row per stage
  constexpr int BK = BKB / ES;    // elements of K per stage
  constexpr int ROWB = BKB + 16;  // LDS row pitch in bytes: 16-byte reads of 16 lanes hit distinct banks
  constexpr int VPR = BKB / 16;   // vectors per row
  constexpr int RPP = NT / VPR;   // rows loaded per pass
  constexpr int A_IT = (BM + RPP - 1) / RPP, B_IT = (BN + RPP - 1) / RPP;
  static_assert(BM % RPP == 0 || BM < RPP, "pixel tile must be a multiple of the rows per pass");
  static_assert(BN % RPP == 0 || BN < RPP, "channel tile must be a multiple of the rows per pass");
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int EPI_PITCH = WN + 4;  // 4-byte words per staged pixel row
  constexpr int MAIN_BYTES = (BM + BN) * ROWB;
  constexpr int EPI_BYTES = NW * 32 * EPI_PITCH * 4;
  constexpr int SMEM_BYTES = MAIN_BYTES > EPI_BYTES ? MAIN_BYTES : EPI_BYTES;
  using Acc = typename Mma<TIn>::Acc;
  using AccE = typename Epi::AccE;
  using TOut = typename EpiTraits<Epi>::TOut;

  __shared__ __attribute__((aligned(16))) unsigned char smem[SMEM_BYTES];
  unsigned char* As = smem;
  unsigned char* Bs = smem + BM * ROWB;

  const int tid = threadIdx.x;
  const int M = p.N * p.Ho * p.Wo;
  const int tiles_n = (p.Kout + BN - 1) / BN;

  // Workgroups are dealt round-robin to the 8 XCDs; renumber them so that the
  // workgroups sharing one pixel tile (all its channel tiles) and neighbouring
  // pixel tiles land on the same XCD and hit in its L2.
  int bid = blockIdx.x;
  {
    const int per = gridDim.x >> 3;
    if (bid < (per << 3)) bid = (bid & 7) * per + (bid >> 3);
  }
  const int tile_n = bid % tiles_n;
  const int tile_m = bid / tiles_n;
  const int z = blockIdx.z;

  const TIn* x = reinterpret_cast<const TIn*>(p.x) + (int64_t)z * p.x_bs;
  const TIn* w = reinterpret_cast<const TIn*>(p.w) + (int64_t)z * p.w_bs;

  const int kv = tid % VPR;
  const int row0 = tid / VPR;

  // ---- per-thread gather state for its A (pixel) rows ----
  const TIn* a_ptr[A_IT];
  int a_hi0[A_IT], a_wi0[A_IT];
  const int HoWo = p.Ho * p.Wo;
#pragma unroll
  for (int i = 0; i < A_IT; ++i) {
    const int m = tile_m * BM + row0 + i * RPP;
    const bool ok = (m < M) && ((BM % RPP == 0) || (row0 + i * RPP < BM));
    const int mm = ok ? m : 0;
    const int n_img = mm / HoWo;
    const int rem = mm - n_img * HoWo;
    const int ho = rem / p.Wo;
    const int wo = rem - ho * p.Wo;
    a_hi0[i] = ok ? ho * p.sh - p.ph : -(1 << 28);  // out-of-range rows never pass the bounds test
    a_wi0[i] = wo * p.sw - p.pw;
    a_ptr[i] = x + (int64_t)n_img * p.H * p.W * p.xcs;
  }
  // ---- per-thread state for its B (weight) rows ----
  const TIn* b_ptr[B_IT];
#pragma unroll
  for (int i = 0; i < B_IT; ++i) {
    const int n = tile_n * BN + row0 + i * RPP;
    const bool in_tile = (BN % RPP == 0) || (row0 + i * RPP < BN);
    b_ptr[i] = (in_tile && n < p.w_rows) ? (w + (int64_t)n * p.w_rs + kv * VEC) : nullptr;
  }

  // k position of this thread's vector, decomposed into tap (r, s) and channel c.
  int kc = kv * VEC, kr = 0, ks = 0;
  while (kc >= p.C) {
    kc -= p.C;
    if (++ks == p.S) { ks = 0; ++kr; }
  }
  int kcol = kv * VEC;

  uintx4 fillv;
  {
    const unsigned f = (unsigned)(p.a_fill & 0xff) * 0x01010101u;
    fillv = (uintx4){f, f, f, f};
  }
  const uintx4 zerov = {0u, 0u, 0u, 0u};

  uintx4 ra[A_IT], rb[B_IT];
  auto gload = [&]() {
    const int hoff = kr * p.dh, woff = ks * p.dw;
#pragma unroll
    for (int i = 0; i < A_IT; ++i) {
      const int hi = a_hi0[i] + hoff, wi = a_wi0[i] + woff;
      const bool ok = (kr < p.R) && ((unsigned)hi < (unsigned)p.H) && ((unsigned)wi < (unsigned)p.W);
      ra[i] = ok ? *reinterpret_cast<const uintx4*>(a_ptr[i] + ((hi * p.W + wi) * p.xcs + kc)) : fillv;
    }
#pragma unroll
    for (int i = 0; i < B_IT; ++i) {
      const bool ok = (b_ptr[i] != nullptr) && (kcol < p.w_cols);
      rb[i] = ok ? *reinterpret_cast<const uintx4*>(b_ptr[i]) : zerov;
      if (b_ptr[i] != nullptr) b_ptr[i] += BK;
    }
    kcol += BK;
    kc += BK;
    while (kc >= p.C) {
      kc -= p.C;
      if (++ks == p.S) { ks = 0; ++kr; }
    }
  };
  auto lds_store = [&]() {
    unsigned char* ab = As + row0 * ROWB + kv * 16;
#pragma unroll
    for (int i = 0; i < A_IT; ++i)
      if (BM % RPP == 0 || row0 + i * RPP < BM) *reinterpret_cast<uintx4*>(ab + i * RPP * ROWB) = ra[i];
    unsigned char* bb = Bs + row0 * ROWB + kv * 16;
#pragma unroll
    for (int i = 0; i < B_IT; ++i)
      if (BN % RPP == 0 || row0 + i * RPP < BN) *reinterpret_cast<uintx4*>(bb + i * RPP * ROWB) = rb[i];
  };

  const int wave = tid >> 6, lane = tid & 63;
  const int wm = wave % (BM / WM), wn = wave / (BM / WM);
  const int l32 = lane & 31, lg = lane >> 5;

  Acc acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

  const int ktot = p.R * p.S * p.C;
  const int nkt = (ktot + BK - 1) / BK;
  const unsigned char* ab = As + (wm * WM + l32) * ROWB + lg * 16;
  const unsigned char* bb = Bs + (wn * WN + l32) * ROWB + lg * 16;

  gload();
  for (int kt = 0; kt < nkt; ++kt) {
    if (kt > 0) __syncthreads();  // everyone finished reading the previous stage
    lds_store();
    __syncthreads();
    if (kt + 1 < nkt) gload();
#pragma unroll
    for (int kk = 0; kk < BKB / 32; ++kk) {
      uintx4 fa[TM], fb[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) fa[i] = *reinterpret_cast<const uintx4*>(ab + i * 32 * ROWB + kk * 32);
#pragma unroll
      for (int j = 0; j < TN; ++j) fb[j] = *reinterpret_cast<const uintx4*>(bb + j * 32 * ROWB + kk * 32);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = Mma<TIn>::run(fb[j], fa[i], acc[i][j]);
    }
  }

  // ---- epilogue ----
  TOut* ybase = reinterpret_cast<TOut*>(p.y) + (int64_t)z * p.y_bs;
  const TOut* rbase = p.residual ? reinterpret_cast<const TOut*>(p.residual) + (int64_t)z * p.r_bs : nullptr;
  const AccE* bias = p.bias ? reinterpret_cast<const AccE*>(p.bias) + (int64_t)z * p.bias_bs : nullptr;

  AccE* stage = reinterpret_cast<AccE*>(smem) + wave * (32 * EPI_PITCH);
  constexpr int LPP = WN / 8;    // lanes per pixel row in the read-back
  constexpr int PPP = 64 / LPP;  // pixels per read-back pass
  const int rp = lane / LPP;     // pixel within a pass
  const int c8 = (lane % LPP) * 8;
  const int n = tile_n * BN + wn * WN + c8;
  int nvalid = p.Kout - n;
  nvalid = nvalid < 0 ? 0 : (nvalid > 8 ? 8 : nvalid);
  const bool vec = epi_vec && nvalid == 8;

  // lane-constant epilogue operands: the lane's eight channels are the same in every pass
  AccE b8[8];
  float m8[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) { b8[e] = 0; m8[e] = 0.f; }
  if (nvalid > 0) {
    if (bias != nullptr) {
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

  // residual vectors of every pass are requested now so that their latency
  // overlaps with the staging below instead of serialising the passes
  constexpr int NPASS = 32 / PPP;
  using RVec = typename Epi::RVec;
  RVec rpre[TM][NPASS];
  const bool have_rpre = Epi::kPrefetchResidual && vec && rbase != nullptr;
  if constexpr (Epi::kPrefetchResidual) {
    if (have_rpre) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int ps = 0; ps < NPASS; ++ps) {
          const int m = tile_m * BM + wm * WM + i * 32 + ps * PPP + rp;
          const int mc = m < M ? m : M - 1;
          rpre[i][ps] = *reinterpret_cast<const RVec*>(rbase + (int64_t)mc * p.rcs + n);
        }
    }
  }

  __syncthreads();  // the K loop's LDS reads are done; the buffer becomes the staging area
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
#pragma unroll
    for (int ps = 0; ps < NPASS; ++ps) {
      const int pix = ps * PPP + rp;
      const int m = tile_m * BM + wm * WM + i * 32 + pix;
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
      if (m < M && nvalid > 0) {
        TOut* yrow = ybase + (int64_t)m * p.ycs + n;
        const TOut* rrow = rbase ? rbase + (int64_t)m * p.rcs + n : nullptr;
        Epi::store8(p, a8, nvalid, vec, b8, m8, yrow, rrow, have_rpre, rpre[i][ps]);
      }
    }
    if (i + 1 < TM) {
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
  }
}

// ---------------------------------------------------------------------------
// Host side: validation, variant choice, launch.

namespace {

struct Variant { int bm, bn; const char* name; };

template <typename TIn, typename Epi, int BM, int BN, int WM, int WN>
hipError_t launch_variant(const IgemmParams& p, int epi_vec, hipStream_t stream) {
  const int64_t M = (int64_t)p.N * p.Ho * p.Wo;
  const int64_t tiles = ((M + BM - 1) / BM) * ((p.Kout + BN - 1) / BN);
  if (tiles <= 0 || tiles > 0x7fffffff) return hipErrorInvalidValue;
  dim3 grid((unsigned)tiles, 1, (unsigned)p.batch);
  dim3 block((BM / WM) * (BN / WN) * 64);
  hipLaunchKernelGGL((igemm_kernel<TIn, Epi, BM, BN, WM, WN>), grid, block, 0, stream, p, epi_vec);
  return hipGetLastError();
}

// Tile choice: channel tile as wide as the layer allows (the pixel tile is then
// read from HBM once), pixel tile shrunk when the layer has few pixels so that
// the launch still covers the 256 CUs.
Variant choose_variant(const IgemmParams& p) {
  const int64_t M = (int64_t)p.N * p.Ho * p.Wo;
  if (p.Kout <= 32) return {128, 32, "128x32"};
  if (p.Kout <= 64) return {128, 64, "128x64"};
  const int64_t blocks128 = ((M + 127) / 128) * ((p.Kout + 127) / 128) * p.batch;
  if (blocks128 < 512) return {64, 128, "64x128"};
  return {128, 128, "128x128"};
}

template <typename TIn, typename Epi>
hipError_t dispatch_tiles(const IgemmParams& p, int epi_vec, hipStream_t s) {
  const Variant v = choose_variant(p);
  if (v.bn == 32) return launch_variant<TIn, Epi, 128, 32, 32, 32>(p, epi_vec, s);
  if (v.bn == 64) return launch_variant<TIn, Epi, 128, 64, 64, 32>(p, epi_vec, s);
  if (v.bm == 64) return launch_variant<TIn, Epi, 64, 128, 32, 64>(p, epi_vec, s);
  return launch_variant<TIn, Epi, 128, 128, 64, 64>(p, epi_vec, s);
}

bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; }

}  // namespace

const char* igemm_variant_name(const IgemmParams& p) { return choose_variant(p).name; }

hipError_t launch_igemm(const IgemmParams& p, hipStream_t stream) {
  const int es = dtype_size(p.in_dt);
  if (es == 0 || p.x == nullptr || p.w == nullptr || p.y == nullptr) return hipErrorInvalidValue;
  const int vec = 16 / es;
  if (p.C <= 0 || p.C % vec != 0 || p.xcs % vec != 0 || p.w_rs % vec != 0) return hipErrorInvalidValue;
  if (p.x_bs % vec != 0 || p.w_bs % vec != 0) return hipErrorInvalidValue;
  if (!aligned16(p.x) || !aligned16(p.w)) return hipErrorInvalidValue;
  if (p.N <= 0 || p.H <= 0 || p.W <= 0 || p.Ho <= 0 || p.Wo <= 0 || p.Kout <= 0 || p.batch <= 0)
    return hipErrorInvalidValue;
  if (p.act != ACT_NONE && p.act != ACT_RELU && p.act != ACT_LEAKY && p.act != ACT_CLAMP) return hipErrorInvalidValue;
  if (p.R <= 0 || p.S <= 0 || p.sh <= 0 || p.sw <= 0 || p.dh <= 0 || p.dw <= 0) return hipErrorInvalidValue;
  if (p.xcs < p.C || p.ycs < p.Kout) return hipErrorInvalidValue;
  if ((int64_t)p.H * p.W * p.xcs >= (1ll << 31)) return hipErrorInvalidValue;
  if ((int64_t)p.N * p.Ho * p.Wo >= (1ll << 31)) return hipErrorInvalidValue;
  if (p.w_rows <= 0 || p.w_cols <= 0 || p.w_cols > p.w_rs) return hipErrorInvalidValue;
  if (p.w_cols % vec != 0) return hipErrorInvalidValue;
  if (p.residual != nullptr && p.rcs < p.Kout) return hipErrorInvalidValue;
  // the last output pixel's receptive field must start inside the padded input
  if ((int64_t)(p.Ho - 1) * p.sh - p.ph >= p.H || (int64_t)(p.Wo - 1) * p.sw - p.pw >= p.W)
    return hipErrorInvalidValue;

  const int oes = dtype_size(p.out_dt);
  // Eight consecutive output elements are accessed as one vector (16 bytes, or
  // 8 bytes for 8-bit output, two 16-byte vectors for 4-byte output) when rows
  // and base pointers are aligned accordingly.
  const int64_t vbytes = oes == 1 ? 8 : 16;
  auto rows_ok = [&](const void* ptr, int64_t cs, int64_t bs) {
    return ((cs * oes) % vbytes == 0) && ((bs * oes) % vbytes == 0) &&
           ((reinterpret_cast<uintptr_t>(ptr) % (uintptr_t)vbytes) == 0);
  };
  int epi_vec = rows_ok(p.y, p.ycs, p.y_bs);
  if (p.residual != nullptr) epi_vec = epi_vec && rows_ok(p.residual, p.rcs, p.r_bs);
  if (p.bias != nullptr) epi_vec = epi_vec && ((reinterpret_cast<uintptr_t>(p.bias) % 16) == 0) && (p.bias_bs % 4 == 0);

  switch (p.in_dt) {
    case DT_F32:
      if (p.out_dt != DT_F32) return hipErrorInvalidValue;
      return dispatch_tiles<float, EpiFloat<float>>(p, epi_vec, stream);
    case DT_F16:
      if (p.out_dt == DT_F16) return dispatch_tiles<f16_t, EpiFloat<f16_t>>(p, epi_vec, stream);
      if (p.out_dt == DT_F32) return dispatch_tiles<f16_t, EpiFloat<float>>(p, epi_vec, stream);
      return hipErrorInvalidValue;
    case DT_BF16:
      if (p.out_dt == DT_BF16) return dispatch_tiles<bf16_t, EpiFloat<bf16_t>>(p, epi_vec, stream);
      if (p.out_dt == DT_F32) return dispatch_tiles<bf16_t, EpiFloat<float>>(p, epi_vec, stream);
      return hipErrorInvalidValue;
    case DT_I8:
      if (p.out_dt == DT_I8) {
        if (p.qmul == nullptr) return hipErrorInvalidValue;
        return dispatch_tiles<int8_t, EpiQuant<0>>(p, epi_vec, stream);
      }
      if (p.out_dt == DT_F32) {
        if (p.qmul == nullptr) return hipErrorInvalidValue;
        return dispatch_tiles<int8_t, EpiQuant<1>>(p, 0, stream);
      }
      if (p.out_dt == DT_I32) return dispatch_tiles<int8_t, EpiQuant<2>>(p, 0, stream);
      return hipErrorInvalidValue;
    default:
      return hipErrorInvalidValue;
  }
}

// ---------------------------------------------------------------------------
// Weight repacking: dst[g][o][ (r*S+s)*Cp + c ] = src(o_global, c, r, s), zero
// elsewhere (padded channels, padded rows, padded row tail).

template <typename TS, typename TD>
__device__ __forceinline__ TD cvt_weight(TS v);
template <> __device__ __forceinline__ float cvt_weight<float, float>(float v) { return v; }
template <> __device__ __forceinline__ f16_t cvt_weight<float, f16_t>(float v) { return f16_t{f32_to_f16(v)}; }
template <> __device__ __forceinline__ bf16_t cvt_weight<float, bf16_t>(float v) { return bf16_t{f32_to_bf16(v)}; }
template <> __device__ __forceinline__ f16_t cvt_weight<f16_t, f16_t>(f16_t v) { return v; }
template <> __device__ __forceinline__ bf16_t cvt_weight<bf16_t, bf16_t>(bf16_t v) { return v; }
template <> __device__ __forceinline__ float cvt_weight<f16_t, float>(f16_t v) { return f16_to_f32(v.bits); }
template <> __device__ __forceinline__ float cvt_weight<bf16_t, float>(bf16_t v) { return bf16_to_f32(v.bits); }
template <> __device__ __forceinline__ int8_t cvt_weight<int8_t, int8_t>(int8_t v) { return v; }

template <typename TS, typename TD>
__global__ void pack_weights_kernel(PackWeightsParams p) {
  const int64_t total = (int64_t)p.G * p.rows_pad * p.w_rs;
  const int taps = p.R * p.S;
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int col = (int)(i % p.w_rs);
    const int64_t rowg = i / p.w_rs;
    const int o = (int)(rowg % p.rows_pad);
    const int g = (int)(rowg / p.rows_pad);
    const int tap = col / p.Cp;
    const int c = col - tap * p.Cp;
    TD out;
    __builtin_memset(&out, 0, sizeof(TD));
    if (o < p.Og && tap < taps && c < p.Cg) {
      const int r = tap / p.S, s = tap - r * p.S;
      const int64_t og = (int64_t)g * p.Og + o;
      const TS v = reinterpret_cast<const TS*>(p.src)[og * p.so + c * p.si + r * p.sr + s * p.ss];
      out = cvt_weight<TS, TD>(v);
    }
    reinterpret_cast<TD*>(p.dst)[i] = out;
  }
}

hipError_t launch_pack_weights(const PackWeightsParams& p, hipStream_t stream) {
  if (p.src == nullptr || p.dst == nullptr) return hipErrorInvalidValue;
  if (p.G <= 0 || p.Og <= 0 || p.Cg <= 0 || p.Cp < p.Cg || p.rows_pad < p.Og) return hipErrorInvalidValue;
  if ((int64_t)p.R * p.S * p.Cp > p.w_rs) return hipErrorInvalidValue;
  const int64_t total = (int64_t)p.G * p.rows_pad * p.w_rs;
  const int grid = grid_for(total, 256);
#define PACK_CASE(S_, D_, TS_, TD_)                                                      \
  if (p.src_dt == S_ && p.dst_dt == D_) {                                                \
    hipLaunchKernelGGL((pack_weights_kernel<TS_, TD_>), dim3(grid), dim3(256), 0, stream, p); \
    return hipGetLastError();                                                            \
  }
  PACK_CASE(DT_F32, DT_F32, float, float)
  PACK_CASE(DT_F32, DT_F16, float, f16_t)
  PACK_CASE(DT_F32, DT_BF16, float, bf16_t)
  PACK_CASE(DT_F16, DT_F16, f16_t, f16_t)
  PACK_CASE(DT_BF16, DT_BF16, bf16_t, bf16_t)
  PACK_CASE(DT_F16, DT_F32, f16_t, float)
  PACK_CASE(DT_BF16, DT_F32, bf16_t, float)
  PACK_CASE(DT_I8, DT_I8, int8_t, int8_t)
#undef PACK_CASE
  return hipErrorInvalidValue;
}

}  // namespace ohip
