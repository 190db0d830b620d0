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
// Epilogues.  Each handles four consecutive output channels n..n+3 of one
// output row; `full` says all four are in range and 16-byte style access is ok.

template <typename TOut>
struct EpiFloat {
  using AccE = float;
  __device__ static __forceinline__ void run(const IgemmParams& p, const float* acc, int n,
                                             const float* bias4, void* yrow, const void* rrow,
                                             bool full) {
    float v[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = acc[e] * p.alpha + bias4[e];
    TOut* y = reinterpret_cast<TOut*>(yrow) + n;
    const TOut* r = reinterpret_cast<const TOut*>(rrow) + n;
    if (full) {
      if (rrow != nullptr) {
        if constexpr (sizeof(TOut) == 4) {
          floatx4 rv = *reinterpret_cast<const floatx4*>(r);
          v[0] += rv.x; v[1] += rv.y; v[2] += rv.z; v[3] += rv.w;
        } else {
          uintx2 rv = *reinterpret_cast<const uintx2*>(r);
          const TOut* re = reinterpret_cast<const TOut*>(&rv);
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] += Store<TOut>::ld(re + e);
        }
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = apply_act(v[e], p.act, p.act_a, p.act_b);
      if constexpr (sizeof(TOut) == 4) {
        floatx4 o = {v[0], v[1], v[2], v[3]};
        *reinterpret_cast<floatx4*>(y) = o;
      } else {
        uintx2 o;
        TOut* oe = reinterpret_cast<TOut*>(&o);
#pragma unroll
        for (int e = 0; e < 4; ++e) Store<TOut>::st(oe + e, v[e]);
        *reinterpret_cast<uintx2*>(y) = o;
      }
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (n + e < p.Kout) {
          float t = v[e];
          if (rrow != nullptr) t += Store<TOut>::ld(r + e);
          Store<TOut>::st(y + e, apply_act(t, p.act, p.act_a, p.act_b));
        }
      }
    }
  }
};

// int8 operands, int32 accumulators.  MODE 0: requantised 8-bit output (stored
// q-128), MODE 1: dequantised fp32 output, MODE 2: raw int32 accumulators.
template <int MODE>
struct EpiQuant {
  using AccE = int;
  __device__ static __forceinline__ int requant(const IgemmParams& p, int acc, float mul) {
    float r = (float)acc * mul;          // v_cvt_f32_i32 (RNE) then one v_mul_f32
    int q = (int)rintf(r) + p.q_zp;      // v_rndne_f32
    q = q < p.q_lo ? p.q_lo : q;
    q = q > 255 ? 255 : q;
    return q;
  }
  __device__ static __forceinline__ void run(const IgemmParams& p, const int* acc, int n,
                                             const int* bias4, void* yrow, const void* rrow,
                                             bool full) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (!full && n + e >= p.Kout) continue;
      const int a = acc[e] + bias4[e];
      if constexpr (MODE == 2) {
        reinterpret_cast<int*>(yrow)[n + e] = a;
      } else if constexpr (MODE == 1) {
        float f = (float)a * p.qmul[n + e];
        if (rrow != nullptr) f += reinterpret_cast<const float*>(rrow)[n + e];
        reinterpret_cast<float*>(yrow)[n + e] = apply_act(f, p.act, p.act_a, p.act_b);
      } else {
        int q = requant(p, a, p.qmul[n + e]);
        if (rrow != nullptr) {
          const int rq = q_from_stored(reinterpret_cast<const int8_t*>(rrow)[n + e]);
          const float fa = (float)(q - p.q_zp) * p.q_scale;
          const float fb = (float)(rq - p.r_zp) * p.r_scale;
          const float f = fa + fb;
          q = (int)rintf(f * p.s_inv) + p.s_zp;
          q = q < p.s_lo ? p.s_lo : q;
          q = q > 255 ? 255 : q;
        }
        reinterpret_cast<int8_t*>(yrow)[n + e] = q_to_stored(q);
      }
    }
  }
};

template <typename Epi> struct EpiOutSize;
template <typename T> struct EpiOutSize<EpiFloat<T>> { static constexpr int v = sizeof(T); };
template <> struct EpiOutSize<EpiQuant<0>> { static constexpr int v = 1; };
template <> struct EpiOutSize<EpiQuant<1>> { static constexpr int v = 4; };
template <> struct EpiOutSize<EpiQuant<2>> { static constexpr int v = 4; };

// ---------------------------------------------------------------------------
template <typename TIn, typename Epi, int BM, int BN, int WM, int WN>
__global__ void __launch_bounds__((BM / WM) * (BN / WN) * 64)
igemm_kernel(const IgemmParams p, const int epi_vec) {
  constexpr int NW = (BM / WM) * (BN / WN);
  constexpr int NT = NW * 64;
  constexpr int ES = sizeof(TIn);
  constexpr int VEC = 16 / ES;   // elements per 16-byte vector
  constexpr int BKB = 64;        // bytes of K per row per stage
  constexpr int BK = BKB / ES;   // elements of K per stage
  constexpr int ROWB = BKB + 16; // LDS row pitch in bytes
  constexpr int VPR = BKB / 16;  // vectors per row
  constexpr int RPP = NT / VPR;  // rows loaded per pass
  constexpr int A_IT = (BM + RPP - 1) / RPP, B_IT = (BN + RPP - 1) / RPP;
  static_assert(BM % RPP == 0 || BM < RPP, "pixel tile must be a multiple of the rows per pass");
  static_assert(BN % RPP == 0 || BN < RPP, "channel tile must be a multiple of the rows per pass");
  constexpr int TM = WM / 32, TN = WN / 32;
  using Acc = typename Mma<TIn>::Acc;
  using AccE = typename Epi::AccE;

  __shared__ __attribute__((aligned(16))) unsigned char smem[2 * (BM + BN) * ROWB];
  unsigned char* As = smem;
  unsigned char* Bs = smem + 2 * BM * ROWB;

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
  auto lds_store = [&](int buf) {
    unsigned char* ab = As + buf * (BM * ROWB) + row0 * ROWB + kv * 16;
#pragma unroll
    for (int i = 0; i < A_IT; ++i)
      if (BM % RPP == 0 || row0 + i * RPP < BM) *reinterpret_cast<uintx4*>(ab + i * RPP * ROWB) = ra[i];
    unsigned char* bb = Bs + buf * (BN * ROWB) + row0 * ROWB + kv * 16;
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

  gload();
  lds_store(0);
  __syncthreads();
  for (int kt = 0; kt < nkt; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < nkt) gload();
    const unsigned char* ab = As + buf * (BM * ROWB) + (wm * WM + l32) * ROWB + lg * 16;
    const unsigned char* bb = Bs + buf * (BN * ROWB) + (wn * WN + l32) * ROWB + lg * 16;
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
    if (kt + 1 < nkt) lds_store(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue ----
  constexpr int OES = EpiOutSize<Epi>::v;
  unsigned char* ybase = reinterpret_cast<unsigned char*>(p.y) + (int64_t)z * p.y_bs * OES;
  const unsigned char* rbase =
      p.residual ? reinterpret_cast<const unsigned char*>(p.residual) + (int64_t)z * p.r_bs * OES : nullptr;
  const AccE* bias = p.bias ? reinterpret_cast<const AccE*>(p.bias) + (int64_t)z * p.bias_bs : nullptr;

#pragma unroll
  for (int j = 0; j < TN; ++j) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int n = tile_n * BN + wn * WN + j * 32 + q * 8 + lg * 4;
      if (n >= p.Kout) continue;
      AccE b4[4] = {0, 0, 0, 0};
      if (bias != nullptr) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (n + e < p.Kout) b4[e] = bias[n + e];
      }
      const bool full = epi_vec && (n + 3 < p.Kout);
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int m = tile_m * BM + wm * WM + i * 32 + l32;
        if (m >= M) continue;
        AccE a4[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) a4[e] = acc[i][j][q * 4 + e];
        void* yrow = ybase + (int64_t)m * p.ycs * OES;
        const void* rrow = rbase ? rbase + (int64_t)m * p.rcs * OES : nullptr;
        Epi::run(p, a4, n, b4, yrow, rrow, full);
      }
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
  // Four consecutive output elements are accessed as one vector when this holds.
  int epi_vec = (p.ycs % 4 == 0) && (p.y_bs % 4 == 0) &&
                ((reinterpret_cast<uintptr_t>(p.y) & (uintptr_t)(4 * oes - 1)) == 0);
  if (p.residual != nullptr)
    epi_vec = epi_vec && (p.rcs % 4 == 0) && (p.r_bs % 4 == 0) &&
              ((reinterpret_cast<uintptr_t>(p.residual) & (uintptr_t)(4 * oes - 1)) == 0);

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
        return dispatch_tiles<int8_t, EpiQuant<0>>(p, 0, stream);
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
