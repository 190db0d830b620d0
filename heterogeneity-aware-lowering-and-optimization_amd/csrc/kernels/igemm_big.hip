// Implicit-GEMM convolution / GEMM with large workgroup tiles for the layers
// that are bound by the matrix cores.
//
// A CU's vector-memory path delivers about 64 bytes per clock while its four
// matrix pipes consume a 128 x 128 tile's operands at exactly that rate, so a
// 128 x 128 workgroup tile cannot pass half of the MFMA peak however well it
// is pipelined.  Here a workgroup owns 256 x 256 (or 256 x 128 / 128 x 256)
// outputs, i.e. fetches half as many operand bytes per MFMA, and
//   - BOTH operands arrive by direct-to-LDS loads (global_load_lds_dwordx4: no
//     registers, no LDS store instructions) into a ring of STAGES buffers of
//     64 bytes of K per row, STAGES-1 stages ahead of their use;
//   - every wavefront computes a 128 x 64 block of the tile (4 x 2 MFMA blocks
//     of 32 x 32: six 16-byte fragment reads feed eight MFMAs);
//   - the one workgroup barrier per stage sits in the MIDDLE of the stage's
//     MFMAs: a wavefront issues the first half of a stage's MFMAs, then waits
//     for the next stage's data and for its neighbours, requests a new stage
//     into the buffer everybody has left, reads the first fragments of the next
//     stage and issues the second half - the matrix pipe stays fed across the
//     barrier and the fragment reads behind it.
//
// LDS layout of a stage: row r of the combined operand tile (pixel rows first,
// then weight rows; 64 bytes = four 16-byte chunks each) at r * 64, chunk c in
// slot c ^ ((r >> 2) & 3).  A direct-to-LDS load writes lane l of a wavefront at
// base + 16 l, i.e. one request fills 16 rows and lane l fetches, for row l / 4,
// the chunk that belongs in slot l % 4; the fragment reads of 16 consecutive
// rows then fall into 16 distinct 16-byte bank groups.
//
// The pixel operand is gathered on the fly (implicit im2col): the input
// channels of one filter tap are contiguous (channels-last activations), the
// tap walk is wavefront-uniform, a thread keeps one address and one validity
// mask per row it feeds; padding taps and rows beyond the tensor fetch a
// 16-byte fill vector.  Requirements (checked by igemm_big_variant): constant
// row-major weights [Cout][w_rs], C * sizeof(T) a multiple of 64, at most 32
// taps.
#include "igemm_common.h"

#include <cstdlib>
#include <cstring>

namespace ohip {

// 16-byte vectors of every byte value: the fill for padding taps (0 for the
// floating-point types, the stored byte of the zero point for 8-bit tensors).
struct FillTable { unsigned char v[256][16]; };
constexpr FillTable make_fill_table() {
  FillTable t{};
  for (int b = 0; b < 256; ++b)
    for (int i = 0; i < 16; ++i) t.v[b][i] = (unsigned char)b;
  return t;
}
static __device__ const FillTable g_fill_table = make_fill_table();

template <typename TIn, typename Epi, int BM, int BN, int WAVES_M, int WAVES_N, int STAGES>
// two wavefronts per SIMD (one workgroup of eight, or two of four): 256 registers
__global__ void __launch_bounds__(WAVES_M* WAVES_N * 64, 2)
igemm_big_kernel(const IgemmParams p, const int epi_vec) {
  constexpr int NW = WAVES_M * WAVES_N;
  constexpr int ES = sizeof(TIn);
  constexpr int BKB = 64, BK = BKB / ES;  // K per stage, bytes / elements
  constexpr int VEC = 16 / ES;
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int ROWS = BM + BN;
  constexpr int STAGE_BYTES = ROWS * BKB;
  constexpr int NREQ = ROWS / 16 / NW;       // direct-to-LDS requests per wavefront and stage
  constexpr int NREQ_A = BM / 16 / NW;       // ... of which the first NREQ_A feed pixel rows
  constexpr int D = STAGES - 1;              // stages requested ahead
  static_assert((BM / 16) % NW == 0 && (BN / 16) % NW == 0, "whole requests per wavefront and operand");
  static_assert(D >= 2, "at least three buffers");
  constexpr int EPI_BYTES = NW * 32 * (WN + 4) * 4;
  static_assert(STAGES * STAGE_BYTES >= EPI_BYTES, "epilogue staging must fit in the ring");
  using Acc = typename Mma<TIn>::Acc;
  // s_waitcnt immediates (vmcnt only; expcnt / lgkmcnt left at their maxima)
  constexpr int kWaitLanded = 0x0f70 | ((D - 1) * NREQ);      // at most D-1 younger stages in flight
  static_assert((D - 1) * NREQ < 16, "vmcnt immediate");

  __shared__ __attribute__((aligned(1024))) unsigned char smem[STAGES * STAGE_BYTES];

  const int tid = threadIdx.x;
  const int M = p.N * p.Ho * p.Wo;
  const int tiles_n = (p.Kout + BN - 1) / BN;
  // Workgroups are dealt round-robin to the 8 XCDs; renumber them so that the
  // channel tiles of one pixel tile and neighbouring pixel tiles share an L2.
  int bid = blockIdx.x;
  {
    const int per = gridDim.x >> 3;
    if (bid < (per << 3)) bid = (bid & 7) * per + (bid >> 3);
  }
  const int tile_n = bid % tiles_n;
  const int tile_m = bid / tiles_n;
  const int z = blockIdx.z;
  const int wave = tid >> 6, lane = tid & 63;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int wm = wave_u % WAVES_M, wn = wave_u / WAVES_M;  // the numbering igemm_epilogue uses
  const int l32 = lane & 31, lg = lane >> 5;

  const TIn* x = reinterpret_cast<const TIn*>(p.x) + (int64_t)z * p.x_bs;
  const TIn* w = reinterpret_cast<const TIn*>(p.w) + (int64_t)z * p.w_bs;
  const uint64_t fill_u = reinterpret_cast<uint64_t>(&g_fill_table.v[p.a_fill & 0xff][0]);

  // ---- what this thread feeds: request i covers rows (i * NW + wave) * 16 .. + 15 of the
  // combined tile; the thread supplies row (lane / 4) of them, slot lane % 4 ----
  const int rrow = lane >> 2;
  uint64_t src[NREQ];       // pixel rows: address of the chunk at tap (0,0), channel 0 (may lie outside the image);
                            // weight rows: address of the chunk at k = 0
  unsigned amask[NREQ];     // pixel rows: one validity bit per tap
  const int HoWo = p.Ho * p.Wo;
#pragma unroll
  for (int i = 0; i < NREQ; ++i) {
    const int row = (i * NW + wave_u) * 16 + rrow;  // row of the combined tile
    const int kv = (lane & 3) ^ ((row >> 2) & 3);   // the chunk that belongs in this lane's slot
    if (i < NREQ_A) {
      const int m = tile_m * BM + row;
      const bool ok = m < M;
      const int mm = ok ? m : 0;
      const int n_img = fast_div(mm, p.howo_magic, p.howo_shift);
      const int rem = mm - n_img * HoWo;
      const int ho = fast_div(rem, p.wo_magic, p.wo_shift);
      const int wo = rem - ho * p.Wo;
      const int hi0 = ho * p.sh - p.ph, wi0 = wo * p.sw - p.pw;
      src[i] = reinterpret_cast<uint64_t>(x + (((int64_t)n_img * p.H + hi0) * p.W + wi0) * p.xcs + kv * VEC);
      unsigned mask = 0u;
      int t = 0;
      for (int r = 0; r < p.R; ++r)
        for (int q = 0; q < p.S; ++q, ++t) {
          const int hi = hi0 + r * p.dh, wi = wi0 + q * p.dw;
          if (ok && (unsigned)hi < (unsigned)p.H && (unsigned)wi < (unsigned)p.W) mask |= 1u << t;
        }
      amask[i] = mask;
    } else {
      int n = tile_n * BN + (row - BM);
      n = n < p.w_rows ? n : p.w_rows - 1;  // rows past the end are computed but never stored
      src[i] = reinterpret_cast<uint64_t>(w + (int64_t)n * p.w_rs + kv * VEC);
    }
  }

  // ---- requests of one stage; all bookkeeping is wavefront-uniform and incremental ----
  using lds_ptr = __attribute__((address_space(3))) void*;
  const int RS = p.R * p.S;
  const int nkt = RS * (p.C / BK);   // stages of the whole reduction (C is a multiple of BK)
  int ld_kt = 0;                     // stage the next call requests
  int tap = 0, tap_s = 0, kc0 = 0;
  int toff = 0;                      // element offset of (tap, kc0) from tap (0,0), channel 0
  unsigned tapbit = 1u;              // 1 << tap, 0 behind the last tap
  const int step_s = p.dw * p.xcs;
  const int step_r = p.dh * p.W * p.xcs - (p.S - 1) * step_s;
  auto dma = [&](const int buf) {
    unsigned char* dst = smem + buf * STAGE_BYTES + wave_u * 1024;
    const bool live = ld_kt < nkt;   // requests past the reduction (the pipeline's run-out) fetch the fill vector
    const int64_t woff = (int64_t)ld_kt * BKB;
#pragma unroll
    for (int i = 0; i < NREQ; ++i) {
      uint64_t a;
      if (i < NREQ_A) a = (amask[i] & tapbit) != 0u ? src[i] + (int64_t)toff * ES : fill_u;
      else a = live ? src[i] + woff : fill_u;
#if defined(__HIP_DEVICE_COMPILE__)  // (the builtin is unknown to the host pass, which only needs the launch stub)
      __builtin_amdgcn_global_load_lds(reinterpret_cast<const TIn*>(a), (lds_ptr)(dst + i * (NW * 1024)), 16, 0, 0);
#else
      (void)a; (void)dst;
#endif
    }
    ++ld_kt;
    kc0 += BK;
    toff += BK;
    if (kc0 >= p.C) {
      kc0 = 0;
      toff -= p.C;
      ++tap;
      tapbit = tap < RS ? tapbit << 1 : 0u;
      if (++tap_s == p.S) { tap_s = 0; toff += step_r; }
      else toff += step_s;
    }
  };

  Acc acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

  if constexpr (EpiTraits<Epi>::quant) acc_init_bias<TM, TN>(p, z, tile_n * BN + wn * WN, lg, acc);

  // fragment read offsets inside a stage: row (l32 + 32 i), chunk 2 kk + lg, swizzled by the row
  const int sw = (l32 >> 2) & 3;
  const int rd0 = l32 * BKB + ((lg ^ sw) << 4);        // kk = 0
  const int rd1 = l32 * BKB + (((2 + lg) ^ sw) << 4);  // kk = 1
  const int a_base = wm * WM * BKB, b_base = (BM + wn * WN) * BKB;
  const unsigned lds0 = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)smem;

  // Fragment reads and their waits are issued by hand.  Left to the compiler, every
  // wait for LDS data in this loop becomes a wait for ALL LDS data in flight - the
  // fragments just requested for the next half included - which leaves the matrix
  // pipe idle for an LDS round trip twice per stage.  LDS operations return in
  // order, so "at most six younger requests outstanding" is exact.  A request names
  // its register quad as output; the matching wait names the quads it releases as
  // input and output, so the compiler sees them occupied from the request to the
  // wait and orders the MFMAs behind the wait.  (The host pass only needs the
  // kernel's launch stub; it cannot parse the vector-register constraints.)
#if defined(__HIP_DEVICE_COMPILE__)
#define BIG_DS_READ(dst, addr, OFF) asm volatile("ds_read_b128 %0, %1 offset:" #OFF : "=v"(dst) : "v"(addr))
#else
#define BIG_DS_READ(dst, addr, OFF) (dst) = uintx4{(unsigned)(addr), 0u, 0u, 0u}
#endif
  auto read4 = [&](uintx4& dst, const unsigned addr, const int k) __attribute__((always_inline)) {
    if (k == 0) BIG_DS_READ(dst, addr, 0);
    else if (k == 1) BIG_DS_READ(dst, addr, 2048);
    else if (k == 2) BIG_DS_READ(dst, addr, 4096);
    else BIG_DS_READ(dst, addr, 6144);
  };
  static_assert(TM <= 4 && TN <= 4 && 32 * BKB == 2048, "offsets of read4");
  auto read_frags = [&](const int buf, const int rd, uintx4 (&fa)[TM], uintx4 (&fb)[TN]) __attribute__((always_inline)) {
    const unsigned s = lds0 + buf * STAGE_BYTES + rd;
    const unsigned sa = s + a_base, sb = s + b_base;
#pragma unroll
    for (int i = 0; i < TM; ++i) read4(fa[i], sa, i);
#pragma unroll
    for (int j = 0; j < TN; ++j) read4(fb[j], sb, j);
  };
  // fa / fb are valid once at most TM + TN younger requests (the other fragment set) are in flight
  static_assert(TM == 4 || TM == 2, "wait_frags names the fragments one by one");
  static_assert(TN == 2, "wait_frags names the fragments one by one");
  auto wait_frags = [&](uintx4 (&fa)[TM], uintx4 (&fb)[TN], const bool all) __attribute__((always_inline)) {
#if defined(__HIP_DEVICE_COMPILE__)
    if constexpr (TM == 4) {
      if (all)
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(fa[0]), "+v"(fa[1]), "+v"(fa[2]), "+v"(fa[3]), "+v"(fb[0]), "+v"(fb[1]));
      else
        asm volatile("s_waitcnt lgkmcnt(6)" : "+v"(fa[0]), "+v"(fa[1]), "+v"(fa[2]), "+v"(fa[3]), "+v"(fb[0]), "+v"(fb[1]));
    } else {
      if (all)
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(fa[0]), "+v"(fa[1]), "+v"(fb[0]), "+v"(fb[1]));
      else
        asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(fa[0]), "+v"(fa[1]), "+v"(fb[0]), "+v"(fb[1]));
    }
#else
    (void)fa; (void)fb; (void)all;
#endif
  };
  auto mma_all = [&](const uintx4 (&fa)[TM], const uintx4 (&fb)[TN]) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) acc[i][j] = Mma<TIn>::run(fb[j], fa[i], acc[i][j]);
  };
  auto fence = [&]() __attribute__((always_inline)) {
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("" ::: "memory");
  };

  // pipeline fill: stages 0 .. D-1 requested, stage 0 landed for everybody
#pragma unroll
  for (int s = 0; s < D; ++s) dma(s);
  fence();
  __builtin_amdgcn_s_waitcnt(kWaitLanded);
  fence();
  __builtin_amdgcn_s_barrier();
  fence();
  uintx4 fa0[TM], fb0[TN], fa1[TM], fb1[TN];
  read_frags(0, rd0, fa0, fb0);

  int buf = 0;       // buffer of stage kt
  int nxt = 1;       // buffer of stage kt + 1
  int refill = D;    // buffer of stage kt + D: the one stage kt - 1 was read from
  for (int kt = 0; kt < nkt; ++kt) {
    // first half of the stage: the second half's fragments are requested before the
    // first half's MFMAs are issued, so that the reads have the whole half to return,
    // behind the MFMAs of both wavefronts of the SIMD
    read_frags(buf, rd1, fa1, fb1);
    wait_frags(fa0, fb0, false);
    mma_all(fa0, fb0);
    fence();
    // the next stage has landed (mine: at most D-2 younger stages in flight), and
    // everybody's has; everybody has also finished the reads of stage kt - 1, whose
    // buffer the next requests go to
    __builtin_amdgcn_s_waitcnt(0x0f70 | ((D - 2) * NREQ));
    fence();
    __builtin_amdgcn_s_barrier();
    fence();
    dma(refill);
    fence();
    // second half, likewise
    read_frags(nxt, rd0, fa0, fb0);
    wait_frags(fa1, fb1, false);
    mma_all(fa1, fb1);
    fence();
    buf = nxt;
    nxt = nxt + 1 == STAGES ? 0 : nxt + 1;
    refill = refill + 1 == STAGES ? 0 : refill + 1;
  }
  // The fragments requested last belong to a run-out stage and are not used, but they
  // must have arrived before their registers serve another purpose.
  wait_frags(fa0, fb0, true);
  fence();
#undef BIG_DS_READ
  igemm_epilogue<TIn, Epi, BM, BN, WM, WN>(p, epi_vec, acc, smem, tile_m, tile_n, z, M, wave, lane);
}

// ---------------------------------------------------------------------------
namespace {

template <typename TIn, typename Epi, int BM, int BN, int WAVES_M, int WAVES_N, int STAGES>
hipError_t launch_one(const IgemmParams& p, int epi_vec, hipStream_t stream) {
  const int64_t M = (int64_t)p.N * p.Ho * p.Wo;
  const int64_t tiles = ((M + BM - 1) / BM) * ((p.Kout + BN - 1) / BN);
  if (tiles <= 0 || tiles > 0x7fffffff) return hipErrorInvalidValue;
  hipLaunchKernelGGL((igemm_big_kernel<TIn, Epi, BM, BN, WAVES_M, WAVES_N, STAGES>), dim3((unsigned)tiles, 1, (unsigned)p.batch),
                     dim3(WAVES_M * WAVES_N * 64), 0, stream, p, epi_vec);
  return hipGetLastError();
}

template <typename TIn, typename Epi>
hipError_t launch_variant(const IgemmParams& p, int epi_vec, int variant, hipStream_t stream) {
  switch (variant) {
    case 1: return launch_one<TIn, Epi, 256, 256, 2, 4, 4>(p, epi_vec, stream);
    case 2: return launch_one<TIn, Epi, 256, 128, 2, 2, 3>(p, epi_vec, stream);
    case 3: return launch_one<TIn, Epi, 128, 256, 1, 4, 3>(p, epi_vec, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace

// 0: the shape is not for these kernels; 1: 256 x 256, 2: 256 pixels x 128 channels,
// 3: 128 pixels x 256 channels.
int igemm_big_variant(const IgemmParams& p) {
  const int es = dtype_size(p.in_dt);
  if (p.in_dt != DT_F16 && p.in_dt != DT_BF16 && p.in_dt != DT_I8) return 0;
  if (p.out_dt != p.in_dt) return 0;
  // (the transcendental epilogues are instantiated for bf16 only: the feed-forward GEMMs of the encoder)
  const bool rich = p.act == ACT_GELU_ERF || p.act == ACT_GELU_TANH || p.act == ACT_SIGMOID || p.act == ACT_TANH;
  if (rich && p.in_dt != DT_BF16) return 0;
  if ((p.C * es) % 64 != 0 || (p.w_rs * es) % 64 != 0 || p.R * p.S > 32) return 0;
  if ((int64_t)p.R * p.S * p.C > p.w_rs || p.w_cols != p.R * p.S * p.C) return 0;
  if ((p.w_bs * es) % 16 != 0 || (p.x_bs * es) % 16 != 0) return 0;
  const char* force = getenv("ODLA_HIP_IGEMM_TILE");  // tuning aid
  if (force != nullptr && force[0] != 0) {
    if (strcmp(force, "big256x256") == 0) return 1;
    if (strcmp(force, "big256x128") == 0) return 2;
    if (strcmp(force, "big128x256") == 0) return 3;
    return 0;
  }
  return 0;
}

hipError_t launch_igemm_big(const IgemmParams& p, int epi_vec, int variant, hipStream_t stream) {
  const bool rich = p.act == ACT_GELU_ERF || p.act == ACT_GELU_TANH || p.act == ACT_SIGMOID || p.act == ACT_TANH;
  switch (p.in_dt) {
    case DT_F16:
      if (rich) return hipErrorInvalidValue;
      return launch_variant<f16_t, EpiFloat<f16_t>>(p, epi_vec, variant, stream);
    case DT_BF16:
      if (rich) return launch_variant<bf16_t, EpiFloat<bf16_t, true>>(p, epi_vec, variant, stream);
      return launch_variant<bf16_t, EpiFloat<bf16_t>>(p, epi_vec, variant, stream);
    case DT_I8:
      if (p.qmul == nullptr) return hipErrorInvalidValue;
      return launch_variant<int8_t, EpiQuant<0>>(p, epi_vec, variant, stream);
    default:
      return hipErrorInvalidValue;
  }
}

}  // namespace ohip
