// Implicit-GEMM convolution / GEMM for gfx950 (CDNA4) matrix cores.
//
// Two kernels cover odla_Conv and odla_Gemm for fp32, fp16, bf16 and int8
// operands.  Activations are channels-last, so the reduction index
// k = (r, s, c) is contiguous in c and every global load is a 16-byte vector;
// a workgroup owns a tile of BM pixels x BN output channels built from 32x32
// MFMA blocks, 128 bytes of K per row and stage.
//   igemm_kernel       both operands staged through LDS from registers (rows
//                      padded to 144 bytes so that the 16-byte fragment reads of
//                      16 consecutive lanes fall into distinct banks), one stage
//                      of register prefetch; any shape.
//   igemm_wreg_kernel  constant weights read in MFMA fragment order straight
//                      into registers, pixel tile through a ring of
//                      direct-to-LDS loads, two stages ahead; layers with more
//                      than 64 output channels.
//
// The weight rows are the MFMA "A" operand and the pixel rows the "B" operand:
// in the 32x32 accumulator layout lane l then holds, for pixel (l % 32), groups
// of four consecutive output channels, which is what a channels-last store
// wants.  Both operands use the same k -> (lane group, element) assignment, so
// the exact k permutation inside one MFMA is irrelevant to the result.
#include "igemm_common.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <type_traits>

namespace ohip {

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
// (the 128 x 128 tile is held to three wavefronts per SIMD: 168 registers)
__global__ void __launch_bounds__((BM / WM) * (BN / WN) * 64, (BM == 128 && BN == 128) ? 3 : 1)
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
    const int n_img = fast_div(mm, p.howo_magic, p.howo_shift);
    const int rem = mm - n_img * HoWo;
    const int ho = fast_div(rem, p.wo_magic, p.wo_shift);
    const int wo = rem - ho * p.Wo;
    a_hi0[i] = ok ? ho * p.sh - p.ph : -(1 << 28);  // out-of-range rows never pass the bounds test
    a_wi0[i] = wo * p.sw - p.pw;
    // address of tap (0, 0), channel 0 of this row - possibly outside the image, and only
    // dereferenced behind the bounds test: a stage then adds one per-thread tap offset
    // instead of multiplying out (hi * W + wi) * xcs per row (integer multiplies run at a
    // quarter of the VALU rate)
    a_ptr[i] = x + ((int64_t)n_img * p.H * p.W + (int64_t)(ok ? ho * p.sh - p.ph : 0) * p.W + a_wi0[i]) * p.xcs;
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
    const int toff = (hoff * p.W + woff) * p.xcs + kc;   // from tap (0, 0), channel 0
#pragma unroll
    for (int i = 0; i < A_IT; ++i) {
      const int hi = a_hi0[i] + hoff, wi = a_wi0[i] + woff;
      const bool ok = (kr < p.R) && ((unsigned)hi < (unsigned)p.H) && ((unsigned)wi < (unsigned)p.W);
      ra[i] = ok ? *reinterpret_cast<const uintx4*>(a_ptr[i] + toff) : fillv;
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

  if constexpr (EpiTraits<Epi>::quant)
    acc_init_bias_vec<TM, TN>(p, z, tile_n * BN + __builtin_amdgcn_readfirstlane(wn) * WN, lg, acc);

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

  igemm_epilogue<TIn, Epi, BM, BN, WM, WN>(p, epi_vec, acc, smem, tile_m, tile_n, z, M, wave, lane);
}

// ---------------------------------------------------------------------------
// Variant for constant weights: a deeper pipeline with less LDS traffic.
//
// Measured on this part, LDS stores from registers run at a quarter of the LDS
// load rate, and one K stage of register prefetch does not cover the latency of
// the gathered pixel loads, so a kernel that stages both operands through
// registers into LDS is bound by exactly those two things.  Here
//   - only the 128-pixel tile goes through LDS, written by direct-to-LDS global
//     loads (no registers, no LDS store instructions) into a ring of three
//     buffers, two K stages ahead of its use, one barrier per stage;
//   - the four wavefronts split the 128 output channels; each reads its
//     32-channel weight fragments straight from global memory into registers,
//     also two stages ahead.  The fragments were stored at plan time in MFMA
//     operand order (one contiguous KiB per 32-channel x 32-byte fragment,
//     lane-major), so every weight byte is fetched by exactly one wavefront
//     with fully coalesced 16-byte loads.
//
// LDS layout of a pixel buffer: row r (128 bytes = eight 16-byte chunks) at
// r*128, chunk c stored in slot c ^ ((r >> 1) & 7).  A direct-to-LDS load
// writes lane l of a wavefront at base + 16*l, so lane l fetches, for row
// base_row + l/8, the chunk that belongs in slot l%8; the fragment reads of 16
// consecutive rows then fall into 16 distinct 16-byte bank groups.
//
// Vector-memory operations retire in issue order, so every load stream has the
// same depth (two stages) and every load is issued unconditionally (clamped to
// valid addresses at the ends): the number of operations in flight at each
// wait is a compile-time constant.  Padding taps and out-of-range rows fetch a
// 16-byte fill vector stored behind the weight fragments.
//
// NJ = 2: every wavefront owns two 32-channel slices (channels wave*32 and 128 +
// wave*32 of a 256-channel tile), i.e. twice the MFMA work for the same pixel
// fragments read from LDS and the same pixel requests; it pays for that with twice
// the accumulators and weight fragments (two wavefronts per SIMD).
//
// KS = 2: eight wavefronts in two groups of four, each group with its own ring and one half
// of the K stages; the second group's accumulators are added to the first's through LDS
// before the epilogue, which the first group runs alone.  For layers with fewer tiles than
// compute units (13 x 13 feature maps at batch 16): their time is the latency chain of the K
// stages of one workgroup, and two chains of half the length run side by side.
template <typename TIn, typename Epi, int NJ, int KS = 1>
// NJ = 1: three wavefronts per SIMD: at most 168 registers (two with the
// transcendental activations in the epilogue, which need more)
__global__ void __launch_bounds__(256 * KS, (EpiTraits<Epi>::rich || NJ == 2) ? 2 : 3)
igemm_wreg_kernel(const IgemmParams p, const int epi_vec) {
  constexpr int BM = 128, BN = 128 * NJ, WM = 128, NW = 4;
  constexpr int NWF = 4 * NJ;  // weight fragments of a wavefront per K stage
  constexpr int ES = sizeof(TIn);
  constexpr int BKB = 128, BK = BKB / ES;
  constexpr int VEC = 16 / ES, A_IT = 4;
  constexpr int TM = WM / 32;
  constexpr int BUF_BYTES = BM * BKB;  // 16 KiB
  constexpr int NBUF = 3;
  constexpr int EPI_BYTES = 2 * 32 * (128 + 4) * 4;
  static_assert(NBUF * BUF_BYTES >= EPI_BYTES, "staging area must fit in the pixel buffers");
  using Acc = typename Mma<TIn>::Acc;
  // s_waitcnt immediates (vmcnt only; expcnt / lgkmcnt left at their maxima):
  // vmcnt(0), and vmcnt(2 * NWF + 4) = 12 / 20 for the wait at the top of a stage
  constexpr int kWaitVm0 = 0x0f70, kWaitVmStage = NJ == 1 ? 0x0f7c : 0x4f74;

  // (8-bit results: the multipliers of the tile's channels wait behind the pixel rings)
  constexpr bool kMulLds = std::is_same<Epi, EpiQuant<0>>::value;
  constexpr int RING_BYTES = KS * NBUF * BUF_BYTES;
  static_assert(KS == 1 || (KS == 2 && NJ == 1), "two K groups with one slice per wavefront only");
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];   // RING_BYTES (+ NJ * 512 for the multipliers)

  const int tid = threadIdx.x;
  const int M = p.N * p.Ho * p.Wo;
  const int tiles_n = (p.Kout + BN - 1) / BN;
  int bid = blockIdx.x;
  {
    const int per = gridDim.x >> 3;
    if (bid < (per << 3)) bid = (bid & 7) * per + (bid >> 3);
  }
  const int tile_n = bid % tiles_n;
  const int tile_m = bid / tiles_n;
  const int z = blockIdx.z;
  const int wave = (tid >> 6) & 3, lane = tid & 63;   // wavefront within its K group
  const int l32 = lane & 31, lg = lane >> 5;
  const int kg_u = KS == 1 ? 0 : __builtin_amdgcn_readfirstlane(tid >> 8);   // K group

  const TIn* x = reinterpret_cast<const TIn*>(p.x) + (int64_t)z * p.x_bs;
  // fragment q of a 32-channel slice: 1 KiB at wf[j] + q * 1024, this lane's 16 bytes at lane * 16.
  // The slice's address is wavefront-uniform (scalar registers, scalar arithmetic for the
  // stage offsets); the lane adds one 32-bit offset.
  // (Measured on ResNet-50 at batch 256, same box: the scalar form is 1.3 % faster per fp16
  //  step - three registers and the 64-bit stage-offset additions of every wavefront less -
  //  and 0.3 % slower per int8 step, whose stages are half as long; the 8-bit kernels keep
  //  the per-lane address.)
  constexpr bool kScalarW = sizeof(TIn) != 1;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const unsigned lane_off = (unsigned)lane * 16u;
  const unsigned char* wf[NJ];
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    int wtile = (tile_n * NJ + j) * 4 + wave_u;
    wtile = wtile < p.wf_tiles ? wtile : p.wf_tiles - 1;  // surplus slices compute channels that are never stored
    wf[j] = reinterpret_cast<const unsigned char*>(p.w_frag) + ((int64_t)z * p.wf_tiles + wtile) * p.wf_chunks * 1024;
    if constexpr (!kScalarW) wf[j] += lane_off;   // (a per-lane address in a vector register pair)
  }
  const TIn* fill_ptr = reinterpret_cast<const TIn*>(reinterpret_cast<const unsigned char*>(p.w_frag) +
                                                     (int64_t)p.batch * p.wf_tiles * p.wf_chunks * 1024);

  // (the launcher gives two K groups an even number of stages)
  const int nkt = p.wf_chunks / 4 / KS;
  const int kt0 = kg_u * nkt;   // this group's first stage
  if constexpr (KS > 1) {
#pragma unroll
    for (int j = 0; j < NJ; ++j) wf[j] += (int64_t)kt0 * 4096;
  }

  // Weight fragment requests and their waits are issued by hand: next to the
  // direct-to-LDS loads the compiler would otherwise treat the vector-memory
  // counter as unordered and wait for everything in flight at each use.
  // wload: dst <- ptr[off bytes]; wwait<n>: dst is valid once at most n younger
  // vector-memory operations are still in flight.  A request inside the K loop
  // names its register as input and output, which ties every request for a
  // fragment to one physical register, and the wait behind the loop names all
  // eight: the compiler then sees them occupied on every path out of the loop,
  // also on those where the last requests are never consumed, and cannot hand
  // one of them to another value while data is still on its way into it.
  // (The host pass only needs the kernel's launch stub; it cannot parse the
  // vector-register constraints.)
#if defined(__HIP_DEVICE_COMPILE__)
// (The address is a scalar register pair.  A vector-memory instruction must not read a scalar
//  register within five wait states of a VECTOR instruction writing it, and the compiler does
//  not look into the asm for that: the addresses here come from scalar arithmetic, and a test
//  of the generated code checks the distance.)
#define IGEMM_WLOAD(dst, ptr, OFF)                                                                                         \
  do {                                                                                                                    \
    if constexpr (kScalarW)                                                                                               \
      asm volatile("global_load_dwordx4 %0, %1, %2 offset:" #OFF : "=v"(dst) : "v"(lane_off), "s"(ptr) : "memory");       \
    else                                                                                                                  \
      asm volatile("global_load_dwordx4 %0, %1, off offset:" #OFF : "=v"(dst) : "v"(ptr) : "memory");                     \
  } while (0)
#define IGEMM_WRELOAD(dst, ptr, OFF)                                                                                       \
  do {                                                                                                                    \
    if constexpr (kScalarW)                                                                                               \
      asm volatile("global_load_dwordx4 %0, %1, %2 offset:" #OFF : "+v"(dst) : "v"(lane_off), "s"(ptr) : "memory");       \
    else                                                                                                                  \
      asm volatile("global_load_dwordx4 %0, %1, off offset:" #OFF : "+v"(dst) : "v"(ptr) : "memory");                     \
  } while (0)
#define IGEMM_WWAIT(N, dst) asm volatile("s_waitcnt vmcnt(" #N ")" : "+v"(dst) : : "memory")
#define IGEMM_WDRAIN8(a, b)                                                                                    \
  asm volatile("s_waitcnt vmcnt(0)"                                                                            \
               : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(b[0]), "+v"(b[1]), "+v"(b[2]), "+v"(b[3]) \
               :                                                                                               \
               : "memory")
#else
#define IGEMM_WLOAD(dst, ptr, OFF) (dst) = *reinterpret_cast<const uintx4*>((ptr) + (kScalarW ? lane_off : 0u) + (OFF))
#define IGEMM_WRELOAD(dst, ptr, OFF) (dst) = *reinterpret_cast<const uintx4*>((ptr) + (kScalarW ? lane_off : 0u) + (OFF))
#define IGEMM_WWAIT(N, dst) (void)(dst)
#define IGEMM_WDRAIN8(a, b) (void)(a), (void)(b)
#endif
  // fragment kk of slice j sits at position kk * NJ + j: the order of use
  uintx4 w0[NWF], w1[NWF];
  auto wload = [&](uintx4& dst, const unsigned char* ptr, const int kk) __attribute__((always_inline)) {
    if (kk == 0) { IGEMM_WLOAD(dst, ptr, 0); }
    else if (kk == 1) { IGEMM_WLOAD(dst, ptr, 1024); }
    else if (kk == 2) { IGEMM_WLOAD(dst, ptr, 2048); }
    else { IGEMM_WLOAD(dst, ptr, 3072); }
  };
  auto wreload = [&](uintx4& dst, const unsigned char* ptr, const int kk) __attribute__((always_inline)) {
    if (kk == 0) { IGEMM_WRELOAD(dst, ptr, 0); }
    else if (kk == 1) { IGEMM_WRELOAD(dst, ptr, 1024); }
    else if (kk == 2) { IGEMM_WRELOAD(dst, ptr, 2048); }
    else { IGEMM_WRELOAD(dst, ptr, 3072); }
  };
  {
    const int64_t second = (int64_t)(nkt > 1 ? 1 : 0) * 4096;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk)
#pragma unroll
      for (int j = 0; j < NJ; ++j) wload(w0[kk * NJ + j], wf[j], kk);
#pragma unroll
    for (int kk = 0; kk < 4; ++kk)
#pragma unroll
      for (int j = 0; j < NJ; ++j) wload(w1[kk * NJ + j], wf[j] + second, kk);
  }
  // (requested this early, the fragments travel while the gather state below is computed)

  // ---- gather state: this thread feeds rows row0 + 32*i, slot lane%8 ----
  // C is a multiple of the stage depth, so a stage lies inside one filter tap
  // and the tap walk is wavefront-uniform (scalar registers).  Per row the
  // thread keeps the address of its chunk at tap (0,0), channel 0 - possibly
  // outside the image - and one validity bit per tap.
  const int row0 = (tid & 255) >> 3;
  const int kv = (lane & 7) ^ ((row0 >> 1) & 7);  // the chunk that belongs in this lane's slot
  const int RS = p.R * p.S;
  const TIn* a_row[A_IT];
  unsigned a_mask[A_IT];
  const int HoWo = p.Ho * p.Wo;
#pragma unroll
  for (int i = 0; i < A_IT; ++i) {
    const int m = tile_m * BM + row0 + i * 32;
    const bool ok = m < M;
    const int mm = ok ? m : 0;
    const int n_img = fast_div(mm, p.howo_magic, p.howo_shift);
    const int rem = mm - n_img * HoWo;
    const int ho = fast_div(rem, p.wo_magic, p.wo_shift);
    const int wo = rem - ho * p.Wo;
    const int hi0 = ho * p.sh - p.ph, wi0 = wo * p.sw - p.pw;
    a_row[i] = x + (((int64_t)n_img * p.H + hi0) * p.W + wi0) * p.xcs + kv * VEC;
    unsigned mask = 0u;
    int t = 0;
    for (int r = 0; r < p.R; ++r)
      for (int q = 0; q < p.S; ++q, ++t) {
        const int hi = hi0 + r * p.dh, wi = wi0 + q * p.dw;
        if (ok && (unsigned)hi < (unsigned)p.H && (unsigned)wi < (unsigned)p.W) mask |= 1u << t;
      }
    a_mask[i] = mask;
  }
  using lds_ptr = __attribute__((address_space(3))) void*;
  // Requests the next K stage of the pixel tile into buffer `buf`.  Requests
  // past the last tap (the pipeline's run-out) fetch the fill vector.  All the
  // bookkeeping is wavefront-uniform and incremental - the element offset of
  // the stage from tap (0,0), the bit of the tap in the validity masks, the LDS
  // address - so that a stage costs one select and one request per row.
  int tap = 0, tap_s = 0, kc0 = 0;
  int toff = 0;             // offset of (tap, kc0) from tap (0,0), channel 0, in elements
  unsigned tapbit = 1u;     // 1 << tap, 0 behind the last tap
  const int step_s = p.dw * p.xcs;                              // to the next tap of the row
  const int step_r = p.dh * p.W * p.xcs - (p.S - 1) * step_s;   // from the last tap of a row to the first of the next
  if constexpr (KS > 1) {
    // the walk starts at this group's first stage
    const int e0 = kt0 * BK;          // elements of K before it
    tap = e0 / p.C;
    kc0 = e0 - tap * p.C;
    const int tap_r = tap / p.S;
    tap_s = tap - tap_r * p.S;
    toff = (tap_r * p.dh * p.W + tap_s * p.dw) * p.xcs + kc0;
    tapbit = tap < RS ? 1u << tap : 0u;
  }
  const uint64_t fill_u = reinterpret_cast<uint64_t>(fill_ptr);
  auto dma = [&](const int buf) {
    unsigned char* dst = smem + (kg_u * NBUF + buf) * BUF_BYTES + wave_u * 1024;
#pragma unroll
    for (int i = 0; i < A_IT; ++i) {
      const uint64_t live = reinterpret_cast<uint64_t>(a_row[i] + toff);
      const uint64_t src = (a_mask[i] & tapbit) != 0u ? live : fill_u;
#if defined(__HIP_DEVICE_COMPILE__)  // (the builtin is unknown to the host pass, which only needs the launch stub)
      __builtin_amdgcn_global_load_lds(reinterpret_cast<const TIn*>(src), (lds_ptr)(dst + i * 4096), 16, 0, 0);
#else
      (void)src; (void)dst;
#endif
    }
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

  Acc acc[NJ][TM][1];
#pragma unroll
  for (int j = 0; j < NJ; ++j)
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[j][i][0][e] = 0;
  if constexpr (EpiTraits<Epi>::quant) {
    // 8-bit layers: the int32 bias starts in the accumulators (element q*4 + r of
    // a lane is channel wave*32 + q*8 + (lane/32)*4 + r), which takes its addition
    // out of the requantising epilogue, the busiest part of these layers.  Eight
    // 16-byte loads per slice, consumed right here: they are older than every
    // request the K loop counts, so its waits stay valid.
    if (KS == 1 || kg_u == 0) {   // (once per tile: the second K group starts from zero)
#pragma unroll
      for (int j = 0; j < NJ; ++j) acc_init_bias_vec<TM, 1>(p, z, (tile_n * NJ + j) * 128 + wave_u * 32, lg, acc[j]);
    }
  }
  if constexpr (kMulLds) {
    // The multipliers of this wavefront's channels, into LDS behind the ring (requested
    // and consumed here, like the bias; read back by the same wavefront in the epilogue,
    // which then begins without a round trip to memory).
    float* mt = reinterpret_cast<float*>(smem + RING_BYTES);
    const int last = p.Kout - 1;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int c = (tile_n * NJ + j) * 128 + wave_u * 32 + l32;
      const float v = p.qmul[c < last ? c : last];
      if (lg == 0) mt[j * 128 + wave_u * 32 + l32] = v;
    }
  }

  // fragment read offsets: row l32 (+32*i), chunk 2*kk + lg, swizzled
  const int sw = (l32 >> 1) & 7;
  const int rd_base = l32 * 128 + ((lg ^ (sw & 1)) * 16);
  const int rd_t = sw >> 1;

  dma(0);
  dma(1);

  // One K stage.  wc = this stage's weight fragments; each is re-requested for
  // stage kt+2 right after its use.
  auto stage = [&](const int kt, const int buf, uintx4 (&wc)[NWF]) {
    // the pixel vectors of this stage have landed (mine), and everyone's have
    // (a bare barrier: the fence of __syncthreads would also wait for the
    // requests of the stages still in flight).  Behind them in flight: this
    // stage's NWF fragments and the 4 + NWF operations of the stage between.
    if (kt < 2) __builtin_amdgcn_s_waitcnt(kWaitVm0);
    else __builtin_amdgcn_s_waitcnt(kWaitVmStage);
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    // every wavefront has also left stage kt-1, whose buffer is (kt+2) % 3
    dma(buf == 0 ? 2 : buf - 1);
    __builtin_amdgcn_sched_barrier(0);
    const unsigned char* ab = smem + (kg_u * NBUF + buf) * BUF_BYTES + rd_base;
    const int ktn = kt + 2 < nkt ? kt + 2 : nkt - 1;
    const unsigned char* wnext[NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j) wnext[j] = wf[j] + (int64_t)ktn * 4096;
    uintx4 fa[2][TM];
#pragma unroll
    for (int i = 0; i < TM; ++i) fa[0][i] = *reinterpret_cast<const uintx4*>(ab + ((0 ^ rd_t) * 32) + i * 4096);
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      if (kk < 3) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
          fa[(kk + 1) & 1][i] = *reinterpret_cast<const uintx4*>(ab + (((kk + 1) ^ rd_t) * 32) + i * 4096);
      }
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int k = kk * NJ + j;
        __builtin_amdgcn_sched_barrier(0);
        // In flight behind wc[k] (requested two stages ago at this position):
        // NWF-1-k fragments of that stage, 4 + NWF operations of the stage
        // between, the 4 pixel requests above and k fragments of this stage:
        // always 2 * NWF + 7.
        if constexpr (NJ == 1) IGEMM_WWAIT(15, wc[k]);
        else IGEMM_WWAIT(23, wc[k]);
#pragma unroll
        for (int i = 0; i < TM; ++i) acc[j][i][0] = Mma<TIn>::run(wc[k], fa[kk & 1][i], acc[j][i][0]);
        __builtin_amdgcn_sched_barrier(0);
        wreload(wc[k], wnext[j], kk);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  int buf = 0;
  for (int kt = 0; kt < nkt; kt += 2) {
    stage(kt, buf, w0);
    buf = buf == 2 ? 0 : buf + 1;
    if (kt + 1 < nkt) {
      stage(kt + 1, buf, w1);
      buf = buf == 2 ? 0 : buf + 1;
    }
  }
  // the ring becomes the staging area: no direct-to-LDS write may still be in
  // flight, and neither may a weight fragment be
  if constexpr (NJ == 1) {
    IGEMM_WDRAIN8(w0, w1);
  } else {
    uintx4(&w0a)[4] = reinterpret_cast<uintx4(&)[4]>(w0[0]);
    uintx4(&w0b)[4] = reinterpret_cast<uintx4(&)[4]>(w0[4]);
    uintx4(&w1a)[4] = reinterpret_cast<uintx4(&)[4]>(w1[0]);
    uintx4(&w1b)[4] = reinterpret_cast<uintx4(&)[4]>(w1[4]);
    // (one wait names all sixteen: with two the compiler could release eight of
    // them after the first, while their data is still in flight)
#if defined(__HIP_DEVICE_COMPILE__)
    asm volatile("s_waitcnt vmcnt(0)"
                 : "+v"(w0a[0]), "+v"(w0a[1]), "+v"(w0a[2]), "+v"(w0a[3]), "+v"(w0b[0]), "+v"(w0b[1]), "+v"(w0b[2]),
                   "+v"(w0b[3]), "+v"(w1a[0]), "+v"(w1a[1]), "+v"(w1a[2]), "+v"(w1a[3]), "+v"(w1b[0]), "+v"(w1b[1]),
                   "+v"(w1b[2]), "+v"(w1b[3])
                 :
                 : "memory");
#endif
  }
  __builtin_amdgcn_sched_barrier(0);
#undef IGEMM_WLOAD
#undef IGEMM_WRELOAD
#undef IGEMM_WWAIT
#undef IGEMM_WDRAIN8
  if constexpr (KS == 2) {
    // The second group's partial sums join the first's: 16 vectors per lane through the rings
    // (64 KiB of them), which nobody reads any more once every wavefront has passed the first
    // barrier.  Barriers for LDS traffic only, as in the epilogue.
    using V4 = typename std::conditional<std::is_same<TIn, int8_t>::value, intx4, floatx4>::type;
    auto lds_barrier = [&]() {
      __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
      __builtin_amdgcn_sched_barrier(0);
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      __builtin_amdgcn_sched_barrier(0);
    };
    V4* red = reinterpret_cast<V4*>(smem) + (wave_u * 16) * 64 + lane;
    lds_barrier();
    if (kg_u == 1) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q)
          red[(i * 4 + q) * 64] = (V4){acc[0][i][0][q * 4 + 0], acc[0][i][0][q * 4 + 1], acc[0][i][0][q * 4 + 2], acc[0][i][0][q * 4 + 3]};
    }
    lds_barrier();
    if (kg_u == 0) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const V4 v = red[(i * 4 + q) * 64];
          acc[0][i][0][q * 4 + 0] += v.x; acc[0][i][0][q * 4 + 1] += v.y;
          acc[0][i][0][q * 4 + 2] += v.z; acc[0][i][0][q * 4 + 3] += v.w;
        }
    }
    lds_barrier();   // the sums are read: the rings become the epilogue's staging area
    // (a wavefront that has ended no longer counts at the workgroup's barriers)
    if (kg_u == 1) return;
  }
#pragma unroll
  for (int j = 0; j < NJ; ++j)
    igemm_epilogue_rows128<TIn, Epi>(p, epi_vec, acc[j], smem, tile_m, tile_n * NJ + j, z, M, wave, lane,
                                     kMulLds ? reinterpret_cast<const float*>(smem + RING_BYTES) + j * 128 : nullptr);
}

// ---------------------------------------------------------------------------
// Variant for 1x1 filters over few input channels (K = 64 or 128 bytes per
// pixel, no padding): such layers are pure streaming - one short burst of
// matrix instructions between reading 8-16 KiB and writing 16-32 KiB per tile -
// and with a K loop, operand staging and workgroup barriers their time is the
// sum of the latencies of those phases.  Here nothing is staged and nothing is
// shared: every wavefront owns 32 pixels x 128 channels, reads its pixel
// fragments and the (fragment-ordered, L2-resident) weights straight from
// global memory into MFMA operand registers, keeps the weights for all the
// pixel tiles it walks, and requests the pixels of its next tile before it
// runs the epilogue of the current one.  The epilogue parks 64 channels at a
// time in the wavefront's private LDS slice (no workgroup barrier anywhere).
// NKK = 32-byte K steps per pixel; NJ = 32-channel slices per wavefront (the
// tile is 32 NJ channels wide: 4 slices of 4 K steps do not fit the registers).
template <typename TIn, typename Epi, int NKK, int NJ>
__global__ void __launch_bounds__(256, 3)
igemm_lean_kernel(const IgemmParams p, const int epi_vec, const int tiles_per_wg) {
  constexpr int BM = 128, BN = 32 * NJ;
  using Acc = typename Mma<TIn>::Acc;
  __shared__ __attribute__((aligned(16))) unsigned char smem[4 * 32 * (64 + 4) * 4];

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int l32 = lane & 31, lg = lane >> 5;
  const int M = p.N * p.Ho * p.Wo;
  const int tiles_m = (M + BM - 1) / BM;
  const int tiles_n = (p.Kout + BN - 1) / BN;
  int bid = blockIdx.x;
  {
    const int per = gridDim.x >> 3;
    if (bid < (per << 3)) bid = (bid & 7) * per + (bid >> 3);
  }
  const int tile_n = bid % tiles_n;
  const int tm0 = (bid / tiles_n) * tiles_per_wg;
  const int tm1 = tm0 + tiles_per_wg < tiles_m ? tm0 + tiles_per_wg : tiles_m;

  const TIn* x = reinterpret_cast<const TIn*>(p.x);
  const uintx4* wf = reinterpret_cast<const uintx4*>(p.w_frag) + lane;
  uintx4 w[NJ][NKK];
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    int wtile = tile_n * NJ + j;
    wtile = wtile < p.wf_tiles ? wtile : p.wf_tiles - 1;  // surplus slices compute channels that are never stored
#pragma unroll
    for (int kk = 0; kk < NKK; ++kk) w[j][kk] = wf[((int64_t)wtile * p.wf_chunks + kk) * 64];
  }
  const int HoWo = p.Ho * p.Wo;
  // lane (l32, lg) supplies bytes [32 kk + 16 lg, +16) of pixel row l32
  auto load_a = [&](const int tile_m, uintx4 (&a)[NKK]) {
    int m = tile_m * BM + wave * 32 + l32;
    m = m < M ? m : M - 1;
    const int n_img = fast_div(m, p.howo_magic, p.howo_shift);
    const int rem = m - n_img * HoWo;
    const int ho = fast_div(rem, p.wo_magic, p.wo_shift);
    const int wo = rem - ho * p.Wo;
    const uintx4* row =
        reinterpret_cast<const uintx4*>(x + (((int64_t)n_img * p.H + ho * p.sh) * p.W + wo * p.sw) * p.xcs) + lg;
#pragma unroll
    for (int kk = 0; kk < NKK; ++kk) a[kk] = row[2 * kk];
  };
  uintx4 a_cur[NKK], a_nxt[NKK];
  load_a(tm0, a_cur);
  for (int tile_m = tm0; tile_m < tm1; ++tile_m) {
    // (requested only where a next tile exists: a workgroup walks two or three tiles, and re-reading
    //  the last one instead - which would let the compiler count the requests in flight - costs more
    //  than the wait it saves: 64 -> 256 + residual at 56 x 56, fp16, 175 -> 186 us)
    if (tile_m + 1 < tm1) load_a(tile_m + 1, a_nxt);
    // 64 channels at a time: half the accumulator registers, half the staging space
#pragma unroll
    for (int h = 0; h < NJ / 2; ++h) {
      Acc acc[1][2];
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[0][j][e] = 0;
#pragma unroll
      for (int kk = 0; kk < NKK; ++kk)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[0][j] = Mma<TIn>::run(w[2 * h + j][kk], a_cur[kk], acc[0][j]);
      igemm_epilogue<TIn, Epi, BM, BN, 32, 64, false>(p, epi_vec, acc, smem, tile_m, tile_n, 0, M, wave, lane, h * 64);
      // the same wavefront parks into its slice again next: order it behind the read-back
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
#pragma unroll
    for (int kk = 0; kk < NKK; ++kk) a_cur[kk] = a_nxt[kk];
  }
}

// ---------------------------------------------------------------------------
// Variant for filters over one or two 16-byte vectors of channels per tap
// (network stems: three input channels padded to a vector, or their
// space-to-depth form).  K is R*S short taps and the layer is pure streaming
// like the 1x1 case above; the 16 bytes a lane supplies to a matrix
// instruction are exactly one vector of one tap of its pixel, so they come
// straight from global memory into the operand register (the overlap between
// the windows of neighbouring pixels is served by the caches), nothing is
// staged and nothing is shared.  Every wavefront owns 32 pixels x 64 channels
// and keeps the fragment-ordered weights of all K steps in registers for the
// pixel tiles it walks; the pixels of the next tile are requested between the
// matrix instructions of the current one and its epilogue.  A tap's position
// is tested against the image only for pixel blocks that touch the border.
// NKK = 32-byte K steps (R*S*VPT 16-byte units, rounded up to a pair);
// VPT = 16-byte vectors per tap (xcs * sizeof(TIn) / 16).
template <typename TIn, typename Epi, int NKK, int VPT, int NJ>
__global__ void __launch_bounds__(256, 2)
igemm_taps_kernel(const IgemmParams p, const int epi_vec, const int tiles_per_wg) {
  // NJ = 2: four wavefronts on four 32-pixel blocks, 64 channels each; NJ = 1 (K rows too
  // long to keep 64 channels of weights in registers): two blocks, two channel halves
  constexpr int BM = NJ == 2 ? 128 : 64, BN = 64, WN = 32 * NJ;
  using Acc = typename Mma<TIn>::Acc;
  __shared__ __attribute__((aligned(16))) unsigned char smem[4 * 32 * (64 + 4) * 4];

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int l32 = lane & 31, lg = lane >> 5;
  const int wm = wave % (BM / 32), wn = wave / (BM / 32);
  const int M = p.N * p.Ho * p.Wo;
  const int tiles_m = (M + BM - 1) / BM;
  const int tiles_n = (p.Kout + BN - 1) / BN;
  int bid = blockIdx.x;
  {
    const int per = gridDim.x >> 3;
    if (bid < (per << 3)) bid = (bid & 7) * per + (bid >> 3);
  }
  const int tile_n = bid % tiles_n;
  const int tm0 = (bid / tiles_n) * tiles_per_wg;
  const int tm1 = tm0 + tiles_per_wg < tiles_m ? tm0 + tiles_per_wg : tiles_m;

  const uintx4* wf = reinterpret_cast<const uintx4*>(p.w_frag) + lane;
  uintx4 w[NJ][NKK];
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    int wtile = tile_n * 2 + wn * NJ + j;
    wtile = wtile < p.wf_tiles ? wtile : p.wf_tiles - 1;  // a surplus slice computes channels that are never stored
#pragma unroll
    for (int kk = 0; kk < NKK; ++kk) w[j][kk] = wf[((int64_t)wtile * p.wf_chunks + kk) * 64];
  }

  // The accumulators start at the bias (held for every pixel tile this wavefront walks),
  // and the multipliers of an 8-bit layer are parked once: the epilogues then begin with
  // no vector-memory wait, behind which the next tile's pixels would have to queue.
  Acc acc0[1][NJ];
#pragma unroll
  for (int j = 0; j < NJ; ++j)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc0[0][j][e] = 0;
  IgemmParams pe = p;   // the epilogue's view: no bias left to add
  if constexpr (EpiTraits<Epi>::quant) {
    acc_init_bias_vec<1, NJ>(p, 0, tile_n * BN + wn * WN, lg, acc0);
    constexpr int TILE = 32 * (WN + 16);
    float* mtile = reinterpret_cast<float*>(smem + wave * (2 * TILE + WN * 4) + 2 * TILE);
    if (lane < WN / 4) *reinterpret_cast<floatx4*>(mtile + lane * 4) = load_qmul4(p.qmul, tile_n * BN + wn * WN + lane * 4, p.Kout);
  } else {
    if (p.bias != nullptr) {
      const float* bias = reinterpret_cast<const float*>(p.bias);
      const int last = p.Kout - 1;   // channels past the end are computed but never stored
#pragma unroll
      for (int j = 0; j < NJ; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int c = tile_n * BN + wn * WN + j * 32 + q * 8 + lg * 4 + r;
            acc0[0][j][q * 4 + r] = p.alpha == 1.0f ? bias[c < last ? c : last] : 0.f;
          }
      if (p.alpha == 1.0f) pe.bias = nullptr;   // (a scaled accumulator keeps its bias in the epilogue)
    }
  }

  // unit u = 2 kk + lg of the K row is vector (u % VPT) of tap (u / VPT) = (tr, tc), tr = tap / S
  // through a multiplication (taps < 64, S <= 8: exact).  Taps outside the image and units
  // past the last tap (their weights are zero) are read at a clamped position and replaced
  // by the fill value before use: the requests themselves are unconditional.
  const int units = p.R * p.S * VPT;
  const unsigned s_inv = (65536u + (unsigned)p.S - 1u) / (unsigned)p.S;
  const unsigned fill_w = (unsigned)(p.a_fill & 0xff) * 0x01010101u;
  const uintx4 fillv = {fill_w, fill_w, fill_w, fill_w};
  const uintx4* x16 = reinterpret_cast<const uintx4*>(p.x);
  const int HoWo = p.Ho * p.Wo;

  uintx4 a[NKK];
  unsigned okmask = 0;   // bit kk: this lane's unit of K step kk is real data
  auto load_a = [&](const int tile_m) {
    int m = tile_m * BM + wm * 32 + l32;
    m = m < M ? m : M - 1;
    const int n_img = fast_div(m, p.howo_magic, p.howo_shift);
    const int rem = m - n_img * HoWo;
    const int ho = fast_div(rem, p.wo_magic, p.wo_shift);
    const int wo = rem - ho * p.Wo;
    const int hi0 = ho * p.sh - p.ph, wi0 = wo * p.sw - p.pw;
    const int img = n_img * p.H;   // (the whole source has fewer than 2^31 16-byte units)
    okmask = 0;
#pragma unroll
    for (int kk = 0; kk < NKK; ++kk) {
      const int u = 2 * kk + lg;
      const int tap = u / VPT;
      const int tr = (int)(((unsigned)tap * s_inv) >> 16), tc = tap - tr * p.S;
      const int hi = hi0 + tr, wi = wi0 + tc;
      const bool ok = u < units && (unsigned)hi < (unsigned)p.H && (unsigned)wi < (unsigned)p.W;
      const int hc = hi < 0 ? 0 : (hi < p.H ? hi : p.H - 1), wc = wi < 0 ? 0 : (wi < p.W ? wi : p.W - 1);
      a[kk] = x16[(unsigned)(((img + hc) * p.W + wc) * VPT + u % VPT)];
      okmask |= ok ? 1u << kk : 0u;
    }
  };

  load_a(tm0);
  for (int tile_m = tm0; tile_m < tm1; ++tile_m) {
    if (__builtin_amdgcn_ballot_w64(okmask != (1u << NKK) - 1u) != 0) {   // a border block
#pragma unroll
      for (int kk = 0; kk < NKK; ++kk) a[kk] = (okmask >> kk) & 1u ? a[kk] : fillv;
    }
    Acc acc[1][NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j) acc[0][j] = Mma<TIn>::run(w[j][0], a[0], acc0[0][j]);
#pragma unroll
    for (int kk = 1; kk < NKK; ++kk)
#pragma unroll
      for (int j = 0; j < NJ; ++j) acc[0][j] = Mma<TIn>::run(w[j][kk], a[kk], acc[0][j]);
    // the operand registers are free again: the next tile's pixels travel during the epilogue
    // (always requested: the last tile re-reads itself)
    load_a(tile_m + 1 < tm1 ? tile_m + 1 : tile_m);
    igemm_epilogue<TIn, Epi, BM, BN, 32, WN, false, true>(pe, epi_vec, acc, smem, tile_m, tile_n, 0, M, wave, lane, 0);
    // the same wavefront parks into its slice again next: order it behind the read-back
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
}

// Rearranges packed weight rows ([batch][rows][row_bytes], zero padded) into
// MFMA fragment order, followed by kWfragTailBytes of the fill byte: 16-byte unit ((b * tiles + t) * chunks + q) * 64 + lane
// holds bytes [q*32 + (lane/32)*16, +16) of row t*32 + lane%32.
__global__ void __launch_bounds__(256) wfrag_pack_kernel(WfragPackParams p) {
  const int64_t total = (int64_t)p.batch * p.tiles * p.chunks * 64;
  const uintx4* src = reinterpret_cast<const uintx4*>(p.src);
  uintx4* dst = reinterpret_cast<uintx4*>(p.dst);
  if (blockIdx.x == 0 && threadIdx.x < kWfragTailBytes / 16) {  // the fill vectors behind the fragments
    const unsigned f = (unsigned)(p.fill & 0xff) * 0x01010101u;
    dst[total + threadIdx.x] = (uintx4){f, f, f, f};
  }
  for (int64_t u = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; u < total; u += (int64_t)gridDim.x * blockDim.x) {
    const int lane = (int)(u & 63);
    int64_t t = u >> 6;
    const int q = (int)(t % p.chunks);
    t /= p.chunks;
    const int tile = (int)(t % p.tiles);
    const int64_t b = t / p.tiles;
    const int row = tile * 32 + (lane & 31);
    const int off = q * 32 + (lane >> 5) * 16;
    uintx4 v = {0u, 0u, 0u, 0u};
    if (row < p.rows && off < p.row_bytes) v = src[((b * p.rows + row) * p.row_bytes + off) >> 4];
    dst[u] = v;
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
  if (const char* force = getenv("ODLA_HIP_IGEMM_TILE")) {  // tuning aid: "128x64" etc.
    int bm = 0, bn = 0;
    if (sscanf(force, "%dx%d", &bm, &bn) == 2) {
      if (bm == 128 && bn == 32) return {128, 32, "128x32"};
      if (bm == 128 && bn == 64) return {128, 64, "128x64"};
      if (bm == 64 && bn == 128) return {64, 128, "64x128"};
      if (bm == 128 && bn == 128) return {128, 128, "128x128"};
    }
  }
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

// 32-channel slices per wavefront of the weights-in-registers kernel.
int wreg_slices(const IgemmParams& p) {
  if (const char* force = getenv("ODLA_HIP_WREG_SLICES")) {  // tuning aid
    const int v = atoi(force);
    if (v == 1 || v == 2) return v;
  }
  // Two slices halve the workgroups and the LDS reads per MFMA but leave two
  // wavefronts per SIMD: measured faster only on long K loops whose grid still
  // covers the chip (ResNet-50 at batch 256: the 3x3 256 -> 256 layers, 784 -> 392
  // workgroups, 88 -> 76 us, and 1024 -> 256, 48 -> 43 us), slower on short ones.
  const int64_t M = (int64_t)p.N * p.Ho * p.Wo;
  const int64_t stages = (int64_t)p.R * p.S * p.C * dtype_size(p.in_dt) / 128;
  const int64_t tiles2 = ((M + 127) / 128) * ((p.Kout + 255) / 256);
  if (p.Kout % 256 == 0 && stages >= 16 && tiles2 >= 320 && tiles2 <= 512) return 2;
  return 1;
}

// K groups of the weights-in-registers kernel (one slice per wavefront): two where the launch has
// far fewer workgroups than the chip has compute units and the K loop is long enough to be worth
// splitting (an even number of stages, at least 24: measured on YOLOv3 at batch 16, 72 stages
// 53 -> 46 us, 16 stages unchanged, 8 stages 14.6 -> 16 .. 21 us).
int wreg_k_groups(const IgemmParams& p, const int64_t workgroups) {
  const int64_t stages = (int64_t)p.wf_chunks / 4;
  const bool legal = stages % 2 == 0 && stages >= 4;
  if (const char* force = getenv("ODLA_HIP_WREG_KSPLIT")) {  // tuning aid: 0 = never, 2 = wherever legal
    const int v = atoi(force);
    if (v == 0) return 1;
    if (v == 2) return legal ? 2 : 1;
  }
  // (fp32 layers keep one summation chain per result: their parity bound is relative to single
  //  results, which a second chain's rounding can exceed where a sum nearly cancels)
  if (p.in_dt == DT_F32) return 1;
  // (at most 180 workgroups: a workgroup of this form takes a compute unit's LDS for itself, and
  //  when two half-batch copies of a plan run side by side the other copy's launch wants the
  //  units this one leaves - BERT-base halves of 32 sequences, 192 workgroups of 48 stages,
  //  2.36 -> 2.43 ms per step with it)
  return legal && stages >= 24 && workgroups <= 180 ? 2 : 1;
}

template <typename TIn, typename Epi>
hipError_t launch_wreg(const IgemmParams& p, int epi_vec, hipStream_t stream) {
  const int64_t M = (int64_t)p.N * p.Ho * p.Wo;
  // what the kernel's tap walk assumes: whole K stages per tap, one mask bit per tap
  if (p.C % (128 / (int)sizeof(TIn)) != 0 || p.R * p.S > 32) return hipErrorInvalidValue;
  // (the transcendental epilogues do not fit beside twice the accumulators)
  const int nj = EpiTraits<Epi>::rich ? 1 : wreg_slices(p);
  const int64_t tiles = ((M + 127) / 128) * ((p.Kout + 128 * nj - 1) / (128 * nj));
  if (tiles <= 0 || tiles > 0x7fffffff) return hipErrorInvalidValue;
  // pixel ring(s) and, for 8-bit results, the tile's multipliers
  constexpr size_t ring = 3 * 128 * 128;
  constexpr size_t mul = std::is_same<Epi, EpiQuant<0>>::value ? 512 : 0;
  if constexpr (!EpiTraits<Epi>::rich) {
    if (nj == 2) {
      hipLaunchKernelGGL((igemm_wreg_kernel<TIn, Epi, 2>), dim3((unsigned)tiles, 1, (unsigned)p.batch), dim3(256),
                         ring + 2 * mul, stream, p, epi_vec);
      return hipGetLastError();
    }
    if (wreg_k_groups(p, tiles * p.batch) == 2) {
      static bool ready = false;   // (repeating the call is harmless: no lock)
      if (!ready) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&igemm_wreg_kernel<TIn, Epi, 1, 2>),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)(2 * ring + mul));
        if (e != hipSuccess) return e;
        ready = true;
      }
      hipLaunchKernelGGL((igemm_wreg_kernel<TIn, Epi, 1, 2>), dim3((unsigned)tiles, 1, (unsigned)p.batch), dim3(512),
                         2 * ring + mul, stream, p, epi_vec);
      return hipGetLastError();
    }
  }
  hipLaunchKernelGGL((igemm_wreg_kernel<TIn, Epi, 1>), dim3((unsigned)tiles, 1, (unsigned)p.batch), dim3(256), ring + mul,
                     stream, p, epi_vec);
  return hipGetLastError();
}

// 1x1 filters with at most one K stage and no padding: the streaming variant.
int lean_steps(const IgemmParams& p) {
  if (const char* force = getenv("ODLA_HIP_IGEMM_TILE")) {  // tuning aid
    if (strcmp(force, "lean") != 0 && force[0] != 0) return 0;
  }
  const int kbytes = p.C * dtype_size(p.in_dt);
  if (p.R != 1 || p.S != 1 || p.ph != 0 || p.pw != 0 || p.batch != 1 || p.Kout < 64) return 0;
  // no padding behind the image either: every output pixel reads a pixel that exists
  if ((int64_t)(p.Ho - 1) * p.sh >= p.H || (int64_t)(p.Wo - 1) * p.sw >= p.W) return 0;
  // (8-bit layers of this shape are bound by the arithmetic of the requantising
  // epilogue, not by their staging, and do not gain from it)
  if (p.in_dt != DT_F16 && p.in_dt != DT_BF16) return 0;
  if (kbytes != 64 && kbytes != 128) return 0;
  return kbytes / 32;
}

template <typename TIn, typename Epi>
hipError_t launch_lean(const IgemmParams& p, int epi_vec, hipStream_t stream) {
  const int64_t M = (int64_t)p.N * p.Ho * p.Wo;
  const int steps = lean_steps(p);
  const int bn = steps == 2 ? 128 : 64;
  const int64_t tiles_m = (M + 127) / 128, tiles_n = (p.Kout + bn - 1) / bn;
  // a few pixel tiles per workgroup: the weights are fetched once for all of
  // them and the next tile's pixels are in flight during each epilogue
  int tpw = 1;
  while (tpw < 8 && tiles_m * tiles_n / (tpw * 2) >= 4096) tpw *= 2;
  if (const char* force = getenv("ODLA_HIP_LEAN_TILES")) {  // test aid: pixel tiles per workgroup
    const int v = atoi(force);
    if (v >= 1 && v <= 64) tpw = v;
  }
  const int64_t groups = (tiles_m + tpw - 1) / tpw;
  const int64_t wgs = groups * tiles_n;
  if (wgs <= 0 || wgs > 0x7fffffff) return hipErrorInvalidValue;
  if (steps == 2)
    hipLaunchKernelGGL((igemm_lean_kernel<TIn, Epi, 2, 4>), dim3((unsigned)wgs), dim3(256), 0, stream, p, epi_vec, tpw);
  else
    hipLaunchKernelGGL((igemm_lean_kernel<TIn, Epi, 4, 2>), dim3((unsigned)wgs), dim3(256), 0, stream, p, epi_vec, tpw);
  return hipGetLastError();
}

// The layers that run on the short-tap streaming variant.  Returns its K steps
// and vectors per tap, or {0, 0}.
struct TapsShape { int nkk, vpt; };
TapsShape taps_shape(const IgemmParams& p) {
  if (const char* force = getenv("ODLA_HIP_IGEMM_TILE")) {  // tuning aid
    if (strcmp(force, "taps") != 0 && force[0] != 0) return {0, 0};
  }
  const int es = dtype_size(p.in_dt);
  if (p.in_dt != DT_F16 && p.in_dt != DT_BF16 && p.in_dt != DT_I8) return {0, 0};
  if (p.out_dt != p.in_dt || p.batch != 1 || p.dh != 1 || p.dw != 1 || p.C != p.xcs) return {0, 0};
  if (p.y_rdiv > 0 || p.y_zdiv > 0) return {0, 0};
  if (p.act != ACT_NONE && p.act != ACT_RELU && p.act != ACT_LEAKY && p.act != ACT_CLAMP) return {0, 0};
  const int pix_bytes = p.xcs * es;
  // (8-bit 1x1 filters over 64 channels into at most 64: one "tap" of four vectors; ResNet-50's
  // first bottleneck at batch 256: 35 -> 27 us.  With more output channels, or longer pixel
  // rows, the same layers were measured slower here than on the other kernels.)
  if (es == 1 && p.R * p.S == 1 && pix_bytes == 64 && p.Kout <= 64 && (int64_t)p.N * p.H * p.W * 4 < (1ll << 31))
    return {2, 4};
  if (pix_bytes != 16 && pix_bytes != 32) return {0, 0};
  const int vpt = pix_bytes / 16;
  if (p.R * p.S < 2 || p.S > 8 || p.Kout > 128) return {0, 0};
  const int nkk = (p.R * p.S * vpt + 1) / 2;
  // the indices of the 16-byte units of the whole source fit 31 bits
  if ((int64_t)p.N * p.H * p.W * vpt >= (1ll << 31)) return {0, 0};
  // Built and selected where it was measured faster than the two-operand kernel: 16 taps of
  // one 8-bit vector (the space-to-depth form of a 7x7 stride-2 stem; ResNet-50 at batch
  // 256: 159 -> 122 us).  The 2-byte forms of the same layers request twice the bytes per
  // pixel from the vector-memory pipeline, which then bounds them (215 -> 288 us), and stay
  // on the two-operand kernel.
  const bool built = vpt == 1 && nkk == 8 && es == 1;
  return built ? TapsShape{nkk, vpt} : TapsShape{0, 0};
}

template <typename TIn, typename Epi>
hipError_t launch_taps(const IgemmParams& p, int epi_vec, hipStream_t stream) {
  const int64_t M = (int64_t)p.N * p.Ho * p.Wo;
  const TapsShape ts = taps_shape(p);
  const int64_t tiles_m = (M + 127) / 128, tiles_n = (p.Kout + 63) / 64;
  // several pixel tiles per workgroup (the weights are fetched once for all of them),
  // as long as the chip keeps eight workgroups per compute unit
  int tpw = 1;
  while (tpw < 16 && tiles_m * tiles_n / (tpw * 2) >= 2048) tpw *= 2;
  if (const char* force = getenv("ODLA_HIP_LEAN_TILES")) {  // test aid: pixel tiles per workgroup
    const int v = atoi(force);
    if (v >= 1 && v <= 64) tpw = v;
  }
  const int64_t wgs = ((tiles_m + tpw - 1) / tpw) * tiles_n;
  if (wgs <= 0 || wgs > 0x7fffffff) return hipErrorInvalidValue;
  const dim3 grid((unsigned)wgs), block(256);
  if (ts.vpt == 1) hipLaunchKernelGGL((igemm_taps_kernel<TIn, Epi, 8, 1, 2>), grid, block, 0, stream, p, epi_vec, tpw);
  else hipLaunchKernelGGL((igemm_taps_kernel<TIn, Epi, 2, 4, 2>), grid, block, 0, stream, p, epi_vec, tpw);
  return hipGetLastError();
}

// The weights-in-registers kernel pays off once a layer has enough output
// channels to give each of the four wavefronts its own 32-channel slice.
bool wreg_shape(const IgemmParams& p) {
  if (const char* force = getenv("ODLA_HIP_IGEMM_TILE")) {  // tuning aid
    if (strcmp(force, "wreg") == 0) return true;
    if (force[0] != 0) return false;
  }
  const int bk = 128 / dtype_size(p.in_dt);
  // A K stage must lie inside one filter tap.  (The kernel also handles 1x1
  // filters with any channel count, but with less than one full stage of K the
  // two-operand kernel is faster: measured on the 64 -> 256 int8 layers.)
  return p.Kout > 64 && p.C % bk == 0 && p.R * p.S <= 32;
}

template <typename TIn, typename Epi>
hipError_t dispatch(const IgemmParams& p, int epi_vec, hipStream_t s) {
  // (the streaming kernel serves the 2-byte types only: no instantiation for the others)
  if constexpr (std::is_same<TIn, f16_t>::value || std::is_same<TIn, bf16_t>::value) {
    if (p.w_frag != nullptr && lean_steps(p) > 0) return launch_lean<TIn, Epi>(p, epi_vec, s);
  }
  // (the streaming 1x1 kernel and the short-tap kernel are built for 8-bit layers with 8-bit results)
  if constexpr (std::is_same<Epi, EpiQuant<0>>::value) {
    if (p.w_frag != nullptr && (epi_vec & 2) && igemm_stream_q8_geometry(p)) return launch_igemm_stream_q8(p, s);
    if (p.w_frag != nullptr && taps_shape(p).nkk > 0) return launch_taps<TIn, Epi>(p, epi_vec, s);
  }
  if (p.w_frag != nullptr && wreg_shape(p)) return launch_wreg<TIn, Epi>(p, epi_vec, s);
  return dispatch_tiles<TIn, Epi>(p, epi_vec, s);
}

}  // namespace

bool igemm_wants_wfrag(const IgemmParams& p) {
  return wreg_shape(p) || lean_steps(p) > 0 || taps_shape(p).nkk > 0 || igemm_stream_q8_geometry(p) || igemm_c3_geometry(p);
}

hipError_t launch_wfrag_pack(const WfragPackParams& p, hipStream_t stream) {
  if (p.src == nullptr || p.dst == nullptr || p.rows <= 0 || p.row_bytes <= 0 || p.row_bytes % 16 != 0 ||
      p.tiles * 32 < p.rows || p.chunks * 32 < p.row_bytes || p.chunks % 4 != 0 || p.batch <= 0)
    return hipErrorInvalidValue;
  if (!aligned16(p.src) || !aligned16(p.dst)) return hipErrorInvalidValue;
  const int64_t total = (int64_t)p.batch * p.tiles * p.chunks * 64;
  hipLaunchKernelGGL(wfrag_pack_kernel, dim3(grid_for(total, 256)), dim3(256), 0, stream, p);
  return hipGetLastError();
}

const char* igemm_variant_name(const IgemmParams& p) {
  switch (igemm_big_variant(p)) {
    case 1: return "256x256";
    case 2: return "256x128";
    case 3: return "128x256";
    default: break;
  }
  if (gemm_rowdot_shape(p)) return "rowdot";
  if (p.w_frag != nullptr && igemm_c3_geometry(p)) return "patch3x3";
  if (p.w_frag != nullptr && igemm_stream_q8_geometry(p)) return "stream";
  if (p.w_frag != nullptr && lean_steps(p) > 0) return "128x128s";
  if (p.w_frag != nullptr && taps_shape(p).nkk > 0) return "128x64t";
  if (p.w_frag != nullptr && wreg_shape(p)) {
    const bool rich = p.act == ACT_GELU_ERF || p.act == ACT_GELU_TANH || p.act == ACT_SIGMOID || p.act == ACT_TANH;
    const int nj = rich ? 1 : wreg_slices(p);
    const int64_t M = (int64_t)p.N * p.Ho * p.Wo;
    const int64_t tiles = ((M + 127) / 128) * ((p.Kout + 128 * nj - 1) / (128 * nj));
    if (!rich && nj == 1 && wreg_k_groups(p, tiles * p.batch) == 2) return "128x128w2k";   // two K groups per workgroup
    return "128x128w";
  }
  return choose_variant(p).name;
}

hipError_t launch_igemm(const IgemmParams& p_in, hipStream_t stream) {
  IgemmParams p = p_in;
  if (p.Ho > 0 && p.Wo > 0) {
    div_magic(p.Ho * p.Wo, &p.howo_magic, &p.howo_shift);
    div_magic(p.Wo, &p.wo_magic, &p.wo_shift);
  }
  if (p.y_rdiv > 0 && p.y_cdiv > 0) {
    div_magic(p.y_rdiv, &p.yr_magic, &p.yr_shift);
    div_magic(p.y_cdiv, &p.yc_magic, &p.yc_shift);
  }
  const int es = dtype_size(p.in_dt);
  if (es == 0 || p.x == nullptr || p.w == nullptr || p.y == nullptr) return hipErrorInvalidValue;
  const int vec = 16 / es;
  if (p.C <= 0 || p.C % vec != 0 || p.xcs % vec != 0 || p.w_rs % vec != 0) return hipErrorInvalidValue;
  if (p.x_bs % vec != 0 || p.w_bs % vec != 0) return hipErrorInvalidValue;
  if (!aligned16(p.x) || !aligned16(p.w)) return hipErrorInvalidValue;
  if (p.N <= 0 || p.H <= 0 || p.W <= 0 || p.Ho <= 0 || p.Wo <= 0 || p.Kout <= 0 || p.batch <= 0)
    return hipErrorInvalidValue;
  const bool rich = p.act == ACT_GELU_ERF || p.act == ACT_GELU_TANH || p.act == ACT_SIGMOID || p.act == ACT_TANH;
  if (p.act != ACT_NONE && p.act != ACT_RELU && p.act != ACT_LEAKY && p.act != ACT_CLAMP && !rich) return hipErrorInvalidValue;
  if (rich && (p.in_dt == DT_I8 || p.out_dt != p.in_dt)) return hipErrorInvalidValue;
  if (p.R <= 0 || p.S <= 0 || p.sh <= 0 || p.sw <= 0 || p.dh <= 0 || p.dw <= 0) return hipErrorInvalidValue;
  if (p.xcs < p.C || p.ycs < p.Kout) return hipErrorInvalidValue;
  if ((int64_t)p.H * p.W * p.xcs >= (1ll << 31)) return hipErrorInvalidValue;
  if ((int64_t)p.N * p.Ho * p.Wo >= (1ll << 31)) return hipErrorInvalidValue;
  if (p.w_rows <= 0 || p.w_cols <= 0 || p.w_cols > p.w_rs) return hipErrorInvalidValue;
  if (p.w_cols % vec != 0) return hipErrorInvalidValue;
  if (p.residual != nullptr && p.rcs < p.Kout) return hipErrorInvalidValue;
  if (p.y_rdiv > 0 || p.y_zdiv > 0) {
    // remapped result addressing: float results without residual; eight consecutive columns stay together
    if (!dtype_is_float(p.out_dt) || p.residual != nullptr) return hipErrorInvalidValue;
    if (p.y_rdiv > 0 && (p.y_cdiv <= 0 || p.y_cdiv % 8 != 0 || p.Kout % p.y_cdiv != 0 || p.y_rlo < p.y_cdiv)) return hipErrorInvalidValue;
  }
  if (p.w_frag != nullptr) {
    const int64_t kbytes = (int64_t)p.R * p.S * p.C * es;
    if (!aligned16(p.w_frag) || p.wf_chunks <= 0 || p.wf_chunks % 4 != 0 || (int64_t)p.wf_chunks * 32 < kbytes ||
        (int64_t)p.wf_chunks * 32 >= kbytes + 128 || (int64_t)p.wf_tiles * 32 < p.Kout)
      return hipErrorInvalidValue;
  }
  // (An output pixel may lie entirely in the padding: every tap is then masked.)
  // Source coordinates are computed in 32 bits.
  if ((int64_t)(p.Ho - 1) * p.sh + (int64_t)(p.R - 1) * p.dh >= (1ll << 30) ||
      (int64_t)(p.Wo - 1) * p.sw + (int64_t)(p.S - 1) * p.dw >= (1ll << 30) || p.ph >= (1 << 30) || p.pw >= (1 << 30))
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
  if (p.y_rdiv > 0) epi_vec = epi_vec && rows_ok(p.y, p.y_rlo, p.y_rhi) && rows_ok(p.y, p.y_chi, p.y_chi);
  if (p.y_zdiv > 0) epi_vec = epi_vec && rows_ok(p.y, p.ycs, p.y_bs_hi);
  if (p.residual != nullptr) epi_vec = epi_vec && rows_ok(p.residual, p.rcs, p.r_bs);
  if (p.bias != nullptr) epi_vec = epi_vec && ((reinterpret_cast<uintptr_t>(p.bias) % 16) == 0) && (p.bias_bs % 4 == 0);
  if (oes == 1) {
    // bit 2: 8-bit rows allow 16-byte accesses (the requantising epilogue moves 16 channels per lane)
    auto rows16 = [&](const void* ptr, int64_t cs, int64_t bs) {
      return cs % 16 == 0 && bs % 16 == 0 && (reinterpret_cast<uintptr_t>(ptr) % 16u) == 0;
    };
    bool ok16 = rows16(p.y, p.ycs, p.y_bs);
    if (p.residual != nullptr) ok16 = ok16 && rows16(p.residual, p.rcs, p.r_bs);
    if (ok16) epi_vec |= 2;
  }

  if (p.f_y != nullptr) {
    // a second layer rides in this launch: only the streaming row kernel computes it
    if (p.in_dt != DT_I8 || p.out_dt != DT_I8 || p.w_frag == nullptr || !(epi_vec & 2)) return hipErrorInvalidValue;
    return launch_igemm_stream_q8(p, stream);
  }
  if (gemm_rowdot_shape(p)) return launch_gemm_rowdot(p, stream);
  if (p.row_softmax != 0) return hipErrorInvalidValue;   // (no other kernel finishes with a Softmax)
  if (const int big = igemm_big_variant(p)) return launch_igemm_big(p, epi_vec, big, stream);
  if (p.w_frag != nullptr && igemm_c3_geometry(p)) return launch_igemm_c3(p, epi_vec, stream);

  switch (p.in_dt) {
    case DT_F32:
      if (p.out_dt != DT_F32) return hipErrorInvalidValue;
      if (rich) return dispatch<float, EpiFloat<float, true>>(p, epi_vec, stream);
      return dispatch<float, EpiFloat<float>>(p, epi_vec, stream);
    case DT_F16:
      if (p.out_dt == DT_F16 && rich) return dispatch<f16_t, EpiFloat<f16_t, true>>(p, epi_vec, stream);
      if (p.out_dt == DT_F16) return dispatch<f16_t, EpiFloat<f16_t>>(p, epi_vec, stream);
      if (p.out_dt == DT_F32) return dispatch<f16_t, EpiFloat<float>>(p, epi_vec, stream);
      return hipErrorInvalidValue;
    case DT_BF16:
      if (p.out_dt == DT_BF16 && rich) return dispatch<bf16_t, EpiFloat<bf16_t, true>>(p, epi_vec, stream);
      if (p.out_dt == DT_BF16) return dispatch<bf16_t, EpiFloat<bf16_t>>(p, epi_vec, stream);
      if (p.out_dt == DT_F32) return dispatch<bf16_t, EpiFloat<float>>(p, epi_vec, stream);
      return hipErrorInvalidValue;
    case DT_I8:
      if (p.out_dt == DT_I8) {
        if (p.qmul == nullptr) return hipErrorInvalidValue;
        return dispatch<int8_t, EpiQuant<0>>(p, epi_vec, stream);
      }
      if (p.out_dt == DT_F32) {
        if (p.qmul == nullptr) return hipErrorInvalidValue;
        return dispatch<int8_t, EpiQuant<1>>(p, 0, stream);
      }
      if (p.out_dt == DT_I32) return dispatch<int8_t, EpiQuant<2>>(p, 0, stream);
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
    bool live = o < p.Og && tap < taps && c < p.Cg;
    int cs = c;
    if (p.dense_groups > 0) {
      const int cg = p.Cg / p.dense_groups;
      cs = c - (o / (p.Og / p.dense_groups)) * cg;
      live = live && cs >= 0 && cs < cg;
    }
    if (live) {
      const int r = tap / p.S, s = tap - r * p.S;
      const int64_t og = (int64_t)g * p.Og + o;
      const TS v = reinterpret_cast<const TS*>(p.src)[og * p.so + cs * p.si + r * p.sr + s * p.ss];
      out = cvt_weight<TS, TD>(v);
    }
    reinterpret_cast<TD*>(p.dst)[i] = out;
  }
}

hipError_t launch_pack_weights(const PackWeightsParams& p, hipStream_t stream) {
  if (p.src == nullptr || p.dst == nullptr) return hipErrorInvalidValue;
  if (p.G <= 0 || p.Og <= 0 || p.Cg <= 0 || p.Cp < p.Cg || p.rows_pad < p.Og) return hipErrorInvalidValue;
  if (p.dense_groups < 0 || (p.dense_groups > 0 && (p.G != 1 || p.Og % p.dense_groups || p.Cg % p.dense_groups)))
    return hipErrorInvalidValue;
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
