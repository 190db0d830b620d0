// Streaming kernel for 8-bit 1x1 convolutions over short pixel rows (gfx950).
//
// The 1x1 layers of a network's first stages move far more bytes than they
// compute: 64 -> 256 channels at 56 x 56 and batch 256 reads 51 MB (+ 205 MB of
// residual) and writes 205 MB for 26 GOP.  A tiled GEMM with a K loop, operand
// staging and workgroup barriers turns such a layer into a chain of latencies
// per tile.  Here nothing is staged per tile and nothing is shared but the
// weights:
//   * a workgroup keeps ALL weights of the layer (Kout x K bytes <= 64 KiB, in
//     MFMA fragment order), the int32 bias and the multipliers in LDS for its
//     whole life and walks pixel groups with a grid stride;
//   * a wavefront owns 32 pixels x all output channels: the 16 bytes a lane
//     feeds to v_mfma_i32_32x32x32_i8 are one contiguous piece of its pixel's
//     row, so the pixel operand goes straight from global memory into the
//     operand registers, once per tile;
//   * per 32-channel slice: the weight fragments come from LDS, the
//     accumulators start at the bias, the requantisation runs in the accumulator
//     layout (four consecutive channels of one pixel per dword), and the 16-byte
//     row vectors of the result - and of the residual, in the other direction -
//     are formed by exchanging dwords between lanes l and l + 32
//     (v_permlane32_swap): no LDS round trip, no barrier, no wave-level fence.
// The arithmetic of the result is that of igemm_epilogue_q8 (requant4).
#include "igemm_common.h"

#include <cstdlib>
#include <cstring>

namespace ohip {

namespace {

// X' = [X.lo | Y.lo], Y' = [X.hi | Y.hi] over the two 32-lane halves (its own inverse).
__device__ __forceinline__ void swap32(unsigned& x, unsigned& y) {
#if defined(__HIP_DEVICE_COMPILE__)
  const uintx2 r = __builtin_amdgcn_permlane32_swap(x, y, false, false);
  x = r.x;
  y = r.y;
#endif
}

// Accumulator layout of one 32 x 32 block: lane (l32, lg) holds, for pixel l32,
// the dwords of channel groups q*8 + lg*4 (q = 0..3).  Row layout: lane (l32, lg)
// holds the 16 consecutive channels lg*16 .. lg*16 + 15 of pixel l32.
// For lg = 0 the row vector holds the groups (q0,0) (q0,1) (q1,0) (q1,1), for lg = 1
// (q2,0) (q2,1) (q3,0) (q3,1), where group (q, s) = channels q*8 + s*4 .. + 3.
// rows -> accumulator dwords d[q]
__device__ __forceinline__ void rows_to_acc(const uintx4 v, unsigned (&d)[4]) {
  unsigned a = v.x, b = v.y, c = v.z, e = v.w;
  swap32(a, b);   // a' = [(q0,0) | (q0,1)]: group q0 at every lane's own lg;  b' = [(q2,0) | (q2,1)]
  swap32(c, e);   // c' = [(q1,0) | (q1,1)],  e' = [(q3,0) | (q3,1)]
  d[0] = a; d[2] = b; d[1] = c; d[3] = e;
}
// accumulator dwords d[q] -> rows
__device__ __forceinline__ uintx4 acc_to_rows(const unsigned (&d)[4]) {
  unsigned a = d[0], b = d[2], c = d[1], e = d[3];
  swap32(a, b);   // a' = [(q0,0) | (q2,0)], b' = [(q0,1) | (q2,1)]
  swap32(c, e);   // c' = [(q1,0) | (q3,0)], e' = [(q1,1) | (q3,1)]
  return uintx4{a, b, c, e};
}

constexpr int kStreamMaxLds = 64 * 1024 + 8 * 1024;

template <int NKK, int NS, int NW>
__global__ void __launch_bounds__(NW * 64, 2)
igemm_stream_q8_kernel(const IgemmParams p, const int groups) {
  // NKK: 32-byte K steps per pixel row; NS: 32-channel slices (Kout / 32); NW: wavefronts
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int l32 = lane & 31, lg = lane >> 5;
  const int M = p.N * p.Ho * p.Wo;
  constexpr int KOUT = NS * 32;            // channels of this workgroup: [n0, n0 + KOUT)
  const int n0 = blockIdx.y * KOUT;

  uintx4* wl = reinterpret_cast<uintx4*>(smem);                              // [NS][NKK][64] fragments
  int* bl = reinterpret_cast<int*>(smem + (size_t)NS * NKK * 1024);          // [Kout] bias
  float* ml = reinterpret_cast<float*>(bl + KOUT);                           // [Kout] multipliers
  {
    const uintx4* wf = reinterpret_cast<const uintx4*>(p.w_frag);
    constexpr int per_slice = NKK * 64;
    for (int u = tid; u < NS * per_slice; u += NW * 64) {
      const int t = u / per_slice, rem = u - t * per_slice;
      wl[u] = wf[(int64_t)(n0 / 32 + t) * p.wf_chunks * 64 + rem];
    }
    const int* bias = reinterpret_cast<const int*>(p.bias);
    for (int c = tid; c < KOUT; c += NW * 64) {
      bl[c] = bias != nullptr ? bias[n0 + c] : 0;
      ml[c] = p.qmul[n0 + c];
    }
  }
  __syncthreads();

  const int8_t* x = reinterpret_cast<const int8_t*>(p.x);
  int8_t* y = reinterpret_cast<int8_t*>(p.y);
  const int8_t* res = reinterpret_cast<const int8_t*>(p.residual);
  const bool has_res = res != nullptr;
  const bool clamp = p.q_lo > 0.f;   // (a lower bound of 0 is what the saturating conversion applies anyway)
  const int HoWo = p.Ho * p.Wo;
  const bool plain = p.sh == 1 && p.sw == 1 && p.Ho == p.H && p.Wo == p.W;   // output pixel m reads input pixel m

  // this lane's piece of the pixel operand of group g: bytes [32 kk + 16 lg, +16) of its pixel's row
  auto load_b = [&](const int g, uintx4 (&b)[NKK]) {
    int m = (g * NW + wave) * 32 + l32;
    m = m < M ? m : M - 1;
    int64_t xin = m;
    if (!plain) {
      const int n_img = fast_div(m, p.howo_magic, p.howo_shift);
      const int rem = m - n_img * HoWo;
      const int ho = fast_div(rem, p.wo_magic, p.wo_shift);
      const int wo = rem - ho * p.Wo;
      xin = ((int64_t)n_img * p.H + ho * p.sh) * p.W + wo * p.sw;
    }
    const uintx4* xrow = reinterpret_cast<const uintx4*>(x + xin * p.xcs) + lg;
#pragma unroll
    for (int kk = 0; kk < NKK; ++kk) b[kk] = xrow[2 * kk];
  };

  uintx4 b[NKK], bnext[NKK];
  if ((int)blockIdx.x < groups) load_b(blockIdx.x, b);
  for (int g = blockIdx.x; g < groups; g += gridDim.x) {
    const int m = (g * NW + wave) * 32 + l32;
    const bool live = m < M;
    const int mc = live ? m : M - 1;
    int8_t* yrow = y + (int64_t)mc * p.ycs + n0 + lg * 16;
    // the residual rows travel up to PRE slices ahead of their use: PRE KiB per wavefront in flight
    constexpr int PRE = NS < 8 ? NS : 8;
    uintx4 rr[NS];
    const int8_t* rrow = has_res ? res + (int64_t)mc * p.rcs + n0 + lg * 16 : nullptr;
    if (has_res) {
#pragma unroll
      for (int j = 0; j < PRE; ++j) rr[j] = *reinterpret_cast<const uintx4*>(rrow + j * 32);
    }
    // ... and so is the pixel operand of this wavefront's next tile
    const int gn = g + (int)gridDim.x;
    if (gn < groups) load_b(gn, bnext);

#pragma unroll
    for (int j = 0; j < NS; j += 2) {
      // (unrolled for the static indices of rr[]; the scheduler must not pull the LDS reads of
      //  every later pair up here, which would cost more registers than the chip has)
      __builtin_amdgcn_sched_barrier(0);
      if (has_res && j + PRE < NS) {
        rr[j + PRE] = *reinterpret_cast<const uintx4*>(rrow + (j + PRE) * 32);
        rr[j + PRE + 1] = *reinterpret_cast<const uintx4*>(rrow + (j + PRE + 1) * 32);
      }
      intx16 acc[2];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int* bj = bl + (j + h) * 32 + lg * 4;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const intx4 bv = *reinterpret_cast<const intx4*>(bj + q * 8);
          acc[h][q * 4 + 0] = bv.x; acc[h][q * 4 + 1] = bv.y; acc[h][q * 4 + 2] = bv.z; acc[h][q * 4 + 3] = bv.w;
        }
      }
      const uintx4* wj = wl + (size_t)j * NKK * 64 + lane;
#pragma unroll
      for (int kk = 0; kk < NKK; ++kk) {
        const uintx4 w0 = wj[kk * 64], w1 = wj[(NKK + kk) * 64];
        acc[0] = Mma<int8_t>::run(w0, b[kk], acc[0]);
        acc[1] = Mma<int8_t>::run(w1, b[kk], acc[1]);
      }
      auto finish = [&](auto with_res, auto with_clamp) __attribute__((always_inline)) {
        constexpr bool kRes = decltype(with_res)::value;
        constexpr bool kClamp = decltype(with_clamp)::value;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const float* mj = ml + (j + h) * 32 + lg * 4;
          unsigned out[4], rd[4] = {0u, 0u, 0u, 0u};
          if constexpr (kRes) rows_to_acc(rr[j + h], rd);
#pragma unroll
          for (int q = 0; q < 4; ++q)
            out[q] = requant4<kRes, kClamp>(acc[h][q * 4 + 0], acc[h][q * 4 + 1], acc[h][q * 4 + 2], acc[h][q * 4 + 3],
                                            *reinterpret_cast<const floatx4*>(mj + q * 8), rd[q], p);
          const uintx4 v = acc_to_rows(out);
          // (plain stores: a row leaves in 32-byte pieces, which only the cache assembles into lines;
          //  written around the cache such pieces cost several times the traffic)
          if (live) *reinterpret_cast<uintx4*>(yrow + (j + h) * 32) = v;
        }
      };
      // (wavefront-uniform choices)
      if (has_res) { if (clamp) finish(std::true_type{}, std::true_type{}); else finish(std::true_type{}, std::false_type{}); }
      else { if (clamp) finish(std::false_type{}, std::true_type{}); else finish(std::false_type{}, std::false_type{}); }
    }
#pragma unroll
    for (int kk = 0; kk < NKK; ++kk) b[kk] = bnext[kk];
  }
}

// The same walk with a row epilogue: a wavefront computes 128 channels (four slices) of its 32
// pixels at a time, requantises them in the accumulator layout (requant4, the arithmetic of
// igemm_epilogue_q8), turns the bytes into full 128-byte rows through its own LDS tile and moves
// rows (and residual rows) with non-temporal 16-byte accesses - eight lanes per row, where the
// lane-exchange form above moves 32-byte pieces.
//
// Order of the memory operations.  Loads and stores share one in-order counter, and the stores
// sit in branches (pixels past the end), so the compiler cannot count them: every wait for a
// load that comes after a store waits for that store too.  Hence: every request - the pixels of
// the next group, the residual rows of the NEXT 128-channel step - is made after the stores of
// the step before and is waited for (epi_settle) right before the stores of the current step.
// A step's MFMAs and requantisation then cover the latency of its requests, and a store burst
// has a whole step to drain before anything waits behind it.
// NG: groups of 128 channels of this workgroup (blockIdx.y selects its share of the layer's).
// NF > 0: a second 1x1 layer of NF * 32 channels over this layer's KOUT (all of them: one channel
// share) is computed from the staged byte tiles - after each 128-channel step the wavefront
// multiplies the tile it has just requantised, as it lies in LDS, into NF more accumulators, and
// after the last step requantises those with the second layer's parameters and writes them as
// rows of NF * 32 bytes (see IgemmParams::f_y).
template <int NKK, int NG, int NW, bool kRes, bool kClamp, int NF = 0>
__device__ __forceinline__ void stream_rows_body(const IgemmParams& p, const int groups, unsigned char* smem) {
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int l32 = lane & 31, lg = lane >> 5;
  const int M = p.N * p.Ho * p.Wo;
  constexpr int NS = NG * 4;
  constexpr int KOUT = NS * 32;
  constexpr int PITCH = 128 + 16, TILE = 32 * PITCH;   // a staged [32 pixels][128 channels] byte tile
  const int n0 = blockIdx.y * KOUT;

  uintx4* wl = reinterpret_cast<uintx4*>(smem);                              // [NS][NKK][64] fragments
  int* bl = reinterpret_cast<int*>(smem + (size_t)NS * NKK * 1024);          // [KOUT] bias
  float* ml = reinterpret_cast<float*>(bl + KOUT);                           // [KOUT] multipliers
  // second layer: fragments [NF][KOUT / 32][64], bias and multipliers [NF * 32]
  uintx4* wl2 = reinterpret_cast<uintx4*>(ml + KOUT);
  int* bl2 = reinterpret_cast<int*>(wl2 + (size_t)NF * (KOUT / 32) * 64);
  float* ml2 = reinterpret_cast<float*>(bl2 + NF * 32);
  unsigned char* otile = reinterpret_cast<unsigned char*>(ml2 + NF * 32) + wave * (2 * TILE);
  unsigned char* rtile = otile + TILE;
  if constexpr (NF > 0) {
    const uintx4* wf2 = reinterpret_cast<const uintx4*>(p.f_wfrag);
    constexpr int per_slice2 = (KOUT / 32) * 64;
    for (int u = tid; u < NF * per_slice2; u += NW * 64) {
      const int t = u / per_slice2, rem = u - t * per_slice2;
      wl2[u] = wf2[(int64_t)t * p.f_wf_chunks * 64 + rem];
    }
    const int* bias2 = reinterpret_cast<const int*>(p.f_bias);
    for (int c = tid; c < NF * 32; c += NW * 64) {
      bl2[c] = bias2 != nullptr ? bias2[c] : 0;
      ml2[c] = p.f_qmul[c];
    }
  }
  {
    const uintx4* wf = reinterpret_cast<const uintx4*>(p.w_frag);
    constexpr int per_slice = NKK * 64;
    for (int u = tid; u < NS * per_slice; u += NW * 64) {
      const int t = u / per_slice, rem = u - t * per_slice;
      wl[u] = wf[(int64_t)(n0 / 32 + t) * p.wf_chunks * 64 + rem];
    }
    const int* bias = reinterpret_cast<const int*>(p.bias);
    for (int c = tid; c < KOUT; c += NW * 64) {
      bl[c] = bias != nullptr ? bias[n0 + c] : 0;
      ml[c] = p.qmul[n0 + c];
    }
  }
  __syncthreads();

  const int8_t* x = reinterpret_cast<const int8_t*>(p.x);
  int8_t* ybase = reinterpret_cast<int8_t*>(p.y);
  const int8_t* rbase = reinterpret_cast<const int8_t*>(p.residual);
  const int HoWo = p.Ho * p.Wo;
  const bool plain = p.sh == 1 && p.sw == 1 && p.Ho == p.H && p.Wo == p.W;
  auto load_b = [&](const int g, uintx4 (&b)[NKK]) {
    int m = (g * NW + wave) * 32 + l32;
    m = m < M ? m : M - 1;
    int64_t xin = m;
    if (!plain) {
      const int n_img = fast_div(m, p.howo_magic, p.howo_shift);
      const int rem = m - n_img * HoWo;
      const int ho = fast_div(rem, p.wo_magic, p.wo_shift);
      const int wo = rem - ho * p.Wo;
      xin = ((int64_t)n_img * p.H + ho * p.sh) * p.W + wo * p.sw;
    }
    const uintx4* xrow = reinterpret_cast<const uintx4*>(x + xin * p.xcs) + lg;
#pragma unroll
    for (int kk = 0; kk < NKK; ++kk) b[kk] = xrow[2 * kk];
  };
  // row passes: lane handles channels c16 .. c16 + 15 of pixel ps * 8 + rp
  const int rp = lane >> 3, c16 = (lane & 7) * 16;
  auto rreq = [&](const int g, const int grp, uintx4 (&r)[4]) {
#pragma unroll
    for (int ps = 0; ps < 4; ++ps) {
      int m = (g * NW + wave) * 32 + ps * 8 + rp;
      m = m < M ? m : M - 1;
      r[ps] = __builtin_nontemporal_load(reinterpret_cast<const uintx4*>(rbase + (int64_t)m * p.rcs + n0 + grp * 128 + c16));
    }
  };
  auto wave_fence = [&]() {
    // a wavefront only touches its own tiles and its LDS operations complete in issue order
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };

  uintx4 b[NKK], bnext[NKK], rnx[4];
#pragma unroll
  for (int ps = 0; ps < 4; ++ps) rnx[ps] = uintx4{0u, 0u, 0u, 0u};
  int g = blockIdx.x;   // (the launcher starts no more workgroups than there are pixel groups)
  load_b(g, b);
  if constexpr (kRes) rreq(g, 0, rnx);
  for (; g < groups; g += gridDim.x) {
    // (behind the last group a workgroup re-reads that group: a request that is always made is
    //  one the compiler can count)
    const int gn = g + (int)gridDim.x < groups ? g + (int)gridDim.x : g;
    load_b(gn, bnext);
    intx16 acc2[NF > 0 ? NF : 1];
    if constexpr (NF > 0) {
#pragma unroll
      for (int f = 0; f < NF; ++f) {
        const int* bj = bl2 + f * 32 + lg * 4;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const intx4 bv = *reinterpret_cast<const intx4*>(bj + q * 8);
          acc2[f][q * 4 + 0] = bv.x; acc2[f][q * 4 + 1] = bv.y; acc2[f][q * 4 + 2] = bv.z; acc2[f][q * 4 + 3] = bv.w;
        }
      }
    }
    static_for<NG>([&](auto grp_no) __attribute__((always_inline)) {
      constexpr int grp = decltype(grp_no)::value;
      intx16 acc[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int* bj = bl + (grp * 4 + j) * 32 + lg * 4;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const intx4 bv = *reinterpret_cast<const intx4*>(bj + q * 8);
          acc[j][q * 4 + 0] = bv.x; acc[j][q * 4 + 1] = bv.y; acc[j][q * 4 + 2] = bv.z; acc[j][q * 4 + 3] = bv.w;
        }
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uintx4* wj = wl + (size_t)(grp * 4 + j) * NKK * 64 + lane;
#pragma unroll
        for (int kk = 0; kk < NKK; ++kk) acc[j] = Mma<int8_t>::run(wj[kk * 64], b[kk], acc[j]);
      }
      if constexpr (kRes) {
        // this step's residual rows (settled before the stores of the step before) into LDS
#pragma unroll
        for (int ps = 0; ps < 4; ++ps)
          *reinterpret_cast<uintx4*>(rtile + (ps * 8 + rp) * PITCH + c16) = q8_swz_chunk(rnx[ps], ps * 8 + rp);
        wave_fence();
        // the next step's: the other channel group of these pixels, or the first of the next pixels
        if constexpr (grp + 1 < NG) rreq(g, grp + 1, rnx);
        else rreq(gn, 0, rnx);
      }
      // requantise in the accumulator layout: lane holds, for pixel l32, channels j*32 + q*8 + lg*4 + (0..3)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int ch = j * 32 + q * 8 + lg * 4;
          const int off = (l32 * PITCH + ch) ^ q8_swz(l32);
          const floatx4 m = *reinterpret_cast<const floatx4*>(ml + grp * 128 + ch);
          const unsigned rs = kRes ? *reinterpret_cast<const unsigned*>(rtile + off) : 0u;
          *reinterpret_cast<unsigned*>(otile + off) =
              requant4<kRes, kClamp>(acc[j][q * 4 + 0], acc[j][q * 4 + 1], acc[j][q * 4 + 2], acc[j][q * 4 + 3], m, rs, p);
        }
      wave_fence();
      if constexpr (NF > 0) {
        // the tile as the pixel operand of the second layer: lane (pixel l32, K half lg) takes
        // 16 stored bytes of each of the step's four 32-channel K steps
#pragma unroll
        for (int k2 = 0; k2 < 4; ++k2) {
          const uintx4 a2 = q8_swz_chunk(*reinterpret_cast<const uintx4*>(otile + l32 * PITCH + k2 * 32 + lg * 16), l32);
#pragma unroll
          for (int f = 0; f < NF; ++f)
            acc2[f] = Mma<int8_t>::run(wl2[(size_t)(f * (KOUT / 32) + grp * 4 + k2) * 64 + lane], a2, acc2[f]);
        }
      }
      uintx4 v[4];
#pragma unroll
      for (int ps = 0; ps < 4; ++ps) v[ps] = q8_swz_chunk(*reinterpret_cast<const uintx4*>(otile + (ps * 8 + rp) * PITCH + c16), ps * 8 + rp);
      // everything requested is complete before the first store
      if constexpr (kRes) {
#pragma unroll
        for (int ps = 0; ps < 4; ++ps) epi_settle(rnx[ps]);
      }
      if constexpr (grp == 0) {
#pragma unroll
        for (int kk = 0; kk < NKK; ++kk) epi_settle(bnext[kk]);
      }
#pragma unroll
      for (int ps = 0; ps < 4; ++ps) {
        const int m = (g * NW + wave) * 32 + ps * 8 + rp;
        if (m < M) store_row16(ybase + (int64_t)m * p.ycs + n0 + grp * 128 + c16, v[ps], true, 16, p.stream_out);
      }
      wave_fence();   // the tiles are written again by the next step
    });
    if constexpr (NF > 0) {
      IgemmParams p2;   // (only the two fields requant4 reads without a residual)
      p2.q_add = p.f_q_add;
      p2.q_lo = p.f_q_lo;
      const bool clamp2 = p.f_q_lo > 0.f;   // (wavefront-uniform)
#pragma unroll
      for (int f = 0; f < NF; ++f)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int ch = f * 32 + q * 8 + lg * 4;
          const int off = (l32 * PITCH + ch) ^ q8_swz(l32);
          const floatx4 m = *reinterpret_cast<const floatx4*>(ml2 + ch);
          *reinterpret_cast<unsigned*>(otile + off) =
              clamp2 ? requant4<false, true>(acc2[f][q * 4 + 0], acc2[f][q * 4 + 1], acc2[f][q * 4 + 2], acc2[f][q * 4 + 3], m, 0u, p2)
                     : requant4<false, false>(acc2[f][q * 4 + 0], acc2[f][q * 4 + 1], acc2[f][q * 4 + 2], acc2[f][q * 4 + 3], m, 0u, p2);
        }
      wave_fence();
      // rows of NF * 32 bytes: LR lanes per row, 64 / LR rows per pass (kept in the cache: the
      // next launch reads them)
      constexpr int LR = NF * 2, RPP = 64 / LR;
      const int rp2 = lane / LR, c2 = (lane % LR) * 16;
      int8_t* y2 = reinterpret_cast<int8_t*>(p.f_y);
#pragma unroll
      for (int ps = 0; ps < 32 / RPP; ++ps) {
        const int row = ps * RPP + rp2;
        const uintx4 v2 = q8_swz_chunk(*reinterpret_cast<const uintx4*>(otile + row * PITCH + c2), row);
        const int m = (g * NW + wave) * 32 + row;
        if (m < M) store_row16(y2 + (int64_t)m * p.f_ycs + c2, v2, true, 16, false);
      }
      wave_fence();
    }
#pragma unroll
    for (int kk = 0; kk < NKK; ++kk) b[kk] = bnext[kk];
  }
}

template <int NKK, int NG, int NW, int NF = 0>
__global__ void __launch_bounds__(NW * 64, 2)
igemm_stream_q8_rows_kernel(const IgemmParams p, const int groups, const int epi_vec) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  (void)epi_vec;   // rows and bases are 16-byte aligned and the channels whole groups of 128 (checked by the launcher)
  // (workgroup-uniform choices: the body is compiled once per case, so that none of its memory
  //  requests sits in a branch)
  if (p.residual != nullptr) {
    if (p.q_lo > 0.f) stream_rows_body<NKK, NG, NW, true, true, NF>(p, groups, smem);
    else stream_rows_body<NKK, NG, NW, true, false, NF>(p, groups, smem);
  } else {
    if (p.q_lo > 0.f) stream_rows_body<NKK, NG, NW, false, true, NF>(p, groups, smem);
    else stream_rows_body<NKK, NG, NW, false, false, NF>(p, groups, smem);
  }
}

}  // namespace

// Layers the streaming kernel serves: 8-bit 1x1 filters without padding, 8-bit
// result, K = 64 .. 512 bytes per pixel, a multiple of 64 output channels, all
// weights within 64 KiB, 16-byte aligned rows.
// Output channels a workgroup keeps the weights of (at most 64 KiB): all of them, or an
// equal share when the layer has more.
static int stream_q8_channels_per_wg(const IgemmParams& p) {
  if (p.C <= 0 || p.Kout <= 0) return 0;
  const int cap = (64 * 1024 / p.C) / 64 * 64;
  if (cap <= 0) return 0;
  if (p.Kout <= cap) return p.Kout;
  int n = cap;
  while (n >= 64 && p.Kout % n != 0) n -= 64;
  return n >= 64 ? n : 0;
}

bool igemm_stream_q8_geometry(const IgemmParams& p) {
  if (const char* force = getenv("ODLA_HIP_IGEMM_TILE")) {  // tuning aid
    if (strcmp(force, "stream") != 0 && force[0] != 0) return false;
  }
  if (const char* off = getenv("ODLA_HIP_STREAM_Q8")) {     // tuning aid: "0" turns the kernel off
    if (off[0] == '0') return false;
  }
  if (p.in_dt != DT_I8 || p.out_dt != DT_I8) return false;
  if (p.R != 1 || p.S != 1 || p.ph != 0 || p.pw != 0 || p.batch != 1) return false;
  if (p.C != 64 && p.C != 128 && p.C != 256 && p.C != 512) return false;
  if (p.xcs < p.C || p.xcs % 16 != 0) return false;
  if (p.Kout % 64 != 0 || p.Kout < 64) return false;
  {  // the instantiations that exist: K bytes per pixel / output channels per workgroup
    const int k = p.C, n = stream_q8_channels_per_wg(p);
    const bool built = (k == 64 && (n == 64 || n == 256)) || (k == 128 && (n == 128 || n == 512)) ||
                       (k == 256 && (n == 64 || n == 128 || n == 256)) || (k == 512 && n == 128);
    if (!built || p.Kout % n != 0) return false;
    // 512-byte pixel rows are built (and parity-clean) but selected only on request
    // (ODLA_HIP_STREAM_Q8=all): a lane's 16-byte piece of its pixel is then one of 32 pieces of
    // the row and every load touches 32 cache lines.  Measured on ResNet-50 at batch 256 against
    // the kernels that stage whole rows through LDS: 512 -> 128 at 28 x 28 33 -> 37 us, 512 -> 2048
    // at 7 x 7 32 -> 40 us.  256-byte rows are selected: with the row-epilogue form, same box,
    // 256 -> 128 at 56 x 56 81 -> 65 us, 256 -> 512 stride 2 72 -> 64 us, 256 -> 1024 + residual
    // 43.5 -> 41 us, 256 -> 64 (lane-exchange form) 57 -> 52 us.
    if (k > 256) {
      const char* sel = getenv("ODLA_HIP_STREAM_Q8");
      if (sel == nullptr || strcmp(sel, "all") != 0) return false;
    }
  }
  if ((int64_t)(p.Ho - 1) * p.sh >= p.H || (int64_t)(p.Wo - 1) * p.sw >= p.W) return false;
  if (p.ycs % 16 != 0 || (p.residual != nullptr && p.rcs % 16 != 0)) return false;
  if (p.y_rdiv > 0 || p.y_zdiv > 0) return false;
  return true;
}

static bool stream_q8_ready(const IgemmParams& p) {
  auto al16 = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15u) == 0; };
  return igemm_stream_q8_geometry(p) && p.w_frag != nullptr && p.qmul != nullptr && p.wf_chunks >= p.C / 32 &&
         al16(p.x) && al16(p.y) && al16(p.residual) && al16(p.w_frag);
}

// Pairs the row-epilogue form computes in one launch: 64 -> 256 channels (one channel share of two
// 128-channel groups) followed by a plain 1x1 layer 256 -> 64 or 256 -> 128 over the same pixels.  With more
// channels on either side the two layers' weights and the staged tiles no longer fit the LDS of a
// compute unit next to a second workgroup.
bool igemm_stream_q8_fusable(const IgemmParams& a, const IgemmParams& b) {
  if (const char* e = getenv("ODLA_HIP_STREAM_FUSE")) {   // tuning aid: 0 keeps the layers apart
    if (e[0] == '0') return false;
  }
  if (const char* e = getenv("ODLA_HIP_STREAM_ROWS")) {
    if (e[0] == '0') return false;
  }
  if (!igemm_stream_q8_geometry(a) || !igemm_stream_q8_geometry(b)) return false;
  if (a.C != 64 || a.Kout != 256 || a.ycs != 256) return false;
  if (b.C != 256 || b.xcs != 256 || (b.Kout != 64 && b.Kout != 128) || b.residual != nullptr || b.ycs % 16 != 0) return false;
  if (b.sh != 1 || b.sw != 1 || b.H != a.Ho || b.W != a.Wo || b.N != a.N || b.Ho != b.H || b.Wo != b.W) return false;
  return true;
}

// The row-epilogue form: 128-channel groups, four wavefronts, the layer's channels split over
// blockIdx.y so that a share's weights stay within 32 KiB.
static hipError_t launch_stream_q8_rows(const IgemmParams& p, hipStream_t stream) {
  const int64_t M = (int64_t)p.N * p.Ho * p.Wo;
  const int nkk = p.C / 32;
  int ng = p.Kout / 128;                          // groups per workgroup
  while (ng > 1 && (ng * 128 * p.C > 32 * 1024 || (ng != 1 && ng != 2))) ng = (ng % 2 == 0) ? ng / 2 : 1;
  const int nsplit = p.Kout / (ng * 128);
  const int nf = p.f_y != nullptr ? p.f_kout / 32 : 0;
  // (a second layer of 128 channels: its weights leave room for one workgroup per compute unit,
  //  which then has eight wavefronts instead of four)
  const int nw = nf == 4 ? 8 : 4;
  const int64_t groups = (M + nw * 32 - 1) / (nw * 32);
  if (nf != 0) {   // (igemm_stream_q8_fusable)
    auto al16 = [](const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15u) == 0; };
    if (nsplit != 1 || nkk != 2 || ng != 2 || (nf != 2 && nf != 4) || p.f_kout != nf * 32 || p.f_wfrag == nullptr ||
        p.f_qmul == nullptr || p.f_wf_chunks < 8 || p.f_ycs % 16 != 0 || !al16(p.f_y) || !al16(p.f_wfrag))
      return hipErrorInvalidValue;
  }
  // weights, bias and multipliers of the share (and of the second layer), two staged byte tiles per wavefront
  const size_t lds = (size_t)ng * 4 * nkk * 1024 + (size_t)ng * 128 * 8 + (size_t)nf * (ng * 4) * 1024 + (size_t)nf * 32 * 8 +
                     (size_t)nw * (2 * 32 * 144);
  if (groups > 0x7fffffff) return hipErrorInvalidValue;
  int per_cu = (int)((160 * 1024) / (lds + 512));
  per_cu = per_cu > 4 ? 4 : (per_cu < 1 ? 1 : per_cu);
  if (const char* e = getenv("ODLA_HIP_STREAM_WGS")) {
    const int v = atoi(e);
    if (v >= 1 && v <= 8) per_cu = v;
  }
  int64_t grid = (256 * per_cu + nsplit - 1) / nsplit;
  if (grid > groups) grid = groups;
  const int epi_vec = 3;   // rows and bases are 16-byte aligned (stream_q8_ready)
#define ROWS_CASE(NKK_, NG_)                                                                                         \
  if (nkk == NKK_ && ng == NG_) {                                                                                    \
    static bool attr_set = false;                                                                                   \
    if (!attr_set) {                                                                                                \
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&igemm_stream_q8_rows_kernel<NKK_, NG_, 4>), \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024);                    \
      if (e != hipSuccess) return e;                                                                                \
      attr_set = true;                                                                                              \
    }                                                                                                               \
    hipLaunchKernelGGL((igemm_stream_q8_rows_kernel<NKK_, NG_, 4>), dim3((unsigned)grid, (unsigned)nsplit), dim3(4 * 64), lds, stream, \
                       p, (int)groups, epi_vec);                                                                    \
    return hipGetLastError();                                                                                       \
  }
#define FUSED_CASE(NF_, NW_)                                                                                          \
  if (nf == NF_) {                                                                                                    \
    static bool attr_set = false;                                                                                    \
    if (!attr_set) {                                                                                                 \
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&igemm_stream_q8_rows_kernel<2, 2, NW_, NF_>), \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, 144 * 1024);                    \
      if (e != hipSuccess) return e;                                                                                 \
      attr_set = true;                                                                                               \
    }                                                                                                                \
    hipLaunchKernelGGL((igemm_stream_q8_rows_kernel<2, 2, NW_, NF_>), dim3((unsigned)grid, 1u), dim3(NW_ * 64), lds, stream, p, \
                       (int)groups, epi_vec);                                                                        \
    return hipGetLastError();                                                                                        \
  }
  FUSED_CASE(2, 4)
  FUSED_CASE(4, 8)
#undef FUSED_CASE
  ROWS_CASE(2, 1)
  ROWS_CASE(2, 2)
  ROWS_CASE(4, 1)
  ROWS_CASE(4, 2)
  ROWS_CASE(8, 1)
#undef ROWS_CASE
  return hipErrorInvalidValue;
}

hipError_t launch_igemm_stream_q8(const IgemmParams& p, hipStream_t stream) {
  if (!stream_q8_ready(p)) return hipErrorInvalidValue;
  // Layers with whole groups of 128 channels take the row-epilogue form.  Measured on ResNet-50
  // int8 at batch 256, same box: 64 -> 256 + residual 116 -> 96 us, 128 -> 512 + residual 63.5 -> 58 us,
  // and the layers that read these results lose the penalty the lane-exchange form's plain
  // residual loads left in the cache (256 -> 64 60 -> 57 us, 512 -> 128 39 -> 34 us, 512 -> 256 55 -> 48 us):
  // 2.68 -> 2.57 ms per step.  ODLA_HIP_STREAM_ROWS=0 keeps the lane-exchange form.
  if (p.Kout % 128 == 0 && (p.C == 64 || p.C == 128 || p.C == 256)) {
    const char* e = getenv("ODLA_HIP_STREAM_ROWS");
    if (e == nullptr || e[0] != '0' || p.f_y != nullptr) {
      const hipError_t r = launch_stream_q8_rows(p, stream);
      if (r != hipErrorInvalidValue) return r;
    }
  }
  if (p.f_y != nullptr) return hipErrorInvalidValue;   // (the lane-exchange form computes no second layer)
  const int64_t M = (int64_t)p.N * p.Ho * p.Wo;
  const int kout_wg = stream_q8_channels_per_wg(p);
  const int nkk = p.C / 32, ns = kout_wg / 32, nsplit = p.Kout / kout_wg;
  // wavefronts per workgroup as instantiated below (four where registers or LDS hold the
  // compute unit to fewer wavefronts: more, smaller workgroups then fill it better)
  const int nw = ((nkk == 4 && ns == 16) || (nkk == 8 && ns >= 4) || nkk == 16) ? 4 : 8;
  const int64_t groups = (M + nw * 32 - 1) / (nw * 32);
  const size_t lds = (size_t)ns * nkk * 1024 + (size_t)kout_wg * 8;
  if (lds > (size_t)kStreamMaxLds || groups > 0x7fffffff) return hipErrorInvalidValue;
  // resident workgroups walk the pixel groups with a grid stride
  int per_cu = (int)((160 * 1024) / (lds + 512));
  const int by_waves = 16 / nw;   // up to four wavefronts per SIMD
  if (per_cu > by_waves) per_cu = by_waves;
  if (per_cu < 1) per_cu = 1;
  if (const char* e = getenv("ODLA_HIP_STREAM_WGS")) {  // tuning aid: workgroups per compute unit
    const int v = atoi(e);
    if (v >= 1 && v <= 8) per_cu = v;
  }
  int64_t grid = (256 * per_cu + nsplit - 1) / nsplit;   // per channel share
  if (grid > groups) grid = groups;
#define STREAM_CASE(NKK_, NS_, NW_)                                                                                 \
  if (nkk == NKK_ && ns == NS_) {                                                                          \
    static bool attr_set = false;                                                                                   \
    if (!attr_set) {                                                                                                \
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&igemm_stream_q8_kernel<NKK_, NS_, NW_>),   \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, kStreamMaxLds);               \
      if (e != hipSuccess) return e;                                                                                \
      attr_set = true;                                                                                              \
    }                                                                                                               \
    hipLaunchKernelGGL((igemm_stream_q8_kernel<NKK_, NS_, NW_>), dim3((unsigned)grid, (unsigned)nsplit), dim3(NW_ * 64), lds, stream, \
                       p, (int)groups);                                                                             \
    return hipGetLastError();                                                                                       \
  }
  STREAM_CASE(2, 2, 8)
  STREAM_CASE(2, 8, 8)
  STREAM_CASE(4, 4, 8)
  STREAM_CASE(4, 16, 4)
  STREAM_CASE(8, 2, 8)
  STREAM_CASE(8, 4, 4)
  STREAM_CASE(8, 8, 4)
  STREAM_CASE(16, 4, 4)
#undef STREAM_CASE
  return hipErrorInvalidValue;
}

}  // namespace ohip
