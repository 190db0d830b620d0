// 3x3 convolutions with stride 1 and padding 1 (NHWC, constant weights) whose
// input patch lives in LDS: a workgroup of WS wavefronts computes a tile of 4 pixel
// blocks (BR rows x BC columns each, stacked vertically, BR * BC <= 32) of ONE image
// for 32 * WS * NJ output channels; every wavefront owns NJ 32-channel slices and all
// four blocks, so that a weight fragment feeds four MFMAs and a pixel fragment NJ.  Per chunk of NKK * 32 bytes of input channels it
// stages the (4 BR + 2) x (BC + 2) patch of input pixels around the tile once and
// runs all nine taps on it: nine K stages of MFMAs per patch, where the gathering
// kernels fetch 128 pixel rows per stage (the same input bytes nine times).
//
// LDS layout of a patch chunk: one plane of 3 KiB per 16-byte piece of the chunk,
// plane[c][patch pixel] - the 32 pixels a fragment read covers are 16-byte slots of one
// plane, a tap is a constant offset from the lane's base address: (r * PW + s) * 16, and
// which MFMA column takes which pixel of a block is chosen such that the sixteen lanes the
// LDS serves in one pass read sixteen different banks (c3_lane_table).
// Patch pixels outside the image hold the byte that represents 0.
//
// Weights come fragment-ordered from the packed copy (p.w_frag), one K stage
// (tap x chunk) ahead, straight into registers.  Two patch buffers alternate: the
// next chunk's patch is requested at the start of a chunk, parked in registers
// during its nine stages and written to the other buffer at its end; one
// workgroup barrier per chunk.
//
// The epilogues are the shared ones, told through a table in LDS which output
// pixel each of the tile's 128 positions is (-1: none - rows past the image,
// lanes past BR * BC).
#include <hip/hip_runtime.h>

#include <cstdlib>
#include <type_traits>

#include "igemm_common.h"

namespace ohip {
namespace {

struct C3Geom {
  int br = 0, bc = 0;            // pixel block
  int pw = 0, npp = 0;           // patch width (bc + 2) and pixels ((4 br + 2) * pw)
  int tiles_x = 0, tiles_y = 0;  // tiles per image
  int tiles_n = 0;               // channel tiles of 32 * ws * nj channels
  int nck = 0;                   // channel chunks
  int cpt = 0;                   // 32-byte K chunks per tap (C * element size / 32)
  int nkk = 0, ws = 0, nj = 0;   // template choice
  int main_bytes = 0;            // LDS ahead of the pixel table
  float eff = 0.f;               // share of the MFMA columns that are output pixels
  // Which position of a pixel block (row-major, br x bc) MFMA column l takes: byte l of
  // lane_pos[l / 8]; bit 7 marks a column past the block, which reads the pixel of another
  // column of its LDS pass and stores nothing.
  unsigned long long lane_pos[4] = {0, 0, 0, 0};
};

constexpr int kC3Plane = 3072;   // bytes of a patch plane: 192 patch pixels x 16 bytes
// LDS ahead of the pixel table: the patch buffers (two; one when the layer has a single chunk),
// or the epilogue's staging tiles if those are larger
inline int c3_main_bytes(const int nkk, const int ws, const int nck) {
  const int bufs = (nck > 1 ? 2 : 1) * nkk * 2 * kC3Plane;
  const int epi = ws == 4 ? 2 * 32 * (128 + 4) * 4 : 2 * 32 * (32 + 4) * 4;
  return bufs > epi ? bufs : epi;
}

// NJ = 2: every wavefront owns two 32-channel slices, i.e. every pixel fragment read from LDS
// feeds two MFMAs (with one slice the LDS read rate saturates together with the matrix pipes).
template <typename TIn, typename Epi, int NKK, int WS, int NJ>
__global__ __launch_bounds__(WS * 64, NJ == 1 ? 3 : 2) void igemm_c3_kernel(const IgemmParams p, const int epi_vec, const C3Geom g) {
  constexpr int NCH = NKK * 2;   // 16-byte planes of a chunk
  constexpr int CKB = NKK * 32;  // bytes of a chunk
  constexpr int PLANE = kC3Plane;
  constexpr int BUF = NCH * PLANE;
  constexpr int NB = 4;          // pixel blocks of the tile, all of them in every wavefront
  constexpr int NT = WS * 64;    // threads
  constexpr int PR = (kC3Plane / 16 + NT - 1) / NT;   // patch pixels per thread
  using Acc = typename Mma<TIn>::Acc;
  static_assert(WS == 4 || WS == 2, "four wavefronts, or two");

  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];  // g.main_bytes + 512
  int* mtab = reinterpret_cast<int*>(smem + g.main_bytes);

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int l32 = lane & 31, lg = lane >> 5;
  const int M = p.N * p.H * p.W;

  int bid = blockIdx.x;
  {
    // neighbouring tiles (which share weights and patch borders) on one XCD's L2
    const int per = gridDim.x >> 3;
    if (bid < (per << 3)) bid = (bid & 7) * per + (bid >> 3);
  }
  const int tile_n = bid % g.tiles_n;
  int t = bid / g.tiles_n;
  const int tx = t % g.tiles_x;
  t /= g.tiles_x;
  const int ty = t % g.tiles_y;
  const int n_img = t / g.tiles_y;
  const int y0 = ty * 4 * g.br, x0 = tx * g.bc;

  // which output pixel each position of the tile is
  auto lane_pos = [&](const int l) __attribute__((always_inline)) {
    const unsigned long long w = l < 16 ? (l < 8 ? g.lane_pos[0] : g.lane_pos[1]) : (l < 24 ? g.lane_pos[2] : g.lane_pos[3]);
    return (int)((w >> ((l & 7) * 8)) & 0xff);
  };
  if (tid < 128) {
    const int blk = tid >> 5, q = lane_pos(tid & 31);
    const int br = (q & 0x7f) / g.bc, bc = (q & 0x7f) - br * g.bc;
    const int yy = y0 + blk * g.br + br, xx = x0 + bc;
    mtab[tid] = (q < 0x80 && yy < p.H && xx < p.W) ? (n_img * p.H + yy) * p.W + xx : -1;
  }

  // this thread's patch pixels: tid, tid + NT, ..
  const unsigned fill_w = (unsigned)(p.a_fill & 0xff) * 0x01010101u;
  const uintx4 fill = {fill_w, fill_w, fill_w, fill_w};
  const unsigned char* src[PR];
  bool inside[PR];
#pragma unroll
  for (int r = 0; r < PR; ++r) {
    const int pp = tid + r * NT;
    const int py = pp / g.pw, px = pp - py * g.pw;
    const int gy = y0 - 1 + py, gx = x0 - 1 + px;
    inside[r] = pp < g.npp && gy >= 0 && gy < p.H && gx >= 0 && gx < p.W;
    src[r] = reinterpret_cast<const unsigned char*>(p.x) +
             ((int64_t)(n_img * p.H + (inside[r] ? gy : 0)) * p.W + (inside[r] ? gx : 0)) * p.xcs * (int64_t)sizeof(TIn);
  }

  // The patch of the next chunk travels through registers in PH pieces of NCH / PH planes, so
  // that a thread parks 32 bytes at a time (the whole patch at once for the first chunk, whose
  // registers nothing else needs yet).
  constexpr int PH = 2 * PR < NCH ? 2 * PR : NCH;   // pieces
  constexpr int PP = NCH / PH;                      // planes per piece
  uintx4 pr[PR][PP];
  // Requests are unconditional (a position outside the image or past the patch reads the
  // image's first pixel and is replaced by the fill value when it is parked): a request inside a
  // branch is waited for right there, with everything else in flight, because the compiler
  // copies its result out of the branch.
  auto patch_load = [&](const int ck, const int c0) __attribute__((always_inline)) {
#pragma unroll
    for (int r = 0; r < PR; ++r)
#pragma unroll
      for (int c = 0; c < PP; ++c) pr[r][c] = *reinterpret_cast<const uintx4*>(src[r] + (int64_t)ck * CKB + (c0 + c) * 16);
  };
  auto patch_store = [&](const int buf, const int c0) __attribute__((always_inline)) {
    // (the wait for the requests sits here, in straight-line code, not inside the branch below)
#pragma unroll
    for (int r = 0; r < PR; ++r)
#pragma unroll
      for (int c = 0; c < PP; ++c) epi_settle(pr[r][c]);
#pragma unroll
    for (int r = 0; r < PR; ++r) {
      const int pp = tid + r * NT;
      if (pp < g.npp) {
#pragma unroll
        for (int c = 0; c < PP; ++c)
          *reinterpret_cast<uintx4*>(smem + buf * BUF + (c0 + c) * PLANE + pp * 16) = inside[r] ? pr[r][c] : fill;
      }
    }
  };

  // this wavefront's channel slices: slice j is block wave of channel tile tile_n * NJ + j (the
  // epilogue's view: WS blocks of 32 channels side by side per tile)
  const unsigned char* wfp[NJ];
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    int wtile = (tile_n * NJ + j) * WS + wave;
    wtile = wtile < p.wf_tiles ? wtile : p.wf_tiles - 1;
    wfp[j] = reinterpret_cast<const unsigned char*>(p.w_frag) + (int64_t)wtile * p.wf_chunks * 1024 + lane * 16;
  }
  // fragments of K step st (tap st / NKK, 32-byte piece st % NKK) of chunk ck
  auto wload = [&](uintx4 (&dst)[NJ], const int ck, const int st) __attribute__((always_inline)) {
    const int64_t off = (int64_t)((st / NKK) * g.cpt + ck * NKK + st % NKK) * 1024;
#pragma unroll
    for (int j = 0; j < NJ; ++j) dst[j] = *reinterpret_cast<const uintx4*>(wfp[j] + off);
  };

  // LDS address of the window's top left pixel, per block
  unsigned base[NB];
  {
    const int q = lane_pos(l32) & 0x7f;
    const int br = q / g.bc;
    const int bc = q - br * g.bc;
#pragma unroll
    for (int i = 0; i < NB; ++i) base[i] = (unsigned)(((i * g.br + br) * g.pw + bc) * 16 + lg * PLANE);
  }

  // Weight fragments: a ring of RW K steps, requested RW - 1 steps ahead of their use.  The
  // steps of a chunk are a multiple of RW, so step st of every chunk sits in slot st % RW.
  constexpr int STEPS = 9 * NKK;
  // (deeper rings were measured slower: 9 and 12 steps against 6, ResNet-50 at batch 256, the
  //  3x3 layers at 14 x 14: int8 250 -> 259 -> 264 us, fp16 435 -> 465 -> 504 us for the six)
  constexpr int RW = NJ == 1 ? 6 : (STEPS % 4 == 0 ? 4 : 3), AHEAD = RW - 1;
  static_assert(STEPS % RW == 0, "the ring position of a step must not depend on the chunk");
  uintx4 w[RW][NJ];
  {
    // the first patch: every request of a thread in flight at once (its registers are free:
    // the accumulators are not live yet)
    // (conditional here: with two wavefronts most threads have no second patch pixel, and
    //  nothing else is in flight yet that a wait inside the branch could hold up)
    uintx4 first[PR][NCH];
#pragma unroll
    for (int r = 0; r < PR; ++r) {
#pragma unroll
      for (int c = 0; c < NCH; ++c) first[r][c] = fill;
      if (inside[r]) {
#pragma unroll
        for (int c = 0; c < NCH; ++c) first[r][c] = *reinterpret_cast<const uintx4*>(src[r] + c * 16);
      }
    }
#pragma unroll
    for (int r = 0; r < PR; ++r) {
      const int pp = tid + r * NT;
      if (pp < g.npp) {
#pragma unroll
        for (int c = 0; c < NCH; ++c) *reinterpret_cast<uintx4*>(smem + c * PLANE + pp * 16) = first[r][c];
      }
    }
  }
#pragma unroll
  for (int st = 0; st < AHEAD; ++st) wload(w[st], 0, st);

  Acc acc[NJ][NB][1];
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[j][i][0][e] = 0;
    if constexpr (EpiTraits<Epi>::quant) acc_init_bias_vec<NB, 1>(p, 0, ((tile_n * NJ + j) * WS + wave) * 32, lg, acc[j]);
  }
  __syncthreads();

  // pixel fragments of the step in flight and of the next one
  uintx4 b[2][NB];
  auto bread = [&](uintx4 (&dst)[NB], const unsigned char* buf, const int tap, const int kk) __attribute__((always_inline)) {
    const unsigned off = (unsigned)(((tap / 3) * g.pw + (tap % 3)) * 16) + kk * 2 * PLANE;
#pragma unroll
    for (int i = 0; i < NB; ++i) dst[i] = *reinterpret_cast<const uintx4*>(buf + base[i] + off);
  };

  for (int ck = 0; ck < g.nck; ++ck) {
    const unsigned char* buf = smem + (ck & 1) * BUF;
    // (two wavefronts x one slice serve single-chunk layers only: no code for a second patch)
    const bool more = !(WS == 2 && NJ == 1) && ck + 1 < g.nck;
    const int nbuf = (ck + 1) & 1;
    bread(b[0], buf, 0, 0);
    // The scheduling barriers keep the requests where they are written - ahead of the MFMAs
    // of the steps before their use; left alone, the compiler moves every request down to
    // its use and waits for it there.
#pragma unroll
    for (int st = 0; st < STEPS; ++st) {
      // (behind the last chunk the ring re-reads that chunk's first steps: a request that is
      //  always made keeps the number of operations in flight a constant the compiler can count)
      if (st + AHEAD < STEPS) wload(w[(st + AHEAD) % RW], ck, st + AHEAD);
      else wload(w[(st + AHEAD) % RW], more ? ck + 1 : ck, st + AHEAD - STEPS);
      // The next chunk's patch, piece k requested at step k * STEPS / (PH + 1) and written at the
      // next of these points.  Nobody reads the other buffer any more: every wavefront has
      // passed the barrier that ended the chunk before, i.e. has finished that chunk's reads.
      if (more) {
#pragma unroll
        for (int k = 0; k <= PH; ++k)
          if (st == k * STEPS / (PH + 1)) {
            if (k > 0) patch_store(nbuf, (k - 1) * PP);
            if (k < PH) patch_load(ck + 1, k * PP);
          }
      }
      if (st + 1 < STEPS) bread(b[(st + 1) & 1], buf, (st + 1) / NKK, (st + 1) % NKK);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int j = 0; j < NJ; ++j)
#pragma unroll
        for (int i = 0; i < NB; ++i) acc[j][i][0] = Mma<TIn>::run(w[st % RW][j], b[st & 1][i], acc[j][i][0]);
      __builtin_amdgcn_sched_barrier(0);
    }
    __syncthreads();
  }

#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    if constexpr (WS == 4) {
      igemm_epilogue_rows128<TIn, Epi, 4, false>(p, epi_vec, acc[j], smem, 0, tile_n * NJ + j, 0, M, wave, lane, nullptr, mtab);
    } else {
      igemm_epilogue<TIn, Epi, 128, 64, 128, 32>(p, epi_vec, acc[j], smem, 0, tile_n * NJ + j, 0, M, wave, lane, 0, mtab);
    }
  }
}

// LDS passes of a pixel-fragment read.  A 16-byte read of a wavefront is served in four passes
// of sixteen lanes - within each half of the wavefront lanes {0-3, 12-15, 20-27} and lanes
// {4-11, 16-19, 28-31} (measured: two lanes that trade their slots cost a pass exactly when
// they are of different sets) - and two lanes of a pass conflict when their 16-byte slots are
// equal modulo 16 (256 bytes = all banks).  Position q of a block sits in slot
// (q / bc) * (bc + 2) + q % bc of its plane (plus a common offset); which MFMA column takes
// which position is free, so the positions are dealt to the two sets such that a set holds
// every slot residue once where the block's shape allows that (no residue more than twice).
// Returns the passes of the worse set and writes the table (C3Geom::lane_pos).
int c3_lane_table(const int br, const int bc, unsigned long long (*table)[4]) {
  static const int kSet[2][16] = {{0, 1, 2, 3, 12, 13, 14, 15, 20, 21, 22, 23, 24, 25, 26, 27},
                                  {4, 5, 6, 7, 8, 9, 10, 11, 16, 17, 18, 19, 28, 29, 30, 31}};
  int members[2][16], count[2] = {0, 0}, used[2][16] = {{0}, {0}};
  for (int q = 0; q < br * bc; ++q) {
    const int r = ((q / bc) * (bc + 2) + q % bc) & 15;
    int s;
    if (count[0] >= 16) s = 1;
    else if (count[1] >= 16) s = 0;
    else if (used[0][r] != used[1][r]) s = used[0][r] < used[1][r] ? 0 : 1;
    else s = count[0] <= count[1] ? 0 : 1;
    members[s][count[s]++] = q;
    ++used[s][r];
  }
  int worst = 1;
  unsigned char pos[32];
  for (int s = 0; s < 2; ++s) {
    for (int r = 0; r < 16; ++r) worst = used[s][r] > worst ? used[s][r] : worst;
    // (a column past the block reads what another column of its pass reads: one address, no conflict)
    const int spare = count[s] > 0 ? members[s][0] : 0;
    for (int k = 0; k < 16; ++k) pos[kSet[s][k]] = (unsigned char)(k < count[s] ? members[s][k] : (spare | 0x80));
  }
  if (table)
    for (int w = 0; w < 4; ++w) {
      (*table)[w] = 0;
      for (int b = 0; b < 8; ++b) (*table)[w] |= (unsigned long long)pos[w * 8 + b] << (b * 8);
    }
  return worst;
}

bool c3_geometry(const IgemmParams& p, C3Geom* out) {
  if (const char* e = getenv("ODLA_HIP_C3")) {  // tuning aid: 0 keeps these layers on the gathering kernels
    if (e[0] == '0') return false;
  }
  const int es = dtype_size(p.in_dt);
  if (p.in_dt != DT_F16 && p.in_dt != DT_BF16 && p.in_dt != DT_I8) return false;
  if (p.out_dt != p.in_dt || p.batch != 1) return false;
  if (p.R != 3 || p.S != 3 || p.sh != 1 || p.sw != 1 || p.dh != 1 || p.dw != 1 || p.ph != 1 || p.pw != 1) return false;
  if (p.Ho != p.H || p.Wo != p.W) return false;
  if (p.y_rdiv > 0 || p.y_zdiv > 0) return false;
  if (p.act != ACT_NONE && p.act != ACT_RELU && p.act != ACT_LEAKY && p.act != ACT_CLAMP) return false;
  C3Geom g;
  const int cb = p.C * es;
  if (cb % 128 == 0) g.nkk = 4;
  else if (cb == 64) g.nkk = 2;
  else return false;
  g.nck = cb / (g.nkk * 32);
  g.cpt = cb / 32;
  // Wavefronts x slices per wavefront: 4 x 1 (128 channels per workgroup) or 2 x 1 (64).  Two
  // slices per wavefront (4 x 2: 256 channels, 2 x 2: 128) halve the LDS reads per MFMA and were
  // measured no faster (ResNet-50 int8 at batch 256, 3x3 256 -> 256 at 14 x 14: 41.5 against
  // 40 us; 128 -> 128 at 28 x 28 as 2 x 2: 50 against 41 us): with the K loop removed these
  // launches still take 13 and 27 us, and in the loop a wavefront waits for weight fragments,
  // not for LDS.  ODLA_HIP_C3_SLICES=2 selects them for measurement.
  int nj2 = 0;
  if (const char* e = getenv("ODLA_HIP_C3_SLICES")) nj2 = atoi(e) == 2 ? 1 : 0;
  if (p.Kout % 256 == 0 && nj2) { g.ws = 4; g.nj = 2; }
  else if (p.Kout % 128 == 0 && nj2 && g.nkk == 4) { g.ws = 2; g.nj = 2; }
  else if (p.Kout % 128 == 0) { g.ws = 4; g.nj = 1; }
  else if (p.Kout == 64 && g.nck == 1) { g.ws = 2; g.nj = 1; }
  else return false;
  g.tiles_n = p.Kout / (32 * g.ws * g.nj);
  g.main_bytes = c3_main_bytes(g.nkk, g.ws, g.nck);
  // The block shape that wastes the fewest MFMA columns (lanes past the block, rows past the
  // image), a shape whose fragment reads take two LDS passes counting as 15 % worse (measured
  // on 56-column images: 28 x 1 blocks, 12.5 % of the columns idle but conflict-free, against
  // 8 x 4: int8 49 -> 46.5 us, fp16 88 -> 85.7 us); among equals the smallest patch per pixel.
  float best_halo = 0.f, best_score = 0.f;
  int force_bc = 0;
  if (const char* e = getenv("ODLA_HIP_C3_BC")) force_bc = atoi(e);   // tuning aid: block columns
  for (int bc = 32; bc >= 4; --bc) {
    // Blocks of 16 or 32 columns may hang over the right edge (a 30-column image as blocks of
    // 32 x 1); other widths must divide the image's.
    const bool over = (bc == 16 || bc == 32) && p.W % bc != 0;
    if ((p.W % bc != 0 && !over) || (force_bc > 0 && (p.W % force_bc == 0 || force_bc == 16 || force_bc == 32) && bc != force_bc)) continue;
    int br = 32 / bc;
    if (br > p.H) br = p.H;
    const int th = 4 * br, ty = (p.H + th - 1) / th;
    const int tx = (p.W + bc - 1) / bc;
    const float eff = (float)(br * bc) / 32.f * (float)p.H / (float)(ty * th) * (float)p.W / (float)(tx * bc);
    const int npp = (th + 2) * (bc + 2);
    if (npp > kC3Plane / 16) continue;
    const float halo = (float)npp / (float)(th * bc);
    const float score = c3_lane_table(br, bc, nullptr) == 1 ? eff : 0.85f * eff;
    if (score > best_score + 1e-6f || (score > best_score - 1e-6f && halo < best_halo)) {
      g.eff = eff; best_halo = halo; best_score = score;
      g.br = br; g.bc = bc; g.pw = bc + 2; g.npp = npp;
      g.tiles_x = tx; g.tiles_y = ty;
    }
  }
  float min_eff = 0.7f;
  if (const char* e = getenv("ODLA_HIP_C3_MIN_FILL")) min_eff = (float)atof(e);  // tuning aid
  if (g.bc == 0 || g.eff < min_eff) return false;
  c3_lane_table(g.br, g.bc, &g.lane_pos);
  const int64_t wgs = (int64_t)p.N * g.tiles_y * g.tiles_x * g.tiles_n;
  if (wgs <= 0 || wgs > 0x7fffffff) return false;
  if ((int64_t)p.N * p.H * p.W * p.xcs * es >= (1ll << 40)) return false;
  if (out) *out = g;
  return true;
}

template <typename TIn, typename Epi>
hipError_t launch_c3(const IgemmParams& p, const int epi_vec, const C3Geom& g, hipStream_t stream) {
  const dim3 grid((unsigned)((int64_t)p.N * g.tiles_y * g.tiles_x * g.tiles_n)), block(g.ws * 64);
  // (more than the 64 KiB a kernel may use without asking)
#define C3_CASE(NKK, WS, NJ)                                                                                            \
  if (g.nkk == NKK && g.ws == WS && g.nj == NJ) {                                                                       \
    static bool ready = false; /* (repeating the call is harmless: no lock) */                                          \
    if (!ready) {                                                                                                       \
      const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&igemm_c3_kernel<TIn, Epi, NKK, WS, NJ>), \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, c3_main_bytes(NKK, WS, 2) + 512); \
      if (e != hipSuccess) return e;                                                                                    \
      ready = true;                                                                                                     \
    }                                                                                                                   \
    hipLaunchKernelGGL((igemm_c3_kernel<TIn, Epi, NKK, WS, NJ>), grid, block, lds, stream, p, epi_vec, g);             \
    return hipGetLastError();                                                                                           \
  }
  const int lds = g.main_bytes + 512;
  C3_CASE(4, 4, 1)
  C3_CASE(4, 2, 1)
  C3_CASE(2, 4, 1)
  C3_CASE(2, 2, 1)
  C3_CASE(4, 4, 2)
  C3_CASE(4, 2, 2)
  C3_CASE(2, 4, 2)
#undef C3_CASE
  return hipErrorInvalidValue;
}

}  // namespace

bool igemm_c3_geometry(const IgemmParams& p) { return c3_geometry(p, nullptr); }

hipError_t launch_igemm_c3(const IgemmParams& p, const int epi_vec, hipStream_t stream) {
  C3Geom g;
  if (p.w_frag == nullptr || !c3_geometry(p, &g)) return hipErrorInvalidValue;
  switch (p.in_dt) {
    case DT_F16: return launch_c3<f16_t, EpiFloat<f16_t>>(p, epi_vec, g, stream);
    case DT_BF16: return launch_c3<bf16_t, EpiFloat<bf16_t>>(p, epi_vec, g, stream);
    case DT_I8:
      if (p.qmul == nullptr) return hipErrorInvalidValue;
      return launch_c3<int8_t, EpiQuant<0>>(p, epi_vec, g, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace ohip
