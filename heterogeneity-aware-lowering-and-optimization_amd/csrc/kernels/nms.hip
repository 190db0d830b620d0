// Batched non-maximum suppression for gfx950: one launch over all boxes for the
// class reduction, then one workgroup per image.
//
// Phase 1  every box competes with its best class score (first maximum over
//          the class axis); boxes with score > score_thr become candidates.
//          scores are [C][B] per image, so for a fixed class consecutive lanes
//          read consecutive boxes.  The reduction over the classes reads the
//          whole score tensor and runs chip-wide (one thread per box); the
//          per-image workgroup only thresholds and appends.
// Phase 2  candidates are ordered by (score descending, box index ascending)
//          with a bitonic sort of 64-bit keys.
// Phase 3  greedy suppression in sorted order: the workgroup walks the list;
//          an unsuppressed candidate is emitted and all lanes mark the later
//          candidates whose IoU with it is >= iou_thr.  A suppressed candidate
//          never suppresses others, so the result equals the sequential
//          "compare with every kept box" rule.
//
// Up to 8192 candidates per image (the usual case by far) phases 2 and 3 keep
// everything on the compute unit: a thread holds its (up to eight) keys in
// registers, compare-exchange steps between lanes of a wavefront are lane
// shuffles, only steps between wavefronts go through LDS; in phase 3 a thread
// holds its candidates' boxes, areas, classes and liveness in registers, and a
// round reads one box and 64 liveness flags from LDS.  Longer lists are sorted
// and walked in the workspace.
//
// IoU uses the same fp32 operation order as the CPU formulation (corner boxes
// normalised with min/max, zero when either area is <= 0).  Boxes and scores
// are read in their storage type (fp32 / fp16 / bf16); the conversion to fp32 is
// exact.
#include "device_utils.h"

namespace ohip {
namespace {

constexpr int kNmsThreads = 1024;

__host__ __device__ inline int64_t next_pow2(int64_t v) {
  int64_t p = 1;
  while (p < v) p <<= 1;
  return p;
}

struct Box4 { float y1, x1, y2, x2; };

template <typename TB>
__device__ __forceinline__ Box4 norm_box(const TB* b) {
  const float b0 = Store<TB>::ld(b), b1 = Store<TB>::ld(b + 1), b2 = Store<TB>::ld(b + 2), b3 = Store<TB>::ld(b + 3);
  Box4 r;
  r.y1 = fminf(b0, b2);
  r.x1 = fminf(b1, b3);
  r.y2 = fmaxf(b0, b2);
  r.x2 = fmaxf(b1, b3);
  return r;
}

__device__ __forceinline__ float box_area(const Box4& a) { return (a.y2 - a.y1) * (a.x2 - a.x1); }

__device__ __forceinline__ float iou_of(const Box4& a, const float area_a, const Box4& b, const float area_b) {
  if (area_a <= 0.f || area_b <= 0.f) return 0.f;
  const float ih = fmaxf(fminf(a.y2, b.y2) - fmaxf(a.y1, b.y1), 0.f);
  const float iw = fmaxf(fminf(a.x2, b.x2) - fmaxf(a.x1, b.x1), 0.f);
  const float inter = ih * iw;
  return inter / (area_a + area_b - inter);
}

// best[n][b] = max over classes (first maximum), cls[n][b] = its class
template <typename TS>
__global__ void __launch_bounds__(256)
nms_best_class_kernel(const TS* __restrict__ scores, int C, int B, float* __restrict__ best_ws,
                      int32_t* __restrict__ cls_ws) {
  const int n = blockIdx.y;
  const int b = blockIdx.x * 256 + threadIdx.x;
  if (b >= B) return;
  const TS* sc = scores + (int64_t)n * C * B + b;
  float best = Store<TS>::ld(sc);
  int bc = 0;
  int c = 1;
  for (; c + 8 <= C; c += 8) {   // eight loads in flight; the comparisons keep the class order
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = Store<TS>::ld(sc + (int64_t)(c + u) * B);
#pragma unroll
    for (int u = 0; u < 8; ++u)
      if (v[u] > best) { best = v[u]; bc = c + u; }
  }
  for (; c < C; ++c) {
    const float v = Store<TS>::ld(sc + (int64_t)c * B);
    if (v > best) { best = v; bc = c; }
  }
  best_ws[(int64_t)n * B + b] = best;
  cls_ws[(int64_t)n * B + b] = bc;
}

// One compare-exchange of the bitonic network seen from element i: `mine` stays or
// is replaced by `other` (the value of element i ^ j).
__device__ __forceinline__ unsigned long long bitonic_pick(const unsigned long long mine, const unsigned long long other,
                                                           const int i, const int j, const int k) {
  const bool lower = (i & j) == 0, up = (i & k) == 0;
  const unsigned long long lo = mine < other ? mine : other, hi = mine < other ? other : mine;
  return lower == up ? lo : hi;
}

constexpr int kNmsPerThread = 8;   // candidates a thread holds when the list stays on the compute unit

// Phases 2 and 3 for a list of at most lds_slots candidates (M of them, P = next
// power of two), whose keys phase 1 left in `lds` [0, M).
template <typename TB>
__device__ __forceinline__ void nms_on_cu(const TB* __restrict__ bx, const int32_t* __restrict__ cls, int32_t* __restrict__ o,
                                          unsigned long long* lds, const int n, const int M, const int P,
                                          const int max_out, const float iou_thr) {
  const int tid = threadIdx.x;
  const int R = P > kNmsThreads ? P / kNmsThreads : 1;   // elements per thread: i = tid + m * kNmsThreads
  unsigned long long e[kNmsPerThread];
#pragma unroll
  for (int m = 0; m < kNmsPerThread; ++m) {
    const int i = tid + m * kNmsThreads;
    e[m] = (m < R && i < M) ? lds[i] : ~0ull;
  }
  __syncthreads();   // the keys are in registers: LDS becomes two exchange buffers of P keys

  int xsel = 0;
  for (int k = 2; k <= P; k <<= 1) {
    for (int j = k >> 1; j > 0; j >>= 1) {
      if (j >= kNmsThreads) {   // both elements in this thread
#pragma unroll
        for (int db = 0; db < 3; ++db) {
          if ((j / kNmsThreads) != (1 << db)) continue;
#pragma unroll
          for (int m = 0; m < kNmsPerThread; ++m) {
            if ((m & (1 << db)) != 0 || m >= R) continue;
            const int i = tid + m * kNmsThreads;
            const unsigned long long a = e[m], b = e[m | (1 << db)];
            e[m] = bitonic_pick(a, b, i, j, k);
            e[m | (1 << db)] = bitonic_pick(b, a, i | j, j, k);
          }
        }
      } else if (j >= 64) {     // the other element is in another wavefront: through LDS
        unsigned long long* x = lds + xsel * P;
        xsel ^= 1;   // the buffers alternate, so one barrier per step is enough
#pragma unroll
        for (int m = 0; m < kNmsPerThread; ++m) {
          const int i = tid + m * kNmsThreads;
          if (m < R && i < P) x[i] = e[m];
        }
        __syncthreads();
#pragma unroll
        for (int m = 0; m < kNmsPerThread; ++m) {
          const int i = tid + m * kNmsThreads;
          if (m < R && i < P) e[m] = bitonic_pick(e[m], x[i ^ j], i, j, k);
        }
      } else {                  // the other element is in another lane of this wavefront
#pragma unroll
        for (int m = 0; m < kNmsPerThread; ++m) {
          if (m >= R) continue;
          const int i = tid + m * kNmsThreads;
          const unsigned long long other = __shfl_xor(e[m], j, 64);
          e[m] = bitonic_pick(e[m], other, i, j, k);
        }
      }
    }
  }
  __syncthreads();   // every exchange has been read: LDS becomes the candidates' boxes and flags

  Box4* lbox = reinterpret_cast<Box4*>(lds);
  unsigned char* lsup = reinterpret_cast<unsigned char*>(lbox + P);
  Box4 mb[kNmsPerThread];
  float marea[kNmsPerThread];
  int mbi[kNmsPerThread], mcls[kNmsPerThread], mrow[kNmsPerThread];
  unsigned alive = 0;
#pragma unroll
  for (int m = 0; m < kNmsPerThread; ++m) {
    const int i = tid + m * kNmsThreads;
    mb[m] = Box4{0.f, 0.f, 0.f, 0.f};
    marea[m] = 0.f;
    mbi[m] = 0;
    mcls[m] = 0;
    mrow[m] = -1;
    if (m < R && i < M) {
      mbi[m] = (int)(e[m] & 0xffffffffu);
      mb[m] = norm_box(bx + (int64_t)mbi[m] * 4);
      marea[m] = box_area(mb[m]);
      mcls[m] = cls[mbi[m]];
      lbox[i] = mb[m];
      lsup[i] = 0;
      alive |= 1u << m;
    }
  }
  __syncthreads();

  const int lane = tid & 63;
  int kept = 0;   // every thread counts the kept boxes itself: one barrier per kept box
  int i = 0;
  while (i < M) {
    // (uniform: the flags were written before the last barrier.)  The next candidate
    // that is still alive, 64 flags per read.
    const int probe = i + lane;
    const unsigned long long live = __ballot(probe < M && lsup[probe] == 0);
    if (live == 0) { i += 64; continue; }
    i += __ffsll(live) - 1;
    if (kept >= max_out) break;
    const Box4 a = lbox[i];
    const float area_a = box_area(a);
    if (tid == (i & (kNmsThreads - 1))) {   // its owner notes the output row (written behind the walk:
#pragma unroll                              // a round has no access to memory in it)
      for (int m = 0; m < kNmsPerThread; ++m)
        if (m == i / kNmsThreads) mrow[m] = kept;
    }
#pragma unroll
    for (int m = 0; m < kNmsPerThread; ++m) {
      const int j = tid + m * kNmsThreads;
      // candidate j plays the role of "I", the kept box of "J" in the reference
      // formula; the expression is symmetric in fp32.
      if (m < R && j > i && ((alive >> m) & 1u) && iou_of(mb[m], marea[m], a, area_a) >= iou_thr) {
        alive &= ~(1u << m);
        lsup[j] = 1;
      }
    }
    ++kept;
    ++i;
    __syncthreads();
  }
#pragma unroll
  for (int m = 0; m < kNmsPerThread; ++m) {
    if (mrow[m] >= 0) {
      o[mrow[m] * 3 + 0] = n;
      o[mrow[m] * 3 + 1] = mcls[m];
      o[mrow[m] * 3 + 2] = mbi[m];
    }
  }
}

template <typename TB>
__global__ void __launch_bounds__(kNmsThreads)
nms_kernel(const TB* __restrict__ boxes, const float* __restrict__ best_ws, int B,
           int max_out, float iou_thr, float score_thr, int32_t* __restrict__ out,
           unsigned long long* keys_ws, const int32_t* cls_ws, unsigned char* sup_ws, int64_t bpad,
           int lds_slots, int image_base) {
  const int n = blockIdx.x;
  const int tid = threadIdx.x;
  const TB* bx = boxes + (int64_t)n * B * 4;
  const float* bestv = best_ws + (int64_t)n * B;
  unsigned long long* keys = keys_ws + (int64_t)n * bpad;
  const int32_t* cls = cls_ws + (int64_t)n * B;
  unsigned char* sup = sup_ws + (int64_t)n * bpad;
  int32_t* o = out + (int64_t)n * max_out * 3;
  extern __shared__ unsigned long long lds_keys[];

  __shared__ int s_count;
  if (tid == 0) s_count = 0;
  for (int i = tid; i < max_out * 3; i += kNmsThreads) o[i] = -1;
  __syncthreads();

  // ---- phase 1 (second half): threshold, append (to the workspace, and to LDS while it has room) ----
  for (int b0 = 0; b0 < B; b0 += 4 * kNmsThreads) {
    float v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int b = b0 + u * kNmsThreads + tid;
      v[u] = b < B ? bestv[b] : score_thr;   // (not above the threshold)
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (v[u] > score_thr) {
        const int b = b0 + u * kNmsThreads + tid;
        const int slot = atomicAdd(&s_count, 1);
        unsigned w = __float_as_uint(v[u]);
        w = (w & 0x80000000u) ? ~w : (w | 0x80000000u);  // ascending in w == ascending in value
        const unsigned long long key = ((unsigned long long)(~w) << 32) | (unsigned)b;  // score desc, then box asc
        keys[slot] = key;
        if (slot < lds_slots) lds_keys[slot] = key;
      }
    }
  }
  __syncthreads();
  const int M = s_count;
  if (M == 0 || max_out == 0) return;
  const int P = (int)next_pow2(M);
  if (P <= lds_slots && P <= kNmsThreads * kNmsPerThread) {
    nms_on_cu<TB>(bx, cls, o, lds_keys, image_base + n, M, P, max_out, iou_thr);
    return;
  }

  // ---- the list does not fit: phases 2 and 3 in the workspace ----
  for (int i = M + tid; i < P; i += kNmsThreads) keys[i] = ~0ull;
  for (int i = tid; i < M; i += kNmsThreads) sup[i] = 0;
  __syncthreads();
  for (int k = 2; k <= P; k <<= 1) {
    for (int j = k >> 1; j > 0; j >>= 1) {
      for (int i = tid; i < P; i += kNmsThreads) {
        const int l = i ^ j;
        if (l > i) {
          const unsigned long long a = keys[i], b = keys[l];
          const bool up = (i & k) == 0;
          if ((a > b) == up) { keys[i] = b; keys[l] = a; }
        }
      }
      __syncthreads();
    }
  }
  int kept = 0;  // every thread counts the kept boxes itself: one barrier per kept box
  const bool flags8 = (reinterpret_cast<uintptr_t>(sup) & 7u) == 0;
  for (int i = 0; i < M; ++i) {
    // (uniform: the flags were written before the last barrier.)  Runs of
    // suppressed candidates are skipped eight flags per read: the walk is a chain
    // of dependent reads, one per step.
    if (flags8 && (i & 7) == 0) {
      while (i + 8 <= M && *reinterpret_cast<const unsigned long long*>(sup + i) == 0x0101010101010101ull) i += 8;
      if (i >= M) break;
    }
    if (sup[i]) continue;
    if (kept >= max_out) break;
    const int bi = (int)(keys[i] & 0xffffffffu);
    if (tid == 0) {
      o[kept * 3 + 0] = image_base + n;   // (the image's number in the caller's batch)
      o[kept * 3 + 1] = cls[bi];
      o[kept * 3 + 2] = bi;
    }
    const Box4 a = norm_box(bx + (int64_t)bi * 4);
    const float area_a = box_area(a);
    for (int j = i + 1 + tid; j < M; j += kNmsThreads) {
      if (!sup[j]) {
        const Box4 b = norm_box(bx + (int64_t)(keys[j] & 0xffffffffu) * 4);
        if (iou_of(b, box_area(b), a, area_a) >= iou_thr) sup[j] = 1;
      }
    }
    ++kept;
    __syncthreads();
  }
}

}  // namespace

size_t nms_workspace_bytes(int N, int B) {
  const int64_t bpad = next_pow2(B);
  // keys (8 B) + suppression flags (1 B) per padded slot, class and best score per box (4 B each)
  size_t bytes = (size_t)N * bpad * 8;
  bytes += (size_t)N * B * 4 * 2;
  bytes += (size_t)N * bpad;
  return (bytes + 255) & ~(size_t)255;
}

template <typename TB>
static hipError_t launch_nms_kernel(const void* boxes, const float* best, int N, int B, int max_out, float iou_thr,
                                    float score_thr, int32_t* out, unsigned long long* keys, const int32_t* cls,
                                    unsigned char* sup, int64_t bpad, int image_base, hipStream_t stream) {
  // candidate list on the compute unit - first the keys (two exchange buffers of 8 B per
  // slot), then boxes and flags in their place (16 + 1 B per slot): up to 8192 candidates
  const int lds_slots = (int)(bpad < 8192 ? bpad : 8192);
  const size_t lds_bytes = (size_t)lds_slots * 17;
  static bool lds_limit_raised = false;  // (benign if two threads both do it)
  if (!lds_limit_raised) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(nms_kernel<TB>), hipFuncAttributeMaxDynamicSharedMemorySize,
                            8192 * 17) != hipSuccess)
      return hipErrorInvalidValue;
    lds_limit_raised = true;
  }
  hipLaunchKernelGGL(nms_kernel<TB>, dim3(N), dim3(kNmsThreads), lds_bytes, stream, (const TB*)boxes, best, B, max_out,
                     iou_thr, score_thr, out, keys, cls, sup, bpad, lds_slots, image_base);
  return hipGetLastError();
}

hipError_t launch_nms(const void* boxes, DType boxes_dt, const void* scores, DType scores_dt, int N, int C, int B,
                      int max_out, float iou_thr, float score_thr, int32_t* out, void* workspace,
                      hipStream_t stream, int image_base) {
  if (!boxes || !scores || !out || !workspace || N <= 0 || C <= 0 || B <= 0 || max_out < 0)
    return hipErrorInvalidValue;
  if ((reinterpret_cast<uintptr_t>(workspace) & 7u) != 0) return hipErrorInvalidValue;
  const int64_t bpad = next_pow2(B);
  if (bpad > (1 << 24)) return hipErrorInvalidValue;
  unsigned long long* keys = reinterpret_cast<unsigned long long*>(workspace);
  int32_t* cls = reinterpret_cast<int32_t*>(keys + (int64_t)N * bpad);
  float* best = reinterpret_cast<float*>(cls + (int64_t)N * B);
  unsigned char* sup = reinterpret_cast<unsigned char*>(best + (int64_t)N * B);
  if (N > 65535) return hipErrorInvalidValue;
  const dim3 grid1((unsigned)((B + 255) / 256), (unsigned)N);
  switch (scores_dt) {
    case DT_F32: hipLaunchKernelGGL(nms_best_class_kernel<float>, grid1, dim3(256), 0, stream, (const float*)scores, C, B, best, cls); break;
    case DT_F16: hipLaunchKernelGGL(nms_best_class_kernel<f16_t>, grid1, dim3(256), 0, stream, (const f16_t*)scores, C, B, best, cls); break;
    case DT_BF16: hipLaunchKernelGGL(nms_best_class_kernel<bf16_t>, grid1, dim3(256), 0, stream, (const bf16_t*)scores, C, B, best, cls); break;
    default: return hipErrorInvalidValue;
  }
  switch (boxes_dt) {
    case DT_F32: return launch_nms_kernel<float>(boxes, best, N, B, max_out, iou_thr, score_thr, out, keys, cls, sup, bpad, image_base, stream);
    case DT_F16: return launch_nms_kernel<f16_t>(boxes, best, N, B, max_out, iou_thr, score_thr, out, keys, cls, sup, bpad, image_base, stream);
    case DT_BF16: return launch_nms_kernel<bf16_t>(boxes, best, N, B, max_out, iou_thr, score_thr, out, keys, cls, sup, bpad, image_base, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace ohip
