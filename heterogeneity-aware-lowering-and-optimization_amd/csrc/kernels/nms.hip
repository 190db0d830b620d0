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
//          with an in-place bitonic sort of 64-bit keys in the workspace.
// Phase 3  greedy suppression in sorted order: the workgroup walks the list;
//          an unsuppressed candidate is emitted and all lanes mark the later
//          candidates whose IoU with it is >= iou_thr.  A suppressed candidate
//          never suppresses others, so the result equals the sequential
//          "compare with every kept box" rule.
//
// IoU uses the same fp32 operation order as the CPU formulation (corner boxes
// normalised with min/max, zero when either area is <= 0).
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

__device__ __forceinline__ Box4 norm_box(const float* b) {
  Box4 r;
  r.y1 = fminf(b[0], b[2]);
  r.x1 = fminf(b[1], b[3]);
  r.y2 = fmaxf(b[0], b[2]);
  r.x2 = fmaxf(b[1], b[3]);
  return r;
}

__device__ __forceinline__ float iou_of(const Box4& a, const Box4& b) {
  const float area_a = (a.y2 - a.y1) * (a.x2 - a.x1);
  const float area_b = (b.y2 - b.y1) * (b.x2 - b.x1);
  if (area_a <= 0.f || area_b <= 0.f) return 0.f;
  const float ih = fmaxf(fminf(a.y2, b.y2) - fmaxf(a.y1, b.y1), 0.f);
  const float iw = fmaxf(fminf(a.x2, b.x2) - fmaxf(a.x1, b.x1), 0.f);
  const float inter = ih * iw;
  return inter / (area_a + area_b - inter);
}

// best[n][b] = max over classes (first maximum), cls[n][b] = its class
__global__ void __launch_bounds__(256)
nms_best_class_kernel(const float* __restrict__ scores, int C, int B, float* __restrict__ best_ws,
                      int32_t* __restrict__ cls_ws) {
  const int n = blockIdx.y;
  const int b = blockIdx.x * 256 + threadIdx.x;
  if (b >= B) return;
  const float* sc = scores + (int64_t)n * C * B + b;
  float best = sc[0];
  int bc = 0;
  for (int c = 1; c < C; ++c) {
    const float v = sc[(int64_t)c * B];
    if (v > best) { best = v; bc = c; }
  }
  best_ws[(int64_t)n * B + b] = best;
  cls_ws[(int64_t)n * B + b] = bc;
}

__global__ void __launch_bounds__(kNmsThreads)
nms_kernel(const float* __restrict__ boxes, const float* __restrict__ best_ws, int B,
           int max_out, float iou_thr, float score_thr, int32_t* __restrict__ out,
           unsigned long long* keys_ws, const int32_t* cls_ws, unsigned char* sup_ws, int64_t bpad,
           int lds_slots) {
  const int n = blockIdx.x;
  const int tid = threadIdx.x;
  const float* bx = boxes + (int64_t)n * B * 4;
  const float* bestv = best_ws + (int64_t)n * B;
  unsigned long long* keys = keys_ws + (int64_t)n * bpad;
  const int32_t* cls = cls_ws + (int64_t)n * B;
  unsigned char* sup = sup_ws + (int64_t)n * bpad;
  int32_t* o = out + (int64_t)n * max_out * 3;

  __shared__ int s_count;
  if (tid == 0) s_count = 0;
  for (int i = tid; i < max_out * 3; i += kNmsThreads) o[i] = -1;
  __syncthreads();

  // ---- phase 1 (second half): threshold, append ----
  for (int b = tid; b < B; b += kNmsThreads) {
    const float best = bestv[b];
    if (best > score_thr) {
      const int slot = atomicAdd(&s_count, 1);
      unsigned u = __float_as_uint(best);
      u = (u & 0x80000000u) ? ~u : (u | 0x80000000u);  // ascending in u == ascending in value
      keys[slot] = ((unsigned long long)(~u) << 32) | (unsigned)b;  // score desc, then box asc
    }
  }
  __syncthreads();
  const int M = s_count;
  if (M == 0 || max_out == 0) return;
  const int P = (int)next_pow2(M);
  for (int i = M + tid; i < P; i += kNmsThreads) keys[i] = ~0ull;
  for (int i = tid; i < M; i += kNmsThreads) sup[i] = 0;
  __syncthreads();

  // ---- phase 2: bitonic sort of keys[0..P) ascending; in LDS when the list fits ----
  extern __shared__ unsigned long long lds_keys[];
  unsigned long long* sk = P <= lds_slots ? lds_keys : keys;
  if (sk != keys) {
    for (int i = tid; i < P; i += kNmsThreads) sk[i] = keys[i];
    __syncthreads();
  }
  for (int k = 2; k <= P; k <<= 1) {
    for (int j = k >> 1; j > 0; j >>= 1) {
      for (int i = tid; i < P; i += kNmsThreads) {
        const int l = i ^ j;
        if (l > i) {
          const unsigned long long a = sk[i], b = sk[l];
          const bool up = (i & k) == 0;
          if ((a > b) == up) { sk[i] = b; sk[l] = a; }
        }
      }
      __syncthreads();
    }
  }
  // With the list in LDS the sorted keys go back to memory and the candidates'
  // boxes and suppression flags take their place: the walk below is a chain of
  // short rounds, each as long as its slowest read.
  const bool in_lds = sk != keys;
  Box4* lbox = reinterpret_cast<Box4*>(lds_keys);
  unsigned char* lsup = reinterpret_cast<unsigned char*>(lbox + lds_slots);
  if (in_lds) {
    for (int i = tid; i < M; i += kNmsThreads) keys[i] = sk[i];
    __syncthreads();
    for (int i = tid; i < M; i += kNmsThreads) {
      lbox[i] = norm_box(bx + (int64_t)(keys[i] & 0xffffffffu) * 4);
      lsup[i] = 0;
    }
    __syncthreads();
  }
  unsigned char* const supf = in_lds ? lsup : sup;

  // ---- phase 3: greedy suppression ----
  int kept = 0;  // every thread counts the kept boxes itself: one barrier per kept box
  const bool flags8 = (reinterpret_cast<uintptr_t>(supf) & 7u) == 0;
  for (int i = 0; i < M; ++i) {
    // (uniform: the flags were written before the last barrier.)  Runs of
    // suppressed candidates are skipped eight flags per read: the walk is a chain
    // of dependent reads, one per step.
    if (flags8 && (i & 7) == 0) {
      while (i + 8 <= M && *reinterpret_cast<const unsigned long long*>(supf + i) == 0x0101010101010101ull) i += 8;
      if (i >= M) break;
    }
    if (supf[i]) continue;
    if (kept >= max_out) break;
    const int bi = (int)(keys[i] & 0xffffffffu);
    if (tid == 0) {
      o[kept * 3 + 0] = n;
      o[kept * 3 + 1] = cls[bi];
      o[kept * 3 + 2] = bi;
    }
    const Box4 a = in_lds ? lbox[i] : norm_box(bx + (int64_t)bi * 4);
    for (int j = i + 1 + tid; j < M; j += kNmsThreads) {
      if (!supf[j]) {
        const Box4 b = in_lds ? lbox[j] : norm_box(bx + (int64_t)(keys[j] & 0xffffffffu) * 4);
        // candidate j plays the role of "I", the kept box of "J" in the
        // reference formula; the expression is symmetric in fp32.
        if (iou_of(b, a) >= iou_thr) supf[j] = 1;
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

hipError_t launch_nms(const float* boxes, const float* scores, int N, int C, int B, int max_out,
                      float iou_thr, float score_thr, int32_t* out, void* workspace,
                      hipStream_t stream) {
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
  hipLaunchKernelGGL(nms_best_class_kernel, dim3((unsigned)((B + 255) / 256), (unsigned)N), dim3(256), 0, stream,
                     scores, C, B, best, cls);
  // candidate list in LDS - first the keys (8 B per slot), then boxes and flags in
  // their place (16 + 1 B per slot): up to 8192 candidates per image
  const int lds_slots = (int)(bpad < 8192 ? bpad : 8192);
  const size_t lds_bytes = (size_t)lds_slots * 17;
  static bool lds_limit_raised = false;  // (benign if two threads both do it)
  if (!lds_limit_raised) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(nms_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            8192 * 17) != hipSuccess)
      return hipErrorInvalidValue;
    lds_limit_raised = true;
  }
  hipLaunchKernelGGL(nms_kernel, dim3(N), dim3(kNmsThreads), lds_bytes, stream, boxes, best, B, max_out,
                     iou_thr, score_thr, out, keys, cls, sup, bpad, lds_slots);
  return hipGetLastError();
}

}  // namespace ohip
