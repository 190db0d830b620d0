// YOLOv3 post-processing as one operator: box decode of the three heads and the
// per-class suppression walk of the reference's post-processor.
// [ref: models/vision/detection/yolo/yolov3_postproc.cc:34-88 (decode), :90-153
//  (per-class walk); ODLA/platforms/odla_popart/custom_ops/codelets_nms.cpp:24-125
//  (the same two steps as device code of the PostProcess custom operator)]
#include <hip/hip_runtime.h>

#include <cfloat>
#include <climits>

#include "kernels.h"

namespace ohip {
namespace {

// One thread per (anchor, cell) of a head stored as [3 * (5 + classes)][dim][dim];
// cells are the fast index so that every channel read is coalesced.  The box
// lands at position first + cell * 3 + anchor, the order in which the reference
// walks its channels-last copy of the head.
__global__ void __launch_bounds__(256)
yolo_decode_kernel(const float* __restrict__ head, const int dim, const int classes, const int first,
                   const int total, const int anchor_w0, const int anchor_h0, const int anchor_w1,
                   const int anchor_h1, const int anchor_w2, const int anchor_h2,
                   const int* __restrict__ img_w_ptr, const int* __restrict__ img_h_ptr,
                   float* __restrict__ boxes, float* __restrict__ scores) {
  const int cells = dim * dim;
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= 3 * cells) return;
  const int a = t / cells, cell = t - a * cells;
  const int gy = cell / dim, gx = cell - gy * dim;
  const float img_w = (float)(unsigned)img_w_ptr[0], img_h = (float)(unsigned)img_h_ptr[0];
  // letterbox of the source image inside the 416 x 416 network input
  const float scale = fminf(416.0f / img_h, 416.0f / img_w);
  const float new_h = roundf(img_h * scale), new_w = roundf(img_w * scale);
  const float offset_h = (416.0f - new_h) / 2.0f / 416.0f, offset_w = (416.0f - new_w) / 2.0f / 416.0f;
  const float scale_h = 416.0f / new_h, scale_w = 416.0f / new_w;
  const float aw = (float)(a == 0 ? anchor_w0 : a == 1 ? anchor_w1 : anchor_w2);
  const float ah = (float)(a == 0 ? anchor_h0 : a == 1 ? anchor_h1 : anchor_h2);

  const float* p = head + (int64_t)a * (5 + classes) * cells + cell;
  // every logit goes through exp first; sigmoid(v) is then e / (e + 1)
  const float e0 = expf(p[0]), e1 = expf(p[cells]), e2 = expf(p[2 * cells]), e3 = expf(p[3 * cells]);
  const float e4 = expf(p[4 * cells]);
  float dx = ((e0 / (e0 + 1.0f)) + (float)gx) / (float)dim;
  dx = (dx - offset_w) * scale_w;
  float dy = ((e1 / (e1 + 1.0f)) + (float)gy) / (float)dim;
  dy = (dy - offset_h) * scale_h;
  const float dw = (e2 * aw) / 416.0f * scale_w;
  const float dh = (e3 * ah) / 416.0f * scale_h;
  const int idx = first + cell * 3 + a;
  float* b = boxes + (int64_t)idx * 4;
  b[0] = (dy - dh / 2.0f) * img_h;  // y min
  b[1] = (dx - dw / 2.0f) * img_w;  // x min
  b[2] = (dy + dh / 2.0f) * img_h;  // y max
  b[3] = (dx + dw / 2.0f) * img_w;  // x max
  const float conf = e4 / (e4 + 1.0f);
  for (int c = 0; c < classes; ++c) {
    const float e = expf(p[(int64_t)(5 + c) * cells]);
    scores[(int64_t)c * total + idx] = e / (e + 1.0f) * conf;
  }
}

__device__ __forceinline__ bool yolo_overlapping(const float4 s, const float4 c, const float iou_thr) {
  const float y_top = fmaxf(s.x, c.x), x_left = fmaxf(s.y, c.y);
  const float y_bot = fminf(s.z, c.z), x_right = fminf(s.w, c.w);
  if (x_right < x_left || y_bot < y_top) return false;
  const float common = (x_right - x_left) * (y_bot - y_top);
  const float s_area = (s.z - s.x) * (s.w - s.y);
  const float c_area = (c.z - c.x) * (c.w - c.y);
  return common / (s_area + c_area - common) > iou_thr;
}

// One workgroup per class.  The reference sorts the boxes that pass the score
// threshold by falling score and walks them once, keeping a box when it does not
// overlap the box kept last.  The box kept after `s` is therefore the best box
// that comes behind `s` in that order and does not overlap `s`: one parallel
// search per kept box, no sort.  Equal scores are ordered by rising box index.
__global__ void __launch_bounds__(256)
yolo_class_walk_kernel(const float* __restrict__ boxes, const float* __restrict__ scores, const int total,
                       const int capacity, const float iou_thr, const float score_thr,
                       float* __restrict__ info, int* __restrict__ num) {
  const int cls = blockIdx.x, tid = threadIdx.x;
  const float* sc = scores + (int64_t)cls * total;
  const float4* bx = reinterpret_cast<const float4*>(boxes);
  float* out = info + (int64_t)cls * capacity * 5;
  __shared__ float red_s[4];
  __shared__ int red_i[4];
  __shared__ float cur_s;
  __shared__ int cur_i;

  int kept = 0;
  int s_idx = -1;
  float s_score = 0.f;
  float4 s_box = make_float4(0.f, 0.f, 0.f, 0.f);
  while (kept < capacity) {
    float best = -FLT_MAX;
    int best_i = INT_MAX;
    for (int j = tid; j < total; j += 256) {
      const float v = sc[j];
      if (!(v >= score_thr)) continue;
      if (s_idx >= 0) {
        const bool behind = v < s_score || (v == s_score && j > s_idx);
        if (!behind) continue;
        if (yolo_overlapping(s_box, bx[j], iou_thr)) continue;
      }
      if (best_i == INT_MAX || v > best) { best = v; best_i = j; }  // j rises: the first of equal scores stays
    }
    // wavefront, then workgroup: highest score, lowest index among equals
    for (int off = 32; off > 0; off >>= 1) {
      const float ov = __shfl_down(best, off);
      const int oi = __shfl_down(best_i, off);
      if (oi != INT_MAX && (best_i == INT_MAX || ov > best || (ov == best && oi < best_i))) { best = ov; best_i = oi; }
    }
    if ((tid & 63) == 0) { red_s[tid >> 6] = best; red_i[tid >> 6] = best_i; }
    __syncthreads();
    if (tid == 0) {
      for (int w = 1; w < 4; ++w) {
        const float ov = red_s[w];
        const int oi = red_i[w];
        if (oi != INT_MAX && (best_i == INT_MAX || ov > best || (ov == best && oi < best_i))) { best = ov; best_i = oi; }
      }
      cur_s = best;
      cur_i = best_i;
    }
    __syncthreads();
    s_idx = cur_i;
    s_score = cur_s;
    __syncthreads();  // everyone has read the result before the next round overwrites it
    if (s_idx == INT_MAX) break;
    s_box = bx[s_idx];
    if (tid == 0) {
      float* o = out + (int64_t)kept * 5;
      o[0] = s_box.x; o[1] = s_box.y; o[2] = s_box.z; o[3] = s_box.w; o[4] = s_score;
    }
    ++kept;
  }
  // rows behind the last kept box read as zeros
  for (int j = kept * 5 + tid; j < capacity * 5; j += 256) out[j] = 0.f;
  if (tid == 0) num[cls] = kept;
}

}  // namespace

hipError_t launch_yolo_postprocess(const float* const heads[3], const int dims[3], int classes,
                                   const int anchors[3][6], const int* img_w, const int* img_h, float iou_thr,
                                   float score_thr, int capacity, float* boxes, float* scores, float* info,
                                   int* num, hipStream_t stream) {
  if (classes < 1 || capacity < 1) return hipErrorInvalidValue;
  int total = 0;
  for (int h = 0; h < 3; ++h) {
    if (dims[h] < 1 || heads[h] == nullptr) return hipErrorInvalidValue;
    total += 3 * dims[h] * dims[h];
  }
  if ((reinterpret_cast<uintptr_t>(boxes) & 15u) != 0) return hipErrorInvalidValue;
  int first = 0;
  for (int h = 0; h < 3; ++h) {
    const int n = 3 * dims[h] * dims[h];
    const int* an = anchors[h];
    hipLaunchKernelGGL(yolo_decode_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, heads[h], dims[h],
                       classes, first, total, an[0], an[1], an[2], an[3], an[4], an[5], img_w, img_h, boxes, scores);
    first += n;
  }
  hipLaunchKernelGGL(yolo_class_walk_kernel, dim3((unsigned)classes), dim3(256), 0, stream, boxes, scores, total,
                     capacity, iou_thr, score_thr, info, num);
  return hipGetLastError();
}

}  // namespace ohip
