// ODLA graph builders: each odla_<Op> call validates its operands, infers the
// result shape and appends one node to the calling thread's current
// computation.  Nothing touches the GPU here; kernels are chosen when the
// first context of the computation is created.
//
// Node attribute slots (Node::i / Node::f / Node::iv) per operator:
//   CONV       i0 layout, i1 group, i2 kernel layout, i3-4 stride, i5-6 dilation,
//              i7-8 pad front, i9-10 pad back; in = {x, kernel, bias?}
//   GEMM       i0 transA, i1 transB; f0 alpha, f1 beta; in = {A, B, C?}
//   BINARY     i0 BinKind;  UNARY  i0 ActKind, f0 f1 parameters
//   BATCHNORM  i0 layout; f0 eps, f1 scalar scale, f2 scalar offset;
//              in = {x, mean, var, scale?, offset?}
//   LAYERNORM  i0 number of trailing axes; f0 eps; in = {x, scale?, offset?}
//   POOL       i0 layout, i1 is_max, i2-3 window, i4-5 stride, i6-7 pad front,
//              i8-9 pad back, i10 padding_included
//   REDUCE     i0 ReduceKind, i1 keep_dims, iv axes
//   SOFTMAX    i0 axis, i1 log;  CONCAT i0 axis;  GATHER i0 axis
//   RESIZE     i0 interpolation, i1 coordinate mode
//   SLICE      iv = start[r] end[r] stride[r];  TRANSPOSE iv = permutation
//   QUANTIZE / DEQUANTIZE  i0 axis; in = {x, scale, zero_point?}
//   NMS        i0 max outputs; f0 iou threshold, f1 score threshold
#include <cmath>
#include <cstring>

#include "internal.h"

using namespace ohip;

namespace {

_odla_computation* comp_of(odla_value a, odla_value b = nullptr) {
  if (a != nullptr && a->comp != nullptr) return a->comp;
  if (b != nullptr && b->comp != nullptr) return b->comp;
  return current_computation();
}

Node* add_node(_odla_computation* c, OpKind op, std::vector<odla_value> in, odla_element_type et,
               const Shape& shape, const odla_value_id id) {
  odla_value out = new_value(c, _odla_value::TEMP, et, shape, id);
  c->nodes.emplace_back();
  Node& n = c->nodes.back();
  n.op = op;
  n.in = std::move(in);
  n.out = out;
  out->producer = (int)c->nodes.size() - 1;
  return &n;
}

bool is_float_type(odla_element_type t) {
  return t == ODLA_FLOAT32 || t == ODLA_FLOAT16 || t == ODLA_BFLOAT16;
}

#define REQUIRE(cond, ...)      \
  do {                          \
    if (!(cond)) {              \
      OHIP_ERR(__VA_ARGS__);    \
      return nullptr;           \
    }                           \
  } while (0)

// Right-aligned sliding alignment of a lower-rank operand, as the reference
// does it: the operand's dims are matched against a window of the larger
// shape, starting at the trailing position and moving left until every pair
// is equal or has a 1.  [ref: ODLA/platforms/dnnl/odla_dnnl.h:301-343]
bool expand_like_reference(Shape* src, const Shape& dst) {
  const int sn = src->rank, dn = dst.rank;
  for (int j = dn - 1; j >= sn - 1; --j) {
    bool ok = true;
    for (int k = 0; k < sn; ++k) {
      const int64_t a = dst.d[j - k], b = src->d[sn - 1 - k];
      if (a != b && a != 1 && b != 1) { ok = false; break; }
    }
    if (ok) {
      Shape r;
      r.rank = dn;
      for (int i = 0; i < dn; ++i) r.d[i] = 1;
      for (int k = 0; k < sn; ++k) r.d[j - k] = src->d[sn - 1 - k];
      *src = r;
      return true;
    }
  }
  return false;
}

odla_value binary(BinKind kind, odla_value lhs, odla_value rhs, const odla_value_id id) {
  REQUIRE(lhs && rhs, "binary op: null operand");
  _odla_computation* c = comp_of(lhs, rhs);
  REQUIRE(c, "binary op: no current computation");
  Shape a = lhs->shape, b = rhs->shape;
  if (a.rank != b.rank) {
    Shape& lo = a.rank < b.rank ? a : b;
    const Shape& hi = a.rank < b.rank ? b : a;
    REQUIRE(expand_like_reference(&lo, hi), "binary op: shapes %s and %s do not broadcast",
            lhs->shape.str().c_str(), rhs->shape.str().c_str());
  }
  Shape o;
  o.rank = a.rank;
  for (int i = 0; i < a.rank; ++i) {
    REQUIRE(a.d[i] == b.d[i] || a.d[i] == 1 || b.d[i] == 1, "binary op: shapes %s and %s do not broadcast",
            lhs->shape.str().c_str(), rhs->shape.str().c_str());
    o.d[i] = a.d[i] > b.d[i] ? a.d[i] : b.d[i];
  }
  Node* n = add_node(c, OP_BINARY, {lhs, rhs}, lhs->etype, o, id);
  n->i[0] = kind;
  // remember the aligned operand shapes for the planner
  n->iv.clear();
  n->iv.push_back(a.rank);
  for (int i = 0; i < a.rank; ++i) n->iv.push_back(a.d[i]);
  for (int i = 0; i < b.rank; ++i) n->iv.push_back(b.d[i]);
  return n->out;
}

odla_value unary(ActKind kind, odla_value x, float a, float b, const odla_value_id id) {
  REQUIRE(x, "unary op: null operand");
  _odla_computation* c = comp_of(x);
  REQUIRE(c, "unary op: no current computation");
  REQUIRE(is_float_type(x->etype), "unary op on non-float value '%s'", x->name.c_str());
  Node* n = add_node(c, OP_UNARY, {x}, x->etype, x->shape, id);
  n->i[0] = kind;
  n->f[0] = a;
  n->f[1] = b;
  return n->out;
}

// Spatial output extent of a strided window.
int64_t out_extent(int64_t in, int64_t k, int64_t s, int64_t pf, int64_t pb, int64_t dil = 1) {
  const int64_t eff = (k - 1) * dil + 1;
  return (in + pf + pb - eff) / s + 1;
}

odla_value pool(bool is_max, odla_value input, odla_memory_layout layout, const odla_uint32* window,
                const odla_uint32* strides, const odla_uint32* pf, const odla_uint32* pb,
                bool padding_included, const odla_value_shape& output_dims, const odla_value_id id) {
  REQUIRE(input && window && strides && pf && pb, "pool: null argument");
  _odla_computation* c = comp_of(input);
  REQUIRE(c, "pool: no current computation");
  REQUIRE(input->shape.rank == 4, "pool: only 2-D pooling of rank-4 tensors is supported (got %s)",
          input->shape.str().c_str());
  const bool cl = layout == ODLA_CHANNELS_LAST;
  const int hd = cl ? 1 : 2, wd = cl ? 2 : 3;
  Shape o = input->shape;
  o.d[hd] = out_extent(input->shape.d[hd], window[0], strides[0], pf[0], pb[0]);
  o.d[wd] = out_extent(input->shape.d[wd], window[1], strides[1], pf[1], pb[1]);
  // A caller-provided shape that only differs by the ceil-mode extra row/col is honoured.
  if (shape_valid(output_dims) && output_dims.size == 4) {
    const Shape u = shape_from(output_dims);
    if ((u.d[hd] == o.d[hd] || u.d[hd] == o.d[hd] + 1) && (u.d[wd] == o.d[wd] || u.d[wd] == o.d[wd] + 1)) {
      o.d[hd] = u.d[hd];
      o.d[wd] = u.d[wd];
    }
  }
  REQUIRE(o.d[hd] > 0 && o.d[wd] > 0, "pool: empty output");
  Node* n = add_node(c, OP_POOL, {input}, input->etype, o, id);
  n->i[0] = layout;
  n->i[1] = is_max;
  n->i[2] = window[0]; n->i[3] = window[1];
  n->i[4] = strides[0]; n->i[5] = strides[1];
  n->i[6] = pf[0]; n->i[7] = pf[1];
  n->i[8] = pb[0]; n->i[9] = pb[1];
  n->i[10] = padding_included;
  return n->out;
}

odla_value reduce(ReduceKind kind, odla_value input, odla_size_t num_axes, const odla_uint32* axes,
                  odla_bool keep_dims, const odla_value_id id) {
  REQUIRE(input && (axes || num_axes == 0), "reduce: null argument");
  _odla_computation* c = comp_of(input);
  REQUIRE(c, "reduce: no current computation");
  const int r = input->shape.rank;
  bool red[ODLA_MAX_DIMENSION] = {false};
  if (num_axes == 0)
    for (int i = 0; i < r; ++i) red[i] = true;
  for (odla_size_t i = 0; i < num_axes; ++i) {
    REQUIRE((int)axes[i] < r, "reduce: axis %u out of range for %s", axes[i], input->shape.str().c_str());
    red[axes[i]] = true;
  }
  Shape o;
  for (int i = 0; i < r; ++i) {
    if (red[i]) {
      if (keep_dims) o.d[o.rank++] = 1;
    } else {
      o.d[o.rank++] = input->shape.d[i];
    }
  }
  if (o.rank == 0) { o.rank = 1; o.d[0] = 1; }
  Node* n = add_node(c, OP_REDUCE, {input}, input->etype, o, id);
  n->i[0] = kind;
  n->i[1] = keep_dims;
  for (int i = 0; i < r; ++i)
    if (red[i]) n->iv.push_back(i);
  return n->out;
}

}  // namespace

extern "C" {

odla_value odla_Conv(odla_value input, odla_memory_layout input_layout, odla_uint32 group,
                     odla_value kernel, odla_memory_layout kernel_layout, const odla_uint32* strides,
                     const odla_uint32* dilations, const odla_uint32* paddings_front,
                     const odla_uint32* paddings_back, odla_value bias, odla_value_shape output_dims,
                     const odla_value_id id) {
  (void)output_dims;
  REQUIRE(input && kernel && strides && dilations && paddings_front && paddings_back, "odla_Conv: null argument");
  _odla_computation* c = comp_of(input, kernel);
  REQUIRE(c, "odla_Conv: no current computation");
  REQUIRE(input->shape.rank == 4 && kernel->shape.rank == 4, "odla_Conv: only 2-D convolution is supported");
  // Callers of the reference test-suite pass uninitialised layout enums; anything
  // that is not a known alternative means the ONNX default (NCHW / OIHW).
  const bool cl = input_layout == ODLA_CHANNELS_LAST;
  if (input_layout != ODLA_CHANNELS_LAST) input_layout = ODLA_CHANNELS_FIRST;
  if (kernel_layout != ODLA_SIO && kernel_layout != ODLA_SOI && kernel_layout != ODLA_IOS) kernel_layout = ODLA_OIS;
  if (group == 0) group = 1;
  const Shape& x = input->shape;
  const Shape& k = kernel->shape;
  int64_t O, I, R, S;
  switch (kernel_layout) {
    case ODLA_SIO: R = k.d[0]; S = k.d[1]; I = k.d[2]; O = k.d[3]; break;
    case ODLA_SOI: R = k.d[0]; S = k.d[1]; O = k.d[2]; I = k.d[3]; break;
    case ODLA_IOS: I = k.d[0]; O = k.d[1]; R = k.d[2]; S = k.d[3]; break;
    default: O = k.d[0]; I = k.d[1]; R = k.d[2]; S = k.d[3]; break;
  }
  const int64_t N = x.d[0], C = cl ? x.d[3] : x.d[1], H = cl ? x.d[1] : x.d[2], W = cl ? x.d[2] : x.d[3];
  REQUIRE(C == I * group, "odla_Conv: input channels %lld != kernel in-channels %lld x group %u",
          (long long)C, (long long)I, group);
  REQUIRE(O % group == 0, "odla_Conv: out channels %lld not divisible by group %u", (long long)O, group);
  REQUIRE(strides[0] > 0 && strides[1] > 0 && dilations[0] > 0 && dilations[1] > 0, "odla_Conv: bad stride/dilation");
  const int64_t Ho = out_extent(H, R, strides[0], paddings_front[0], paddings_back[0], dilations[0]);
  const int64_t Wo = out_extent(W, S, strides[1], paddings_front[1], paddings_back[1], dilations[1]);
  REQUIRE(Ho > 0 && Wo > 0, "odla_Conv: empty output");
  if (bias) REQUIRE(bias->shape.numel() == O, "odla_Conv: bias has %lld elements, expected %lld",
                    (long long)bias->shape.numel(), (long long)O);
  Shape o;
  o.rank = 4;
  o.d[0] = N;
  if (cl) { o.d[1] = Ho; o.d[2] = Wo; o.d[3] = O; } else { o.d[1] = O; o.d[2] = Ho; o.d[3] = Wo; }
  Node* n = add_node(c, OP_CONV, {input, kernel, bias}, input->etype, o, id);
  n->i[0] = input_layout;
  n->i[1] = group;
  n->i[2] = kernel_layout;
  n->i[3] = strides[0]; n->i[4] = strides[1];
  n->i[5] = dilations[0]; n->i[6] = dilations[1];
  n->i[7] = paddings_front[0]; n->i[8] = paddings_front[1];
  n->i[9] = paddings_back[0]; n->i[10] = paddings_back[1];
  return n->out;
}

odla_value odla_Gemm(odla_value A, odla_bool tA, odla_value B, odla_bool tB, odla_float32 alpha,
                     odla_float32 beta, odla_value C, odla_value_shape output_dims,
                     const odla_value_id id) {
  (void)output_dims;
  REQUIRE(A && B, "odla_Gemm: null operand");
  _odla_computation* c = comp_of(A, B);
  REQUIRE(c, "odla_Gemm: no current computation");
  const Shape& a = A->shape;
  const Shape& b = B->shape;
  REQUIRE(a.rank >= 2 && b.rank >= 2, "odla_Gemm: operands must have rank >= 2 (%s, %s)", a.str().c_str(), b.str().c_str());
  const int64_t M = tA ? a.d[a.rank - 1] : a.d[a.rank - 2];
  const int64_t K = tA ? a.d[a.rank - 2] : a.d[a.rank - 1];
  const int64_t Kb = tB ? b.d[b.rank - 1] : b.d[b.rank - 2];
  const int64_t N = tB ? b.d[b.rank - 2] : b.d[b.rank - 1];
  REQUIRE(K == Kb, "odla_Gemm: inner dims differ (%s%s x %s%s)", a.str().c_str(), tA ? "^T" : "", b.str().c_str(), tB ? "^T" : "");
  Shape o;
  if (b.rank == 2) {
    o = a;
    o.d[a.rank - 2] = M;
    o.d[a.rank - 1] = N;
  } else {
    REQUIRE(a.rank == b.rank, "odla_Gemm: batched operands must have equal rank (%s, %s)", a.str().c_str(), b.str().c_str());
    for (int i = 0; i < a.rank - 2; ++i)
      REQUIRE(a.d[i] == b.d[i], "odla_Gemm: batch dims differ (%s, %s)", a.str().c_str(), b.str().c_str());
    o = a;
    o.d[a.rank - 2] = M;
    o.d[a.rank - 1] = N;
  }
  Node* n = add_node(c, OP_GEMM, {A, B, C}, A->etype, o, id);
  n->i[0] = tA ? 1 : 0;
  n->i[1] = tB ? 1 : 0;
  n->f[0] = alpha;
  n->f[1] = C ? beta : 0.f;
  return n->out;
}

odla_value odla_BatchMatMul(odla_value A, odla_bool tA, odla_value B, odla_bool tB,
                            odla_value_shape output_dims, const odla_value_id id) {
  return odla_Gemm(A, tA, B, tB, 1.f, 0.f, nullptr, output_dims, id);
}

odla_value odla_Add(odla_value l, odla_value r, const odla_value_id id) { return binary(BIN_ADD, l, r, id); }
odla_value odla_Sub(odla_value l, odla_value r, const odla_value_id id) { return binary(BIN_SUB, l, r, id); }
odla_value odla_Mul(odla_value l, odla_value r, const odla_value_id id) { return binary(BIN_MUL, l, r, id); }
odla_value odla_Div(odla_value l, odla_value r, const odla_value_id id) { return binary(BIN_DIV, l, r, id); }
odla_value odla_Max(odla_value l, odla_value r, const odla_value_id id) { return binary(BIN_MAX, l, r, id); }
odla_value odla_Min(odla_value l, odla_value r, const odla_value_id id) { return binary(BIN_MIN, l, r, id); }

odla_value odla_Relu(odla_value x, const odla_value_id id) { return unary(ACT_RELU, x, 0, 0, id); }
odla_value odla_LeakyRelu(odla_value x, odla_float32 alpha, const odla_value_id id) { return unary(ACT_LEAKY, x, alpha, 0, id); }
odla_value odla_Sigmoid(odla_value x, const odla_value_id id) { return unary(ACT_SIGMOID, x, 0, 0, id); }
odla_value odla_Tanh(odla_value x, const odla_value_id id) { return unary(ACT_TANH, x, 0, 0, id); }
odla_value odla_Exp(odla_value x, const odla_value_id id) { return unary(ACT_EXP, x, 0, 0, id); }
odla_value odla_Log(odla_value x, const odla_value_id id) { return unary(ACT_LOG, x, 0, 0, id); }
odla_value odla_Sqrt(odla_value x, const odla_value_id id) { return unary(ACT_SQRT, x, 0, 0, id); }
odla_value odla_Rsqrt(odla_value x, const odla_value_id id) { return unary(ACT_RSQRT, x, 0, 0, id); }
odla_value odla_Erf(odla_value x, const odla_value_id id) { return unary(ACT_ERF, x, 0, 0, id); }
odla_value odla_Abs(odla_value x, const odla_value_id id) { return unary(ACT_ABS, x, 0, 0, id); }
odla_value odla_Neg(odla_value x, const odla_value_id id) { return unary(ACT_NEG, x, 0, 0, id); }
odla_value odla_Round(odla_value x, const odla_value_id id) { return unary(ACT_ROUND, x, 0, 0, id); }
odla_value odla_Clamp(odla_value x, odla_float32 lo, odla_float32 hi, const odla_value_id id) { return unary(ACT_CLAMP, x, lo, hi, id); }
odla_value odla_Gelu(odla_value x, odla_bool use_approx, const odla_value_id id) {
  return unary(use_approx ? ACT_GELU_TANH : ACT_GELU_ERF, x, 0, 0, id);
}

odla_value odla_BatchNormalization(odla_value input, odla_memory_layout layout, odla_value mean,
                                   odla_value var, odla_float32 epsilon, odla_value scale,
                                   odla_value offset, odla_float32 scalar_scale,
                                   odla_float32 scalar_offset, const odla_value_id id) {
  REQUIRE(input && mean && var, "odla_BatchNormalization: null operand");
  _odla_computation* c = comp_of(input);
  REQUIRE(c, "odla_BatchNormalization: no current computation");
  REQUIRE(input->shape.rank >= 2, "odla_BatchNormalization: rank < 2");
  if (layout != ODLA_CHANNELS_LAST) layout = ODLA_CHANNELS_FIRST;
  const int64_t C = layout == ODLA_CHANNELS_LAST ? input->shape.d[input->shape.rank - 1] : input->shape.d[1];
  REQUIRE(mean->shape.numel() == C && var->shape.numel() == C, "odla_BatchNormalization: statistics must have %lld elements", (long long)C);
  if (scale) REQUIRE(scale->shape.numel() == C, "odla_BatchNormalization: scale size");
  if (offset) REQUIRE(offset->shape.numel() == C, "odla_BatchNormalization: offset size");
  Node* n = add_node(c, OP_BATCHNORM, {input, mean, var, scale, offset}, input->etype, input->shape, id);
  n->i[0] = layout;
  n->f[0] = epsilon;
  n->f[1] = scalar_scale;
  n->f[2] = scalar_offset;
  return n->out;
}

odla_value odla_LayerNorm(odla_value input, odla_size_t axes_size, const odla_int32* axes,
                          odla_float32 epsilon, odla_value scale, odla_value offset,
                          const odla_value_id id) {
  REQUIRE(input, "odla_LayerNorm: null operand");
  _odla_computation* c = comp_of(input);
  REQUIRE(c, "odla_LayerNorm: no current computation");
  const int r = input->shape.rank;
  // the normalised axes must be the trailing ones
  int n_axes = 1;
  if (axes_size > 0 && axes != nullptr) {
    bool used[ODLA_MAX_DIMENSION] = {false};
    for (odla_size_t i = 0; i < axes_size; ++i) {
      int a = axes[i] < 0 ? axes[i] + r : axes[i];
      REQUIRE(a >= 0 && a < r, "odla_LayerNorm: axis out of range");
      used[a] = true;
    }
    n_axes = 0;
    for (int i = r - 1; i >= 0 && used[i]; --i) ++n_axes;
    REQUIRE(n_axes == (int)axes_size, "odla_LayerNorm: axes must be the trailing dimensions");
  }
  int64_t len = 1;
  for (int i = r - n_axes; i < r; ++i) len *= input->shape.d[i];
  if (scale) REQUIRE(scale->shape.numel() == len, "odla_LayerNorm: scale must have %lld elements", (long long)len);
  if (offset) REQUIRE(offset->shape.numel() == len, "odla_LayerNorm: offset must have %lld elements", (long long)len);
  Node* n = add_node(c, OP_LAYERNORM, {input, scale, offset}, input->etype, input->shape, id);
  n->i[0] = n_axes;
  n->f[0] = epsilon;
  return n->out;
}

odla_value odla_MaxPool(odla_value input, odla_memory_layout layout, const odla_uint32* window,
                        const odla_uint32* strides, const odla_uint32* pf, const odla_uint32* pb,
                        odla_value_shape output_dims, const odla_value_id id) {
  return pool(true, input, layout, window, strides, pf, pb, false, output_dims, id);
}
odla_value odla_AveragePool(odla_value input, odla_memory_layout layout, const odla_uint32* window,
                            const odla_uint32* strides, const odla_uint32* pf, const odla_uint32* pb,
                            odla_bool padding_included, odla_value_shape output_dims,
                            const odla_value_id id) {
  return pool(false, input, layout, window, strides, pf, pb, padding_included != 0, output_dims, id);
}

odla_value odla_ReduceMean(odla_value input, odla_size_t n, const odla_uint32* axes, odla_bool keep,
                           odla_value_shape, const odla_value_id id) {
  return reduce(RED_MEAN, input, n, axes, keep, id);
}
odla_value odla_ReduceSum(odla_value input, odla_size_t n, const odla_uint32* axes, odla_bool keep,
                          odla_value_shape, const odla_value_id id) {
  return reduce(RED_SUM, input, n, axes, keep, id);
}
odla_value odla_ReduceMax(odla_value input, odla_size_t n, const odla_uint32* axes, odla_bool keep,
                          odla_value_shape, const odla_value_id id) {
  return reduce(RED_MAX, input, n, axes, keep, id);
}

static odla_value softmax_impl(odla_value input, odla_int32 axis, bool logsm, const odla_value_id id) {
  REQUIRE(input, "softmax: null operand");
  _odla_computation* c = comp_of(input);
  REQUIRE(c, "softmax: no current computation");
  const int r = input->shape.rank;
  // the reference maps every negative axis to the last one [ref: odla_dnnl.cc:1632]
  if (axis < 0) axis = r - 1;
  REQUIRE(axis < r, "softmax: axis %d out of range for %s", axis, input->shape.str().c_str());
  Node* n = add_node(c, OP_SOFTMAX, {input}, input->etype, input->shape, id);
  n->i[0] = axis;
  n->i[1] = logsm;
  return n->out;
}
odla_value odla_Softmax(odla_value input, odla_int32 axis, const odla_value_id id) { return softmax_impl(input, axis, false, id); }
odla_value odla_LogSoftmax(odla_value input, odla_int32 axis, const odla_value_id id) { return softmax_impl(input, axis, true, id); }

odla_value odla_Cast(odla_value input, odla_element_type target, const odla_value_id id) {
  REQUIRE(input, "odla_Cast: null operand");
  _odla_computation* c = comp_of(input);
  REQUIRE(c, "odla_Cast: no current computation");
  REQUIRE(dtype_from_odla(target) != DT_INVALID, "odla_Cast: unsupported target type %d", (int)target);
  Node* n = add_node(c, OP_CAST, {input}, target, input->shape, id);
  return n->out;
}

odla_value odla_Concat(odla_values inputs, odla_int32 axis, odla_value_shape, const odla_value_id id) {
  REQUIRE(inputs.size >= 1 && inputs.size <= ODLA_MAX_OUTPUTS, "odla_Concat: bad input count");
  odla_value first = inputs.values[0];
  REQUIRE(first, "odla_Concat: null input");
  _odla_computation* c = comp_of(first);
  REQUIRE(c, "odla_Concat: no current computation");
  const int r = first->shape.rank;
  if (axis < 0) axis += r;
  REQUIRE(axis >= 0 && axis < r, "odla_Concat: axis out of range");
  Shape o = first->shape;
  std::vector<odla_value> in;
  in.push_back(first);
  for (size_t k = 1; k < inputs.size; ++k) {
    odla_value v = inputs.values[k];
    REQUIRE(v && v->shape.rank == r && v->etype == first->etype, "odla_Concat: mismatching input %zu", k);
    for (int i = 0; i < r; ++i)
      if (i != axis) REQUIRE(v->shape.d[i] == o.d[i], "odla_Concat: input %zu shape %s mismatches", k, v->shape.str().c_str());
    o.d[axis] += v->shape.d[axis];
    in.push_back(v);
  }
  Node* n = add_node(c, OP_CONCAT, in, first->etype, o, id);
  n->i[0] = axis;
  return n->out;
}

odla_value odla_Gather(odla_value input, odla_value indices, odla_int32 axis, odla_value_shape,
                       const odla_value_id id) {
  REQUIRE(input && indices, "odla_Gather: null operand");
  _odla_computation* c = comp_of(input, indices);
  REQUIRE(c, "odla_Gather: no current computation");
  REQUIRE(indices->etype == ODLA_INT32 || indices->etype == ODLA_INT64, "odla_Gather: indices must be int32/int64");
  const int r = input->shape.rank;
  if (axis < 0) axis += r;
  REQUIRE(axis >= 0 && axis < r, "odla_Gather: axis out of range");
  Shape o;
  for (int i = 0; i < axis; ++i) o.d[o.rank++] = input->shape.d[i];
  for (int i = 0; i < indices->shape.rank; ++i) o.d[o.rank++] = indices->shape.d[i];
  for (int i = axis + 1; i < r; ++i) o.d[o.rank++] = input->shape.d[i];
  REQUIRE(o.rank <= ODLA_MAX_DIMENSION, "odla_Gather: result rank too large");
  Node* n = add_node(c, OP_GATHER, {input, indices}, input->etype, o, id);
  n->i[0] = axis;
  return n->out;
}

odla_value odla_Reshape(odla_value input, odla_value_shape output_dims, const odla_value_id id) {
  REQUIRE(input, "odla_Reshape: null operand");
  _odla_computation* c = comp_of(input);
  REQUIRE(c, "odla_Reshape: no current computation");
  REQUIRE(output_dims.size >= 0 && output_dims.size <= ODLA_MAX_DIMENSION, "odla_Reshape: bad output rank");
  Shape o = shape_from(output_dims);
  // one dimension may be -1 (inferred)
  int64_t known = 1;
  int unk = -1;
  for (int i = 0; i < o.rank; ++i) {
    if (o.d[i] == -1) { REQUIRE(unk < 0, "odla_Reshape: more than one -1"); unk = i; }
    else known *= o.d[i];
  }
  if (unk >= 0) {
    REQUIRE(known > 0 && input->shape.numel() % known == 0, "odla_Reshape: cannot infer dimension");
    o.d[unk] = input->shape.numel() / known;
  }
  REQUIRE(o.numel() == input->shape.numel(), "odla_Reshape: %s -> %s changes the element count",
          input->shape.str().c_str(), o.str().c_str());
  Node* n = add_node(c, OP_RESHAPE, {input}, input->etype, o, id);
  return n->out;
}

odla_value odla_Resize(odla_value input, odla_interpolation_mode interpolation,
                       odla_resize_coordinate_mode mode, odla_uint32 axes_mask,
                       odla_value_shape output_dims, const odla_value_id id) {
  (void)axes_mask;
  REQUIRE(input, "odla_Resize: null operand");
  _odla_computation* c = comp_of(input);
  REQUIRE(c, "odla_Resize: no current computation");
  REQUIRE(input->shape.rank == 4 && output_dims.size == 4, "odla_Resize: rank-4 tensors only");
  REQUIRE(interpolation == ODLA_NEAREST, "odla_Resize: only nearest interpolation is supported");
  Shape o = shape_from(output_dims);
  REQUIRE(o.d[0] == input->shape.d[0] && o.d[1] == input->shape.d[1] && o.d[2] > 0 && o.d[3] > 0,
          "odla_Resize: output %s must keep batch and channels of %s", o.str().c_str(), input->shape.str().c_str());
  Node* n = add_node(c, OP_RESIZE, {input}, input->etype, o, id);
  n->i[0] = interpolation;
  n->i[1] = mode;
  return n->out;
}

odla_value odla_Slice(odla_value input, const odla_int32* start, const odla_int32* end,
                      const odla_int32* stride, odla_value_shape, const odla_value_id id) {
  REQUIRE(input && start && end && stride, "odla_Slice: null argument");
  _odla_computation* c = comp_of(input);
  REQUIRE(c, "odla_Slice: no current computation");
  const int r = input->shape.rank;
  Shape o;
  o.rank = r;
  std::vector<int64_t> iv(3 * r);
  for (int i = 0; i < r; ++i) {
    REQUIRE(stride[i] > 0, "odla_Slice: only positive strides are supported");
    int64_t s = start[i], e = end[i];
    const int64_t d = input->shape.d[i];
    if (s < 0) s += d;
    if (e < 0) e += d;
    s = s < 0 ? 0 : (s > d ? d : s);
    e = e < 0 ? 0 : (e > d ? d : e);
    o.d[i] = (e - s + stride[i] - 1) / stride[i];
    REQUIRE(o.d[i] > 0, "odla_Slice: empty result along dim %d", i);
    iv[i] = s; iv[r + i] = e; iv[2 * r + i] = stride[i];
  }
  Node* n = add_node(c, OP_SLICE, {input}, input->etype, o, id);
  n->iv = iv;
  return n->out;
}

odla_value odla_Transpose(odla_value input, odla_value_shape permutations, odla_value_shape,
                          const odla_value_id id) {
  REQUIRE(input, "odla_Transpose: null operand");
  _odla_computation* c = comp_of(input);
  REQUIRE(c, "odla_Transpose: no current computation");
  const int r = input->shape.rank;
  REQUIRE(permutations.size == r, "odla_Transpose: permutation rank %d != input rank %d", permutations.size, r);
  Shape o;
  o.rank = r;
  bool seen[ODLA_MAX_DIMENSION] = {false};
  std::vector<int64_t> perm(r);
  for (int i = 0; i < r; ++i) {
    const int64_t p = permutations.dims[i];
    REQUIRE(p >= 0 && p < r && !seen[p], "odla_Transpose: invalid permutation");
    seen[p] = true;
    perm[i] = p;
    o.d[i] = input->shape.d[p];
  }
  Node* n = add_node(c, OP_TRANSPOSE, {input}, input->etype, o, id);
  n->iv = perm;
  return n->out;
}

static odla_value qdq(OpKind op, odla_value input, odla_value scale, odla_value zp, odla_int32 axis,
                      odla_element_type target, const odla_value_id id) {
  REQUIRE(input && scale, "quantize/dequantize: null operand");
  _odla_computation* c = comp_of(input);
  REQUIRE(c, "quantize/dequantize: no current computation");
  REQUIRE(scale->kind == _odla_value::CONSTANT && (!zp || zp->kind == _odla_value::CONSTANT),
          "quantize/dequantize: scale and zero point must be constants");
  const int r = input->shape.rank;
  const int64_t ns = scale->shape.numel();
  if (axis < 0) axis += r;
  if (ns > 1) REQUIRE(axis >= 0 && axis < r && input->shape.d[axis] == ns, "quantize/dequantize: per-axis scale size mismatch");
  if (zp) REQUIRE(zp->shape.numel() == ns, "quantize/dequantize: zero point / scale size mismatch");
  if (op == OP_QUANTIZE) {
    REQUIRE(target == ODLA_INT8 || target == ODLA_UINT8 || target == ODLA_QINT8 || target == ODLA_QUINT8,
            "odla_Quantize: target must be an 8-bit integer type");
    REQUIRE(is_float_type(input->etype), "odla_Quantize: input must be floating point");
  } else {
    REQUIRE(target == ODLA_FLOAT32, "odla_Dequantize: target must be FLOAT32");
  }
  Node* n = add_node(c, op, {input, scale, zp}, target, input->shape, id);
  n->i[0] = axis;
  return n->out;
}
odla_value odla_Quantize(odla_value input, odla_value scale, odla_value zp, odla_int32 axis,
                         odla_element_type target, const odla_value_id id) {
  return qdq(OP_QUANTIZE, input, scale, zp, axis, target, id);
}
odla_value odla_Dequantize(odla_value input, odla_value scale, odla_value zp, odla_int32 axis,
                           odla_element_type target, const odla_value_id id) {
  return qdq(OP_DEQUANTIZE, input, scale, zp, axis, target, id);
}

odla_value odla_NMS(odla_value boxes, odla_value scores, odla_uint32 max_num_outputs,
                    odla_float32 iou_threshold, odla_float32 score_threshold,
                    odla_value_type output_value_type, const odla_value_id id) {
  REQUIRE(boxes && scores, "odla_NMS: null operand");
  _odla_computation* c = comp_of(boxes, scores);
  REQUIRE(c, "odla_NMS: no current computation");
  REQUIRE(boxes->shape.rank == 3 && boxes->shape.d[2] == 4, "odla_NMS: boxes must be [N,B,4], got %s", boxes->shape.str().c_str());
  REQUIRE(scores->shape.rank == 3 && scores->shape.d[0] == boxes->shape.d[0] && scores->shape.d[2] == boxes->shape.d[1],
          "odla_NMS: scores must be [N,C,B], got %s", scores->shape.str().c_str());
  odla_element_type et = output_value_type.element_type == ODLA_INT64 ? ODLA_INT64 : ODLA_INT32;
  Shape o;
  o.rank = 2;
  o.d[0] = boxes->shape.d[0] * (int64_t)max_num_outputs;
  o.d[1] = 3;
  REQUIRE(o.d[0] > 0, "odla_NMS: max_num_outputs must be positive");
  Node* n = add_node(c, OP_NMS, {boxes, scores}, et, o, id);
  n->i[0] = max_num_outputs;
  n->f[0] = iou_threshold;
  n->f[1] = score_threshold;
  return n->out;
}

}  // extern "C"
