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
//   EWISE      i0 EwiseOp; iv = rank, then one aligned shape per operand
//   ARGEXT     i0 is_max, i1 axis, i2 last index on ties
//   COPYND     i0 fill first; iv = rank R, dims[R], src strides[R], dst strides[R], src offset,
//              dst offset (elements; row-major source and result)
//   TOPK       i0 K, i1 largest, i2 axis; out = values, out2 = indices
//   LRN        i0 layout, i1 window; f0 alpha, f1 beta, f2 bias
//   ROWNORM    i0 layout; f0 eps, f1 scalar scale, f2 scalar offset; in = {x, scale?, offset?}
#include <climits>
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

// Appends a node and its result value.  Returns nullptr (and logs) when the
// computation no longer takes operators - it has been compiled and a caller's
// context runs its plan - or when an operand belongs to another computation.
// One thread records into a computation at a time; the lock only orders the
// append against a compilation running on another thread.
Node* add_node(_odla_computation* c, OpKind op, std::vector<odla_value> in, odla_element_type et,
               const Shape& shape, const odla_value_id id) {
  for (const odla_value v : in) {
    if (v != nullptr && v->comp != c) {
      OHIP_ERR("odla_%s: operand '%s' belongs to another computation", op_name(op), v->name.c_str());
      return nullptr;
    }
  }
  std::lock_guard<std::mutex> lk(c->mu);
  if (c->plan && c->live_contexts > 0) {
    OHIP_ERR("odla_%s: the computation is compiled and has contexts; operators recorded now would not run", op_name(op));
    return nullptr;
  }
  odla_value out = new_value(c, _odla_value::TEMP, et, shape, id);
  c->nodes.emplace_back();
  Node& n = c->nodes.back();
  n.op = op;
  n.in = std::move(in);
  n.out = out;
  out->producer = (int)c->nodes.size() - 1;
  return &n;
}

#define ADD_NODE_FAILED {}

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

odla_value ewise_same_type(EwiseOp op, odla_value l, odla_value r, const char* what, const odla_value_id id);

odla_value binary(BinKind kind, odla_value lhs, odla_value rhs, const odla_value_id id) {
  REQUIRE(lhs && rhs, "binary op: null operand");
  if (!is_float_type(lhs->etype) || !is_float_type(rhs->etype)) {
    // integer arithmetic [ref: ODLA/platforms/dnnl/odla_dnnl.cc:567-610]
    static const EwiseOp map[] = {EW_ADD, EW_SUB, EW_MUL, EW_DIV, EW_MAX, EW_MIN};
    return ewise_same_type(map[kind], lhs, rhs, "binary op", id);
  }
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
  if (n == nullptr) return ADD_NODE_FAILED;
  n->i[0] = kind;
  // remember the aligned operand shapes for the planner
  n->iv.clear();
  n->iv.push_back(a.rank);
  for (int i = 0; i < a.rank; ++i) n->iv.push_back(a.d[i]);
  for (int i = 0; i < b.rank; ++i) n->iv.push_back(b.d[i]);
  return n->out;
}

// Typed element-wise node over up to three operands, broadcast like binary():
// lower-rank operands are aligned against the operand of highest rank.
odla_value ewise(EwiseOp op, std::vector<odla_value> in, odla_element_type out_type, const char* what,
                 const odla_value_id id, const Shape* target = nullptr) {
  for (odla_value v : in) REQUIRE(v, "%s: null operand", what);
  _odla_computation* c = comp_of(in[0], in.size() > 1 ? in[1] : nullptr);
  REQUIRE(c, "%s: no current computation", what);
  Shape hi = target ? *target : in[0]->shape;
  if (!target)
    for (odla_value v : in)
      if (v->shape.rank > hi.rank) hi = v->shape;
  std::vector<Shape> al;
  for (odla_value v : in) {
    Shape s = v->shape;
    if (s.rank != hi.rank)
      REQUIRE(s.rank < hi.rank && expand_like_reference(&s, hi), "%s: shapes %s and %s do not broadcast", what,
              v->shape.str().c_str(), hi.str().c_str());
    al.push_back(s);
  }
  Shape o;
  o.rank = hi.rank;
  for (int i = 0; i < o.rank; ++i) {
    o.d[i] = 1;
    for (const Shape& s : al)
      if (s.d[i] > o.d[i]) o.d[i] = s.d[i];
    for (const Shape& s : al)
      REQUIRE(s.d[i] == o.d[i] || s.d[i] == 1, "%s: operand shapes do not broadcast in dim %d", what, i);
  }
  if (target) REQUIRE(o == *target, "%s: operands do not broadcast to %s", what, target->str().c_str());
  Node* n = add_node(c, OP_EWISE, in, out_type, o, id);
  if (n == nullptr) return ADD_NODE_FAILED;
  n->i[0] = op;
  n->iv.push_back(o.rank);
  for (const Shape& s : al)
    for (int i = 0; i < o.rank; ++i) n->iv.push_back(s.d[i]);
  return n->out;
}

odla_value ewise_same_type(EwiseOp op, odla_value l, odla_value r, const char* what, const odla_value_id id) {
  REQUIRE(l && r, "%s: null operand", what);
  REQUIRE(l->etype == r->etype, "%s: operands '%s' and '%s' differ in element type", what, l->name.c_str(),
          r->name.c_str());
  REQUIRE(l->etype != ODLA_BOOL, "%s: arithmetic on boolean values", what);
  return ewise(op, {l, r}, l->etype, what, id);
}
odla_value ewise_compare(EwiseOp op, odla_value l, odla_value r, const char* what, const odla_value_id id) {
  REQUIRE(l && r, "%s: null operand", what);
  REQUIRE(l->etype == r->etype, "%s: operands '%s' and '%s' differ in element type", what, l->name.c_str(),
          r->name.c_str());
  return ewise(op, {l, r}, ODLA_BOOL, what, id);
}
odla_value ewise_logic(EwiseOp op, odla_value l, odla_value r, const char* what, const odla_value_id id) {
  REQUIRE(l && r, "%s: null operand", what);
  REQUIRE(l->etype == ODLA_BOOL && r->etype == ODLA_BOOL, "%s: operands must be boolean", what);
  return ewise(op, {l, r}, ODLA_BOOL, what, id);
}

odla_value unary(ActKind kind, odla_value x, float a, float b, const odla_value_id id) {
  REQUIRE(x, "unary op: null operand");
  _odla_computation* c = comp_of(x);
  REQUIRE(c, "unary op: no current computation");
  REQUIRE(is_float_type(x->etype), "unary op on non-float value '%s'", x->name.c_str());
  Node* n = add_node(c, OP_UNARY, {x}, x->etype, x->shape, id);
  if (n == nullptr) return ADD_NODE_FAILED;
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
  if (n == nullptr) return ADD_NODE_FAILED;
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
                  odla_bool keep_dims, const odla_value_id id, float eps = 0.f) {
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
  if (n == nullptr) return ADD_NODE_FAILED;
  n->i[0] = kind;
  n->i[1] = keep_dims;
  n->f[0] = eps;
  for (int i = 0; i < r; ++i)
    if (red[i]) n->iv.push_back(i);
  return n->out;
}

// Strided gather / scatter copy node over a row-major source and result.
odla_value copynd(_odla_computation* c, odla_value x, const Shape& out, const std::vector<int64_t>& dims,
                  const std::vector<int64_t>& sx, const std::vector<int64_t>& sy, int64_t x_off, int64_t y_off,
                  bool fill, const odla_value_id id) {
  Node* n = add_node(c, OP_COPYND, {x}, x->etype, out, id);
  if (n == nullptr) return ADD_NODE_FAILED;
  n->i[0] = fill;
  n->iv.push_back((int64_t)dims.size());
  n->iv.insert(n->iv.end(), dims.begin(), dims.end());
  n->iv.insert(n->iv.end(), sx.begin(), sx.end());
  n->iv.insert(n->iv.end(), sy.begin(), sy.end());
  n->iv.push_back(x_off);
  n->iv.push_back(y_off);
  return n->out;
}
odla_value_shape undefined_shape() {
  odla_value_shape s;
  memset(&s, 0, sizeof(s));
  return s;
}
std::vector<int64_t> row_major_strides(const Shape& s) {
  std::vector<int64_t> st(s.rank);
  int64_t acc = 1;
  for (int i = s.rank - 1; i >= 0; --i) { st[i] = acc; acc *= s.d[i]; }
  return st;
}

// [ref: ODLA/platforms/dnnl/odla_dnnl_statistics.cc:203-300]
odla_value arg_extreme(bool is_max, odla_value input, odla_int32 axis, odla_bool keep_dims,
                       odla_bool return_last_index, const odla_value_type& out_type, const odla_value_id id) {
  REQUIRE(input, "ArgMax/ArgMin: null operand");
  _odla_computation* c = comp_of(input);
  REQUIRE(c, "ArgMax/ArgMin: no current computation");
  REQUIRE(is_float_type(input->etype), "ArgMax/ArgMin: operand must be a float type");
  const int r = input->shape.rank;
  if (axis < 0) axis += r;
  REQUIRE(axis >= 0 && axis < r, "ArgMax/ArgMin: axis out of range for %s", input->shape.str().c_str());
  const odla_element_type et = out_type.element_type == ODLA_INT64 ? ODLA_INT64 : ODLA_INT32;
  REQUIRE(out_type.element_type == ODLA_INT64 || out_type.element_type == ODLA_INT32,
          "ArgMax/ArgMin: the index type must be INT32 or INT64");
  Shape o;
  for (int i = 0; i < r; ++i) {
    if (i == axis) {
      if (keep_dims) o.d[o.rank++] = 1;
    } else {
      o.d[o.rank++] = input->shape.d[i];
    }
  }
  if (o.rank == 0) { o.rank = 1; o.d[0] = 1; }
  Node* n = add_node(c, OP_ARGEXT, {input}, et, o, id);
  if (n == nullptr) return ADD_NODE_FAILED;
  n->i[0] = is_max;
  n->i[1] = axis;
  n->i[2] = return_last_index != 0;
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
  if (n == nullptr) return ADD_NODE_FAILED;
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
  // The GEMM launch itself adds a constant row / scalar (any beta) or a
  // run-time matrix of the result's shape (beta 1).  Every other C operand - a
  // constant matrix, a column, a run-time row, another beta - becomes
  // Gemm -> Add(beta * C), with the reference's broadcasting rules for the Add.
  bool fused_c = true;
  if (C != nullptr && beta != 0.f) {
    const int64_t cn = C->shape.numel();
    const bool row_const = C->kind == _odla_value::CONSTANT && is_float_type(C->etype) &&
                           (cn == 1 || (cn == N && C->shape.d[C->shape.rank - 1] == N));
    const bool full_runtime = C->kind != _odla_value::CONSTANT && C->shape == o && beta == 1.f;
    fused_c = row_const || full_runtime;
  }
  if (!fused_c) {
    REQUIRE(is_float_type(C->etype), "odla_Gemm: C operand must be a float type");
    odla_value g = odla_Gemm(A, tA, B, tB, alpha, 0.f, nullptr, output_dims, nullptr);
    if (g == nullptr) return nullptr;
    odla_value cs = C;
    if (beta != 1.f) {
      auto buf = std::make_unique<std::vector<uint8_t>>(sizeof(float));
      memcpy(buf->data(), &beta, sizeof(float));
      Shape one;
      one.rank = 1;
      one.d[0] = 1;
      odla_value k = new_value(c, _odla_value::CONSTANT, ODLA_FLOAT32, one, nullptr);
      k->host_data = buf->data();
      c->owned_data.push_back(std::move(buf));
      cs = binary(BIN_MUL, C, k, nullptr);
      if (cs == nullptr) return nullptr;
    }
    return binary(BIN_ADD, g, cs, id);
  }
  Node* n = add_node(c, OP_GEMM, {A, B, C}, A->etype, o, id);
  if (n == nullptr) return ADD_NODE_FAILED;
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

odla_value odla_Pow(odla_value l, odla_value r, const odla_value_id id) { return ewise_same_type(EW_POW, l, r, "odla_Pow", id); }
odla_value odla_Mod(odla_value l, odla_value r, odla_int64 fmod, const odla_value_id id) {
  return ewise_same_type(fmod == 1 ? EW_FMOD : EW_MOD, l, r, "odla_Mod", id);
}
odla_value odla_SquaredDifference(odla_value l, odla_value r, const odla_value_id id) {
  return ewise_same_type(EW_SQDIFF, l, r, "odla_SquaredDifference", id);
}
odla_value odla_PRelu(odla_value x, odla_value slope, const odla_value_id id) {
  return ewise_same_type(EW_PRELU, x, slope, "odla_PRelu", id);
}
odla_value odla_Equal(odla_value l, odla_value r, const odla_value_id id) { return ewise_compare(EW_EQ, l, r, "odla_Equal", id); }
odla_value odla_NotEqual(odla_value l, odla_value r, const odla_value_id id) { return ewise_compare(EW_NE, l, r, "odla_NotEqual", id); }
odla_value odla_Less(odla_value l, odla_value r, const odla_value_id id) { return ewise_compare(EW_LT, l, r, "odla_Less", id); }
odla_value odla_LessOrEqual(odla_value l, odla_value r, const odla_value_id id) { return ewise_compare(EW_LE, l, r, "odla_LessOrEqual", id); }
odla_value odla_Greater(odla_value l, odla_value r, const odla_value_id id) { return ewise_compare(EW_GT, l, r, "odla_Greater", id); }
odla_value odla_GreaterOrEqual(odla_value l, odla_value r, const odla_value_id id) { return ewise_compare(EW_GE, l, r, "odla_GreaterOrEqual", id); }
odla_value odla_And(odla_value l, odla_value r, const odla_value_id id) { return ewise_logic(EW_AND, l, r, "odla_And", id); }
odla_value odla_Or(odla_value l, odla_value r, const odla_value_id id) { return ewise_logic(EW_OR, l, r, "odla_Or", id); }
odla_value odla_Xor(odla_value l, odla_value r, const odla_value_id id) { return ewise_logic(EW_XOR, l, r, "odla_Xor", id); }
odla_value odla_Not(odla_value x, const odla_value_id id) {
  REQUIRE(x, "odla_Not: null operand");
  REQUIRE(x->etype == ODLA_BOOL, "odla_Not: operand must be boolean");
  return ewise(EW_NOT, {x}, ODLA_BOOL, "odla_Not", id);
}
odla_value odla_IsNaN(odla_value x, const odla_value_id id) {
  REQUIRE(x, "odla_IsNaN: null operand");
  REQUIRE(is_float_type(x->etype), "odla_IsNaN: operand must be a float type");
  return ewise(EW_ISNAN, {x}, ODLA_BOOL, "odla_IsNaN", id);
}
odla_value odla_IsInf(odla_value x, odla_bool detect_pos, odla_bool detect_neg, const odla_value_id id) {
  REQUIRE(x, "odla_IsInf: null operand");
  REQUIRE(is_float_type(x->etype), "odla_IsInf: operand must be a float type");
  // neither flag set selects the negative test, as in the reference [ref: odla_dnnl_unary.cc:229-238]
  const EwiseOp op = (detect_pos && detect_neg) ? EW_ISINF : (detect_pos ? EW_ISINF_POS : EW_ISINF_NEG);
  return ewise(op, {x}, ODLA_BOOL, "odla_IsInf", id);
}
odla_value odla_Select(odla_value cond, odla_value a, odla_value b, odla_value_shape output_dims,
                       const odla_value_id id) {
  REQUIRE(cond && a && b, "odla_Select: null operand");
  REQUIRE(cond->etype == ODLA_BOOL, "odla_Select: the condition must be boolean");
  REQUIRE(a->etype == b->etype, "odla_Select: branches differ in element type");
  if (shape_valid(output_dims)) {
    const Shape t = shape_from(output_dims);
    return ewise(EW_SELECT, {cond, a, b}, a->etype, "odla_Select", id, &t);
  }
  return ewise(EW_SELECT, {cond, a, b}, a->etype, "odla_Select", id);
}
// Element-wise mean of n same-shaped (or broadcastable) values.
// [ref: ODLA/platforms/dnnl/odla_dnnl.cc:2432-2441]
odla_value odla_Mean(odla_values inputs, const odla_value_id id) {
  REQUIRE(inputs.size >= 1 && inputs.size <= ODLA_MAX_OUTPUTS, "odla_Mean: bad operand count");
  odla_value acc = inputs.values[0];
  REQUIRE(acc, "odla_Mean: null operand");
  REQUIRE(is_float_type(acc->etype), "odla_Mean: operands must be a float type");
  for (odla_size_t i = 1; i < inputs.size; ++i) {
    acc = binary(BIN_ADD, acc, inputs.values[i], nullptr);
    if (acc == nullptr) return nullptr;
  }
  _odla_computation* c = comp_of(acc);
  Node* n = add_node(c, OP_UNARY, {acc}, acc->etype, acc->shape, id);
  if (n == nullptr) return ADD_NODE_FAILED;
  n->i[0] = ACT_DIV_CONST;
  n->f[0] = (float)inputs.size;
  return n->out;
}

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
odla_value odla_Reciprocal(odla_value x, const odla_value_id id) { return unary(ACT_RECIP, x, 0, 0, id); }
odla_value odla_Ceil(odla_value x, const odla_value_id id) { return unary(ACT_CEIL, x, 0, 0, id); }
odla_value odla_Floor(odla_value x, const odla_value_id id) { return unary(ACT_FLOOR, x, 0, 0, id); }
odla_value odla_Sign(odla_value x, const odla_value_id id) { return unary(ACT_SIGN, x, 0, 0, id); }
odla_value odla_Sin(odla_value x, const odla_value_id id) { return unary(ACT_SIN, x, 0, 0, id); }
odla_value odla_Cos(odla_value x, const odla_value_id id) { return unary(ACT_COS, x, 0, 0, id); }
odla_value odla_Tan(odla_value x, const odla_value_id id) { return unary(ACT_TAN, x, 0, 0, id); }
odla_value odla_ASin(odla_value x, const odla_value_id id) { return unary(ACT_ASIN, x, 0, 0, id); }
odla_value odla_ACos(odla_value x, const odla_value_id id) { return unary(ACT_ACOS, x, 0, 0, id); }
odla_value odla_ATan(odla_value x, const odla_value_id id) { return unary(ACT_ATAN, x, 0, 0, id); }
odla_value odla_Sinh(odla_value x, const odla_value_id id) { return unary(ACT_SINH, x, 0, 0, id); }
odla_value odla_Cosh(odla_value x, const odla_value_id id) { return unary(ACT_COSH, x, 0, 0, id); }
odla_value odla_ASinh(odla_value x, const odla_value_id id) { return unary(ACT_ASINH, x, 0, 0, id); }
odla_value odla_ACosh(odla_value x, const odla_value_id id) { return unary(ACT_ACOSH, x, 0, 0, id); }
odla_value odla_ATanh(odla_value x, const odla_value_id id) { return unary(ACT_ATANH, x, 0, 0, id); }
odla_value odla_Elu(odla_value x, odla_float32 alpha, const odla_value_id id) { return unary(ACT_ELU, x, alpha, 0, id); }
odla_value odla_Selu(odla_value x, odla_float32 alpha, odla_float32 gamma, const odla_value_id id) {
  return unary(ACT_SELU, x, alpha, gamma, id);
}
odla_value odla_Celu(odla_value x, odla_float32 alpha, const odla_value_id id) {
  if (alpha == 0.f) {
    OHIP_ERR("odla_Celu: alpha must not be zero");
    return nullptr;
  }
  return unary(ACT_CELU, x, alpha, 0, id);
}
odla_value odla_HardSigmoid(odla_value x, odla_float32 alpha, odla_float32 beta, const odla_value_id id) {
  return unary(ACT_HARDSIGMOID, x, alpha, beta, id);
}
odla_value odla_Softplus(odla_value x, const odla_value_id id) { return unary(ACT_SOFTPLUS, x, 0, 0, id); }
odla_value odla_Softsign(odla_value x, const odla_value_id id) { return unary(ACT_SOFTSIGN, x, 0, 0, id); }
odla_value odla_ThresholdedRelu(odla_value x, odla_float32 alpha, const odla_value_id id) {
  return unary(ACT_THRESHOLDED, x, alpha, 0, id);
}
odla_value odla_Shrink(odla_value x, odla_float32 bias, odla_float32 lambd, const odla_value_id id) {
  return unary(ACT_SHRINK, x, bias, lambd, id);
}
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
  if (n == nullptr) return ADD_NODE_FAILED;
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
  if (n == nullptr) return ADD_NODE_FAILED;
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
odla_value odla_ReduceMin(odla_value input, odla_size_t n, const odla_uint32* axes, odla_bool keep,
                          odla_value_shape, const odla_value_id id) {
  return reduce(RED_MIN, input, n, axes, keep, id);
}
odla_value odla_ReduceProd(odla_value input, odla_size_t n, const odla_uint32* axes, odla_bool keep,
                           odla_value_shape, const odla_value_id id) {
  return reduce(RED_PROD, input, n, axes, keep, id);
}
odla_value odla_ReduceL1(odla_value input, odla_size_t n, const odla_uint32* axes, odla_bool keep,
                         odla_float32 epsilon, odla_value_shape, const odla_value_id id) {
  return reduce(RED_L1, input, n, axes, keep, id, epsilon);
}
odla_value odla_ReduceL2(odla_value input, odla_size_t n, const odla_uint32* axes, odla_bool keep,
                         odla_float32 epsilon, odla_value_shape, const odla_value_id id) {
  return reduce(RED_L2, input, n, axes, keep, id, epsilon);
}
odla_value odla_ReduceSumSquare(odla_value input, odla_size_t n, const odla_uint32* axes, odla_bool keep,
                                odla_value_shape, const odla_value_id id) {
  return reduce(RED_SUMSQ, input, n, axes, keep, id);
}
odla_value odla_ReduceLogSum(odla_value input, odla_size_t n, const odla_uint32* axes, odla_bool keep,
                             odla_value_shape, const odla_value_id id) {
  return reduce(RED_LOGSUM, input, n, axes, keep, id);
}
// log(sum(exp(x - max))) + max, composed from the existing operators as the
// reference does.  [ref: ODLA/platforms/dnnl/odla_dnnl_statistics.cc:77-105]
odla_value odla_ReduceLogSumExp(odla_value input, odla_size_t n, const odla_uint32* axes, odla_bool keep,
                                odla_value_shape, const odla_value_id id) {
  odla_value mx = reduce(RED_MAX, input, n, axes, 1, nullptr);
  if (mx == nullptr) return nullptr;
  odla_value delta = binary(BIN_SUB, input, mx, nullptr);
  if (delta == nullptr) return nullptr;
  odla_value ex = unary(ACT_EXP, delta, 0, 0, nullptr);
  odla_value ls = reduce(RED_LOGSUM, ex, n, axes, 1, nullptr);
  if (ls == nullptr) return nullptr;
  odla_value sum = binary(BIN_ADD, ls, mx, keep ? id : nullptr);
  if (sum == nullptr || keep) return sum;
  // drop the reduced dims
  bool red[ODLA_MAX_DIMENSION] = {false};
  const int r = input->shape.rank;
  if (n == 0)
    for (int i = 0; i < r; ++i) red[i] = true;
  for (odla_size_t i = 0; i < n; ++i) red[axes[i]] = true;
  Shape o;
  for (int i = 0; i < r; ++i)
    if (!red[i]) o.d[o.rank++] = input->shape.d[i];
  if (o.rank == 0) { o.rank = 1; o.d[0] = 1; }
  return odla_Reshape(sum, shape_to(o), id);
}
odla_value odla_ArgMax(odla_value input, odla_int32 axis, odla_bool keep_dims, odla_bool return_last_index,
                       odla_value_type output_value_type, const odla_value_id id) {
  return arg_extreme(true, input, axis, keep_dims, return_last_index, output_value_type, id);
}
odla_value odla_ArgMin(odla_value input, odla_int32 axis, odla_bool keep_dims, odla_bool return_last_index,
                       odla_value_type output_value_type, const odla_value_id id) {
  return arg_extreme(false, input, axis, keep_dims, return_last_index, output_value_type, id);
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
  if (n == nullptr) return ADD_NODE_FAILED;
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
  if (n == nullptr) return ADD_NODE_FAILED;
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
  if (n == nullptr) return ADD_NODE_FAILED;
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
  if (n == nullptr) return ADD_NODE_FAILED;
  n->i[0] = axis;
  return n->out;
}

// ---------------------------------------------------------------------------
// Operators along one axis (OP_AXISOP): i[0] = AxisOp, i[1] = axis (resolved, >= 0).
// CumSum: i[2] = exclusive, i[3] = reverse.  Compress: i[2] = conditions used,
// i[3] = 1 when the operand is taken as one flat axis.

// [ref: ops/odla_ops_process.h:187-201; dnnl odla_dnnl.cc:509-567]
odla_value odla_GatherElements(odla_value input, odla_value indices, odla_int32 axis, odla_value_shape,
                               const odla_value_id id) {
  REQUIRE(input && indices, "odla_GatherElements: null operand");
  _odla_computation* c = comp_of(input, indices);
  REQUIRE(c, "odla_GatherElements: no current computation");
  REQUIRE(indices->etype == ODLA_INT32 || indices->etype == ODLA_INT64, "odla_GatherElements: indices must be int32/int64");
  const int r = input->shape.rank;
  REQUIRE(indices->shape.rank == r, "odla_GatherElements: indices %s and input %s differ in rank", indices->shape.str().c_str(),
          input->shape.str().c_str());
  if (axis < 0) axis += r;
  REQUIRE(axis >= 0 && axis < r, "odla_GatherElements: axis out of range");
  // The operands are walked as [i][j][k] with j the axis (like the reference): the leading and
  // trailing extents of the indices may be smaller than the input's only where that keeps
  // the flattened walk meaningful - a smaller extent in the first of the merged dims.
  for (int i = 0; i < r; ++i) {
    if (i == axis) continue;
    REQUIRE(indices->shape.d[i] <= input->shape.d[i], "odla_GatherElements: indices %s exceed the input %s",
            indices->shape.str().c_str(), input->shape.str().c_str());
    const bool first_of_group = i == 0 || i == axis + 1;
    REQUIRE(indices->shape.d[i] == input->shape.d[i] || first_of_group,
            "odla_GatherElements: indices %s may only be smaller than the input %s along the axis, dim 0 or the dim behind the axis",
            indices->shape.str().c_str(), input->shape.str().c_str());
  }
  Node* n = add_node(c, OP_AXISOP, {input, indices}, input->etype, indices->shape, id);
  if (n == nullptr) return ADD_NODE_FAILED;
  n->i[0] = AX_GATHER_ELEMENTS;
  n->i[1] = axis;
  return n->out;
}

// The axis is a constant scalar (INT32 or INT64); the reference reads it when the
// computation runs, here it is read when the node is recorded.
// [ref: ops/odla_ops_math.h:239-241; dnnl odla_dnnl_statistics.cc:147-200]
odla_value odla_CumSum(odla_value input, odla_value axis, odla_bool exclusion, odla_bool reverse, const odla_value_id id) {
  REQUIRE(input && axis, "odla_CumSum: null operand");
  _odla_computation* c = comp_of(input);
  REQUIRE(c, "odla_CumSum: no current computation");
  REQUIRE(is_float_type(input->etype), "odla_CumSum: operand must be a float type");
  REQUIRE(axis->kind == _odla_value::CONSTANT && axis->host_data != nullptr && axis->shape.numel() >= 1 &&
              (axis->etype == ODLA_INT32 || axis->etype == ODLA_INT64),
          "odla_CumSum: the axis must be a constant INT32 / INT64 scalar");
  int64_t ax = axis->etype == ODLA_INT32 ? (int64_t) * static_cast<const int32_t*>(axis->host_data)
                                         : *static_cast<const int64_t*>(axis->host_data);
  const int r = input->shape.rank;
  if (ax < 0) ax += r;
  REQUIRE(ax >= 0 && ax < r, "odla_CumSum: axis out of range for %s", input->shape.str().c_str());
  Node* n = add_node(c, OP_AXISOP, {input}, input->etype, input->shape, id);
  if (n == nullptr) return ADD_NODE_FAILED;
  n->i[0] = AX_CUMSUM;
  n->i[1] = ax;
  n->i[2] = exclusion != 0;
  n->i[3] = reverse != 0;
  return n->out;
}

// One-hot of the first largest element along the axis (a negative axis counts from the
// end; the reference takes every negative axis as the last one in its second half).
// [ref: ops/odla_ops_nn.h:114-126; dnnl odla_dnnl.cc:1688-1727]
odla_value odla_Hardmax(odla_value input, odla_int32 axis, const odla_value_id id) {
  REQUIRE(input, "odla_Hardmax: null operand");
  _odla_computation* c = comp_of(input);
  REQUIRE(c, "odla_Hardmax: no current computation");
  REQUIRE(is_float_type(input->etype), "odla_Hardmax: operand must be a float type");
  const int r = input->shape.rank;
  if (axis < 0) axis += r;
  REQUIRE(axis >= 0 && axis < r, "odla_Hardmax: axis out of range for %s", input->shape.str().c_str());
  Node* n = add_node(c, OP_AXISOP, {input}, input->etype, input->shape, id);
  if (n == nullptr) return ADD_NODE_FAILED;
  n->i[0] = AX_HARDMAX;
  n->i[1] = axis;
  return n->out;
}

// The result has the declared maximum shape; the selected slices fill it densely from the
// start ([outer][selected][inner]) and the rest is zero (undefined in the reference).
// axis == INT_MAX: the operand is taken as one flat axis.
// [ref: ops/odla_ops_process.h:83-98; dnnl odla_dnnl.cc:1280-1328]
odla_value odla_Compress(odla_value input, odla_value condition, odla_int32 axis, odla_value_shape max_output_shape,
                         const odla_value_id id) {
  REQUIRE(input && condition, "odla_Compress: null operand");
  _odla_computation* c = comp_of(input, condition);
  REQUIRE(c, "odla_Compress: no current computation");
  REQUIRE(condition->etype == ODLA_BOOL && condition->shape.rank == 1, "odla_Compress: the condition must be a boolean vector");
  REQUIRE(shape_valid(max_output_shape) && max_output_shape.size >= 1, "odla_Compress: the maximum result shape is required");
  const Shape o = shape_from(max_output_shape);
  const int r = input->shape.rank;
  const bool flat = axis == INT_MAX;
  int64_t used = condition->shape.d[0];
  if (flat) {
    axis = 0;
    used = std::min(used, std::min(o.numel(), input->shape.numel()));
  } else {
    if (axis < 0) axis += r;
    REQUIRE(axis >= 0 && axis < r, "odla_Compress: axis out of range for %s", input->shape.str().c_str());
    used = std::min(used, input->shape.d[axis]);
    int64_t outer = 1, inner = 1;
    for (int i = 0; i < axis; ++i) outer *= input->shape.d[i];
    for (int i = axis + 1; i < r; ++i) inner *= input->shape.d[i];
    REQUIRE(outer * used * inner <= o.numel(), "odla_Compress: the maximum result shape %s cannot hold %lld slices",
            o.str().c_str(), (long long)used);
  }
  REQUIRE(used < (1ll << 31), "odla_Compress: too many conditions");
  Node* n = add_node(c, OP_AXISOP, {input, condition}, input->etype, o, id);
  if (n == nullptr) return ADD_NODE_FAILED;
  n->i[0] = AX_COMPRESS;
  n->i[1] = axis;
  n->i[2] = used;
  n->i[3] = flat;
  return n->out;
}

// Logical shifts of unsigned integers (UINT8, UINT32, UINT64; no 16-bit integer storage
// here); a shift by the width of the type or more gives 0 (undefined in the reference).
// [ref: ops/odla_ops_math.h:863-876; dnnl odla_dnnl.cc:947-1010]
odla_value odla_Shift(odla_value input, odla_value shift_amount, odla_bool is_left_shift, const odla_value_id id) {
  REQUIRE(input && shift_amount, "odla_Shift: null operand");
  REQUIRE(input->etype == ODLA_UINT8 || input->etype == ODLA_UINT32 || input->etype == ODLA_UINT64,
          "odla_Shift: operand must be UINT8, UINT32 or UINT64");
  REQUIRE(input->etype == shift_amount->etype, "odla_Shift: operand and shift amount differ in element type");
  return ewise(is_left_shift ? EW_SHL : EW_SHR, {input, shift_amount}, input->etype, "odla_Shift", id);
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
  if (n == nullptr) return ADD_NODE_FAILED;
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
  REQUIRE(interpolation == ODLA_NEAREST || interpolation == ODLA_LINEAR, "odla_Resize: nearest and linear interpolation are supported");
  REQUIRE(interpolation == ODLA_NEAREST || input->etype == ODLA_FLOAT32 || input->etype == ODLA_FLOAT16 ||
              input->etype == ODLA_BFLOAT16,
          "odla_Resize: linear interpolation needs a float input");
  Shape o = shape_from(output_dims);
  REQUIRE(o.d[0] == input->shape.d[0] && o.d[1] == input->shape.d[1] && o.d[2] > 0 && o.d[3] > 0,
          "odla_Resize: output %s must keep batch and channels of %s", o.str().c_str(), input->shape.str().c_str());
  Node* n = add_node(c, OP_RESIZE, {input}, input->etype, o, id);
  if (n == nullptr) return ADD_NODE_FAILED;
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
  if (n == nullptr) return ADD_NODE_FAILED;
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
  if (n == nullptr) return ADD_NODE_FAILED;
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
  if (n == nullptr) return ADD_NODE_FAILED;
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

// Zero padding.  [ref: ODLA/include/ODLA/ops/odla_ops_process.h:221-236]
odla_value odla_Pad(odla_value input, const odla_uint32* padding_front, const odla_uint32* padding_back,
                    odla_value_shape, const odla_value_id id) {
  REQUIRE(input && padding_front && padding_back, "odla_Pad: null argument");
  _odla_computation* c = comp_of(input);
  REQUIRE(c, "odla_Pad: no current computation");
  const Shape& xs = input->shape;
  REQUIRE(xs.rank <= 8, "odla_Pad: rank > 8");
  Shape o = xs;
  for (int i = 0; i < xs.rank; ++i) o.d[i] = xs.d[i] + padding_front[i] + padding_back[i];
  const std::vector<int64_t> sx = row_major_strides(xs), sy = row_major_strides(o);
  int64_t y_off = 0;
  for (int i = 0; i < xs.rank; ++i) y_off += (int64_t)padding_front[i] * sy[i];
  std::vector<int64_t> dims(xs.d, xs.d + xs.rank);
  return copynd(c, input, o, dims, sx, sy, 0, y_off, true, id);
}

// Repeats the input `repeat[i]` times along dim i.
// [ref: ops/odla_ops_process.h:437-451; dnnl odla_dnnl.cc:2183-2254]
odla_value odla_Tile(odla_value input, const odla_uint32* repeat, odla_value_shape, const odla_value_id id) {
  REQUIRE(input && repeat, "odla_Tile: null argument");
  _odla_computation* c = comp_of(input);
  REQUIRE(c, "odla_Tile: no current computation");
  const Shape& xs = input->shape;
  REQUIRE(xs.rank <= 4, "odla_Tile: rank > 4");
  Shape o = xs;
  std::vector<int64_t> dims, sx, sy;
  for (int i = 0; i < xs.rank; ++i) {
    REQUIRE(repeat[i] >= 1, "odla_Tile: repeat count 0");
    o.d[i] = xs.d[i] * repeat[i];
  }
  const std::vector<int64_t> xst = row_major_strides(xs), yst = row_major_strides(o);
  for (int i = 0; i < xs.rank; ++i) {
    dims.push_back(repeat[i]); sx.push_back(0); sy.push_back(yst[i] * xs.d[i]);
    dims.push_back(xs.d[i]); sx.push_back(xst[i]); sy.push_back(yst[i]);
  }
  return copynd(c, input, o, dims, sx, sy, 0, 0, false, id);
}

// Broadcast to `output_dims`.  [ref: ops/odla_ops_process.h:117-130]
odla_value odla_ExpandDims(odla_value input, odla_value_shape output_dims, const odla_value_id id) {
  REQUIRE(input, "odla_ExpandDims: null argument");
  REQUIRE(shape_valid(output_dims), "odla_ExpandDims: the output shape is required");
  _odla_computation* c = comp_of(input);
  REQUIRE(c, "odla_ExpandDims: no current computation");
  const Shape o = shape_from(output_dims);
  REQUIRE(o.rank <= 8, "odla_ExpandDims: rank > 8");
  Shape al = input->shape;
  if (al.rank != o.rank)
    REQUIRE(al.rank < o.rank && expand_like_reference(&al, o), "odla_ExpandDims: %s does not broadcast to %s",
            input->shape.str().c_str(), o.str().c_str());
  std::vector<int64_t> dims(o.d, o.d + o.rank), sx = row_major_strides(al), sy = row_major_strides(o);
  for (int i = 0; i < o.rank; ++i) {
    REQUIRE(al.d[i] == o.d[i] || al.d[i] == 1, "odla_ExpandDims: %s does not broadcast to %s",
            input->shape.str().c_str(), o.str().c_str());
    if (al.d[i] == 1) sx[i] = 0;
  }
  return copynd(c, input, o, dims, sx, sy, 0, 0, false, id);
}

// Removes the listed 1-sized dims (all of them when none is listed).
// [ref: ops/odla_ops_process.h:397-412]
odla_value odla_Squeeze(odla_value input, odla_size_t num_of_axes, const odla_uint32* axes, odla_value_shape,
                        const odla_value_id id) {
  REQUIRE(input && (axes || num_of_axes == 0), "odla_Squeeze: null argument");
  const Shape& xs = input->shape;
  bool drop[ODLA_MAX_DIMENSION] = {false};
  for (odla_size_t i = 0; i < num_of_axes; ++i) {
    REQUIRE((int)axes[i] < xs.rank && xs.d[axes[i]] == 1, "odla_Squeeze: axis %u of %s is not 1", axes[i], xs.str().c_str());
    drop[axes[i]] = true;
  }
  Shape o;
  for (int i = 0; i < xs.rank; ++i) {
    const bool d = num_of_axes == 0 ? xs.d[i] == 1 : drop[i];
    if (!d) o.d[o.rank++] = xs.d[i];
  }
  if (o.rank == 0) { o.rank = 1; o.d[0] = 1; }
  return odla_Reshape(input, shape_to(o), id);
}

// Joins same-shaped values along a new axis.  [ref: ops/odla_ops_process.h:414-430]
odla_value odla_Stack(odla_values inputs, odla_int32 axis, odla_value_shape, const odla_value_id id) {
  REQUIRE(inputs.size >= 1 && inputs.size <= ODLA_MAX_OUTPUTS && inputs.values[0], "odla_Stack: bad operand list");
  const Shape& xs = inputs.values[0]->shape;
  if (axis < 0) axis += xs.rank + 1;
  REQUIRE(axis >= 0 && axis <= xs.rank && xs.rank < ODLA_MAX_DIMENSION, "odla_Stack: axis out of range");
  Shape one;
  one.rank = xs.rank + 1;
  for (int i = 0, j = 0; i < one.rank; ++i) one.d[i] = i == axis ? 1 : xs.d[j++];
  odla_values parts;
  parts.size = inputs.size;
  for (odla_size_t i = 0; i < inputs.size; ++i) {
    REQUIRE(inputs.values[i] && inputs.values[i]->shape == xs, "odla_Stack: operands differ in shape");
    parts.values[i] = odla_Reshape(inputs.values[i], shape_to(one), nullptr);
    if (parts.values[i] == nullptr) return nullptr;
  }
  return odla_Concat(parts, axis, undefined_shape(), id);
}

// K largest / smallest elements along `axis`, best first, and their indices.
// [ref: ops/odla_ops_process.h (odla_TopK); dnnl odla_dnnl.cc:2064-2111]
odla_values odla_TopK(odla_value input, odla_uint32 K, odla_bool largest, odla_bool sorted, odla_uint32 axis,
                      odla_value_type output_value_type, odla_value_type output_value_index_type,
                      const odla_value_ids value_ids) {
  (void)sorted;  // results are always ordered
  (void)output_value_type;
  odla_values none;
  none.size = 0;
  auto bail = [&](const char* msg) { OHIP_ERR("odla_TopK: %s", msg); return none; };
  if (input == nullptr) return bail("null operand");
  _odla_computation* c = comp_of(input);
  if (c == nullptr) return bail("no current computation");
  if (!is_float_type(input->etype)) return bail("operand must be a float type");
  const Shape& xs = input->shape;
  if ((int)axis >= xs.rank) return bail("axis out of range");
  if (K < 1 || (int64_t)K > xs.d[axis]) return bail("K out of range");
  const odla_element_type it = output_value_index_type.element_type == ODLA_INT64 ? ODLA_INT64 : ODLA_INT32;
  Shape o = xs;
  o.d[axis] = K;
  Node* n = add_node(c, OP_TOPK, {input}, input->etype, o, value_ids.size > 0 ? value_ids.value_ids[0] : nullptr);
  if (n == nullptr) return ADD_NODE_FAILED;
  n->out2 = new_value(c, _odla_value::TEMP, it, o, value_ids.size > 1 ? value_ids.value_ids[1] : nullptr);
  n->out2->producer = n->out->producer;
  n->i[0] = K;
  n->i[1] = largest != 0;
  n->i[2] = axis;
  odla_values r;
  r.size = 2;
  r.values[0] = n->out;
  r.values[1] = n->out2;
  return r;
}

// YOLOv3 post-processing of one image: decode of the 13-, 26- and 52-cell heads
// and, per class, the boxes that survive the suppression walk.  Results: value
// "<id>0" [classes, N / 169, 5] rows {y min, x min, y max, x max, score} in
// source-image pixels, zero padded, and "<id>1" [classes] rows kept (N = boxes
// of the three heads; the reference leaves the padding undefined and has no
// bound on the rows of a class - here a class stops at its N / 169 rows).
// [ref: ops/odla_ops_nn.h:744-759 (odla_PostProcess); popart odla_ops_nn.cc:462-484,
//  custom_ops/postprocess.cc:67-81 (result shapes), :139-290, codelets_nms.cpp:24-125]
odla_values odla_PostProcess(odla_value orig_img_w, odla_value orig_img_h, odla_value bb13, odla_value bb26,
                             odla_value bb52, const odla_value_id value_id) {
  odla_values none;
  none.size = 0;
  auto bail = [&](const char* msg) { OHIP_ERR("odla_PostProcess: %s", msg); return none; };
  if (!orig_img_w || !orig_img_h || !bb13 || !bb26 || !bb52) return bail("null operand");
  _odla_computation* c = comp_of(bb13);
  if (c == nullptr) return bail("no current computation");
  const odla_value heads[3] = {bb13, bb26, bb52};
  const odla_value sizes[2] = {orig_img_w, orig_img_h};
  for (odla_value s : sizes) {
    if (s->etype != ODLA_UINT32 && s->etype != ODLA_INT32) return bail("the image size must be 32-bit integers");
    if (s->shape.numel() != 1) return bail("the image size must be scalars");
  }
  int64_t total = 0;
  for (odla_value h : heads) {
    if (!is_float_type(h->etype)) return bail("the heads must be float tensors");
    const Shape& s = h->shape;
    if (s.rank != 4 || s.d[0] != 1) return bail("the heads must be [1, 3 * (5 + classes), dim, dim]");
    if (s.d[2] != s.d[3] || s.d[2] < 1) return bail("a head is not square");
    if (s.d[1] != bb13->shape.d[1]) return bail("the heads differ in channels");
    total += 3 * s.d[2] * s.d[2];
  }
  const int64_t ch = bb13->shape.d[1];
  if (ch % 3 != 0 || ch / 3 < 6) return bail("the channels of a head must be 3 * (5 + classes)");
  const int64_t classes = ch / 3 - 5, capacity = total / 169;
  if (capacity < 1) return bail("fewer than 169 boxes");
  const std::string base = value_id ? std::string(reinterpret_cast<const char*>(value_id)) : std::string();
  const std::string n0 = base + "0", n1 = base + "1";
  Shape o0, o1;
  o0.rank = 3; o0.d[0] = classes; o0.d[1] = capacity; o0.d[2] = 5;
  o1.rank = 1; o1.d[0] = classes;
  Node* n = add_node(c, OP_POSTPROCESS, {orig_img_w, orig_img_h, bb13, bb26, bb52}, ODLA_FLOAT32, o0,
                     value_id ? (const odla_value_id)n0.c_str() : nullptr);
  if (n == nullptr) return ADD_NODE_FAILED;
  n->out2 = new_value(c, _odla_value::TEMP, ODLA_UINT32, o1, value_id ? (const odla_value_id)n1.c_str() : nullptr);
  n->out2->producer = n->out->producer;
  n->f[0] = 0.45f;  // IoU above which a box is suppressed
  n->f[1] = 0.3f;   // lowest score that takes part
  odla_values r;
  r.size = 2;
  r.values[0] = n->out;
  r.values[1] = n->out2;
  return r;
}

// [ref: ops/odla_ops_nn.h (odla_LRN); dnnl odla_dnnl.cc:1553-1581]
odla_value odla_LRN(odla_value input, odla_memory_layout layout, odla_int32 window_size, odla_float32 alpha,
                    odla_float32 beta, odla_float32 bias, const odla_value_id id) {
  REQUIRE(input, "odla_LRN: null argument");
  _odla_computation* c = comp_of(input);
  REQUIRE(c, "odla_LRN: no current computation");
  REQUIRE(is_float_type(input->etype), "odla_LRN: operand must be a float type");
  REQUIRE(input->shape.rank >= 3, "odla_LRN: rank < 3");
  REQUIRE(window_size >= 1 && (window_size & 1), "odla_LRN: the window must be odd");
  Node* n = add_node(c, OP_LRN, {input}, input->etype, input->shape, id);
  if (n == nullptr) return ADD_NODE_FAILED;
  n->i[0] = layout == ODLA_CHANNELS_LAST ? ODLA_CHANNELS_LAST : ODLA_CHANNELS_FIRST;
  n->i[1] = window_size;
  n->f[0] = alpha; n->f[1] = beta; n->f[2] = bias;
  return n->out;
}

// Normalisation over the spatial dims of every (sample, channel) pair.
// [ref: ops/odla_ops_nn.h (odla_InstanceNormalization); dnnl odla_dnnl.cc:1583-1626]
odla_value odla_InstanceNormalization(odla_value input, odla_memory_layout layout, odla_float32 epsilon,
                                      odla_value scale, odla_value offset, odla_float32 scalar_scale,
                                      odla_float32 scalar_offset, const odla_value_id id) {
  REQUIRE(input, "odla_InstanceNormalization: null argument");
  _odla_computation* c = comp_of(input);
  REQUIRE(c, "odla_InstanceNormalization: no current computation");
  REQUIRE(is_float_type(input->etype), "odla_InstanceNormalization: operand must be a float type");
  const Shape& xs = input->shape;
  REQUIRE(xs.rank >= 3, "odla_InstanceNormalization: rank < 3");
  const bool cl = layout == ODLA_CHANNELS_LAST;
  const int64_t C = cl ? xs.d[xs.rank - 1] : xs.d[1];
  if (scale) REQUIRE(scale->kind == _odla_value::CONSTANT && scale->shape.numel() == C,
                     "odla_InstanceNormalization: scale must be a constant with one element per channel");
  if (offset) REQUIRE(offset->kind == _odla_value::CONSTANT && offset->shape.numel() == C,
                      "odla_InstanceNormalization: offset must be a constant with one element per channel");
  Node* n = add_node(c, OP_ROWNORM, {input, scale, offset}, input->etype, xs, id);
  if (n == nullptr) return ADD_NODE_FAILED;
  n->i[0] = cl ? ODLA_CHANNELS_LAST : ODLA_CHANNELS_FIRST;
  n->f[0] = epsilon; n->f[1] = scalar_scale; n->f[2] = scalar_offset;
  return n->out;
}

// Transposed convolution, rewritten as a stride-1 convolution of the
// zero-stuffed input with the flipped, in/out-swapped kernel.
// [ref: ops/odla_ops_nn.h (odla_DeConv); dnnl odla_dnnl.cc:1131-1232]
odla_value odla_DeConv(odla_value input, odla_memory_layout input_layout, odla_uint32 group, odla_value kernel,
                       odla_memory_layout kernel_layout, const odla_uint32* strides, const odla_uint32* dilations,
                       const odla_uint32* paddings_front, const odla_uint32* paddings_back, odla_value bias,
                       odla_value_shape output_dims, const odla_value_id id) {
  REQUIRE(input && kernel && strides && dilations && paddings_front && paddings_back, "odla_DeConv: null argument");
  _odla_computation* c = comp_of(input, kernel);
  REQUIRE(c, "odla_DeConv: no current computation");
  REQUIRE(input->shape.rank == 4 && kernel->shape.rank == 4, "odla_DeConv: only 2-D is supported");
  REQUIRE(input_layout != ODLA_CHANNELS_LAST, "odla_DeConv: channels-last input is not supported");
  REQUIRE(kernel->kind == _odla_value::CONSTANT && kernel->host_data != nullptr, "odla_DeConv: the kernel must be a constant");
  REQUIRE(kernel->etype == ODLA_FLOAT32, "odla_DeConv: the kernel must be FLOAT32");
  REQUIRE(dilations[0] == 1 && dilations[1] == 1, "odla_DeConv: dilation is not supported");
  REQUIRE(strides[0] >= 1 && strides[1] >= 1, "odla_DeConv: bad stride");
  if (group == 0) group = 1;
  const Shape& x = input->shape;
  const Shape& k = kernel->shape;
  // element (o_in_group, c, r, s) of the kernel, c = input channel, o = output channel within its group
  int64_t Cin, Og, R, S, so, sc, sr, ss;
  switch (kernel_layout) {
    case ODLA_IOS: Cin = k.d[0]; Og = k.d[1]; R = k.d[2]; S = k.d[3]; sc = Og * R * S; so = R * S; sr = S; ss = 1; break;
    case ODLA_SIO: R = k.d[0]; S = k.d[1]; Cin = k.d[2]; Og = k.d[3]; sr = S * Cin * Og; ss = Cin * Og; sc = Og; so = 1; break;
    case ODLA_SOI: R = k.d[0]; S = k.d[1]; Og = k.d[2]; Cin = k.d[3]; sr = S * Cin * Og; ss = Cin * Og; so = Cin; sc = 1; break;
    default: Og = k.d[0]; Cin = k.d[1]; R = k.d[2]; S = k.d[3]; so = Cin * R * S; sc = R * S; sr = S; ss = 1; break;
  }
  const int64_t N = x.d[0], C = x.d[1], H = x.d[2], W = x.d[3];
  REQUIRE(C == Cin && C % group == 0, "odla_DeConv: input channels %lld do not match the kernel (%lld, group %u)",
          (long long)C, (long long)Cin, group);
  const int64_t O = Og * group, Cg = C / group;
  const int64_t st[2] = {strides[0], strides[1]}, KS[2] = {R, S}, IN[2] = {H, W};
  int64_t out_hw[2], pf[2], pb[2], up[2];
  for (int d = 0; d < 2; ++d) {
    up[d] = (IN[d] - 1) * st[d] + 1;
    int64_t want = up[d] + KS[d] - 1 - (int64_t)paddings_front[d] - (int64_t)paddings_back[d];
    if (shape_valid(output_dims) && output_dims.size == 4 && output_dims.dims[2 + d] >= want &&
        output_dims.dims[2 + d] < want + st[d])
      want = output_dims.dims[2 + d];  // output padding
    out_hw[d] = want;
    pf[d] = KS[d] - 1 - (int64_t)paddings_front[d];
    pb[d] = want - (up[d] + pf[d] - KS[d] + 1);
    REQUIRE(pf[d] >= 0 && pb[d] >= 0 && want > 0, "odla_DeConv: padding larger than the kernel is not supported");
  }
  if (bias) REQUIRE(bias->shape.numel() == O, "odla_DeConv: bias has %lld elements, expected %lld",
                    (long long)bias->shape.numel(), (long long)O);
  // flipped kernel in OIHW order with per-group input channels
  auto buf = std::make_unique<std::vector<uint8_t>>((size_t)(O * Cg * R * S) * sizeof(float));
  float* wf = reinterpret_cast<float*>(buf->data());
  const float* w = static_cast<const float*>(kernel->host_data);
  for (int64_t g = 0; g < group; ++g)
    for (int64_t oi = 0; oi < Og; ++oi)
      for (int64_t ci = 0; ci < Cg; ++ci)
        for (int64_t r = 0; r < R; ++r)
          for (int64_t s = 0; s < S; ++s)
            wf[(((g * Og + oi) * Cg + ci) * R + r) * S + s] =
                w[oi * so + (g * Cg + ci) * sc + (R - 1 - r) * sr + (S - 1 - s) * ss];
  Shape ks;
  ks.rank = 4;
  ks.d[0] = O; ks.d[1] = Cg; ks.d[2] = R; ks.d[3] = S;
  odla_value kf = new_value(c, _odla_value::CONSTANT, ODLA_FLOAT32, ks, nullptr);
  kf->host_data = wf;
  c->owned_data.push_back(std::move(buf));
  // zero-stuffed input
  odla_value xu = input;
  if (st[0] > 1 || st[1] > 1) {
    Shape us = x;
    us.d[2] = up[0]; us.d[3] = up[1];
    std::vector<int64_t> dims(x.d, x.d + 4), sx = row_major_strides(x), sy = row_major_strides(us);
    sy[2] *= st[0];
    sy[3] *= st[1];
    xu = copynd(c, input, us, dims, sx, sy, 0, 0, true, nullptr);
  }
  Shape o;
  o.rank = 4;
  o.d[0] = N; o.d[1] = O; o.d[2] = out_hw[0]; o.d[3] = out_hw[1];
  Node* n = add_node(c, OP_CONV, {xu, kf, bias}, input->etype, o, id);
  if (n == nullptr) return ADD_NODE_FAILED;
  n->i[0] = ODLA_CHANNELS_FIRST;
  n->i[1] = group;
  n->i[2] = ODLA_OIS;
  n->i[3] = 1; n->i[4] = 1;
  n->i[5] = 1; n->i[6] = 1;
  n->i[7] = pf[0]; n->i[8] = pf[1];
  n->i[9] = pb[0]; n->i[10] = pb[1];
  return n->out;
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
  if (n == nullptr) return ADD_NODE_FAILED;
  n->i[0] = max_num_outputs;
  n->f[0] = iou_threshold;
  n->f[1] = score_threshold;
  return n->out;
}

}  // extern "C"
