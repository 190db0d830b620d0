// Dynamic batch: a computation is recorded once, with the largest batch as the
// leading extent of its arguments, and executed at any smaller batch through a
// copy of the recording whose shapes were rescaled.  Each copy is planned like
// any other computation (own kernel selection, arena and hipGraph), so a small
// batch runs kernels sized for it instead of the largest batch with idle rows.
// [ref: ODLA/platforms/tensorrt/odla_tensorrt.cc:138-179 (computation items),
//  :251-268 (odla_SetRuntimeShape), :286-296 (ODLA_RUN_BATCH_SIZE), :642-656
//  (every input's leading extent is the batch); the generated code passes -1 as
//  the batch extent: lib/target/generic_cpp/generic_cxx_codegen.cc:624-637]
#include <cstring>

#include "internal.h"

namespace ohip {

int recorded_batch(const _odla_computation& c) {
  if (!c.dynamic_batch || c.max_batch <= 0) return 0;
  return c.max_batch;
}

namespace {

struct Rescaler {
  const _odla_computation& src;
  int64_t from, to;
  std::vector<char> carries;  // by value index: the leading extent is a multiple of the batch
  bool ok = true;

  bool carry(const _odla_value* v) const { return v != nullptr && carries[v->index] != 0; }

  bool quiet = false;   // a refusal is not an error: the caller has another way to run the computation

  void reject(const Node& n, const char* why) {
    if (ok && !quiet)
      OHIP_ERR("dynamic batch: %s '%s' %s; run this computation at its recorded batch %lld", api_op_name(n),
               n.out ? n.out->name.c_str() : "", why, (long long)from);
    else if (ok)
      OHIP_DEBUG("batch halves: %s '%s' %s", api_op_name(n), n.out ? n.out->name.c_str() : "", why);
    ok = false;
  }
  bool scalable(int64_t d) const { return d % from == 0; }
  int64_t scale(int64_t d) const { return d / from * to; }

  // An operand that does not depend on the arguments may only meet one that
  // does where it is broadcast along the leading extent.
  void need_broadcast_lead(const Node& n, const _odla_value* v, int out_rank) {
    if (v == nullptr || carry(v)) return;
    if (v->shape.rank == out_rank && v->shape.d[0] != 1) reject(n, "combines the batch with a constant that is not broadcast along it");
  }
};

}  // namespace

std::unique_ptr<_odla_computation> clone_for_batch(const _odla_computation& c, int64_t from, int64_t to, bool rows_apart) {
  if (from <= 0 || to <= 0) return nullptr;
  Rescaler rs{c, from, to, std::vector<char>(c.values.size(), 0)};
  rs.quiet = rows_apart;

  bool flagged = false;
  for (const _odla_value* a : c.args) flagged = flagged || a->dyn_batch;
  for (const _odla_value* a : c.args) {
    if (a->eager) {
      if (!rows_apart) OHIP_ERR("dynamic batch: values made by odla_CreateValue have no batch");
      return nullptr;
    }
    // without an explicit -1 every argument's leading extent is the batch, as in the reference
    if (flagged ? a->dyn_batch : a->shape.d[0] == from) rs.carries[a->index] = 1;
  }

  // per-node copies of the attribute vectors that hold shapes
  std::vector<std::vector<int64_t>> new_iv(c.nodes.size());
  for (size_t ni = 0; ni < c.nodes.size() && rs.ok; ++ni) {
    const Node& n = c.nodes[ni];
    new_iv[ni] = n.iv;
    bool any = false;
    for (const _odla_value* v : n.in) any = any || rs.carry(v);
    if (!any) continue;
    const _odla_value* x = n.in.empty() ? nullptr : n.in[0];
    const int out_rank = n.out ? n.out->shape.rank : 0;
    switch (n.op) {
      case OP_CONV:
        if (!rs.carry(x) || rs.carry(n.in[1])) rs.reject(n, "has a kernel that depends on the batch");
        break;
      case OP_GEMM: {
        const _odla_value* A = n.in[0];
        const _odla_value* B = n.in[1];
        if (rs.carry(A) && A->shape.rank == 2 && n.i[0]) rs.reject(n, "transposes the batch into the reduction");
        if (rs.carry(B) && (B->shape.rank == 2 || !rs.carry(A))) rs.reject(n, "has a right operand whose rows are the batch");
        if (!rs.carry(A) && !rs.carry(B)) rs.reject(n, "adds a batch-dependent matrix to a constant product");
        if (n.in.size() > 2) rs.need_broadcast_lead(n, n.in[2], out_rank);
        break;
      }
      case OP_BINARY:
      case OP_EWISE: {
        // iv = rank, then the operand shapes aligned to that rank
        const int r = (int)n.iv[0];
        for (size_t k = 0; k < n.in.size(); ++k) {
          const _odla_value* v = n.in[k];
          if (v == nullptr) continue;
          int64_t& lead = new_iv[ni][1 + k * r];
          if (rs.carry(v)) {
            if (lead != v->shape.d[0] || !rs.scalable(lead)) rs.reject(n, "aligns the batch of an operand away from the leading extent");
            else lead = rs.scale(lead);
          } else if (lead != 1) {
            rs.reject(n, "combines the batch with a constant that is not broadcast along it");
          }
        }
        break;
      }
      case OP_LAYERNORM:
        if (n.i[0] >= x->shape.rank) rs.reject(n, "normalises over the batch");
        break;
      case OP_SOFTMAX:
        if (n.i[0] == 0) rs.reject(n, "runs along the batch");
        break;
      case OP_REDUCE:
        for (int64_t ax : n.iv)
          if (ax == 0) rs.reject(n, "reduces over the batch");
        break;
      case OP_ARGEXT:
        if (n.i[1] == 0) rs.reject(n, "runs along the batch");
        break;
      case OP_TOPK:
        if (n.i[2] == 0) rs.reject(n, "runs along the batch");
        break;
      case OP_CONCAT:
        for (const _odla_value* v : n.in)
          if (!rs.carry(v)) rs.reject(n, "joins the batch with a constant");
        // (batches laid end to end: the rows of one half of the batch are not one half of the result)
        if (rows_apart && n.i[0] == 0) rs.reject(n, "joins along the batch");
        break;
      case OP_GATHER:
        if (rs.carry(n.in[0]) && (n.i[0] == 0 || rs.carry(n.in[1]))) rs.reject(n, "gathers along the batch");
        if (!rs.carry(n.in[0]) && n.i[0] != 0) rs.reject(n, "puts the batch behind the leading extent");
        break;
      case OP_SLICE: {
        const int r = x->shape.rank;
        if (n.iv[0] != 0 || n.iv[r] != x->shape.d[0] || n.iv[2 * r] != 1) rs.reject(n, "cuts the batch");
        else new_iv[ni][r] = rs.scale(n.iv[r]);
        break;
      }
      case OP_TRANSPOSE:
        if (n.iv[0] != 0) rs.reject(n, "moves the batch out of the leading extent");
        break;
      case OP_COPYND: {
        // iv = nd, extents[nd], source strides[nd], result strides[nd], source offset, result offset
        const int nd = (int)n.iv[0];
        const int64_t lead = n.iv[1];
        const int64_t x_row = x->shape.numel() / x->shape.d[0], y_row = n.out->shape.numel() / n.out->shape.d[0];
        if (nd < 1 || lead != x->shape.d[0] || lead != n.out->shape.d[0] || n.iv[1 + nd] != x_row ||
            n.iv[1 + 2 * nd] != y_row || !rs.scalable(lead))
          rs.reject(n, "pads, tiles or broadcasts along the batch");
        else
          new_iv[ni][1] = rs.scale(lead);
        break;
      }
      case OP_BATCHNORM: case OP_ROWNORM:
        for (size_t k = 1; k < n.in.size(); ++k)
          if (rs.carry(n.in[k])) rs.reject(n, "has parameters that depend on the batch");
        break;
      case OP_POSTPROCESS:
        rs.reject(n, "works on one image");
        break;
      case OP_AXISOP:
        if (n.i[1] == 0 || (n.i[0] == AX_COMPRESS && n.i[3] != 0)) rs.reject(n, "runs along the batch");
        else if (n.i[0] == AX_GATHER_ELEMENTS && !rs.carry(n.in[1])) rs.reject(n, "has indices that do not depend on the batch");
        else if (n.i[0] == AX_COMPRESS) rs.reject(n, "has a result of a declared maximum shape");
        break;
      case OP_QUANTIZE: case OP_DEQUANTIZE:
        for (size_t k = 1; k < n.in.size(); ++k)
          if (rs.carry(n.in[k])) rs.reject(n, "has a scale that depends on the batch");
        if (n.i[0] == 0 && n.in.size() > 1 && n.in[1] != nullptr && n.in[1]->shape.numel() > 1)
          rs.reject(n, "has one scale per row of the batch");
        break;
      case OP_NMS:
        if (!rs.carry(n.in[0]) || !rs.carry(n.in[1])) rs.reject(n, "has boxes or scores that do not depend on the batch");
        // (every image owns max_num_outputs rows of the result, and the image numbers written there
        //  start at the executing context's image_base: a half-batch copy gives the whole batch's rows)
        break;
      case OP_UNARY: case OP_POOL: case OP_CAST: case OP_RESHAPE: case OP_RESIZE: case OP_LRN:
        break;
      default:
        rs.reject(n, "is not known to keep the batch in the leading extent");
        break;
    }
    for (const _odla_value* o : {n.out, n.out2}) {
      if (o == nullptr) continue;
      if (!rs.scalable(o->shape.d[0])) rs.reject(n, "has a result whose leading extent is not a multiple of the batch");
      rs.carries[o->index] = 1;
    }
  }
  if (!rs.ok) return nullptr;

  auto d = std::make_unique<_odla_computation>();
  d->opts = c.opts;
  d->values.reserve(c.values.size());
  for (const auto& up : c.values) {
    auto v = std::make_unique<_odla_value>(*up);
    v->comp = d.get();
    if (rs.carries[v->index]) v->shape.d[0] = rs.scale(v->shape.d[0]);
    if (!v->name.empty()) d->by_name[v->name] = v.get();
    d->values.push_back(std::move(v));
  }
  auto map = [&](const _odla_value* v) -> _odla_value* { return v ? d->values[v->index].get() : nullptr; };
  d->nodes.reserve(c.nodes.size());
  for (size_t ni = 0; ni < c.nodes.size(); ++ni) {
    Node n = c.nodes[ni];
    n.absorbed = false;
    for (auto& v : n.in) v = map(v);
    n.out = map(n.out);
    n.out2 = map(n.out2);
    n.iv = new_iv[ni];
    d->nodes.push_back(std::move(n));
  }
  for (const _odla_value* v : c.args) d->args.push_back(map(v));
  for (const _odla_value* v : c.outputs) d->outputs.push_back(map(v));
  // constants made by the library stay owned by `c`, which outlives its copies
  return d;
}

}  // namespace ohip
