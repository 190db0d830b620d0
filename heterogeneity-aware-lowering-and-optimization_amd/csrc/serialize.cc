// Stored computations and executables.
//
// The reference's executable cache keeps a vendor engine (TensorRT plan files,
// ODLA/platforms/tensorrt/odla_tensorrt.cc:537-559,703-811 of the reference
// tree).  Compiling is cheap here (weights are packed and the arena planned in
// milliseconds when the first context is created), so what is worth storing is
// the recorded computation itself: values, constants (by value), nodes with
// their attributes, outputs, precision options and the quantisation table.  A
// loaded computation owns everything it needs and compiles like a recorded one.
//
// File layout (little endian): "ODLAHIP3", then the sections written by
// Writer below; every variable-length item is preceded by its 64-bit length;
// the last eight bytes are the FNV-1a hash of everything before them, so a
// truncated or damaged file is refused before any of it is interpreted.  What
// passes the hash is still checked record by record (validate_loaded): shapes,
// element types and, per operator, the operands and attributes the planner
// will index.
#include <cstdio>
#include <cstring>
#include <memory>
#include <string>
#include <vector>

#include "internal.h"

using namespace ohip;

namespace {

const char kMagic[8] = {'O', 'D', 'L', 'A', 'H', 'I', 'P', '3'};

uint64_t fnv1a(const uint8_t* p, size_t n) {
  uint64_t h = 1469598103934665603ull;
  for (size_t i = 0; i < n; ++i) { h ^= p[i]; h *= 1099511628211ull; }
  return h;
}

struct Writer {
  std::vector<uint8_t> buf;
  void raw(const void* p, size_t n) { const uint8_t* b = static_cast<const uint8_t*>(p); buf.insert(buf.end(), b, b + n); }
  void i64(int64_t v) { raw(&v, 8); }
  void f32(float v) { raw(&v, 4); }
  void str(const std::string& s) { i64((int64_t)s.size()); raw(s.data(), s.size()); }
};

struct Reader {
  const uint8_t* p;
  size_t n, pos = 0;
  bool ok = true;
  bool raw(void* dst, size_t len) {
    if (!ok || len > n - pos) { ok = false; return false; }
    memcpy(dst, p + pos, len);
    pos += len;
    return true;
  }
  int64_t i64() { int64_t v = 0; raw(&v, 8); return v; }
  float f32() { float v = 0; raw(&v, 4); return v; }
  std::string str() {
    const int64_t len = i64();
    if (!ok || len < 0 || (size_t)len > n - pos) { ok = false; return std::string(); }
    std::string s(reinterpret_cast<const char*>(p + pos), (size_t)len);
    pos += (size_t)len;
    return s;
  }
};

odla_status serialize(_odla_computation* c, std::vector<uint8_t>* out) {
  std::lock_guard<std::mutex> lk(c->mu);
  Writer w;
  w.raw(kMagic, 8);
  const Options& o = c->opts;
  w.i64(o.fp16); w.i64((int64_t)o.bf16); w.i64(o.int8); w.i64(o.raw_acc);
  w.i64(c->dynamic_batch); w.i64(c->min_batch); w.i64(c->max_batch); w.i64(c->opt_batch);
  w.i64(o.qtable != nullptr ? o.qtable_size : 0);
  for (int i = 0; o.qtable != nullptr && i < o.qtable_size; ++i) {
    const odla_value_quant_info& q = o.qtable[i];
    w.str(q.value_id ? reinterpret_cast<const char*>(q.value_id) : "");
    w.i64(q.ch_idx); w.f32(q.scale); w.f32(q.offset); w.f32(q.min); w.f32(q.max);
  }
  w.i64((int64_t)c->values.size());
  for (const auto& up : c->values) {
    const _odla_value& v = *up;
    w.i64((int64_t)v.kind); w.i64((int64_t)v.etype); w.i64(v.shape.rank);
    for (int i = 0; i < v.shape.rank; ++i) w.i64(v.shape.d[i]);
    w.str(v.name);
    w.i64(v.is_output); w.i64(v.eager); w.i64(v.producer); w.i64(v.dyn_batch);
    if (v.kind == _odla_value::CONSTANT) {
      const size_t bytes = (size_t)v.shape.numel() * (size_t)odla_type_size(v.etype);
      if (v.host_data == nullptr || bytes == 0) {
        OHIP_ERR("cannot store constant '%s': no data", v.name.c_str());
        return ODLA_FAILURE;
      }
      w.i64((int64_t)bytes);
      w.raw(v.host_data, bytes);
    }
  }
  auto idx_list = [&](const std::vector<_odla_value*>& vs) {
    w.i64((int64_t)vs.size());
    for (const _odla_value* v : vs) w.i64(v->index);
  };
  idx_list(c->args);
  idx_list(c->outputs);
  w.i64((int64_t)c->nodes.size());
  for (const Node& n : c->nodes) {
    w.i64((int64_t)n.op);
    w.i64((int64_t)n.in.size());
    for (const _odla_value* v : n.in) w.i64(v ? v->index : -1);
    w.i64(n.out ? n.out->index : -1);
    w.i64(n.out2 ? n.out2->index : -1);
    for (int i = 0; i < 24; ++i) w.i64(n.i[i]);
    for (int i = 0; i < 8; ++i) w.f32(n.f[i]);
    w.i64((int64_t)n.iv.size());
    for (int64_t v : n.iv) w.i64(v);
  }
  const uint64_t h = fnv1a(w.buf.data(), w.buf.size());
  w.raw(&h, 8);
  *out = std::move(w.buf);
  return ODLA_SUCCESS;
}

// ---------------------------------------------------------------------------
// What a node of each operator must look like for the planner to index it
// safely: operand slots (count and which may be empty), second result, the
// length of the integer list, attribute ranges.  Mirrors what the builders in
// api_ops.cc record.
struct OpRule {
  int min_in, max_in;   // operand slots
  unsigned required;    // bit k: slot k must hold a value
  bool out2;
};

bool op_rule(OpKind op, OpRule* r) {
  switch (op) {
    case OP_CONV: *r = {3, 3, 0x3, false}; return true;
    case OP_GEMM: *r = {3, 3, 0x3, false}; return true;
    case OP_BINARY: *r = {2, 2, 0x3, false}; return true;
    case OP_UNARY: *r = {1, 1, 0x1, false}; return true;
    case OP_BATCHNORM: *r = {5, 5, 0x7, false}; return true;
    case OP_LAYERNORM: *r = {3, 3, 0x1, false}; return true;
    case OP_POOL: *r = {1, 1, 0x1, false}; return true;
    case OP_REDUCE: *r = {1, 1, 0x1, false}; return true;
    case OP_SOFTMAX: *r = {1, 1, 0x1, false}; return true;
    case OP_CAST: *r = {1, 1, 0x1, false}; return true;
    case OP_CONCAT: *r = {1, ODLA_MAX_OUTPUTS, ~0u, false}; return true;
    case OP_GATHER: *r = {2, 2, 0x3, false}; return true;
    case OP_RESHAPE: *r = {1, 1, 0x1, false}; return true;
    case OP_RESIZE: *r = {1, 1, 0x1, false}; return true;
    case OP_SLICE: *r = {1, 1, 0x1, false}; return true;
    case OP_TRANSPOSE: *r = {1, 1, 0x1, false}; return true;
    case OP_QUANTIZE: case OP_DEQUANTIZE: *r = {3, 3, 0x3, false}; return true;
    case OP_NMS: *r = {2, 2, 0x3, false}; return true;
    case OP_EWISE: *r = {1, 3, ~0u, false}; return true;
    case OP_ARGEXT: *r = {1, 1, 0x1, false}; return true;
    case OP_COPYND: *r = {1, 1, 0x1, false}; return true;
    case OP_TOPK: *r = {1, 1, 0x1, true}; return true;
    case OP_LRN: *r = {1, 1, 0x1, false}; return true;
    case OP_ROWNORM: *r = {3, 3, 0x1, false}; return true;
    case OP_POSTPROCESS: *r = {5, 5, 0x1f, true}; return true;
    case OP_AXISOP: *r = {1, 2, ~0u, false}; return true;
  }
  return false;
}

#define LOADED_REQUIRE(cond, ...)                                   \
  do {                                                              \
    if (!(cond)) {                                                  \
      OHIP_ERR("stored computation rejected: " __VA_ARGS__);        \
      return ODLA_INVALID_PARAM;                                    \
    }                                                               \
  } while (0)

odla_status validate_loaded(const _odla_computation* c) {
  const int64_t nn = (int64_t)c->nodes.size();
  for (const auto& up : c->values) {
    const _odla_value& v = *up;
    LOADED_REQUIRE(dtype_from_odla(v.etype) != DT_INVALID, "value %d has element type %d", v.index, (int)v.etype);
    LOADED_REQUIRE(v.shape.rank >= 1, "value %d has rank %d", v.index, v.shape.rank);
    for (int i = 0; i < v.shape.rank; ++i)
      LOADED_REQUIRE(v.shape.d[i] > 0 && v.shape.d[i] < (1ll << 40), "value %d has extent %lld", v.index, (long long)v.shape.d[i]);
    LOADED_REQUIRE(v.shape.numel() < (1ll << 48), "value %d is implausibly large", v.index);
    if (v.kind == _odla_value::TEMP) {
      LOADED_REQUIRE(v.producer >= 0 && v.producer < nn, "value %d names producer %d", v.index, v.producer);
      const Node& p = c->nodes[(size_t)v.producer];
      LOADED_REQUIRE(p.out == &v || p.out2 == &v, "value %d is not a result of its producer", v.index);
    } else {
      LOADED_REQUIRE(v.producer == -1, "argument / constant %d has a producer", v.index);
    }
  }
  for (const _odla_value* v : c->args) LOADED_REQUIRE(v->kind == _odla_value::ARG, "argument list names value %d", v->index);
  for (int64_t k = 0; k < nn; ++k) {
    const Node& n = c->nodes[(size_t)k];
    OpRule r;
    LOADED_REQUIRE(op_rule(n.op, &r), "node %lld has operator %d", (long long)k, (int)n.op);
    const char* name = op_name(n.op);
    const int nin = (int)n.in.size();
    LOADED_REQUIRE(nin >= r.min_in && nin <= r.max_in, "%s node %lld has %d operand slots", name, (long long)k, nin);
    for (int i = 0; i < nin; ++i) {
      const _odla_value* v = n.in[(size_t)i];
      if (v == nullptr) {
        // (an operator that requires every slot says so with all bits set: that covers slots
        //  beyond the 32 the mask has a bit for - a Concat may have up to ODLA_MAX_OUTPUTS)
        const bool must = r.required == ~0u || (i < 32 && ((r.required >> i) & 1u));
        LOADED_REQUIRE(!must, "%s node %lld lacks operand %d", name, (long long)k, i);
        continue;
      }
      // operands are defined before their use
      LOADED_REQUIRE(v->kind != _odla_value::TEMP || v->producer < k, "%s node %lld uses value %d before it is computed",
                     name, (long long)k, v->index);
    }
    LOADED_REQUIRE(n.out != nullptr && n.out->kind == _odla_value::TEMP && n.out->producer == k,
                   "%s node %lld: result does not point back at it", name, (long long)k);
    LOADED_REQUIRE(!r.out2 || (n.out2 != nullptr && n.out2->kind == _odla_value::TEMP && n.out2->producer == k),
                   "%s node %lld lacks its second result", name, (long long)k);
    const _odla_value* x = n.in[0];
    const int xr = x->shape.rank, orank = n.out->shape.rank;
    const size_t niv = n.iv.size();
    switch (n.op) {
      case OP_CONV:
        LOADED_REQUIRE(xr == 4 && n.in[1]->shape.rank == 4 && orank == 4, "Conv node %lld: operands must have rank 4", (long long)k);
        LOADED_REQUIRE(n.i[1] >= 1 && n.i[3] >= 1 && n.i[4] >= 1 && n.i[5] >= 1 && n.i[6] >= 1 && n.i[7] >= 0 &&
                       n.i[8] >= 0 && n.i[9] >= 0 && n.i[10] >= 0, "Conv node %lld: bad stride / dilation / padding / group", (long long)k);
        LOADED_REQUIRE(n.i[0] >= ODLA_CHANNELS_FIRST && n.i[0] <= ODLA_CHANNELS_LAST && n.i[2] >= ODLA_SIO && n.i[2] <= ODLA_IOS,
                       "Conv node %lld: bad layout", (long long)k);
        break;
      case OP_GEMM:
        LOADED_REQUIRE(xr >= 2 && n.in[1]->shape.rank >= 2, "Gemm node %lld: operands must have rank >= 2", (long long)k);
        break;
      case OP_BINARY:
        LOADED_REQUIRE(n.i[0] >= BIN_ADD && n.i[0] <= BIN_MIN, "Binary node %lld: kind %lld", (long long)k, (long long)n.i[0]);
        LOADED_REQUIRE(niv >= 1 && n.iv[0] >= 1 && n.iv[0] <= ODLA_MAX_DIMENSION && niv == 1 + 2 * (size_t)n.iv[0] && n.iv[0] == orank,
                       "Binary node %lld: aligned shapes are malformed", (long long)k);
        for (size_t i = 1; i < niv; ++i) LOADED_REQUIRE(n.iv[i] >= 1, "Binary node %lld: aligned extent %lld", (long long)k, (long long)n.iv[i]);
        break;
      case OP_EWISE:
        LOADED_REQUIRE(niv >= 1 && n.iv[0] == orank && niv == 1 + (size_t)nin * (size_t)orank, "Elementwise node %lld: aligned shapes are malformed", (long long)k);
        for (size_t i = 1; i < niv; ++i) LOADED_REQUIRE(n.iv[i] >= 1, "Elementwise node %lld: aligned extent %lld", (long long)k, (long long)n.iv[i]);
        break;
      case OP_UNARY:
        LOADED_REQUIRE(n.i[0] >= ACT_NONE && n.i[0] <= ACT_DIV_CONST, "Unary node %lld: kind %lld", (long long)k, (long long)n.i[0]);
        break;
      case OP_LAYERNORM:
        LOADED_REQUIRE(n.i[0] >= 1 && n.i[0] <= xr, "LayerNorm node %lld: %lld axes", (long long)k, (long long)n.i[0]);
        break;
      case OP_POOL:
        LOADED_REQUIRE(xr == 4 && orank == 4, "Pool node %lld: operands must have rank 4", (long long)k);
        LOADED_REQUIRE(n.i[2] >= 1 && n.i[3] >= 1 && n.i[4] >= 1 && n.i[5] >= 1 && n.i[6] >= 0 && n.i[7] >= 0 && n.i[8] >= 0 && n.i[9] >= 0,
                       "Pool node %lld: bad window / stride / padding", (long long)k);
        break;
      case OP_REDUCE:
        LOADED_REQUIRE(niv >= 1 && niv <= (size_t)xr, "Reduce node %lld: %zu axes", (long long)k, niv);
        for (int64_t a : n.iv) LOADED_REQUIRE(a >= 0 && a < xr, "Reduce node %lld: axis %lld", (long long)k, (long long)a);
        break;
      case OP_SOFTMAX:
        LOADED_REQUIRE(n.i[0] >= -xr && n.i[0] < xr, "Softmax node %lld: axis %lld", (long long)k, (long long)n.i[0]);
        break;
      case OP_CONCAT:
        LOADED_REQUIRE(n.i[0] >= 0 && n.i[0] < xr, "Concat node %lld: axis %lld", (long long)k, (long long)n.i[0]);
        for (const _odla_value* v : n.in) LOADED_REQUIRE(v->shape.rank == xr, "Concat node %lld: operands of different rank", (long long)k);
        break;
      case OP_GATHER:
      case OP_ARGEXT:
        LOADED_REQUIRE(n.i[n.op == OP_ARGEXT ? 1 : 0] >= 0 && n.i[n.op == OP_ARGEXT ? 1 : 0] < xr, "%s node %lld: axis out of range", name, (long long)k);
        break;
      case OP_RESHAPE:
        LOADED_REQUIRE(x->shape.numel() == n.out->shape.numel(), "Reshape node %lld changes the element count", (long long)k);
        break;
      case OP_RESIZE:
        LOADED_REQUIRE(n.i[0] == ODLA_NEAREST || n.i[0] == ODLA_LINEAR, "Resize node %lld: interpolation %lld", (long long)k, (long long)n.i[0]);
        [[fallthrough]];
      case OP_LRN:
        LOADED_REQUIRE(xr == 4 && orank == 4, "%s node %lld: operands must have rank 4", name, (long long)k);
        break;
      case OP_SLICE:
        LOADED_REQUIRE(niv == 3 * (size_t)xr && orank == xr, "Slice node %lld: malformed bounds", (long long)k);
        for (int i = 0; i < xr; ++i)
          LOADED_REQUIRE(n.iv[i] >= 0 && n.iv[i] < n.iv[xr + i] && n.iv[xr + i] <= x->shape.d[i] && n.iv[2 * xr + i] >= 1,
                         "Slice node %lld: bounds outside the operand along dim %d", (long long)k, i);
        break;
      case OP_TRANSPOSE: {
        LOADED_REQUIRE(niv == (size_t)xr && orank == xr, "Transpose node %lld: malformed permutation", (long long)k);
        unsigned seen = 0;
        for (int64_t a : n.iv) {
          LOADED_REQUIRE(a >= 0 && a < xr && !((seen >> a) & 1u), "Transpose node %lld: not a permutation", (long long)k);
          seen |= 1u << a;
        }
        break;
      }
      case OP_QUANTIZE:
      case OP_DEQUANTIZE:
        LOADED_REQUIRE(n.i[0] >= -xr && n.i[0] < xr, "%s node %lld: axis %lld", name, (long long)k, (long long)n.i[0]);
        break;
      case OP_NMS:
        LOADED_REQUIRE(xr == 3 && n.in[1]->shape.rank == 3 && x->shape.d[2] == 4 && n.i[0] >= 0, "NMS node %lld: malformed operands", (long long)k);
        break;
      case OP_COPYND: {
        LOADED_REQUIRE(niv >= 1 && n.iv[0] >= 1 && n.iv[0] <= ODLA_MAX_DIMENSION && niv == 3 + 3 * (size_t)n.iv[0],
                       "CopyND node %lld: malformed extents", (long long)k);
        // every element the copy touches lies inside its operand / result
        const int r0 = (int)n.iv[0];
        int64_t xmax = n.iv[1 + 3 * r0], ymax = n.iv[2 + 3 * r0];
        LOADED_REQUIRE(xmax >= 0 && ymax >= 0, "CopyND node %lld: negative offset", (long long)k);
        for (int i = 0; i < r0; ++i) {
          const int64_t d = n.iv[1 + i], sx = n.iv[1 + r0 + i], sy = n.iv[1 + 2 * r0 + i];
          LOADED_REQUIRE(d >= 1 && d < (1ll << 40) && sx >= 0 && sy >= 0 && sx < (1ll << 40) && sy < (1ll << 40),
                         "CopyND node %lld: bad extent or stride", (long long)k);
          xmax += (d - 1) * sx;
          ymax += (d - 1) * sy;
        }
        LOADED_REQUIRE(xmax < x->shape.numel() && ymax < n.out->shape.numel(), "CopyND node %lld reaches outside its tensors", (long long)k);
        break;
      }
      case OP_AXISOP: {
        LOADED_REQUIRE(n.i[0] >= AX_GATHER_ELEMENTS && n.i[0] <= AX_COMPRESS, "AxisOp node %lld: kind %lld", (long long)k, (long long)n.i[0]);
        LOADED_REQUIRE(n.i[1] >= 0 && n.i[1] < xr, "AxisOp node %lld: axis out of range", (long long)k);
        const bool two = n.i[0] == AX_GATHER_ELEMENTS || n.i[0] == AX_COMPRESS;
        LOADED_REQUIRE(n.in.size() == (two ? 2u : 1u), "AxisOp node %lld: %zu operands", (long long)k, n.in.size());
        if (n.i[0] == AX_GATHER_ELEMENTS) {
          const Shape& is = n.in[1]->shape;
          LOADED_REQUIRE(is.rank == xr && n.out->shape == is, "GatherElements node %lld: malformed indices", (long long)k);
          for (int i = 0; i < xr; ++i)
            LOADED_REQUIRE(i == n.i[1] || is.d[i] == x->shape.d[i] || ((i == 0 || i == n.i[1] + 1) && is.d[i] <= x->shape.d[i]),
                           "GatherElements node %lld: indices exceed the operand", (long long)k);
        } else if (n.i[0] == AX_COMPRESS) {
          const int64_t lim = n.i[3] ? std::min(x->shape.numel(), n.out->shape.numel()) : x->shape.d[n.i[1]];
          LOADED_REQUIRE(n.in[1]->shape.rank == 1 && n.i[2] >= 0 && n.i[2] <= n.in[1]->shape.d[0] && n.i[2] <= lim,
                         "Compress node %lld: malformed condition", (long long)k);
          if (!n.i[3]) {
            int64_t rest = 1;
            for (int i = 0; i < xr; ++i) if (i != n.i[1]) rest *= x->shape.d[i];
            LOADED_REQUIRE(rest * n.i[2] <= n.out->shape.numel(), "Compress node %lld: result too small", (long long)k);
          } else {
            LOADED_REQUIRE(n.i[1] == 0, "Compress node %lld: flat form with an axis", (long long)k);
          }
        } else {
          LOADED_REQUIRE(n.out->shape == x->shape, "AxisOp node %lld: result shape differs from the operand's", (long long)k);
        }
        break;
      }
      case OP_TOPK:
        LOADED_REQUIRE(n.i[2] >= 0 && n.i[2] < xr && n.i[0] >= 1 && n.i[0] <= x->shape.d[n.i[2]], "TopK node %lld: bad axis or K", (long long)k);
        break;
      default:
        break;
    }
  }
  for (const _odla_value* v : c->outputs) LOADED_REQUIRE(v != nullptr, "output list names a missing value");
  return ODLA_SUCCESS;
}

odla_status deserialize(const uint8_t* data, size_t size, _odla_computation* c) {
  if (size < 16 || data == nullptr || memcmp(data, kMagic, 8) != 0) {
    OHIP_ERR("not a stored computation of this library version (bad signature)");
    return ODLA_INVALID_PARAM;
  }
  uint64_t stored = 0;
  memcpy(&stored, data + size - 8, 8);
  if (stored != fnv1a(data, size - 8)) {
    OHIP_ERR("stored computation is truncated or damaged (hash mismatch)");
    return ODLA_INVALID_PARAM;
  }
  size -= 8;
  Reader r{data, size};
  char magic[8];
  r.raw(magic, 8);
  Options& o = c->opts;
  o.fp16 = r.i64() != 0; o.bf16 = (odla_bf16_mode)r.i64(); o.int8 = r.i64() != 0; o.raw_acc = r.i64() != 0;
  c->dynamic_batch = r.i64() != 0;
  c->min_batch = (int)r.i64(); c->max_batch = (int)r.i64(); c->opt_batch = (int)r.i64();
  if (!r.ok || c->min_batch < 0 || c->max_batch < 0 || c->opt_batch < 0) return ODLA_INVALID_PARAM;
  const int64_t nq = r.i64();
  if (!r.ok || nq < 0 || nq > (1 << 24)) return ODLA_INVALID_PARAM;
  c->owned_qnames.reserve((size_t)nq);
  for (int64_t i = 0; i < nq; ++i) {
    c->owned_qnames.push_back(r.str());
    odla_value_quant_info q;
    memset(&q, 0, sizeof(q));
    q.ch_idx = (int)r.i64(); q.scale = r.f32(); q.offset = r.f32(); q.min = r.f32(); q.max = r.f32();
    c->owned_qtable.push_back(q);
  }
  for (size_t i = 0; i < c->owned_qtable.size(); ++i)  // the strings no longer move
    c->owned_qtable[i].value_id = reinterpret_cast<odla_value_id>(const_cast<char*>(c->owned_qnames[i].c_str()));
  if (nq > 0) { o.qtable = c->owned_qtable.data(); o.qtable_size = (int)nq; }

  const int64_t nv = r.i64();
  if (!r.ok || nv < 0 || nv > (1 << 24)) return ODLA_INVALID_PARAM;
  for (int64_t k = 0; k < nv; ++k) {
    const int64_t kind = r.i64(), et = r.i64(), rank = r.i64();
    if (!r.ok || rank < 0 || rank > ODLA_MAX_DIMENSION || kind < 0 || kind > 2) return ODLA_INVALID_PARAM;
    if (et < 0 || et > (int64_t)ODLA_STRING) {   // checked before the number becomes an enumerator
      OHIP_ERR("stored computation rejected: value %lld has element type %lld", (long long)k, (long long)et);
      return ODLA_INVALID_PARAM;
    }
    Shape s;
    s.rank = (int)rank;
    for (int i = 0; i < s.rank; ++i) s.d[i] = r.i64();
    const std::string name = r.str();
    _odla_value* v = new_value(c, (_odla_value::Kind)kind, (odla_element_type)et, s,
                               name.empty() ? nullptr : reinterpret_cast<odla_value_id>(const_cast<char*>(name.c_str())));
    v->is_output = r.i64() != 0;
    v->eager = r.i64() != 0;
    v->producer = (int)r.i64();
    v->dyn_batch = r.i64() != 0;
    if (v->kind == _odla_value::CONSTANT) {
      const int64_t bytes = r.i64();
      if (!r.ok || bytes <= 0 || (size_t)bytes > r.n - r.pos ||
          (size_t)bytes != (size_t)s.numel() * (size_t)odla_type_size(v->etype))
        return ODLA_INVALID_PARAM;
      auto buf = std::make_unique<std::vector<uint8_t>>((size_t)bytes);
      r.raw(buf->data(), (size_t)bytes);
      v->host_data = buf->data();
      c->owned_data.push_back(std::move(buf));
    }
  }
  auto value_at = [&](int64_t i) -> _odla_value* {
    if (i < 0 || i >= (int64_t)c->values.size()) { r.ok = false; return nullptr; }
    return c->values[(size_t)i].get();
  };
  auto idx_list = [&](std::vector<_odla_value*>* vs) {
    const int64_t n = r.i64();
    if (!r.ok || n < 0 || n > nv) { r.ok = false; return; }
    for (int64_t i = 0; i < n; ++i) vs->push_back(value_at(r.i64()));
  };
  idx_list(&c->args);
  idx_list(&c->outputs);
  const int64_t nn = r.i64();
  if (!r.ok || nn < 0 || nn > (1 << 24)) return ODLA_INVALID_PARAM;
  for (int64_t k = 0; k < nn; ++k) {
    Node n;
    const int64_t op = r.i64();
    if (op < 0 || op > (int64_t)OP_AXISOP) return ODLA_INVALID_PARAM;
    n.op = (OpKind)op;
    const int64_t nin = r.i64();
    if (!r.ok || nin < 0 || nin > ODLA_MAX_OUTPUTS) return ODLA_INVALID_PARAM;
    for (int64_t i = 0; i < nin; ++i) {
      const int64_t vi = r.i64();
      n.in.push_back(vi < 0 ? nullptr : value_at(vi));
    }
    const int64_t oi = r.i64(), o2 = r.i64();
    n.out = oi < 0 ? nullptr : value_at(oi);
    n.out2 = o2 < 0 ? nullptr : value_at(o2);
    for (int i = 0; i < 24; ++i) n.i[i] = r.i64();
    for (int i = 0; i < 8; ++i) n.f[i] = r.f32();
    const int64_t niv = r.i64();
    if (!r.ok || niv < 0 || (size_t)niv > (r.n - r.pos) / 8) return ODLA_INVALID_PARAM;
    for (int64_t i = 0; i < niv; ++i) n.iv.push_back(r.i64());
    if (!r.ok || n.out == nullptr) return ODLA_INVALID_PARAM;
    c->nodes.push_back(std::move(n));
  }
  if (!r.ok || r.pos != r.n) {
    OHIP_ERR("stored computation is truncated or corrupt");
    return ODLA_INVALID_PARAM;
  }
  return validate_loaded(c);
}

odla_status write_location(const odla_resource_location& loc, const std::vector<uint8_t>& bytes) {
  if (loc.location_type != ODLA_LOCATION_PATH || loc.location == nullptr) {
    OHIP_ERR("only ODLA_LOCATION_PATH can be written");
    return ODLA_INVALID_PARAM;
  }
  FILE* f = fopen(static_cast<const char*>(loc.location), "wb");
  if (f == nullptr) {
    OHIP_ERR("cannot open '%s' for writing", static_cast<const char*>(loc.location));
    return ODLA_FILE_NOT_EXIST;
  }
  const bool good = fwrite(bytes.data(), 1, bytes.size(), f) == bytes.size();
  return (fclose(f) == 0 && good) ? ODLA_SUCCESS : ODLA_FAILURE;
}

odla_status read_location(const odla_resource_location& loc, std::vector<uint8_t>* bytes, const uint8_t** data, size_t* size) {
  if (loc.location == nullptr) return ODLA_INVALID_PARAM;
  if (loc.location_type == ODLA_LOCATION_MEMORY) {
    *data = static_cast<const uint8_t*>(loc.location);
    *size = loc.size;
    return ODLA_SUCCESS;
  }
  if (loc.location_type != ODLA_LOCATION_PATH) return ODLA_INVALID_PARAM;
  FILE* f = fopen(static_cast<const char*>(loc.location), "rb");
  if (f == nullptr) {
    OHIP_ERR("cannot open '%s'", static_cast<const char*>(loc.location));
    return ODLA_FILE_NOT_EXIST;
  }
  fseek(f, 0, SEEK_END);
  const long len = ftell(f);
  fseek(f, 0, SEEK_SET);
  if (len < 0) { fclose(f); return ODLA_FAILURE; }
  bytes->resize((size_t)len);
  const bool good = fread(bytes->data(), 1, (size_t)len, f) == (size_t)len;
  fclose(f);
  if (!good) return ODLA_FAILURE;
  *data = bytes->data();
  *size = bytes->size();
  return ODLA_SUCCESS;
}

}  // namespace

extern "C" {

odla_status odla_StoreComputation(odla_resource_location location, odla_computation computation) {
  if (computation == nullptr) return ODLA_INVALID_PARAM;
  std::vector<uint8_t> bytes;
  odla_status st = serialize(computation, &bytes);
  if (st != ODLA_SUCCESS) return st;
  return write_location(location, bytes);
}

odla_status odla_LoadComputation(odla_resource_location location, odla_computation* computation) {
  if (computation == nullptr) return ODLA_INVALID_PARAM;
  *computation = nullptr;
  std::vector<uint8_t> owned;
  const uint8_t* data = nullptr;
  size_t size = 0;
  odla_status st = read_location(location, &owned, &data, &size);
  if (st != ODLA_SUCCESS) return st;
  odla_computation c = nullptr;
  st = odla_CreateComputation(&c);  // becomes the calling thread's current computation
  if (st != ODLA_SUCCESS) return st;
  st = deserialize(data, size, c);
  if (st != ODLA_SUCCESS) {
    (void)odla_DestroyComputation(c);
    return st;
  }
  *computation = c;
  return ODLA_SUCCESS;
}

odla_status odla_CompileComputation(const odla_computation computation, const odla_device device,
                                    odla_executable* executable) {
  (void)device;
  if (computation == nullptr || executable == nullptr) return ODLA_INVALID_PARAM;
  *executable = nullptr;
  odla_status st = ohip::compile_computation(computation);
  if (st != ODLA_SUCCESS) return st;
  computation->executable.comp = computation;
  *executable = &computation->executable;
  return ODLA_SUCCESS;
}

odla_status odla_StoreExecutable(odla_resource_location location, odla_executable executable) {
  if (executable == nullptr || executable->comp == nullptr) return ODLA_INVALID_PARAM;
  return odla_StoreComputation(location, executable->comp);
}

odla_status odla_LoadExecutable(odla_resource_location location, odla_device device, odla_executable* executable) {
  (void)device;
  if (executable == nullptr) return ODLA_INVALID_PARAM;
  *executable = nullptr;
  odla_computation c = nullptr;
  odla_status st = odla_LoadComputation(location, &c);
  if (st != ODLA_SUCCESS) return st;
  c->executable.comp = c;
  c->executable.owns = true;
  *executable = &c->executable;
  return ODLA_SUCCESS;
}

odla_status odla_LaunchExecutable(odla_executable executable, odla_context context) {
  if (executable == nullptr || executable->comp == nullptr || context == nullptr) return ODLA_INVALID_PARAM;
  return odla_ExecuteComputation(executable->comp, context, ODLA_COMPUTE_INFERENCE, nullptr);
}

odla_status odla_GetNumOfArgsFromExecutable(const odla_executable executable, odla_uint32* num_args) {
  if (executable == nullptr) return ODLA_INVALID_PARAM;
  return odla_GetNumOfArgsFromComputation(executable->comp, num_args);
}
odla_status odla_GetArgFromExecutableByIdx(const odla_executable executable, const odla_uint32 arg_idx,
                                           odla_value* arg_value) {
  if (executable == nullptr) return ODLA_INVALID_PARAM;
  return odla_GetArgFromComputationByIdx(executable->comp, arg_idx, arg_value);
}
odla_status odla_GetNumOfOutputsFromExecutable(const odla_executable executable, odla_uint32* num_outputs) {
  if (executable == nullptr) return ODLA_INVALID_PARAM;
  return odla_GetNumOfOutputsFromComputation(executable->comp, num_outputs);
}
odla_status odla_GetOutputFromExecutableByIdx(const odla_executable executable, const odla_uint32 output_idx,
                                              odla_value* output_value) {
  if (executable == nullptr) return ODLA_INVALID_PARAM;
  return odla_GetOutputFromComputationByIdx(executable->comp, output_idx, output_value);
}

odla_status odla_DestroyExecutable(odla_executable executable) {
  if (executable == nullptr) return ODLA_INVALID_PARAM;
  if (executable->owns && executable->comp != nullptr) return odla_DestroyComputation(executable->comp);
  return ODLA_SUCCESS;  // an executable compiled from a caller's computation lives and dies with it
}

}  // extern "C"
