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
// File layout (little endian): "ODLAHIP1", then the sections written by
// Writer below; every variable-length item is preceded by its 64-bit length.
#include <cstdio>
#include <cstring>
#include <memory>
#include <string>
#include <vector>

#include "internal.h"

using namespace ohip;

namespace {

const char kMagic[8] = {'O', 'D', 'L', 'A', 'H', 'I', 'P', '2'};

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
  *out = std::move(w.buf);
  return ODLA_SUCCESS;
}

odla_status deserialize(const uint8_t* data, size_t size, _odla_computation* c) {
  Reader r{data, size};
  char magic[8];
  if (!r.raw(magic, 8) || memcmp(magic, kMagic, 8) != 0) {
    OHIP_ERR("not a stored computation (bad signature)");
    return ODLA_INVALID_PARAM;
  }
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
    if (op < 0 || op > (int64_t)OP_POSTPROCESS) return ODLA_INVALID_PARAM;
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
  if (!r.ok) {
    OHIP_ERR("stored computation is truncated or corrupt");
    return ODLA_INVALID_PARAM;
  }
  return ODLA_SUCCESS;
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
