// Graph -> plan compiler of libodla_hip.so.
//
// build_plan() walks the recorded nodes once and lowers them to kernel launch
// steps over physical device tensors:
//   * storage type: FLOAT32 graph values are kept as fp32, or as fp16 / bf16
//     when ODLA_FP16_MODE / ODLA_BF16_MODE is set (fp32 accumulate in every
//     kernel); in the int8 plan values with a quant-table entry are kept as
//     8-bit levels;
//   * layout: rank-4 values flowing through Conv / Pool / Resize live
//     channels-last on the device, everything else row-major; conversions are
//     inserted where a consumer needs the other form and cached per value;
//   * fusion: per-channel Add / Mul / BatchNorm after a Conv or Gemm fold into
//     its weights and bias, a same-shape residual Add and a trailing activation
//     fold into its epilogue;
//   * memory: constants are packed once into one device pool; temporaries get
//     offsets in one arena by liveness (first fit over step intervals).
#include <algorithm>
#include <cmath>
#include <cstring>
#include <unordered_set>

#include "internal.h"

namespace ohip {
namespace {

constexpr size_t kAlign = 256;
constexpr int kUnset = 1 << 30;  // PTensor::def_step before any step touched the tensor
// Convolution results of at least this size are written with non-temporal stores
// (the chip's last-level cache holds 256 MiB); ODLA_HIP_STREAM_OUT_MB overrides it.
size_t stream_out_bytes() {
  static const size_t v = [] {
    const char* e = getenv("ODLA_HIP_STREAM_OUT_MB");
    return (size_t)(e != nullptr ? atol(e) : 150) << 20;
  }();
  return v;
}
size_t align_up(size_t v, size_t a = kAlign) { return (v + a - 1) / a * a; }
int round_up_i(int v, int a) { return (v + a - 1) / a * a; }

float half_bits_to_float(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1f, man = h & 0x3ffu, u;
  if (exp == 0) {
    if (man == 0) u = sign;
    else {
      exp = 127 - 15 + 1;
      while ((man & 0x400u) == 0) { man <<= 1; --exp; }
      man &= 0x3ffu;
      u = sign | (exp << 23) | (man << 13);
    }
  } else if (exp == 31) u = sign | 0x7f800000u | (man << 13);
  else u = sign | ((exp + 127 - 15) << 23) | (man << 13);
  float f;
  memcpy(&f, &u, 4);
  return f;
}

struct PlanError {
  odla_status status;
  std::string msg;
};
[[noreturn]] void fail(odla_status st, const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  throw PlanError{st, buf};
}

// FORM_OPERAND: the 16-bit copy a Conv / Gemm reads under BF16_ACCURACY_MODE, where values
// are stored as fp32; in every other mode it is the same thing as FORM_FLOAT.
enum Form { FORM_FLOAT = 0, FORM_QUANT = 1, FORM_OPERAND = 2 };

struct VState {
  int slot[2][3] = {{-1, -1, -1}, {-1, -1, -1}};  // [layout][form] -> tensor id
  int main = -1;
};

// Epilogue collected while fusing followers into a Conv / Gemm.
struct Epilogue {
  std::vector<float> row_scale;  // per output channel multiplier folded into weights
  float scalar = 1.f;            // uniform multiplier applied to the accumulator (kernel alpha)
  std::vector<float> bias;       // per output channel
  bool has_bias = false;
  _odla_value* residual = nullptr;
  ActKind act = ACT_NONE;
  float act_a = 0.f, act_b = 0.f;
  _odla_value* pre_residual_value = nullptr;  // value right before the residual Add
  bool res_after_act = false;                 // the residual joins behind the activation
  _odla_value* final_value = nullptr;
};

class Planner {
 public:
  Planner(_odla_computation* c, Plan* p) : comp_(c), plan_(p) {}
  void run();

 private:
  _odla_computation* comp_;
  Plan* plan_;
  std::vector<VState> vs_;
  std::vector<std::vector<int>> consumers_;  // value index -> node indices
  std::unordered_map<std::string, QuantEntry> qmap_;
  DType cdt_ = DT_F32;     // storage type of FLOAT32 graph values
  DType op_dt_ = DT_F32;   // type in which Conv / Gemm read their operands
  // BF16_ACCURACY_MODE [ref: ODLA/include/ODLA/odla_compute.h:72-78; odla_dnnl.cc:1024-1026,
  // 1780-1802]: values stay fp32, only the operands of Conv / Gemm are rounded to bf16.
  bool acc_mode_ = false;
  std::vector<signed char> operand_only_;   // per value, memo of operand_only(): -1 unknown
  bool in_init_ = false;

  // ---------------------------------------------------------------- tensors
  int new_tensor(DType dt, Layout layout, const Shape& shape, int cs, Space space) {
    PTensor t;
    t.dt = dt;
    t.layout = layout;
    t.shape = shape;
    t.cs = cs;
    t.space = space;
    t.bytes = (size_t)t.phys_elems() * dtype_size(dt);
    t.def_step = kUnset;
    t.last_step = -1;
    if (space == SP_CONST) { t.offset = plan_->const_bytes; plan_->const_bytes += align_up(t.bytes); }
    if (space == SP_INIT) { t.offset = plan_->init_bytes; plan_->init_bytes += align_up(t.bytes); }
    plan_->tensors.push_back(t);
    return (int)plan_->tensors.size() - 1;
  }
  int raw_buffer(size_t bytes, Space space) {
    Shape s;
    s.rank = 1;
    s.d[0] = (int64_t)bytes;
    return new_tensor(DT_U8, L_ROWMAJOR, s, 0, space);
  }
  int alias_tensor(int src, const Shape& shape) {
    PTensor t = plan_->tensors[src];
    t.shape = shape;
    t.layout = L_ROWMAJOR;
    t.cs = 0;
    t.alias_of = root(src);
    plan_->tensors.push_back(t);
    return (int)plan_->tensors.size() - 1;
  }
  // a dense row-major view of `shape` that starts `byte_off` bytes into `src`
  int view_tensor(int src, const Shape& shape, size_t byte_off) {
    PTensor t = plan_->tensors[src];
    t.shape = shape;
    t.layout = L_ROWMAJOR;
    t.cs = 0;
    t.alias_of = root(src);
    t.alias_off = plan_->tensors[src].alias_off + byte_off;
    t.bytes = (size_t)shape.numel() * dtype_size(t.dt);
    plan_->tensors.push_back(t);
    return (int)plan_->tensors.size() - 1;
  }
  std::unordered_set<int> arena_only_;   // root tensors that some step writes, or reads relying on the arena
  // The 8-bit convolution steps, kept so that a plain 1x1 layer over the result of one can ride in
  // its launch (lower_conv; igemm_stream_q8_fusable decides).
  struct FuseProducer {
    int step = -1;
    const _odla_value* out = nullptr;
    IgemmParams ip;
    int tx = -1, tw = -1, ty = -1, tb = -1, tm = -1, tr = -1, tf = -1;
  };
  std::unordered_map<const _odla_value*, FuseProducer> fuse_prods_;   // by result value
  int root(int t) const {
    while (plan_->tensors[t].alias_of >= 0) t = plan_->tensors[t].alias_of;
    return t;
  }
  PTensor& T(int t) { return plan_->tensors[t]; }

  // pointer resolution inside steps
  struct Ref {
    const Plan* plan;
    int t;
    char* operator()(const ExecEnv& env) const {
      int r = t;
      while (plan->tensors[r].alias_of >= 0) r = plan->tensors[r].alias_of;
      const PTensor& pt = plan->tensors[r];
      if (pt.ext_slot >= 0 && env.ext != nullptr && env.ext[pt.ext_slot] != nullptr)
        return const_cast<char*>(env.ext[pt.ext_slot]) + plan->tensors[t].alias_off;
      return env.base[pt.space] + pt.offset + plan->tensors[t].alias_off;  // (alias offsets are relative to the root)
    }
  };
  Ref ref(int t) const { return Ref{plan_, t}; }

  // exact_reader: the launch reads exactly the elements of its sources and tests their alignment
  // itself (the layout conversions launch_nchw_to_nhwc / launch_nchw_to_s2d do), so a source that
  // is an argument's staging tensor may be the caller's own device buffer.  Every other reader
  // may rely on the arena (256-byte bases, slack behind a tensor) and pins its sources to it.
  void emit(const std::string& name, std::initializer_list<int> reads, std::initializer_list<int> writes,
            std::function<hipError_t(const ExecEnv&, hipStream_t)> fn, bool exact_reader = false) {
    emit_lists(name, std::vector<int>(reads), std::vector<int>(writes), std::move(fn), exact_reader);
  }
  void emit_lists(const std::string& name, const std::vector<int>& reads, const std::vector<int>& writes,
                  std::function<hipError_t(const ExecEnv&, hipStream_t)> fn, bool exact_reader = false) {
    if (in_init_) {
      plan_->init_steps.push_back({name, std::move(fn)});
      return;
    }
    const int idx = (int)plan_->steps.size();
    auto touch = [&](int t) {
      if (t < 0) return;
      PTensor& p = T(root(t));
      if (p.space != SP_ARENA) return;
      if (idx < p.def_step) p.def_step = idx;
      if (idx > p.last_step) p.last_step = idx;
    };
    for (int t : reads) touch(t);
    for (int t : writes) touch(t);
    for (int t : reads) if (t >= 0 && !exact_reader) arena_only_.insert(root(t));
    for (int t : writes) if (t >= 0) arena_only_.insert(root(t));
    plan_->steps.push_back({name, std::move(fn)});
  }

  // -------------------------------------------------------------- constants
  size_t add_blob(Space space, size_t offset, const void* src, size_t bytes, std::vector<uint8_t>* owned) {
    Plan::Blob b;
    b.space = space;
    b.offset = offset;
    b.bytes = bytes;
    if (owned) { b.owned = std::move(*owned); b.src = nullptr; } else b.src = src;
    plan_->blobs.push_back(std::move(b));
    return offset;
  }
  // device tensor in the constant pool holding `bytes` of host data
  int const_from_host(DType dt, const Shape& shape, const void* src, std::vector<uint8_t>* owned) {
    const int t = new_tensor(dt, L_ROWMAJOR, shape, 0, SP_CONST);
    add_blob(SP_CONST, T(t).offset, src, T(t).bytes, owned);
    return t;
  }
  template <typename E>
  int const_vector(DType dt, const std::vector<E>& v) {
    Shape s;
    s.rank = 1;
    s.d[0] = (int64_t)v.size();
    std::vector<uint8_t> raw(v.size() * sizeof(E));
    memcpy(raw.data(), v.data(), raw.size());
    return const_from_host(dt, s, nullptr, &raw);
  }

  std::vector<float> const_as_float(const _odla_value* v) {
    if (v->kind != _odla_value::CONSTANT || v->host_data == nullptr) fail(ODLA_INVALID_PARAM, "value '%s' is not a constant", v->name.c_str());
    const int64_t n = v->shape.numel();
    std::vector<float> out((size_t)n);
    switch (dtype_from_odla(v->etype)) {
      case DT_F32: memcpy(out.data(), v->host_data, (size_t)n * 4); break;
      case DT_F16: for (int64_t i = 0; i < n; ++i) out[i] = half_bits_to_float(((const uint16_t*)v->host_data)[i]); break;
      case DT_BF16: for (int64_t i = 0; i < n; ++i) { uint32_t u = (uint32_t)((const uint16_t*)v->host_data)[i] << 16; memcpy(&out[i], &u, 4); } break;
      case DT_I32: for (int64_t i = 0; i < n; ++i) out[i] = (float)((const int32_t*)v->host_data)[i]; break;
      case DT_I64: for (int64_t i = 0; i < n; ++i) out[i] = (float)((const int64_t*)v->host_data)[i]; break;
      case DT_I8: for (int64_t i = 0; i < n; ++i) out[i] = (float)((const int8_t*)v->host_data)[i]; break;
      case DT_U8: for (int64_t i = 0; i < n; ++i) out[i] = (float)((const uint8_t*)v->host_data)[i]; break;
      default: fail(ODLA_UNSUPPORTED_DATATYPE, "constant '%s' has an unsupported element type", v->name.c_str());
    }
    return out;
  }

  // ------------------------------------------------------------- dtype rules
  DType storage_dtype(const _odla_value* v) const {
    const DType d = dtype_from_odla(v->etype);
    if (d == DT_F32) return cdt_;
    return d;
  }
  // Type of the tensor a Conv / Gemm reads for a FLOAT32 operand.
  DType mm_dtype(const _odla_value* v) const {
    const DType d = dtype_from_odla(v->etype);
    return d == DT_F32 ? op_dt_ : d;
  }
  // Every reader of `v` is a Conv / Gemm operand slot (through Reshape / Transpose, which move
  // bits): storing it in the operand type loses nothing that the readers would keep.
  bool operand_only(const _odla_value* v) {
    if (v == nullptr || v->is_output || consumers_[v->index].empty()) return false;
    signed char& memo = operand_only_[v->index];
    if (memo >= 0) return memo != 0;
    bool all = true;
    for (int ci : consumers_[v->index]) {
      const Node& c = comp_->nodes[ci];
      if (c.op == OP_GEMM || c.op == OP_CONV) {
        const bool as_operand = c.in[0] == v || c.in[1] == v;
        const bool as_addend = c.in.size() > 2 && c.in[2] == v;
        all = all && as_operand && !as_addend;
      } else if (c.op == OP_RESHAPE || c.op == OP_TRANSPOSE) {
        all = all && operand_only(c.out);
      } else {
        all = false;
      }
      if (!all) break;
    }
    operand_only_[v->index] = all ? 1 : 0;
    return all;
  }
  // Storage type of what a Conv / Gemm / Softmax launch writes for the FLOAT32 value `v`.
  DType result_dtype(const _odla_value* v) {
    const DType d = dtype_from_odla(v->etype);
    if (d != DT_F32) return d;
    if (acc_mode_) return operand_only(v) ? op_dt_ : DT_F32;
    return cdt_;
  }
  // `v` in the given layout as some float tensor, preferring what exists: data movement
  // (Reshape, Transpose, Slice, Concat) keeps whatever type its source is stored in.
  int get_moved(const _odla_value* v, Layout want) {
    const VState& s = vs_[v->index];
    const bool narrow = acc_mode_ && dtype_from_odla(v->etype) == DT_F32 && s.main >= 0 && !T(s.main).quant &&
                        T(s.main).dt == op_dt_ && s.slot[want][FORM_FLOAT] < 0;
    return get(v, want, narrow ? FORM_OPERAND : FORM_FLOAT);
  }
  const QuantEntry* qentry(const _odla_value* v) const {
    if (!comp_->opts.int8 || v == nullptr || v->name.empty()) return nullptr;
    if (dtype_from_odla(v->etype) != DT_F32) return nullptr;
    auto it = qmap_.find(v->name);
    return it == qmap_.end() ? nullptr : &it->second;
  }

  // --------------------------------------------------- value -> device tensor
  // Returns a tensor holding `v` in the requested layout and form, inserting
  // (and caching) a conversion step when the value lives in another one.
  // `cvec` > 0 asks for a channels-last pitch that is a multiple of cvec.
  int get(const _odla_value* v, Layout want, Form form = FORM_FLOAT, int cvec = 0) {
    if (form == FORM_OPERAND && (!acc_mode_ || dtype_from_odla(v->etype) != DT_F32)) form = FORM_FLOAT;
    VState& s = vs_[v->index];
    if (s.main < 0) materialize_source(v);
    if (want == L_NHWC && v->shape.rank != 4) fail(ODLA_INTERNAL_LOGIC_ERR, "channels-last form requested for rank-%d value", v->shape.rank);
    int& slot = s.slot[want][form];
    if (slot >= 0 && (want != L_NHWC || cvec <= 1 || T(slot).cs % cvec == 0)) return slot;
    const int have = pick_source(s, want, form);
    const int made = convert(v, have, want, form, cvec);
    slot = made;
    return made;
  }

  int pick_source(const VState& s, Layout want, Form form) const {
    // prefer same form, then same layout, then main
    if (s.slot[want][form] >= 0) return s.slot[want][form];
    if (s.slot[1 - want][form] >= 0) return s.slot[1 - want][form];
    for (int f = 0; f < 3; ++f)
      if (f != form && s.slot[want][f] >= 0) return s.slot[want][f];
    return s.main;
  }

  void set_main(const _odla_value* v, int t) {
    VState& s = vs_[v->index];
    s.main = t;
    const PTensor p = T(t);  // by value: the tensor table may grow below
    const int form = p.quant ? FORM_QUANT
                             : (acc_mode_ && p.dt == op_dt_ && dtype_from_odla(v->etype) == DT_F32 ? FORM_OPERAND : FORM_FLOAT);
    s.slot[p.layout][form] = t;
    // a channels-last tensor with one pixel (or one channel) and no padding is
    // also a valid row-major tensor, and vice versa
    if (p.shape.rank == 4) {
      const bool trivial = (p.shape.d[2] * p.shape.d[3] == 1) || (p.shape.d[1] == 1);
      if (trivial && (p.layout == L_ROWMAJOR || p.cs == p.shape.d[1])) {
        const int other = 1 - (int)p.layout;
        if (s.slot[other][form] < 0) {
          PTensor a = p;
          a.alias_of = root(t);
          a.layout = (Layout)other;
          a.cs = other == L_NHWC ? (int)p.shape.d[1] : 0;
          plan_->tensors.push_back(a);
          s.slot[other][form] = (int)plan_->tensors.size() - 1;
        }
      }
    }
  }

  // Arguments and constants enter the plan in their declared type, row-major.
  void materialize_source(const _odla_value* v) {
    if (v->kind == _odla_value::ARG) {
      fail(ODLA_INTERNAL_LOGIC_ERR, "argument '%s' was not staged", v->name.c_str());
    } else if (v->kind == _odla_value::CONSTANT) {
      const DType src = dtype_from_odla(v->etype);
      const DType dst = storage_dtype(v);
      int t;
      if (src == dst) {
        t = const_from_host(src, v->shape, v->host_data, nullptr);
      } else {
        const int raw = new_tensor(src, L_ROWMAJOR, v->shape, 0, SP_INIT);
        add_blob(SP_INIT, T(raw).offset, v->host_data, T(raw).bytes, nullptr);
        t = new_tensor(dst, L_ROWMAJOR, v->shape, 0, SP_CONST);
        const int64_t n = v->shape.numel();
        const Ref a = ref(raw), b = ref(t);
        const bool was_init = in_init_;
        in_init_ = true;
        emit("const.cast", {}, {}, [=](const ExecEnv& e, hipStream_t st) { return launch_cast(a(e), src, b(e), dst, n, st); });
        in_init_ = was_init;
      }
      set_main(v, t);
    } else {
      fail(ODLA_INTERNAL_LOGIC_ERR, "value '%s' is used before it is produced", v->name.c_str());
    }
  }

  int convert(const _odla_value* v, int have, Layout want, Form form, int cvec) {
    const PTensor src = T(have);
    const QuantEntry* q = qentry(v);
    const bool src_q = src.quant;
    const bool dst_q = form == FORM_QUANT;
    if (dst_q && q == nullptr && !src_q) fail(ODLA_INTERNAL_LOGIC_ERR, "quantised form of '%s' requested without a table entry", v->name.c_str());
    const float scale = src_q ? src.qscale : (q ? q->scale : 1.f);
    const int zp = src_q ? src.qzp : (q ? q->zp : 0);
    const DType fdt = dst_q ? DT_I8 : (form == FORM_OPERAND ? op_dt_ : storage_dtype(v));
    const Space space = SP_ARENA;
    const Shape& sh = v->shape;

    // Layout change (with optional type / form change fused in) -----------
    if (src.layout != want || (want == L_NHWC && cvec > 1 && src.cs % cvec != 0)) {
      if (sh.rank != 4) fail(ODLA_INTERNAL_LOGIC_ERR, "layout conversion of a rank-%d value", sh.rank);
      int from = have;
      if (src.layout == L_NHWC && want == L_NHWC) {
        // repitch: go through row-major
        from = get(v, L_ROWMAJOR, src_q ? FORM_QUANT : (form == FORM_OPERAND ? FORM_OPERAND : FORM_FLOAT));
      }
      const PTensor s2 = T(from);
      LayoutParams lp;
      lp.N = (int)sh.d[0]; lp.C = (int)sh.d[1]; lp.HW = (int)(sh.d[2] * sh.d[3]);
      lp.scale = scale; lp.zp = zp;
      // the layout kernels convert between float types and to/from 8-bit levels
      if (s2.quant && dst_q) {
        // 8-bit to 8-bit relayout: byte-wise strided copy
        return relayout_bytes(v, from, want, cvec);
      }
      lp.src_dt = s2.dt;
      lp.dst_dt = fdt;
      if (want == L_NHWC) {
        const int cs = cvec > 1 ? round_up_i((int)sh.d[1], cvec) : (int)sh.d[1];
        lp.cs = cs;
        const int dst = new_tensor(fdt, L_NHWC, sh, cs, space);
        set_quant(dst, dst_q, scale, zp);
        const Ref a = ref(from), b = ref(dst);
        emit("to_nhwc:" + v->name, {from}, {dst}, [=](const ExecEnv& e, hipStream_t st) {
          LayoutParams p = lp; p.src = a(e); p.dst = b(e);
          return launch_nchw_to_nhwc(p, st);
        }, /*exact_reader=*/true);
        return dst;
      } else {
        lp.cs = s2.cs;
        const int dst = new_tensor(fdt, L_ROWMAJOR, sh, 0, space);
        set_quant(dst, dst_q, scale, zp);
        const Ref a = ref(from), b = ref(dst);
        emit("to_nchw:" + v->name, {from}, {dst}, [=](const ExecEnv& e, hipStream_t st) {
          LayoutParams p = lp; p.src = a(e); p.dst = b(e);
          return launch_nhwc_to_nchw(p, st);
        });
        return dst;
      }
    }
    // Same layout, form change ----------------------------------------------
    const int dst = new_tensor(fdt, src.layout, sh, src.cs, space);
    set_quant(dst, dst_q, scale, zp);
    const int64_t n = src.phys_elems();
    const Ref a = ref(have), b = ref(dst);
    if (src_q && !dst_q) {
      const int sc = const_vector<float>(DT_F32, {scale});
      const int zc = const_vector<int32_t>(DT_I32, {zp});
      const Ref rs = ref(sc), rz = ref(zc);
      const DType ddt = fdt;
      emit("dequant:" + v->name, {have}, {dst}, [=](const ExecEnv& e, hipStream_t st) {
        QuantParams p; p.src = a(e); p.dst = b(e); p.src_dt = DT_I8; p.dst_dt = ddt; p.n = n;
        p.scale = (const float*)rs(e); p.zp = (const int32_t*)rz(e);
        return launch_dequantize(p, st);
      });
    } else if (!src_q && dst_q) {
      const int sc = const_vector<float>(DT_F32, {scale});
      const int zc = const_vector<int32_t>(DT_I32, {zp});
      const Ref rs = ref(sc), rz = ref(zc);
      const DType sdt = src.dt;
      emit("quant:" + v->name, {have}, {dst}, [=](const ExecEnv& e, hipStream_t st) {
        QuantParams p; p.src = a(e); p.dst = b(e); p.src_dt = sdt; p.dst_dt = DT_I8; p.n = n;
        p.scale = (const float*)rs(e); p.zp = (const int32_t*)rz(e);
        return launch_quantize(p, st);
      });
    } else if (src.dt != fdt) {
      const DType sdt = src.dt, ddt = fdt;
      emit("cast:" + v->name, {have}, {dst}, [=](const ExecEnv& e, hipStream_t st) { return launch_cast(a(e), sdt, b(e), ddt, n, st); });
    } else {
      fail(ODLA_INTERNAL_LOGIC_ERR, "no conversion needed for '%s'", v->name.c_str());
    }
    return dst;
  }

  int relayout_bytes(const _odla_value* v, int from, Layout want, int cvec) {
    const PTensor s = T(from);
    const Shape& sh = v->shape;
    const int64_t N = sh.d[0], C = sh.d[1], H = sh.d[2], W = sh.d[3];
    const int cs = want == L_NHWC ? (cvec > 1 ? round_up_i((int)C, cvec) : (int)C) : 0;
    if (want == L_NHWC && cs != C) fail(ODLA_UNSUPPORTED_OP, "8-bit relayout with channel padding is not supported ('%s')", v->name.c_str());
    const int dst = new_tensor(s.dt, want, sh, cs, SP_ARENA);
    set_quant(dst, s.quant, s.qscale, s.qzp);
    StridedCopyParams cp;
    cp.elem_size = dtype_size(s.dt);
    cp.rank = 4;
    if (want == L_NHWC) {  // iterate N,H,W,C over the destination
      cp.dims[0] = N; cp.dims[1] = H; cp.dims[2] = W; cp.dims[3] = C;
      cp.sy[0] = H * W * cs; cp.sy[1] = W * cs; cp.sy[2] = cs; cp.sy[3] = 1;
      cp.sx[0] = C * H * W; cp.sx[1] = W; cp.sx[2] = 1; cp.sx[3] = H * W;
    } else {  // iterate N,C,H,W over the destination
      cp.dims[0] = N; cp.dims[1] = C; cp.dims[2] = H; cp.dims[3] = W;
      cp.sy[0] = C * H * W; cp.sy[1] = H * W; cp.sy[2] = W; cp.sy[3] = 1;
      cp.sx[0] = H * W * s.cs; cp.sx[1] = 1; cp.sx[2] = W * s.cs; cp.sx[3] = s.cs;
    }
    const Ref a = ref(from), b = ref(dst);
    emit("relayout:" + v->name, {from}, {dst}, [=](const ExecEnv& e, hipStream_t st) {
      StridedCopyParams p = cp; p.x = a(e); p.y = b(e);
      return launch_strided_copy(p, st);
    });
    return dst;
  }

  void set_quant(int t, bool q, float scale, int zp) {
    T(t).quant = q;
    T(t).qscale = q ? scale : 1.f;
    T(t).qzp = q ? zp : 0;
  }

  // New output tensor of a node in float storage.
  int out_tensor(const _odla_value* v, Layout layout, int cs = 0, DType dt = DT_INVALID) {
    if (dt == DT_INVALID) dt = storage_dtype(v);
    if (layout == L_NHWC && cs == 0) cs = (int)v->shape.d[1];
    return new_tensor(dt, layout, v->shape, cs, SP_ARENA);
  }

  // Is `v` available as 8-bit levels (already stored so, or quantisable from the table)?
  bool q8_value(const _odla_value* v) {
    if (!comp_->opts.int8 || v == nullptr) return false;
    if (qentry(v) != nullptr) return true;
    const VState& s = vs_[v->index];
    return s.main >= 0 && T(s.main).quant;
  }
  int use_count(const _odla_value* v) const { return (int)consumers_[v->index].size() + (v->is_output ? 1 : 0); }
  bool available(const _odla_value* v) const {
    return v->kind != _odla_value::TEMP || vs_[v->index].main >= 0;
  }

  // ------------------------------------------------------------------ nodes
  void lower(int ni);
  void lower_conv(int ni);
  void lower_gemm(int ni);
  void lower_binary(int ni);
  void lower_unary(int ni);
  void lower_batchnorm(int ni);
  void lower_layernorm(int ni);
  void lower_pool(int ni);
  void lower_reduce(int ni);
  void lower_softmax(int ni);
  void lower_cast(int ni);
  void lower_concat(int ni);
  void lower_gather(int ni);
  void lower_reshape(int ni);
  void lower_resize(int ni);
  void lower_slice(int ni);
  void lower_transpose(int ni);
  void lower_qdq(int ni);
  void lower_nms(int ni);
  void lower_ewise(int ni);
  void lower_argext(int ni);
  void lower_copynd(int ni);
  void lower_topk(int ni);
  void lower_lrn(int ni);
  void lower_rownorm(int ni);
  void lower_postprocess(int ni);
  void lower_axisop(int ni);
  bool lower_fused_group(int seed, int from);
  bool fuse_slice_seed(int ni) const;
  bool fuse_candidate(int ni) const;
  bool gemm_epilogue(int ni, Epilogue* ep);
  bool try_fused_attention(int ni);
  std::unordered_map<int, Epilogue> gemm_ep_ahead_;  // epilogues collected while looking for sibling GEMMs
  std::vector<char> gemm_merged_;                    // nodes already lowered inside a sibling's launch
  std::vector<char> no_fuse_;                        // nodes of an element-wise group that was given up
  void emit_stats(const _odla_value* v, const char* op_type, int forced_axis, const Node* producer);
  bool calib_ = false;
  struct SoftmaxAdd { const _odla_value* x; const _odla_value* mask; int64_t div; };
  std::unordered_map<int, SoftmaxAdd> softmax_add_;  // index of a folded Add's result -> its operands

  void collect_epilogue(int ni, int64_t out_channels, int channel_axis_of_output, Epilogue* ep);
  bool per_channel_constant(const _odla_value* k, const Shape& aligned, const Shape& out, int ch_axis,
                            int64_t channels, std::vector<float>* vals);
  void bn_params_host(const Node& n, int64_t C, std::vector<float>* scale, std::vector<float>* shift);
  // dense_groups > 0: G is 1, Og / Cg are the totals and the kernel holds that many groups
  int pack_weights(const _odla_value* kernel, DType dst_dt, int G, int Og, int Cg, int R, int S, int Cp,
                   int64_t so, int64_t si, int64_t sr, int64_t ss, const std::vector<float>& row_scale,
                   int* w_rs_out, const std::vector<float>* wq_scale, int dense_groups = 0);
  int make_wfrag(const std::string& name, IgemmParams* ip, int tw);
  // Debug-level log line "<launch>: kernel <variant>" (the device pointers that the
  // choice looks at are replaced by stand-ins: only their presence matters).
  void log_igemm_choice(const std::string& name, IgemmParams ip, bool has_wfrag, bool has_residual) {
    static int dummy;
    ip.w_frag = has_wfrag ? &dummy : nullptr;
    ip.residual = has_residual ? &dummy : nullptr;
    OHIP_DEBUG("%s: kernel %s", name.c_str(), igemm_variant_name(ip));
  }
  // A value whose only use is Reshape -> [B, S, heads, d] -> Transpose (0, 2, 1, 3): the
  // GEMM that computes it can store [B, heads, S, d] directly (IgemmParams::y_rdiv).
  struct HeadSplit { int reshape = -1, transpose = -1; int64_t B = 0, S = 0, heads = 0, d = 0; _odla_value* out = nullptr; };
  bool head_split_behind(const _odla_value* v, int64_t rows, int64_t cols, HeadSplit* hs) const;
  // The Transpose (0, 2, 1, 3) that is the only use of a rank-4 value, or -1.
  int head_merge_behind(const _odla_value* v) const;
  void finish_igemm(const std::string& name, IgemmParams ip, int tx, int tw, int ty, const Epilogue& ep,
                    int64_t Kout_total);
  int strided_copy_step(const std::string& name, int src, int dst, const StridedCopyParams& cp_in);
  void assign_arena();
  void parse_quant_table();
};

// ============================================================================

void Planner::parse_quant_table() {
  const Options& o = comp_->opts;
  if (!o.int8) return;
  if (o.qtable == nullptr || o.qtable_size <= 0) fail(ODLA_INVALID_PARAM, "int8 data type selected but no ODLA_QUANT_TABLE / ODLA_QUANT_TABLE_SIZE was set");
  QuantEntry* cur = nullptr;
  for (int i = 0; i < o.qtable_size; ++i) {
    const odla_value_quant_info& r = o.qtable[i];
    if (r.value_id == nullptr) continue;
    const std::string name(reinterpret_cast<const char*>(r.value_id));
    if (r.ch_idx < 0) {
      QuantEntry& e = qmap_[name];
      e.scale = r.scale;
      e.zp = (int)std::lrintf(r.offset);
      e.min = r.min;
      e.max = r.max;
      e.ch_min.assign((size_t)(-r.ch_idx), 0.f);
      e.ch_max.assign((size_t)(-r.ch_idx), 0.f);
      cur = &e;
      if (!(e.scale > 0.f) || e.zp < 0 || e.zp > 255) fail(ODLA_INVALID_PARAM, "quant table entry '%s' has scale %g / zero point %d", name.c_str(), e.scale, e.zp);
    } else {
      auto it = qmap_.find(name);
      QuantEntry* e = it != qmap_.end() ? &it->second : cur;
      if (e == nullptr || (size_t)r.ch_idx >= e->ch_min.size()) fail(ODLA_INVALID_PARAM, "quant table channel record %d of '%s' has no tensor record", r.ch_idx, name.c_str());
      e->ch_min[r.ch_idx] = r.min;
      e->ch_max[r.ch_idx] = r.max;
    }
  }
}

// Calibration: partial minima / maxima of a named fp32 value, kept in a pinned
// arena tensor until the execution has finished.
void Planner::emit_stats(const _odla_value* v, const char* op_type, int forced_axis, const Node* producer) {
  const Options& o = comp_->opts;
  if (v == nullptr || v->name.empty() || dtype_from_odla(v->etype) != DT_F32) return;
  const int tx = get(v, L_ROWMAJOR, FORM_FLOAT);
  if (T(tx).dt != DT_F32) return;
  const Shape& s = v->shape;
  Plan::StatRec rec;
  rec.name = v->name;
  rec.op_type = op_type;
  rec.shape = s;
  int axis = forced_axis >= 0 ? forced_axis : (o.calib_axis < 0 ? s.rank + o.calib_axis : o.calib_axis);
  int64_t outer = 1, inner = 1, C = 1;
  if (o.calib_channels && axis >= 0 && axis < s.rank && s.d[axis] <= 65535) {
    rec.per_channel = true;
    C = s.d[axis];
    for (int i = 0; i < axis; ++i) outer *= s.d[i];
    for (int i = axis + 1; i < s.rank; ++i) inner *= s.d[i];
  } else {
    inner = s.numel();
  }
  rec.channels = (int)C;
  const int64_t per = outer * inner;
  int64_t splits = (per + 8191) / 8192;
  const int64_t cap = 2048 / C > 1 ? 2048 / C : 1;   // enough workgroups to fill the chip, few partials
  if (splits > cap) splits = cap;
  rec.splits = (int)(splits < 1 ? 1 : splits);
  rec.tensor = raw_buffer((size_t)C * rec.splits * 2 * sizeof(float), SP_ARENA);
  if (producer != nullptr)
    for (const _odla_value* in : producer->in)
      if (in != nullptr && !in->name.empty()) rec.inputs.push_back(in->name);
  const Ref a = ref(tx), b = ref(rec.tensor);
  const int Ci = (int)C, sp = rec.splits;
  emit("stats:" + v->name, {tx}, {rec.tensor}, [=](const ExecEnv& e, hipStream_t st) {
    return launch_minmax_partial((const float*)a(e), (float*)b(e), outer, Ci, inner, sp, st);
  });
  PTensor& p = T(rec.tensor);
  p.pinned = true;
  p.last_step = 1 << 30;
  plan_->stat_recs.push_back(std::move(rec));
}

void Planner::run() {
  const Options& o = comp_->opts;
  calib_ = o.calibrate;
  plan_->calibrated = calib_;
  if (calib_) cdt_ = DT_F32;
  else if (o.fp16) cdt_ = DT_F16;
  else if (o.bf16 == BF16_ACCURACY_MODE && !o.int8) acc_mode_ = true;   // values fp32, Conv / Gemm operands bf16
  else if (o.bf16 != BF16_DISABLE) cdt_ = DT_BF16;                      // (performance and auto modes)
  op_dt_ = acc_mode_ ? DT_BF16 : cdt_;
  if (!calib_) parse_quant_table();

  vs_.assign(comp_->values.size(), VState());
  operand_only_.assign(comp_->values.size(), (signed char)-1);
  consumers_.assign(comp_->values.size(), {});
  for (size_t ni = 0; ni < comp_->nodes.size(); ++ni)
    for (_odla_value* v : comp_->nodes[ni].in)
      if (v != nullptr) consumers_[v->index].push_back((int)ni);

  // Arguments: one staging tensor each (declared type, row-major), alive from
  // the start of the execution because the H2D copy precedes every step.
  for (_odla_value* a : comp_->args) {
    const DType d = dtype_from_odla(a->etype);
    const int t = new_tensor(d, L_ROWMAJOR, a->shape, 0, SP_ARENA);
    T(t).pinned = true;
    T(t).def_step = -1;
    Plan::IO io;
    io.v = a;
    io.tensor = t;
    io.bytes = T(t).bytes;
    plan_->inputs.push_back(io);
    VState& s = vs_[a->index];
    s.main = t;
    if (d == storage_dtype(a)) {
      set_main(a, t);
    }
    // otherwise no slot is filled: consumers convert from the staging tensor
  }

  if (calib_) {
    for (_odla_value* a : comp_->args) emit_stats(a, a->eager ? "odla_SetValueData" : "odla_CreateArgument", -1, nullptr);
    if (!o.calib_skip_weights) {
      // kernels of convolutions get one range per output channel whatever the channel axis is
      std::unordered_map<const _odla_value*, int> kernel_axis;
      for (const Node& n : comp_->nodes)
        if (n.op == OP_CONV && n.in[1] != nullptr) {
          const int kl = (int)n.i[2];
          kernel_axis[n.in[1]] = kl == ODLA_SIO ? 3 : (kl == ODLA_SOI ? 2 : (kl == ODLA_IOS ? 1 : 0));
        }
      for (const auto& up : comp_->values) {
        const _odla_value* v = up.get();
        if (v->kind != _odla_value::CONSTANT || consumers_[v->index].empty()) continue;
        auto it = kernel_axis.find(v);
        emit_stats(v, "odla_CreateConstant", it == kernel_axis.end() ? -1 : it->second, nullptr);
      }
    }
  }
  for (size_t ni = 0; ni < comp_->nodes.size(); ++ni) {
    if (comp_->nodes[ni].absorbed) continue;
    if (!calib_ && !o.int8) {
      if (fuse_candidate((int)ni) && lower_fused_group((int)ni, (int)ni)) continue;
      if (fuse_slice_seed((int)ni) && lower_fused_group(consumers_[comp_->nodes[ni].out->index][0], (int)ni) &&
          comp_->nodes[ni].absorbed)
        continue;
    }
    lower((int)ni);
    if (calib_) {
      const Node& n = comp_->nodes[ni];
      emit_stats(n.out, api_op_name(n), -1, &n);
      if (n.out2 != nullptr) emit_stats(n.out2, api_op_name(n), -1, &n);
    }
  }

  // Outputs: row-major, declared element type.
  for (_odla_value* ov : comp_->outputs) {
    const DType want = dtype_from_odla(ov->etype);
    int t = get(ov, L_ROWMAJOR, FORM_FLOAT);
    bool converted = false;
    if (T(t).dt != want) {
      const int dst = new_tensor(want, L_ROWMAJOR, ov->shape, 0, SP_ARENA);
      const int64_t n = ov->shape.numel();
      const DType sdt = T(t).dt;
      const Ref a = ref(t), b = ref(dst);
      emit("out.cast:" + ov->name, {t}, {dst}, [=](const ExecEnv& e, hipStream_t st) { return launch_cast(a(e), sdt, b(e), want, n, st); });
      t = dst;
      converted = true;
    }
    PTensor& p = T(root(t));
    if (p.space == SP_ARENA) { p.pinned = true; p.last_step = 1 << 30; }
    Plan::IO io;
    io.v = ov;
    io.tensor = root(t);
    io.offset = T(t).alias_off;
    io.bytes = (size_t)ov->shape.numel() * dtype_size(want);
    // The conversion to the declared type is the only step that touches its result, and it
    // writes exactly the result's elements: it can write the caller's device buffer directly.
    if (converted && !calib_ && io.tensor == t && io.offset == 0) {
      io.in_place_ok = true;
      T(t).ext_slot = (int)(plan_->inputs.size() + plan_->outputs.size());
    }
    plan_->outputs.push_back(io);
  }
  // Arguments whose staging tensor only layout conversions read: the conversion can read the
  // caller's device buffer, and the copy into the arena is skipped.
  for (size_t k = 0; k < plan_->inputs.size(); ++k) {
    Plan::IO& io = plan_->inputs[k];
    const int r = root(io.tensor);
    bool ok = !calib_ && r == io.tensor && T(r).space == SP_ARENA && T(r).last_step >= 0 && !arena_only_.count(r);
    for (const Plan::IO& o : plan_->outputs) ok = ok && root(o.tensor) != r;
    for (const auto& ft : plan_->final_tensor) ok = ok && root(ft.second) != r;
    if (ok) {
      io.in_place_ok = true;
      T(r).ext_slot = (int)k;
    }
  }
  assign_arena();
}

// Staged arguments whose declared type differs from the storage type have no
// slot; pick_source() then falls back to `main` (the staging tensor).

void Planner::assign_arena() {
  struct Item { int t; int a, b; size_t bytes; size_t off; };
  std::vector<Item> items;
  for (size_t i = 0; i < plan_->tensors.size(); ++i) {
    PTensor& p = plan_->tensors[i];
    if (p.space != SP_ARENA || p.alias_of >= 0) continue;
    int a = p.def_step, b = p.last_step;
    if (a == kUnset) { a = 0; if (b < 0) b = 0; }  // never touched by a step: still give it room
    if (b < a) b = a;
    items.push_back({(int)i, a, b, align_up(p.bytes ? p.bytes : 1), 0});
  }
  std::sort(items.begin(), items.end(), [](const Item& x, const Item& y) {
    if (x.a != y.a) return x.a < y.a;
    return x.bytes > y.bytes;
  });
  std::vector<Item> placed;
  size_t total = 0;
  for (Item& it : items) {
    std::vector<std::pair<size_t, size_t>> busy;
    for (const Item& q : placed)
      if (!(q.b < it.a || it.b < q.a)) busy.push_back({q.off, q.off + q.bytes});
    std::sort(busy.begin(), busy.end());
    size_t off = 0;
    for (auto& r : busy) {
      if (off + it.bytes <= r.first) break;
      if (r.second > off) off = r.second;
    }
    it.off = off;
    placed.push_back(it);
    plan_->tensors[it.t].offset = off;
    if (off + it.bytes > total) total = off + it.bytes;
  }
  plan_->arena_bytes = total;
}

void Planner::lower(int ni) {
  const Node& n = comp_->nodes[ni];
  switch (n.op) {
    case OP_CONV: lower_conv(ni); break;
    case OP_GEMM: lower_gemm(ni); break;
    case OP_BINARY: lower_binary(ni); break;
    case OP_UNARY: lower_unary(ni); break;
    case OP_BATCHNORM: lower_batchnorm(ni); break;
    case OP_LAYERNORM: lower_layernorm(ni); break;
    case OP_POOL: lower_pool(ni); break;
    case OP_REDUCE: lower_reduce(ni); break;
    case OP_SOFTMAX: lower_softmax(ni); break;
    case OP_CAST: lower_cast(ni); break;
    case OP_CONCAT: lower_concat(ni); break;
    case OP_GATHER: lower_gather(ni); break;
    case OP_RESHAPE: lower_reshape(ni); break;
    case OP_RESIZE: lower_resize(ni); break;
    case OP_SLICE: lower_slice(ni); break;
    case OP_TRANSPOSE: lower_transpose(ni); break;
    case OP_QUANTIZE: case OP_DEQUANTIZE: lower_qdq(ni); break;
    case OP_NMS: lower_nms(ni); break;
    case OP_EWISE: lower_ewise(ni); break;
    case OP_ARGEXT: lower_argext(ni); break;
    case OP_COPYND: lower_copynd(ni); break;
    case OP_TOPK: lower_topk(ni); break;
    case OP_LRN: lower_lrn(ni); break;
    case OP_ROWNORM: lower_rownorm(ni); break;
    case OP_POSTPROCESS: lower_postprocess(ni); break;
    case OP_AXISOP: lower_axisop(ni); break;
  }
}

// ------------------------------------------------------------------ fusion --

// Is `k` a constant that varies only along `ch_axis` of `out` (or is a scalar)?
bool Planner::per_channel_constant(const _odla_value* k, const Shape& aligned, const Shape& out,
                                   int ch_axis, int64_t channels, std::vector<float>* vals) {
  if (k->kind != _odla_value::CONSTANT) return false;
  const int64_t n = k->shape.numel();
  if (n == 1) {
    const float v = const_as_float(k)[0];
    vals->assign((size_t)channels, v);
    return true;
  }
  if (n != channels || aligned.rank != out.rank) return false;
  for (int i = 0; i < aligned.rank; ++i) {
    if (i == ch_axis) { if (aligned.d[i] != channels) return false; }
    else if (aligned.d[i] != 1) return false;
  }
  *vals = const_as_float(k);
  return true;
}

void Planner::bn_params_host(const Node& n, int64_t C, std::vector<float>* scale, std::vector<float>* shift) {
  const std::vector<float> mean = const_as_float(n.in[1]), var = const_as_float(n.in[2]);
  std::vector<float> g((size_t)C, n.f[1]), b((size_t)C, n.f[2]);
  if (n.in[3]) g = const_as_float(n.in[3]);
  if (n.in[4]) b = const_as_float(n.in[4]);
  scale->resize((size_t)C);
  shift->resize((size_t)C);
  for (int64_t c = 0; c < C; ++c) {
    const float m = g[c] / std::sqrt(var[c] + n.f[0]);
    (*scale)[c] = m;
    (*shift)[c] = b[c] - mean[c] * m;
  }
}

// Walk the single-consumer chain behind node `ni` and fold what the igemm
// epilogue can do.  `ch_axis` is the logical axis of the output that indexes
// output channels.
void Planner::collect_epilogue(int ni, int64_t channels, int ch_axis, Epilogue* ep) {
  _odla_value* cur = comp_->nodes[ni].out;
  ep->final_value = cur;
  if (calib_) return;  // every value of the graph must exist to be measured
  const bool q8 = comp_->opts.int8;
  while (true) {
    if (cur->is_output || consumers_[cur->index].size() != 1) break;
    const int ci = consumers_[cur->index][0];
    Node& nx = comp_->nodes[ci];
    if (nx.absorbed) break;
    bool took = false;
    if (nx.op == OP_BATCHNORM && nx.in[0] == cur && ep->residual == nullptr && ep->act == ACT_NONE && !q8) {
      const bool cf = nx.i[0] != ODLA_CHANNELS_LAST;
      const int bn_axis = cf ? 1 : cur->shape.rank - 1;
      bool all_const = nx.in[1]->kind == _odla_value::CONSTANT && nx.in[2]->kind == _odla_value::CONSTANT &&
                       (!nx.in[3] || nx.in[3]->kind == _odla_value::CONSTANT) &&
                       (!nx.in[4] || nx.in[4]->kind == _odla_value::CONSTANT);
      if (all_const && bn_axis == ch_axis) {
        std::vector<float> sc, sh;
        bn_params_host(nx, channels, &sc, &sh);
        if (ep->row_scale.empty()) ep->row_scale.assign((size_t)channels, 1.f);
        if (ep->bias.empty()) ep->bias.assign((size_t)channels, 0.f);
        for (int64_t c = 0; c < channels; ++c) {
          ep->row_scale[c] *= sc[c];
          ep->bias[c] = ep->bias[c] * sc[c] + sh[c];
        }
        ep->has_bias = true;
        took = true;
      }
    } else if (nx.op == OP_BINARY && (nx.i[0] == BIN_ADD || nx.i[0] == BIN_MUL || nx.i[0] == BIN_SUB || nx.i[0] == BIN_DIV)) {
      const bool cur_is_lhs = nx.in[0] == cur;
      _odla_value* other = cur_is_lhs ? nx.in[1] : nx.in[0];
      if (other != cur && nx.out->shape == cur->shape) {
        // aligned operand shapes recorded by the builder
        const int r = (int)nx.iv[0];
        Shape al;
        al.rank = r;
        for (int i = 0; i < r; ++i) al.d[i] = nx.iv[1 + (cur_is_lhs ? r : 0) + i];
        std::vector<float> vals;
        if (ep->residual == nullptr && ep->act == ACT_NONE && !q8 &&
            per_channel_constant(other, al, nx.out->shape, ch_axis, channels, &vals)) {
          if (ep->bias.empty()) ep->bias.assign((size_t)channels, 0.f);
          if (nx.i[0] == BIN_ADD) {
            for (int64_t c = 0; c < channels; ++c) ep->bias[c] += vals[c];
            ep->has_bias = true;
            took = true;
          } else if (nx.i[0] == BIN_SUB && cur_is_lhs) {
            for (int64_t c = 0; c < channels; ++c) ep->bias[c] -= vals[c];
            ep->has_bias = true;
            took = true;
          } else if (nx.i[0] == BIN_MUL && other->shape.numel() == 1) {
            ep->scalar *= vals[0];
            for (int64_t c = 0; c < channels; ++c) ep->bias[c] *= vals[0];
            took = true;
          } else if (nx.i[0] == BIN_DIV && cur_is_lhs && other->shape.numel() == 1 && vals[0] != 0.f) {
            const float inv = 1.0f / vals[0];
            ep->scalar *= inv;
            for (int64_t c = 0; c < channels; ++c) ep->bias[c] *= inv;
            took = true;
          } else if (nx.i[0] == BIN_MUL) {
            if (ep->row_scale.empty()) ep->row_scale.assign((size_t)channels, 1.f);
            for (int64_t c = 0; c < channels; ++c) { ep->row_scale[c] *= vals[c]; ep->bias[c] *= vals[c]; }
            took = true;
          }
        } else if (nx.i[0] == BIN_ADD && ep->residual == nullptr && ep->act == ACT_NONE &&
                   other->kind != _odla_value::CONSTANT && other->shape == cur->shape && available(other) &&
                   storage_dtype(other) == storage_dtype(cur)) {
          bool ok = true;
          if (q8) {  // both sides must be 8-bit
            ok = qentry(cur) != nullptr && q8_value(other);
          }
          if (ok) {
            ep->residual = other;
            ep->pre_residual_value = cur;
            took = true;
          }
        }
      }
    } else if (nx.op == OP_UNARY && ep->act == ACT_NONE) {
      const ActKind a = (ActKind)nx.i[0];
      // the 8-bit epilogue clamps only; the float ones also have a variant with
      // the transcendental activations (GELU behind a feed-forward GEMM)
      const bool rich = a == ACT_GELU_ERF || a == ACT_GELU_TANH || a == ACT_SIGMOID || a == ACT_TANH;
      // (the epilogues with the transcendental functions exist for results of the operand type only)
      const bool rich_ok = rich && ep->residual == nullptr && result_dtype(nx.out) == mm_dtype(nx.out);
      const bool fusable = q8 ? (a == ACT_RELU) : (a == ACT_RELU || a == ACT_LEAKY || a == ACT_CLAMP || rich_ok);
      if (fusable) {
        ep->act = a;
        ep->act_a = nx.f[0];
        ep->act_b = nx.f[1];
        took = true;
      }
    }
    if (!took) break;
    nx.absorbed = true;
    cur = nx.out;
    ep->final_value = cur;
    if (ep->act != ACT_NONE) break;
  }
  // Shortcut behind the activation (y = act(conv) + x, the Darknet order): one more follower.
  if (!q8 && ep->act != ACT_NONE && ep->residual == nullptr && !cur->is_output && consumers_[cur->index].size() == 1) {
    Node& nx = comp_->nodes[consumers_[cur->index][0]];
    if (!nx.absorbed && nx.op == OP_BINARY && nx.i[0] == BIN_ADD && nx.out->shape == cur->shape) {
      _odla_value* other = nx.in[0] == cur ? nx.in[1] : nx.in[0];
      if (other != cur && other->kind != _odla_value::CONSTANT && other->shape == cur->shape && available(other) &&
          storage_dtype(other) == storage_dtype(cur)) {
        ep->residual = other;
        ep->pre_residual_value = cur;
        ep->res_after_act = true;
        nx.absorbed = true;
        ep->final_value = nx.out;
      }
    }
  }
}

// ------------------------------------------------------------------ weights --

int Planner::pack_weights(const _odla_value* kernel, DType dst_dt, int G, int Og, int Cg, int R, int S,
                          int Cp, int64_t so, int64_t si, int64_t sr, int64_t ss,
                          const std::vector<float>& row_scale, int* w_rs_out,
                          const std::vector<float>* wq_scale, int dense_groups) {
  const int es = dtype_size(dst_dt);
  const int bk = 64 / es;
  const int w_rs = round_up_i(R * S * Cp, bk);
  *w_rs_out = w_rs;
  Shape ws;
  ws.rank = 3;
  ws.d[0] = G; ws.d[1] = Og; ws.d[2] = w_rs;
  PackWeightsParams pp;
  pp.G = G; pp.Og = Og; pp.Cg = Cg; pp.R = R; pp.S = S; pp.Cp = Cp;
  pp.rows_pad = Og; pp.w_rs = w_rs;
  pp.so = so; pp.si = si; pp.sr = sr; pp.ss = ss;
  pp.dst_dt = dst_dt;
  pp.dense_groups = dense_groups;
  const int64_t Ci = dense_groups > 0 ? Cg / dense_groups : Cg;  // in-channels per output row in the source

  if (kernel->kind == _odla_value::CONSTANT) {
    const int64_t n = kernel->shape.numel();
    const int dst = new_tensor(dst_dt, L_ROWMAJOR, ws, 0, SP_CONST);
    int raw;
    if (dst_dt == DT_I8) {
      // symmetric per-output-channel quantisation on the host:
      // q = clip(rne(w / s[o]), -127, 127)
      std::vector<float> w = const_as_float(kernel);
      std::vector<uint8_t> q((size_t)n);
      const int64_t O = (int64_t)G * Og;
      // element (o,i,r,s) at o*so + i*si + r*sr + s*ss
      for (int64_t o = 0; o < O; ++o) {
        const float s = (*wq_scale)[o];
        for (int64_t i = 0; i < Ci; ++i)
          for (int r = 0; r < R; ++r)
            for (int t = 0; t < S; ++t) {
              const int64_t idx = o * so + i * si + r * sr + t * ss;
              float v = std::nearbyintf(w[idx] / s);
              v = v < -127.f ? -127.f : (v > 127.f ? 127.f : v);
              q[idx] = (uint8_t)(int8_t)(int)v;
            }
      }
      raw = new_tensor(DT_I8, L_ROWMAJOR, kernel->shape, 0, SP_INIT);
      add_blob(SP_INIT, T(raw).offset, nullptr, T(raw).bytes, &q);
      pp.src_dt = DT_I8;
    } else if (!row_scale.empty()) {
      std::vector<float> w = const_as_float(kernel);
      const int64_t O = (int64_t)G * Og;
      for (int64_t o = 0; o < O; ++o)
        for (int64_t i = 0; i < Ci; ++i)
          for (int r = 0; r < R; ++r)
            for (int t = 0; t < S; ++t) w[o * so + i * si + r * sr + t * ss] *= row_scale[o];
      std::vector<uint8_t> bytes((size_t)n * 4);
      memcpy(bytes.data(), w.data(), bytes.size());
      raw = new_tensor(DT_F32, L_ROWMAJOR, kernel->shape, 0, SP_INIT);
      add_blob(SP_INIT, T(raw).offset, nullptr, T(raw).bytes, &bytes);
      pp.src_dt = DT_F32;
    } else {
      const DType sdt = dtype_from_odla(kernel->etype);
      raw = new_tensor(sdt, L_ROWMAJOR, kernel->shape, 0, SP_INIT);
      add_blob(SP_INIT, T(raw).offset, kernel->host_data, T(raw).bytes, nullptr);
      pp.src_dt = sdt;
    }
    const Ref a = ref(raw), b = ref(dst);
    const bool was_init = in_init_;
    in_init_ = true;
    emit("pack:" + kernel->name, {}, {}, [=](const ExecEnv& e, hipStream_t st) {
      PackWeightsParams p = pp; p.src = a(e); p.dst = b(e);
      return launch_pack_weights(p, st);
    });
    in_init_ = was_init;
    return dst;
  }
  // run-time kernel (argument or computed value): repack on every execution
  if (dst_dt == DT_I8) fail(ODLA_UNSUPPORTED_OP, "int8 convolution needs a constant kernel ('%s')", kernel->name.c_str());
  if (!row_scale.empty()) fail(ODLA_INTERNAL_LOGIC_ERR, "cannot fold a scale into a run-time kernel");
  const VState& s = vs_[kernel->index];
  if (s.main < 0) fail(ODLA_INTERNAL_LOGIC_ERR, "kernel '%s' is not available", kernel->name.c_str());
  const int src = s.main;  // staging tensor (declared type) or produced tensor, row-major
  if (T(src).layout != L_ROWMAJOR) fail(ODLA_UNSUPPORTED_OP, "run-time kernel '%s' must be row-major", kernel->name.c_str());
  pp.src_dt = T(src).dt;
  const int dst = new_tensor(dst_dt, L_ROWMAJOR, ws, 0, SP_ARENA);
  const Ref a = ref(src), b = ref(dst);
  emit("pack:" + kernel->name, {src}, {dst}, [=](const ExecEnv& e, hipStream_t st) {
    PackWeightsParams p = pp; p.src = a(e); p.dst = b(e);
    return launch_pack_weights(p, st);
  });
  return dst;
}

int Planner::strided_copy_step(const std::string& name, int src, int dst, const StridedCopyParams& cp_in) {
  StridedCopyParams cp = cp_in;
  // Move 16-byte elements when the innermost run is contiguous on both sides and
  // every stride / offset keeps 16-byte alignment (tensor bases are 256-byte aligned).
  {
    const int r = cp.rank;
    const int w = cp.elem_size > 0 && cp.elem_size < 16 ? 16 / cp.elem_size : 0;
    bool ok = w > 1 && r >= 1 && cp.sx[r - 1] == 1 && cp.sy[r - 1] == 1 && cp.dims[r - 1] % w == 0 &&
              cp.x_off % w == 0 && cp.y_off % w == 0;
    for (int d = 0; ok && d < r - 1; ++d) ok = cp.sx[d] % w == 0 && cp.sy[d] % w == 0;
    if (ok) {
      cp.elem_size = 16;
      cp.dims[r - 1] /= w;
      for (int d = 0; d < r - 1; ++d) { cp.sx[d] /= w; cp.sy[d] /= w; }
      cp.x_off /= w;
      cp.y_off /= w;
    }
  }
  const Ref a = ref(src), b = ref(dst);
  emit(name, {src}, {dst}, [=](const ExecEnv& e, hipStream_t st) {
    StridedCopyParams p = cp; p.x = a(e); p.y = b(e);
    return launch_strided_copy(p, st);
  });
  return dst;
}

// Constant weights of layers that use the weights-in-registers kernel get a
// second copy in MFMA fragment order, built once at initialisation.  Returns
// the tensor (and fills ip->wf_*), or -1 when the layer does not use one.
int Planner::make_wfrag(const std::string& name, IgemmParams* ip, int tw) {
  if (T(tw).space != SP_CONST || !igemm_wants_wfrag(*ip)) return -1;
  if (ip->batch != 1 && (int64_t)ip->w_bs != (int64_t)ip->w_rows * ip->w_rs) return -1;
  const int es = dtype_size(ip->in_dt);
  WfragPackParams fp;
  fp.batch = ip->batch;
  fp.rows = ip->w_rows;
  fp.row_bytes = ip->w_rs * es;
  fp.tiles = (ip->w_rows + 31) / 32;
  fp.chunks = (int)(((int64_t)ip->R * ip->S * ip->C * es + 127) / 128) * 4;
  fp.fill = ip->a_fill;
  const int tf = raw_buffer((size_t)fp.batch * fp.tiles * fp.chunks * 1024 + kWfragTailBytes, SP_CONST);
  ip->wf_chunks = fp.chunks;
  ip->wf_tiles = fp.tiles;
  const Ref a = ref(tw), b = ref(tf);
  const bool was_init = in_init_;
  in_init_ = true;
  emit("wfrag:" + name, {}, {}, [=](const ExecEnv& e, hipStream_t st) {
    WfragPackParams p = fp; p.src = a(e); p.dst = b(e);
    return launch_wfrag_pack(p, st);
  });
  in_init_ = was_init;
  return tf;
}

// Common tail of Conv / Gemm lowering: bias / residual / activation wiring and
// the launch step.  tx, tw, ty are the operand tensors.
void Planner::finish_igemm(const std::string& name, IgemmParams ip, int tx, int tw, int ty,
                           const Epilogue& ep, int64_t Kout_total) {
  int tb = -1, tr = -1;
  if (ep.has_bias) {
    std::vector<float> b = ep.bias;
    b.resize((size_t)Kout_total, 0.f);
    tb = const_vector<float>(DT_F32, b);
  }
  if (ep.residual != nullptr) {
    const PTensor yo = T(ty);
    tr = get(ep.residual, yo.layout, FORM_FLOAT);
    if (T(tr).dt != yo.dt) fail(ODLA_INTERNAL_LOGIC_ERR, "residual type mismatch ('%s')", name.c_str());
    ip.rcs = yo.layout == L_NHWC ? T(tr).cs : ip.ycs;
  }
  ip.act = ep.act;
  ip.act_a = ep.act_a;
  ip.act_b = ep.act_b;
  ip.res_after_act = ep.res_after_act;
  // A result much larger than the last-level cache cannot be kept there for its
  // consumer; written around the cache it leaves the lines of smaller tensors alone.
  ip.stream_out = T(ty).bytes >= stream_out_bytes();
  const int tf = make_wfrag(name, &ip, tw);
  const bool hf = tf >= 0;
  log_igemm_choice(name, ip, hf, tr >= 0);
  const Ref rf = ref(hf ? tf : tx);
  const Ref rx = ref(tx), rw = ref(tw), ry = ref(ty);
  const Ref rb = ref(tb >= 0 ? tb : tx), rr = ref(tr >= 0 ? tr : tx);
  const bool hb = tb >= 0, hr = tr >= 0;
  emit(name, {tx, tw, tr}, {ty}, [=](const ExecEnv& e, hipStream_t st) {
    IgemmParams p = ip;
    p.x = rx(e); p.w = rw(e); p.y = ry(e);
    p.bias = hb ? rb(e) : nullptr;
    p.residual = hr ? rr(e) : nullptr;
    p.w_frag = hf ? rf(e) : nullptr;
    return launch_igemm(p, st);
  });
}

// ---------------------------------------------------------------- Conv ----
void Planner::lower_conv(int ni) {
  Node& n = comp_->nodes[ni];
  const _odla_value* x = n.in[0];
  const _odla_value* k = n.in[1];
  const _odla_value* bias = n.in[2];
  const bool cl = n.i[0] == ODLA_CHANNELS_LAST;
  const int G = (int)n.i[1];
  const int kl = (int)n.i[2];
  const Shape& ks = k->shape;
  int64_t O, I, R, S, so, si, sr, ss;
  switch (kl) {
    case ODLA_SIO: R = ks.d[0]; S = ks.d[1]; I = ks.d[2]; O = ks.d[3]; sr = S * I * O; ss = I * O; si = O; so = 1; break;
    case ODLA_SOI: R = ks.d[0]; S = ks.d[1]; O = ks.d[2]; I = ks.d[3]; sr = S * O * I; ss = O * I; so = I; si = 1; break;
    case ODLA_IOS: I = ks.d[0]; O = ks.d[1]; R = ks.d[2]; S = ks.d[3]; si = O * R * S; so = R * S; sr = S; ss = 1; break;
    default: O = ks.d[0]; I = ks.d[1]; R = ks.d[2]; S = ks.d[3]; so = I * R * S; si = R * S; sr = S; ss = 1; break;
  }
  const Shape& xs = x->shape;
  const Shape& os = n.out->shape;
  const int64_t N = xs.d[0];
  int64_t C = cl ? xs.d[3] : xs.d[1], H = cl ? xs.d[1] : xs.d[2], W = cl ? xs.d[2] : xs.d[3];
  const int64_t Ho = cl ? os.d[1] : os.d[2], Wo = cl ? os.d[2] : os.d[3];
  const int Og = (int)(O / G);
  int Cg = (int)I;
  int str_h = (int)n.i[3], str_w = (int)n.i[4], dil_h = (int)n.i[5], dil_w = (int)n.i[6];
  int pad_t = (int)n.i[7], pad_l = (int)n.i[8];

  Epilogue ep;
  if (bias != nullptr) {
    if (bias->kind == _odla_value::CONSTANT) { ep.bias = const_as_float(bias); ep.has_bias = true; }
  }
  const bool runtime_bias = bias != nullptr && bias->kind != _odla_value::CONSTANT;
  const bool const_kernel = k->kind == _odla_value::CONSTANT;
  if (!runtime_bias) {
    collect_epilogue(ni, O, cl ? 3 : 1, &ep);
    if (!const_kernel && !ep.row_scale.empty()) fail(ODLA_UNSUPPORTED_OP, "scale folding into a run-time kernel");
  } else {
    ep.final_value = n.out;
  }
  _odla_value* outv = ep.final_value;

  // int8 plan?
  const QuantEntry* qk = qentry(k);
  // the input is 8-bit if it already lives as levels (e.g. the result of a
  // quantised producer or of a max-pool that kept its input's scale) or has a
  // table entry to quantise it with
  const bool x_q8 = q8_value(x);
  const bool q8 = comp_->opts.int8 && x_q8 && qk != nullptr && const_kernel && !cl && G == 1 &&
                  !runtime_bias;

  // ---- few-channel stride-2 convolution on an NCHW source (a network stem) ----
  // Rewritten as a stride-1 convolution over the space-to-depth form of the
  // input: source row 2*ho - pad + r = 2*(ho + dy) + py with dy = floor((r -
  // pad) / 2), so the R taps collapse into dy_max - dy_min + 1 taps over four
  // times the channels, channel (py*2 + px)*C + c.  7x7 / stride 2 / 3 channels
  // becomes 4x4 / stride 1 / 12 channels: K shrinks from 49 x 8 (channels padded
  // to one 16-byte vector) to 16 x 16 elements.
  const _odla_value* kpack = k;  // the kernel tensor that is packed
  _odla_value k_s2d;
  int tx_s2d = -1;
  {
    const VState& xv = vs_[x->index];
    const bool src_ok = xv.main >= 0 && T(xv.main).layout == L_ROWMAJOR && !T(xv.main).quant;
    if (!cl && G == 1 && const_kernel && !runtime_bias && C <= 4 && str_h == 2 && str_w == 2 && dil_h == 1 &&
        dil_w == 1 && (R > 2 || S > 2) && src_ok) {
      auto floor2 = [](int e) { return e >= 0 ? e / 2 : -((-e + 1) / 2); };
      const int dy0 = floor2(-pad_t), dy1 = floor2((int)R - 1 - pad_t);
      const int dx0 = floor2(-pad_l), dx1 = floor2((int)S - 1 - pad_l);
      const int R2 = dy1 - dy0 + 1, S2 = dx1 - dx0 + 1, C2 = 4 * (int)C;
      const std::vector<float> w = const_as_float(k);
      auto buf = std::make_unique<std::vector<uint8_t>>((size_t)O * C2 * R2 * S2 * 4, (uint8_t)0);
      float* w2 = reinterpret_cast<float*>(buf->data());
      for (int64_t o = 0; o < O; ++o)
        for (int64_t c = 0; c < C; ++c)
          for (int r = 0; r < R; ++r)
            for (int t = 0; t < S; ++t) {
              const int ey = r - pad_t, ex = t - pad_l;
              const int dy = floor2(ey), dx = floor2(ex);
              const int py = ey - 2 * dy, px = ex - 2 * dx;
              const int64_t c2 = (py * 2 + px) * C + c;
              w2[((o * C2 + c2) * R2 + (dy - dy0)) * S2 + (dx - dx0)] = w[o * so + c * si + r * sr + t * ss];
            }
      k_s2d.kind = _odla_value::CONSTANT;
      k_s2d.name = k->name;
      k_s2d.etype = ODLA_FLOAT32;
      k_s2d.shape.rank = 4;
      k_s2d.shape.d[0] = O; k_s2d.shape.d[1] = C2; k_s2d.shape.d[2] = R2; k_s2d.shape.d[3] = S2;
      k_s2d.host_data = w2;
      comp_->owned_data.push_back(std::move(buf));
      kpack = &k_s2d;
      so = (int64_t)C2 * R2 * S2; si = (int64_t)R2 * S2; sr = S2; ss = 1;

      // converted input: [N][ceil(H/2)][ceil(W/2)][C2 padded to one vector]
      const DType fdt = q8 ? DT_I8 : mm_dtype(x);
      const int vec = 16 / dtype_size(fdt);
      const int cs = round_up_i(C2, vec);
      const int64_t H2 = (H + 1) / 2, W2 = (W + 1) / 2;
      Shape sh2;
      sh2.rank = 4;
      sh2.d[0] = N; sh2.d[1] = C2; sh2.d[2] = H2; sh2.d[3] = W2;
      tx_s2d = new_tensor(fdt, L_NHWC, sh2, cs, SP_ARENA);
      S2dParams sp;
      sp.src_dt = T(xv.main).dt; sp.dst_dt = fdt;
      sp.N = (int)N; sp.C = (int)C; sp.H = (int)H; sp.W = (int)W; sp.cs = cs;
      if (q8) {
        const QuantEntry* qx = qentry(x);
        if (qx == nullptr) fail(ODLA_INTERNAL_LOGIC_ERR, "int8 stem without a table entry for '%s'", x->name.c_str());
        sp.scale = qx->scale; sp.zp = qx->zp;
        set_quant(tx_s2d, true, qx->scale, qx->zp);
      }
      const int from = xv.main;
      const Ref a = ref(from), b = ref(tx_s2d);
      emit("to_s2d:" + x->name, {from}, {tx_s2d}, [=](const ExecEnv& e, hipStream_t st) {
        S2dParams p = sp; p.src = a(e); p.dst = b(e);
        return launch_nchw_to_s2d(p, st);
      }, /*exact_reader=*/true);
      C = C2; Cg = C2; H = H2; W = W2; R = R2; S = S2;
      str_h = str_w = 1;
      pad_t = -dy0; pad_l = -dx0;
    }
  }

  if (q8) {
    // ---- int8 x int8 -> int32 with fused requantisation ----
    const int vec = 16;
    const int tx = tx_s2d >= 0 ? tx_s2d : get(x, L_NHWC, FORM_QUANT, vec);
    const int Cp = T(tx).cs;
    if (qk->ch_min.size() != (size_t)O) fail(ODLA_INVALID_PARAM, "quant table entry of kernel '%s' needs %lld channel records", k->name.c_str(), (long long)O);
    std::vector<float> sw((size_t)O);
    for (int64_t o = 0; o < O; ++o) {
      const float m = std::fmax(std::fabs(qk->ch_min[o]), std::fabs(qk->ch_max[o]));
      sw[o] = m > 0.f ? m / 127.f : 1.f;
    }
    int w_rs = 0;
    const int tw = pack_weights(kpack, DT_I8, 1, (int)O, Cg, (int)R, (int)S, Cp, so, si, sr, ss, {}, &w_rs, &sw);
    // int32 bias: rne(b / (s_x * s_w[o])) minus the zero-point correction
    // (zp_x - 128) * sum_k w_q[o][k]; activations are stored as q - 128.
    std::vector<float> wf = const_as_float(kpack);
    std::vector<int32_t> bi((size_t)O, 0);
    const float sx = T(tx).qscale;  // parameters of the tensor actually consumed
    const int zx = T(tx).qzp;
    for (int64_t o = 0; o < O; ++o) {
      int64_t wsum = 0;
      for (int64_t i = 0; i < Cg; ++i)
        for (int r = 0; r < R; ++r)
          for (int t = 0; t < S; ++t) {
            float v = std::nearbyintf(wf[o * so + i * si + r * sr + t * ss] / sw[o]);
            v = v < -127.f ? -127.f : (v > 127.f ? 127.f : v);
            wsum += (int64_t)v;
          }
      int64_t b = 0;
      if (ep.has_bias) {
        const float bs = sx * sw[o];
        float r = std::nearbyintf(ep.bias[o] / bs);
        r = r < -2147483648.f ? -2147483648.f : (r > 2147483520.f ? 2147483520.f : r);
        b = (int64_t)r;
      }
      b -= (int64_t)(zx - 128) * wsum;
      bi[o] = (int32_t)b;
    }
    const int tb = const_vector<int32_t>(DT_I32, bi);

    IgemmParams ip;
    ip.N = (int)N; ip.H = (int)H; ip.W = (int)W; ip.C = Cp; ip.xcs = Cp;
    ip.Ho = (int)Ho; ip.Wo = (int)Wo; ip.Kout = (int)O;
    ip.R = (int)R; ip.S = (int)S; ip.sh = str_h; ip.sw = str_w;
    ip.dh = dil_h; ip.dw = dil_w; ip.ph = pad_t; ip.pw = pad_l;
    ip.w_rows = (int)O; ip.w_cols = w_rs; ip.w_rs = w_rs;
    ip.in_dt = DT_I8;
    ip.a_fill = (zx - 128) & 0xff;

    const QuantEntry* qf = qentry(outv);
    std::vector<float> mul((size_t)O);
    int ty;
    if (qf != nullptr && ep.pre_residual_value != nullptr && ep.pre_residual_value != outv &&
        qentry(ep.pre_residual_value) != nullptr)
      OHIP_INFO("int8 plan: the quant-table entry of '%s' is not used - the residual Add behind it is fused and the "
                "convolution requantises once, to the entry of '%s'", ep.pre_residual_value->name.c_str(), outv->name.c_str());
    if (qf != nullptr) {
      // One requantisation per convolution, whatever is fused behind it: the result
      // (after the residual add and the ReLU, if any) takes the scale and zero point
      // of the last fused value.
      for (int64_t o = 0; o < O; ++o) mul[o] = (sx * sw[o]) / qf->scale;
      ip.out_dt = DT_I8;
      ip.q_add = (float)qf->zp;
      ip.q_lo = ep.act == ACT_RELU ? (float)qf->zp : 0.f;
      ty = new_tensor(DT_I8, L_NHWC, outv->shape, (int)O, SP_ARENA);
      set_quant(ty, true, qf->scale, qf->zp);
    } else if (comp_->opts.raw_acc && ep.residual == nullptr && ep.act == ACT_NONE) {
      ip.out_dt = DT_I32;
      ty = new_tensor(DT_I32, L_NHWC, outv->shape, (int)O, SP_ARENA);
    } else {
      if (ep.residual != nullptr) fail(ODLA_UNSUPPORTED_OP, "int8 residual fusion needs quant entries for '%s'", outv->name.c_str());
      for (int64_t o = 0; o < O; ++o) mul[o] = sx * sw[o];
      ip.out_dt = DT_F32;
      ip.act = ep.act; ip.act_a = ep.act_a; ip.act_b = ep.act_b;
      ty = new_tensor(DT_F32, L_NHWC, outv->shape, (int)O, SP_ARENA);
    }
    ip.ycs = (int)O;
    const int tm = const_vector<float>(DT_F32, mul);
    int tr = -1;
    if (ep.residual) {
      tr = get(ep.residual, L_NHWC, FORM_QUANT);
      ip.rcs = T(tr).cs;
      // the residual's levels enter as fma(float(r), r_mul, r_add), r_add carrying both zero points
      const QuantEntry* qy = qentry(outv);
      ip.r_mul = T(tr).qscale / qy->scale;
      ip.r_add = (float)qy->zp - (float)T(tr).qzp * ip.r_mul;
    }
    ip.stream_out = T(ty).bytes >= stream_out_bytes();
    const int tf = make_wfrag("conv.i8:" + outv->name, &ip, tw);
    const bool hf = tf >= 0;
    log_igemm_choice("conv.i8:" + outv->name, ip, hf, tr >= 0);
    const Ref rf = ref(hf ? tf : tx);
    const Ref rx = ref(tx), rw = ref(tw), ry = ref(ty), rb = ref(tb), rm = ref(tm), rr = ref(tr >= 0 ? tr : tx);
    const bool hr = tr >= 0;
    const auto prod = fuse_prods_.find(x);
    if (prod != fuse_prods_.end() && !in_init_ && hf && !hr && ip.out_dt == DT_I8 && tx == prod->second.ty &&
        igemm_stream_q8_fusable(prod->second.ip, ip)) {
      // This layer reads the result of the step before it pixel by pixel: that step computes it
      // too, from its staged tiles, and writes both results - one launch and one pass over the
      // wide tensor less.
      const FuseProducer fp = prod->second;
      fuse_prods_.erase(prod);   // (one rider per launch)
      IgemmParams fa = fp.ip;
      fa.f_kout = ip.Kout; fa.f_ycs = ip.ycs; fa.f_wf_chunks = ip.wf_chunks;
      fa.f_q_add = ip.q_add; fa.f_q_lo = ip.q_lo;
      const Ref ax = ref(fp.tx), aw = ref(fp.tw), ay = ref(fp.ty), ab = ref(fp.tb), am = ref(fp.tm), af = ref(fp.tf);
      const Ref ar = ref(fp.tr >= 0 ? fp.tr : fp.tx);
      const bool ahr = fp.tr >= 0;
      Step& sa = plan_->steps[(size_t)fp.step];
      OHIP_INFO("int8 plan: '%s' is computed in the launch of '%s' (from its tiles in LDS)", outv->name.c_str(), sa.name.c_str());
      sa.name += "+" + outv->name;
      sa.fn = [=](const ExecEnv& e, hipStream_t st) {
        IgemmParams p = fa;
        p.x = ax(e); p.w = aw(e); p.y = ay(e); p.bias = ab(e);
        p.qmul = (const float*)am(e);
        p.residual = ahr ? ar(e) : nullptr;
        p.w_frag = af(e);
        p.f_wfrag = rf(e); p.f_bias = rb(e); p.f_qmul = (const float*)rm(e); p.f_y = ry(e);
        return launch_igemm(p, st);
      };
      {  // the second result is written by that step
        PTensor& yt = T(root(ty));
        if (yt.space == SP_ARENA) {
          if (fp.step < yt.def_step) yt.def_step = fp.step;
          if (fp.step > yt.last_step) yt.last_step = fp.step;
        }
        arena_only_.insert(root(ty));
      }
      set_main(outv, ty);
      return;
    }
    emit("conv.i8:" + outv->name, {tx, tw, tr}, {ty}, [=](const ExecEnv& e, hipStream_t st) {
      IgemmParams p = ip;
      p.x = rx(e); p.w = rw(e); p.y = ry(e); p.bias = rb(e);
      p.qmul = (const float*)rm(e);
      p.residual = hr ? rr(e) : nullptr;
      p.w_frag = hf ? rf(e) : nullptr;
      return launch_igemm(p, st);
    });
    if (!in_init_ && hf && ip.out_dt == DT_I8 && !calib_) {
      FuseProducer& fp = fuse_prods_[outv];
      fp.step = (int)plan_->steps.size() - 1;
      fp.out = outv;
      fp.ip = ip;
      fp.tx = tx; fp.tw = tw; fp.ty = ty; fp.tb = tb; fp.tm = tm; fp.tr = tr; fp.tf = tf;
    }
    if (ip.out_dt == DT_I32) {
      // raw accumulators are exposed through the FLOAT32-typed value as bit patterns
      T(ty).dt = DT_F32;
    }
    if (ip.out_dt == DT_F32 && cdt_ != DT_F32) {
      const int tc = new_tensor(cdt_, L_NHWC, outv->shape, (int)O, SP_ARENA);
      const int64_t ne = T(ty).phys_elems();
      const Ref a = ref(ty), b = ref(tc);
      const DType ddt = cdt_;
      emit("cast:" + outv->name, {ty}, {tc}, [=](const ExecEnv& e, hipStream_t st) { return launch_cast(a(e), DT_F32, b(e), ddt, ne, st); });
      ty = tc;
    }
    set_main(outv, ty);
    return;
  }

  // ---- floating-point path ----
  const DType dt = mm_dtype(x);
  if (!dtype_is_float(dt)) fail(ODLA_UNSUPPORTED_DATATYPE, "odla_Conv on element type %d", (int)x->etype);
  // a result with a residual takes the residual's (storage) type
  const DType odt = ep.residual != nullptr ? storage_dtype(outv) : result_dtype(outv);
  const int vec = 16 / dtype_size(dt);
  int tx;
  int xcs;
  if (cl) {
    tx = get(x, L_ROWMAJOR, FORM_OPERAND);
    xcs = (int)C;
  } else {
    tx = tx_s2d >= 0 ? tx_s2d : get(x, L_NHWC, FORM_OPERAND, vec);
    xcs = T(tx).cs;
  }
  if (T(tx).dt != dt) fail(ODLA_INTERNAL_LOGIC_ERR, "conv input storage type mismatch");
  // Groups with fewer channels than one 16-byte K vector run as one dense
  // convolution over block-diagonal weights (zero outside each group's block).
  const bool densify = G > 1 && Cg % vec != 0;
  const int Ge = densify ? 1 : G, Oge = densify ? (int)O : Og;
  int Cp;
  if (Ge == 1) {
    if (xcs % vec != 0) fail(ODLA_UNSUPPORTED_OP, "channels-last convolution input with %d channels needs a multiple of %d", xcs, vec);
    Cp = xcs;
  } else {
    Cp = Cg;
  }
  int w_rs = 0;
  const int tw = densify ? pack_weights(kpack, dt, 1, (int)O, (int)C, (int)R, (int)S, Cp, so, si, sr, ss, ep.row_scale,
                                        &w_rs, nullptr, G)
                         : pack_weights(kpack, dt, G, Og, Cg, (int)R, (int)S, Cp, so, si, sr, ss, ep.row_scale, &w_rs,
                                        nullptr);

  IgemmParams ip;
  ip.N = (int)N; ip.H = (int)H; ip.W = (int)W; ip.C = Cp; ip.xcs = xcs;
  ip.Ho = (int)Ho; ip.Wo = (int)Wo; ip.Kout = Oge;
  ip.R = (int)R; ip.S = (int)S; ip.sh = str_h; ip.sw = str_w;
  ip.dh = dil_h; ip.dw = dil_w; ip.ph = pad_t; ip.pw = pad_l;
  ip.w_rows = Oge; ip.w_cols = w_rs; ip.w_rs = w_rs;
  ip.in_dt = dt; ip.out_dt = odt;
  ip.batch = Ge;
  ip.alpha = ep.scalar;
  if (Ge > 1) { ip.x_bs = Cg; ip.w_bs = (int64_t)Og * w_rs; ip.y_bs = Og; ip.r_bs = Og; ip.bias_bs = Og; }
  ip.ycs = (int)O;

  int ty;
  if (cl) ty = new_tensor(odt, L_ROWMAJOR, outv->shape, 0, SP_ARENA);
  else ty = new_tensor(odt, L_NHWC, outv->shape, (int)O, SP_ARENA);

  if (runtime_bias) {
    // bias supplied at run time: read it as fp32 from its staging tensor
    const VState& bs = vs_[bias->index];
    if (bs.main < 0 || T(bs.main).dt != DT_F32) fail(ODLA_UNSUPPORTED_OP, "run-time conv bias must be FLOAT32");
    const int tb = bs.main;
    const Ref rx = ref(tx), rw = ref(tw), ry = ref(ty), rb = ref(tb);
    emit("conv:" + outv->name, {tx, tw, tb}, {ty}, [=](const ExecEnv& e, hipStream_t st) {
      IgemmParams p = ip;
      p.x = rx(e); p.w = rw(e); p.y = ry(e); p.bias = rb(e);
      return launch_igemm(p, st);
    });
  } else {
    finish_igemm("conv:" + outv->name, ip, tx, tw, ty, ep, O);
  }
  set_main(outv, ty);
}

// ---------------------------------------------------------------- Gemm ----
// Bias operand of a Gemm node (alpha*(A.B) + beta*C) and the operators folded
// behind it.  Returns false when C is a run-time matrix (then it rides as the
// residual and nothing else is folded).
bool Planner::gemm_epilogue(int ni, Epilogue* ep) {
  Node& n = comp_->nodes[ni];
  const _odla_value* Cv = n.in[2];
  const Shape& os = n.out->shape;
  const int64_t Nn = os.d[os.rank - 1];
  const float beta = n.f[1];
  _odla_value* full_c = nullptr;
  if (Cv != nullptr && beta != 0.f) {
    const int64_t cn = Cv->shape.numel();
    if (Cv->kind == _odla_value::CONSTANT && (cn == 1 || cn == Nn)) {
      std::vector<float> c = const_as_float(Cv);
      ep->bias.assign((size_t)Nn, 0.f);
      for (int64_t j = 0; j < Nn; ++j) ep->bias[j] = beta * c[cn == 1 ? 0 : j];
      ep->has_bias = true;
    } else if (beta == 1.f && Cv->shape == os && Cv->kind != _odla_value::CONSTANT) {
      full_c = const_cast<_odla_value*>(Cv);
    } else {
      fail(ODLA_UNSUPPORTED_OP, "odla_Gemm: C operand of shape %s with beta %g is not supported", Cv->shape.str().c_str(), beta);
    }
  }
  if (full_c == nullptr) collect_epilogue(ni, Nn, os.rank - 1, ep);
  else { ep->residual = full_c; ep->final_value = n.out; }
  return full_c == nullptr;
}

bool Planner::head_split_behind(const _odla_value* v, int64_t rows, int64_t cols, HeadSplit* hs) const {
  if (calib_ || v == nullptr || v->is_output || consumers_[v->index].size() != 1) return false;
  const int ri = consumers_[v->index][0];
  const Node& r = comp_->nodes[ri];
  if (r.op != OP_RESHAPE || r.absorbed || r.out->is_output || r.out->shape.rank != 4) return false;
  const Shape& s4 = r.out->shape;
  if (s4.d[0] * s4.d[1] != rows || s4.d[2] * s4.d[3] != cols || s4.d[3] % 8 != 0) return false;
  if (consumers_[r.out->index].size() != 1) return false;
  const int ti = consumers_[r.out->index][0];
  const Node& t = comp_->nodes[ti];
  if (t.op != OP_TRANSPOSE || t.absorbed || t.out->is_output || t.iv.size() != 4) return false;
  if (t.iv[0] != 0 || t.iv[1] != 2 || t.iv[2] != 1 || t.iv[3] != 3) return false;
  hs->reshape = ri; hs->transpose = ti;
  hs->B = s4.d[0]; hs->S = s4.d[1]; hs->heads = s4.d[2]; hs->d = s4.d[3];
  hs->out = t.out;
  return true;
}

int Planner::head_merge_behind(const _odla_value* v) const {
  if (calib_ || v == nullptr || v->is_output || v->shape.rank != 4 || consumers_[v->index].size() != 1) return -1;
  const int ti = consumers_[v->index][0];
  const Node& t = comp_->nodes[ti];
  if (t.op != OP_TRANSPOSE || t.absorbed || t.iv.size() != 4) return -1;
  if (t.iv[0] != 0 || t.iv[1] != 2 || t.iv[2] != 1 || t.iv[3] != 3) return -1;
  return ti;
}

// q . k^T -> [scalar Mul / Div] -> [+ mask] -> Softmax -> . v (-> head merge): the attention block
// of an encoder layer as ONE launch [ref: the reference's compiler matches the same block,
// lib/transforms/fusion.cc:315-348].  `ni` is the q . k^T product; on success every node of the
// block is marked as done and the block's result exists.
bool Planner::try_fused_attention(int ni) {
  if (calib_ || comp_->opts.int8) return false;
  Node& n = comp_->nodes[ni];
  const _odla_value* Q = n.in[0];
  const _odla_value* K = n.in[1];
  if (Q == nullptr || K == nullptr || (n.in.size() > 2 && n.in[2] != nullptr)) return false;
  if (n.i[0] != 0 || n.i[1] == 0) return false;   // q . k^T
  const Shape& qs = Q->shape;
  if (qs.rank != 4 || !(K->shape == qs) || Q->kind == _odla_value::CONSTANT || K->kind == _odla_value::CONSTANT) return false;
  const int64_t B = qs.d[0], heads = qs.d[1], S = qs.d[2], d = qs.d[3];
  const DType dt = mm_dtype(Q);
  if (mm_dtype(K) != dt || !available(Q) || !available(K)) return false;
  auto sole_reader = [&](const _odla_value* v) -> int {
    if (v->is_output || consumers_[v->index].size() != 1) return -1;
    const int c = consumers_[v->index][0];
    return comp_->nodes[c].absorbed ? -1 : c;
  };
  std::vector<int> block;   // nodes behind `ni` that the launch covers
  float scale = n.f[0];
  const _odla_value* cur = n.out;
  int ci = sole_reader(cur);
  if (ci < 0) return false;
  // a scalar factor (scores / sqrt(d))
  if (comp_->nodes[ci].op == OP_BINARY && (comp_->nodes[ci].i[0] == BIN_MUL || comp_->nodes[ci].i[0] == BIN_DIV)) {
    const Node& m = comp_->nodes[ci];
    const bool lhs = m.in[0] == cur;
    const _odla_value* other = lhs ? m.in[1] : m.in[0];
    if (other == cur || other->kind != _odla_value::CONSTANT || other->shape.numel() != 1 || !(m.out->shape == cur->shape)) return false;
    const float c = const_as_float(other)[0];
    if (m.i[0] == BIN_DIV) {
      if (!lhs || c == 0.f) return false;
      scale *= 1.0f / c;
    } else {
      scale *= c;
    }
    block.push_back(ci);
    cur = m.out;
    if ((ci = sole_reader(cur)) < 0) return false;
  }
  // an additive mask: one row of S values per batch entry (or one for all)
  const _odla_value* mask = nullptr;
  int64_t mask_bs = 0;
  if (comp_->nodes[ci].op == OP_BINARY && comp_->nodes[ci].i[0] == BIN_ADD) {
    const Node& a = comp_->nodes[ci];
    const bool lhs = a.in[0] == cur;
    const _odla_value* other = lhs ? a.in[1] : a.in[0];
    const int r = (int)a.iv[0];
    if (other == cur || r != 4 || !(a.out->shape == cur->shape) || !available(other)) return false;
    int64_t al[4];
    for (int i = 0; i < 4; ++i) al[i] = a.iv[1 + (lhs ? r : 0) + i];
    if ((al[0] != B && al[0] != 1) || al[1] != 1 || al[2] != 1 || al[3] != S) return false;
    const DType mdt = storage_dtype(other);
    if (mdt != dt && mdt != DT_F32) return false;
    mask = other;
    mask_bs = al[0] == 1 ? 0 : S;
    block.push_back(ci);
    cur = a.out;
    if ((ci = sole_reader(cur)) < 0) return false;
  }
  {
    const Node& sm = comp_->nodes[ci];
    if (sm.op != OP_SOFTMAX || (int)sm.i[0] != 3 || sm.i[1] != 0) return false;
    block.push_back(ci);
    cur = sm.out;
    if ((ci = sole_reader(cur)) < 0) return false;
  }
  const Node& g2 = comp_->nodes[ci];
  if (g2.op != OP_GEMM || g2.in[0] != cur || g2.i[0] != 0 || g2.i[1] != 0 || g2.f[0] != 1.f ||
      (g2.in.size() > 2 && g2.in[2] != nullptr))
    return false;
  const _odla_value* V = g2.in[1];
  if (V == nullptr || !(V->shape == qs) || V->kind == _odla_value::CONSTANT || mm_dtype(V) != dt || !available(V)) return false;
  if (gemm_ep_ahead_.count(ci) || (ci < (int)gemm_merged_.size() && gemm_merged_[ci])) return false;
  block.push_back(ci);
  _odla_value* fv = g2.out;
  const int ti = head_merge_behind(fv);   // [B, heads, S, d] -> [B, S, heads, d] behind it: stored that way
  if (ti >= 0) fv = comp_->nodes[ti].out;
  if (result_dtype(fv) != dt) return false;

  AttentionParams ap;
  ap.dt = dt;
  ap.mask_dt = mask != nullptr ? storage_dtype(mask) : dt;
  ap.B = (int)B; ap.heads = (int)heads; ap.S = (int)S; ap.d = (int)d;
  ap.scale = scale;
  ap.q_bs = ap.k_bs = ap.v_bs = heads * S * d;
  ap.q_hs = ap.k_hs = ap.v_hs = S * d;
  ap.q_rs = ap.k_rs = ap.v_rs = d;
  if (ti >= 0) { ap.o_bs = S * heads * d; ap.o_hs = d; ap.o_rs = heads * d; }
  else { ap.o_bs = heads * S * d; ap.o_hs = S * d; ap.o_rs = d; }
  ap.mask_bs = mask_bs;
  if (B * heads > 0x7fffffff || !attention_supported(ap)) return false;

  // ---- from here on the plan changes
  const int tq = get(Q, L_ROWMAJOR, FORM_OPERAND), tk = get(K, L_ROWMAJOR, FORM_OPERAND), tv = get(V, L_ROWMAJOR, FORM_OPERAND);
  const int tm = mask != nullptr ? get(mask, L_ROWMAJOR, FORM_FLOAT) : -1;
  if (T(tq).dt != dt || T(tk).dt != dt || T(tv).dt != dt || (tm >= 0 && T(tm).dt != ap.mask_dt))
    fail(ODLA_INTERNAL_LOGIC_ERR, "attention operand storage type mismatch ('%s')", fv->name.c_str());
  const int ty = new_tensor(dt, L_ROWMAJOR, fv->shape, 0, SP_ARENA);
  const Ref rq = ref(tq), rk = ref(tk), rv = ref(tv), ry = ref(ty), rm = ref(tm >= 0 ? tm : tq);
  const bool hm = tm >= 0;
  emit("attention:" + fv->name, {tq, tk, tv, tm}, {ty}, [=](const ExecEnv& e, hipStream_t st) {
    AttentionParams p = ap;
    p.q = rq(e); p.k = rk(e); p.v = rv(e); p.out = ry(e);
    p.mask = hm ? rm(e) : nullptr;
    return launch_attention(p, st);
  });
  for (int j : block) comp_->nodes[j].absorbed = true;
  if (ti >= 0) comp_->nodes[ti].absorbed = true;
  set_main(fv, ty);
  return true;
}

void Planner::lower_gemm(int ni) {
  if (ni < (int)gemm_merged_.size() && gemm_merged_[ni]) return;  // computed by an earlier sibling's launch
  if (try_fused_attention(ni)) return;
  Node& n = comp_->nodes[ni];
  const _odla_value* A = n.in[0];
  const _odla_value* B = n.in[1];
  const bool tA = n.i[0] != 0, tB = n.i[1] != 0;
  const Shape& as = A->shape;
  const Shape& bs = B->shape;
  const Shape& os = n.out->shape;
  const int64_t M = os.d[os.rank - 2], Nn = os.d[os.rank - 1];
  const int64_t K = tA ? as.d[as.rank - 2] : as.d[as.rank - 1];
  int64_t lead = 1;
  for (int i = 0; i < as.rank - 2; ++i) lead *= as.d[i];
  const bool shared_b = bs.rank == 2;
  const DType dt = mm_dtype(A);
  if (!dtype_is_float(dt)) fail(ODLA_UNSUPPORTED_DATATYPE, "odla_Gemm on element type %d", (int)A->etype);
  const int vec = 16 / dtype_size(dt);

  Epilogue ep;
  const float alpha = n.f[0];
  bool plain_c = true;
  {
    auto ahead = gemm_ep_ahead_.find(ni);
    if (ahead != gemm_ep_ahead_.end()) { ep = ahead->second; gemm_ep_ahead_.erase(ahead); }
    else plain_c = gemm_epilogue(ni, &ep);
  }
  _odla_value* outv = ep.final_value;
  // a result with a residual takes the residual's (storage) type
  const DType odt = ep.residual != nullptr ? storage_dtype(outv) : result_dtype(outv);

  // ---- sibling GEMMs: the same left operand against several constant matrices
  // of one shape (the query / key / value projections of an attention block),
  // each too small to fill the chip.  They run as ONE batched launch whose
  // batch stride on the left operand is zero; every result is a slice of the
  // launch's output.
  std::vector<int> group;  // node indices, this one first
  std::vector<Epilogue> group_ep;
  {
    const int es0 = dtype_size(dt);
    const int64_t rows = lead * M;
    const int64_t tiles = ((rows + 127) / 128) * ((Nn + 127) / 128);
    auto simple = [&](const Epilogue& e) {
      return e.residual == nullptr && e.row_scale.empty() && e.final_value != nullptr &&
             result_dtype(e.final_value) == odt && !e.final_value->is_output;
    };
    if (!calib_ && plain_c && B->kind == _odla_value::CONSTANT && shared_b && !tA && K % vec == 0 && Nn % 32 == 0 &&
        A->kind != _odla_value::CONSTANT && tiles <= 512 && (int64_t)K * es0 >= 256 && simple(ep)) {
      group.push_back(ni);
      group_ep.push_back(ep);
      for (int mi = ni + 1; mi < (int)comp_->nodes.size() && group.size() < 8; ++mi) {
        Node& m = comp_->nodes[mi];
        if (m.op != OP_GEMM || m.absorbed || m.in[0] != A || (m.i[0] != 0) != tA || (m.i[1] != 0) != tB) continue;
        if (m.f[0] != alpha || m.in[1] == nullptr || m.in[1]->kind != _odla_value::CONSTANT) continue;
        if (!(m.in[1]->shape == bs) || !(m.out->shape == os) || m.out->etype != n.out->etype) continue;
        if (gemm_ep_ahead_.count(mi) || (mi < (int)gemm_merged_.size() && gemm_merged_[mi])) continue;
        Epilogue em;
        const bool plain = gemm_epilogue(mi, &em);
        if (plain && simple(em) && em.act == ep.act && em.act_a == ep.act_a && em.act_b == ep.act_b &&
            em.scalar == ep.scalar && em.res_after_act == ep.res_after_act) {
          group.push_back(mi);
          group_ep.push_back(em);
        } else {
          gemm_ep_ahead_[mi] = em;  // folded nodes are marked already: keep what was collected for its own turn
        }
      }
      if (group.size() < 2) { group.clear(); group_ep.clear(); }
    }
  }

  // ---- A operand: row-major [lead][M][K], K padded to the vector width ----
  int ta = get(A, L_ROWMAJOR, FORM_OPERAND);
  if (T(ta).dt != dt) fail(ODLA_INTERNAL_LOGIC_ERR, "gemm input storage type mismatch");
  int Kp = round_up_i((int)K, vec);
  if (tA || Kp != K) {
    // materialise A^T and/or zero-pad K
    Shape s2;
    s2.rank = 3;
    s2.d[0] = lead; s2.d[1] = M; s2.d[2] = Kp;
    const int t2 = new_tensor(dt, L_ROWMAJOR, s2, 0, SP_ARENA);
    if (Kp != K) {
      const Ref b = ref(t2);
      const int64_t words = (int64_t)(T(t2).bytes / 4);
      emit("gemm.zero:" + outv->name, {}, {t2}, [=](const ExecEnv& e, hipStream_t st) { return launch_fill_i32((int32_t*)b(e), words, 0, st); });
    }
    StridedCopyParams cp;
    cp.elem_size = dtype_size(dt);
    cp.rank = 3;
    cp.dims[0] = lead; cp.dims[1] = M; cp.dims[2] = K;
    cp.sy[0] = M * Kp; cp.sy[1] = Kp; cp.sy[2] = 1;
    cp.sx[0] = M * K; cp.sx[1] = tA ? 1 : K; cp.sx[2] = tA ? M : 1;
    strided_copy_step("gemm.a:" + outv->name, ta, t2, cp);
    ta = t2;
  }

  IgemmParams ip;
  ip.H = 1; ip.W = 1; ip.Ho = 1; ip.Wo = 1;
  ip.C = Kp; ip.xcs = Kp;
  ip.Kout = (int)Nn;
  ip.in_dt = dt; ip.out_dt = odt;
  ip.alpha = alpha * ep.scalar;
  ip.ycs = (int)Nn;
  int tw;
  if (!group.empty()) {
    const int G = (int)group.size();
    // one constant [G*N][K] matrix (row n of matrix g = column n of B_g) packed like any other
    auto buf = std::make_unique<std::vector<uint8_t>>((size_t)G * Nn * K * sizeof(float));
    float* wcat = reinterpret_cast<float*>(buf->data());
    std::vector<float> bias_all((size_t)G * Nn, 0.f);
    bool any_bias = false;
    for (int g = 0; g < G; ++g) {
      const std::vector<float> bg = const_as_float(comp_->nodes[group[g]].in[1]);
      for (int64_t nn = 0; nn < Nn; ++nn)
        for (int64_t k = 0; k < K; ++k)
          wcat[((int64_t)g * Nn + nn) * K + k] = tB ? bg[nn * K + k] : bg[k * Nn + nn];
      if (group_ep[g].has_bias) {
        any_bias = true;
        for (int64_t nn = 0; nn < Nn && nn < (int64_t)group_ep[g].bias.size(); ++nn) bias_all[(size_t)(g * Nn + nn)] = group_ep[g].bias[nn];
      }
    }
    _odla_value kcat;
    kcat.kind = _odla_value::CONSTANT;
    kcat.name = B->name;
    kcat.etype = ODLA_FLOAT32;
    kcat.shape.rank = 2;
    kcat.shape.d[0] = (int64_t)G * Nn; kcat.shape.d[1] = K;
    kcat.host_data = wcat;
    comp_->owned_data.push_back(std::move(buf));
    int w_rs = 0;
    const int twc = pack_weights(&kcat, dt, 1, (int)(G * Nn), (int)K, 1, 1, Kp, K, 1, 0, 0, {}, &w_rs, nullptr);
    ip.w_rows = (int)Nn; ip.w_cols = w_rs; ip.w_rs = w_rs;
    ip.N = (int)(lead * M);
    ip.batch = G;
    ip.x_bs = 0; ip.w_bs = Nn * w_rs; ip.y_bs = lead * M * Nn; ip.bias_bs = Nn;
    Shape all;
    all.rank = 3;
    all.d[0] = G; all.d[1] = lead * M; all.d[2] = Nn;
    const int tall = new_tensor(odt, L_ROWMAJOR, all, 0, SP_ARENA);
    Epilogue eall = ep;
    eall.has_bias = any_bias;
    eall.bias = bias_all;
    // Every member feeds Reshape -> Transpose into [B, heads, S, d] (the head split of an
    // attention block): the launch stores that order itself and the transposes vanish.
    std::vector<HeadSplit> hs((size_t)G);
    bool split = true;
    for (int g = 0; g < G && split; ++g) {
      split = head_split_behind(group_ep[g].final_value, lead * M, Nn, &hs[g]);
      if (split && g > 0) split = hs[g].S == hs[0].S && hs[g].d == hs[0].d && hs[g].heads == hs[0].heads;
    }
    if (split) {
      ip.y_rdiv = (int)hs[0].S; ip.y_rlo = hs[0].d; ip.y_rhi = hs[0].heads * hs[0].S * hs[0].d;
      ip.y_cdiv = (int)hs[0].d; ip.y_chi = hs[0].S * hs[0].d;
    }
    finish_igemm("gemm.x" + std::to_string(G) + ":" + outv->name, ip, ta, twc, tall, eall, (int64_t)G * Nn);
    if (gemm_merged_.size() < comp_->nodes.size()) gemm_merged_.resize(comp_->nodes.size(), 0);
    const size_t slice_bytes = (size_t)(lead * M * Nn) * dtype_size(odt);
    for (int g = 0; g < G; ++g) {
      if (split) {
        set_main(hs[g].out, view_tensor(tall, hs[g].out->shape, (size_t)g * slice_bytes));
        comp_->nodes[hs[g].reshape].absorbed = true;
        comp_->nodes[hs[g].transpose].absorbed = true;
      } else {
        set_main(group_ep[g].final_value, view_tensor(tall, group_ep[g].final_value->shape, (size_t)g * slice_bytes));
      }
      if (g > 0) gemm_merged_[group[g]] = 1;
    }
    return;
  }
  if (B->kind == _odla_value::CONSTANT && (shared_b || lead == 1)) {
    // weights: pack once.  B[k][n] (so=1, si=N) or B^T[n][k] (so=K, si=1)
    int w_rs = 0;
    const int64_t so = tB ? K : 1, si = tB ? 1 : Nn;
    tw = pack_weights(B, dt, 1, (int)Nn, (int)K, 1, 1, Kp, so, si, 0, 0, ep.row_scale, &w_rs, nullptr);
    ip.w_rows = (int)Nn; ip.w_cols = w_rs; ip.w_rs = w_rs;
    ip.N = (int)(lead * M);
    ip.batch = 1;
    // Few output tiles and a long K (classifier heads): the tiles would walk K
    // one after the other on a handful of CUs.  Split K into independent
    // problems (grid.z) that write fp32 partial sums, then add them up.
    {
      const int es = dtype_size(dt);
      const int64_t rows = lead * M;
      const int64_t tiles = ((rows + 127) / 128) * ((Nn + 127) / 128);
      const int stage = 128 / es;  // K elements per 128-byte stage
      int splits = 1;
      if (!calib_ && ep.residual == nullptr && ep.act == ACT_NONE && tiles <= 64 && (int64_t)Kp * es >= 2048) {
        while (splits < 16 && Kp % (splits * 2 * stage) == 0 && Kp / (splits * 2) >= 4 * stage && tiles * splits * 2 <= 1024)
          splits *= 2;
      }
      if (splits > 1) {
        const int Kc = Kp / splits;
        Shape ps;
        ps.rank = 3;
        ps.d[0] = splits; ps.d[1] = rows; ps.d[2] = Nn;
        const int tp = new_tensor(DT_F32, L_ROWMAJOR, ps, 0, SP_ARENA);
        int tb = -1;
        if (ep.has_bias) {  // the first partial carries the bias
          std::vector<float> b((size_t)splits * Nn, 0.f);
          for (int64_t i = 0; i < Nn && i < (int64_t)ep.bias.size(); ++i) b[(size_t)i] = ep.bias[(size_t)i];
          tb = const_vector<float>(DT_F32, b);
        }
        IgemmParams sp = ip;
        sp.C = Kc;
        sp.w_cols = Kc;
        sp.batch = splits;
        sp.x_bs = Kc; sp.w_bs = Kc; sp.y_bs = rows * Nn; sp.bias_bs = Nn;
        sp.out_dt = DT_F32;
        const Ref rx = ref(ta), rw = ref(tw), rp = ref(tp), rb = ref(tb >= 0 ? tb : ta);
        const bool hb = tb >= 0;
        emit("gemm.splitk:" + outv->name, {ta, tw}, {tp}, [=](const ExecEnv& e, hipStream_t st) {
          IgemmParams p = sp;
          p.x = rx(e); p.w = rw(e); p.y = rp(e);
          p.bias = hb ? rb(e) : nullptr;
          return launch_igemm(p, st);
        });
        const int ty = new_tensor(odt, L_ROWMAJOR, outv->shape, 0, SP_ARENA);
        const Ref ry = ref(ty);
        const int64_t inner = rows * Nn;
        emit("gemm.sum:" + outv->name, {tp}, {ty}, [=](const ExecEnv& e, hipStream_t st) {
          return launch_reduce(rp(e), ry(e), DT_F32, odt, 1, splits, inner, RED_SUM, st);
        });
        set_main(outv, ty);
        return;
      }
    }
  } else {
    if (!ep.row_scale.empty()) fail(ODLA_UNSUPPORTED_OP, "odla_Gemm: scale folding into a run-time operand");
    int tb = get(B, L_ROWMAJOR, FORM_OPERAND);
    if (T(tb).dt != dt) fail(ODLA_INTERNAL_LOGIC_ERR, "gemm operand storage type mismatch");
    const int64_t blead = shared_b ? 1 : lead;
    if (!tB || Kp != K) {
      // need [blead][N][Kp]
      Shape s2;
      s2.rank = 3;
      s2.d[0] = blead; s2.d[1] = Nn; s2.d[2] = Kp;
      const int t2 = new_tensor(dt, L_ROWMAJOR, s2, 0, SP_ARENA);
      if (Kp != K) {
        const Ref b = ref(t2);
        const int64_t words = (int64_t)(T(t2).bytes / 4);
        emit("gemm.zero:" + outv->name, {}, {t2}, [=](const ExecEnv& e, hipStream_t st) { return launch_fill_i32((int32_t*)b(e), words, 0, st); });
      }
      if (!tB) {
        // [blead][K][N] -> [blead][N][Kp]: LDS-tiled transpose
        const Ref a2 = ref(tb), b2 = ref(t2);
        const int es2 = dtype_size(dt), bl = (int)blead, Ki = (int)K, Ni = (int)Nn, Kpi = Kp;
        emit("gemm.b:" + outv->name, {tb}, {t2}, [=](const ExecEnv& e, hipStream_t st) {
          return launch_transpose2d(a2(e), b2(e), es2, bl, Ki, Ni, Kpi, st);
        });
      } else {
        StridedCopyParams cp;
        cp.elem_size = dtype_size(dt);
        cp.rank = 3;
        cp.dims[0] = blead; cp.dims[1] = Nn; cp.dims[2] = K;
        cp.sy[0] = Nn * Kp; cp.sy[1] = Kp; cp.sy[2] = 1;
        cp.sx[0] = K * Nn; cp.sx[1] = K; cp.sx[2] = 1;
        strided_copy_step("gemm.b:" + outv->name, tb, t2, cp);
      }
      tb = t2;
    }
    tw = tb;
    ip.w_rows = (int)Nn; ip.w_cols = Kp; ip.w_rs = Kp;
    if (shared_b) { ip.N = (int)(lead * M); ip.batch = 1; }
    else {
      ip.N = (int)M; ip.batch = (int)lead;
      ip.x_bs = M * Kp; ip.w_bs = Nn * Kp; ip.y_bs = M * Nn; ip.r_bs = M * Nn; ip.bias_bs = 0;
    }
  }
  if (ep.residual == nullptr) {
    HeadSplit hs;
    if (ip.batch == 1 && head_split_behind(outv, lead * M, Nn, &hs)) {
      // [B*S, heads*d] stored as [B, heads, S, d]: the Reshape -> Transpose behind it costs nothing
      ip.y_rdiv = (int)hs.S; ip.y_rlo = hs.d; ip.y_rhi = hs.heads * hs.S * hs.d;
      ip.y_cdiv = (int)hs.d; ip.y_chi = hs.S * hs.d;
      ip.out_dt = result_dtype(hs.out);
      const int ty = new_tensor(ip.out_dt, L_ROWMAJOR, hs.out->shape, 0, SP_ARENA);
      finish_igemm("gemm:" + outv->name, ip, ta, tw, ty, ep, Nn);
      set_main(hs.out, ty);
      comp_->nodes[hs.reshape].absorbed = true;
      comp_->nodes[hs.transpose].absorbed = true;
      return;
    }
    const int ti = ip.batch > 1 && os.rank == 4 && outv->shape == os ? head_merge_behind(outv) : -1;
    if (ti >= 0) {
      // a [B*heads] batch of [S, d] results stored as [B, S, heads, d]: the head merge behind
      // an attention block's context product
      Node& t = comp_->nodes[ti];
      const int64_t heads = os.d[1], S = os.d[2], d = os.d[3];
      ip.y_zdiv = (int)heads; ip.y_bs_hi = S * heads * d; ip.y_bs = d; ip.ycs = (int)(heads * d);
      ip.out_dt = result_dtype(t.out);
      const int ty = new_tensor(ip.out_dt, L_ROWMAJOR, t.out->shape, 0, SP_ARENA);
      finish_igemm("gemm:" + outv->name, ip, ta, tw, ty, ep, Nn);
      set_main(t.out, ty);
      t.absorbed = true;
      return;
    }
  }
  // A Softmax over the columns of a product with very few of them (a classifier head like
  // mnist_simple's Gemm -> Add -> Softmax): the one-wavefront-per-row kernel has every column of
  // its row in registers and finishes with it - one launch for the whole head.
  if (!calib_ && ep.residual == nullptr && ip.batch == 1 && dt == DT_F32 && odt == DT_F32 && ip.y_rdiv == 0 &&
      ip.y_zdiv == 0 && !outv->is_output && consumers_[outv->index].size() == 1) {
    Node& sm = comp_->nodes[consumers_[outv->index][0]];
    IgemmParams probe = ip;
    probe.act = ep.act;
    probe.ycs = ip.ycs > 0 ? ip.ycs : (int)Nn;
    if (sm.op == OP_SOFTMAX && !sm.absorbed && (int)sm.i[0] == sm.in[0]->shape.rank - 1 && sm.in[0] == outv &&
        result_dtype(sm.out) == DT_F32 && softmax_add_.find(outv->index) == softmax_add_.end() && gemm_rowdot_shape(probe)) {
      ip.row_softmax = sm.i[1] != 0 ? 2 : 1;
      sm.absorbed = true;
      const int ty = new_tensor(DT_F32, L_ROWMAJOR, sm.out->shape, 0, SP_ARENA);
      finish_igemm("gemm+softmax:" + sm.out->name, ip, ta, tw, ty, ep, Nn);
      set_main(sm.out, ty);
      return;
    }
  }
  const int ty = new_tensor(odt, L_ROWMAJOR, outv->shape, 0, SP_ARENA);
  finish_igemm("gemm:" + outv->name, ip, ta, tw, ty, ep, Nn);
  set_main(outv, ty);
}

// -------------------------------------------------------------- Binary ----
namespace {
// element stride of each logical dim of a physical tensor
void logical_strides(const PTensor& t, int64_t* st) {
  const Shape& s = t.shape;
  if (t.layout == L_NHWC) {
    st[0] = s.d[2] * s.d[3] * t.cs;
    st[1] = 1;
    st[2] = s.d[3] * t.cs;
    st[3] = t.cs;
    return;
  }
  int64_t acc = 1;
  for (int i = s.rank - 1; i >= 0; --i) { st[i] = acc; acc *= s.d[i]; }
}
}  // namespace

void Planner::lower_binary(int ni) {
  Node& n = comp_->nodes[ni];
  const _odla_value* a = n.in[0];
  const _odla_value* b = n.in[1];
  _odla_value* outv = n.out;
  const Shape& os = outv->shape;
  const int r = (int)n.iv[0];
  Shape sa, sb;
  sa.rank = sb.rank = r;
  for (int i = 0; i < r; ++i) { sa.d[i] = n.iv[1 + i]; sb.d[i] = n.iv[1 + r + i]; }
  const DType dt = storage_dtype(outv);

  // x + mask -> Softmax over the last axis (attention): the Softmax launch adds
  // the mask itself.  The mask must hold whole rows shared by a block of
  // consecutive rows of x: leading dims equal, then 1s, then the row length.
  if (!calib_ && n.i[0] == BIN_ADD && dtype_is_float(dt) && !outv->is_output && consumers_[outv->index].size() == 1 && r >= 2) {
    const Node& nx = comp_->nodes[consumers_[outv->index][0]];
    const int64_t len = os.d[r - 1];
    const int vecn = 16 / dtype_size(dt);
    if (nx.op == OP_SOFTMAX && !nx.absorbed && (int)nx.i[0] == r - 1 && len % vecn == 0 && len / vecn <= 256) {
      for (int side = 0; side < 2; ++side) {
        const _odla_value* xv = side == 0 ? a : b;
        const _odla_value* mv = side == 0 ? b : a;
        const Shape& sx = side == 0 ? sa : sb;
        const Shape& sm = side == 0 ? sb : sa;
        if (!(sx == os) || sm.d[r - 1] != len || storage_dtype(mv) != dt) continue;
        int p = 0;
        while (p < r - 1 && sm.d[p] == os.d[p]) ++p;
        bool ones = true;
        int64_t div = 1;
        for (int i = p; i < r - 1; ++i) { ones = ones && sm.d[i] == 1; div *= os.d[i]; }
        if (!ones) continue;
        softmax_add_[outv->index] = {xv, mv, div};
        return;  // nothing to launch here: lower_softmax picks it up
      }
    }
  }

  // optional trailing activation
  ActKind act = ACT_NONE;
  float act_a = 0.f, act_b = 0.f;
  const bool q8 = comp_->opts.int8 && q8_value(a) && q8_value(b) && a->shape == os && b->shape == os &&
                  (n.i[0] == BIN_ADD) && a->kind != _odla_value::CONSTANT && b->kind != _odla_value::CONSTANT;
  if (!calib_ && !outv->is_output && consumers_[outv->index].size() == 1) {
    Node& nx = comp_->nodes[consumers_[outv->index][0]];
    if (nx.op == OP_UNARY && !nx.absorbed) {
      const ActKind k = (ActKind)nx.i[0];
      if (k == ACT_RELU || (!q8 && (k == ACT_LEAKY || k == ACT_CLAMP))) {
        if (!q8 || qentry(nx.out) != nullptr) {
          act = k; act_a = nx.f[0]; act_b = nx.f[1];
          nx.absorbed = true;
          outv = nx.out;
        }
      }
    }
  }
  const QuantEntry* qo = qentry(outv);

  if (q8 && qo != nullptr) {
    // both operands 8-bit, same shape: stay in the quantised domain
    const Layout lay = (os.rank == 4 && vs_[a->index].slot[L_NHWC][FORM_QUANT] >= 0) ? L_NHWC : L_ROWMAJOR;
    const int ta = get(a, lay, FORM_QUANT);
    const int tb = get(b, lay, FORM_QUANT);
    if (lay == L_NHWC && T(ta).cs != T(tb).cs) fail(ODLA_UNSUPPORTED_OP, "quantised add of differently padded tensors");
    const int ty = new_tensor(DT_I8, lay, os, T(ta).cs, SP_ARENA);
    set_quant(ty, true, qo->scale, qo->zp);
    BinaryParams bp;
    bp.dt = DT_I8;
    bp.op = BIN_ADD;
    bp.rank = 1;
    bp.dims[0] = T(ta).phys_elems();
    bp.sa[0] = 1; bp.sb[0] = 1;
    bp.a_scale = T(ta).qscale; bp.a_zp = T(ta).qzp;
    bp.b_scale = T(tb).qscale; bp.b_zp = T(tb).qzp;
    bp.y_inv = 1.0f / qo->scale; bp.y_zp = qo->zp; bp.y_lo = act == ACT_RELU ? qo->zp : 0;
    const Ref ra = ref(ta), rb = ref(tb), ry = ref(ty);
    emit("add.q8:" + outv->name, {ta, tb}, {ty}, [=](const ExecEnv& e, hipStream_t st) {
      BinaryParams p = bp; p.a = ra(e); p.b = rb(e); p.y = ry(e);
      return launch_binary(p, st);
    });
    set_main(outv, ty);
    return;
  }

  if (!dtype_is_float(dt)) fail(ODLA_UNSUPPORTED_DATATYPE, "element-wise arithmetic on non-float values ('%s')", outv->name.c_str());
  // Output layout: channels-last if either full-size operand already lives that way.
  Layout lay = L_ROWMAJOR;
  if (os.rank == 4) {
    auto nhwc_main = [&](const _odla_value* v) {
      const VState& s = vs_[v->index];
      return v->shape == os && s.main >= 0 && T(s.main).layout == L_NHWC;
    };
    if (nhwc_main(a) || nhwc_main(b)) lay = L_NHWC;
  }
  auto operand = [&](const _odla_value* v, const Shape& aligned) -> int {
    // full-shape rank-4 operands follow the output layout; broadcast operands stay row-major
    if (lay == L_NHWC && v->shape == os) return get(v, L_NHWC, FORM_FLOAT);
    (void)aligned;
    return get(v, L_ROWMAJOR, FORM_FLOAT);
  };
  int ta = operand(a, sa), tb = operand(b, sb);
  int ocs = 0;
  if (lay == L_NHWC) {
    ocs = (int)os.d[1];
    if ((a->shape == os && T(ta).cs != ocs) || (b->shape == os && T(tb).cs != ocs)) {
      // a channels-last operand whose pixels are padded to a vector multiple: the
      // flat kernels assume dense rows, so this one runs on row-major copies
      lay = L_ROWMAJOR;
      ocs = 0;
      ta = get(a, L_ROWMAJOR, FORM_FLOAT);
      tb = get(b, L_ROWMAJOR, FORM_FLOAT);
    }
  }
  if (T(ta).dt != dt || T(tb).dt != dt) fail(ODLA_UNSUPPORTED_DATATYPE, "mixed storage types in element-wise op '%s'", outv->name.c_str());
  const int ty = new_tensor(dt, lay, os, ocs, SP_ARENA);

  // physical iteration order of the output and per-operand strides
  int order[ODLA_MAX_DIMENSION];
  int64_t odims[ODLA_MAX_DIMENSION];
  if (lay == L_NHWC) {
    order[0] = 0; order[1] = 2; order[2] = 3; order[3] = 1;
  } else {
    for (int i = 0; i < r; ++i) order[i] = i;
  }
  auto strides_for = [&](int t, const Shape& aligned, int64_t* st_phys) {
    // strides of the operand's own logical dims, mapped through the aligned shape
    PTensor pt = T(t);
    int64_t ls[ODLA_MAX_DIMENSION] = {0};
    if (pt.layout == L_NHWC) {
      logical_strides(pt, ls);
    } else {
      // the operand is row-major over its aligned shape (alignment only adds 1-dims)
      int64_t acc = 1;
      for (int i = r - 1; i >= 0; --i) { ls[i] = acc; acc *= aligned.d[i]; }
    }
    for (int i = 0; i < r; ++i) {
      const int ld = order[i];
      st_phys[i] = (aligned.d[ld] == 1 && os.d[ld] != 1) ? 0 : ls[ld];
      if (aligned.d[ld] == 1) st_phys[i] = 0;
    }
  };
  int64_t pa[ODLA_MAX_DIMENSION], pb[ODLA_MAX_DIMENSION];
  strides_for(ta, sa, pa);
  strides_for(tb, sb, pb);
  for (int i = 0; i < r; ++i) odims[i] = os.d[order[i]];
  // collapse to at most 6 dims by merging adjacent dims that are contiguous in all three
  BinaryParams bp;
  bp.dt = dt;
  bp.op = (BinKind)n.i[0];
  bp.act = act; bp.act_a = act_a; bp.act_b = act_b;
  {
    // output strides in physical order
    int64_t py[ODLA_MAX_DIMENSION];
    if (lay == L_NHWC) { py[0] = os.d[2] * os.d[3] * ocs; py[1] = os.d[3] * ocs; py[2] = ocs; py[3] = 1; }
    else { int64_t acc = 1; for (int i = r - 1; i >= 0; --i) { py[i] = acc; acc *= os.d[i]; } }
    std::vector<int64_t> d, xa, xb, xy;
    for (int i = 0; i < r; ++i) {
      if (odims[i] == 1) continue;
      if (!d.empty()) {
        const size_t l = d.size() - 1;
        const bool merge = xa[l] == pa[i] * odims[i] && xb[l] == pb[i] * odims[i] && xy[l] == py[i] * odims[i];
        if (merge) { d[l] *= odims[i]; xa[l] = pa[i]; xb[l] = pb[i]; xy[l] = py[i]; continue; }
      }
      d.push_back(odims[i]); xa.push_back(pa[i]); xb.push_back(pb[i]); xy.push_back(py[i]);
    }
    if (d.empty()) { d.push_back(1); xa.push_back(0); xb.push_back(0); xy.push_back(1); }
    if (d.size() > 6) fail(ODLA_UNSUPPORTED_OP, "element-wise op '%s' needs more than 6 broadcast dims", outv->name.c_str());
    // the kernel assumes a contiguous output over dims[]; that holds unless channel padding was dropped
    int64_t acc = 1;
    for (int i = (int)d.size() - 1; i >= 0; --i) {
      if (xy[i] != acc) fail(ODLA_UNSUPPORTED_OP, "element-wise op '%s' on a padded channels-last tensor", outv->name.c_str());
      acc *= d[i];
    }
    bp.rank = (int)d.size();
    for (size_t i = 0; i < d.size(); ++i) { bp.dims[i] = d[i]; bp.sa[i] = xa[i]; bp.sb[i] = xb[i]; }
  }
  const Ref ra = ref(ta), rb = ref(tb), ry = ref(ty);
  emit("binary:" + outv->name, {ta, tb}, {ty}, [=](const ExecEnv& e, hipStream_t st) {
    BinaryParams p = bp; p.a = ra(e); p.b = rb(e); p.y = ry(e);
    return launch_binary(p, st);
  });
  set_main(outv, ty);
}

// ------------------------------------------------- typed element-wise ----
// Integer arithmetic, comparisons, logic, predicates and Select: row-major
// operands, broadcast through per-dim element strides.
void Planner::lower_ewise(int ni) {
  Node& n = comp_->nodes[ni];
  const Shape& os = n.out->shape;
  const int r = (int)n.iv[0];
  const int nin = (int)n.in.size();
  const EwiseOp op = (EwiseOp)n.i[0];
  int tin[3] = {-1, -1, -1};
  int64_t st[3][ODLA_MAX_DIMENSION] = {{0}};
  for (int k = 0; k < nin; ++k) {
    tin[k] = get(n.in[k], L_ROWMAJOR, FORM_FLOAT);
    int64_t acc = 1;
    for (int i = r - 1; i >= 0; --i) {
      const int64_t d = n.iv[1 + k * r + i];
      st[k][i] = d == 1 ? 0 : acc;
      acc *= d;
    }
  }
  const DType odt = storage_dtype(n.out);
  // element type of the typed operands (Select: of the two branches)
  const DType dt = T(tin[op == EW_SELECT ? 1 : 0]).dt;
  for (int k = (op == EW_SELECT ? 1 : 0); k < nin; ++k)
    if (T(tin[k]).dt != dt) fail(ODLA_UNSUPPORTED_DATATYPE, "mixed storage types in element-wise op '%s'", n.out->name.c_str());
  const int ty = new_tensor(odt, L_ROWMAJOR, os, 0, SP_ARENA);
  EwiseParams ep;
  ep.dt = dt;
  ep.op = op;
  {
    // merge adjacent dims that are contiguous in every operand
    std::vector<int64_t> d, x[3];
    for (int i = 0; i < r; ++i) {
      if (os.d[i] == 1) continue;
      if (!d.empty()) {
        const size_t l = d.size() - 1;
        bool merge = true;
        for (int k = 0; k < nin; ++k) merge = merge && x[k][l] == st[k][i] * os.d[i];
        if (merge) {
          d[l] *= os.d[i];
          for (int k = 0; k < nin; ++k) x[k][l] = st[k][i];
          continue;
        }
      }
      d.push_back(os.d[i]);
      for (int k = 0; k < nin; ++k) x[k].push_back(st[k][i]);
    }
    if (d.empty()) { d.push_back(1); for (int k = 0; k < nin; ++k) x[k].push_back(0); }
    if (d.size() > 6) fail(ODLA_UNSUPPORTED_OP, "element-wise op '%s' needs more than 6 broadcast dims", n.out->name.c_str());
    ep.rank = (int)d.size();
    for (size_t i = 0; i < d.size(); ++i) {
      ep.dims[i] = d[i];
      ep.sa[i] = x[0][i];
      if (nin > 1) ep.sb[i] = x[1][i];
      if (nin > 2) ep.sc[i] = x[2][i];
    }
  }
  const Ref ra = ref(tin[0]), rb = ref(tin[nin > 1 ? 1 : 0]), rc = ref(tin[nin > 2 ? 2 : 0]), ry = ref(ty);
  emit("ewise:" + n.out->name, {tin[0], tin[1], tin[2]}, {ty}, [=](const ExecEnv& e, hipStream_t s) {
    EwiseParams p = ep;
    p.a = ra(e);
    if (nin > 1) p.b = rb(e);
    if (nin > 2) p.c = rc(e);
    p.y = ry(e);
    return launch_ewise(p, s);
  });
  set_main(n.out, ty);
}

// --------------------------------------------------------------- Unary ----
void Planner::lower_unary(int ni) {
  Node& n = comp_->nodes[ni];
  const _odla_value* x = n.in[0];
  const VState& s = vs_[x->index];
  const ActKind act = (ActKind)n.i[0];
  // 8-bit ReLU keeps the levels: q = max(q, zp), expressed as add-with-zero is
  // overkill; dequantise instead unless the producer fused it (the common case).
  Layout lay = L_ROWMAJOR;
  if (s.main >= 0 && !T(s.main).quant) lay = T(s.main).layout;
  else if (x->shape.rank == 4 && s.slot[L_NHWC][FORM_FLOAT] >= 0) lay = L_NHWC;
  else if (s.main >= 0 && T(s.main).quant) lay = T(s.main).layout;
  const int tx = get(x, lay, FORM_FLOAT);
  const PTensor px = T(tx);
  const int ty = new_tensor(px.dt, px.layout, n.out->shape, px.cs, SP_ARENA);
  const int64_t ne = px.phys_elems();
  const float fa = n.f[0], fb = n.f[1];
  const DType dt = px.dt;
  const Ref a = ref(tx), b = ref(ty);
  emit(std::string("unary:") + n.out->name, {tx}, {ty}, [=](const ExecEnv& e, hipStream_t st) {
    return launch_unary(a(e), b(e), dt, ne, act, fa, fb, st);
  });
  set_main(n.out, ty);
}

// ------------------------------------------- element-wise group fusion ----
// Float unary / binary operators on values of rank <= 3 (rank-4 values belong
// to the convolution epilogues and may live channels-last) that feed each other
// run as one launch: launch_fused_eltwise evaluates the whole group per element.
// Slices of available tensors become strided loads; a Concat of group results
// or a Transpose of one becomes a strided store.  The group is emitted at its
// first operator, so every outside operand must already be available there;
// whatever does not fit is left to the ordinary one-launch-per-operator path.
bool Planner::fuse_candidate(int ni) const {
  const Node& n = comp_->nodes[ni];
  if (n.absorbed || (!no_fuse_.empty() && no_fuse_[ni])) return false;
  if (n.op != OP_UNARY && n.op != OP_BINARY) return false;
  const Shape& os = n.out->shape;
  if (os.rank < 1 || os.rank > 3) return false;
  const DType dt = storage_dtype(n.out);
  if (!dtype_is_float(dt)) return false;
  for (const _odla_value* v : n.in)
    if (v == nullptr || storage_dtype(v) != dt || v->shape.rank > 3) return false;
  return true;
}

// A Slice met before the operators that read it: the first of them seeds the group.
bool Planner::fuse_slice_seed(int ni) const {
  const Node& n = comp_->nodes[ni];
  if (n.op != OP_SLICE || n.absorbed || n.out->is_output || consumers_[n.out->index].empty()) return false;
  if (n.out->shape.rank > 3 || !dtype_is_float(storage_dtype(n.out))) return false;
  return fuse_candidate(consumers_[n.out->index][0]);
}

// `seed`: the operator the group grows from; `from` <= seed: the node being
// lowered, where the group's launch is emitted.
static constexpr int64_t kTransposeSinkMax = 1 << 22;

bool Planner::lower_fused_group(int seed, int from) {
  const int n_nodes = (int)comp_->nodes.size();
  if (no_fuse_.empty()) no_fuse_.assign((size_t)n_nodes, 0);
  const int scan_end = std::min(n_nodes, seed + 512);
  const DType dt = storage_dtype(comp_->nodes[seed].out);

  // ---- operators and slices that could run at the seed's position
  std::unordered_map<const _odla_value*, int> member_of, slice_of;
  for (int j = from; j < scan_end; ++j) {
    const Node& n = comp_->nodes[j];
    if (n.absorbed) continue;
    if (n.op == OP_SLICE && n.out->shape.rank <= 3 && !n.out->is_output && storage_dtype(n.out) == dt &&
        dtype_is_float(dt) && available(n.in[0]) && !consumers_[n.out->index].empty()) {
      bool ok = true;
      for (int c : consumers_[n.out->index]) ok = ok && (comp_->nodes[c].op == OP_UNARY || comp_->nodes[c].op == OP_BINARY);
      if (ok) slice_of[n.out] = j;
      continue;
    }
    if (!fuse_candidate(j) || storage_dtype(n.out) != dt) continue;
    bool ok = true;
    for (const _odla_value* v : n.in) ok = ok && (member_of.count(v) || slice_of.count(v) || available(v));
    if (ok) member_of[n.out] = j;
  }
  {
    auto m = member_of.find(comp_->nodes[seed].out);
    if (m == member_of.end() || m->second != seed) return false;   // an operand of the seed is not ready here
  }
  // ---- the connected part that holds the seed
  std::vector<int> members;
  std::vector<int> slices;
  {
    std::vector<char> seen((size_t)n_nodes, 0);
    std::vector<int> todo{seed};
    seen[seed] = 1;
    auto push = [&](int j) { if (!seen[j]) { seen[j] = 1; todo.push_back(j); } };
    while (!todo.empty()) {
      const int j = todo.back();
      todo.pop_back();
      const Node& n = comp_->nodes[j];
      if (n.op == OP_SLICE) {
        slices.push_back(j);
        for (int c : consumers_[n.out->index]) if (member_of.count(comp_->nodes[c].out) && member_of[comp_->nodes[c].out] == c) push(c);
        continue;
      }
      members.push_back(j);
      for (const _odla_value* v : n.in) {
        auto m = member_of.find(v);
        if (m != member_of.end()) push(m->second);
        auto sl = slice_of.find(v);
        if (sl != slice_of.end()) push(sl->second);
      }
      for (int c : consumers_[n.out->index]) {
        const Node& cn = comp_->nodes[c];
        auto m = member_of.find(cn.out);
        if (m != member_of.end() && m->second == c) push(c);
        if (cn.op == OP_CONCAT && !cn.absorbed) {   // the parts of a Concat belong together
          bool all = true;
          for (const _odla_value* ci : cn.in) all = all && member_of.count(ci);
          if (all) for (const _odla_value* ci : cn.in) push(member_of[ci]);
        }
      }
    }
  }
  std::sort(members.begin(), members.end());
  auto give_up = [&]() { for (int j : members) no_fuse_[j] = 1; return false; };
  if (members.size() < 2) return give_up();
  std::unordered_map<const _odla_value*, int> in_group;   // value -> member node
  for (int j : members) in_group[comp_->nodes[j].out] = j;
  for (int j : slices)
    for (int c : consumers_[comp_->nodes[j].out->index])
      if (!in_group.count(comp_->nodes[c].out) || in_group[comp_->nodes[c].out] != c) return give_up();

  // ---- iteration space: every member's shape, right-aligned, is 1 or S per dim
  int R = 1;
  for (int j : members) R = std::max(R, comp_->nodes[j].out->shape.rank);
  auto padded = [&](const Shape& sh) {
    Shape o;
    o.rank = R;
    for (int i = 0; i < R; ++i) o.d[i] = 1;
    for (int i = 0; i < sh.rank; ++i) o.d[R - sh.rank + i] = sh.d[i];
    return o;
  };
  Shape S = padded(comp_->nodes[members[0]].out->shape);
  for (int j : members) {
    const Shape p = padded(comp_->nodes[j].out->shape);
    for (int i = 0; i < R; ++i) S.d[i] = std::max(S.d[i], p.d[i]);
  }
  for (int j : members) {
    const Shape p = padded(comp_->nodes[j].out->shape);
    for (int i = 0; i < R; ++i) if (p.d[i] != 1 && p.d[i] != S.d[i]) return give_up();
  }
  // operand shape as the consuming operator aligns it
  auto aligned_operand = [&](const Node& n, int k) {
    if (n.op == OP_UNARY) return n.in[0]->shape;
    const int r = (int)n.iv[0];
    Shape a;
    a.rank = r;
    for (int i = 0; i < r; ++i) a.d[i] = n.iv[1 + k * r + i];
    return a;
  };

  // ---- program over virtual registers
  struct View { int tensor = -1; const _odla_value* value = nullptr; int64_t off = 0; int64_t st[3] = {0, 0, 0}; bool store = false; };
  std::vector<View> views;
  struct VI { int op, dst, a, b, kind; float fa, fb; };
  std::vector<VI> prog;
  std::unordered_map<const _odla_value*, int> reg_of;   // member result or loaded operand -> virtual register
  int n_vregs = 0;
  struct PendingLoad { const _odla_value* v; Shape aligned; int reg; };
  std::vector<PendingLoad> loads;
  for (int j : members) {
    const Node& n = comp_->nodes[j];
    int src[2] = {-1, -1};
    float imm[2] = {0.f, 0.f};
    const int n_in = n.op == OP_UNARY ? 1 : 2;
    for (int k = 0; k < n_in; ++k) {
      const _odla_value* v = n.in[k];
      const Shape al = aligned_operand(n, k);
      if (al.rank > R) return give_up();
      if (in_group.count(v)) {
        if (!(padded(al) == padded(v->shape))) return give_up();
        src[k] = reg_of.at(v);
        continue;
      }
      if (n.op == OP_BINARY && v->kind == _odla_value::CONSTANT && v->shape.numel() == 1 && v->host_data != nullptr) {
        imm[k] = const_as_float(v)[0];
        continue;   // src stays -1: immediate operand
      }
      auto it = reg_of.find(v);
      if (it != reg_of.end()) {
        // the same outside value twice: both uses must see it with the same alignment
        bool same = false;
        for (const PendingLoad& l : loads) if (l.v == v) same = padded(l.aligned) == padded(al);
        if (!same) return give_up();
        src[k] = it->second;
        continue;
      }
      const Shape pal = padded(al);
      for (int i = 0; i < R; ++i) if (pal.d[i] != 1 && pal.d[i] != S.d[i]) return give_up();
      if (al.numel() != v->shape.numel()) return give_up();
      const int reg = n_vregs++;
      reg_of[v] = reg;
      loads.push_back({v, al, reg});
      prog.push_back({FOP_LOAD, reg, (int)loads.size() - 1, 0, 0, 0.f, 0.f});   // a = load index for now
      src[k] = reg;
    }
    const int dst = n_vregs++;
    reg_of[n.out] = dst;
    if (n.op == OP_UNARY) {
      prog.push_back({FOP_UNARY, dst, src[0], 0, (int)n.i[0], n.f[0], n.f[1]});
    } else {
      if (src[0] < 0 && src[1] < 0) return give_up();
      prog.push_back({FOP_BINARY, dst, src[0], src[1], (int)n.i[0], src[0] < 0 ? imm[0] : imm[1], 0.f});
    }
  }
  // ---- results that leave the group: plain, through a Concat, through a Transpose
  struct Sink { int node; const _odla_value* src; int kind; /* 0 plain, 1 concat part, 2 transpose */ int part; };
  std::vector<Sink> sinks;
  std::vector<int> sink_nodes;
  for (int j : members) {
    const Node& n = comp_->nodes[j];
    const _odla_value* v = n.out;
    bool plain = v->is_output;
    for (int c : consumers_[v->index]) {
      const Node& cn = comp_->nodes[c];
      if (in_group.count(cn.out) && in_group[cn.out] == c) continue;
      const bool full = v->shape.rank == R && v->shape == S;
      if (cn.op == OP_CONCAT && !cn.absorbed && full && storage_dtype(cn.out) == dt && cn.out->shape.rank == R) {
        bool all = true;
        for (const _odla_value* ci : cn.in) all = all && in_group.count(ci) && ci->shape.rank == R;
        if (all) {
          const int axis = (int)cn.i[0];
          for (const _odla_value* ci : cn.in)
            for (int i = 0; i < R; ++i) if (i != axis && ci->shape.d[i] != S.d[i]) all = false;
          for (const _odla_value* ci : cn.in) if (!(ci->shape == S)) all = false;
        }
        if (all) {
          if (std::find(sink_nodes.begin(), sink_nodes.end(), c) == sink_nodes.end()) {
            sink_nodes.push_back(c);
            for (size_t k = 0; k < cn.in.size(); ++k) sinks.push_back({c, cn.in[k], 1, (int)k});
          }
          continue;
        }
      }
      // A Transpose that moves the innermost dim turns the group's stores into single
      // elements a row apart; beyond a few million elements the tiled copy
      // behind a plain store is several times faster than that.
      if (cn.op == OP_TRANSPOSE && !cn.absorbed && full && storage_dtype(cn.out) == dt && (int)cn.iv.size() == R &&
          (cn.iv[R - 1] == R - 1 || S.numel() <= kTransposeSinkMax)) {
        if (std::find(sink_nodes.begin(), sink_nodes.end(), c) == sink_nodes.end()) {
          sink_nodes.push_back(c);
          sinks.push_back({c, v, 2, 0});
        }
        continue;
      }
      plain = true;
    }
    if (plain) {
      if (!(padded(v->shape) == S)) return give_up();
      sinks.push_back({j, v, 0, 0});
    }
  }
  if (sinks.empty()) return give_up();
  if ((int)(loads.size() + sinks.size()) > kFusedMaxViews || (int)(prog.size() + sinks.size()) > kFusedMaxInstr) return give_up();

  // ---- physical registers: a register is free again after its last reader
  std::vector<int> last_use((size_t)n_vregs, -1);
  for (size_t k = 0; k < prog.size(); ++k) {
    if (prog[k].op != FOP_LOAD && prog[k].a >= 0) last_use[prog[k].a] = (int)k;
    if (prog[k].op == FOP_BINARY && prog[k].b >= 0) last_use[prog[k].b] = (int)k;
  }
  for (const Sink& sk : sinks) last_use[reg_of.at(sk.src)] = (int)prog.size();   // stores come last
  std::vector<int> phys((size_t)n_vregs, -1);
  {
    std::vector<int> free_regs;
    for (int i = kFusedMaxRegs - 1; i >= 0; --i) free_regs.push_back(i);
    for (size_t k = 0; k < prog.size(); ++k) {
      VI& in = prog[k];
      const int va = in.op != FOP_LOAD ? in.a : -1, vb = in.op == FOP_BINARY ? in.b : -1;
      // operands read before the result is written: a register freed here may take the result
      if (va >= 0 && last_use[va] == (int)k) free_regs.push_back(phys[va]);
      if (vb >= 0 && vb != va && last_use[vb] == (int)k) free_regs.push_back(phys[vb]);
      if (free_regs.empty()) return give_up();
      phys[in.dst] = free_regs.back();
      free_regs.pop_back();
      if (last_use[in.dst] < 0) free_regs.push_back(phys[in.dst]);   // never read: reusable at once
    }
  }

  // ---- from here on the plan changes: nothing below gives up
  // outside operands (conversion steps, if any, are emitted here, before the group)
  FusedParams fp;
  fp.dt = dt;
  std::vector<int> read_tensors, write_tensors;
  std::vector<int64_t> in_main_stride;   // per load: used to pick the iteration order
  for (const PendingLoad& l : loads) {
    View vw;
    auto sl = slice_of.find(l.v);
    const Shape pal = padded(l.aligned);
    if (sl != slice_of.end() && std::find(slices.begin(), slices.end(), sl->second) != slices.end()) {
      const Node& sn = comp_->nodes[sl->second];
      const _odla_value* x = sn.in[0];
      const int r = x->shape.rank;
      vw.tensor = get(x, L_ROWMAJOR, FORM_FLOAT);
      // strides of the slice's own dims, then mapped through the aligned shape (which only adds 1-dims)
      std::vector<int64_t> own_st((size_t)r);
      int64_t acc = 1;
      for (int i = r - 1; i >= 0; --i) {
        own_st[i] = acc * sn.iv[2 * r + i];
        vw.off += sn.iv[i] * acc;
        acc *= x->shape.d[i];
      }
      // walk the non-1 dims of the slice result and of the aligned shape together
      int oi = 0;
      for (int i = 0; i < R; ++i) {
        if (pal.d[i] == 1) continue;
        while (oi < r && sn.out->shape.d[oi] == 1) ++oi;
        vw.st[i] = own_st[oi++];
      }
    } else {
      vw.tensor = get(l.v, L_ROWMAJOR, FORM_FLOAT);
      int64_t acc = 1;
      for (int i = R - 1; i >= 0; --i) { vw.st[i] = pal.d[i] == 1 ? 0 : acc; acc *= pal.d[i]; }
    }
    if (T(vw.tensor).dt != dt) fail(ODLA_UNSUPPORTED_DATATYPE, "mixed storage types in the element-wise group at '%s'", comp_->nodes[seed].out->name.c_str());
    vw.value = l.v;
    views.push_back(vw);
    read_tensors.push_back(vw.tensor);
  }
  const size_t n_loads = views.size();
  std::unordered_map<int, int> sink_tensor;   // sink node -> its result tensor
  std::vector<std::pair<_odla_value*, int>> results;
  auto row_major = [&](const Shape& sh, int64_t* st) { int64_t acc = 1; for (int i = sh.rank - 1; i >= 0; --i) { st[i] = acc; acc *= sh.d[i]; } };
  for (const Sink& sk : sinks) {
    const Node& sn = comp_->nodes[sk.node];
    View vw;
    vw.store = true;
    vw.value = sk.src;
    int64_t st[ODLA_MAX_DIMENSION] = {0};
    if (sk.kind == 0) {
      vw.tensor = new_tensor(dt, L_ROWMAJOR, sk.src->shape, 0, SP_ARENA);
      results.push_back({sn.out, vw.tensor});
      row_major(S, st);
      for (int i = 0; i < R; ++i) vw.st[i] = st[i];
    } else {
      auto it = sink_tensor.find(sk.node);
      if (it == sink_tensor.end()) {
        const int t = new_tensor(dt, L_ROWMAJOR, sn.out->shape, 0, SP_ARENA);
        it = sink_tensor.emplace(sk.node, t).first;
        results.push_back({sn.out, t});
      }
      vw.tensor = it->second;
      row_major(sn.out->shape, st);
      if (sk.kind == 1) {
        const int axis = (int)sn.i[0];
        int64_t before = 0;
        for (int k = 0; k < sk.part; ++k) before += sn.in[k]->shape.d[axis];
        vw.off = before * st[axis];
        for (int i = 0; i < R; ++i) vw.st[i] = st[i];
      } else {
        for (int i = 0; i < R; ++i) vw.st[(int)sn.iv[i]] = st[i];   // result dim i walks source dim perm[i]
      }
    }
    views.push_back(vw);
    if (std::find(write_tensors.begin(), write_tensors.end(), vw.tensor) == write_tensors.end()) write_tensors.push_back(vw.tensor);
  }

  // ---- iteration order: stores contiguous across threads, loads along a thread's walk
  int d3 = R - 1, d2 = -1;
  {
    const View& mo = views[n_loads];
    int64_t best = 0;
    for (int i = 0; i < R; ++i)
      if (S.d[i] > 1 && mo.st[i] > 0 && (best == 0 || mo.st[i] < best)) { best = mo.st[i]; d3 = i; }
    int64_t most = -1;
    const View* mi = nullptr;
    for (size_t k = 0; k < n_loads; ++k) {
      int64_t elems = 1;
      for (int i = 0; i < R; ++i) if (views[k].st[i] != 0) elems *= S.d[i];
      if (elems > most) { most = elems; mi = &views[k]; }
    }
    if (mi != nullptr && mi->st[d3] != 1)
      for (int i = 0; i < R; ++i) if (i != d3 && S.d[i] > 1 && mi->st[i] == 1) d2 = i;
    // no such dim: with points to spare, a thread still takes four per decoded instruction,
    // along the longest other dim
    if (d2 < 0 && S.numel() >= (int64_t)4 * 256 * 2048)
      for (int i = 0; i < R; ++i) if (i != d3 && S.d[i] >= 4 && (d2 < 0 || S.d[i] > S.d[d2])) d2 = i;
  }
  int order[4] = {-1, -1, d2, d3};
  {
    int slot = 1;
    for (int i = R - 1; i >= 0; --i) if (i != d2 && i != d3) order[slot--] = i;
  }
  for (int k = 0; k < 4; ++k) fp.dims[k] = order[k] < 0 ? 1 : S.d[order[k]];
  {
    // every step of a walk waits for its loads: keep walks short until the chip has
    // a few resident threads per lane (256 CUs x 2048 threads x 2)
    const int64_t base = fp.dims[0] * fp.dims[1] * fp.dims[3];
    const int64_t want = 256 * 2048 * 2;
    int64_t w = fp.dims[2] * base / want;
    fp.walk = std::min<int64_t>(fp.dims[2], std::max<int64_t>(4, w / 4 * 4));   // whole groups of four points
  }
  for (size_t k = 0; k < views.size(); ++k) {
    fp.view[k].off = views[k].off;
    for (int q = 0; q < 4; ++q) fp.view[k].st[q] = order[q] < 0 ? 0 : views[k].st[order[q]];
  }
  int ni = 0;
  for (const VI& in : prog) {
    FusedInstr& o = fp.prog[ni++];
    o.op = in.op; o.kind = in.kind; o.fa = in.fa; o.fb = in.fb;
    o.dst = phys[in.dst];
    o.a = in.op == FOP_LOAD ? in.a : (in.a < 0 ? -1 : phys[in.a]);
    o.b = in.op == FOP_BINARY ? (in.b < 0 ? -1 : phys[in.b]) : 0;
  }
  for (size_t k = 0; k < sinks.size(); ++k) {
    FusedInstr& o = fp.prog[ni++];
    o.op = FOP_STORE;
    o.dst = (int)(n_loads + k);
    o.a = phys[reg_of.at(sinks[k].src)];
  }
  fp.n_instr = ni;

  std::vector<Ref> refs;
  for (const View& vw : views) refs.push_back(ref(vw.tensor));
  std::vector<int64_t> elem_off;
  const std::string name = "fused:" + comp_->nodes[members.back()].out->name + "(" + std::to_string(members.size()) + ")";
  emit_lists(name, read_tensors, write_tensors, [=](const ExecEnv& e, hipStream_t st) {
    FusedParams p = fp;
    for (size_t k = 0; k < refs.size(); ++k) p.view[k].base = refs[k](e);
    return launch_fused_eltwise(p, st);
  });
  for (int j : members) comp_->nodes[j].absorbed = true;
  for (int j : slices) comp_->nodes[j].absorbed = true;
  for (int j : sink_nodes) comp_->nodes[j].absorbed = true;
  for (auto& rv : results) set_main(rv.first, rv.second);
  return true;
}

// ----------------------------------------------------------- BatchNorm ----
void Planner::lower_batchnorm(int ni) {
  Node& n = comp_->nodes[ni];
  const _odla_value* x = n.in[0];
  const bool cf = n.i[0] != ODLA_CHANNELS_LAST;
  const Shape& xs = x->shape;
  const int64_t C = cf ? xs.d[1] : xs.d[xs.rank - 1];
  const VState& s = vs_[x->index];
  Layout lay = L_ROWMAJOR;
  if (cf && xs.rank == 4 && s.main >= 0 && T(s.main).layout == L_NHWC) lay = L_NHWC;
  const int tx = get(x, lay, FORM_FLOAT);
  const PTensor px = T(tx);
  const int ty = new_tensor(px.dt, px.layout, n.out->shape, px.cs, SP_ARENA);
  int64_t inner;
  int channels;
  if (lay == L_NHWC) { inner = 1; channels = px.cs; }
  else if (cf) { inner = 1; for (int i = 2; i < xs.rank; ++i) inner *= xs.d[i]; channels = (int)C; }
  else { inner = 1; channels = (int)C; }

  bool all_const = true;
  for (int i = 1; i <= 4; ++i)
    if (n.in[i] && n.in[i]->kind != _odla_value::CONSTANT) all_const = false;
  int tscale, tshift;
  if (all_const) {
    std::vector<float> sc, sh;
    bn_params_host(n, C, &sc, &sh);
    sc.resize((size_t)channels, 1.f);
    sh.resize((size_t)channels, 0.f);
    tscale = const_vector<float>(DT_F32, sc);
    tshift = const_vector<float>(DT_F32, sh);
  } else {
    // statistics arrive at run time (fp32 arguments): fold them on the device
    if (channels != C) fail(ODLA_UNSUPPORTED_OP, "run-time BatchNorm parameters on a padded tensor");
    int tp[5] = {-1, -1, -1, -1, -1};
    for (int i = 1; i <= 4; ++i) {
      if (!n.in[i]) continue;
      const _odla_value* pv = n.in[i];
      if (dtype_from_odla(pv->etype) != DT_F32) fail(ODLA_UNSUPPORTED_DATATYPE, "BatchNorm parameters must be FLOAT32");
      if (pv->kind == _odla_value::CONSTANT) tp[i] = const_from_host(DT_F32, pv->shape, pv->host_data, nullptr);
      else {
        const VState& ps = vs_[pv->index];
        if (ps.main < 0 || T(ps.main).dt != DT_F32) fail(ODLA_UNSUPPORTED_OP, "BatchNorm parameter '%s' must be a FLOAT32 argument", pv->name.c_str());
        tp[i] = ps.main;
      }
    }
    Shape cs1;
    cs1.rank = 1;
    cs1.d[0] = C;
    tscale = new_tensor(DT_F32, L_ROWMAJOR, cs1, 0, SP_ARENA);
    tshift = new_tensor(DT_F32, L_ROWMAJOR, cs1, 0, SP_ARENA);
    const Ref rm = ref(tp[1]), rv = ref(tp[2]), rg = ref(tp[3] >= 0 ? tp[3] : tp[1]), rb = ref(tp[4] >= 0 ? tp[4] : tp[1]);
    const bool hg = tp[3] >= 0, hb = tp[4] >= 0;
    const Ref rs = ref(tscale), rt = ref(tshift);
    const float sg = n.f[1], sb = n.f[2], eps = n.f[0];
    const int Ci = (int)C;
    emit("bn.fold:" + n.out->name, {tp[1], tp[2], tp[3], tp[4]}, {tscale, tshift}, [=](const ExecEnv& e, hipStream_t st) {
      return launch_bn_fold((const float*)rm(e), (const float*)rv(e), hg ? (const float*)rg(e) : nullptr,
                            hb ? (const float*)rb(e) : nullptr, sg, sb, eps, Ci, (float*)rs(e), (float*)rt(e), st);
    });
  }
  const int64_t ne = px.phys_elems();
  const DType dt = px.dt;
  const Ref a = ref(tx), b = ref(ty), rs = ref(tscale), rt = ref(tshift);
  emit("bn:" + n.out->name, {tx, tscale, tshift}, {ty}, [=](const ExecEnv& e, hipStream_t st) {
    return launch_channel_affine(a(e), b(e), dt, ne, inner, channels, (const float*)rs(e), (const float*)rt(e), st);
  });
  set_main(n.out, ty);
}

// ----------------------------------------------------------- LayerNorm ----
void Planner::lower_layernorm(int ni) {
  Node& n = comp_->nodes[ni];
  const _odla_value* x = n.in[0];
  const int tx = get(x, L_ROWMAJOR, FORM_FLOAT);
  const Shape& xs = x->shape;
  const int na = (int)n.i[0];
  int64_t len = 1;
  for (int i = xs.rank - na; i < xs.rank; ++i) len *= xs.d[i];
  const int64_t rows = xs.numel() / len;
  int tg = -1, tb = -1;
  if (n.in[1]) { std::vector<float> g = const_as_float(n.in[1]); tg = const_vector<float>(DT_F32, g); }
  if (n.in[2]) { std::vector<float> b = const_as_float(n.in[2]); tb = const_vector<float>(DT_F32, b); }
  const DType dt = T(tx).dt;
  const int ty = new_tensor(dt, L_ROWMAJOR, n.out->shape, 0, SP_ARENA);
  const Ref a = ref(tx), b = ref(ty), rg = ref(tg >= 0 ? tg : tx), rb = ref(tb >= 0 ? tb : tx);
  const bool hg = tg >= 0, hb = tb >= 0;
  const float eps = n.f[0];
  // Accuracy mode (fp32 tensors, 2-byte matrix operands): a result that matrix products read as
  // their operand leaves this launch in both forms - the separate conversion launch per
  // LayerNorm (25 per BERT-base step) is gone.
  int t2 = -1;
  if (acc_mode_ && dt == DT_F32 && dtype_from_odla(n.out->etype) == DT_F32 && layernorm_dual_ok(dt, len)) {
    for (int ci : consumers_[n.out->index]) {
      const Node& c = comp_->nodes[ci];
      if ((c.op == OP_GEMM || c.op == OP_CONV) && (c.in[0] == n.out || c.in[1] == n.out)) t2 = -2;
    }
    if (t2 == -2) t2 = new_tensor(op_dt_, L_ROWMAJOR, n.out->shape, 0, SP_ARENA);
  }
  const Ref b2 = ref(t2 >= 0 ? t2 : ty);
  const bool dual = t2 >= 0;
  const DType dt2 = op_dt_;
  emit("layernorm:" + n.out->name, {tx}, {ty, t2}, [=](const ExecEnv& e, hipStream_t st) {
    return launch_layernorm(a(e), b(e), dt, rows, len, hg ? (const float*)rg(e) : nullptr,
                            hb ? (const float*)rb(e) : nullptr, eps, st, dual ? b2(e) : nullptr, dt2);
  });
  set_main(n.out, ty);
  if (dual) vs_[n.out->index].slot[L_ROWMAJOR][FORM_OPERAND] = t2;
}

// ---------------------------------------------------------------- Pool ----
void Planner::lower_pool(int ni) {
  Node& n = comp_->nodes[ni];
  const _odla_value* x = n.in[0];
  const bool cl = n.i[0] == ODLA_CHANNELS_LAST;
  const Shape& xs = x->shape;
  const Shape& os = n.out->shape;
  const bool is_max = n.i[1] != 0;
  // 8-bit max pooling keeps levels (the result inherits the input's scale)
  const VState& s = vs_[x->index];
  const bool q8 = is_max && !cl && s.main >= 0 && T(s.main).quant && (xs.d[1] % 16 == 0);
  int tx;
  if (cl) tx = get(x, L_ROWMAJOR, FORM_FLOAT);
  else tx = get(x, L_NHWC, q8 ? FORM_QUANT : FORM_FLOAT);
  const PTensor px = T(tx);
  PoolParams pp;
  pp.dt = px.dt;
  pp.N = (int)xs.d[0];
  pp.H = (int)(cl ? xs.d[1] : xs.d[2]);
  pp.W = (int)(cl ? xs.d[2] : xs.d[3]);
  pp.C = (int)(cl ? xs.d[3] : xs.d[1]);
  pp.cs = cl ? pp.C : px.cs;
  pp.Ho = (int)(cl ? os.d[1] : os.d[2]);
  pp.Wo = (int)(cl ? os.d[2] : os.d[3]);
  pp.ycs = pp.C;
  pp.kh = (int)n.i[2]; pp.kw = (int)n.i[3]; pp.sh = (int)n.i[4]; pp.sw = (int)n.i[5];
  pp.ph = (int)n.i[6]; pp.pw = (int)n.i[7];
  pp.is_max = is_max;
  pp.count_include_pad = n.i[10] != 0;
  int ty;
  if (cl) ty = new_tensor(px.dt, L_ROWMAJOR, os, 0, SP_ARENA);
  else ty = new_tensor(px.dt, L_NHWC, os, pp.C, SP_ARENA);
  if (q8) set_quant(ty, true, px.qscale, px.qzp);
  const Ref a = ref(tx), b = ref(ty);
  emit(std::string(is_max ? "maxpool:" : "avgpool:") + n.out->name, {tx}, {ty}, [=](const ExecEnv& e, hipStream_t st) {
    PoolParams p = pp; p.x = a(e); p.y = b(e);
    return launch_pool2d(p, st);
  });
  set_main(n.out, ty);
}

// -------------------------------------------------------------- Reduce ----
void Planner::lower_reduce(int ni) {
  Node& n = comp_->nodes[ni];
  const _odla_value* x = n.in[0];
  const Shape& xs = x->shape;
  const ReduceKind kind = (ReduceKind)n.i[0];
  const float eps = n.f[0];
  const std::vector<int64_t>& axes = n.iv;
  const VState& s = vs_[x->index];
  // spatial reduction of a channels-last tensor (global pooling)
  const bool spatial = xs.rank == 4 && axes.size() == 2 && axes[0] == 2 && axes[1] == 3;
  // (a float tensor whose pixels are padded to a vector multiple takes the general path below)
  if (spatial && s.main >= 0 && T(s.main).layout == L_NHWC && (T(s.main).cs == xs.d[1] || T(s.main).quant)) {
    const PTensor px = T(s.main);
    const int64_t outer = xs.d[0], len = xs.d[2] * xs.d[3], inner = px.cs;
    if (px.cs != xs.d[1]) fail(ODLA_UNSUPPORTED_OP, "reduction over a padded 8-bit channels-last tensor");
    Shape o4;
    o4.rank = 4;
    o4.d[0] = xs.d[0]; o4.d[1] = xs.d[1]; o4.d[2] = 1; o4.d[3] = 1;
    const Ref a = ref(s.main);
    int ty;
    if (px.quant) {
      if (kind != RED_MEAN) fail(ODLA_UNSUPPORTED_OP, "only ReduceMean is supported on 8-bit tensors");
      ty = new_tensor(DT_F32, L_ROWMAJOR, n.out->shape, 0, SP_ARENA);
      const Ref b = ref(ty);
      const float sc = px.qscale;
      const int zp = px.qzp;
      emit("reduce.q8:" + n.out->name, {s.main}, {ty}, [=](const ExecEnv& e, hipStream_t st) {
        return launch_reduce_q8_mean(a(e), (float*)b(e), outer, len, inner, sc, zp, st);
      });
      if (cdt_ != DT_F32) {
        const int tc = new_tensor(cdt_, L_ROWMAJOR, n.out->shape, 0, SP_ARENA);
        const Ref c = ref(tc);
        const int64_t ne = n.out->shape.numel();
        const DType ddt = cdt_;
        emit("cast:" + n.out->name, {ty}, {tc}, [=](const ExecEnv& e, hipStream_t st) { return launch_cast(b(e), DT_F32, c(e), ddt, ne, st); });
        ty = tc;
      }
    } else {
      ty = new_tensor(px.dt, L_ROWMAJOR, n.out->shape, 0, SP_ARENA);
      const Ref b = ref(ty);
      const DType dt = px.dt;
      emit("reduce:" + n.out->name, {s.main}, {ty}, [=](const ExecEnv& e, hipStream_t st) {
        return launch_reduce(a(e), b(e), dt, dt, outer, len, inner, kind, st, eps);
      });
    }
    set_main(n.out, ty);
    return;
  }
  // general case: one launch when the reduced axes are adjacent in row-major
  // order; otherwise a permuted copy that moves them behind the kept ones first
  bool adjacent = true;
  for (size_t i = 1; i < axes.size(); ++i)
    if (axes[i] != axes[i - 1] + 1) adjacent = false;
  int tx = get(x, L_ROWMAJOR, FORM_FLOAT);
  const DType dt = T(tx).dt;
  int64_t outer = 1, len = 1, inner = 1;
  if (adjacent) {
    for (int i = 0; i < xs.rank; ++i) {
      if (i < axes.front()) outer *= xs.d[i];
      else if (i <= axes.back()) len *= xs.d[i];
      else inner *= xs.d[i];
    }
  } else {
    const int r = xs.rank;
    if (r > 8) fail(ODLA_UNSUPPORTED_OP, "reduction over non-adjacent axes of a rank > 8 value");
    std::vector<int> order;
    for (int i = 0; i < r; ++i)
      if (std::find(axes.begin(), axes.end(), (int64_t)i) == axes.end()) order.push_back(i);
    for (int64_t a : axes) order.push_back((int)a);
    int64_t xstr[ODLA_MAX_DIMENSION];
    {
      int64_t acc = 1;
      for (int i = r - 1; i >= 0; --i) { xstr[i] = acc; acc *= xs.d[i]; }
    }
    Shape ps;
    ps.rank = r;
    for (int i = 0; i < r; ++i) ps.d[i] = xs.d[order[i]];
    const int tp = new_tensor(dt, L_ROWMAJOR, ps, 0, SP_ARENA);
    StridedCopyParams cp;
    cp.elem_size = dtype_size(dt);
    cp.rank = r;
    int64_t sy = 1;
    for (int i = r - 1; i >= 0; --i) {
      cp.dims[i] = ps.d[i];
      cp.sx[i] = xstr[order[i]];
      cp.sy[i] = sy;
      sy *= ps.d[i];
    }
    strided_copy_step("reduce.gather:" + n.out->name, tx, tp, cp);
    tx = tp;
    for (int64_t a : axes) len *= xs.d[a];
    outer = xs.numel() / len;
  }
  const int ty = new_tensor(dt, L_ROWMAJOR, n.out->shape, 0, SP_ARENA);
  const Ref a = ref(tx), b = ref(ty);
  emit("reduce:" + n.out->name, {tx}, {ty}, [=](const ExecEnv& e, hipStream_t st) {
    return launch_reduce(a(e), b(e), dt, dt, outer, len, inner, kind, st, eps);
  });
  set_main(n.out, ty);
}

// ---------------------------------------------------- ArgMax / ArgMin ----
void Planner::lower_argext(int ni) {
  Node& n = comp_->nodes[ni];
  const _odla_value* x = n.in[0];
  const Shape& xs = x->shape;
  const int axis = (int)n.i[1];
  const int tx = get(x, L_ROWMAJOR, FORM_FLOAT);
  int64_t outer = 1, inner = 1;
  for (int i = 0; i < axis; ++i) outer *= xs.d[i];
  for (int i = axis + 1; i < xs.rank; ++i) inner *= xs.d[i];
  const int64_t len = xs.d[axis];
  const DType dt = T(tx).dt, odt = storage_dtype(n.out);
  const int ty = new_tensor(odt, L_ROWMAJOR, n.out->shape, 0, SP_ARENA);
  const bool is_max = n.i[0] != 0, last = n.i[2] != 0;
  const Ref a = ref(tx), b = ref(ty);
  emit(std::string(is_max ? "argmax:" : "argmin:") + n.out->name, {tx}, {ty}, [=](const ExecEnv& e, hipStream_t st) {
    return launch_arg_extreme(a(e), b(e), dt, odt, outer, len, inner, is_max, last, st);
  });
  set_main(n.out, ty);
}

// ------------------------------------------------------------- Softmax ----
void Planner::lower_softmax(int ni) {
  Node& n = comp_->nodes[ni];
  const _odla_value* x = n.in[0];
  const Shape& xs = x->shape;
  const int axis = (int)n.i[0];
  int tadd = -1;
  int64_t add_div = 1;
  {
    auto it = softmax_add_.find(x->index);
    if (it != softmax_add_.end()) {  // the Add in front was folded into this launch
      x = it->second.x;
      tadd = get(it->second.mask, L_ROWMAJOR, FORM_FLOAT);
      add_div = it->second.div;
    }
  }
  const int tx = get(x, L_ROWMAJOR, FORM_FLOAT);
  int64_t outer = 1, inner = 1;
  for (int i = 0; i < axis; ++i) outer *= xs.d[i];
  for (int i = axis + 1; i < xs.rank; ++i) inner *= xs.d[i];
  const int64_t len = xs.d[axis];
  const DType dt = T(tx).dt;
  if (tadd >= 0 && T(tadd).dt != dt) fail(ODLA_INTERNAL_LOGIC_ERR, "softmax mask storage type mismatch");
  // a graph output is written in fp32 directly
  const bool to_f32 = n.out->is_output && dtype_from_odla(n.out->etype) == DT_F32 && consumers_[n.out->index].empty();
  // (accuracy mode: probabilities that only feed a matrix product are stored in its operand type)
  const DType odt = to_f32 ? DT_F32 : (acc_mode_ && dt == DT_F32 && operand_only(n.out) ? op_dt_ : dt);
  const int ty = new_tensor(odt, L_ROWMAJOR, n.out->shape, 0, SP_ARENA);
  const bool logsm = n.i[1] != 0;
  const Ref a = ref(tx), b = ref(ty), m = ref(tadd >= 0 ? tadd : tx);
  const bool has_add = tadd >= 0;
  emit("softmax:" + n.out->name, {tx, tadd}, {ty}, [=](const ExecEnv& e, hipStream_t st) {
    return launch_softmax(a(e), b(e), dt, odt, outer, len, inner, logsm, st, has_add ? m(e) : nullptr, add_div);
  });
  set_main(n.out, ty);
}

// ---------------------------------------------------------------- Cast ----
void Planner::lower_cast(int ni) {
  Node& n = comp_->nodes[ni];
  const _odla_value* x = n.in[0];
  const int tx = get(x, L_ROWMAJOR, FORM_FLOAT);
  const DType sdt = T(tx).dt;
  const DType ddt = storage_dtype(n.out);
  if (sdt == ddt) {
    set_main(n.out, alias_tensor(tx, n.out->shape));
    return;
  }
  const int ty = new_tensor(ddt, L_ROWMAJOR, n.out->shape, 0, SP_ARENA);
  const int64_t ne = x->shape.numel();
  const Ref a = ref(tx), b = ref(ty);
  emit("cast:" + n.out->name, {tx}, {ty}, [=](const ExecEnv& e, hipStream_t st) { return launch_cast(a(e), sdt, b(e), ddt, ne, st); });
  set_main(n.out, ty);
}

// -------------------------------------------------------------- Concat ----
void Planner::lower_concat(int ni) {
  Node& n = comp_->nodes[ni];
  const Shape& os = n.out->shape;
  const int axis = (int)n.i[0];
  // channel concat of channels-last tensors stays channels-last
  bool nhwc = os.rank == 4 && axis == 1;
  if (nhwc) {
    bool any = false;
    for (_odla_value* v : n.in) {
      const VState& s = vs_[v->index];
      if (s.main >= 0 && T(s.main).layout == L_NHWC && !T(s.main).quant) any = true;
    }
    nhwc = any;
  }
  const Layout lay = nhwc ? L_NHWC : L_ROWMAJOR;
  std::vector<int> tin;
  for (_odla_value* v : n.in) tin.push_back(get(v, lay, FORM_FLOAT));
  const DType dt = T(tin[0]).dt;
  const int es = dtype_size(dt);
  const int ty = new_tensor(dt, lay, os, nhwc ? (int)os.d[1] : 0, SP_ARENA);
  int64_t off = 0;
  for (size_t k = 0; k < n.in.size(); ++k) {
    const PTensor pi = T(tin[k]);
    if (pi.dt != dt) fail(ODLA_UNSUPPORTED_DATATYPE, "odla_Concat of mixed storage types");
    const Shape& is = n.in[k]->shape;
    StridedCopyParams cp;
    cp.elem_size = es;
    if (nhwc) {
      const int64_t pixels = is.d[0] * is.d[2] * is.d[3];
      cp.rank = 2;
      cp.dims[0] = pixels; cp.dims[1] = is.d[1];
      cp.sx[0] = pi.cs; cp.sx[1] = 1;
      cp.sy[0] = os.d[1]; cp.sy[1] = 1;
      cp.y_off = off;
      off += is.d[1];
    } else {
      int64_t outer = 1, inner = 1;
      for (int i = 0; i < axis; ++i) outer *= is.d[i];
      for (int i = axis + 1; i < is.rank; ++i) inner *= is.d[i];
      cp.rank = 2;
      cp.dims[0] = outer; cp.dims[1] = is.d[axis] * inner;
      cp.sx[0] = is.d[axis] * inner; cp.sx[1] = 1;
      cp.sy[0] = os.d[axis] * inner; cp.sy[1] = 1;
      cp.y_off = off;
      off += is.d[axis] * inner;
    }
    // widen to 16-byte elements when everything is aligned
    const int w = 16 / es;
    if (cp.dims[1] % w == 0 && cp.sx[0] % w == 0 && cp.sy[0] % w == 0 && cp.y_off % w == 0) {
      cp.elem_size = 16;
      cp.dims[1] /= w; cp.sx[0] /= w; cp.sy[0] /= w; cp.y_off /= w;
    }
    strided_copy_step("concat:" + n.out->name, tin[k], ty, cp);
  }
  set_main(n.out, ty);
}

// -------------------------------------------------------------- Gather ----
void Planner::lower_gather(int ni) {
  Node& n = comp_->nodes[ni];
  const _odla_value* x = n.in[0];
  const _odla_value* idx = n.in[1];
  const int axis = (int)n.i[0];
  const int tx = get(x, L_ROWMAJOR, FORM_FLOAT);
  const int ti = get(idx, L_ROWMAJOR, FORM_FLOAT);
  const Shape& xs = x->shape;
  int64_t outer = 1, inner = 1;
  for (int i = 0; i < axis; ++i) outer *= xs.d[i];
  for (int i = axis + 1; i < xs.rank; ++i) inner *= xs.d[i];
  const DType dt = T(tx).dt;
  const DType idt = T(ti).dt;
  const int64_t n_src = xs.d[axis], n_idx = idx->shape.numel();
  const int64_t row_bytes = inner * dtype_size(dt);
  const int ty = new_tensor(dt, L_ROWMAJOR, n.out->shape, 0, SP_ARENA);
  const Ref a = ref(tx), ri = ref(ti), b = ref(ty);
  emit("gather:" + n.out->name, {tx, ti}, {ty}, [=](const ExecEnv& e, hipStream_t st) {
    return launch_gather_rows(a(e), ri(e), idt, b(e), outer, n_src, n_idx, row_bytes, st);
  });
  set_main(n.out, ty);
}

// ------------------------------- GatherElements, CumSum, Hardmax, Compress ----
void Planner::lower_axisop(int ni) {
  Node& n = comp_->nodes[ni];
  const _odla_value* x = n.in[0];
  const Shape& xs = x->shape;
  const AxisOp op = (AxisOp)n.i[0];
  const int axis = (int)n.i[1];
  const int tx = get(x, L_ROWMAJOR, FORM_FLOAT);
  const DType dt = T(tx).dt;
  int64_t outer = 1, inner = 1;
  for (int i = 0; i < axis; ++i) outer *= xs.d[i];
  for (int i = axis + 1; i < xs.rank; ++i) inner *= xs.d[i];
  const int64_t len = xs.d[axis];
  const int ty = new_tensor(dt, L_ROWMAJOR, n.out->shape, 0, SP_ARENA);
  const Ref a = ref(tx), b = ref(ty);
  switch (op) {
    case AX_GATHER_ELEMENTS: {
      const _odla_value* idx = n.in[1];
      const int ti = get(idx, L_ROWMAJOR, FORM_FLOAT);
      const DType idt = T(ti).dt;
      int64_t ii = 1, ik = 1;
      for (int i = 0; i < axis; ++i) ii *= idx->shape.d[i];
      for (int i = axis + 1; i < xs.rank; ++i) ik *= idx->shape.d[i];
      const int64_t ij = idx->shape.d[axis];
      const int es = dtype_size(dt);
      const Ref ri = ref(ti);
      emit("gather_elements:" + n.out->name, {tx, ti}, {ty}, [=](const ExecEnv& e, hipStream_t st) {
        return launch_gather_elements(a(e), ri(e), idt, b(e), es, ii, ij, ik, outer, len, inner, st);
      });
      break;
    }
    case AX_CUMSUM: {
      const bool exclusive = n.i[2] != 0, reverse = n.i[3] != 0;
      emit("cumsum:" + n.out->name, {tx}, {ty}, [=](const ExecEnv& e, hipStream_t st) {
        return launch_cumsum(a(e), b(e), dt, outer, len, inner, exclusive, reverse, st);
      });
      break;
    }
    case AX_HARDMAX: {
      // the index of the first largest element, then its one-hot form (the reference's two steps)
      Shape is;
      is.rank = 1;
      is.d[0] = outer * inner;
      const int tm = new_tensor(DT_I32, L_ROWMAJOR, is, 0, SP_ARENA);
      const Ref m = ref(tm);
      emit("hardmax.argmax:" + n.out->name, {tx}, {tm}, [=](const ExecEnv& e, hipStream_t st) {
        return launch_arg_extreme(a(e), m(e), dt, DT_I32, outer, len, inner, true, false, st);
      });
      emit("hardmax:" + n.out->name, {tm}, {ty}, [=](const ExecEnv& e, hipStream_t st) {
        return launch_onehot_axis(m(e), DT_I32, b(e), dt, outer, len, inner, st);
      });
      break;
    }
    case AX_COMPRESS: {
      const int tc = get(n.in[1], L_ROWMAJOR, FORM_FLOAT);
      const int n_cond = (int)n.i[2];
      const bool flat = n.i[3] != 0;
      const int64_t o2 = flat ? 1 : outer, l2 = flat ? xs.numel() : len, i2 = flat ? 1 : inner;
      const int64_t n_out = n.out->shape.numel();
      const int es = dtype_size(dt);
      const int tsel = raw_buffer(((size_t)n_cond + 1) * sizeof(int32_t), SP_ARENA);
      const Ref rc = ref(tc), rs = ref(tsel);
      emit("compress:" + n.out->name, {tx, tc}, {ty, tsel}, [=](const ExecEnv& e, hipStream_t st) {
        return launch_compress(a(e), rc(e), n_cond, reinterpret_cast<int32_t*>(rs(e)), b(e), es, o2, l2, i2, n_out, st);
      });
      break;
    }
    default:
      fail(ODLA_INTERNAL_LOGIC_ERR, "unknown axis operator %d", (int)op);
  }
  set_main(n.out, ty);
}

// ------------------------------------------------------------- Reshape ----
void Planner::lower_reshape(int ni) {
  Node& n = comp_->nodes[ni];
  const _odla_value* x = n.in[0];
  const VState& s = vs_[x->index];
  // keep 8-bit data 8-bit through a reshape when it is already row-major
  int tx;
  if (s.main >= 0 && T(s.main).quant && s.slot[L_ROWMAJOR][FORM_QUANT] >= 0 && qentry(n.out) != nullptr)
    tx = s.slot[L_ROWMAJOR][FORM_QUANT];
  else
    tx = get_moved(x, L_ROWMAJOR);
  const int ty = alias_tensor(tx, n.out->shape);
  set_main(n.out, ty);
}

// -------------------------------------------------------------- Resize ----
void Planner::lower_resize(int ni) {
  Node& n = comp_->nodes[ni];
  const _odla_value* x = n.in[0];
  const int tx = get(x, L_NHWC, FORM_FLOAT);
  const PTensor px = T(tx);
  const Shape& xs = x->shape;
  const Shape& os = n.out->shape;
  const int ty = new_tensor(px.dt, L_NHWC, os, px.cs, SP_ARENA);
  const int es = dtype_size(px.dt);
  const int N = (int)xs.d[0], H = (int)xs.d[2], W = (int)xs.d[3], cs = px.cs, Ho = (int)os.d[2], Wo = (int)os.d[3];
  const Ref a = ref(tx), b = ref(ty);
  if (n.i[0] == ODLA_LINEAR) {
    const DType dt = px.dt;
    if (!dtype_is_float(dt)) fail(ODLA_UNSUPPORTED_DATATYPE, "linear odla_Resize of a non-float value ('%s')", n.out->name.c_str());
    emit("resize.linear:" + n.out->name, {tx}, {ty}, [=](const ExecEnv& e, hipStream_t st) {
      return launch_resize_linear_nhwc(a(e), b(e), dt, N, H, W, cs, Ho, Wo, st);
    });
  } else {
    emit("resize:" + n.out->name, {tx}, {ty}, [=](const ExecEnv& e, hipStream_t st) {
      return launch_resize_nearest_nhwc(a(e), b(e), es, N, H, W, cs, Ho, Wo, st);
    });
  }
  set_main(n.out, ty);
}

// --------------------------------------------------------------- Slice ----
void Planner::lower_slice(int ni) {
  Node& n = comp_->nodes[ni];
  const _odla_value* x = n.in[0];
  const int tx = get(x, L_ROWMAJOR, FORM_FLOAT);
  const Shape& xs = x->shape;
  const Shape& os = n.out->shape;
  const int r = xs.rank;
  if (r > 8) fail(ODLA_UNSUPPORTED_OP, "odla_Slice of rank > 8");
  const DType dt = T(tx).dt;
  const int ty = new_tensor(dt, L_ROWMAJOR, os, 0, SP_ARENA);
  StridedCopyParams cp;
  cp.elem_size = dtype_size(dt);
  cp.rank = r;
  int64_t sx = 1, sy = 1;
  for (int i = r - 1; i >= 0; --i) {
    cp.dims[i] = os.d[i];
    cp.sx[i] = sx * n.iv[2 * r + i];
    cp.sy[i] = sy;
    cp.x_off += n.iv[i] * sx;
    sx *= xs.d[i];
    sy *= os.d[i];
  }
  strided_copy_step("slice:" + n.out->name, tx, ty, cp);
  set_main(n.out, ty);
}

// ------------------------------------- Pad / Tile / broadcast / stuffing ----
void Planner::lower_copynd(int ni) {
  Node& n = comp_->nodes[ni];
  const _odla_value* x = n.in[0];
  const int tx = get(x, L_ROWMAJOR, FORM_FLOAT);
  const DType dt = T(tx).dt;
  const int ty = new_tensor(dt, L_ROWMAJOR, n.out->shape, 0, SP_ARENA);
  const int r = (int)n.iv[0];
  if (r > 8) fail(ODLA_UNSUPPORTED_OP, "copy of rank > 8 ('%s')", n.out->name.c_str());
  StridedCopyParams cp;
  cp.elem_size = dtype_size(dt);
  cp.rank = r;
  for (int i = 0; i < r; ++i) {
    cp.dims[i] = n.iv[1 + i];
    cp.sx[i] = n.iv[1 + r + i];
    cp.sy[i] = n.iv[1 + 2 * r + i];
  }
  cp.x_off = n.iv[1 + 3 * r];
  cp.y_off = n.iv[2 + 3 * r];
  if (n.i[0] != 0) {
    // the value 0 has an all-zero encoding in every storage type
    const size_t bytes = (T(ty).bytes + 3) & ~(size_t)3;
    const Ref b = ref(ty);
    emit("fill:" + n.out->name, {}, {ty}, [=](const ExecEnv& e, hipStream_t st) { return launch_fill_bytes(b(e), bytes, 0u, st); });
  }
  strided_copy_step("copy:" + n.out->name, tx, ty, cp);
  set_main(n.out, ty);
}

// ---------------------------------------------------------------- TopK ----
void Planner::lower_topk(int ni) {
  Node& n = comp_->nodes[ni];
  const _odla_value* x = n.in[0];
  const Shape& xs = x->shape;
  const int axis = (int)n.i[2], K = (int)n.i[0];
  const bool largest = n.i[1] != 0;
  const int tx = get(x, L_ROWMAJOR, FORM_FLOAT);
  int64_t outer = 1, inner = 1;
  for (int i = 0; i < axis; ++i) outer *= xs.d[i];
  for (int i = axis + 1; i < xs.rank; ++i) inner *= xs.d[i];
  const int64_t len = xs.d[axis];
  const DType dt = T(tx).dt, idt = storage_dtype(n.out2);
  const int tv = new_tensor(dt, L_ROWMAJOR, n.out->shape, 0, SP_ARENA);
  const int ti = new_tensor(idt, L_ROWMAJOR, n.out2->shape, 0, SP_ARENA);
  const Ref a = ref(tx), rv = ref(tv), ri = ref(ti);
  emit("topk:" + n.out->name, {tx}, {tv, ti}, [=](const ExecEnv& e, hipStream_t st) {
    return launch_topk(a(e), rv(e), ri(e), dt, idt, outer, len, inner, K, largest, st);
  });
  set_main(n.out, tv);
  set_main(n.out2, ti);
}

// ----------------------------------------------------------------- LRN ----
void Planner::lower_lrn(int ni) {
  Node& n = comp_->nodes[ni];
  const _odla_value* x = n.in[0];
  const Shape& xs = x->shape;
  const bool cl = n.i[0] == ODLA_CHANNELS_LAST;
  const int tx = get(x, L_ROWMAJOR, FORM_FLOAT);
  const DType dt = T(tx).dt;
  const int ty = new_tensor(dt, L_ROWMAJOR, xs, 0, SP_ARENA);
  // row-major [N][C][inner]; channels-last data is the case inner == 1
  int64_t N, inner;
  int C;
  if (cl) {
    C = (int)xs.d[xs.rank - 1];
    N = xs.numel() / C;
    inner = 1;
  } else {
    N = xs.d[0];
    C = (int)xs.d[1];
    inner = xs.numel() / (N * C);
  }
  const int half = ((int)n.i[1] - 1) / 2;
  const float alpha = n.f[0], beta = n.f[1], bias = n.f[2];
  const Ref a = ref(tx), b = ref(ty);
  emit("lrn:" + n.out->name, {tx}, {ty}, [=](const ExecEnv& e, hipStream_t st) {
    return launch_lrn(a(e), b(e), dt, N, C, inner, half, alpha, beta, bias, st);
  });
  set_main(n.out, ty);
}

// ------------------------------------------------- InstanceNormalization ----
void Planner::lower_rownorm(int ni) {
  Node& n = comp_->nodes[ni];
  const _odla_value* x = n.in[0];
  const Shape& xs = x->shape;
  if (n.i[0] == ODLA_CHANNELS_LAST) fail(ODLA_UNSUPPORTED_OP, "channels-last instance normalisation ('%s')", n.out->name.c_str());
  const int tx = get(x, L_ROWMAJOR, FORM_FLOAT);
  const DType dt = T(tx).dt;
  const int ty = new_tensor(dt, L_ROWMAJOR, xs, 0, SP_ARENA);
  const int C = (int)xs.d[1];
  const int64_t rows = xs.d[0] * C, len = xs.numel() / rows;
  int tg = -1, tb = -1;
  if (n.in[1]) tg = const_vector<float>(DT_F32, const_as_float(n.in[1]));
  if (n.in[2]) tb = const_vector<float>(DT_F32, const_as_float(n.in[2]));
  const float eps = n.f[0], sg = n.f[1], sb = n.f[2];
  const Ref a = ref(tx), b = ref(ty), rg = ref(tg >= 0 ? tg : tx), rb = ref(tb >= 0 ? tb : tx);
  const bool hg = tg >= 0, hb = tb >= 0;
  emit("instnorm:" + n.out->name, {tx}, {ty}, [=](const ExecEnv& e, hipStream_t st) {
    return launch_rownorm(a(e), b(e), dt, rows, len, C, hg ? (const float*)rg(e) : nullptr,
                          hb ? (const float*)rb(e) : nullptr, sg, sb, eps, st);
  });
  set_main(n.out, ty);
}

// ----------------------------------------------------------- Transpose ----
void Planner::lower_transpose(int ni) {
  Node& n = comp_->nodes[ni];
  const _odla_value* x = n.in[0];
  const Shape& xs = x->shape;
  const Shape& os = n.out->shape;
  const int r = xs.rank;
  if (r > 8) fail(ODLA_UNSUPPORTED_OP, "odla_Transpose of rank > 8");
  // N,C,H,W -> N,H,W,C of a value that already lives channels-last is free
  const VState& s = vs_[x->index];
  if (r == 4 && n.iv[0] == 0 && n.iv[1] == 2 && n.iv[2] == 3 && n.iv[3] == 1 && s.main >= 0 &&
      T(s.main).layout == L_NHWC && !T(s.main).quant && T(s.main).cs == xs.d[1]) {
    set_main(n.out, alias_tensor(s.main, os));
    return;
  }
  const int tx = get_moved(x, L_ROWMAJOR);
  const DType dt = T(tx).dt;
  const int ty = new_tensor(dt, L_ROWMAJOR, os, 0, SP_ARENA);
  int64_t xstr[ODLA_MAX_DIMENSION];
  {
    int64_t acc = 1;
    for (int i = r - 1; i >= 0; --i) { xstr[i] = acc; acc *= xs.d[i]; }
  }
  StridedCopyParams cp;
  cp.elem_size = dtype_size(dt);
  cp.rank = r;
  int64_t sy = 1;
  for (int i = r - 1; i >= 0; --i) {
    cp.dims[i] = os.d[i];
    cp.sx[i] = xstr[n.iv[i]];
    cp.sy[i] = sy;
    sy *= os.d[i];
  }
  strided_copy_step("transpose:" + n.out->name, tx, ty, cp);
  set_main(n.out, ty);
}

// ------------------------------------------------- Quantize/Dequantize ----
void Planner::lower_qdq(int ni) {
  Node& n = comp_->nodes[ni];
  const _odla_value* x = n.in[0];
  const bool quant = n.op == OP_QUANTIZE;
  const int tx = get(x, L_ROWMAJOR, FORM_FLOAT);
  const Shape& xs = x->shape;
  const int axis = (int)n.i[0];
  std::vector<float> sc = const_as_float(n.in[1]);
  std::vector<int32_t> zp;
  if (n.in[2]) { std::vector<float> z = const_as_float(n.in[2]); for (float v : z) zp.push_back((int32_t)v); }
  const int channels = (int)sc.size();
  int64_t inner = 1;
  if (channels > 1) for (int i = axis + 1; i < xs.rank; ++i) inner *= xs.d[i];
  const int ts = const_vector<float>(DT_F32, sc);
  const int tz = zp.empty() ? -1 : const_vector<int32_t>(DT_I32, zp);
  const DType odt = storage_dtype(n.out);
  const int ty = new_tensor(odt, L_ROWMAJOR, n.out->shape, 0, SP_ARENA);
  QuantParams qp;
  qp.n = xs.numel(); qp.inner = inner; qp.channels = channels;
  qp.src_dt = T(tx).dt; qp.dst_dt = odt;
  qp.dst_signed = quant ? (odt == DT_I8) : (T(tx).dt == DT_I8);
  const Ref a = ref(tx), b = ref(ty), rs = ref(ts), rz = ref(tz >= 0 ? tz : ts);
  const bool hz = tz >= 0;
  emit(std::string(quant ? "quantize:" : "dequantize:") + n.out->name, {tx}, {ty}, [=](const ExecEnv& e, hipStream_t st) {
    QuantParams p = qp; p.src = a(e); p.dst = b(e); p.scale = (const float*)rs(e); p.zp = hz ? (const int32_t*)rz(e) : nullptr;
    return quant ? launch_quantize(p, st) : launch_dequantize(p, st);
  });
  set_main(n.out, ty);
}

// ----------------------------------------------------------------- NMS ----
void Planner::lower_nms(int ni) {
  Node& n = comp_->nodes[ni];
  const _odla_value* boxes = n.in[0];
  const _odla_value* scores = n.in[1];
  // fp32 / fp16 / bf16 are read as they are stored; anything else is converted first
  auto as_float = [&](const _odla_value* v) -> int {
    int t = get(v, L_ROWMAJOR, FORM_FLOAT);
    if (T(t).dt == DT_F32 || T(t).dt == DT_F16 || T(t).dt == DT_BF16) return t;
    const int d = new_tensor(DT_F32, L_ROWMAJOR, v->shape, 0, SP_ARENA);
    const int64_t ne = v->shape.numel();
    const DType sdt = T(t).dt;
    const Ref a = ref(t), b = ref(d);
    emit("nms.cast:" + v->name, {t}, {d}, [=](const ExecEnv& e, hipStream_t st) { return launch_cast(a(e), sdt, b(e), DT_F32, ne, st); });
    return d;
  };
  const int tb = as_float(boxes), ts = as_float(scores);
  const DType bdt = T(tb).dt, sdt = T(ts).dt;
  const int N = (int)boxes->shape.d[0], B = (int)boxes->shape.d[1], C = (int)scores->shape.d[1];
  const int max_out = (int)n.i[0];
  const float iou = n.f[0], thr = n.f[1];
  const int tw = raw_buffer(nms_workspace_bytes(N, B), SP_ARENA);
  Shape o32 = n.out->shape;
  const int ty = new_tensor(DT_I32, L_ROWMAJOR, o32, 0, SP_ARENA);
  const Ref rb = ref(tb), rs = ref(ts), rw = ref(tw), ry = ref(ty);
  emit("nms:" + n.out->name, {tb, ts, tw}, {ty, tw}, [=](const ExecEnv& e, hipStream_t st) {
    return launch_nms(rb(e), bdt, rs(e), sdt, N, C, B, max_out, iou, thr, (int32_t*)ry(e), rw(e), st, e.image_base);
  });
  if (dtype_from_odla(n.out->etype) == DT_I64) {
    const int t64 = new_tensor(DT_I64, L_ROWMAJOR, o32, 0, SP_ARENA);
    const int64_t ne = o32.numel();
    const Ref c = ref(t64);
    emit("nms.i64:" + n.out->name, {ty}, {t64}, [=](const ExecEnv& e, hipStream_t st) { return launch_cast(ry(e), DT_I32, c(e), DT_I64, ne, st); });
    set_main(n.out, t64);
  } else {
    set_main(n.out, ty);
  }
}

// -------------------------------------------------------- PostProcess ----
// [ref: ODLA/platforms/odla_popart/custom_ops/postprocess.cc:139-290: anchors of
//  the 13-, 26- and 52-cell heads, thresholds 0.45 / 0.3, N / 169 rows per class]
void Planner::lower_postprocess(int ni) {
  Node& n = comp_->nodes[ni];
  auto as_f32 = [&](const _odla_value* v) -> int {
    int t = get(v, L_ROWMAJOR, FORM_FLOAT);
    if (T(t).dt == DT_F32) return t;
    const int d = new_tensor(DT_F32, L_ROWMAJOR, v->shape, 0, SP_ARENA);
    const int64_t ne = v->shape.numel();
    const DType sdt = T(t).dt;
    const Ref a = ref(t), b = ref(d);
    emit("postprocess.cast:" + v->name, {t}, {d}, [=](const ExecEnv& e, hipStream_t st) { return launch_cast(a(e), sdt, b(e), DT_F32, ne, st); });
    return d;
  };
  const int tw = get(n.in[0], L_ROWMAJOR, FORM_FLOAT), th = get(n.in[1], L_ROWMAJOR, FORM_FLOAT);
  if (T(tw).dt != DT_I32 || T(th).dt != DT_I32) fail(ODLA_UNSUPPORTED_DATATYPE, "odla_PostProcess: the image size must be 32-bit integers");
  const int t0 = as_f32(n.in[2]), t1 = as_f32(n.in[3]), t2 = as_f32(n.in[4]);
  struct Args { int dims[3]; int anchors[3][6]; } a;
  static const int kAnchors[3][6] = {{116, 90, 156, 198, 373, 326}, {30, 61, 62, 45, 59, 119}, {10, 13, 16, 30, 33, 23}};
  int total = 0;
  for (int h = 0; h < 3; ++h) {
    a.dims[h] = (int)n.in[2 + h]->shape.d[2];
    total += 3 * a.dims[h] * a.dims[h];
    for (int k = 0; k < 6; ++k) a.anchors[h][k] = kAnchors[h][k];
  }
  const int classes = (int)n.out->shape.d[0], capacity = (int)n.out->shape.d[1];
  Shape bs, ss;
  bs.rank = 2; bs.d[0] = total; bs.d[1] = 4;
  ss.rank = 2; ss.d[0] = classes; ss.d[1] = total;
  const int tb = new_tensor(DT_F32, L_ROWMAJOR, bs, 0, SP_ARENA);
  const int ts = new_tensor(DT_F32, L_ROWMAJOR, ss, 0, SP_ARENA);
  const int ti = new_tensor(DT_F32, L_ROWMAJOR, n.out->shape, 0, SP_ARENA);
  const int tn = new_tensor(DT_I32, L_ROWMAJOR, n.out2->shape, 0, SP_ARENA);
  const float iou = n.f[0], thr = n.f[1];
  const Ref rw = ref(tw), rh = ref(th), r0 = ref(t0), r1 = ref(t1), r2 = ref(t2), rb = ref(tb), rs = ref(ts), ri = ref(ti), rn = ref(tn);
  emit("postprocess:" + n.out->name, {tw, th, t0, t1, t2}, {tb, ts, ti, tn}, [=](const ExecEnv& e, hipStream_t st) {
    const float* heads[3] = {(const float*)r0(e), (const float*)r1(e), (const float*)r2(e)};
    return launch_yolo_postprocess(heads, a.dims, classes, a.anchors, (const int*)rw(e), (const int*)rh(e), iou, thr,
                                   capacity, (float*)rb(e), (float*)rs(e), (float*)ri(e), (int*)rn(e), st);
  });
  set_main(n.out, ti);
  set_main(n.out2, tn);
}

}  // namespace

// ============================================================================
odla_status plan_summary(_odla_computation* comp, int* launches, int* init_launches, size_t* arena_bytes,
                         size_t* const_bytes) {
  auto plan = std::make_unique<Plan>();
  for (Node& n : comp->nodes) n.absorbed = false;
  odla_status st = ODLA_SUCCESS;
  try {
    Planner p(comp, plan.get());
    p.run();
  } catch (const PlanError& e) {
    OHIP_ERR("cannot compile computation: %s", e.msg.c_str());
    st = e.status;
  } catch (const std::exception& e) {
    OHIP_ERR("cannot compile computation: %s", e.what());
    st = ODLA_FAILURE;
  }
  for (Node& n : comp->nodes) n.absorbed = false;
  if (st != ODLA_SUCCESS) return st;
  for (const Step& sp : plan->steps) OHIP_DEBUG("step %s", sp.name.c_str());
  *launches = (int)plan->steps.size();
  *init_launches = (int)plan->init_steps.size();
  *arena_bytes = plan->arena_bytes;
  *const_bytes = plan->const_bytes;
  return ODLA_SUCCESS;
}

odla_status build_plan(_odla_computation* comp, std::unique_ptr<Plan>* out) {
  auto plan = std::make_unique<Plan>();
  // fusion marks are per-plan
  for (Node& n : comp->nodes) n.absorbed = false;
  try {
    Planner p(comp, plan.get());
    p.run();
  } catch (const PlanError& e) {
    OHIP_ERR("cannot compile computation: %s", e.msg.c_str());
    return e.status;
  } catch (const std::exception& e) {
    OHIP_ERR("cannot compile computation: %s", e.what());
    return ODLA_FAILURE;
  }

  // ---- constant pool + one-time initialisation steps ----
  char* init_tmp = nullptr;
  auto cleanup = [&]() { if (init_tmp) (void)hipFree(init_tmp); };
  if (plan->const_bytes > 0 &&
      hipMalloc(reinterpret_cast<void**>(&plan->const_pool), plan->const_bytes) != hipSuccess) {
    OHIP_ERR("cannot allocate %zu bytes for constants", plan->const_bytes);
    return ODLA_MEM_ERROR;
  }
  if (plan->init_bytes > 0 && hipMalloc(reinterpret_cast<void**>(&init_tmp), plan->init_bytes) != hipSuccess) {
    OHIP_ERR("cannot allocate %zu bytes of initialisation scratch", plan->init_bytes);
    return ODLA_MEM_ERROR;
  }
  for (const Plan::Blob& b : plan->blobs) {
    char* base = b.space == SP_CONST ? plan->const_pool : init_tmp;
    const void* src = b.src ? b.src : b.owned.data();
    if (hipMemcpy(base + b.offset, src, b.bytes, hipMemcpyHostToDevice) != hipSuccess) {
      OHIP_ERR("upload of a constant failed");
      cleanup();
      return ODLA_FAILURE;
    }
  }
  ExecEnv env;
  env.base[SP_CONST] = plan->const_pool;
  env.base[SP_INIT] = init_tmp;
  for (const Step& s : plan->init_steps) {
    hipError_t e = s.fn(env, nullptr);
    if (e != hipSuccess) {
      OHIP_ERR("initialisation step '%s' failed: %s", s.name.c_str(), hipGetErrorString(e));
      cleanup();
      return ODLA_FAILURE;
    }
  }
  if (hipDeviceSynchronize() != hipSuccess) {
    OHIP_ERR("device error while preparing constants");
    cleanup();
    return ODLA_FAILURE;
  }
  cleanup();
  plan->blobs.clear();
  plan->blobs.shrink_to_fit();
  plan->init_steps.clear();
  OHIP_INFO("plan: %zu steps, arena %.1f MiB, constants %.1f MiB", plan->steps.size(),
            plan->arena_bytes / 1048576.0, plan->const_bytes / 1048576.0);
  *out = std::move(plan);
  return ODLA_SUCCESS;
}

}  // namespace ohip
