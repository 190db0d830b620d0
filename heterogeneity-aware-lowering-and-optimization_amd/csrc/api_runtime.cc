// ODLA control plane of libodla_hip.so: computations, contexts, binding,
// execution (hipGraph replay), value introspection, device / memory / logging.
#include <atomic>
#include <cstdlib>
#include <chrono>
#include <cstring>

#include "internal.h"

using namespace ohip;

// ---------------------------------------------------------------- logging --
namespace {
std::atomic<int> g_log_level{ODLA_LOG_LEVEL_ERROR};

void default_logger(const char* file, int line, const char* func, odla_log_level level, const char* msg) {
  (void)func;
  if ((int)level > g_log_level.load()) return;
  static const char tags[] = {'-', 'F', 'E', 'W', 'I', 'D', 'T'};
  const char tag = (level >= 0 && level <= ODLA_LOG_LEVEL_TRACE) ? tags[level] : '?';
  if (file != nullptr && line > 0) fprintf(stderr, "[odla_hip %c] %s:%d %s\n", tag, file, line, msg);
  else fprintf(stderr, "[odla_hip %c] %s\n", tag, msg);
}
std::atomic<odla_logging_func> g_logger{default_logger};

std::mutex g_registry_mu;
std::vector<_odla_computation*> g_computations;  // live computations, creation order
thread_local _odla_computation* t_current = nullptr;

const char* kVersion = "odla_hip 0.5.0 (gfx950)";
}  // namespace

namespace ohip {

void log_msg(const char* file, int line, const char* func, odla_log_level lvl, const char* fmt, ...) {
  if ((int)lvl > g_log_level.load() && g_logger.load() == default_logger) return;
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  const char* base = file ? strrchr(file, '/') : nullptr;
  g_logger.load()(base ? base + 1 : file, line, func, lvl, buf);
}

const char* op_name(OpKind k) {
  static const char* names[] = {"Conv", "Gemm", "Binary", "Unary", "BatchNorm", "LayerNorm", "Pool",
                                "Reduce", "Softmax", "Cast", "Concat", "Gather", "Reshape", "Resize",
                                "Slice", "Transpose", "Quantize", "Dequantize", "NMS", "Elementwise", "ArgExtreme",
                                "CopyND", "TopK", "LRN", "RowNorm", "PostProcess", "AxisOp"};
  static_assert(sizeof(names) / sizeof(names[0]) == (size_t)OP_AXISOP + 1, "one name per OpKind");
  if ((int)k < 0 || (int)k > (int)OP_AXISOP) return "?";
  return names[(int)k];
}

std::string Shape::str() const {
  std::string s = "[";
  for (int i = 0; i < rank; ++i) {
    if (i) s += ",";
    s += std::to_string(d[i]);
  }
  return s + "]";
}

Shape shape_from(const odla_value_shape& s) {
  Shape r;
  if (s.size <= 0) {  // scalar: rewritten to {1} as the reference does [ref: odla_dnnl.cc:181-190]
    r.rank = 1;
    r.d[0] = 1;
    return r;
  }
  r.rank = s.size > ODLA_MAX_DIMENSION ? ODLA_MAX_DIMENSION : s.size;
  for (int i = 0; i < r.rank; ++i) r.d[i] = s.dims[i];
  return r;
}

odla_value_shape shape_to(const Shape& s) {
  odla_value_shape r;
  memset(&r, 0, sizeof(r));
  r.size = s.rank;
  for (int i = 0; i < s.rank; ++i) r.dims[i] = s.d[i];
  return r;
}

bool shape_valid(const odla_value_shape& s) {
  if (s.size < 1 || s.size > ODLA_MAX_DIMENSION) return false;
  for (int i = 0; i < s.size; ++i)
    if (s.dims[i] <= 0 || s.dims[i] > (1ll << 40)) return false;
  return true;
}

DType dtype_from_odla(odla_element_type t) {
  switch (t) {
    case ODLA_FLOAT32: return DT_F32;
    case ODLA_FLOAT16: return DT_F16;
    case ODLA_BFLOAT16: return DT_BF16;
    case ODLA_INT8: case ODLA_QINT8: return DT_I8;
    case ODLA_UINT8: case ODLA_QUINT8: return DT_U8;
    case ODLA_INT32: case ODLA_QINT32: case ODLA_UINT32: return DT_I32;
    case ODLA_INT64: case ODLA_UINT64: return DT_I64;
    case ODLA_BOOL: return DT_BOOL;
    default: return DT_INVALID;
  }
}

int odla_type_size(odla_element_type t) { return dtype_size(dtype_from_odla(t)); }

_odla_computation* current_computation() {
  if (t_current != nullptr) return t_current;
  std::lock_guard<std::mutex> lk(g_registry_mu);
  return g_computations.empty() ? nullptr : g_computations.back();
}
void set_current_computation(_odla_computation* c) { t_current = c; }
void forget_computation(_odla_computation* c) {
  if (t_current == c) t_current = nullptr;
  std::lock_guard<std::mutex> lk(g_registry_mu);
  for (size_t i = 0; i < g_computations.size(); ++i)
    if (g_computations[i] == c) { g_computations.erase(g_computations.begin() + i); break; }
}

_odla_value* new_value(_odla_computation* c, _odla_value::Kind kind, odla_element_type et,
                       const Shape& shape, const odla_value_id id) {
  auto v = std::make_unique<_odla_value>();
  v->kind = kind;
  v->etype = et;
  v->shape = shape;
  v->comp = c;
  v->index = (int)c->values.size();
  if (id != nullptr) {
    v->name = reinterpret_cast<const char*>(id);
    if (!v->name.empty()) c->by_name[v->name] = v.get();
  }
  _odla_value* raw = v.get();
  c->values.push_back(std::move(v));
  return raw;
}

Plan::~Plan() {
  if (const_pool != nullptr) (void)hipFree(const_pool);
}

}  // namespace ohip

namespace {

bool is_live(_odla_computation* c) {
  std::lock_guard<std::mutex> lk(g_registry_mu);
  for (auto* p : g_computations)
    if (p == c) return true;
  return false;
}

odla_status ensure_plan(_odla_computation* c) {
  std::lock_guard<std::mutex> lk(c->mu);
  if (c->plan) return ODLA_SUCCESS;
  if (c->plan_failed) return ODLA_FAILURE;
  std::unique_ptr<Plan> plan;
  profiler_configure(&c->opts);
  odla_status st = build_plan(c, &plan);
  if (st != ODLA_SUCCESS) {
    c->plan_failed = true;
    return st;
  }
  c->plan = std::move(plan);
  c->planned_nodes = c->nodes.size();
  return ODLA_SUCCESS;
}

}  // namespace
namespace ohip {
odla_status compile_computation(_odla_computation* c) { return ensure_plan(c); }
}  // namespace ohip
namespace {

void drop_graph(_odla_context* ctx) {
  if (ctx->graph_exec) { (void)hipGraphExecDestroy(ctx->graph_exec); ctx->graph_exec = nullptr; }
  if (ctx->graph) { (void)hipGraphDestroy(ctx->graph); ctx->graph = nullptr; }
  ctx->graph_ext.clear();
  for (_odla_context::ParkedGraph& g : ctx->parked_graphs) {
    if (g.exec) (void)hipGraphExecDestroy(g.exec);
    if (g.graph) (void)hipGraphDestroy(g.graph);
  }
  ctx->parked_graphs.clear();
}

constexpr size_t kMaxParkedGraphs = 3;

// The captured launches hold the argument buffers they read in place.  When the
// caller has bound other buffers, the current graph is set aside and one captured
// for these buffers comes back, if there is one; otherwise graph_exec stays null and
// the caller captures.
void select_graph(_odla_context* ctx, const std::vector<const char*>& ext) {
  if (ctx->graph_exec == nullptr || ctx->graph_ext == ext) return;
  ctx->parked_graphs.push_back({ctx->graph_ext, ctx->graph, ctx->graph_exec});
  ctx->graph = nullptr;
  ctx->graph_exec = nullptr;
  for (size_t i = 0; i < ctx->parked_graphs.size(); ++i) {
    if (ctx->parked_graphs[i].ext != ext) continue;
    ctx->graph = ctx->parked_graphs[i].graph;
    ctx->graph_exec = ctx->parked_graphs[i].exec;
    ctx->graph_ext = ext;
    ctx->parked_graphs.erase(ctx->parked_graphs.begin() + (long)i);
    return;
  }
  if (ctx->parked_graphs.size() > kMaxParkedGraphs) {
    (void)hipGraphExecDestroy(ctx->parked_graphs.front().exec);
    (void)hipGraphDestroy(ctx->parked_graphs.front().graph);
    ctx->parked_graphs.erase(ctx->parked_graphs.begin());
  }
}

// ODLA_HIP_IN_PLACE_ARGS=0 copies every argument into the arena, as for host buffers.
bool in_place_args_enabled() {
  static const bool on = [] {
    const char* e = getenv("ODLA_HIP_IN_PLACE_ARGS");
    return e == nullptr || strcmp(e, "0") != 0;
  }();
  return on;
}

bool is_device_memory(const void* p) {
  hipPointerAttribute_t attr;
  if (hipPointerGetAttributes(&attr, p) != hipSuccess) {
    (void)hipGetLastError();   // ordinary host memory is reported as an error
    return false;
  }
  return attr.type == hipMemoryTypeDevice;
}

odla_status run_steps(_odla_context* ctx, const Plan& plan, char* arena, const std::vector<const char*>* ext = nullptr) {
  ExecEnv env;
  env.base[SP_ARENA] = arena;
  env.base[SP_CONST] = plan.const_pool;
  env.ext = ext != nullptr && !ext->empty() ? ext->data() : nullptr;
  env.image_base = ctx->image_base;
  for (const Step& s : plan.steps) {
    hipError_t e = s.fn(env, ctx->stream);
    if (e != hipSuccess) {
      OHIP_ERR("step '%s' failed: %s", s.name.c_str(), hipGetErrorString(e));
      return ODLA_FAILURE;
    }
  }
  return ODLA_SUCCESS;
}

// Copies the bound arguments into their staging tensors.  With `ext`, an argument
// that lives in device memory and that the plan can read in place is not copied:
// its buffer is entered in (*ext)[k] instead (nullptr for the copied ones).
odla_status stage_inputs(_odla_context* ctx, const Plan& plan, char* arena, std::vector<const char*>* ext = nullptr) {
  if (ext != nullptr) ext->assign(plan.inputs.size() + plan.outputs.size(), nullptr);
  for (size_t k = 0; k < plan.inputs.size(); ++k) {
    const Plan::IO& io = plan.inputs[k];
    auto it = ctx->bound_in.find(io.v);
    if (it == ctx->bound_in.end()) {
      OHIP_ERR("argument '%s' is not bound", io.v->name.c_str());
      return ODLA_INVALID_PARAM;
    }
    if (ext != nullptr && io.in_place_ok && !ctx->in_place_off && in_place_args_enabled() && is_device_memory(it->second)) {
      (*ext)[k] = static_cast<const char*>(it->second);
      OHIP_DEBUG("argument '%s' is read in place", io.v->name.c_str());
      continue;
    }
    char* dst = arena + plan.tensors[io.tensor].offset;
    if (hipMemcpyAsync(dst, it->second, io.bytes, hipMemcpyDefault, ctx->stream) != hipSuccess) {
      OHIP_ERR("copy of argument '%s' failed", io.v->name.c_str());
      return ODLA_FAILURE;
    }
  }
  return ODLA_SUCCESS;
}

// Results bound to device memory that the final conversion can write directly: their
// buffers are entered behind the arguments in *ext (filled by stage_inputs).  A buffer
// that overlaps an argument read in place keeps its copy.
void place_outputs(_odla_context* ctx, const Plan& plan, std::vector<const char*>* ext) {
  if (!in_place_args_enabled() || ctx->in_place_off) return;
  const size_t n_in = plan.inputs.size();
  for (size_t k = 0; k < plan.outputs.size(); ++k) {
    const Plan::IO& io = plan.outputs[k];
    if (!io.in_place_ok) continue;
    auto it = ctx->bound_out.find(io.v);
    if (it == ctx->bound_out.end() || it->second == nullptr) continue;
    const char* p = static_cast<const char*>(it->second);
    if ((reinterpret_cast<uintptr_t>(p) & 15u) != 0 || !is_device_memory(p)) continue;
    bool clash = false;
    for (size_t j = 0; j < n_in + k && !clash; ++j) {
      const char* q = (*ext)[j];
      if (q == nullptr) continue;
      const size_t qb = j < n_in ? plan.inputs[j].bytes : plan.outputs[j - n_in].bytes;
      clash = p < q + qb && q < p + io.bytes;
    }
    if (clash) continue;
    (*ext)[n_in + k] = p;
    OHIP_DEBUG("result '%s' is written in place", io.v->name.c_str());
  }
}

// Copies the bound results out of `arena` (or the constant pool) and waits for the stream.
odla_status fetch_outputs(_odla_context* ctx, const Plan& plan, const char* arena,
                          const std::vector<const char*>* ext = nullptr, const bool wait = true) {
  for (size_t k = 0; k < plan.outputs.size(); ++k) {
    const Plan::IO& io = plan.outputs[k];
    auto it = ctx->bound_out.find(io.v);
    if (it == ctx->bound_out.end()) continue;
    if (ext != nullptr && !ext->empty() && (*ext)[plan.inputs.size() + k] != nullptr) continue;   // already there
    const PTensor& t = plan.tensors[io.tensor];
    const char* src = (t.space == SP_CONST ? plan.const_pool : arena) + t.offset + io.offset;
    if (hipMemcpyAsync(it->second, src, io.bytes, hipMemcpyDefault, ctx->stream) != hipSuccess) {
      OHIP_ERR("copy of output '%s' failed", io.v->name.c_str());
      return ODLA_FAILURE;
    }
  }
  if (!wait) return ODLA_SUCCESS;   // (the caller waits for the stream itself)
  hipError_t e = hipStreamSynchronize(ctx->stream);
  if (e != hipSuccess) {
    OHIP_ERR("device error: %s", hipGetErrorString(e));
    return ODLA_FAILURE;
  }
  return ODLA_SUCCESS;
}

odla_status create_context_for(_odla_computation* c, odla_context* context);

// The context that executes `ctx`'s computation at batch `bs`: `ctx` itself at
// the recorded batch, otherwise a context over a rescaled copy of the recording
// (made, planned and given an arena on first use).
// Destroys a context and the contexts it holds over batch variants.
void destroy_context_tree(_odla_context* ctx) {
  for (auto& kv : ctx->variant_ctx) destroy_context_tree(kv.second.ctx);
  ctx->variant_ctx.clear();
  for (_odla_context*& h : ctx->split.half) {
    if (h != nullptr) destroy_context_tree(h);
    h = nullptr;
  }
  ctx->split.comp.reset();
  if (ctx->stream) (void)hipStreamSynchronize(ctx->stream);
  drop_graph(ctx);
  if (ctx->inputs_staged) (void)hipEventDestroy(ctx->inputs_staged);
  if (ctx->arena) (void)hipFree(ctx->arena);
  if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
  delete ctx;
}

// Smallest batch at which a context tries two half-batch copies against the whole batch (see split_threshold).
constexpr int kMinTrialBatch = 8;

// Batches (other than the recorded one) a context keeps planned at a time.
int max_batch_variants() {
  static const int n = [] {
    const char* e = getenv("ODLA_HIP_MAX_BATCH_VARIANTS");
    const int v = e ? atoi(e) : 0;
    return v >= 1 ? v : 4;
  }();
  return n;
}

odla_status variant_context(_odla_context* ctx, int bs, _odla_context** out) {
  _odla_computation* c = ctx->comp;
  const int rec = recorded_batch(*c);
  if (bs == 0 || bs == rec) { *out = ctx; return ODLA_SUCCESS; }
  auto have = ctx->variant_ctx.find(bs);
  if (have != ctx->variant_ctx.end()) {
    have->second.last_use = ++ctx->variant_clock;
    *out = have->second.ctx;
    return ODLA_SUCCESS;
  }
  // make room first, so that the peak stays within the bound
  while ((int)ctx->variant_ctx.size() >= max_batch_variants()) {
    auto lru = ctx->variant_ctx.begin();
    for (auto it = ctx->variant_ctx.begin(); it != ctx->variant_ctx.end(); ++it)
      if (it->second.last_use < lru->second.last_use) lru = it;
    destroy_context_tree(lru->second.ctx);
    ctx->variant_ctx.erase(lru);  // drops this context's share of the variant: the last share frees its plan
  }
  std::shared_ptr<_odla_computation> v;
  {
    std::lock_guard<std::mutex> lk(c->mu);
    auto it = c->variants.find(bs);
    if (it != c->variants.end()) v = it->second.lock();
    if (!v) {
      std::unique_ptr<_odla_computation> copy = clone_for_batch(*c, rec, bs);
      if (!copy) return ODLA_UNSUPPORTED_OP;
      v = std::move(copy);
      c->variants[bs] = v;
    }
  }
  odla_context sub = nullptr;
  odla_status st = create_context_for(v.get(), &sub);
  if (st != ODLA_SUCCESS) return st;
  _odla_context::Variant& slot = ctx->variant_ctx[bs];
  slot.comp = std::move(v);
  slot.ctx = sub;
  slot.last_use = ++ctx->variant_clock;
  *out = sub;
  return ODLA_SUCCESS;
}

odla_status set_run_batch(_odla_context* ctx, int bs) {
  const int rec = recorded_batch(*ctx->comp);
  if (rec == 0) {
    OHIP_ERR("ODLA_RUN_BATCH_SIZE: the computation was not recorded with ODLA_DYNAMIC_BATCH and ODLA_MAX_BATCH_SIZE");
    return ODLA_FAILURE;
  }
  const int lo = ctx->comp->min_batch > 0 ? ctx->comp->min_batch : 1;
  if (bs < lo || bs > rec) {
    OHIP_ERR("ODLA_RUN_BATCH_SIZE: %d is outside %d..%d (ODLA_MIN_BATCH_SIZE .. ODLA_MAX_BATCH_SIZE)", bs, lo, rec);
    return ODLA_FAILURE;
  }
  _odla_context* sub = nullptr;
  odla_status st = variant_context(ctx, bs, &sub);  // compiled here, so that a graph that cannot be rescaled fails early
  if (st != ODLA_SUCCESS) return st;
  ctx->run_batch = bs;
  return ODLA_SUCCESS;
}

_odla_value* find_value(_odla_computation* c, const odla_value_id id) {
  if (c == nullptr || id == nullptr) return nullptr;
  auto it = c->by_name.find(reinterpret_cast<const char*>(id));
  return it == c->by_name.end() ? nullptr : it->second;
}

}  // namespace

extern "C" {

// ------------------------------------------------------------ computation --
odla_status odla_CreateComputation(odla_computation* computation) {
  if (computation == nullptr) return ODLA_INVALID_PARAM;
  auto* c = new (std::nothrow) _odla_computation();
  if (c == nullptr) return ODLA_MEM_ERROR;
  {
    std::lock_guard<std::mutex> lk(g_registry_mu);
    g_computations.push_back(c);
  }
  set_current_computation(c);
  *computation = c;
  return ODLA_SUCCESS;
}

static void destroy_context(odla_context ctx);

odla_status odla_DestroyComputation(odla_computation c) {
  if (c == nullptr) return ODLA_INVALID_PARAM;
  if (!is_live(c)) return ODLA_INVALID_PARAM;
  forget_computation(c);
  (void)hipDeviceSynchronize();
  if (c->eager_ctx != nullptr) destroy_context(c->eager_ctx);
  delete c;
  return ODLA_SUCCESS;
}

odla_status odla_SetComputationItem(odla_computation c, odla_item_type type, odla_item_value value) {
  if (c == nullptr) return ODLA_INVALID_PARAM;
  std::lock_guard<std::mutex> lk(c->mu);
  if (c->plan) {
    OHIP_WARN("odla_SetComputationItem(%d) after the computation was compiled is ignored", (int)type);
    return ODLA_FAILURE;
  }
  switch ((int)type) {
    case ODLA_FP16_MODE:
      if (value == nullptr) return ODLA_INVALID_PARAM;
      c->opts.fp16 = *reinterpret_cast<const bool*>(value);
      return ODLA_SUCCESS;
    case ODLA_BF16_MODE:
      if (value == nullptr) return ODLA_INVALID_PARAM;
      c->opts.bf16 = *reinterpret_cast<const odla_bf16_mode*>(value);
      return ODLA_SUCCESS;
    case ODLA_USE_DATA_TYPE: {
      if (value == nullptr) return ODLA_INVALID_PARAM;
      const odla_element_type t = *reinterpret_cast<const odla_element_type*>(value);
      if (t == ODLA_INT8 || t == ODLA_QINT8 || t == ODLA_QUINT8 || t == ODLA_UINT8) c->opts.int8 = true;
      else if (t == ODLA_FLOAT16) c->opts.fp16 = true;
      else if (t == ODLA_BFLOAT16) c->opts.bf16 = BF16_PERFORMACE_MODE;
      else if (t == ODLA_FLOAT32) { c->opts.int8 = false; c->opts.fp16 = false; c->opts.bf16 = BF16_DISABLE; }
      else return ODLA_UNSUPPORTED_DATATYPE;
      return ODLA_SUCCESS;
    }
    case ODLA_DYNAMIC_BATCH:
      if (value == nullptr) return ODLA_INVALID_PARAM;
      c->dynamic_batch = *reinterpret_cast<const bool*>(value);
      return ODLA_SUCCESS;
    case ODLA_MIN_BATCH_SIZE:
    case ODLA_MAX_BATCH_SIZE:
    case ODLA_OPT_BATCH_SIZE: {
      if (value == nullptr) return ODLA_INVALID_PARAM;
      const int n = *reinterpret_cast<const int*>(value);
      if (n < 1) return ODLA_INVALID_PARAM;
      if ((int)type == ODLA_MAX_BATCH_SIZE && !c->args.empty() && n != c->max_batch) {
        OHIP_ERR("odla_SetComputationItem: the largest batch must be set before the first argument is created");
        return ODLA_FAILURE;
      }
      ((int)type == ODLA_MIN_BATCH_SIZE ? c->min_batch : (int)type == ODLA_MAX_BATCH_SIZE ? c->max_batch : c->opt_batch) = n;
      return ODLA_SUCCESS;
    }
    case ODLA_QUANT_TABLE:
      c->opts.qtable = reinterpret_cast<const odla_value_quant_info*>(value);
      return ODLA_SUCCESS;
    case ODLA_QUANT_TABLE_SIZE:
      if (value == nullptr) return ODLA_INVALID_PARAM;
      c->opts.qtable_size = *reinterpret_cast<const int*>(value);
      return ODLA_SUCCESS;
    case 1000:  // ODLA_HIP_ITEM_RAW_INT32_ACC
      if (value == nullptr) return ODLA_INVALID_PARAM;
      c->opts.raw_acc = *reinterpret_cast<const bool*>(value);
      return ODLA_SUCCESS;
    default:
      OHIP_DEBUG("odla_SetComputationItem: item %d accepted and ignored", (int)type);
      return ODLA_SUCCESS;
  }
}

// ---------------------------------------------------------------- context --
odla_status odla_CreateContext(odla_context* context) {
  if (context == nullptr) return ODLA_INVALID_PARAM;
  _odla_computation* c = current_computation();
  if (c == nullptr) {
    OHIP_ERR("odla_CreateContext: no computation exists");
    return ODLA_FAILURE;
  }
  odla_status st = create_context_for(c, context);
  if (st == ODLA_SUCCESS) {
    std::lock_guard<std::mutex> lk(c->mu);
    ++c->live_contexts;
  }
  return st;
}

}  // extern "C"
namespace {
odla_status create_context_for(_odla_computation* c, odla_context* context) {
  odla_status st = ensure_plan(c);
  if (st != ODLA_SUCCESS) return st;
  auto ctx = std::make_unique<_odla_context>();
  ctx->comp = c;
  if (hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking) != hipSuccess) {
    OHIP_ERR("odla_CreateContext: cannot create a HIP stream");
    return ODLA_FAILURE;
  }
  ctx->arena_bytes = c->plan->arena_bytes;
  if (ctx->arena_bytes > 0) {
    hipError_t e = hipMalloc(reinterpret_cast<void**>(&ctx->arena), ctx->arena_bytes);
    if (e != hipSuccess) {
      OHIP_ERR("odla_CreateContext: cannot allocate a %zu-byte device arena: %s", ctx->arena_bytes, hipGetErrorString(e));
      (void)hipStreamDestroy(ctx->stream);
      return ODLA_MEM_ERROR;
    }
  }
  // set-up for odla_hip_ExecuteComputationStatic: resolve this device's copy of the static
  // scratch now, so that the entry point itself only reads the cached address
  {
    void* base = nullptr;
    if (static_arena(&base, nullptr) != hipSuccess) OHIP_WARN("odla_CreateContext: the static scratch could not be resolved");
  }
  *context = ctx.release();
  return ODLA_SUCCESS;
}
}  // namespace
extern "C" {

static void destroy_context(odla_context ctx) { destroy_context_tree(ctx); }

odla_status odla_DestroyContext(odla_context ctx) {
  if (ctx == nullptr) return ODLA_INVALID_PARAM;
  if (ctx->comp != nullptr && is_live(ctx->comp)) {
    std::lock_guard<std::mutex> lk(ctx->comp->mu);
    if (ctx->comp->live_contexts > 0) --ctx->comp->live_contexts;
  }
  destroy_context(ctx);
  return ODLA_SUCCESS;
}

odla_status odla_SetContextItem(odla_context ctx, odla_item_type type, odla_item_value value) {
  if (ctx == nullptr) return ODLA_INVALID_PARAM;
  if (type == ODLA_AGGREGATE_OPS) {
    if (value == nullptr) return ODLA_INVALID_PARAM;
    ctx->use_graph = *reinterpret_cast<const bool*>(value);
    if (!ctx->use_graph) drop_graph(ctx);
    return ODLA_SUCCESS;
  }
  if (type == ODLA_RUN_BATCH_SIZE) {
    if (value == nullptr) return ODLA_INVALID_PARAM;
    return set_run_batch(ctx, *reinterpret_cast<const int*>(value));
  }
  OHIP_DEBUG("odla_SetContextItem: item %d accepted and ignored", (int)type);
  return ODLA_SUCCESS;
}

odla_status odla_SetRuntimeShape(odla_context ctx, odla_value value, odla_value_shape shape) {
  if (ctx == nullptr || value == nullptr) return ODLA_INVALID_PARAM;
  // only arguments, as in the reference [ref: odla_tensorrt.cc:251-258]
  if (value->kind != _odla_value::ARG || value->comp != ctx->comp) return ODLA_FAILURE;
  const Shape want = shape_from(shape);
  if (want.rank != value->shape.rank || want.d[0] < 1) return ODLA_INVALID_PARAM;
  for (int i = 1; i < want.rank; ++i) {
    if (want.d[i] != value->shape.d[i]) {
      OHIP_ERR("odla_SetRuntimeShape: only the leading extent of '%s' %s may change at run time (asked for %s)",
               value->name.c_str(), value->shape.str().c_str(), want.str().c_str());
      return ODLA_UNSUPPORTED_OP;
    }
  }
  const int rec = recorded_batch(*ctx->comp);
  if (rec == 0 || value->shape.d[0] != rec) {
    if (want.d[0] == value->shape.d[0]) return ODLA_SUCCESS;
    OHIP_ERR("odla_SetRuntimeShape: '%s' was not recorded with a dynamic batch", value->name.c_str());
    return ODLA_UNSUPPORTED_OP;
  }
  return set_run_batch(ctx, (int)want.d[0]);
}

odla_status odla_SetRuntimeValueType(odla_context ctx, odla_value value, odla_value_type type) {
  if (value != nullptr && type.element_type != value->etype) return ODLA_UNSUPPORTED_DATATYPE;
  return odla_SetRuntimeShape(ctx, value, type.shape);
}

odla_status odla_GetRuntimeValueType(odla_context ctx, odla_value value, odla_value_type* type) {
  if (value == nullptr || type == nullptr) return ODLA_INVALID_PARAM;
  type->element_type = value->etype;
  return odla_GetRuntimeShape(ctx, value, &type->shape);
}

odla_status odla_BindToArgument(odla_value value, const odla_void* data_ptr, odla_context ctx) {
  if (value == nullptr || data_ptr == nullptr || ctx == nullptr) return ODLA_INVALID_PARAM;
  if (value->kind != _odla_value::ARG || value->comp != ctx->comp) {
    OHIP_ERR("odla_BindToArgument: '%s' is not an argument of this computation", value->name.c_str());
    return ODLA_INVALID_PARAM;
  }
  ctx->bound_in[value] = data_ptr;
  return ODLA_SUCCESS;
}

odla_status odla_BindToArgumentById(const odla_value_id id, const odla_void* data_ptr, odla_context ctx) {
  if (ctx == nullptr || id == nullptr) return ODLA_INVALID_PARAM;
  _odla_value* v = find_value(ctx->comp, id);
  if (v == nullptr) {
    OHIP_ERR("odla_BindToArgumentById: unknown value id '%s'", reinterpret_cast<const char*>(id));
    return ODLA_INVALID_PARAM;
  }
  return odla_BindToArgument(v, data_ptr, ctx);
}

odla_status odla_BindToOutput(odla_value value, odla_void* data_ptr, odla_context ctx) {
  if (value == nullptr || data_ptr == nullptr || ctx == nullptr) return ODLA_INVALID_PARAM;
  if (!value->is_output || value->comp != ctx->comp) {
    OHIP_ERR("odla_BindToOutput: '%s' is not an output of this computation", value->name.c_str());
    return ODLA_INVALID_PARAM;
  }
  ctx->bound_out[value] = data_ptr;
  return ODLA_SUCCESS;
}

odla_status odla_BindToOutputById(const odla_value_id id, odla_void* data_ptr, odla_context ctx) {
  if (ctx == nullptr || id == nullptr) return ODLA_INVALID_PARAM;
  _odla_value* v = find_value(ctx->comp, id);
  if (v == nullptr) {
    OHIP_ERR("odla_BindToOutputById: unknown value id '%s'", reinterpret_cast<const char*>(id));
    return ODLA_INVALID_PARAM;
  }
  return odla_BindToOutput(v, data_ptr, ctx);
}

namespace {

// Launch sequences shorter than this run uncaptured: replaying a hipGraph costs a fixed amount
// per execution that a few direct launches stay below.  Measured on chains of 1 .. 24 small
// launches (device-resident buffers, one execution after the other): replay 34.5 us for one
// launch, 35.8 for five, 37.2 for six, 65.9 for 24; direct launches 17.8, 27.0, 45.0 (the
// runtime hands over more than five queued launches differently), 92.4.
// ODLA_HIP_GRAPH_MIN_STEPS overrides (read per execution: tests of the capture path set it to 1).
size_t min_graph_steps() {
  const char* e = getenv("ODLA_HIP_GRAPH_MIN_STEPS");
  const long n = e ? atol(e) : 0;
  return (size_t)(n > 0 ? n : 6);
}

odla_status execute_impl(odla_context ctx, odla_compute_mode mode, odla_device device, bool wait, bool whole = false);

// Leading extent shared by every argument of `c` (the batch, as in the reference's runtimes), 0 if
// there is none.
int64_t common_batch(const _odla_computation& c) {
  int64_t b = 0;
  for (const _odla_value* a : c.args) {
    if (a->shape.rank < 1 || a->eager) return 0;
    if (b != 0 && a->shape.d[0] != b) return 0;
    b = a->shape.d[0];
  }
  return b;
}

// An execution as two half-batch copies side by side.  A network's launches alternate between
// bandwidth-bound and MFMA-bound ones and each runs as few rounds of workgroups with a serial head
// and tail; two half-batch replicas on two streams fill each other's gaps.  Whether that beats
// the smaller, less efficient launches of a half batch depends on the work per image.  Measured
// on one box, whole batch against two halves: ResNet-50 int8 at batch 512 / 256 / 128 / 32: +4.2 /
// +3.8 / +1.6 / -4.2 %; fp16 at 256 / 128 / 64 / 8: +5.9 / +3.9 / +6.5 / -7.3 %; BERT-base bf16 at
// 64 / 16 sequences: +8.7 / -8.6 %; YOLOv3 fp16 at 16 images of 416 x 416: +8.8 %.  So a context
// measures (see _odla_context::Split) unless ODLA_HIP_BATCH_SPLIT decides: 0 = never, n > 0 =
// always from batch n on.  Plans of fewer than 16 launches and batches below 8 are not tried
// (two graph launches and two waits cost ~10 us).
// Returns the threshold (0: never) and whether it came from the environment.
int64_t split_threshold(bool* forced) {
  const char* e = getenv("ODLA_HIP_BATCH_SPLIT");   // (read per execution: a test switches it)
  *forced = e != nullptr && e[0] != 0;
  if (!*forced) return (int64_t)kMinTrialBatch;
  return (int64_t)atoll(e);
}

// Executes `ctx` as two half-batch contexts.  *handled = false: not applicable (odd or small batch,
// an unbound argument or result, a graph that does not follow the batch) - the caller runs as usual.
odla_status execute_split(_odla_context* ctx, odla_compute_mode mode, odla_device device, bool* handled) {
  *handled = false;
  _odla_computation* c = ctx->comp;
  _odla_context::Split& sp = ctx->split;
  if (sp.tried && !sp.ok) return ODLA_SUCCESS;
  if (!c->plan) return ODLA_SUCCESS;
  const Plan& plan = *c->plan;
  // results are fetched from the halves' arenas only through bound buffers
  for (const Plan::IO& io : plan.inputs)
    if (ctx->bound_in.find(io.v) == ctx->bound_in.end()) return ODLA_SUCCESS;
  for (const Plan::IO& io : plan.outputs)
    if (ctx->bound_out.find(io.v) == ctx->bound_out.end()) return ODLA_SUCCESS;
  if (!plan.stat_recs.empty()) return ODLA_SUCCESS;   // (value statistics are collected on the whole batch)
  // A result buffer that overlaps an argument buffer: one half could write (in place) what the
  // other still reads.  The whole batch has its own guard for that case.
  for (const Plan::IO& in : plan.inputs) {
    const char* a0 = static_cast<const char*>(ctx->bound_in[in.v]);
    for (const Plan::IO& out : plan.outputs) {
      const char* b0 = static_cast<const char*>(ctx->bound_out[out.v]);
      if (a0 < b0 + out.bytes && b0 < a0 + in.bytes) return ODLA_SUCCESS;
    }
  }
  if (!sp.tried) {
    sp.tried = true;
    const int64_t B = common_batch(*c);
    if (B < 2 || B % 2 != 0) return ODLA_SUCCESS;
    std::shared_ptr<_odla_computation> v;
    {
      std::lock_guard<std::mutex> lk(c->mu);
      // (kept under the negative batch: a copy made for a smaller dynamic batch was not checked
      //  for keeping the images' rows apart)
      const int key = -(int)(B / 2);
      auto it = c->variants.find(key);
      if (it != c->variants.end()) v = it->second.lock();
      if (!v) {
        std::unique_ptr<_odla_computation> copy = clone_for_batch(*c, B, B / 2, /*rows_apart=*/true);
        if (!copy) return ODLA_SUCCESS;
        v = std::move(copy);
        c->variants[key] = v;
      }
    }
    for (int k = 0; k < 2; ++k) {
      odla_context sub = nullptr;
      if (create_context_for(v.get(), &sub) != ODLA_SUCCESS) {
        for (_odla_context*& h : sp.half) { if (h) destroy_context_tree(h); h = nullptr; }
        return ODLA_SUCCESS;
      }
      sub->is_half = true;
      sub->defer_fetch = true;
      sub->image_base = ctx->image_base + k * (int)(B / 2);
      sp.half[k] = sub;
    }
    if (hipEventCreateWithFlags(&sp.half[0]->inputs_staged, hipEventDisableTiming) == hipSuccess)
      sp.half[1]->wait_inputs = sp.half[0]->inputs_staged;
    else
      sp.half[0]->inputs_staged = nullptr;
    sp.comp = std::move(v);
    sp.ok = true;
    OHIP_DEBUG("odla_ExecuteComputation: two half-batch copies of batch %lld planned", (long long)B);
  }
  *handled = true;
  const Plan& hp = *sp.comp->plan;
  for (int k = 0; k < 2; ++k) {
    _odla_context* sub = sp.half[k];
    if (sub->use_graph != ctx->use_graph) {
      sub->use_graph = ctx->use_graph;
      if (!sub->use_graph) drop_graph(sub);
    }
    sub->bound_in.clear();
    sub->bound_out.clear();
    // a value whose leading extent was halved takes its half of the caller's buffer
    auto offset = [&](const _odla_value* whole, const Plan::IO& io) -> size_t {
      return io.v->shape.rank >= 1 && io.v->shape.d[0] * 2 == whole->shape.d[0] ? (size_t)k * io.bytes : 0;
    };
    for (size_t i = 0; i < plan.inputs.size(); ++i) {
      const _odla_value* whole = plan.inputs[i].v;
      const Plan::IO* io = nullptr;
      for (const Plan::IO& cand : hp.inputs)
        if (cand.v->index == whole->index) io = &cand;
      if (io == nullptr) continue;
      sub->bound_in[io->v] = static_cast<const char*>(ctx->bound_in[whole]) + offset(whole, *io);
    }
    for (size_t i = 0; i < plan.outputs.size(); ++i) {
      const _odla_value* whole = plan.outputs[i].v;
      const Plan::IO* io = nullptr;
      for (const Plan::IO& cand : hp.outputs)
        if (cand.v->index == whole->index) io = &cand;
      if (io == nullptr) continue;
      sub->bound_out[io->v] = static_cast<char*>(ctx->bound_out[whole]) + offset(whole, *io);
    }
  }
  odla_status st = ODLA_SUCCESS;
  for (int k = 0; k < 2 && st == ODLA_SUCCESS; ++k) st = execute_impl(sp.half[k], mode, device, /*wait=*/false);
  // both halves are queued: now their results' copies
  for (int k = 0; k < 2 && st == ODLA_SUCCESS; ++k)
    st = fetch_outputs(sp.half[k], hp, sp.half[k]->arena, &sp.half[k]->last_ext, /*wait=*/false);
  for (int k = 0; k < 2; ++k) {
    const hipError_t e = hipStreamSynchronize(sp.half[k]->stream);
    if (e != hipSuccess) {
      OHIP_ERR("device error: %s", hipGetErrorString(e));
      st = ODLA_FAILURE;
    }
  }
  ctx->executed = st == ODLA_SUCCESS;
  ctx->last_split = ctx->executed;
  return st;
}

}  // namespace

odla_status odla_ExecuteComputation(const odla_computation comp, const odla_context ctx,
                                    const odla_compute_mode mode, odla_device device) {
  if (ctx == nullptr) return ODLA_INVALID_PARAM;
  if (comp != nullptr && comp != ctx->comp) {
    OHIP_ERR("odla_ExecuteComputation: context belongs to another computation");
    return ODLA_INVALID_PARAM;
  }
  return execute_impl(ctx, mode, device, /*wait=*/true);
}

namespace {

// whole: run the batch as it is (no half-batch copies, no measuring)
odla_status execute_impl(const odla_context ctx, const odla_compute_mode mode, odla_device device, const bool wait, const bool whole) {
  (void)device;
  if (mode == ODLA_COMPUTE_TRAINING) return ODLA_UNSUPPORTED_OP;
  _odla_computation* c = ctx->comp;
  if (!whole && !ctx->is_half && (ctx->run_batch == 0 || ctx->run_batch == recorded_batch(*c))) {
    bool forced = false;
    const int64_t from = split_threshold(&forced);
    const int64_t B = from > 0 ? common_batch(*c) : 0;
    _odla_context::Split& sp = ctx->split;
    if (from > 0 && B >= from && forced) {
      // the environment decides: halves wherever they apply
      bool handled = false;
      const odla_status st = execute_split(ctx, mode, device, &handled);
      if (handled) {
        if (sp.choice != 2) OHIP_INFO("odla_ExecuteComputation: batch %lld runs as two halves side by side", (long long)B);
        sp.choice = 2;
        return st;
      }
    } else if (from > 0 && B >= from && c->plan && c->plan->steps.size() >= 16 && sp.choice != 1) {
      if (sp.choice == 2) {
        bool handled = false;
        const odla_status st = execute_split(ctx, mode, device, &handled);
        if (handled) return st;
      } else if (wait) {
        // measuring: six executions whole, then ten in halves, the fastest of the last three
        // (whole) and four (halves) counts.  A fresh context needs some five replays to reach its
        // steady time - clocks, caches, the graphs' first launches - and the halves, coming
        // second with two fresh graphs, more: over 40 runs of the ResNet-50 plans their figure
        // here read 3 - 10 % above what the same halves reached afterwards, the whole batch's
        // about right.  Halves are therefore kept as soon as they are not slower.
        constexpr int kWhole = 6, kHalves = 10, kCount = 3, kCountHalves = 4;
        const int t = sp.trial;
        const auto t0 = std::chrono::steady_clock::now();
        odla_status st = ODLA_SUCCESS;
        bool handled = true;
        if (t < kWhole) {
          st = execute_impl(ctx, mode, device, wait, /*whole=*/true);
        } else {
          st = execute_split(ctx, mode, device, &handled);
        }
        if (!handled) {
          sp.choice = 1;   // does not apply to this graph or these bindings: whole from now on
        } else {
          const double ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
          if (st != ODLA_SUCCESS) return st;
          if (t >= kWhole - kCount && t < kWhole && (t == kWhole - kCount || ms < sp.whole_ms)) sp.whole_ms = ms;
          if (t >= kWhole + kHalves - kCountHalves && (t == kWhole + kHalves - kCountHalves || ms < sp.halves_ms)) sp.halves_ms = ms;
          sp.trial = t + 1;
          if (sp.trial == kWhole + kHalves) {
            sp.choice = sp.halves_ms < sp.whole_ms ? 2 : 1;
            if (sp.choice == 2)
              OHIP_INFO("odla_ExecuteComputation: batch %lld runs as two halves side by side (%.3f ms against %.3f ms whole)",
                        (long long)B, sp.halves_ms, sp.whole_ms);
            else
              OHIP_INFO("odla_ExecuteComputation: batch %lld stays whole (%.3f ms against %.3f ms in two halves)",
                        (long long)B, sp.whole_ms, sp.halves_ms);
            if (sp.choice == 1) {   // the halves' arenas, streams and graphs are not needed again
              for (_odla_context*& h : sp.half) { if (h) destroy_context_tree(h); h = nullptr; }
              sp.comp.reset();
              sp.ok = false;
            }
          }
          return st;
        }
      }
    }
  }
  if (ctx->run_batch > 0 && ctx->run_batch != recorded_batch(*c)) {
    // another batch than the recorded one: the same bindings, on the copy planned for that batch
    _odla_context* sub = nullptr;
    odla_status st = variant_context(ctx, ctx->run_batch, &sub);
    if (st != ODLA_SUCCESS) return st;
    if (sub->use_graph != ctx->use_graph) {
      sub->use_graph = ctx->use_graph;
      if (!sub->use_graph) drop_graph(sub);
    }
    sub->bound_in.clear();
    sub->bound_out.clear();
    for (const auto& kv : ctx->bound_in) sub->bound_in[sub->comp->values[kv.first->index].get()] = kv.second;
    for (const auto& kv : ctx->bound_out) sub->bound_out[sub->comp->values[kv.first->index].get()] = kv.second;
    st = execute_impl(sub, mode, device, wait);
    ctx->executed = st == ODLA_SUCCESS;
    return st;
  }
  if (!c->plan) return ODLA_FAILURE;
  const Plan& plan = *c->plan;

  // 1. stage arguments (host -> device across PCIe, or device -> device; device buffers
  //    that the first steps can read where they are stay there)
  std::vector<const char*> ext;
  {
    if (ctx->wait_inputs != nullptr) (void)hipStreamWaitEvent(ctx->stream, ctx->wait_inputs, 0);
    odla_status st = stage_inputs(ctx, plan, ctx->arena, &ext);
    if (st != ODLA_SUCCESS) return st;
    if (ctx->inputs_staged != nullptr) (void)hipEventRecord(ctx->inputs_staged, ctx->stream);
    place_outputs(ctx, plan, &ext);
  }

  // 2. launch sequence: captured once into a hipGraph, replayed afterwards
  if (ctx->use_graph && plan.steps.size() >= min_graph_steps()) {
    select_graph(ctx, ext);
    // A caller that brings new buffers every time would capture every time: after a few
    // captures in a row this context goes back to staging copies and one graph.
    constexpr int kCaptureStreakLimit = 8;
    if (ctx->graph_exec != nullptr) {
      ctx->capture_streak = 0;
    } else if (++ctx->capture_streak > kCaptureStreakLimit && !ctx->in_place_off) {
      bool any = false;
      for (const char* p : ext) any = any || p != nullptr;
      if (any) {
        OHIP_INFO("odla_ExecuteComputation: %d executions in a row with new device buffers; arguments and results are copied from now on", ctx->capture_streak);
        ctx->in_place_off = true;
        drop_graph(ctx);
        odla_status st2 = stage_inputs(ctx, plan, ctx->arena, &ext);
        if (st2 != ODLA_SUCCESS) return st2;
      }
    }
    if (ctx->graph_exec == nullptr) {
      if (hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal) != hipSuccess) {
        OHIP_ERR("odla_ExecuteComputation: hipStreamBeginCapture failed");
        return ODLA_FAILURE;
      }
      odla_status st = run_steps(ctx, plan, ctx->arena, &ext);
      hipGraph_t g = nullptr;
      hipError_t e = hipStreamEndCapture(ctx->stream, &g);
      if (st != ODLA_SUCCESS || e != hipSuccess || g == nullptr) {
        if (g) (void)hipGraphDestroy(g);
        OHIP_ERR("odla_ExecuteComputation: graph capture failed");
        return ODLA_FAILURE;
      }
      ctx->graph = g;
      ctx->graph_ext = ext;
      if (hipGraphInstantiate(&ctx->graph_exec, g, nullptr, nullptr, 0) != hipSuccess) {
        drop_graph(ctx);
        OHIP_ERR("odla_ExecuteComputation: hipGraphInstantiate failed");
        return ODLA_FAILURE;
      }
    }
    if (hipGraphLaunch(ctx->graph_exec, ctx->stream) != hipSuccess) {
      OHIP_ERR("odla_ExecuteComputation: hipGraphLaunch failed");
      return ODLA_FAILURE;
    }
  } else {
    if (ctx->use_graph && !plan.steps.empty() && !ctx->said_uncaptured) {
      ctx->said_uncaptured = true;
      OHIP_INFO("odla_ExecuteComputation: %zu launches per execution run uncaptured (a graph replay costs more than that few)", plan.steps.size());
    }
    odla_status st = run_steps(ctx, plan, ctx->arena, &ext);
    if (st != ODLA_SUCCESS) return st;
  }

  // 3. results
  if (ctx->defer_fetch) {   // (a half: its parent fetches, see execute_split)
    ctx->last_ext = ext;
    ctx->executed = true;
    ctx->last_split = false;
    return ODLA_SUCCESS;
  }
  odla_status st = fetch_outputs(ctx, plan, ctx->arena, &ext, wait);
  if (st != ODLA_SUCCESS) return st;
  ctx->last_ext = ext;
  ctx->executed = true;
  ctx->last_split = false;
  if (!plan.stat_recs.empty()) return profiler_collect(plan, ctx->arena);
  return ODLA_SUCCESS;
}

}  // namespace

static_assert(kStaticArenaBytes == ODLA_HIP_STATIC_SCRATCH_BYTES, "the header states the size of the static scratch");

// odla_ExecuteComputation for callers that must not allocate device memory.
// The plan's temporaries live in the library's static device scratch instead
// of the context's arena, and the launch sequence runs un-captured (building a
// hipGraph allocates), so the call performs no hipMalloc / hipFree.  The
// context supplies the stream and the bindings; its own arena is not touched.
odla_status odla_hip_ExecuteComputationStatic(odla_computation comp, odla_context ctx,
                                              const odla_compute_mode mode, odla_device device) {
  (void)device;
  if (ctx == nullptr) return ODLA_INVALID_PARAM;
  if (comp != nullptr && comp != ctx->comp) {
    OHIP_ERR("odla_hip_ExecuteComputationStatic: context belongs to another computation");
    return ODLA_INVALID_PARAM;
  }
  if (mode == ODLA_COMPUTE_TRAINING) return ODLA_UNSUPPORTED_OP;
  _odla_computation* c = ctx->comp;
  if (ctx->run_batch > 0 && ctx->run_batch != recorded_batch(*c)) {
    // another batch runs a copy of the recording that is planned on first use: that allocates
    OHIP_ERR("odla_hip_ExecuteComputationStatic: runs the recorded batch only (context is set to batch %d)", ctx->run_batch);
    return ODLA_UNSUPPORTED_OP;
  }
  if (!c->plan) return ODLA_FAILURE;
  const Plan& plan = *c->plan;
  if (!plan.stat_recs.empty()) {
    OHIP_ERR("odla_hip_ExecuteComputationStatic: calibration plans are not supported");
    return ODLA_UNSUPPORTED_OP;
  }
  void* base = nullptr;
  size_t cap = 0;
  hipError_t e = static_arena(&base, &cap);
  if (e != hipSuccess) {
    OHIP_ERR("odla_hip_ExecuteComputationStatic: static scratch unavailable: %s", hipGetErrorString(e));
    return ODLA_FAILURE;
  }
  if (plan.arena_bytes > cap) {
    OHIP_ERR("odla_hip_ExecuteComputationStatic: the plan needs %zu bytes of temporaries, the static scratch holds %zu; "
             "use odla_ExecuteComputation", plan.arena_bytes, cap);
    return ODLA_MEM_ERROR;
  }
  char* arena = static_cast<char*>(base);
  odla_status st = stage_inputs(ctx, plan, arena);
  if (st != ODLA_SUCCESS) return st;
  st = run_steps(ctx, plan, arena);
  if (st != ODLA_SUCCESS) return st;
  return fetch_outputs(ctx, plan, arena);
}

// Diagnostic: run the launch sequence un-captured `iters` times with a HIP
// event pair around every step on the context's stream and report the mean
// duration of each step.  Arguments must be bound.
odla_status odla_hip_PlanSummary(odla_computation c, odla_hip_plan_summary* summary) {
  if (c == nullptr || summary == nullptr || !is_live(c)) return ODLA_INVALID_PARAM;
  std::lock_guard<std::mutex> lk(c->mu);
  if (c->plan && c->live_contexts > 0) {
    OHIP_ERR("odla_hip_PlanSummary: the computation is compiled and has live contexts");
    return ODLA_FAILURE;   // the fusion marks of the nodes belong to the live plan
  }
  int launches = 0, init_launches = 0;
  size_t arena = 0, consts = 0;
  profiler_configure(&c->opts);
  const odla_status st = plan_summary(c, &launches, &init_launches, &arena, &consts);
  if (st != ODLA_SUCCESS) return st;
  summary->launches = launches;
  summary->init_launches = init_launches;
  summary->arena_bytes = arena;
  summary->constant_bytes = consts;
  return ODLA_SUCCESS;
}

odla_status odla_hip_ProfileSteps(odla_context ctx, odla_int32 iters, odla_hip_step_time* out,
                                  odla_int32 capacity, odla_int32* count) {
  if (ctx == nullptr || out == nullptr || count == nullptr || iters <= 0) return ODLA_INVALID_PARAM;
  _odla_computation* c = ctx->comp;
  if (!c->plan) return ODLA_FAILURE;
  const Plan& plan = *c->plan;
  const int n = (int)plan.steps.size();
  if (n > capacity) return ODLA_INVALID_PARAM;
  std::vector<hipEvent_t> ev((size_t)n * 2);
  for (auto& e : ev)
    if (hipEventCreate(&e) != hipSuccess) return ODLA_FAILURE;
  std::vector<double> acc((size_t)n, 0.0);
  ExecEnv env;
  env.base[SP_ARENA] = ctx->arena;
  env.base[SP_CONST] = plan.const_pool;
  odla_status st = ODLA_SUCCESS;
  for (int it = 0; it < iters && st == ODLA_SUCCESS; ++it) {
    st = stage_inputs(ctx, plan, ctx->arena);
    for (int i = 0; i < n && st == ODLA_SUCCESS; ++i) {
      (void)hipEventRecord(ev[2 * i], ctx->stream);
      if (plan.steps[i].fn(env, ctx->stream) != hipSuccess) st = ODLA_FAILURE;
      (void)hipEventRecord(ev[2 * i + 1], ctx->stream);
    }
    if (hipStreamSynchronize(ctx->stream) != hipSuccess) st = ODLA_FAILURE;
    for (int i = 0; i < n && st == ODLA_SUCCESS; ++i) {
      float ms = 0.f;
      if (hipEventElapsedTime(&ms, ev[2 * i], ev[2 * i + 1]) != hipSuccess) st = ODLA_FAILURE;
      acc[i] += ms;
    }
  }
  for (auto& e : ev) (void)hipEventDestroy(e);
  if (st != ODLA_SUCCESS) return st;
  for (int i = 0; i < n; ++i) {
    snprintf(out[i].name, sizeof(out[i].name), "%s", plan.steps[i].name.c_str());
    out[i].ms = (float)(acc[i] / iters);
  }
  *count = n;
  return ODLA_SUCCESS;
}

// ----------------------------------------------------------- introspection --
odla_status odla_GetNumOfArgsFromComputation(const odla_computation c, odla_uint32* n) {
  if (c == nullptr || n == nullptr) return ODLA_INVALID_PARAM;
  *n = (odla_uint32)c->args.size();
  return ODLA_SUCCESS;
}
odla_status odla_GetArgFromComputationByIdx(const odla_computation c, const odla_uint32 idx, odla_value* v) {
  if (c == nullptr || v == nullptr) return ODLA_INVALID_PARAM;
  *v = nullptr;
  if (idx >= c->args.size()) return ODLA_INVALID_PARAM;
  *v = c->args[idx];
  return ODLA_SUCCESS;
}
odla_status odla_GetNumOfOutputsFromComputation(const odla_computation c, odla_uint32* n) {
  if (c == nullptr || n == nullptr) return ODLA_INVALID_PARAM;
  *n = (odla_uint32)c->outputs.size();
  return ODLA_SUCCESS;
}
odla_status odla_GetOutputFromComputationByIdx(const odla_computation c, const odla_uint32 idx, odla_value* v) {
  if (c == nullptr || v == nullptr) return ODLA_INVALID_PARAM;
  *v = nullptr;
  if (idx >= c->outputs.size()) return ODLA_INVALID_PARAM;
  *v = c->outputs[idx];
  return ODLA_SUCCESS;
}
odla_status odla_GetRuntimeShape(odla_context ctx, odla_value value, odla_value_shape* shape) {
  if (value == nullptr || shape == nullptr) return ODLA_INVALID_PARAM;
  *shape = shape_to(value->shape);
  if (ctx != nullptr && value->comp == ctx->comp && ctx->run_batch > 0) {
    // the value's shape at the batch this context runs at
    auto it = ctx->variant_ctx.find(ctx->run_batch);
    if (it != ctx->variant_ctx.end()) *shape = shape_to(it->second.comp->values[value->index]->shape);
  }
  return ODLA_SUCCESS;
}

odla_status odla_GetValueType(const odla_value value, odla_value_type* type) {
  if (value == nullptr || type == nullptr) return ODLA_INVALID_PARAM;
  type->element_type = value->etype;
  type->shape = shape_to(value->shape);
  return ODLA_SUCCESS;
}
odla_status odla_GetValueId(const odla_value value, odla_value_id* id) {
  if (value == nullptr || id == nullptr) return ODLA_INVALID_PARAM;
  *id = reinterpret_cast<odla_value_id>(const_cast<char*>(value->name.c_str()));
  return ODLA_SUCCESS;
}
odla_status odla_FindValueById(const odla_value_id id, odla_value* value) {
  if (id == nullptr || value == nullptr) return ODLA_INVALID_PARAM;
  *value = find_value(current_computation(), id);
  return *value ? ODLA_SUCCESS : ODLA_INVALID_PARAM;
}

odla_status odla_SetValueAsOutput(odla_value value) {
  if (value == nullptr || value->comp == nullptr) return ODLA_INVALID_PARAM;
  _odla_computation* c = value->comp;
  std::lock_guard<std::mutex> lk(c->mu);
  if (c->plan) {
    OHIP_ERR("odla_SetValueAsOutput: computation is already compiled");
    return ODLA_FAILURE;
  }
  if (!value->is_output) {
    value->is_output = true;
    c->outputs.push_back(value);
  }
  return ODLA_SUCCESS;
}
odla_status odla_SetValuesAsOutput(odla_values values) {
  if (values.size > ODLA_MAX_OUTPUTS) return ODLA_INVALID_PARAM;
  for (size_t i = 0; i < values.size; ++i) {
    odla_status st = odla_SetValueAsOutput(values.values[i]);
    if (st != ODLA_SUCCESS) return st;
  }
  return ODLA_SUCCESS;
}
odla_status odla_SetValueAsOutputById(const odla_value_id id) {
  return odla_SetValueAsOutput(find_value(current_computation(), id));
}

// Interpret mode: values made by odla_CreateValue carry their own data
// (odla_SetValueData), operators are recorded as usual, and asking for a
// value's data with no context compiles what has been recorded so far (again
// only when the graph has grown or the value was not yet a result), runs it on
// an internal context and copies the value back.
// [ref: ODLA/platforms/dnnl/odla_dnnl.cc:161-179,225-230,276-295]
static odla_status eager_evaluate(_odla_value* value, void* data_ptr) {
  _odla_computation* c = value->comp;
  if (c == nullptr || !is_live(c)) return ODLA_INVALID_PARAM;
  {
    std::lock_guard<std::mutex> lk(c->mu);
    const bool stale = !c->plan || c->planned_nodes != c->nodes.size() || !value->is_output ||
                       c->plan->calibrated != profiler_active();
    if (stale) {
      if (c->live_contexts > 0) {
        OHIP_ERR("odla_GetValueData: '%s' is not a result of the compiled computation and contexts are still alive",
                 value->name.c_str());
        return ODLA_FAILURE;
      }
      if (c->eager_ctx != nullptr) { destroy_context(c->eager_ctx); c->eager_ctx = nullptr; }
      if (!value->is_output) { value->is_output = true; c->outputs.push_back(value); }
      c->plan.reset();
      c->plan_failed = false;
      for (Node& n : c->nodes) n.absorbed = false;
    }
  }
  if (c->eager_ctx == nullptr) {
    odla_status st = create_context_for(c, &c->eager_ctx);
    if (st != ODLA_SUCCESS) return st;
    c->eager_ctx->use_graph = false;
  }
  _odla_context* ctx = c->eager_ctx;
  for (_odla_value* a : c->args) {
    if (!a->eager) continue;
    if (a->eager_data == nullptr) {
      OHIP_ERR("odla_GetValueData: value '%s' has no data (odla_SetValueData)", a->name.c_str());
      return ODLA_INVALID_PARAM;
    }
    ctx->bound_in[a] = a->eager_data;
  }
  odla_status st = odla_ExecuteComputation(c, ctx, ODLA_COMPUTE_INFERENCE, nullptr);
  if (st != ODLA_SUCCESS) return st;
  return odla_GetValueData(value, data_ptr, ctx);
}

odla_value odla_CreateValue(odla_value_type type, const odla_value_id id) {
  if (current_computation() == nullptr) {
    odla_computation c = nullptr;  // the interpreter works on an implicit computation
    if (odla_CreateComputation(&c) != ODLA_SUCCESS) return nullptr;
  }
  odla_value v = odla_CreateArgument(type, id);
  if (v != nullptr) v->eager = true;
  return v;
}

odla_status odla_SetValueData(odla_value value, const odla_void* data_ptr) {
  if (value == nullptr || data_ptr == nullptr) return ODLA_INVALID_PARAM;
  if (!value->eager) {
    OHIP_ERR("odla_SetValueData: '%s' was not made by odla_CreateValue", value->name.c_str());
    return ODLA_INVALID_PARAM;
  }
  value->eager_data = data_ptr;
  return ODLA_SUCCESS;
}

odla_status odla_SetValueDataById(const odla_value_id id, const odla_void* data_ptr) {
  return odla_SetValueData(find_value(current_computation(), id), data_ptr);
}

odla_status odla_GetValueDataById(const odla_value_id id, odla_void* data_ptr) {
  return odla_GetValueData(find_value(current_computation(), id), data_ptr, nullptr);
}

odla_status odla_GetValueData(const odla_value value, odla_void* data_ptr, odla_context ctx) {
  if (value == nullptr || data_ptr == nullptr) return ODLA_INVALID_PARAM;
  if (ctx == nullptr) return eager_evaluate(value, data_ptr);
  if (ctx->run_batch > 0 && value->comp == ctx->comp) {
    auto it = ctx->variant_ctx.find(ctx->run_batch);
    if (it != ctx->variant_ctx.end())
      return odla_GetValueData(it->second.comp->values[value->index].get(), data_ptr, it->second.ctx);
  }
  if (!ctx->executed || !ctx->comp->plan) return ODLA_FAILURE;
  if (ctx->last_split && value->comp == ctx->comp && ctx->split.ok) {
    // the last execution ran as two halves: each holds its rows of the result
    const Plan& hp = *ctx->split.comp->plan;
    for (int k = 0; k < 2; ++k) {
      _odla_value* hv = ctx->split.comp->values[value->index].get();
      size_t off = 0;
      for (const Plan::IO& io : hp.outputs)
        if (io.v == hv && hv->shape.rank >= 1 && hv->shape.d[0] * 2 == value->shape.d[0]) off = (size_t)k * io.bytes;
      const odla_status st = odla_GetValueData(hv, static_cast<char*>(data_ptr) + off, ctx->split.half[k]);
      if (st != ODLA_SUCCESS) return st;
    }
    return ODLA_SUCCESS;
  }
  const Plan& plan = *ctx->comp->plan;
  for (size_t k = 0; k < plan.outputs.size(); ++k) {
    const Plan::IO& io = plan.outputs[k];
    if (io.v != value) continue;
    const PTensor& t = plan.tensors[io.tensor];
    const char* src = (t.space == SP_CONST ? plan.const_pool : ctx->arena) + t.offset + io.offset;
    const size_t slot = plan.inputs.size() + k;
    if (slot < ctx->last_ext.size() && ctx->last_ext[slot] != nullptr) src = ctx->last_ext[slot];   // written in place
    if (hipMemcpy(data_ptr, src, io.bytes, hipMemcpyDefault) != hipSuccess) return ODLA_FAILURE;
    return ODLA_SUCCESS;
  }
  OHIP_ERR("odla_GetValueData: '%s' is not an output; only outputs stay resident after execution", value->name.c_str());
  return ODLA_INVALID_PARAM;
}
odla_status odla_ReleaseValue(odla_value value) { return value ? ODLA_SUCCESS : ODLA_INVALID_PARAM; }

odla_value odla_CreateArgument(const odla_value_type type, const odla_value_id id) {
  _odla_computation* c = current_computation();
  if (c == nullptr) { OHIP_ERR("odla_CreateArgument: no current computation"); return nullptr; }
  if (dtype_from_odla(type.element_type) == DT_INVALID) {
    OHIP_ERR("odla_CreateArgument: unsupported element type %d", (int)type.element_type);
    return nullptr;
  }
  if (type.shape.size > ODLA_MAX_DIMENSION) { OHIP_ERR("odla_CreateArgument: rank too large"); return nullptr; }
  Shape s = shape_from(type.shape);
  bool dyn = false;
  if (s.d[0] < 0) {
    // the batch of a computation recorded with ODLA_DYNAMIC_BATCH: planned at the largest batch
    if (recorded_batch(*c) == 0) {
      OHIP_ERR("odla_CreateArgument: a negative leading extent needs ODLA_DYNAMIC_BATCH and ODLA_MAX_BATCH_SIZE set before");
      return nullptr;
    }
    s.d[0] = recorded_batch(*c);
    dyn = true;
  }
  for (int i = 0; i < s.rank; ++i)
    if (s.d[i] <= 0) { OHIP_ERR("odla_CreateArgument: only the leading extent may be dynamic (%s)", s.str().c_str()); return nullptr; }
  std::lock_guard<std::mutex> lk(c->mu);
  _odla_value* v = new_value(c, _odla_value::ARG, type.element_type, s, id);
  v->dyn_batch = dyn;
  c->args.push_back(v);
  return v;
}

odla_value odla_CreateConstant(const odla_value_type type, const odla_void* data_ptr, const odla_value_id id) {
  _odla_computation* c = current_computation();
  if (c == nullptr) { OHIP_ERR("odla_CreateConstant: no current computation"); return nullptr; }
  if (data_ptr == nullptr) { OHIP_ERR("odla_CreateConstant: null data"); return nullptr; }
  if (dtype_from_odla(type.element_type) == DT_INVALID) {
    OHIP_ERR("odla_CreateConstant: unsupported element type %d", (int)type.element_type);
    return nullptr;
  }
  if (type.shape.size > ODLA_MAX_DIMENSION) { OHIP_ERR("odla_CreateConstant: rank too large"); return nullptr; }
  Shape s = shape_from(type.shape);
  for (int i = 0; i < s.rank; ++i)
    if (s.d[i] <= 0) { OHIP_ERR("odla_CreateConstant: bad shape %s", s.str().c_str()); return nullptr; }
  std::lock_guard<std::mutex> lk(c->mu);
  _odla_value* v = new_value(c, _odla_value::CONSTANT, type.element_type, s, id);
  v->host_data = data_ptr;
  return v;
}

// ------------------------------------------------------------------ device --
odla_status odla_AllocateDevice(odla_vendor vendor, odla_device_name name, odla_int32 idx, odla_device* device) {
  (void)vendor;
  if (device == nullptr) return ODLA_INVALID_PARAM;
  *device = nullptr;
  if (name != ODLA_DEVICE_DEFAULT) return ODLA_UNSUPPORTED_DEVICE_TYPE;
  int count = 0;
  if (hipGetDeviceCount(&count) != hipSuccess || count <= 0) return ODLA_FAILURE;
  if (idx < 0 || idx >= count) return ODLA_INVALID_PARAM;
  auto* d = new (std::nothrow) _odla_device();
  if (d == nullptr) return ODLA_MEM_ERROR;
  d->index = idx;
  *device = d;
  return ODLA_SUCCESS;
}

odla_status odla_GetDeviceInfo(odla_device device, odla_device_info info, odla_scalar_value* out) {
  if (device == nullptr || out == nullptr) return ODLA_INVALID_PARAM;
  static thread_local char text[256];
  hipDeviceProp_t prop;
  switch (info) {
    case ODLA_DEVICE_INFO_ODLA_LIB_VERSION:
      out->data_type = ODLA_STRING; out->val_str = kVersion; return ODLA_SUCCESS;
    case ODLA_DEVICE_INFO_DEV_COUNT: {
      int n = 0;
      if (hipGetDeviceCount(&n) != hipSuccess) return ODLA_FAILURE;
      out->data_type = ODLA_INT32; out->val_int32 = n; return ODLA_SUCCESS;
    }
    case ODLA_DEVICE_INFO_DEV_INDEX:
      out->data_type = ODLA_INT32; out->val_int32 = device->index; return ODLA_SUCCESS;
    case ODLA_DEVICE_INFO_DEV_TYPE:
      if (hipGetDeviceProperties(&prop, device->index) != hipSuccess) return ODLA_FAILURE;
      snprintf(text, sizeof(text), "%s (%s)", prop.name, prop.gcnArchName);
      out->data_type = ODLA_STRING; out->val_str = text; return ODLA_SUCCESS;
    case ODLA_DEVICE_INFO_DEV_UUID: {
      hipUUID uuid;
      if (hipDeviceGetUuid(&uuid, device->index) != hipSuccess) return ODLA_FAILURE;
      memcpy(text, uuid.bytes, 16); text[16] = 0;
      out->data_type = ODLA_STRING; out->val_str = text; return ODLA_SUCCESS;
    }
    case ODLA_DEVICE_INFO_TOTAL_MEMORY:
    case ODLA_DEVICE_INFO_USED_MEMORY:
    case ODLA_DEVICE_INFO_MEMORY_UTIL: {
      size_t free_b = 0, total_b = 0;
      int prev = 0;
      (void)hipGetDevice(&prev);
      if (hipSetDevice(device->index) != hipSuccess) return ODLA_FAILURE;
      hipError_t e = hipMemGetInfo(&free_b, &total_b);
      (void)hipSetDevice(prev);
      if (e != hipSuccess) return ODLA_FAILURE;
      if (info == ODLA_DEVICE_INFO_TOTAL_MEMORY) { out->data_type = ODLA_INT64; out->val_int64 = (odla_int64)total_b; }
      else if (info == ODLA_DEVICE_INFO_USED_MEMORY) { out->data_type = ODLA_INT64; out->val_int64 = (odla_int64)(total_b - free_b); }
      else { out->data_type = ODLA_FLOAT32; out->val_fp32 = total_b ? (float)(total_b - free_b) / (float)total_b : 0.f; }
      return ODLA_SUCCESS;
    }
    // Utilisation and power need the SMI library; a neutral value is reported
    // so that generic monitors keep working.
    case ODLA_DEVICE_INFO_PROCESSOR_UTIL:
    case ODLA_DEVICE_INFO_POWER_USAGE:
    case ODLA_DEVICE_INFO_POWER_LIMIT:
      out->data_type = ODLA_FLOAT32; out->val_fp32 = 0.f; return ODLA_SUCCESS;
    case ODLA_DEVICE_INFO_DRIVER_VERSION: {
      int v = 0;
      if (hipDriverGetVersion(&v) != hipSuccess) return ODLA_FAILURE;
      snprintf(text, sizeof(text), "%d", v);
      out->data_type = ODLA_STRING; out->val_str = text; return ODLA_SUCCESS;
    }
    case ODLA_DEVICE_INFO_SDK_VERSION: {
      int v = 0;
      if (hipRuntimeGetVersion(&v) != hipSuccess) return ODLA_FAILURE;
      snprintf(text, sizeof(text), "HIP %d", v);
      out->data_type = ODLA_STRING; out->val_str = text; return ODLA_SUCCESS;
    }
  }
  return ODLA_INVALID_PARAM;
}

odla_status odla_SetCurrentDevice(odla_device device) {
  if (device == nullptr) return ODLA_INVALID_PARAM;
  return hipSetDevice(device->index) == hipSuccess ? ODLA_SUCCESS : ODLA_FAILURE;
}
odla_status odla_DestroyDevice(odla_device device) {
  if (device == nullptr) return ODLA_INVALID_PARAM;
  delete device;
  return ODLA_SUCCESS;
}

// ------------------------------------------------------------------ memory --
odla_status odla_AllocateDeviceMemory(odla_void** dev_ptr, odla_size_t size) {
  if (dev_ptr == nullptr || size == 0) return ODLA_INVALID_PARAM;
  return hipMalloc(dev_ptr, size) == hipSuccess ? ODLA_SUCCESS : ODLA_MEM_ERROR;
}
odla_status odla_FreeDeviceMemory(odla_void* ptr) {
  return hipFree(ptr) == hipSuccess ? ODLA_SUCCESS : ODLA_MEM_ERROR;
}
odla_status odla_AllocateHostMemory(odla_void** host_ptr, odla_size_t size) {
  if (host_ptr == nullptr || size == 0) return ODLA_INVALID_PARAM;
  return hipHostMalloc(host_ptr, size, hipHostMallocDefault) == hipSuccess ? ODLA_SUCCESS : ODLA_MEM_ERROR;
}
odla_status odla_FreeHostMemory(odla_void* ptr) {
  return hipHostFree(ptr) == hipSuccess ? ODLA_SUCCESS : ODLA_MEM_ERROR;
}
odla_status odla_CopyMemory(odla_void* dst, odla_void* src, odla_size_t size, odla_memcpy_type type) {
  if (dst == nullptr || src == nullptr) return ODLA_INVALID_PARAM;
  hipMemcpyKind kind;
  switch (type) {
    case ODLA_MEMCPY_H2H: kind = hipMemcpyHostToHost; break;
    case ODLA_MEMCPY_H2D: kind = hipMemcpyHostToDevice; break;
    case ODLA_MEMCPY_D2H: kind = hipMemcpyDeviceToHost; break;
    case ODLA_MEMCPY_D2D: kind = hipMemcpyDeviceToDevice; break;
    default: return ODLA_INVALID_PARAM;
  }
  return hipMemcpy(dst, src, size, kind) == hipSuccess ? ODLA_SUCCESS : ODLA_FAILURE;
}

// ----------------------------------------------------------------- logging --
odla_status odla_SetLogLevel(odla_log_level level) {
  g_log_level.store((int)level);
  return ODLA_SUCCESS;
}
odla_status odla_SetLogger(odla_logging_func logger) {
  g_logger.store(logger ? logger : default_logger);
  return ODLA_SUCCESS;
}
odla_logging_func odla_GetLogger(void) { return g_logger.load(); }

const odla_char* odla_GetVersionString(void) { return kVersion; }

}  // extern "C"
