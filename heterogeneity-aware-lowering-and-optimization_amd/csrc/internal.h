// Private structures of libodla_hip.so: the recorded graph (values + nodes),
// the compiled plan (physical tensors + launch steps) and the execution
// context (device arena, stream, captured hipGraph).
#ifndef ODLA_HIP_INTERNAL_H_
#define ODLA_HIP_INTERNAL_H_

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <functional>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "../../include/odla_hip.h"
#include "kernels/kernels.h"

namespace ohip {

// ---------------------------------------------------------------- logging --
void log_msg(const char* file, int line, const char* func, odla_log_level lvl, const char* fmt, ...)
    __attribute__((format(printf, 5, 6)));
#define OHIP_LOG(lvl, ...) ::ohip::log_msg(__FILE__, __LINE__, __func__, lvl, __VA_ARGS__)
#define OHIP_ERR(...) OHIP_LOG(ODLA_LOG_LEVEL_ERROR, __VA_ARGS__)
#define OHIP_WARN(...) OHIP_LOG(ODLA_LOG_LEVEL_WARN, __VA_ARGS__)
#define OHIP_INFO(...) OHIP_LOG(ODLA_LOG_LEVEL_INFO, __VA_ARGS__)
#define OHIP_DEBUG(...) OHIP_LOG(ODLA_LOG_LEVEL_DEBUG, __VA_ARGS__)

// ------------------------------------------------------------------ graph --
enum OpKind : int {
  OP_CONV, OP_GEMM, OP_BINARY, OP_UNARY, OP_BATCHNORM, OP_LAYERNORM, OP_POOL, OP_REDUCE,
  OP_SOFTMAX, OP_CAST, OP_CONCAT, OP_GATHER, OP_RESHAPE, OP_RESIZE, OP_SLICE, OP_TRANSPOSE,
  OP_QUANTIZE, OP_DEQUANTIZE, OP_NMS, OP_EWISE, OP_ARGEXT, OP_COPYND, OP_TOPK, OP_LRN, OP_ROWNORM,
  OP_POSTPROCESS, OP_AXISOP
};
// sub-kinds of OP_AXISOP (Node::i[0])
enum AxisOp : int { AX_GATHER_ELEMENTS = 0, AX_CUMSUM, AX_HARDMAX, AX_COMPRESS };
const char* op_name(OpKind k);

struct Shape {
  int rank = 0;
  int64_t d[ODLA_MAX_DIMENSION] = {0};
  int64_t numel() const {
    int64_t n = 1;
    for (int i = 0; i < rank; ++i) n *= d[i];
    return n;
  }
  bool operator==(const Shape& o) const {
    if (rank != o.rank) return false;
    for (int i = 0; i < rank; ++i)
      if (d[i] != o.d[i]) return false;
    return true;
  }
  bool operator!=(const Shape& o) const { return !(*this == o); }
  std::string str() const;
};
Shape shape_from(const odla_value_shape& s);    // scalars become {1}
odla_value_shape shape_to(const Shape& s);
bool shape_valid(const odla_value_shape& s);     // plausible caller-provided shape?

struct Node;

}  // namespace ohip

struct _odla_computation;

struct _odla_value {
  enum Kind { ARG, CONSTANT, TEMP };
  Kind kind = TEMP;
  std::string name;  // empty for anonymous temporaries
  odla_element_type etype = ODLA_FLOAT32;
  ohip::Shape shape;
  const void* host_data = nullptr;  // CONSTANT: borrowed from the caller
  int index = -1;                   // position in computation->values
  int producer = -1;                // node index, -1 for ARG / CONSTANT
  bool is_output = false;
  bool dyn_batch = false;           // ARG declared with a negative leading extent (the run-time batch)
  bool eager = false;               // created by odla_CreateValue: data comes from odla_SetValueData
  const void* eager_data = nullptr; // borrowed from the caller
  _odla_computation* comp = nullptr;
};

namespace ohip {

struct Node {
  OpKind op;
  std::vector<_odla_value*> in;  // nullptr entries allowed for optional operands
  _odla_value* out = nullptr;
  _odla_value* out2 = nullptr;  // second result (TopK indices)
  // attributes (meaning depends on op; see api_ops.cc)
  int64_t i[24] = {0};
  float f[8] = {0};
  std::vector<int64_t> iv;
  bool absorbed = false;  // set by the planner when fused into another node
};

struct Options {
  bool fp16 = false;
  odla_bf16_mode bf16 = BF16_DISABLE;
  bool int8 = false;
  bool raw_acc = false;
  const odla_value_quant_info* qtable = nullptr;
  int qtable_size = 0;
  // calibration: fp32, nothing fused, range statistics behind every named fp32 value
  bool calibrate = false;
  bool calib_channels = false;   // also per-channel ranges
  int calib_axis = -1;           // channel axis (negative: from the end)
  bool calib_skip_weights = false;
};

// ------------------------------------------------------------------- plan --
enum Layout : int { L_ROWMAJOR = 0, L_NHWC = 1 };
enum Space : int { SP_ARENA = 0, SP_CONST = 1, SP_INIT = 2, SP_NONE = 3 };

// A physical device tensor.  For L_NHWC the logical shape is N,C,H,W and the
// memory order N,H,W,cs with cs >= C.
struct PTensor {
  DType dt = DT_F32;
  Layout layout = L_ROWMAJOR;
  Shape shape;      // logical
  int cs = 0;       // channel pitch (L_NHWC only)
  Space space = SP_NONE;
  size_t offset = 0;
  size_t bytes = 0;
  int alias_of = -1;     // shares storage with another tensor (Reshape, a slice of a merged result)
  size_t alias_off = 0;  // byte offset of an alias inside the root tensor's storage
  int def_step = -1, last_step = -1;
  bool pinned = false;   // lives for the whole execution (inputs being staged, outputs)
  int ext_slot = -1;     // argument staging tensor that steps may read in the caller's buffer instead (ExecEnv::ext)
  bool quant = false;    // 8-bit affine levels stored as q-128
  float qscale = 1.f;
  int qzp = 0;
  int64_t phys_elems() const {
    if (layout == L_NHWC) return shape.d[0] * shape.d[2] * shape.d[3] * cs;
    return shape.numel();
  }
};

struct ExecEnv {
  char* base[3] = {nullptr, nullptr, nullptr};  // indexed by Space
  // Per argument (Plan::inputs order), then per result (Plan::outputs order): the caller's
  // device buffer when the steps read / write it in place, nullptr when the data goes
  // through the staging tensor in the arena.
  const char* const* ext = nullptr;
  // Number, in the caller's batch, of the first image this execution works on (not 0 for the
  // second of two half-batch copies): operators that write image numbers add it.
  int image_base = 0;
};

struct Step {
  std::string name;
  std::function<hipError_t(const ExecEnv&, hipStream_t)> fn;
};

struct QuantEntry {
  float scale = 0.f;
  int zp = 0;
  float min = 0.f, max = 0.f;
  std::vector<float> ch_min, ch_max;
};

struct Plan {
  std::vector<PTensor> tensors;
  std::vector<Step> steps;       // replayed on every execution
  std::vector<Step> init_steps;  // run once when the plan is created
  size_t arena_bytes = 0;
  size_t const_bytes = 0;
  size_t init_bytes = 0;
  char* const_pool = nullptr;
  struct IO {
    _odla_value* v = nullptr;
    int tensor = -1;  // staging tensor in the arena: row-major, declared element type
    size_t offset = 0;  // byte offset inside that tensor (results that are slices of a merged launch)
    size_t bytes = 0;
    // arguments: every step that touches the staging tensor reads exactly its elements and
    // checks alignment itself, and nothing writes it: a device buffer can be read in place;
    // results: only the final conversion to the declared type touches the tensor, and it
    // writes exactly its elements: a device buffer can be written in place
    bool in_place_ok = false;
  };
  std::vector<IO> inputs, outputs;
  std::unordered_map<const _odla_value*, int> final_tensor;  // for odla_GetValueData
  // calibration plans: one record per profiled value; its partial minima /
  // maxima live in a pinned arena tensor as [channels][splits][2] floats
  struct StatRec {
    std::string name, op_type;
    Shape shape;
    int channels = 1;       // partial rows (1 when no per-channel ranges were asked for)
    bool per_channel = false;
    int splits = 1;
    int tensor = -1;
    std::vector<std::string> inputs;
  };
  std::vector<StatRec> stat_recs;
  bool calibrated = false;
  // host blobs copied into the constant pool / init scratch when the plan is built
  struct Blob { Space space; size_t offset; std::vector<uint8_t> owned; const void* src; size_t bytes; };
  std::vector<Blob> blobs;
  ~Plan();
};

odla_status build_plan(_odla_computation* comp, std::unique_ptr<Plan>* out);
// Host-only lowering: the plan is built, measured and dropped (no device call).
odla_status plan_summary(_odla_computation* comp, int* launches, int* init_launches, size_t* arena_bytes,
                         size_t* const_bytes);

// Calibration profiler (the control functions StartProfiling .. are exported
// with the reference profiler's names).
bool profiler_active();
void profiler_configure(Options* o);
// Reads the statistics of one finished execution and appends them to the open run.
odla_status profiler_collect(const Plan& plan, const char* arena);
const char* api_op_name(const Node& n);

DType dtype_from_odla(odla_element_type t);
int odla_type_size(odla_element_type t);

}  // namespace ohip

struct _odla_executable {
  _odla_computation* comp = nullptr;
  bool owns = false;  // made by odla_LoadExecutable: destroying it destroys the computation
};

struct _odla_computation {
  std::vector<std::unique_ptr<_odla_value>> values;
  std::vector<ohip::Node> nodes;
  std::vector<_odla_value*> args, outputs;
  std::unordered_map<std::string, _odla_value*> by_name;
  // library-created constants (scalars, folded parameters)
  std::vector<std::unique_ptr<std::vector<uint8_t>>> owned_data;
  ohip::Options opts;
  std::mutex mu;
  std::unique_ptr<ohip::Plan> plan;
  bool plan_failed = false;
  size_t planned_nodes = 0;          // size of `nodes` when the plan was built
  int live_contexts = 0;             // contexts created by the caller
  _odla_context* eager_ctx = nullptr;  // context behind odla_GetValueData(value, ptr, NULL)
  _odla_executable executable;       // handle given out by odla_CompileComputation / odla_LoadExecutable
  // dynamic batch [ref: ODLA/platforms/tensorrt/odla_tensorrt.cc:138-179]: arguments are
  // recorded with max_batch as their leading extent; a context that asks for
  // another batch runs a copy of the recording whose shapes were rescaled
  bool dynamic_batch = false;
  int min_batch = 0, max_batch = 0, opt_batch = 0;
  // by run-time batch; owned by the contexts that run them (see _odla_context::variant_ctx):
  // a variant, its plan and its packed constants go away with its last user
  std::map<int, std::weak_ptr<_odla_computation>> variants;
  // quantisation table of a loaded computation (the caller's table is borrowed otherwise)
  std::vector<odla_value_quant_info> owned_qtable;
  std::vector<std::string> owned_qnames;
};

struct _odla_context {
  _odla_computation* comp = nullptr;
  hipStream_t stream = nullptr;
  char* arena = nullptr;
  size_t arena_bytes = 0;
  bool use_graph = true;
  hipGraph_t graph = nullptr;
  hipGraphExec_t graph_exec = nullptr;
  std::vector<const char*> graph_ext;   // the caller's buffers the captured launches read / write in place
  std::vector<const char*> last_ext;    // those of the last execution (odla_GetValueData finds results there)
  int capture_streak = 0;               // executions in a row that had to capture for new buffers
  bool in_place_off = false;            // the caller binds new buffers every time: copy instead
  // Graphs captured for other sets of argument buffers (a caller that alternates between a
  // few device buffers replays instead of capturing again); bounded, oldest dropped first.
  struct ParkedGraph { std::vector<const char*> ext; hipGraph_t graph; hipGraphExec_t exec; };
  std::vector<ParkedGraph> parked_graphs;
  std::unordered_map<const _odla_value*, const void*> bound_in;
  std::unordered_map<const _odla_value*, void*> bound_out;
  bool executed = false;
  int run_batch = 0;                              // 0: the recorded shapes
  // Contexts over comp->variants, by batch.  Every batch a context has run keeps a
  // planned copy of the recording alive (packed constants, arena, stream, graph),
  // so the map is bounded: beyond kMaxBatchVariants (ODLA_HIP_MAX_BATCH_VARIANTS)
  // entries the one used longest ago is destroyed and rebuilt if it is asked for again.
  struct Variant {
    std::shared_ptr<_odla_computation> comp;
    _odla_context* ctx = nullptr;
    uint64_t last_use = 0;
  };
  std::map<int, Variant> variant_ctx;
  uint64_t variant_clock = 0;
  // Two contexts over ONE copy of the recording at half the batch, executed side by side on
  // their own streams, each on its half of the caller's buffers (see execute_split).
  struct Split {
    bool tried = false, ok = false;
    std::shared_ptr<_odla_computation> comp;
    _odla_context* half[2] = {nullptr, nullptr};
    // Without ODLA_HIP_BATCH_SPLIT the context measures: six executions whole, eight in halves,
    // the fastest of the last three of each counts; then the faster way is kept.
    int trial = 0;            // executions counted so far (stops at 14)
    double whole_ms = 0, halves_ms = 0;
    int choice = 0;           // 0 undecided, 1 whole, 2 halves
  } split;
  bool is_half = false;   // this context is one of those halves: it runs as it is
  int image_base = 0;        // see ExecEnv::image_base
  // Halves only: the second half stages its arguments after the first has staged its own
  // (copies from host memory then follow each other at full PCIe rate, and the first half
  // computes while the second half's arguments travel).  The first half records
  // `inputs_staged` behind its copies (it owns the event), the second waits for `wait_inputs`.
  hipEvent_t inputs_staged = nullptr;
  hipEvent_t wait_inputs = nullptr;
  // Halves only: the execution returns once the launches are queued; the parent queues the
  // copies of the results of both halves afterwards (a copy into pageable host memory blocks
  // the calling thread until the stream has reached it - the second half would not even be
  // queued before the first has finished).
  bool defer_fetch = false;
  bool last_split = false;   // the last execution ran as halves: results live in their arenas / the caller's buffers
  bool said_uncaptured = false;   // the note that a short launch sequence runs without a graph has been logged
};

struct _odla_device {
  int index = 0;
};

namespace ohip {
_odla_computation* current_computation();
void set_current_computation(_odla_computation* c);
void forget_computation(_odla_computation* c);
_odla_value* new_value(_odla_computation* c, _odla_value::Kind kind, odla_element_type et,
                       const Shape& shape, const odla_value_id id);
odla_status compile_computation(_odla_computation* c);  // builds the plan if there is none yet
// Leading extent the dynamic-batch arguments of `c` were recorded with (0: none).
int recorded_batch(const _odla_computation& c);
// A copy of the recording of `c` in which every value that depends on an
// argument has its leading extent rescaled from `from` to `to`; nullptr (and a
// log line) when the graph moves the batch out of the leading position.
// rows_apart: the copy is to run on one part of the batch while another copy runs on the rest, so
// the graph must also keep the rows of different images apart in every result (refusals are then
// logged at debug level only).
std::unique_ptr<_odla_computation> clone_for_batch(const _odla_computation& c, int64_t from, int64_t to,
                                                   bool rows_apart = false);
}  // namespace ohip

#endif
