// Calibration profiler: records the value ranges of a computation while it
// runs on the GPU and writes them in the reference profiler's JSON layout.
//
// The reference does this with an interposer library that forwards every
// odla_<Op> call to its CPU interpreter, copies each result to the host and
// scans it there [ref: ODLA/platforms/odla_profiler.cc:133-226].  Here the
// library itself has a calibration mode: while profiling is on, computations
// are compiled in fp32 with nothing fused and a range-statistics kernel behind
// every named fp32 value; after each execution the few partial minima / maxima
// are read back and one record per value is appended to the open run.  The
// control functions keep the reference's names and meaning
// [ref: odla_profiler.cc:228-285], so a harness written for the reference's
// profiler (utils/halo_pgq.py:205-239) drives this one unchanged.
#include <algorithm>
#include <cstdio>
#include <cstring>
#include <limits>
#include <map>
#include <mutex>
#include <string>
#include <vector>

#include "internal.h"

namespace ohip {

namespace {
struct ProfilerState {
  std::mutex mu;
  bool active = false;
  FILE* out = nullptr;     // null: stdout
  int rec_cnt = 0, run_cnt = 0;
  bool in_run = false;
  bool channels = false;
  int axis = -1;
  bool skip_weights = false;
  std::map<std::string, std::vector<std::string>> uses;  // value -> names of its operands
};
ProfilerState g_prof;

FILE* os() { return g_prof.out ? g_prof.out : stdout; }

void put_float(FILE* f, float v) {
  if (v != v) fputs("NaN", f);
  else if (v == std::numeric_limits<float>::infinity()) fputs("Infinity", f);
  else if (v == -std::numeric_limits<float>::infinity()) fputs("-Infinity", f);
  else fprintf(f, "%.9g", (double)v);
}
void put_list(FILE* f, const std::vector<float>& v) {
  fputc('[', f);
  for (size_t i = 0; i < v.size(); ++i) {
    if (i) fputs(", ", f);
    put_float(f, v[i]);
  }
  fputc(']', f);
}
}  // namespace

bool profiler_active() {
  std::lock_guard<std::mutex> lk(g_prof.mu);
  return g_prof.active;
}

void profiler_configure(Options* o) {
  std::lock_guard<std::mutex> lk(g_prof.mu);
  o->calibrate = g_prof.active;
  o->calib_channels = g_prof.channels;
  o->calib_axis = g_prof.axis;
  o->calib_skip_weights = g_prof.skip_weights;
}

odla_status profiler_collect(const Plan& plan, const char* arena) {
  std::lock_guard<std::mutex> lk(g_prof.mu);
  if (!g_prof.active || !g_prof.in_run) return ODLA_SUCCESS;  // executions outside a run are not recorded
  std::vector<float> part;
  for (const Plan::StatRec& r : plan.stat_recs) {
    const PTensor& t = plan.tensors[r.tensor];
    const size_t n = (size_t)r.channels * r.splits * 2;
    part.resize(n);
    if (hipMemcpy(part.data(), arena + t.offset, n * sizeof(float), hipMemcpyDeviceToHost) != hipSuccess) {
      OHIP_ERR("profiler: cannot read the statistics of '%s'", r.name.c_str());
      return ODLA_FAILURE;
    }
    std::vector<float> ch_min, ch_max;
    float lo = std::numeric_limits<float>::infinity(), hi = -lo;
    for (int c = 0; c < r.channels; ++c) {
      float cl = std::numeric_limits<float>::infinity(), ch = -cl;
      for (int s = 0; s < r.splits; ++s) {
        cl = std::min(cl, part[((size_t)c * r.splits + s) * 2]);
        ch = std::max(ch, part[((size_t)c * r.splits + s) * 2 + 1]);
      }
      lo = std::min(lo, cl);
      hi = std::max(hi, ch);
      if (r.per_channel) { ch_min.push_back(cl); ch_max.push_back(ch); }
    }
    FILE* f = os();
    if (g_prof.rec_cnt > 0) fputc(',', f);
    fprintf(f, "\n\"%s\" : {\"op_type\": \"%s\", \"shape\": [", r.name.c_str(), r.op_type.c_str());
    for (int i = 0; i < r.shape.rank; ++i) fprintf(f, "%s%lld", i ? ", " : "", (long long)r.shape.d[i]);
    fprintf(f, "], \"channels\": %zu, \"min_value\": ", ch_min.size());
    put_float(f, lo);
    fputs(", \"max_value\": ", f);
    put_float(f, hi);
    fputs(", \"channels_min\": ", f);
    put_list(f, ch_min);
    fputs(", \"channels_max\": ", f);
    put_list(f, ch_max);
    fputc('}', f);
    ++g_prof.rec_cnt;
    if (!r.inputs.empty()) g_prof.uses[r.name] = r.inputs;
  }
  return ODLA_SUCCESS;
}

const char* api_op_name(const Node& n) {
  static const char* bin[] = {"odla_Add", "odla_Sub", "odla_Mul", "odla_Div", "odla_Max", "odla_Min"};
  static const char* red[] = {"odla_ReduceMean", "odla_ReduceSum", "odla_ReduceMax", "odla_ReduceMin", "odla_ReduceProd",
                              "odla_ReduceL1", "odla_ReduceL2", "odla_ReduceSumSquare", "odla_ReduceLogSum"};
  static const char* act[] = {
      "odla_Identity", "odla_Relu", "odla_LeakyRelu", "odla_Clamp", "odla_Sigmoid", "odla_Tanh", "odla_Gelu", "odla_Gelu",
      "odla_Exp", "odla_Log", "odla_Sqrt", "odla_Rsqrt", "odla_Erf", "odla_Abs", "odla_Neg", "odla_Round",
      "odla_Reciprocal", "odla_Ceil", "odla_Floor", "odla_Sign", "odla_Sin", "odla_Cos", "odla_Tan", "odla_ASin",
      "odla_ACos", "odla_ATan", "odla_Sinh", "odla_Cosh", "odla_ASinh", "odla_ACosh", "odla_ATanh", "odla_Elu",
      "odla_Selu", "odla_Celu", "odla_HardSigmoid", "odla_Softplus", "odla_Softsign", "odla_ThresholdedRelu",
      "odla_Shrink", "odla_Mean"};
  static const char* ew[] = {"odla_Add", "odla_Sub", "odla_Mul", "odla_Div", "odla_Max", "odla_Min", "odla_Pow", "odla_Mod",
                             "odla_Mod", "odla_PRelu", "odla_SquaredDifference", "odla_Select", "odla_Equal",
                             "odla_NotEqual", "odla_Less", "odla_LessOrEqual", "odla_Greater", "odla_GreaterOrEqual",
                             "odla_And", "odla_Or", "odla_Xor", "odla_Not", "odla_IsNaN", "odla_IsInf", "odla_IsInf",
                             "odla_IsInf"};
  auto pick = [](const char* const* tbl, size_t n, int64_t i) { return i >= 0 && (size_t)i < n ? tbl[i] : "odla_Op"; };
  switch (n.op) {
    case OP_CONV: return "odla_Conv";
    case OP_GEMM: return "odla_Gemm";
    case OP_BINARY: return pick(bin, sizeof(bin) / sizeof(*bin), n.i[0]);
    case OP_UNARY: return pick(act, sizeof(act) / sizeof(*act), n.i[0]);
    case OP_BATCHNORM: return "odla_BatchNormalization";
    case OP_LAYERNORM: return "odla_LayerNorm";
    case OP_POOL: return n.i[1] ? "odla_MaxPool" : "odla_AveragePool";
    case OP_REDUCE: return pick(red, sizeof(red) / sizeof(*red), n.i[0]);
    case OP_SOFTMAX: return n.i[1] ? "odla_LogSoftmax" : "odla_Softmax";
    case OP_CAST: return "odla_Cast";
    case OP_CONCAT: return "odla_Concat";
    case OP_GATHER: return "odla_Gather";
    case OP_RESHAPE: return "odla_Reshape";
    case OP_RESIZE: return "odla_Resize";
    case OP_SLICE: return "odla_Slice";
    case OP_TRANSPOSE: return "odla_Transpose";
    case OP_QUANTIZE: return "odla_Quantize";
    case OP_DEQUANTIZE: return "odla_Dequantize";
    case OP_NMS: return "odla_NMS";
    case OP_EWISE: return pick(ew, sizeof(ew) / sizeof(*ew), n.i[0]);
    case OP_ARGEXT: return n.i[0] ? "odla_ArgMax" : "odla_ArgMin";
    case OP_COPYND: return n.i[0] ? "odla_Pad" : "odla_Tile";
    case OP_TOPK: return "odla_TopK";
    case OP_LRN: return "odla_LRN";
    case OP_ROWNORM: return "odla_InstanceNormalization";
    case OP_POSTPROCESS: return "odla_PostProcess";
    case OP_AXISOP:
      switch ((AxisOp)n.i[0]) {
        case AX_GATHER_ELEMENTS: return "odla_GatherElements";
        case AX_CUMSUM: return "odla_CumSum";
        case AX_HARDMAX: return "odla_Hardmax";
        case AX_COMPRESS: return "odla_Compress";
      }
      return "?";
  }
  return "odla_Op";
}

}  // namespace ohip

using ohip::g_prof;

extern "C" {

void EnableChannelWiseProf(void) {
  std::lock_guard<std::mutex> lk(g_prof.mu);
  g_prof.channels = true;
}
void SetChannelAxis(int axis) {
  std::lock_guard<std::mutex> lk(g_prof.mu);
  g_prof.axis = axis;
}
void SkipWeightsProfiling(bool skip) {
  std::lock_guard<std::mutex> lk(g_prof.mu);
  g_prof.skip_weights = skip;
}

void StartProfiling(const char* data_path) {
  std::lock_guard<std::mutex> lk(g_prof.mu);
  if (g_prof.out != nullptr) { fclose(g_prof.out); g_prof.out = nullptr; }
  g_prof.rec_cnt = 0;
  g_prof.run_cnt = 0;
  g_prof.in_run = false;
  g_prof.uses.clear();
  if (data_path != nullptr) {
    g_prof.out = fopen(data_path, "w");
    if (g_prof.out == nullptr) OHIP_ERR("StartProfiling: cannot open '%s'; writing to stdout", data_path);
  }
  g_prof.active = true;
  fputs("{\n\"ProfilingResults\": {\n", ohip::os());
}

void StartOneRun(const char* tag) {
  std::lock_guard<std::mutex> lk(g_prof.mu);
  if (!g_prof.active) return;
  FILE* f = ohip::os();
  if (g_prof.run_cnt > 0) fputc(',', f);
  ++g_prof.run_cnt;
  fprintf(f, "\"%s\" : {\n", tag ? tag : "");
  g_prof.rec_cnt = 0;
  g_prof.in_run = true;
}

void StopOneRun(void) {
  std::lock_guard<std::mutex> lk(g_prof.mu);
  if (!g_prof.active || !g_prof.in_run) return;
  fputs("}\n", ohip::os());
  g_prof.in_run = false;
}

void StopProfiling(void) {
  std::lock_guard<std::mutex> lk(g_prof.mu);
  if (!g_prof.active) return;
  FILE* f = ohip::os();
  if (g_prof.in_run) { fputs("}\n", f); g_prof.in_run = false; }
  fputs("}, \n\"NetworkInfo\": {\n", f);
  bool first = true;
  for (const auto& kv : g_prof.uses) {
    fprintf(f, "%s\"%s\" :{\n  \"inputs\":[", first ? "" : ", \n", kv.first.c_str());
    for (size_t i = 0; i < kv.second.size(); ++i) fprintf(f, "%s\"%s\"", i ? ", " : "", kv.second[i].c_str());
    fputs("]\n}", f);
    first = false;
  }
  fputs("}\n}\n", f);
  if (g_prof.out != nullptr) { fclose(g_prof.out); g_prof.out = nullptr; }
  else fflush(stdout);
  g_prof.active = false;
  g_prof.channels = false;
  g_prof.axis = -1;
  g_prof.skip_weights = false;
}

}  // extern "C"
