// Host-visible launch interface of the gfx950 kernels behind libodla_hip.so.
//
// Every launcher validates its operands on the host before enqueueing work on
// `stream` and returns hipErrorInvalidValue instead of launching a kernel whose
// indexing assumptions do not hold.  Nothing here allocates memory.
#ifndef ODLA_HIP_KERNELS_H_
#define ODLA_HIP_KERNELS_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ohip {

// Size of the statically allocated device scratch behind
// odla_hip_ExecuteComputationStatic (kernels/static_arena.hip): plans whose
// temporaries need more are refused by that entry point.
constexpr size_t kStaticArenaBytes = 64u << 20;
// Address (on the calling thread's current device) and size of that scratch.
// Allocates nothing; the first call on a device resolves the symbol.
hipError_t static_arena(void** ptr, size_t* bytes);

// Storage types of device tensors.
enum DType : int {
  DT_F32 = 0,
  DT_F16 = 1,
  DT_BF16 = 2,
  DT_I8 = 3,  // quantised activations are stored as (q - 128) in int8 so that
              // unsigned 8-bit data feeds the signed MFMA; weights are plain s8
  DT_U8 = 4,
  DT_I32 = 5,
  DT_I64 = 6,
  DT_BOOL = 7,
  DT_INVALID = -1
};

inline int dtype_size(DType t) {
  switch (t) {
    case DT_F32: case DT_I32: return 4;
    case DT_F16: case DT_BF16: return 2;
    case DT_I8: case DT_U8: case DT_BOOL: return 1;
    case DT_I64: return 8;
    default: return 0;
  }
}
inline bool dtype_is_float(DType t) { return t == DT_F32 || t == DT_F16 || t == DT_BF16; }

// Magic pair for the kernels' fast_div(n, magic, shift) = n / d, 0 <= n < 2^31, 1 <= d < 2^31:
// shift = ceil(log2 d), magic = ceil(2^(31+shift) / d).
inline void div_magic(int d, unsigned* magic, int* shift) {
  int s = 0;
  while ((1ll << s) < d) ++s;
  *shift = s;
  *magic = (unsigned)((((unsigned long long)1 << (31 + s)) + (unsigned long long)d - 1) / (unsigned long long)d);
}

// Activation applied in a GEMM epilogue or by the unary kernel.
enum ActKind : int {
  ACT_NONE = 0, ACT_RELU, ACT_LEAKY, ACT_CLAMP, ACT_SIGMOID, ACT_TANH,
  ACT_GELU_ERF, ACT_GELU_TANH, ACT_EXP, ACT_LOG, ACT_SQRT, ACT_RSQRT, ACT_ERF,
  ACT_ABS, ACT_NEG, ACT_ROUND, ACT_RECIP,
  ACT_CEIL, ACT_FLOOR, ACT_SIGN, ACT_SIN, ACT_COS, ACT_TAN, ACT_ASIN, ACT_ACOS, ACT_ATAN,
  ACT_SINH, ACT_COSH, ACT_ASINH, ACT_ACOSH, ACT_ATANH,
  ACT_ELU,          // x > 0 ? x : a * (exp(x) - 1)
  ACT_SELU,         // b * elu(x, a)
  ACT_CELU,         // max(0, x) + min(0, a * (exp(x / a) - 1))
  ACT_HARDSIGMOID,  // clamp(a * x + b, 0, 1)
  ACT_SOFTPLUS,     // log(exp(x) + 1)
  ACT_SOFTSIGN,     // x / (|x| + 1)
  ACT_THRESHOLDED,  // x > a ? x : 0
  ACT_SHRINK,       // x > b ? x - a : (x < -b ? x + a : 0)
  ACT_DIV_CONST     // x / a
};

enum BinKind : int { BIN_ADD = 0, BIN_SUB, BIN_MUL, BIN_DIV, BIN_MAX, BIN_MIN };

// ---------------------------------------------------------------------------
// Implicit-GEMM convolution / GEMM on MFMA.
//
//   y[z][m][n] = epilogue( sum_k A[z][m][k] * Wt[z][n][k] )
//
// A is gathered on the fly from a channels-last activation tensor
// x[z][N][H][W][xcs] (m = (n,ho,wo), k = (r,s,c), c < C); a plain GEMM is the
// case H = W = R = S = 1.  Wt is a row-major [w_rows][w_rs] matrix whose row n
// holds output channel n with k ordered (r,s,c); rows >= w_rows and columns
// >= w_cols are read as zero.  C and w_rs must be multiples of 16 bytes worth
// of elements, x and w 16-byte aligned.
struct IgemmParams {
  const void* x = nullptr;
  const void* w = nullptr;
  void* y = nullptr;
  const void* bias = nullptr;      // float[Kout] (int32[Kout] for int8), or null
  const void* residual = nullptr;  // same type/geometry as y, or null
  int N = 1, H = 1, W = 1, C = 0;  // C = reduction channels per tap
  int xcs = 0;                     // element stride between pixels of x
  int Ho = 1, Wo = 1, Kout = 0;
  int R = 1, S = 1, sh = 1, sw = 1, ph = 0, pw = 0, dh = 1, dw = 1;
  int w_rows = 0, w_cols = 0, w_rs = 0;
  int ycs = 0;                     // element stride between rows of y
  int rcs = 0;                     // element stride between rows of residual
  int batch = 1;                   // grid.z: independent problems (groups, heads)
  int64_t x_bs = 0, w_bs = 0, y_bs = 0, r_bs = 0, bias_bs = 0;  // per-z element strides
  // Result addressing beyond "row m at m * ycs" (float types, no residual), so that a
  // transposition behind the GEMM costs nothing:
  //   y_rdiv > 0: row m = (a, b) with b = m % y_rdiv lies at a * y_rhi + b * y_rlo, and
  //               column n = (c, d) with d = n % y_cdiv at c * y_chi + d - a [B*S, heads*d]
  //               result stored as [B, heads, S, d];
  //   y_zdiv > 0: problem z = (u, v) with v = z % y_zdiv starts at u * y_bs_hi + v * y_bs -
  //               a [B*heads] batch of [S, d] results stored as [B, S, heads, d] (ycs = heads*d).
  int y_rdiv = 0, y_cdiv = 1, y_zdiv = 0;
  int64_t y_rhi = 0, y_rlo = 0, y_chi = 0, y_bs_hi = 0;
  DType in_dt = DT_F32;            // type of x and w
  DType out_dt = DT_F32;           // type of y and residual
  // Optional copy of w in MFMA fragment order (see WfragPackParams); when set,
  // layers with enough output channels read their weights from it directly
  // into registers.  wf_chunks = 32-byte K chunks per row (a multiple of 4
  // covering R*S*C), wf_tiles = 32-row tiles per batch entry.
  const void* w_frag = nullptr;
  int wf_chunks = 0, wf_tiles = 0;
  // filled in by launch_igemm: magic pairs for the divisions by Ho*Wo, Wo, y_rdiv and y_cdiv
  unsigned howo_magic = 0, wo_magic = 0, yr_magic = 0, yc_magic = 0;
  int howo_shift = 0, wo_shift = 0, yr_shift = 0, yc_shift = 0;
  float alpha = 1.0f;              // scales the accumulator before bias (float types)
  ActKind act = ACT_NONE;
  float act_a = 0.0f, act_b = 0.0f;  // leaky slope / clamp lo,hi
  bool res_after_act = false;        // float types: y = act(..) + residual instead of act(.. + residual)
  bool stream_out = false;           // 2-byte results leave with non-temporal stores (results far larger than the last-level cache)
  // Softmax (1) or LogSoftmax (2) over the Kout columns of every result row, behind bias and
  // activation: only the one-wavefront-per-row kernel computes it (gemm_rowdot_shape).
  int row_softmax = 0;
  // int8 only -----------------------------------------------------------
  // acc = int32 accumulator + int32 bias; fma = one fused multiply-add in fp32
  // (a single rounding); sat8 = round to nearest even and saturate to [0, 255].
  // out_dt == DT_I8 : q = sat8(max(fma(float(acc), qmul[n], q_add), q_lo))
  //                   with q_add = the zero point of the result, or, with a
  //                   residual r (levels of an 8-bit tensor):
  //                   q = sat8(max(fma(float(acc), qmul[n], fma(float(r), r_mul, r_add)), q_lo))
  //                   qmul[n] = s_x s_w[n] / s_y, r_mul = s_r / s_y,
  //                   r_add = zp_y - zp_r * r_mul: convolution, residual add and
  //                   ReLU (q_lo = zp_y) are requantised ONCE.
  // out_dt == DT_F32: y = float(acc) * qmul[n]    (dequantised result)
  // out_dt == DT_I32: y = acc                     (raw accumulators)
  const float* qmul = nullptr;
  int a_fill = 0;  // stored byte that represents the real value 0 in x
  float q_add = 0.f, q_lo = 0.f;
  float r_mul = 0.f, r_add = 0.f;
  // A second 8-bit 1x1 layer computed from this layer's result while a pixel tile of it is still
  // in LDS (f_y != nullptr; igemm_stream_q8_fusable says which pairs): y2 = requant(y . w2 + bias2)
  // with the second layer's own fragment-ordered weights, int32 bias, multipliers, zero point and
  // lower bound.  Both results are written; the second layer's read of y from memory is what is saved.
  const void* f_wfrag = nullptr;
  const void* f_bias = nullptr;
  const float* f_qmul = nullptr;
  void* f_y = nullptr;
  int f_kout = 0, f_ycs = 0, f_wf_chunks = 0;
  float f_q_add = 0.f, f_q_lo = 0.f;
};
hipError_t launch_igemm(const IgemmParams& p, hipStream_t stream);
// Name of the kernel variant launch_igemm would pick (for reports).
const char* igemm_variant_name(const IgemmParams& p);

// Products with at most 16 output columns, a long reduction and few rows (gemm_rowdot.hip): one
// wavefront per output row.  Whether the shape qualifies, and the launch (launch_igemm uses both).
bool gemm_rowdot_shape(const IgemmParams& p);
hipError_t launch_gemm_rowdot(const IgemmParams& p, hipStream_t stream);

// Large-tile kernels (igemm_big.hip) for matrix-core-bound layers: the variant
// launch_igemm uses for this shape (0: none), and the launch itself.
int igemm_big_variant(const IgemmParams& p);
hipError_t launch_igemm_big(const IgemmParams& p, int epi_vec, int variant, hipStream_t stream);

// Streaming kernel for 8-bit 1x1 filters over short pixel rows (igemm_stream.hip):
// whether the layer's geometry qualifies (no pointer is looked at), and the launch
// (p.w_frag, p.qmul and the division magics must be set; launch_igemm does that).
bool igemm_stream_q8_geometry(const IgemmParams& p);
// Whether layer b (its x being a's result) can ride in a's launch (see IgemmParams::f_y); no
// pointer is looked at.
bool igemm_stream_q8_fusable(const IgemmParams& a, const IgemmParams& b);
hipError_t launch_igemm_stream_q8(const IgemmParams& p, hipStream_t stream);
// 3x3, stride 1, padding 1 with the input patch of a tile held in LDS (igemm_c3.hip): whether
// the layer is one of its shapes, and its launch (called by launch_igemm with its epi_vec).
bool igemm_c3_geometry(const IgemmParams& p);
hipError_t launch_igemm_c3(const IgemmParams& p, int epi_vec, hipStream_t stream);

// True when launch_igemm would use a fragment-ordered weight copy for this shape.
bool igemm_wants_wfrag(const IgemmParams& p);
// [batch][rows][row_bytes] packed weight rows -> fragment order: the 16-byte
// unit ((b * tiles + t) * chunks + q) * 64 + lane holds bytes
// [q*32 + (lane/32)*16, +16) of row t*32 + lane%32; rows and bytes beyond the
// source are zero.
// The destination holds batch * tiles * chunks KiB of fragments followed by
// kWfragTailBytes bytes of `fill` (the stored byte that represents the real
// value 0 of the activation operand; padding taps fetch it).
constexpr int kWfragTailBytes = 256;
struct WfragPackParams {
  const void* src = nullptr; void* dst = nullptr;
  int batch = 1, rows = 0, row_bytes = 0, tiles = 0, chunks = 0;
  int fill = 0;
};
hipError_t launch_wfrag_pack(const WfragPackParams& p, hipStream_t stream);

// Repack a weight tensor into the [G][rows_pad][w_rs] matrix launch_igemm reads.
// src element (o, i, r, s) lives at o*so + i*si + r*sr + s*ss.
struct PackWeightsParams {
  const void* src = nullptr; void* dst = nullptr;
  DType src_dt = DT_F32, dst_dt = DT_F32;
  int G = 1, Og = 0, Cg = 0, R = 1, S = 1;  // per-group out / in channels
  int Cp = 0;                               // padded in-channels per tap (>= Cg)
  // dense_groups > 0 (with G == 1): the source holds that many groups of
  // Og / dense_groups rows with Cg / dense_groups in-channels each; the result
  // is the block-diagonal matrix of the equivalent ungrouped convolution.
  int dense_groups = 0;
  int rows_pad = 0, w_rs = 0;
  int64_t so = 0, si = 0, sr = 0, ss = 0;
};
hipError_t launch_pack_weights(const PackWeightsParams& p, hipStream_t stream);

// ---------------------------------------------------------------------------
// One-launch attention (attention.hip):
//   out[b, h] = softmax(scale * q[b, h] . k[b, h]^T + mask[b]) . v[b, h]
// q, k, v: [S][d] matrices of 16-bit elements per (batch, head), rows of d = 64
// contiguous values; S = 32, 64, 96 or 128.  mask: one row of S values per batch
// (added to every query's scores), of the operands' type or fp32, or null.
// All strides in elements.
struct AttentionParams {
  const void* q = nullptr; const void* k = nullptr; const void* v = nullptr;
  void* out = nullptr;
  const void* mask = nullptr;
  DType dt = DT_BF16;        // q, k, v, out
  DType mask_dt = DT_BF16;
  int B = 0, heads = 0, S = 0, d = 0;
  float scale = 1.f;
  int64_t q_bs = 0, q_hs = 0, q_rs = 0;   // batch / head / row strides
  int64_t k_bs = 0, k_hs = 0, k_rs = 0;
  int64_t v_bs = 0, v_hs = 0, v_rs = 0;
  int64_t o_bs = 0, o_hs = 0, o_rs = 0;
  int64_t mask_bs = 0;                    // between batches (0: one row for all)
};
// Shapes / types the kernel serves (no pointer is looked at).
bool attention_supported(const AttentionParams& p);
hipError_t launch_attention(const AttentionParams& p, hipStream_t stream);

// ---------------------------------------------------------------------------
// Layout conversion between row-major N,C,HW (any float type) and
// channels-last N,HW,cs with optional channel padding (pad lanes get `fill`).
struct LayoutParams {
  const void* src = nullptr; void* dst = nullptr;
  DType src_dt = DT_F32, dst_dt = DT_F32;
  int N = 0, C = 0, HW = 0;
  int cs = 0;          // channel stride of the channels-last side (>= C)
  // Optional affine quantisation when dst_dt == DT_I8 (to_nhwc) or
  // dequantisation when src_dt == DT_I8 (to_nchw).
  float scale = 1.f; int zp = 0;
};
hipError_t launch_nchw_to_nhwc(const LayoutParams& p, hipStream_t stream);
// NCHW [N][C<=4][H][W] -> channels-last space-to-depth [N][ceil(H/2)][ceil(W/2)][cs],
// channel (py*2 + px)*C + c = src[n][c][2hh+py][2ww+px]; missing source rows /
// columns and channels 4C..cs-1 hold the real value 0 (quantised like the rest
// when dst_dt == DT_I8).
struct S2dParams {
  const void* src = nullptr; void* dst = nullptr;
  DType src_dt = DT_F32, dst_dt = DT_F32;
  int N = 0, C = 0, H = 0, W = 0, cs = 0;
  float scale = 1.f; int zp = 0;
};
hipError_t launch_nchw_to_s2d(const S2dParams& p, hipStream_t stream);
hipError_t launch_nhwc_to_nchw(const LayoutParams& p, hipStream_t stream);

// Flat conversions -------------------------------------------------------
hipError_t launch_cast(const void* src, DType sdt, void* dst, DType ddt, int64_t n,
                       hipStream_t stream);
// q = sat(rne(x / scale[c]) + zp[c]); channel c = (i / inner) % channels.
struct QuantParams {
  const void* src = nullptr; void* dst = nullptr;
  DType src_dt = DT_F32, dst_dt = DT_U8;   // DT_I8 here means "stored q-128" of an unsigned q
  bool dst_signed = false;                 // true: saturate to [-128,127] and store as is
  const float* scale = nullptr;            // [channels]
  const int32_t* zp = nullptr;             // [channels] or null
  int64_t n = 0, inner = 1; int channels = 1;
};
hipError_t launch_quantize(const QuantParams& p, hipStream_t stream);
hipError_t launch_dequantize(const QuantParams& p, hipStream_t stream);  // src int, dst float

// ---------------------------------------------------------------------------
// Streaming element-wise kernels (flat, 16-byte vectorised).
hipError_t launch_unary(const void* x, void* y, DType dt, int64_t n, ActKind act,
                        float a, float b, hipStream_t stream);
// y = x * scale[c] + shift[c], c = (i / inner) % channels   (folded BatchNorm)
hipError_t launch_channel_affine(const void* x, void* y, DType dt, int64_t n,
                                 int64_t inner, int channels, const float* scale,
                                 const float* shift, hipStream_t stream);
// scale/shift from BatchNorm statistics, computed on the device for
// non-constant operands.  Any of gamma/beta may be null (scalars used instead).
hipError_t launch_bn_fold(const float* mean, const float* var, const float* gamma,
                          const float* beta, float sgamma, float sbeta, float eps,
                          int channels, float* scale, float* shift, hipStream_t stream);

// Binary with broadcast.  Output is described by up to 6 physical dims; each
// operand has one element stride per dim (0 where it broadcasts).
struct BinaryParams {
  const void* a = nullptr; const void* b = nullptr; void* y = nullptr;
  DType dt = DT_F32;        // all three tensors
  BinKind op = BIN_ADD;
  int rank = 1;
  int64_t dims[6] = {1, 1, 1, 1, 1, 1};
  int64_t sa[6] = {0}, sb[6] = {0};
  ActKind act = ACT_NONE; float act_a = 0.f, act_b = 0.f;
  // int8 tensors (dt == DT_I8): f = (a-a_zp)*a_scale op (b-b_zp)*b_scale;
  // q = clamp(rne(f * y_inv) + y_zp, y_lo, 255)
  float a_scale = 0.f, b_scale = 0.f, y_inv = 0.f; int a_zp = 0, b_zp = 0, y_zp = 0, y_lo = 0;
};
hipError_t launch_binary(const BinaryParams& p, hipStream_t stream);

// A connected group of float unary / binary operators run as one launch.
// Every thread evaluates the whole group for one point of the iteration space
// dims[0..3]: threads enumerate (dims[0], dims[1], pieces of dims[2], dims[3])
// with dims[3] fastest and walk their piece of dims[2] themselves, so that the
// planner can give stores a unit stride across threads and loads a unit stride
// along a thread's walk.
// The group is a short program over per-thread registers: loads and stores go
// through views (base pointer, element offset, one element stride per dim; a
// stride of 0 broadcasts), all of storage type `dt`; arithmetic is fp32.
enum FusedOp : int { FOP_LOAD = 0, FOP_UNARY, FOP_BINARY, FOP_STORE };
struct FusedView {
  const void* base = nullptr;   // stores cast the const away
  int64_t off = 0;
  int64_t st[4] = {0, 0, 0, 0};
};
struct FusedInstr {
  int op = FOP_LOAD;   // FusedOp
  int dst = 0;         // register written (FOP_STORE: view index)
  int a = 0, b = 0;    // registers read (FOP_LOAD: a = view index; FOP_BINARY: -1 = the immediate fa)
  int kind = 0;        // ActKind / BinKind
  float fa = 0.f, fb = 0.f;   // FOP_UNARY: the activation's parameters
};
constexpr int kFusedMaxRegs = 32, kFusedMaxViews = 24, kFusedMaxInstr = 64;
struct FusedParams {
  DType dt = DT_F32;
  int n_instr = 0;
  int64_t dims[4] = {1, 1, 1, 1};
  int64_t walk = 0;    // points of dims[2] per thread (0: all of them); short walks give more threads
  FusedView view[kFusedMaxViews];
  FusedInstr prog[kFusedMaxInstr];
};
hipError_t launch_fused_eltwise(const FusedParams& p, hipStream_t stream);

// Typed element-wise operators with broadcast (row-major operands, up to 6
// collapsed dims, one element stride per dim and operand, 0 where it
// broadcasts).  EW_ADD .. EW_SQDIFF: y has the operands' type `dt` (float types
// and integers).  EW_EQ .. EW_GE: operands of type dt, boolean result.
// EW_AND .. EW_NOT: boolean operands and result.  EW_ISNAN ..: float operand,
// boolean result.  EW_SELECT: y = a ? b : c with a boolean, b / c / y of type dt.
enum EwiseOp : int {
  EW_ADD = 0, EW_SUB, EW_MUL, EW_DIV, EW_MAX, EW_MIN, EW_POW,
  EW_MOD,    // a - b * floor(a / b)
  EW_FMOD,   // a - b * trunc(a / b)
  EW_PRELU,  // a < 0 ? a * b : a
  EW_SQDIFF, // (a - b)^2
  EW_SELECT,
  EW_EQ, EW_NE, EW_LT, EW_LE, EW_GT, EW_GE,
  EW_AND, EW_OR, EW_XOR, EW_NOT,
  EW_ISNAN, EW_ISINF, EW_ISINF_POS, EW_ISINF_NEG,
  EW_SHL, EW_SHR   // bit shifts of unsigned integers (logical; a shift by the width or more gives 0)
};
struct EwiseParams {
  const void* a = nullptr; const void* b = nullptr; const void* c = nullptr; void* y = nullptr;
  DType dt = DT_F32;
  EwiseOp op = EW_ADD;
  int rank = 1;
  int64_t dims[6] = {1, 1, 1, 1, 1, 1};
  int64_t sa[6] = {0}, sb[6] = {0}, sc[6] = {0};
};
hipError_t launch_ewise(const EwiseParams& p, hipStream_t stream);

// ---------------------------------------------------------------------------
// Pooling on channels-last tensors x[N][H][W][cs] -> y[N][Ho][Wo][ycs].
struct PoolParams {
  const void* x = nullptr; void* y = nullptr;
  DType dt = DT_F32;
  int N = 0, H = 0, W = 0, C = 0, cs = 0, Ho = 0, Wo = 0, ycs = 0;
  int kh = 1, kw = 1, sh = 1, sw = 1, ph = 0, pw = 0;
  bool is_max = true;
  bool count_include_pad = false;
  // int8 average pooling: q = clamp(rne(mean(q_in - zp_in) * mul) + zp_out)
  float q_mul = 1.f; int zp_in = 0, zp_out = 0;
  // filled in by launch_pool2d: magic pairs for the divisions by Wo * (C / vector) and C / vector
  unsigned row_magic = 0, cv_magic = 0;
  int row_shift = 0, cv_shift = 0;
};
hipError_t launch_pool2d(const PoolParams& p, hipStream_t stream);

// Row reductions / normalisations over a contiguous inner axis:
// x viewed as [outer][len][inner]; one result column per (outer, inner).
// RED_L1 = sum |x| + eps, RED_L2 = sqrt(sum x^2 + eps), RED_LOGSUM = log(sum x).
enum ReduceKind : int {
  RED_MEAN = 0, RED_SUM, RED_MAX, RED_MIN, RED_PROD, RED_L1, RED_L2, RED_SUMSQ, RED_LOGSUM
};
hipError_t launch_reduce(const void* x, void* y, DType in_dt, DType out_dt, int64_t outer,
                         int64_t len, int64_t inner, ReduceKind kind, hipStream_t stream,
                         float eps = 0.f);
// Index (int32 / int64) of the largest or smallest element along the middle
// axis; ties resolve to the first index, or to the last when `last` is set.
hipError_t launch_arg_extreme(const void* x, void* y, DType in_dt, DType out_dt, int64_t outer,
                              int64_t len, int64_t inner, bool is_max, bool last, hipStream_t stream);
// Mean over the middle axis of 8-bit levels (stored q-128): fp32 result
// y = ((sum q - len*zp) / len) * scale.
hipError_t launch_reduce_q8_mean(const void* x, float* y, int64_t outer, int64_t len, int64_t inner,
                                 float scale, int zp, hipStream_t stream);
// add (optional, type of x): softmax(x + add) where add holds one row of `len`
// values per add_div consecutive rows of x (an attention mask); only for
// inner == 1 and rows of at most 256 16-byte vectors.
hipError_t launch_softmax(const void* x, void* y, DType in_dt, DType out_dt, int64_t outer,
                          int64_t len, int64_t inner, bool log_softmax, hipStream_t stream,
                          const void* add = nullptr, int64_t add_div = 1);
// y = (x - mean) * rsqrt(var + eps) * gamma + beta over the last `len` elements.
// y2 (optional): a second copy of the result in y2_dt (DT_F16 / DT_BF16), written by the same
// launch - for fp32 rows that layernorm_dual_ok accepts.
hipError_t launch_layernorm(const void* x, void* y, DType dt, int64_t rows, int64_t len,
                            const float* gamma, const float* beta, float eps,
                            hipStream_t stream, void* y2 = nullptr, DType y2_dt = DT_F32);
bool layernorm_dual_ok(DType dt, int64_t len);

// ---------------------------------------------------------------------------
// Data movement.
// Generic strided copy: y (contiguous, `rank` dims) <- x with element strides.
struct StridedCopyParams {
  const void* x = nullptr; void* y = nullptr;
  int elem_size = 4;
  int rank = 1;
  int64_t dims[8] = {1, 1, 1, 1, 1, 1, 1, 1};
  int64_t sx[8] = {0};      // source strides (elements)
  int64_t sy[8] = {0};      // destination strides (elements)
  int64_t x_off = 0, y_off = 0;  // element offsets
};
hipError_t launch_strided_copy(const StridedCopyParams& p, hipStream_t stream);
// Batched 2-D transpose: y[b][c][r] = x[b][r][c], destination row pitch dst_pitch >= rows.
hipError_t launch_transpose2d(const void* x, void* y, int elem_size, int batch, int rows, int cols,
                              int dst_pitch, hipStream_t stream);
// Nearest-neighbour resize, channels-last: src index = floor(dst * in / out).
hipError_t launch_resize_nearest_nhwc(const void* x, void* y, int elem_size, int N, int H,
                                      int W, int cs, int Ho, int Wo, hipStream_t stream);
// Bilinear resize, channels-last, float types: half-pixel centres, edges clamped.
hipError_t launch_resize_linear_nhwc(const void* x, void* y, DType dt, int N, int H, int W, int cs,
                                     int Ho, int Wo, hipStream_t stream);
// Row gather: y[o][j][:] = x[o][idx[j]][:], rows of row_bytes bytes.
hipError_t launch_gather_rows(const void* x, const void* idx, DType idx_dt, void* y,
                              int64_t outer, int64_t n_src_rows, int64_t n_idx,
                              int64_t row_bytes, hipStream_t stream);
// Operators along one axis of a row-major tensor [outer][len][inner] (axis_ops.hip).
// GatherElements: y[i][j][k] = x[i][idx[i][j][k]][k] with idx [ii][ij][ik] (INT32 / INT64) and
// x [di][dj][dk], ii <= di, ik <= dk; a negative index counts from the end, one outside
// the axis is clamped into it.
hipError_t launch_gather_elements(const void* x, const void* idx, DType idx_dt, void* y, int elem_size, int64_t ii,
                                  int64_t ij, int64_t ik, int64_t di, int64_t dj, int64_t dk, hipStream_t stream);
// Running sum along the axis (fp32 accumulation; exclusive: the element itself is left out;
// reverse: from the end of the axis).
hipError_t launch_cumsum(const void* x, void* y, DType dt, int64_t outer, int64_t len, int64_t inner, bool exclusive,
                         bool reverse, hipStream_t stream);
// y[o][i][in] = 1 where i == amax[o][in], else 0 (the second half of Hardmax).
hipError_t launch_onehot_axis(const void* amax, DType idx_dt, void* y, DType dt, int64_t outer, int64_t len, int64_t inner,
                              hipStream_t stream);
// Compress: the slices x[o][j][:] with cond[j] != 0 (j < n_cond <= len), dense from the start of
// y as [outer][selected][inner]; the rest of y's n_out elements is zero.  sel: n_cond + 1 int32
// of scratch memory.
hipError_t launch_compress(const void* x, const void* cond, int n_cond, int32_t* sel, void* y, int elem_size,
                           int64_t outer, int64_t len, int64_t inner, int64_t n_out, hipStream_t stream);

hipError_t launch_fill_i32(int32_t* p, int64_t n, int32_t v, hipStream_t stream);
// Fills `bytes` (a multiple of 4) with a repeated 32-bit pattern.
hipError_t launch_fill_bytes(void* p, size_t bytes, uint32_t pattern, hipStream_t stream);

// ---------------------------------------------------------------------------
// TopK along the middle axis of x[outer][len][inner] -> vals / idxs
// [outer][K][inner], best first, equal values by ascending index.
hipError_t launch_topk(const void* x, void* vals, void* idxs, DType dt, DType idx_dt, int64_t outer,
                       int64_t len, int64_t inner, int K, bool largest, hipStream_t stream);
// Calibration statistics: part[c][s] = {min, max} of the s-th share of channel
// c of x[outer][C][inner] (fp32), s < splits, C <= 65535.
hipError_t launch_minmax_partial(const float* x, float* part, int64_t outer, int C, int64_t inner, int splits,
                                 hipStream_t stream);
// LRN across the channels of x[N][C][inner]:
// y = x / (bias + alpha / (2 half + 1) * sum_{|c'-c| <= half} x[c']^2) ^ beta
hipError_t launch_lrn(const void* x, void* y, DType dt, int64_t N, int C, int64_t inner, int half, float alpha,
                      float beta, float bias, hipStream_t stream);
// Rows of x[rows][len] normalised to zero mean / unit (biased) variance, then
// scaled by gamma[r % channels] and shifted by beta[r % channels] (scalars
// sgamma / sbeta where the vectors are null).
hipError_t launch_rownorm(const void* x, void* y, DType dt, int64_t rows, int64_t len, int channels,
                          const float* gamma, const float* beta, float sgamma, float sbeta, float eps,
                          hipStream_t stream);

// ---------------------------------------------------------------------------
// Batched NMS.  boxes [N][B][4] fp32 corners, scores [N][C][B] fp32.
// out int32 [N][max_out][3] = {image, class, box}, -1 padded.
// workspace: at least nms_workspace_bytes(N, B) bytes of device memory.
size_t nms_workspace_bytes(int N, int B);
// boxes / scores are read in their storage type (DT_F32, DT_F16 or DT_BF16).
hipError_t launch_nms(const void* boxes, DType boxes_dt, const void* scores, DType scores_dt, int N, int C, int B,
                      int max_out, float iou_thr, float score_thr, int32_t* out,
                      void* workspace, hipStream_t stream, int image_base = 0);

// YOLOv3 post-processing of one image: decode of three heads [3*(5+classes)][dim][dim]
// (fp32, channels first) into `boxes` [total][4] (y min, x min, y max, x max in
// source-image pixels) and `scores` [classes][total] (total = 3 * sum dim^2),
// then per class the reference's suppression walk: `info` [classes][capacity][5]
// rows {box, score}, zero padded, and `num` [classes] rows kept (at most capacity).
// anchors[h] = {w0, h0, w1, h1, w2, h2} in pixels of the 416 x 416 network input.
hipError_t launch_yolo_postprocess(const float* const heads[3], const int dims[3], int classes,
                                   const int anchors[3][6], const int* img_w, const int* img_h, float iou_thr,
                                   float score_thr, int capacity, float* boxes, float* scores, float* info,
                                   int* num, hipStream_t stream);

}  // namespace ohip
#endif
