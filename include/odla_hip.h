/*
 * odla_hip.h -- C ABI of libodla_hip.so, an ODLA runtime platform for one AMD
 * Instinct MI355X (gfx950).
 *
 * The library is a drop-in ODLA backend: model code emitted by the HALO
 * compiler (or any program written against the headers under ODLA/include/ODLA
 * of the reference tree) links against it in place of libodla_dnnl.so /
 * libodla_tensorrt.so.  Every type below is binary compatible with the
 * reference declaration it cites (x86-64 SysV): enumerator order, struct
 * member order and sizes are part of the ABI and must not change.
 *
 * Citations of the form  [ref: <file>:<line>]  name the reference interface a
 * declaration replaces; paths are relative to the reference tree root.
 *
 * All functions are plain C symbols with default visibility.  Control
 * functions return odla_status (ODLA_SUCCESS == 0); graph builders return an
 * odla_value handle, or NULL after logging the reason when the request is
 * malformed or unsupported.  No C++ exception crosses this boundary.
 */
#ifndef ODLA_HIP_H_
#define ODLA_HIP_H_

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------------ */
/* Scalar and handle types                [ref: ODLA/include/ODLA/odla_common.h:63-137] */
/* ------------------------------------------------------------------------ */
typedef int8_t odla_int8;
typedef int16_t odla_int16;
typedef int32_t odla_int32;
typedef int64_t odla_int64;
typedef uint8_t odla_uint8;
typedef uint16_t odla_uint16;
typedef uint32_t odla_uint32;
typedef uint64_t odla_uint64;
typedef uint16_t odla_float16;  /* IEEE binary16 bit pattern */
typedef uint16_t odla_bfloat16; /* bfloat16 bit pattern      */
typedef float odla_float32;
typedef double odla_float64;
typedef const char* odla_string;
typedef odla_uint32 odla_bool;
typedef char odla_char;
typedef size_t odla_size_t;
typedef void odla_void;

/* Element types.                          [ref: ODLA/include/ODLA/odla_common.h:102-128] */
typedef enum {
  ODLA_INT8, ODLA_INT16, ODLA_INT32, ODLA_INT64,
  ODLA_UINT8, ODLA_UINT16, ODLA_UINT32, ODLA_UINT64,
  ODLA_QINT8, ODLA_QINT16, ODLA_QINT32, ODLA_QINT64,
  ODLA_QUINT8, ODLA_QUINT16, ODLA_QUINT32, ODLA_QUINT64,
  ODLA_FLOAT16, ODLA_BFLOAT16, ODLA_FLOAT32, ODLA_FLOAT64,
  ODLA_BOOL, ODLA_STRING
} odla_element_type;

/* Status codes.                           [ref: ODLA/include/ODLA/odla_common.h:140-165] */
typedef enum {
  ODLA_SUCCESS,
  ODLA_DL_ERROR,
  ODLA_FILE_NOT_EXIST,
  ODLA_INVALID_PARAM,
  ODLA_MEM_ERROR,
  ODLA_UNSUPPORTED_DATATYPE,
  ODLA_UNSUPPORTED_DEVICE_TYPE,
  ODLA_UNSUPPORTED_OP,
  ODLA_TIMEOUT,
  ODLA_INTERNAL_LOGIC_ERR,
  ODLA_RECOVERABLE_ERR,
  ODLA_PARTITION_RESET,
  ODLA_FULL_RESET,
  ODLA_UNRECOVERABLE_ERR,
  ODLA_FAILURE
} odla_status;

/* Shapes, value types, value lists.       [ref: ODLA/include/ODLA/odla_value.h:32-80] */
#define ODLA_MAX_DIMENSION 10
#define ODLA_MAX_OUTPUTS 64

typedef struct {
  odla_element_type data_type;
  union {
    odla_int32 val_int32;
    odla_uint32 val_uint32;
    odla_int64 val_int64;
    odla_uint64 val_uint64;
    odla_float32 val_fp32;
    odla_float64 val_fp64;
    odla_string val_str;
  };
} odla_scalar_value;

typedef struct {
  odla_int32 size; /* rank; 0 = scalar, -1 = undefined */
  odla_int64 dims[ODLA_MAX_DIMENSION];
} odla_value_shape; /* 88 bytes */

typedef struct {
  odla_element_type element_type;
  odla_value_shape shape;
} odla_value_type; /* 96 bytes */

typedef struct _odla_value* odla_value;
typedef struct _odla_value_id* odla_value_id; /* NUL-terminated name, or NULL */

typedef struct {
  odla_size_t size;
  odla_value values[ODLA_MAX_OUTPUTS];
} odla_values; /* 520 bytes */

typedef struct {
  odla_size_t size;
  odla_value_id value_ids[ODLA_MAX_OUTPUTS];
} odla_value_ids;

/* Compute objects.                        [ref: ODLA/include/ODLA/odla_compute.h:34-112] */
typedef enum {
  ODLA_COMPUTE_DEFAULT, ODLA_COMPUTE_INFERENCE, ODLA_COMPUTE_TRAINING
} odla_compute_mode;

typedef enum {
  ODLA_DYNAMIC_BATCH, ODLA_MIN_BATCH_SIZE, ODLA_MAX_BATCH_SIZE,
  ODLA_OPT_BATCH_SIZE, ODLA_RUN_BATCH_SIZE, ODLA_DYNAMIC_SHAPE,
  ODLA_MIN_SHAPE, ODLA_MAX_SHAPE, ODLA_OPT_SHAPE, ODLA_DYNAMIC_VALUE,
  ODLA_MIN_VALUE, ODLA_MAX_VALUE, ODLA_OPT_VALUE,
  ODLA_BF16_MODE,        /* value: odla_bf16_mode*                           */
  ODLA_FP16_MODE,        /* value: bool*; fp16 storage, fp32 accumulate      */
  ODLA_USE_SIM_MODE, ODLA_PROCESSOR_NUM, ODLA_BATCHES_PER_STEP,
  ODLA_USE_DATA_TYPE,    /* value: odla_element_type*; ODLA_INT8/QINT8/QUINT8
                            selects the int8 plan driven by the quant table  */
  ODLA_LOAD_ENGINE_MODE, ODLA_USE_DLA_CORE,
  ODLA_QUANT_TABLE,      /* value: const odla_value_quant_info*              */
  ODLA_QUANT_TABLE_SIZE, /* value: const int*                                */
  ODLA_AGGREGATE_OPS,    /* context item, value: bool*; hipGraph replay      */
  ODLA_ENABLE_ENGINE_CACHE, ODLA_CACHE_DIR,
  ODLA_ASYNC_CALLBACK_FUNC, ODLA_ASYNC_CALLBACK_ARG
} odla_item_type;

/* Library-private computation item (no counterpart in the reference): when
 * set to true before the first context is created, every int8 Conv/Gemm whose
 * result has no quant-table entry writes its raw int32 accumulator (+ int32
 * bias) bit pattern into the 4-byte elements of its FLOAT32-typed result, so
 * that tests can compare accumulators bit for bit. */
#define ODLA_HIP_ITEM_RAW_INT32_ACC ((odla_item_type)1000)

typedef enum {
  BF16_DISABLE, BF16_ACCURACY_MODE, BF16_PERFORMACE_MODE, BF16_AUTO_MODE
} odla_bf16_mode;

typedef struct _odla_computation* odla_computation;
typedef struct _odla_executable* odla_executable;
typedef struct _odla_context* odla_context;
typedef struct _odla_item_value* odla_item_value;

/* Device objects.                         [ref: ODLA/include/ODLA/odla_device.h:33-88] */
typedef enum {
  ODLA_VENDOR_DEFAULT, ODLA_VENDOR_ALIBABA, ODLA_VENDOR_ARM,
  ODLA_VENDOR_CAMBRICON, ODLA_VENDOR_GRAPHCORE, ODLA_VENDOR_HABANA,
  ODLA_VENDOR_INTEL, ODLA_VENDOR_NVIDIA, ODLA_VENDOR_QUALCOMM
} odla_vendor_name;

typedef enum {
  ODLA_DEVICE_DEFAULT, ODLA_DEVICE_ALIBABA_HANGUANG, ODLA_DEVICE_ARM_CORTEX_M,
  ODLA_DEVICE_CAMBRICON_MLU220, ODLA_DEVICE_CAMBRICON_MLU270,
  ODLA_DEVICE_GRAPHCORE_IPU, ODLA_DEVICE_HABANA_GAUDI, ODLA_DEVICE_HABANA_GOYA,
  ODLA_DEVICE_INTEL_X86, ODLA_DEVICE_INTEL_DNNL, ODLA_DEVICE_NVIDIA_GPU,
  ODLA_DEVICE_NVIDIA_TENSORRT, ODLA_DEVICE_QUALCOMM_AIC100
} odla_device_name;

typedef enum {
  ODLA_DEVICE_INFO_ODLA_LIB_VERSION, /* string */
  ODLA_DEVICE_INFO_DEV_COUNT,        /* int32  */
  ODLA_DEVICE_INFO_DEV_INDEX,        /* int32  */
  ODLA_DEVICE_INFO_DEV_TYPE,         /* string */
  ODLA_DEVICE_INFO_DEV_UUID,         /* string */
  ODLA_DEVICE_INFO_PROCESSOR_UTIL,   /* fp32 in [0,1] */
  ODLA_DEVICE_INFO_MEMORY_UTIL,      /* fp32 in [0,1] */
  ODLA_DEVICE_INFO_TOTAL_MEMORY,     /* int64 bytes */
  ODLA_DEVICE_INFO_USED_MEMORY,      /* int64 bytes */
  ODLA_DEVICE_INFO_POWER_USAGE,      /* fp32 watt */
  ODLA_DEVICE_INFO_POWER_LIMIT,      /* fp32 watt */
  ODLA_DEVICE_INFO_DRIVER_VERSION,   /* string */
  ODLA_DEVICE_INFO_SDK_VERSION       /* string */
} odla_device_info;

typedef struct _odla_vendor* odla_vendor;
typedef struct _odla_device* odla_device;

/* Memory, logging.   [ref: ODLA/include/ODLA/odla_memory.h:33-38, odla_log.h:29-45] */
typedef enum {
  ODLA_MEMCPY_H2H, ODLA_MEMCPY_H2D, ODLA_MEMCPY_D2H, ODLA_MEMCPY_D2D
} odla_memcpy_type;

typedef enum {
  ODLA_LOG_LEVEL_OFF, ODLA_LOG_LEVEL_FATAL, ODLA_LOG_LEVEL_ERROR,
  ODLA_LOG_LEVEL_WARN, ODLA_LOG_LEVEL_INFO, ODLA_LOG_LEVEL_DEBUG,
  ODLA_LOG_LEVEL_TRACE
} odla_log_level;

typedef void (*odla_logging_func)(const char* file_name, int line,
                                  const char* func_name, odla_log_level level,
                                  const char* msg);

/* Operator attribute enums.
 * [ref: ODLA/include/ODLA/ops/odla_ops_nn.h:35-43, odla_ops_process.h:33-48] */
typedef enum {
  ODLA_CHANNELS_FIRST, /* activations N,C,spatial  */
  ODLA_CHANNELS_LAST,  /* activations N,spatial,C  */
  ODLA_SIO,            /* kernel spatial,in,out    */
  ODLA_SOI,            /* kernel spatial,out,in    */
  ODLA_OIS,            /* kernel out,in,spatial    */
  ODLA_IOS             /* kernel in,out,spatial    */
} odla_memory_layout;

typedef enum { ODLA_NEAREST, ODLA_LINEAR, ODLA_CUBIC } odla_interpolation_mode;

typedef enum {
  ODLA_ASSYMMETRIC, ODLA_HALF_PIXEL, ODLA_HALF_PIXEL_TF, ODLA_ALIGN_CORNERS
} odla_resize_coordinate_mode;

/* One record of a quantization table.  A tensor is described by one record
 * with ch_idx = -(number of channels) carrying the per-tensor scale, offset
 * (zero point) and range, optionally followed by one record per channel
 * (ch_idx = c) carrying that channel's min/max.
 * [ref: ODLA/include/ODLA/ops/odla_ops_quantization.h:33-41; writer
 *  utils/halo_pgq.py:308-332] */
typedef struct {
  odla_value_id value_id;
  int ch_idx;
  odla_float32 scale;
  odla_float32 offset;
  odla_float32 min;
  odla_float32 max;
} odla_value_quant_info; /* 32 bytes */

/* ------------------------------------------------------------------------ */
/* Computation / context / execution                                         */
/* ------------------------------------------------------------------------ */

/* Create an empty graph and make it the calling thread's current computation.
 * [ref: ODLA/include/ODLA/odla_compute.h:114-122; dnnl odla_dnnl.cc:98-105] */
odla_status odla_CreateComputation(odla_computation* computation);

/* Release the graph, its packed weights and every value handle it owns.
 * [ref: odla_compute.h:223-230; tensorrt odla_tensorrt.cc:104-113] */
odla_status odla_DestroyComputation(odla_computation computation);

/* Property bag.  Honoured: ODLA_FP16_MODE, ODLA_BF16_MODE, ODLA_USE_DATA_TYPE,
 * ODLA_QUANT_TABLE, ODLA_QUANT_TABLE_SIZE, ODLA_HIP_ITEM_RAW_INT32_ACC.  Other
 * items are accepted and ignored (ODLA_SUCCESS) so that harnesses that set
 * ODLA_USE_SIM_MODE or batch hints keep working.
 * [ref: odla_compute.h:232-241; dnnl odla_dnnl.cc:84-96; tensorrt :130-199] */
odla_status odla_SetComputationItem(odla_computation computation,
                                    odla_item_type type, odla_item_value value);

/* Create an execution context (device arena + stream + captured hipGraph)
 * for the calling thread's current computation (the most recently created one
 * when the thread has none).
 * [ref: odla_compute.h:420-427; dnnl odla_dnnl.cc:122-126; tensorrt :319-329] */
odla_status odla_CreateContext(odla_context* context);
odla_status odla_DestroyContext(odla_context context); /* [ref: odla_compute.h:440-446] */

/* Honoured: ODLA_AGGREGATE_OPS (bool*, default true: replay through hipGraph).
 * [ref: odla_compute.h:429-438; tensorrt odla_tensorrt.cc:284-317] */
odla_status odla_SetContextItem(odla_context context, odla_item_type type,
                                odla_item_value value);

/* Attach caller memory to an argument / output for the next execution.  The
 * pointer may be host memory (copied across PCIe inside Execute) or device
 * memory obtained from odla_AllocateDeviceMemory (copied on the device).
 * [ref: odla_compute.h:448-505; dnnl odla_dnnl.cc:246-303,380-407;
 *  tensorrt odla_tensorrt.cc:422-448] */
odla_status odla_BindToArgument(odla_value value, const odla_void* data_ptr,
                                odla_context context);
odla_status odla_BindToArgumentById(const odla_value_id value_id,
                                    const odla_void* data_ptr,
                                    odla_context context);
odla_status odla_BindToOutput(odla_value value, odla_void* data_ptr,
                              odla_context context);
odla_status odla_BindToOutputById(const odla_value_id value_id,
                                  odla_void* data_ptr, odla_context context);

/* Run the graph once: stage bound arguments, replay the planned launch
 * sequence, write every bound output, and return after the device is idle.
 * The sequence is replayed from a hipGraph captured at the first execution,
 * except that sequences of fewer than six launches are launched directly (a
 * replay has a fixed cost that so few launches stay below;
 * ODLA_HIP_GRAPH_MIN_STEPS in the environment sets another bound, 1 = always
 * a graph) and that a context whose ODLA_AGGREGATE_OPS item is false never
 * captures.
 * Where that is faster (a context measures during its first sixteen executions;
 * ODLA_HIP_BATCH_SPLIT in the environment: 0 = never, n = always from batch n
 * on) a graph that keeps the images' rows apart in every result runs as two
 * copies at half the batch (every argument's leading extent), side by side on
 * two streams, each on its half of the bound buffers: same buffers, same
 * results, a second pair of arenas in the context.
 * [ref: odla_compute.h:158-170; dnnl odla_dnnl.cc:133-159;
 *  tensorrt odla_tensorrt.cc:866-968] */
odla_status odla_ExecuteComputation(const odla_computation computation,
                                    const odla_context context,
                                    const odla_compute_mode mode,
                                    odla_device device);

/* Introspection used by generic harnesses.
 * [ref: odla_compute.h:184-221; dnnl odla_dnnl.cc:208-244,363-378] */
odla_status odla_GetNumOfArgsFromComputation(const odla_computation computation,
                                             odla_uint32* num_args);
odla_status odla_GetArgFromComputationByIdx(const odla_computation computation,
                                            const odla_uint32 arg_idx,
                                            odla_value* arg_value);
odla_status odla_GetNumOfOutputsFromComputation(
    const odla_computation computation, odla_uint32* num_outputs);
odla_status odla_GetOutputFromComputationByIdx(
    const odla_computation computation, const odla_uint32 output_idx,
    odla_value* output_value);
/* Dynamic batch.  A computation recorded after
 *   odla_SetComputationItem(comp, ODLA_DYNAMIC_BATCH, &true) and
 *   odla_SetComputationItem(comp, ODLA_MAX_BATCH_SIZE, &n)
 * declares its batch as a leading extent of -1 (odla_CreateArgument; -1 in the
 * output dims of odla_Reshape is inferred) and is planned at batch n.  A context
 * runs it at any batch 1..n chosen with
 *   odla_SetContextItem(ctx, ODLA_RUN_BATCH_SIZE, &bs)   or
 *   odla_SetRuntimeShape(ctx, argument, shape with the leading extent bs);
 * bound buffers then hold bs rows.  Each batch is planned on first use from a
 * copy of the recording with rescaled shapes (its own kernels, arena and
 * hipGraph); graphs that move the batch out of the leading extent (a transpose
 * of it, a reduction, slice or softmax along it) are refused with
 * ODLA_UNSUPPORTED_OP.  Only the leading extent may change at run time.
 * odla_GetRuntimeShape returns a value's shape at the context's batch.
 * [ref: ODLA/include/ODLA/odla_compute.h:275-299,532-545;
 *  ODLA/platforms/tensorrt/odla_tensorrt.cc:138-179,251-296] */
odla_status odla_SetRuntimeShape(odla_context context, odla_value value,
                                 odla_value_shape value_shape);
odla_status odla_GetRuntimeShape(odla_context context, odla_value value,
                                 odla_value_shape* value_shape_ptr);
odla_status odla_SetRuntimeValueType(odla_context context, odla_value value,
                                     odla_value_type value_type);
odla_status odla_GetRuntimeValueType(odla_context context, odla_value value,
                                     odla_value_type* value_type_ptr);

/* Values.                      [ref: ODLA/include/ODLA/odla_value.h:82-214] */
odla_status odla_GetValueType(const odla_value value,
                              odla_value_type* value_type);
odla_status odla_GetValueId(const odla_value value, odla_value_id* value_id);
odla_status odla_FindValueById(const odla_value_id value_id, odla_value* value);
odla_status odla_SetValueAsOutput(odla_value value);
odla_status odla_SetValuesAsOutput(odla_values values);
odla_status odla_SetValueAsOutputById(const odla_value_id value_id);
/* Copy the device-resident result of `value` from the last execution of
 * `context` to host memory.  With a NULL context (interpret mode) the
 * operators recorded so far are compiled - again only when the graph has
 * grown or `value` was not yet a result - and run on an internal context with
 * the data of the odla_CreateValue values; `value` then stays a result of the
 * computation.  Fails while caller-made contexts of the computation exist and
 * a recompilation would be needed.
 * [ref: odla_compute.h:556-565; dnnl odla_dnnl.cc:161-179,286-295] */
odla_status odla_GetValueData(const odla_value value, odla_void* data_ptr,
                              odla_context context);
odla_status odla_GetValueDataById(const odla_value_id value_id,
                                  odla_void* data_ptr);
/* Interpret mode: a value that carries its own data.  The pointer given to
 * odla_SetValueData is borrowed (not copied) and read at every evaluation, as
 * the reference CPU backend does; without a current computation an implicit
 * one is created.
 * [ref: ops/odla_ops_basic.h:50-52; odla_value.h:82-120;
 *  dnnl odla_dnnl.cc:74-82,225-230,276-284] */
odla_value odla_CreateValue(odla_value_type value_type,
                            const odla_value_id value_id);
odla_status odla_SetValueData(odla_value value, const odla_void* data_ptr);
odla_status odla_SetValueDataById(const odla_value_id value_id,
                                  const odla_void* data_ptr);
odla_status odla_ReleaseValue(odla_value value); /* no-op; values die with the graph */

/* Graph inputs and constants.  A constant's host data must stay valid until
 * the first context of the computation has been created; it is then resident
 * on the device.
 * [ref: ODLA/include/ODLA/ops/odla_ops_basic.h:39-75;
 *  dnnl odla_dnnl.cc:192-206,305-330] */
odla_value odla_CreateArgument(const odla_value_type value_type,
                               const odla_value_id value_id);
odla_value odla_CreateConstant(const odla_value_type value_type,
                               const odla_void* data_ptr,
                               const odla_value_id value_id);

/* ------------------------------------------------------------------------ */
/* Device, memory, logging, version                                          */
/* ------------------------------------------------------------------------ */
/* [ref: odla_device.h:118-174; tensorrt/odla_device.cc:60-200;
 *  tests/ODLA/device_test.cc:63-89] */
odla_status odla_AllocateDevice(odla_vendor vendor, odla_device_name device_name,
                                odla_int32 device_idx, odla_device* device);
odla_status odla_GetDeviceInfo(odla_device device, odla_device_info info_type,
                               odla_scalar_value* info_value);
odla_status odla_SetCurrentDevice(odla_device device);
odla_status odla_DestroyDevice(odla_device device);

/* [ref: ODLA/include/ODLA/odla_memory.h:47-87] */
odla_status odla_AllocateDeviceMemory(odla_void** dev_ptr, odla_size_t size);
odla_status odla_FreeDeviceMemory(odla_void* ptr);
odla_status odla_AllocateHostMemory(odla_void** host_ptr, odla_size_t size);
odla_status odla_FreeHostMemory(odla_void* ptr);
odla_status odla_CopyMemory(odla_void* dst, odla_void* src, odla_size_t size,
                            odla_memcpy_type type);

/* [ref: ODLA/include/ODLA/odla_log.h:47-68; platforms/common/utils.cc:21-60] */
odla_status odla_SetLogLevel(odla_log_level level);
odla_status odla_SetLogger(odla_logging_func logger);
odla_logging_func odla_GetLogger(void);

/* [ref: ODLA/include/ODLA/odla_version.h:33-43] */
const odla_char* odla_GetVersionString(void);

/* ------------------------------------------------------------------------ */
/* Graph builders.  `output_dims` may be left undefined (size <= 0 or          */
/* garbage): the library infers every result shape itself and only uses a     */
/* caller-provided shape where inference is ambiguous (Reshape, Resize).      */
/* ------------------------------------------------------------------------ */

/* 2-D cross-correlation with groups and optional bias.
 * [ref: ops/odla_ops_nn.h:213-219; dnnl odla_dnnl.cc:1014-1129] */
odla_value odla_Conv(odla_value input, odla_memory_layout input_layout,
                     odla_uint32 group, odla_value kernel,
                     odla_memory_layout kernel_layout,
                     const odla_uint32* strides, const odla_uint32* dilations,
                     const odla_uint32* paddings_front,
                     const odla_uint32* paddings_back, odla_value bias,
                     odla_value_shape output_dims, const odla_value_id value_id);

/* alpha * op(A) * op(B) + beta * C, rank 2 or batched.
 * [ref: ops/odla_ops_math.h:361-364; dnnl odla_dnnl.cc:1730-1866] */
odla_value odla_Gemm(odla_value A, odla_bool A_transpose, odla_value B,
                     odla_bool B_transpose, odla_float32 alpha,
                     odla_float32 beta, odla_value C,
                     odla_value_shape output_dims, const odla_value_id value_id);
/* [ref: ops/odla_ops_math.h:337-339] */
odla_value odla_BatchMatMul(odla_value A, odla_bool A_transpose, odla_value B,
                            odla_bool B_transpose, odla_value_shape output_dims,
                            const odla_value_id value_id);

/* Element-wise binary with numpy-style broadcast.
 * [ref: ops/odla_ops_math.h:75,228,601,643,683,968; dnnl odla_dnnl.cc:585-633,
 *  odla_dnnl.h:301-394] */
odla_value odla_Add(odla_value lhs, odla_value rhs, const odla_value_id value_id);
odla_value odla_Sub(odla_value lhs, odla_value rhs, const odla_value_id value_id);
odla_value odla_Mul(odla_value lhs, odla_value rhs, const odla_value_id value_id);
odla_value odla_Div(odla_value lhs, odla_value rhs, const odla_value_id value_id);
odla_value odla_Max(odla_value lhs, odla_value rhs, const odla_value_id value_id);
odla_value odla_Min(odla_value lhs, odla_value rhs, const odla_value_id value_id);

/* Element-wise unary.
 * [ref: ops/odla_ops_nn.h:431,586,678; ops/odla_ops_math.h:163,253,287,553,
 *  870,883,941,1009; dnnl odla_dnnl.cc:432-453,635-696,834-837,1868-1904] */
odla_value odla_Relu(odla_value input, const odla_value_id value_id);
odla_value odla_LeakyRelu(odla_value input, odla_float32 alpha,
                          const odla_value_id value_id);
odla_value odla_Sigmoid(odla_value input, const odla_value_id value_id);
odla_value odla_Tanh(odla_value input, const odla_value_id value_id);
odla_value odla_Exp(odla_value input, const odla_value_id value_id);
odla_value odla_Log(odla_value input, const odla_value_id value_id);
odla_value odla_Sqrt(odla_value input, const odla_value_id value_id);
odla_value odla_Rsqrt(odla_value input, const odla_value_id value_id);
odla_value odla_Erf(odla_value input, const odla_value_id value_id);
odla_value odla_Abs(odla_value input, const odla_value_id value_id);
odla_value odla_Neg(odla_value input, const odla_value_id value_id);
odla_value odla_Round(odla_value input, const odla_value_id value_id);
odla_value odla_Clamp(odla_value input, odla_float32 lo, odla_float32 hi,
                      const odla_value_id value_id);
odla_value odla_Gelu(odla_value input, odla_bool use_approx,
                     const odla_value_id value_id);

/* Inference batch normalisation with global statistics.
 * [ref: ops/odla_ops_nn.h:172-176; dnnl odla_dnnl.cc:1448-1524] */
odla_value odla_BatchNormalization(odla_value input,
                                   odla_memory_layout input_layout,
                                   odla_value mean, odla_value var,
                                   odla_float32 epsilon, odla_value scale,
                                   odla_value offset, odla_float32 scalar_scale,
                                   odla_float32 scalar_offset,
                                   const odla_value_id value_id);

/* Layer normalisation over the trailing axes.  The reference code generator
 * emits this call but no reference header declares it.
 * [ref: lib/target/generic_cpp/batchnorm.cc:100-113;
 *  lib/transforms/fusion.cc:296-313] */
odla_value odla_LayerNorm(odla_value input, odla_size_t axes_size,
                          const odla_int32* axes, odla_float32 epsilon,
                          odla_value scale, odla_value offset,
                          const odla_value_id value_id);

/* Pooling.  [ref: ops/odla_ops_nn.h:107-112,463-467; dnnl odla_dnnl.cc:1360-1446] */
odla_value odla_MaxPool(odla_value input, odla_memory_layout input_layout,
                        const odla_uint32* window_dims,
                        const odla_uint32* strides,
                        const odla_uint32* paddings_front,
                        const odla_uint32* paddings_back,
                        odla_value_shape output_dims,
                        const odla_value_id value_id);
odla_value odla_AveragePool(odla_value input, odla_memory_layout input_layout,
                            const odla_uint32* window_dims,
                            const odla_uint32* strides,
                            const odla_uint32* paddings_front,
                            const odla_uint32* paddings_back,
                            odla_bool padding_included,
                            odla_value_shape output_dims,
                            const odla_value_id value_id);

/* Reductions.  [ref: ops/odla_ops_math.h:742-820; dnnl odla_dnnl_statistics.cc:20-117] */
odla_value odla_ReduceMean(odla_value input, odla_size_t num_of_axes,
                           const odla_uint32* axes, odla_bool keep_dims,
                           odla_value_shape output_dims,
                           const odla_value_id value_id);
odla_value odla_ReduceSum(odla_value input, odla_size_t num_of_axes,
                          const odla_uint32* axes, odla_bool keep_dims,
                          odla_value_shape output_dims,
                          const odla_value_id value_id);
odla_value odla_ReduceMax(odla_value input, odla_size_t num_of_axes,
                          const odla_uint32* axes, odla_bool keep_dims,
                          odla_value_shape output_dims,
                          const odla_value_id value_id);

/* Softmax along one axis (negative axis = last).
 * [ref: ops/odla_ops_nn.h:440,691; dnnl odla_dnnl.cc:1628-1669] */
odla_value odla_Softmax(odla_value input, odla_int32 axis,
                        const odla_value_id value_id);
odla_value odla_LogSoftmax(odla_value input, odla_int32 axis,
                           const odla_value_id value_id);

/* Data movement.  odla_Resize: rank-4 channels-first values; ODLA_NEAREST takes
 * source index floor(dst * in / out), ODLA_LINEAR is bilinear with pixel
 * centres at half-integers and clamped edges (the coordinate mode is ignored,
 * as in the reference's oneDNN backend); ODLA_CUBIC is refused.
 * [ref: ops/odla_ops_process.h:80-84,113-116,160-163,253-256,281-284,355-359,
 *  434-437; dnnl odla_dnnl.cc:455-508,869-898,1331-1358,1526-1551,1906-1990;
 *  odla_eigen.cc:602-632] */
odla_value odla_Cast(odla_value input, odla_element_type target_type,
                     const odla_value_id value_id);
odla_value odla_Concat(odla_values inputs, odla_int32 axis,
                       odla_value_shape output_shape,
                       const odla_value_id value_id);
odla_value odla_Gather(odla_value input, odla_value indices, odla_int32 axis,
                       odla_value_shape output_dims,
                       const odla_value_id value_id);
odla_value odla_Reshape(odla_value input, odla_value_shape output_dims,
                        const odla_value_id value_id);
odla_value odla_Resize(odla_value input, odla_interpolation_mode interpolation,
                       odla_resize_coordinate_mode mode, odla_uint32 axes_mask,
                       odla_value_shape output_dims,
                       const odla_value_id value_id);
odla_value odla_Slice(odla_value input, const odla_int32* start,
                      const odla_int32* end, const odla_int32* stride,
                      odla_value_shape output_dims,
                      const odla_value_id value_id);
odla_value odla_Transpose(odla_value input, odla_value_shape permutations,
                          odla_value_shape output_dims,
                          const odla_value_id value_id);

/* Affine (de)quantisation; scale with more than one element is per-`axis`.
 * q = saturate(round_half_even(x / scale) + zero_point);  x = (q - zp) * scale.
 * [ref: ops/odla_ops_quantization.h:55-73; dnnl odla_dnnl_quantization.cc:33-90] */
odla_value odla_Quantize(odla_value input, odla_value scale,
                         odla_value zero_point, odla_int32 axis,
                         odla_element_type target_data_type,
                         const odla_value_id value_id);
odla_value odla_Dequantize(odla_value input, odla_value scale,
                           odla_value zero_point, odla_int32 axis,
                           odla_element_type target_data_type,
                           const odla_value_id value_id);

/* Batched non-maximum suppression.  boxes [N,B,4] as (y1,x1,y2,x2) corners,
 * scores [N,C,B]; result int32 [N*max_num_outputs,3] rows {image, class, box}
 * in selection order, unused rows filled with -1.  Selection rule per image:
 * each box competes with its best class score; keep score > score_threshold;
 * order by (score desc, box index asc); greedily drop a box whose IoU with an
 * already kept box is >= iou_threshold.
 * [ref: ops/odla_ops_nn.h:504-507; dnnl odla_dnnl.cc:2113-2181;
 *  dnnl_utils_avx512.h:977-1079] */
odla_value odla_NMS(odla_value boxes, odla_value scores,
                    odla_uint32 max_num_outputs, odla_float32 iou_threshold,
                    odla_float32 score_threshold,
                    odla_value_type output_value_type,
                    const odla_value_id value_id);

/* ------------------------------------------------------------------------ */
/* Wider operator surface (not used by the benchmark graphs).                 */
/* ------------------------------------------------------------------------ */

/* More element-wise unary operators on float values.
 * [ref: ops/odla_ops_math.h (ACos .. Tan, Ceil, Floor, Reciprocal, Sign),
 *  ops/odla_ops_nn.h (Elu, Selu, Celu, HardSigmoid, Softplus, Softsign,
 *  ThresholdedRelu, Shrink); dnnl odla_dnnl_unary.cc:21-306,
 *  odla_dnnl.cc:409-430,660-832,1671-1688] */
odla_value odla_Reciprocal(odla_value input, const odla_value_id value_id);
odla_value odla_Ceil(odla_value input, const odla_value_id value_id);
odla_value odla_Floor(odla_value input, const odla_value_id value_id);
odla_value odla_Sign(odla_value input, const odla_value_id value_id);
odla_value odla_Sin(odla_value input, const odla_value_id value_id);
odla_value odla_Cos(odla_value input, const odla_value_id value_id);
odla_value odla_Tan(odla_value input, const odla_value_id value_id);
odla_value odla_ASin(odla_value input, const odla_value_id value_id);
odla_value odla_ACos(odla_value input, const odla_value_id value_id);
odla_value odla_ATan(odla_value input, const odla_value_id value_id);
odla_value odla_Sinh(odla_value input, const odla_value_id value_id);
odla_value odla_Cosh(odla_value input, const odla_value_id value_id);
odla_value odla_ASinh(odla_value input, const odla_value_id value_id);
odla_value odla_ACosh(odla_value input, const odla_value_id value_id);
odla_value odla_ATanh(odla_value input, const odla_value_id value_id);
/* x > 0 ? x : alpha * (exp(x) - 1) */
odla_value odla_Elu(odla_value input, odla_float32 alpha,
                    const odla_value_id value_id);
/* gamma * elu(x, alpha) */
odla_value odla_Selu(odla_value input, odla_float32 alpha, odla_float32 gamma,
                     const odla_value_id value_id);
/* max(0, x) + min(0, alpha * (exp(x / alpha) - 1)) */
odla_value odla_Celu(odla_value input, odla_float32 alpha,
                     const odla_value_id value_id);
/* clamp(alpha * x + beta, 0, 1) */
odla_value odla_HardSigmoid(odla_value input, odla_float32 alpha,
                            odla_float32 beta, const odla_value_id value_id);
odla_value odla_Softplus(odla_value input, const odla_value_id value_id);
odla_value odla_Softsign(odla_value input, const odla_value_id value_id);
/* x > alpha ? x : 0 */
odla_value odla_ThresholdedRelu(odla_value input, odla_float32 alpha,
                                const odla_value_id value_id);
/* x > lambd ? x - bias : (x < -lambd ? x + bias : 0) */
odla_value odla_Shrink(odla_value input, odla_float32 bias, odla_float32 lambd,
                       const odla_value_id value_id);

/* Binary operators with broadcast beyond the six above; Add .. Min also accept
 * integer operands.  Mod: fmod == 1 takes the sign of the dividend (C fmod),
 * otherwise of the divisor.  PRelu: x < 0 ? x * slope : x.
 * [ref: ops/odla_ops_math.h (Pow, Mod, SquaredDifference), ops/odla_ops_nn.h
 *  (PRelu); dnnl odla_dnnl_binary.cc:21-298, odla_dnnl.cc:567-610,698-718] */
odla_value odla_Pow(odla_value base, odla_value exponent,
                    const odla_value_id value_id);
odla_value odla_Mod(odla_value lhs, odla_value rhs, odla_int64 fmod,
                    const odla_value_id value_id);
odla_value odla_SquaredDifference(odla_value lhs, odla_value rhs,
                                  const odla_value_id value_id);
odla_value odla_PRelu(odla_value input, odla_value slope,
                      const odla_value_id value_id);
/* Element-wise mean of the operands.  [ref: dnnl odla_dnnl.cc:2432-2441] */
odla_value odla_Mean(odla_values inputs, const odla_value_id value_id);

/* Comparisons (operands of one type, BOOL result), logic on BOOL values and
 * float predicates.
 * [ref: ops/odla_ops_math.h (Equal .. Xor, IsNaN, IsInf);
 *  dnnl odla_dnnl_binary.cc:40-90,222-270, odla_dnnl_unary.cc:47-60,140-160,225-238] */
odla_value odla_Equal(odla_value lhs, odla_value rhs, const odla_value_id value_id);
odla_value odla_NotEqual(odla_value lhs, odla_value rhs, const odla_value_id value_id);
odla_value odla_Less(odla_value lhs, odla_value rhs, const odla_value_id value_id);
odla_value odla_LessOrEqual(odla_value lhs, odla_value rhs, const odla_value_id value_id);
odla_value odla_Greater(odla_value lhs, odla_value rhs, const odla_value_id value_id);
odla_value odla_GreaterOrEqual(odla_value lhs, odla_value rhs, const odla_value_id value_id);
odla_value odla_And(odla_value lhs, odla_value rhs, const odla_value_id value_id);
odla_value odla_Or(odla_value lhs, odla_value rhs, const odla_value_id value_id);
odla_value odla_Xor(odla_value lhs, odla_value rhs, const odla_value_id value_id);
odla_value odla_Not(odla_value input, const odla_value_id value_id);
odla_value odla_IsNaN(odla_value input, const odla_value_id value_id);
odla_value odla_IsInf(odla_value input, odla_bool detect_pos,
                      odla_bool detect_neg, const odla_value_id value_id);
/* condition ? a : b, all three broadcast to the result shape.
 * [ref: ops/odla_ops_process.h (odla_Select); dnnl odla_dnnl.cc:2372-2430] */
odla_value odla_Select(odla_value condition, odla_value a, odla_value b,
                       odla_value_shape output_dims,
                       const odla_value_id value_id);

/* out[i][j][k] = input[i][indices[i][j][k]][k] with j the axis: `indices` (INT32 or
 * INT64) has the rank of `input` and the shape of the result.  A negative index
 * counts from the end of the axis; an index outside the axis is clamped into it
 * (the reference reads outside the tensor).
 * [ref: ops/odla_ops_process.h:187-201; dnnl odla_dnnl.cc:509-567] */
odla_value odla_GatherElements(odla_value input, odla_value indices,
                               odla_int32 axis, odla_value_shape output_dims,
                               const odla_value_id value_id);
/* Running sum along `axis`, a constant INT32 / INT64 scalar that is read when the
 * node is recorded (the reference reads it at run time).  exclusion: an element's
 * own value is left out of its sum; reverse: sums run from the end of the axis.
 * [ref: ops/odla_ops_math.h:239-241; dnnl odla_dnnl_statistics.cc:147-200] */
odla_value odla_CumSum(odla_value input, odla_value axis, odla_bool exclusion,
                       odla_bool reverse, const odla_value_id value_id);
/* 1 at the first largest element along `axis`, 0 elsewhere.
 * [ref: ops/odla_ops_nn.h:114-126; dnnl odla_dnnl.cc:1688-1727] */
odla_value odla_Hardmax(odla_value input, odla_int32 axis,
                        const odla_value_id value_id);
/* The slices of `input` along `axis` whose entry of the boolean vector `condition`
 * is set.  The result has the declared maximum shape; the selected slices are
 * packed densely from its start ([outer][selected][inner]) and the rest is zero
 * (undefined in the reference).  axis == INT_MAX: `input` is one flat axis.
 * [ref: ops/odla_ops_process.h:83-98; dnnl odla_dnnl.cc:1280-1328] */
odla_value odla_Compress(odla_value input, odla_value condition, odla_int32 axis,
                         odla_value_shape max_output_shape,
                         const odla_value_id value_id);
/* Logical bit shift of UINT8 / UINT32 / UINT64 values by `shift_amount` (same
 * type, broadcast like the binary operators); a shift by the width of the type
 * or more gives 0.  UINT16 is not a storage type of this library.
 * [ref: ops/odla_ops_math.h:863-876; dnnl odla_dnnl.cc:947-1010] */
odla_value odla_Shift(odla_value input, odla_value shift_amount,
                      odla_bool is_left_shift, const odla_value_id value_id);

/* More reductions.  L1 = sum|x| + epsilon, L2 = sqrt(sum x^2 + epsilon).
 * [ref: ops/odla_ops_math.h:657-819; dnnl odla_dnnl_statistics.cc:21-160] */
odla_value odla_ReduceMin(odla_value input, odla_size_t num_of_axes,
                          const odla_uint32* axes, odla_bool keep_dims,
                          odla_value_shape output_dims,
                          const odla_value_id value_id);
odla_value odla_ReduceProd(odla_value input, odla_size_t num_of_axes,
                           const odla_uint32* axes, odla_bool keep_dims,
                           odla_value_shape output_dims,
                           const odla_value_id value_id);
odla_value odla_ReduceL1(odla_value input, odla_size_t num_of_axes,
                         const odla_uint32* axes, odla_bool keep_dims,
                         odla_float32 epsilon, odla_value_shape output_dims,
                         const odla_value_id value_id);
odla_value odla_ReduceL2(odla_value input, odla_size_t num_of_axes,
                         const odla_uint32* axes, odla_bool keep_dims,
                         odla_float32 epsilon, odla_value_shape output_dims,
                         const odla_value_id value_id);
odla_value odla_ReduceSumSquare(odla_value input, odla_size_t num_of_axes,
                                const odla_uint32* axes, odla_bool keep_dims,
                                odla_value_shape output_dims,
                                const odla_value_id value_id);
odla_value odla_ReduceLogSum(odla_value input, odla_size_t num_of_axes,
                             const odla_uint32* axes, odla_bool keep_dims,
                             odla_value_shape output_dims,
                             const odla_value_id value_id);
odla_value odla_ReduceLogSumExp(odla_value input, odla_size_t num_of_axes,
                                const odla_uint32* axes, odla_bool keep_dims,
                                odla_value_shape output_dims,
                                const odla_value_id value_id);
/* Index of the extreme element along `axis` (INT32 or INT64); ties keep the
 * first index, or the last when return_last_index is set.
 * [ref: ops/odla_ops_math.h (ArgMax, ArgMin);
 *  dnnl odla_dnnl_statistics.cc:203-300] */
odla_value odla_ArgMax(odla_value input, odla_int32 axis, odla_bool keep_dims,
                       odla_bool return_last_index,
                       odla_value_type output_value_type,
                       const odla_value_id value_id);
odla_value odla_ArgMin(odla_value input, odla_int32 axis, odla_bool keep_dims,
                       odla_bool return_last_index,
                       odla_value_type output_value_type,
                       const odla_value_id value_id);
/* values[0] = the K best elements along `axis`, best first; values[1] =
 * their indices (INT32 or INT64).  Equal elements are ordered by ascending
 * index; `sorted` is ignored (the result is always ordered).
 * [ref: ops/odla_ops_process.h (odla_TopK); dnnl odla_dnnl.cc:2064-2111] */
odla_values odla_TopK(odla_value input, odla_uint32 K, odla_bool largest,
                      odla_bool sorted, odla_uint32 axis,
                      odla_value_type output_value_type,
                      odla_value_type output_value_index_type,
                      const odla_value_ids value_ids);
/* YOLOv3 post-processing of one image (heads [1, 3*(5+classes), dim, dim],
 * image size as two 32-bit integer scalars bound at run time): values[0] =
 * "<id>0" FLOAT32 [classes, N/169, 5] rows {y min, x min, y max, x max,
 * score} in source-image pixels, best first, zero padded; values[1] = "<id>1"
 * UINT32 [classes] rows kept.  N = boxes of the three heads.  Score threshold
 * 0.3 (>=), IoU threshold 0.45 (>), a box is compared with the box kept last
 * only, equal scores are ordered by ascending box index.  The reference leaves
 * the padding undefined and writes past N/169 rows; here a class stops there.
 * [ref: ops/odla_ops_nn.h:744-759; popart odla_ops_nn.cc:462-484,
 *  custom_ops/postprocess.cc:67-81, :139-290, custom_ops/codelets_nms.cpp:24-125;
 *  models/vision/detection/yolo/yolov3_postproc.cc:34-153 (the host version)] */
odla_values odla_PostProcess(odla_value orig_img_w, odla_value orig_img_h,
                             odla_value bb13, odla_value bb26, odla_value bb52,
                             const odla_value_id value_id);

/* Data movement.
 * [ref: ops/odla_ops_process.h:117-130 (ExpandDims = broadcast), :221-236
 *  (Pad, zero fill), :397-451 (Squeeze, Stack, Tile); dnnl odla_dnnl.cc:2183-2254] */
odla_value odla_Pad(odla_value input, const odla_uint32* padding_front,
                    const odla_uint32* padding_back,
                    odla_value_shape output_dims, const odla_value_id value_id);
odla_value odla_Tile(odla_value input, const odla_uint32* repeat,
                     odla_value_shape output_dims, const odla_value_id value_id);
odla_value odla_ExpandDims(odla_value input, odla_value_shape output_dims,
                           const odla_value_id value_id);
odla_value odla_Squeeze(odla_value input, odla_size_t num_of_axes,
                        const odla_uint32* axes, odla_value_shape output_dims,
                        const odla_value_id value_id);
odla_value odla_Stack(odla_values inputs, odla_int32 axis,
                      odla_value_shape output_shape,
                      const odla_value_id value_id);

/* Cross-channel local response normalisation:
 * y = x / (bias + alpha / window * sum_{window} x^2) ^ beta.
 * [ref: ops/odla_ops_nn.h (odla_LRN); dnnl odla_dnnl.cc:1553-1581] */
odla_value odla_LRN(odla_value input, odla_memory_layout input_layout,
                    odla_int32 window_size, odla_float32 alpha,
                    odla_float32 beta, odla_float32 bias,
                    const odla_value_id value_id);
/* Per (sample, channel) normalisation over the spatial dims (channels-first
 * input; scale / offset constants with one element per channel, or null to
 * use the scalars).
 * [ref: ops/odla_ops_nn.h (odla_InstanceNormalization);
 *  dnnl odla_dnnl.cc:1583-1626] */
odla_value odla_InstanceNormalization(
    odla_value input, odla_memory_layout input_layout, odla_float32 epsilon,
    odla_value scale, odla_value offset, odla_float32 scalar_scale,
    odla_float32 scalar_offset, const odla_value_id value_id);
/* Transposed 2-D convolution (channels-first input, constant FLOAT32 kernel,
 * dilation 1).  An output shape larger than the minimal one, by less than the
 * stride, selects the output padding.
 * [ref: ops/odla_ops_nn.h (odla_DeConv); dnnl odla_dnnl.cc:1131-1232] */
odla_value odla_DeConv(odla_value input, odla_memory_layout input_layout,
                       odla_uint32 group, odla_value kernel,
                       odla_memory_layout kernel_layout,
                       const odla_uint32* strides, const odla_uint32* dilations,
                       const odla_uint32* paddings_front,
                       const odla_uint32* paddings_back, odla_value bias,
                       odla_value_shape output_dims,
                       const odla_value_id value_id);

/* ------------------------------------------------------------------------ */
/* Stored computations and executables.  What is stored is the recorded       */
/* computation (values, constants by value, nodes, outputs, precision options */
/* and quantisation table); compiling it again is a matter of milliseconds.   */
/* Store while the constants' host data is still valid.  A loaded computation */
/* becomes the calling thread's current one and owns all its data.            */
/* ODLA_LOCATION_PATH for both directions, ODLA_LOCATION_MEMORY for loading.  */
/* [ref: odla_compute.h:80-97,123-156,338-440;                                */
/*  tensorrt/odla_tensorrt.cc:537-559,561-700,703-811]                        */
/* ------------------------------------------------------------------------ */
typedef enum {
  ODLA_LOCATION_PATH,   /* NUL-terminated file path  */
  ODLA_LOCATION_MEMORY, /* address + size of a buffer */
  ODLA_LOCATION_URI     /* not supported             */
} odla_resource_location_type;
typedef struct {
  odla_resource_location_type location_type;
  const void* location;
  odla_size_t size;
} odla_resource_location;

odla_status odla_StoreComputation(odla_resource_location location,
                                  odla_computation computation);
odla_status odla_LoadComputation(odla_resource_location location,
                                 odla_computation* computation);
/* Compiles (plans) the computation now instead of at the first
 * odla_CreateContext; the executable is a handle on the computation. */
odla_status odla_CompileComputation(const odla_computation computation,
                                    const odla_device device,
                                    odla_executable* executable);
odla_status odla_StoreExecutable(odla_resource_location location,
                                 odla_executable executable);
odla_status odla_LoadExecutable(odla_resource_location location,
                                odla_device device, odla_executable* executable);
/* = odla_ExecuteComputation on the executable's computation */
odla_status odla_LaunchExecutable(odla_executable executable,
                                  odla_context context);
odla_status odla_GetNumOfArgsFromExecutable(const odla_executable executable,
                                            odla_uint32* num_args);
odla_status odla_GetArgFromExecutableByIdx(const odla_executable executable,
                                           const odla_uint32 arg_idx,
                                           odla_value* arg_value);
odla_status odla_GetNumOfOutputsFromExecutable(const odla_executable executable,
                                               odla_uint32* num_outputs);
odla_status odla_GetOutputFromExecutableByIdx(const odla_executable executable,
                                              const odla_uint32 output_idx,
                                              odla_value* output_value);
/* Destroys the computation behind a loaded executable; a compiled one lives
 * and dies with the caller's computation. */
odla_status odla_DestroyExecutable(odla_executable executable);

/* ------------------------------------------------------------------------ */
/* Calibration profiler.  The control functions keep the names and meaning of */
/* the reference's profiler library; between StartProfiling and StopProfiling */
/* computations are compiled in fp32 with nothing fused and range statistics  */
/* behind every named FLOAT32 value (arguments and constants included), and   */
/* every execution inside StartOneRun / StopOneRun appends, per value,        */
/*   "<id>" : {"op_type", "shape", "channels", "min_value", "max_value",     */
/*             "channels_min", "channels_max"}                                */
/* to the "ProfilingResults" object of the JSON file; StopProfiling adds the  */
/* "NetworkInfo" object (the operands of every value).  Kernels of            */
/* convolutions are always profiled along their output-channel axis.  Start   */
/* profiling before the computation's first context exists.                   */
/* [ref: ODLA/platforms/odla_profiler.cc:133-285; utils/halo_pgq.py:205-239] */
/* ------------------------------------------------------------------------ */
void StartProfiling(const char* data_path); /* NULL: write to stdout */
void StartOneRun(const char* tag);
void StopOneRun(void);
void StopProfiling(void);
void EnableChannelWiseProf(void);
void SetChannelAxis(int axis); /* negative: counted from the last dim */
void SkipWeightsProfiling(bool skip);

/* ------------------------------------------------------------------------ */
/* Diagnostics (no counterpart in the reference).                            */
/* ------------------------------------------------------------------------ */
typedef struct {
  char name[64]; /* "<kernel class>:<value id>", e.g. "conv:l1b0c2.relu" */
  float ms;      /* mean duration of the launch                          */
} odla_hip_step_time;

/* Runs the compiled launch sequence of `context` un-captured `iters` times,
 * with a HIP event pair around every launch on the context's stream, and
 * reports the mean duration of each launch in plan order.  Arguments must be
 * bound.  Used by the benchmark to price kernels against their roofline. */
odla_status odla_hip_ProfileSteps(odla_context context, odla_int32 iters,
                                  odla_hip_step_time* out, odla_int32 capacity,
                                  odla_int32* count);

typedef struct {
  odla_int32 launches;        /* kernel launches of one execution              */
  odla_int32 init_launches;   /* one-time launches that prepare the constants  */
  odla_uint64 arena_bytes;    /* temporaries of one context                    */
  odla_uint64 constant_bytes; /* packed constants, shared by all contexts      */
} odla_hip_plan_summary;

/* Lowers what has been recorded in `computation` to its launch sequence on the
 * host, reports its size and discards it.  No device is touched: a build
 * machine without a GPU can check that a model compiles (unsupported operators
 * and shapes are reported exactly as odla_CreateContext would report them) and
 * how much device memory it will need.  The computation itself is unchanged
 * and can be compiled, extended or stored afterwards.  No counterpart in the
 * reference. */
odla_status odla_hip_PlanSummary(odla_computation computation, odla_hip_plan_summary* summary);

/* ------------------------------------------------------------------------ */
/* Execution without device-memory allocation.                               */
/* No counterpart in the reference.  For callers that cannot allocate device */
/* memory while they run: code under HIP graph capture, tight serving loops, */
/* harnesses that forbid hipMalloc.                                          */
/* ------------------------------------------------------------------------ */
/* Temporaries larger than this are refused (ODLA_MEM_ERROR). */
#define ODLA_HIP_STATIC_SCRATCH_BYTES (64u << 20)

/* odla_ExecuteComputation with the plan's temporaries placed in a statically
 * allocated device buffer of ODLA_HIP_STATIC_SCRATCH_BYTES (one per GPU, held
 * from the library's load to the end of the process) instead of the context's
 * arena, and the launch sequence issued directly on the context's stream (no
 * hipGraph is built).  The call performs no hipMalloc / hipFree and calls no
 * allocating library routine; bind device pointers for arguments and outputs
 * so that the copies in and out are device-to-device.  `context` comes from
 * odla_CreateContext as usual (created ahead of time; it supplies the stream
 * and the bindings) and must run the recorded batch.  Results are delivered
 * through bound outputs only (odla_GetValueData reads a context's own arena).
 * Returns ODLA_MEM_ERROR when the plan's temporaries exceed the buffer,
 * ODLA_UNSUPPORTED_OP for another run-time batch or a calibration plan.
 * All calls on one GPU share that GPU's buffer, which keeps the previous
 * call's contents (no launch relies on them): calls that overlap in time on
 * one GPU race and must be serialised by the caller. */
odla_status odla_hip_ExecuteComputationStatic(odla_computation computation,
                                              odla_context context,
                                              odla_compute_mode mode,
                                              odla_device device);

#ifdef __cplusplus
} /* extern "C" */
#endif
#endif /* ODLA_HIP_H_ */
