/*
 * glow_mi355x_host.h - flat C view of the MI355X backend's host layer
 * (glow_amd/host: MI355XBackend, MI355XFunction, MI355XDeviceManager), for
 * harnesses and tests that are not C++. The C++ classes mirror glow::Backend,
 * glow::CompiledFunction and glow::runtime::DeviceManager (reference
 * include/glow/Backend/Backend.h:67-325, include/glow/Backend/CompiledFunction.h:29-98,
 * include/glow/Backends/DeviceManager.h:47-241); this header only wraps them:
 * build a module of constants, placeholders and lowered instructions, compile
 * it, make it resident on the device, run it.
 *
 * Every int-returning function gives a non-negative result on success and
 * -(error code) on failure, where the error code is one of
 * MI355X_HOST_ERR_* (the names follow glow::ErrorValue::ErrorCode, reference
 * include/glow/Support/Error.h:292-337); mi355x_host_last_error() holds the
 * message for the calling thread.
 */
#ifndef GLOW_MI355X_HOST_H
#define GLOW_MI355X_HOST_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
  MI355X_HOST_SUCCESS = 0,
  MI355X_HOST_ERR_UNKNOWN = 1,
  MI355X_HOST_ERR_RUNTIME_ERROR = 2,
  MI355X_HOST_ERR_RUNTIME_OUT_OF_DEVICE_MEMORY = 3,
  MI355X_HOST_ERR_RUNTIME_NET_NOT_FOUND = 4,
  MI355X_HOST_ERR_RUNTIME_REQUEST_REFUSED = 5,
  MI355X_HOST_ERR_RUNTIME_DEVICE_NOT_FOUND = 6,
  MI355X_HOST_ERR_RUNTIME_DEVICE_NONRECOVERABLE = 7,
  MI355X_HOST_ERR_RUNTIME_NET_BUSY = 8,
  MI355X_HOST_ERR_DEVICE_FEATURE_NOT_SUPPORTED = 9,
  MI355X_HOST_ERR_COMPILE_UNSUPPORTED_NODE_AFTER_OPTIMIZE = 10,
  MI355X_HOST_ERR_COMPILE_CONTEXT_MALFORMED = 11
};
const char *mi355x_host_last_error(void);
const char *mi355x_host_error_name(int code);

/* glow::ElemKind subset (reference include/glow/Base/Type.h:401-433) */
enum {
  MI355X_HOST_FLOAT = 0, MI355X_HOST_FLOAT16 = 1, MI355X_HOST_INT8Q = 2,
  MI355X_HOST_INT32Q = 3, MI355X_HOST_INT32I = 4, MI355X_HOST_INT64I = 5,
  MI355X_HOST_UINT8_FUSED = 6, MI355X_HOST_UINT8_FUSED_FP16 = 7,
  MI355X_HOST_UINT4_FUSED_FP16 = 8, MI355X_HOST_UINT4_FUSED = 9,
  MI355X_HOST_BOOL = 10, MI355X_HOST_INT16Q = 11
};

/* Instruction kinds: Glow's IR instruction names (operand order of
 * tools/ClassGen/InstrGen.cpp, destination first). */
enum {
  MI355X_HOST_QUANTIZE = 0,            /* Dest, Src */
  MI355X_HOST_DEQUANTIZE = 1,          /* Dest, Src */
  MI355X_HOST_RESCALE_QUANTIZED = 2,   /* Dest, Src */
  MI355X_HOST_FULLY_CONNECTED = 3,     /* Dest, Src, Weights[K,N], Bias */
  MI355X_HOST_ROWWISE_QUANTIZED_FC = 4,/* Dest, Src, Weights[N,K], Bias, Scales, Offsets */
  MI355X_HOST_MATMUL = 5,              /* Dest, LHS, RHS */
  MI355X_HOST_CONVOLUTION = 6,         /* Dest, Src, Filter, Bias; 12 iattrs */
  MI355X_HOST_CHANNELWISE_QUANTIZED_CONV = 7, /* + FilterScales, FilterOffsets, BiasScales, BiasOffsets */
  MI355X_HOST_FRWQ_SLWS = 8,           /* Dest, Data, Weights, Indices, Lengths; iattrs {useFP16Accumulation} */
  MI355X_HOST_FRWQ_SLS = 9,            /* Dest, Data, Indices, Lengths; iattrs {useFP16Accumulation} */
  MI355X_HOST_ELEMENT_ADD = 10,        /* Dest, LHS, RHS */
  MI355X_HOST_RELU = 11,               /* Dest, Src */
  MI355X_HOST_MAX_POOL = 12,           /* Dest, Src; iattrs kernelH, kernelW, strideH, strideW, padT, padL, padB, padR */
  MI355X_HOST_AVG_POOL = 13,           /* Dest, Src; MaxPool's iattrs + countIncludePads */
  MI355X_HOST_SOFTMAX = 14,            /* Dest, Src (float, [rows x cols]) */
  MI355X_HOST_CONVERT_TO = 15,         /* Dest float, Src float16 */
  MI355X_HOST_INSERT_TENSOR = 16,      /* Dest [R,W], Src [R,w]; iattrs {inner offset} */
  MI355X_HOST_TRANSPOSE = 17,          /* Dest, Src int8; iattrs shuffle {1,0} or {0,2,1} */
  MI355X_HOST_GATHER = 18,             /* Dest, Data, Indices; iattrs {batchDims} */
  MI355X_HOST_BATCH_MATMUL = 19,       /* Dest [B,M,N], LHS [B,M,K], RHS [B,K,N] int8 */
  MI355X_HOST_SIGMOID = 20,            /* Dest, Src float */
  MI355X_HOST_RWQ_SLWS = 21,           /* Dest, Data u8, Scales, Offsets, Weights, Indices, Lengths */
  MI355X_HOST_EMBEDDING_BAG_BYTE_ROWWISE_OFFSETS = 22, /* Dest, Data, Weights, Indices, Offsets; iattrs {hasEndOffset} */
  MI355X_HOST_COPY = 23                /* Dest, Src: same bytes (CopyInst) */
};
/* Convolution iattrs: kernelH, kernelW, strideH, strideW, padT, padL, padB,
 * padR, group, dilationH, dilationW, fusedActivation (glow::FusedActivation);
 * fattrs: the float activation arguments (Clip {min,max}, LeakyRelu {alpha}). */

typedef struct mi355x_host_module mi355x_host_module;
typedef struct mi355x_host_dm mi355x_host_dm;

mi355x_host_module *mi355x_host_module_create(const char *name);
void mi355x_host_module_destroy(mi355x_host_module *m);
/* Module::createConstant / createPlaceholder; return the value id. */
int mi355x_host_add_constant(mi355x_host_module *m, const char *name, int elem_kind,
                             const int64_t *dims, int ndims, float scale, int32_t offset,
                             const void *payload);
int mi355x_host_add_placeholder(mi355x_host_module *m, const char *name, int elem_kind,
                                const int64_t *dims, int ndims, float scale, int32_t offset);
/* Module::createFunction; returns the function index. */
int mi355x_host_create_function(mi355x_host_module *m, const char *name);
/* AllocActivationInst of one function; returns the value id. */
int mi355x_host_add_activation(mi355x_host_module *m, int function, const char *name,
                               int elem_kind, const int64_t *dims, int ndims, float scale,
                               int32_t offset);
/* TensorViewInst: a value of another type over the bytes of `source` (reshape). */
int mi355x_host_add_view(mi355x_host_module *m, const char *name, int source, int elem_kind,
                         const int64_t *dims, int ndims, float scale, int32_t offset);
/* The same with the view starting `byte_offset` bytes into a placeholder or
 * constant (a slice of its outermost dimension, as TensorViewInst's offsets
 * give; reference lib/Backends/BackendUtils.cpp:600-636). */
int mi355x_host_add_view_at(mi355x_host_module *m, const char *name, int source, int elem_kind,
                            const int64_t *dims, int ndims, float scale, int32_t offset,
                            size_t byte_offset);
int mi355x_host_add_instruction(mi355x_host_module *m, int function, int kind, const char *name,
                                const int *operands, int n_operands, const int64_t *iattrs,
                                int n_iattrs, const float *fattrs, int n_fattrs);
/* Backend::isOpSupported for one would-be instruction: 1, or 0 with the
 * reason in mi355x_host_last_error(). */
int mi355x_host_is_op_supported(mi355x_host_module *m, int kind, const int *operands,
                                int n_operands, const int64_t *iattrs, int n_iattrs,
                                const float *fattrs, int n_fattrs);
/* Backend::compile of one function; the compiled function stays with the
 * module. `options` is a set of MI355X_HOST_OPT_* bits (BackendOptions). */
enum {
  MI355X_HOST_OPT_WEIGHT_ROW_SUMS = 1, /* form sum_k W[n][k] once at load time */
  MI355X_HOST_OPT_FUSE_ADD_RELU = 2,   /* ElementAdd + Relu of its result in one pass */
  MI355X_HOST_OPT_FUSE_CONV_ADD = 4,   /* convolution + ElementAdd (+ Relu) in one kernel */
  MI355X_HOST_OPT_SPACE_TO_DEPTH_STEM = 8, /* stride-2 convolutions over <= 4 channels via space-to-depth */
  MI355X_HOST_OPT_FUSE_SLS_CHAINS = 16, /* pooled lookups + ConvertTo/Quantize/InsertTensor, many tables per launch */
  MI355X_HOST_OPT_FUSE_TRANSPOSE_MATMUL = 32, /* BatchMatMul(L, Transpose(R)) reads R as it lies */
  MI355X_HOST_OPT_FUSE_FC_RELU = 64, /* RowwiseQuantizedFullyConnected + Relu in one kernel */
  MI355X_HOST_OPT_PAD_TABLE_ROWS = 128, /* constant lookup tables with rows of 33..63 bytes are copied
                                          at load time to rows 64 bytes apart */
  MI355X_HOST_OPT_FUSE_INSERT = 256, /* Gather / RescaleQuantized whose result is only inserted into a
                                        wider tensor write there directly */
  MI355X_HOST_OPT_FUSE_DEQUANTIZE_SIGMOID = 512, /* Dequantize + the Sigmoid or SoftMax of its result in one kernel */
  MI355X_HOST_OPT_DERIVE_BAG_OFFSETS = 1024, /* lookups whose lengths are an input placeholder read
                                              * their bags as positions that the device manager sums
                                              * on the host when it uploads the lengths */
  MI355X_HOST_OPT_REUSE_ACTIVATIONS = 2048, /* activations whose lives do not meet in the dependence
                                             * graph share memory (AllocationsInfo.cpp:128-156); off:
                                             * every value has bytes of its own */
  MI355X_HOST_OPT_FUSE_QUANTIZE_STEM = 4096, /* a Quantize read only by a convolution that goes
                                              * through space-to-depth is applied by that pass */
  MI355X_HOST_OPT_SPLIT_K = 8192, /* matrix-core launches with few output tiles and a long K get
                                   * a workspace in the generated region, so the kernel library
                                   * may split their K loop over workgroups */
  MI355X_HOST_OPT_DEFAULT = 16383
};
int mi355x_host_compile(mi355x_host_module *m, int function, int options);
/* Listing of the compiled function's launches and derived parameters; returns
 * the length needed (text is truncated to cap-1 bytes). */
int mi355x_host_describe(mi355x_host_module *m, int function, char *buf, size_t cap);
/* RuntimeBundle sizes: out = {constants, generated, mutable, activations}. */
int mi355x_host_bundle_sizes(mi355x_host_module *m, int function, uint64_t out[4]);

/* DeviceManager. memory_bytes 0 = what the device reports free.
 * use_launch_graphs: 0 = launch kernel by kernel; 1 = record each function as a
 * launch graph whose independent launches form parallel branches (default
 * width); n > 1 = the same with up to n branches. For n >= 1 the first nine
 * requests of a function compare its recordings with all branches, as one
 * chain and with two branches, and the fastest serves the requests after
 * them. n < 0 = exactly -n branches (-1 = a chain), nothing compared. */
mi355x_host_dm *mi355x_host_dm_create(int device, uint64_t memory_bytes, int use_launch_graphs);
/* The same with DeviceConfig::slwsMath: the arithmetic this device manager's
 * SparseLengths launches ask for with every call (MI355X_SLWS_MATH_*; -1 = the
 * library's default). Each device manager passes its own setting explicitly, so
 * several of them in one process do not influence one another. */
mi355x_host_dm *mi355x_host_dm_create_opts(int device, uint64_t memory_bytes,
                                           int use_launch_graphs, int slws_math);
void mi355x_host_dm_destroy(mi355x_host_dm *dm);
int mi355x_host_dm_init(mi355x_host_dm *dm);
int mi355x_host_dm_stop(mi355x_host_dm *dm);
/* addNetwork with every compiled function of the module; waits for the callback. */
int mi355x_host_dm_add_network(mi355x_host_dm *dm, mi355x_host_module *m);
/* addNetwork with a subset of the module's compiled functions (by function
 * index): the reference's FunctionMapTy may hold any part of a module, and the
 * rest may follow in a later call (DeviceManagerTest.cpp:573 "ReuseModule"). */
int mi355x_host_dm_add_functions(mi355x_host_dm *dm, mi355x_host_module *m, const int *functions,
                                 int n);
/* DeviceManager::transferStaticPlaceholderToDevice (reference
 * include/glow/Backends/DeviceManager.h:166-171): host bytes -> the device
 * slot of the module's placeholder `name`; blocks until copied. */
int mi355x_host_dm_transfer_static_placeholder(mi355x_host_dm *dm, mi355x_host_module *m,
                                               const char *name, void *buffer, size_t bytes);
int mi355x_host_dm_evict_network(mi355x_host_dm *dm, const char *function_name);
/* runFunction; binds n host buffers to placeholders by name (inputs are read,
 * outputs written, `bytes[i]` may be smaller than the placeholder), waits for
 * the result callback. */
int mi355x_host_dm_run(mi355x_host_dm *dm, const char *function_name, const char *const *names,
                       void *const *buffers, const size_t *bytes, int n);
/* Benchmark aid (no counterpart in the reference): replays a resident function
 * `iterations` times on the data already in its placeholders, without host
 * copies, and reports the average device milliseconds per replay. */
int mi355x_host_dm_time_function(mi355x_host_dm *dm, const char *function_name, int iterations,
                                 float *ms_per_iteration);
uint64_t mi355x_host_dm_maximum_memory(mi355x_host_dm *dm);
uint64_t mi355x_host_dm_available_memory(mi355x_host_dm *dm);

#ifdef __cplusplus
}
#endif
#endif /* GLOW_MI355X_HOST_H */
