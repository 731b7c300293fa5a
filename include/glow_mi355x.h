/*
 * glow_mi355x.h - C ABI of the MI355X (gfx950) kernel library for Glow's
 * quantized-inference hot path.
 *
 * This is the layer a glow::Backend / CompiledFunction / DeviceManager for
 * MI355X calls where Glow's CPU backend calls into libjit: one entry point
 * per lowered quantized instruction, taking DEVICE pointers, plain sizes and
 * the same integer parameters the CPU code generator derives
 * (lib/LLVMIRCodeGen/LLVMIRGen.cpp). Each entry point cites the libjit
 * function it replaces; "reference" paths are relative to the pytorch/glow
 * tree.
 *
 * Conventions
 *   - every function returns MI355X_OK (0) or a negative mi355x_status; the
 *     message of the last failure on the calling thread is
 *     mi355x_last_error().
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).
 *     Launches are asynchronous; nothing here synchronises unless it says so.
 *   - all tensors are dense, row-major, in device memory unless a parameter
 *     is documented as a host pointer.
 *   - shift amounts (pre, post) must lie in [0, 31].
 */
#ifndef GLOW_MI355X_H
#define GLOW_MI355X_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Status codes; the names follow glow::ErrorValue::ErrorCode
 * (reference include/glow/Support/Error.h:292-337) where one applies. */
typedef enum {
  MI355X_OK = 0,
  MI355X_ERR_INVALID_ARGUMENT = -1,
  MI355X_ERR_RUNTIME = -2,              /* RUNTIME_ERROR: a HIP call failed   */
  MI355X_ERR_OUT_OF_DEVICE_MEMORY = -3, /* RUNTIME_OUT_OF_DEVICE_MEMORY        */
  MI355X_ERR_NOT_SUPPORTED = -4,        /* DEVICE_FEATURE_NOT_SUPPORTED        */
  MI355X_ERR_NET_NOT_FOUND = -5,        /* RUNTIME_NET_NOT_FOUND               */
  MI355X_ERR_DEVICE_NOT_FOUND = -6,     /* RUNTIME_DEVICE_NOT_FOUND            */
  MI355X_ERR_NET_BUSY = -7              /* RUNTIME_NET_BUSY                    */
} mi355x_status;

const char *mi355x_last_error(void);

/* ---- device, memory, streams, events ------------------------------------ */
/* Replaces what CPUDeviceManager gets from the host OS: device discovery and
 * memory accounting (reference lib/Backends/CPU/CPUDeviceManager.cpp:36-63,
 * DeviceManager.h:189-204). */

typedef struct {
  char name[128];
  char arch[64];            /* e.g. "gfx950:sramecc+:xnack-" */
  int32_t compute_units;
  int32_t clock_khz;
  uint64_t total_memory;
  uint64_t free_memory;
  int32_t device;
  int32_t lds_bytes_per_block;
} mi355x_info;

int mi355x_num_devices(int *count);
/* Selects `device` for the calling thread and checks that it is a gfx950. */
int mi355x_init(int device);
int mi355x_device_info(mi355x_info *info);

int mi355x_malloc(void **dptr, size_t bytes);
int mi355x_free(void *dptr);
/* Pinned host memory for I/O buffers (DeviceManager::allocateDeviceIOBuffer,
 * reference include/glow/Backends/DeviceManager.h:122-127). */
int mi355x_host_alloc(void **hptr, size_t bytes);
int mi355x_host_free(void *hptr);
int mi355x_memcpy_h2d(void *dst, const void *src, size_t bytes, void *stream);
int mi355x_memcpy_d2h(void *dst, const void *src, size_t bytes, void *stream);
int mi355x_memcpy_d2d(void *dst, const void *src, size_t bytes, void *stream);
/* Fills with a kernel (safe inside a captured graph). */
int mi355x_fill_u8(void *dst, int value, size_t bytes, void *stream);
/* Device-to-device copy done by a kernel: a graph node with a known HBM
 * footprint (bytes read + bytes written), which is also what the hardware
 * byte counters are calibrated against. */
int mi355x_copy_u8(void *dst, const void *src, size_t bytes, void *stream);

/* Measurement aid (no counterpart in the reference): one wavefront waits
 * `micros` microseconds of the device's constant-rate clock and writes
 * out2[0] = shader-clock cycles that went by, out2[1] = constant-rate ticks
 * (mi355x_wall_clock_khz per millisecond), both uint64 in DEVICE memory. Run on
 * a second stream while a kernel runs on the first, cycles / ticks is the
 * shader clock the part holds under that kernel's power draw. */
int mi355x_shader_clock_probe(uint64_t *out2, uint32_t micros, void *stream);
int mi355x_wall_clock_khz(int *khz);

int mi355x_stream_create(void **stream);
int mi355x_stream_destroy(void *stream);
int mi355x_stream_sync(void *stream);
int mi355x_device_sync(void);
int mi355x_event_create(void **event);
int mi355x_event_destroy(void *event);
int mi355x_event_record(void *event, void *stream);
/* Work queued on `stream` after this call waits for `event`. Inside a graph
 * capture this makes `stream` a branch of the captured graph. */
int mi355x_stream_wait_event(void *stream, void *event);
int mi355x_event_sync(void *event);
int mi355x_event_elapsed_ms(void *start, void *stop, float *ms);

/* ---- per-launch options ------------------------------------------------------ */
/* Every entry point whose result bits or kernel choice can be steered has a
 * twin <name>_opts with one more argument, `const mi355x_launch_opts *opts`,
 * declared directly behind it; the options hold for that one call and nothing
 * of them outlives it, so callers on one thread or on many (two device
 * managers in a process) cannot change each other's launches. opts == NULL
 * means the calling thread's defaults, which is also what the plain entry
 * point uses. No counterpart in the reference, whose kernels have one form.
 *   struct_size   sizeof(mi355x_launch_opts) (MI355X_LAUNCH_OPTS_INIT sets it)
 *   gemm_tile     matrix-core launches (FullyConnected, MatMul, convolution):
 *                 the workgroup tile, -1 = chosen from the problem shape. Values
 *                 as listed at mi355x_gemm_tile_override. Results do not depend
 *                 on it. A tile in 6..8 or 12 names one special kernel; a launch
 *                 that kernel cannot serve fails with MI355X_ERR_NOT_SUPPORTED (a
 *                 tuner skips the candidate) instead of running another one.
 *   requant_hint  MI355X_REQUANT_* guarantees about the launch's constants, as
 *                 mi355x_gemm_requant_hint_host derives them; 0 = none. A wrong
 *                 guarantee gives wrong results, so only pass what that
 *                 function returned for this launch's own vectors.
 *   slws_math     arithmetic of the SparseLengths entry points, -1 = the
 *                 default (MI355X_SLWS_MATH_ELEMENT unless
 *                 mi355x_slws_set_fused_math changed it):
 *                 MI355X_SLWS_MATH_STRICT    acc = acc + (s*q + o)*w with every
 *                   operation rounded on its own, in bag order: the bits of a
 *                   plain (no fast-math) build of libjit.cpp:1253-1276;
 *                 MI355X_SLWS_MATH_ELEMENT   v = fma(s, q, o); acc = fma(w, v,
 *                   acc): the same expression per element without the two
 *                   intermediate roundings (three vector instructions per
 *                   element instead of five); rows of 32, 64, 128 or 256 data
 *                   bytes with fp32 accumulation, anything else runs strict;
 *                 MI355X_SLWS_MATH_REGROUPED sum_j (w_j s_j) q_jk + sum_j w_j o_j
 *                   (two instructions per element); its error is relative to
 *                   the magnitude a bag adds up, not to the result, and
 *                   exceeds 1e-5 of results that cancel: on request only.
 *   workspace, workspace_bytes   device memory the launch may use for sums that
 *                 several workgroups share (matrix-core launches whose K loop is
 *                 split over workgroups, see mi355x_gemm_splitk_workspace_bytes
 *                 for the size and the zero-fill rule); NULL = none. A caller
 *                 built before these two fields existed passes the smaller
 *                 struct_size and gets none. */
enum { MI355X_SLWS_MATH_STRICT = 0, MI355X_SLWS_MATH_ELEMENT = 1, MI355X_SLWS_MATH_REGROUPED = 2 };
typedef struct {
  uint32_t struct_size;
  int32_t gemm_tile;
  int32_t requant_hint;
  int32_t slws_math;
  void *workspace;
  uint64_t workspace_bytes;
} mi355x_launch_opts;
#define MI355X_LAUNCH_OPTS_INIT { (uint32_t)sizeof(mi355x_launch_opts), -1, 0, -1, 0, 0 }

/* ---- launch graphs ---------------------------------------------------------- */
/* A compiled function is a fixed sequence of kernel launches on fixed
 * addresses (Glow plans all memory statically), so the sequence can be
 * recorded once and replayed per inference without paying the host-side
 * launch cost of every kernel; replaces the per-instruction dispatch loop of
 * LLVMCompiledFunction::execute / jitmain (reference
 * lib/LLVMIRCodeGen/LLVMCompiledFunction.cpp:73-150). Capture needs a stream
 * made by mi355x_stream_create (not the default stream). No launch entry
 * point allocates. */
typedef struct mi355x_graph mi355x_graph;
int mi355x_graph_begin_capture(void *stream);
int mi355x_graph_end_capture(void *stream, mi355x_graph **graph);
int mi355x_graph_launch(mi355x_graph *graph, void *stream);
int mi355x_graph_destroy(mi355x_graph *graph);

/* ---- static memory plan ---------------------------------------------------- */
/* One HBM allocation per compiled function laid out as
 * constants | mutable (placeholders) | activations with the byte offsets
 * Glow's RuntimeBundle assigns (reference lib/Backend/BackendUtils.cpp:702-730,
 * RuntimeSymbolInfo BackendUtils.h:41-62); replaces the per-run host
 * allocations of LLVMCompiledFunction::execute
 * (lib/LLVMIRCodeGen/LLVMCompiledFunction.cpp:81-96). */
typedef struct mi355x_arena mi355x_arena;
enum { MI355X_REGION_CONSTANTS = 0, MI355X_REGION_MUTABLE = 1,
       MI355X_REGION_ACTIVATIONS = 2 };
int mi355x_arena_create(size_t const_bytes, size_t mutable_bytes,
                        size_t activation_bytes, mi355x_arena **arena);
int mi355x_arena_destroy(mi355x_arena *arena);
/* Device address of region base + offset (NULL and an error when outside). */
int mi355x_arena_ptr(mi355x_arena *arena, int region, size_t offset,
                     void **dptr);
int mi355x_arena_upload(mi355x_arena *arena, int region, size_t offset,
                        const void *host, size_t bytes, void *stream);
int mi355x_arena_download(mi355x_arena *arena, int region, size_t offset,
                          void *host, size_t bytes, void *stream);
uint64_t mi355x_arena_bytes(const mi355x_arena *arena);

/* ---- host-side parameter derivation (no GPU involved) ----------------------- */

/* quantization::quantizeScaleOffset32To8 (reference
 * lib/Quantization/Base/Base.cpp:234-359). out = {pre, post, scale, offset}. */
void mi355x_quantize_scale_offset_32to8(float scale, int32_t offset,
                                        int32_t out[4]);

/* quantization::Schema (reference include/glow/Quantization/Base/Base.h:217) */
enum { MI355X_SCHEMA_ASYMMETRIC = 0, MI355X_SCHEMA_SYMMETRIC = 1,
       MI355X_SCHEMA_SYMMETRIC_WITH_UNSIGNED = 2,
       MI355X_SCHEMA_SYMMETRIC_POWER2 = 3 };
/* Quantized element kinds for the range lookup (Base.cpp:361-403). */
enum { MI355X_QTY_INT8 = 8, MI355X_QTY_INT16 = 16, MI355X_QTY_INT32 = 32,
       MI355X_QTY_UINT8 = 108 };
/* quantization::chooseQuantizationParams with Calibration::None (reference
 * lib/Quantization/Base/Base.cpp:433-565). */
int mi355x_choose_quantization_params(float min, float max, int schema,
                                      int qty, float *scale, int32_t *offset);

/* quantization::specializeBiasWeightsQuantizationParams (reference
 * lib/Quantization/Base/Base.cpp:594-629): makes the bias scale equal
 * inputScale * weightsScale (adjusting the weights scale for an int32 bias whose
 * own scale is larger), offset 0 for an int32 bias. In/out: bias_scale,
 * bias_offset, weights_scale. */
int mi355x_specialize_bias_weights_qparams(float *bias_scale, int32_t *bias_offset,
                                           float input_scale, float *weights_scale,
                                           int bias_is_i32, int bias_is_zero);

/* quantization::specializeBiasQuantizationParams (reference
 * lib/Quantization/Base/Base.cpp:567-592): what the quantizer applies to the
 * bias of a Convolution or FullyConnected whose weights keep their scale
 * (lib/Quantization/Quantization.cpp:103-113). In/out: bias_scale, bias_offset. */
int mi355x_specialize_bias_qparams(float *bias_scale, int32_t *bias_offset, float input_scale,
                                   float weights_scale, int bias_is_i32, int bias_is_zero);

/* The constant preparation of Function::createChannelwiseQuantizedConv for a
 * float filter and a float bias without given parameters, int8 filter and
 * int32 bias (reference lib/Graph/Graph.cpp:3576-3700, what
 * Quantizer::enableChannelwise triggers, lib/Quantization/Quantization.cpp:762-844):
 * per output channel, filter parameters from the channel's range
 * (getTensorQuantizationParams, Base.cpp:632-691), bias parameters from the
 * channel's bias value as an Int32QTy range, both specialised by
 * specializeBiasWeightsQuantizationParams (Base.cpp:594-629), then the filter
 * and the bias quantized with them (quantizeTensor, Base.cpp:707-760).
 * HOST buffers; filter is [channels x per_channel] row-major. */
int mi355x_channelwise_quantize_conv_host(const float *filter, const float *bias,
                                          size_t channels, size_t per_channel,
                                          float input_scale, int schema, int8_t *filter_q,
                                          int32_t *bias_q, float *filter_scales,
                                          int32_t *filter_offsets, float *bias_scales,
                                          int32_t *bias_offsets);

/* Fused-rowwise element kinds (reference include/glow/Base/Type.h:424-433):
 * row = [data | scale | offset], scale/offset fp32 or fp16; 4-bit rows hold
 * two columns per byte, even column in the low nibble. */
enum { MI355X_FUSED_U8_F32 = 0, MI355X_FUSED_U8_F16 = 1,
       MI355X_FUSED_U4_F16 = 2, MI355X_FUSED_U4_F32 = 3 };
size_t mi355x_fused_row_bytes(size_t cols, int kind);
/* quantization::tensorFusedRowwiseQuantization<T> on HOST buffers (reference
 * include/glow/Quantization/Base/Base.h:598-678). */
int mi355x_fused_rowwise_quantize_host(const float *in, size_t rows,
                                       size_t cols, int kind, uint8_t *out);
/* quantization::tensorRowwiseQuantization<float,int32_t,int8_t> on HOST
 * buffers (reference Base.h:522-557): per-row parameters + int8 weights. */
int mi355x_rowwise_quantize_i8_host(const float *in, size_t rows, size_t cols,
                                    int schema, int8_t *out, float *scales,
                                    int32_t *offsets);

/* ---- elementwise ------------------------------------------------------------ */

/* libjit_element_quantize_kernel_i8 (reference
 * lib/LLVMIRCodeGen/libjit/libjit.cpp:2998-3002) over n elements. */
int mi355x_quantize_i8(int8_t *dst, const float *src, size_t n, float scale,
                       int32_t offset, void *stream);
/* libjit_element_dequantize_kernel_i8 (libjit.cpp:3016-3019). */
int mi355x_dequantize_i8(float *dst, const int8_t *src, size_t n, float scale,
                         int32_t offset, void *stream);
/* libjit_element_rescale_kernel_i8 (libjit.cpp:3031-3038). */
int mi355x_rescale_i8(int8_t *dst, const int8_t *src, size_t n,
                      int32_t out_offset, int32_t in_offset, int32_t pre,
                      int32_t post, int32_t scale, void *stream);
/* The 16- and 32-bit forms: libjit_element_quantize_kernel_i16 / _i32
 * (libjit.cpp:3004-3014; the 32-bit one does not clip),
 * libjit_element_dequantize_kernel_i16 / _i32 (libjit.cpp:3021-3029) and
 * libjit_element_rescale_kernel_i16 / _i32 (libjit.cpp:3040-3056, which run
 * libjit_scale<int64_t>: 64-bit products, result truncated to 32 bits). */
int mi355x_quantize_i16(int16_t *dst, const float *src, size_t n, float scale,
                        int32_t offset, void *stream);
int mi355x_quantize_i32(int32_t *dst, const float *src, size_t n, float scale,
                        int32_t offset, void *stream);
int mi355x_dequantize_i16(float *dst, const int16_t *src, size_t n, float scale,
                          int32_t offset, void *stream);
int mi355x_dequantize_i32(float *dst, const int32_t *src, size_t n, float scale,
                          int32_t offset, void *stream);
int mi355x_rescale_i16(int16_t *dst, const int16_t *src, size_t n,
                       int32_t out_offset, int32_t in_offset, int32_t pre,
                       int32_t post, int32_t scale, void *stream);
int mi355x_rescale_i32(int32_t *dst, const int32_t *src, size_t n,
                       int32_t out_offset, int32_t in_offset, int32_t pre,
                       int32_t post, int32_t scale, void *stream);
/* The same rescale of a [rows x cols] tensor, written as a slice of a wider
 * tensor: row r goes to dst + r*dst_row_stride (the caller adds the slice's
 * offset to dst). RescaleQuantized followed by the InsertTensor that is the
 * only reader of its result (libjit.cpp:3031-3038, then libjit_insert_tensor
 * :156-260) in one pass. */
int mi355x_rescale_rows_i8(int8_t *dst, const int8_t *src, size_t rows, size_t cols,
                           size_t dst_row_stride, int32_t out_offset, int32_t in_offset,
                           int32_t pre, int32_t post, int32_t scale, void *stream);
/* Dequantize (libjit.cpp:3016-3019) followed by Sigmoid (libjit.cpp:1913-1916)
 * of its result in one pass; the dequantized value is the same fp32 number,
 * the sigmoid agrees with the CPU to fp32 rounding of expf (1e-5 relative). */
int mi355x_dequantize_sigmoid(float *dst, const int8_t *src, size_t n, float scale,
                              int32_t offset, void *stream);
/* Dequantize (libjit.cpp:3016-3019) followed by SoftMax over the rows of its
 * result (libjit_softmax_f, libjit.cpp:3058-3082) in one pass: the dequantized
 * values are the same fp32 numbers, the rest is mi355x_softmax_f32. */
int mi355x_dequantize_softmax(float *out, const int8_t *in, size_t rows, size_t cols, float scale,
                              int32_t offset, void *stream);

/* ---- int8 glue operators ------------------------------------------------------ */

/* libjit_element_add_kernel_i8 (reference lib/LLVMIRCodeGen/libjit/libjit.cpp:
 * 1593-1603, 1675-1676) over n elements: clip(scale(lhs - lhs_offset; lhsP) +
 * scale(rhs - rhs_offset; rhsP) + dest_offset), parameters as derived in
 * LLVMIRGen.cpp:1716-1771 (lhsScale/destScale, rhsScale/destScale). */
int mi355x_add_i8(int8_t *dst, const int8_t *lhs, const int8_t *rhs, size_t n,
                  int32_t dest_offset, int32_t lhs_offset, int32_t rhs_offset,
                  int32_t lhs_pre, int32_t lhs_post, int32_t lhs_scale,
                  int32_t rhs_pre, int32_t rhs_post, int32_t rhs_scale,
                  void *stream);
/* ElementAdd followed by Relu in one pass over memory (the CPU backend stacks
 * both data-parallel instructions into one loop, LLVMIRGen.cpp:1465-1499 for
 * Relu's parameters): the sum is clipped to int8 at `sum_offset` exactly as the
 * separate add would store it, then libjit_element_relu_i8 is applied with that
 * value as its source. */
int mi355x_add_relu_i8(int8_t *dst, const int8_t *lhs, const int8_t *rhs,
                       size_t n, int32_t sum_offset, int32_t lhs_offset,
                       int32_t rhs_offset, int32_t lhs_pre, int32_t lhs_post,
                       int32_t lhs_scale, int32_t rhs_pre, int32_t rhs_post,
                       int32_t rhs_scale, int32_t dest_offset, int32_t dest_pre,
                       int32_t dest_post, int32_t dest_scale, void *stream);
/* libjit_element_relu_i8 (libjit.cpp:1851-1858): clip(scale(max(src,
 * src_offset) - src_offset; destP, dest_offset)). */
int mi355x_relu_i8(int8_t *dst, const int8_t *src, size_t n, int32_t src_offset,
                   int32_t dest_offset, int32_t dest_pre, int32_t dest_post,
                   int32_t dest_scale, void *stream);
/* libjit_element_clip_i8 (libjit.cpp:1865-1873), the un-lowered ClipInst on
 * int8: clip(scale(min(max(src, clip_min), clip_max) - src_offset; destP,
 * dest_offset)). clip_min / clip_max are the float bounds quantized with the
 * SOURCE tensor's parameters and destP = quantizeScaleOffset32To8(srcScale /
 * destScale) (LLVMIRGen.cpp:1501-1546). */
int mi355x_clip_i8(int8_t *dst, const int8_t *src, size_t n, int32_t clip_min,
                   int32_t clip_max, int32_t src_offset, int32_t dest_offset,
                   int32_t dest_pre, int32_t dest_post, int32_t dest_scale, void *stream);
/* libjit_element_leaky_relu_i8 (libjit.cpp:1880-1892), the un-lowered
 * LeakyReluInst on int8: values at or above src_offset are rescaled with posP =
 * quantizeScaleOffset32To8(srcScale / destScale), the others with negP =
 * quantizeScaleOffset32To8(srcScale * alpha / destScale) (LLVMIRGen.cpp:1549-1590);
 * clip(scale(src - src_offset; P, dest_offset)). */
int mi355x_leaky_relu_i8(int8_t *dst, const int8_t *src, size_t n, int32_t src_offset,
                         int32_t dest_offset, int32_t pos_pre, int32_t pos_post,
                         int32_t pos_scale, int32_t neg_pre, int32_t neg_post,
                         int32_t neg_scale, void *stream);
/* libjit_element_maxsplat_kernel_i8 (lib/Backends/CPU/libjit_cpu/libjit_cpu.cpp:45-46),
 * the CPU backend's CPUMaxSplatInst (Max(x, Splat(v)): a Relu that keeps its
 * input's type): max(src, value), value = v quantized with the source
 * tensor's parameters (CPULLVMIRGen.cpp:135-167). */
int mi355x_max_splat_i8(int8_t *dst, const int8_t *src, size_t n, int32_t value,
                        void *stream);
/* libjit_batchedadd_i8 / libjit_batchedadd_i32_i8 (libjit.cpp:997-1015,
 * 1945-1969), BatchedAddInst (what a FullyConnected lowers to behind its
 * MatMul): dest[n][i] = clip(scale(batch[n][i] - batch_offset; batchP, 0) +
 * scale(slice[i] - slice_offset; sliceP, 0) + dest_offset) for num_slices
 * slices of slice_size elements; slice is int8, or int32 when slice_is_i32.
 * batchP / sliceP = quantizeScaleOffset32To8(scale / destScale)
 * (LLVMIRGen.cpp:2322-2375). */
int mi355x_batched_add_i8(int8_t *dst, const int8_t *batch, const void *slice,
                          int slice_is_i32, size_t num_slices, size_t slice_size,
                          int32_t dest_offset, int32_t batch_offset, int32_t slice_offset,
                          int32_t batch_pre, int32_t batch_post, int32_t batch_scale,
                          int32_t slice_pre, int32_t slice_post, int32_t slice_scale,
                          void *stream);
/* libjit_max_pool_i8 (libjit.cpp:812-884, 2592-2597): NHWC int8, pads {top,
 * left}; a window with no valid tap yields out_offset. */
int mi355x_max_pool_i8(int8_t *out, const int8_t *in, size_t N, size_t IH,
                       size_t IW, size_t C, size_t OH, size_t OW, size_t kH,
                       size_t kW, size_t sH, size_t sW, size_t padT,
                       size_t padL, int32_t out_offset, void *stream);
/* libjit_avg_pool_i8 (libjit.cpp:2812-2880); the scale parameters are those of
 * LLVMIRGen.cpp:3003-3048 (srcScale/destScale, divided by the kernel area when
 * count_include_pads). */
int mi355x_avg_pool_i8(int8_t *out, const int8_t *in, size_t N, size_t IH,
                       size_t IW, size_t C, size_t OH, size_t OW, size_t kH,
                       size_t kW, size_t sH, size_t sW, size_t padT,
                       size_t padL, int count_include_pads, int32_t out_offset,
                       int32_t in_offset, int32_t out_pre, int32_t out_post,
                       int32_t out_scale, void *stream);
/* libjit_softmax_f (libjit.cpp:3058-3082) on fp32 [rows x cols]. The row sum is
 * reduced in parallel, so results match the CPU to fp32 rounding (1e-5
 * relative), not bit for bit. */
int mi355x_softmax_f32(float *out, const float *in, size_t rows, size_t cols,
                       void *stream);

/* ---- data movement and the small operators of ranking models ------------------ */

/* ConvertTo Float16 -> Float (exact). */
int mi355x_convert_f16_to_f32(float *dst, const void *src, size_t n, void *stream);
/* InsertTensor of a 2-D slice along the inner dimension, as Concat lowers to
 * (reference libjit_insert_tensor, libjit.cpp:156-260): for each of `rows`
 * rows, row_bytes bytes of src go to dst + r*dst_row_stride + dst_offset. */
int mi355x_insert_rows(void *dst, const void *src, size_t rows, size_t row_bytes,
                       size_t dst_row_stride, size_t dst_offset, void *stream);
/* Transpose of the two inner dimensions of [batch x rows x cols] int8. */
int mi355x_batch_transpose_i8(int8_t *dst, const int8_t *src, size_t batch, size_t rows,
                              size_t cols, void *stream);
/* libjit_gather (libjit.cpp:418-440, gather64/gather32 entry points :2083-2130):
 * dest[sample][i] = slice indices[i] of data[sample]; slices of slice_bytes
 * bytes, samples of sample_bytes bytes. Unlike the reference an index outside
 * the sample yields zeros instead of an out-of-bounds read. */
int mi355x_gather(void *dst, const void *data, const void *indices, int idx_is_64,
                  size_t num_indices, size_t slice_bytes, size_t num_samples,
                  size_t sample_bytes, void *stream);
/* The same gather with the samples of the result dst_sample_stride bytes apart
 * (Gather followed by the InsertTensor that is the only reader of its result;
 * the caller adds the slice's offset to dst). */
int mi355x_gather_rows(void *dst, const void *data, const void *indices, int idx_is_64,
                       size_t num_indices, size_t slice_bytes, size_t num_samples,
                       size_t sample_bytes, size_t dst_sample_stride, void *stream);
/* BatchMatMul of small int8 matrices, i.e. libjit_matmul_i8
 * (libjit_matmul.cpp:353-371) on every [M x K] x [K x N] pair of the batch (what
 * the node lowers to). (M + N) * K must not exceed 64 KiB. */
int mi355x_batch_matmul_i8(int8_t *out, const int8_t *lhs, const int8_t *rhs, size_t batch,
                           size_t M, size_t K, size_t N, int32_t out_offset, int32_t lhs_offset,
                           int32_t rhs_offset, int32_t out_pre, int32_t out_post,
                           int32_t out_scale, void *stream);
/* The same product with the right operand given K-contiguous, rhs_nk [N x K]
 * per sample: out = lhs x transpose(rhs_nk), i.e. BatchMatMul(lhs,
 * Transpose(rhs_nk, {0,2,1})) without materialising the transpose (the feature
 * interaction of a ranking model multiplies a matrix with its own transpose).
 * Runs on the matrix cores, one wavefront per sample. K % 16 == 0, operands
 * 16-byte aligned. Same arithmetic as libjit_matmul_i8 (libjit_matmul.cpp:353-371). */
int mi355x_batch_matmul_nt_i8(int8_t *out, const int8_t *lhs, const int8_t *rhs_nk, size_t batch,
                              size_t M, size_t K, size_t N, int32_t out_offset,
                              int32_t lhs_offset, int32_t rhs_offset, int32_t out_pre,
                              int32_t out_post, int32_t out_scale, void *stream);
/* The same product of which only chosen elements are kept: element (m, n) of
 * sample b goes to out[b*out_sample_stride + dest_of[m*N + n]] when that entry
 * of the DEVICE array dest_of[M*N] is not negative (the caller keeps the
 * entries below out_sample_stride and free of repeats). BatchMatMul followed by
 * a Gather of single elements with a constant index list (libjit_gather,
 * libjit.cpp:418-440) and possibly the InsertTensor of the gathered rows, in
 * one pass; dest_of NULL writes the whole matrix. No counterpart in the
 * reference. */
int mi355x_batch_matmul_nt_select_i8(int8_t *out, const int8_t *lhs, const int8_t *rhs_nk,
                                     size_t batch, size_t M, size_t K, size_t N,
                                     int32_t out_offset, int32_t lhs_offset, int32_t rhs_offset,
                                     int32_t out_pre, int32_t out_post, int32_t out_scale,
                                     const int32_t *dest_of, size_t out_sample_stride,
                                     void *stream);
/* Space-to-depth by 2 of a padded NHWC int8 image, the layout change that turns
 * a stride-2 convolution over few channels into a stride-1 convolution over
 * 4x the channels (SpaceToDepth with block size 2, plus padding):
 * dst[n][bh][bw][(dh*2+dw)*C + c] = src[n][2bh+dh-padT][2bw+dw-padL][c], `fill`
 * outside the image and in channels [4C, Cout). dst is [N, BH, BW, Cout]. */
int mi355x_space_to_depth2_i8(int8_t *dst, const int8_t *src, size_t N, size_t IH, size_t IW,
                              size_t C, size_t padT, size_t padL, size_t BH, size_t BW,
                              size_t Cout, int32_t fill, void *stream);
/* mi355x_quantize_i8 (libjit_quantize_kernel, libjit.cpp:1683-1698 over
 * libjit_defs.h:118-124) followed by mi355x_space_to_depth2_i8 in one pass over
 * the float image [N, IH, IW, C], C of 3 or 4 into Cout = 16: the same bytes,
 * without the int8 image in between. No counterpart in the reference. */
int mi355x_quantize_space_to_depth2_i8(int8_t *dst, const float *src, size_t N, size_t IH,
                                       size_t IW, size_t C, size_t padT, size_t padL, size_t BH,
                                       size_t BW, size_t Cout, int32_t fill, float scale,
                                       int32_t offset, void *stream);
/* libjit_sigmoid_kernel_f (libjit.cpp:1913-1916): 1 / (expf(-x) + 1); agrees
 * with the CPU to fp32 rounding of expf (1e-5 relative). */
int mi355x_sigmoid_f32(float *dst, const float *src, size_t n, void *stream);

/* ---- FullyConnected / MatMul -------------------------------------------------- */

/* sums[r] = sum over k of rows[r][k] for an int8 matrix [n_rows x K] with K
 * contiguous. The matrix-core kernels below contract raw bytes and apply the
 * operand offsets afterwards, which needs sum_k W[n][k] per output column
 * whenever the input offset is non-zero. Weights and filters are constants, so
 * a backend computes these sums once when a network is loaded and passes them
 * as `weights_row_sums` / `filter_row_sums`; with NULL there the kernels form
 * the sums on the fly at a visible cost in matrix-core utilisation. No
 * counterpart in the reference (its scalar loops subtract the offsets
 * element by element). */
int mi355x_rowsum_i8(int32_t *sums, const int8_t *rows, size_t n_rows, size_t K,
                     void *stream);

/* libjit_rowwise_quantized_fc_i8_i32 / _i8_i8 (reference
 * lib/LLVMIRCodeGen/libjit/libjit_matmul.cpp:284-316, 425-450).
 * in [M x K], weights [N x K] (not transposed), bias int32[N] or int8[N]
 * (bias_is_i8), seven int32[N] per-row parameter vectors, out int8 [M x N].
 * weights_offsets_all_zero != 0 promises that every weights_offsets[j] is 0
 * (symmetric weights), which skips the activation row sums. */
int mi355x_rwq_fc_i8(int8_t *out, const int8_t *in, const int8_t *weights,
                     const void *bias, int bias_is_i8,
                     const int32_t *weights_offsets, const int32_t *bias_pre,
                     const int32_t *bias_post, const int32_t *bias_scale,
                     const int32_t *out_pre, const int32_t *out_post,
                     const int32_t *out_scale, size_t M, size_t K, size_t N,
                     int32_t out_offset, int32_t in_offset,
                     int32_t bias_offset, int weights_offsets_all_zero,
                     const int32_t *weights_row_sums, void *stream);
int mi355x_rwq_fc_i8_opts(int8_t *out, const int8_t *in, const int8_t *weights,
                     const void *bias, int bias_is_i8,
                     const int32_t *weights_offsets, const int32_t *bias_pre,
                     const int32_t *bias_post, const int32_t *bias_scale,
                     const int32_t *out_pre, const int32_t *out_post,
                     const int32_t *out_scale, size_t M, size_t K, size_t N,
                     int32_t out_offset, int32_t in_offset,
                     int32_t bias_offset, int weights_offsets_all_zero,
                     const int32_t *weights_row_sums, void *stream,
                     const mi355x_launch_opts *opts);

/* RowwiseQuantizedFullyConnected followed by a Relu instruction of its result
 * (libjit_element_relu_i8, reference libjit.cpp:1851-1858, parameters from
 * LLVMIRGen.cpp:1465-1499) in one kernel. The FullyConnected result is
 * clipped to int8 at `fc_offset` exactly as mi355x_rwq_fc_i8 would store it;
 * then out = clip(scale(max(v, fc_offset) - fc_offset; reluP) + relu_offset)
 * with reluP = quantizeScaleOffset32To8(fcScale / reluScale). */
int mi355x_rwq_fc_relu_i8(int8_t *out, const int8_t *in, const int8_t *weights,
                          const void *bias, int bias_is_i8,
                          const int32_t *weights_offsets, const int32_t *bias_pre,
                          const int32_t *bias_post, const int32_t *bias_scale,
                          const int32_t *out_pre, const int32_t *out_post,
                          const int32_t *out_scale, size_t M, size_t K, size_t N,
                          int32_t fc_offset, int32_t in_offset, int32_t bias_offset,
                          int weights_offsets_all_zero, const int32_t *weights_row_sums,
                          int32_t relu_offset, int32_t relu_pre, int32_t relu_post,
                          int32_t relu_scale, void *stream);
int mi355x_rwq_fc_relu_i8_opts(int8_t *out, const int8_t *in, const int8_t *weights,
                          const void *bias, int bias_is_i8,
                          const int32_t *weights_offsets, const int32_t *bias_pre,
                          const int32_t *bias_post, const int32_t *bias_scale,
                          const int32_t *out_pre, const int32_t *out_post,
                          const int32_t *out_scale, size_t M, size_t K, size_t N,
                          int32_t fc_offset, int32_t in_offset, int32_t bias_offset,
                          int weights_offsets_all_zero, const int32_t *weights_row_sums,
                          int32_t relu_offset, int32_t relu_pre, int32_t relu_post,
                          int32_t relu_scale, void *stream,
                          const mi355x_launch_opts *opts);

/* libjit_fc_i8_i32 / _i8_i8 (libjit_matmul.cpp:254-280, 395-422).
 * weights_kn is [K x N] as Glow stores FullyConnected weights; the kernel
 * consumes the [N x K] transpose, which is written to `weights_nk_workspace`
 * (K*N bytes, device) when repack != 0 and read from there otherwise (weights
 * are constants: repack once at load time). weights_row_sums, if given, are
 * the row sums of that [N x K] transpose. */
int mi355x_fc_i8(int8_t *out, const int8_t *in, const int8_t *weights_kn,
                 int8_t *weights_nk_workspace, int repack, const void *bias,
                 int bias_is_i8, size_t M, size_t K, size_t N,
                 int32_t out_offset, int32_t in_offset, int32_t weights_offset,
                 int32_t bias_offset, int32_t bias_pre, int32_t bias_post,
                 int32_t bias_scale, int32_t out_pre, int32_t out_post,
                 int32_t out_scale, const int32_t *weights_row_sums,
                 void *stream);
int mi355x_fc_i8_opts(int8_t *out, const int8_t *in, const int8_t *weights_kn,
                 int8_t *weights_nk_workspace, int repack, const void *bias,
                 int bias_is_i8, size_t M, size_t K, size_t N,
                 int32_t out_offset, int32_t in_offset, int32_t weights_offset,
                 int32_t bias_offset, int32_t bias_pre, int32_t bias_post,
                 int32_t bias_scale, int32_t out_pre, int32_t out_post,
                 int32_t out_scale, const int32_t *weights_row_sums,
                 void *stream,
                 const mi355x_launch_opts *opts);

/* libjit_matmul_i8 (libjit_matmul.cpp:353-371). lhs [M x K], rhs_kn [K x N];
 * workspace and repack as for mi355x_fc_i8. */
int mi355x_matmul_i8(int8_t *out, const int8_t *lhs, const int8_t *rhs_kn,
                     int8_t *rhs_nk_workspace, int repack, size_t M, size_t K,
                     size_t N, int32_t out_offset, int32_t lhs_offset,
                     int32_t rhs_offset, int32_t out_pre, int32_t out_post,
                     int32_t out_scale, void *stream);
int mi355x_matmul_i8_opts(int8_t *out, const int8_t *lhs, const int8_t *rhs_kn,
                     int8_t *rhs_nk_workspace, int repack, size_t M, size_t K,
                     size_t N, int32_t out_offset, int32_t lhs_offset,
                     int32_t rhs_offset, int32_t out_pre, int32_t out_post,
                     int32_t out_scale, void *stream,
                     const mi355x_launch_opts *opts);

/* Tuning aid (no counterpart in the reference): forces the workgroup tile of
 * the following matrix-core launches of the calling thread: 0 = 256x256,
 * 1 = 128x128, 2 = 128x64, 3 = 64x64, 4 = 256x128, 5 = 128x256, 6 = 32x32 with
 * the K loop split over the workgroup's waves (FullyConnected forms with
 * symmetric weights, precomputed row sums and K % 32 == 0 only), 7 = the 3x3
 * stride-1 convolution over 64, 128, 256 or 512 input channels with the input
 * rows resident in LDS (tiles 0..6 keep such a convolution on the tiled
 * kernels), 8 = the streaming kernel for K of 64, 128 or 256 (FullyConnected
 * and pointwise convolutions with symmetric weights and precomputed row sums:
 * weights and constants resident in LDS, rows straight from memory into
 * registers), 9 = 128x128, 10 = 256x128 and 11 = 256x256 with eight waves per
 * workgroup instead of four, 12 = 128x128 with eight waves and the K loop
 * split over two to four workgroups per output tile, which leave their int32
 * sums in the workspace of the launch's options (what the library also picks
 * by itself when the options bring a workspace and the 128x128 grid would
 * leave half of the CUs idle; int32 sums wrap, so the order in which they are
 * added does not matter: the reference's sum, libjit_matmul.cpp:284-316);
 * -1 = chosen from the problem shape (the default). Results do not depend on
 * the tile. A tile in 6..8 or 12 names one kernel: a launch that kernel cannot
 * serve fails with MI355X_ERR_NOT_SUPPORTED. A device manager uses the tiles
 * to time the candidates of each layer once, when a network is loaded. */
int mi355x_gemm_tile_override(int tile);

/* Bytes of workspace a K-split launch of the product [M x K] x [K x N] (times
 * `groups` for a grouped convolution, M = output pixels, K = taps x channels
 * of a group, N = channels of a group) uses: with named = 0 what the library
 * would split by itself (0: it would not), with named != 0 what tile 12 needs
 * (0: K has fewer than two steps of 64). The workspace is device memory,
 * 256-byte aligned, zero-filled once before its first use (its first bytes are
 * per-tile counters, which every launch leaves zero again); launches that may
 * run at the same time need workspaces of their own. No counterpart in the
 * reference. */
int mi355x_gemm_splitk_workspace_bytes(size_t M, size_t N, size_t K, size_t groups, int named,
                                       size_t *bytes);

/* Requantisation hints (no counterpart in the reference) for the following
 * matrix-core launches of the calling thread (FullyConnected, MatMul and
 * convolution entry points); 0 = none (the default).
 *   MI355X_REQUANT_ACC24: the caller guarantees, for every output column n,
 *     that whatever the operand bytes are, the value in front of the output
 *     multiply of libjit_scale (accumulator + offset corrections + rescaled
 *     bias, shifted right by out_pre[n]) is below 2^23 in magnitude, that
 *     |out_scale[n]| < 2^23, and that product + rounding term +
 *     (out_offset << out_post[n]) stays inside 32 bits. The epilogue then
 *     requantises with one 24-bit multiply-add and one shift: the same bits in
 *     half the instruction slots.
 *   MI355X_REQUANT_NO_PRE_SHIFT (only with ACC24): every out_pre[n] is zero; the
 *     column constant is folded through the multiply as well.
 * A wrong guarantee gives wrong results, not a fault.
 * mi355x_gemm_requant_hint_host derives the flags from HOST copies of a
 * launch's parameter vectors with worst-case operand bytes (vectors of N
 * entries; w_offsets NULL = all zero; bias NULL = no bias; bias_offsets NULL =
 * bias_offset for every column). */
enum { MI355X_REQUANT_ACC24 = 1, MI355X_REQUANT_NO_PRE_SHIFT = 2 };
int mi355x_gemm_requant_hint(int flags);
int mi355x_gemm_requant_hint_host(size_t K, size_t N, int32_t in_offset, int32_t out_offset,
                                  const int32_t *w_offsets, const void *bias, int bias_is_i8,
                                  const int32_t *bias_offsets, int32_t bias_offset,
                                  const int32_t *bias_pre, const int32_t *bias_post,
                                  const int32_t *bias_scale, const int32_t *out_pre,
                                  const int32_t *out_post, const int32_t *out_scale,
                                  int *flags);

/* libjit_transpose_i8 for a 2-D tensor: dst [cols x rows] = src [rows x cols]^T */
int mi355x_transpose2d_i8(int8_t *dst, const int8_t *src, size_t rows,
                          size_t cols, void *stream);

/* libjit_transpose_i8 / _f / _u / _b (libjit.cpp:565-653, 3162-3184) for 1 to 6
 * dimensions and elements of 1, 2, 4 or 8 bytes: output dimension d is input
 * dimension shuffle[d] (in_dims and shuffle are HOST arrays of num_dims). */
int mi355x_transpose_nd(void *dst, const void *src, const size_t *in_dims,
                        const size_t *shuffle, size_t num_dims, size_t elem_size,
                        void *stream);

/* ---- Convolution -------------------------------------------------------------- */

/* NHWC input [N,IH,IW,IC], filter [OC,KH,KW,IC/group], output [N,OH,OW,OC];
 * pads are {top, left}; the output size carries bottom/right. */
typedef struct {
  int32_t N, IH, IW, IC;
  int32_t OH, OW, OC;
  int32_t KH, KW;
  int32_t strideH, strideW;
  int32_t padT, padL;
  int32_t dilH, dilW;
  int32_t group;
} mi355x_conv_geom;

/* glow::FusedActivation (reference include/glow/Graph/Nodes.h:276-283);
 * act_args are the quantized arguments emitConstQuantActivationArgs builds
 * (LLVMIRGen.cpp:618-662): CLIP {min, max}; LEAKY_RELU {pre, post, scale}. */
enum { MI355X_ACT_NONE = 0, MI355X_ACT_RELU = 1, MI355X_ACT_CLIP = 2,
       MI355X_ACT_TANH = 3, MI355X_ACT_SIGMOID = 4, MI355X_ACT_LEAKY_RELU = 5 };

/* libjit_channelwise_quantized_conv2d_i8_i32 / _i8_i8 (reference
 * lib/LLVMIRCodeGen/libjit/libjit_conv.cpp:151-239, 530-562). Eight int32[OC]
 * per-channel vectors on the device; act_args is a HOST array of 3 ints.
 * filter_row_sums (optional) = mi355x_rowsum_i8 of the filter viewed as
 * [OC x KH*KW*IC/group]. */
int mi355x_cwq_conv2d_i8(int8_t *out, const int8_t *in, const int8_t *filter,
                         const void *bias, int bias_is_i8,
                         const mi355x_conv_geom *geom, int32_t out_offset,
                         int32_t in_offset, const int32_t *filter_offsets,
                         const int32_t *bias_offsets, const int32_t *bias_pre,
                         const int32_t *bias_post, const int32_t *bias_scale,
                         const int32_t *out_pre, const int32_t *out_post,
                         const int32_t *out_scale, int32_t act_type,
                         const int32_t *act_args,
                         int filter_offsets_all_zero,
                         const int32_t *filter_row_sums, void *stream);
int mi355x_cwq_conv2d_i8_opts(int8_t *out, const int8_t *in, const int8_t *filter,
                         const void *bias, int bias_is_i8,
                         const mi355x_conv_geom *geom, int32_t out_offset,
                         int32_t in_offset, const int32_t *filter_offsets,
                         const int32_t *bias_offsets, const int32_t *bias_pre,
                         const int32_t *bias_post, const int32_t *bias_scale,
                         const int32_t *out_pre, const int32_t *out_post,
                         const int32_t *out_scale, int32_t act_type,
                         const int32_t *act_args,
                         int filter_offsets_all_zero,
                         const int32_t *filter_row_sums, void *stream,
                         const mi355x_launch_opts *opts);

/* NTHWC input [N,IT,IH,IW,IC], filter [OC,KT,KH,KW,IC/group], output
 * [N,OT,OH,OW,OC]; pads are {near, top, left}; the output size carries
 * far/bottom/right. */
typedef struct {
  int32_t N, IT, IH, IW, IC;
  int32_t OT, OH, OW, OC;
  int32_t KT, KH, KW;
  int32_t strideT, strideH, strideW;
  int32_t padN, padT, padL;
  int32_t group;
} mi355x_conv3d_geom;

/* libjit_channelwise_quantized_conv3d_i8_i32 / _i8_i8 (reference
 * lib/LLVMIRCodeGen/libjit/libjit_conv.cpp:244-349, 564-596; no dilation, as
 * there). Parameters as mi355x_cwq_conv2d_i8; the per-channel shifts must lie
 * in [0, 31]. */
int mi355x_cwq_conv3d_i8(int8_t *out, const int8_t *in, const int8_t *filter,
                         const void *bias, int bias_is_i8,
                         const mi355x_conv3d_geom *geom, int32_t out_offset,
                         int32_t in_offset, const int32_t *filter_offsets,
                         const int32_t *bias_offsets, const int32_t *bias_pre,
                         const int32_t *bias_post, const int32_t *bias_scale,
                         const int32_t *out_pre, const int32_t *out_post,
                         const int32_t *out_scale, int32_t act_type,
                         const int32_t *act_args, void *stream);

/* ChannelwiseQuantizedConvolution whose result feeds an ElementAdd with a
 * residual tensor of the output's shape, optionally followed by Relu: the
 * three instructions in one kernel. The convolution result is clipped to int8
 * at `conv_offset` exactly as mi355x_cwq_conv2d_i8 would store it; then
 * libjit_element_add_kernel_i8 (libjit.cpp:1593-1603) with that value and
 * residual[i], and, when add->relu, libjit_element_relu_i8 (libjit.cpp:1851-1858)
 * are applied while the tile is written. `out` receives the final tensor. */
typedef struct {
  int32_t sum_offset;                              /* ElementAdd's destination offset */
  int32_t residual_offset;
  int32_t conv_pre, conv_post, conv_scale;         /* convScale / sumScale */
  int32_t residual_pre, residual_post, residual_scale; /* residualScale / sumScale */
  int32_t relu;                                    /* 0: store the sum */
  int32_t dest_offset, dest_pre, dest_post, dest_scale; /* Relu: sumScale / destScale */
} mi355x_fused_add;
int mi355x_cwq_conv2d_add_i8(
    int8_t *out, const int8_t *in, const int8_t *filter, const void *bias,
    int bias_is_i8, const mi355x_conv_geom *geom, int32_t conv_offset,
    int32_t in_offset, const int32_t *filter_offsets,
    const int32_t *bias_offsets, const int32_t *bias_pre,
    const int32_t *bias_post, const int32_t *bias_scale, const int32_t *out_pre,
    const int32_t *out_post, const int32_t *out_scale, int32_t act_type,
    const int32_t *act_args, int filter_offsets_all_zero,
    const int32_t *filter_row_sums, const int8_t *residual,
    const mi355x_fused_add *add, void *stream);
int mi355x_cwq_conv2d_add_i8_opts(
    int8_t *out, const int8_t *in, const int8_t *filter, const void *bias,
    int bias_is_i8, const mi355x_conv_geom *geom, int32_t conv_offset,
    int32_t in_offset, const int32_t *filter_offsets,
    const int32_t *bias_offsets, const int32_t *bias_pre,
    const int32_t *bias_post, const int32_t *bias_scale, const int32_t *out_pre,
    const int32_t *out_post, const int32_t *out_scale, int32_t act_type,
    const int32_t *act_args, int filter_offsets_all_zero,
    const int32_t *filter_row_sums, const int8_t *residual,
    const mi355x_fused_add *add, void *stream,
    const mi355x_launch_opts *opts);

/* libjit_conv2d_i8_i32 / _i8_i8 (libjit_conv.cpp:49-147, 496-528). */
int mi355x_conv2d_i8(int8_t *out, const int8_t *in, const int8_t *filter,
                     const void *bias, int bias_is_i8,
                     const mi355x_conv_geom *geom, int32_t out_offset,
                     int32_t in_offset, int32_t filter_offset,
                     int32_t bias_offset, int32_t bias_pre, int32_t bias_post,
                     int32_t bias_scale, int32_t out_pre, int32_t out_post,
                     int32_t out_scale, int32_t act_type,
                     const int32_t *act_args, const int32_t *filter_row_sums,
                     void *stream);
int mi355x_conv2d_i8_opts(int8_t *out, const int8_t *in, const int8_t *filter,
                     const void *bias, int bias_is_i8,
                     const mi355x_conv_geom *geom, int32_t out_offset,
                     int32_t in_offset, int32_t filter_offset,
                     int32_t bias_offset, int32_t bias_pre, int32_t bias_post,
                     int32_t bias_scale, int32_t out_pre, int32_t out_post,
                     int32_t out_scale, int32_t act_type,
                     const int32_t *act_args, const int32_t *filter_row_sums,
                     void *stream,
                     const mi355x_launch_opts *opts);

/* ---- fused-rowwise SparseLengths(Weighted)Sum ----------------------------------- */

/* libjit_fused_rowwise_quantized_sparse_lengths_weighted_sum_f_u / _f_i32
 * (reference lib/LLVMIRCodeGen/libjit/libjit.cpp:1253-1276, 2416-2428) for
 * MI355X_FUSED_U8_F32 with fp32 weights and output, and the Interpreter's
 * fwdFusedRowwiseQuantizedSparseLengthsWeightedSumImpl (reference
 * lib/Backends/Interpreter/InterpreterNodes.cpp:5764-5889) for the other
 * kinds, fp16 weights/output and fp16 accumulation.
 *   dest     [segments x out_line_size] fp32, or fp16 when out_is_f16
 *   data     [data_rows x in_line_size] fused rows; in_line_size is the distance
 *            between rows and may exceed the fused row's own size (quantized
 *            bytes of out_line_size columns, then scale and offset): a table
 *            re-laid with padded rows, e.g. 36-byte rows 64 bytes apart so
 *            that a lookup touches one 64-byte piece of memory instead of 1.5
 *   weights  fp32 (or fp16 when weights_are_f16); NULL = all ones
 *            (FusedRowwiseQuantizedSparseLengthsSum, Lower.cpp:1590-1606)
 *   indices  int64 when idx_is_64 else int32, num_indices entries of which
 *            the first sum(lengths) are used
 *   lengths  int32[segments]
 * Every output row is written (empty bags give zeros). Unlike the reference,
 * an index outside [0, data_rows) or a position beyond num_indices is skipped
 * instead of read. */
int mi355x_frwq_slws(void *dest, int out_is_f16, const uint8_t *data,
                     size_t data_rows, int kind, const void *weights,
                     int weights_are_f16, const void *indices, int idx_is_64,
                     size_t num_indices, const int32_t *lengths,
                     size_t segments, size_t in_line_size,
                     size_t out_line_size, int fp16_accum, void *stream);
int mi355x_frwq_slws_opts(void *dest, int out_is_f16, const uint8_t *data,
                     size_t data_rows, int kind, const void *weights,
                     int weights_are_f16, const void *indices, int idx_is_64,
                     size_t num_indices, const int32_t *lengths,
                     size_t segments, size_t in_line_size,
                     size_t out_line_size, int fp16_accum, void *stream,
                     const mi355x_launch_opts *opts);

/* mi355x_frwq_slws with the bags given as positions instead of lengths: the
 * same operator (libjit.cpp:1253-1276; InterpreterNodes.cpp:5764-5889) for a
 * caller that holds the lengths on the host anyway (a device manager about to
 * upload them) and hands their exclusive prefix sums along. bag_offsets has
 * segments + 1 entries, bag i covering index positions
 * [bag_offsets[i], bag_offsets[i + 1]); with the vector that
 * mi355x_slws_bag_offsets_host makes of `lengths` the result is bit for bit
 * that of mi355x_frwq_slws(lengths). A bag then reads its two ends instead of
 * summing the lengths in front of it: no scratch, one launch for any number
 * of bags. Ends outside [0, num_indices] or decreasing give short or empty
 * bags, never a read outside the index list. */
int mi355x_frwq_slws_offsets(void *dest, int out_is_f16, const uint8_t *data,
                             size_t data_rows, int kind, const void *weights,
                             int weights_are_f16, const void *indices, int idx_is_64,
                             size_t num_indices, const int32_t *bag_offsets,
                             size_t segments, size_t in_line_size,
                             size_t out_line_size, int fp16_accum, void *stream);
int mi355x_frwq_slws_offsets_opts(void *dest, int out_is_f16, const uint8_t *data,
                             size_t data_rows, int kind, const void *weights,
                             int weights_are_f16, const void *indices, int idx_is_64,
                             size_t num_indices, const int32_t *bag_offsets,
                             size_t segments, size_t in_line_size,
                             size_t out_line_size, int fp16_accum, void *stream,
                             const mi355x_launch_opts *opts);

/* Host side, no GPU call: bag_offsets[0] = 0, bag_offsets[i + 1] =
 * bag_offsets[i] + max(lengths[i], 0) (negative lengths count as empty bags,
 * as in the kernels). Fails with MI355X_ERR_INVALID_ARGUMENT when the sum does
 * not fit int32; such batches go through mi355x_frwq_slws. */
int mi355x_slws_bag_offsets_host(const int32_t *lengths, size_t segments,
                                 int32_t *bag_offsets);

/* Scratch of the lengths-mode SparseLengths entry points (mi355x_frwq_slws,
 * mi355x_rwq_slws). With more than 4096 bags a small pre-pass sums the lengths
 * of each 4096-bag chunk into a 256 KiB buffer that belongs to the (device,
 * stream) pair of the launch: launches on one stream are ordered and share it,
 * launches on different streams never do. mi355x_init gives the device's
 * default stream its buffer, mi355x_stream_create every stream it makes; a
 * stream made elsewhere is registered here once (this call allocates, launches
 * do not; a launch with more than 4096 bags on an unregistered stream fails
 * with MI355X_ERR_INVALID_ARGUMENT). No counterpart in the reference. */
int mi355x_slws_reserve_stream(void *stream);

/* mi355x_frwq_slws for callers that cannot allocate device memory at all (code
 * under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc): same arguments, same kernels, same results, but the scratch of
 * the bag-offset pre-pass is a fixed 32 KiB array inside the library's code
 * object (one copy per GPU, held until the process ends) instead of a
 * per-stream buffer, so neither this call nor any set-up it needs calls
 * hipMalloc or hipFree. At most 4096 * 4096 = 16 777 216 bags per call (more
 * is MI355X_ERR_INVALID_ARGUMENT). All calls on one GPU share the array: calls
 * that overlap in time on one GPU (different streams) race on it when either
 * has more than 4096 bags; calls on one stream are ordered and safe. Nothing
 * in the array has to start at zero: the pre-pass writes every entry the
 * lookup reads. No counterpart in the reference. */
int mi355x_frwq_slws_noalloc(void *dest, int out_is_f16, const uint8_t *data,
                             size_t data_rows, int kind, const void *weights,
                             int weights_are_f16, const void *indices, int idx_is_64,
                             size_t num_indices, const int32_t *lengths,
                             size_t segments, size_t in_line_size,
                             size_t out_line_size, int fp16_accum, void *stream);
int mi355x_frwq_slws_noalloc_opts(void *dest, int out_is_f16, const uint8_t *data,
                             size_t data_rows, int kind, const void *weights,
                             int weights_are_f16, const void *indices, int idx_is_64,
                             size_t num_indices, const int32_t *lengths,
                             size_t segments, size_t in_line_size,
                             size_t out_line_size, int fp16_accum, void *stream,
                             const mi355x_launch_opts *opts);

/* Process-wide default of mi355x_launch_opts::slws_math for the calls that do
 * not name an arithmetic themselves (the plain entry points, and _opts calls
 * with slws_math = -1): MI355X_SLWS_MATH_STRICT, _ELEMENT (what the library
 * starts with) or _REGROUPED. Kept for tools that time or test one arithmetic
 * across many calls; a caller that shares the process passes slws_math with
 * its calls instead. No counterpart in the reference. */
int mi355x_slws_set_fused_math(int math);

/* Measurement aid (no counterpart in the reference): the uint8 / fp32
 * SparseLengthsWeightedSum over rows of 128 columns (int64 indices, fp32
 * weights, lengths), cut off behind one of its dependent stages, to time what
 * a launch costs up to there. stage 0: a launch of the same shape that does
 * nothing; 1: the bags' positions (the prefix over the lengths); 2: index and
 * weight of every lookup; 3: scale and offset of every row; 4: every row read,
 * no arithmetic. The output holds values that depend on what was read and
 * nothing else of use. */
int mi355x_frwq_slws_probe(int stage, float *dest, const uint8_t *data, size_t data_rows,
                           const float *weights, const int64_t *indices,
                           size_t num_indices, const int32_t *lengths, size_t segments,
                           size_t in_line_size, void *stream);

/* libjit_rowwise_quantized_sparse_lengths_weighted_sum_f_u / _f_i32 (reference
 * libjit.cpp:1232-1251, 2400-2414): the table holds uint8 rows of line_size
 * bytes, the fp32 scale and offset of row r are scales[r] and offsets[r].
 * weights NULL = all ones. */
int mi355x_rwq_slws(float *dest, const uint8_t *data, size_t data_rows,
                    const float *scales, const float *offsets, const float *weights,
                    const void *indices, int idx_is_64, size_t num_indices,
                    const int32_t *lengths, size_t segments, size_t line_size,
                    void *stream);
int mi355x_rwq_slws_opts(float *dest, const uint8_t *data, size_t data_rows,
                    const float *scales, const float *offsets, const float *weights,
                    const void *indices, int idx_is_64, size_t num_indices,
                    const int32_t *lengths, size_t segments, size_t line_size,
                    void *stream,
                    const mi355x_launch_opts *opts);

/* FusedRowwiseQuantizedSparseLengthsSum over several tables of one shape in ONE
 * launch (a ranking model pools dozens of tables per request, each too small
 * to fill the chip on its own), optionally with the instructions that follow
 * each lookup folded into its store. No counterpart in the reference, whose
 * CPU backend runs the tables one after another.
 *   tables    DEVICE array of n_tables entries (all pointers device pointers;
 *             data 16-byte aligned)
 *   segments  bags per table (at most 4096); every table has in_line_size-byte
 *             rows of `kind`, at most max_data_rows of them
 *   out_kind  MI355X_SLS_OUT_F32 / _F16: dense [segments x out_line_size] rows at
 *             tables[t].dest, as mi355x_frwq_slws writes them;
 *             MI355X_SLS_OUT_I8 / _I8_VIA_F16: Quantize(out_scale, out_offset) of
 *             the fp32 result (_I8) or of the result rounded to fp16 and
 *             converted back (_I8_VIA_F16: lookup with a Float16 result, ConvertTo
 *             Float, Quantize), int8 rows dest_row_stride bytes apart starting at
 *             tables[t].dest (InsertTensor into a wider tensor).
 * Indices are int64 (idx_is_64) or int32 for all tables; no weights.
 * A table whose bag_offsets is not NULL gives its bags as segments + 1 positions
 * (see mi355x_frwq_slws_offsets) and its lengths are not read. */
typedef struct {
  const uint8_t *data;
  const void *indices;
  const int32_t *lengths;
  void *dest;
  uint64_t data_rows;
  uint64_t num_indices;
  const int32_t *bag_offsets;
} mi355x_sls_table;
enum { MI355X_SLS_OUT_F32 = 0, MI355X_SLS_OUT_F16 = 1, MI355X_SLS_OUT_I8 = 2,
       MI355X_SLS_OUT_I8_VIA_F16 = 3 };
int mi355x_frwq_sls_multi(const mi355x_sls_table *tables, size_t n_tables,
                          size_t max_data_rows, int kind, int idx_is_64,
                          size_t segments, size_t in_line_size,
                          size_t out_line_size, int out_kind, float out_scale,
                          int32_t out_offset, size_t dest_row_stride,
                          int fp16_accum, void *stream);
int mi355x_frwq_sls_multi_opts(const mi355x_sls_table *tables, size_t n_tables,
                          size_t max_data_rows, int kind, int idx_is_64,
                          size_t segments, size_t in_line_size,
                          size_t out_line_size, int out_kind, float out_scale,
                          int32_t out_offset, size_t dest_row_stride,
                          int fp16_accum, void *stream,
                          const mi355x_launch_opts *opts);

/* libjit_embedding_bag_byte_rowwise_offsets_f (libjit.cpp:2454-2481) and the
 * Interpreter's 4-bit / fp16 twin: bags are given by int32 start offsets
 * (`segments` entries, the last one being the end offset when
 * has_end_offset). Output has segments - has_end_offset rows. */
int mi355x_embedding_bag_rowwise_offsets(
    void *dest, int out_is_f16, const uint8_t *data, size_t data_rows,
    int kind, const void *weights, int weights_are_f16, const int32_t *indices,
    size_t num_indices, const int32_t *offsets, size_t segments,
    int has_end_offset, size_t in_line_size, size_t out_line_size,
    int fp16_accum, void *stream);
int mi355x_embedding_bag_rowwise_offsets_opts(
    void *dest, int out_is_f16, const uint8_t *data, size_t data_rows,
    int kind, const void *weights, int weights_are_f16, const int32_t *indices,
    size_t num_indices, const int32_t *offsets, size_t segments,
    int has_end_offset, size_t in_line_size, size_t out_line_size,
    int fp16_accum, void *stream,
    const mi355x_launch_opts *opts);

#ifdef __cplusplus
}
#endif
#endif /* GLOW_MI355X_H */
