/*
 * CPU restatement of Glow's quantized-inference arithmetic (CPU backend,
 * "libjit"), plus the Interpreter-only 4-bit / fp16 fused-rowwise SLS formula.
 *
 * THIS IS TEST INFRASTRUCTURE. It is the checker the HIP kernels are compared
 * against and the timed CPU baseline; nothing that ships calls into it.
 *
 * Every function cites the reference file:line whose behaviour it restates
 * (paths relative to the pytorch/glow tree). Integer paths wrap modulo 2^32
 * exactly like the compiled reference (two's complement, arithmetic >>).
 * Float paths are compiled without fast-math and without FMA contraction, so
 * each multiply and add rounds separately, in the reference's loop order.
 *
 * How each function is pinned (none is "parity unpinned"):
 *   go_scale_i32 / go_clip_i8 / go_quantize_i8 / go_dequantize_i8 /
 *   go_rescale_i8 / go_fc_i8 / go_rwq_fc_i8 / go_matmul_i8 / go_conv2d_i8 /
 *   go_cwq_conv2d_i8 / go_cwq_conv3d_i8 / go_frwq_slws_f32 / glue ops /
 *   go_quantize_i16, _i32 / go_dequantize_i16, _i32 / go_rescale_i16, _i32 /
 *   go_transpose
 *       -> compared against the reference's own libjit sources compiled into
 *          oracle/_ref (tests/test_oracle_vs_ref.py), committed golden vectors
 *          produced by that build (tests/golden), the exact known-answer
 *          conv test OperatorTest.cpp:11407-11485 and the SLWS known answers
 *          OperatorTest.cpp:16941-17040, 17314-17380, 17411-17511.
 *   go_quantize_scale_offset_32to8
 *       -> QuantizationTest.cpp:223-247 (+-1 property over 39 scales x int8),
 *          :249-275 (exact power-of-two cases), hand-derived cases.
 *   go_choose_qparams
 *       -> exact offsets / scales of QuantizationTest.cpp:1751-1855, 2069-2116.
 *   go_fused_rowwise_quantize / go_rowwise_quantize_i8
 *       -> round trips QuantizationTest.cpp:444-489, closed forms, numpy fp16.
 *   go_frwq_slws_generic (Interpreter formula, 4-bit and fp16 scale)
 *       -> near-exact KAT OperatorTest.cpp:16152-16295, KATs :17401-17407,
 *          :17531-17547, brute force in numpy on tiny tables, and equality
 *          with go_frwq_slws_f32 on the 8-bit/fp32 form; the float16
 *          accumulator branch (InterpreterNodes.cpp:5799-5836 with AccumT =
 *          float16_t) by a numpy-float16 brute force on inputs that are not
 *          representable in half, on which dropping either rounding (of the
 *          product, of the partial sum) changes bits.
 */
#ifndef GLOW_ORACLE_H
#define GLOW_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- scalar helpers ---------------------------------------------------- */

/* libjit_defs.h:158-173 (libjit_scale<int32_t>) */
int32_t go_scale_i32(int32_t input, int32_t pre, int32_t post, int32_t scale,
                     int32_t offset);
/* libjit_defs.h:147-148 */
int8_t go_clip_i8(int32_t v);
/* libjit_defs.h:206-233; actType follows glow::FusedActivation, Nodes.h:276 */
int32_t go_activation_i32(int32_t input, int32_t offset, int32_t actType,
                          const int32_t *actArgs);

/* IEEE binary16 <-> binary32, round-to-nearest-even (Float16.h:38) */
uint16_t go_f32_to_f16(float f);
float go_f16_to_f32(uint16_t h);

/* ---- host-side parameter derivation ----------------------------------- */

/* lib/Quantization/Base/Base.cpp:234-359. out = {pre, post, scale, offset} */
void go_quantize_scale_offset_32to8(float scale, int32_t offset,
                                    int32_t out[4]);

/* Schema values follow quantization::Schema, Base.h:217-236. */
enum { GO_ASYMMETRIC = 0, GO_SYMMETRIC = 1, GO_SYMMETRIC_WITH_UNSIGNED = 2,
       GO_SYMMETRIC_POW2 = 3 };
/* qty: 8 -> Int8QTy, 16 -> Int16QTy, 32 -> Int32QTy (int30 range),
 * 108 -> UInt8QTy. Base.cpp:361-403. */
/* Base.cpp:433-565 with Calibration::None. */
void go_choose_qparams(float min, float max, int schema, int qty,
                       float *scale, int32_t *offset);
/* Base.cpp:594-629 (specializeBiasWeightsQuantizationParams). biasIsI32 != 0
 * for an Int32QTy bias. Updates *biasScale, *biasOffset, *weightsScale. */
void go_specialize_bias_weights_qparams(float *biasScale, int32_t *biasOffset,
                                        float inputScale, float *weightsScale,
                                        int biasIsI32, int biasZero);
/* Base.cpp:567-592 (specializeBiasQuantizationParams). Updates *biasScale,
 * *biasOffset. */
void go_specialize_bias_qparams(float *biasScale, int32_t *biasOffset, float inputScale,
                                float weightsScale, int biasIsI32, int biasZero);
/* Graph.cpp:3576-3700: constants of a ChannelwiseQuantizedConvolution from a
 * float filter [channels x perChannel] and float bias. Pinned by the closed
 * forms tests/test_oracle_kats.py states (bias scale == input scale * filter
 * scale bit for bit; the filter scale gives way exactly when the bias would
 * saturate; round trip within half a step). */
void go_channelwise_quantize_conv(const float *filter, const float *bias, size_t channels,
                                  size_t perChannel, float inputScale, int schema,
                                  int8_t *filterQ, int32_t *biasQ, float *filterScales,
                                  int32_t *filterOffsets, float *biasScales,
                                  int32_t *biasOffsets);

/* Base.h:323-329 quantize<int8_t> / quantize<int32_t> on one value. */
int8_t go_quantize_value_i8(float x, float scale, int32_t offset);
int32_t go_quantize_value_i32(float x, float scale, int32_t offset);

/* Base.h:522-557 with ScaleT=float, OffsetT=int32, QP=int8 (FC weights):
 * per-row chooseQuantizationParams + quantize. in [rows x cols] row-major. */
void go_rowwise_quantize_i8(const float *in, size_t rows, size_t cols,
                            int schema, int8_t *out, float *scales,
                            int32_t *offsets);

/* Fused-rowwise kinds, Type.h:424-433. */
enum { GO_U8_F32 = 0, GO_U8_F16 = 1, GO_U4_F16 = 2, GO_U4_F32 = 3 };
/* bytes per fused row holding `cols` logical columns of `kind`. */
size_t go_fused_row_bytes(size_t cols, int kind);
/* Base.h:598-678 tensorFusedRowwiseQuantization<T>. out is rows x
 * go_fused_row_bytes(cols, kind). */
void go_fused_rowwise_quantize(const float *in, size_t rows, size_t cols,
                               int kind, uint8_t *out);

/* ---- elementwise ------------------------------------------------------- */

/* libjit.cpp:2998-3002 */
void go_quantize_i8(int8_t *dst, const float *src, size_t n, float scale,
                    int32_t offset);
/* libjit.cpp:3016-3019 */
void go_dequantize_i8(float *dst, const int8_t *src, size_t n, float scale,
                      int32_t offset);
/* libjit.cpp:3031-3038 */
void go_rescale_i8(int8_t *dst, const int8_t *src, size_t n, int32_t outOffset,
                   int32_t inOffset, int32_t pre, int32_t post, int32_t scale);

/* libjit.cpp:3004-3014, 3021-3029, 3040-3056: the 16- and 32-bit forms (the
 * rescales run libjit_scale<int64_t>; the 32-bit quantize does not clip). */
void go_quantize_i16(int16_t *dst, const float *src, size_t n, float scale, int32_t offset);
void go_quantize_i32(int32_t *dst, const float *src, size_t n, float scale, int32_t offset);
void go_dequantize_i16(float *dst, const int16_t *src, size_t n, float scale, int32_t offset);
void go_dequantize_i32(float *dst, const int32_t *src, size_t n, float scale, int32_t offset);
void go_rescale_i16(int16_t *dst, const int16_t *src, size_t n, int32_t outOffset,
                    int32_t inOffset, int32_t pre, int32_t post, int32_t scale);
void go_rescale_i32(int32_t *dst, const int32_t *src, size_t n, int32_t outOffset,
                    int32_t inOffset, int32_t pre, int32_t post, int32_t scale);

/* libjit.cpp:565-653, 3162-3184: transpose of up to 6 dimensions; output
 * dimension d is input dimension shuffle[d]. */
void go_transpose(void *out, const void *in, const size_t *idim, const size_t *shuffle,
                  size_t numDims, size_t elemSize);

/* ---- FullyConnected / MatMul ------------------------------------------ */

/* libjit_matmul.cpp:254-280. in [M x K], weights [K x N], bias int32 or int8
 * (biasIsI8), out [M x N]. */
void go_fc_i8(int8_t *out, const int8_t *in, const int8_t *weights,
              const void *bias, int biasIsI8, size_t M, size_t K, size_t N,
              int32_t outOffset, int32_t inOffset, int32_t weightsOffset,
              int32_t biasOffset, int32_t biasPre, int32_t biasPost,
              int32_t biasScale, int32_t outPre, int32_t outPost,
              int32_t outScale);

/* libjit_matmul.cpp:284-316. weights [N x K]; per-row parameter arrays of
 * length N. */
void go_rwq_fc_i8(int8_t *out, const int8_t *in, const int8_t *weights,
                  const void *bias, int biasIsI8, const int32_t *weightsOffsets,
                  const int32_t *biasPre, const int32_t *biasPost,
                  const int32_t *biasScale, const int32_t *outPre,
                  const int32_t *outPost, const int32_t *outScale, size_t M,
                  size_t K, size_t N, int32_t outOffset, int32_t inOffset,
                  int32_t biasOffset);

/* libjit_matmul.cpp:353-371. lhs [M x K], rhs [K x N]. */
void go_matmul_i8(int8_t *out, const int8_t *lhs, const int8_t *rhs, size_t M,
                  size_t K, size_t N, int32_t outOffset, int32_t lhsOffset,
                  int32_t rhsOffset, int32_t outPre, int32_t outPost,
                  int32_t outScale);

/* ---- Convolution -------------------------------------------------------- */

/* Geometry shared by both convolutions. NHWC input, filter
 * [OC, KH, KW, IC/group], pads = {top, left, bottom, right}. */
typedef struct {
  int32_t N, IH, IW, IC;
  int32_t OH, OW, OC;
  int32_t KH, KW;
  int32_t strideH, strideW;
  int32_t padT, padL;
  int32_t dilH, dilW;
  int32_t group;
} go_conv_geom;

/* libjit_conv.cpp:49-147 (results do not depend on depthUnroll). */
void go_conv2d_i8(int8_t *out, const int8_t *in, const int8_t *filter,
                  const void *bias, int biasIsI8, const go_conv_geom *g,
                  int32_t outOffset, int32_t inOffset, int32_t filterOffset,
                  int32_t biasOffset, int32_t biasPre, int32_t biasPost,
                  int32_t biasScale, int32_t outPre, int32_t outPost,
                  int32_t outScale, int32_t actType, const int32_t *actArgs);

/* libjit_conv.cpp:151-239; per-output-channel arrays of length OC. */
void go_cwq_conv2d_i8(int8_t *out, const int8_t *in, const int8_t *filter,
                      const void *bias, int biasIsI8, const go_conv_geom *g,
                      int32_t outOffset, int32_t inOffset,
                      const int32_t *filterOffsets, const int32_t *biasOffsets,
                      const int32_t *biasPre, const int32_t *biasPost,
                      const int32_t *biasScale, const int32_t *outPre,
                      const int32_t *outPost, const int32_t *outScale,
                      int32_t actType, const int32_t *actArgs);

typedef struct {
  int32_t N, IT, IH, IW, IC;
  int32_t OT, OH, OW, OC;
  int32_t KT, KH, KW;
  int32_t strideT, strideH, strideW;
  int32_t padN, padT, padL; /* near, top, left */
  int32_t group;
} go_conv3d_geom;

/* libjit_conv.cpp:244-349, 564-596 */
void go_cwq_conv3d_i8(int8_t *out, const int8_t *in, const int8_t *filter, const void *bias,
                      int biasIsI8, const go_conv3d_geom *g, int32_t outOffset,
                      int32_t inOffset, const int32_t *filterOffsets,
                      const int32_t *biasOffsets, const int32_t *biasPre,
                      const int32_t *biasPost, const int32_t *biasScale, const int32_t *outPre,
                      const int32_t *outPost, const int32_t *outScale, int32_t actType,
                      const int32_t *actArgs);

/* ---- FusedRowwiseQuantizedSparseLengthsWeightedSum -------------------- */

/* libjit.cpp:1253-1276 (8-bit data, fp32 scale/offset, fp32 weights/out).
 * indices are int64 (idxIs64) or int32. */
void go_frwq_slws_f32(float *dest, const uint8_t *data, const float *weights,
                      const void *indices, int idxIs64, const int32_t *lengths,
                      size_t segments, size_t inLineSize, size_t outLineSize);

/* lib/Backends/Interpreter/InterpreterNodes.cpp:5764-5889 with
 * Base.h:383-406 dequantizers. weights / dest are fp32, or fp16 bit patterns
 * when weightsAreF16 / outIsF16. weights == NULL means all-ones
 * (FusedRowwiseQuantizedSparseLengthsSum, Lower.cpp:1590-1606).
 * fp16Accum follows the dispatch at :5866-5887 (only honoured for fp16
 * output with an fp16-scale kind). */
void go_frwq_slws_generic(void *dest, int outIsF16, const uint8_t *data,
                          int kind, const void *weights, int weightsAreF16,
                          const void *indices, int idxIs64,
                          const int32_t *lengths, size_t segments,
                          size_t inLineSize, size_t outLineSize,
                          int fp16Accum);

/* libjit.cpp:1232-1251 (RowwiseQuantizedSparseLengthsWeightedSum: separate
 * per-row scales and offsets). */
void go_rwq_slws_f32(float *dest, const uint8_t *data, const float *scales,
                     const float *offsets, const float *weights,
                     const void *indices, int indicesAre64, const int32_t *lengths,
                     size_t segments, size_t lineSize);

/* libjit.cpp:2454-2481 (EmbeddingBagByteRowwiseOffsets, int32 indices and
 * offsets). */
void go_embedding_bag_byte_rowwise_offsets_f32(
    float *dest, const uint8_t *data, const float *weights,
    const int32_t *indices, const int32_t *offsets, size_t segments,
    size_t numIndices, size_t inLineSize, size_t outLineSize,
    int hasEndOffset);

/* ---- int8 glue operators (ResNet-style graphs) --------------------------- */

/* libjit_element_add_kernel_i8 (libjit.cpp:1593-1603, 1675-1676) over n. */
void go_add_i8(int8_t *dest, const int8_t *lhs, const int8_t *rhs, size_t n,
               int32_t destOffset, int32_t lhsOffset, int32_t rhsOffset,
               int32_t lhsPre, int32_t lhsPost, int32_t lhsScale,
               int32_t rhsPre, int32_t rhsPost, int32_t rhsScale);
/* libjit_element_clip_i8 (libjit.cpp:1865-1873) over n. */
void go_clip_elem_i8(int8_t *dest, const int8_t *src, size_t n, int8_t clipMin, int8_t clipMax,
                     int8_t srcOffset, int8_t destOffset, int32_t destPre, int32_t destPost,
                     int32_t destScale);
/* libjit_element_leaky_relu_i8 (libjit.cpp:1880-1892) over n. */
void go_leaky_relu_i8(int8_t *dest, const int8_t *src, size_t n, int8_t srcOffset,
                      int8_t destOffset, int32_t posPre, int32_t posPost, int32_t posScale,
                      int32_t negPre, int32_t negPost, int32_t negScale);
/* libjit_element_maxsplat_kernel_i8 (libjit_cpu.cpp:45-46) over n. */
void go_max_splat_i8(int8_t *dest, const int8_t *src, size_t n, int8_t value);
/* libjit_batchedadd_i8 / _i32_i8 (libjit.cpp:997-1015, 1945-1969). */
void go_batched_add_i8(int8_t *dest, const int8_t *batch, const void *slice, int sliceIsI32,
                       size_t numSlice, size_t sliceSize, int32_t destOffset,
                       int32_t batchOffset, int32_t sliceOffset, int32_t batchPre,
                       int32_t batchPost, int32_t batchScale, int32_t slicePre,
                       int32_t slicePost, int32_t sliceScale);
/* libjit_element_relu_i8 (libjit.cpp:1851-1858) over n. */
void go_relu_i8(int8_t *dest, const int8_t *src, size_t n, int8_t srcOffset,
                int8_t destOffset, int32_t destPre, int32_t destPost,
                int32_t destScale);
/* libjit_max_pool_i8 (libjit.cpp:812-884, 2592-2597); NHWC, pads {top, left}. */
void go_max_pool_i8(int8_t *out, const int8_t *in, size_t N, size_t IH,
                    size_t IW, size_t C, size_t OH, size_t OW, size_t kH,
                    size_t kW, size_t sH, size_t sW, size_t padT, size_t padL,
                    int32_t outOffset);
/* libjit_avg_pool_i8 (libjit.cpp:2812-2880). */
void go_avg_pool_i8(int8_t *out, const int8_t *in, size_t N, size_t IH,
                    size_t IW, size_t C, size_t OH, size_t OW, size_t kH,
                    size_t kW, size_t sH, size_t sW, size_t padT, size_t padL,
                    int countIncludePads, int32_t outOffset, int32_t inOffset,
                    int32_t outPre, int32_t outPost, int32_t outScale);
/* libjit_softmax_f (libjit.cpp:3058-3082) on [rows x cols]. */
void go_softmax_f32(float *out, const float *in, size_t rows, size_t cols);
/* libjit_sigmoid_kernel_f (libjit.cpp:1913-1916, the build without fast-math). */
void go_sigmoid_f32(float *out, const float *in, size_t n);
/* libjit_gather (libjit.cpp:418-440) on byte slices. */
void go_gather(uint8_t *dest, const uint8_t *data, const int64_t *indices,
               size_t numIndices, size_t sliceBytes, size_t numSamples,
               size_t sampleBytes);

#ifdef __cplusplus
}
#endif
#endif
