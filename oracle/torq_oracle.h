/*
 * CPU oracle for the quantized TorqHL operator path.  TEST INFRASTRUCTURE ONLY.
 *
 * This is a plain-C restatement of what the reference computes for
 * torq_hl.{conv2d, depthwise_conv2d, fully_connected, matmul, maxpool2d,
 * avg_pool2d, add} and of the compile-side parameter derivations that feed
 * them.  It exists to check the HIP backend; the product never links, loads
 * or calls it.  The only legitimate users are the test-suite, the smoke
 * check and the benchmark's CPU-baseline leg.
 *
 * The reference's own executor for these ops is a closed simulator that is
 * not available, and its tests hold no expected outputs, so every function
 * here is pinned by (1) the cited source text, (2) closed forms / brute force
 * / invariants exercised by tests/test_oracle_*.py and (3) known answers
 * worked out by hand from constants that the reference's fixtures hold
 * (tests/golden/).  No function in this file is "parity unpinned".
 *
 * Each function cites the reference file:line it follows (paths relative to
 * the reference checkout).
 */
#ifndef TORQ_ORACLE_H_
#define TORQ_ORACLE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Tensor layouts for the 4-D activation operands. */
enum { TORQ_LAYOUT_NCHW = 0, TORQ_LAYOUT_NHWC = 1 };

/* Requantisation parameters shared by all ops (ACT unit "rescaleClamp").
 * compiler/torq/Utils/Kernel.h:610-624. */
typedef struct torq_requant_t {
    int32_t shift;      /* shift_factor / act_rsh, 0..63 */
    int32_t output_zp;  /* must fit int16: third_party/torq-hw/ct/torq_api.c:572 */
    int32_t output_min;
    int32_t output_max;
} torq_requant_t;

/* R1. One element of the ACT rescale-clamp.  Returns the clamped value
 * before truncation to the output element type. */
int64_t torq_act_rescale_clamp(int32_t acc, int32_t bias, int32_t scale, const torq_requant_t *rq);

/* Number of OpenMP threads the op functions will use (1 if built without). */
int torq_oracle_threads(void);
void torq_oracle_set_threads(int n);

/* torq_hl.conv2d.  weights are O x I x KH x KW int8, scale_bias is the
 * interleaved [bias0, scale0, bias1, scale1, ...] int32 vector, pad is
 * [left, right, top, bottom], stride is [h, w].  `layout` selects NCHW (the
 * literal reference layout) or NHWC for BOTH input and output.
 * out_elem_bytes in {1,2,4}. Returns 0 on success, -1 on a bad argument. */
int torq_conv2d(const int8_t *input, const int8_t *weights, const int32_t *scale_bias, void *out,
                int N, int C, int H, int W, int O, int KH, int KW, const int64_t pad[4],
                const int64_t stride[2], int32_t input_zp, const torq_requant_t *rq, int layout,
                int out_elem_bytes);

/* torq_hl.depthwise_conv2d.  weights are C x 1 x KH x KW. */
int torq_depthwise_conv2d(const int8_t *input, const int8_t *weights, const int32_t *scale_bias,
                          void *out, int N, int C, int H, int W, int KH, int KW,
                          const int64_t pad[4], const int64_t stride[2], int32_t input_zp,
                          const torq_requant_t *rq, int layout, int out_elem_bytes);

/* torq_hl.fully_connected.  input M x K, weights N x K, scale_bias 2N. */
int torq_fully_connected(const int8_t *input, const int8_t *weights, const int32_t *scale_bias,
                         void *out, int M, int K, int N, const torq_requant_t *rq,
                         int out_elem_bytes);

/* torq_hl.matmul.  input1 B x M x K, input2 B x K x N, ONE (bias, scale)
 * pair in scale_bias[0..1].  bcast1/bcast2 non-zero means that operand has
 * batch 1 and is reused for every batch. */
int torq_matmul(const int8_t *input1, const int8_t *input2, const int32_t *scale_bias, void *out,
                int B, int M, int K, int N, int bcast1, int bcast2, const torq_requant_t *rq,
                int out_elem_bytes);

/* ---- bf16 rows (floating-point partials: bias only, no scale, no shift) ---- */

/* bfloat16 <-> float: the upper 16 bits of the IEEE single; to bf16 rounds to nearest, ties to even. */
float torq_bf16_to_f32(uint16_t h);
uint16_t torq_f32_to_bf16(float f);

/* torq_hl.fully_connected on bf16: input M x K, weights N x K (bf16 bit patterns), bias N floats.
 * clip_min / clip_max are float bit patterns (0xff800000 / 0x7f800000 = no clamp). */
int torq_fully_connected_bf16(const uint16_t *input, const uint16_t *weights, const float *bias,
                              uint16_t *out, int M, int K, int N, int32_t clip_min, int32_t clip_max);

/* torq_hl.matmul on bf16: input1 B x M x K, input2 B x K x N, ONE float bias. */
int torq_matmul_bf16(const uint16_t *input1, const uint16_t *input2, const float *bias, uint16_t *out,
                     int B, int M, int K, int N, int bcast1, int bcast2, int32_t clip_min, int32_t clip_max);

/* torq_hl.conv2d on bf16: weights O x I x KH x KW (bf16), bias O floats, padding with +0.0;
 * layout as for the int8 op. */
int torq_conv2d_bf16(const uint16_t *input, const uint16_t *weights, const float *bias, uint16_t *out,
                     int N, int C, int H, int W, int O, int KH, int KW, const int64_t pad[4],
                     const int64_t stride[2], int32_t clip_min, int32_t clip_max, int layout);

/* torq_hl.depthwise_conv2d on bf16: weights C x 1 x KH x KW, bias C floats. */
int torq_depthwise_conv2d_bf16(const uint16_t *input, const uint16_t *weights, const float *bias, uint16_t *out,
                               int N, int C, int H, int W, int KH, int KW, const int64_t pad[4],
                               const int64_t stride[2], int32_t clip_min, int32_t clip_max, int layout);

/* torq_hl.add on bf16: out = bf16(clamp(in1 * w[0] + in2 * w[1] + bias)), two bf16 weights, ONE float bias. */
int torq_add_bf16(const uint16_t *input1, const uint16_t *input2, const uint16_t weights[2], const float *bias,
                  uint16_t *out, size_t count, int32_t clip_min, int32_t clip_max);

/* torq_hl.avg_pool2d (global) on bf16: out[n][c] = bf16(clamp(sum_u x[n][u][c] * weight + bias[0])), summed
 * over the frame in order, in fp32. */
int torq_avg_pool2d_bf16(const uint16_t *input, uint16_t weight, const float *bias, uint16_t *out,
                         int N, int H, int W, int C, int32_t clip_min, int32_t clip_max);

/* torq_hl.expand_weights: int8 weights K x N, bf16 scales and float biases per block of block_size rows
 * (bias rows are bias_cols >= N wide): out = bf16(clamp(weight * scale + bias)). */
int torq_expand_weights(const int8_t *weights, const uint16_t *scale, const float *bias, uint16_t *out,
                        int K, int N, int block_size, int bias_cols, int32_t clip_min, int32_t clip_max);

/* torq_hl.maxpool2d.  No rescale; padding value is input_zp; result is
 * clamped to [output_min, output_max]. */
int torq_maxpool2d(const int8_t *input, int8_t *out, int N, int C, int H, int W, int KH, int KW,
                   const int64_t pad[4], const int64_t stride[2], int32_t input_zp,
                   int32_t output_min, int32_t output_max, int layout);

/* torq_hl.avg_pool2d (global).  Input is NHWC, output N x C; only pair 0 of
 * scale_bias is used; `weight` is the single int8 weight (1). */
int torq_avg_pool2d(const int8_t *input, int8_t weight, const int32_t *scale_bias, int8_t *out,
                    int N, int H, int W, int C, const torq_requant_t *rq);

/* torq_hl.add (tensor + tensor).  weights are two int16; scale_bias is one
 * [bias, scale] pair. */
int torq_add(const int8_t *input1, const int8_t *input2, const int16_t weights[2],
             const int32_t scale_bias[2], int8_t *out, size_t count, const torq_requant_t *rq);

/* torq_hl.fma (the stand-alone rescale): out = R1(input * weight) with one [bias, scale] pair; int8 / int16 /
 * int32 elements (in_bytes, out_bytes = 1, 2, 4). */
int torq_fma(const void *input, int in_bytes, int32_t weight, const int32_t scale_bias[2], void *out, int out_bytes,
             size_t count, const torq_requant_t *rq);

/* torq_hl.mul: out = R1(input1 * input2) with one [bias, scale] pair; an input of one element is broadcast. */
int torq_mul(const void *input1, size_t count1, const void *input2, size_t count2, int in_bytes,
             const int32_t scale_bias[2], void *out, int out_bytes, size_t count, const torq_requant_t *rq);

/* torq_hl.act on integers; mode 0 clamp [min_int, max_int], 1 abs, 2 negate (both clipped to the output type),
 * 3 i2i (truncating conversion). */
int torq_act(const void *input, int in_bytes, void *out, int out_bytes, size_t count, int mode, int64_t min_int,
             int64_t max_int);

/* torq_hl.elementwisebinary: mode 0 and, 1 or, 2 xor, 4 minimum, 5 maximum; both inputs and the output of one integer
 * type (bytes = 1, 2, 4); is_unsigned (16-bit only) compares as unsigned. */
int torq_elementwise_binary(int mode, const void *input1, const void *input2, int bytes, int is_unsigned, void *out, size_t count);

/* torq_hl.elementwisebinary, comparison and logical modes (6 greater, 7 greater-equal, 8 equal on int8 / int16 /
 * int32; 9 and, 10 or, 11 xor on i1 bytes): the result is an i1 tensor, one byte of 0 or 1 per element. */
int torq_elementwise_compare(int mode, const void *input1, const void *input2, int bytes, int is_unsigned, uint8_t *out, size_t count);

/* torq_hl.elementwiseunary: 3 bitwise not (int8 / int16 / int32), 12 logical not (i1 bytes). */
int torq_elementwise_unary(int mode, const void *input, int bytes, void *out, size_t count);

/* torq_hl.elementwiseshift: 0 logical right, 1 logical left, 2 arithmetic right; round: half up on right shifts;
 * input2 holds each element's count. */
int torq_elementwise_shift(int mode, int round, const void *input1, const void *input2, int bytes, void *out, size_t count);

/* torq_hl.table as the lookup patterns use it: the (bias, scale) pair turns each input (its low byte, signed) into
 * 9.7 fixed point, the integer part selects one of table_count segment words, the result is the word's base
 * (>> 8 for a 1-byte result).  Returns -1 where an interpolation would be needed (non-zero fraction). */
int torq_table(const void *input, int in_bytes, const int32_t *table, int table_count, int32_t bias, int32_t scale, void *out, int out_bytes, size_t count);

/* ---- R2: compile-side parameter derivations ---- */

/* Conv / depthwise / FC: per-channel TOSA (multiplier, shift) -> one global
 * shift_factor = min shift and scale[c] = multiplier[c] >> (shift[c] - min);
 * bias[c] = tosa_bias[c] - input_zp * weight_sum[c]; writes interleaved
 * scale_bias (2*channels) and returns shift_factor. */
int32_t torq_derive_scale_bias(const int32_t *multiplier, const int8_t *shift,
                               const int32_t *tosa_bias, const int64_t *weight_sum,
                               int32_t input_zp, int channels, int32_t *scale_bias);

/* Sum of the weights feeding each output channel (O x per_channel int8). */
void torq_per_channel_sum(const int8_t *weights, int channels, int per_channel, int64_t *sums);

/* Quantised add: multipliers m_k = output_scale * input_scale_k (doubles),
 * S = 2^12.  Returns 0, or -1 when a weight would overflow int16 (the
 * reference rejects the match). `sign` is +1 for add, -1 for sub. */
int torq_derive_add_params(double m0, double m1, int32_t zp0, int32_t zp1, int sign,
                           int16_t weights[2], int32_t scale_bias[2], int32_t *shift_factor);

/* Global average pool: scale = floor(2^20 / (H*W)), bias = -(pre-scale
 * subtract constant) = -H*W*input_zp, shift_factor = 20. */
void torq_derive_avgpool_params(int H, int W, int32_t input_zp, int32_t scale_bias[2],
                                int32_t *shift_factor);

#ifdef __cplusplus
}
#endif
#endif /* TORQ_ORACLE_H_ */
