/*
 * thip -- C-ABI of the MI355X (gfx950) backend for the quantized TorqHL
 * operator path.
 *
 * Plain C linkage, plain pointers and sizes.  Two halves, mirroring the two
 * places where the reference's NPU-specific code is replaced:
 *
 *   compile side  thip_program_* / thip_hl_*  : accepts torq_hl.{conv2d,
 *                 depthwise_conv2d, fully_connected, matmul, maxpool2d,
 *                 avg_pool2d, add} records with the reference's operand and
 *                 attribute names and serialises a dispatch descriptor
 *                 (role of KernelSelection + EncodeTensors + serializeTorqHW).
 *   run side      thip_device_* / thip_executable_* : loads a descriptor and
 *                 runs it on bindings (role of the torq HAL driver's
 *                 native_executable + TorqExecutable + TorqHw).
 *
 * Every entry point returns a thip_status_t whose numeric values are the
 * status categories the reference returns through iree_status_t; the text of
 * the last failure on the calling thread is available from
 * thip_status_message().  No exception crosses this boundary.
 *
 * Reference paths below are relative to the reference checkout.
 */
#ifndef THIP_H_
#define THIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------------ */
/* Status                                                                   */
/* ------------------------------------------------------------------------ */

/* Same categories (and numeric codes) as the iree_status_t values used by
 * runtime/driver/TorqExecutable.cc:640-705 and
 * runtime/driver/torq_command_buffer.c:453-494. */
typedef int32_t thip_status_t;
enum {
    THIP_OK = 0,
    THIP_INVALID_ARGUMENT = 3,
    THIP_RESOURCE_EXHAUSTED = 8,
    THIP_FAILED_PRECONDITION = 9,
    THIP_OUT_OF_RANGE = 11,
    THIP_UNIMPLEMENTED = 12,
    THIP_INTERNAL = 13,
    THIP_UNAVAILABLE = 14
};

/* Message of the last non-OK status returned on this thread ("" if none). */
const char *thip_status_message(void);

/* Library version (major << 16 | minor) and the descriptor version it reads. */
uint32_t thip_version(void);
uint32_t thip_descriptor_version(void);

/* ------------------------------------------------------------------------ */
/* Compile side: TorqHL program -> dispatch descriptor                      */
/* ------------------------------------------------------------------------ */

typedef struct thip_program_t thip_program_t;

/* A tensor value of the program (index into the program's value table). */
typedef int32_t thip_value_t;

/* BF16 values are bfloat16 bit patterns (16 bits); F32 is used for the bias of the bf16 ops. */
/* THIP_DTYPE_I1: a truth value (MLIR's i1), one byte per element holding 0 or 1. */
enum { THIP_DTYPE_I8 = 1, THIP_DTYPE_I16 = 2, THIP_DTYPE_I32 = 3, THIP_DTYPE_BF16 = 4, THIP_DTYPE_F32 = 5, THIP_DTYPE_I1 = 6 };

#define THIP_MAX_RANK 4

/* torq_hl VectorizationModeEnum (compiler/torq/Dialect/TorqHL/TorqHLAttrs.td:149-239).
 * The patterns emit None; the NPU kernel-selection pass picks the others.  The
 * field is carried for signature compatibility and ignored by this backend. */
enum { THIP_VECTORIZATION_NONE = 0 };

thip_status_t thip_program_create(thip_program_t **out_program);
void thip_program_destroy(thip_program_t *program);

/* Declares the tensor carried by dispatch binding `binding` (the
 * hal.interface.binding of the dispatch; table entry of
 * runtime/schemas/torq_executable_def.fbs:29-48). */
/* Name of the hal.executable.export the program comes from (the reference keeps it as
 * ExecutableDef.executable_name, runtime/schemas/torq_executable_def.fbs:172-173, and names its dump directories
 * and profile rows after it).  1..63 characters of [A-Za-z0-9_.$-]; "thip_dispatch" when never set. */
thip_status_t thip_program_set_name(thip_program_t *program, const char *name);

thip_status_t thip_program_binding(thip_program_t *program, uint32_t binding, int32_t dtype,
                                   int32_t rank, const int64_t *shape, thip_value_t *out_value);

/* Declares a compile-time constant (arith.constant); the bytes are copied. */
thip_status_t thip_program_constant(thip_program_t *program, int32_t dtype, int32_t rank,
                                    const int64_t *shape, const void *data, size_t data_size,
                                    thip_value_t *out_value);

/* Declares an intermediate tensor (tensor.empty used as `init` of an op whose
 * result feeds another op of the same program). */
thip_status_t thip_program_tensor(thip_program_t *program, int32_t dtype, int32_t rank,
                                  const int64_t *shape, thip_value_t *out_value);

/* The same bytes under another shape: `shape` elements of `base` (a binding or an intermediate), starting
 * `element_offset` elements into it.  What tensor.collapse_shape / tensor.expand_shape around an op (the patterns
 * create them, compiler/torq/Conversions/LinalgToTorqHL/Conv2DMatmulPattern.cpp:105,134,411) and a contiguous
 * tensor.extract_slice / insert_slice become once bufferized: no op, no copy.  A view may be read and may be the
 * `init` of fully_connected, matmul, add, transpose and the elementwise ops; the rank-4 image ops take whole values. */
thip_status_t thip_program_view(thip_program_t *program, thip_value_t base, int64_t element_offset,
                                int32_t rank, const int64_t *shape, thip_value_t *out_value);

/* The op records.  Field names and meaning are those of the TorqHL op
 * definitions; `init` is the destination-passing-style output operand
 * (compiler/torq/Dialect/TorqHL/TorqHLOps.td:27-46). */

/* torq_hl.conv2d -- TorqHLOps.td:119-143.  input N,C,H,W (N,H,W,C when
 * nhwc_input), weights O,I,KH,KW, scale_bias int32[2*O] = [bias0, scale0, ...],
 * pad = [left, right, top, bottom], stride = [h, w].  With nhwc_input the init
 * tensor is N,OH,OW,O as well.  groups must be 1, dilation [1,1] (folded into
 * the weights by the patterns), weight_zp 0. */
typedef struct thip_hl_conv2d_t {
    thip_value_t init;
    int32_t input_zp;
    int32_t weight_zp;
    int32_t output_zp;
    int32_t output_min;
    int32_t output_max;
    int32_t shift_factor;
    int32_t groups;
    int64_t pad[4];
    int64_t stride[2];
    int64_t dilation[2];
    int32_t vectorization_mode;
    thip_value_t weights;
    thip_value_t scale_bias;
    thip_value_t input;
    int32_t nhwc_input;
    int32_t segment_output;
} thip_hl_conv2d_t;

/* torq_hl.depthwise_conv2d -- TorqHLOps.td:145-170.  weights C,1,KH,KW. */
typedef struct thip_hl_depthwise_conv2d_t {
    thip_value_t init;
    int32_t input_zp;
    int32_t weight_zp;
    int32_t output_zp;
    int32_t output_min;
    int32_t output_max;
    int32_t shift_factor;
    int32_t groups;
    int64_t pad[4];
    int64_t stride[2];
    int64_t dilation[2];
    int32_t vectorization_mode;
    thip_value_t weights;
    thip_value_t scale_bias;
    thip_value_t input;
    int32_t nhwc_input;
    int32_t segment_output;
    int32_t is_dw1d_stride1;
} thip_hl_depthwise_conv2d_t;

/* torq_hl.fully_connected -- TorqHLOps.td:172-190.  input M,K; weights N,K;
 * scale_bias int32[2*N].
 * bf16 form (input, weights and init BF16): the ACT stage has no scale and no shift
 * (compiler/torq/Utils/Kernel.h:626-632): scale_bias is F32[N] (bias only), shift_factor and the
 * zero points must be 0, output_min / output_max are float bit patterns (0xff800000 / 0x7f800000
 * when there is no clamp, compiler/torq/Utils/ConversionUtils.cpp:33-39); fp32 accumulate,
 * result rounded to bf16.  K must be a multiple of 8. */
typedef struct thip_hl_fully_connected_t {
    thip_value_t init;
    int32_t input_zp;
    int32_t weight_zp;
    int32_t output_zp;
    int32_t output_min;
    int32_t output_max;
    int32_t shift_factor;
    int32_t vectorization_mode;
    thip_value_t weights;
    thip_value_t scale_bias;
    thip_value_t input;
} thip_hl_fully_connected_t;

/* torq_hl.matmul -- TorqHLOps.td:85-99.  input1 [B,]M,K; input2 [B,]K,N; one
 * (bias, scale) pair in scale_bias; a batch of 1 broadcasts.
 * bf16 form (both inputs and init BF16): scale_bias is F32 with one bias value, shift and output_zp
 * 0, output_min / output_max float bit patterns, as for fully_connected. */
typedef struct thip_hl_matmul_t {
    thip_value_t init;
    int32_t output_zp;
    int32_t output_min;
    int32_t output_max;
    int32_t shift;
    thip_value_t scale_bias;
    thip_value_t input1;
    thip_value_t input2;
} thip_hl_matmul_t;

/* torq_hl.maxpool2d -- TorqHLOps.td:435-453.  input N,C,H,W; kernel = [kh, kw];
 * weights / scale_bias are the dummies the pattern creates and may be -1.
 * nhwc_input is this backend's addition (same meaning as on conv2d). */
typedef struct thip_hl_maxpool2d_t {
    thip_value_t init;
    int32_t input_zp;
    int32_t output_min;
    int32_t output_max;
    int64_t stride[2];
    int64_t pad[4];
    int64_t kernel[2];
    thip_value_t weights;
    thip_value_t scale_bias;
    thip_value_t input;
    int32_t segment_output;
    int32_t nhwc_input;
} thip_hl_maxpool2d_t;

/* torq_hl.avg_pool2d -- TorqHLOps.td:192-208.  Global: input N,H,W,C (NHWC),
 * init N,1,1,C; weights one int8; pair 0 of scale_bias applies to every channel.
 * bf16 form (compiler/torq/Conversions/LinalgToTorqHL/PoolingPattern.cpp:448-457): weights one BF16 (1.0 or a
 * folded multiplier), scale_bias F32[1] (bias only), shift_factor and zero points 0, output_min / output_max
 * float bit patterns; the frame is summed in order in fp32. */
typedef struct thip_hl_avg_pool2d_t {
    thip_value_t init;
    int32_t input_zp;
    int32_t output_zp;
    int32_t output_min;
    int32_t output_max;
    int32_t shift_factor;
    thip_value_t weights;
    thip_value_t scale_bias;
    thip_value_t input;
} thip_hl_avg_pool2d_t;

/* torq_hl.add -- TorqHLOps.td:48-69.  weights int16[2]; scale_bias int32[2];
 * `name` is "add" or "sub" (the sign already lives in weights[1]).
 * bf16 form (inputs and init BF16): weights BF16[2], scale_bias F32[1] (bias only), shift_factor and
 * zero points 0, output_min / output_max float bit patterns. */
typedef struct thip_hl_add_t {
    thip_value_t init;
    const char *name;
    int32_t input_zp;
    int32_t output_zp;
    int32_t output_min;
    int32_t output_max;
    int32_t shift_factor;
    thip_value_t weights;
    thip_value_t scale_bias;
    thip_value_t input1;
    thip_value_t input2;
    int32_t segment_output;
    int32_t rhs_is_scalar;
} thip_hl_add_t;

/* torq_hl.transpose -- TorqHLOps.td:397-407.  out.shape[i] = in.shape[perm[i]].
 * Rank-4 perms [0,2,3,1] (NCHW->NHWC) and [0,3,1,2] (NHWC->NCHW) and the swap of
 * the two innermost dimensions of a rank-2/3 tensor are supported; between two
 * ops of one program they fold into the producing kernel's layout. */
typedef struct thip_hl_transpose_t {
    thip_value_t init;
    int32_t rank;
    int64_t perm[THIP_MAX_RANK];
    thip_value_t input;
} thip_hl_transpose_t;

/* torq_hl.expand_weights -- TorqHLOps.td:943-957 (fields in the op's order); the block-quantized right-hand
 * side of a bf16 matmul (compiler/torq/Conversions/LinalgToTorqHL/MatmulPattern.cpp:596-680).  input int8
 * K,N; scale BF16 K/block_size,N; scale_bias F32 K/block_size,cols with cols >= N (the float bias
 * -zero_point * scale, columns rounded up to even, MatmulPattern.cpp:322-400); init BF16 K,N or 1,K,N:
 * init = bf16(clamp(input * scale + scale_bias)), output_min / output_max float bit patterns.  When every
 * operand is a constant and the only reader of init is input2 of a bf16 torq_hl.matmul, no kernel is
 * emitted: the matmul streams the int8 weights and expands them in registers (few rows), or reads weights
 * expanded at serialisation (many rows). */
typedef struct thip_hl_expand_weights_t {
    thip_value_t init;
    thip_value_t scale_bias;
    int32_t output_min;
    int32_t output_max;
    thip_value_t scale;
    thip_value_t input;
    int32_t block_size;
} thip_hl_expand_weights_t;

/* torq_hl.fma -- TorqHLOps.td:926-941: the stand-alone rescale
 * (compiler/torq/Conversions/LinalgToTorqHL/Patterns.cpp:1896-1946: weight 1, bias = -input_zp, scale = the
 * multiplier).  input and init int8 / int16 / int32 of the same element count; weights ONE int8 (or int16) value;
 * scale_bias int32[2] = [bias, scale]: init = R1(input * weights[0]). */
typedef struct thip_hl_fma_t {
    thip_value_t init;
    int32_t output_zp;
    int32_t output_min;
    int32_t output_max;
    int32_t shift_factor;
    thip_value_t weights;
    thip_value_t scale_bias;
    thip_value_t input;
} thip_hl_fma_t;

/* torq_hl.mul -- TorqHLOps.td:101-117.  input1 / input2 int8 or int16 (the same type), of init's element count or of
 * one element (broadcast); scale_bias int32[2] = [bias, scale]: init = R1(input1 * input2) with shift `shift`. */
typedef struct thip_hl_mul_t {
    thip_value_t init;
    int32_t output_zp;
    int32_t output_min;
    int32_t output_max;
    thip_value_t scale_bias;
    int32_t shift;
    thip_value_t input1;
    thip_value_t input2;
} thip_hl_mul_t;

/* torq_hl.act -- TorqHLOps.td:291-309, integer tensors.  name: "clamp" (clip to [min_int, max_int]), "abs",
 * "negate" (both clipped to the range of init's element type; the zero-point attributes are carried but, as in
 * compiler/torq/Conversions/TorqHLToTorqHW/ActPattern.cpp:60-140, not used), "i2i" (conversion by truncation).
 * weights (the unsigned-cast multiplier) must be THIP_NO_VALUE; the float names (ceil, floor, i2f, f2i, f2f, clz)
 * are not on this path. */
#define THIP_NO_VALUE (-1)
typedef struct thip_hl_act_t {
    thip_value_t init;
    const char *name;
    int32_t input_zp;
    int32_t output_zp;
    int64_t min_int;
    int64_t max_int;
    float min_fp;
    float max_fp;
    thip_value_t input;
    thip_value_t weights;
} thip_hl_act_t;

/* torq_hl.elementwisebinary -- TorqHLOps.td:248-260.  op_type: the reference's ElementwiseOpEnum value
 * (TorqHLAttrs.td:219-235).  BITWISE_AND 0, BITWISE_OR 1, BITWISE_XOR 2, MINIMUM 4, MAXIMUM 5: input1, input2 and
 * init are int8 / int16 / int32 tensors of one type and shape.  GREATER 6, GREATER_EQUAL 7, EQUAL 8: inputs of one
 * such type, init an i1 tensor (THIP_DTYPE_I1).  LOGICAL_AND 9, LOGICAL_OR 10, LOGICAL_XOR 11: i1 in, i1 out.
 * is_unsigned (16-bit operands only) makes MINIMUM / MAXIMUM and the comparisons read their operands as unsigned.
 * The int32 ADD / SUB through the 48-bit accumulator (13, 14) are not on this path. */
typedef struct thip_hl_elementwisebinary_t {
    thip_value_t init;
    int32_t op_type;
    thip_value_t input1;
    thip_value_t input2;
    int32_t is_unsigned;
} thip_hl_elementwisebinary_t;

/* torq_hl.elementwiseunary -- TorqHLOps.td:262-273.  op_type (ElementwiseOpEnum): 3 BITWISE_NOT on int8 / int16 /
 * int32 (init of the same type), 12 LOGICAL_NOT on i1 (init i1). */
typedef struct thip_hl_elementwiseunary_t {
    thip_value_t init;
    int32_t op_type;
    thip_value_t input;
} thip_hl_elementwiseunary_t;

/* torq_hl.elementwiseshift -- TorqHLOps.td:275-289.  op_type (ShiftModeEnum, TorqHLAttrs.td:239-246): 0 LSR, 1 LSL,
 * 2 ASR (3 ASL is refused, as the reference's lowering refuses it).  input1, input2 (the per-element shift counts)
 * and init share one type of int8 / int16 / int32 and one element count.  round: right shifts round half up. */
typedef struct thip_hl_elementwiseshift_t {
    thip_value_t init;
    int32_t op_type;
    int32_t round;
    thip_value_t input1;
    thip_value_t input2;
} thip_hl_elementwiseshift_t;

/* torq_hl.table -- TorqHLOps.td:311-327, in the forms the lookup patterns produce
 * (compiler/torq/Conversions/LinalgToTorqHL/ExtractPattern.cpp:30-62,285-298,432-545): a 256-entry table of segment
 * words (slope << 16) | (base & 0xFFFF) and scale_bias = int32[2] = [-128, 128].  That scale puts the input into
 * the ACT unit's 9.7 fixed point with a zero fraction, so the slope never contributes and the op is the lookup its
 * source program states: init[i] = value(table[int8(input[i]) + 128]) with value = base >> 8 for an int8 init (the
 * words are sext(lut[i]) << 8; a base whose low byte is not zero is refused) and value = base for an int16 init
 * (the words are zext(lut[i])).  input int8, or int16 of which the low byte is taken as the patterns' trunci does.
 * The table comes either as static_table (static_table_count entries, the attribute a later reference pass folds
 * it into) or as dynamic_table, which must then be a constant int32 tensor (THIP_NO_VALUE when absent); a run-time
 * table is torq_hl.gather in the reference and is not on this path.  Any other scale_bias (the interpolating
 * tables of the bf16 activation functions) is refused: how the ACT unit rounds an interpolated value is not in the
 * sources present. */
typedef struct thip_hl_table_t {
    thip_value_t init;
    thip_value_t scale_bias;
    thip_value_t input;
    thip_value_t dynamic_table;
    const int32_t *static_table;
    int32_t static_table_count;
} thip_hl_table_t;

thip_status_t thip_hl_conv2d(thip_program_t *program, const thip_hl_conv2d_t *op);
thip_status_t thip_hl_depthwise_conv2d(thip_program_t *program,
                                       const thip_hl_depthwise_conv2d_t *op);
thip_status_t thip_hl_fully_connected(thip_program_t *program,
                                      const thip_hl_fully_connected_t *op);
thip_status_t thip_hl_matmul(thip_program_t *program, const thip_hl_matmul_t *op);
thip_status_t thip_hl_maxpool2d(thip_program_t *program, const thip_hl_maxpool2d_t *op);
thip_status_t thip_hl_avg_pool2d(thip_program_t *program, const thip_hl_avg_pool2d_t *op);
thip_status_t thip_hl_add(thip_program_t *program, const thip_hl_add_t *op);
thip_status_t thip_hl_transpose(thip_program_t *program, const thip_hl_transpose_t *op);
thip_status_t thip_hl_expand_weights(thip_program_t *program, const thip_hl_expand_weights_t *op);
thip_status_t thip_hl_fma(thip_program_t *program, const thip_hl_fma_t *op);
thip_status_t thip_hl_mul(thip_program_t *program, const thip_hl_mul_t *op);
thip_status_t thip_hl_elementwiseunary(thip_program_t *program, const thip_hl_elementwiseunary_t *op);
thip_status_t thip_hl_elementwiseshift(thip_program_t *program, const thip_hl_elementwiseshift_t *op);
thip_status_t thip_hl_table(thip_program_t *program, const thip_hl_table_t *op);
thip_status_t thip_hl_act(thip_program_t *program, const thip_hl_act_t *op);
thip_status_t thip_hl_elementwisebinary(thip_program_t *program, const thip_hl_elementwisebinary_t *op);

/* Serialises the program (role of TargetBackend::serializeExecutable,
 * compiler/torq/Target/TorqTarget.cpp:115-151, and serializeTorqHW,
 * compiler/torq/Serialization/Serialization.cpp:265-302): picks a kernel
 * variant per op, pre-packs weights for the MFMA operand layout, splits
 * scale_bias, lays out intermediates.  The blob is malloc'ed; release it with
 * thip_blob_free. */
thip_status_t thip_program_serialize(thip_program_t *program, void **out_blob, size_t *out_size);
void thip_blob_free(void *blob);

/* ------------------------------------------------------------------------ */
/* Run side: device, executable, dispatch                                   */
/* ------------------------------------------------------------------------ */

typedef struct thip_device_t thip_device_t;
typedef struct thip_executable_t thip_executable_t;

/* Opens GPU `ordinal` (role of the driver factory's try_create for "torq",
 * runtime/driver/registration/driver_module.c:95-168).  Fails with
 * THIP_UNAVAILABLE when no gfx950 device is present. */
thip_status_t thip_device_create(int32_t ordinal, thip_device_t **out_device);
void thip_device_destroy(thip_device_t *device);
/* Writes the device's architecture name ("gfx950") into `name`. */
thip_status_t thip_device_name(thip_device_t *device, char *name, size_t capacity);

/* Device memory (role of TorqHw::allocateDeviceBuffer / writeXram / readXram,
 * runtime/torq_hw/inc/TorqHw.h:96-121). */
thip_status_t thip_device_alloc(thip_device_t *device, size_t size, void **out_ptr);
thip_status_t thip_device_free(thip_device_t *device, void *ptr);
thip_status_t thip_device_h2d(thip_device_t *device, void *dst_device, const void *src_host,
                              size_t size);
thip_status_t thip_device_d2h(thip_device_t *device, void *dst_host, const void *src_device,
                              size_t size);
thip_status_t thip_device_synchronize(thip_device_t *device);

/* Calibration for the benchmark (no counterpart in the reference): the rate, in TOP/s with 1 multiply-add = 2 ops,
 * that `workgroups` workgroups of four waves sustain when they issue v_mfma_i32_32x32x32_i8 back to back on
 * register operands and touch no memory.  random_operands != 0: uniformly random operand bytes; 0: every byte 1.
 * The card runs against a power limit, so the two differ: it is the ceiling of any int8 GEMM on such data. */
thip_status_t thip_device_mfma_rate(thip_device_t *device, int32_t random_operands, int32_t workgroups,
                                    int32_t iterations, double *out_tops);

/* Calibration for the benchmark (no counterpart in the reference): microseconds per launch of the fastest of a family
 * of kernels with next to no arithmetic (1 to 8 16-byte items per thread, one pass or a persistent grid-stride grid,
 * default or non-temporal cache policy) that read reads_per_write (1, 2 or 4) 16-byte pieces for every 16 bytes they
 * write, write_bytes written per launch: what this memory system gives a bandwidth-bound op of that size and
 * read/write mix.  cold != 0: every launch on other buffers, more of them than the last-level cache holds.
 * The _tuned form also names the winner ("stream_floor<reads, items per thread, persistent, non-temporal>"). */
thip_status_t thip_device_stream_floor(thip_device_t *device, int32_t reads_per_write, size_t write_bytes,
                                       int32_t cold, double *out_microseconds);
thip_status_t thip_device_stream_floor_tuned(thip_device_t *device, int32_t reads_per_write, size_t write_bytes,
                                             int32_t cold, double *out_microseconds, char *out_variant,
                                             size_t variant_capacity);

/* What a descriptor blob holds, in the terms of the reference's executable schema
 * (runtime/schemas/torq_executable_def.fbs): ExecutableDef :168-197, Binding :28-48, Segment :13-24.  These read
 * the blob only (no device) and validate it first, like thip_descriptor_validate. */
typedef struct thip_descriptor_info_t {
    char executable_name[64];     /* ExecutableDef.executable_name */
    uint32_t runtime_version;     /* ExecutableDef.runtime_version: the descriptor version the runtime gates on */
    uint32_t hw_id;               /* ExecutableDef.hw_id: 950 = gfx950 */
    uint32_t action_count;        /* ExecutableDef.actions: here one kernel record each */
    uint32_t binding_count;       /* ExecutableDef.bindings */
    uint32_t segment_count;       /* ExecutableDef.code: the constant segments uploaded once at create */
    uint32_t intermediate_count;  /* device buffers the executable allocates for itself */
    uint64_t intermediate_bytes;
    uint64_t total_size;
} thip_descriptor_info_t;
thip_status_t thip_descriptor_info(const void *blob, size_t size, thip_descriptor_info_t *out_info);

typedef struct thip_binding_info_t {
    uint32_t id;            /* Binding.id: index into the dispatch's binding table */
    uint64_t address;       /* Binding.address: always 0 (bindings arrive as pointers with each dispatch) */
    uint64_t offset;        /* Binding.offset: always 0 */
    uint64_t size;          /* Binding.size: bytes of the binding the program touches */
    uint8_t is_read_only;   /* Binding.is_read_only */
    uint8_t is_write_only;  /* Binding.is_write_only */
    uint8_t is_used;        /* 0: the id is declared but no kernel touches it */
} thip_binding_info_t;
thip_status_t thip_descriptor_binding(const void *blob, size_t size, uint32_t index,
                                      thip_binding_info_t *out_binding);

typedef struct thip_segment_info_t {
    uint64_t address;     /* Segment.xram_address: here the offset inside the executable's constant buffer */
    uint64_t size;        /* Segment.size */
    const uint8_t *data;  /* Segment.data: points into the blob */
} thip_segment_info_t;
thip_status_t thip_descriptor_segment(const void *blob, size_t size, uint32_t index,
                                      thip_segment_info_t *out_segment);

/* Debug dumps, the roles of the reference's --torq_dump_io_data_dir and --torq_dump_buffers_dir
 * (runtime/driver/TorqDump.cc:34-35,329-428).  io_data_dir: every blocking dispatch writes the raw bytes of its
 * host bindings to <io_data_dir>/thip_dispatch/npu.{in,out}.host_binding.<i>.torq_binding.<i>.bin (the reference's
 * file names).  buffers_dir: dispatches run one kernel record at a time and after record <a> the buffer it wrote
 * is saved as <buffers_dir>/thip_dispatch/action<a>/buffer<id>.npy (a NumPy array; id = binding<k> or temp<k>;
 * activations are N,H,W,C as the kernels hold them), with an index buffers.csv in the reference's columns.
 * NULL or "" switches a dump off.  Dumps are for debugging: they serialise the GPU and copy every result back. */
thip_status_t thip_device_set_dump_dirs(thip_device_t *device, const char *io_data_dir,
                                        const char *buffers_dir);

/* Validates a descriptor blob and writes the format string
 * ("thip-gfx950") -- iree_hal_torq_native_executable_infer_format,
 * runtime/driver/native_executable.cc:151-178. */
thip_status_t thip_infer_format(const void *blob, size_t size, size_t format_capacity,
                                char *format, size_t *out_inferred_size);

/* Everything thip_executable_create checks about a blob before it touches the GPU: header (magic, version,
 * target), table extents, every operand reference and every kernel record's footprint inside the buffer it
 * names, k-table entries inside their windows.  Needs no device.  The blob must be 8-byte aligned.  (The
 * reference verifies its flatbuffer the same way before use, runtime/driver/native_executable.cc:151-170.) */
thip_status_t thip_descriptor_validate(const void *blob, size_t size);

/* Creates an executable from a descriptor: copies the blob, uploads its
 * constant segments, allocates intermediates --
 * iree_hal_torq_native_executable_create, runtime/driver/native_executable.h:42-46,
 * native_executable.cc:41-108.  `constants` are the executable-level constants
 * of iree_hal_executable_params_t (copied; may be NULL when count is 0). */
thip_status_t thip_executable_create(thip_device_t *device, const void *blob, size_t size,
                                     const uint32_t *constants, size_t constant_count,
                                     thip_executable_t **out_executable);
void thip_executable_destroy(thip_executable_t *executable);

/* Binding flags (role of IREE_HAL_TORQ_BINDING_FLAG_ZERO_COPY_*,
 * runtime/driver/torq_command_buffer.h:29-30). */
enum {
    THIP_BINDING_HOST = 0x0,  /* host pointer: staged through device memory */
    THIP_BINDING_DEVICE = 0x1 /* device pointer: used in place */
};

/* The subset of iree_hal_executable_dispatch_state_v0_t that the reference
 * consumes (runtime/driver/torq_command_buffer.c:423-499) plus the per-binding
 * flags of iree_hal_torq_dispatch_state_v0_t (torq_command_buffer.h:17-27).
 * binding_flags may be NULL (all host). */
typedef struct thip_dispatch_state_t {
    uint32_t constant_count;
    const uint32_t *constants;
    uint32_t binding_count;
    void *const *binding_ptrs;
    const size_t *binding_lengths;
    const uint8_t *binding_flags;
} thip_dispatch_state_t;

/* Runs the dispatch and returns when the outputs are in the bindings --
 * iree_hal_torq_native_executable_run, runtime/driver/native_executable.h:57-58,
 * TorqExecutable::executeDispatch, runtime/driver/TorqExecutable.cc:1025-1125.
 * Blocking; one dispatch at a time per executable (internal mutex). */
thip_status_t thip_executable_run(thip_executable_t *executable,
                                  const thip_dispatch_state_t *state);

/* Same dispatch without the final wait: enqueues on the executable's stream.
 * Only device bindings are allowed.  Pair with thip_executable_wait. */
thip_status_t thip_executable_enqueue(thip_executable_t *executable,
                                      const thip_dispatch_state_t *state);
thip_status_t thip_executable_wait(thip_executable_t *executable);

/* Every wait for the GPU (run, wait, time) gives up after this many milliseconds (default 120 000, or the
 * environment's THIP_WAIT_TIMEOUT_MS when the executable is created; <= 0: no limit) and returns THIP_INTERNAL,
 * as the reference turns a hardware wait that exceeds its timeout into IREE_STATUS_INTERNAL
 * (runtime/torq_hw/src/TorqHw.cpp:172-186, runtime/driver/TorqExecutable.cc:640-643).  The executable is then
 * abandoned: its kernels may still be running, every later call on it fails with THIP_FAILED_PRECONDITION, and
 * destroying it leaves its device memory in place.  The process itself stays usable. */
thip_status_t thip_executable_set_wait_timeout(thip_executable_t *executable, int64_t milliseconds);

/* thip_executable_enqueue for callers that cannot allocate device memory at dispatch time (tight serving loops,
 * harnesses that forbid hipMalloc after start-up, a process one of whose other streams is under HIP graph capture,
 * during which allocation is not permitted).  It has no counterpart in the reference.  The dispatch is enqueued on
 * the executable's own stream like every other dispatch (its kernels do not become part of a graph somebody else is
 * capturing), kernel by kernel (no graph is built), on device bindings only, and makes no hipMalloc / hipFree or allocating
 * library call: the scratch memory of the program's kernels (the partial sums of a bf16
 * fully_connected / matmul whose K is split over blocks) is taken from an array that is part of the library's
 * device image instead of the executable's intermediates.  The results are those of thip_executable_enqueue.
 * A program whose kernels need more scratch than the array holds (2 MiB) is refused with
 * THIP_RESOURCE_EXHAUSTED.  Each GPU has one such array, shared by every executable and kept until the process
 * ends: calls that overlap in time on one GPU (from different executables, whose streams differ) race on it, so
 * wait for one to finish before enqueueing the next.  Pair with thip_executable_wait. */
thip_status_t thip_executable_enqueue_noalloc(thip_executable_t *executable,
                                              const thip_dispatch_state_t *state);

/* Enqueues the dispatch `iterations` times between two HIP events recorded on
 * the executable's stream and returns the mean time of one dispatch in
 * milliseconds (role of the per-dispatch profile scopes,
 * runtime/driver/torq_profile_scope.h).  Device bindings only. */
thip_status_t thip_executable_time(thip_executable_t *executable,
                                   const thip_dispatch_state_t *state, int32_t iterations,
                                   float *out_ms_per_dispatch);

/* Same measurement with dispatch i taking states[i % state_count]: with enough distinct buffer sets the working
 * set exceeds the last-level cache and a bandwidth-bound program is timed on memory that is cold in every
 * dispatch.  Device bindings only.  (No counterpart in the reference; benchmark support like the one above.) */
thip_status_t thip_executable_time_rotating(thip_executable_t *executable,
                                            const thip_dispatch_state_t *states, uint32_t state_count,
                                            int32_t iterations, float *out_ms_per_dispatch);

/* Introspection used by the harness and the tests. */
thip_status_t thip_executable_op_count(thip_executable_t *executable, uint32_t *out_count);
/* Name of the kernel that op `index` launches, as a profiler shows it without namespace and argument list
 * (e.g. "igemm_dense_i8<256,256,2,2,4,1,1,0>", "depthwise3x3_strip_i8<2,2,1,3,1>").  It is settled when the
 * executable is created (from the record, the alignment of its operands and the THIP_* environment switches as
 * they are then) and does not change afterwards. */
thip_status_t thip_executable_op_kernel(thip_executable_t *executable, uint32_t index,
                                        char *name, size_t capacity);
thip_status_t thip_executable_binding_count(thip_executable_t *executable, uint32_t *out_count);
thip_status_t thip_executable_binding_size(thip_executable_t *executable, uint32_t binding,
                                           size_t *out_size);

/* The GEMM tile that thip_program_serialize gives an integer conv2d / fully_connected / matmul of M output pixels
 * (rows), N output channels and a reduction of K bytes, without building the program: `addressing` 0 = a dense
 * [M][K] operand (1x1 convolution, fully_connected, matmul), 1 = gathered taps, 2 = whole window rows of a
 * few-channel image, 3 = a KxK window on an image of C channels; `add_follows`: the result's only reader is a
 * torq_hl.add right behind it.  *out_variant is the record's tile number, `name` its tile ("igemm_dense_i8_256x256x64", ...).  The
 * THIP_* tuning switches apply as they do at serialisation.  (The role the kernel selectors of
 * compiler/torq/Conversions/TorqHLToTorqHW/Conv2DToHw.cpp:150-186 play for the NPU; for tuning tools and tests.) */
thip_status_t thip_gemm_tile_choice(int32_t addressing, int64_t M, int64_t N, int64_t K, int64_t C, int32_t out_dtype,
                                    int32_t add_follows, uint32_t *out_variant, char *name, size_t capacity);

/* Per-dispatch event log (role of TorqEventLog, runtime/torq_hw/inc/TorqEventLog.h:19-46, .cpp:48,97-101): when a
 * path is set every dispatch appends rows in the reference's runtime CSV columns (doc/user-manual/profiling.md:53-63)
 * dispatch_name, invocation_id, action_id, timestamp_us, event -- event an EventType name plus _BEGIN / _END:
 * DISPATCH, DISPATCH_SYNC_BINDINGS_IN / _OUT, DISPATCH_EXECUTE_ACTIONS, NSS_START per kernel launch (action_id = the
 * op's index), NSS_WAIT -- and a sixth column, kernel, naming the kernel of a launch row.  An empty path closes the
 * log.  While a log is open dispatches are not replayed as graphs. */
thip_status_t thip_device_set_event_log(thip_device_t *device, const char *csv_path);

#ifdef __cplusplus
}
#endif
#endif /* THIP_H_ */
