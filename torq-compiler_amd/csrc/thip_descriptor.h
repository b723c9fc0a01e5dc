// Dispatch descriptor: the on-disk / in-memory program format that the emitter
// writes and the driver reads.  It plays the role of the reference's "SNPU"
// flatbuffer (runtime/schemas/torq_executable_def.fbs:17-199: code segments,
// binding table, host actions) for a GPU target: a little-endian header, a
// binding table, a table of intermediate buffers, a table of constant
// segments, a list of fixed-size kernel records, and the constant bytes.
// All structs are plain data with explicit sizes; offsets are from the start
// of the blob.
#pragma once

#include <stdint.h>

namespace thip {

constexpr uint32_t kMagic = 0x50494854u;  // "THIP"
constexpr uint32_t kDescriptorVersion = 2;
constexpr uint32_t kArchGfx950 = 950;
constexpr uint64_t kDataAlign = 256;

// Memory spaces an operand reference can name.
enum Space : uint32_t { kSpaceNone = 0, kSpaceBinding = 1, kSpaceTemp = 2, kSpaceConst = 3 };

struct DescRef {
    uint32_t space;
    uint32_t index;
    uint64_t offset;  // bytes into the buffer
};

struct DescHeader {
    uint32_t magic;
    uint32_t version;
    uint32_t arch;
    uint32_t flags;
    uint32_t op_count;
    uint32_t binding_count;
    uint32_t temp_count;
    uint32_t const_count;
    uint64_t ops_offset;
    uint64_t bindings_offset;
    uint64_t temps_offset;
    uint64_t consts_offset;
    uint64_t data_offset;
    uint64_t total_size;
    // name of the hal.executable.export this program was made from (the reference's ExecutableDef.executable_name,
    // runtime/schemas/torq_executable_def.fbs:172-173), NUL-terminated and NUL-padded
    char name[64];
};

enum BindingFlags : uint32_t { kBindingRead = 1, kBindingWritten = 2 };

struct DescBinding {
    uint32_t id;
    uint32_t flags;
    uint64_t size;  // bytes the program touches
};

struct DescTemp {
    uint64_t size;
};

struct DescConst {
    uint64_t offset;  // from DescHeader::data_offset
    uint64_t size;
};

// Kernel kinds.  One record = one kernel launch.
enum Kind : uint32_t {
    kKindTranspose = 1,  // [B, R, S] -> [B, S, R] elements of `gran` bytes (0 or 1: bytes; 2: bf16), output rows TP elements apart
    // conv2d / fully_connected / matmul on MFMA.  A residual add fused by the emitter (pixel-streaming variant, dense
    // loader, int8): in1 = the add's other operand, table = ResidualAddParams (in1.space none: no add)
    kKindIgemm = 2,
    kKindFcSkinny = 3,   // fully_connected with few rows: weight streaming
    kKindDepthwise = 4,
    kKindMaxPool = 5,
    kKindAvgPool = 6,
    kKindAdd = 7,
    kKindAddBf16 = 9,    // bf16 add: w0 / w1 bf16 bits, bias0 / output_min / output_max float bits, C = element count
    kKindIm2colBf16 = 10,     // bf16 N,H,W,C image -> [M][Kp] patch matrix, k = (kh * KW + kw) * C + ci, zero padded
    kKindDepthwiseBf16 = 11,  // bf16 depthwise: weights [KH][KW][C] bf16, bias f32[C]
    // bf16 fully_connected / matmul: fp32 accumulate, float bias, float clamp (output_min/max bits).  loader: weight
    // layout, 0 rows, 1 fragment order, 2 block-quantized int8 in fragment order (a folded torq_hl.expand_weights):
    // scale = bf16 scales [K / gran][Np], table = float biases [K / gran][Np], gran = rows per block, bias0 / scale0
    // = float bits of the expansion's clamp.
    kKindFcBf16 = 8,
    kKindAvgPoolBf16 = 12,    // bf16 global average pool: w0 = bf16 bits of the weight, bias0 = float bits of the bias
    // torq_hl.expand_weights: in0 int8 [K][Nn], scale bf16 [K / gran][Nn], bias float [K / gran][Np], out bf16 [K][Nn]
    kKindExpandWeights = 13,
    // integer elementwise ops: variant = EltwiseOp (0 fma, 1 mul, 2 clamp, 3 abs, 4 negate, 5 i2i, 6 and, 7 or, 8 xor,
    // 9 min, 10 max: two inputs of the output's type, w0 = compare as unsigned), C = element
    // count, gran = input element size, out_dtype, w0 = fma weight, w1 = mul broadcast (1: in0, 2: in1 has one
    // element), bias0 / scale0 / shift / output_zp / output_min / output_max = the ACT stage (fma, mul) or
    // output_min / output_max = the clip range (the others)
    kKindEltwise = 14,
    // Decode-shaped bf16 linear on block-quantized int8 weights (torq_hl.expand_weights folded into torq_hl.matmul),
    // up to three matrices on the same M <= 32 input rows in one launch, the torq_hl.add behind it folded in:
    // in0 = x [M][K] bf16 (K % 128 == 0), gran = rows per quantisation block (a multiple of 128), w0 = number of
    // matrices, w1 = DecLinearFlags, output_min / output_max = float bits of the matmuls' clamp, bias0 / scale0 =
    // float bits of the expansions' clamp, table = a DecLinearExt in the constant segment (the per-matrix operands),
    // out = the first buffer the launch writes, Nn = its row length.
    kKindDecLinear = 15,
    // Batch of small bf16 matmuls against a run-time operand held [N][K]: in0 = a [TB][M][K] (w0 != 0: one [M][K] for
    // every batch), weights = [TB][Nn][K] (w1 != 0: shared), out [TB][M][Nn]; M <= 32; bias0 = float bits of the one
    // bias, output_min / output_max = float bits of the clamp.
    kKindDecMatmul = 16,
};

enum DecLinearFlags : int32_t {
    kDecPair = 1,         // two matrices of equal width; a workgroup owns the same columns of both, the add joins them
    kDecAddResidual = 2,  // add_out = add(res, y) (kDecResFirst) or add(y, res)
    kDecAddPair = 4,      // add_out = add(y0, y1)
    kDecResFirst = 8,
};

// Per-matrix operands of a kKindDecLinear record.  weights: int8 in the dec16 slot order with the block scales (and,
// has_qbias, block biases) inline (thip_kernels.h), bias: float [N], out: bf16 [M][N] (space none: not stored, the
// folded add is its only reader).
struct DecLinearExt {
    DescRef weights[3], bias[3], out[3];
    int32_t N[3];
    int32_t has_qbias;
    DescRef res, add_out;
    int32_t aw0, aw1;           // bf16 bits of the add's two weights
    int32_t abias, alo, ahi;    // float bits of its bias and clamp
    int32_t reserved1[3];
};
static_assert(sizeof(DecLinearExt) == 9 * 16 + 16 + 2 * 16 + 32, "DecLinearExt layout");

// Variants of kKindIgemm: how the A (activation) tile is gathered.
enum IgemmLoader : uint32_t {
    kLoaderDense = 0,   // A is a dense [M, K] matrix with K % 16 == 0
    kLoaderGather = 1,  // implicit-GEMM gather through the k-table, `gran` bytes at a time
    // few input channels (KW * C <= 16): K is laid out as one 16-byte group per window row,
    // [kw][ci] bytes then zero-weight padding, so that a window row is ONE unaligned 16-byte load
    // (what it reads past the KW * C bytes meets zero weights).  Table: one entry per group,
    // kh in bits 24..30, run length KW * C in bits 0..15.
    kLoaderRuns = 2,
    // a convolution window over an image with C % 16 == 0, addressed by the LDS-DMA ring kernel itself: every 16-byte
    // chunk of a k-tile is 16 channels of one tap, K = KH * KW * C, Kp = K rounded up to whole k-tiles (zero weights
    // beyond K).  Table: 128 bytes of input_zp (what a tap outside the image reads).
    kLoaderWindow = 3,
};

// torq_hl.add folded into the epilogue of the convolution that produces one of its operands.
struct ResidualAddParams {
    int32_t w0, w1, bias, scale;             // the add's weights and its one (bias, scale) pair
    int32_t shift, output_zp, output_min, output_max;
    int32_t other_first;                     // the operand read from memory is the add's input1
    int32_t reserved[3];
};
static_assert(sizeof(ResidualAddParams) == 48, "ResidualAddParams layout");

struct DescOp {
    uint32_t kind;
    uint32_t variant;    // tile configuration index (igemm) / vector width (bandwidth kernels)
    uint32_t loader;     // IgemmLoader
    uint32_t gran;       // gather granularity in bytes: 16, 8, 4, 2 or 1
    int32_t out_dtype;   // THIP_DTYPE_*
    int32_t input_zp;
    int32_t output_zp;
    int32_t output_min;
    int32_t output_max;
    int32_t shift;
    // activation geometry (NHWC)
    int32_t N, H, W, C;
    int32_t OH, OW, OC;
    int32_t KH, KW, SH, SW;
    int32_t PL, PR, PT, PB;
    // GEMM view: M x K times (N x K)^T; Kp/Np are the padded sizes of the packed weights
    int32_t M, K, Kp, Nn, Np;
    // uniform parameters (add weights; matmul / avgpool / add single pair)
    int32_t w0, w1;
    int32_t bias0, scale0;
    // transpose: batch, rows, cols
    int32_t TB, TR, TS;
    // igemm / depthwise: left shift of (acc + bias) the emitter proved lossless, with shift + pre_shift == 33
    // (0 = none); lets the kernels requantise with 32-bit arithmetic
    int32_t pre_shift;
    // with pre_shift: clamp (acc + bias) to [-t0_clamp, t0_clamp] first (0 = no clamp).  The emitter sets it
    // when the bound of |acc + bias| is too large for pre_shift but every channel's result already saturates
    // at +-t0_clamp, so the clamp cannot change a result.
    int32_t t0_clamp;
    // transpose: elements from one output row to the next (0: TR, rows packed); a wider pitch leaves the rest of
    // each row as it was (the zero padding of a run-time matmul operand)
    int32_t TP;
    DescRef in0;
    DescRef in1;
    DescRef weights;  // packed weights
    DescRef bias;     // int32[Np] (de-interleaved)
    DescRef scale;    // int32[Np]
    DescRef table;    // k-table of the gather loader
    DescRef out;
};

// k-table entry of the gather loader: one per `gran` bytes of the padded K axis.
// bits 0..15 channel offset, 16..23 kw, 24..30 kh, bit 31 set = beyond K (feeds zeros).
inline uint32_t packKEntry(int kh, int kw, int ci) {
    return (uint32_t)ci | ((uint32_t)kw << 16) | ((uint32_t)kh << 24);
}
constexpr uint32_t kKEntryInvalid = 0x80000000u;

}  // namespace thip
