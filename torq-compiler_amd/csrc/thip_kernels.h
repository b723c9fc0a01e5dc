// Launch interface of the gfx950 kernels.  Host code fills one argument
// struct per launch; every launcher validates what the kernel and its grid
// assume before anything reaches the GPU.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace thip {

// Output requantisation shared by every kernel: the ACT rescale-clamp of the
// reference (compiler/torq/Utils/Kernel.h:610-624).
struct Requant {
    int32_t shift;
    int32_t out_zp;
    int32_t out_min;
    int32_t out_max;
    // 0, or 33 - shift for a shift below 33 when (acc + bias) << pre_shift is known to fit 32 bits:
    // the MFMA and 3x3 depthwise kernels then take their 32-bit tail (the result is the same).
    int32_t pre_shift;
    // > 0 with pre_shift: (acc + bias) is clamped to [-t0_clamp, t0_clamp] before the shift; whoever sets it has
    // checked that every channel's result is already saturated at those values
    int32_t t0_clamp;
};

// Tuning and test switches, read from the environment once per executable (when it is created), never on the launch
// path: a record keeps the kernel it was given for as long as its executable lives.
struct Tuning {
    bool noStreamDeep = false;      // THIP_NO_STREAM_DEEP: pixel-streaming GEMM, no ring over several pixel groups
    bool streamGuarded = false;     // THIP_STREAM_GUARDED: pixel-streaming GEMM, the bounds-checked loop only
    int streamStage = -1;           // THIP_STREAM_STAGE=0 / 1: staged stores never / wherever they fit (-1: by size)
    bool noDirectEpilogue = false;  // THIP_NO_DIRECT_EPILOGUE: dense GEMM, results through LDS
    bool skinnyDot4 = false;        // THIP_SKINNY_DOT4: few-row fully_connected on v_dot4 only
    int depthwiseStrip = -1;        // THIP_DEPTHWISE_STRIP=0 / 1 / 2: rolling-window kernel off / on / on with one column per thread at stride 2
    int depthwiseTile = -1;         // THIP_DEPTHWISE_TILE=0 / 1: register-tile kernel off / on
    long long depthwiseTileMin = 0; // THIP_DEPTHWISE_TILE_MIN: thread-outputs from which the tile kernel is taken
    int depthwisePixels = 0;        // THIP_DEPTHWISE_P: pixels per thread of the window-row kernel
    int fcWideU = 0;                // THIP_FC_WIDE_U: k-steps per register buffer of the wide bf16 kernel
    int fcWideWaves = 0;            // THIP_FC_WIDE_WAVES=4 / 8 / 16: waves per block of the wide bf16 kernel (0: by weight format and rows)
    int denseShortK = 384;          // THIP_DENSE_SHORT_K: padded K up to which the 128 x 128 dense tile runs two stages deep, four blocks per CU
    bool noK128 = false;            // THIP_NO_K128: no 128-byte k-tiles chosen at launch (the emitter reads the same switch for its own choice)
    bool noFcDeep = false;          // THIP_NO_FC_DEEP
    bool noFcWide = false;          // THIP_NO_FC_WIDE
    bool addGeneric = false;        // THIP_ADD_GENERIC: the quantised add always through the 64-bit ACT stage
    bool maxpoolGeneric = false;    // THIP_MAXPOOL_GENERIC: the any-window max pool kernel also for 2 x 2 stride 2
    int decAblate = 0;              // THIP_DEC_ABLATE: parts of dec_linear left out, for timing experiments (wrong results)
    int decTargetGroups = 0;        // THIP_DEC_TARGET_WORKGROUPS: workgroups a dec_linear launch with few column tiles shares its rows out to (0: 256)
};
Tuning tuningFromEnvironment();

// How a launcher is called.  name == nullptr: enqueue the kernel on `stream`.  Otherwise: validate the arguments,
// configure the kernel it would launch (dynamic LDS limit, occupancy query: things that must not happen inside a
// stream capture), write that kernel's name ("kernel<template arguments>") to `name` and enqueue nothing.
struct LaunchCtx {
    hipStream_t stream;
    const Tuning *tuning;
    char *name;
    size_t name_capacity;
};

struct IgemmArgs {
    const int8_t *A;        // activations: NHWC image batch, or dense [M, K]
    const int8_t *Bp;       // packed weights [Np][Kp], K contiguous, zero padded
    const int32_t *bias;    // [Np]
    const int32_t *scale;   // [Np]
    const uint32_t *ktab;   // gather loader only: Kp / gran entries
    void *out;              // [M][N] elements of out_dtype
    int32_t M, N, K, Kp, Np;
    int32_t H, W, C, OH, OW, SH, SW, PT, PL;
    int32_t KH, KW;         // window loader only
    int32_t input_zp;
    int32_t out_dtype;
    int64_t a_bytes;        // size of A in bytes (the run loader keeps its 16-byte loads inside it)
    uint32_t loader;
    uint32_t gran;
    Requant rq;
    // a residual add fused behind the requant (pixel-streaming kernel only; null: none): the other operand, laid
    // out like out, and the parameters of torq_hl.add.  add_skip_first: the other operand is the add's input1.
    const int8_t *skip;
    int32_t add_skip_first, add_w0, add_w1, add_bias, add_scale;
    Requant arq;
    int32_t stream_guarded;  // pixel-streaming kernel: keep every load and store under its bounds check (tests, tuning)
    int32_t stream_stage;    // pixel-streaming kernel: results leave through a per-wave LDS slice as whole rows (its launcher sets it)
};

// Tile configurations of the igemm kernel.
enum IgemmVariant : uint32_t {
    kIgemm128x128x64 = 0,
    kIgemm256x256x64 = 1,
    kIgemm64x64x64 = 2,
    kIgemm256x128x64 = 3,
    // dense [M, K] operand only: tiles moved by LDS DMA through a ring of stages
    kIgemmDense256x256 = 4,
    kIgemmDense128x128 = 5,
    kIgemmDense128x256 = 6,
    kIgemmDense64x64 = 7,
    kIgemmDense256x128 = 8,
    kIgemmDense256x64 = 9,   // narrow-N tiles for the pointwise convolutions of mobile networks
    kIgemmDense256x32 = 10,
    // dense operand, weights of at most 64 KiB resident in LDS, N <= 256, int8 output: streams the pixels
    kIgemmStream = 11,
    kIgemmDense128x64 = 12,  // mid-sized problems: enough tiles to fill the chip at a better ratio of loads to MFMAs than 64x64
    kIgemmDense64x128 = 13,
    kIgemmDense256x256K128 = 14,  // k-tiles of 128 bytes: whole cache lines per tile row, two stages
    kIgemmVariantCount = 15,
};
struct IgemmTile {
    int bm, bn, bk;
    const char *name;
};
const IgemmTile &igemmTile(uint32_t variant);
// The streaming variant splits the (padded) output channels into equal chunks of at most 256, a
// multiple of 32 each; one grid row per chunk, whose weights stay in LDS.
__host__ __device__ inline int igemmStreamChunk(int Np) {
    const int blocks = Np / 32, chunks = (Np + 255) / 256;
    return (blocks + chunks - 1) / chunks * 32;
}
// Whether the streaming variant takes this shape (its launcher checks the same): a chunk of the
// weights fits 64 KiB of LDS, and re-reading the activations once per chunk costs no more than
// the output itself.
inline bool igemmStreamFits(int64_t N, int64_t K, int32_t out_dtype) {
    if (out_dtype != 1 || N <= 0 || K <= 0 || N % 16 != 0 || K % 16 != 0 || N > 65536 || K > 65536) return false;
    const int64_t Np = (N + 31) / 32 * 32, Kp = (K + 31) / 32 * 32;
    const int64_t chunk = igemmStreamChunk((int)Np), chunks = (Np + chunk - 1) / chunk;
    return chunk * Kp + 8 * chunk + Kp / 4 <= 64 * 1024 && (chunks - 1) * K <= N;
}
hipError_t launchIgemm(const IgemmArgs &a, uint32_t variant, const LaunchCtx &ctx);

struct FcSkinnyArgs {
    const int8_t *x;      // [M][K]
    const int8_t *w;      // [N][K] (as given by the op)
    const int32_t *bias;  // [N]
    const int32_t *scale; // [N]
    void *out;            // [M][N]
    int32_t M, N, K;
    int32_t out_dtype;
    Requant rq;
};
constexpr int kFcSkinnyMaxRows = 16;
hipError_t launchFcSkinny(const FcSkinnyArgs &a, const LaunchCtx &ctx);

// bf16 fully_connected: out[m][n] = bf16(clamp(sum_k x[m][k] * w[n][k] + bias[n])), fp32 accumulate.
struct FcBf16Args {
    const uint16_t *x;  // [M][K] bf16 bit patterns
    const uint16_t *w;  // [N][K], or in fragment order (w_fragments)
    const float *bias;  // [N]
    uint16_t *out;      // [M][N]
    int32_t M, K, N;
    float lo, hi;       // clamp (-inf / +inf for none)
    // K split over `ksplit` blocks per output tile (1 = no split): the blocks leave their partial tiles in
    // `workspace` (tiles * ksplit * 1024 floats; nothing in it has to be initialised) and a second kernel adds them.
    int32_t ksplit;
    void *workspace;
    // weights in fragment order: for column block nb (32 columns), k-step s (64 elements) and piece c (0..3),
    // 64 lanes x 16 bytes, lane l = column l & 31, elements 32 (l >> 5) + 8 c .. + 7 of the step; zero padded
    // to whole blocks and steps.  One wave load is then 1 KiB of consecutive memory.
    // 2: block-quantized int8 weights expanded while they are loaded (torq_hl.expand_weights folded into the
    // matmul that consumes it): w then holds int8 in the same order, 64 lanes x 16 bytes per half h2 (0..1) of
    // a step, byte e of lane l = element 32 (l >> 5) + 16 h2 + e; weight (n, k) stands for
    // bf16(clamp(w * qscale[k / qblock][n] + qbias[k / qblock][n], qlo, qhi)).  qblock % 32 == 0; the two
    // tables are qcols (a multiple of 32, >= N) wide.
    int32_t w_fragments;
    const uint16_t *qscale;
    const float *qbias;
    int32_t qblock, qcols;
    float qlo, qhi;
};
// Byte offset of int8 weight (n, k) in the block-quantized fragment order.
inline size_t fcBf16Q8FragmentOffset(int n, int k, int steps) {
    const int nb = n >> 5, r = n & 31, s = k >> 6, kk = k & 63, h = kk >> 5, h2 = (kk & 31) >> 4, e = kk & 15;
    return ((((size_t)nb * steps + s) * 2 + h2) * 64 + (size_t)(h * 32 + r)) * 16 + (size_t)e;
}
// Byte offset of element (n, k) in the fragment order, for K padded to `steps` steps of 64.
inline size_t fcBf16FragmentOffset(int n, int k, int steps) {
    const int nb = n >> 5, r = n & 31, s = k >> 6, kk = k & 63, h = kk >> 5, c = (kk & 31) >> 3, e = kk & 7;
    return ((((size_t)nb * steps + s) * 4 + c) * 64 + (size_t)(h * 32 + r)) * 16 + (size_t)e * 2;
}
// Bytes of workspace a launch with this split needs.
inline size_t fcBf16WorkspaceBytes(int M, int N, int ksplit) {
    const size_t tiles = (size_t)((N + 31) / 32) * ((M + 31) / 32);
    return ksplit <= 1 ? 0 : tiles * ksplit * 1024 * 4;
}
// The split the launcher's heuristics would like for this shape (the emitter allocates the workspace for it).
inline int fcBf16PreferredSplit(int M, int N, int K) {
    const long long tiles = (long long)((N + 31) / 32) * ((M + 31) / 32);
    const int steps = (K + 63) / 64;
    // The second kernel costs a dependent launch (2-3 us): the split pays where a block would otherwise walk a long
    // K alone while most CUs idle (a CU streams 30-50 GB/s whatever its waves do).  About 12 k-steps per block, at
    // most one block per CU (a second round would double the time); measured: 32 x 6912 -> 1152 20.7 us whole, 8.1
    // split 7 ways; 6912 -> 256 20.5 / 7.2; 4096 -> 1024 10.8 / 7.9; 2048 -> 2048 9.4 / 7.1; K = 1152 and 1024: 7.0-7.4
    // whole, 6.7-7.1 split.
    if (steps < 32) return 1;
    long long split = 256 / tiles;
    if (split > (steps + 6) / 12) split = (steps + 6) / 12;
    if (split > 16) split = 16;
    return split < 2 ? 1 : (int)split;
}
hipError_t launchFcBf16(const FcBf16Args &a, const LaunchCtx &ctx);
// ---- decode-shaped bf16 programs: at most 32 input rows, the weights dominate the traffic ---------------------
//
// dec_linear: out[m][n] = bf16(clamp(sum_k x[m][k] * W[k][n] + bias[n])) with W = the expansion of block-quantized
// int8 weights (torq_hl.expand_weights folded into its matmul): W[k][n] = bf16(clamp(w * qscale[k / qblock][n] +
// qbias[k / qblock][n], qlo, qhi)).  One launch serves up to three matrices that read the same input rows
// (`nseg` segments: q, k, v of an attention block), or two matrices of equal width whose results are added
// (`pair`: gate and up), and can apply the torq_hl.add that follows to its result (a residual connection).  A
// workgroup owns 16 output columns: it brings its whole share of the weights into LDS with one burst of LDS-DMA
// loads, its eight to sixteen waves split K, and their partial sums meet in LDS; where few column tiles meet many
// input rows, several workgroups share a tile and take a group of the rows each.
//
// Weight layout ("dec16"): for column tile t (16 columns) and k-block b (128 input rows) one slot of kDecSlotBytes
// (+ 64 with block biases): first 2 KiB of weights, piece p (0, 1) = 64 lanes x 16 bytes, lane l = column l & 15 and
// k-group g = l >> 4; bytes 0..7 of the lane are rows 32 (2 p) + 8 g + 0..7 of the k-block, bytes 8..15 rows
// 32 (2 p + 1) + 8 g + 0..7 (what one lane feeds to two v_mfma_f32_16x16x32_bf16); zero padded to whole k-blocks.
// Then the block's 16 scales as floats (the scale of quantisation block b * 128 / qblock: repeated per k-block, so
// that a workgroup's whole share is one contiguous stretch), then, if the record has block biases, its 16 biases.
constexpr int kDecMaxSegments = 3;
constexpr int kDecMaxRows = 32;
constexpr int kDecSlotBytes = 2048 + 64;
struct DecLinearArgs {
    const uint16_t *x;  // [M][K] bf16
    int32_t M, K, qblock;
    int32_t nseg;       // matrices of this launch, 1..3
    int32_t pair;       // 1: two matrices of equal N; a workgroup owns the same 16 columns of both and adds its two results
    int32_t has_qbias;  // the slots carry block biases (all matrices of a launch, or none)
    const int8_t *w[kDecMaxSegments];
    const float *bias[kDecMaxSegments];   // [N] per matrix
    uint16_t *out[kDecMaxSegments];       // [M][N] per matrix; null: not stored (the fused add is its only reader)
    int32_t N[kDecMaxSegments];           // multiples of 16
    float lo, hi;                         // the matmuls' clamp
    float qlo, qhi;                       // the expansions' clamp
    // the torq_hl.add behind the matmul(s): 0 none; 1 add_out = add(res, y) when res_first, else add(y, res), res laid out
    // like the result (one matrix only); 2 add_out = add(y0, y1) (pair)
    int32_t add_mode, res_first;
    const uint16_t *res;
    uint16_t *add_out;
    float aw0, aw1, abias, alo, ahi;
    int32_t nwaves;  // waves per workgroup; the launcher sets it (decLinearWaves)
    int32_t rows_per_group;  // input rows of a workgroup; the launcher sets it (grid.y workgroups share a column tile)
    int32_t ablate;  // timing experiments only (THIP_DEC_ABLATE; results are wrong): 1 no weight loads, 2 no arithmetic
};
inline int decSlotBytes(bool hasBias) { return kDecSlotBytes + (hasBias ? 64 : 0); }
// Byte offset of int8 weight (n, k) in the dec16 order, for K padded to `kblocks` blocks of 128.
inline size_t decWeightOffset(int n, int k, int kblocks, bool hasBias) {
    const int t = n >> 4, c = n & 15, b = k >> 7, kk = k & 127, j = kk >> 5, g = (kk & 31) >> 3, e = kk & 7;
    return ((size_t)t * kblocks + b) * decSlotBytes(hasBias) + ((size_t)(j >> 1) * 64 + (size_t)(g * 16 + c)) * 16 + (size_t)((j & 1) * 8 + e);
}
// Byte offset of the scale (which = 0) or bias (which = 1) of column n for k-block b.
inline size_t decScaleOffset(int n, int b, int kblocks, bool hasBias, int which) {
    return ((size_t)(n >> 4) * kblocks + b) * decSlotBytes(hasBias) + 2048 + (size_t)which * 64 + (size_t)(n & 15) * 4;
}
inline size_t decWeightBytes(int N, int K, bool hasBias) { return (size_t)((N + 15) / 16) * ((K + 127) / 128) * decSlotBytes(hasBias); }
int decLinearWaves(int K);
hipError_t launchDecLinear(const DecLinearArgs &a, const LaunchCtx &ctx);

// dec_matmul: out[b][m][n] = bf16(clamp(sum_k a[b][m][k] * w[b][n][k] + bias)) for a batch of small matmuls whose
// second operand is a run-time tensor held [N][K] (a key cache; a value cache kept dimension-major): M <= 32 rows
// (the query heads of one sequence), K % 8 == 0.  a_stride / w_stride / out_stride: elements between batches (0:
// the operand is shared by every batch).
struct DecMatmulArgs {
    const uint16_t *a;
    const uint16_t *w;
    uint16_t *out;
    int32_t B, M, K, N;
    int64_t a_stride, w_stride, out_stride;
    float bias, lo, hi;
};
hipError_t launchDecMatmul(const DecMatmulArgs &a, const LaunchCtx &ctx);

// Sustained v_mfma_i32_32x32x32_i8 rate (TOP/s, 1 multiply-add = 2 ops) of `blocks` workgroups of four waves that
// do nothing else, on constant or on random operand bytes.  Allocates and frees its own few KiB.
hipError_t measureMfmaRate(int randomOperands, int blocks, int iterations, hipStream_t stream, double *outTops);

// Microseconds per launch of the fastest of a family of streaming kernels with next to no arithmetic (1, 2, 4 or 8
// 16-byte items per thread, one pass or a persistent grid-stride grid, default or non-temporal cache policy) that
// read readsPerWrite (1, 2 or 4) 16-byte pieces per 16 bytes written, writeBytes written per launch; cold: on
// rotating buffer sets larger than the last-level cache.  outVariant (may be null) receives the winner's name,
// "stream_floor<reads, items per thread, persistent, non-temporal>".  Allocates and frees its buffers.
hipError_t measureStreamRate(int readsPerWrite, size_t writeBytes, int cold, hipStream_t stream, double *outMicroseconds, char *outVariant = nullptr,
                             size_t variantCapacity = 0);

// The library's static scratch array (device memory that needs no allocation): its size and its address on the
// current device (ask once per device, with that device current).
constexpr size_t kStaticScratchBytes = 2u << 20;
hipError_t staticScratchAddress(void **out);

// Integer elementwise ops with the ACT stage behind them.  fma: out = R1(in0 * w0); mul: out = R1(in0 * in1) (an
// input of one element is broadcast); both with ONE (bias, scale) pair.  clamp / abs / negate / i2i: the input
// passed through the mode, then clipped to [lo, hi] and truncated to the output type.
// and / or / xor / min / max: two inputs and the output of one type, no ACT stage; w0 != 0 (16-bit only): min / max
// compare as unsigned.  not: bitwise complement.  greater / greater-equal / equal: two inputs of one integer type
// (w0 != 0, 16-bit only: unsigned), the result one byte of 0 or 1 per element; logical and / or / xor / not: such
// bytes in (non-zero = true), such bytes out.  lsr / lsl / asr: in0 shifted by the counts in in1 (clamped to
// 0 .. bits-1), same type out; w0 != 0: right shifts round half up.  table: out = lut[int8(in0) + 128], in1 = the
// 256 entries of the output's type (int8 or int16); in0 int8 or int16 (its low byte).
enum EltwiseOp : int32_t {
    kEltFma = 0, kEltMul = 1, kEltClamp = 2, kEltAbs = 3, kEltNegate = 4, kEltCast = 5,
    kEltAnd = 6, kEltOr = 7, kEltXor = 8, kEltMin = 9, kEltMax = 10,
    kEltNot = 11, kEltGreater = 12, kEltGreaterEqual = 13, kEltEqual = 14,
    kEltLogicalAnd = 15, kEltLogicalOr = 16, kEltLogicalXor = 17, kEltLogicalNot = 18,
    kEltLsr = 19, kEltLsl = 20, kEltAsr = 21,
    kEltTable = 22,
    kEltLast = kEltTable,
};
// Ops that read a second tensor, and those whose result has the inputs' element type.
__host__ __device__ inline bool eltwiseTwoInputs(int32_t op) {
    return op == kEltMul || (op >= kEltAnd && op <= kEltMax) || (op >= kEltGreater && op <= kEltLogicalXor) || op >= kEltLsr;
}
__host__ __device__ inline bool eltwiseSameType(int32_t op) {
    return (op >= kEltAnd && op <= kEltNot) || (op >= kEltLogicalAnd && op <= kEltLogicalNot) || (op >= kEltLsr && op <= kEltAsr);
}
struct EltwiseArgs {
    const void *in0;
    const void *in1;  // mul and the two-input ops
    void *out;
    int64_t count;
    int32_t op;
    int32_t in_bytes, out_bytes;  // 1, 2 or 4 (int8 / int16 / int32)
    int32_t bcast;                // mul: 0 none, 1 in0 has one element, 2 in1 has one element
    int32_t w0, bias, scale;
    int32_t lo, hi;               // clamp / abs / negate / i2i
    Requant rq;                   // fma / mul
};
hipError_t launchEltwise(const EltwiseArgs &a, const LaunchCtx &ctx);

// bf16 global average pool: out[n][c] = bf16(clamp(sum_u in[n][u][c] * weight + bias)), summed over the frame
// in order, in fp32.
struct AvgPoolBf16Args {
    const uint16_t *in;  // [N][HW][C]
    uint16_t *out;       // [N][C]
    int32_t N, HW, C;
    float weight, bias, lo, hi;
};
hipError_t launchAvgPoolBf16(const AvgPoolBf16Args &a, const LaunchCtx &ctx);

// torq_hl.expand_weights: out[k][n] = bf16(clamp(w[k][n] * scale[k / block][n] + bias[k / block][n])).
struct ExpandWeightsArgs {
    const int8_t *w;        // [K][N]
    const uint16_t *scale;  // [K / block][N] bf16
    const float *bias;      // [K / block][bias_cols]
    uint16_t *out;          // [K][N]
    int32_t K, N, block, bias_cols;
    float lo, hi;
};
hipError_t launchExpandWeights(const ExpandWeightsArgs &a, const LaunchCtx &ctx);

struct DepthwiseArgs {
    const int8_t *in;     // NHWC
    const int8_t *wpk;    // variant 0: [KH][KW][C] bytes; variant 1: [KH][C] dwords, byte kw of a dword = tap kw
    const int32_t *bias;  // [C]
    const int32_t *scale; // [C]
    int8_t *out;          // NHWC
    int32_t N, H, W, C, OH, OW, KH, KW, SH, SW, PT, PL;
    int32_t input_zp;
    uint32_t variant;     // DepthwiseVariant
    Requant rq;
};
enum DepthwiseVariant : uint32_t {
    kDepthwiseGeneric = 0,  // any window, any channel count
    kDepthwiseDot4Rows = 1, // 3x3 window, C % 16 == 0: one v_dot4 per window row and channel
};
hipError_t launchDepthwise(const DepthwiseArgs &a, const LaunchCtx &ctx);

struct MaxPoolArgs {
    const int8_t *in;  // NHWC
    int8_t *out;       // NHWC
    int32_t N, H, W, C, OH, OW, KH, KW, SH, SW, PT, PL;
    int32_t input_zp, out_min, out_max;
};
hipError_t launchMaxPool(const MaxPoolArgs &a, const LaunchCtx &ctx);

struct AvgPoolArgs {
    const int8_t *in;  // [N][HW][C]
    int8_t *out;       // [N][C]
    int32_t N, HW, C;
    int32_t weight, bias, scale;
    Requant rq;
};
hipError_t launchAvgPool(const AvgPoolArgs &a, const LaunchCtx &ctx);

struct AddArgs {
    const int8_t *in0;
    const int8_t *in1;
    int8_t *out;
    int64_t count;
    int32_t w0, w1, bias, scale;
    Requant rq;
};
hipError_t launchAdd(const AddArgs &a, const LaunchCtx &ctx);

// bf16 patch matrix of a convolution: out[m][k] with m = (n * OH + oy) * OW + ox and k = (kh * KW + kw) * C + ci,
// rows padded with zeros to Kp; positions outside the image are zero.
struct Im2colBf16Args {
    const uint16_t *in;  // NHWC
    uint16_t *out;       // [M][Kp]
    int32_t N, H, W, C, OH, OW, KH, KW, SH, SW, PT, PL, Kp;
};
hipError_t launchIm2colBf16(const Im2colBf16Args &a, const LaunchCtx &ctx);

// bf16 depthwise convolution: fp32 accumulation over (kh, kw), float bias and clamp.
struct DepthwiseBf16Args {
    const uint16_t *in;   // NHWC
    const uint16_t *wpk;  // [KH][KW][C]
    const float *bias;    // [C]
    uint16_t *out;        // NHWC
    int32_t N, H, W, C, OH, OW, KH, KW, SH, SW, PT, PL;
    float lo, hi;
};
hipError_t launchDepthwiseBf16(const DepthwiseBf16Args &a, const LaunchCtx &ctx);

// bf16 add: out = bf16(clamp(in0 * w0 + in1 * w1 + bias)) in fp32.
struct AddBf16Args {
    const uint16_t *in0;
    const uint16_t *in1;
    uint16_t *out;
    int64_t count;
    float w0, w1, bias, lo, hi;
};
hipError_t launchAddBf16(const AddBf16Args &a, const LaunchCtx &ctx);

struct TransposeArgs {
    const int8_t *in;  // [B][R][S]
    int8_t *out;       // [B][S][R]
    int32_t B, R, S;
    int32_t elem;      // element size in bytes: 1 or 2
    int32_t out_pitch; // elements between output rows (>= R); the batch stride of the output is S * out_pitch
};
hipError_t launchTranspose(const TransposeArgs &a, const LaunchCtx &ctx);

}  // namespace thip
