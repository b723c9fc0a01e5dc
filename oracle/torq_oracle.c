/*
 * CPU oracle for the quantized TorqHL operator path.  TEST INFRASTRUCTURE ONLY
 * (see torq_oracle.h).  Plain C, int64 intermediates, straightforward loop
 * nests; OpenMP over the outermost independent loop so that the same code
 * doubles as the timed CPU baseline.
 */
#include "torq_oracle.h"

#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

static int g_threads = 0; /* 0 = OpenMP default */

int torq_oracle_threads(void) {
#ifdef _OPENMP
    return g_threads > 0 ? g_threads : omp_get_max_threads();
#else
    return 1;
#endif
}

void torq_oracle_set_threads(int n) {
    g_threads = n;
#ifdef _OPENMP
    if (n > 0) {
        omp_set_num_threads(n);
    }
#endif
}

/*
 * R1 -- ACT rescaleClamp.
 * Pseudocode: compiler/torq/Utils/Kernel.h:610-624.  The shift is act_rsh
 * bits (0..63): third_party/torq-hw/ct/torq_api.c:572-583 (act_sh obsolete,
 * torq_api.h:82-83).  Rounding NTP = nearest, tie towards +inf:
 * compiler/torq/Dialect/TorqHW/TorqHWAttrs.td:123-136, default for
 * EasyKernel lowerings compiler/torq/Serialization/DescGen.cpp:271-291.
 * t0 is an int32 add (two's-complement wrap here; callers keep it in range).
 */
int64_t torq_act_rescale_clamp(int32_t acc, int32_t bias, int32_t scale, const torq_requant_t *rq) {
    int32_t t0 = (int32_t)((uint32_t)acc + (uint32_t)bias);
    int64_t t1 = (int64_t)t0 * (int64_t)scale;
    int sh = rq->shift;
    int64_t t2 = sh > 0 ? t1 + ((int64_t)1 << (sh - 1)) : t1;
    int64_t t3 = t2 >> sh; /* arithmetic shift */
    int64_t t4 = t3 + (int64_t)rq->output_zp;
    if (t4 < rq->output_min) t4 = rq->output_min;
    if (t4 > rq->output_max) t4 = rq->output_max;
    return t4;
}

static inline void store_elem(void *out, size_t idx, int64_t v, int bytes) {
    switch (bytes) {
    case 1: ((int8_t *)out)[idx] = (int8_t)v; break;
    case 2: ((int16_t *)out)[idx] = (int16_t)v; break;
    default: ((int32_t *)out)[idx] = (int32_t)v; break;
    }
}

static int bad_out_bytes(int b) { return !(b == 1 || b == 2 || b == 4); }

/* Strides (in elements) of a 4-D activation tensor for the chosen layout. */
typedef struct {
    size_t n, c, h, w;
} strides4_t;

static strides4_t act_strides(int layout, int C, int H, int W) {
    strides4_t s;
    if (layout == TORQ_LAYOUT_NHWC) {
        s.c = 1;
        s.w = (size_t)C;
        s.h = (size_t)W * C;
        s.n = (size_t)H * W * C;
    } else {
        s.w = 1;
        s.h = (size_t)W;
        s.c = (size_t)H * W;
        s.n = (size_t)C * H * W;
    }
    return s;
}

static int out_dim(int in, int k, int64_t p0, int64_t p1, int64_t stride) {
    int64_t span = (int64_t)in + p0 + p1 - k;
    if (span < 0 || stride <= 0) return 0;
    return (int)(span / stride) + 1;
}

/*
 * torq_hl.conv2d -- signature compiler/torq/Dialect/TorqHL/TorqHLOps.td:119-143;
 * executed loop nest compiler/torq/Conversions/TorqHLToTorqHW/Conv2DToHw.cpp:150-186:
 * for every output pixel and output channel, accumulate over (ic, kh, kw) the
 * product of the padded input and the weight, then rescaleClamp with the
 * channel's (bias, scale).  Padding value is input_zp (Conv2DToHw.cpp:117-121).
 */
int torq_conv2d(const int8_t *input, const int8_t *weights, const int32_t *scale_bias, void *out,
                int N, int C, int H, int W, int O, int KH, int KW, const int64_t pad[4],
                const int64_t stride[2], int32_t input_zp, const torq_requant_t *rq, int layout,
                int out_elem_bytes) {
    if (bad_out_bytes(out_elem_bytes)) return -1;
    const int64_t pl = pad[0], pr = pad[1], pt = pad[2], pb = pad[3];
    const int64_t sh = stride[0], sw = stride[1];
    const int OH = out_dim(H, KH, pt, pb, sh), OW = out_dim(W, KW, pl, pr, sw);
    const strides4_t is = act_strides(layout, C, H, W);
    const strides4_t os = act_strides(layout, O, OH, OW);
#pragma omp parallel for collapse(2) schedule(static)
    for (int n = 0; n < N; n++) {
        for (int oy = 0; oy < OH; oy++) {
            for (int ox = 0; ox < OW; ox++) {
                for (int o = 0; o < O; o++) {
                    int32_t acc = 0;
                    for (int kh = 0; kh < KH; kh++) {
                        const int64_t iy = (int64_t)oy * sh - pt + kh;
                        for (int kw = 0; kw < KW; kw++) {
                            const int64_t ix = (int64_t)ox * sw - pl + kw;
                            const int inside = iy >= 0 && iy < H && ix >= 0 && ix < W;
                            const int8_t *wp = weights + (((size_t)o * C) * KH + kh) * KW + kw;
                            const size_t wstep = (size_t)KH * KW;
                            if (inside) {
                                const int8_t *ip = input + n * is.n + (size_t)iy * is.h + (size_t)ix * is.w;
                                for (int ic = 0; ic < C; ic++) {
                                    acc += (int32_t)ip[ic * is.c] * (int32_t)wp[ic * wstep];
                                }
                            } else {
                                for (int ic = 0; ic < C; ic++) {
                                    acc += input_zp * (int32_t)wp[ic * wstep];
                                }
                            }
                        }
                    }
                    int64_t q = torq_act_rescale_clamp(acc, scale_bias[2 * o], scale_bias[2 * o + 1], rq);
                    store_elem(out, n * os.n + (size_t)o * os.c + (size_t)oy * os.h + (size_t)ox * os.w, q,
                               out_elem_bytes);
                }
            }
        }
    }
    return 0;
}

/*
 * torq_hl.depthwise_conv2d -- signature TorqHLOps.td:145-170; weights C x 1 x KH x KW
 * (compiler/torq/Conversions/LinalgToTorqHL/Conv2DPattern.cpp:404-424); executed
 * compiler/torq/Conversions/TorqHLToTorqHW/DWToHw.cpp:223-251.
 */
int torq_depthwise_conv2d(const int8_t *input, const int8_t *weights, const int32_t *scale_bias,
                          void *out, int N, int C, int H, int W, int KH, int KW,
                          const int64_t pad[4], const int64_t stride[2], int32_t input_zp,
                          const torq_requant_t *rq, int layout, int out_elem_bytes) {
    if (bad_out_bytes(out_elem_bytes)) return -1;
    const int64_t pl = pad[0], pr = pad[1], pt = pad[2], pb = pad[3];
    const int64_t sh = stride[0], sw = stride[1];
    const int OH = out_dim(H, KH, pt, pb, sh), OW = out_dim(W, KW, pl, pr, sw);
    const strides4_t is = act_strides(layout, C, H, W);
    const strides4_t os = act_strides(layout, C, OH, OW);
#pragma omp parallel for collapse(2) schedule(static)
    for (int n = 0; n < N; n++) {
        for (int oy = 0; oy < OH; oy++) {
            for (int ox = 0; ox < OW; ox++) {
                for (int c = 0; c < C; c++) {
                    int32_t acc = 0;
                    for (int kh = 0; kh < KH; kh++) {
                        const int64_t iy = (int64_t)oy * sh - pt + kh;
                        for (int kw = 0; kw < KW; kw++) {
                            const int64_t ix = (int64_t)ox * sw - pl + kw;
                            int32_t x = input_zp;
                            if (iy >= 0 && iy < H && ix >= 0 && ix < W) {
                                x = input[n * is.n + (size_t)c * is.c + (size_t)iy * is.h + (size_t)ix * is.w];
                            }
                            acc += x * (int32_t)weights[((size_t)c * KH + kh) * KW + kw];
                        }
                    }
                    int64_t q = torq_act_rescale_clamp(acc, scale_bias[2 * c], scale_bias[2 * c + 1], rq);
                    store_elem(out, n * os.n + (size_t)c * os.c + (size_t)oy * os.h + (size_t)ox * os.w, q,
                               out_elem_bytes);
                }
            }
        }
    }
    return 0;
}

/*
 * torq_hl.fully_connected -- signature TorqHLOps.td:172-190; weights [N(out), K(in)]
 * (compiler/torq/Conversions/LinalgToTorqHL/Conv2DMatmulPattern.cpp:121-125);
 * executed compiler/torq/Conversions/TorqHLToTorqHW/FCToHw.cpp:55-76:
 * acc[m][n] = sum_k x[m][k] * w[n][k], rescaleClamp with pair n.
 */
int torq_fully_connected(const int8_t *input, const int8_t *weights, const int32_t *scale_bias,
                         void *out, int M, int K, int N, const torq_requant_t *rq,
                         int out_elem_bytes) {
    if (bad_out_bytes(out_elem_bytes)) return -1;
#pragma omp parallel for collapse(2) schedule(static)
    for (int m = 0; m < M; m++) {
        for (int n = 0; n < N; n++) {
            const int8_t *x = input + (size_t)m * K;
            const int8_t *w = weights + (size_t)n * K;
            int32_t acc = 0;
            for (int k = 0; k < K; k++) {
                acc += (int32_t)x[k] * (int32_t)w[k];
            }
            int64_t q = torq_act_rescale_clamp(acc, scale_bias[2 * n], scale_bias[2 * n + 1], rq);
            store_elem(out, (size_t)m * N + n, q, out_elem_bytes);
        }
    }
    return 0;
}

/*
 * torq_hl.matmul -- signature TorqHLOps.td:85-99; executed
 * compiler/torq/Conversions/TorqHLToTorqHW/MatMulPattern.cpp:66-86: batch
 * broadcast allowed, ONE (bias, scale) pair loaded before the loops (:66).
 */
int torq_matmul(const int8_t *input1, const int8_t *input2, const int32_t *scale_bias, void *out,
                int B, int M, int K, int N, int bcast1, int bcast2, const torq_requant_t *rq,
                int out_elem_bytes) {
    if (bad_out_bytes(out_elem_bytes)) return -1;
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < B; b++) {
        for (int m = 0; m < M; m++) {
            const int8_t *a = input1 + (bcast1 ? 0 : (size_t)b * M * K) + (size_t)m * K;
            const int8_t *bm = input2 + (bcast2 ? 0 : (size_t)b * K * N);
            for (int n = 0; n < N; n++) {
                int32_t acc = 0;
                for (int k = 0; k < K; k++) {
                    acc += (int32_t)a[k] * (int32_t)bm[(size_t)k * N + n];
                }
                int64_t q = torq_act_rescale_clamp(acc, scale_bias[0], scale_bias[1], rq);
                store_elem(out, ((size_t)b * M + m) * N + n, q, out_elem_bytes);
            }
        }
    }
    return 0;
}

/*
 * bf16 rows.  With floating-point partials the ACT stage has no scale and no shift
 * (compiler/torq/Utils/Kernel.h:626-632):
 *     float t0 = pdata + bias;   float t1 = t0 < clipMin ? clipMin : t0 > clipMax ? clipMax : t0;   qdata = t1
 * with the clamp bounds given as float bit patterns (compiler/torq/Utils/ConversionUtils.cpp:33-39: -inf / +inf
 * when there is no clamp).  The products of two bf16 values are exact in fp32; they are accumulated in fp32 in
 * k order (the ALU's scalarProductAccumulate loop, compiler/torq/Conversions/TorqHLToTorqHW/MatMulPattern.cpp:66-78)
 * and the result is rounded to bf16 to nearest even, which is what the reference's own expected values use
 * (python/torq/testing/numpy.py:42-53, float32 matmul cast to the output type).
 */
float torq_bf16_to_f32(uint16_t h) {
    union {
        uint32_t u;
        float f;
    } v;
    v.u = (uint32_t)h << 16;
    return v.f;
}

uint16_t torq_f32_to_bf16(float f) {
    union {
        uint32_t u;
        float f;
    } v;
    v.f = f;
    if ((v.u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((v.u >> 16) | 0x0040u); /* NaN stays NaN */
    return (uint16_t)((v.u + 0x7fffu + ((v.u >> 16) & 1u)) >> 16);
}

static float float_from_bits(int32_t bits) {
    union {
        int32_t i;
        float f;
    } v;
    v.i = bits;
    return v.f;
}

static uint16_t act_float(float acc, float bias, float lo, float hi) {
    float t0 = acc + bias;
    float t1 = t0 < lo ? lo : (t0 > hi ? hi : t0);
    return torq_f32_to_bf16(t1);
}

int torq_fully_connected_bf16(const uint16_t *input, const uint16_t *weights, const float *bias,
                              uint16_t *out, int M, int K, int N, int32_t clip_min, int32_t clip_max) {
    const float lo = float_from_bits(clip_min), hi = float_from_bits(clip_max);
#pragma omp parallel for collapse(2) schedule(static)
    for (int m = 0; m < M; m++) {
        for (int n = 0; n < N; n++) {
            const uint16_t *x = input + (size_t)m * K, *w = weights + (size_t)n * K;
            float acc = 0.0f;
            for (int k = 0; k < K; k++) acc += torq_bf16_to_f32(x[k]) * torq_bf16_to_f32(w[k]);
            out[(size_t)m * N + n] = act_float(acc, bias[n], lo, hi);
        }
    }
    return 0;
}

int torq_matmul_bf16(const uint16_t *input1, const uint16_t *input2, const float *bias, uint16_t *out,
                     int B, int M, int K, int N, int bcast1, int bcast2, int32_t clip_min, int32_t clip_max) {
    const float lo = float_from_bits(clip_min), hi = float_from_bits(clip_max);
#pragma omp parallel for collapse(2) schedule(static)
    for (int b = 0; b < B; b++) {
        for (int m = 0; m < M; m++) {
            const uint16_t *a = input1 + (bcast1 ? 0 : (size_t)b * M * K) + (size_t)m * K;
            const uint16_t *bm = input2 + (bcast2 ? 0 : (size_t)b * K * N);
            for (int n = 0; n < N; n++) {
                float acc = 0.0f;
                for (int k = 0; k < K; k++) acc += torq_bf16_to_f32(a[k]) * torq_bf16_to_f32(bm[(size_t)k * N + n]);
                out[((size_t)b * M + m) * N + n] = act_float(acc, bias[0], lo, hi);
            }
        }
    }
    return 0;
}

/*
 * torq_hl.conv2d / depthwise_conv2d on bf16 -- the loop nests of the int8 ops
 * (compiler/torq/Conversions/TorqHLToTorqHW/Conv2DToHw.cpp:150-186, DWToHw.cpp:223-251) with bf16 operands
 * (Conv2DPattern.cpp:96-106: alu_format = act_format = BF, 4-byte bias, no scale), fp32 accumulation over
 * (kh, kw, ic), and the float ACT stage.  The padding value is the op's input_zp, which is 0 for bf16 tensors:
 * positions outside the image contribute nothing.
 */
int torq_conv2d_bf16(const uint16_t *input, const uint16_t *weights, const float *bias, uint16_t *out,
                     int N, int C, int H, int W, int O, int KH, int KW, const int64_t pad[4],
                     const int64_t stride[2], int32_t clip_min, int32_t clip_max, int layout) {
    const float lo = float_from_bits(clip_min), hi = float_from_bits(clip_max);
    const int64_t pl = pad[0], pr = pad[1], pt = pad[2], pb = pad[3];
    const int64_t sh = stride[0], sw = stride[1];
    const int OH = out_dim(H, KH, pt, pb, sh), OW = out_dim(W, KW, pl, pr, sw);
    const strides4_t is = act_strides(layout, C, H, W);
    const strides4_t os = act_strides(layout, O, OH, OW);
#pragma omp parallel for collapse(2) schedule(static)
    for (int n = 0; n < N; n++) {
        for (int oy = 0; oy < OH; oy++) {
            for (int ox = 0; ox < OW; ox++) {
                for (int o = 0; o < O; o++) {
                    float acc = 0.0f;
                    for (int kh = 0; kh < KH; kh++) {
                        const int64_t iy = (int64_t)oy * sh - pt + kh;
                        for (int kw = 0; kw < KW; kw++) {
                            const int64_t ix = (int64_t)ox * sw - pl + kw;
                            if (iy < 0 || iy >= H || ix < 0 || ix >= W) continue;
                            const uint16_t *wp = weights + (((size_t)o * C) * KH + kh) * KW + kw;
                            const uint16_t *ip = input + n * is.n + (size_t)iy * is.h + (size_t)ix * is.w;
                            for (int ic = 0; ic < C; ic++) {
                                acc += torq_bf16_to_f32(ip[ic * is.c]) * torq_bf16_to_f32(wp[(size_t)ic * KH * KW]);
                            }
                        }
                    }
                    out[n * os.n + (size_t)o * os.c + (size_t)oy * os.h + (size_t)ox * os.w] = act_float(acc, bias[o], lo, hi);
                }
            }
        }
    }
    return 0;
}

int torq_depthwise_conv2d_bf16(const uint16_t *input, const uint16_t *weights, const float *bias, uint16_t *out,
                               int N, int C, int H, int W, int KH, int KW, const int64_t pad[4],
                               const int64_t stride[2], int32_t clip_min, int32_t clip_max, int layout) {
    const float lo = float_from_bits(clip_min), hi = float_from_bits(clip_max);
    const int64_t pl = pad[0], pr = pad[1], pt = pad[2], pb = pad[3];
    const int64_t sh = stride[0], sw = stride[1];
    const int OH = out_dim(H, KH, pt, pb, sh), OW = out_dim(W, KW, pl, pr, sw);
    const strides4_t is = act_strides(layout, C, H, W);
    const strides4_t os = act_strides(layout, C, OH, OW);
#pragma omp parallel for collapse(2) schedule(static)
    for (int n = 0; n < N; n++) {
        for (int oy = 0; oy < OH; oy++) {
            for (int ox = 0; ox < OW; ox++) {
                for (int c = 0; c < C; c++) {
                    float acc = 0.0f;
                    for (int kh = 0; kh < KH; kh++) {
                        const int64_t iy = (int64_t)oy * sh - pt + kh;
                        for (int kw = 0; kw < KW; kw++) {
                            const int64_t ix = (int64_t)ox * sw - pl + kw;
                            if (iy < 0 || iy >= H || ix < 0 || ix >= W) continue;
                            acc += torq_bf16_to_f32(input[n * is.n + (size_t)c * is.c + (size_t)iy * is.h + (size_t)ix * is.w]) *
                                   torq_bf16_to_f32(weights[((size_t)c * KH + kh) * KW + kw]);
                        }
                    }
                    out[n * os.n + (size_t)c * os.c + (size_t)oy * os.h + (size_t)ox * os.w] = act_float(acc, bias[c], lo, hi);
                }
            }
        }
    }
    return 0;
}

/*
 * torq_hl.add on bf16 -- compiler/torq/Conversions/TorqHLToTorqHW/AddPattern.cpp:262-281 with floating-point
 * partials: the two products (exact in fp32) are accumulated in tensor order, then the float ACT stage
 * (one bias: biasScaleWidth is 1 for bf16, AddPattern.cpp:118-121,197-200).
 */
int torq_add_bf16(const uint16_t *input1, const uint16_t *input2, const uint16_t weights[2], const float *bias,
                  uint16_t *out, size_t count, int32_t clip_min, int32_t clip_max) {
    const float lo = float_from_bits(clip_min), hi = float_from_bits(clip_max);
    const float w0 = torq_bf16_to_f32(weights[0]), w1 = torq_bf16_to_f32(weights[1]);
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < count; i++) {
        float acc = torq_bf16_to_f32(input1[i]) * w0;
        acc += torq_bf16_to_f32(input2[i]) * w1;
        out[i] = act_float(acc, bias[0], lo, hi);
    }
    return 0;
}

/*
 * torq_hl.avg_pool2d on bf16 -- created compiler/torq/Conversions/LinalgToTorqHL/PoolingPattern.cpp:448-457
 * (ONE bf16 weight: 1.0, or the constant of a mulf/divf that follows the pool, folded in; scale_bias is a
 * single float bias 0.0; clamp at -inf/+inf); executed by the same slice program as the int8 op
 * (compiler/torq/Conversions/TorqHLToTorqHW/AvgpoolPattern.cpp:67-83): for each channel the products
 * x[u] * w are accumulated over the frame u = 0 .. H*W-1 in order, in fp32, then the float ACT stage.
 */
int torq_avg_pool2d_bf16(const uint16_t *input, uint16_t weight, const float *bias, uint16_t *out,
                         int N, int H, int W, int C, int32_t clip_min, int32_t clip_max) {
    const float lo = float_from_bits(clip_min), hi = float_from_bits(clip_max);
    const float w = torq_bf16_to_f32(weight);
    const size_t HW = (size_t)H * W;
#pragma omp parallel for collapse(2) schedule(static)
    for (int n = 0; n < N; n++) {
        for (int c = 0; c < C; c++) {
            float acc = 0.0f;
            for (size_t u = 0; u < HW; u++) acc += torq_bf16_to_f32(input[((size_t)n * HW + u) * C + c]) * w;
            out[(size_t)n * C + c] = act_float(acc, bias[0], lo, hi);
        }
    }
    return 0;
}

/*
 * torq_hl.expand_weights -- signature TorqHLOps.td:943-957; created for the right-hand side of a matmul by
 * compiler/torq/Conversions/LinalgToTorqHL/MatmulPattern.cpp:596-680 (weights [G, B, N] flattened to [K, N],
 * scales [G, N], scale_bias = the float bias -zero_point * scale, [G, cols rounded up to even]
 * MatmulPattern.cpp:322-400; clamp = the float range -inf/+inf); executed
 * compiler/torq/Conversions/TorqHLToTorqHW/ExpandWeightsPattern.cpp:42-98: per block of `block_size` rows
 * one scale and one bias per column, out = weight * scale (elementwise product in fp32, exact for an 8-bit
 * weight and a bf16 scale) then the float ACT stage (+ bias, clamp, round to bf16).
 */
int torq_expand_weights(const int8_t *weights, const uint16_t *scale, const float *bias, uint16_t *out,
                        int K, int N, int block_size, int bias_cols, int32_t clip_min, int32_t clip_max) {
    const float lo = float_from_bits(clip_min), hi = float_from_bits(clip_max);
    if (block_size <= 0 || K % block_size != 0 || bias_cols < N) return -1;
#pragma omp parallel for schedule(static)
    for (int k = 0; k < K; k++) {
        const size_t g = (size_t)(k / block_size);
        for (int n = 0; n < N; n++) {
            const float p = (float)weights[(size_t)k * N + n] * torq_bf16_to_f32(scale[g * N + n]);
            out[(size_t)k * N + n] = act_float(p, bias[g * bias_cols + n], lo, hi);
        }
    }
    return 0;
}

/*
 * torq_hl.maxpool2d -- signature TorqHLOps.td:435-453; created
 * compiler/torq/Conversions/LinalgToTorqHL/PoolingPattern.cpp:199-236 (pad value
 * becomes input_zp, output_min/max = element type range); executed
 * compiler/torq/Conversions/TorqHLToTorqHW/MaxPool2dToHw.cpp:28-333 (ALU MAX
 * accumulate, ACT load: no rescale).
 */
int torq_maxpool2d(const int8_t *input, int8_t *out, int N, int C, int H, int W, int KH, int KW,
                   const int64_t pad[4], const int64_t stride[2], int32_t input_zp,
                   int32_t output_min, int32_t output_max, int layout) {
    const int64_t pl = pad[0], pr = pad[1], pt = pad[2], pb = pad[3];
    const int64_t sh = stride[0], sw = stride[1];
    const int OH = out_dim(H, KH, pt, pb, sh), OW = out_dim(W, KW, pl, pr, sw);
    const strides4_t is = act_strides(layout, C, H, W);
    const strides4_t os = act_strides(layout, C, OH, OW);
#pragma omp parallel for collapse(2) schedule(static)
    for (int n = 0; n < N; n++) {
        for (int oy = 0; oy < OH; oy++) {
            for (int ox = 0; ox < OW; ox++) {
                for (int c = 0; c < C; c++) {
                    int32_t best = INT32_MIN;
                    for (int kh = 0; kh < KH; kh++) {
                        const int64_t iy = (int64_t)oy * sh - pt + kh;
                        for (int kw = 0; kw < KW; kw++) {
                            const int64_t ix = (int64_t)ox * sw - pl + kw;
                            int32_t x = input_zp;
                            if (iy >= 0 && iy < H && ix >= 0 && ix < W) {
                                x = input[n * is.n + (size_t)c * is.c + (size_t)iy * is.h + (size_t)ix * is.w];
                            }
                            if (x > best) best = x;
                        }
                    }
                    if (best < output_min) best = output_min;
                    if (best > output_max) best = output_max;
                    out[n * os.n + (size_t)c * os.c + (size_t)oy * os.h + (size_t)ox * os.w] = (int8_t)best;
                }
            }
        }
    }
    return 0;
}

/*
 * torq_hl.avg_pool2d -- signature TorqHLOps.td:192-208; global only
 * (compiler/torq/Conversions/LinalgToTorqHL/PoolingPattern.cpp:289-291); executed
 * compiler/torq/Conversions/TorqHLToTorqHW/AvgpoolPattern.cpp:67-83: per channel,
 * scalar-product-accumulate the whole frame with the single weight, then
 * rescaleClamp with bias/scale pair 0 (:58-59).  Input NHWC (:36).
 */
int torq_avg_pool2d(const int8_t *input, int8_t weight, const int32_t *scale_bias, int8_t *out,
                    int N, int H, int W, int C, const torq_requant_t *rq) {
    const size_t frame = (size_t)H * W;
#pragma omp parallel for collapse(2) schedule(static)
    for (int n = 0; n < N; n++) {
        for (int c = 0; c < C; c++) {
            int32_t acc = 0;
            const int8_t *p = input + (size_t)n * frame * C + c;
            for (size_t u = 0; u < frame; u++) {
                acc += (int32_t)p[u * C] * (int32_t)weight;
            }
            out[(size_t)n * C + c] = (int8_t)torq_act_rescale_clamp(acc, scale_bias[0], scale_bias[1], rq);
        }
    }
    return 0;
}

/*
 * torq_hl.add -- signature TorqHLOps.td:48-69; executed
 * compiler/torq/Conversions/TorqHLToTorqHW/AddPattern.cpp:262-281:
 * acc = in1*w[0] + in2*w[1] (int16 weights), rescaleClamp with one pair.
 */
int torq_add(const int8_t *input1, const int8_t *input2, const int16_t weights[2],
             const int32_t scale_bias[2], int8_t *out, size_t count, const torq_requant_t *rq) {
    const int32_t w0 = weights[0], w1 = weights[1];
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < count; i++) {
        int32_t acc = (int32_t)input1[i] * w0 + (int32_t)input2[i] * w1;
        out[i] = (int8_t)torq_act_rescale_clamp(acc, scale_bias[0], scale_bias[1], rq);
    }
    return 0;
}

static inline int64_t load_elem(const void *in, size_t idx, int bytes) {
    switch (bytes) {
    case 1: return ((const int8_t *)in)[idx];
    case 2: return ((const int16_t *)in)[idx];
    default: return ((const int32_t *)in)[idx];
    }
}

/*
 * torq_hl.fma -- signature TorqHLOps.td:926-941; the stand-alone rescale, created
 * compiler/torq/Conversions/LinalgToTorqHL/Patterns.cpp:1896-1946 (weight 1, bias = -input_zp, scale = the
 * multiplier, shift_factor = the shift); executed compiler/torq/Conversions/TorqHLToTorqHW/FMAPattern.cpp:19-50:
 * acc = input * weights[0] (one scalar weight), rescaleClamp with ONE (bias, scale) pair.
 */
int torq_fma(const void *input, int in_bytes, int32_t weight, const int32_t scale_bias[2], void *out, int out_bytes,
             size_t count, const torq_requant_t *rq) {
    if (bad_out_bytes(in_bytes) || bad_out_bytes(out_bytes)) return -1;
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < count; i++) {
        const int32_t acc = (int32_t)((uint32_t)load_elem(input, i, in_bytes) * (uint32_t)weight);
        store_elem(out, i, torq_act_rescale_clamp(acc, scale_bias[0], scale_bias[1], rq), out_bytes);
    }
    return 0;
}

/*
 * torq_hl.mul -- signature TorqHLOps.td:101-117; created
 * compiler/torq/Conversions/LinalgToTorqHL/MulPattern.cpp:178-212,354-378 (no input zero points: bias 0 or the
 * folded constant, one scale, `shift`); executed compiler/torq/Conversions/TorqHLToTorqHW/MulPattern.cpp:19-62:
 * the inputs broadcast to the output, acc = input1 * input2 elementwise, rescaleClamp with ONE pair.
 * count1 / count2: elements of each input, `count` or 1 (a one-element tensor is broadcast).
 */
int torq_mul(const void *input1, size_t count1, const void *input2, size_t count2, int in_bytes,
             const int32_t scale_bias[2], void *out, int out_bytes, size_t count, const torq_requant_t *rq) {
    if (bad_out_bytes(in_bytes) || bad_out_bytes(out_bytes)) return -1;
    if ((count1 != count && count1 != 1) || (count2 != count && count2 != 1)) return -1;
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < count; i++) {
        const int64_t a = load_elem(input1, count1 == 1 ? 0 : i, in_bytes), b = load_elem(input2, count2 == 1 ? 0 : i, in_bytes);
        const int32_t acc = (int32_t)((uint32_t)(int32_t)a * (uint32_t)(int32_t)b);
        store_elem(out, i, torq_act_rescale_clamp(acc, scale_bias[0], scale_bias[1], rq), out_bytes);
    }
    return 0;
}

/*
 * torq_hl.act on integers -- signature TorqHLOps.td:291-309; executed
 * compiler/torq/Conversions/TorqHLToTorqHW/ActPattern.cpp:60-140,196-212: the ALU passes the input through and
 * the ACT unit applies `mode`, then clips: "clamp" clips to [min_int, max_int]; "abs" and "negate" clip to the
 * range of the output type (abs(-128) is 127 in int8; the zero-point attributes are not read by the lowering);
 * "i2i" clips to the int32 range, i.e. converts by truncation.
 * mode: 0 clamp, 1 abs, 2 negate, 3 i2i.
 */
int torq_act(const void *input, int in_bytes, void *out, int out_bytes, size_t count, int mode, int64_t min_int,
             int64_t max_int) {
    if (bad_out_bytes(in_bytes) || bad_out_bytes(out_bytes) || mode < 0 || mode > 3) return -1;
    int64_t lo = min_int, hi = max_int;
    if (mode == 1 || mode == 2) {
        lo = out_bytes == 1 ? INT8_MIN : out_bytes == 2 ? INT16_MIN : INT32_MIN;
        hi = out_bytes == 1 ? INT8_MAX : out_bytes == 2 ? INT16_MAX : INT32_MAX;
    } else if (mode == 3) {
        lo = INT32_MIN;
        hi = INT32_MAX;
    }
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < count; i++) {
        int64_t v = load_elem(input, i, in_bytes);
        if (mode == 1) v = v < 0 ? -v : v;
        if (mode == 2) v = -v;
        v = v < lo ? lo : (v > hi ? hi : v);
        store_elem(out, i, v, out_bytes);
    }
    return 0;
}

/*
 * torq_hl.elementwisebinary -- signature TorqHLOps.td:248-260, modes TorqHLAttrs.td:219-235; executed
 * compiler/torq/Conversions/TorqHLToTorqHW/ElementWiseBinaryPattern.cpp:93-107 (ALU op1 modes BAND / BOR / BXOR /
 * MIN / MAX on two tensors of one element type, no ACT rescale) and :70-84 (16-bit operands compare as unsigned
 * when is_unsigned is set).  mode: 0 and, 1 or, 2 xor, 4 minimum, 5 maximum (the enum's values).
 */
int torq_elementwise_binary(int mode, const void *input1, const void *input2, int bytes, int is_unsigned, void *out, size_t count) {
    if (bad_out_bytes(bytes) || !(mode == 0 || mode == 1 || mode == 2 || mode == 4 || mode == 5)) return -1;
    if (is_unsigned && bytes != 2) return -1;
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < count; i++) {
        const int64_t a = load_elem(input1, i, bytes), b = load_elem(input2, i, bytes);
        int64_t r;
        switch (mode) {
        case 0: r = a & b; break;
        case 1: r = a | b; break;
        case 2: r = a ^ b; break;
        default: {
            const int64_t ka = is_unsigned ? (a & 0xffff) : a, kb = is_unsigned ? (b & 0xffff) : b;
            r = (mode == 4) == (ka < kb) ? a : b;
            break;
        }
        }
        store_elem(out, i, r, bytes);
    }
    return 0;
}

/*
 * The comparisons and logical modes of torq_hl.elementwisebinary (TorqHLAttrs.td:226-231: GREATER 6, GREATER_EQUAL 7,
 * EQUAL 8, LOGICAL_AND 9, LOGICAL_OR 10, LOGICAL_XOR 11), created from arith.cmpi / cmpf and i1 and / or / xor
 * (compiler/torq/Conversions/LinalgToTorqHL/ArithToTorqHLPattern.cpp:104-131,181-222; a "less" predicate arrives
 * with its inputs swapped, "not equal" as EQUAL followed by LOGICAL_NOT :239-251).  The result is an i1 tensor:
 * one byte per element holding 0 or 1.  What pins the values is the arith op each mode replaces; the NPU's own
 * encoding of a truth value before its right shift by 16 (ElementWiseBinaryPattern.cpp:108-119) is internal to it.
 * Logical modes read i1 bytes (any non-zero byte is true).  is_unsigned (16-bit operands only, as :70-79).
 */
int torq_elementwise_compare(int mode, const void *input1, const void *input2, int bytes, int is_unsigned, uint8_t *out, size_t count) {
    if (bad_out_bytes(bytes) || mode < 6 || mode > 11) return -1;
    if (is_unsigned && bytes != 2) return -1;
    if (mode >= 9 && bytes != 1) return -1;
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < count; i++) {
        int64_t a = load_elem(input1, i, bytes), b = load_elem(input2, i, bytes);
        if (is_unsigned) {
            a &= 0xffff;
            b &= 0xffff;
        }
        int r;
        switch (mode) {
        case 6: r = a > b; break;
        case 7: r = a >= b; break;
        case 8: r = a == b; break;
        case 9: r = (a != 0) && (b != 0); break;
        case 10: r = (a != 0) || (b != 0); break;
        default: r = (a != 0) != (b != 0); break;
        }
        out[i] = (uint8_t)r;
    }
    return 0;
}

/*
 * torq_hl.elementwiseunary -- signature TorqHLOps.td:262-273; modes BITWISE_NOT (3) and LOGICAL_NOT (12), created
 * from arith.xori with an all-ones constant (ArithToTorqHLPattern.cpp:322-340: LOGICAL_NOT when the result is i1);
 * executed ElementWiseUnaryPattern.cpp:31-36 (ALU op1 BNOT / NOT).  BITWISE_NOT complements every bit of an
 * int8 / int16 / int32 element; LOGICAL_NOT maps an i1 byte to 1 if it is zero, else 0.
 */
int torq_elementwise_unary(int mode, const void *input, int bytes, void *out, size_t count) {
    if (bad_out_bytes(bytes) || !(mode == 3 || mode == 12) || (mode == 12 && bytes != 1)) return -1;
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < count; i++) {
        const int64_t a = load_elem(input, i, bytes);
        store_elem(out, i, mode == 3 ? ~a : (int64_t)(a == 0), bytes);
    }
    return 0;
}

/*
 * torq_hl.elementwiseshift -- signature TorqHLOps.td:275-289, modes TorqHLAttrs.td:239-246 (LSR 0, LSL 1, ASR 2; ASL
 * is refused by the lowering, ElementWiseShiftPattern.cpp:77-90); both inputs and the result share one integer type,
 * input2 holds the shift count of each element.  `round` selects the ACT rounding mode NTP (:91-93); the op stands
 * for exactly this arithmetic (ArithToTorqHLPattern.cpp:367-379, the linalg body RoundingRightShiftPattern matches):
 *     r = x >> s;  if (s > 0 && ((x >> (s - 1)) & 1)) r += 1
 * i.e. round half up, on the signed value for ASR and on the unsigned bit pattern for LSR.  LSL drops the bits
 * shifted out.  Counts must lie in 0 .. bits-1 (arith.shrsi / shli are undefined beyond); here they are clamped.
 */
int torq_elementwise_shift(int mode, int round, const void *input1, const void *input2, int bytes, void *out, size_t count) {
    if (bad_out_bytes(bytes) || mode < 0 || mode > 2) return -1;
    const int bits = 8 * bytes;
    const uint64_t mask = bits == 32 ? 0xffffffffull : ((1ull << bits) - 1);
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < count; i++) {
        const int64_t x = load_elem(input1, i, bytes);
        int64_t s = load_elem(input2, i, bytes);
        s = s < 0 ? 0 : (s > bits - 1 ? bits - 1 : s);
        int64_t r;
        if (mode == 1) {
            r = (int64_t)(((uint64_t)x << s) & mask);
        } else {
            const int64_t v = mode == 2 ? x : (int64_t)((uint64_t)x & mask);
            r = v >> s;
            if (round && s > 0 && ((v >> (s - 1)) & 1)) r += 1;
        }
        store_elem(out, i, r, bytes);  /* keeps the low `bits` bits */
    }
    return 0;
}

/*
 * torq_hl.table -- signature and segment-word format TorqHLOps.td:311-327: word = (slope << 16) | (base & 0xFFFF).
 * The ACT stage first applies the one (bias, scale) pair (TablePattern.cpp:58-63: rescaleClamp with shift 0), which
 * yields a 16-bit 9.7 fixed-point number; its upper nine bits, read as signed, select the entry (-256 .. 255 ->
 * 0 .. 511) and its lower seven are the fraction the slope is multiplied with (TablePattern.cpp:20-27).  The lookup
 * patterns (LinalgToTorqHL/ExtractPattern.cpp:56-62) pass bias -128 and scale 128, so the fraction is zero, the
 * slope contributes nothing and the selected entry is int8(x) + 128 of a 256-entry table: the op then equals the
 * program it replaced, out = lut[x + 128] (ExtractPattern.cpp:285-298 for an int8 table packed as sext(v) << 8,
 * :432-545 for an int16 table packed as zext(v); an int16 input is truncated to int8 first, :485-497).  The value
 * of an entry is base >> 8 for an int8 result and base for an int16 result.
 * How an interpolated value (non-zero fraction) is rounded is not in the sources present: such an input returns -1,
 * as does an int8 result from a base with a non-zero low byte and an index beyond the table.
 */
int torq_table(const void *input, int in_bytes, const int32_t *table, int table_count, int32_t bias, int32_t scale, void *out, int out_bytes, size_t count) {
    if ((in_bytes != 1 && in_bytes != 2) || (out_bytes != 1 && out_bytes != 2) || table_count <= 0) return -1;
    int bad = 0;
#pragma omp parallel for schedule(static) reduction(| : bad)
    for (size_t i = 0; i < count; i++) {
        const int64_t x = (int8_t)(load_elem(input, i, in_bytes) & 0xff);
        const int64_t t = (x + bias) * (int64_t)scale;
        const int16_t fixed = (int16_t)(uint16_t)((uint64_t)t & 0xffffu);
        const int frac = fixed & 127, index = (fixed >> 7) + 256;
        if (frac != 0 || index < 0 || index >= table_count) {
            bad |= 1;
            continue;
        }
        const int16_t base = (int16_t)(uint16_t)((uint32_t)table[index] & 0xffffu);
        if (out_bytes == 1 && (base & 0xff)) {
            bad |= 1;
            continue;
        }
        store_elem(out, i, out_bytes == 1 ? base >> 8 : base, out_bytes);
    }
    return bad ? -1 : 0;
}

/* ---- R2 ---- */

/* compiler/torq/Utils/ConversionUtils.cpp:122-141 (per_channel_sum). */
void torq_per_channel_sum(const int8_t *weights, int channels, int per_channel, int64_t *sums) {
    for (int o = 0; o < channels; o++) {
        int64_t s = 0;
        for (int i = 0; i < per_channel; i++) s += weights[(size_t)o * per_channel + i];
        sums[o] = s;
    }
}

/*
 * shift_factor = min_c shift[c]: compiler/torq/Conversions/LinalgToTorqHL/PatternUtils.cpp:3230-3283;
 * scale[c] = multiplier[c] >> (shift[c] - shift_factor) (arith.shrsi): PatternUtils.cpp:3536-3548;
 * bias[c] = tosa_bias[c] - weight_sum[c] * input_zp: compiler/torq/Utils/ConversionUtils.h:301-329;
 * interleave [bias, scale]: compiler/torq/Utils/ConversionUtils.cpp:88-103.
 */
int32_t torq_derive_scale_bias(const int32_t *multiplier, const int8_t *shift,
                               const int32_t *tosa_bias, const int64_t *weight_sum,
                               int32_t input_zp, int channels, int32_t *scale_bias) {
    int32_t min_shift = INT8_MAX;
    for (int c = 0; c < channels; c++) {
        if (shift[c] < min_shift) min_shift = shift[c];
    }
    for (int c = 0; c < channels; c++) {
        int64_t b = (int64_t)(tosa_bias ? tosa_bias[c] : 0) -
                    (weight_sum ? weight_sum[c] : 0) * (int64_t)input_zp;
        scale_bias[2 * c] = (int32_t)b;
        scale_bias[2 * c + 1] = multiplier[c] >> (shift[c] - min_shift);
    }
    return min_shift;
}

/*
 * compiler/torq/Conversions/LinalgToTorqHL/ElementWiseBinaryPattern.cpp:459-487,
 * 564-597: S = 2^12, weights = (int16)trunc(m_k * S) (w1 times sign),
 * bias = -trunc(m0*S*zp0) - sign*trunc(m1*S*zp1), scale = 1, shift 12.
 * doubleToInt is a C cast: compiler/torq/Utils/TorqUtils.h:55-62.
 */
int torq_derive_add_params(double m0, double m1, int32_t zp0, int32_t zp1, int sign,
                           int16_t weights[2], int32_t scale_bias[2], int32_t *shift_factor) {
    const int sh = 12;
    const int scale_factor = 1 << sh;
    if (m0 * scale_factor > INT16_MAX || m0 * scale_factor < INT16_MIN ||
        m1 * scale_factor > INT16_MAX || m1 * scale_factor < INT16_MIN) {
        return -1;
    }
    int16_t w0 = (int16_t)(m0 * scale_factor);
    int32_t b0 = -(int32_t)(m0 * scale_factor * zp0);
    int16_t w1 = (int16_t)((int16_t)(m1 * scale_factor) * sign);
    int32_t b1 = -(int32_t)(m1 * scale_factor * zp1) * sign;
    weights[0] = w0;
    weights[1] = w1;
    scale_bias[0] = b0 + b1;
    scale_bias[1] = 1;
    *shift_factor = sh;
    return 0;
}

/*
 * compiler/torq/Conversions/LinalgToTorqHL/PoolingPattern.cpp:325-328 (scale =
 * int32(1.0 * 2^shift / itemsPerChannel), bias = -scInfo.bias) with shift 20
 * (:598,600); the folded pre-scale subtract constant of a TFLite-origin mean is
 * H*W*input_zp.
 */
void torq_derive_avgpool_params(int H, int W, int32_t input_zp, int32_t scale_bias[2],
                                int32_t *shift_factor) {
    const int sh = 20;
    const int items = H * W;
    scale_bias[0] = -(items * input_zp);
    scale_bias[1] = (int32_t)(1.0 * (double)(1 << sh) / items);
    *shift_factor = sh;
}
