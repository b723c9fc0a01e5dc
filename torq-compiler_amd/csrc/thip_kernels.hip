// gfx950 (CDNA4) kernels of the quantized TorqHL operator path.
//
//   igemm_i8      conv2d / fully_connected / matmul as implicit GEMM on
//                 v_mfma_i32_32x32x32_i8, LDS double-buffered tiles, requant fused
//                 on the accumulator registers.
//   fc_skinny     fully_connected with at most 16 rows: weight streaming with
//                 v_dot4_i32_i8 and wave-shuffle reductions (HBM bound).
//   depthwise / maxpool / avgpool / add / transpose: bandwidth-bound kernels
//                 with 128-bit accesses on NHWC tensors.
//
// Every kernel ends with the reference's ACT rescale-clamp
// (compiler/torq/Utils/Kernel.h:610-624): int32 add of the bias, 32x32->64 bit
// multiply by the scale, add of 2^(shift-1), arithmetic right shift, add of the
// output zero point, clamp.
#include "thip_kernels.h"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <initializer_list>
#include <mutex>
#include <string>
#include <type_traits>
#include <vector>

#include "thip_descriptor.h"

namespace thip {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kDtypeI8 = 1, kDtypeI16 = 2, kDtypeI32 = 3;

// "name<a,b,...>": the kernel instantiation as a profiler shows it (without its namespace and argument list).
static std::string kernelLabel(const char *name, std::initializer_list<int> params) {
    std::string s = name;
    char sep = '<';
    for (int v : params) {
        s += sep;
        s += std::to_string(v);
        sep = ',';
    }
    return s + ">";
}
static const char *labelText(const char *s) { return s; }
static const char *labelText(const std::string &s) { return s.c_str(); }
// A launch site.  With ctx.name set the launcher is only asked which kernel it would launch for these arguments (the
// driver asks once per record when an executable is created): the name is written and nothing is enqueued.
#define THIP_ENQUEUE(ctx, label, kernel, grid, block, lds, ...)                           \
    do {                                                                                  \
        if ((ctx).name) {                                                                 \
            snprintf((ctx).name, (ctx).name_capacity, "%s", labelText(label));            \
        } else {                                                                          \
            hipLaunchKernelGGL(kernel, grid, block, lds, (ctx).stream, __VA_ARGS__);      \
        }                                                                                 \
    } while (0)

__device__ __forceinline__ int32_t requant(int32_t acc, int32_t bias, int32_t scale, long long rnd,
                                           const Requant &rq) {
    const int32_t t0 = (int32_t)((uint32_t)acc + (uint32_t)bias);
    const long long t3 = ((long long)t0 * (long long)scale + rnd) >> rq.shift;
    // clamp(t3 + zp, min, max) == clamp(t3, min - zp, max - zp) + zp; the bounds cannot overflow
    // 64 bits, and the sum of the low words is exact because the result fits 32 bits
    const long long lo = (long long)rq.out_min - (long long)rq.out_zp;
    const long long hi = (long long)rq.out_max - (long long)rq.out_zp;
    uint32_t q = (uint32_t)t3;
    q = t3 < lo ? (uint32_t)lo : q;
    q = t3 > hi ? (uint32_t)hi : q;
    return (int32_t)(q + (uint32_t)rq.out_zp);
}

// Same result when shift >= 33, with 32-bit work only.  Write the product as H * 2^32 + L.  The
// rounding term 2^(shift-1) is then a multiple of 2^32, so it adds r = 2^(shift-33) to H, and
// floor((H + r + L / 2^32) / 2^(shift-32)) = (H + r) >> (shift - 32) because L / 2^32 < 1 cannot
// carry an integer across a multiple of 2^(shift-32).  |H| <= 2^30 and r <= 2^29: no overflow.
// A smaller shift gets there through rq.pre_shift = 33 - shift: t0 * 2^pre * scale >> (shift + pre)
// is the same number, provided t0 * 2^pre still fits 32 bits; whoever fills rq.pre_shift has
// bounded |t0| from the weights and the bias to make sure of that, or passes rq.t0_clamp: t0 is
// then clamped to a range that fits, chosen so wide that every result outside it is saturated by
// the output clamp anyway (the result is monotonic in t0).  Where no clamp is needed the kernels do not shift
// at all: the bound says that the result fits 32 bits, so it is read out of the 64-bit sum directly
// (requantPreShift).  shift == 32 needs neither: the result is the high word of product + 2^31.
struct WideRequant {
    bool on;  // rq.shift + rq.pre_shift >= 33, or rq.shift == 32
    int pre, shiftMinus32;
    int32_t rnd, lo, hi, zp;
    long long rnd64;     // added to the 64-bit product: rnd * 2^32 adds rnd to the product's high word
    int32_t t0lo, t0hi;  // clamp of acc + bias (the whole int32 range when rq.t0_clamp == 0)
    bool plain;          // on, pre == 0, no clamp of t0, zero point folded: requantWideT0<true> applies
    bool preOnly;        // on, pre > 0, no clamp of t0, zero point folded: requantPreShift applies
    int alignShift;      // preOnly: rq.shift (3..31)
    long long rndAlign;  // preOnly: 2^(shift-1) + zp * 2^shift, added to the product before its bits [shift, shift+32) are taken
};
__device__ __forceinline__ WideRequant wideRequant(const Requant &rq) {
    WideRequant w;
    // shift == 32: the result is the high word of product + 2^31, exact for every acc + bias; a pre-shift or a clamp
    // of acc + bias that the op carries is not needed (either changes nothing in the result)
    const bool whole = rq.shift == 32;
    const int sh = whole ? 32 : rq.shift + rq.pre_shift;
    w.on = sh >= 32;
    w.pre = whole ? 0 : rq.pre_shift;
    w.shiftMinus32 = sh - 32;
    w.rnd = sh >= 33 ? (int32_t)(1u << (sh - 33)) : 0;
    const long long lo64 = (long long)rq.out_min - rq.out_zp, hi64 = (long long)rq.out_max - rq.out_zp;
    w.lo = (int32_t)(lo64 < INT32_MIN ? INT32_MIN : lo64);
    w.hi = (int32_t)(hi64 > INT32_MAX ? INT32_MAX : hi64);
    w.zp = rq.out_zp;
    const bool clampT0 = !whole && rq.t0_clamp > 0;
    w.t0lo = clampT0 ? -rq.t0_clamp : INT32_MIN;
    w.t0hi = clampT0 ? rq.t0_clamp : INT32_MAX;
    // ((H + r) >> s) + zp == (H + r + zp * 2^s) >> s: fold the zero point into the rounding term
    // where that cannot overflow (|H| <= 2^30, r <= 2^29, so |zp| * 2^s up to 2^29 is safe)
    if (w.on && w.shiftMinus32 <= 13 && rq.out_zp >= -32768 && rq.out_zp <= 32767 && rq.out_min <= rq.out_max) {
        w.rnd += rq.out_zp * (1 << w.shiftMinus32);  // |out_zp| < 2^15 (checked when the program is built)
        w.lo = rq.out_min;
        w.hi = rq.out_max;
        w.zp = 0;
    }
    w.rnd64 = (long long)w.rnd * 4294967296LL + (whole ? 2147483648LL : 0LL);  // rnd may be negative (a folded negative zero point)
    w.plain = w.on && w.pre == 0 && !clampT0 && w.zp == 0;
    w.preOnly = w.on && w.pre > 0 && !clampT0 && w.zp == 0;
    w.alignShift = rq.shift & 31;
    w.rndAlign = (w.preOnly ? 1LL << (w.alignShift - 1) : 0LL) + (long long)rq.out_zp * (1LL << w.alignShift);
    return w;
}
// `v` has to be the result of an ordinary VALU instruction the compiler emitted (every caller passes a shift's):
// the compiler does not look into the asm for the wait states that the result of a dot-product instruction needs
// before another kind of VALU instruction may read it, and a v_med3 issued right behind a v_dot4c reads a stale value.
__device__ __forceinline__ int32_t med3(int32_t v, int32_t lo, int32_t hi) {
    int32_t r;
    asm("v_med3_i32 %0, %1, %2, %3" : "=v"(r) : "v"(v), "v"(lo), "v"(hi));
    return r;
}
// High word of t0 * scale, plus the rounding term: one v_mad_i64_i32 (full rate) instead of a v_mul_hi_i32 and an
// add.  |t0 * scale| < 2^62 and rnd * 2^32 < 2^62: the sum cannot overflow.
__device__ __forceinline__ int32_t mulhiPlusRnd(int32_t t0, int32_t scale, const WideRequant &w) {
    return (int32_t)(((long long)t0 * (long long)scale + w.rnd64) >> 32);
}
// `t0` is acc + bias (with int32 wrap).  PLAIN: no pre-shift, no clamp of t0, zero point folded into the
// rounding term (WideRequant::plain), which is the usual case and four instructions shorter.
template <bool PLAIN>
__device__ __forceinline__ int32_t requantWideT0(int32_t t0, int32_t scale, const WideRequant &w) {
    if (PLAIN) return med3(mulhiPlusRnd(t0, scale, w) >> w.shiftMinus32, w.lo, w.hi);
    // t0 may come straight out of a dot product (accumulators that start at the bias): clamp it with compiler-visible code
    t0 = t0 < w.t0lo ? w.t0lo : t0;
    t0 = t0 > w.t0hi ? w.t0hi : t0;
    t0 = (int32_t)((uint32_t)t0 << w.pre);
    const int32_t t3 = med3(mulhiPlusRnd(t0, scale, w) >> w.shiftMinus32, w.lo, w.hi);  // lo <= hi
    return (int32_t)((uint32_t)t3 + (uint32_t)w.zp);
}
// The tail of an op with a shift below 32 and a proven bound |acc + bias| < 2^(31 - pre) = 2^(shift - 2), no clamp of
// t0 and the zero point folded (WideRequant::preOnly).  |t0 * scale| < 2^(shift + 29), so the rounded, shifted sum
// fits 32 bits and is bits [shift, shift + 32) of the 64-bit sum: one v_mad_i64_i32 and one v_alignbit_b32, the
// same number as shifting t0 left by pre first and the high word right afterwards, two instructions shorter.
__device__ __forceinline__ int32_t requantPreShift(int32_t t0, int32_t scale, const WideRequant &w) {
    const long long sum = (long long)t0 * (long long)scale + w.rndAlign;
    return med3((int32_t)__builtin_amdgcn_alignbit((uint32_t)(sum >> 32), (uint32_t)sum, (uint32_t)w.alignShift), w.lo, w.hi);
}
__device__ __forceinline__ int32_t requantWideShift(int32_t acc, int32_t bias, int32_t scale, const WideRequant &w) {
    return requantWideT0<false>((int32_t)((uint32_t)acc + (uint32_t)bias), scale, w);
}
// The requant tails as a compile-time choice made once per kernel: f(tag) with tag::value
// 0 = generic 64-bit, 1 = 32-bit general, 2 = 32-bit plain, 3 = 32-bit pre-shifted only.
template <typename F>
__device__ __forceinline__ void withRequantMode(const WideRequant &w, F &&f) {
    if (!w.on) {
        f(std::integral_constant<int, 0>{});
    } else if (w.plain) {
        f(std::integral_constant<int, 2>{});
    } else if (w.preOnly) {
        f(std::integral_constant<int, 3>{});
    } else {
        f(std::integral_constant<int, 1>{});
    }
}
template <int MODE>
__device__ __forceinline__ int32_t requantT0(int32_t t0, int32_t scale, long long rnd, const Requant &rq, const WideRequant &w) {
    if (MODE == 0) return requant(t0, 0, scale, rnd, rq);
    if (MODE == 3) return requantPreShift(t0, scale, w);
    return requantWideT0<MODE == 2>(t0, scale, w);
}
// Four requantised values (each within int8 after the clamp) as the bytes of one dword.
__device__ __forceinline__ uint32_t packBytes(int32_t a, int32_t b, int32_t c, int32_t d) {
    const uint32_t ab = __builtin_amdgcn_perm((uint32_t)b, (uint32_t)a, 0x0c0c0400u);  // [a.0, b.0, 0, 0]
    const uint32_t cd = __builtin_amdgcn_perm((uint32_t)d, (uint32_t)c, 0x04000c0cu);  // [0, 0, c.0, d.0]
    return ab | cd;
}

// float -> bfloat16 bit pattern.
__device__ __forceinline__ uint16_t bf16Bits(float f) {
    const uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);  // NaN stays NaN
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);                      // nearest, ties to even
}

__device__ __forceinline__ long long roundTerm(int shift) {
    return shift > 0 ? (1LL << (shift - 1)) : 0LL;
}

__device__ __forceinline__ void storeElem(void *out, size_t idx, int32_t v, int dtype) {
    if (dtype == kDtypeI8) {
        ((int8_t *)out)[idx] = (int8_t)v;
    } else if (dtype == kDtypeI16) {
        ((int16_t *)out)[idx] = (int16_t)v;
    } else {
        ((int32_t *)out)[idx] = v;
    }
}

// ---------------------------------------------------------------------------
// Epilogue shared by the MFMA kernels.  The accumulators come from MFMAs that took the weights as
// the row operand: register r of lane l of tile (j, i) holds
// C[m = 32 i + (l & 31)][n = 32 j + 8 (r / 4) + 4 (l >> 5) + (r & 3)], four consecutive output
// channels per register group.  `smem` is the kernel's LDS, free by now, of at least
// igemmEpilogueLds<...>() bytes; myBias / myScale are the (bias, scale) of channel n0 + threadIdx.x.
// ---------------------------------------------------------------------------
__device__ __forceinline__ void blockBarrier() { asm volatile("s_barrier" : : : "memory"); }

template <int WTM, int NW, int BN>
constexpr size_t igemmEpilogueLds() {
    return (size_t)NW * WTM * (32 * 4 + 16) + 2 * (size_t)BN * 4;
}

template <int WTM, int WTN, int NW, int BN>
__device__ __forceinline__ void igemmEpilogue(v16i (&acc)[WTN / 32][WTM / 32], int8_t *smem, const IgemmArgs &p, int m0,
                                              int n0, int wm, int wn, int32_t myBias, int32_t myScale) {
    // Epilogue.  Lane l owns row m = l & 31 of each MFMA tile and, per register group g,
    // channels n = 8 g + 4 (l >> 5) + {0..3}.  The stage ring is free now and serves as staging
    // so that results leave as 128-bit row-contiguous stores.
    blockBarrier();
    constexpr int EROW = 32 * 4 + 16;          // bytes per staged row: 32 int32 + padding against bank conflicts
    constexpr int PARAMS = NW * WTM * EROW;    // bias[BN], scale[BN] behind the staging slices
    constexpr int TM = WTM / 32, TN = WTN / 32;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, fr = lane & 31;
    int32_t *ldsBias = (int32_t *)(smem + PARAMS), *ldsScale = ldsBias + BN;
    if (tid < BN) {
        ldsBias[tid] = myBias;
        ldsScale[tid] = myScale;
    }
    __syncthreads();
    const long long rnd = roundTerm(p.rq.shift);
    const int hi4 = (lane >> 5) * 4;
    const bool wide = p.out_dtype == kDtypeI8 && (p.N & 15) == 0 && (((uintptr_t)p.out) & 15) == 0;
    const WideRequant wrq = wideRequant(p.rq);
    // One 32-channel column of MFMA tiles at a time goes through the wave's own LDS slice as int32;
    // a compact loop then requantises 16 consecutive channels of one row per lane and stores them
    // as one 128-bit word.  (Kept as a loop: unrolled over the whole tile it outgrows the
    // instruction cache.)
    int8_t *stageOut = smem + wave * (WTM * EROW);
    const int erow = lane >> 1, ecol = (lane & 1) * 16;  // read-back: 2 lanes per row, 16 channels each
#pragma unroll
    for (int j = 0; j < TN; j++) {
#pragma unroll
        for (int i = 0; i < TM; i++) {
#pragma unroll
            for (int g = 0; g < 4; g++) {
                v4i v = {acc[j][i][4 * g], acc[j][i][4 * g + 1], acc[j][i][4 * g + 2], acc[j][i][4 * g + 3]};
                *(v4i *)(stageOut + (i * 32 + fr) * EROW + (8 * g + hi4) * 4) = v;
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory");  // wave-private slice: no block barrier needed
        const int nl = wn * WTN + j * 32 + ecol;  // first of this lane's 16 channels, relative to n0
        const int nb = n0 + nl;
        int32_t bias[16], scale[16];
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const v4i b4 = *(const v4i *)(ldsBias + nl + 4 * q);
            const v4i s4 = *(const v4i *)(ldsScale + nl + 4 * q);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                bias[4 * q + e] = b4[e];
                scale[4 * q + e] = s4[e];
            }
        }
        // the shift >= 33 case (the usual one for TFLite-derived scales) has a cheaper tail; the
        // choice is made once per column, outside the row loop
        auto rows = [&](auto wideShiftTag) {
            constexpr bool kWideShift = decltype(wideShiftTag)::value;
            for (int r0 = 0; r0 < WTM; r0 += 32) {
                const int row = r0 + erow;
                const int m = m0 + wm * WTM + row;
                int32_t q[16];
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    const v4i v = *(const v4i *)(stageOut + row * EROW + (ecol + 4 * c) * 4);
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        q[4 * c + e] = kWideShift ? requantWideShift(v[e], bias[4 * c + e], scale[4 * c + e], wrq)
                                                  : requant(v[e], bias[4 * c + e], scale[4 * c + e], rnd, p.rq);
                    }
                }
                if (m < p.M) {
                    if (wide && nb + 15 < p.N) {
                        v4i w;
#pragma unroll
                        for (int c = 0; c < 4; c++) {
                            w[c] = (int)packBytes(q[4 * c], q[4 * c + 1], q[4 * c + 2], q[4 * c + 3]);
                        }
                        *(v4i *)((int8_t *)p.out + (size_t)m * p.N + nb) = w;
                    } else {
#pragma unroll
                        for (int e = 0; e < 16; e++) {
                            if (nb + e < p.N) storeElem(p.out, (size_t)m * p.N + nb + e, q[e], p.out_dtype);
                        }
                    }
                }
            }
        };
        if (wrq.on) {
            rows(std::true_type{});
        } else {
            rows(std::false_type{});
        }
        asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory");  // reads done before the slice is overwritten
    }
}

// torq_hl.add on 16 requantised bytes and 16 bytes of the other operand.  The patterns give an add scale 1 and shift
// 12: then bias, rounding term and zero point fold into one 32-bit constant `folded` and a value costs two
// multiply-adds, a shift and a clamp (FAST; the launcher proves that nothing overflows).  Anything else takes the
// generic 64-bit ACT stage.
template <bool FAST>
__device__ __forceinline__ v4i residualAdd16(v4i mine, v4i other, bool otherFirst, int32_t w0, int32_t w1, int32_t bias, int32_t scale,
                                             long long rnd, const Requant &rq, int32_t folded) {
    v4i r;
    const int32_t wm = otherFirst ? w1 : w0, wo = otherFirst ? w0 : w1;
#pragma unroll
    for (int g = 0; g < 4; g++) {
        int32_t v[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int32_t a = (int32_t)(int8_t)((uint32_t)mine[g] >> (8 * e)), b = (int32_t)(int8_t)((uint32_t)other[g] >> (8 * e));
            if (FAST) {
                v[e] = med3((a * wm + b * wo + folded) >> rq.shift, rq.out_min, rq.out_max);
            } else {
                v[e] = requant(a * wm + b * wo, bias, scale, rnd, rq);
            }
        }
        r[g] = (int)packBytes(v[0], v[1], v[2], v[3]);
    }
    return r;
}
// Whether the FAST form applies, and its constant: ((sum + bias) + 2^(shift-1)) >> shift, + zp, clamp equals
// (sum + bias + 2^(shift-1) + zp * 2^shift) >> shift, clamp, as long as the 32-bit sum cannot overflow.
__host__ __device__ inline bool residualAddFolded(int32_t w0, int32_t w1, int32_t bias, int32_t scale, const Requant &rq, int32_t *folded) {
    if (scale != 1 || rq.shift < 1 || rq.shift > 20 || rq.out_min > rq.out_max) return false;
    const long long aw0 = w0 < 0 ? -(long long)w0 : w0, aw1 = w1 < 0 ? -(long long)w1 : w1;
    const long long c = (long long)bias + (1LL << (rq.shift - 1)) + (long long)rq.out_zp * (1LL << rq.shift);
    const long long bound = 128 * (aw0 + aw1) + (c < 0 ? -c : c);
    if (bound >= (1LL << 31)) return false;
    *folded = (int32_t)c;
    return true;
}

// The same epilogue without the LDS round trip, for int8 outputs with N % 16 == 0 and the plain
// 32-bit requant tail (no pre-shift, zero point folded into the rounding term): each accumulator tile is requantised in place, two v_permlane32_swap exchange
// register groups between the wave halves so that a lane owns 16 consecutive channels of its row
// (see igemm_stream_i8), and the lane stores them as one 128-bit word.  Only the (bias, scale)
// vectors pass through LDS.
template <int WTM, int WTN, int NW, int BN, bool ADD, bool PLAIN>  // ADD: a residual add behind the requant (IgemmArgs::skip); PLAIN: see requantWideT0
__device__ __forceinline__ void igemmEpilogueDirect(v16i (&acc)[WTN / 32][WTM / 32], int8_t *smem, const IgemmArgs &p, int m0,
                                                    int n0, int wm, int wn, int32_t myBias, int32_t myScale) {
    blockBarrier();
    constexpr int TM = WTM / 32, TN = WTN / 32;
    const int tid = threadIdx.x, lane = tid & 63, fr = lane & 31, half = lane >> 5;
    int32_t *ldsBias = (int32_t *)smem, *ldsScale = ldsBias + BN;
    if (tid < BN) {
        ldsBias[tid] = myBias;
        ldsScale[tid] = myScale;
    }
    __syncthreads();
    const WideRequant wrq = wideRequant(p.rq);  // a 32-bit tail applies (the launcher checks); PLAIN: no pre-shift, no clamp of acc + bias, zero point folded
    const long long addRnd = roundTerm(p.arq.shift);
    int32_t addFolded = 0;
    const bool addFast = ADD && residualAddFolded(p.add_w0, p.add_w1, p.add_bias, p.add_scale, p.arq, &addFolded);
#pragma unroll
    for (int j = 0; j < TN; j++) {
        const int nl = wn * WTN + j * 32;  // first channel of this tile column, relative to n0
        v4i b4[4], s4[4];
#pragma unroll
        for (int q = 0; q < 4; q++) {
            b4[q] = *(const v4i *)(ldsBias + nl + 8 * q + 4 * half);
            s4[q] = *(const v4i *)(ldsScale + nl + 8 * q + 4 * half);
        }
        const int n = n0 + nl + 16 * half;
#pragma unroll
        for (int i = 0; i < TM; i++) {
            uint32_t d4[4];
#pragma unroll
            for (int q = 0; q < 4; q++) {
                int32_t v[4];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    v[e] = requantWideT0<PLAIN>((int32_t)((uint32_t)acc[j][i][4 * q + e] + (uint32_t)b4[q][e]), s4[q][e], wrq);
                }
                d4[q] = packBytes(v[0], v[1], v[2], v[3]);
            }
            const auto s02 = __builtin_amdgcn_permlane32_swap(d4[0], d4[2], false, false);
            const auto s13 = __builtin_amdgcn_permlane32_swap(d4[1], d4[3], false, false);
            v4i outv = {(int)s02[0], (int)s02[1], (int)s13[0], (int)s13[1]};
            const int m = m0 + wm * WTM + i * 32 + fr;
            if (m < p.M && n < p.N) {
                if (ADD) {
                    const v4i other = *(const v4i *)(p.skip + (size_t)m * p.N + n);
                    outv = addFast ? residualAdd16<true>(outv, other, p.add_skip_first != 0, p.add_w0, p.add_w1, p.add_bias, p.add_scale, addRnd, p.arq, addFolded)
                                   : residualAdd16<false>(outv, other, p.add_skip_first != 0, p.add_w0, p.add_w1, p.add_bias, p.add_scale, addRnd, p.arq, 0);
                }
                *(v4i *)((int8_t *)p.out + (size_t)m * p.N + n) = outv;
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Linear work index -> (channel group, x, y, image).  A 64-bit division by a run-time divisor costs a
// couple of hundred instructions, more than the whole body of a pooling thread, so the launchers
// precompute multipliers: for n < 2^31 and a divisor d with s = ceil(log2 d),
// n / d == umulhi(n, ceil(2^(31+s) / d)) >> (s - 1) (the multiplier fits 32 bits because
// d > 2^(s-1)).  Work counts of 2^31 and more take the plain 64-bit path.
// ---------------------------------------------------------------------------
struct FastDiv {
    uint32_t mul;    // 0: the divisor is 1
    uint32_t shift;  // s - 1
    uint32_t d;
};
__host__ __device__ static inline FastDiv makeFastDiv(uint32_t d) {
    FastDiv f{0, 0, d};
    if (d <= 1) return f;
    uint32_t s = 0;
    while ((1ull << s) < d) s++;
    f.mul = (uint32_t)((((unsigned long long)1 << (31 + s)) + d - 1) / d);
    f.shift = s - 1;
    return f;
}
struct WorkSplit {
    FastDiv cg, xs, ys;  // channel groups, x positions, y positions per image
    int wide;            // the work count does not fit 31 bits
};
static WorkSplit makeWorkSplit(long long total, int cg, int xs, int ys) {
    return WorkSplit{makeFastDiv((uint32_t)cg), makeFastDiv((uint32_t)xs), makeFastDiv((uint32_t)ys), total >= (1LL << 31)};
}
__device__ __forceinline__ uint32_t fastDiv(uint32_t n, const FastDiv &f) { return f.mul ? __umulhi(n, f.mul) >> f.shift : n; }
__device__ __forceinline__ void splitWork(long long t, const WorkSplit &w, int &c, int &x, int &y, int &n) {
    if (!w.wide) {
        uint32_t u = (uint32_t)t, q = fastDiv(u, w.cg);
        c = (int)(u - q * w.cg.d);
        u = q;
        q = fastDiv(u, w.xs);
        x = (int)(u - q * w.xs.d);
        u = q;
        q = fastDiv(u, w.ys);
        y = (int)(u - q * w.ys.d);
        n = (int)q;
    } else {
        c = (int)(t % w.cg.d);
        long long pix = t / w.cg.d;
        x = (int)(pix % w.xs.d);
        pix /= w.xs.d;
        y = (int)(pix % w.ys.d);
        n = (int)(pix / w.ys.d);
    }
}

// ---------------------------------------------------------------------------
// igemm_i8
// ---------------------------------------------------------------------------
//
// C[m][n] = sum_k A[m][k] * B[n][k]; block tile BM x BN x BK, 256 threads =
// 4 waves in a 2 x 2 arrangement, each wave owns (BM/2) x (BN/2) as a grid of
// 32 x 32 MFMA tiles.  One MFMA consumes 32 rows x 32 k of each operand: lane l
// supplies row (l & 31), 16 consecutive k bytes starting at 16 * (l >> 5).  The weights are
// the MFMA's row operand; the accumulator layout is described at igemmEpilogue.
//
// LDS rows are padded by 16 bytes so that the 16 lanes of one ds_read_b128
// phase fall into distinct banks.

template <int G>
__device__ __forceinline__ v4i gatherChunk(const int8_t *__restrict__ A,
                                           const uint32_t *__restrict__ entries, int iy0, int ix0,
                                           size_t base, int H, int W, int C, uint32_t zp4) {
    union {
        v4i v;
        uint64_t d[2];
        uint32_t w[4];
        uint16_t h[8];
        uint8_t b[16];
    } u;
#pragma unroll
    for (int j = 0; j < 16 / G; j++) {
        const uint32_t e = entries[j];
        const int kh = (int)((e >> 24) & 0x7f), kw = (int)((e >> 16) & 0xff);
        const int ci = (int)(e & 0xffff);
        const int iy = iy0 + kh, ix = ix0 + kw;
        const bool beyond = (e & kKEntryInvalid) != 0;
        const bool inside = !beyond && (unsigned)iy < (unsigned)H && (unsigned)ix < (unsigned)W;
        const int8_t *src = A + base + ((size_t)iy * W + ix) * C + ci;
        const uint32_t fill = beyond ? 0u : zp4;
        if (G == 16) {
            if (inside) {
                u.v = *(const v4i *)src;
            } else {
                u.w[0] = fill; u.w[1] = fill; u.w[2] = fill; u.w[3] = fill;
            }
        } else if (G == 8) {
            u.d[j] = inside ? *(const uint64_t *)src : ((uint64_t)fill << 32 | fill);
        } else if (G == 4) {
            u.w[j] = inside ? *(const uint32_t *)src : fill;
        } else if (G == 2) {
            u.h[j] = inside ? *(const uint16_t *)src : (uint16_t)fill;
        } else {
            u.b[j] = inside ? *(const uint8_t *)src : (uint8_t)fill;
        }
    }
    return u.v;
}

// One window row of a few-channel convolution: 16 bytes starting at pixel (iy, ix0), channel 0.
struct __attribute__((packed)) UnalignedV4 {
    v4i v;
};
__device__ __forceinline__ v4i gatherRun(const int8_t *__restrict__ A, uint32_t entry, int iy0, int ix0, size_t base,
                                         int H, int W, int C, uint32_t zpb, long long aBytes) {
    if (entry & kKEntryInvalid) return v4i{0, 0, 0, 0};
    const int kh = (int)((entry >> 24) & 0x7f), len = (int)(entry & 0xffff);
    const int iy = iy0 + kh;
    const bool rowIn = (unsigned)iy < (unsigned)H;
    const long long off = (long long)base + ((long long)iy * W + ix0) * C;
    const uint32_t zp4 = zpb * 0x01010101u;
    if (!rowIn) return v4i{(int)zp4, (int)zp4, (int)zp4, (int)zp4};  // bytes past the run meet zero weights
    if (off >= 0 && off + 16 <= aBytes) {
        v4i v = ((const UnalignedV4 *)(A + off))->v;
        // bytes [lo, hi) of the run lie inside the image row; the others are padding
        const int lo = ix0 < 0 ? (-ix0 * C < len ? -ix0 * C : len) : 0;
        const int room = (W - ix0) * C;
        const int hi = room < len ? (room > 0 ? room : 0) : len;
        if (lo == 0 && hi == len) return v;
#pragma unroll
        for (int d = 0; d < 4; d++) {
            const int a = lo - 4 * d, b = hi - 4 * d;
            const uint32_t below = a <= 0 ? 0u : a >= 4 ? 0xffffffffu : (1u << (8 * a)) - 1u;
            const uint32_t upto = b <= 0 ? 0u : b >= 4 ? 0xffffffffu : (1u << (8 * b)) - 1u;
            const uint32_t m = upto & ~below;
            v[d] = (int)(((uint32_t)v[d] & m) | (zp4 & ~m));
        }
        return v;
    }
    // window row touches the padding (or the last bytes of the tensor): byte by byte
    union {
        v4i v;
        uint8_t b[16];
    } u;
    int kw = 0, ci = 0;
#pragma unroll
    for (int b = 0; b < 16; b++) {
        uint8_t x = 0;
        if (b < len) {
            const int ix = ix0 + kw;
            x = (rowIn && (unsigned)ix < (unsigned)W) ? (uint8_t)A[off + b] : (uint8_t)zpb;
            if (++ci == C) {
                ci = 0;
                kw++;
            }
        }
        u.b[b] = x;
    }
    return u.v;
}

template <int BM, int BN, int BK, int LOADER, int G>
__global__ __launch_bounds__(256) void igemm_i8(IgemmArgs p) {
    constexpr int LDK = BK + 16;            // padded LDS row
    constexpr int CPR = BK / 16;            // 16-byte chunks per tile row
    constexpr int RPP = 256 / CPR;          // rows loaded per pass
    constexpr int PA = BM / RPP;            // passes over the A tile
    constexpr int PB = BN / RPP;            // passes over the B tile
    constexpr int WTM = BM / 2, WTN = BN / 2;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    static_assert(BM % RPP == 0 && BN % RPP == 0, "tile rows must be a multiple of a load pass");
    static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tile must be a multiple of the MFMA tile");

    extern __shared__ __align__(16) int8_t smem[];
    int8_t *As = smem;                       // [2][BM][LDK]
    int8_t *Bs = smem + 2 * BM * LDK;        // [2][BN][LDK]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;

    // Block -> tile: blocks are dealt round-robin to the 8 XCDs, so give every
    // XCD a contiguous range of tiles (its L2 then sees neighbouring tiles), and
    // walk each range in groups of 8 tile rows so that A and B tiles are reused.
    const int tilesM = (p.M + BM - 1) / BM;
    const int tilesN = p.Np / BN;
    int lin;
    {
        const int nb = (int)gridDim.x, pid = (int)blockIdx.x;
        const int per = nb / 8, rem = nb % 8;
        const int xcd = pid % 8, idx = pid / 8;
        lin = xcd * per + (xcd < rem ? xcd : rem) + idx;
    }
    constexpr int GROUP = 8;
    const int width = GROUP * tilesN;
    const int group = lin / width;
    const int firstM = group * GROUP;
    const int gsize = (tilesM - firstM) < GROUP ? (tilesM - firstM) : GROUP;
    const int tileM = firstM + (lin % width) % gsize;
    const int tileN = (lin % width) / gsize;
    const int m0 = tileM * BM, n0 = tileN * BN;

    const int lrow = tid / CPR, lkc = tid % CPR;
    const uint32_t zpb = (uint32_t)(p.input_zp & 0xff);
    const uint32_t zp4 = zpb * 0x01010101u;

    // Per-row state of the A loader.
    int rIy0[PA], rIx0[PA];
    size_t rBase[PA];
#pragma unroll
    for (int i = 0; i < PA; i++) {
        const int m = m0 + lrow + i * RPP;
        if (LOADER == kLoaderDense) {
            rBase[i] = (size_t)m * p.K;
            rIy0[i] = m < p.M ? 0 : -1;
            rIx0[i] = 0;
        } else {
            const int ohw = p.OH * p.OW;
            const int img = m / ohw, rem = m % ohw;
            const int oy = rem / p.OW, ox = rem % p.OW;
            rBase[i] = (size_t)img * p.H * p.W * p.C;
            // rows past M gather nothing but padding; they are never stored
            rIy0[i] = m < p.M ? oy * p.SH - p.PT : -(1 << 20);
            rIx0[i] = ox * p.SW - p.PL;
        }
    }

    v4i ra[PA], rb[PB];
    auto loadGlobal = [&](int kt) {
        const int k0 = kt * BK + lkc * 16;
#pragma unroll
        for (int i = 0; i < PA; i++) {
            if (LOADER == kLoaderDense) {
                v4i v = {0, 0, 0, 0};
                if (rIy0[i] == 0 && k0 < p.K) {
                    v = *(const v4i *)(p.A + rBase[i] + k0);
                }
                ra[i] = v;
            } else if (LOADER == kLoaderRuns) {
                ra[i] = gatherRun(p.A, p.ktab[k0 / 16], rIy0[i], rIx0[i], rBase[i], p.H, p.W, p.C, zpb, p.a_bytes);
            } else {
                ra[i] = gatherChunk<G>(p.A, p.ktab + k0 / G, rIy0[i], rIx0[i], rBase[i], p.H, p.W,
                                       p.C, zp4);
            }
        }
#pragma unroll
        for (int i = 0; i < PB; i++) {
            const int n = n0 + lrow + i * RPP;
            rb[i] = *(const v4i *)(p.Bp + (size_t)n * p.Kp + k0);
        }
    };
    auto storeLds = [&](int stage) {
#pragma unroll
        for (int i = 0; i < PA; i++) {
            *(v4i *)(As + (stage * BM + lrow + i * RPP) * LDK + lkc * 16) = ra[i];
        }
#pragma unroll
        for (int i = 0; i < PB; i++) {
            *(v4i *)(Bs + (stage * BN + lrow + i * RPP) * LDK + lkc * 16) = rb[i];
        }
    };

    v16i acc[TN][TM];
#pragma unroll
    for (int j = 0; j < TN; j++) {
#pragma unroll
        for (int i = 0; i < TM; i++) {
#pragma unroll
            for (int r = 0; r < 16; r++) acc[j][i][r] = 0;
        }
    }
    // One (bias, scale) pair per thread, fetched now and parked in LDS by the epilogue.
    int32_t myBias = 0, myScale = 0;
    if (tid < BN) {
        myBias = p.bias[n0 + tid];  // arrays are padded to Np
        myScale = p.scale[n0 + tid];
    }

    const int KT = p.Kp / BK;
    loadGlobal(0);
    storeLds(0);
    __syncthreads();

    const int aRow = wm * WTM + (lane & 31);
    const int bRow = wn * WTN + (lane & 31);
    const int kOff = (lane >> 5) * 16;

    for (int kt = 0; kt < KT; kt++) {
        const int cur = kt & 1;
        if (kt + 1 < KT) {
            loadGlobal(kt + 1);
        }
#pragma unroll
        for (int kk = 0; kk < BK / 32; kk++) {
            v4i af[TM], bf[TN];
#pragma unroll
            for (int i = 0; i < TM; i++) {
                af[i] = *(const v4i *)(As + (cur * BM + aRow + i * 32) * LDK + kk * 32 + kOff);
            }
#pragma unroll
            for (int j = 0; j < TN; j++) {
                bf[j] = *(const v4i *)(Bs + (cur * BN + bRow + j * 32) * LDK + kk * 32 + kOff);
            }
#pragma unroll
            for (int j = 0; j < TN; j++) {
#pragma unroll
                for (int i = 0; i < TM; i++) {
                    // weights as the row operand: a lane then holds 4 consecutive output channels
                    acc[j][i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bf[j], af[i], acc[j][i], 0, 0, 0);
                }
            }
        }
        if (kt + 1 < KT) {
            storeLds(cur ^ 1);
        }
        __syncthreads();
    }

    igemmEpilogue<WTM, WTN, 4, BN>(acc, smem, p, m0, n0, wm, wn, myBias, myScale);
}

// ---------------------------------------------------------------------------
// igemm_dense_i8: the dense [M, K] x [N, K]^T case (fully_connected, matmul,
// stride-1 1x1 conv2d) with the tiles moved global -> LDS by the DMA path
// (global_load_lds_dwordx4: no VGPRs, no ds_write) through a ring of STAGES
// LDS stages, so several k-tiles of loads are in flight while one is computed.
//
// One DMA instruction of a wave writes 64 lanes x 16 bytes = 1 KiB of
// consecutive LDS, i.e. 16 tile rows of 64 bytes; lanes cannot scatter.  Bank
// conflicts are therefore avoided on the global side: the 16-byte slot at
// position p of row r holds the logical k-chunk p ^ ((r >> 2) & 3), which makes
// the 16 rows read by one ds_read_b128 phase fall into 16 distinct bank groups.
//
// The loads are issued by inline asm and waited on by hand (s_waitcnt vmcnt(n)
// with n = loads of the tiles still allowed in flight).  Every wave issues the
// same number of loads per k-tile (out-of-range rows and k-chunks are clamped
// to valid addresses rather than skipped) so that the count is exact.
//
// The MFMA takes the weights as its row operand and the activations as its
// column operand: accumulator register r of lane l then holds
// C[m = l & 31][n = 8 * (r / 4) + 4 * (l >> 5) + (r & 3)], four consecutive
// output channels per register group, which requantise into one 32-bit store.
__device__ __forceinline__ void dmaLoad16(const void *gptr, unsigned ldsAddr) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" : : "s"(ldsAddr), "v"(gptr) : "memory", "m0");
}

// Same with the address split into a wave-uniform 64-bit base (SGPR pair) and a 32-bit per-lane
// offset: advancing along K is then scalar work only.
__device__ __forceinline__ void dmaLoad16(const void *base, uint32_t laneOffset, unsigned ldsAddr) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(ldsAddr), "v"(laneOffset), "s"(base) : "memory", "m0");
}

template <int N>
__device__ __forceinline__ void waitVmcnt() {
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

// DIRECT selects the epilogue: 0 staged through LDS (any output type, ragged N, the 64-bit requant tail), or in
// registers (int8 output, N % 16 == 0: the launcher checks) with 1 the plain 32-bit tail or 2 the general 32-bit tail
// (a pre-shift, a clamp of acc + bias or a zero point that does not fold: e.g. small shifts under large scales,
// where every result beyond a small |acc + bias| saturates).
//
// CONV: the activation operand is not a dense matrix but the patch matrix of a convolution over an N,H,W,C image
// with C % BK == 0, so that a k-tile is BK consecutive channels of ONE window tap (kh, kw) and its chunk order is
// the dense one.  Row m of the patch matrix is output pixel (n, oy, ox); the lane that loads it keeps the pixel's
// window origin and, per k-tile, adds the tap's offset (wave-uniform, advanced with scalar selects: no division
// and no branch in the loop).  A tap outside the image reads a 128-byte page of input_zp bytes instead (p.ktab):
// the same number of loads whatever the padding, as the hand-counted waits need.
//
// BK = 128: a k-tile is 128 bytes of K, so that the eight lanes that load one tile row fetch a whole 128-byte line
// (with BK = 64 every request to L2 is half a line, and the path L2 -> LDS is bound by requests, not bytes: the bare
// DMA stream of a 4096^3 problem takes 44 us in half lines and 30 us in whole ones).  One DMA instruction then covers
// 8 rows, slot p of row r holds chunk p ^ ((r >> 1) & 7) (row pitch 128 bytes = 32 banks: the 16 rows of a ds_read_b128
// phase again fall into 16 distinct bank groups), and a k-tile is four MFMA phases.
template <int BM, int BN, int WAVES_M, int WAVES_N, int STAGES, int BLOCKS_PER_CU, int DIRECT, bool ADD = false, bool CONV = false, int BK = 64>
__global__ __launch_bounds__(WAVES_M *WAVES_N * 64, BLOCKS_PER_CU) void igemm_dense_i8(IgemmArgs p) {
    static_assert(BK == 64 || BK == 128, "k-tile of 64 or 128 bytes");
    constexpr int CH = BK / 16;    // 16-byte chunks per tile row
    constexpr int RPI = 64 / CH;   // tile rows one DMA instruction covers
    constexpr int NP = BK / 32;    // MFMA phases per k-tile
    constexpr int NW = WAVES_M * WAVES_N;
    constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    constexpr int BWL = BN / RPI;                          // wave-loads (RPI rows each) that make up the B tile
    constexpr int LA = BM / RPI / NW, LB = (BWL + NW - 1) / NW;  // DMA instructions per wave per k-tile
    constexpr int LPT = LA + LB;
    constexpr int A_STAGE = BM * BK, B_STAGE = BN * BK, STAGE = A_STAGE + B_STAGE;
    // every wave must issue the same number of loads: a narrow B tile (fewer wave-loads than
    // waves) is loaded redundantly, several waves writing the same bytes to the same place
    static_assert(BM % (RPI * NW) == 0 && BN % RPI == 0 && (BWL % NW == 0 || BWL < NW), "unbalanced DMA loads");
    static_assert(BK == 64 || (NW % 2 == 0 && BWL % 2 == 0), "the 128-byte swizzle takes the parity of a wave-load from the wave");
    static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tile must be a multiple of the MFMA tile");
    static_assert(STAGES >= 2 && STAGES <= 8 && LPT * (STAGES - 1) < 64, "vmcnt is a 6-bit counter");

    extern __shared__ __align__(16) int8_t smem[];
    const unsigned ldsBase = (unsigned)(uintptr_t)(__attribute__((address_space(3))) int8_t *)smem;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;

    const int tilesM = (p.M + BM - 1) / BM;
    const int tilesN = p.Np / BN;
    int lin;
    {
        const int nb = (int)gridDim.x, pid = (int)blockIdx.x;
        const int per = nb / 8, rem = nb % 8;
        const int xcd = pid % 8, idx = pid / 8;
        lin = xcd * per + (xcd < rem ? xcd : rem) + idx;
    }
    constexpr int GROUP = 8;
    const int width = GROUP * tilesN;
    const int group = lin / width;
    const int firstM = group * GROUP;
    const int gsize = (tilesM - firstM) < GROUP ? (tilesM - firstM) : GROUP;
    const int tileM = firstM + (lin % width) % gsize;
    const int tileN = (lin % width) / gsize;
    const int m0 = tileM * BM, n0 = tileN * BN;

    // DMA source pointers: lane l of a wave-load covers row l / 4 of its 16 rows and
    // fetches the logical chunk that belongs at slot l % 4 of that row.
    const int lrow = lane / CH;
    // the swizzle of the row a lane loads: (row >> 2) & 3 for 64-byte rows; (row >> 1) & 7 for 128-byte rows, where
    // row = 8 * (wave-load index) + lrow and the index has the wave's parity (NW and BWL are even)
    const int lchunk = BK == 64 ? ((lane & 3) ^ ((lane >> 4) & 3)) : ((lane & 7) ^ ((((wave & 1) << 2) + (lrow >> 1)) & 7));
    // per-lane byte offsets from the tile origins (rows past M are clamped to the last row: their
    // results are never stored, and every wave must issue the same number of loads)
    const int8_t *aTile = CONV ? p.A : p.A + (size_t)m0 * p.K;
    const int8_t *bTile = p.Bp + (size_t)n0 * p.Kp;
    uint32_t aOff[LA], bOff[LB];
    int winY[CONV ? LA : 1], winX[CONV ? LA : 1];  // CONV: input row / column of tap (0, 0) of the lane's output pixels
#pragma unroll
    for (int i = 0; i < LA; i++) {
        int r = RPI * (wave + NW * i) + lrow;
        r = m0 + r < p.M ? r : p.M - 1 - m0;
        if constexpr (CONV) {
            const int m = m0 + r, frame = p.OH * p.OW;
            const int n = m / frame, rem = m - n * frame;
            const int oy = rem / p.OW, ox = rem - oy * p.OW;
            winY[i] = oy * p.SH - p.PT;
            winX[i] = ox * p.SW - p.PL;
            // byte offset of the window origin (modulo 2^32: it may lie before the image; origin + tap does not)
            aOff[i] = ((uint32_t)(n * p.H + winY[i]) * (uint32_t)p.W + (uint32_t)winX[i]) * (uint32_t)p.C;
        } else {
            aOff[i] = (uint32_t)r * (uint32_t)p.K + (uint32_t)lchunk * 16u;
        }
    }
    // CONV: the tap the lane's 16-byte chunk of the next k-tile to be issued belongs to, the chunk's first channel and
    // its byte offset from a window origin.  C is a multiple of 16, so a chunk never straddles two taps, but the chunks
    // of one tile row may (C need not be a multiple of BK, and may be less): the state is per lane.  Chunks of the last tile past
    // KH * KW * C carry on into row KH of the window: inside the image they read valid bytes, which meet zero weights.
    int tapH = 0, tapW = 0, tapC = CONV ? lchunk * 16 : 0;
    uint32_t tapOff = (uint32_t)tapC;
    const uint32_t rowJump = CONV ? ((uint32_t)p.W - (uint32_t)p.KW) * (uint32_t)p.C : 0u;
    // brings tapC back below C once: on to the next column of the window, at the end of a window row on to the next row
    auto tapWrap = [&]() {
        const bool endC = tapC >= p.C;
        tapC -= endC ? p.C : 0;
        const bool endW = endC && tapW + 1 == p.KW;
        tapW = endC ? (endW ? 0 : tapW + 1) : tapW;
        tapH += endW ? 1 : 0;
        tapOff += endW ? rowJump : 0u;
    };
    if constexpr (CONV) {
        if (p.C < BK) {  // the chunks of the first k-tile already span several taps
#pragma unroll
            for (int extra = 1; extra < CH; extra++) tapWrap();
        }
    }
    const int8_t *zpPage = CONV ? (const int8_t *)p.ktab + lchunk * 16 : nullptr;
#pragma unroll
    for (int i = 0; i < LB; i++) {
        bOff[i] = (uint32_t)(RPI * ((wave + NW * i) % BWL) + lrow) * (uint32_t)p.Kp + (uint32_t)lchunk * 16u;
    }
    v16i acc[TN][TM];
#pragma unroll
    for (int j = 0; j < TN; j++) {
#pragma unroll
        for (int i = 0; i < TM; i++) {
#pragma unroll
            for (int r = 0; r < 16; r++) acc[j][i][r] = 0;
        }
    }

    // Fragment addresses: row (l & 31) of a 32-row MFMA tile, logical chunk 2 * kk + (l >> 5).
    const int fr = lane & 31;
    const int swz = BK == 64 ? ((fr >> 2) & 3) : ((fr >> 1) & 7);
    const int off0 = (((lane >> 5)) ^ swz) * 16;  // phase kk = 0; phase kk is off0 ^ (32 kk)
    const int aFrag = (wm * WTM + fr) * BK + off0;
    const int bFrag = A_STAGE + (wn * WTN + fr) * BK + off0;

    // One (bias, scale) pair per thread, fetched now and parked in LDS for the epilogue.
    int32_t myBias = 0, myScale = 0;
    if (tid < BN) {
        myBias = p.bias[n0 + tid];  // arrays are padded to Np
        myScale = p.scale[n0 + tid];
    }

    const int KT = p.Kp / BK;

    // Software pipeline.  The ring holds tiles kt+1 .. kt+STAGES while tile kt is computed.
    // Each k-tile is NP MFMA phases (k slices of 32; described here for two).  While phase 0 runs, the fragments
    // of phase 1 are read from LDS; then the wave waits for tile kt+1, meets the block at the
    // barrier, and while phase 1 runs it refills the stage it just finished with tile
    // kt+STAGES and reads phase 0 of tile kt+1.  LDS latency and the DMA issue thus hide
    // under MFMAs; sched_barrier pins the interleaving the source spells out.
    auto issueTile = [&](int kt, int part, int parts, auto wholeTag) {
        // issues this wave's DMA loads number [part * LPT / parts, (part + 1) * LPT / parts) of tile kt;
        // `whole` promises that the tile lies entirely below K
        constexpr bool kWhole = decltype(wholeTag)::value;
        const unsigned stage = ldsBase + (unsigned)(kt % STAGES) * STAGE;
        const int8_t *aBase = aTile + kt * BK;
        const int8_t *bBase = bTile + kt * BK;
        // beyond K the weights are zero, so any valid bytes will do: such lanes read chunk 0 of the
        // same k-tile (always below K) by dropping their chunk offset; offsets stay non-negative
        const uint32_t back = (!kWhole && kt * BK + lchunk * 16 >= p.K) ? (uint32_t)(lchunk * 16) : 0u;
#pragma unroll
        for (int x = 0; x < LPT; x++) {
            if (x * parts / LPT != part) continue;
            if (x < LA) {
                if constexpr (CONV) {
                    const int y = winY[x] + tapH, xx = winX[x] + tapW;
                    const bool inside = (unsigned)y < (unsigned)p.H && (unsigned)xx < (unsigned)p.W;
                    const int8_t *src = inside ? p.A + (size_t)(uint32_t)(aOff[x] + tapOff) : zpPage;
                    dmaLoad16(src, stage + (unsigned)(wave + NW * x) * 1024u);
                } else {
                    dmaLoad16(aBase, aOff[x] - back, stage + (unsigned)(wave + NW * x) * 1024u);
                }
            } else {
                dmaLoad16(bBase, bOff[x - LA], stage + A_STAGE + (unsigned)((wave + NW * (x - LA)) % BWL) * 1024u);
            }
        }
        if constexpr (CONV) {
            if (part == parts - 1) {
                // on to tile kt + 1: BK bytes further along the window.  Channels and columns of one window row are
                // contiguous in the image, so the offset moves on by BK, and by the rest of the image row as well
                // wherever a window row ends (modulo 2^32 where the window is wider than the image).  With C >= BK
                // that is one wrap of the channel at most; fewer channels wrap up to BK / 16 times.
                // (Recomputing (tapH * W + tapW) * C + tapC instead becomes a 64-bit multiply-add whose unused upper
                // addend lands in a register with a load in flight, and the compiler then drains vmcnt in every
                // k-tile: 17.0 us against 12.8 for 256 -> 256 channels at 14 x 14.)
                tapC += BK;
                tapOff += (uint32_t)BK;
                tapWrap();
                if (p.C < BK) {
#pragma unroll
                    for (int extra = 1; extra < CH; extra++) tapWrap();
                }
            }
        }
    };
    // reads fragment number x (first the TM activation fragments, then the TN weight fragments)
    auto readFrag = [&](const int8_t *st, int kk, int x, v4i(&af)[TM], v4i(&bf)[TN]) {
        if (x < TM) {
            af[x] = *(const v4i *)(st + ((aFrag + x * 32 * BK) ^ (kk * 32)));
        } else {
            bf[x - TM] = *(const v4i *)(st + ((bFrag + (x - TM) * 32 * BK) ^ (kk * 32)));
        }
    };
    constexpr int NF = TM + TN;

#pragma unroll
    for (int t = 0; t < STAGES; t++) {
        if (t < KT) issueTile(t, 0, 1, std::false_type{});
    }
    // tile 0 landed?  (tiles 1 .. STAGES-1 may stay in flight)
    if (KT >= STAGES) {
        waitVmcnt<LPT *(STAGES - 1)>();
    } else {
        waitVmcnt<0>();
    }
    blockBarrier();
    v4i af0[TM], bf0[TN], af1[TM], bf1[TN];
#pragma unroll
    for (int x = 0; x < NF; x++) readFrag(smem, 0, x, af0, bf0);

    // One k-tile.  `steady` (a compile-time flag) is the branch-free body used while the tile it
    // refills the ring with exists and lies wholly below K; the rest go through the general body.
    auto step = [&](int kt, auto steady) {
        constexpr bool kSteady = decltype(steady)::value;
        const int8_t *st = smem + (kt % STAGES) * STAGE;
        const int8_t *stNext = smem + ((kt + 1) % STAGES) * STAGE;
        // every phase but the last: MFMAs on the current fragments; the reads of the next phase's go out behind the
        // first weight row (so that the wait in front of that row only covers reads issued a phase ago) and
        // complete under the remaining rows
        auto phase = [&](v4i(&afC)[TM], v4i(&bfC)[TN], v4i(&afN)[TM], v4i(&bfN)[TN], int kkNext) {
#pragma unroll
            for (int j = 0; j < TN; j++) {
#pragma unroll
                for (int i = 0; i < TM; i++) acc[j][i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bfC[j], afC[i], acc[j][i], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
                if (j == 0) {
#pragma unroll
                    for (int x = 0; x < NF; x++) readFrag(st, kkNext, x, afN, bfN);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        };
        phase(af0, bf0, af1, bf1, 1);
        if constexpr (NP == 4) {
            phase(af1, bf1, af0, bf0, 2);
            phase(af0, bf0, af1, bf1, 3);
        }
        // tile kt+1 must have landed; tiles kt+2 .. kt+STAGES-1 may stay in flight
        const bool more = kSteady || kt + 1 < KT;
        if (kSteady) {
            waitVmcnt<LPT *(STAGES - 2)>();
        } else if (more) {
            const int inFlight = (KT - 2 - kt) < (STAGES - 2) ? (KT - 2 - kt) : (STAGES - 2);
            if (inFlight >= 6) {
                waitVmcnt<(LPT * 6 < 64 ? LPT * 6 : 0)>();
            } else if (inFlight == 5) {
                waitVmcnt<(LPT * 5 < 64 ? LPT * 5 : 0)>();
            } else if (inFlight == 4) {
                waitVmcnt<(LPT * 4 < 64 ? LPT * 4 : 0)>();
            } else if (inFlight == 3) {
                waitVmcnt<LPT * 3>();
            } else if (inFlight == 2) {
                waitVmcnt<LPT * 2>();
            } else if (inFlight == 1) {
                waitVmcnt<LPT>();
            } else {
                waitVmcnt<0>();
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory");  // this wave's reads of tile kt are complete
        blockBarrier();  // tile kt+1 is visible to everyone, and nobody reads stage kt % STAGES any more
        const bool refill = kSteady || kt + STAGES < KT;
        // last phase: MFMAs on (af1, bf1), the reads of the next phase 0 behind the first weight row,
        // the refill of the freed stage spread between the rows
#pragma unroll
        for (int j = 0; j < TN; j++) {
            if (refill) issueTile(kt + STAGES, j, TN, steady);
#pragma unroll
            for (int i = 0; i < TM; i++) acc[j][i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bf1[j], af1[i], acc[j][i], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            if (j == 0 && more) {
#pragma unroll
                for (int x = 0; x < NF; x++) readFrag(stNext, 0, x, af0, bf0);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };
    int kt = 0;
    for (; kt + STAGES < KT - 1; kt++) step(kt, std::true_type{});
    for (; kt < KT; kt++) step(kt, std::false_type{});

    if (DIRECT) {
        igemmEpilogueDirect<WTM, WTN, NW, BN, ADD, DIRECT == 1>(acc, smem, p, m0, n0, wm, wn, myBias, myScale);
    } else {
        igemmEpilogue<WTM, WTN, NW, BN>(acc, smem, p, m0, n0, wm, wn, myBias, myScale);
    }
}


// ---------------------------------------------------------------------------
// igemm_stream_i8: pointwise convolution / fully_connected with a small weight matrix
// (Np * Kp of at most 64 KiB, N <= 256), the shape of the expand and project convolutions of
// mobile networks at high resolution.  These are bandwidth-bound: a tile kernel spends its time
// in load -> MFMA -> epilogue phases that do not overlap.  Here the whole weight matrix sits in
// LDS in MFMA fragment order and every wave streams 32-pixel groups: per k-step one 16-byte
// activation load per lane and NB MFMAs (weights as the row operand), then the requant on the
// accumulator registers.  Lane l of an accumulator holds, for pixel l & 31, the channels
// 8 g + 4 (l >> 5) + {0..3} of register group g; two v_permlane32_swap exchange groups between
// the wave halves so that each lane owns 16 consecutive channels and stores them as one 128-bit
// word: no LDS round trip and no barrier after the prologue.  Activation loads run RING k-steps
// ahead, across group boundaries.  K % 16 == 0, N % 16 == 0, int8 output.
// ---------------------------------------------------------------------------
constexpr int kStreamRing = 4;
constexpr size_t kStreamMaxLds = 64 * 1024;
// LDS of the streaming kernel: weights [chunk][Kp], bias and scale [chunk] each, the run table, then (16-byte
// aligned) the staging slices of the four waves: 32 rows of chunk + 16 bytes each (the 16 keep the 128-bit writes
// of 16 lanes, one row each, on distinct banks)
__host__ __device__ inline size_t igemmStreamStageOffset(int chunk, int Kp, bool runs) {
    const size_t used = (size_t)chunk * Kp + 8 * (size_t)chunk + (runs ? (size_t)Kp / 16 * 4 : 0);
    return (used + 15) & ~(size_t)15;
}
__host__ __device__ inline size_t igemmStreamStageBytes(int chunk) { return (size_t)4 * 32 * (chunk + 16); }

// KS: 0, or the number of k-steps (1 or 2) when that is known at compile time and divides the ring: the ring then
// runs over RING / KS pixel groups instead of one, so that loads stay RING k-steps ahead of the MFMAs even where a
// group has only one or two of them (the expanding pointwise convolutions of a mobile network: K = 16 .. 64).
template <int NB, int LOADER, bool ADD, int KS>  // ADD: a residual add behind the requant (its code costs the others registers)
__global__ __launch_bounds__(256, NB <= 2 ? 4 : 2) void igemm_stream_i8(IgemmArgs p) {
    static_assert(KS == 0 || (kStreamRing % KS == 0 && LOADER == kLoaderDense), "the ring holds whole groups");
    extern __shared__ __attribute__((aligned(16))) int8_t smem[];
    constexpr int RING = kStreamRing;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int fr = lane & 31, half = lane >> 5;
    // this grid row's chunk of output channels
    const int chunk = igemmStreamChunk(p.Np), n0 = blockIdx.y * chunk;
    const int chunkN = (p.Np - n0 < chunk ? p.Np - n0 : chunk);
    const int ksteps = p.Kp / 32, nblocks = chunkN / 32;
    // weights [chunkN][Kp] -> fragment order: fragment (s, j) = 64 lanes x 16 bytes, lane (n & 31) + 32 (kc & 1)
    {
        const int chunksPerRow = p.Kp / 16, total = chunkN * chunksPerRow;
        for (int c = tid; c < total; c += 256) {
            const int n = c / chunksPerRow, kc = c - n * chunksPerRow;
            const v4i v = *(const v4i *)(p.Bp + (size_t)(n0 + n) * p.Kp + kc * 16);
            *(v4i *)(smem + ((((kc >> 1) * nblocks + (n >> 5)) * 64 + (kc & 1) * 32 + (n & 31)) << 4)) = v;
        }
    }
    int32_t *ldsBias = (int32_t *)(smem + (size_t)chunkN * p.Kp), *ldsScale = ldsBias + chunkN;
    for (int c = tid; c < chunkN; c += 256) {
        ldsBias[c] = p.bias[n0 + c];
        ldsScale[c] = p.scale[n0 + c];
    }
    // run loader: the k-table next to them, so that a gather does not wait for a table load from memory
    uint32_t *ldsTab = (uint32_t *)(ldsScale + chunkN);
    if (LOADER == kLoaderRuns) {
        for (int c = tid; c < p.Kp / 16; c += 256) ldsTab[c] = p.ktab[c];
    }
    __syncthreads();

    const int groups = (p.M + 31) / 32, stride = gridDim.x * 4;
    const int kstepsRing = (ksteps + RING - 1) / RING * RING;
    // 16 bytes of pixel row (32 g + fr) at k-step s; zero past K or past the last group.  With the
    // run loader (few input channels: one 16-byte run per window row) the row is gathered from the
    // image, at the window position `pos` of the lane's pixel in group g.
    struct Pos {
        int iy0, ix0;
        size_t base;
    };
    // pixel index -> (image, row, column) with multiply-shift divisions (M < 2^31): two run-time integer divisions
    // per group cost this loader about a fifth of its instructions
    const FastDiv divPlane = makeFastDiv(LOADER == kLoaderRuns ? (uint32_t)(p.OH * p.OW) : 1u), divOw = makeFastDiv(LOADER == kLoaderRuns ? (uint32_t)p.OW : 1u);
    auto locate = [&](int g) -> Pos {
        if (LOADER != kLoaderRuns) return Pos{0, 0, 0};
        int m = g * 32 + fr;
        m = m < p.M ? m : p.M - 1;
        const int plane = p.OH * p.OW;
        const int img = (int)fastDiv((uint32_t)m, divPlane), rem = m - img * plane;
        const int oy = (int)fastDiv((uint32_t)rem, divOw), ox = rem - oy * p.OW;
        return Pos{oy * p.SH - p.PT, ox * p.SW - p.PL, (size_t)img * p.H * p.W * p.C};
    };
    const uint32_t zpb = (uint32_t)(p.input_zp & 0xff);
    auto fetch = [&](int g, int s, const Pos &pos) -> v4i {
        const int k = s * 32 + half * 16;
        if (g >= groups || k >= p.K) return v4i{0, 0, 0, 0};
        if (LOADER == kLoaderRuns) {
            return gatherRun(p.A, ldsTab[k >> 4], pos.iy0, pos.ix0, pos.base, p.H, p.W, p.C, zpb, p.a_bytes);
        }
        int m = g * 32 + fr;
        m = m < p.M ? m : p.M - 1;
        return *(const v4i *)(p.A + (size_t)m * p.K + k);
    };
    const WideRequant wrq = wideRequant(p.rq);
    const long long rnd = roundTerm(p.rq.shift), addRnd = roundTerm(p.arq.shift);
    int32_t addFolded = 0;
    const bool addFast = ADD && residualAddFolded(p.add_w0, p.add_w1, p.add_bias, p.add_scale, p.arq, &addFolded);

    // accumulators start at the bias: register 4 q + e of block j holds channel 32 j + 8 q + 4 half + e
    auto initAcc = [&](v16i (&acc)[NB]) {
#pragma unroll
        for (int j = 0; j < NB; j++) {
            if (j < nblocks) {
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const v4i b4 = *(const v4i *)(ldsBias + j * 32 + 8 * q + 4 * half);
#pragma unroll
                    for (int e = 0; e < 4; e++) acc[j][4 * q + e] = b4[e];
                }
            }
        }
    };
    auto multiply = [&](int s, const v4i &a, v16i (&acc)[NB]) {
        const int8_t *wfrag = smem + ((size_t)(s * nblocks) * 64 + lane) * 16;
#pragma unroll
        for (int j = 0; j < NB; j++) {
            if (j < nblocks) {
                const v4i w = *(const v4i *)(wfrag + j * 1024);
                acc[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(w, a, acc[j], 0, 0, 0);
            }
        }
    };
    auto epilogue = [&](int g, v16i (&acc)[NB]) {
        const int m = g * 32 + fr;
        withRequantMode(wrq, [&](auto mode) {
            constexpr int kMode = decltype(mode)::value;
#pragma unroll
            for (int j = 0; j < NB; j++) {
                if (j < nblocks) {
                    uint32_t d4[4];
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        const v4i s4 = *(const v4i *)(ldsScale + j * 32 + 8 * q + 4 * half);
                        int32_t v[4];
#pragma unroll
                        for (int e = 0; e < 4; e++) v[e] = requantT0<kMode>(acc[j][4 * q + e], s4[e], rnd, p.rq, wrq);
                        d4[q] = packBytes(v[0], v[1], v[2], v[3]);
                    }
                    // lower half lanes: channels 0-3, 8-11, 16-19, 24-27; upper half: 4-7, 12-15, 20-23, 28-31.
                    // Swap (upper of d4[0], lower of d4[2]) and (upper of d4[1], lower of d4[3]):
                    // then {d4[0], d4[2], d4[1], d4[3]} are 16 consecutive channels, 0-15 below, 16-31 above.
                    const auto s02 = __builtin_amdgcn_permlane32_swap(d4[0], d4[2], false, false);
                    const auto s13 = __builtin_amdgcn_permlane32_swap(d4[1], d4[3], false, false);
                    v4i outv = {(int)s02[0], (int)s02[1], (int)s13[0], (int)s13[1]};
                    const int n = n0 + j * 32 + 16 * half;
                    if (m < p.M && n < p.N) {
                        if (ADD) {
                            const v4i other = *(const v4i *)(p.skip + (size_t)m * p.N + n);
                            outv = addFast ? residualAdd16<true>(outv, other, p.add_skip_first != 0, p.add_w0, p.add_w1, p.add_bias, p.add_scale, addRnd, p.arq, addFolded)
                                           : residualAdd16<false>(outv, other, p.add_skip_first != 0, p.add_w0, p.add_w1, p.add_bias, p.add_scale, addRnd, p.arq, 0);
                        }
                        *(v4i *)((int8_t *)p.out + (size_t)m * p.N + n) = outv;
                    }
                }
            }
        });
    };

    int g = blockIdx.x * 4 + wave;
    v4i ring[RING];
    // The steady state of the dense loader: every load and every store unconditional and branch-free, so that the
    // compiler's s_waitcnt before an MFMA counts exactly the memory operations issued after the load it needs (a
    // load or a store under a branch counts as zero, and the wait then drains the whole queue, prefetches included).
    // A row past M reads row M - 1 and bytes past the end of A the last 16: they meet zero weights (K..Kp) or
    // belong to rows that are not stored.  Full groups only; what is left goes through the guarded code below.
    if (LOADER == kLoaderDense && !ADD && nblocks == NB && !p.stream_guarded) {
        const long long lastRun = (long long)p.M * p.K - 16;
        auto fetchDense = [&](int gq, int sq) -> v4i {
            int m = gq * 32 + fr;
            m = m < p.M ? m : p.M - 1;
            long long off = (long long)m * p.K + (sq < ksteps ? sq : 0) * 32 + half * 16;
            off = off < lastRun ? off : lastRun;
            return *(const v4i *)(p.A + off);
        };
        const int groupsFull = p.M / 32;
        const bool ragged = p.N - n0 < NB * 32;  // the upper 16 channels of the last block do not exist (N % 16 == 0)
        // Staged stores: a group's 32 rows of this chunk go through the wave's LDS slice and leave as 16-byte pieces in
        // row order, consecutive lanes taking consecutive pieces, so that a store instruction writes whole pixel rows
        // (1 KiB of consecutive bytes where the chunk is the whole row) instead of 32 bytes per pixel: with 32-byte
        // pieces the partly written lines of the output do not survive in L2 next to the activation reads.
        // Piece q = i * 64 + lane of a group is the same for every group: its LDS and global offsets are computed once.
        const bool stage = KS > 0 && p.stream_stage != 0;  // (the widths with more k-steps would pay for the offsets with a wave per SIMD)
        const int pitch = chunk + 16;
        int8_t *slice = smem + igemmStreamStageOffset(chunk, p.Kp, false) + (size_t)wave * 32 * pitch;
        const int piecesPerRow = (p.N - n0 < chunkN ? p.N - n0 : chunkN) >> 4;
        int pieceLds[NB], pieceOut[NB];
        {
            const FastDiv divPieces = makeFastDiv((uint32_t)piecesPerRow);
#pragma unroll
            for (int i = 0; i < NB; i++) {
                const int q = i * 64 + lane;
                int row = (int)fastDiv((uint32_t)q, divPieces);
                const int c = q - row * piecesPerRow;
                // the last instruction may run past the 32 rows: those lanes write their first piece again (with one
                // piece per row and one instruction, the piece of the lane 32 below)
                if (i == 0) row = row < 32 ? row : row - 32;
                pieceLds[i] = row < 32 ? row * pitch + c * 16 : pieceLds[0];
                pieceOut[i] = row < 32 ? row * p.N + c * 16 : pieceOut[0];
            }
        }
        // bias and scale are read from LDS again for every group: kept in registers across the loop (where the compiler
        // hoists loop-invariant loads to) they would be 32 registers per block of channels and spill; an offset of
        // zero that the compiler cannot see through keeps the reads where they are
        auto perGroupZero = [] {
            int zero = 0;
            asm volatile("" : "+v"(zero));
            return zero;
        };
        auto initAll = [&](v16i (&acc)[NB]) {
            const int32_t *bias = ldsBias + perGroupZero();
#pragma unroll
            for (int j = 0; j < NB; j++) {
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const v4i b4 = *(const v4i *)(bias + j * 32 + 8 * q + 4 * half);
#pragma unroll
                    for (int e = 0; e < 4; e++) acc[j][4 * q + e] = b4[e];
                }
            }
        };
        auto multiplyAll = [&](int sq, const v4i &a, v16i (&acc)[NB]) {
            const int8_t *wfrag = smem + ((size_t)(sq * NB) * 64 + lane) * 16;
#pragma unroll
            for (int j = 0; j < NB; j++) {
                const v4i w = *(const v4i *)(wfrag + j * 1024);
                acc[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(w, a, acc[j], 0, 0, 0);
            }
        };
        withRequantMode(wrq, [&](auto mode) {
            constexpr int kMode = decltype(mode)::value;
            auto storeFull = [&](int gq, v16i (&acc)[NB]) {
                int8_t *orow = (int8_t *)p.out + (size_t)(gq * 32 + fr) * p.N + n0 + 16 * half;
                const int32_t *scale = ldsScale + perGroupZero();
#pragma unroll
                for (int j = 0; j < NB; j++) {
                    uint32_t d4[4];
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        const v4i s4 = *(const v4i *)(scale + j * 32 + 8 * q + 4 * half);
                        int32_t v[4];
#pragma unroll
                        for (int e = 0; e < 4; e++) v[e] = requantT0<kMode>(acc[j][4 * q + e], s4[e], rnd, p.rq, wrq);
                        d4[q] = packBytes(v[0], v[1], v[2], v[3]);
                    }
                    const auto s02 = __builtin_amdgcn_permlane32_swap(d4[0], d4[2], false, false);
                    const auto s13 = __builtin_amdgcn_permlane32_swap(d4[1], d4[3], false, false);
                    v4i outv = {(int)s02[0], (int)s02[1], (int)s13[0], (int)s13[1]};
                    if (stage) {
                        *(v4i *)(slice + fr * pitch + j * 32 + 16 * half) = outv;
                    } else if (j == NB - 1 && ragged) {
                        // ragged last block: its 16 channels sit in the lower half lanes; the upper half lanes take over
                        // the second 8 of them, so that every lane stores (one store on either side of this branch)
                        const auto hi0 = __builtin_amdgcn_permlane32_swap((uint32_t)outv[2], (uint32_t)outv[2], false, false);
                        const auto hi1 = __builtin_amdgcn_permlane32_swap((uint32_t)outv[3], (uint32_t)outv[3], false, false);
                        const v2i part = {half ? (int)hi0[0] : outv[0], half ? (int)hi1[0] : outv[1]};
                        *(v2i *)(orow + j * 32 - 8 * half) = part;
                    } else {
                        *(v4i *)(orow + j * 32) = outv;
                    }
                }
                if (stage) {
                    // LDS operations of a wave complete in order: the reads see the writes above, and the next group's
                    // writes come behind these reads
                    int8_t *obase = (int8_t *)p.out + (size_t)gq * 32 * p.N + n0;
#pragma unroll
                    for (int i = 0; i < NB; i++) *(v4i *)(obase + pieceOut[i]) = *(const v4i *)(slice + pieceLds[i]);
                }
            };
            if (KS > 0) {
                // slot d holds k-step d % KS of group g + (d / KS) * stride; a revolution of the ring covers GPI groups
                constexpr int KSS = KS > 0 ? KS : 1, GPI = RING / KSS;
#pragma unroll
                for (int d = 0; d < RING; d++) ring[d] = fetchDense(g + (d / KSS) * stride, d % KSS);
                for (; g + (GPI - 1) * stride < groupsFull; g += GPI * stride) {
#pragma unroll
                    for (int gi = 0; gi < GPI; gi++) {
                        const int gd = g + gi * stride;
                        v16i acc[NB];
                        initAll(acc);
#pragma unroll
                        for (int ks = 0; ks < KSS; ks++) {
                            // the MFMAs read the slot before its next load is issued: the slot keeps its registers
                            multiplyAll(ks, ring[gi * KSS + ks], acc);
                            ring[gi * KSS + ks] = fetchDense(gd + GPI * stride, ks);
                        }
                        storeFull(gd, acc);
                    }
                }
                // the wave's last groups (fewer than a revolution, the last one perhaps short): their data is in the ring
#pragma unroll
                for (int gi = 0; gi < GPI; gi++) {
                    const int gd = g + gi * stride;
                    if (gd < groups) {
                        v16i acc[NB];
                        initAcc(acc);
#pragma unroll
                        for (int ks = 0; ks < KSS; ks++) multiply(ks, ring[gi * KSS + ks], acc);
                        epilogue(gd, acc);
                    }
                }
            } else {
#pragma unroll
                for (int d = 0; d < RING; d++) ring[d] = fetchDense(g, d);
                auto revolve = [&](int gq, v16i (&acc)[NB]) {
                    for (int s0 = 0; s0 < kstepsRing; s0 += RING) {
#pragma unroll
                        for (int d = 0; d < RING; d++) {
                            const int sq = s0 + d;
                            if (sq < ksteps) multiplyAll(sq, ring[d], acc);
                            // slot d next holds k-step s + RING of this group, or the same slot of the next group
                            const bool wrap = sq + RING >= kstepsRing;
                            ring[d] = fetchDense(wrap ? gq + stride : gq, wrap ? sq + RING - kstepsRing : sq + RING);
                        }
                    }
                };
                for (; g < groupsFull; g += stride) {
                    v16i acc[NB];
                    initAll(acc);
                    revolve(g, acc);
                    storeFull(g, acc);
                }
                if (g < groups) {  // the short last group
                    v16i acc[NB];
                    initAcc(acc);
                    revolve(g, acc);
                    epilogue(g, acc);
                }
            }
        });
        return;
    }
    Pos here = locate(g);
#pragma unroll
    for (int d = 0; d < RING; d++) ring[d] = fetch(g, d, here);
    for (; g < groups; g += stride) {
        const Pos next = locate(g + stride < groups ? g + stride : g);
        v16i acc[NB];
        initAcc(acc);
        for (int s0 = 0; s0 < kstepsRing; s0 += RING) {
#pragma unroll
            for (int d = 0; d < RING; d++) {
                const int s = s0 + d;
                const v4i a = ring[d];
                // slot d next holds k-step s + RING of this group, or the same slot of the next group
                const bool wrap = s + RING >= kstepsRing;
                ring[d] = fetch(wrap ? g + stride : g, wrap ? s + RING - kstepsRing : s + RING, wrap ? next : here);
                if (s < ksteps) multiply(s, a, acc);
            }
        }
        epilogue(g, acc);
        here = next;
    }
}

template <int NB, int LOADER, bool ADD, int KS>
static hipError_t launchIgemmStreamA(const IgemmArgs &a, size_t smem, const LaunchCtx &ctx) {
    auto kernel = igemm_stream_i8<NB, LOADER, ADD, KS>;
    // every block copies the weights into LDS once, then strides over the pixel groups:
    // one resident set of blocks, each with several groups where the image is large
    // blocks one CU holds: by registers (asked once per kernel, with no LDS in the way) and by LDS
    static std::once_flag once;
    static hipError_t configured = hipSuccess;
    static int byRegs = 0;
    std::call_once(once, [&] {
        configured = hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kStreamMaxLds);
        int n = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, (const void *)kernel, 256, 0) != hipSuccess || n <= 0) {
            (void)hipGetLastError();
            n = NB <= 1 ? 7 : NB <= 2 ? 5 : NB <= 4 ? 4 : NB <= 6 ? 3 : 2;
        }
        byRegs = n;
    });
    if (configured != hipSuccess) return configured;
    const int perCu = (int)std::min<size_t>((size_t)std::min(byRegs, 8), (160 * 1024) / ((smem + 1023) / 1024 * 1024));
    const int groups = (a.M + 31) / 32;
    const int chunk = igemmStreamChunk(a.Np), chunks = (a.Np + chunk - 1) / chunk;
    const int blocks = std::min((groups + 3) / 4, std::max(1, 256 * perCu / chunks));
    THIP_ENQUEUE(ctx, kernelLabel("igemm_stream_i8", {NB, LOADER, ADD, KS}), kernel, dim3((unsigned)blocks, (unsigned)chunks), dim3(256), smem, a);
    return hipGetLastError();
}

template <int NB, int LOADER>
static hipError_t launchIgemmStreamT(const IgemmArgs &a, size_t smem, const LaunchCtx &ctx) {
    if (a.skip != nullptr) {
        // the residual add comes with the accumulator widths 1, 2, 4, 6, 8 only (its caller rounds up)
        if constexpr (LOADER == kLoaderDense && (NB <= 2 || NB % 2 == 0)) {
            return launchIgemmStreamA<NB, kLoaderDense, true, 0>(a, smem, ctx);
        } else {
            return hipErrorInvalidValue;
        }
    }
    // one or two k-steps per pixel group: the ring runs over several groups (THIP_NO_STREAM_DEEP: never)
    if (LOADER == kLoaderDense && a.Kp <= 64 && !ctx.tuning->noStreamDeep) {
        return a.Kp <= 32 ? launchIgemmStreamA<NB, kLoaderDense, false, 1>(a, smem, ctx) : launchIgemmStreamA<NB, kLoaderDense, false, 2>(a, smem, ctx);
    }
    return launchIgemmStreamA<NB, LOADER, false, 0>(a, smem, ctx);
}

static hipError_t launchIgemmStream(const IgemmArgs &a, const LaunchCtx &ctx) {
    if ((a.loader != kLoaderDense && a.loader != kLoaderRuns) || a.out_dtype != kDtypeI8) return hipErrorInvalidValue;
    if (a.N % 16 != 0 || ((uintptr_t)a.out & 15) != 0 || ((uintptr_t)a.skip & 15) != 0) return hipErrorInvalidValue;
    const int chunk = igemmStreamChunk(a.Np);
    size_t smem = (size_t)chunk * a.Kp + 8 * (size_t)chunk + (a.loader == kLoaderRuns ? (size_t)a.Kp / 16 * 4 : 0);
    if (chunk > 256 || smem > kStreamMaxLds) return hipErrorInvalidValue;
    const int nb = chunk / 32;
    if (a.loader == kLoaderRuns) {
        // the first layer of an image network: few output channels
        if (nb <= 1) return launchIgemmStreamT<1, kLoaderRuns>(a, smem, ctx);
        if (nb <= 2) return launchIgemmStreamT<2, kLoaderRuns>(a, smem, ctx);
        if (nb <= 4) return launchIgemmStreamT<4, kLoaderRuns>(a, smem, ctx);
        return hipErrorInvalidValue;
    }
    if (a.skip == nullptr) {
        // the branch-free steady state needs the block count at compile time (THIP_STREAM_GUARDED: the guarded loop only)
        IgemmArgs b = a;
        b.stream_guarded = ctx.tuning->streamGuarded;
        // staged stores where the slices fit beside the weights, the stores outweigh the loads and the output is far larger than
        // the caches (measured on a mobile network at batch 256: ahead from about 100 MB of output, behind at 40 MB);
        // THIP_STREAM_STAGE=0 / 1: never / wherever they fit
        const size_t staged = igemmStreamStageOffset(chunk, a.Kp, false) + igemmStreamStageBytes(chunk);
        const int stageMode = ctx.tuning->streamStage;
        b.stream_stage = staged <= kStreamMaxLds && a.skip == nullptr && (stageMode >= 0 ? stageMode == 1 : a.N >= 2 * a.K && a.N >= 32 && (long long)a.M * a.N >= (64LL << 20)) && a.Kp <= 64;
        if (b.stream_stage) smem = staged;
        switch (nb) {
        case 1: return launchIgemmStreamT<1, kLoaderDense>(b, smem, ctx);
        case 2: return launchIgemmStreamT<2, kLoaderDense>(b, smem, ctx);
        case 3: return launchIgemmStreamT<3, kLoaderDense>(b, smem, ctx);
        case 4: return launchIgemmStreamT<4, kLoaderDense>(b, smem, ctx);
        case 5: return launchIgemmStreamT<5, kLoaderDense>(b, smem, ctx);
        case 6: return launchIgemmStreamT<6, kLoaderDense>(b, smem, ctx);
        case 7: return launchIgemmStreamT<7, kLoaderDense>(b, smem, ctx);
        default: return launchIgemmStreamT<8, kLoaderDense>(b, smem, ctx);
        }
    }
    if (nb <= 1) return launchIgemmStreamT<1, kLoaderDense>(a, smem, ctx);
    if (nb <= 2) return launchIgemmStreamT<2, kLoaderDense>(a, smem, ctx);
    if (nb <= 4) return launchIgemmStreamT<4, kLoaderDense>(a, smem, ctx);
    if (nb <= 6) return launchIgemmStreamT<6, kLoaderDense>(a, smem, ctx);
    return launchIgemmStreamT<8, kLoaderDense>(a, smem, ctx);
}

template <int BM, int BN, int BK, int LOADER, int G>
static hipError_t launchIgemmTile(const IgemmArgs &a, const LaunchCtx &ctx) {
    constexpr int LDK = BK + 16;
    constexpr size_t tiles = (size_t)2 * (BM + BN) * LDK;
    constexpr size_t epilogue = igemmEpilogueLds<BM / 2, 4, BN>();
    constexpr size_t smem = tiles > epilogue ? tiles : epilogue;
    auto kernel = igemm_i8<BM, BN, BK, LOADER, G>;
    // once per kernel, when an executable that uses it is created: launches may sit inside a stream capture, where only stream work belongs
    static std::once_flag once;
    static hipError_t configured = hipSuccess;
    std::call_once(once, [&] { configured = hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem); });
    if (configured != hipSuccess) return configured;
    const int tilesM = (a.M + BM - 1) / BM;
    const int tilesN = a.Np / BN;
    const dim3 grid((unsigned)(tilesM * tilesN));
    THIP_ENQUEUE(ctx, kernelLabel("igemm_i8", {BM, BN, BK, LOADER, G}), kernel, grid, dim3(256), smem, a);
    return hipGetLastError();
}

template <int BM, int BN, int BK>
static hipError_t launchIgemmLoader(const IgemmArgs &a, const LaunchCtx &ctx) {
    if (a.loader == kLoaderDense) {
        return launchIgemmTile<BM, BN, BK, kLoaderDense, 16>(a, ctx);
    }
    if (a.loader == kLoaderRuns) {
        return launchIgemmTile<BM, BN, BK, kLoaderRuns, 16>(a, ctx);
    }
    switch (a.gran) {
    case 16: return launchIgemmTile<BM, BN, BK, kLoaderGather, 16>(a, ctx);
    case 8: return launchIgemmTile<BM, BN, BK, kLoaderGather, 8>(a, ctx);
    case 4: return launchIgemmTile<BM, BN, BK, kLoaderGather, 4>(a, ctx);
    case 2: return launchIgemmTile<BM, BN, BK, kLoaderGather, 2>(a, ctx);
    case 1: return launchIgemmTile<BM, BN, BK, kLoaderGather, 1>(a, ctx);
    default: return hipErrorInvalidValue;
    }
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int STAGES, int BLOCKS_PER_CU, int DIRECT, bool ADD = false, bool CONV = false, int BK = 64>
static hipError_t launchIgemmDenseE(const IgemmArgs &a, const LaunchCtx &ctx) {
    // the stage ring, reused by the epilogue as staging slices (one per wave) plus bias/scale
    constexpr size_t ring = (size_t)STAGES * (BM + BN) * BK;
    constexpr size_t epilogue = (size_t)(BM / WAVES_M) * (WAVES_M * WAVES_N) * (32 * 4 + 16) + 2 * BN * 4;
    constexpr size_t smem = ring > epilogue ? ring : epilogue;
    static_assert(smem * BLOCKS_PER_CU <= 160 * 1024, "LDS of one CU");
    auto kernel = igemm_dense_i8<BM, BN, WAVES_M, WAVES_N, STAGES, BLOCKS_PER_CU, DIRECT, ADD, CONV, BK>;
    static std::once_flag once;
    static hipError_t configured = hipSuccess;
    std::call_once(once, [&] { configured = hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem); });
    if (configured != hipSuccess) return configured;
    const int tilesM = (a.M + BM - 1) / BM;
    const int tilesN = a.Np / BN;
    THIP_ENQUEUE(ctx, kernelLabel(CONV ? "igemm_dense_conv_i8" : BK == 128 ? "igemm_dense_k128_i8" : "igemm_dense_i8", {BM, BN, WAVES_M, WAVES_N, STAGES, BLOCKS_PER_CU, DIRECT, ADD}), kernel, dim3((unsigned)(tilesM * tilesN)), dim3(WAVES_M * WAVES_N * 64), smem, a);
    return hipGetLastError();
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int STAGES, int BLOCKS_PER_CU, bool CONV = false, int BK = 64>
static hipError_t launchIgemmDense(const IgemmArgs &a, const LaunchCtx &ctx) {
    // the in-register epilogue takes the 32-bit requant tails: the plain one (what wideRequant() calls plain), or the
    // general one (any shift of 32 and up, or a smaller one that the record's pre_shift lifts to 33; on the small tiles
    // it is 2-9 % ahead of the staged epilogue: 512 x 4096 x 4096 with the literal requant range, 14.4 -> 14.1 us)
    const bool plain = a.rq.shift >= 33 && a.rq.shift <= 45 && a.rq.pre_shift == 0 && a.rq.t0_clamp == 0 &&
                       a.rq.out_zp >= -32768 && a.rq.out_zp <= 32767 && a.rq.out_min <= a.rq.out_max;
    const bool wide = (a.rq.shift >= 32 || (a.rq.pre_shift > 0 && a.rq.shift + a.rq.pre_shift == 33)) && a.rq.out_min <= a.rq.out_max;
    const bool inRegisters = a.out_dtype == kDtypeI8 && a.N % 16 == 0 && ((uintptr_t)a.out & 15) == 0 && !ctx.tuning->noDirectEpilogue;
    const bool direct = inRegisters && plain;
    if (a.skip != nullptr) {
        // a residual add: the in-register epilogue of the small tile only (what a network's late, small layers take)
        if constexpr (BM == 64 && BN == 64 && !CONV) {
            if (!direct || ((uintptr_t)a.skip & 15) != 0) return hipErrorInvalidValue;
            return launchIgemmDenseE<BM, BN, WAVES_M, WAVES_N, STAGES, BLOCKS_PER_CU, 1, true>(a, ctx);
        } else {
            return hipErrorInvalidValue;
        }
    }
    if (direct) return launchIgemmDenseE<BM, BN, WAVES_M, WAVES_N, STAGES, BLOCKS_PER_CU, 1, false, CONV, BK>(a, ctx);
    if (inRegisters && wide) return launchIgemmDenseE<BM, BN, WAVES_M, WAVES_N, STAGES, BLOCKS_PER_CU, 2, false, CONV, BK>(a, ctx);
    return launchIgemmDenseE<BM, BN, WAVES_M, WAVES_N, STAGES, BLOCKS_PER_CU, 0, false, CONV, BK>(a, ctx);
}

hipError_t launchIgemm(const IgemmArgs &a, uint32_t variant, const LaunchCtx &ctx) {
    if (variant >= kIgemmVariantCount) return hipErrorInvalidValue;
    const IgemmTile &t = igemmTile(variant);
    // What the kernel assumes: padded sizes are whole tiles, the real sizes fit
    // inside them, the dense loader reads whole 16-byte chunks of each row.
    if (a.M <= 0 || a.N <= 0 || a.K <= 0) return hipErrorInvalidValue;
    if (a.Kp % t.bk != 0 || a.Np % t.bn != 0 || a.K > a.Kp || a.N > a.Np) return hipErrorInvalidValue;
    if (!a.A || !a.Bp || !a.bias || !a.scale || !a.out) return hipErrorInvalidValue;
    if (a.loader == kLoaderDense) {
        if (a.K % 16 != 0 || ((uintptr_t)a.A & 15) != 0) return hipErrorInvalidValue;
    } else if (a.loader == kLoaderRuns) {
        if (!a.ktab || a.C <= 0 || a.C > 16 || a.a_bytes < 16) return hipErrorInvalidValue;
        if (a.OH <= 0 || a.OW <= 0 || a.M % (a.OH * a.OW) != 0) return hipErrorInvalidValue;
        if (a.a_bytes != (long long)(a.M / (a.OH * a.OW)) * a.H * a.W * a.C) return hipErrorInvalidValue;
    } else if (a.loader == kLoaderGather) {
        if (!a.ktab || a.C <= 0 || a.C % (int)a.gran != 0) return hipErrorInvalidValue;
        if (a.OH <= 0 || a.OW <= 0 || a.M % (a.OH * a.OW) != 0) return hipErrorInvalidValue;
        if (((uintptr_t)a.A & (a.gran - 1)) != 0) return hipErrorInvalidValue;
    } else if (a.loader == kLoaderWindow) {
        // the ring kernel's window addressing: whole 16-byte chunks per tap (so the walk wraps the channel at most
        // bk / 16 times per k-tile), 32-bit byte offsets into the image, a page of zero-point bytes behind ktab,
        // every tap offset non-negative once the tap lies inside the image, K rounded up to whole k-tiles
        if (!a.ktab || ((uintptr_t)a.ktab & 15) != 0 || a.C < 16 || a.C % 16 != 0 || a.KH <= 0 || a.KW <= 0) return hipErrorInvalidValue;
        if (a.H <= 0 || a.W <= 0 || a.OH <= 0 || a.OW <= 0 || a.SH <= 0 || a.SW <= 0 || a.PT < 0 || a.PL < 0) return hipErrorInvalidValue;
        if (a.M % (a.OH * a.OW) != 0 || (long long)a.K != (long long)a.KH * a.KW * a.C || a.Kp != (a.K + t.bk - 1) / t.bk * t.bk) return hipErrorInvalidValue;
        if (a.a_bytes != (long long)(a.M / (a.OH * a.OW)) * a.H * a.W * a.C || a.a_bytes >= (1LL << 32)) return hipErrorInvalidValue;
        if (((uintptr_t)a.A & 15) != 0 || a.skip != nullptr) return hipErrorInvalidValue;
        switch (variant) {
        case kIgemmDense256x256: return launchIgemmDense<256, 256, 2, 2, 4, 1, true>(a, ctx);
        case kIgemmDense128x256:
            // a long K in whole 128-byte k-tiles: whole cache lines per tile row, two stages (512 -> 512 at 14 x 14,
            // batch 64: 34.5 us against 36.8; on 128 x 128, batch 32: 21.4 against 24.4)
            if (a.Kp >= 2304 && a.Kp % 128 == 0 && !ctx.tuning->noK128) return launchIgemmDense<128, 256, 2, 2, 2, 1, true, 128>(a, ctx);
            return launchIgemmDense<128, 256, 2, 2, 3, 2, true>(a, ctx);
        case kIgemmDense128x128:
            if (a.Kp >= 2304 && a.Kp % 128 == 0 && !ctx.tuning->noK128) return launchIgemmDense<128, 128, 2, 2, 2, 2, true, 128>(a, ctx);
            return launchIgemmDense<128, 128, 2, 2, 4, 2, true>(a, ctx);
        case kIgemmDense256x128: return launchIgemmDense<256, 128, 2, 2, 3, 2, true>(a, ctx);
        case kIgemmDense256x64: return launchIgemmDense<256, 64, 4, 1, 3, 2, true>(a, ctx);
        case kIgemmDense64x64: return launchIgemmDense<64, 64, 2, 2, 4, 4, true>(a, ctx);  // four stages: measured against three and five
        case kIgemmDense256x32: return launchIgemmDense<256, 32, 4, 1, 3, 2, true>(a, ctx);
        case kIgemmDense256x256K128: return launchIgemmDense<256, 256, 2, 2, 2, 1, true, 128>(a, ctx);  // 128 channels per k-tile
        default: return hipErrorInvalidValue;
        }
    } else {
        return hipErrorInvalidValue;
    }
    if (variant >= kIgemmDense256x256 && a.loader != kLoaderDense && !(variant == kIgemmStream && a.loader == kLoaderRuns)) {
        return hipErrorInvalidValue;
    }
    if (((uintptr_t)a.Bp & 15) != 0) return hipErrorInvalidValue;
    if (a.out_dtype < kDtypeI8 || a.out_dtype > kDtypeI32) return hipErrorInvalidValue;
    if (a.skip != nullptr && variant != kIgemmStream && variant != kIgemmDense64x64) return hipErrorInvalidValue;  // the kernels that can add a residual
    switch (variant) {
    case kIgemm128x128x64: return launchIgemmLoader<128, 128, 64>(a, ctx);
    case kIgemm256x256x64: return launchIgemmLoader<256, 256, 64>(a, ctx);
    case kIgemm64x64x64: return launchIgemmLoader<64, 64, 64>(a, ctx);
    case kIgemm256x128x64: return launchIgemmLoader<256, 128, 64>(a, ctx);
    case kIgemmDense256x256: return launchIgemmDense<256, 256, 2, 2, 4, 1>(a, ctx);
    case kIgemmDense128x128:
        // a short K (up to four k-tiles) never fills a deep ring: two stages leave LDS for four blocks per CU, whose
        // prologues and epilogues overlap (256 -> 1024 channels at 56 x 56, batch 8: 13.5 us against 17.4)
        // (with fewer than two tiles per CU there is nothing to overlap, and the deeper ring is 2 us ahead)
        if (a.Kp <= ctx.tuning->denseShortK && (long long)((a.M + 127) / 128) * (a.Np / 128) >= 512) return launchIgemmDense<128, 128, 2, 2, 2, 4>(a, ctx);
        // a long K in whole 128-byte k-tiles and more tiles than CUs: whole cache lines per tile row, two stages
        // (1536 x 4096 x 4096: 28.8 us against 35.1; with one tile per CU the four-stage ring is ahead, 20.8 against 22.7)
        if (a.Kp >= 4096 && a.Kp % 128 == 0 && (long long)((a.M + 127) / 128) * (a.Np / 128) > 256 && !ctx.tuning->noK128) {
            return launchIgemmDense<128, 128, 2, 2, 2, 2, false, 128>(a, ctx);
        }
        return launchIgemmDense<128, 128, 2, 2, 4, 2>(a, ctx);
    case kIgemmDense128x256:
        // (the same on this tile, one block per CU: 1024 x 8192 x 8192 64.1 us against 72.3, never behind)
        if (a.Kp >= 4096 && a.Kp % 128 == 0 && !ctx.tuning->noK128) return launchIgemmDense<128, 256, 2, 2, 2, 1, false, 128>(a, ctx);
        return launchIgemmDense<128, 256, 2, 2, 3, 2>(a, ctx);
    case kIgemmDense64x64: return launchIgemmDense<64, 64, 2, 2, 4, 4>(a, ctx);
    case kIgemmDense256x128: return launchIgemmDense<256, 128, 2, 2, 3, 2>(a, ctx);
    case kIgemmDense256x64: return launchIgemmDense<256, 64, 4, 1, 3, 2>(a, ctx);
    case kIgemmDense256x32: return launchIgemmDense<256, 32, 4, 1, 3, 2>(a, ctx);
    case kIgemmStream: return launchIgemmStream(a, ctx);
    case kIgemmDense128x64: return launchIgemmDense<128, 64, 2, 2, 4, 2>(a, ctx);
    case kIgemmDense64x128:
        // a long K in whole 128-byte k-tiles: whole cache lines per tile row here as well, three stages deep
        // (512 x 4096 x 4096: 12.8 us against 13.9, 256 x 4096 x 8192: 13.1 against 15.0; at K = 2048 the 64-byte
        // k-tiles with four stages are ahead, 7.7 against 8.1)
        if (a.Kp >= 4096 && a.Kp % 128 == 0 && !ctx.tuning->noK128) return launchIgemmDense<64, 128, 2, 2, 3, 2, false, 128>(a, ctx);
        return launchIgemmDense<64, 128, 2, 2, 4, 2>(a, ctx);
    case kIgemmDense256x256K128: return launchIgemmDense<256, 256, 2, 2, 2, 1, false, 128>(a, ctx);
    default: return hipErrorInvalidValue;
    }
}

// ---------------------------------------------------------------------------
// fc_skinny: out[m][n] = requant(sum_k x[m][k] * w[n][k]) for M <= 16.
// One wave per NW output columns; lanes split K in 16-byte chunks, so one wave
// load of a weight row is 1 KiB contiguous.  Partial sums are reduced with
// wave shuffles.  K % 16 == 0.
// ---------------------------------------------------------------------------
template <int MR, int NW>
__global__ __launch_bounds__(256) void fc_skinny(FcSkinnyArgs p) {
    const int lane = threadIdx.x & 63;
    const int wave = (int)((blockIdx.x * 256 + threadIdx.x) >> 6);
    const int n0 = wave * NW;
    if (n0 >= p.N) return;
    int32_t acc[MR][NW];
#pragma unroll
    for (int m = 0; m < MR; m++) {
#pragma unroll
        for (int j = 0; j < NW; j++) acc[m][j] = 0;
    }
    const int chunks = p.K / 16;
    for (int c = lane; c < chunks; c += 64) {
        v4i wv[NW];
#pragma unroll
        for (int j = 0; j < NW; j++) {
            const int n = (n0 + j) < p.N ? (n0 + j) : (p.N - 1);
            wv[j] = *(const v4i *)(p.w + (size_t)n * p.K + (size_t)c * 16);
        }
#pragma unroll
        for (int m = 0; m < MR; m++) {
            if (m < p.M) {
                const v4i xv = *(const v4i *)(p.x + (size_t)m * p.K + (size_t)c * 16);
#pragma unroll
                for (int j = 0; j < NW; j++) {
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        acc[m][j] = __builtin_amdgcn_sdot4(xv[q], wv[j][q], acc[m][j], false);
                    }
                }
            }
        }
    }
#pragma unroll
    for (int m = 0; m < MR; m++) {
#pragma unroll
        for (int j = 0; j < NW; j++) {
            int32_t v = acc[m][j];
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
            acc[m][j] = v;
        }
    }
    if (lane == 0) {
        const long long rnd = roundTerm(p.rq.shift);
#pragma unroll
        for (int j = 0; j < NW; j++) {
            const int n = n0 + j;
            if (n < p.N) {
                const int32_t bias = p.bias[n], scale = p.scale[n];
#pragma unroll
                for (int m = 0; m < MR; m++) {
                    if (m < p.M) {
                        storeElem(p.out, (size_t)m * p.N + n, requant(acc[m][j], bias, scale, rnd, p.rq),
                                  p.out_dtype);
                    }
                }
            }
        }
    }
}

// fc_skinny_mfma: the same op for 2 .. 16 rows on v_mfma_i32_16x16x64_i8.  A block owns 16 output
// columns; its four waves split K and add their partial sums through LDS.  Per 256 bytes of K a lane
// loads 64 contiguous bytes of one weight row and of one activation row (lane l: row l & 15, bytes
// 64 (l >> 4) .. + 63 of the 256), and MFMA step s takes 16-byte piece s of every lane: the k order
// inside the 256 bytes is permuted, identically for both operands, so that every load instruction
// of a wave covers whole 256-byte stretches of 16 rows.  The weights are the MFMA's first operand:
// lane l then holds out[m = l & 15][n0 + 4 (l >> 4) + r], r = 0 .. 3: four consecutive columns.
__global__ __launch_bounds__(256) void fc_skinny_mfma(FcSkinnyArgs p) {
    __shared__ int32_t partial[3][4][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 15, kg = lane >> 4;
    const int n0 = blockIdx.x * 16;
    const int nrow = n0 + r < p.N ? n0 + r : p.N - 1;  // clamped: such columns are never stored
    const int mrow = r < p.M ? r : p.M - 1;
    const int8_t *wrow = p.w + (size_t)nrow * p.K;
    const int8_t *xrow = p.x + (size_t)mrow * p.K;
    // this wave's share of K, in whole 256-byte steps
    const int steps = (p.K + 255) / 256, per = (steps + 3) / 4;
    const int sBeg = wave * per, sEnd = (sBeg + per) < steps ? (sBeg + per) : steps;
    v4i acc = {0, 0, 0, 0};
    for (int s = sBeg; s < sEnd; s++) {
        const int k = s * 256 + 64 * kg;
        v4i wv[4], xv[4];
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const bool in = k + 16 * c < p.K;  // K % 16 == 0: a piece is inside K or outside
            wv[c] = in ? *(const v4i *)(wrow + k + 16 * c) : v4i{0, 0, 0, 0};
            xv[c] = in ? *(const v4i *)(xrow + k + 16 * c) : v4i{0, 0, 0, 0};
        }
#pragma unroll
        for (int c = 0; c < 4; c++) acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(wv[c], xv[c], acc, 0, 0, 0);
    }
    if (wave > 0) {
#pragma unroll
        for (int e = 0; e < 4; e++) partial[wave - 1][e][lane] = acc[e];
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int w = 0; w < 3; w++) {
#pragma unroll
        for (int e = 0; e < 4; e++) acc[e] += partial[w][e][lane];
    }
    const int m = r, n = n0 + 4 * kg;
    if (m >= p.M || n >= p.N) return;
    const long long rnd = roundTerm(p.rq.shift);
    int32_t q[4];
#pragma unroll
    for (int e = 0; e < 4; e++) {
        const int ne = n + e < p.N ? n + e : p.N - 1;
        q[e] = requant(acc[e], p.bias[ne], p.scale[ne], rnd, p.rq);
    }
    if (p.out_dtype == kDtypeI8 && (p.N & 3) == 0) {
        *(uint32_t *)((int8_t *)p.out + (size_t)m * p.N + n) = packBytes(q[0], q[1], q[2], q[3]);
    } else {
#pragma unroll
        for (int e = 0; e < 4; e++) {
            if (n + e < p.N) storeElem(p.out, (size_t)m * p.N + n + e, q[e], p.out_dtype);
        }
    }
}

template <int MR, int NW>
static hipError_t launchFcSkinnyT(const FcSkinnyArgs &a, const LaunchCtx &ctx) {
    const int waves = (a.N + NW - 1) / NW;
    const dim3 grid((unsigned)((waves + 3) / 4));
    THIP_ENQUEUE(ctx, kernelLabel("fc_skinny", {MR, NW}), (fc_skinny<MR, NW>), grid, dim3(256), 0, a);
    return hipGetLastError();
}

hipError_t launchFcSkinny(const FcSkinnyArgs &a, const LaunchCtx &ctx) {
    if (a.M <= 0 || a.M > kFcSkinnyMaxRows || a.N <= 0 || a.K <= 0 || a.K % 16 != 0) {
        return hipErrorInvalidValue;
    }
    if (!a.x || !a.w || !a.bias || !a.scale || !a.out) return hipErrorInvalidValue;
    if ((((uintptr_t)a.x) | ((uintptr_t)a.w)) & 15) return hipErrorInvalidValue;
    if (a.out_dtype < kDtypeI8 || a.out_dtype > kDtypeI32) return hipErrorInvalidValue;
    if (a.M == 1) return launchFcSkinnyT<1, 4>(a, ctx);
    if (a.M >= 2 && ((uintptr_t)a.out & 3) == 0 && !ctx.tuning->skinnyDot4) {  // two rows: 3.4 us against 5.6 on the dot-product kernel (2048 x 2048)
        THIP_ENQUEUE(ctx, "fc_skinny_mfma", fc_skinny_mfma, dim3((unsigned)((a.N + 15) / 16)), dim3(256), 0, a);
        return hipGetLastError();
    }
    if (a.M <= 4) return launchFcSkinnyT<4, 4>(a, ctx);
    if (a.M <= 8) return launchFcSkinnyT<8, 2>(a, ctx);
    return launchFcSkinnyT<16, 2>(a, ctx);
}

// ---------------------------------------------------------------------------
// Bandwidth-bound kernels.  One thread = VEC consecutive channels of one
// output pixel (NHWC), VEC bytes per load/store (16 when C % 16 == 0).
// ---------------------------------------------------------------------------
template <int VEC>
struct ByteVec;
template <>
struct ByteVec<16> {
    typedef v4i type;
};
template <>
struct ByteVec<8> {
    typedef v2i type;
};
template <>
struct ByteVec<4> {
    typedef int type;
};
template <>
struct ByteVec<1> {
    typedef int8_t type;
};

template <int VEC>
union Pack {
    typename ByteVec<VEC>::type v;
    int8_t b[VEC];
};

template <int VEC, int KS>  // KS > 0: square KS x KS window known at compile time
__global__ __launch_bounds__(256) void depthwise_i8(DepthwiseArgs p, WorkSplit ws) {
    const int cg = p.C / VEC;
    const long long total = (long long)p.N * p.OH * p.OW * cg;
    const long long t = (long long)blockIdx.x * 256 + threadIdx.x;
    if (t >= total) return;
    int cgi, ox, oy, n;
    splitWork(t, ws, cgi, ox, oy, n);
    const int c0 = cgi * VEC;
    const int KH = KS > 0 ? KS : p.KH, KW = KS > 0 ? KS : p.KW;
    const int iy0 = oy * p.SH - p.PT, ix0 = ox * p.SW - p.PL;
    const int8_t *img = p.in + (size_t)n * p.H * p.W * p.C + c0;
    int32_t acc[VEC];
#pragma unroll
    for (int v = 0; v < VEC; v++) acc[v] = 0;
#pragma unroll
    for (int kh = 0; kh < KH; kh++) {
        const int iy = iy0 + kh;
#pragma unroll
        for (int kw = 0; kw < KW; kw++) {
            const int ix = ix0 + kw;
            Pack<VEC> x, w;
            w.v = *(const typename ByteVec<VEC>::type *)(p.wpk + (size_t)(kh * KW + kw) * p.C + c0);
            if ((unsigned)iy < (unsigned)p.H && (unsigned)ix < (unsigned)p.W) {
                x.v = *(const typename ByteVec<VEC>::type *)(img + ((size_t)iy * p.W + ix) * p.C);
#pragma unroll
                for (int v = 0; v < VEC; v++) acc[v] += (int32_t)x.b[v] * (int32_t)w.b[v];
            } else {
#pragma unroll
                for (int v = 0; v < VEC; v++) acc[v] += p.input_zp * (int32_t)w.b[v];
            }
        }
    }
    const long long rnd = roundTerm(p.rq.shift);
    Pack<VEC> o;
#pragma unroll
    for (int v = 0; v < VEC; v++) {
        o.b[v] = (int8_t)requant(acc[v], p.bias[c0 + v], p.scale[c0 + v], rnd, p.rq);
    }
    *(typename ByteVec<VEC>::type *)(p.out + (((size_t)n * p.OH + oy) * p.OW + ox) * p.C + c0) = o.v;
}

// Blocks are handed to the eight XCDs in turn (block b runs on XCD b % 8), each with an L2 of its own.  This
// renumbering gives every XCD one contiguous eighth of the blocks, so that blocks whose threads read the same input
// (neighbouring column strips share two of four columns) find it in their own L2 instead of fetching it eight times.
__device__ __forceinline__ unsigned xcdContiguousBlock() {
    const unsigned nb = gridDim.x, x = blockIdx.x & 7u, i = blockIdx.x >> 3, per = nb >> 3, rem = nb & 7u;
    return x * per + (x < rem ? x : rem) + i;
}

// 3x3 depthwise with the window row as the dot dimension.  A thread owns 16 channels of P
// horizontally adjacent output pixels.  The three taps of a window row are brought together per
// channel with two byte permutes ([x(kw0), x(kw1), x(kw2), 0] in one register) and multiplied by the
// matching packed weights with one v_dot4_i32_i8: 3 dot4 + 6 permutes per channel instead of 9
// multiply-adds on unpacked bytes.  P > 1 shares the input columns that neighbouring windows have
// in common and loads weights, bias and scale once for P outputs, which is what matters here:
// the kernel is bound by the traffic through the vector L1, not by arithmetic.
// SWT is the horizontal stride when it is 1 or 2 (P > 1 needs it at compile time), 0 = run time.
template <int P, int SWT>
__global__ __launch_bounds__(256) void depthwise3x3_dot4_i8(DepthwiseArgs p, WorkSplit ws) {
    static_assert(P == 1 || SWT > 0, "several pixels per thread need a compile-time stride");
    const int SW = SWT > 0 ? SWT : p.SW;
    constexpr int NC = SWT > 0 ? (P - 1) * SWT + 3 : 3;  // input columns one window row of the thread spans
    const int cg = p.C / 16;
    const int oxGroups = (p.OW + P - 1) / P;
    const long long total = (long long)p.N * p.OH * oxGroups * cg;
    const long long t = (long long)xcdContiguousBlock() * 256 + threadIdx.x;
    if (t >= total) return;
    int cgi, oxg, oy, n;
    splitWork(t, ws, cgi, oxg, oy, n);
    const int c0 = cgi * 16, ox0 = oxg * P;
    const int iy0 = oy * p.SH - p.PT, ix0 = ox0 * SW - p.PL;
    const int8_t *img = p.in + (size_t)n * p.H * p.W * p.C + c0;
    const uint32_t zp4 = (uint32_t)(p.input_zp & 0xff) * 0x01010101u;
    const uint32_t *wrow = (const uint32_t *)p.wpk + c0;
    // the accumulators start at the bias: the first dot product takes it as its addend, which saves clearing the
    // accumulator and adding the bias afterwards (int32 wrap-around is the same in either order)
    int32_t acc[P][16];
#pragma unroll
    for (int g = 0; g < 4; g++) {
        const v4i b4 = *(const v4i *)(p.bias + c0 + 4 * g);
#pragma unroll
        for (int q = 0; q < P; q++) {
#pragma unroll
            for (int c = 0; c < 4; c++) acc[q][4 * g + c] = b4[c];
        }
    }
#pragma unroll
    for (int kh = 0; kh < 3; kh++) {
        const int iy = iy0 + kh;
        const bool rowIn = (unsigned)iy < (unsigned)p.H;
        v4i d[NC];
#pragma unroll
        for (int j = 0; j < NC; j++) {
            const int ix = ix0 + j;
            if (rowIn && (unsigned)ix < (unsigned)p.W) {
                d[j] = *(const v4i *)(img + ((size_t)iy * p.W + ix) * p.C);
            } else {
                d[j] = v4i{(int)zp4, (int)zp4, (int)zp4, (int)zp4};
            }
        }
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const v4i w4 = *(const v4i *)(wrow + (size_t)kh * p.C + 4 * g);
#pragma unroll
            for (int q = 0; q < P; q++) {
                const int j0 = SWT > 0 ? q * SWT : 0;
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    // byte c of column j0, byte c of column j0+1, then byte c of column j0+2, then zero
                    const uint32_t t01 = __builtin_amdgcn_perm((uint32_t)d[j0 + 1][g], (uint32_t)d[j0][g], 0x0c0c0000u | ((4u + c) << 8) | (uint32_t)c);
                    const uint32_t x3 = __builtin_amdgcn_perm((uint32_t)d[j0 + 2][g], t01, 0x0c000100u | ((4u + c) << 16));
                    acc[q][4 * g + c] = __builtin_amdgcn_sdot4((int)x3, w4[c], acc[q][4 * g + c], false);
                }
            }
        }
    }
    const WideRequant wrq = wideRequant(p.rq);
    const long long rnd = roundTerm(p.rq.shift);
    v4i o[P];
    withRequantMode(wrq, [&](auto mode) {
        constexpr int kMode = decltype(mode)::value;
#pragma unroll
        for (int g = 0; g < 4; g++) {
            const v4i s4 = *(const v4i *)(p.scale + c0 + 4 * g);
#pragma unroll
            for (int q = 0; q < P; q++) {
                int32_t v[4];
#pragma unroll
                for (int c = 0; c < 4; c++) v[c] = requantT0<kMode>(acc[q][4 * g + c], s4[c], rnd, p.rq, wrq);
                o[q][g] = (int)packBytes(v[0], v[1], v[2], v[3]);
            }
        }
    });
#pragma unroll
    for (int q = 0; q < P; q++) {
        if (ox0 + q < p.OW) *(v4i *)(p.out + (((size_t)n * p.OH + oy) * p.OW + ox0 + q) * p.C + c0) = o[q];
    }
}

template <int P, int SWT>
static hipError_t launchDepthwiseDot4(const DepthwiseArgs &a, const LaunchCtx &ctx) {
    const long long total = (long long)a.N * a.OH * ((a.OW + P - 1) / P) * (a.C / 16);
    const WorkSplit ws = makeWorkSplit(total, a.C / 16, (a.OW + P - 1) / P, a.OH);
    THIP_ENQUEUE(ctx, kernelLabel("depthwise3x3_dot4_i8", {P, SWT}), (depthwise3x3_dot4_i8<P, SWT>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, a, ws);
    return hipGetLastError();
}

// 3x3 depthwise for large images: a thread owns 16 channels of a tile of R x P output pixels
// (stride S in both directions).  Each input row of the tile is loaded once and serves every
// output row that overlaps it.  Per group of 4 channels, four adjacent columns of a row (one
// dword each, a byte per channel) are transposed with 8 byte permutes into one dword per channel
// holding that channel at the four columns; a v_dot4_i32_i8 with the weights [w0, w1, w2, 0]
// gives the window row at the block's first column and, for stride 1, with [0, w0, w1, w2] the
// one at its second column.  That is about one permute and three dot products per output instead
// of six and three.
template <int G>
struct DwordVec {
    typedef v4i type;
};
template <>
struct DwordVec<2> {
    typedef v2i type;
};
template <>
struct DwordVec<1> {
    typedef int type;
};
template <int G>
__device__ __forceinline__ void loadDwords(const int8_t *src, int (&dst)[G]) {
    union {
        typename DwordVec<G>::type v;
        int w[G];
    } u;
    u.v = *(const typename DwordVec<G>::type *)src;
#pragma unroll
    for (int g = 0; g < G; g++) dst[g] = u.w[g];
}

// G = channels per thread / 4.  Fewer channels per thread mean fewer registers and more waves per SIMD
// (the loads stay coalesced: neighbouring lanes hold neighbouring channel groups).
template <int P, int R, int S, int G>
__global__ __launch_bounds__(256) void depthwise3x3_tile_i8(DepthwiseArgs p, WorkSplit ws) {
    static_assert(S == 1 || S == 2, "stride 1 or 2");
    static_assert(S == 2 || P % 2 == 0, "stride 1 pairs the pixels of a block");
    constexpr int NC = (P - 1) * S + 3, NR = (R - 1) * S + 3;
    constexpr int NBK = S == 1 ? P / 2 : P;  // blocks of four columns per row; block b starts at column 2 b
    constexpr int CV = 4 * G;
    const int cg = p.C / CV;
    const int oxGroups = (p.OW + P - 1) / P, oyGroups = (p.OH + R - 1) / R;
    const long long total = (long long)p.N * oyGroups * oxGroups * cg;
    const long long t = (long long)xcdContiguousBlock() * 256 + threadIdx.x;
    if (t >= total) return;
    int cgi, oxg, oyg, n;
    splitWork(t, ws, cgi, oxg, oyg, n);
    const int c0 = cgi * CV, ox0 = oxg * P, oy0 = oyg * R;
    const int iy0 = oy0 * S - p.PT, ix0 = ox0 * S - p.PL;
    const int8_t *img = p.in + (size_t)n * p.H * p.W * p.C + c0;
    const int zp4 = (int)((uint32_t)(p.input_zp & 0xff) * 0x01010101u);
    int d[NR][NC][G];
    if (iy0 >= 0 && iy0 + NR <= p.H && ix0 >= 0 && ix0 + NC <= p.W) {
        const int8_t *base = img + ((size_t)iy0 * p.W + ix0) * p.C;
#pragma unroll
        for (int i = 0; i < NR; i++) {
#pragma unroll
            for (int j = 0; j < NC; j++) loadDwords<G>(base + ((size_t)i * p.W + j) * p.C, d[i][j]);
        }
    } else {
#pragma unroll
        for (int i = 0; i < NR; i++) {
            const int iy = iy0 + i;
            const int iyc = iy < 0 ? 0 : iy >= p.H ? p.H - 1 : iy;
#pragma unroll
            for (int j = 0; j < NC; j++) {
                const int ix = ix0 + j;
                const int ixc = ix < 0 ? 0 : ix >= p.W ? p.W - 1 : ix;
                loadDwords<G>(img + ((size_t)iyc * p.W + ixc) * p.C, d[i][j]);
                const bool inside = iy == iyc && ix == ixc;
#pragma unroll
                for (int g = 0; g < G; g++) d[i][j][g] = inside ? d[i][j][g] : zp4;
            }
        }
    }
    const WideRequant wrq = wideRequant(p.rq);
    const long long rnd = roundTerm(p.rq.shift);
    const uint32_t *wrow = (const uint32_t *)p.wpk + c0;
    int o[R][P][G];
    withRequantMode(wrq, [&](auto mode) {
        constexpr int kMode = decltype(mode)::value;
#pragma unroll
        for (int g = 0; g < G; g++) {
            v4i wk[3];
#pragma unroll
            for (int kh = 0; kh < 3; kh++) wk[kh] = *(const v4i *)(wrow + (size_t)kh * p.C + 4 * g);
            const v4i b4 = *(const v4i *)(p.bias + c0 + 4 * g);
            const v4i s4 = *(const v4i *)(p.scale + c0 + 4 * g);
            int32_t acc[R][P][4];
#pragma unroll
            for (int r = 0; r < R; r++) {
#pragma unroll
                for (int q = 0; q < P; q++) {
#pragma unroll
                    for (int c = 0; c < 4; c++) acc[r][q][c] = 0;
                }
            }
#pragma unroll
            for (int i = 0; i < NR; i++) {
#pragma unroll
                for (int b = 0; b < NBK; b++) {
                    const uint32_t x0 = (uint32_t)d[i][2 * b][g], x1 = (uint32_t)d[i][2 * b + 1][g], x2 = (uint32_t)d[i][2 * b + 2][g];
                    // the last block of a stride-2 row has no fourth column; its weight is zero
                    const uint32_t x3 = (uint32_t)d[i][2 * b + 3 < NC ? 2 * b + 3 : 2 * b + 2][g];
                    // 4 x 4 byte transpose: tr[c] = channel c at columns 2b .. 2b+3
                    const uint32_t lo01 = __builtin_amdgcn_perm(x1, x0, 0x05010400u), hi01 = __builtin_amdgcn_perm(x1, x0, 0x07030602u);
                    const uint32_t lo23 = __builtin_amdgcn_perm(x3, x2, 0x05010400u), hi23 = __builtin_amdgcn_perm(x3, x2, 0x07030602u);
                    const uint32_t tr[4] = {__builtin_amdgcn_perm(lo23, lo01, 0x05040100u), __builtin_amdgcn_perm(lo23, lo01, 0x07060302u),
                                            __builtin_amdgcn_perm(hi23, hi01, 0x05040100u), __builtin_amdgcn_perm(hi23, hi01, 0x07060302u)};
#pragma unroll
                    for (int r = 0; r < R; r++) {
                        const int kh = i - r * S;
                        if (kh < 0 || kh > 2) continue;
#pragma unroll
                        for (int c = 0; c < 4; c++) {
                            if (S == 1) {
                                acc[r][2 * b][c] = __builtin_amdgcn_sdot4((int)tr[c], wk[kh][c], acc[r][2 * b][c], false);
                                acc[r][2 * b + 1][c] = __builtin_amdgcn_sdot4((int)tr[c], (int)((uint32_t)wk[kh][c] << 8), acc[r][2 * b + 1][c], false);
                            } else {
                                acc[r][b][c] = __builtin_amdgcn_sdot4((int)tr[c], wk[kh][c], acc[r][b][c], false);
                            }
                        }
                    }
                }
            }
#pragma unroll
            for (int r = 0; r < R; r++) {
#pragma unroll
                for (int q = 0; q < P; q++) {
                    int32_t v[4];
#pragma unroll
                    for (int c = 0; c < 4; c++) {
                        v[c] = requantT0<kMode>((int32_t)((uint32_t)acc[r][q][c] + (uint32_t)b4[c]), s4[c], rnd, p.rq, wrq);
                    }
                    o[r][q][g] = (int)packBytes(v[0], v[1], v[2], v[3]);
                }
            }
        }
    });
#pragma unroll
    for (int r = 0; r < R; r++) {
#pragma unroll
        for (int q = 0; q < P; q++) {
            if (oy0 + r < p.OH && ox0 + q < p.OW) {
                union {
                    typename DwordVec<G>::type v;
                    int w[G];
                } u;
#pragma unroll
                for (int g = 0; g < G; g++) u.w[g] = o[r][q][g];
                *(typename DwordVec<G>::type *)(p.out + (((size_t)n * p.OH + oy0 + r) * p.OW + ox0 + q) * p.C + c0) = u.v;
            }
        }
    }
}

template <int P, int R, int S, int G>
static hipError_t launchDepthwiseTile(const DepthwiseArgs &a, const LaunchCtx &ctx) {
    const long long total = (long long)a.N * ((a.OH + R - 1) / R) * ((a.OW + P - 1) / P) * (a.C / (4 * G));
    const WorkSplit ws = makeWorkSplit(total, a.C / (4 * G), (a.OW + P - 1) / P, (a.OH + R - 1) / R);
    THIP_ENQUEUE(ctx, kernelLabel("depthwise3x3_tile_i8", {P, R, S, G}), (depthwise3x3_tile_i8<P, R, S, G>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, a, ws);
    return hipGetLastError();
}

// 3x3 depthwise as a rolling window: a thread owns 4 G channels of P adjacent output columns and walks down a
// segment of `seg` output rows.  Every input row is loaded once per thread, transposed once (the byte transposes
// of depthwise3x3_tile_i8) into a ring of three rows held in registers, and then serves the three output rows
// whose windows contain it.  The loads for the next output row are issued before the arithmetic of the current
// one, so a wave overlaps its own memory latency with its own arithmetic instead of relying on the other waves
// of the SIMD for that; weights, bias and scale stay in registers for the whole segment.
// The row loop is unrolled three times so that the ring slots are compile-time indices.  S is the stride (1 or
// 2, both directions); OCC is the number of waves per SIMD the register allocation aims for; D (1 or 3) is how
// many output rows ahead the loads run.
template <int P, int S, int G, int OCC, int D>
__global__ __launch_bounds__(256, OCC) void depthwise3x3_strip_i8(DepthwiseArgs p, WorkSplit ws, int seg) {
    static_assert(D == 1 || D == 3, "the prefetch buffers rotate with the row loop's unrolling");
    static_assert(S == 1 || S == 2, "stride 1 or 2");
    static_assert(S == 2 || P % 2 == 0, "stride 1 pairs the pixels of a block");
    constexpr int NC = (P - 1) * S + 3;      // input columns under the thread's P windows
    constexpr int NBK = S == 1 ? P / 2 : P;  // blocks of four columns per row; block b starts at column 2 b
    constexpr int CV = 4 * G;
    constexpr int NEW = S;                   // input rows that enter the window per output row
    const int cg = p.C / CV;
    const int oxGroups = (p.OW + P - 1) / P, nseg = (p.OH + seg - 1) / seg;
    const long long total = (long long)p.N * nseg * oxGroups * cg;
    const long long t = (long long)xcdContiguousBlock() * 256 + threadIdx.x;
    if (t >= total) return;
    int cgi, oxg, sg, n;
    splitWork(t, ws, cgi, oxg, sg, n);
    const int c0 = cgi * CV, ox0 = oxg * P, oy0 = sg * seg;
    const int oyEnd = oy0 + seg < p.OH ? oy0 + seg : p.OH;
    const int ix0 = ox0 * S - p.PL;
    const int8_t *img = p.in + (size_t)n * p.H * p.W * p.C + c0;
    int8_t *outImg = p.out + (size_t)n * p.OH * p.OW * p.C + c0;
    const int zp4 = (int)((uint32_t)(p.input_zp & 0xff) * 0x01010101u);
    // every load is in bounds: coordinates are clamped and what the clamp moved is replaced by the zero point
    int colOff[NC];
    bool colIn[NC];
#pragma unroll
    for (int j = 0; j < NC; j++) {
        const int ix = ix0 + j;
        const int ixc = ix < 0 ? 0 : ix >= p.W ? p.W - 1 : ix;
        colOff[j] = ixc * p.C;
        colIn[j] = ix == ixc;
    }
    const int rowBytes = p.W * p.C;
    auto issue = [&](int iy, int (&raw)[NC][G]) {
        const int iyc = iy < 0 ? 0 : iy >= p.H ? p.H - 1 : iy;
        const int8_t *row = img + (size_t)iyc * rowBytes;
#pragma unroll
        for (int j = 0; j < NC; j++) loadDwords<G>(row + colOff[j], raw[j]);
    };
    auto settle = [&](int iy, const int (&raw)[NC][G], uint32_t (&tr)[NBK][G][4]) {
        const bool rowIn = (unsigned)iy < (unsigned)p.H;
        uint32_t x[NC][G];
#pragma unroll
        for (int j = 0; j < NC; j++) {
            const bool in = rowIn && colIn[j];
#pragma unroll
            for (int g = 0; g < G; g++) x[j][g] = in ? (uint32_t)raw[j][g] : (uint32_t)zp4;
        }
#pragma unroll
        for (int b = 0; b < NBK; b++) {
#pragma unroll
            for (int g = 0; g < G; g++) {
                // the last block of a stride-2 row has no fourth column; its weight is zero
                const uint32_t x0 = x[2 * b][g], x1 = x[2 * b + 1][g], x2 = x[2 * b + 2][g], x3 = x[2 * b + 3 < NC ? 2 * b + 3 : NC - 1][g];
                // 4 x 4 byte transpose: tr[c] = channel c at columns 2b .. 2b+3
                const uint32_t lo01 = __builtin_amdgcn_perm(x1, x0, 0x05010400u), hi01 = __builtin_amdgcn_perm(x1, x0, 0x07030602u);
                const uint32_t lo23 = __builtin_amdgcn_perm(x3, x2, 0x05010400u), hi23 = __builtin_amdgcn_perm(x3, x2, 0x07030602u);
                tr[b][g][0] = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u);
                tr[b][g][1] = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u);
                tr[b][g][2] = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u);
                tr[b][g][3] = __builtin_amdgcn_perm(hi23, hi01, 0x07060302u);
            }
        }
    };
    const WideRequant wrq = wideRequant(p.rq);
    const long long rnd = roundTerm(p.rq.shift);
    const uint32_t *wrow = (const uint32_t *)p.wpk + c0;
    // wk = [w0, w1, w2, 0] serves the window at a block's first column, wks = [0, w0, w1, w2] the one at its second
    int wk[G][3][4], wks[G][3][4], bs[G][4], sc[G][4];
#pragma unroll
    for (int g = 0; g < G; g++) {
#pragma unroll
        for (int kh = 0; kh < 3; kh++) {
            const v4i w4 = *(const v4i *)(wrow + (size_t)kh * p.C + 4 * g);
#pragma unroll
            for (int c = 0; c < 4; c++) {
                wk[g][kh][c] = w4[c];
                wks[g][kh][c] = (int)((uint32_t)w4[c] << 8);
            }
        }
        const v4i b4 = *(const v4i *)(p.bias + c0 + 4 * g);
        const v4i s4 = *(const v4i *)(p.scale + c0 + 4 * g);
#pragma unroll
        for (int c = 0; c < 4; c++) {
            bs[g][c] = b4[c];
            sc[g][c] = s4[c];
        }
    }
    uint32_t ring[3][NBK][G][4];  // window row kh of the J-th output row of a round of three sits in slot (J S + kh) % 3
    int raw[D][NEW][NC][G];
    const int iyFirst = oy0 * S - p.PT;
    {
        // every load of the prologue goes out before the first one is waited for: the rows that complete the first
        // window and the D rows of prefetch cost one memory round trip together, not one each
        int first[3 - NEW][NC][G];
#pragma unroll
        for (int kh = 0; kh < 3 - NEW; kh++) issue(iyFirst + kh, first[kh]);
#pragma unroll
        for (int d = 0; d < D; d++) {
#pragma unroll
            for (int e = 0; e < NEW; e++) issue(iyFirst + d * S + 3 - NEW + e, raw[d][e]);
        }
#pragma unroll
        for (int kh = 0; kh < 3 - NEW; kh++) settle(iyFirst + kh, first[kh], ring[kh]);
    }
    withRequantMode(wrq, [&](auto mode) {
        constexpr int kMode = decltype(mode)::value;
        auto step = [&](auto round, int oy) {
            constexpr int J = decltype(round)::value;
            constexpr int slots[3] = {(J * S) % 3, (J * S + 1) % 3, (J * S + 2) % 3};
            const int base = oy * S - p.PT;
#pragma unroll
            for (int e = 0; e < NEW; e++) settle(base + 3 - NEW + e, raw[J % D][e], ring[slots[3 - NEW + e]]);
            // the rows that output row oy + D adds (clamped: past the segment's end they are loaded and not used)
#pragma unroll
            for (int e = 0; e < NEW; e++) issue(base + D * S + 3 - NEW + e, raw[J % D][e]);
            int o[P][G];
#pragma unroll
            for (int g = 0; g < G; g++) {
                int32_t acc[P][4];  // starts at the bias (int32 wrap-around is the same in either order)
#pragma unroll
                for (int q = 0; q < P; q++) {
#pragma unroll
                    for (int c = 0; c < 4; c++) acc[q][c] = bs[g][c];
                }
#pragma unroll
                for (int kh = 0; kh < 3; kh++) {
#pragma unroll
                    for (int b = 0; b < NBK; b++) {
#pragma unroll
                        for (int c = 0; c < 4; c++) {
                            const int x = (int)ring[slots[kh]][b][g][c];
                            if (S == 1) {
                                acc[2 * b][c] = __builtin_amdgcn_sdot4(x, wk[g][kh][c], acc[2 * b][c], false);
                                acc[2 * b + 1][c] = __builtin_amdgcn_sdot4(x, wks[g][kh][c], acc[2 * b + 1][c], false);
                            } else {
                                acc[b][c] = __builtin_amdgcn_sdot4(x, wk[g][kh][c], acc[b][c], false);
                            }
                        }
                    }
                }
#pragma unroll
                for (int q = 0; q < P; q++) {
                    int32_t v[4];
#pragma unroll
                    for (int c = 0; c < 4; c++) v[c] = requantT0<kMode>(acc[q][c], sc[g][c], rnd, p.rq, wrq);
                    o[q][g] = (int)packBytes(v[0], v[1], v[2], v[3]);
                }
            }
            if (oy < oyEnd) {
                int8_t *orow = outImg + ((size_t)oy * p.OW + ox0) * p.C;
#pragma unroll
                for (int q = 0; q < P; q++) {
                    if (ox0 + q < p.OW) {
                        union {
                            typename DwordVec<G>::type v;
                            int w[G];
                        } u;
#pragma unroll
                        for (int g = 0; g < G; g++) u.w[g] = o[q][g];
                        *(typename DwordVec<G>::type *)(orow + (size_t)q * p.C) = u.v;
                    }
                }
            }
        };
        // the same trip count for every thread (rows past a short last segment are computed and not stored)
        for (int oy = oy0; oy < oy0 + seg; oy += 3) {
            step(std::integral_constant<int, 0>{}, oy);
            step(std::integral_constant<int, 1>{}, oy + 1);
            step(std::integral_constant<int, 2>{}, oy + 2);
        }
    });
}

// Rows per segment: enough segments that every SIMD gets several waves (they hide what the prefetch does not),
// segments of at least six rows (each one re-reads two rows of its neighbour and reloads the weights).
static int depthwiseStripSegment(const DepthwiseArgs &a, int P, int G, long long *waves) {
    const long long stripWaves = ((long long)a.N * ((a.OW + P - 1) / P) * (a.C / (4 * G)) + 63) / 64;
    long long nseg = (6 * 1024 + stripWaves - 1) / stripWaves;
    const long long most = a.OH / 6 > 0 ? a.OH / 6 : 1;
    nseg = nseg < 1 ? 1 : nseg > most ? most : nseg;
    const int seg = (int)((a.OH + nseg - 1) / nseg);
    *waves = stripWaves * ((a.OH + seg - 1) / seg);
    return seg;
}

template <int P, int S, int G, int OCC, int D>
static hipError_t launchDepthwiseStrip(const DepthwiseArgs &a, int seg, const LaunchCtx &ctx) {
    const int nseg = (a.OH + seg - 1) / seg, xs = (a.OW + P - 1) / P;
    const long long total = (long long)a.N * nseg * xs * (a.C / (4 * G));
    const WorkSplit ws = makeWorkSplit(total, a.C / (4 * G), xs, nseg);
    THIP_ENQUEUE(ctx, kernelLabel("depthwise3x3_strip_i8", {P, S, G, OCC, D}), (depthwise3x3_strip_i8<P, S, G, OCC, D>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, a, ws, seg);
    return hipGetLastError();
}

static int pickVec(int C, const void *a, const void *b, const void *c) {
    const uintptr_t bits = (uintptr_t)a | (uintptr_t)b | (uintptr_t)c;
    if (C % 16 == 0 && (bits & 15) == 0) return 16;
    if (C % 8 == 0 && (bits & 7) == 0) return 8;
    if (C % 4 == 0 && (bits & 3) == 0) return 4;
    return 1;
}

static bool poolGeometryOk(int N, int H, int W, int C, int OH, int OW, int KH, int KW, int SH,
                           int SW, int PT, int PL) {
    if (N <= 0 || H <= 0 || W <= 0 || C <= 0 || OH <= 0 || OW <= 0) return false;
    if (KH <= 0 || KW <= 0 || SH <= 0 || SW <= 0 || PT < 0 || PL < 0) return false;
    return true;
}

template <int VEC>
static hipError_t launchDepthwiseV(const DepthwiseArgs &a, const LaunchCtx &ctx) {
    const long long total = (long long)a.N * a.OH * a.OW * (a.C / VEC);
    const dim3 grid((unsigned)((total + 255) / 256));
    const WorkSplit ws = makeWorkSplit(total, a.C / VEC, a.OW, a.OH);
    if (a.KH == 3 && a.KW == 3) {
        THIP_ENQUEUE(ctx, kernelLabel("depthwise_i8", {VEC, 3}), (depthwise_i8<VEC, 3>), grid, dim3(256), 0, a, ws);
    } else {
        THIP_ENQUEUE(ctx, kernelLabel("depthwise_i8", {VEC, 0}), (depthwise_i8<VEC, 0>), grid, dim3(256), 0, a, ws);
    }
    return hipGetLastError();
}

hipError_t launchDepthwise(const DepthwiseArgs &a, const LaunchCtx &ctx) {
    if (!poolGeometryOk(a.N, a.H, a.W, a.C, a.OH, a.OW, a.KH, a.KW, a.SH, a.SW, a.PT, a.PL)) {
        return hipErrorInvalidValue;
    }
    if (!a.in || !a.wpk || !a.bias || !a.scale || !a.out) return hipErrorInvalidValue;
    if ((long long)a.N * a.OH * a.OW * a.C >= (1LL << 40)) return hipErrorInvalidValue;
    if (a.variant == kDepthwiseDot4Rows) {
        const uintptr_t bits = (uintptr_t)a.in | (uintptr_t)a.out | (uintptr_t)a.wpk | (uintptr_t)a.bias | (uintptr_t)a.scale;
        if (a.KH != 3 || a.KW != 3 || a.C % 16 != 0 || (bits & 15) != 0) return hipErrorInvalidValue;
        // several pixels per thread once there is enough work to still fill the chip
        const long long outputs = (long long)a.N * a.OH * a.OW * (a.C / 16);
        // a register tile of outputs per thread where that still leaves every CU several blocks
        // (THIP_DEPTHWISE_TILE=0 / 1 switches that kernel off / on for every size, for tests and tuning)
        // the rolling-window kernel where it has at least 0.6 waves (stride 1) or 1.9 waves (stride 2) per SIMD
        // (THIP_DEPTHWISE_STRIP=0 / 1 / 2 switches it off / on / on with one column per thread at stride 2, for every
        // size, for tests and tuning)
        const int stripMode = ctx.tuning->depthwiseStrip;
        const bool stripOff = stripMode == 0, stripOn = stripMode == 1 || stripMode == 2;
        const bool stripOne = stripMode == 2;
        if (!stripOff && a.SH == a.SW && (a.SW == 1 || a.SW == 2) && (long long)a.W * a.C < (1LL << 24)) {
            long long waves = 0;
            const int seg = depthwiseStripSegment(a, 2, 1, &waves);
            if (a.SW == 1 && (stripOn || (a.OH >= 6 && waves >= 640))) return launchDepthwiseStrip<2, 1, 1, 4, 3>(a, seg, ctx);
            if (a.SW == 2 && (stripOne || (!stripOn && a.OH >= 12))) {
                // with plenty of work (the six waves per SIMD that the segment length aims for), one column per thread, more
                // waves and the deeper prefetch measured 7-11 % ahead
                long long waves1 = 0;
                const int seg1 = depthwiseStripSegment(a, 1, 1, &waves1);
                if (stripOne || waves1 >= 6 * 1024) return launchDepthwiseStrip<1, 2, 1, 4, 3>(a, seg1, ctx);
            }
            if (a.SW == 2 && (stripOn || (a.OH >= 12 && 10 * waves >= 19 * 1024))) return launchDepthwiseStrip<2, 2, 1, 3, 1>(a, seg, ctx);
            // too few waves for two columns per thread, enough for one (112 x 112 x 96 at batch 8: 6.8 us against 7.7 for
            // the window-row kernel; 56 x 56 x 144 at batch 32: 7.2 against 8.2)
            if (a.SW == 2 && !stripOn && a.OH >= 12) {
                long long waves1 = 0;
                const int seg1 = depthwiseStripSegment(a, 1, 1, &waves1);
                if (waves1 >= 1280) return launchDepthwiseStrip<1, 2, 1, 4, 3>(a, seg1, ctx);
            }
        }
        const bool tileOff = ctx.tuning->depthwiseTile == 0, tileOn = ctx.tuning->depthwiseTile == 1;
        if (!tileOff) {
            // 16 channels per thread: 8 or 4 (more waves, fewer registers) measured 5 % and 12 % slower
            const long long tileMin = ctx.tuning->depthwiseTileMin > 0 ? ctx.tuning->depthwiseTileMin : 8 * 65536;  // measured on a mobile network at batch 32 and 256: even or ahead from about half a million thread-outputs
            if (a.SW == 1 && a.SH == 1 && (tileOn || outputs >= tileMin)) return launchDepthwiseTile<4, 2, 1, 4>(a, ctx);
        }
        // pixels per thread (THIP_DEPTHWISE_P forces 1, 2 or 4, for tuning)
        int pix = outputs >= 4 * 65536 ? 4 : outputs >= 2 * 65536 ? 2 : 1;
        if (ctx.tuning->depthwisePixels > 0) pix = ctx.tuning->depthwisePixels;
        if (a.SW == 1 && pix == 4) return launchDepthwiseDot4<4, 1>(a, ctx);
        if (a.SW == 2 && pix == 4) return launchDepthwiseDot4<4, 2>(a, ctx);
        if (a.SW == 1 && pix == 2) return launchDepthwiseDot4<2, 1>(a, ctx);
        if (a.SW == 2 && pix == 2) return launchDepthwiseDot4<2, 2>(a, ctx);
        return launchDepthwiseDot4<1, 0>(a, ctx);
    }
    if (a.variant != kDepthwiseGeneric) return hipErrorInvalidValue;
    switch (pickVec(a.C, a.in, a.out, a.wpk)) {
    case 16: return launchDepthwiseV<16>(a, ctx);
    case 8: return launchDepthwiseV<8>(a, ctx);
    case 4: return launchDepthwiseV<4>(a, ctx);
    default: return launchDepthwiseV<1>(a, ctx);
    }
}

template <int VEC>
__global__ __launch_bounds__(256) void maxpool_i8(MaxPoolArgs p, WorkSplit ws) {
    const int cg = p.C / VEC;
    const long long total = (long long)p.N * p.OH * p.OW * cg;
    const long long t = (long long)blockIdx.x * 256 + threadIdx.x;
    if (t >= total) return;
    int cgi, ox, oy, n;
    splitWork(t, ws, cgi, ox, oy, n);
    const int c0 = cgi * VEC;
    const int iy0 = oy * p.SH - p.PT, ix0 = ox * p.SW - p.PL;
    const int8_t *img = p.in + (size_t)n * p.H * p.W * p.C + c0;
    int32_t best[VEC];
#pragma unroll
    for (int v = 0; v < VEC; v++) best[v] = -(1 << 30);
    bool padded = false;
    for (int kh = 0; kh < p.KH; kh++) {
        const int iy = iy0 + kh;
        for (int kw = 0; kw < p.KW; kw++) {
            const int ix = ix0 + kw;
            if ((unsigned)iy < (unsigned)p.H && (unsigned)ix < (unsigned)p.W) {
                Pack<VEC> x;
                x.v = *(const typename ByteVec<VEC>::type *)(img + ((size_t)iy * p.W + ix) * p.C);
#pragma unroll
                for (int v = 0; v < VEC; v++) best[v] = best[v] > (int32_t)x.b[v] ? best[v] : (int32_t)x.b[v];
            } else {
                padded = true;
            }
        }
    }
    Pack<VEC> o;
#pragma unroll
    for (int v = 0; v < VEC; v++) {
        int32_t b = best[v];
        if (padded) b = b > p.input_zp ? b : p.input_zp;
        b = b < p.out_min ? p.out_min : b;
        b = b > p.out_max ? p.out_max : b;
        o.b[v] = (int8_t)b;
    }
    *(typename ByteVec<VEC>::type *)(p.out + (((size_t)n * p.OH + oy) * p.OW + ox) * p.C + c0) = o.v;
}

// Signed maximum of the four bytes of two dwords.  Bytes 0 and 2 move to the upper byte of their 16-bit half (a byte
// permute), bytes 1 and 3 are masked in place; a packed 16-bit signed maximum then orders each pair exactly as the
// bytes order (the lower byte of every half is zero on both sides).  Halves stay split between calls.
struct SplitBytes {
    uint32_t even, odd;  // [0, b0, 0, b2] and [0, b1, 0, b3] as bytes 0..3
};
__device__ __forceinline__ SplitBytes splitBytes(uint32_t x) {
    return SplitBytes{__builtin_amdgcn_perm(x, x, 0x020c000cu), x & 0xff00ff00u};
}
typedef short v2s __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pkMaxI16(uint32_t a, uint32_t b) {
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(v2s, a), __builtin_bit_cast(v2s, b)));
}
__device__ __forceinline__ SplitBytes maxSplit(SplitBytes a, SplitBytes b) { return SplitBytes{pkMaxI16(a.even, b.even), pkMaxI16(a.odd, b.odd)}; }
__device__ __forceinline__ uint32_t joinBytes(SplitBytes m) { return __builtin_amdgcn_perm(m.odd, m.even, 0x07030501u); }

// The common pooling window as its own kernel: 2 x 2, stride 2, no padding touched, C % 16 == 0, no clamp beyond the
// int8 range.  A thread owns 16 channels of one output pixel: its four 128-bit loads are issued together (the
// general kernel walks a run-time window, one load in flight per thread) and the maxima are taken on packed bytes.
__global__ __launch_bounds__(256) void maxpool2x2_i8(MaxPoolArgs p, WorkSplit ws) {
    const int cg = p.C / 16;
    const long long total = (long long)p.N * p.OH * p.OW * cg;
    const long long t = (long long)blockIdx.x * 256 + threadIdx.x;
    if (t >= total) return;
    int cgi, ox, oy, n;
    splitWork(t, ws, cgi, ox, oy, n);
    const int8_t *src = p.in + (((size_t)n * p.H + 2 * oy) * p.W + 2 * ox) * p.C + cgi * 16;
    const size_t row = (size_t)p.W * p.C;
    const v4i a = *(const v4i *)src, b = *(const v4i *)(src + p.C), c = *(const v4i *)(src + row), d = *(const v4i *)(src + row + p.C);
    v4i o;
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const SplitBytes m = maxSplit(maxSplit(splitBytes((uint32_t)a[q]), splitBytes((uint32_t)b[q])),
                                      maxSplit(splitBytes((uint32_t)c[q]), splitBytes((uint32_t)d[q])));
        o[q] = (int)joinBytes(m);
    }
    *(v4i *)(p.out + (((size_t)n * p.OH + oy) * p.OW + ox) * p.C + cgi * 16) = o;
}

template <int VEC>
static hipError_t launchMaxPoolV(const MaxPoolArgs &a, const LaunchCtx &ctx) {
    const long long total = (long long)a.N * a.OH * a.OW * (a.C / VEC);
    const dim3 grid((unsigned)((total + 255) / 256));
    const WorkSplit ws = makeWorkSplit(total, a.C / VEC, a.OW, a.OH);
    THIP_ENQUEUE(ctx, kernelLabel("maxpool_i8", {VEC}), (maxpool_i8<VEC>), grid, dim3(256), 0, a, ws);
    return hipGetLastError();
}

hipError_t launchMaxPool(const MaxPoolArgs &a, const LaunchCtx &ctx) {
    if (!poolGeometryOk(a.N, a.H, a.W, a.C, a.OH, a.OW, a.KH, a.KW, a.SH, a.SW, a.PT, a.PL)) {
        return hipErrorInvalidValue;
    }
    if (!a.in || !a.out) return hipErrorInvalidValue;
    if ((long long)a.N * a.OH * a.OW * a.C >= (1LL << 40)) return hipErrorInvalidValue;
    const int vec = pickVec(a.C, a.in, a.out, nullptr);
    if (vec == 16 && a.KH == 2 && a.KW == 2 && a.SH == 2 && a.SW == 2 && a.PT == 0 && a.PL == 0 && 2 * a.OH <= a.H && 2 * a.OW <= a.W &&
        a.out_min <= -128 && a.out_max >= 127 && !ctx.tuning->maxpoolGeneric) {
        const long long total = (long long)a.N * a.OH * a.OW * (a.C / 16);
        const WorkSplit ws = makeWorkSplit(total, a.C / 16, a.OW, a.OH);
        THIP_ENQUEUE(ctx, "maxpool2x2_i8", maxpool2x2_i8, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, a, ws);
        return hipGetLastError();
    }
    switch (vec) {
    case 16: return launchMaxPoolV<16>(a, ctx);
    case 8: return launchMaxPoolV<8>(a, ctx);
    case 4: return launchMaxPoolV<4>(a, ctx);
    default: return launchMaxPoolV<1>(a, ctx);
    }
}

// Global average pool: one wave covers CC channel groups of VEC channels; the
// 64 / CC lanes that share a channel group split the H*W pixels and are
// combined with wave shuffles.
template <int VEC, int CC>
__global__ __launch_bounds__(256) void avgpool_i8(AvgPoolArgs p) {
    constexpr int PG = 64 / CC;  // lanes per channel group
    const int lane = threadIdx.x & 63;
    const int wave = (int)((blockIdx.x * 256 + threadIdx.x) >> 6);
    const int cgroups = p.C / VEC;
    const int wavesPerImage = (cgroups + CC - 1) / CC;
    const int n = wave / wavesPerImage;
    if (n >= p.N) return;
    const int cgi = (wave % wavesPerImage) * CC + (lane % CC);
    const int pg = lane / CC;
    const bool active = cgi < cgroups;
    const int c0 = cgi * VEC;
    int32_t acc[VEC];
#pragma unroll
    for (int v = 0; v < VEC; v++) acc[v] = 0;
    if (active) {
        const int8_t *src = p.in + (size_t)n * p.HW * p.C + c0;
        // four pixels per round, all four loads issued before the first is used (a pixel past the frame re-reads the
        // lane's first one and is weighted 0): a 7 x 7 frame costs one memory round trip instead of four
        for (int u0 = pg; u0 < p.HW; u0 += 4 * PG) {
            Pack<VEC> x[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int u = u0 + j * PG;
                x[j].v = *(const typename ByteVec<VEC>::type *)(src + (size_t)(u < p.HW ? u : pg) * p.C);
            }
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int32_t wj = u0 + j * PG < p.HW ? p.weight : 0;
#pragma unroll
                for (int v = 0; v < VEC; v++) acc[v] += (int32_t)x[j].b[v] * wj;
            }
        }
    }
#pragma unroll
    for (int v = 0; v < VEC; v++) {
        int32_t s = acc[v];
#pragma unroll
        for (int off = 32; off >= CC; off >>= 1) s += __shfl_xor(s, off, 64);
        acc[v] = s;
    }
    if (active && pg == 0) {
        const long long rnd = roundTerm(p.rq.shift);
        Pack<VEC> o;
#pragma unroll
        for (int v = 0; v < VEC; v++) o.b[v] = (int8_t)requant(acc[v], p.bias, p.scale, rnd, p.rq);
        *(typename ByteVec<VEC>::type *)(p.out + (size_t)n * p.C + c0) = o.v;
    }
}

template <int VEC>
static hipError_t launchAvgPoolV(const AvgPoolArgs &a, const LaunchCtx &ctx) {
    constexpr int CC = 4;
    const int cgroups = a.C / VEC;
    const long long waves = (long long)a.N * ((cgroups + CC - 1) / CC);
    const dim3 grid((unsigned)((waves + 3) / 4));
    THIP_ENQUEUE(ctx, kernelLabel("avgpool_i8", {VEC, CC}), (avgpool_i8<VEC, CC>), grid, dim3(256), 0, a);
    return hipGetLastError();
}

hipError_t launchAvgPool(const AvgPoolArgs &a, const LaunchCtx &ctx) {
    if (a.N <= 0 || a.HW <= 0 || a.C <= 0 || !a.in || !a.out) return hipErrorInvalidValue;
    switch (pickVec(a.C, a.in, a.out, nullptr)) {
    case 16: return launchAvgPoolV<16>(a, ctx);
    case 8: return launchAvgPoolV<8>(a, ctx);
    case 4: return launchAvgPoolV<4>(a, ctx);
    default: return launchAvgPoolV<1>(a, ctx);
    }
}

// FAST (16 bytes per thread only): the add's scale is 1 and its 32-bit sum cannot overflow, so bias, rounding term
// and zero point are one constant and a value costs two multiply-adds, a shift and a clamp (residualAdd16).
template <int VEC, bool FAST>
__global__ __launch_bounds__(256) void add_i8(AddArgs p, int32_t folded) {
    const long long t = (long long)blockIdx.x * 256 + threadIdx.x;
    const long long i0 = t * VEC;
    if (i0 >= p.count) return;
    const long long rnd = roundTerm(p.rq.shift);
    if (i0 + VEC <= p.count) {
        if constexpr (FAST && VEC == 16) {
            const v4i a = *(const v4i *)(p.in0 + i0), b = *(const v4i *)(p.in1 + i0);
            *(v4i *)(p.out + i0) = residualAdd16<true>(a, b, false, p.w0, p.w1, p.bias, p.scale, rnd, p.rq, folded);
        } else {
            Pack<VEC> a, b, o;
            a.v = *(const typename ByteVec<VEC>::type *)(p.in0 + i0);
            b.v = *(const typename ByteVec<VEC>::type *)(p.in1 + i0);
#pragma unroll
            for (int v = 0; v < VEC; v++) {
                const int32_t acc = (int32_t)a.b[v] * p.w0 + (int32_t)b.b[v] * p.w1;
                o.b[v] = (int8_t)requant(acc, p.bias, p.scale, rnd, p.rq);
            }
            *(typename ByteVec<VEC>::type *)(p.out + i0) = o.v;
        }
    } else {
        for (long long i = i0; i < p.count; i++) {
            const int32_t acc = (int32_t)p.in0[i] * p.w0 + (int32_t)p.in1[i] * p.w1;
            p.out[i] = (int8_t)requant(acc, p.bias, p.scale, rnd, p.rq);
        }
    }
}

hipError_t launchAdd(const AddArgs &a, const LaunchCtx &ctx) {
    if (a.count <= 0 || !a.in0 || !a.in1 || !a.out) return hipErrorInvalidValue;
    const uintptr_t bits = (uintptr_t)a.in0 | (uintptr_t)a.in1 | (uintptr_t)a.out;
    if ((bits & 15) == 0) {
        const long long threads = (a.count + 15) / 16;
        const dim3 grid((unsigned)((threads + 255) / 256));
        int32_t folded = 0;
        // what the patterns emit (scale 1, shift 12, int8 clamp) folds; anything else takes the 64-bit ACT stage
        if (a.rq.out_min >= -128 && a.rq.out_max <= 127 && residualAddFolded(a.w0, a.w1, a.bias, a.scale, a.rq, &folded) && !ctx.tuning->addGeneric) {
            THIP_ENQUEUE(ctx, "add_i8<16,1>", (add_i8<16, true>), grid, dim3(256), 0, a, folded);
        } else {
            THIP_ENQUEUE(ctx, "add_i8<16,0>", (add_i8<16, false>), grid, dim3(256), 0, a, 0);
        }
    } else {
        THIP_ENQUEUE(ctx, "add_i8<1,0>", (add_i8<1, false>), dim3((unsigned)((a.count + 255) / 256)), dim3(256), 0, a, 0);
    }
    return hipGetLastError();
}

// Patch matrix of a bf16 convolution (the GEMM that follows streams it like any other input): one
// thread per element.  Not a fast path: the int8 convolutions gather inside the GEMM instead.
__global__ __launch_bounds__(256) void im2col_bf16(Im2colBf16Args p, long long total) {
    const long long t = (long long)blockIdx.x * 256 + threadIdx.x;
    if (t >= total) return;
    const int k = (int)(t % p.Kp);
    const long long m = t / p.Kp;
    uint16_t v = 0;
    if (k < p.KH * p.KW * p.C) {
        const int ci = k % p.C, pos = k / p.C, kw = pos % p.KW, kh = pos / p.KW;
        const int ox = (int)(m % p.OW);
        const long long r = m / p.OW;
        const int oy = (int)(r % p.OH), n = (int)(r / p.OH);
        const int iy = oy * p.SH - p.PT + kh, ix = ox * p.SW - p.PL + kw;
        if ((unsigned)iy < (unsigned)p.H && (unsigned)ix < (unsigned)p.W) v = p.in[(((size_t)n * p.H + iy) * p.W + ix) * p.C + ci];
    }
    p.out[t] = v;
}

hipError_t launchIm2colBf16(const Im2colBf16Args &a, const LaunchCtx &ctx) {
    if (!a.in || !a.out || !poolGeometryOk(a.N, a.H, a.W, a.C, a.OH, a.OW, a.KH, a.KW, a.SH, a.SW, a.PT, a.PL)) return hipErrorInvalidValue;
    if (a.Kp < a.KH * a.KW * a.C) return hipErrorInvalidValue;
    const long long total = (long long)a.N * a.OH * a.OW * a.Kp;
    if (total >= (1LL << 39)) return hipErrorInvalidValue;
    THIP_ENQUEUE(ctx, "im2col_bf16", im2col_bf16, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, a, total);
    return hipGetLastError();
}

// bf16 depthwise: one thread per output element, taps accumulated in (kh, kw) order in fp32 (the
// products are exact, so a fused multiply-add gives the same sums as a multiply and an add).
__global__ __launch_bounds__(256) void depthwise_bf16(DepthwiseBf16Args p, long long total) {
    const long long t = (long long)blockIdx.x * 256 + threadIdx.x;
    if (t >= total) return;
    const int c = (int)(t % p.C);
    long long r = t / p.C;
    const int ox = (int)(r % p.OW);
    r /= p.OW;
    const int oy = (int)(r % p.OH), n = (int)(r / p.OH);
    float acc = 0.0f;
    for (int kh = 0; kh < p.KH; kh++) {
        const int iy = oy * p.SH - p.PT + kh;
        if ((unsigned)iy >= (unsigned)p.H) continue;
        for (int kw = 0; kw < p.KW; kw++) {
            const int ix = ox * p.SW - p.PL + kw;
            if ((unsigned)ix >= (unsigned)p.W) continue;
            const float x = __uint_as_float((uint32_t)p.in[(((size_t)n * p.H + iy) * p.W + ix) * p.C + c] << 16);
            const float w = __uint_as_float((uint32_t)p.wpk[((size_t)kh * p.KW + kw) * p.C + c] << 16);
            acc = __fadd_rn(acc, __fmul_rn(x, w));
        }
    }
    const float t0 = __fadd_rn(acc, p.bias[c]);
    p.out[t] = bf16Bits(t0 < p.lo ? p.lo : (t0 > p.hi ? p.hi : t0));
}

hipError_t launchDepthwiseBf16(const DepthwiseBf16Args &a, const LaunchCtx &ctx) {
    if (!a.in || !a.wpk || !a.bias || !a.out) return hipErrorInvalidValue;
    if (!poolGeometryOk(a.N, a.H, a.W, a.C, a.OH, a.OW, a.KH, a.KW, a.SH, a.SW, a.PT, a.PL)) return hipErrorInvalidValue;
    const long long total = (long long)a.N * a.OH * a.OW * a.C;
    if (total >= (1LL << 39)) return hipErrorInvalidValue;
    THIP_ENQUEUE(ctx, "depthwise_bf16", depthwise_bf16, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, a, total);
    return hipGetLastError();
}

// bf16 add: 8 elements (16 bytes) per thread when the tensors allow it.  No fused multiply-add: the second
// product is added to the first (both exact in fp32), then the bias, as the ACT stage does.
template <int VEC>
__global__ __launch_bounds__(256) void add_bf16(AddBf16Args p) {
    const int64_t i0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * VEC;
    if (i0 >= p.count) return;
    union Pack16 {
        v4i v;
        uint16_t h[8];
    } a, b, o;
    if (VEC == 8) {
        a.v = *(const v4i *)(p.in0 + i0);
        b.v = *(const v4i *)(p.in1 + i0);
    } else {
        a.h[0] = p.in0[i0];
        b.h[0] = p.in1[i0];
    }
#pragma unroll
    for (int e = 0; e < VEC; e++) {
        const float x0 = __uint_as_float((uint32_t)a.h[e] << 16), x1 = __uint_as_float((uint32_t)b.h[e] << 16);
        float acc = __fmul_rn(x0, p.w0);
        acc = __fadd_rn(acc, __fmul_rn(x1, p.w1));
        const float t0 = __fadd_rn(acc, p.bias);
        o.h[e] = bf16Bits(t0 < p.lo ? p.lo : (t0 > p.hi ? p.hi : t0));
    }
    if (VEC == 8) {
        *(v4i *)(p.out + i0) = o.v;
    } else {
        p.out[i0] = o.h[0];
    }
}

hipError_t launchAddBf16(const AddBf16Args &a, const LaunchCtx &ctx) {
    if (!a.in0 || !a.in1 || !a.out || a.count <= 0) return hipErrorInvalidValue;
    const bool vec = a.count % 8 == 0 && ((((uintptr_t)a.in0) | ((uintptr_t)a.in1) | ((uintptr_t)a.out)) & 15) == 0;
    const int64_t threads = vec ? a.count / 8 : a.count;
    if (threads >= (1LL << 39)) return hipErrorInvalidValue;
    const dim3 grid((unsigned)((threads + 255) / 256));
    if (vec) {
        THIP_ENQUEUE(ctx, "add_bf16<8>", add_bf16<8>, grid, dim3(256), 0, a);
    } else {
        THIP_ENQUEUE(ctx, "add_bf16<1>", add_bf16<1>, grid, dim3(256), 0, a);
    }
    return hipGetLastError();
}

// Integer elementwise ops: a thread owns VEC neighbouring elements (one wide load per input, one wide store).
template <typename T, int VEC>
struct alignas(sizeof(T) * VEC) EltVec {
    T e[VEC];
};
template <typename TIN, typename TOUT, int VEC>
__global__ __launch_bounds__(256) void eltwise_int(EltwiseArgs p) {
    const int64_t i0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * VEC;
    if (i0 >= p.count) return;
    const TIN *in0 = (const TIN *)p.in0, *in1 = (const TIN *)p.in1;
    TOUT *out = (TOUT *)p.out;
    const bool whole = i0 + VEC <= p.count;
    EltVec<TIN, VEC> a, b;
    EltVec<TOUT, VEC> o;
#pragma unroll
    for (int v = 0; v < VEC; v++) b.e[v] = (TIN)0;  // the one-input ops never look at it
    if (whole && p.bcast != 1) {
        a = *(const EltVec<TIN, VEC> *)(in0 + i0);
    } else {
#pragma unroll
        for (int v = 0; v < VEC; v++) a.e[v] = p.bcast == 1 ? in0[0] : (i0 + v < p.count ? in0[i0 + v] : (TIN)0);
    }
    if (eltwiseTwoInputs(p.op)) {
        if (whole && p.bcast != 2) {
            b = *(const EltVec<TIN, VEC> *)(in1 + i0);
        } else {
#pragma unroll
            for (int v = 0; v < VEC; v++) b.e[v] = p.bcast == 2 ? in1[0] : (i0 + v < p.count ? in1[i0 + v] : (TIN)0);
        }
    }
    if (p.op == kEltFma || p.op == kEltMul) {
        const WideRequant wrq = wideRequant(p.rq);
        const long long rnd = roundTerm(p.rq.shift);
        withRequantMode(wrq, [&](auto mode) {
            constexpr int kMode = decltype(mode)::value;
#pragma unroll
            for (int v = 0; v < VEC; v++) {
                const uint32_t rhs = p.op == kEltMul ? (uint32_t)(int32_t)b.e[v] : (uint32_t)p.w0;
                const int32_t t0 = (int32_t)((uint32_t)(int32_t)a.e[v] * rhs + (uint32_t)p.bias);
                o.e[v] = (TOUT)requantT0<kMode>(t0, p.scale, rnd, p.rq, wrq);
            }
        });
    } else if (p.op >= kEltNot) {
        constexpr int BITS = 8 * (int)sizeof(TIN);
        const uint32_t typeMask = BITS == 32 ? 0xffffffffu : ((1u << BITS) - 1u);
#pragma unroll
        for (int v = 0; v < VEC; v++) {
            const int32_t x = (int32_t)a.e[v], y = (int32_t)b.e[v];
            int32_t r;
            if (p.op == kEltNot) {
                r = ~x;
            } else if (p.op <= kEltEqual) {
                const int32_t kx = p.w0 ? (x & 0xffff) : x, ky = p.w0 ? (y & 0xffff) : y;
                r = p.op == kEltGreater ? kx > ky : p.op == kEltGreaterEqual ? kx >= ky : kx == ky;
            } else if (p.op <= kEltLogicalNot) {
                const bool tx = x != 0, ty = y != 0;
                r = p.op == kEltLogicalAnd ? (tx && ty) : p.op == kEltLogicalOr ? (tx || ty) : p.op == kEltLogicalXor ? (tx != ty) : !tx;
            } else {
                int32_t s = y < 0 ? 0 : (y > BITS - 1 ? BITS - 1 : y);
                if (p.op == kEltLsl) {
                    r = (int32_t)((uint32_t)x << s);
                } else {
                    // arithmetic: the sign-extended value; logical: the element's own bits, zero-extended
                    const long long val = p.op == kEltAsr ? (long long)x : (long long)((uint32_t)x & typeMask);
                    long long q = val >> s;
                    if (p.w0 && s > 0 && ((val >> (s - 1)) & 1)) q += 1;
                    r = (int32_t)q;
                }
            }
            o.e[v] = (TOUT)r;
        }
    } else if (p.op >= kEltAnd) {
        const int32_t mask = p.w0 ? 0xffff : -1;  // unsigned 16-bit comparison
#pragma unroll
        for (int v = 0; v < VEC; v++) {
            const int32_t x = (int32_t)a.e[v], y = (int32_t)b.e[v];
            const bool less = p.w0 ? (x & mask) < (y & mask) : x < y;
            const int32_t r = p.op == kEltAnd ? (x & y) : p.op == kEltOr ? (x | y) : p.op == kEltXor ? (x ^ y) : (p.op == kEltMin) == less ? x : y;
            o.e[v] = (TOUT)r;
        }
    } else {
#pragma unroll
        for (int v = 0; v < VEC; v++) {
            long long x = (long long)a.e[v];
            if (p.op == kEltAbs) x = x < 0 ? -x : x;
            if (p.op == kEltNegate) x = -x;
            x = x < p.lo ? (long long)p.lo : (x > p.hi ? (long long)p.hi : x);
            o.e[v] = (TOUT)x;
        }
    }
    if (whole) {
        *(EltVec<TOUT, VEC> *)(out + i0) = o;
    } else {
#pragma unroll
        for (int v = 0; v < VEC; v++) {
            if (i0 + v < p.count) out[i0 + v] = o.e[v];
        }
    }
}

// torq_hl.table as a plain lookup: the block copies the 256 entries into LDS, a thread looks up VEC neighbouring
// elements by the low byte of each input (read as signed, plus 128).
template <typename TIN, typename TOUT, int VEC>
__global__ __launch_bounds__(256) void table_lookup(EltwiseArgs p) {
    __shared__ TOUT lut[256];
    lut[threadIdx.x] = ((const TOUT *)p.in1)[threadIdx.x];
    __syncthreads();
    const int64_t i0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * VEC;
    if (i0 >= p.count) return;
    const TIN *in0 = (const TIN *)p.in0;
    TOUT *out = (TOUT *)p.out;
    const bool whole = i0 + VEC <= p.count;
    EltVec<TIN, VEC> a;
    EltVec<TOUT, VEC> o;
    if (whole) {
        a = *(const EltVec<TIN, VEC> *)(in0 + i0);
    } else {
#pragma unroll
        for (int v = 0; v < VEC; v++) a.e[v] = i0 + v < p.count ? in0[i0 + v] : (TIN)0;
    }
#pragma unroll
    for (int v = 0; v < VEC; v++) o.e[v] = lut[((uint32_t)(int32_t)a.e[v] & 0xffu) ^ 0x80u];
    if (whole) {
        *(EltVec<TOUT, VEC> *)(out + i0) = o;
    } else {
#pragma unroll
        for (int v = 0; v < VEC; v++) {
            if (i0 + v < p.count) out[i0 + v] = o.e[v];
        }
    }
}

template <typename TIN, typename TOUT>
static hipError_t launchTableT(const EltwiseArgs &a, const LaunchCtx &ctx) {
    constexpr int VEC = sizeof(TIN) == 1 && sizeof(TOUT) == 1 ? 16 : 8;
    const bool aligned = (((uintptr_t)a.in0) & (sizeof(TIN) * VEC - 1)) == 0 && (((uintptr_t)a.out) & (sizeof(TOUT) * VEC - 1)) == 0;
    if (aligned) {
        const long long threads = (a.count + VEC - 1) / VEC;
        THIP_ENQUEUE(ctx, kernelLabel("table_lookup", {(int)sizeof(TIN), (int)sizeof(TOUT), VEC}), (table_lookup<TIN, TOUT, VEC>), dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, a);
    } else {
        THIP_ENQUEUE(ctx, kernelLabel("table_lookup", {(int)sizeof(TIN), (int)sizeof(TOUT), 1}), (table_lookup<TIN, TOUT, 1>), dim3((unsigned)((a.count + 255) / 256)), dim3(256), 0, a);
    }
    return hipGetLastError();
}

template <typename TIN, typename TOUT>
static hipError_t launchEltwiseT(const EltwiseArgs &a, const LaunchCtx &ctx) {
    constexpr int VEC = sizeof(TIN) == 1 && sizeof(TOUT) == 1 ? 16 : 8;
    const uintptr_t bits = (uintptr_t)a.in0 | (eltwiseTwoInputs(a.op) ? (uintptr_t)a.in1 : 0);
    const bool aligned = (bits & (sizeof(TIN) * VEC - 1)) == 0 && (((uintptr_t)a.out) & (sizeof(TOUT) * VEC - 1)) == 0;
    if (aligned) {
        const long long threads = (a.count + VEC - 1) / VEC;
        THIP_ENQUEUE(ctx, kernelLabel("eltwise_int", {(int)sizeof(TIN), (int)sizeof(TOUT), VEC}), (eltwise_int<TIN, TOUT, VEC>), dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, a);
    } else {
        THIP_ENQUEUE(ctx, kernelLabel("eltwise_int", {(int)sizeof(TIN), (int)sizeof(TOUT), 1}), (eltwise_int<TIN, TOUT, 1>), dim3((unsigned)((a.count + 255) / 256)), dim3(256), 0, a);
    }
    return hipGetLastError();
}

hipError_t launchEltwise(const EltwiseArgs &a, const LaunchCtx &ctx) {
    if (!a.in0 || !a.out || a.count <= 0 || a.count >= (1LL << 39) || a.op < kEltFma || a.op > kEltLast) return hipErrorInvalidValue;
    const bool two = eltwiseTwoInputs(a.op);
    if (two && (!a.in1 || a.bcast < 0 || a.bcast > 2)) return hipErrorInvalidValue;
    if (a.op != kEltMul && a.bcast != 0) return hipErrorInvalidValue;
    if (eltwiseSameType(a.op) && a.in_bytes != a.out_bytes) return hipErrorInvalidValue;
    if (a.op >= kEltAnd && a.op <= kEltEqual && a.w0 != 0 && a.in_bytes != 2) return hipErrorInvalidValue;  // unsigned: 16-bit only
    if (a.op >= kEltGreater && a.op <= kEltEqual && a.out_bytes != 1) return hipErrorInvalidValue;            // a truth value is one byte
    if (a.op >= kEltLogicalAnd && a.op <= kEltLogicalNot && a.in_bytes != 1) return hipErrorInvalidValue;
    if ((((uintptr_t)a.in0) & (a.in_bytes - 1)) || (((uintptr_t)a.out) & (a.out_bytes - 1))) return hipErrorInvalidValue;
    if (a.op == kEltTable) {
        // the 256 entries have the output's type; an int8 table serves int8 inputs only
        if ((((uintptr_t)a.in1) & (a.out_bytes - 1)) || a.in_bytes > 2 || a.out_bytes > 2 || a.out_bytes < a.in_bytes) return hipErrorInvalidValue;
        if (a.in_bytes == 1) return a.out_bytes == 1 ? launchTableT<int8_t, int8_t>(a, ctx) : launchTableT<int8_t, int16_t>(a, ctx);
        return launchTableT<int16_t, int16_t>(a, ctx);
    }
    if (two && (((uintptr_t)a.in1) & (a.in_bytes - 1))) return hipErrorInvalidValue;
    switch (a.in_bytes * 8 + a.out_bytes) {
    case 1 * 8 + 1: return launchEltwiseT<int8_t, int8_t>(a, ctx);
    case 1 * 8 + 2: return launchEltwiseT<int8_t, int16_t>(a, ctx);
    case 1 * 8 + 4: return launchEltwiseT<int8_t, int32_t>(a, ctx);
    case 2 * 8 + 1: return launchEltwiseT<int16_t, int8_t>(a, ctx);
    case 2 * 8 + 2: return launchEltwiseT<int16_t, int16_t>(a, ctx);
    case 2 * 8 + 4: return launchEltwiseT<int16_t, int32_t>(a, ctx);
    case 4 * 8 + 1: return launchEltwiseT<int32_t, int8_t>(a, ctx);
    case 4 * 8 + 2: return launchEltwiseT<int32_t, int16_t>(a, ctx);
    case 4 * 8 + 4: return launchEltwiseT<int32_t, int32_t>(a, ctx);
    default: return hipErrorInvalidValue;
    }
}

// Batched transpose [B][R][S] -> [B][S][R] of 1- or 2-byte elements through a 64 x 64 LDS tile; output rows are
// out_pitch elements apart (what lies between R and the pitch is not written).
template <typename T>
__global__ __launch_bounds__(256) void transpose_i8(TransposeArgs p) {
    __shared__ T tile[64][65];
    const int tilesS = (p.S + 63) / 64, tilesR = (p.R + 63) / 64;
    int bid = (int)blockIdx.x;
    const int ts = bid % tilesS;
    bid /= tilesS;
    const int tr = bid % tilesR;
    const int b = bid / tilesR;
    const int r0 = tr * 64, s0 = ts * 64;
    const T *src = (const T *)p.in + (size_t)b * p.R * p.S;
    T *dst = (T *)p.out + (size_t)b * p.S * p.out_pitch;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    for (int r = ty; r < 64; r += 4) {
        if (r0 + r < p.R && s0 + tx < p.S) tile[r][tx] = src[(size_t)(r0 + r) * p.S + s0 + tx];
    }
    __syncthreads();
    for (int s = ty; s < 64; s += 4) {
        if (s0 + s < p.S && r0 + tx < p.R) dst[(size_t)(s0 + s) * p.out_pitch + r0 + tx] = tile[tx][s];
    }
}

hipError_t launchTranspose(const TransposeArgs &a, const LaunchCtx &ctx) {
    if (!a.in || !a.out || a.B <= 0 || a.R <= 0 || a.S <= 0 || (a.elem != 1 && a.elem != 2) || a.out_pitch < a.R) return hipErrorInvalidValue;
    if (a.elem == 2 && ((((uintptr_t)a.in) | ((uintptr_t)a.out)) & 1)) return hipErrorInvalidValue;
    const long long blocks = (long long)a.B * ((a.R + 63) / 64) * ((a.S + 63) / 64);
    if (blocks >= (1LL << 31)) return hipErrorInvalidValue;
    if (a.elem == 2) {
        THIP_ENQUEUE(ctx, "transpose_i8<2>", transpose_i8<uint16_t>, dim3((unsigned)blocks), dim3(256), 0, a);
    } else {
        THIP_ENQUEUE(ctx, "transpose_i8<1>", transpose_i8<int8_t>, dim3((unsigned)blocks), dim3(256), 0, a);
    }
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// fc_bf16: bf16 fully_connected / matmul with the weights streamed once per 32 rows of the input
// (decode-shaped: few rows, weight traffic dominates).  A block owns 32 output columns of 32 input
// rows; its four waves split K and add their fp32 partial sums through LDS.
// v_mfma_f32_32x32x16_bf16, weights as the first operand: register r of lane l ends up with
// out[m = l & 31][n = 8 (r / 4) + 4 (l >> 5) + (r & 3)].  Per 64 elements of K a lane loads 64
// contiguous bytes of one weight row and of one input row (lane l: row l & 31, elements
// 32 (l >> 5) .. + 31 of the 64) and MFMA step c takes 16-byte piece c of every lane: the k order
// inside the 64 is permuted, identically for both operands, so that a wave's loads cover whole
// 128-byte stretches of 32 rows.  fp32 products of bf16 values are exact; only the order of the
// additions differs from a sequential sum.  K % 8 == 0.
// ---------------------------------------------------------------------------
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
typedef float v2f __attribute__((ext_vector_type(2)));

// Four int8 weights of a dword to bf16 pairs: w * scale + bias in fp32 (the product of an 8-bit weight and a
// bf16 scale is exact, so the fused multiply-add rounds once, like a multiply followed by an add), optional
// clamp, round to nearest even.
template <bool CLAMP>
__device__ __forceinline__ void expandQ8(int d, float sc, float bi, float lo, float hi, int *o0, int *o1) {
    float f[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        f[j] = __builtin_fmaf((float)(int8_t)(d >> (8 * j)), sc, bi);
        if (CLAMP) f[j] = f[j] < lo ? lo : (f[j] > hi ? hi : f[j]);
    }
    *o0 = __builtin_bit_cast(int, __builtin_convertvector((v2f){f[0], f[1]}, v2bf));
    *o1 = __builtin_bit_cast(int, __builtin_convertvector((v2f){f[2], f[3]}, v2bf));
}

// Bias, clamp, round to bf16 and store one 32 x 32 accumulator tile: register 4 q + e of lane (r, h) is
// out[m0 + r][n0 + 8 q + 4 h + e].  fcBf16StoreQuad stores the four registers of one q.
__device__ __forceinline__ void fcBf16StoreQuad(const FcBf16Args &p, const float (&a)[4], int m0, int n0, int r, int h, int q) {
    const int m = m0 + r;
    if (m >= p.M) return;
    const int n = n0 + 8 * q + 4 * h;
    uint16_t o[4];
#pragma unroll
    for (int e = 0; e < 4; e++) {
        const int ne = n + e < p.N ? n + e : p.N - 1;
        const float t0 = a[e] + p.bias[ne];
        o[e] = bf16Bits(t0 < p.lo ? p.lo : (t0 > p.hi ? p.hi : t0));
    }
    if ((p.N & 3) == 0 && n + 3 < p.N) {
        *(v2i *)(p.out + (size_t)m * p.N + n) = v2i{(int)((uint32_t)o[0] | ((uint32_t)o[1] << 16)), (int)((uint32_t)o[2] | ((uint32_t)o[3] << 16))};
    } else {
#pragma unroll
        for (int e = 0; e < 4; e++) {
            if (n + e < p.N) p.out[(size_t)m * p.N + n + e] = o[e];
        }
    }
}
__device__ __forceinline__ void fcBf16Store(const FcBf16Args &p, const v16f &acc, int m0, int n0, int r, int h) {
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const float a[4] = {acc[4 * q], acc[4 * q + 1], acc[4 * q + 2], acc[4 * q + 3]};
        fcBf16StoreQuad(p, a, m0, n0, r, h, q);
    }
}

// waves of a block = ways K is split; Q8: 0 bf16 weights, 1 int8 expanded, 2 with clamp; UNR: k-steps whose loads are
// in flight together (6 for the small grids of a decoder's linears: a wave's whole share of K <= 1536 in one round trip)
template <int NWAVES, int Q8, int UNR = 4>
__global__ __launch_bounds__(NWAVES * 64) void fc_bf16(FcBf16Args p, FastDiv qblk) {
    __shared__ float partial[NWAVES - 1][16][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 31, h = lane >> 5;
    const int n0 = blockIdx.x * 32, m0 = blockIdx.y * 32;
    const int nrow = n0 + r < p.N ? n0 + r : p.N - 1;  // clamped rows are never stored
    const int mrow = m0 + r < p.M ? m0 + r : p.M - 1;
    const uint16_t *wrow = p.w + (size_t)nrow * p.K;
    const uint16_t *xrow = p.x + (size_t)mrow * p.K;
    // this block's slice of K (blockIdx.z of ksplit), then this wave's share of the slice
    const int steps = (p.K + 63) / 64;
    const int zBeg = (int)((long long)steps * blockIdx.z / p.ksplit), zEnd = (int)((long long)steps * (blockIdx.z + 1) / p.ksplit);
    const int per = (zEnd - zBeg + NWAVES - 1) / NWAVES;
    const int sBeg = zBeg + wave * per, sEnd = (sBeg + per) < zEnd ? (sBeg + per) : zEnd;
    v16f acc;
#pragma unroll
    for (int e = 0; e < 16; e++) acc[e] = 0.0f;
    // UNR steps of loads are issued before their MFMAs: one memory round trip per UNR * 64 elements of K
    for (int s0 = sBeg; s0 < sEnd; s0 += UNR) {
        v4i wv[Q8 ? 1 : UNR][4], xv[UNR][4];
        v4i wq[Q8 ? UNR : 1][2];
        uint16_t qs[Q8 ? UNR : 1];  // raw bf16 bits: converting here would wait for the load, and for every older one
        float qb[Q8 ? UNR : 1];
#pragma unroll
        for (int u = 0; u < UNR; u++) {
            const int k = (s0 + u) * 64 + 32 * h;
            if (Q8) {
                // the lane's 32 weights of this step lie in one block: one scale, one bias.  Loads only, no branch:
                // a step past the end re-reads the last one and meets zero input rows
                const int sq = s0 + u < sEnd ? s0 + u : sEnd - 1, kq = sq * 64 + 32 * h;
                const size_t g = fastDiv((uint32_t)(kq < p.K ? kq : 0), qblk);  // beyond K the input rows are zero
                qs[u] = p.qscale[g * p.qcols + n0 + r];
                qb[u] = p.qbias[g * p.qcols + n0 + r];
#pragma unroll
                for (int h2 = 0; h2 < 2; h2++) {
                    wq[u][h2] = *(const v4i *)((const int8_t *)p.w + ((((size_t)blockIdx.x * steps + sq) * 2 + h2) * 64 + lane) * 16);
                }
            }
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const bool in = s0 + u < sEnd && k + 8 * c < p.K;  // K % 8 == 0: a piece is inside K or outside
                if (Q8) {
                } else if (p.w_fragments) {
                    // whole (zero padded) steps: every lane of the wave loads, 1 KiB in a row
                    const int8_t *frag = (const int8_t *)p.w + ((((size_t)blockIdx.x * steps + (s0 + u)) * 4 + c) * 64 + lane) * 16;
                    wv[Q8 ? 0 : u][c] = s0 + u < sEnd ? *(const v4i *)frag : v4i{0, 0, 0, 0};
                } else {
                    wv[Q8 ? 0 : u][c] = in ? *(const v4i *)(wrow + k + 8 * c) : v4i{0, 0, 0, 0};
                }
                xv[u][c] = in ? *(const v4i *)(xrow + k + 8 * c) : v4i{0, 0, 0, 0};
            }
        }
#pragma unroll
        for (int u = 0; u < UNR; u++) {
#pragma unroll
            for (int c = 0; c < 4; c++) {
                v4i wpiece;
                if (Q8) {
                    // piece c = bytes 8 (c & 1) .. + 7 of half c >> 1; the k rows beyond K are zero in the input
                    int o[4];
                    const float sc = __uint_as_float((uint32_t)qs[u] << 16);
                    expandQ8<Q8 == 2>(wq[u][c >> 1][2 * (c & 1)], sc, qb[u], p.qlo, p.qhi, &o[0], &o[1]);
                    expandQ8<Q8 == 2>(wq[u][c >> 1][2 * (c & 1) + 1], sc, qb[u], p.qlo, p.qhi, &o[2], &o[3]);
                    wpiece = v4i{o[0], o[1], o[2], o[3]};
                } else {
                    wpiece = wv[u][c];
                }
                acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, wpiece), __builtin_bit_cast(v8bf, xv[u][c]), acc, 0, 0, 0);
            }
        }
    }
    if (wave > 0) {
#pragma unroll
        for (int e = 0; e < 16; e++) partial[wave - 1][e][lane] = acc[e];
    }
    __syncthreads();
    if (wave > 0) return;
    for (int w = 0; w < NWAVES - 1; w++) {
#pragma unroll
        for (int e = 0; e < 16; e++) acc[e] += partial[w][e][lane];
    }
    if (p.ksplit > 1) {
        // K split over blocks: every block leaves its partial tile in the workspace and fc_bf16_reduce, launched
        // behind this kernel, adds the slices in slice order.  (One kernel with a fence, a counter per tile and the
        // last block to arrive doing the sum measured 5-7 us slower: the fence writes the XCD's L2 back.)
        const int tile = blockIdx.y * gridDim.x + blockIdx.x;
        float *mine = (float *)p.workspace + ((size_t)tile * p.ksplit + blockIdx.z) * 1024;
#pragma unroll
        for (int e = 0; e < 16; e++) mine[e * 64 + lane] = acc[e];
        return;
    }
    fcBf16Store(p, acc, m0, n0, r, h);
}

// Second kernel of a K split: a block per output tile adds the slices' partial tiles in slice order and finishes the
// tile (bias, clamp, bf16).  Wave q owns registers 4 q .. 4 q + 3 of the tile's accumulator layout; the loads of
// every slice (at most 16) are issued before the first addition, so the kernel is one memory round trip.
__global__ __launch_bounds__(256) void fc_bf16_reduce(FcBf16Args p) {
    const int lane = threadIdx.x & 63, q = threadIdx.x >> 6, r = lane & 31, h = lane >> 5;
    const int tile = blockIdx.y * gridDim.x + blockIdx.x;
    const float *parts = (const float *)p.workspace + (size_t)tile * p.ksplit * 1024 + (size_t)(4 * q) * 64 + lane;
    float v[16][4];
#pragma unroll
    for (int z = 0; z < 16; z++) {
        const int zc = z < p.ksplit ? z : p.ksplit - 1;  // loads only, no branch: slices past the split re-read the last one
#pragma unroll
        for (int e = 0; e < 4; e++) v[z][e] = parts[(size_t)zc * 1024 + e * 64];
    }
    float a[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int z = 0; z < 16; z++) {
#pragma unroll
        for (int e = 0; e < 4; e++) a[e] += z < p.ksplit ? v[z][e] : 0.0f;
    }
    fcBf16StoreQuad(p, a, blockIdx.y * 32, blockIdx.x * 32, r, h, q);
}

// fc_bf16_wide: the same product for a very wide N and a short K (a vocabulary projection): a wave owns a
// column block for the whole of K, so nothing is reduced across waves, and it streams the weights through two
// register buffers, the loads of one in flight while the other feeds the MFMAs.  The input rows of the block
// (at most 32, and one slot of zeros for the lanes of rows it does not have) sit in LDS in fragment order, read
// 16 bytes per lane right before each MFMA: with few rows that is a few KiB, and registers set the occupancy.
// Weights in fragment order only (layouts 1 and 2).
constexpr int kFcBf16WideMaxSteps = 24;  // 99 KiB of LDS for 32 input rows
template <int Q8, int U, int W = 4>  // U: k-steps per register buffer; W: waves per block (they share the block's input rows in LDS)
__global__ __launch_bounds__(64 * W) void fc_bf16_wide(FcBf16Args p, FastDiv qblk) {
    extern __shared__ __attribute__((aligned(16))) int8_t xs[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 31, h = lane >> 5;
    const int steps = (p.K + 63) / 64;
    const int m0 = blockIdx.y * 32;
    // rows the block really has, plus one slot of zeros that the lanes of the missing rows all read
    const int mt = p.M - m0 < 32 ? p.M - m0 : 32, slots = 2 * (mt + 1);
    for (int i = threadIdx.x; i < steps * 4 * slots; i += 64 * W) {
        const int slot = i % slots, sc = i / slots, c = sc & 3, s = sc >> 2;
        const int hh = slot / (mt + 1), rr = slot - hh * (mt + 1);
        const int k = s * 64 + 32 * hh + 8 * c;
        v4i v = {0, 0, 0, 0};
        if (rr < mt && k < p.K) v = *(const v4i *)(p.x + (size_t)(m0 + rr) * p.K + k);
        *(v4i *)(xs + (size_t)i * 16) = v;
    }
    __syncthreads();
    const int xslot = (h * (mt + 1) + (r < mt ? r : mt)) * 16;
    const int nb = blockIdx.x * W + wave;
    if (nb >= (p.N + 31) / 32) return;
    const int n0 = nb * 32;
    constexpr int PIECES = Q8 ? 2 : 4;  // 16-byte loads per lane per step
    const int8_t *wbase = (const int8_t *)p.w + (size_t)nb * steps * (PIECES * 1024) + lane * 16;
    struct Buf {
        v4i w[U][PIECES];
        uint16_t qs[U];  // raw bf16 bits: converting here would wait for the load, and with it for every older one
        float qb[U];
    };
    // Loads only, no use of a loaded value and no branch: the steps past the end re-read the last one (never used).
    auto loadGroup = [&](int s0, Buf &b) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int s = s0 + u < steps ? s0 + u : steps - 1;
#pragma unroll
            for (int c = 0; c < PIECES; c++) b.w[u][c] = *(const v4i *)(wbase + ((size_t)s * PIECES + c) * 1024);
            if (Q8) {
                const int k = s * 64 + 32 * h;
                const size_t g = fastDiv((uint32_t)(k < p.K ? k : 0), qblk);  // beyond K the input rows are zero
                b.qs[u] = p.qscale[g * p.qcols + n0 + r];
                b.qb[u] = p.qbias[g * p.qcols + n0 + r];
            }
        }
    };
    v16f acc;
#pragma unroll
    for (int e = 0; e < 16; e++) acc[e] = 0.0f;
    auto compute = [&](int s0, const Buf &b) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int s = s0 + u;
            if (s >= steps) break;
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const v4i xpiece = *(const v4i *)(xs + (size_t)(s * 4 + c) * slots * 16 + xslot);
                v4i wpiece;
                if (Q8) {
                    int o[4];
                    const float sc = __uint_as_float((uint32_t)b.qs[u] << 16);
                    expandQ8<Q8 == 2>(b.w[u][c >> 1][2 * (c & 1)], sc, b.qb[u], p.qlo, p.qhi, &o[0], &o[1]);
                    expandQ8<Q8 == 2>(b.w[u][c >> 1][2 * (c & 1) + 1], sc, b.qb[u], p.qlo, p.qhi, &o[2], &o[3]);
                    wpiece = v4i{o[0], o[1], o[2], o[3]};
                } else {
                    wpiece = b.w[u][c & (PIECES - 1)];
                }
                acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, wpiece), __builtin_bit_cast(v8bf, xpiece), acc, 0, 0, 0);
            }
        }
    };
    Buf b0, b1;
    loadGroup(0, b0);
    for (int s0 = 0; s0 < steps; s0 += 2 * U) {
        loadGroup(s0 + U, b1);
        compute(s0, b0);
        loadGroup(s0 + 2 * U, b0);
        compute(s0 + U, b1);
    }
    fcBf16Store(p, acc, m0, n0, r, h);
}

template <int Q8, int U, int W>
static hipError_t launchFcBf16WideUW(const FcBf16Args &a, FastDiv blk, const LaunchCtx &ctx) {
    auto kernel = fc_bf16_wide<Q8, U, W>;
    static std::once_flag once;
    static hipError_t configured = hipSuccess;
    std::call_once(once, [&] { configured = hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, kFcBf16WideMaxSteps * 4 * 66 * 16); });
    if (configured != hipSuccess) return configured;
    const int steps = (a.K + 63) / 64, nblocks = (a.N + 31) / 32;
    const dim3 grid((unsigned)((nblocks + W - 1) / W), (unsigned)((a.M + 31) / 32));
    const int mt = a.M < 32 ? a.M : 32;
    THIP_ENQUEUE(ctx, kernelLabel("fc_bf16_wide", {Q8, U, W}), kernel, grid, dim3(64 * W), (size_t)steps * 4 * 2 * (mt + 1) * 16, a, blk);
    return hipGetLastError();
}

template <int Q8, int U>
static hipError_t launchFcBf16WideU(const FcBf16Args &a, FastDiv blk, const LaunchCtx &ctx) {
    // Waves per block: they share one copy of the block's input rows in LDS (up to 99 KiB, read from L2 once per block),
    // so more waves mean fewer copies and more waves per CU.  Measured at K = 1152, N = 65536, 1 / 32 / 64 rows, in us:
    // bf16 weights 26.3 / 34.4 / 64.8 with four waves, 26.0 / 30.3 / 53.0 with eight, 26.6 / 29.3 / 30.2 with sixteen;
    // block-scaled int8 weights 19.7 / 27.6 / 50.4, 19.4 / 23.5 / 34.3 and 23.9 / 26.2 / 28.6 (one block of sixteen
    // waves per CU: its prologue overlaps with nothing).  THIP_FC_WIDE_WAVES forces a count.
    constexpr bool fitsSixteen = U <= (Q8 ? 4 : 2);  // beyond that 128 registers per lane are not enough
    int waves = ctx.tuning->fcWideWaves;
    if (waves != 4 && waves != 8 && waves != 16) waves = (!Q8 || a.M > 32) ? 16 : 8;
    if constexpr (fitsSixteen) {
        if (waves == 16) return launchFcBf16WideUW<Q8, U, 16>(a, blk, ctx);
    }
    return waves == 4 ? launchFcBf16WideUW<Q8, U, 4>(a, blk, ctx) : launchFcBf16WideUW<Q8, U, 8>(a, blk, ctx);
}

template <int Q8>
static hipError_t launchFcBf16Wide(const FcBf16Args &a, FastDiv blk, const LaunchCtx &ctx) {
    const int u = ctx.tuning->fcWideU > 0 ? ctx.tuning->fcWideU : (Q8 ? 4 : 2);
    if (u == 8 && Q8) return launchFcBf16WideU<Q8, 8>(a, blk, ctx);
    if (u == 4) return launchFcBf16WideU<Q8, 4>(a, blk, ctx);
    return launchFcBf16WideU<Q8, Q8 ? 4 : 2>(a, blk, ctx);
}

hipError_t launchFcBf16(const FcBf16Args &a, const LaunchCtx &ctx) {
    if (!a.x || !a.w || !a.bias || !a.out || a.M <= 0 || a.N <= 0 || a.K <= 0 || a.K % 8 != 0) return hipErrorInvalidValue;
    if (((((uintptr_t)a.x) | ((uintptr_t)a.w)) & 15) || (((uintptr_t)a.out) & (a.N % 4 == 0 ? 7 : 1)) || (((uintptr_t)a.bias) & 3)) return hipErrorInvalidValue;
    if (a.ksplit < 1 || a.ksplit > 16 || (a.ksplit > 1 && (!a.workspace || ((uintptr_t)a.workspace & 255)))) return hipErrorInvalidValue;
    const dim3 grid((unsigned)((a.N + 31) / 32), (unsigned)((a.M + 31) / 32), (unsigned)a.ksplit);
    if (grid.y > 65535) return hipErrorInvalidValue;
    // few blocks (registers do not limit anything then) and 5 or 6 k-steps per wave: one deeper round of loads instead of two
    const int stepsPerWave = (((a.K + 63) / 64 + a.ksplit - 1) / a.ksplit + 3) / 4;
    const bool deep = (long long)grid.x * grid.y * grid.z <= 512 && stepsPerWave > 4 && stepsPerWave <= 6 && !ctx.tuning->noFcDeep;
    // a very wide N with a short K and no K split: every wave streams its own columns (THIP_NO_FC_WIDE: off)
    const bool wide = a.w_fragments >= 1 && a.ksplit == 1 && (a.K + 63) / 64 <= kFcBf16WideMaxSteps && (a.N + 31) / 32 >= 1024 &&
                      !ctx.tuning->noFcWide;
    if (a.w_fragments == 2) {
        if (!a.qscale || !a.qbias || a.qblock < 32 || a.qblock % 32 != 0 || a.qcols < (a.N + 31) / 32 * 32 || a.qcols % 32 != 0) return hipErrorInvalidValue;
        if ((((uintptr_t)a.qscale) & 1) || (((uintptr_t)a.qbias) & 3)) return hipErrorInvalidValue;
        const FastDiv blk = makeFastDiv((uint32_t)a.qblock);
        const bool clamp = !(a.qlo == -INFINITY && a.qhi == INFINITY);
        if (wide) return clamp ? launchFcBf16Wide<2>(a, blk, ctx) : launchFcBf16Wide<1>(a, blk, ctx);
        if (clamp) THIP_ENQUEUE(ctx, "fc_bf16<4,2,4>", (fc_bf16<4, 2>), grid, dim3(256), 0, a, blk);
        else if (deep) THIP_ENQUEUE(ctx, "fc_bf16<4,1,6>", (fc_bf16<4, 1, 6>), grid, dim3(256), 0, a, blk);
        else THIP_ENQUEUE(ctx, "fc_bf16<4,1,4>", (fc_bf16<4, 1>), grid, dim3(256), 0, a, blk);
        if (a.ksplit > 1 && !ctx.name) hipLaunchKernelGGL(fc_bf16_reduce, dim3(grid.x, grid.y), dim3(256), 0, ctx.stream, a);
        return hipGetLastError();
    }
    if (wide) return launchFcBf16Wide<0>(a, makeFastDiv(1), ctx);
    if (deep) THIP_ENQUEUE(ctx, "fc_bf16<4,0,6>", (fc_bf16<4, 0, 6>), grid, dim3(256), 0, a, makeFastDiv(1));
    else THIP_ENQUEUE(ctx, "fc_bf16<4,0,4>", (fc_bf16<4, 0>), grid, dim3(256), 0, a, makeFastDiv(1));
    if (a.ksplit > 1 && !ctx.name) hipLaunchKernelGGL(fc_bf16_reduce, dim3(grid.x, grid.y), dim3(256), 0, ctx.stream, a);
    return hipGetLastError();
}

// bf16 global average pool: a thread owns VEC neighbouring channels of one image and walks the frame in
// order (the sums then equal a sequential fp32 accumulation bit for bit); a wave's loads cover 64 * VEC
// neighbouring channels of one pixel.
template <int VEC>
__global__ __launch_bounds__(256) void avgpool_bf16(AvgPoolBf16Args p) {
    const int cgroups = p.C / VEC;
    const long long t = (long long)blockIdx.x * 256 + threadIdx.x;
    if (t >= (long long)p.N * cgroups) return;
    const int n = (int)(t / cgroups), c0 = (int)(t % cgroups) * VEC;
    const uint16_t *src = p.in + (size_t)n * p.HW * p.C + c0;
    float acc[VEC];
#pragma unroll
    for (int v = 0; v < VEC; v++) acc[v] = 0.0f;
#pragma unroll 8
    for (int u = 0; u < p.HW; u++) {
        uint16_t x[VEC];
        if (VEC == 2) {
            const uint32_t d = *(const uint32_t *)(src + (size_t)u * p.C);
            x[0] = (uint16_t)d;
            x[VEC - 1] = (uint16_t)(d >> 16);
        } else {
            x[0] = src[(size_t)u * p.C];
        }
#pragma unroll
        for (int v = 0; v < VEC; v++) acc[v] = __fadd_rn(acc[v], __fmul_rn(__uint_as_float((uint32_t)x[v] << 16), p.weight));
    }
#pragma unroll
    for (int v = 0; v < VEC; v++) {
        const float t0 = __fadd_rn(acc[v], p.bias);
        p.out[(size_t)n * p.C + c0 + v] = bf16Bits(t0 < p.lo ? p.lo : (t0 > p.hi ? p.hi : t0));
    }
}

hipError_t launchAvgPoolBf16(const AvgPoolBf16Args &a, const LaunchCtx &ctx) {
    if (a.N <= 0 || a.HW <= 0 || a.C <= 0 || !a.in || !a.out) return hipErrorInvalidValue;
    const bool pairs = a.C % 2 == 0 && (((uintptr_t)a.in) & 3) == 0;
    const long long threads = (long long)a.N * (pairs ? a.C / 2 : a.C);
    const dim3 grid((unsigned)((threads + 255) / 256));
    if (pairs) THIP_ENQUEUE(ctx, "avgpool_bf16<2>", avgpool_bf16<2>, grid, dim3(256), 0, a);
    else THIP_ENQUEUE(ctx, "avgpool_bf16<1>", avgpool_bf16<1>, grid, dim3(256), 0, a);
    return hipGetLastError();
}

// torq_hl.expand_weights as an op of its own (the result is a binding, or has several readers): a thread
// expands four neighbouring columns of one row.
__global__ __launch_bounds__(256) void expand_weights_bf16(ExpandWeightsArgs p, FastDiv blk, int quads) {
    const long long t = (long long)blockIdx.x * 256 + threadIdx.x;
    if (t >= (long long)p.K * quads) return;
    const int k = (int)(t / quads), n0 = (int)(t % quads) * 4;
    const size_t g = fastDiv((uint32_t)k, blk);
#pragma unroll
    for (int e = 0; e < 4; e++) {
        const int n = n0 + e;
        if (n >= p.N) break;
        const float sc = __uint_as_float((uint32_t)p.scale[g * p.N + n] << 16);
        const float t0 = __fadd_rn(__fmul_rn((float)p.w[(size_t)k * p.N + n], sc), p.bias[g * p.bias_cols + n]);
        p.out[(size_t)k * p.N + n] = bf16Bits(t0 < p.lo ? p.lo : (t0 > p.hi ? p.hi : t0));
    }
}

hipError_t launchExpandWeights(const ExpandWeightsArgs &a, const LaunchCtx &ctx) {
    if (!a.w || !a.scale || !a.bias || !a.out || a.K <= 0 || a.N <= 0 || a.block <= 0 || a.K % a.block != 0 || a.bias_cols < a.N) return hipErrorInvalidValue;
    const int quads = (a.N + 3) / 4;
    const long long threads = (long long)a.K * quads;
    if (threads >= (1LL << 39)) return hipErrorInvalidValue;
    THIP_ENQUEUE(ctx, "expand_weights_bf16", expand_weights_bf16, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, a, makeFastDiv((uint32_t)a.block), quads);
    return hipGetLastError();
}

}  // namespace thip

namespace thip {

// ---------------------------------------------------------------------------
// Scratch memory that exists without any allocation: a device array of the library's image.  Every GPU the
// library runs on holds its own copy, at its own address, until the process ends.  In host code the array's name
// is only a handle for hipGetSymbolAddress; the address that call returns is what kernels, fills and copies take.
// ---------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

hipError_t staticScratchAddress(void **out) {
    // asked once per device, with that device current; kept for the life of the process
    static std::mutex mutex;
    static void *known[64] = {nullptr};
    int device = -1;
    hipError_t err = hipGetDevice(&device);
    if (err != hipSuccess) return err;
    if (device < 0 || device >= 64) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(mutex);
    if (!known[device]) {
        void *ptr = nullptr;
        err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (err != hipSuccess) return err;
        if (!ptr || ((uintptr_t)ptr & 255) != 0) return hipErrorInvalidSymbol;
        known[device] = ptr;
    }
    *out = known[device];
    return hipSuccess;
}

// ---------------------------------------------------------------------------
// Calibration: what the matrix cores sustain on this GPU with nothing else going on.  Every wave owns a 4 x 4 grid of
// 32 x 32 accumulators (the register layout of the 256 x 256 GEMM tile) and issues v_mfma_i32_32x32x32_i8 back to
// back on operands it loaded once; no memory traffic inside the loop.  The rate depends on the operand VALUES: the
// card runs against a power limit, and random bytes toggle far more of the datapath than constants do.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void mfma_rate_i8(int iterations, const v4i *__restrict__ operands, int *__restrict__ sink) {
    v16i acc[4][4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
#pragma unroll
            for (int r = 0; r < 16; r++) acc[j][i][r] = 0;
        }
    }
    v4i a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        a[i] = operands[threadIdx.x + 256 * i];
        b[i] = operands[threadIdx.x + 256 * (4 + i)];
    }
    for (int it = 0; it < iterations; it++) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
#pragma unroll
            for (int i = 0; i < 4; i++) acc[j][i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(b[j], a[i], acc[j][i], 0, 0, 0);
        }
        // the operands stay live and opaque, so the loop is not folded
        asm volatile("" : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(b[0]), "+v"(b[1]), "+v"(b[2]), "+v"(b[3]));
    }
    int s = 0;
#pragma unroll
    for (int j = 0; j < 4; j++) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
#pragma unroll
            for (int r = 0; r < 16; r++) s += acc[j][i][r];
        }
    }
    sink[blockIdx.x * 256 + threadIdx.x] = s;
}

hipError_t measureMfmaRate(int randomOperands, int blocks, int iterations, hipStream_t stream, double *outTops) {
    if (blocks <= 0 || blocks > 65536 || iterations <= 0 || !outTops) return hipErrorInvalidValue;
    constexpr size_t kOperandBytes = 256 * 8 * 16;
    uint8_t host[kOperandBytes];
    uint32_t x = 0x9e3779b9u;
    for (size_t i = 0; i < kOperandBytes; i++) {
        x ^= x << 13; x ^= x >> 17; x ^= x << 5;  // xorshift: any uniform bytes will do
        host[i] = randomOperands ? (uint8_t)(x >> 11) : (uint8_t)1;
    }
    v4i *operands = nullptr;
    int *sink = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    hipError_t err = hipMalloc((void **)&operands, kOperandBytes);
    if (err == hipSuccess) err = hipMalloc((void **)&sink, (size_t)blocks * 256 * 4);
    if (err == hipSuccess) err = hipMemcpy(operands, host, kOperandBytes, hipMemcpyHostToDevice);
    if (err == hipSuccess) err = hipEventCreate(&e0);
    if (err == hipSuccess) err = hipEventCreate(&e1);
    if (err == hipSuccess) {
        hipLaunchKernelGGL(mfma_rate_i8, dim3((unsigned)blocks), dim3(256), 0, stream, iterations / 20 + 1, operands, sink);  // warm-up
        err = hipEventRecord(e0, stream);
        hipLaunchKernelGGL(mfma_rate_i8, dim3((unsigned)blocks), dim3(256), 0, stream, iterations, operands, sink);
        if (err == hipSuccess) err = hipGetLastError();
        if (err == hipSuccess) err = hipEventRecord(e1, stream);
        if (err == hipSuccess) err = hipEventSynchronize(e1);
        float ms = 0.f;
        if (err == hipSuccess) err = hipEventElapsedTime(&ms, e0, e1);
        // per wave and iteration: 16 MFMAs of 32 x 32 x 32 multiply-adds, 2 ops each
        if (err == hipSuccess) *outTops = (double)blocks * 4 * iterations * 16 * 32768.0 * 2 / ((double)ms * 1e-3) / 1e12;
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (operands) (void)hipFree(operands);
    if (sink) (void)hipFree(sink);
    return err;
}

// Calibration: what a kernel with no arithmetic to speak of reaches on this memory system for a transfer of a given
// size: every thread reads RD 16-byte pieces (from RD separate streams, perfectly coalesced), combines them with one
// instruction each and writes 16 bytes.  RD = 1 is a plain copy, RD = 2 the traffic shape of an elementwise add,
// RD = 4 that of a 2 x 2 pooling or a stride-2 3 x 3 depthwise convolution.
template <int RD>
__global__ __launch_bounds__(256) void stream_floor(const v4i *__restrict__ in, v4i *__restrict__ out, size_t items) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= items) return;
    v4i v[RD];
#pragma unroll
    for (int r = 0; r < RD; r++) v[r] = in[(size_t)r * items + i];
    v4i m = v[0];
#pragma unroll
    for (int r = 1; r < RD; r++) {
        m[0] ^= v[r][0];
        m[1] ^= v[r][1];
        m[2] ^= v[r][2];
        m[3] ^= v[r][3];
    }
    out[i] = m;
}

hipError_t measureStreamRate(int readsPerWrite, size_t writeBytes, int cold, hipStream_t stream, double *outMicroseconds) {
    if ((readsPerWrite != 1 && readsPerWrite != 2 && readsPerWrite != 4) || writeBytes < 4096 || writeBytes % 16 != 0 || writeBytes > (1ull << 31) ||
        !outMicroseconds) {
        return hipErrorInvalidValue;
    }
    const size_t items = writeBytes / 16, perSet = writeBytes * (size_t)(readsPerWrite + 1);
    // cold: dispatch i works on buffer set i mod n, the sets together twice the size of the 256 MiB last-level cache
    int sets = cold ? (int)((512ull << 20) / perSet) + 1 : 1;
    sets = sets < (cold ? 2 : 1) ? 2 : (sets > 160 ? 160 : sets);
    std::vector<v4i *> in((size_t)sets, nullptr), out((size_t)sets, nullptr);
    hipEvent_t e0 = nullptr, e1 = nullptr;
    hipError_t err = hipSuccess;
    for (int s = 0; s < sets && err == hipSuccess; s++) {
        err = hipMalloc((void **)&in[(size_t)s], writeBytes * (size_t)readsPerWrite);
        if (err == hipSuccess) err = hipMalloc((void **)&out[(size_t)s], writeBytes);
        if (err == hipSuccess) err = hipMemsetAsync(in[(size_t)s], s + 1, writeBytes * (size_t)readsPerWrite, stream);
    }
    auto launch = [&](int s) {
        const dim3 grid((unsigned)((items + 255) / 256));
        if (readsPerWrite == 1) hipLaunchKernelGGL(stream_floor<1>, grid, dim3(256), 0, stream, in[(size_t)s], out[(size_t)s], items);
        else if (readsPerWrite == 2) hipLaunchKernelGGL(stream_floor<2>, grid, dim3(256), 0, stream, in[(size_t)s], out[(size_t)s], items);
        else hipLaunchKernelGGL(stream_floor<4>, grid, dim3(256), 0, stream, in[(size_t)s], out[(size_t)s], items);
    };
    if (err == hipSuccess) err = hipEventCreate(&e0);
    if (err == hipSuccess) err = hipEventCreate(&e1);
    if (err == hipSuccess) {
        for (int s = 0; s < sets; s++) launch(s);  // first touch
        const int iterations = sets * 3 > 30 ? sets * 3 : 30;
        err = hipEventRecord(e0, stream);
        for (int i = 0; i < iterations; i++) launch(i % sets);
        if (err == hipSuccess) err = hipGetLastError();
        if (err == hipSuccess) err = hipEventRecord(e1, stream);
        if (err == hipSuccess) err = hipEventSynchronize(e1);
        float ms = 0.f;
        if (err == hipSuccess) err = hipEventElapsedTime(&ms, e0, e1);
        if (err == hipSuccess) *outMicroseconds = (double)ms * 1e3 / iterations;
    }
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    for (int s = 0; s < sets; s++) {
        if (in[(size_t)s]) (void)hipFree(in[(size_t)s]);
        if (out[(size_t)s]) (void)hipFree(out[(size_t)s]);
    }
    return err;
}

Tuning tuningFromEnvironment() {
    Tuning t;
    auto flag = [](const char *name) { return getenv(name) != nullptr; };
    auto digit = [](const char *name, int unset) {
        const char *v = getenv(name);
        return v && v[0] >= '0' && v[0] <= '9' ? v[0] - '0' : unset;
    };
    t.noStreamDeep = flag("THIP_NO_STREAM_DEEP");
    t.streamGuarded = flag("THIP_STREAM_GUARDED");
    t.streamStage = digit("THIP_STREAM_STAGE", -1);
    if (t.streamStage > 1) t.streamStage = -1;
    t.noDirectEpilogue = flag("THIP_NO_DIRECT_EPILOGUE");
    t.skinnyDot4 = flag("THIP_SKINNY_DOT4");
    t.depthwiseStrip = digit("THIP_DEPTHWISE_STRIP", -1);
    if (t.depthwiseStrip > 2) t.depthwiseStrip = -1;
    t.depthwiseTile = digit("THIP_DEPTHWISE_TILE", -1);
    if (t.depthwiseTile > 1) t.depthwiseTile = -1;
    if (const char *v = getenv("THIP_DEPTHWISE_TILE_MIN")) t.depthwiseTileMin = atoll(v);
    if (const char *v = getenv("THIP_DEPTHWISE_P")) t.depthwisePixels = atoi(v);
    if (const char *v = getenv("THIP_FC_WIDE_U")) t.fcWideU = atoi(v);
    if (const char *v = getenv("THIP_FC_WIDE_WAVES")) t.fcWideWaves = atoi(v);
    if (const char *v = getenv("THIP_DENSE_SHORT_K")) t.denseShortK = atoi(v);
    t.noK128 = flag("THIP_NO_K128");
    t.noFcDeep = flag("THIP_NO_FC_DEEP");
    t.noFcWide = flag("THIP_NO_FC_WIDE");
    t.maxpoolGeneric = flag("THIP_MAXPOOL_GENERIC");
    t.addGeneric = flag("THIP_ADD_GENERIC");
    return t;
}

}  // namespace thip
