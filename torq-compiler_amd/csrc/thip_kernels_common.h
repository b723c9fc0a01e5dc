// Device-side helpers shared by the gfx950 kernel files: vector types, the launch-site macro, the requantisation
// tails (the reference's ACT rescale-clamp, compiler/torq/Utils/Kernel.h:610-624: int32 add of the bias, 32x32->64
// bit multiply by the scale, add of 2^(shift-1), arithmetic right shift, add of the output zero point, clamp),
// bf16 rounding and the precomputed divisions of the bandwidth kernels' work split.
#pragma once

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

__device__ __forceinline__ void blockBarrier() { asm volatile("s_barrier" : : : "memory"); }

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

// torq_hl.add on bf16, one element: no fused multiply-add -- the second product is added to the first (both exact in
// fp32), then the bias, as the ACT stage does; clamp; round to nearest even.
__device__ __forceinline__ uint16_t addBf16One(uint16_t a, uint16_t b, float w0, float w1, float bias, float lo, float hi) {
    const float x0 = __uint_as_float((uint32_t)a << 16), x1 = __uint_as_float((uint32_t)b << 16);
    float acc = __fmul_rn(x0, w0);
    acc = __fadd_rn(acc, __fmul_rn(x1, w1));
    const float t0 = __fadd_rn(acc, bias);
    return bf16Bits(t0 < lo ? lo : (t0 > hi ? hi : t0));
}

// global -> LDS without registers (global_load_lds_dwordx4): the 64 lanes of a wave write 64 x 16 bytes = 1 KiB of
// consecutive LDS starting at ldsAddr (wave-uniform), each from its own global address.  The load counts in vmcnt
// like any other; the compiler does not see it, so whoever issues it waits for it by hand (waitVmcnt).
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


// Loads and stores of data that is used once (a bandwidth-bound op's input and output): the non-temporal cache policy.
// A plain copy of 64 MB .. 512 MB reaches 5.7 .. 6.5 TB/s with it against 4.9 .. 5.7 TB/s with the default policy
// (the calibration family of thip_device_stream_floor: the non-temporal member wins every shape).
template <typename T>
__device__ __forceinline__ T streamLoad(const void *p) {
    return __builtin_nontemporal_load((const T *)p);
}
template <typename T>
__device__ __forceinline__ void streamStore(void *p, T v) {
    __builtin_nontemporal_store(v, (T *)p);
}

}  // namespace thip
