// gfx950 kernels of the bandwidth-bound ops: depthwise convolution, max / average pooling, the quantised add, the
// integer elementwise ops, table lookups, transposes, and the small bf16 ops (im2col, depthwise, add).
#include "thip_kernels_common.h"

namespace thip {

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
    u.v = *(const typename DwordVec<G>::type *)src;  // neighbouring threads and strips read the same bytes again: default cache policy
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
                        // written once, read by another kernel: the non-temporal policy at stride 2 (56 x 56 x 144, batch 64:
                        // 11.4 -> 10.8 us cold); at stride 1 the 4-byte pieces of neighbouring threads complete each other's
                        // lines in the cache, and the same policy costs 58 -> 64 us at batch 256
                        if (S == 2) streamStore<typename DwordVec<G>::type>(orow + (size_t)q * p.C, u.v);
                        else *(typename DwordVec<G>::type *)(orow + (size_t)q * p.C) = u.v;
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
    const v4i a = streamLoad<v4i>(src), b = streamLoad<v4i>(src + p.C), c = streamLoad<v4i>(src + row), d = streamLoad<v4i>(src + row + p.C);
    v4i o;
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const SplitBytes m = maxSplit(maxSplit(splitBytes((uint32_t)a[q]), splitBytes((uint32_t)b[q])),
                                      maxSplit(splitBytes((uint32_t)c[q]), splitBytes((uint32_t)d[q])));
        o[q] = (int)joinBytes(m);
    }
    streamStore<v4i>(p.out + (((size_t)n * p.OH + oy) * p.OW + ox) * p.C + cgi * 16, o);
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
            const v4i a = streamLoad<v4i>(p.in0 + i0), b = streamLoad<v4i>(p.in1 + i0);
            streamStore<v4i>(p.out + i0, residualAdd16<true>(a, b, false, p.w0, p.w1, p.bias, p.scale, rnd, p.rq, folded));
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
        o.h[e] = addBf16One(a.h[e], b.h[e], p.w0, p.w1, p.bias, p.lo, p.hi);
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
    // 16 bytes of the wider side per thread: the widest access is then 16 bytes, the alignment every device binding has
    // (a wider one would make the kernel depend on where a binding happens to lie, dispatch by dispatch)
    constexpr int VEC = 16 / (int)(sizeof(TIN) > sizeof(TOUT) ? sizeof(TIN) : sizeof(TOUT));
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
    // 16 bytes of the wider side per thread: the widest access is then 16 bytes, the alignment every device binding has
    // (a wider one would make the kernel depend on where a binding happens to lie, dispatch by dispatch)
    constexpr int VEC = 16 / (int)(sizeof(TIN) > sizeof(TOUT) ? sizeof(TIN) : sizeof(TOUT));
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

}  // namespace thip
