// gfx950 kernels of the bf16 rows: fully_connected / matmul with fp32 accumulation on v_mfma_f32_32x32x16_bf16
// (weights in bf16 or block-quantized int8 expanded in registers), the global average pool and torq_hl.expand_weights.
#include "thip_kernels_common.h"

namespace thip {

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
