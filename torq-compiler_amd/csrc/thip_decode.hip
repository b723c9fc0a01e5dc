// gfx950 kernels of decode-shaped bf16 programs (a decoder's step: at most 32 input rows per linear, so every
// matrix is read once and the weights are the traffic): dec_linear, the grouped linear on block-quantized int8
// weights (torq_hl.expand_weights folded into torq_hl.matmul, the add behind it folded into the epilogue), and
// dec_matmul, the batched small matmul against a run-time operand held [N][K] (the attention's two products).
//
// Both use v_mfma_f32_16x16x32_bf16 with the weights as the row operand: a lane (c = lane & 15, g = lane >> 4) feeds
// weight column c and input row c, each with the 8 consecutive k of group g, and receives
// D[n = 4 g + e][m = c] in register e: four neighbouring output columns of one input row.  fp32 products of bf16
// values are exact; only the order of the additions differs from a sum in k order.
#include "thip_kernels_common.h"

namespace thip {

typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kDecWaves = 8;      // waves of a dec_matmul workgroup = ways K is split inside it
constexpr int kDecMaxWaves = 16;  // dec_linear: between 8 and 16, one k-block each where K allows (DecLinearArgs::nwaves)

__device__ __forceinline__ unsigned ldsOffset(const void *p) {
    return (unsigned)(uintptr_t)(__attribute__((address_space(3))) const int8_t *)p;
}

// 64 lanes x 4 bytes, global -> LDS (see dmaLoad16).
__device__ __forceinline__ void dmaLoad4(const void *gptr, unsigned ldsAddr) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dword %1, off" : : "s"(ldsAddr), "v"(gptr) : "memory", "m0");
}

// s_waitcnt vmcnt(n) for a wave-uniform run-time n (the instruction takes an immediate).
__device__ __forceinline__ void waitVmcntDyn(int n) {
#define THIP_VMCNT_CASE(k) \
    case k: waitVmcnt<k>(); break;
    switch (n) {
        THIP_VMCNT_CASE(0) THIP_VMCNT_CASE(1) THIP_VMCNT_CASE(2) THIP_VMCNT_CASE(3) THIP_VMCNT_CASE(4) THIP_VMCNT_CASE(5) THIP_VMCNT_CASE(6) THIP_VMCNT_CASE(7)
        THIP_VMCNT_CASE(8) THIP_VMCNT_CASE(9) THIP_VMCNT_CASE(10) THIP_VMCNT_CASE(11) THIP_VMCNT_CASE(12) THIP_VMCNT_CASE(13) THIP_VMCNT_CASE(14) THIP_VMCNT_CASE(15)
        THIP_VMCNT_CASE(16) THIP_VMCNT_CASE(17) THIP_VMCNT_CASE(18) THIP_VMCNT_CASE(19) THIP_VMCNT_CASE(20) THIP_VMCNT_CASE(21) THIP_VMCNT_CASE(22) THIP_VMCNT_CASE(23)
        THIP_VMCNT_CASE(24) THIP_VMCNT_CASE(25) THIP_VMCNT_CASE(26) THIP_VMCNT_CASE(27) THIP_VMCNT_CASE(28) THIP_VMCNT_CASE(29) THIP_VMCNT_CASE(30) THIP_VMCNT_CASE(31)
        THIP_VMCNT_CASE(32) THIP_VMCNT_CASE(33) THIP_VMCNT_CASE(34) THIP_VMCNT_CASE(35) THIP_VMCNT_CASE(36) THIP_VMCNT_CASE(37) THIP_VMCNT_CASE(38) THIP_VMCNT_CASE(39)
        THIP_VMCNT_CASE(40) THIP_VMCNT_CASE(41) THIP_VMCNT_CASE(42) THIP_VMCNT_CASE(43) THIP_VMCNT_CASE(44) THIP_VMCNT_CASE(45) THIP_VMCNT_CASE(46) THIP_VMCNT_CASE(47)
    default: break;  // 48 or more may stay in flight: more than a wave of these kernels ever has
    }
#undef THIP_VMCNT_CASE
}

constexpr int kDecLdsSlot = 2048 + 128;  // a k-block's weights, scales and (room for) biases in LDS

// MR: groups of 16 input rows (1 or 2).  XLDS: the input rows come through LDS as well (at most four rows): then every
// global load of a wave is an LDS-DMA load issued up front and each k-block is computed as soon as it has landed.
// Otherwise the rows come through registers, CH k-blocks at a time, double-buffered.  QB: the slots carry block biases.
// QC: the expansion clamps.
template <int MR, int CH, bool XLDS, bool QB, bool QC>
__global__ __launch_bounds__(kDecMaxWaves * 64) void dec_linear(DecLinearArgs p) {
    extern __shared__ __attribute__((aligned(16))) int8_t smem[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int NW = p.nwaves;  // waves of this workgroup: k-blocks wave, wave + NW, ... are this wave's
    const int c = lane & 15, g = lane >> 4;
    // the input rows of this workgroup: grid.y workgroups share a column tile, rows_per_group rows each
    const int row0 = (int)blockIdx.y * p.rows_per_group;
    const int M = p.M - row0 < p.rows_per_group ? p.M - row0 : p.rows_per_group;
    const uint16_t *x = p.x + (size_t)row0 * p.K;
    // the tile of this workgroup: (matrix, 16 columns of it); a pair owns the same columns of both matrices
    int tile = (int)blockIdx.x, seg = 0;
    if (!p.pair) {
        if (p.nseg > 1 && tile >= p.N[0] / 16) {
            tile -= p.N[0] / 16;
            seg = 1;
            if (p.nseg > 2 && tile >= p.N[1] / 16) {
                tile -= p.N[1] / 16;
                seg = 2;
            }
        }
    }
    const int nmat = p.pair ? 2 : 1;
    const int kblocks = p.K >> 7;  // K % 128 == 0
    const int nkb = wave < kblocks ? (kblocks - wave + NW - 1) / NW : 0;  
    const int maxkb = (kblocks + NW - 1) / NW;
    const int slotBytes = kDecSlotBytes + (QB ? 64 : 0);
    const int xRowBytes = XLDS ? M * 256 : 0;  // a k-block of the input rows in LDS
    const unsigned regionBytes = (unsigned)maxkb * (unsigned)(xRowBytes + nmat * kDecLdsSlot);
    int8_t *region = smem + (size_t)wave * regionBytes;
    int8_t *slots = region + (size_t)maxkb * xRowBytes;
    const unsigned regionLds = ldsOffset(smem) + (unsigned)wave * regionBytes;
    const unsigned slotsLds = regionLds + (unsigned)(maxkb * xRowBytes);
    const int8_t *wsrc[2];
    {
        const int s0 = p.pair ? 0 : seg, s1 = p.pair ? 1 : seg;
        wsrc[0] = s0 == 0 ? p.w[0] : s0 == 1 ? p.w[1] : p.w[2];
        wsrc[1] = s1 == 0 ? p.w[0] : s1 == 1 ? p.w[1] : p.w[2];
    }
    if (XLDS) {
        // lane l brings 16 bytes of row l >> 4: a k-block of one row is 16 lanes x 16 bytes
        for (int i = 0; i < nkb; i++) {
            const int kb = wave + NW * i;
            if (lane < 16 * M) dmaLoad16(x + (size_t)(lane >> 4) * p.K + kb * 128 + (lane & 15) * 8, regionLds + (unsigned)(i * xRowBytes));
        }
    }
    // the wave's whole share of the weights, one burst: per k-block and matrix 2 KiB and the scales, straight into LDS
    for (int i = 0; i < ((p.ablate & 1) ? 0 : nkb); i++) {
        const int kb = wave + NW * i;
        for (int m = 0; m < nmat; m++) {
            const int8_t *src = wsrc[m] + ((size_t)tile * kblocks + kb) * slotBytes;
            const unsigned dst = slotsLds + (unsigned)(i * nmat + m) * kDecLdsSlot;
            dmaLoad16(src + (size_t)lane * 16, dst);
            dmaLoad16(src + 1024 + (size_t)lane * 16, dst + 1024u);
            if (lane < (QB ? 32 : 16)) dmaLoad4(src + 2048 + (size_t)lane * 4, dst + 2048u);
        }
    }
    v4f acc[2][MR];
#pragma unroll
    for (int m = 0; m < 2; m++) {
#pragma unroll
        for (int mr = 0; mr < MR; mr++) acc[m][mr] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
    }
    // one k-block of one matrix: 32 weights of the lane expanded, four MFMAs per row group
    auto kblock = [&](int i, int m, const v4i (&xp)[4][MR]) {
        const int8_t *slot = slots + (size_t)(i * nmat + m) * kDecLdsSlot;
        const v4i p0 = *(const v4i *)(slot + lane * 16), p1 = *(const v4i *)(slot + 1024 + lane * 16);
        const float sc = *(const float *)(slot + 2048 + c * 4);
        const float bi = QB ? *(const float *)(slot + 2048 + 64 + c * 4) : 0.0f;
        const int dw[8] = {p0[0], p0[1], p0[2], p0[3], p1[0], p1[1], p1[2], p1[3]};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            int o[4];
            expandQ8<QC>(dw[2 * j], sc, bi, p.qlo, p.qhi, &o[0], &o[1]);
            expandQ8<QC>(dw[2 * j + 1], sc, bi, p.qlo, p.qhi, &o[2], &o[3]);
            const v8bf wfrag = __builtin_bit_cast(v8bf, v4i{o[0], o[1], o[2], o[3]});
#pragma unroll
            for (int mr = 0; mr < MR; mr++) {
                acc[m][mr] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wfrag, __builtin_bit_cast(v8bf, xp[j][mr]), acc[m][mr], 0, 0, 0);
            }
        }
    };
    if constexpr (XLDS) {
        const int xrow = (c < M ? c : 0) * 256 + g * 16;  // lanes of rows the input does not have read row 0 (never stored)
        for (int i = 0; i < ((p.ablate & 2) ? 0 : nkb); i++) {
            waitVmcntDyn((p.ablate & 1) ? 0 : (nkb - 1 - i) * 3 * nmat);  // everything up to this k-block has landed
            v4i xp[4][MR];
#pragma unroll
            for (int j = 0; j < 4; j++) xp[j][0] = *(const v4i *)(region + (size_t)i * xRowBytes + xrow + j * 64);
            kblock(i, 0, xp);
            if (nmat > 1) kblock(i, 1, xp);
        }
    } else {
        struct XBuf {
            v4i x[CH][4][MR];
        };
        // Loads only; a k-block the wave does not have and a row beyond M read nothing and feed zeros.
        auto loadChunk = [&](int ch, XBuf &b) {
#pragma unroll
            for (int u = 0; u < CH; u++) {
                const int i = ch * CH + u;
                const int kb = wave + NW * i;
#pragma unroll
                for (int j = 0; j < 4; j++) {
#pragma unroll
                    for (int mr = 0; mr < MR; mr++) {
                        const int row = c + 16 * mr;
                        b.x[u][j][mr] = (i < nkb && row < M) ? *(const v4i *)(x + (size_t)row * p.K + kb * 128 + 32 * j + 8 * g) : v4i{0, 0, 0, 0};
                    }
                }
            }
        };
        auto computeChunk = [&](int ch, const XBuf &b) {
#pragma unroll
            for (int u = 0; u < CH; u++) {
                const int i = ch * CH + u;
                if (i >= nkb) break;
                kblock(i, 0, b.x[u]);
                if (nmat > 1) kblock(i, 1, b.x[u]);
            }
        };
        const int nchunks = (nkb + CH - 1) / CH;
        XBuf b0, b1;
        loadChunk(0, b0);
        waitVmcnt<0>();  // the DMA burst (and the first chunk's rows) has landed; the compiler counts only its own loads
        for (int ch = 0; ch < nchunks; ch += 2) {
            if (ch + 1 < nchunks) loadChunk(ch + 1, b1);
            computeChunk(ch, b0);
            if (ch + 1 < nchunks) {
                if (ch + 2 < nchunks) loadChunk(ch + 2, b0);
                computeChunk(ch + 1, b1);
            }
        }
    }
    // the waves' partial sums meet in LDS: each leaves its own in its own region (its weights are used up)
    asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory");
#pragma unroll
    for (int m = 0; m < 2; m++) {
#pragma unroll
        for (int mr = 0; mr < MR; mr++) {
            if (m < nmat) ((v4f *)region)[(m * MR + mr) * 64 + lane] = acc[m][mr];
        }
    }
    __syncthreads();
    if (wave >= MR) return;
    const int mr = wave;  // this wave finishes row group `wave`
    if (c + 16 * mr >= M) return;
    const int row = row0 + c + 16 * mr;  // as the whole launch counts them
    const int s0 = p.pair ? 0 : seg;
    const int Nseg = s0 == 0 ? p.N[0] : s0 == 1 ? p.N[1] : p.N[2];
    const int n = tile * 16 + 4 * g;
    // what the epilogue reads from memory, issued before the sums are collected
    v4f bias4[2];
#pragma unroll
    for (int m = 0; m < 2; m++) {
        const int sm = p.pair ? m : seg;
        const float *bias = sm == 0 ? p.bias[0] : sm == 1 ? p.bias[1] : p.bias[2];
        bias4[m] = m < nmat ? *(const v4f *)(bias + n) : v4f{0.0f, 0.0f, 0.0f, 0.0f};
    }
    v2i rv = v2i{0, 0};
    if (p.add_mode == 1) rv = *(const v2i *)(p.res + (size_t)row * Nseg + n);
    uint16_t y[2][4];
#pragma unroll
    for (int m = 0; m < 2; m++) {
        if (m >= nmat) break;
        v4f s = v4f{0.0f, 0.0f, 0.0f, 0.0f};
        for (int w = 0; w < NW; w++) {
            const v4f t = ((const v4f *)(smem + (size_t)w * regionBytes))[(m * MR + mr) * 64 + lane];
            s += t;
        }
        const int sm = p.pair ? m : seg;
        uint16_t *out = sm == 0 ? p.out[0] : sm == 1 ? p.out[1] : p.out[2];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const float t0 = s[e] + bias4[m][e];
            y[m][e] = bf16Bits(t0 < p.lo ? p.lo : (t0 > p.hi ? p.hi : t0));
        }
        if (out) {
            *(v2i *)(out + (size_t)row * Nseg + n) = v2i{(int)((uint32_t)y[m][0] | ((uint32_t)y[m][1] << 16)), (int)((uint32_t)y[m][2] | ((uint32_t)y[m][3] << 16))};
        }
    }
    if (p.add_mode == 0) return;
    uint16_t z[4];
    if (p.add_mode == 1) {
        const uint16_t r[4] = {(uint16_t)rv[0], (uint16_t)((uint32_t)rv[0] >> 16), (uint16_t)rv[1], (uint16_t)((uint32_t)rv[1] >> 16)};
#pragma unroll
        for (int e = 0; e < 4; e++) {
            z[e] = p.res_first ? addBf16One(r[e], y[0][e], p.aw0, p.aw1, p.abias, p.alo, p.ahi) : addBf16One(y[0][e], r[e], p.aw0, p.aw1, p.abias, p.alo, p.ahi);
        }
    } else {
#pragma unroll
        for (int e = 0; e < 4; e++) z[e] = addBf16One(y[0][e], y[1][e], p.aw0, p.aw1, p.abias, p.alo, p.ahi);
    }
    *(v2i *)(p.add_out + (size_t)row * Nseg + n) = v2i{(int)((uint32_t)z[0] | ((uint32_t)z[1] << 16)), (int)((uint32_t)z[2] | ((uint32_t)z[3] << 16))};
}

template <int MR, int CH, bool XLDS, bool QB, bool QC>
static hipError_t launchDecLinearT(const DecLinearArgs &a, int tiles, size_t lds, const LaunchCtx &ctx) {
    auto kernel = dec_linear<MR, CH, XLDS, QB, QC>;
    static std::once_flag once;
    static hipError_t configured = hipSuccess;
    std::call_once(once, [&] { configured = hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024); });
    if (configured != hipSuccess) return configured;
    const int groups = (a.M + a.rows_per_group - 1) / a.rows_per_group;
    THIP_ENQUEUE(ctx, kernelLabel("dec_linear", {MR, CH, (int)XLDS, (int)QB, (int)QC, a.pair ? 2 : a.nseg, a.add_mode}), kernel, dim3((unsigned)tiles, (unsigned)groups),
                 dim3((unsigned)a.nwaves * 64), lds, a);
    return hipGetLastError();
}

// LDS a launch needs: every wave's share of the weights, and of the input rows when they come through LDS (the
// partial sums reuse it).
static size_t decLinearLds(int K, int nmat, int xRows, int nwaves) {
    const int kblocks = K / 128, maxkb = (kblocks + nwaves - 1) / nwaves;
    return (size_t)nwaves * maxkb * (size_t)(xRows * 256 + nmat * kDecLdsSlot);
}
// Waves per workgroup: one k-block each where K has between 8 and 16 of them, 16 for a longer K (a wave's
// arithmetic is the launch's critical path: 128 x 16 weights expanded per k-block and matrix).
int decLinearWaves(int K) {
    const int kblocks = K / 128;
    return kblocks < kDecWaves ? kDecWaves : (kblocks > kDecMaxWaves ? kDecMaxWaves : kblocks);
}
constexpr size_t kDecMaxLds = 152 * 1024;
constexpr int kDecLdsRows = 4;  // up to this many input rows may come through LDS

// Workgroups per column tile.  A workgroup streams its rows of the input next to its 16 columns of the weights: with few
// column tiles and many rows (32 rows of K = 6912 are 442 KB per workgroup against 110 KB of weights, on 72 of 256 CUs)
// the rows are the traffic, and sharing them out over several workgroups, each re-reading the weights, spreads it over
// the chip.  As many groups as keep the launch within one workgroup per CU, at least eight rows each.
static int decLinearRowGroups(int M, int tiles, const Tuning *tuning) {
    if (M <= kDecLdsRows) return 1;
    int groups = (tuning && tuning->decTargetGroups > 0 ? tuning->decTargetGroups : 256) / tiles;
    const int most = (M + 7) / 8;
    groups = groups < 1 ? 1 : (groups > most ? most : groups);
    return groups;
}

template <bool QB, bool QC>
static hipError_t launchDecLinearQ(const DecLinearArgs &in, int tiles, const LaunchCtx &ctx) {
    DecLinearArgs a = in;
    const int nmat = a.pair ? 2 : 1;
    a.rows_per_group = a.M;
    if (a.M <= kDecLdsRows) {
        // the input rows through LDS as well, with the most waves whose regions still fit
        for (int nw = a.nwaves; nw >= kDecWaves; nw--) {
            if (decLinearLds(a.K, nmat, a.M, nw) > kDecMaxLds) continue;
            a.nwaves = nw;
            return launchDecLinearT<1, 1, true, QB, QC>(a, tiles, decLinearLds(a.K, nmat, a.M, nw), ctx);
        }
    }
    const int groups = decLinearRowGroups(a.M, tiles, ctx.tuning);
    a.rows_per_group = (a.M + groups - 1) / groups;
    // more workgroups than CUs: eight waves each, so that two of them (at four waves per SIMD) share a CU and the
    // launch is one round of workgroups rather than two (decoder step at 32 tokens 1247 -> 1216 us, at 8 1028 -> 994)
    if ((long long)tiles * groups > 256 && a.nwaves > kDecWaves) a.nwaves = kDecWaves;
    const size_t lds = decLinearLds(a.K, nmat, 0, a.nwaves);
    if (a.rows_per_group <= 16) return launchDecLinearT<1, 2, false, QB, QC>(a, tiles, lds, ctx);
    return launchDecLinearT<2, 1, false, QB, QC>(a, tiles, lds, ctx);
}

hipError_t launchDecLinear(const DecLinearArgs &in, const LaunchCtx &ctx) {
    DecLinearArgs a = in;
    a.nwaves = a.K > 0 ? decLinearWaves(a.K) : kDecWaves;
    if (!a.x || a.M <= 0 || a.M > kDecMaxRows || a.K <= 0 || a.K % 128 != 0 || a.qblock <= 0 || a.qblock % 128 != 0 || a.K % a.qblock != 0) return hipErrorInvalidValue;
    if (a.nseg < 1 || a.nseg > kDecMaxSegments || (a.pair && a.nseg != 2) || (((uintptr_t)a.x) & 15)) return hipErrorInvalidValue;
    if (a.add_mode < 0 || a.add_mode > 2 || (a.add_mode == 1 && (a.nseg != 1 || !a.res)) || (a.add_mode == 2 && !a.pair) || (a.pair && a.add_mode != 2)) return hipErrorInvalidValue;
    if (a.add_mode != 0 && (!a.add_out || (((uintptr_t)a.add_out) & 7) || (a.res && (((uintptr_t)a.res) & 7)))) return hipErrorInvalidValue;
    long long tiles = 0;
    for (int s = 0; s < a.nseg; s++) {
        if (!a.w[s] || !a.bias[s] || a.N[s] <= 0 || a.N[s] % 16 != 0) return hipErrorInvalidValue;
        if ((((uintptr_t)a.w[s]) & 15) || (((uintptr_t)a.bias[s]) & 15) || (((uintptr_t)a.out[s]) & 7)) return hipErrorInvalidValue;
        if (!a.out[s] && a.add_mode == 0) return hipErrorInvalidValue;  // a result nobody receives
        tiles += a.N[s] / 16;
    }
    if (a.pair) {
        if (a.N[0] != a.N[1]) return hipErrorInvalidValue;
        tiles = a.N[0] / 16;
    }
    if (tiles <= 0 || tiles > 65535 || decLinearLds(a.K, a.pair ? 2 : 1, 0, a.nwaves) > kDecMaxLds) return hipErrorInvalidValue;
    const bool clamp = !(a.qlo == -INFINITY && a.qhi == INFINITY);
    const int t = (int)tiles;
    if (ctx.tuning->decAblate) {
        DecLinearArgs b = a;
        b.ablate = ctx.tuning->decAblate;
        return launchDecLinearQ<false, false>(b, t, ctx);
    }
    if (clamp) return a.has_qbias ? launchDecLinearQ<true, true>(a, t, ctx) : launchDecLinearQ<false, true>(a, t, ctx);
    return a.has_qbias ? launchDecLinearQ<true, false>(a, t, ctx) : launchDecLinearQ<false, false>(a, t, ctx);
}

// dec_matmul: a workgroup owns 16 columns (rows of w) of one batch element; its eight waves split K in steps of 32
// (wave, wave + 8, ...), each lane loading 16 bytes of its weight row and of its input row per step; the partial
// sums meet in LDS.  A wave's loads of up to ST steps are all issued before the first MFMA.
template <int MR, int ST>
__global__ __launch_bounds__(kDecWaves * 64) void dec_matmul(DecMatmulArgs p) {
    __shared__ v4f red[kDecWaves][MR][64];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int c = lane & 15, g = lane >> 4;
    const int n0 = (int)blockIdx.x * 16, b = (int)blockIdx.y;
    const uint16_t *a = p.a + (size_t)b * p.a_stride, *w = p.w + (size_t)b * p.w_stride;
    const int steps = (p.K + 31) >> 5;
    const int nrow = n0 + c < p.N ? n0 + c : p.N - 1;  // clamped columns are never stored
    v4f acc[MR];
#pragma unroll
    for (int mr = 0; mr < MR; mr++) acc[mr] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
    for (int s0 = wave; s0 < steps; s0 += kDecWaves * ST) {
        v4i wv[ST], xv[ST][MR];
#pragma unroll
        for (int u = 0; u < ST; u++) {
            const int k = (s0 + kDecWaves * u) * 32 + 8 * g;
            const bool in = k < p.K;  // K % 8 == 0: a piece lies inside K or outside
            wv[u] = in ? *(const v4i *)(w + (size_t)nrow * p.K + k) : v4i{0, 0, 0, 0};
#pragma unroll
            for (int mr = 0; mr < MR; mr++) {
                const int row = c + 16 * mr;
                xv[u][mr] = (in && row < p.M) ? *(const v4i *)(a + (size_t)row * p.K + k) : v4i{0, 0, 0, 0};
            }
        }
#pragma unroll
        for (int u = 0; u < ST; u++) {
#pragma unroll
            for (int mr = 0; mr < MR; mr++) {
                acc[mr] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, wv[u]), __builtin_bit_cast(v8bf, xv[u][mr]), acc[mr], 0, 0, 0);
            }
        }
    }
#pragma unroll
    for (int mr = 0; mr < MR; mr++) red[wave][mr][lane] = acc[mr];
    __syncthreads();
    if (wave >= MR) return;
    const int mr = wave, row = c + 16 * mr;
    if (row >= p.M) return;
    v4f s = v4f{0.0f, 0.0f, 0.0f, 0.0f};
    for (int wv = 0; wv < kDecWaves; wv++) s += red[wv][mr][lane];
    const int n = n0 + 4 * g;
    uint16_t *out = p.out + (size_t)b * p.out_stride + (size_t)row * p.N;
    uint16_t y[4];
#pragma unroll
    for (int e = 0; e < 4; e++) {
        const float t0 = s[e] + p.bias;
        y[e] = bf16Bits(t0 < p.lo ? p.lo : (t0 > p.hi ? p.hi : t0));
    }
    if ((p.N & 3) == 0 && n + 3 < p.N) {
        *(v2i *)(out + n) = v2i{(int)((uint32_t)y[0] | ((uint32_t)y[1] << 16)), (int)((uint32_t)y[2] | ((uint32_t)y[3] << 16))};
    } else {
#pragma unroll
        for (int e = 0; e < 4; e++) {
            if (n + e < p.N) out[n + e] = y[e];
        }
    }
}

hipError_t launchDecMatmul(const DecMatmulArgs &a, const LaunchCtx &ctx) {
    if (!a.a || !a.w || !a.out || a.B <= 0 || a.B > 65535 || a.M <= 0 || a.M > kDecMaxRows || a.K <= 0 || a.K % 8 != 0 || a.N <= 0) return hipErrorInvalidValue;
    if (a.a_stride < 0 || a.w_stride < 0 || a.out_stride < 0 || a.a_stride % 8 != 0 || a.w_stride % 8 != 0) return hipErrorInvalidValue;
    if (((((uintptr_t)a.a) | ((uintptr_t)a.w)) & 15) || (((uintptr_t)a.out) & (a.N % 4 == 0 ? 7 : 1)) || (a.N % 4 == 0 && a.out_stride % 4 != 0)) return hipErrorInvalidValue;
    const long long tiles = ((long long)a.N + 15) / 16;
    if (tiles > 0x7fffffffLL) return hipErrorInvalidValue;
    const dim3 grid((unsigned)tiles, (unsigned)a.B);
    // steps of 32 per wave: up to four are one round of loads
    const int perWave = ((a.K + 31) / 32 + kDecWaves - 1) / kDecWaves;
    if (a.M <= 16) {
        if (perWave <= 1) THIP_ENQUEUE(ctx, "dec_matmul<1,1>", (dec_matmul<1, 1>), grid, dim3(kDecWaves * 64), 0, a);
        else if (perWave <= 2) THIP_ENQUEUE(ctx, "dec_matmul<1,2>", (dec_matmul<1, 2>), grid, dim3(kDecWaves * 64), 0, a);
        else THIP_ENQUEUE(ctx, "dec_matmul<1,4>", (dec_matmul<1, 4>), grid, dim3(kDecWaves * 64), 0, a);
    } else {
        if (perWave <= 1) THIP_ENQUEUE(ctx, "dec_matmul<2,1>", (dec_matmul<2, 1>), grid, dim3(kDecWaves * 64), 0, a);
        else if (perWave <= 2) THIP_ENQUEUE(ctx, "dec_matmul<2,2>", (dec_matmul<2, 2>), grid, dim3(kDecWaves * 64), 0, a);
        else THIP_ENQUEUE(ctx, "dec_matmul<2,4>", (dec_matmul<2, 4>), grid, dim3(kDecWaves * 64), 0, a);
    }
    return hipGetLastError();
}

}  // namespace thip
