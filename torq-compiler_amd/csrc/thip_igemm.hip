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
#include "thip_kernels_common.h"

namespace thip {

// ---------------------------------------------------------------------------
// Epilogue shared by the MFMA kernels.  The accumulators come from MFMAs that took the weights as
// the row operand: register r of lane l of tile (j, i) holds
// C[m = 32 i + (l & 31)][n = 32 j + 8 (r / 4) + 4 (l >> 5) + (r & 3)], four consecutive output
// channels per register group.  `smem` is the kernel's LDS, free by now, of at least
// igemmEpilogueLds<...>() bytes; myBias / myScale are the (bias, scale) of channel n0 + threadIdx.x.
// ---------------------------------------------------------------------------

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

}  // namespace thip
