// Device-side services of the library that are not ops: the static scratch array, the MFMA-rate and streaming-rate
// calibration kernels, and the tuning switches read from the environment.
#include "thip_kernels_common.h"

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

// ---------------------------------------------------------------------------
// Calibration: what a kernel with next to no arithmetic takes to move a given number of bytes, i.e. the floor under
// every bandwidth-bound op of that traffic shape on this GPU.  RD 16-byte reads per 16-byte write and lane (reads of
// RD planes of one buffer, one xor per extra read).  A family, because the floor must be the best a copy can do, not
// one arbitrary copy: U 16-byte items per thread whose loads are all issued before the first store (1, 2, 4, 8);
// a grid of one item group per thread, or a persistent grid (every CU full, grid-stride loop); default or non-temporal
// cache policy.  measureStreamRate times all of them and reports the fastest.
// ---------------------------------------------------------------------------
template <int RD, int U, bool PERSIST, bool NT>
__global__ __launch_bounds__(256) void stream_floor(const v4i *__restrict__ in, v4i *__restrict__ out, size_t items) {
    const size_t stride = PERSIST ? (size_t)gridDim.x * 256 * U : items + (size_t)256 * U;  // one pass unless persistent
    for (size_t base = (size_t)blockIdx.x * 256 * U; base < items; base += stride) {
        v4i v[U][RD];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const size_t i = base + (size_t)u * 256 + threadIdx.x;  // a wave's loads cover 1 KiB in a row
#pragma unroll
            for (int r = 0; r < RD; r++) {
                if (i < items) v[u][r] = NT ? __builtin_nontemporal_load(in + (size_t)r * items + i) : in[(size_t)r * items + i];
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            const size_t i = base + (size_t)u * 256 + threadIdx.x;
            if (i >= items) continue;
            v4i m = v[u][0];
#pragma unroll
            for (int r = 1; r < RD; r++) {
                m[0] ^= v[u][r][0];
                m[1] ^= v[u][r][1];
                m[2] ^= v[u][r][2];
                m[3] ^= v[u][r][3];
            }
            if (NT) __builtin_nontemporal_store(m, out + i);
            else out[i] = m;
        }
    }
}

struct StreamVariant {
    int u, persist, nt;
};

template <int RD, int U, bool PERSIST, bool NT>
static void launchStreamFloor(const v4i *in, v4i *out, size_t items, int cus, hipStream_t stream) {
    const size_t groups = (items + (size_t)256 * U - 1) / ((size_t)256 * U);
    const size_t resident = (size_t)cus * 8;  // eight workgroups of four waves fill a CU's wave slots
    const unsigned blocks = (unsigned)(PERSIST && groups > resident ? resident : groups);
    hipLaunchKernelGGL((stream_floor<RD, U, PERSIST, NT>), dim3(blocks), dim3(256), 0, stream, in, out, items);
}

template <int RD>
static void launchStreamFloorRd(const StreamVariant &v, const v4i *in, v4i *out, size_t items, int cus, hipStream_t stream) {
#define THIP_STREAM_CASE(U)                                                                                   \
    if (v.u == U) {                                                                                           \
        if (v.persist) {                                                                                      \
            if (v.nt) launchStreamFloor<RD, U, true, true>(in, out, items, cus, stream);                      \
            else launchStreamFloor<RD, U, true, false>(in, out, items, cus, stream);                          \
        } else {                                                                                              \
            if (v.nt) launchStreamFloor<RD, U, false, true>(in, out, items, cus, stream);                     \
            else launchStreamFloor<RD, U, false, false>(in, out, items, cus, stream);                         \
        }                                                                                                     \
        return;                                                                                               \
    }
    THIP_STREAM_CASE(1)
    THIP_STREAM_CASE(2)
    THIP_STREAM_CASE(4)
    THIP_STREAM_CASE(8)
#undef THIP_STREAM_CASE
}

hipError_t measureStreamRate(int readsPerWrite, size_t writeBytes, int cold, hipStream_t stream, double *outMicroseconds, char *outVariant, size_t variantCapacity) {
    if ((readsPerWrite != 1 && readsPerWrite != 2 && readsPerWrite != 4) || writeBytes < 4096 || writeBytes % 16 != 0 || writeBytes > (1ull << 31) ||
        !outMicroseconds) {
        return hipErrorInvalidValue;
    }
    int device = 0, cus = 0;
    hipError_t err = hipGetDevice(&device);
    if (err == hipSuccess) err = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device);
    if (err != hipSuccess) return err;
    const size_t items = writeBytes / 16, perSet = writeBytes * (size_t)(readsPerWrite + 1);
    // cold: dispatch i works on buffer set i mod n, the sets together twice the size of the 256 MiB last-level cache
    int sets = cold ? (int)((512ull << 20) / perSet) + 1 : 1;
    sets = sets < (cold ? 2 : 1) ? 2 : (sets > 160 ? 160 : sets);
    std::vector<v4i *> in((size_t)sets, nullptr), out((size_t)sets, nullptr);
    hipEvent_t e0 = nullptr, e1 = nullptr;
    for (int s = 0; s < sets && err == hipSuccess; s++) {
        err = hipMalloc((void **)&in[(size_t)s], writeBytes * (size_t)readsPerWrite);
        if (err == hipSuccess) err = hipMalloc((void **)&out[(size_t)s], writeBytes);
        if (err == hipSuccess) err = hipMemsetAsync(in[(size_t)s], s + 1, writeBytes * (size_t)readsPerWrite, stream);
    }
    auto launch = [&](const StreamVariant &v, int s) {
        if (readsPerWrite == 1) launchStreamFloorRd<1>(v, in[(size_t)s], out[(size_t)s], items, cus, stream);
        else if (readsPerWrite == 2) launchStreamFloorRd<2>(v, in[(size_t)s], out[(size_t)s], items, cus, stream);
        else launchStreamFloorRd<4>(v, in[(size_t)s], out[(size_t)s], items, cus, stream);
    };
    if (err == hipSuccess) err = hipEventCreate(&e0);
    if (err == hipSuccess) err = hipEventCreate(&e1);
    double best = 0.0;
    StreamVariant bestVariant{1, 0, 0};
    if (err == hipSuccess) {
        for (int s = 0; s < sets; s++) launch(bestVariant, s);  // first touch
        const int iterations = sets * 2 > 24 ? sets * 2 : 24;
        for (int u = 1; u <= 8 && err == hipSuccess; u *= 2) {
            if (readsPerWrite * u > 16) continue;  // more than 64 registers of loads in flight per thread gain nothing
            for (int mode = 0; mode < 4 && err == hipSuccess; mode++) {
                const StreamVariant v{u, mode & 1, mode >> 1};
                err = hipEventRecord(e0, stream);
                for (int i = 0; i < iterations; i++) launch(v, i % sets);
                if (err == hipSuccess) err = hipGetLastError();
                if (err == hipSuccess) err = hipEventRecord(e1, stream);
                if (err == hipSuccess) err = hipEventSynchronize(e1);
                float ms = 0.f;
                if (err == hipSuccess) err = hipEventElapsedTime(&ms, e0, e1);
                const double us = (double)ms * 1e3 / iterations;
                if (err == hipSuccess && (best == 0.0 || us < best)) {
                    best = us;
                    bestVariant = v;
                }
            }
        }
        if (err == hipSuccess) {
            *outMicroseconds = best;
            if (outVariant && variantCapacity) {
                snprintf(outVariant, variantCapacity, "stream_floor<%d,%d,%d,%d>", readsPerWrite, bestVariant.u, bestVariant.persist, bestVariant.nt);
            }
        }
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
    if (const char *v = getenv("THIP_DEC_ABLATE")) t.decAblate = atoi(v);
    if (const char *v = getenv("THIP_DEC_TARGET_WORKGROUPS")) t.decTargetGroups = atoi(v);
    return t;
}

}  // namespace thip
