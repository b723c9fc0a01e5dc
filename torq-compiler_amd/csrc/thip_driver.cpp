// Run side: device, executable and dispatch.
//
// The shape of this file follows the reference's HAL driver for this path:
//   thip_executable_create  <- iree_hal_torq_native_executable_create
//                              (runtime/driver/native_executable.cc:41-108): copy the
//                              program blob and the executable constants, build the
//                              executor object, initialise it (version / target gate,
//                              runtime/driver/TorqExecutable.cc:655-752).
//   thip_executable_run     <- iree_hal_torq_native_executable_run (:180-192) ->
//                              TorqExecutable::executeDispatch
//                              (runtime/driver/TorqExecutable.cc:1025-1125): lock,
//                              write inputs, walk the action list, read outputs.
// Instead of NSS programs on an NPU the action list is a list of kernel
// records, each launched on the executable's HIP stream.
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <errno.h>
#include <sys/stat.h>

#include <chrono>
#include <mutex>
#include <new>
#include <string>
#include <thread>
#include <vector>

#include "thip_descriptor.h"
#include "thip_kernels.h"
#include "thip_status.h"
#include "thip_validate.h"

using namespace thip;

struct thip_device_t {
    int ordinal = 0;
    std::string arch;
    std::mutex logMutex;
    FILE *eventLog = nullptr;
    std::chrono::steady_clock::time_point t0 = std::chrono::steady_clock::now();
    uint8_t *staticScratch = nullptr;    // this GPU's copy of the library's scratch array (kStaticScratchBytes)
    // dump directories (empty: off): bindings of every blocking dispatch / every buffer a kernel record wrote
    std::string dumpIoDir, dumpBuffersDir;
};

struct thip_executable_t {
    thip_device_t *device = nullptr;
    std::vector<uint8_t> blob;           // private copy of the descriptor
    std::vector<uint32_t> constants;     // executable-level constants (copied)
    DescHeader header;
    const DescOp *ops = nullptr;
    const DescBinding *bindings = nullptr;
    const DescTemp *temps = nullptr;
    const DescConst *consts = nullptr;
    uint8_t *constData = nullptr;        // device copy of the constant segment
    std::vector<uint8_t *> tempPtrs;     // device intermediates
    std::vector<uint8_t *> staging;      // device staging of host bindings
    hipStream_t stream = nullptr;
    hipEvent_t evStart = nullptr, evStop = nullptr, evDone = nullptr;
    // A wait for the GPU gives up after this long (the reference turns a wait that exceeds its timeout into
    // IREE_STATUS_INTERNAL, runtime/torq_hw/src/TorqHw.cpp:172-186).  <= 0: no limit.
    int64_t waitTimeoutMs = 120000;
    bool abandoned = false;              // a wait timed out: work may still be running, the executable is unusable
    std::mutex mutex;                    // one dispatch at a time
    // Multi-kernel programs on device bindings are replayed as a HIP graph: the first dispatch on a
    // set of binding pointers runs eagerly, the second is captured, later ones are one graph launch.
    std::vector<uint8_t *> seenPtrs;     // binding pointers of the previous device dispatch
    std::vector<uint8_t *> graphPtrs;    // binding pointers the instantiated graph was captured with
    hipGraph_t graph = nullptr;
    hipGraphExec_t graphExec = nullptr;
    bool graphsDisabled = false;
    uint64_t invocation = 0;             // dispatches so far (the event log's invocation_id)
    Tuning tuning;                       // the environment's switches as they were when the executable was created
    std::vector<std::string> kernelNames;  // per record: the kernel its launcher resolved at creation
    // thip_executable_enqueue_noalloc: where each record's scratch (a K-split workspace) sits in the static array,
    // and the program's total
    std::vector<uint64_t> scratchOffset;
    uint64_t scratchBytes = 0;
};

static thip_status_t hipFail(hipError_t e, const char *what) {
    const thip_status_t code = e == hipErrorOutOfMemory ? THIP_RESOURCE_EXHAUSTED : THIP_INTERNAL;
    return fail(code, "%s: %s", what, hipGetErrorString(e));
}

#define THIP_HIP(call, what)                          \
    do {                                              \
        hipError_t e_ = (call);                       \
        if (e_ != hipSuccess) return hipFail(e_, what); \
    } while (0)

// The kernel family of a record (error messages before the launcher has named the instantiation).
static const char *opKernelName(const DescOp &op) {
    switch (op.kind) {
    case kKindTranspose: return "transpose_i8";
    case kKindIgemm: return igemmTile(op.variant).name;
    case kKindFcSkinny: return "fc_skinny";
    case kKindDepthwise: return op.variant == kDepthwiseDot4Rows ? "depthwise3x3_dot4_i8" : "depthwise_i8";
    case kKindMaxPool: return "maxpool_i8";
    case kKindAvgPool: return "avgpool_i8";
    case kKindAdd: return "add_i8";
    case kKindFcBf16: return "fc_bf16";
    case kKindAddBf16: return "add_bf16";
    case kKindIm2colBf16: return "im2col_bf16";
    case kKindDepthwiseBf16: return "depthwise_bf16";
    case kKindAvgPoolBf16: return "avgpool_bf16";
    case kKindExpandWeights: return "expand_weights_bf16";
    case kKindEltwise: return "eltwise_int";
    case kKindDecLinear: return "dec_linear";
    case kKindDecMatmul: return "dec_matmul";
    default: return "unknown";
    }
}

// One row of the event log, in the reference's runtime CSV columns (doc/user-manual/profiling.md:53-63, written by
// runtime/torq_hw/src/TorqEventLog.cpp:48,97-101): dispatch_name, invocation_id, action_id, timestamp_us, event
// (an EventType name + _BEGIN / _END), plus one column of this backend's own: the kernel of a launch row.
static void logEvent(const thip_executable_t *e, uint64_t invocation, int32_t action, const char *event, const char *phase, const char *kernel) {
    thip_device_t *d = e->device;
    if (!d->eventLog) return;
    std::lock_guard<std::mutex> lock(d->logMutex);
    const auto us = std::chrono::duration_cast<std::chrono::microseconds>(std::chrono::steady_clock::now() - d->t0).count();
    fprintf(d->eventLog, "%s,%llu,%d,%lld,%s_%s,%s\n", e->header.name, (unsigned long long)invocation, action, (long long)us, event, phase, kernel);
}

// Resolves an operand reference against the buffers of this dispatch.
static uint8_t *resolve(const thip_executable_t *e, const DescRef &r, uint8_t *const *bindingPtrs) {
    switch (r.space) {
    case kSpaceBinding: return bindingPtrs[r.index] + r.offset;
    case kSpaceTemp: return e->tempPtrs[r.index] + r.offset;
    case kSpaceConst: return e->constData + e->consts[r.index].offset + r.offset;
    default: return nullptr;
    }
}

// Launches record i, or (ctx.name set) only asks its launcher which kernel it takes for these operands.
// `scratch` (or null): the static scratch array, which then stands in for the record's workspace intermediate.
static thip_status_t launchOp(thip_executable_t *e, uint32_t i, uint8_t *const *bp, const LaunchCtx &ctx, uint8_t *scratch = nullptr) {
    const DescOp &op = e->ops[i];
    const Requant rq{op.shift, op.output_zp, op.output_min, op.output_max, op.pre_shift, op.t0_clamp};
    hipError_t err = hipSuccess;
    switch (op.kind) {
    case kKindTranspose: {
        TransposeArgs a{(const int8_t *)resolve(e, op.in0, bp), (int8_t *)resolve(e, op.out, bp), op.TB, op.TR, op.TS, op.gran == 2 ? 2 : 1, op.TP ? op.TP : op.TR};
        err = launchTranspose(a, ctx);
        break;
    }
    case kKindIgemm: {
        IgemmArgs a;
        memset(&a, 0, sizeof(a));
        a.A = (const int8_t *)resolve(e, op.in0, bp);
        a.Bp = (const int8_t *)resolve(e, op.weights, bp);
        a.bias = (const int32_t *)resolve(e, op.bias, bp);
        a.scale = (const int32_t *)resolve(e, op.scale, bp);
        a.ktab = (const uint32_t *)resolve(e, op.table, bp);
        a.out = resolve(e, op.out, bp);
        a.M = op.M; a.N = op.Nn; a.K = op.K; a.Kp = op.Kp; a.Np = op.Np;
        a.H = op.H; a.W = op.W; a.C = op.C; a.OH = op.OH; a.OW = op.OW;
        a.SH = op.SH; a.SW = op.SW; a.PT = op.PT; a.PL = op.PL;
        a.KH = op.KH; a.KW = op.KW;
        a.input_zp = op.input_zp;
        a.out_dtype = op.out_dtype;
        a.a_bytes = (int64_t)op.N * op.H * op.W * op.C;
        a.loader = op.loader;
        a.gran = op.gran;
        a.rq = rq;
        if (op.in1.space != kSpaceNone) {
            ResidualAddParams ap;
            memcpy(&ap, e->blob.data() + e->header.data_offset + e->consts[op.table.index].offset + op.table.offset, sizeof(ap));
            a.skip = (const int8_t *)resolve(e, op.in1, bp);
            a.add_skip_first = ap.other_first;
            a.add_w0 = ap.w0; a.add_w1 = ap.w1; a.add_bias = ap.bias; a.add_scale = ap.scale;
            a.arq = Requant{ap.shift, ap.output_zp, ap.output_min, ap.output_max, 0, 0};
        }
        err = launchIgemm(a, op.variant, ctx);
        break;
    }
    case kKindFcSkinny: {
        FcSkinnyArgs a{(const int8_t *)resolve(e, op.in0, bp), (const int8_t *)resolve(e, op.weights, bp),
                       (const int32_t *)resolve(e, op.bias, bp), (const int32_t *)resolve(e, op.scale, bp),
                       resolve(e, op.out, bp), op.M, op.Nn, op.K, op.out_dtype, rq};
        err = launchFcSkinny(a, ctx);
        break;
    }
    case kKindDepthwise: {
        DepthwiseArgs a{(const int8_t *)resolve(e, op.in0, bp), (const int8_t *)resolve(e, op.weights, bp),
                        (const int32_t *)resolve(e, op.bias, bp), (const int32_t *)resolve(e, op.scale, bp),
                        (int8_t *)resolve(e, op.out, bp), op.N, op.H, op.W, op.C, op.OH, op.OW, op.KH, op.KW,
                        op.SH, op.SW, op.PT, op.PL, op.input_zp, op.variant, rq};
        err = launchDepthwise(a, ctx);
        break;
    }
    case kKindMaxPool: {
        MaxPoolArgs a{(const int8_t *)resolve(e, op.in0, bp), (int8_t *)resolve(e, op.out, bp), op.N, op.H, op.W, op.C,
                      op.OH, op.OW, op.KH, op.KW, op.SH, op.SW, op.PT, op.PL, op.input_zp, op.output_min, op.output_max};
        err = launchMaxPool(a, ctx);
        break;
    }
    case kKindAvgPool: {
        AvgPoolArgs a{(const int8_t *)resolve(e, op.in0, bp), (int8_t *)resolve(e, op.out, bp), op.N, op.H * op.W, op.C,
                      op.w0, op.bias0, op.scale0, rq};
        err = launchAvgPool(a, ctx);
        break;
    }
    case kKindAdd: {
        AddArgs a{(const int8_t *)resolve(e, op.in0, bp), (const int8_t *)resolve(e, op.in1, bp),
                  (int8_t *)resolve(e, op.out, bp), (int64_t)op.C, op.w0, op.w1, op.bias0, op.scale0, rq};
        err = launchAdd(a, ctx);
        break;
    }
    case kKindIm2colBf16: {
        Im2colBf16Args a{(const uint16_t *)resolve(e, op.in0, bp), (uint16_t *)resolve(e, op.out, bp), op.N, op.H, op.W, op.C,
                         op.OH, op.OW, op.KH, op.KW, op.SH, op.SW, op.PT, op.PL, op.Kp};
        err = launchIm2colBf16(a, ctx);
        break;
    }
    case kKindDepthwiseBf16: {
        float lo, hi;
        memcpy(&lo, &op.output_min, 4);
        memcpy(&hi, &op.output_max, 4);
        DepthwiseBf16Args a{(const uint16_t *)resolve(e, op.in0, bp), (const uint16_t *)resolve(e, op.weights, bp),
                            (const float *)resolve(e, op.bias, bp), (uint16_t *)resolve(e, op.out, bp), op.N, op.H, op.W, op.C,
                            op.OH, op.OW, op.KH, op.KW, op.SH, op.SW, op.PT, op.PL, lo, hi};
        err = launchDepthwiseBf16(a, ctx);
        break;
    }
    case kKindAddBf16: {
        auto asFloat = [](int32_t bits) {
            float f;
            memcpy(&f, &bits, 4);
            return f;
        };
        AddBf16Args a{(const uint16_t *)resolve(e, op.in0, bp), (const uint16_t *)resolve(e, op.in1, bp),
                      (uint16_t *)resolve(e, op.out, bp), (int64_t)op.C, asFloat(op.w0 << 16), asFloat(op.w1 << 16),
                      asFloat(op.bias0), asFloat(op.output_min), asFloat(op.output_max)};
        err = launchAddBf16(a, ctx);
        break;
    }
    case kKindFcBf16: {
        float lo, hi;
        memcpy(&lo, &op.output_min, 4);
        memcpy(&hi, &op.output_max, 4);
        FcBf16Args a{(const uint16_t *)resolve(e, op.in0, bp), (const uint16_t *)resolve(e, op.weights, bp),
                     (const float *)resolve(e, op.bias, bp), (uint16_t *)resolve(e, op.out, bp), op.M, op.K, op.Nn, lo, hi,
                     op.w0 > 1 ? op.w0 : 1, op.w0 > 1 ? (void *)(scratch ? scratch + e->scratchOffset[i] : resolve(e, op.in1, bp)) : nullptr, (int32_t)op.loader,
                     nullptr, nullptr, 0, 0, 0.0f, 0.0f};
        if (op.loader == 2) {
            a.qscale = (const uint16_t *)resolve(e, op.scale, bp);
            a.qbias = (const float *)resolve(e, op.table, bp);
            a.qblock = (int32_t)op.gran;
            a.qcols = op.Np;
            memcpy(&a.qlo, &op.bias0, 4);
            memcpy(&a.qhi, &op.scale0, 4);
        }
        err = launchFcBf16(a, ctx);
        break;
    }
    case kKindAvgPoolBf16: {
        AvgPoolBf16Args a{(const uint16_t *)resolve(e, op.in0, bp), (uint16_t *)resolve(e, op.out, bp), op.N, op.H * op.W, op.C,
                          0.0f, 0.0f, 0.0f, 0.0f};
        const uint32_t wbits = (uint32_t)op.w0 << 16;
        memcpy(&a.weight, &wbits, 4);
        memcpy(&a.bias, &op.bias0, 4);
        memcpy(&a.lo, &op.output_min, 4);
        memcpy(&a.hi, &op.output_max, 4);
        err = launchAvgPoolBf16(a, ctx);
        break;
    }
    case kKindEltwise: {
        EltwiseArgs a{resolve(e, op.in0, bp), eltwiseTwoInputs((int32_t)op.variant) ? resolve(e, op.in1, bp) : nullptr, resolve(e, op.out, bp), (int64_t)op.C,
                      (int32_t)op.variant, (int32_t)op.gran, op.out_dtype == THIP_DTYPE_I8 ? 1 : op.out_dtype == THIP_DTYPE_I16 ? 2 : 4, op.w1,
                      op.w0, op.bias0, op.scale0, op.output_min, op.output_max, rq};
        err = launchEltwise(a, ctx);
        break;
    }
    case kKindExpandWeights: {
        ExpandWeightsArgs a{(const int8_t *)resolve(e, op.in0, bp), (const uint16_t *)resolve(e, op.scale, bp),
                            (const float *)resolve(e, op.bias, bp), (uint16_t *)resolve(e, op.out, bp), op.K, op.Nn,
                            (int32_t)op.gran, op.Np, 0.0f, 0.0f};
        memcpy(&a.lo, &op.output_min, 4);
        memcpy(&a.hi, &op.output_max, 4);
        err = launchExpandWeights(a, ctx);
        break;
    }
    case kKindDecLinear: {
        DecLinearExt x;
        memcpy(&x, e->blob.data() + e->header.data_offset + e->consts[op.table.index].offset + op.table.offset, sizeof(x));  // the host copy
        DecLinearArgs a;
        memset(&a, 0, sizeof(a));
        a.x = (const uint16_t *)resolve(e, op.in0, bp);
        a.M = op.M; a.K = op.K; a.qblock = (int32_t)op.gran;
        a.nseg = op.w0;
        a.pair = (op.w1 & kDecPair) ? 1 : 0;
        a.has_qbias = x.has_qbias;
        for (int m = 0; m < op.w0 && m < kDecMaxSegments; m++) {
            a.w[m] = (const int8_t *)resolve(e, x.weights[m], bp);
            a.bias[m] = (const float *)resolve(e, x.bias[m], bp);
            a.out[m] = (uint16_t *)resolve(e, x.out[m], bp);
            a.N[m] = x.N[m];
        }
        memcpy(&a.lo, &op.output_min, 4);
        memcpy(&a.hi, &op.output_max, 4);
        memcpy(&a.qlo, &op.bias0, 4);
        memcpy(&a.qhi, &op.scale0, 4);
        a.add_mode = (op.w1 & kDecAddResidual) ? 1 : (op.w1 & kDecAddPair) ? 2 : 0;
        a.res_first = (op.w1 & kDecResFirst) ? 1 : 0;
        if (a.add_mode) {
            a.res = (const uint16_t *)resolve(e, x.res, bp);
            a.add_out = (uint16_t *)resolve(e, x.add_out, bp);
            const uint32_t w0 = (uint32_t)x.aw0 << 16, w1 = (uint32_t)x.aw1 << 16;
            memcpy(&a.aw0, &w0, 4);
            memcpy(&a.aw1, &w1, 4);
            memcpy(&a.abias, &x.abias, 4);
            memcpy(&a.alo, &x.alo, 4);
            memcpy(&a.ahi, &x.ahi, 4);
        }
        err = launchDecLinear(a, ctx);
        break;
    }
    case kKindDecMatmul: {
        DecMatmulArgs a{(const uint16_t *)resolve(e, op.in0, bp), (const uint16_t *)resolve(e, op.weights, bp), (uint16_t *)resolve(e, op.out, bp),
                        op.TB, op.M, op.K, op.Nn, op.w0 ? 0 : (int64_t)op.M * op.K, op.w1 ? 0 : (int64_t)op.Nn * op.K, (int64_t)op.M * op.Nn, 0.0f, 0.0f, 0.0f};
        memcpy(&a.bias, &op.bias0, 4);
        memcpy(&a.lo, &op.output_min, 4);
        memcpy(&a.hi, &op.output_max, 4);
        err = launchDecMatmul(a, ctx);
        break;
    }
    default: return fail(THIP_INTERNAL, "op %u has unknown kind %u", i, op.kind);
    }
    if (err != hipSuccess) {
        return fail(THIP_INTERNAL, "op %u (%s): launch failed: %s", i, ctx.name ? opKernelName(op) : e->kernelNames[i].c_str(), hipGetErrorString(err));
    }
    return THIP_OK;
}

// Validates the dispatch state against the binding table.  Mirrors the checks of
// iree_hal_torq_command_buffer_dispatch (runtime/driver/torq_command_buffer.c:453-494).
static thip_status_t checkState(const thip_executable_t *e, const thip_dispatch_state_t *st, bool deviceOnly) {
    if (!st) return fail(THIP_INVALID_ARGUMENT, "dispatch state is NULL");
    if (st->constant_count > 0 && !st->constants) return fail(THIP_FAILED_PRECONDITION, "constants pointer is NULL");
    if (st->binding_count < e->header.binding_count) {
        return fail(THIP_INVALID_ARGUMENT, "dispatch carries %u bindings, the executable uses %u", st->binding_count, e->header.binding_count);
    }
    if (e->header.binding_count > 0 && (!st->binding_ptrs || !st->binding_lengths)) {
        return fail(THIP_FAILED_PRECONDITION, "binding tables are NULL");
    }
    for (uint32_t i = 0; i < e->header.binding_count; i++) {
        if (e->bindings[i].flags == 0) continue;  // declared but unused
        if (!st->binding_ptrs[i]) {
            return fail(THIP_FAILED_PRECONDITION, "required binding %u is NULL; all bindings must have a valid pointer", i);
        }
        if (st->binding_lengths[i] < e->bindings[i].size) {
            return fail(THIP_OUT_OF_RANGE, "binding %u is %zu bytes, the executable touches %llu", i, st->binding_lengths[i],
                        (unsigned long long)e->bindings[i].size);
        }
        const bool isDevice = st->binding_flags && (st->binding_flags[i] & THIP_BINDING_DEVICE);
        if (deviceOnly && !isDevice) return fail(THIP_FAILED_PRECONDITION, "binding %u is a host pointer; this entry point takes device bindings only", i);
        if (isDevice && ((uintptr_t)st->binding_ptrs[i] & 15) != 0) {
            return fail(THIP_FAILED_PRECONDITION, "device binding %u is not 16-byte aligned", i);
        }
    }
    return THIP_OK;
}

// Waits for everything enqueued on the executable's stream, at most waitTimeoutMs.  On expiry the executable is
// marked abandoned (kernels may still be running on its buffers: later calls are refused and destruction does not
// free them) and THIP_INTERNAL comes back; the process goes on and can report the failure.
static thip_status_t waitBounded(thip_executable_t *e, const char *what) {
    if (e->waitTimeoutMs <= 0) {
        THIP_HIP(hipStreamSynchronize(e->stream), what);
        return THIP_OK;
    }
    THIP_HIP(hipEventRecord(e->evDone, e->stream), "hipEventRecord");
    const auto start = std::chrono::steady_clock::now();
    const auto deadline = start + std::chrono::milliseconds(e->waitTimeoutMs);
    for (;;) {
        const hipError_t q = hipEventQuery(e->evDone);
        if (q == hipSuccess) return THIP_OK;
        if (q != hipErrorNotReady) return hipFail(q, what);
        (void)hipGetLastError();  // not-ready is no error
        const auto now = std::chrono::steady_clock::now();
        if (now >= deadline) {
            e->abandoned = true;
            return fail(THIP_INTERNAL, "%s: the GPU did not finish within %lld ms; the executable is abandoned", what, (long long)e->waitTimeoutMs);
        }
        // poll hard at first (dispatches are microseconds to a few milliseconds long, and a sleep of any length costs
        // some 100 us before the thread runs again), then back off
        if (now - start > std::chrono::microseconds(3000)) std::this_thread::sleep_for(std::chrono::microseconds(50));
    }
}

static bool makeDirs(const std::string &path) {
    for (size_t i = 1; i <= path.size(); i++) {
        if (i == path.size() || path[i] == '/') {
            const std::string part = path.substr(0, i);
            if (mkdir(part.c_str(), 0777) != 0 && errno != EEXIST) return false;
        }
    }
    return true;
}

// Raw bytes of a binding, named as the reference names them (runtime/driver/TorqDump.cc:329-339):
// <dir>/<executable>/npu.{in,out}.host_binding.<i>.torq_binding.<i>.bin
static void dumpBinding(const thip_executable_t *e, uint32_t binding, const void *host, size_t size, bool isInput) {
    const thip_device_t *d = e->device;
    if (d->dumpIoDir.empty()) return;
    const std::string dir = d->dumpIoDir + "/" + e->header.name;
    if (!makeDirs(dir)) return;
    const std::string n = std::to_string(binding);
    const std::string path = dir + "/npu" + (isInput ? ".in" : ".out") + ".host_binding." + n + ".torq_binding." + n + ".bin";
    if (FILE *f = fopen(path.c_str(), "wb")) {
        fwrite(host, 1, size, f);
        fclose(f);
    }
}

// What record i wrote, as a NumPy array file <dir>/<executable>/action<i>/buffer<id>.npy (the reference writes one
// .npy per live buffer per action, runtime/driver/TorqDump.cc:341-428), id = "binding<k>" or "temp<k>", plus one
// line of <dir>/<executable>/buffers.csv in the reference's columns.  The record's kernels must have finished.
static thip_status_t dumpOpOutput(thip_executable_t *e, uint32_t i, uint8_t *const *bp) {
    const thip_device_t *d = e->device;
    const DescOp &op = e->ops[i];
    std::vector<int64_t> shape;
    const char *descr = "|i1", *typeName = "i8";
    size_t elem = 1;
    auto outType = [&]() {
        if (op.out_dtype == THIP_DTYPE_I32) { descr = "<i4"; typeName = "i32"; elem = 4; }
        else if (op.out_dtype == THIP_DTYPE_I16) { descr = "<i2"; typeName = "i16"; elem = 2; }
    };
    auto bf16 = [&]() { descr = "<u2"; typeName = "bf16"; elem = 2; };  // bf16 bit patterns, as uint16
    switch (op.kind) {
    case kKindTranspose: shape = {op.TB, op.TS, op.TP ? op.TP : op.TR}; if (op.gran == 2) bf16(); break;
    case kKindIgemm: case kKindFcSkinny: shape = {op.M, op.Nn}; outType(); break;
    case kKindDepthwise: case kKindMaxPool: shape = {op.N, op.OH, op.OW, op.C}; break;
    case kKindAvgPool: shape = {op.N, op.C}; break;
    case kKindAdd: shape = {op.C}; break;
    case kKindEltwise: shape = {op.C}; outType(); break;
    case kKindFcBf16: case kKindDecLinear: shape = {op.M, op.Nn}; bf16(); break;
    case kKindDecMatmul: shape = {op.TB, op.M, op.Nn}; bf16(); break;
    case kKindAddBf16: shape = {op.C}; bf16(); break;
    case kKindIm2colBf16: shape = {op.N, op.OH, op.OW, op.Kp}; bf16(); break;
    case kKindDepthwiseBf16: shape = {op.N, op.OH, op.OW, op.C}; bf16(); break;
    case kKindAvgPoolBf16: shape = {op.N, op.C}; bf16(); break;
    case kKindExpandWeights: shape = {op.K, op.Nn}; bf16(); break;
    default: return THIP_OK;
    }
    size_t count = 1;
    for (int64_t v : shape) count *= (size_t)v;
    if (count == 0 || op.out.space == kSpaceNone) return THIP_OK;  // e.g. a convolution whose result only feeds its fused add
    std::vector<uint8_t> host(count * elem);
    THIP_HIP(hipMemcpy(host.data(), resolve(e, op.out, bp), host.size(), hipMemcpyDeviceToHost), "reading a buffer back for the dump");
    const std::string base = d->dumpBuffersDir + "/" + e->header.name, dir = base + "/action" + std::to_string(i);
    if (!makeDirs(dir)) return fail(THIP_INVALID_ARGUMENT, "cannot create dump directory %s", dir.c_str());
    const std::string id = (op.out.space == kSpaceBinding ? "binding" : "temp") + std::to_string(op.out.index);
    std::string dims, dimsX;
    for (size_t k = 0; k < shape.size(); k++) {
        dims += std::to_string(shape[k]) + ",";
        dimsX += std::to_string(shape[k]) + "x";
    }
    std::string header = std::string("{'descr': '") + descr + "', 'fortran_order': False, 'shape': (" + dims + "), }";
    while ((10 + header.size() + 1) % 64 != 0) header += ' ';
    header += '\n';
    FILE *f = fopen((dir + "/buffer" + id + ".npy").c_str(), "wb");
    if (!f) return fail(THIP_INVALID_ARGUMENT, "cannot write into dump directory %s", dir.c_str());
    const uint8_t magic[10] = {0x93, 'N', 'U', 'M', 'P', 'Y', 1, 0, (uint8_t)(header.size() & 0xff), (uint8_t)(header.size() >> 8)};
    fwrite(magic, 1, sizeof(magic), f);
    fwrite(header.data(), 1, header.size(), f);
    fwrite(host.data(), 1, host.size(), f);
    fclose(f);
    // index of the buffers, one line per record output; started afresh by the first record of every dispatch
    if (FILE *csv = fopen((base + "/buffers.csv").c_str(), i == 0 ? "w" : "a")) {
        if (i == 0) {
            fprintf(csv, "id;type;shape;strides;address;size;allocation_action;last_use_action;deallocation_action;"
                         "allocation_location;last_use_location;deallocation_location\n");
        }
        fprintf(csv, "%s;%s;%s%s;;%llu;%zu;%u;%u;%u;%s;;\n", id.c_str(), op.out.space == kSpaceBinding ? "BINDING" : "INTERMEDIATE", dimsX.c_str(),
                typeName, (unsigned long long)op.out.offset, host.size(), i, i, e->header.op_count - 1, e->kernelNames[i].c_str());
        fclose(csv);
    }
    return THIP_OK;
}

// Enqueues every kernel record of the program.  `bp` holds one device pointer per binding.
static thip_status_t enqueueOps(thip_executable_t *e, uint8_t *const *bp) {
    for (uint32_t i = 0; i < e->header.op_count; i++) {
        // a kernel launch is what starting an NSS task is on the reference's hardware
        logEvent(e, e->invocation, (int32_t)i, "NSS_START", "BEGIN", e->kernelNames[i].c_str());
        if (thip_status_t s = launchOp(e, i, bp, LaunchCtx{e->stream, &e->tuning, nullptr, 0})) return s;
        logEvent(e, e->invocation, (int32_t)i, "NSS_START", "END", e->kernelNames[i].c_str());
        if (!e->device->dumpBuffersDir.empty()) {
            // buffer dumps: each record runs to its end and what it wrote is read back before the next one starts
            if (thip_status_t s = waitBounded(e, "waiting for a record before its dump")) return s;
            if (thip_status_t s = dumpOpOutput(e, i, bp)) return s;
        }
    }
    return THIP_OK;
}

constexpr uint32_t kGraphMinOps = 4;

static void dropGraph(thip_executable_t *e) {
    if (e->graphExec) (void)hipGraphExecDestroy(e->graphExec);
    if (e->graph) (void)hipGraphDestroy(e->graph);
    e->graphExec = nullptr;
    e->graph = nullptr;
    e->graphPtrs.clear();
}

// Enqueues one dispatch on device bindings, through the graph when there is one.
static thip_status_t enqueueDevice(thip_executable_t *e, uint8_t *const *bp) {
    const uint32_t nb = e->header.binding_count;
    const bool eligible = !e->graphsDisabled && e->header.op_count >= kGraphMinOps && !e->device->eventLog && e->device->dumpBuffersDir.empty();
    if (!eligible) return enqueueOps(e, bp);
    std::vector<uint8_t *> key(bp, bp + nb);
    if (e->graphExec && key == e->graphPtrs) {
        THIP_HIP(hipGraphLaunch(e->graphExec, e->stream), "hipGraphLaunch");
        return THIP_OK;
    }
    if (key != e->seenPtrs) {  // first time with these pointers: run eagerly (this also configures the kernels)
        e->seenPtrs = key;
        return enqueueOps(e, bp);
    }
    dropGraph(e);
    THIP_HIP(hipStreamBeginCapture(e->stream, hipStreamCaptureModeThreadLocal), "hipStreamBeginCapture");
    const thip_status_t launched = enqueueOps(e, bp);
    hipGraph_t g = nullptr;
    const hipError_t ended = hipStreamEndCapture(e->stream, &g);
    if (launched != THIP_OK || ended != hipSuccess || !g) {
        if (g) (void)hipGraphDestroy(g);
        e->graphsDisabled = true;  // fall back to eager launches for good
        (void)hipGetLastError();
        if (launched != THIP_OK) return launched;
        return enqueueOps(e, bp);
    }
    e->graph = g;
    if (hipGraphInstantiate(&e->graphExec, g, nullptr, nullptr, 0) != hipSuccess) {
        dropGraph(e);
        e->graphsDisabled = true;
        (void)hipGetLastError();
        return enqueueOps(e, bp);
    }
    e->graphPtrs = key;
    THIP_HIP(hipGraphLaunch(e->graphExec, e->stream), "hipGraphLaunch");
    return THIP_OK;
}

extern "C" {

thip_status_t thip_device_create(int32_t ordinal, thip_device_t **out_device) {
    if (!out_device) return fail(THIP_INVALID_ARGUMENT, "null result pointer");
    *out_device = nullptr;
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0) {
        (void)hipGetLastError();
        return fail(THIP_UNAVAILABLE, "no HIP device is visible (%s)", e == hipSuccess ? "count is 0" : hipGetErrorString(e));
    }
    if (ordinal < 0 || ordinal >= count) return fail(THIP_INVALID_ARGUMENT, "device ordinal %d is outside 0..%d", ordinal, count - 1);
    hipDeviceProp_t prop;
    THIP_HIP(hipGetDeviceProperties(&prop, ordinal), "hipGetDeviceProperties");
    std::string arch = prop.gcnArchName;
    const size_t colon = arch.find(':');
    if (colon != std::string::npos) arch.resize(colon);
    if (arch != "gfx950") return fail(THIP_UNAVAILABLE, "device %d is %s; the kernels are built for gfx950 only", ordinal, arch.c_str());
    THIP_HIP(hipSetDevice(ordinal), "hipSetDevice");
    thip_device_t *d = new (std::nothrow) thip_device_t();
    if (!d) return fail(THIP_RESOURCE_EXHAUSTED, "out of memory");
    d->ordinal = ordinal;
    d->arch = arch;
    {
        // the address of this device's copy of the scratch array (the device is current)
        void *ptr = nullptr;
        const hipError_t se = staticScratchAddress(&ptr);
        if (se != hipSuccess) {
            delete d;
            return hipFail(se, "locating the static scratch array");
        }
        d->staticScratch = (uint8_t *)ptr;
    }
    *out_device = d;
    return THIP_OK;
}

void thip_device_destroy(thip_device_t *device) {
    if (!device) return;
    if (device->eventLog) fclose(device->eventLog);
    delete device;
}

thip_status_t thip_device_name(thip_device_t *device, char *name, size_t capacity) {
    if (!device || !name || capacity == 0) return fail(THIP_INVALID_ARGUMENT, "null argument");
    snprintf(name, capacity, "%s", device->arch.c_str());
    return THIP_OK;
}

thip_status_t thip_device_alloc(thip_device_t *device, size_t size, void **out_ptr) {
    if (!device || !out_ptr) return fail(THIP_INVALID_ARGUMENT, "null argument");
    *out_ptr = nullptr;
    THIP_HIP(hipSetDevice(device->ordinal), "hipSetDevice");
    THIP_HIP(hipMalloc(out_ptr, size ? size : 1), "hipMalloc");
    return THIP_OK;
}

thip_status_t thip_device_free(thip_device_t *device, void *ptr) {
    if (!device) return fail(THIP_INVALID_ARGUMENT, "null device");
    if (ptr) THIP_HIP(hipFree(ptr), "hipFree");
    return THIP_OK;
}

thip_status_t thip_device_h2d(thip_device_t *device, void *dst_device, const void *src_host, size_t size) {
    if (!device || (size && (!dst_device || !src_host))) return fail(THIP_INVALID_ARGUMENT, "null argument");
    if (size) THIP_HIP(hipMemcpy(dst_device, src_host, size, hipMemcpyHostToDevice), "hipMemcpy H2D");
    return THIP_OK;
}

thip_status_t thip_device_d2h(thip_device_t *device, void *dst_host, const void *src_device, size_t size) {
    if (!device || (size && (!dst_host || !src_device))) return fail(THIP_INVALID_ARGUMENT, "null argument");
    if (size) THIP_HIP(hipMemcpy(dst_host, src_device, size, hipMemcpyDeviceToHost), "hipMemcpy D2H");
    return THIP_OK;
}

thip_status_t thip_device_synchronize(thip_device_t *device) {
    if (!device) return fail(THIP_INVALID_ARGUMENT, "null device");
    THIP_HIP(hipDeviceSynchronize(), "hipDeviceSynchronize");
    return THIP_OK;
}

thip_status_t thip_device_set_event_log(thip_device_t *device, const char *csv_path) {
    if (!device) return fail(THIP_INVALID_ARGUMENT, "null device");
    std::lock_guard<std::mutex> lock(device->logMutex);
    if (device->eventLog) {
        fclose(device->eventLog);
        device->eventLog = nullptr;
    }
    if (csv_path && csv_path[0]) {
        device->eventLog = fopen(csv_path, "w");
        if (!device->eventLog) return fail(THIP_INVALID_ARGUMENT, "cannot open event log %s", csv_path);
        fprintf(device->eventLog, "dispatch_name,invocation_id,action_id,timestamp_us,event,kernel\n");
    }
    return THIP_OK;
}

thip_status_t thip_device_mfma_rate(thip_device_t *device, int32_t random_operands, int32_t workgroups, int32_t iterations, double *out_tops) {
    if (!device || !out_tops) return fail(THIP_INVALID_ARGUMENT, "null argument");
    if (workgroups <= 0 || iterations <= 0) return fail(THIP_INVALID_ARGUMENT, "workgroups and iterations must be positive");
    THIP_HIP(hipSetDevice(device->ordinal), "hipSetDevice");
    THIP_HIP(measureMfmaRate(random_operands, workgroups, iterations, nullptr, out_tops), "measuring the MFMA rate");
    return THIP_OK;
}

thip_status_t thip_device_stream_floor(thip_device_t *device, int32_t reads_per_write, size_t write_bytes, int32_t cold, double *out_microseconds) {
    return thip_device_stream_floor_tuned(device, reads_per_write, write_bytes, cold, out_microseconds, nullptr, 0);
}

thip_status_t thip_device_stream_floor_tuned(thip_device_t *device, int32_t reads_per_write, size_t write_bytes, int32_t cold, double *out_microseconds,
                                             char *out_variant, size_t variant_capacity) {
    if (!device || !out_microseconds) return fail(THIP_INVALID_ARGUMENT, "null argument");
    THIP_HIP(hipSetDevice(device->ordinal), "hipSetDevice");
    const hipError_t err = measureStreamRate(reads_per_write, write_bytes, cold, nullptr, out_microseconds, out_variant, variant_capacity);
    if (err == hipErrorInvalidValue) return fail(THIP_INVALID_ARGUMENT, "reads_per_write is 1, 2 or 4; write_bytes a multiple of 16 from 4 KiB to 2 GiB");
    THIP_HIP(err, "measuring the streaming floor");
    return THIP_OK;
}

thip_status_t thip_device_set_dump_dirs(thip_device_t *device, const char *io_data_dir, const char *buffers_dir) {
    if (!device) return fail(THIP_INVALID_ARGUMENT, "null device");
    const std::string io = io_data_dir ? io_data_dir : "", buffers = buffers_dir ? buffers_dir : "";
    for (const std::string *dir : {&io, &buffers}) {
        if (!dir->empty() && !makeDirs(*dir)) return fail(THIP_INVALID_ARGUMENT, "cannot create dump directory %s", dir->c_str());
    }
    device->dumpIoDir = io;
    device->dumpBuffersDir = buffers;
    return THIP_OK;
}

thip_status_t thip_executable_set_wait_timeout(thip_executable_t *e, int64_t milliseconds) {
    if (!e) return fail(THIP_INVALID_ARGUMENT, "null executable");
    std::lock_guard<std::mutex> lock(e->mutex);
    e->waitTimeoutMs = milliseconds;
    return THIP_OK;
}

void thip_executable_destroy(thip_executable_t *e) {
    if (!e) return;
    if (e->abandoned) {
        // a wait on this executable timed out.  If its work has finished since, clean up as usual; if not, kernels may
        // still be using its buffers: leave everything in place (the caller is expected to end the process)
        if (!e->stream || hipStreamQuery(e->stream) != hipSuccess) {
            (void)hipGetLastError();
            return;
        }
    }
    if (e->stream) (void)hipStreamSynchronize(e->stream);
    dropGraph(e);
    for (uint8_t *p : e->tempPtrs) {
        if (p) (void)hipFree(p);
    }
    for (uint8_t *p : e->staging) {
        if (p) (void)hipFree(p);
    }
    if (e->constData) (void)hipFree(e->constData);
    if (e->evStart) (void)hipEventDestroy(e->evStart);
    if (e->evStop) (void)hipEventDestroy(e->evStop);
    if (e->evDone) (void)hipEventDestroy(e->evDone);
    if (e->stream) (void)hipStreamDestroy(e->stream);
    delete e;
}

thip_status_t thip_executable_create(thip_device_t *device, const void *blob, size_t size, const uint32_t *constants,
                                     size_t constant_count, thip_executable_t **out_executable) {
    if (!out_executable) return fail(THIP_INVALID_ARGUMENT, "null result pointer");
    *out_executable = nullptr;
    if (!device) return fail(THIP_INVALID_ARGUMENT, "null device");
    if (constant_count > 0 && !constants) return fail(THIP_INVALID_ARGUMENT, "constants pointer is NULL");
    DescHeader h;
    if (thip_status_t s = validateDescriptor((const uint8_t *)blob, size, &h)) return s;
    thip_executable_t *e = new (std::nothrow) thip_executable_t();
    if (!e) return fail(THIP_RESOURCE_EXHAUSTED, "out of memory");
    e->device = device;
    e->blob.assign((const uint8_t *)blob, (const uint8_t *)blob + h.total_size);
    if (constant_count) e->constants.assign(constants, constants + constant_count);
    e->header = h;
    e->ops = (const DescOp *)(e->blob.data() + h.ops_offset);
    e->bindings = (const DescBinding *)(e->blob.data() + h.bindings_offset);
    e->temps = (const DescTemp *)(e->blob.data() + h.temps_offset);
    e->consts = (const DescConst *)(e->blob.data() + h.consts_offset);
    thip_status_t s = THIP_OK;
    {
        const DescriptorView view{e->blob.data(), h, e->ops, e->bindings, e->temps, e->consts};
        for (uint32_t i = 0; i < h.op_count && s == THIP_OK; i++) s = checkOpFootprint(&view, i);
    }
    auto bail = [&](thip_status_t code) {
        thip_executable_destroy(e);
        return code;
    };
    if (s != THIP_OK) return bail(s);
    hipError_t err = hipSetDevice(device->ordinal);
    if (err == hipSuccess) err = hipStreamCreate(&e->stream);  // default priority
    if (err == hipSuccess) err = hipEventCreate(&e->evStart);
    if (err == hipSuccess) err = hipEventCreate(&e->evStop);
    if (err == hipSuccess) err = hipEventCreateWithFlags(&e->evDone, hipEventDisableTiming);
    if (err != hipSuccess) return bail(hipFail(err, "creating the stream"));
    const uint64_t dataSize = h.total_size - h.data_offset;
    if (dataSize) {
        err = hipMalloc((void **)&e->constData, dataSize);
        if (err == hipSuccess) err = hipMemcpy(e->constData, e->blob.data() + h.data_offset, dataSize, hipMemcpyHostToDevice);
        if (err != hipSuccess) return bail(hipFail(err, "uploading the constant segment"));
    }
    e->tempPtrs.assign(h.temp_count, nullptr);
    for (uint32_t i = 0; i < h.temp_count; i++) {
        const uint64_t bytes = e->temps[i].size ? e->temps[i].size : 1;
        err = hipMalloc((void **)&e->tempPtrs[i], bytes);
        // zero-filled once: padding regions of packed run-time operands rely on it
        if (err == hipSuccess) err = hipMemset(e->tempPtrs[i], 0, bytes);
        if (err != hipSuccess) return bail(hipFail(err, "allocating an intermediate"));
    }
    e->staging.assign(h.binding_count, nullptr);
    e->graphsDisabled = getenv("THIP_NO_GRAPH") != nullptr;
    if (const char *t = getenv("THIP_WAIT_TIMEOUT_MS")) e->waitTimeoutMs = atoll(t);
    // Which kernel each record runs is settled now, from the record, the alignment of its operands and the
    // environment's switches, and kept: the launchers are asked in naming mode (they also configure their kernels,
    // which must not happen later inside a stream capture).  Bindings stand in as aligned placeholder addresses:
    // device bindings must be 16-byte aligned and staged host bindings are, so a dispatch resolves the same way.
    e->scratchOffset.assign(h.op_count, 0);
    for (uint32_t i = 0; i < h.op_count; i++) {
        const DescOp &op = e->ops[i];
        if (op.kind != kKindFcBf16 || op.w0 <= 1) continue;
        e->scratchOffset[i] = e->scratchBytes;
        e->scratchBytes += (fcBf16WorkspaceBytes(op.M, op.Nn, op.w0) + 255) / 256 * 256;
    }
    e->tuning = tuningFromEnvironment();
    e->kernelNames.assign(h.op_count, std::string());
    {
        uint8_t *placeholder[64];
        for (auto &ptr : placeholder) ptr = (uint8_t *)(uintptr_t)0x1000000;
        for (uint32_t i = 0; i < h.op_count; i++) {
            char name[96] = "";
            if (thip_status_t st = launchOp(e, i, placeholder, LaunchCtx{nullptr, &e->tuning, name, sizeof(name)})) return bail(st);
            e->kernelNames[i] = name[0] ? name : opKernelName(e->ops[i]);
        }
    }
    *out_executable = e;
    return THIP_OK;
}

static thip_status_t refuseAbandoned(const thip_executable_t *e) {
    if (!e->abandoned) return THIP_OK;
    return fail(THIP_FAILED_PRECONDITION, "an earlier wait on this executable timed out; it cannot be used any more");
}

static thip_status_t runLocked(thip_executable_t *e, const thip_dispatch_state_t *st) {
    if (thip_status_t s = refuseAbandoned(e)) return s;
    THIP_HIP(hipSetDevice(e->device->ordinal), "hipSetDevice");
    uint8_t *bp[64] = {nullptr};
    const int32_t lastOp = (int32_t)e->header.op_count - 1;
    logEvent(e, e->invocation, 0, "DISPATCH", "BEGIN", "");
    logEvent(e, e->invocation, 0, "DISPATCH_SYNC_BINDINGS_IN", "BEGIN", "");
    // writeInputs: host bindings are staged into device memory (TorqExecutable::writeInputs)
    for (uint32_t i = 0; i < e->header.binding_count; i++) {
        if (e->bindings[i].flags == 0) continue;
        const bool isDevice = st->binding_flags && (st->binding_flags[i] & THIP_BINDING_DEVICE);
        if (isDevice) {
            bp[i] = (uint8_t *)st->binding_ptrs[i];
            continue;
        }
        if (!e->staging[i]) {
            THIP_HIP(hipMalloc((void **)&e->staging[i], e->bindings[i].size ? e->bindings[i].size : 1), "allocating binding staging");
        }
        bp[i] = e->staging[i];
        if (e->bindings[i].flags & kBindingRead) {
            dumpBinding(e, i, st->binding_ptrs[i], e->bindings[i].size, true);
            THIP_HIP(hipMemcpyAsync(bp[i], st->binding_ptrs[i], e->bindings[i].size, hipMemcpyHostToDevice, e->stream), "staging a binding");
        }
    }
    logEvent(e, e->invocation, 0, "DISPATCH_SYNC_BINDINGS_IN", "END", "");
    bool allDevice = true;
    for (uint32_t i = 0; i < e->header.binding_count; i++) {
        if (e->bindings[i].flags != 0 && !(st->binding_flags && (st->binding_flags[i] & THIP_BINDING_DEVICE))) allDevice = false;
    }
    logEvent(e, e->invocation, 0, "DISPATCH_EXECUTE_ACTIONS", "BEGIN", "");
    if (thip_status_t s = allDevice ? enqueueDevice(e, bp) : enqueueOps(e, bp)) {
        // what was enqueued before the failure still runs: wait for it (bounded; the launch error is what is reported)
        std::string message = thip_status_message();
        if (!e->abandoned) (void)waitBounded(e, "waiting after a failed launch");
        e->invocation++;
        return fail(s, "%s", message.c_str());
    }
    logEvent(e, e->invocation, lastOp, "DISPATCH_EXECUTE_ACTIONS", "END", "");
    logEvent(e, e->invocation, lastOp, "DISPATCH_SYNC_BINDINGS_OUT", "BEGIN", "");
    // readOutputs (TorqExecutable::readOutputs, runtime/driver/TorqExecutable.cc:860-918)
    for (uint32_t i = 0; i < e->header.binding_count; i++) {
        const bool isDevice = st->binding_flags && (st->binding_flags[i] & THIP_BINDING_DEVICE);
        if (isDevice || !(e->bindings[i].flags & kBindingWritten)) continue;
        THIP_HIP(hipMemcpyAsync(st->binding_ptrs[i], bp[i], e->bindings[i].size, hipMemcpyDeviceToHost, e->stream), "reading back a binding");
    }
    logEvent(e, e->invocation, lastOp, "NSS_WAIT", "BEGIN", "");
    const thip_status_t waited = waitBounded(e, "waiting for the dispatch");
    const std::string waitMessage = waited == THIP_OK ? std::string() : std::string(thip_status_message());
    logEvent(e, e->invocation, lastOp, "NSS_WAIT", "END", "");
    logEvent(e, e->invocation, lastOp, "DISPATCH_SYNC_BINDINGS_OUT", "END", "");
    logEvent(e, e->invocation, lastOp, "DISPATCH", "END", "");
    e->invocation++;
    if (waited != THIP_OK) return fail(waited, "%s", waitMessage.c_str());
    for (uint32_t i = 0; i < e->header.binding_count; i++) {
        const bool isDevice = st->binding_flags && (st->binding_flags[i] & THIP_BINDING_DEVICE);
        if (!isDevice && (e->bindings[i].flags & kBindingWritten)) dumpBinding(e, i, st->binding_ptrs[i], e->bindings[i].size, false);
    }
    return THIP_OK;
}

thip_status_t thip_executable_run(thip_executable_t *e, const thip_dispatch_state_t *st) {
    if (!e) return fail(THIP_INVALID_ARGUMENT, "null executable");
    if (thip_status_t s = checkState(e, st, false)) return s;
    std::lock_guard<std::mutex> lock(e->mutex);
    return runLocked(e, st);
}

thip_status_t thip_executable_enqueue(thip_executable_t *e, const thip_dispatch_state_t *st) {
    if (!e) return fail(THIP_INVALID_ARGUMENT, "null executable");
    if (thip_status_t s = checkState(e, st, true)) return s;
    std::lock_guard<std::mutex> lock(e->mutex);
    if (thip_status_t s = refuseAbandoned(e)) return s;
    THIP_HIP(hipSetDevice(e->device->ordinal), "hipSetDevice");
    uint8_t *bp[64] = {nullptr};
    for (uint32_t i = 0; i < e->header.binding_count; i++) bp[i] = (uint8_t *)st->binding_ptrs[i];
    const thip_status_t s = enqueueDevice(e, bp);
    e->invocation++;
    return s;
}

thip_status_t thip_executable_enqueue_noalloc(thip_executable_t *e, const thip_dispatch_state_t *st) {
    if (!e) return fail(THIP_INVALID_ARGUMENT, "null executable");
    if (thip_status_t s = checkState(e, st, true)) return s;
    if (e->scratchBytes > kStaticScratchBytes) {
        return fail(THIP_RESOURCE_EXHAUSTED, "the program's kernels need %llu bytes of scratch, the static array holds %llu",
                    (unsigned long long)e->scratchBytes, (unsigned long long)kStaticScratchBytes);
    }
    std::lock_guard<std::mutex> lock(e->mutex);
    if (thip_status_t s = refuseAbandoned(e)) return s;
    THIP_HIP(hipSetDevice(e->device->ordinal), "hipSetDevice");
    uint8_t *scratch = e->device->staticScratch;  // the address hipGetSymbolAddress gave for this device
    if (!scratch) return fail(THIP_INTERNAL, "the static scratch array was not located");
    uint8_t *bp[64] = {nullptr};
    for (uint32_t i = 0; i < e->header.binding_count; i++) bp[i] = (uint8_t *)st->binding_ptrs[i];
    const LaunchCtx ctx{e->stream, &e->tuning, nullptr, 0};
    thip_status_t result = THIP_OK;
    for (uint32_t i = 0; i < e->header.op_count && result == THIP_OK; i++) {
        // the array keeps what the last call left there, whoever made it; nothing in a K-split workspace has to start
        // at zero (every slot that is read has been written by the same dispatch)
        if (result == THIP_OK) result = launchOp(e, i, bp, ctx, scratch);
    }
    e->invocation++;
    return result;
}

thip_status_t thip_executable_wait(thip_executable_t *e) {
    if (!e) return fail(THIP_INVALID_ARGUMENT, "null executable");
    std::lock_guard<std::mutex> lock(e->mutex);
    if (thip_status_t s = refuseAbandoned(e)) return s;
    return waitBounded(e, "waiting for the dispatch");
}

thip_status_t thip_executable_time(thip_executable_t *e, const thip_dispatch_state_t *st, int32_t iterations, float *out_ms) {
    if (!e || !out_ms) return fail(THIP_INVALID_ARGUMENT, "null argument");
    if (iterations <= 0) return fail(THIP_INVALID_ARGUMENT, "iterations must be positive");
    if (thip_status_t s = checkState(e, st, true)) return s;
    std::lock_guard<std::mutex> lock(e->mutex);
    if (thip_status_t as = refuseAbandoned(e)) return as;
    THIP_HIP(hipSetDevice(e->device->ordinal), "hipSetDevice");
    uint8_t *bp[64] = {nullptr};
    for (uint32_t i = 0; i < e->header.binding_count; i++) bp[i] = (uint8_t *)st->binding_ptrs[i];
    THIP_HIP(hipEventRecord(e->evStart, e->stream), "hipEventRecord");
    for (int32_t it = 0; it < iterations; it++) {
        const thip_status_t s = enqueueDevice(e, bp);
        e->invocation++;
        if (s != THIP_OK) {
            (void)hipStreamSynchronize(e->stream);
            return s;
        }
    }
    THIP_HIP(hipEventRecord(e->evStop, e->stream), "hipEventRecord");
    if (thip_status_t ws = waitBounded(e, "waiting for the timed dispatches")) return ws;
    float ms = 0.f;
    THIP_HIP(hipEventElapsedTime(&ms, e->evStart, e->evStop), "hipEventElapsedTime");
    *out_ms = ms / (float)iterations;
    return THIP_OK;
}

thip_status_t thip_executable_time_rotating(thip_executable_t *e, const thip_dispatch_state_t *states, uint32_t state_count,
                                            int32_t iterations, float *out_ms) {
    if (!e || !out_ms || !states) return fail(THIP_INVALID_ARGUMENT, "null argument");
    if (iterations <= 0 || state_count == 0) return fail(THIP_INVALID_ARGUMENT, "iterations and state_count must be positive");
    for (uint32_t s = 0; s < state_count; s++) {
        if (thip_status_t st = checkState(e, &states[s], true)) return st;
    }
    std::lock_guard<std::mutex> lock(e->mutex);
    if (thip_status_t as = refuseAbandoned(e)) return as;
    THIP_HIP(hipSetDevice(e->device->ordinal), "hipSetDevice");
    THIP_HIP(hipEventRecord(e->evStart, e->stream), "hipEventRecord");
    for (int32_t it = 0; it < iterations; it++) {
        const thip_dispatch_state_t &st = states[(uint32_t)it % state_count];
        uint8_t *bp[64] = {nullptr};
        for (uint32_t i = 0; i < e->header.binding_count; i++) bp[i] = (uint8_t *)st.binding_ptrs[i];
        const thip_status_t s = enqueueDevice(e, bp);
        e->invocation++;
        if (s != THIP_OK) {
            (void)hipStreamSynchronize(e->stream);
            return s;
        }
    }
    THIP_HIP(hipEventRecord(e->evStop, e->stream), "hipEventRecord");
    if (thip_status_t ws = waitBounded(e, "waiting for the timed dispatches")) return ws;
    float ms = 0.f;
    THIP_HIP(hipEventElapsedTime(&ms, e->evStart, e->evStop), "hipEventElapsedTime");
    *out_ms = ms / (float)iterations;
    return THIP_OK;
}

thip_status_t thip_executable_op_count(thip_executable_t *e, uint32_t *out_count) {
    if (!e || !out_count) return fail(THIP_INVALID_ARGUMENT, "null argument");
    *out_count = e->header.op_count;
    return THIP_OK;
}

thip_status_t thip_executable_op_kernel(thip_executable_t *e, uint32_t index, char *name, size_t capacity) {
    if (!e || !name || capacity == 0) return fail(THIP_INVALID_ARGUMENT, "null argument");
    if (index >= e->header.op_count) return fail(THIP_OUT_OF_RANGE, "op %u of %u", index, e->header.op_count);
    snprintf(name, capacity, "%s", e->kernelNames[index].c_str());
    return THIP_OK;
}

thip_status_t thip_executable_binding_count(thip_executable_t *e, uint32_t *out_count) {
    if (!e || !out_count) return fail(THIP_INVALID_ARGUMENT, "null argument");
    *out_count = e->header.binding_count;
    return THIP_OK;
}

thip_status_t thip_executable_binding_size(thip_executable_t *e, uint32_t binding, size_t *out_size) {
    if (!e || !out_size) return fail(THIP_INVALID_ARGUMENT, "null argument");
    if (binding >= e->header.binding_count) return fail(THIP_OUT_OF_RANGE, "binding %u of %u", binding, e->header.binding_count);
    *out_size = (size_t)e->bindings[binding].size;
    return THIP_OK;
}

}  // extern "C"
