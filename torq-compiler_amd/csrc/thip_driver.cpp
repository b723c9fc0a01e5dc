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

#include <chrono>
#include <mutex>
#include <new>
#include <string>
#include <vector>

#include "thip_descriptor.h"
#include "thip_kernels.h"
#include "thip_status.h"

using namespace thip;

struct thip_device_t {
    int ordinal = 0;
    std::string arch;
    std::mutex logMutex;
    FILE *eventLog = nullptr;
    std::chrono::steady_clock::time_point t0 = std::chrono::steady_clock::now();
    uint8_t *staticScratch = nullptr;    // this GPU's copy of the library's scratch array (kStaticScratchBytes)
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
    hipEvent_t evStart = nullptr, evStop = nullptr;
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
    // how much of it has to be zero before the launch, and the program's total
    std::vector<uint64_t> scratchOffset, scratchZeroBytes;
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

static thip_status_t validateDescriptor(const uint8_t *p, size_t size, DescHeader *out) {
    if (!p || size < sizeof(DescHeader)) return fail(THIP_INVALID_ARGUMENT, "descriptor is smaller than its header");
    DescHeader h;
    memcpy(&h, p, sizeof(h));
    if (h.magic != kMagic) return fail(THIP_INVALID_ARGUMENT, "descriptor magic 0x%08x is not THIP", h.magic);
    // same gate as `runtime_version != 2 -> UNAVAILABLE`, runtime/driver/TorqExecutable.cc:663-667
    if (h.version != kDescriptorVersion) {
        return fail(THIP_UNAVAILABLE, "descriptor version %u, this runtime reads version %u", h.version, kDescriptorVersion);
    }
    // same gate as isHwCompatible(hwId), runtime/driver/TorqExecutable.cc:701-705
    if (h.arch != kArchGfx950) return fail(THIP_UNAVAILABLE, "descriptor targets arch %u, this runtime drives gfx950", h.arch);
    if (h.total_size > size) return fail(THIP_INVALID_ARGUMENT, "descriptor says %llu bytes, %zu given", (unsigned long long)h.total_size, size);
    auto inside = [&](uint64_t off, uint64_t count, uint64_t each) {
        return off <= h.total_size && count * each <= h.total_size - off;
    };
    if (!inside(h.ops_offset, h.op_count, sizeof(DescOp)) || !inside(h.bindings_offset, h.binding_count, sizeof(DescBinding)) ||
        !inside(h.temps_offset, h.temp_count, sizeof(DescTemp)) || !inside(h.consts_offset, h.const_count, sizeof(DescConst)) ||
        h.data_offset > h.total_size) {
        return fail(THIP_INVALID_ARGUMENT, "descriptor tables run past its end");
    }
    if (h.op_count == 0) return fail(THIP_INVALID_ARGUMENT, "descriptor holds no ops");
    if (h.binding_count > 64) return fail(THIP_INVALID_ARGUMENT, "descriptor declares %u bindings (max 64)", h.binding_count);
    const DescConst *consts = (const DescConst *)(p + h.consts_offset);
    for (uint32_t i = 0; i < h.const_count; i++) {
        if (consts[i].offset > h.total_size - h.data_offset || consts[i].size > h.total_size - h.data_offset - consts[i].offset) {
            return fail(THIP_INVALID_ARGUMENT, "constant segment %u runs past the descriptor", i);
        }
    }
    // every operand reference must name an existing buffer and stay inside it
    const DescOp *ops = (const DescOp *)(p + h.ops_offset);
    const DescBinding *bindings = (const DescBinding *)(p + h.bindings_offset);
    const DescTemp *temps = (const DescTemp *)(p + h.temps_offset);
    for (uint32_t i = 0; i < h.op_count; i++) {
        const DescRef *refs[] = {&ops[i].in0, &ops[i].in1, &ops[i].weights, &ops[i].bias, &ops[i].scale, &ops[i].table, &ops[i].out};
        for (const DescRef *r : refs) {
            uint64_t limit = 0;
            switch (r->space) {
            case kSpaceNone: continue;
            case kSpaceBinding:
                if (r->index >= h.binding_count) return fail(THIP_INVALID_ARGUMENT, "op %u names binding %u of %u", i, r->index, h.binding_count);
                limit = bindings[r->index].size;
                break;
            case kSpaceTemp:
                if (r->index >= h.temp_count) return fail(THIP_INVALID_ARGUMENT, "op %u names intermediate %u of %u", i, r->index, h.temp_count);
                limit = temps[r->index].size;
                break;
            case kSpaceConst:
                if (r->index >= h.const_count) return fail(THIP_INVALID_ARGUMENT, "op %u names constant %u of %u", i, r->index, h.const_count);
                limit = consts[r->index].size;
                break;
            default: return fail(THIP_INVALID_ARGUMENT, "op %u has an operand in unknown space %u", i, r->space);
            }
            if (r->offset > limit) return fail(THIP_INVALID_ARGUMENT, "op %u operand offset %llu is past its buffer (%llu)", i, (unsigned long long)r->offset, (unsigned long long)limit);
        }
    }
    *out = h;
    return THIP_OK;
}

// Bytes an operand reference can still address.
static uint64_t refRoom(const thip_executable_t *e, const DescRef &r) {
    switch (r.space) {
    case kSpaceBinding: return e->bindings[r.index].size - r.offset;
    case kSpaceTemp: return e->temps[r.index].size - r.offset;
    case kSpaceConst: return e->consts[r.index].size - r.offset;
    default: return 0;
    }
}

// Checks, once at creation, that every kernel record stays inside the buffers it names.
static thip_status_t checkOpFootprint(const thip_executable_t *e, uint32_t i) {
    const DescOp &op = e->ops[i];
    auto need = [&](const DescRef &r, uint64_t bytes, const char *name) -> thip_status_t {
        if (r.space == kSpaceNone) return fail(THIP_INVALID_ARGUMENT, "op %u: operand %s is missing", i, name);
        if (refRoom(e, r) < bytes) {
            return fail(THIP_INVALID_ARGUMENT, "op %u: operand %s needs %llu bytes, its buffer has %llu", i, name,
                        (unsigned long long)bytes, (unsigned long long)refRoom(e, r));
        }
        return THIP_OK;
    };
    auto positive = [&](std::initializer_list<int32_t> vals) {
        for (int32_t v : vals) {
            if (v <= 0) return false;
        }
        return true;
    };
    const uint64_t outElem = op.out_dtype == THIP_DTYPE_I32 ? 4 : op.out_dtype == THIP_DTYPE_I16 ? 2 : 1;
    thip_status_t s = THIP_OK;
    if (op.pre_shift != 0 && (op.pre_shift < 0 || op.pre_shift > 30 || op.shift + op.pre_shift != 33 ||
                              (op.kind != kKindIgemm && op.kind != kKindDepthwise))) {
        return fail(THIP_INVALID_ARGUMENT, "op %u: pre_shift %d does not complete shift %d to 33", i, op.pre_shift, op.shift);
    }
    if (op.t0_clamp != 0 && (op.t0_clamp < 0 || op.pre_shift <= 0 || op.pre_shift > 30 || op.t0_clamp >= (1 << (31 - op.pre_shift)))) {
        return fail(THIP_INVALID_ARGUMENT, "op %u: t0_clamp %d does not fit pre_shift %d", i, op.t0_clamp, op.pre_shift);
    }
    switch (op.kind) {
    case kKindTranspose: {
        if (!positive({op.TB, op.TR, op.TS})) return fail(THIP_INVALID_ARGUMENT, "op %u: bad transpose extents", i);
        if (op.gran > 2) return fail(THIP_INVALID_ARGUMENT, "op %u: transpose element size %u", i, op.gran);
        if (op.TP != 0 && op.TP < op.TR) return fail(THIP_INVALID_ARGUMENT, "op %u: transpose pitch %d is below its row length %d", i, op.TP, op.TR);
        const uint64_t elem = op.gran == 2 ? 2 : 1, pitch = op.TP ? (uint64_t)op.TP : (uint64_t)op.TR;
        if ((s = need(op.in0, (uint64_t)op.TB * op.TR * op.TS * elem, "in"))) return s;
        return need(op.out, (uint64_t)op.TB * op.TS * pitch * elem, "out");
    }
    case kKindIgemm: {
        if (!positive({op.M, op.K, op.Kp, op.Nn, op.Np, op.N, op.H, op.W, op.C, op.OH, op.OW})) {
            return fail(THIP_INVALID_ARGUMENT, "op %u: bad igemm extents", i);
        }
        if (op.variant >= kIgemmVariantCount) return fail(THIP_INVALID_ARGUMENT, "op %u: unknown igemm variant %u", i, op.variant);
        const uint64_t inBytes = op.loader == kLoaderDense ? (uint64_t)op.M * op.K : (uint64_t)op.N * op.H * op.W * op.C;
        if (op.loader != kLoaderDense && (uint64_t)op.N * op.OH * op.OW != (uint64_t)op.M) {
            return fail(THIP_INVALID_ARGUMENT, "op %u: igemm rows do not match the output pixels", i);
        }
        if ((s = need(op.in0, inBytes, "in"))) return s;
        if ((s = need(op.weights, (uint64_t)op.Np * op.Kp, "weights"))) return s;
        if ((s = need(op.bias, (uint64_t)op.Np * 4, "bias"))) return s;
        if ((s = need(op.scale, (uint64_t)op.Np * 4, "scale"))) return s;
        if (op.loader > kLoaderRuns) return fail(THIP_INVALID_ARGUMENT, "op %u: unknown igemm loader %u", i, op.loader);
        if (op.loader == kLoaderRuns) {
            if (op.KW * op.C > 16 || op.Kp % 16 != 0) return fail(THIP_INVALID_ARGUMENT, "op %u: window row of %d bytes does not fit a 16-byte run", i, op.KW * op.C);
            if ((s = need(op.table, (uint64_t)op.Kp / 16 * 4, "table"))) return s;
            if (op.table.space != kSpaceConst) return fail(THIP_INVALID_ARGUMENT, "op %u: table must be a constant", i);
            const uint8_t *base = e->blob.data() + e->header.data_offset + e->consts[op.table.index].offset + op.table.offset;
            for (uint32_t t = 0; t < (uint32_t)op.Kp / 16; t++) {
                uint32_t ent;
                memcpy(&ent, base + 4ull * t, 4);
                if (ent & kKEntryInvalid) continue;
                if ((int)((ent >> 24) & 0x7f) >= op.KH || (int)(ent & 0xffff) != op.KW * op.C) return fail(THIP_INVALID_ARGUMENT, "op %u: run table entry %u is outside the window", i, t);
            }
        }
        if (op.loader == kLoaderGather) {
            if (op.gran == 0 || (op.gran & (op.gran - 1)) || op.gran > 16) return fail(THIP_INVALID_ARGUMENT, "op %u: bad gather granularity", i);
            if ((s = need(op.table, (uint64_t)op.Kp / op.gran * 4, "table"))) return s;
            // every valid table entry must stay inside the window and the channel axis
            const uint8_t *base = e->blob.data() + e->header.data_offset + e->consts[op.table.index].offset + op.table.offset;
            if (op.table.space != kSpaceConst) return fail(THIP_INVALID_ARGUMENT, "op %u: table must be a constant", i);
            for (uint32_t t = 0; t < (uint32_t)op.Kp / op.gran; t++) {
                uint32_t ent;
                memcpy(&ent, base + 4ull * t, 4);
                if (ent & kKEntryInvalid) continue;
                const int kh = (ent >> 24) & 0x7f, kw = (ent >> 16) & 0xff, ci = ent & 0xffff;
                if (kh >= op.KH || kw >= op.KW || ci + (int)op.gran > op.C) return fail(THIP_INVALID_ARGUMENT, "op %u: table entry %u is outside the window", i, t);
            }
        }
        if (op.in1.space != kSpaceNone) {  // fused residual add
            if ((op.variant != kIgemmStream && op.variant != kIgemmDense64x64) || op.loader != kLoaderDense || op.out_dtype != THIP_DTYPE_I8 ||
                op.table.space != kSpaceConst) {
                return fail(THIP_INVALID_ARGUMENT, "op %u: a residual add needs the streaming or the small-tile int8 kernel", i);
            }
            if ((s = need(op.in1, (uint64_t)op.M * op.Nn, "residual"))) return s;
            if ((s = need(op.table, sizeof(ResidualAddParams), "residual parameters"))) return s;
            ResidualAddParams ap;
            memcpy(&ap, e->blob.data() + e->header.data_offset + e->consts[op.table.index].offset + op.table.offset, sizeof(ap));
            if (ap.shift < 0 || ap.shift > 63 || ap.output_min > ap.output_max || ap.output_min < -128 || ap.output_max > 127) {
                return fail(THIP_INVALID_ARGUMENT, "op %u: bad residual add parameters", i);
            }
        }
        return need(op.out, (uint64_t)op.M * op.Nn * outElem, "out");
    }
    case kKindFcSkinny: {
        if (!positive({op.M, op.K, op.Nn})) return fail(THIP_INVALID_ARGUMENT, "op %u: bad fc extents", i);
        if ((s = need(op.in0, (uint64_t)op.M * op.K, "in"))) return s;
        if ((s = need(op.weights, (uint64_t)op.Nn * op.K, "weights"))) return s;
        if ((s = need(op.bias, (uint64_t)op.Nn * 4, "bias"))) return s;
        if ((s = need(op.scale, (uint64_t)op.Nn * 4, "scale"))) return s;
        return need(op.out, (uint64_t)op.M * op.Nn * outElem, "out");
    }
    case kKindDepthwise: {
        if (!positive({op.N, op.H, op.W, op.C, op.OH, op.OW, op.KH, op.KW})) return fail(THIP_INVALID_ARGUMENT, "op %u: bad depthwise extents", i);
        if ((s = need(op.in0, (uint64_t)op.N * op.H * op.W * op.C, "in"))) return s;
        if (op.variant > kDepthwiseDot4Rows) return fail(THIP_INVALID_ARGUMENT, "op %u: unknown depthwise variant %u", i, op.variant);
        if ((s = need(op.weights, op.variant == kDepthwiseDot4Rows ? (uint64_t)op.KH * op.C * 4 : (uint64_t)op.KH * op.KW * op.C, "weights"))) return s;
        if ((s = need(op.bias, (uint64_t)op.C * 4, "bias"))) return s;
        if ((s = need(op.scale, (uint64_t)op.C * 4, "scale"))) return s;
        return need(op.out, (uint64_t)op.N * op.OH * op.OW * op.C, "out");
    }
    case kKindMaxPool: {
        if (!positive({op.N, op.H, op.W, op.C, op.OH, op.OW, op.KH, op.KW})) return fail(THIP_INVALID_ARGUMENT, "op %u: bad maxpool extents", i);
        if ((s = need(op.in0, (uint64_t)op.N * op.H * op.W * op.C, "in"))) return s;
        return need(op.out, (uint64_t)op.N * op.OH * op.OW * op.C, "out");
    }
    case kKindAvgPool: {
        if (!positive({op.N, op.H, op.W, op.C})) return fail(THIP_INVALID_ARGUMENT, "op %u: bad avgpool extents", i);
        if ((s = need(op.in0, (uint64_t)op.N * op.H * op.W * op.C, "in"))) return s;
        return need(op.out, (uint64_t)op.N * op.C, "out");
    }
    case kKindAdd: {
        if (!positive({op.C})) return fail(THIP_INVALID_ARGUMENT, "op %u: bad add extent", i);
        if ((s = need(op.in0, (uint64_t)op.C, "in1"))) return s;
        if ((s = need(op.in1, (uint64_t)op.C, "in2"))) return s;
        return need(op.out, (uint64_t)op.C, "out");
    }
    case kKindIm2colBf16: {
        if (!positive({op.N, op.H, op.W, op.C, op.OH, op.OW, op.KH, op.KW, op.Kp}) || op.Kp < op.KH * op.KW * op.C) {
            return fail(THIP_INVALID_ARGUMENT, "op %u: bad im2col extents", i);
        }
        if ((s = need(op.in0, (uint64_t)op.N * op.H * op.W * op.C * 2, "in"))) return s;
        return need(op.out, (uint64_t)op.N * op.OH * op.OW * op.Kp * 2, "out");
    }
    case kKindDepthwiseBf16: {
        if (!positive({op.N, op.H, op.W, op.C, op.OH, op.OW, op.KH, op.KW})) return fail(THIP_INVALID_ARGUMENT, "op %u: bad depthwise extents", i);
        if ((s = need(op.in0, (uint64_t)op.N * op.H * op.W * op.C * 2, "in"))) return s;
        if ((s = need(op.weights, (uint64_t)op.KH * op.KW * op.C * 2, "weights"))) return s;
        if ((s = need(op.bias, (uint64_t)op.C * 4, "bias"))) return s;
        return need(op.out, (uint64_t)op.N * op.OH * op.OW * op.C * 2, "out");
    }
    case kKindAvgPoolBf16: {
        if (!positive({op.N, op.H, op.W, op.C})) return fail(THIP_INVALID_ARGUMENT, "op %u: bad avgpool extents", i);
        if ((s = need(op.in0, (uint64_t)op.N * op.H * op.W * op.C * 2, "in"))) return s;
        return need(op.out, (uint64_t)op.N * op.C * 2, "out");
    }
    case kKindExpandWeights: {
        const int32_t block = (int32_t)op.gran;
        if (!positive({op.K, op.Nn, block}) || op.K % block != 0 || op.Np < op.Nn) return fail(THIP_INVALID_ARGUMENT, "op %u: bad expand_weights extents", i);
        if ((s = need(op.in0, (uint64_t)op.K * op.Nn, "weights"))) return s;
        if ((s = need(op.scale, (uint64_t)(op.K / block) * op.Nn * 2, "scale"))) return s;
        if ((s = need(op.bias, (uint64_t)(op.K / block) * op.Np * 4, "bias"))) return s;
        return need(op.out, (uint64_t)op.K * op.Nn * 2, "out");
    }
    case kKindEltwise: {
        const uint64_t inElem = op.gran, outElem = op.out_dtype == THIP_DTYPE_I8 ? 1 : op.out_dtype == THIP_DTYPE_I16 ? 2 : op.out_dtype == THIP_DTYPE_I32 ? 4 : 0;
        if (!positive({op.C}) || !(inElem == 1 || inElem == 2 || inElem == 4) || outElem == 0 || op.variant > kEltMax || op.w1 < 0 || op.w1 > 2 ||
            (op.variant != kEltMul && op.w1 != 0)) {
            return fail(THIP_INVALID_ARGUMENT, "op %u: bad elementwise record", i);
        }
        if ((s = need(op.in0, (op.w1 == 1 ? 1 : (uint64_t)op.C) * inElem, "in1"))) return s;
        if ((op.variant == kEltMul || op.variant >= kEltAnd) && (s = need(op.in1, (op.w1 == 2 ? 1 : (uint64_t)op.C) * inElem, "in2"))) return s;
        return need(op.out, (uint64_t)op.C * outElem, "out");
    }
    case kKindAddBf16: {
        if (!positive({op.C})) return fail(THIP_INVALID_ARGUMENT, "op %u: bad add extent", i);
        if ((s = need(op.in0, (uint64_t)op.C * 2, "in1"))) return s;
        if ((s = need(op.in1, (uint64_t)op.C * 2, "in2"))) return s;
        return need(op.out, (uint64_t)op.C * 2, "out");
    }
    case kKindFcBf16: {
        if (!positive({op.M, op.K, op.Nn}) || op.K % 8 != 0) return fail(THIP_INVALID_ARGUMENT, "op %u: bad bf16 fully_connected extents", i);
        if ((s = need(op.in0, (uint64_t)op.M * op.K * 2, "in"))) return s;
        if (op.loader > 2) return fail(THIP_INVALID_ARGUMENT, "op %u: unknown bf16 weight layout %u", i, op.loader);
        const uint64_t padded = (uint64_t)((op.Nn + 31) / 32 * 32) * ((op.K + 63) / 64 * 64);
        const uint64_t wBytes = op.loader == 2 ? padded : op.loader == 1 ? padded * 2 : (uint64_t)op.Nn * op.K * 2;
        if ((s = need(op.weights, wBytes, "weights"))) return s;
        if (op.loader == 2) {
            const int32_t block = (int32_t)op.gran;
            if (block < 32 || block % 32 != 0 || op.K % block != 0 || op.Np < (op.Nn + 31) / 32 * 32 || op.Np % 32 != 0) {
                return fail(THIP_INVALID_ARGUMENT, "op %u: bad block-quantized weight tables", i);
            }
            if ((s = need(op.scale, (uint64_t)(op.K / block) * op.Np * 2, "block scales"))) return s;
            if ((s = need(op.table, (uint64_t)(op.K / block) * op.Np * 4, "block biases"))) return s;
        }
        if ((s = need(op.bias, (uint64_t)op.Nn * 4, "bias"))) return s;
        if (op.w0 > 1) {
            // K split over blocks: counters and partial sums live in an intermediate (zero-filled at creation)
            if (op.w0 > 64 || op.in1.space != kSpaceTemp) return fail(THIP_INVALID_ARGUMENT, "op %u: bad split-K workspace", i);
            if ((s = need(op.in1, fcBf16WorkspaceBytes(op.M, op.Nn, op.w0), "workspace"))) return s;
        }
        return need(op.out, (uint64_t)op.M * op.Nn * 2, "out");
    }
    default: return fail(THIP_INVALID_ARGUMENT, "op %u has unknown kind %u", i, op.kind);
    }
}

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
    default: return "unknown";
    }
}

// One row of the event log, in the reference's runtime CSV columns (doc/user-manual/profiling.md:53-63, written by
// runtime/torq_hw/src/TorqEventLog.cpp:48,97-101): dispatch_name, invocation_id, action_id, timestamp_us, event
// (an EventType name + _BEGIN / _END), plus one column of this backend's own: the kernel of a launch row.
static void logEvent(thip_device_t *d, uint64_t invocation, int32_t action, const char *event, const char *phase, const char *kernel) {
    if (!d->eventLog) return;
    std::lock_guard<std::mutex> lock(d->logMutex);
    const auto us = std::chrono::duration_cast<std::chrono::microseconds>(std::chrono::steady_clock::now() - d->t0).count();
    fprintf(d->eventLog, "thip_dispatch,%llu,%d,%lld,%s_%s,%s\n", (unsigned long long)invocation, action, (long long)us, event, phase, kernel);
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
        EltwiseArgs a{resolve(e, op.in0, bp), (op.variant == kEltMul || op.variant >= kEltAnd) ? resolve(e, op.in1, bp) : nullptr, resolve(e, op.out, bp), (int64_t)op.C,
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

// Enqueues every kernel record of the program.  `bp` holds one device pointer per binding.
static thip_status_t enqueueOps(thip_executable_t *e, uint8_t *const *bp) {
    for (uint32_t i = 0; i < e->header.op_count; i++) {
        // a kernel launch is what starting an NSS task is on the reference's hardware
        logEvent(e->device, e->invocation, (int32_t)i, "NSS_START", "BEGIN", e->kernelNames[i].c_str());
        if (thip_status_t s = launchOp(e, i, bp, LaunchCtx{e->stream, &e->tuning, nullptr, 0})) return s;
        logEvent(e->device, e->invocation, (int32_t)i, "NSS_START", "END", e->kernelNames[i].c_str());
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
    const bool eligible = !e->graphsDisabled && e->header.op_count >= kGraphMinOps && !e->device->eventLog;
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

thip_status_t thip_infer_format(const void *blob, size_t size, size_t format_capacity, char *format, size_t *out_inferred_size) {
    DescHeader h;
    if (thip_status_t s = validateDescriptor((const uint8_t *)blob, size, &h)) return s;
    static const char kFormat[] = "thip-gfx950";
    if (!format || format_capacity < sizeof(kFormat)) return fail(THIP_OUT_OF_RANGE, "format buffer too small");
    memcpy(format, kFormat, sizeof(kFormat));
    if (out_inferred_size) *out_inferred_size = (size_t)h.total_size;
    return THIP_OK;
}

void thip_executable_destroy(thip_executable_t *e) {
    if (!e) return;
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
    for (uint32_t i = 0; i < h.op_count && s == THIP_OK; i++) s = checkOpFootprint(e, i);
    auto bail = [&](thip_status_t code) {
        thip_executable_destroy(e);
        return code;
    };
    if (s != THIP_OK) return bail(s);
    hipError_t err = hipSetDevice(device->ordinal);
    if (err == hipSuccess) err = hipStreamCreate(&e->stream);  // default priority
    if (err == hipSuccess) err = hipEventCreate(&e->evStart);
    if (err == hipSuccess) err = hipEventCreate(&e->evStop);
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
    // Which kernel each record runs is settled now, from the record, the alignment of its operands and the
    // environment's switches, and kept: the launchers are asked in naming mode (they also configure their kernels,
    // which must not happen later inside a stream capture).  Bindings stand in as aligned placeholder addresses:
    // device bindings must be 16-byte aligned and staged host bindings are, so a dispatch resolves the same way.
    e->scratchOffset.assign(h.op_count, 0);
    e->scratchZeroBytes.assign(h.op_count, 0);
    for (uint32_t i = 0; i < h.op_count; i++) {
        const DescOp &op = e->ops[i];
        if (op.kind != kKindFcBf16 || op.w0 <= 1) continue;
        e->scratchOffset[i] = e->scratchBytes;
        e->scratchZeroBytes[i] = fcBf16WorkspaceCounterBytes(op.M, op.Nn, op.w0);
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

static thip_status_t runLocked(thip_executable_t *e, const thip_dispatch_state_t *st) {
    THIP_HIP(hipSetDevice(e->device->ordinal), "hipSetDevice");
    uint8_t *bp[64] = {nullptr};
    const int32_t lastOp = (int32_t)e->header.op_count - 1;
    logEvent(e->device, e->invocation, 0, "DISPATCH", "BEGIN", "");
    logEvent(e->device, e->invocation, 0, "DISPATCH_SYNC_BINDINGS_IN", "BEGIN", "");
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
            THIP_HIP(hipMemcpyAsync(bp[i], st->binding_ptrs[i], e->bindings[i].size, hipMemcpyHostToDevice, e->stream), "staging a binding");
        }
    }
    logEvent(e->device, e->invocation, 0, "DISPATCH_SYNC_BINDINGS_IN", "END", "");
    bool allDevice = true;
    for (uint32_t i = 0; i < e->header.binding_count; i++) {
        if (e->bindings[i].flags != 0 && !(st->binding_flags && (st->binding_flags[i] & THIP_BINDING_DEVICE))) allDevice = false;
    }
    logEvent(e->device, e->invocation, 0, "DISPATCH_EXECUTE_ACTIONS", "BEGIN", "");
    if (thip_status_t s = allDevice ? enqueueDevice(e, bp) : enqueueOps(e, bp)) {
        (void)hipStreamSynchronize(e->stream);
        e->invocation++;
        return s;
    }
    logEvent(e->device, e->invocation, lastOp, "DISPATCH_EXECUTE_ACTIONS", "END", "");
    logEvent(e->device, e->invocation, lastOp, "DISPATCH_SYNC_BINDINGS_OUT", "BEGIN", "");
    // readOutputs (TorqExecutable::readOutputs, runtime/driver/TorqExecutable.cc:860-918)
    for (uint32_t i = 0; i < e->header.binding_count; i++) {
        const bool isDevice = st->binding_flags && (st->binding_flags[i] & THIP_BINDING_DEVICE);
        if (isDevice || !(e->bindings[i].flags & kBindingWritten)) continue;
        THIP_HIP(hipMemcpyAsync(st->binding_ptrs[i], bp[i], e->bindings[i].size, hipMemcpyDeviceToHost, e->stream), "reading back a binding");
    }
    logEvent(e->device, e->invocation, lastOp, "NSS_WAIT", "BEGIN", "");
    const hipError_t waited = hipStreamSynchronize(e->stream);
    logEvent(e->device, e->invocation, lastOp, "NSS_WAIT", "END", "");
    logEvent(e->device, e->invocation, lastOp, "DISPATCH_SYNC_BINDINGS_OUT", "END", "");
    logEvent(e->device, e->invocation, lastOp, "DISPATCH", "END", "");
    e->invocation++;
    THIP_HIP(waited, "waiting for the dispatch");
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
    THIP_HIP(hipSetDevice(e->device->ordinal), "hipSetDevice");
    uint8_t *scratch = e->device->staticScratch;  // the address hipGetSymbolAddress gave for this device
    if (!scratch) return fail(THIP_INTERNAL, "the static scratch array was not located");
    uint8_t *bp[64] = {nullptr};
    for (uint32_t i = 0; i < e->header.binding_count; i++) bp[i] = (uint8_t *)st->binding_ptrs[i];
    const LaunchCtx ctx{e->stream, &e->tuning, nullptr, 0};
    thip_status_t result = THIP_OK;
    for (uint32_t i = 0; i < e->header.op_count && result == THIP_OK; i++) {
        // the array keeps what the last call left there, whoever made it: what has to start at zero is cleared
        if (e->scratchZeroBytes[i]) {
            const hipError_t ze = launchZeroFill(scratch + e->scratchOffset[i], (size_t)e->scratchZeroBytes[i], e->stream);
            if (ze != hipSuccess) result = hipFail(ze, "clearing the scratch counters");
        }
        if (result == THIP_OK) result = launchOp(e, i, bp, ctx, scratch);
    }
    e->invocation++;
    return result;
}

thip_status_t thip_executable_wait(thip_executable_t *e) {
    if (!e) return fail(THIP_INVALID_ARGUMENT, "null executable");
    THIP_HIP(hipStreamSynchronize(e->stream), "waiting for the dispatch");
    return THIP_OK;
}

thip_status_t thip_executable_time(thip_executable_t *e, const thip_dispatch_state_t *st, int32_t iterations, float *out_ms) {
    if (!e || !out_ms) return fail(THIP_INVALID_ARGUMENT, "null argument");
    if (iterations <= 0) return fail(THIP_INVALID_ARGUMENT, "iterations must be positive");
    if (thip_status_t s = checkState(e, st, true)) return s;
    std::lock_guard<std::mutex> lock(e->mutex);
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
    THIP_HIP(hipEventSynchronize(e->evStop), "hipEventSynchronize");
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
    THIP_HIP(hipEventSynchronize(e->evStop), "hipEventSynchronize");
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
