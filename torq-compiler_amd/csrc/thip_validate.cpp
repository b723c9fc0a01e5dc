// Validation of a dispatch descriptor: everything that can be checked without a GPU.  The driver runs it when an
// executable is created (and thip_infer_format / thip_descriptor_validate on their own); nothing here calls HIP, so
// the same code is fuzzed on the host under sanitizers.
#include "thip_validate.h"

#include <string.h>

#include <initializer_list>

#include "thip_kernels.h"
#include "thip_status.h"

namespace thip {

// Tile geometry of the igemm variants (what the emitter pads to and the launchers launch).
static const IgemmTile kTiles[kIgemmVariantCount] = {
    {128, 128, 64, "igemm_i8_128x128x64"},
    {256, 256, 64, "igemm_i8_256x256x64"},
    {64, 64, 64, "igemm_i8_64x64x64"},
    {256, 128, 64, "igemm_i8_256x128x64"},
    {256, 256, 64, "igemm_dense_i8_256x256x64"},
    {128, 128, 64, "igemm_dense_i8_128x128x64"},
    {128, 256, 64, "igemm_dense_i8_128x256x64"},
    {64, 64, 64, "igemm_dense_i8_64x64x64"},
    {256, 128, 64, "igemm_dense_i8_256x128x64"},
    {256, 64, 64, "igemm_dense_i8_256x64x64"},
    {256, 32, 64, "igemm_dense_i8_256x32x64"},
    {32, 32, 32, "igemm_stream_i8"},
    {128, 64, 64, "igemm_dense_i8_128x64x64"},
    {64, 128, 64, "igemm_dense_i8_64x128x64"},
    {256, 256, 128, "igemm_dense_i8_256x256x128"},
};

const IgemmTile &igemmTile(uint32_t variant) {
    return kTiles[variant < kIgemmVariantCount ? variant : 0];
}

// Product of non-negative extents, saturating (a corrupt record must not wrap around to a small number).
template <typename... T>
static uint64_t mul(T... factors) {
    unsigned __int128 p = 1;
    for (int64_t f : {(int64_t)factors...}) {
        if (f < 0) return ~0ull >> 8;
        p *= (uint64_t)f;
        if (p > (~0ull >> 8)) return ~0ull >> 8;
    }
    return (uint64_t)p;
}

thip_status_t validateDescriptor(const uint8_t *p, size_t size, DescHeader *out) {
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
    if ((h.ops_offset | h.bindings_offset | h.temps_offset | h.consts_offset) & 7) return fail(THIP_INVALID_ARGUMENT, "descriptor tables are misaligned");
    if (((uintptr_t)p & 7) != 0) return fail(THIP_INVALID_ARGUMENT, "descriptor must be 8-byte aligned in memory");
    if (h.op_count == 0) return fail(THIP_INVALID_ARGUMENT, "descriptor holds no ops");
    {
        size_t n = 0;
        while (n < sizeof(h.name) && h.name[n]) n++;
        if (n == 0 || n == sizeof(h.name)) return fail(THIP_INVALID_ARGUMENT, "descriptor has no terminated executable name");
        for (size_t k = 0; k < sizeof(h.name); k++) {
            const char c = h.name[k];
            const bool ok = k >= n ? c == 0 : ((c >= 'a' && c <= 'z') || (c >= 'A' && c <= 'Z') || (c >= '0' && c <= '9') || c == '_' || c == '-' || (c == '.' && k > 0) || c == '$');
            if (!ok) return fail(THIP_INVALID_ARGUMENT, "descriptor's executable name is malformed");
        }
    }
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
static uint64_t refRoom(const DescriptorView *e, const DescRef &r) {
    switch (r.space) {
    case kSpaceBinding: return e->bindings[r.index].size - r.offset;
    case kSpaceTemp: return e->temps[r.index].size - r.offset;
    case kSpaceConst: return e->consts[r.index].size - r.offset;
    default: return 0;
    }
}

// An operand reference that does not sit in the record itself (it came out of a constant blob): names an existing
// buffer, at an offset inside it.
static thip_status_t checkLooseRef(const DescriptorView *e, uint32_t i, const DescRef &r) {
    uint64_t limit = 0;
    switch (r.space) {
    case kSpaceNone: return THIP_OK;
    case kSpaceBinding:
        if (r.index >= e->header.binding_count) return fail(THIP_INVALID_ARGUMENT, "op %u names binding %u of %u", i, r.index, e->header.binding_count);
        limit = e->bindings[r.index].size;
        break;
    case kSpaceTemp:
        if (r.index >= e->header.temp_count) return fail(THIP_INVALID_ARGUMENT, "op %u names intermediate %u of %u", i, r.index, e->header.temp_count);
        limit = e->temps[r.index].size;
        break;
    case kSpaceConst:
        if (r.index >= e->header.const_count) return fail(THIP_INVALID_ARGUMENT, "op %u names constant %u of %u", i, r.index, e->header.const_count);
        limit = e->consts[r.index].size;
        break;
    default: return fail(THIP_INVALID_ARGUMENT, "op %u has an operand in unknown space %u", i, r.space);
    }
    if (r.offset > limit) return fail(THIP_INVALID_ARGUMENT, "op %u operand offset %llu is past its buffer (%llu)", i, (unsigned long long)r.offset, (unsigned long long)limit);
    return THIP_OK;
}

// Checks, once at creation, that every kernel record stays inside the buffers it names.
thip_status_t checkOpFootprint(const DescriptorView *e, uint32_t i) {
    const DescOp &op = e->ops[i];
    auto need = [&](const DescRef &r, uint64_t bytes, const char *name) -> thip_status_t {
        if (r.space == kSpaceNone) return fail(THIP_INVALID_ARGUMENT, "op %u: operand %s is missing", i, name);
        if (bytes >= (1ull << 48)) return fail(THIP_INVALID_ARGUMENT, "op %u: operand %s has an absurd extent", i, name);
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
    switch (op.kind) {
    case kKindTranspose: {
        if (!positive({op.TB, op.TR, op.TS})) return fail(THIP_INVALID_ARGUMENT, "op %u: bad transpose extents", i);
        if (op.gran > 2) return fail(THIP_INVALID_ARGUMENT, "op %u: transpose element size %u", i, op.gran);
        if (op.TP != 0 && op.TP < op.TR) return fail(THIP_INVALID_ARGUMENT, "op %u: transpose pitch %d is below its row length %d", i, op.TP, op.TR);
        const uint64_t elem = op.gran == 2 ? 2 : 1, pitch = op.TP ? (uint64_t)op.TP : (uint64_t)op.TR;
        if ((s = need(op.in0, mul(op.TB, op.TR, op.TS) * elem, "in"))) return s;
        return need(op.out, mul(op.TB, op.TS) * pitch * elem, "out");
    }
    case kKindIgemm: {
        if (!positive({op.M, op.K, op.Kp, op.Nn, op.Np, op.N, op.H, op.W, op.C, op.OH, op.OW})) {
            return fail(THIP_INVALID_ARGUMENT, "op %u: bad igemm extents", i);
        }
        if (op.variant >= kIgemmVariantCount) return fail(THIP_INVALID_ARGUMENT, "op %u: unknown igemm variant %u", i, op.variant);
        const uint64_t inBytes = op.loader == kLoaderDense ? mul(op.M, op.K) : mul(op.N, op.H, op.W, op.C);
        if (op.loader != kLoaderDense && mul(op.N, op.OH, op.OW) != (uint64_t)op.M) {
            return fail(THIP_INVALID_ARGUMENT, "op %u: igemm rows do not match the output pixels", i);
        }
        if (op.loader == kLoaderDense && mul(op.N, op.H, op.W, op.C) != mul(op.M, op.K)) {
            return fail(THIP_INVALID_ARGUMENT, "op %u: the dense operand's image view is not its M x K matrix", i);
        }
        if ((s = need(op.in0, inBytes, "in"))) return s;
        if ((s = need(op.weights, mul(op.Np, op.Kp), "weights"))) return s;
        if ((s = need(op.bias, (uint64_t)op.Np * 4, "bias"))) return s;
        if ((s = need(op.scale, (uint64_t)op.Np * 4, "scale"))) return s;
        if (op.loader > kLoaderWindow) return fail(THIP_INVALID_ARGUMENT, "op %u: unknown igemm loader %u", i, op.loader);
        if (op.loader == kLoaderWindow) {
            const int32_t bk = igemmTile(op.variant).bk;
            if (!positive({op.KH, op.KW, op.SH, op.SW}) || op.PT < 0 || op.PL < 0 || op.C < 16 || op.C % 16 != 0 || mul(op.KH, op.KW, op.C) != (uint64_t)op.K || op.Kp != (op.K + bk - 1) / bk * bk) {
                return fail(THIP_INVALID_ARGUMENT, "op %u: the window loader needs a multiple of 16 channels and K rounded up to whole k-tiles", i);
            }
            if (inBytes >= (1ull << 32)) return fail(THIP_INVALID_ARGUMENT, "op %u: image too large for the window loader", i);
            switch (op.variant) {
            case kIgemmDense256x256: case kIgemmDense128x256: case kIgemmDense128x128: case kIgemmDense256x128: case kIgemmDense256x64: case kIgemmDense64x64: case kIgemmDense256x32: case kIgemmDense256x256K128: break;
            default: return fail(THIP_INVALID_ARGUMENT, "op %u: the window loader has no kernel for tile variant %u", i, op.variant);
            }
            if (op.table.space != kSpaceConst) return fail(THIP_INVALID_ARGUMENT, "op %u: table must be a constant", i);
            if ((s = need(op.table, 128, "zero-point page"))) return s;
            const uint8_t *page = e->blob + e->header.data_offset + e->consts[op.table.index].offset + op.table.offset;
            for (int b = 0; b < 128; b++) {
                if ((int8_t)page[b] != (int8_t)op.input_zp) return fail(THIP_INVALID_ARGUMENT, "op %u: the zero-point page does not hold input_zp", i);
            }
        }
        if (op.loader == kLoaderRuns) {
            if (!positive({op.KH, op.KW}) || (int64_t)op.KW * op.C > 16 || op.Kp % 16 != 0) return fail(THIP_INVALID_ARGUMENT, "op %u: a window row of %d x %d bytes does not fit a 16-byte run", i, op.KW, op.C);
            if (inBytes < 16) return fail(THIP_INVALID_ARGUMENT, "op %u: the run loader reads 16 bytes at a time, the image has %llu", i, (unsigned long long)inBytes);
            if (op.table.space != kSpaceConst) return fail(THIP_INVALID_ARGUMENT, "op %u: table must be a constant", i);
            if ((s = need(op.table, (uint64_t)op.Kp / 16 * 4, "table"))) return s;
            const uint8_t *base = e->blob + e->header.data_offset + e->consts[op.table.index].offset + op.table.offset;
            for (uint32_t t = 0; t < (uint32_t)op.Kp / 16; t++) {
                uint32_t ent;
                memcpy(&ent, base + 4ull * t, 4);
                if (ent & kKEntryInvalid) continue;
                if ((int)((ent >> 24) & 0x7f) >= op.KH || (int)(ent & 0xffff) != op.KW * op.C) return fail(THIP_INVALID_ARGUMENT, "op %u: run table entry %u is outside the window", i, t);
            }
        }
        if (op.loader == kLoaderGather) {
            if (op.gran == 0 || (op.gran & (op.gran - 1)) || op.gran > 16) return fail(THIP_INVALID_ARGUMENT, "op %u: bad gather granularity", i);
            if (op.table.space != kSpaceConst) return fail(THIP_INVALID_ARGUMENT, "op %u: table must be a constant", i);
            if ((s = need(op.table, (uint64_t)op.Kp / op.gran * 4, "table"))) return s;
            // every valid table entry must stay inside the window and the channel axis
            const uint8_t *base = e->blob + e->header.data_offset + e->consts[op.table.index].offset + op.table.offset;
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
            if ((s = need(op.in1, mul(op.M, op.Nn), "residual"))) return s;
            if ((s = need(op.table, sizeof(ResidualAddParams), "residual parameters"))) return s;
            ResidualAddParams ap;
            memcpy(&ap, e->blob + e->header.data_offset + e->consts[op.table.index].offset + op.table.offset, sizeof(ap));
            if (ap.shift < 0 || ap.shift > 63 || ap.output_min > ap.output_max || ap.output_min < -128 || ap.output_max > 127) {
                return fail(THIP_INVALID_ARGUMENT, "op %u: bad residual add parameters", i);
            }
        }
        return need(op.out, mul(op.M, op.Nn) * outElem, "out");
    }
    case kKindFcSkinny: {
        if (!positive({op.M, op.K, op.Nn})) return fail(THIP_INVALID_ARGUMENT, "op %u: bad fc extents", i);
        if ((s = need(op.in0, mul(op.M, op.K), "in"))) return s;
        if ((s = need(op.weights, mul(op.Nn, op.K), "weights"))) return s;
        if ((s = need(op.bias, (uint64_t)op.Nn * 4, "bias"))) return s;
        if ((s = need(op.scale, (uint64_t)op.Nn * 4, "scale"))) return s;
        return need(op.out, mul(op.M, op.Nn) * outElem, "out");
    }
    case kKindDepthwise: {
        if (!positive({op.N, op.H, op.W, op.C, op.OH, op.OW, op.KH, op.KW})) return fail(THIP_INVALID_ARGUMENT, "op %u: bad depthwise extents", i);
        if ((s = need(op.in0, mul(op.N, op.H, op.W, op.C), "in"))) return s;
        if (op.variant > kDepthwiseDot4Rows) return fail(THIP_INVALID_ARGUMENT, "op %u: unknown depthwise variant %u", i, op.variant);
        if ((s = need(op.weights, op.variant == kDepthwiseDot4Rows ? mul(op.KH, op.C) * 4 : mul(op.KH, op.KW, op.C), "weights"))) return s;
        if ((s = need(op.bias, (uint64_t)op.C * 4, "bias"))) return s;
        if ((s = need(op.scale, (uint64_t)op.C * 4, "scale"))) return s;
        return need(op.out, mul(op.N, op.OH, op.OW, op.C), "out");
    }
    case kKindMaxPool: {
        if (!positive({op.N, op.H, op.W, op.C, op.OH, op.OW, op.KH, op.KW})) return fail(THIP_INVALID_ARGUMENT, "op %u: bad maxpool extents", i);
        if ((s = need(op.in0, mul(op.N, op.H, op.W, op.C), "in"))) return s;
        return need(op.out, mul(op.N, op.OH, op.OW, op.C), "out");
    }
    case kKindAvgPool: {
        if (!positive({op.N, op.H, op.W, op.C})) return fail(THIP_INVALID_ARGUMENT, "op %u: bad avgpool extents", i);
        if ((s = need(op.in0, mul(op.N, op.H, op.W, op.C), "in"))) return s;
        return need(op.out, mul(op.N, op.C), "out");
    }
    case kKindAdd: {
        if (!positive({op.C})) return fail(THIP_INVALID_ARGUMENT, "op %u: bad add extent", i);
        if ((s = need(op.in0, (uint64_t)op.C, "in1"))) return s;
        if ((s = need(op.in1, (uint64_t)op.C, "in2"))) return s;
        return need(op.out, (uint64_t)op.C, "out");
    }
    case kKindIm2colBf16: {
        if (!positive({op.N, op.H, op.W, op.C, op.OH, op.OW, op.KH, op.KW, op.Kp}) || (uint64_t)op.Kp < mul(op.KH, op.KW, op.C)) {
            return fail(THIP_INVALID_ARGUMENT, "op %u: bad im2col extents", i);
        }
        if ((s = need(op.in0, mul(op.N, op.H, op.W, op.C) * 2, "in"))) return s;
        return need(op.out, mul(op.N, op.OH, op.OW, op.Kp) * 2, "out");
    }
    case kKindDepthwiseBf16: {
        if (!positive({op.N, op.H, op.W, op.C, op.OH, op.OW, op.KH, op.KW})) return fail(THIP_INVALID_ARGUMENT, "op %u: bad depthwise extents", i);
        if ((s = need(op.in0, mul(op.N, op.H, op.W, op.C) * 2, "in"))) return s;
        if ((s = need(op.weights, mul(op.KH, op.KW, op.C) * 2, "weights"))) return s;
        if ((s = need(op.bias, (uint64_t)op.C * 4, "bias"))) return s;
        return need(op.out, mul(op.N, op.OH, op.OW, op.C) * 2, "out");
    }
    case kKindAvgPoolBf16: {
        if (!positive({op.N, op.H, op.W, op.C})) return fail(THIP_INVALID_ARGUMENT, "op %u: bad avgpool extents", i);
        if ((s = need(op.in0, mul(op.N, op.H, op.W, op.C) * 2, "in"))) return s;
        return need(op.out, mul(op.N, op.C) * 2, "out");
    }
    case kKindExpandWeights: {
        const int32_t block = (int32_t)op.gran;
        if (!positive({op.K, op.Nn, block}) || op.K % block != 0 || op.Np < op.Nn) return fail(THIP_INVALID_ARGUMENT, "op %u: bad expand_weights extents", i);
        if ((s = need(op.in0, mul(op.K, op.Nn), "weights"))) return s;
        if ((s = need(op.scale, (uint64_t)(op.K / block) * op.Nn * 2, "scale"))) return s;
        if ((s = need(op.bias, (uint64_t)(op.K / block) * op.Np * 4, "bias"))) return s;
        return need(op.out, mul(op.K, op.Nn) * 2, "out");
    }
    case kKindEltwise: {
        const uint64_t inElem = op.gran, outElem = op.out_dtype == THIP_DTYPE_I8 ? 1 : op.out_dtype == THIP_DTYPE_I16 ? 2 : op.out_dtype == THIP_DTYPE_I32 ? 4 : 0;
        if (!positive({op.C}) || !(inElem == 1 || inElem == 2 || inElem == 4) || outElem == 0 || op.variant > kEltLast || op.w1 < 0 || op.w1 > 2 ||
            (op.variant != kEltMul && op.w1 != 0)) {
            return fail(THIP_INVALID_ARGUMENT, "op %u: bad elementwise record", i);
        }
        if ((s = need(op.in0, (op.w1 == 1 ? 1 : (uint64_t)op.C) * inElem, "in1"))) return s;
        if (op.variant == kEltTable) {
            if (inElem > 2 || outElem > 2 || outElem < inElem || op.in1.space != kSpaceConst) return fail(THIP_INVALID_ARGUMENT, "op %u: bad table record", i);
            if ((s = need(op.in1, 256 * outElem, "table"))) return s;
            return need(op.out, (uint64_t)op.C * outElem, "out");
        }
        if (eltwiseTwoInputs((int32_t)op.variant) && (s = need(op.in1, (op.w1 == 2 ? 1 : (uint64_t)op.C) * inElem, "in2"))) return s;
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
        if ((s = need(op.in0, mul(op.M, op.K) * 2, "in"))) return s;
        if (op.loader > 2) return fail(THIP_INVALID_ARGUMENT, "op %u: unknown bf16 weight layout %u", i, op.loader);
        const uint64_t padded = (((uint64_t)op.Nn + 31) / 32 * 32) * (((uint64_t)op.K + 63) / 64 * 64);
        const uint64_t wBytes = op.loader == 2 ? padded : op.loader == 1 ? padded * 2 : mul(op.Nn, op.K) * 2;
        if ((s = need(op.weights, wBytes, "weights"))) return s;
        if (op.loader == 2) {
            const int32_t block = (int32_t)op.gran;
            if (block < 32 || block % 32 != 0 || op.K % block != 0 || (int64_t)op.Np < ((int64_t)op.Nn + 31) / 32 * 32 || op.Np % 32 != 0) {
                return fail(THIP_INVALID_ARGUMENT, "op %u: bad block-quantized weight tables", i);
            }
            if ((s = need(op.scale, (uint64_t)(op.K / block) * op.Np * 2, "block scales"))) return s;
            if ((s = need(op.table, (uint64_t)(op.K / block) * op.Np * 4, "block biases"))) return s;
        }
        if ((s = need(op.bias, (uint64_t)op.Nn * 4, "bias"))) return s;
        if (op.w0 > 1) {
            // K split over blocks: the partial sums live in an intermediate of the record's own
            if (op.w0 > 16 || op.in1.space != kSpaceTemp) return fail(THIP_INVALID_ARGUMENT, "op %u: bad split-K workspace", i);
            if ((s = need(op.in1, fcBf16WorkspaceBytes(op.M, op.Nn, op.w0), "workspace"))) return s;
        }
        return need(op.out, mul(op.M, op.Nn) * 2, "out");
    }
    case kKindDecLinear: {
        if (!positive({op.M, op.K}) || op.M > kDecMaxRows || op.K % 128 != 0 || op.gran == 0 || op.gran % 128 != 0 || (uint32_t)op.K % op.gran != 0 ||
            op.w0 < 1 || op.w0 > kDecMaxSegments || (op.w1 & ~(kDecPair | kDecAddResidual | kDecAddPair | kDecResFirst))) {
            return fail(THIP_INVALID_ARGUMENT, "op %u: bad grouped-linear record", i);
        }
        const bool pair = op.w1 & kDecPair, addRes = op.w1 & kDecAddResidual, addPair = op.w1 & kDecAddPair;
        if ((pair && op.w0 != 2) || pair != addPair || (addRes && (addPair || op.w0 != 1))) return fail(THIP_INVALID_ARGUMENT, "op %u: bad grouped-linear flags", i);
        if ((s = need(op.in0, mul(op.M, op.K) * 2, "in"))) return s;
        if (op.table.space != kSpaceConst) return fail(THIP_INVALID_ARGUMENT, "op %u: the per-matrix operands must be a constant", i);
        if ((s = need(op.table, sizeof(DecLinearExt), "per-matrix operands"))) return s;
        if ((op.table.offset & 7) != 0) return fail(THIP_INVALID_ARGUMENT, "op %u: misaligned per-matrix operands", i);
        DecLinearExt x;
        memcpy(&x, e->blob + e->header.data_offset + e->consts[op.table.index].offset + op.table.offset, sizeof(x));
        if (x.has_qbias != 0 && x.has_qbias != 1) return fail(THIP_INVALID_ARGUMENT, "op %u: bad block-bias flag", i);
        for (int m = 0; m < op.w0; m++) {
            const DescRef *refs[] = {&x.weights[m], &x.bias[m], &x.out[m]};
            for (const DescRef *r : refs) {
                if ((s = checkLooseRef(e, i, *r))) return s;
            }
            if (x.N[m] <= 0 || x.N[m] % 16 != 0 || x.N[m] > (1 << 24)) return fail(THIP_INVALID_ARGUMENT, "op %u: matrix %d has %d columns", i, m, x.N[m]);
            if ((s = need(x.weights[m], decWeightBytes(x.N[m], op.K, x.has_qbias != 0), "weights"))) return s;
            if ((s = need(x.bias[m], (uint64_t)x.N[m] * 4, "bias"))) return s;
            if (x.out[m].space == kSpaceNone) {
                if (!addRes && !addPair) return fail(THIP_INVALID_ARGUMENT, "op %u: matrix %d has no destination", i, m);
            } else if ((s = need(x.out[m], mul(op.M, x.N[m]) * 2, "out"))) {
                return s;
            }
            if ((x.weights[m].offset & 15) || (x.bias[m].offset & 15) || (x.out[m].offset & 7)) {
                return fail(THIP_INVALID_ARGUMENT, "op %u: misaligned operand of matrix %d", i, m);
            }
        }
        if (pair && x.N[0] != x.N[1]) return fail(THIP_INVALID_ARGUMENT, "op %u: a pair of unequal widths", i);
        if (addRes || addPair) {
            if ((s = checkLooseRef(e, i, x.res)) || (s = checkLooseRef(e, i, x.add_out))) return s;
            if (addRes && (s = need(x.res, mul(op.M, x.N[0]) * 2, "residual"))) return s;
            if ((s = need(x.add_out, mul(op.M, x.N[0]) * 2, "sum"))) return s;
            if ((x.res.offset & 7) || (x.add_out.offset & 7)) return fail(THIP_INVALID_ARGUMENT, "op %u: misaligned operand of the folded add", i);
        }
        if ((op.in0.offset & 15) != 0) return fail(THIP_INVALID_ARGUMENT, "op %u: misaligned input", i);
        return THIP_OK;
    }
    case kKindDecMatmul: {
        if (!positive({op.TB, op.M, op.K, op.Nn}) || op.M > kDecMaxRows || op.K % 8 != 0 || op.TB > 65535) return fail(THIP_INVALID_ARGUMENT, "op %u: bad batched-matmul extents", i);
        if ((s = need(op.in0, mul(op.w0 ? 1 : op.TB, op.M, op.K) * 2, "in1"))) return s;
        if ((s = need(op.weights, mul(op.w1 ? 1 : op.TB, op.Nn, op.K) * 2, "in2"))) return s;
        if ((op.in0.offset & 15) || (op.weights.offset & 15) || (op.out.offset & 7)) return fail(THIP_INVALID_ARGUMENT, "op %u: misaligned operand", i);
        return need(op.out, mul(op.TB, op.M, op.Nn) * 2, "out");
    }
    default: return fail(THIP_INVALID_ARGUMENT, "op %u has unknown kind %u", i, op.kind);
    }
}

thip_status_t validateWhole(const uint8_t *blob, size_t size, DescHeader *out) {
    DescHeader h;
    if (thip_status_t s = validateDescriptor(blob, size, &h)) return s;
    const DescriptorView v{blob, h, (const DescOp *)(blob + h.ops_offset), (const DescBinding *)(blob + h.bindings_offset),
                           (const DescTemp *)(blob + h.temps_offset), (const DescConst *)(blob + h.consts_offset)};
    for (uint32_t i = 0; i < h.op_count; i++) {
        if (thip_status_t s = checkOpFootprint(&v, i)) return s;
    }
    if (out) *out = h;
    return THIP_OK;
}

}  // namespace thip

extern "C" thip_status_t thip_descriptor_validate(const void *blob, size_t size) {
    return thip::validateWhole((const uint8_t *)blob, size, nullptr);
}

extern "C" thip_status_t thip_descriptor_info(const void *blob, size_t size, thip_descriptor_info_t *out) {
    if (!out) return thip::fail(THIP_INVALID_ARGUMENT, "null result pointer");
    thip::DescHeader h;
    if (thip_status_t s = thip::validateWhole((const uint8_t *)blob, size, &h)) return s;
    memset(out, 0, sizeof(*out));
    memcpy(out->executable_name, h.name, sizeof(h.name));
    out->runtime_version = h.version;
    out->hw_id = h.arch;
    out->action_count = h.op_count;
    out->binding_count = h.binding_count;
    out->segment_count = h.const_count;
    out->intermediate_count = h.temp_count;
    const thip::DescTemp *temps = (const thip::DescTemp *)((const uint8_t *)blob + h.temps_offset);
    for (uint32_t i = 0; i < h.temp_count; i++) out->intermediate_bytes += temps[i].size;
    out->total_size = h.total_size;
    return THIP_OK;
}

extern "C" thip_status_t thip_descriptor_binding(const void *blob, size_t size, uint32_t index, thip_binding_info_t *out) {
    if (!out) return thip::fail(THIP_INVALID_ARGUMENT, "null result pointer");
    thip::DescHeader h;
    if (thip_status_t s = thip::validateWhole((const uint8_t *)blob, size, &h)) return s;
    if (index >= h.binding_count) return thip::fail(THIP_OUT_OF_RANGE, "binding %u of %u", index, h.binding_count);
    const thip::DescBinding &b = ((const thip::DescBinding *)((const uint8_t *)blob + h.bindings_offset))[index];
    memset(out, 0, sizeof(*out));
    out->id = b.id;
    out->address = 0;  // bindings are passed as pointers with each dispatch; nothing is mapped at a fixed address
    out->offset = 0;   // always from the start of the binding's buffer
    out->size = b.size;
    out->is_read_only = (b.flags & thip::kBindingRead) && !(b.flags & thip::kBindingWritten);
    out->is_write_only = (b.flags & thip::kBindingWritten) && !(b.flags & thip::kBindingRead);
    out->is_used = b.flags != 0;
    return THIP_OK;
}

extern "C" thip_status_t thip_descriptor_segment(const void *blob, size_t size, uint32_t index, thip_segment_info_t *out) {
    if (!out) return thip::fail(THIP_INVALID_ARGUMENT, "null result pointer");
    thip::DescHeader h;
    if (thip_status_t s = thip::validateWhole((const uint8_t *)blob, size, &h)) return s;
    if (index >= h.const_count) return thip::fail(THIP_OUT_OF_RANGE, "segment %u of %u", index, h.const_count);
    const thip::DescConst &c = ((const thip::DescConst *)((const uint8_t *)blob + h.consts_offset))[index];
    out->address = c.offset;
    out->size = c.size;
    out->data = (const uint8_t *)blob + h.data_offset + c.offset;
    return THIP_OK;
}

extern "C" thip_status_t thip_infer_format(const void *blob, size_t size, size_t format_capacity, char *format, size_t *out_inferred_size) {
    thip::DescHeader h;
    if (thip_status_t s = thip::validateWhole((const uint8_t *)blob, size, &h)) return s;
    static const char kFormat[] = "thip-gfx950";
    if (!format || format_capacity < sizeof(kFormat)) return thip::fail(THIP_OUT_OF_RANGE, "format buffer too small");
    memcpy(format, kFormat, sizeof(kFormat));
    if (out_inferred_size) *out_inferred_size = (size_t)h.total_size;
    return THIP_OK;
}
