// Compile side: a TorqHL-level program (the ops that the reference's
// Linalg->TorqHL patterns produce, with the reference's operand and attribute
// names) is turned into a dispatch descriptor for the gfx950 kernels.
//
// This takes the place of the NPU-specific tail of the reference pipeline:
//   * KernelSelection (compiler/torq/Codegen/KernelSelectionPass.cpp:411-636):
//     there weights become O/4.I.H.W.4 blocks for the NPU ALU; here they become a
//     K-contiguous [Np][Kp] matrix, k = (kh, kw, ci), zero padded to whole tiles,
//     which is what one lane of v_mfma_i32_32x32x32_i8 reads with a 128-bit load.
//   * EncodeTensors / scale_bias handling: the interleaved [bias, scale] vector
//     (compiler/torq/Utils/ConversionUtils.cpp:88-103) is split into two arrays.
//   * ConvertNhwcOpToNchw + OptimizeTransposeLayout
//     (compiler/torq/Transforms/Linalg/ConvertNhwcOpToNchwPass.cpp:308-321):
//     the ops arrive NCHW; kernels run NHWC.  Intermediates stay NHWC in memory,
//     so transposes only materialise at NCHW bindings.
//   * serializeTorqHW (compiler/torq/Serialization/Serialization.cpp:265-302).
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <map>
#include <string>
#include <vector>

#include "thip_descriptor.h"
#include "thip_kernels.h"
#include "thip_status.h"

namespace thip {

// kValueView: `shape` elements of value `base` starting `viewOffset` elements into it (thip_program_view); `base`
// is a binding or an intermediate, never another view
enum ValueKind { kValueBinding = 0, kValueConstant = 1, kValueTensor = 2, kValueView = 3 };

struct Value {
    ValueKind kind;
    int32_t dtype;
    int32_t rank;
    int64_t shape[THIP_MAX_RANK];
    uint32_t binding;
    thip_value_t base = -1;
    int64_t viewOffset = 0;
    std::vector<uint8_t> data;
    int64_t numel() const {
        int64_t n = 1;
        for (int i = 0; i < rank; i++) n *= shape[i];
        return n;
    }
};

enum HlKind { kHlConv2d, kHlDepthwise, kHlFullyConnected, kHlMatmul, kHlMaxPool, kHlAvgPool, kHlAdd, kHlTranspose, kHlExpandWeights, kHlFma, kHlMul, kHlAct, kHlBinary, kHlUnary, kHlShift, kHlTable };

struct HlOp {
    HlKind kind;
    union Body {
        thip_hl_conv2d_t conv;
        thip_hl_depthwise_conv2d_t dw;
        thip_hl_fully_connected_t fc;
        thip_hl_matmul_t mm;
        thip_hl_maxpool2d_t mp;
        thip_hl_avg_pool2d_t ap;
        thip_hl_add_t add;
        thip_hl_transpose_t tr;
        thip_hl_expand_weights_t ew;
        thip_hl_fma_t fma;
        thip_hl_mul_t mul;
        thip_hl_act_t act;
        thip_hl_elementwisebinary_t bin;
        thip_hl_elementwiseunary_t un;
        thip_hl_elementwiseshift_t sh;
        thip_hl_table_t tab;
    } u;
    std::string name;
    std::vector<int32_t> staticTable;  // torq_hl.table: the caller's static_table, copied
};

}  // namespace thip

struct thip_program_t {
    std::vector<thip::Value> values;
    std::vector<thip::HlOp> ops;
    std::string name = "thip_dispatch";
};

namespace thip {

static size_t elemSize(int32_t dtype) {
    switch (dtype) {
    case THIP_DTYPE_I8: return 1;
    case THIP_DTYPE_I16: return 2;
    case THIP_DTYPE_I32: return 4;
    case THIP_DTYPE_BF16: return 2;
    case THIP_DTYPE_F32: return 4;
    case THIP_DTYPE_I1: return 1;
    default: return 0;
    }
}

static int64_t roundUp(int64_t v, int64_t m) { return (v + m - 1) / m * m; }

// Where a value lives while the program is being laid out.
struct ValState {
    bool defined = false;
    DescRef ref = {kSpaceNone, 0, 0};
    // The tensor is declared N,C,H,W but stored N,H,W,C (an intermediate between
    // two NCHW ops: the transposes the reference inserts around each cancel).
    bool nhwcOfNchw = false;
};

struct Dims4 {
    int64_t N, C, H, W;
};

class Emitter {
  public:
    explicit Emitter(const thip_program_t &prog) : prog_(prog), state_(prog.values.size()) {}

    thip_status_t run(void **outBlob, size_t *outSize);
    // The tile a GEMM-shaped record of this geometry gets (the rule emitIgemm applies), for thip_gemm_tile_choice.
    static uint32_t tileChoice(uint32_t loader, int64_t M, int64_t N, int64_t K, int64_t C, int32_t outDtype, bool addFollows) {
        return loader == kLoaderWindow ? chooseWindowVariant(M, N, C, K)
                                       : chooseIgemmVariant(M, N, loader == kLoaderDense, K, outDtype, loader == kLoaderRuns, addFollows);
    }

  private:
    const thip_program_t &prog_;
    std::vector<ValState> state_;
    std::vector<DescOp> ops_;
    std::vector<uint64_t> temps_;
    std::vector<std::vector<uint8_t>> consts_;
    std::map<uint32_t, DescBinding> bindings_;
    // Physical channel count of an intermediate whose channels are padded to a multiple of 16
    // (0 = stored as declared).  See planChannelPadding.
    std::vector<int> valueReads_;  // per value: how many op inputs name it (planExpandFolding fills it)
    bool addFollows_ = false;      // the convolution being emitted is read by one op only, the torq_hl.add right behind it
    std::vector<int64_t> cpad_;
    std::vector<int64_t> cdeclared_;  // declared channel count of a padded intermediate

    int64_t physC(thip_value_t id, int64_t C) const {
        return (id >= 0 && (size_t)id < cpad_.size() && cpad_[id]) ? cpad_[id] : C;
    }
    // Elements the value occupies in memory (its channel axis possibly padded).
    int64_t physNumel(thip_value_t id) const {
        const int64_t n = prog_.values[id].numel();
        return cpad_[id] ? n / cdeclared_[id] * cpad_[id] : n;
    }
    void planChannelPadding();
    // torq_hl.expand_weights ops that emit no kernel: every operand a constant and the result read once, as
    // input2 of a bf16 matmul, which then takes the block-quantized weights itself (value id of the result ->
    // the op).  THIP_NO_EXPAND_FOLD keeps every expand_weights a kernel of its own.
    std::map<thip_value_t, const thip_hl_expand_weights_t *> foldedExpand_;
    void planExpandFolding();
    // Folds a torq_hl.add record into the pixel-streaming convolution record right before it that produces one of
    // its operands, when nobody else reads that operand (THIP_NO_ADD_FUSION leaves them apart).
    void fuseResidualAdd();

    thip_status_t checkValue(thip_value_t v, const char *what, const Value **out) const {
        if (v < 0 || (size_t)v >= prog_.values.size()) {
            return fail(THIP_INVALID_ARGUMENT, "%s: value %d does not exist", what, (int)v);
        }
        *out = &prog_.values[v];
        return THIP_OK;
    }

    DescRef newTemp(uint64_t size) {
        temps_.push_back(size);
        return DescRef{kSpaceTemp, (uint32_t)(temps_.size() - 1), 0};
    }

    template <typename T>
    DescRef newConst(const std::vector<T> &data) {
        std::vector<uint8_t> bytes(data.size() * sizeof(T));
        if (!bytes.empty()) memcpy(bytes.data(), data.data(), bytes.size());
        consts_.push_back(std::move(bytes));
        return DescRef{kSpaceConst, (uint32_t)(consts_.size() - 1), 0};
    }

    DescRef bindingRef(const Value &v, bool written) {
        DescBinding &b = bindings_[v.binding];
        b.id = v.binding;
        b.flags |= written ? kBindingWritten : kBindingRead;
        b.size = std::max<uint64_t>(b.size, (uint64_t)v.numel() * elemSize(v.dtype));
        return DescRef{kSpaceBinding, v.binding, 0};
    }

    // Reference to the bytes of an input value exactly as declared.
    thip_status_t literalInput(thip_value_t id, const char *what, DescRef *out) {
        const Value *v;
        if (thip_status_t s = checkValue(id, what, &v)) return s;
        if (v->kind == kValueBinding) {
            *out = bindingRef(*v, false);
        } else if (v->kind == kValueView) {
            if (thip_status_t s = literalInput(v->base, what, out)) return s;
            if (state_[v->base].nhwcOfNchw) return fail(THIP_UNIMPLEMENTED, "%s: a view of an N,C,H,W intermediate", what);
            out->offset += (uint64_t)v->viewOffset * elemSize(v->dtype);
        } else if (v->kind == kValueConstant) {
            if (!state_[id].defined) {
                state_[id].ref = newConst(v->data);
                state_[id].defined = true;
            }
            *out = state_[id].ref;
        } else {
            if (!state_[id].defined) {
                return fail(THIP_FAILED_PRECONDITION, "%s: intermediate tensor %d is read before any op writes it",
                            what, (int)id);
            }
            *out = state_[id].ref;
        }
        return THIP_OK;
    }

    void emitTranspose(DescRef in, DescRef out, int64_t B, int64_t R, int64_t S, uint32_t elem = 1, int64_t outPitch = 0) {
        DescOp op;
        memset(&op, 0, sizeof(op));
        op.kind = kKindTranspose;
        op.gran = elem;
        op.TB = (int32_t)B;
        op.TR = (int32_t)R;
        op.TS = (int32_t)S;
        op.TP = (int32_t)outPitch;
        op.in0 = in;
        op.out = out;
        ops_.push_back(op);
    }

    // A 4-D int8 activation operand, delivered to the kernel as NHWC.
    thip_status_t nhwcInput(thip_value_t id, bool declaredNhwc, const char *what, Dims4 *dims, DescRef *out,
                            int32_t dtype = THIP_DTYPE_I8) {
        const Value *v;
        if (thip_status_t s = checkValue(id, what, &v)) return s;
        if (v->rank != 4) return fail(THIP_INVALID_ARGUMENT, "%s: expected a rank-4 tensor, got rank %d", what, v->rank);
        if (v->dtype != dtype) return fail(THIP_UNIMPLEMENTED, "%s: activation element type not supported here", what);
        if (declaredNhwc) {
            *dims = Dims4{v->shape[0], v->shape[3], v->shape[1], v->shape[2]};
        } else {
            *dims = Dims4{v->shape[0], v->shape[1], v->shape[2], v->shape[3]};
        }
        if (dims->N <= 0 || dims->C <= 0 || dims->H <= 0 || dims->W <= 0) {
            return fail(THIP_INVALID_ARGUMENT, "%s: empty tensor", what);
        }
        DescRef lit;
        if (thip_status_t s = literalInput(id, what, &lit)) return s;
        const bool storedNhwc = declaredNhwc || state_[id].nhwcOfNchw || dims->C == 1 || dims->H * dims->W == 1;
        if (declaredNhwc && state_[id].nhwcOfNchw) {
            return fail(THIP_INVALID_ARGUMENT, "%s: tensor %d was produced as N,C,H,W but is consumed as N,H,W,C", what, (int)id);
        }
        if (storedNhwc) {
            *out = lit;
            return THIP_OK;
        }
        // literal NCHW in memory: transpose [N][C][HW] -> [N][HW][C]
        DescRef t = newTemp((uint64_t)v->numel() * elemSize(dtype));
        emitTranspose(lit, t, dims->N, dims->C, dims->H * dims->W, (uint32_t)elemSize(dtype));
        *out = t;
        return THIP_OK;
    }

    // The init operand of an op whose kernel writes NHWC.  Returns the buffer
    // the kernel writes; *post is set when a transpose into the real
    // destination has to follow (finishOutput emits it).
    struct Pending {
        bool needed = false;
        DescRef from, to;
        int64_t B = 0, R = 0, S = 0;
        uint32_t elem = 1;
    };
    thip_status_t nhwcOutput(thip_value_t id, bool declaredNhwc, const char *what, int32_t dtype, int64_t N,
                             int64_t C, int64_t H, int64_t W, DescRef *out, Pending *post) {
        const Value *v;
        if (thip_status_t s = checkValue(id, what, &v)) return s;
        if (v->rank != 4) return fail(THIP_INVALID_ARGUMENT, "%s: expected a rank-4 init tensor", what);
        const int64_t want[4] = {N, declaredNhwc ? H : C, declaredNhwc ? W : H, declaredNhwc ? C : W};
        for (int i = 0; i < 4; i++) {
            if (v->shape[i] != want[i]) {
                return fail(THIP_INVALID_ARGUMENT, "%s: init dimension %d is %lld, the op produces %lld", what, i,
                            (long long)v->shape[i], (long long)want[i]);
            }
        }
        if (v->dtype != dtype) return fail(THIP_INVALID_ARGUMENT, "%s: init element type mismatch", what);
        if (v->kind == kValueConstant) return fail(THIP_INVALID_ARGUMENT, "%s: init cannot be a constant", what);
        if (v->kind == kValueView) return fail(THIP_UNIMPLEMENTED, "%s: init cannot be a view", what);
        const uint64_t bytes = (uint64_t)(N * H * W * physC(id, C)) * elemSize(dtype);
        const bool sameInMemory = declaredNhwc || C == 1 || H * W == 1;
        if (v->kind == kValueTensor) {
            state_[id].ref = newTemp(bytes);
            state_[id].defined = true;
            state_[id].nhwcOfNchw = !sameInMemory;
            *out = state_[id].ref;
            return THIP_OK;
        }
        DescRef b = bindingRef(*v, true);
        if (sameInMemory) {
            *out = b;
            return THIP_OK;
        }
        if (elemSize(dtype) != 1 && dtype != THIP_DTYPE_BF16) {
            return fail(THIP_UNIMPLEMENTED, "%s: N,C,H,W integer outputs wider than 8 bits need nhwc_input", what);
        }
        DescRef t = newTemp(bytes);
        post->elem = (uint32_t)elemSize(dtype);
        post->needed = true;
        post->from = t;
        post->to = b;
        post->B = N;
        post->R = H * W;
        post->S = C;
        *out = t;
        return THIP_OK;
    }
    void finishOutput(const Pending &post) {
        if (post.needed) emitTranspose(post.from, post.to, post.B, post.R, post.S, post.elem);
    }

    // An output written in its declared order (FC, matmul, avg pool).
    thip_status_t literalOutput(thip_value_t id, const char *what, int32_t dtype, int64_t numel, DescRef *out,
                                int64_t physElems = 0) {
        const Value *v;
        if (thip_status_t s = checkValue(id, what, &v)) return s;
        if (v->dtype != dtype) return fail(THIP_INVALID_ARGUMENT, "%s: init element type mismatch", what);
        if (v->numel() != numel) {
            return fail(THIP_INVALID_ARGUMENT, "%s: init holds %lld elements, the op produces %lld", what,
                        (long long)v->numel(), (long long)numel);
        }
        if (v->kind == kValueConstant) return fail(THIP_INVALID_ARGUMENT, "%s: init cannot be a constant", what);
        if (v->kind == kValueView) {
            // a slice of a binding, or of an intermediate that is allocated whole when its first slice is written
            const Value &b = prog_.values[(size_t)v->base];
            if (b.kind == kValueTensor) {
                if (!state_[v->base].defined) {
                    state_[v->base].ref = newTemp((uint64_t)b.numel() * elemSize(b.dtype));
                    state_[v->base].defined = true;
                    state_[v->base].nhwcOfNchw = false;
                }
                if (state_[v->base].nhwcOfNchw) return fail(THIP_UNIMPLEMENTED, "%s: a view of an N,C,H,W intermediate", what);
                *out = state_[v->base].ref;
            } else {
                *out = bindingRef(b, true);
            }
            out->offset += (uint64_t)v->viewOffset * elemSize(dtype);
        } else if (v->kind == kValueTensor) {
            state_[id].ref = newTemp((uint64_t)(physElems ? physElems : numel) * elemSize(dtype));
            state_[id].defined = true;
            state_[id].nhwcOfNchw = false;
            *out = state_[id].ref;
        } else {
            *out = bindingRef(*v, true);
        }
        return THIP_OK;
    }

    thip_status_t constantData(thip_value_t id, const char *what, int32_t dtype, const Value **out) const {
        const Value *v;
        if (thip_status_t s = checkValue(id, what, &v)) return s;
        if (v->kind != kValueConstant) {
            return fail(THIP_UNIMPLEMENTED, "%s: must be a compile-time constant", what);
        }
        if (v->dtype != dtype) return fail(THIP_INVALID_ARGUMENT, "%s: wrong element type", what);
        *out = v;
        return THIP_OK;
    }

    // Splits the interleaved [bias, scale] vector into two arrays padded to `padded`.
    thip_status_t splitScaleBias(thip_value_t id, const char *what, int64_t channels, int64_t padded, bool single,
                                 DescRef *bias, DescRef *scale) {
        const Value *v;
        if (thip_status_t s = constantData(id, what, THIP_DTYPE_I32, &v)) return s;
        const int64_t need = single ? 2 : 2 * channels;
        if (v->numel() < need) {
            return fail(THIP_INVALID_ARGUMENT, "%s: holds %lld int32 values, %lld needed", what, (long long)v->numel(),
                        (long long)need);
        }
        const int32_t *sb = (const int32_t *)v->data.data();
        std::vector<int32_t> b((size_t)padded, 0), s((size_t)padded, 0);
        for (int64_t c = 0; c < channels; c++) {
            b[(size_t)c] = sb[single ? 0 : 2 * c];
            s[(size_t)c] = sb[single ? 1 : 2 * c + 1];
        }
        *bias = newConst(b);
        *scale = newConst(s);
        return THIP_OK;
    }

    static thip_status_t checkRequant(const char *what, int32_t shift, int32_t zp, int32_t mn, int32_t mx, int32_t dtype) {
        // act_rsh is a 6-bit field and the zero point a 16-bit one:
        // third_party/torq-hw/ct/torq_api.c:572-575.
        if (shift < 0 || shift > 63) return fail(THIP_INVALID_ARGUMENT, "%s: shift %d is outside 0..63", what, shift);
        if (zp < -32768 || zp > 32767) return fail(THIP_INVALID_ARGUMENT, "%s: output_zp %d does not fit 16 bits", what, zp);
        if (mn > mx) return fail(THIP_INVALID_ARGUMENT, "%s: output_min > output_max", what);
        int64_t lo = 0, hi = 0;
        switch (dtype) {
        case THIP_DTYPE_I8: lo = -128; hi = 127; break;
        case THIP_DTYPE_I16: lo = -32768; hi = 32767; break;
        default: lo = INT32_MIN; hi = INT32_MAX; break;
        }
        if (mn < lo || mx > hi) {
            return fail(THIP_INVALID_ARGUMENT, "%s: clamp [%d, %d] exceeds the output element type", what, mn, mx);
        }
        return THIP_OK;
    }

    // Left shift of (acc + bias) that lifts a shift below 33 to 33 without losing a bit, or 0 when
    // there is no such shift.  Activations are int8, so |acc| <= 128 * sum |w| per output channel;
    // with the bias that bounds |acc + bias|, which has to stay below 2^(31 - pre).  If the bound is
    // too large, (acc + bias) may still be clamped to +-(2^(31 - pre) - 1) first, provided every
    // channel's result at those two values already lies at or beyond the output clamp: the result is
    // monotonic in acc + bias, so the clamp then changes nothing.  The kernels requantise such ops with
    // their 32-bit tail; the result is the same number.  THIP_NO_PRE_SHIFT turns it off.
    void planPreShift(DescOp *op, const std::vector<int64_t> &absWeightSum) const {
        op->pre_shift = 0;
        op->t0_clamp = 0;
        const int32_t shift = op->shift;
        if (shift >= 33 || shift < 3 || getenv("THIP_NO_PRE_SHIFT")) return;
        const int32_t pre = 33 - shift;
        const int32_t *b = (const int32_t *)consts_[op->bias.index].data();
        const int32_t *sc = (const int32_t *)consts_[op->scale.index].data();
        const int64_t limit = (1LL << 31) >> pre;
        bool fits = true;
        for (size_t n = 0; n < absWeightSum.size() && fits; n++) {
            fits = 128 * absWeightSum[n] + std::llabs((long long)b[n]) < limit;
        }
        if (fits) {
            op->pre_shift = pre;
            return;
        }
        const int64_t bound = limit - 1;
        const int64_t lo = (int64_t)op->output_min - op->output_zp, hi = (int64_t)op->output_max - op->output_zp;
        auto result = [&](int64_t t0, int64_t scale) { return (t0 * scale + (1LL << (shift - 1))) >> shift; };
        for (size_t n = 0; n < absWeightSum.size(); n++) {
            const int64_t scale = sc[n];
            if (scale == 0) continue;  // the result does not depend on acc + bias
            const int64_t top = result(scale > 0 ? bound : -bound, scale), bottom = result(scale > 0 ? -bound : bound, scale);
            if (top < hi || bottom > lo) return;
        }
        op->pre_shift = pre;
        op->t0_clamp = (int32_t)bound;
    }

    // What the tile choice knows about the machine, and every cut-off measured on it, in one place: a different part
    // (another CU count, another LDS size) is re-tuned here and nowhere else.  Tile counts are in units of the chip.
    struct TileRule {
        static constexpr int64_t kCus = 256;                // compute units (8 XCDs of 32)
        static constexpr int64_t kFillsChip = kCus * 7 / 8; // 224 tiles: a one-block-per-CU tile (nearly) fills the chip
        static constexpr int64_t kFillsChipSmall = kCus * 3 / 4;  // 192: the same for the 128-wide and narrower tiles
        static constexpr int64_t kHalfChip = kCus / 2;      // 128: a window tile with a long K pays from half the CUs on
        static constexpr int64_t kTwoPerCu = 2 * kCus;      // 512 tiles
        static constexpr int64_t kSmallTilesMax = kCus * 5 / 2;   // 640 small tiles: beyond, a tile column reads the image once
        static constexpr int64_t kIdleShareDen = 10;        // a last round of tiles more than 1/10 idle counts as idle
        static constexpr int64_t kPadShareDen = 8;          // padding N (or K) by more than 1/8 counts as wasteful
        // the streaming kernel (weights resident in LDS)
        static constexpr int64_t kStreamMinM = 4096;
        static constexpr int64_t kStreamAlwaysM = 200000;   // K <= 128: ahead from here whatever N
        static constexpr int64_t kStreamExpandM = 40000;    // N >= 2 K, K <= 32
        static constexpr int64_t kStreamLongKExpandM = 25000;     // K > 128, N >= 2 K
        static constexpr int64_t kStreamLongKMaxOutputs = 1LL << 28;
        static constexpr int64_t kStreamAddM = 400000;      // K > 128 with an add behind it
        static constexpr int64_t kStreamShortK = 128, kStreamTinyK = 32;
        // dense tiles
        static constexpr int64_t kColumnMinM = 16384;       // N <= 128: one tile column from this many rows
        static constexpr int64_t kShortK = 256, kShortKMaxOutputs = 1LL << 28, kShortKMaxM = 600000;
        static constexpr int64_t kShortKWide = 384, kShortKWideMaxM = 65536;
        static constexpr int64_t kLargestTileMinK = 512;    // up to here the 256 x 256 tile is mostly prologue and epilogue
        static constexpr int64_t kRoundRuleMaxK = 1024;     // the idle-last-round rule applies up to this K
        static constexpr int64_t kK128From = 4096;          // 128-byte k-tiles on the 128 x 128 tile from this K
        // window tiles
        static constexpr int64_t kWindowLargestMinK = 640;
    };

    // Tile choice.  THIP_IGEMM_VARIANT / THIP_IGEMM_DENSE_VARIANT force one (for tuning runs).  addFollows: the
    // record's only reader is a torq_hl.add right behind it, which the streaming kernel and the 64 x 64 tile can fold.
    static uint32_t chooseIgemmVariant(int64_t M, int64_t N, bool dense, int64_t K = 0, int32_t outDtype = 0, bool runs = false, bool addFollows = false) {
        auto tiles = [&](uint32_t v) {
            const IgemmTile &t = igemmTile(v);
            return ((M + t.bm - 1) / t.bm) * ((N + t.bn - 1) / t.bn);
        };
        if (dense) {
            if (const char *env = getenv("THIP_IGEMM_DENSE_VARIANT"); env && *env) {
                const long v = strtol(env, nullptr, 10);
                if (v >= 0 && v < (long)kIgemmVariantCount && (v != (long)kIgemmStream || igemmStreamFits(N, K, outDtype))) {
                    return (uint32_t)v;
                }
            }
            // A small weight matrix over many pixels: keep it in LDS and stream the pixels.  Measured against the dense
            // tiles on pointwise shapes of 16 .. 960 channels over 12 544 .. 802 816 pixels: with at most four k-steps
            // per pixel group (the depth of its prefetch ring) it is ahead from about 200 000 pixels, and from 40 000
            // where N >= 2 K and K <= 32 (the output dominates: the first expanding convolutions of a mobile network;
            // 64 -> 384 over 50 176 pixels is 9.0 us on a dense tile against 10.6); with a longer K only where N >= 2 K,
            // up to 2^28 outputs (beyond that its passes over the activations, one per 256 channels, cost more), or
            // where an add follows a very large image (the fused add saves more than the dense tile gains); below
            // those sizes a dense tile is 10-50 % faster.
            if (M >= TileRule::kStreamMinM && igemmStreamFits(N, K, outDtype) && !getenv("THIP_NO_STREAM")) {
                const bool expanding = N >= 2 * K;
                const char *em = getenv("THIP_STREAM_EXPAND_MIN_M");  // tuning: the pixel count from which an expanding layer streams
                const bool take = K <= TileRule::kStreamShortK ? (M >= TileRule::kStreamAlwaysM || (expanding && K <= TileRule::kStreamTinyK && M >= (em ? atoll(em) : TileRule::kStreamExpandM)))
                                           : ((expanding && M >= TileRule::kStreamLongKExpandM && M * N < TileRule::kStreamLongKMaxOutputs) || (addFollows && M >= TileRule::kStreamAddM));
                if (take) return kIgemmStream;
            }
            // an add behind it: the small tile folds the add into its epilogue, which beats a larger tile plus an add kernel
            if (addFollows && outDtype == THIP_DTYPE_I8 && N % 16 == 0) return kIgemmDense64x64;
            // N narrower than a tile: one tile column of the narrowest tile that covers N, so the
            // activations are streamed once (these shapes are bandwidth-bound, padded MFMA work is free)
            if (N <= 128 && M >= TileRule::kColumnMinM) {
                return N <= 32 ? kIgemmDense256x32 : N <= 64 ? kIgemmDense256x64 : kIgemmDense256x128;
            }
            // a short K (up to six k-tiles) over at least two tiles per CU: the 128 x 128 tile, which the launcher then runs
            // two stages deep with four blocks per CU, so that the prologues and epilogues that dominate such tiles
            // overlap (256 -> 1024 channels at 56 x 56, batch 8: 13.5 us against 16.2 on 128 x 256; 64 -> 256 over 100 352
            // pixels: 10.4 against 12.0; from 400 000 pixels x 960 channels the wider tile is 3 % ahead again)
            const bool shortK = K > 0 && ((K <= TileRule::kShortK && M * N < TileRule::kShortKMaxOutputs && M < TileRule::kShortKMaxM) || (K <= TileRule::kShortKWide && M < TileRule::kShortKWideMaxM));
            if (shortK && N > 128 && tiles(kIgemmDense128x128) >= TileRule::kTwoPerCu && (roundUp(N, 128) - N) * TileRule::kPadShareDen <= N && !getenv("THIP_NO_SHORTK_TILE")) {
                return kIgemmDense128x128;
            }
            // a long K on the largest tile: k-tiles of 128 bytes, whole cache lines per row (THIP_NO_K128 keeps 64)
            // (one block per CU pays for a mostly empty last round of tiles in full, two half-size blocks per CU run
            // it at nearly twice the speed: with K of 513 .. 1024 and more than a tenth of the last round idle the
            // largest tile is skipped - 100 352 x 768 x 512, 784 tiles: 56.3 us on 128 x 256 against 74.7; K = 1024: 69.3
            // against 80.4; with 392 tiles and K = 1024 both take 39 us, and from K = 1536 the 128-byte k-tiles win)
            const int64_t t256 = tiles(kIgemmDense256x256), rounds256 = (t256 + TileRule::kCus - 1) / TileRule::kCus;
            const bool idleLastRound = (rounds256 * TileRule::kCus - t256) * TileRule::kIdleShareDen > rounds256 * TileRule::kCus;
            const bool skipLargest = K > TileRule::kLargestTileMinK && K <= TileRule::kRoundRuleMaxK && idleLastRound && (K < TileRule::kRoundRuleMaxK || t256 >= TileRule::kTwoPerCu) && !getenv("THIP_NO_ROUND_RULE");
            // (the 128-byte k-tiles are ahead from K = 576 on, padded to whole k-tiles: 8192 x 640 x 4096 32.7 us against
            // 36.8, 16384 x 768 x 4096 71.3 against 78.7, 4096 x 960 x 4096 23.0 against 23.4)
            if (K > TileRule::kLargestTileMinK && (roundUp(K, 128) - K) * TileRule::kPadShareDen <= K && tiles(kIgemmDense256x256) >= TileRule::kFillsChip && !skipLargest && !getenv("THIP_NO_K128")) return kIgemmDense256x256K128;
            // otherwise the largest tile that still gives (nearly) every CU a tile and does not pad N by more than an
            // eighth where a narrower tile that fills the chip would not (padded columns are computed too)
            // a long K in whole 128-byte k-tiles on more 128 x 128 tiles than CUs: the launcher runs that tile with
            // 128-byte k-tiles, ahead of the wider tile (1536 x 4096 x 4096: 28.8 us against 31.7, 3000 rows: 54.5 against 60.1)
            if (K >= TileRule::kK128From && K % 128 == 0 && tiles(kIgemmDense128x128) > TileRule::kCus && (roundUp(N, 128) - N) * TileRule::kPadShareDen <= N && !getenv("THIP_NO_K128")) return kIgemmDense128x128;
            const uint32_t order[] = {kIgemmDense256x256, kIgemmDense128x256, kIgemmDense128x128, kIgemmDense64x128, kIgemmDense128x64};
            auto enough = [&](uint32_t v) { return tiles(v) >= (v == kIgemmDense128x128 || v == kIgemmDense128x64 ? TileRule::kFillsChipSmall : TileRule::kFillsChip); };
            auto wasteful = [&](uint32_t v) { return (roundUp(N, igemmTile(v).bn) - N) * TileRule::kPadShareDen > N; };
            for (size_t i = 0; i < sizeof(order) / sizeof(order[0]); i++) {
                const uint32_t v = order[i];
                // a short K leaves a 256 x 256 tile (one block per CU) mostly prologue and epilogue; two blocks per CU
                // of half the size overlap them (256 -> 1024 channels at 56 x 56, batch 32: 75 -> 54 us)
                if (v == kIgemmDense256x256 && K > 0 && (K <= TileRule::kLargestTileMinK || skipLargest)) continue;
                if (v == kIgemmDense64x128 && (wasteful(v) || getenv("THIP_NO_64X128"))) continue;
                if (!enough(v)) continue;
                bool better = false;
                for (size_t j = i + 1; j < sizeof(order) / sizeof(order[0]) && wasteful(v); j++) better = better || (!wasteful(order[j]) && enough(order[j]));
                if (better) continue;
                return v;
            }
            return kIgemmDense64x64;
        }
        if (const char *env = getenv("THIP_IGEMM_VARIANT"); env && *env) {
            const long v = strtol(env, nullptr, 10);
            if (v >= 0 && v < (long)kIgemmDense256x256) return (uint32_t)v;
        }
        // window-row runs of a few-channel image, few output channels: the streaming kernel gathers them too
        if (runs && M >= TileRule::kStreamMinM && N <= 128 && igemmStreamFits(N, K, outDtype) && !getenv("THIP_NO_STREAM")) return kIgemmStream;
        // Enough 128x128 tiles to give every CU work (and N wide enough to use them); otherwise the small tile.
        if (N > 64 && tiles(kIgemm128x128x64) >= TileRule::kCus) return kIgemm128x128x64;
        return kIgemm64x64x64;
    }

    // Tile of the ring kernel with window addressing: one tile column for few output channels (the image is read
    // once), else the largest tile that still gives every CU a tile, two blocks per CU where there are many.
    static uint32_t chooseWindowVariant(int64_t M, int64_t N, int64_t C, int64_t K) {
        if (const char *env = getenv("THIP_WINDOW_VARIANT"); env && *env) {
            const long v = strtol(env, nullptr, 10);
            if (v == kIgemmDense256x256 || v == kIgemmDense128x256 || v == kIgemmDense128x128 || v == kIgemmDense256x128 || v == kIgemmDense256x64 || v == kIgemmDense64x64 || v == kIgemmDense256x32) return (uint32_t)v;
            if (v == kIgemmDense256x256K128) return (uint32_t)v;
        }
        auto tiles = [&](uint32_t v) {
            const IgemmTile &t = igemmTile(v);
            return ((M + t.bm - 1) / t.bm) * ((N + t.bn - 1) / t.bn);
        };
        // padding N by more than an eighth counts against a wide tile only where the 128-wide fallback pads less
        // (144 channels are 256 either way: 144 -> 144 at 56 x 56, batch 32, 45.1 us on 256 x 256 against 48.3 on 128 x 128)
        auto wasteful = [&](uint32_t v) {
            const int64_t np = roundUp(N, igemmTile(v).bn);
            return np > roundUp(N, 128) && (np - N) * TileRule::kPadShareDen > N;
        };
        // up to two small tiles per CU: the 64 x 64 tile (four blocks per CU) spreads a small convolution over the chip
        // (256 -> 256 at 14 x 14: 10.3 us against 13.7 on 7 tiles of 128 x 128; 512 -> 512 at 14 x 14, batch 16, 392
        // tiles: 17.8 against 24.2; at 784 tiles the 128 x 128 tile is ahead, 14.5 against 19.8)
        if (tiles(kIgemmDense64x64) <= TileRule::kTwoPerCu) return kIgemmDense64x64;
        // few output channels: one tile column, the image is read once (64 -> 64 at 112 x 112, batch 32: 27.8 us against
        // 41.1 with 128 x 128 tiles).  At most 64 output channels never take a wider tile (32 -> 64 at 112 x 112, batch
        // 3 / 4: 6.2 / 7.2 us on 588 / 784 small tiles, 6.5 / 6.6 on one column of 256 x 64, 7.0 / 7.1 on 128 x 128); up
        // to 128 take theirs with a tile per CU, below that the 128 x 128 tile wins (128 -> 128 at 28 x 28, batch 8: 8.5 us
        // against 12.4)
        // (and at most 32 take the 32-wide column: 32 -> 16 at 112 x 112, batch 32: 19.2 us against 22.4)
        if (N <= 64) return tiles(kIgemmDense64x64) <= TileRule::kSmallTilesMax ? kIgemmDense64x64 : N <= 32 ? kIgemmDense256x32 : kIgemmDense256x64;
        if (N <= 128 && tiles(kIgemmDense256x128) >= TileRule::kFillsChip) return kIgemmDense256x128;
        // measured on 3x3 convolutions of 64 .. 512 channels at batch 1 .. 64: the largest tile wins as soon as half the CUs
        // get one (a long K per tile amortises its prologue and epilogue), unless it pads N by more than an eighth
        // (a short K leaves the largest tile mostly prologue and epilogue, as in the dense choice: 64 -> 256 at 56 x 56,
        // batch 32, K = 576: 24.7 us on 128 x 256 against 27.5)
        // (and, as there, up to K = 1024 a mostly idle last round of the largest tiles costs more than two half-size
        // blocks per CU: 112 -> 512 at 56 x 56, batch 32, K = 1008, 3.06 rounds: 68.1 us against 80.1)
        const int64_t t256 = tiles(kIgemmDense256x256), rounds256 = (t256 + TileRule::kCus - 1) / TileRule::kCus;
        const bool idleLastRound = (rounds256 * TileRule::kCus - t256) * TileRule::kIdleShareDen > rounds256 * TileRule::kCus && !getenv("THIP_NO_ROUND_RULE");
        if (K > TileRule::kWindowLargestMinK && !(K <= TileRule::kRoundRuleMaxK && idleLastRound) && tiles(kIgemmDense256x256) >= TileRule::kHalfChip && !wasteful(kIgemmDense256x256)) {
            return (C % 128 == 0 && !getenv("THIP_NO_K128")) ? kIgemmDense256x256K128 : kIgemmDense256x256;
        }
        if (tiles(kIgemmDense128x256) >= TileRule::kHalfChip && !wasteful(kIgemmDense128x256)) return kIgemmDense128x256;
        return kIgemmDense128x128;
    }

    // conv2d / fully_connected / matmul as one igemm record.  `wAt(n, k)` returns
    // weight (n, k) with k = (kh * KW + kw) * C + ci.
    template <typename WeightAt>
    void emitIgemm(DescOp base, int64_t M, int64_t N, int64_t K, uint32_t loader, WeightAt wAt) {
        const bool dense = loader == kLoaderDense;
        const uint32_t variant = tileChoice(loader, M, N, K, base.C, base.out_dtype, addFollows_);
        const IgemmTile &t = igemmTile(variant);
        const int64_t Kp = roundUp(K, t.bk), Np = roundUp(N, t.bn);
        std::vector<int8_t> packed((size_t)(Np * Kp), 0);
        std::vector<int64_t> absSum((size_t)N, 0);
        for (int64_t n = 0; n < N; n++) {
            for (int64_t k = 0; k < K; k++) {
                const int8_t wv = wAt(n, k);
                packed[(size_t)(n * Kp + k)] = wv;
                absSum[(size_t)n] += wv < 0 ? -(int64_t)wv : wv;
            }
        }
        base.weights = newConst(packed);
        finishIgemm(base, M, N, K, loader, variant, absSum);
    }

    // The record of an igemm whose [Np][Kp] weight matrix (base.weights) is in place: requant plan, extents, k-table.
    // absWeightSum[n] bounds sum_k |w[n][k]|.
    void finishIgemm(DescOp base, int64_t M, int64_t N, int64_t K, uint32_t loader, uint32_t variant, const std::vector<int64_t> &absWeightSum) {
        const IgemmTile &t = igemmTile(variant);
        const int64_t Kp = roundUp(K, t.bk), Np = roundUp(N, t.bn);
        const bool dense = loader == kLoaderDense;
        planPreShift(&base, absWeightSum);
        base.kind = kKindIgemm;
        base.variant = variant;
        base.loader = loader;
        base.M = (int32_t)M;
        base.K = (int32_t)K;
        base.Kp = (int32_t)Kp;
        base.Nn = (int32_t)N;
        base.Np = (int32_t)Np;
        if (dense) {
            base.gran = 16;
        } else if (loader == kLoaderWindow) {
            base.gran = 16;
            base.table = newConst(std::vector<int8_t>(128, (int8_t)base.input_zp));
        } else if (loader == kLoaderRuns) {
            // K = KH groups of 16 bytes; entry: kh and the run length KW * C
            base.gran = 16;
            std::vector<uint32_t> tab((size_t)(Kp / 16));
            for (int64_t e = 0; e < Kp / 16; e++) {
                tab[(size_t)e] = e < base.KH ? (((uint32_t)e << 24) | (uint32_t)(base.KW * base.C)) : kKEntryInvalid;
            }
            base.table = newConst(tab);
        } else {
            int g = 16;
            while (base.C % g != 0) g /= 2;
            base.gran = (uint32_t)g;
            std::vector<uint32_t> tab((size_t)(Kp / g));
            for (int64_t e = 0; e < Kp / g; e++) {
                const int64_t k = e * g;
                if (k >= K) {
                    tab[(size_t)e] = kKEntryInvalid;
                } else {
                    const int64_t pos = k / base.C, ci = k % base.C;
                    tab[(size_t)e] = packKEntry((int)(pos / base.KW), (int)(pos % base.KW), (int)ci);
                }
            }
            base.table = newConst(tab);
        }
        ops_.push_back(base);
    }

    thip_status_t emitConv2d(const thip_hl_conv2d_t &c);
    thip_status_t emitDepthwise(const thip_hl_depthwise_conv2d_t &c);
    thip_status_t emitFullyConnected(const thip_hl_fully_connected_t &c);
    thip_status_t emitMatmul(const thip_hl_matmul_t &c);
    // A long K over fewer output tiles than CUs: split K over several blocks per tile; their partial sums live in
    // an intermediate of the record's own (THIP_NO_SPLIT_K turns it off).
    void planFcBf16Split(DescOp *op) {
        int split = getenv("THIP_NO_SPLIT_K") ? 1 : fcBf16PreferredSplit(op->M, op->Nn, op->K);
        // THIP_FC_SPLIT forces a split of 1 .. 16 where K has that many k-steps (for tuning runs)
        if (const char *env = getenv("THIP_FC_SPLIT"); env && *env) {
            const long v = strtol(env, nullptr, 10);
            if (v >= 1 && v <= 16 && v <= (op->K + 63) / 64) split = (int)v;
        }
        op->w0 = split;
        if (split > 1) op->in1 = newTemp(fcBf16WorkspaceBytes(op->M, op->Nn, split));
    }
    // Constant bf16 weights [N][K] in the order the kernel's wave loads read them (THIP_BF16_ROW_MAJOR keeps rows).
    void packBf16Weights(DescOp *op, const uint16_t *w, int64_t N, int64_t K) {
        if (getenv("THIP_BF16_ROW_MAJOR")) {
            op->loader = 0;
            op->weights = newConst(std::vector<uint16_t>(w, w + N * K));
            return;
        }
        const int steps = (int)((K + 63) / 64);
        std::vector<uint8_t> packed((size_t)roundUp(N, 32) * (size_t)steps * 64 * 2, 0);
        for (int64_t n = 0; n < N; n++) {
            for (int64_t k = 0; k < K; k++) memcpy(&packed[fcBf16FragmentOffset((int)n, (int)k, steps)], &w[n * K + k], 2);
        }
        op->loader = 1;
        op->weights = newConst(packed);
    }
    thip_status_t emitConv2dBf16(const thip_hl_conv2d_t &c);
    thip_status_t emitDepthwiseBf16(const thip_hl_depthwise_conv2d_t &c);
    thip_status_t emitFullyConnectedBf16(const thip_hl_fully_connected_t &c);
    thip_status_t emitMatmulBf16(const thip_hl_matmul_t &c);
    thip_status_t emitMaxPool(const thip_hl_maxpool2d_t &c);
    thip_status_t emitAvgPool(const thip_hl_avg_pool2d_t &c);
    thip_status_t emitAdd(const thip_hl_add_t &c);
    thip_status_t emitTransposeOp(const thip_hl_transpose_t &c);
    thip_status_t emitExpandWeights(const thip_hl_expand_weights_t &c);
    thip_status_t emitFma(const thip_hl_fma_t &c);
    thip_status_t emitMul(const thip_hl_mul_t &c);
    thip_status_t emitAct(const thip_hl_act_t &c, const std::string &name);
    thip_status_t emitBinary(const thip_hl_elementwisebinary_t &c);
    thip_status_t emitUnary(const thip_hl_elementwiseunary_t &c);
    thip_status_t emitShift(const thip_hl_elementwiseshift_t &c);
    thip_status_t emitTable(const thip_hl_table_t &c, const std::vector<int32_t> &staticTable);
    // Operands of an integer elementwise op: element types, and the record's common fields.
    thip_status_t eltwiseCommon(const char *what, thip_value_t input, thip_value_t init, DescOp *op);
    thip_status_t emitAvgPoolBf16(const thip_hl_avg_pool2d_t &c);
    // ---- decode-shaped bf16 programs (at most 32 rows per matmul): fewer, wider launches -----------------------
    // A torq_hl.transpose that emits no kernel: its result is read once, as input2 of a bf16 matmul with at most 32
    // rows, which then reads the transpose's input as its [N][K] operand (result value -> index of the transpose).
    std::map<thip_value_t, size_t> foldedTranspose_;
    std::vector<char> consumed_;  // per op of the program: already emitted as part of an earlier op's record
    void planDecodeFolding();
    // A bf16 matmul that the grouped linear kernel can take: two-dimensional input1 of at most 32 rows, input2 a folded
    // expand_weights with blocks of a multiple of 128 rows, N a multiple of 16.
    struct DecCandidate {
        const thip_hl_matmul_t *mm;
        const thip_hl_expand_weights_t *ew;
        int64_t M, K, N, block;
        float bias;
    };
    bool decodeCandidate(size_t at, DecCandidate *out);
    size_t nextLiveOp(size_t at) const;
    thip_status_t tryEmitDecodeLinear(size_t at, bool *handled);
    thip_status_t emitDecodeMatmul(const thip_hl_matmul_t &c, size_t transposeAt);
    // Operands of an expand_weights checked and measured.
    struct ExpandShape {
        const Value *w, *scale, *bias, *init;
        int64_t K, N, G, block, biasCols;
    };
    thip_status_t checkExpandWeights(const thip_hl_expand_weights_t &c, ExpandShape *out);
};

// Round-to-nearest-even bf16 bits of a float (NaN stays NaN).
static uint16_t bf16FromFloat(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1)) >> 16);
}
static float floatFromBf16(uint16_t b) {
    const uint32_t u = (uint32_t)b << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}
static float floatFromBits(int32_t bits) {
    float f;
    memcpy(&f, &bits, 4);
    return f;
}
// One expanded weight, as the kernels compute it: the product of an 8-bit weight and a bf16 scale is exact in
// fp32, so it does not matter whether the compiler fuses the multiply and the add.
static uint16_t expandWeight(int8_t w, uint16_t scale, float bias, float lo, float hi) {
    const float t0 = (float)w * floatFromBf16(scale) + bias;
    return bf16FromFloat(t0 < lo ? lo : (t0 > hi ? hi : t0));
}

static thip_status_t windowGeometry(const char *what, int64_t H, int64_t W, int64_t KH, int64_t KW, const int64_t pad[4],
                                    const int64_t stride[2], int64_t *OH, int64_t *OW) {
    if (stride[0] <= 0 || stride[1] <= 0) return fail(THIP_INVALID_ARGUMENT, "%s: stride must be positive", what);
    for (int i = 0; i < 4; i++) {
        if (pad[i] < 0) return fail(THIP_INVALID_ARGUMENT, "%s: negative padding", what);
    }
    if (KH <= 0 || KW <= 0 || KH > 127 || KW > 255) return fail(THIP_INVALID_ARGUMENT, "%s: unsupported window %lldx%lld", what, (long long)KH, (long long)KW);
    const int64_t spanH = H + pad[2] + pad[3] - KH, spanW = W + pad[0] + pad[1] - KW;
    if (spanH < 0 || spanW < 0) return fail(THIP_INVALID_ARGUMENT, "%s: window larger than the padded input", what);
    *OH = spanH / stride[0] + 1;
    *OW = spanW / stride[1] + 1;
    return THIP_OK;
}

static bool fitsInt32(int64_t v) { return v > 0 && v < (1LL << 31); }

thip_status_t Emitter::emitConv2d(const thip_hl_conv2d_t &c) {
    const char *what = "torq_hl.conv2d";
    {
        const Value *xin;
        if (thip_status_t s = checkValue(c.input, "torq_hl.conv2d input", &xin)) return s;
        if (xin->dtype == THIP_DTYPE_BF16) return emitConv2dBf16(c);
    }
    if (c.groups != 1) return fail(THIP_UNIMPLEMENTED, "%s: groups must be 1", what);
    if (c.weight_zp != 0) return fail(THIP_UNIMPLEMENTED, "%s: weight_zp must be 0 (the patterns fold it into the weights)", what);
    if (c.dilation[0] != 1 || c.dilation[1] != 1) return fail(THIP_UNIMPLEMENTED, "%s: dilation must be [1,1] (the patterns fold it into the weights)", what);
    if (c.segment_output) return fail(THIP_UNIMPLEMENTED, "%s: segment_output is an NPU memory layout", what);
    if (c.input_zp < -128 || c.input_zp > 127) return fail(THIP_INVALID_ARGUMENT, "%s: input_zp outside int8", what);
    const Value *w;
    if (thip_status_t s = constantData(c.weights, "torq_hl.conv2d weights", THIP_DTYPE_I8, &w)) return s;
    if (w->rank != 4) return fail(THIP_INVALID_ARGUMENT, "%s: weights must be O,I,KH,KW", what);
    const Value *init;
    if (thip_status_t s = checkValue(c.init, "torq_hl.conv2d init", &init)) return s;
    if (thip_status_t s = checkRequant(what, c.shift_factor, c.output_zp, c.output_min, c.output_max, init->dtype)) return s;
    Dims4 d;
    DescRef in;
    if (thip_status_t s = nhwcInput(c.input, c.nhwc_input != 0, "torq_hl.conv2d input", &d, &in)) return s;
    const int64_t O = w->shape[0], I = w->shape[1], KH = w->shape[2], KW = w->shape[3];
    if (I != d.C) return fail(THIP_INVALID_ARGUMENT, "%s: weights expect %lld input channels, input has %lld", what, (long long)I, (long long)d.C);
    if (d.C > 65535) return fail(THIP_UNIMPLEMENTED, "%s: more than 65535 input channels", what);
    int64_t OH, OW;
    if (thip_status_t s = windowGeometry(what, d.H, d.W, KH, KW, c.pad, c.stride, &OH, &OW)) return s;
    // channel counts in memory: padded intermediates carry zero-weight channels (planChannelPadding)
    const int64_t Cin = physC(c.input, d.C), Oout = physC(c.init, O);
    const int64_t M = d.N * OH * OW, K = KH * KW * Cin;
    if (!fitsInt32(M) || !fitsInt32(K) || !fitsInt32(M * Oout) || !fitsInt32(d.N * d.H * d.W * Cin)) {
        return fail(THIP_UNIMPLEMENTED, "%s: tensor too large for 32-bit indexing", what);
    }
    DescOp op;
    memset(&op, 0, sizeof(op));
    DescRef out;
    Pending post;
    if (thip_status_t s = nhwcOutput(c.init, c.nhwc_input != 0, "torq_hl.conv2d init", init->dtype, d.N, O, OH, OW, &out, &post)) return s;
    const int64_t tile = 256;
    if (thip_status_t s = splitScaleBias(c.scale_bias, "torq_hl.conv2d scale_bias", O, roundUp(Oout, tile), false, &op.bias, &op.scale)) return s;
    op.out_dtype = init->dtype;
    op.input_zp = c.input_zp;
    op.output_zp = c.output_zp;
    op.output_min = c.output_min;
    op.output_max = c.output_max;
    op.shift = c.shift_factor;
    op.N = (int32_t)d.N; op.H = (int32_t)d.H; op.W = (int32_t)d.W; op.C = (int32_t)Cin;
    op.OH = (int32_t)OH; op.OW = (int32_t)OW; op.OC = (int32_t)Oout;
    op.KH = (int32_t)KH; op.KW = (int32_t)KW; op.SH = (int32_t)c.stride[0]; op.SW = (int32_t)c.stride[1];
    op.PL = (int32_t)c.pad[0]; op.PR = (int32_t)c.pad[1]; op.PT = (int32_t)c.pad[2]; op.PB = (int32_t)c.pad[3];
    op.in0 = in;
    op.out = out;
    const int8_t *wd = (const int8_t *)w->data.data();
    const bool pointwise = KH == 1 && KW == 1 && c.stride[0] == 1 && c.stride[1] == 1 && c.pad[0] == 0 &&
                           c.pad[1] == 0 && c.pad[2] == 0 && c.pad[3] == 0;
    const int64_t C = d.C;
    // (its 16-byte loads stay inside the image by stepping back from its end, so the image must hold 16 bytes)
    if (KW * Cin <= 16 && Cin % 16 != 0 && d.N * d.H * d.W * Cin >= 16 && !getenv("THIP_NO_RUN_LOADER")) {
        // few input channels (the first layer of an image network): one 16-byte run per window row
        emitIgemm(op, M, Oout, KH * 16, kLoaderRuns, [&](int64_t n, int64_t k) -> int8_t {
            const int64_t kh = k / 16, b = k % 16;
            if (b >= KW * C || n >= O) return 0;
            return wd[((n * C + b % C) * KH + kh) * KW + b / C];
        });
    } else {
        // a window over a multiple of 16 channels: the LDS-DMA ring kernel addresses the window itself, at every size
        // (256 -> 256 at 14 x 14, one image: 10.3 us against 15.3 on the gather kernel; 32 -> 32 at 28 x 28: 4.3
        // against 4.8; 96 -> 96 at 56 x 56, batch 32: 17.3 against 29.4).  THIP_NO_WINDOW_RING keeps such convolutions
        // on the gather kernel; THIP_RING_MIN_C, THIP_RING_MIN_M and THIP_RING_MIN_O raise the input channel, pixel and
        // output channel counts from which the ring kernel is taken (tests and tuning).  Few output channels pay as
        // well, padded to a 64-wide tile as on the gather kernel (16 -> 16 at 32 x 32: 3.6 us against 4.2, batch 128: 6.5
        // against 9.8; 32 -> 16 at 112 x 112, batch 32: 22.3 against 28.9).
        const char *minC = getenv("THIP_RING_MIN_C"), *minM = getenv("THIP_RING_MIN_M"), *minO = getenv("THIP_RING_MIN_O");
        const bool ring = !pointwise && Cin % 16 == 0 && Cin >= (minC && *minC ? atoi(minC) : 16) && M >= (minM && *minM ? atoi(minM) : 1) && Oout >= (minO && *minO ? atoi(minO) : 1) &&
                          d.N * d.H * d.W * Cin < (1LL << 32) && !getenv("THIP_NO_WINDOW_RING");
        emitIgemm(op, M, Oout, K, (pointwise && K % 16 == 0) ? kLoaderDense : ring ? kLoaderWindow : kLoaderGather, [&](int64_t n, int64_t k) -> int8_t {
            const int64_t pos = k / Cin, ci = k % Cin;
            const int64_t kh = pos / KW, kw = pos % KW;
            if (ci >= C || n >= O) return 0;  // padded channels meet zero weights
            return wd[((n * C + ci) * KH + kh) * KW + kw];
        });
    }
    finishOutput(post);
    return THIP_OK;
}

thip_status_t Emitter::emitDepthwise(const thip_hl_depthwise_conv2d_t &c) {
    const char *what = "torq_hl.depthwise_conv2d";
    {
        const Value *xin;
        if (thip_status_t s = checkValue(c.input, "torq_hl.depthwise_conv2d input", &xin)) return s;
        if (xin->dtype == THIP_DTYPE_BF16) return emitDepthwiseBf16(c);
    }
    if (c.weight_zp != 0) return fail(THIP_UNIMPLEMENTED, "%s: weight_zp must be 0", what);
    if (c.dilation[0] != 1 || c.dilation[1] != 1) return fail(THIP_UNIMPLEMENTED, "%s: dilation must be [1,1]", what);
    if (c.segment_output) return fail(THIP_UNIMPLEMENTED, "%s: segment_output is an NPU memory layout", what);
    if (c.is_dw1d_stride1) return fail(THIP_UNIMPLEMENTED, "%s: is_dw1d_stride1 is the bf16 1-D special case", what);
    if (c.input_zp < -128 || c.input_zp > 127) return fail(THIP_INVALID_ARGUMENT, "%s: input_zp outside int8", what);
    const Value *w;
    if (thip_status_t s = constantData(c.weights, "torq_hl.depthwise_conv2d weights", THIP_DTYPE_I8, &w)) return s;
    if (w->rank != 4 || w->shape[1] != 1) return fail(THIP_INVALID_ARGUMENT, "%s: weights must be C,1,KH,KW", what);
    const Value *init;
    if (thip_status_t s = checkValue(c.init, "torq_hl.depthwise_conv2d init", &init)) return s;
    if (init->dtype != THIP_DTYPE_I8) return fail(THIP_UNIMPLEMENTED, "%s: only int8 outputs", what);
    if (thip_status_t s = checkRequant(what, c.shift_factor, c.output_zp, c.output_min, c.output_max, init->dtype)) return s;
    Dims4 d;
    DescRef in;
    if (thip_status_t s = nhwcInput(c.input, c.nhwc_input != 0, "torq_hl.depthwise_conv2d input", &d, &in)) return s;
    const int64_t C = w->shape[0], KH = w->shape[2], KW = w->shape[3];
    if (C != d.C) return fail(THIP_INVALID_ARGUMENT, "%s: weights have %lld channels, input has %lld", what, (long long)C, (long long)d.C);
    if (c.groups != C && c.groups != 1 && c.groups != 0) return fail(THIP_INVALID_ARGUMENT, "%s: groups must equal the channel count", what);
    int64_t OH, OW;
    if (thip_status_t s = windowGeometry(what, d.H, d.W, KH, KW, c.pad, c.stride, &OH, &OW)) return s;
    // channels in memory (input and output of a depthwise op are padded alike); padded channels get zero weights
    const int64_t Cp = physC(c.input, C);
    if (!fitsInt32(d.N * OH * OW * Cp) || !fitsInt32(d.N * d.H * d.W * Cp)) return fail(THIP_UNIMPLEMENTED, "%s: tensor too large for 32-bit indexing", what);
    DescOp op;
    memset(&op, 0, sizeof(op));
    DescRef out;
    Pending post;
    if (thip_status_t s = nhwcOutput(c.init, c.nhwc_input != 0, "torq_hl.depthwise_conv2d init", init->dtype, d.N, C, OH, OW, &out, &post)) return s;
    if (thip_status_t s = splitScaleBias(c.scale_bias, "torq_hl.depthwise_conv2d scale_bias", C, roundUp(Cp, 16), false, &op.bias, &op.scale)) return s;
    const int8_t *wd = (const int8_t *)w->data.data();
    std::vector<int8_t> wpk((size_t)(KH * KW * Cp), 0);
    std::vector<int64_t> absSum((size_t)C, 0);
    for (int64_t ch = 0; ch < C; ch++) {
        for (int64_t k = 0; k < KH * KW; k++) {
            const int8_t wv = wd[ch * KH * KW + k];
            wpk[(size_t)(k * Cp + ch)] = wv;
            absSum[(size_t)ch] += wv < 0 ? -(int64_t)wv : wv;
        }
    }
    op.kind = kKindDepthwise;
    op.out_dtype = init->dtype;
    op.input_zp = c.input_zp;
    op.output_zp = c.output_zp;
    op.output_min = c.output_min;
    op.output_max = c.output_max;
    op.shift = c.shift_factor;
    planPreShift(&op, absSum);
    op.N = (int32_t)d.N; op.H = (int32_t)d.H; op.W = (int32_t)d.W; op.C = (int32_t)Cp;
    op.OH = (int32_t)OH; op.OW = (int32_t)OW; op.OC = (int32_t)Cp;
    op.KH = (int32_t)KH; op.KW = (int32_t)KW; op.SH = (int32_t)c.stride[0]; op.SW = (int32_t)c.stride[1];
    op.PL = (int32_t)c.pad[0]; op.PR = (int32_t)c.pad[1]; op.PT = (int32_t)c.pad[2]; op.PB = (int32_t)c.pad[3];
    op.in0 = in;
    op.out = out;
    if (KH == 3 && KW == 3 && Cp % 16 == 0 && !getenv("THIP_DEPTHWISE_GENERIC")) {
        // one dword per (window row, channel): byte kw = tap kw, byte 3 = 0, for v_dot4_i32_i8
        std::vector<uint32_t> wdot((size_t)(KH * Cp), 0);
        for (int64_t ch = 0; ch < C; ch++) {
            for (int64_t kh = 0; kh < KH; kh++) {
                uint32_t v = 0;
                for (int64_t kw = 0; kw < KW; kw++) v |= (uint32_t)(uint8_t)wd[(ch * KH + kh) * KW + kw] << (8 * kw);
                wdot[(size_t)(kh * Cp + ch)] = v;
            }
        }
        op.variant = kDepthwiseDot4Rows;
        op.weights = newConst(wdot);
    } else {
        op.variant = kDepthwiseGeneric;
        op.weights = newConst(wpk);
    }
    ops_.push_back(op);
    finishOutput(post);
    return THIP_OK;
}

thip_status_t Emitter::emitFullyConnected(const thip_hl_fully_connected_t &c) {
    const char *what = "torq_hl.fully_connected";
    {
        const Value *xin;
        if (thip_status_t s = checkValue(c.input, "torq_hl.fully_connected input", &xin)) return s;
        if (xin->dtype == THIP_DTYPE_BF16) return emitFullyConnectedBf16(c);
    }
    if (c.weight_zp != 0) return fail(THIP_UNIMPLEMENTED, "%s: weight_zp must be 0", what);
    const Value *w;
    if (thip_status_t s = constantData(c.weights, "torq_hl.fully_connected weights", THIP_DTYPE_I8, &w)) return s;
    if (w->rank != 2) return fail(THIP_INVALID_ARGUMENT, "%s: weights must be N,K", what);
    const int64_t N = w->shape[0], K = w->shape[1];
    const Value *x;
    if (thip_status_t s = checkValue(c.input, "torq_hl.fully_connected input", &x)) return s;
    if (x->dtype != THIP_DTYPE_I8) return fail(THIP_UNIMPLEMENTED, "%s: only int8 and bf16 inputs", what);
    if (x->rank < 1 || x->shape[x->rank - 1] != K) {
        // a flattened N,C,1,1 / N,1,1,C activation is accepted as M,K too
        if (K <= 0 || x->numel() % K != 0) return fail(THIP_INVALID_ARGUMENT, "%s: input does not end in K=%lld", what, (long long)K);
    }
    if (state_[c.input].nhwcOfNchw) {
        return fail(THIP_UNIMPLEMENTED, "%s: input %d is an N,C,H,W intermediate with H*W > 1; flatten needs a transpose", what, (int)c.input);
    }
    const int64_t M = x->numel() / K;
    const Value *init;
    if (thip_status_t s = checkValue(c.init, "torq_hl.fully_connected init", &init)) return s;
    if (thip_status_t s = checkRequant(what, c.shift_factor, c.output_zp, c.output_min, c.output_max, init->dtype)) return s;
    if (!fitsInt32(M) || !fitsInt32(K) || !fitsInt32(N) || !fitsInt32(M * N) || !fitsInt32(M * K)) {
        return fail(THIP_UNIMPLEMENTED, "%s: tensor too large for 32-bit indexing", what);
    }
    DescOp op;
    memset(&op, 0, sizeof(op));
    if (thip_status_t s = literalInput(c.input, "torq_hl.fully_connected input", &op.in0)) return s;
    if (thip_status_t s = literalOutput(c.init, "torq_hl.fully_connected init", init->dtype, M * N, &op.out)) return s;
    op.out_dtype = init->dtype;
    op.input_zp = c.input_zp;
    op.output_zp = c.output_zp;
    op.output_min = c.output_min;
    op.output_max = c.output_max;
    op.shift = c.shift_factor;
    const int8_t *wd = (const int8_t *)w->data.data();
    const bool skinnyOff = getenv("THIP_NO_SKINNY") != nullptr;
    if (M <= kFcSkinnyMaxRows && K % 16 == 0 && !skinnyOff) {
        if (thip_status_t s = splitScaleBias(c.scale_bias, "torq_hl.fully_connected scale_bias", N, N, false, &op.bias, &op.scale)) return s;
        op.kind = kKindFcSkinny;
        op.M = (int32_t)M; op.K = (int32_t)K; op.Kp = (int32_t)K; op.Nn = (int32_t)N; op.Np = (int32_t)N;
        op.weights = newConst(w->data);
        ops_.push_back(op);
        return THIP_OK;
    }
    if (thip_status_t s = splitScaleBias(c.scale_bias, "torq_hl.fully_connected scale_bias", N, roundUp(N, 256), false, &op.bias, &op.scale)) return s;
    // as a 1x1 convolution over an M x 1 x 1 x K image
    op.N = (int32_t)M; op.H = 1; op.W = 1; op.C = (int32_t)K;
    op.OH = 1; op.OW = 1; op.OC = (int32_t)N;
    op.KH = 1; op.KW = 1; op.SH = 1; op.SW = 1;
    emitIgemm(op, M, N, K, K % 16 == 0 ? kLoaderDense : kLoaderGather, [&](int64_t n, int64_t k) { return wd[n * K + k]; });
    return THIP_OK;
}

thip_status_t Emitter::emitMatmul(const thip_hl_matmul_t &c) {
    const char *what = "torq_hl.matmul";
    const Value *a, *b, *init;
    if (thip_status_t s = checkValue(c.input1, "torq_hl.matmul input1", &a)) return s;
    if (thip_status_t s = checkValue(c.input2, "torq_hl.matmul input2", &b)) return s;
    if (thip_status_t s = checkValue(c.init, "torq_hl.matmul init", &init)) return s;
    if (a->dtype == THIP_DTYPE_BF16) return emitMatmulBf16(c);
    if (a->dtype != THIP_DTYPE_I8 || b->dtype != THIP_DTYPE_I8) return fail(THIP_UNIMPLEMENTED, "%s: only int8 inputs", what);
    if (a->rank < 2 || a->rank > 3 || b->rank < 2 || b->rank > 3) return fail(THIP_UNIMPLEMENTED, "%s: operands must have rank 2 or 3", what);
    if (state_[c.input1].nhwcOfNchw || state_[c.input2].nhwcOfNchw) return fail(THIP_UNIMPLEMENTED, "%s: N,C,H,W intermediates are not accepted", what);
    const int64_t Ba = a->rank == 3 ? a->shape[0] : 1, Bb = b->rank == 3 ? b->shape[0] : 1;
    const int64_t M = a->shape[a->rank - 2], K = a->shape[a->rank - 1];
    const int64_t K2 = b->shape[b->rank - 2], N = b->shape[b->rank - 1];
    if (K != K2) return fail(THIP_INVALID_ARGUMENT, "%s: inner dimensions differ (%lld vs %lld)", what, (long long)K, (long long)K2);
    const int64_t B = std::max(Ba, Bb);
    if ((Ba != B && Ba != 1) || (Bb != B && Bb != 1)) return fail(THIP_INVALID_ARGUMENT, "%s: batch dimensions do not broadcast", what);
    if (thip_status_t s = checkRequant(what, c.shift, c.output_zp, c.output_min, c.output_max, init->dtype)) return s;
    if (!fitsInt32(B * M * N) || !fitsInt32(B * M * K) || !fitsInt32(B * K * N)) return fail(THIP_UNIMPLEMENTED, "%s: tensor too large for 32-bit indexing", what);
    DescRef aRef, outRef;
    if (thip_status_t s = literalInput(c.input1, "torq_hl.matmul input1", &aRef)) return s;
    if (thip_status_t s = literalOutput(c.init, "torq_hl.matmul init", init->dtype, B * M * N, &outRef)) return s;
    DescOp op;
    memset(&op, 0, sizeof(op));
    op.out_dtype = init->dtype;
    op.output_zp = c.output_zp;
    op.output_min = c.output_min;
    op.output_max = c.output_max;
    op.shift = c.shift;
    op.H = 1; op.W = 1; op.C = (int32_t)K; op.OH = 1; op.OW = 1; op.OC = (int32_t)N;
    op.KH = 1; op.KW = 1; op.SH = 1; op.SW = 1;
    const size_t outElem = elemSize(init->dtype);
    if (b->kind == kValueConstant) {
        // weights known at compile time: pack per batch (one record when B is broadcast)
        const int8_t *bd = (const int8_t *)b->data.data();
        const int64_t records = Bb == 1 ? 1 : B;
        for (int64_t r = 0; r < records; r++) {
            DescOp o = op;
            const int64_t rows = Bb == 1 ? (Ba == 1 ? M : B * M) : M;
            o.N = (int32_t)rows;
            o.in0 = aRef;
            o.in0.offset += (uint64_t)(Ba == 1 ? 0 : r * M * K);
            o.out = outRef;
            o.out.offset += (uint64_t)(r * M * N) * outElem;
            if (thip_status_t s = splitScaleBias(c.scale_bias, "torq_hl.matmul scale_bias", N, roundUp(N, 256), true, &o.bias, &o.scale)) return s;
            const int8_t *bb = bd + (Bb == 1 ? 0 : r * K * N);
            emitIgemm(o, rows, N, K, K % 16 == 0 ? kLoaderDense : kLoaderGather, [&](int64_t n, int64_t k) { return bb[k * N + n]; });
        }
        return THIP_OK;
    }
    // input2 produced at run time: transpose each batch into a zero-padded
    // [Np][Kp] buffer (intermediates are zero-filled when the executable is
    // created and the padding is never written), then run the igemm on it: the dense loader
    // when the rows of input1 are whole 16-byte chunks, the gather loader (K as the channel axis
    // of a 1x1 window) otherwise.
    DescRef bRef;
    if (thip_status_t s = literalInput(c.input2, "torq_hl.matmul input2", &bRef)) return s;
    const uint32_t loader = K % 16 == 0 ? kLoaderDense : kLoaderGather;
    const uint32_t variant = chooseIgemmVariant(M, N, loader == kLoaderDense, K, init->dtype);
    const IgemmTile &t = igemmTile(variant);
    const int64_t Kp = roundUp(K, t.bk), Np = roundUp(N, t.bn);
    std::vector<DescRef> packed;
    for (int64_t r = 0; r < (Bb == 1 ? 1 : B); r++) {
        DescRef t2 = newTemp((uint64_t)(Np * Kp));
        DescRef src = bRef;
        src.offset += (uint64_t)(r * K * N);
        emitTranspose(src, t2, 1, K, N, 1, Kp);
        packed.push_back(t2);
    }
    // nothing is known about the values of a run-time operand: every |w| may be 128
    const std::vector<int64_t> absSum((size_t)N, 128 * K);
    for (int64_t batch = 0; batch < B; batch++) {
        DescOp o = op;
        o.N = (int32_t)M;
        o.in0 = aRef;
        o.in0.offset += (uint64_t)(Ba == 1 ? 0 : batch * M * K);
        o.out = outRef;
        o.out.offset += (uint64_t)(batch * M * N) * outElem;
        o.weights = packed[(size_t)(Bb == 1 ? 0 : batch)];
        if (thip_status_t s = splitScaleBias(c.scale_bias, "torq_hl.matmul scale_bias", N, roundUp(N, 256), true, &o.bias, &o.scale)) return s;
        finishIgemm(o, M, N, K, loader, variant, absSum);
    }
    return THIP_OK;
}


// bf16 rows (compiler/torq/Utils/Kernel.h:626-632): float bias, no scale, no shift, float clamp.
static thip_status_t checkFloatAct(const char *what, int32_t shift, int32_t zpA, int32_t zpB, int32_t zpOut) {
    if (shift != 0) return fail(THIP_INVALID_ARGUMENT, "%s: bf16 has no rescale: shift must be 0", what);
    if (zpA != 0 || zpB != 0 || zpOut != 0) return fail(THIP_INVALID_ARGUMENT, "%s: bf16 has no zero points", what);
    return THIP_OK;
}

thip_status_t Emitter::emitConv2dBf16(const thip_hl_conv2d_t &c) {
    const char *what = "torq_hl.conv2d (bf16)";
    if (c.groups != 1) return fail(THIP_UNIMPLEMENTED, "%s: groups must be 1", what);
    if (c.dilation[0] != 1 || c.dilation[1] != 1) return fail(THIP_UNIMPLEMENTED, "%s: dilation must be [1,1]", what);
    if (c.segment_output) return fail(THIP_UNIMPLEMENTED, "%s: segment_output is an NPU memory layout", what);
    if (thip_status_t s = checkFloatAct(what, c.shift_factor, c.input_zp, c.weight_zp, c.output_zp)) return s;
    const Value *w, *init, *b;
    if (thip_status_t s = constantData(c.weights, "torq_hl.conv2d weights", THIP_DTYPE_BF16, &w)) return s;
    if (w->rank != 4) return fail(THIP_INVALID_ARGUMENT, "%s: weights must be O,I,KH,KW", what);
    if (thip_status_t s = checkValue(c.init, "torq_hl.conv2d init", &init)) return s;
    if (init->dtype != THIP_DTYPE_BF16) return fail(THIP_INVALID_ARGUMENT, "%s: init must be bf16", what);
    Dims4 d;
    DescRef in;
    if (thip_status_t s = nhwcInput(c.input, c.nhwc_input != 0, "torq_hl.conv2d input", &d, &in, THIP_DTYPE_BF16)) return s;
    const int64_t O = w->shape[0], I = w->shape[1], KH = w->shape[2], KW = w->shape[3];
    if (I != d.C) return fail(THIP_INVALID_ARGUMENT, "%s: weights expect %lld input channels, input has %lld", what, (long long)I, (long long)d.C);
    if (thip_status_t s = constantData(c.scale_bias, "torq_hl.conv2d scale_bias", THIP_DTYPE_F32, &b)) return s;
    if (b->numel() < O) return fail(THIP_INVALID_ARGUMENT, "%s: scale_bias holds %lld floats, %lld needed", what, (long long)b->numel(), (long long)O);
    int64_t OH, OW;
    if (thip_status_t s = windowGeometry(what, d.H, d.W, KH, KW, c.pad, c.stride, &OH, &OW)) return s;
    const int64_t M = d.N * OH * OW, K = KH * KW * d.C, Kp = roundUp(K, 8);
    if (!fitsInt32(M) || !fitsInt32(Kp) || !fitsInt32(M * O) || !fitsInt32(M * Kp) || !fitsInt32(d.N * d.H * d.W * d.C)) {
        return fail(THIP_UNIMPLEMENTED, "%s: tensor too large for 32-bit indexing", what);
    }
    DescRef out;
    Pending post;
    if (thip_status_t s = nhwcOutput(c.init, c.nhwc_input != 0, "torq_hl.conv2d init", THIP_DTYPE_BF16, d.N, O, OH, OW, &out, &post)) return s;
    // the GEMM operand: the image itself for a pointwise convolution, its patch matrix otherwise
    const bool pointwise = KH == 1 && KW == 1 && c.stride[0] == 1 && c.stride[1] == 1 && c.pad[0] == 0 && c.pad[1] == 0 &&
                           c.pad[2] == 0 && c.pad[3] == 0 && d.C % 8 == 0;
    DescRef a = in;
    if (!pointwise) {
        DescOp g;
        memset(&g, 0, sizeof(g));
        g.kind = kKindIm2colBf16;
        g.N = (int32_t)d.N; g.H = (int32_t)d.H; g.W = (int32_t)d.W; g.C = (int32_t)d.C;
        g.OH = (int32_t)OH; g.OW = (int32_t)OW; g.KH = (int32_t)KH; g.KW = (int32_t)KW;
        g.SH = (int32_t)c.stride[0]; g.SW = (int32_t)c.stride[1]; g.PL = (int32_t)c.pad[0]; g.PT = (int32_t)c.pad[2];
        g.Kp = (int32_t)Kp;
        g.in0 = in;
        a = newTemp((uint64_t)(M * Kp) * 2);
        g.out = a;
        ops_.push_back(g);
    }
    // weights as [O][Kp], k = (kh * KW + kw) * C + ci
    const uint16_t *wd = (const uint16_t *)w->data.data();
    std::vector<uint16_t> wk((size_t)(O * Kp), 0);
    for (int64_t o = 0; o < O; o++) {
        for (int64_t kh = 0; kh < KH; kh++) {
            for (int64_t kw = 0; kw < KW; kw++) {
                for (int64_t ci = 0; ci < d.C; ci++) {
                    wk[(size_t)(o * Kp + (kh * KW + kw) * d.C + ci)] = wd[((o * d.C + ci) * KH + kh) * KW + kw];
                }
            }
        }
    }
    DescOp op;
    memset(&op, 0, sizeof(op));
    op.kind = kKindFcBf16;
    op.out_dtype = THIP_DTYPE_BF16;
    op.output_min = c.output_min;
    op.output_max = c.output_max;
    op.M = (int32_t)M; op.K = (int32_t)Kp; op.Kp = (int32_t)Kp; op.Nn = (int32_t)O; op.Np = (int32_t)O;
    op.in0 = a;
    op.out = out;
    packBf16Weights(&op, wk.data(), O, Kp);
    op.bias = newConst(std::vector<uint8_t>(b->data.begin(), b->data.begin() + (size_t)O * 4));
    planFcBf16Split(&op);
    ops_.push_back(op);
    finishOutput(post);
    return THIP_OK;
}

thip_status_t Emitter::emitDepthwiseBf16(const thip_hl_depthwise_conv2d_t &c) {
    const char *what = "torq_hl.depthwise_conv2d (bf16)";
    if (c.dilation[0] != 1 || c.dilation[1] != 1) return fail(THIP_UNIMPLEMENTED, "%s: dilation must be [1,1]", what);
    if (c.segment_output) return fail(THIP_UNIMPLEMENTED, "%s: segment_output is an NPU memory layout", what);
    if (c.is_dw1d_stride1) return fail(THIP_UNIMPLEMENTED, "%s: is_dw1d_stride1 is the 1-D special case", what);
    if (thip_status_t s = checkFloatAct(what, c.shift_factor, c.input_zp, c.weight_zp, c.output_zp)) return s;
    const Value *w, *init, *b;
    if (thip_status_t s = constantData(c.weights, "torq_hl.depthwise_conv2d weights", THIP_DTYPE_BF16, &w)) return s;
    if (w->rank != 4 || w->shape[1] != 1) return fail(THIP_INVALID_ARGUMENT, "%s: weights must be C,1,KH,KW", what);
    if (thip_status_t s = checkValue(c.init, "torq_hl.depthwise_conv2d init", &init)) return s;
    if (init->dtype != THIP_DTYPE_BF16) return fail(THIP_INVALID_ARGUMENT, "%s: init must be bf16", what);
    Dims4 d;
    DescRef in;
    if (thip_status_t s = nhwcInput(c.input, c.nhwc_input != 0, "torq_hl.depthwise_conv2d input", &d, &in, THIP_DTYPE_BF16)) return s;
    const int64_t C = w->shape[0], KH = w->shape[2], KW = w->shape[3];
    if (C != d.C) return fail(THIP_INVALID_ARGUMENT, "%s: weights have %lld channels, input has %lld", what, (long long)C, (long long)d.C);
    if (thip_status_t s = constantData(c.scale_bias, "torq_hl.depthwise_conv2d scale_bias", THIP_DTYPE_F32, &b)) return s;
    if (b->numel() < C) return fail(THIP_INVALID_ARGUMENT, "%s: scale_bias holds %lld floats, %lld needed", what, (long long)b->numel(), (long long)C);
    int64_t OH, OW;
    if (thip_status_t s = windowGeometry(what, d.H, d.W, KH, KW, c.pad, c.stride, &OH, &OW)) return s;
    if (!fitsInt32(d.N * OH * OW * C) || !fitsInt32(d.N * d.H * d.W * C)) return fail(THIP_UNIMPLEMENTED, "%s: tensor too large for 32-bit indexing", what);
    DescOp op;
    memset(&op, 0, sizeof(op));
    DescRef out;
    Pending post;
    if (thip_status_t s = nhwcOutput(c.init, c.nhwc_input != 0, "torq_hl.depthwise_conv2d init", THIP_DTYPE_BF16, d.N, C, OH, OW, &out, &post)) return s;
    const uint16_t *wd = (const uint16_t *)w->data.data();
    std::vector<uint16_t> wpk((size_t)(KH * KW * C));
    for (int64_t ch = 0; ch < C; ch++) {
        for (int64_t k = 0; k < KH * KW; k++) wpk[(size_t)(k * C + ch)] = wd[ch * KH * KW + k];
    }
    op.kind = kKindDepthwiseBf16;
    op.out_dtype = THIP_DTYPE_BF16;
    op.output_min = c.output_min;
    op.output_max = c.output_max;
    op.N = (int32_t)d.N; op.H = (int32_t)d.H; op.W = (int32_t)d.W; op.C = (int32_t)C;
    op.OH = (int32_t)OH; op.OW = (int32_t)OW; op.OC = (int32_t)C;
    op.KH = (int32_t)KH; op.KW = (int32_t)KW; op.SH = (int32_t)c.stride[0]; op.SW = (int32_t)c.stride[1];
    op.PL = (int32_t)c.pad[0]; op.PR = (int32_t)c.pad[1]; op.PT = (int32_t)c.pad[2]; op.PB = (int32_t)c.pad[3];
    op.in0 = in;
    op.out = out;
    op.weights = newConst(wpk);
    op.bias = newConst(std::vector<uint8_t>(b->data.begin(), b->data.begin() + (size_t)C * 4));
    ops_.push_back(op);
    finishOutput(post);
    return THIP_OK;
}

thip_status_t Emitter::emitFullyConnectedBf16(const thip_hl_fully_connected_t &c) {
    const char *what = "torq_hl.fully_connected (bf16)";
    if (thip_status_t s = checkFloatAct(what, c.shift_factor, c.input_zp, c.weight_zp, c.output_zp)) return s;
    const Value *w, *x, *init, *b;
    if (thip_status_t s = constantData(c.weights, "torq_hl.fully_connected weights", THIP_DTYPE_BF16, &w)) return s;
    if (w->rank != 2) return fail(THIP_INVALID_ARGUMENT, "%s: weights must be N,K", what);
    const int64_t N = w->shape[0], K = w->shape[1];
    if (thip_status_t s = checkValue(c.input, "torq_hl.fully_connected input", &x)) return s;
    if (K <= 0 || x->numel() % K != 0 || x->numel() == 0) return fail(THIP_INVALID_ARGUMENT, "%s: input does not end in K=%lld", what, (long long)K);
    if (K % 8 != 0) return fail(THIP_UNIMPLEMENTED, "%s: K must be a multiple of 8", what);
    if (state_[c.input].nhwcOfNchw) return fail(THIP_UNIMPLEMENTED, "%s: N,C,H,W intermediates are not accepted", what);
    const int64_t M = x->numel() / K;
    if (thip_status_t s = checkValue(c.init, "torq_hl.fully_connected init", &init)) return s;
    if (init->dtype != THIP_DTYPE_BF16) return fail(THIP_INVALID_ARGUMENT, "%s: init must be bf16", what);
    if (thip_status_t s = constantData(c.scale_bias, "torq_hl.fully_connected scale_bias", THIP_DTYPE_F32, &b)) return s;
    if (b->numel() < N) return fail(THIP_INVALID_ARGUMENT, "%s: scale_bias holds %lld floats, %lld needed", what, (long long)b->numel(), (long long)N);
    if (!fitsInt32(M) || !fitsInt32(K) || !fitsInt32(N) || !fitsInt32(M * N) || !fitsInt32(M * K)) {
        return fail(THIP_UNIMPLEMENTED, "%s: tensor too large for 32-bit indexing", what);
    }
    DescOp op;
    memset(&op, 0, sizeof(op));
    op.kind = kKindFcBf16;
    if (thip_status_t s = literalInput(c.input, "torq_hl.fully_connected input", &op.in0)) return s;
    if (thip_status_t s = literalOutput(c.init, "torq_hl.fully_connected init", THIP_DTYPE_BF16, M * N, &op.out)) return s;
    op.out_dtype = THIP_DTYPE_BF16;
    op.output_min = c.output_min;
    op.output_max = c.output_max;
    op.M = (int32_t)M; op.K = (int32_t)K; op.Kp = (int32_t)K; op.Nn = (int32_t)N; op.Np = (int32_t)N;
    packBf16Weights(&op, (const uint16_t *)w->data.data(), N, K);
    std::vector<uint8_t> bias(b->data.begin(), b->data.begin() + (size_t)N * 4);
    op.bias = newConst(bias);
    planFcBf16Split(&op);
    ops_.push_back(op);
    return THIP_OK;
}

thip_status_t Emitter::emitMatmulBf16(const thip_hl_matmul_t &c) {
    const char *what = "torq_hl.matmul (bf16)";
    if (thip_status_t s = checkFloatAct(what, c.shift, 0, 0, c.output_zp)) return s;
    if (const auto ft = foldedTranspose_.find(c.input2); ft != foldedTranspose_.end()) return emitDecodeMatmul(c, ft->second);
    const Value *a, *b, *init, *bv;
    if (thip_status_t s = checkValue(c.input1, "torq_hl.matmul input1", &a)) return s;
    if (thip_status_t s = checkValue(c.input2, "torq_hl.matmul input2", &b)) return s;
    if (thip_status_t s = checkValue(c.init, "torq_hl.matmul init", &init)) return s;
    if (b->dtype != THIP_DTYPE_BF16 || init->dtype != THIP_DTYPE_BF16) return fail(THIP_INVALID_ARGUMENT, "%s: input2 and init must be bf16", what);
    if (a->rank < 2 || a->rank > 3 || b->rank < 2 || b->rank > 3) return fail(THIP_UNIMPLEMENTED, "%s: operands must have rank 2 or 3", what);
    if (state_[c.input1].nhwcOfNchw || state_[c.input2].nhwcOfNchw) return fail(THIP_UNIMPLEMENTED, "%s: N,C,H,W intermediates are not accepted", what);
    const int64_t Ba = a->rank == 3 ? a->shape[0] : 1, Bb = b->rank == 3 ? b->shape[0] : 1;
    const int64_t M = a->shape[a->rank - 2], K = a->shape[a->rank - 1];
    const int64_t K2 = b->shape[b->rank - 2], N = b->shape[b->rank - 1];
    if (K != K2) return fail(THIP_INVALID_ARGUMENT, "%s: inner dimensions differ (%lld vs %lld)", what, (long long)K, (long long)K2);
    if (K % 8 != 0) return fail(THIP_UNIMPLEMENTED, "%s: K must be a multiple of 8", what);
    const int64_t B = std::max(Ba, Bb);
    if ((Ba != B && Ba != 1) || (Bb != B && Bb != 1)) return fail(THIP_INVALID_ARGUMENT, "%s: batch dimensions do not broadcast", what);
    if (thip_status_t s = constantData(c.scale_bias, "torq_hl.matmul scale_bias", THIP_DTYPE_F32, &bv)) return s;
    if (bv->numel() < 1) return fail(THIP_INVALID_ARGUMENT, "%s: scale_bias is empty", what);
    if (!fitsInt32(B * M * N) || !fitsInt32(B * M * K) || !fitsInt32(B * K * N)) return fail(THIP_UNIMPLEMENTED, "%s: tensor too large for 32-bit indexing", what);
    const float bias0 = ((const float *)bv->data.data())[0];
    DescRef biasRef = newConst(std::vector<float>((size_t)N, bias0));
    DescRef aRef, outRef;
    if (thip_status_t s = literalInput(c.input1, "torq_hl.matmul input1", &aRef)) return s;
    if (thip_status_t s = literalOutput(c.init, "torq_hl.matmul init", THIP_DTYPE_BF16, B * M * N, &outRef)) return s;
    // input2 as [N][K] per batch: transposed here when it is a constant, by a kernel when it is not
    std::vector<DescRef> wrefs;
    std::vector<std::vector<uint16_t>> wconst;
    const int64_t wcount = Bb == 1 ? 1 : B;
    // a folded torq_hl.expand_weights: few rows stream the int8 weights and expand them in registers (half the
    // weight traffic), many rows read weights expanded here, once
    const auto folded = foldedExpand_.find(c.input2);
    ExpandShape ex{};
    bool q8 = false;
    if (folded != foldedExpand_.end()) {
        if (thip_status_t s = checkExpandWeights(*folded->second, &ex)) return s;
        const int64_t rows = Ba == 1 ? M : B * M;
        const char *lim = getenv("THIP_EXPAND_INLINE_ROWS");
        q8 = ex.block % 32 == 0 && rows <= (lim ? atoll(lim) : 64);
        if (!q8) {
            const float lo = floatFromBits(folded->second->output_min), hi = floatFromBits(folded->second->output_max);
            const int8_t *wd = (const int8_t *)ex.w->data.data();
            const uint16_t *sd = (const uint16_t *)ex.scale->data.data();
            const float *bd = (const float *)ex.bias->data.data();
            std::vector<uint16_t> t((size_t)(N * K));
            for (int64_t k = 0; k < K; k++) {
                const int64_t g = k / ex.block;
                for (int64_t n = 0; n < N; n++) {
                    t[(size_t)(n * K + k)] = expandWeight(wd[k * N + n], sd[g * N + n], bd[g * ex.biasCols + n], lo, hi);
                }
            }
            wconst.push_back(std::move(t));
        }
    } else if (b->kind == kValueConstant) {
        const uint16_t *bd = (const uint16_t *)b->data.data();
        for (int64_t r = 0; r < wcount; r++) {
            std::vector<uint16_t> t((size_t)(N * K));
            for (int64_t k = 0; k < K; k++) {
                for (int64_t n = 0; n < N; n++) t[(size_t)(n * K + k)] = bd[(size_t)(r * K * N + k * N + n)];
            }
            wconst.push_back(std::move(t));
        }
    } else {
        DescRef bRef;
        if (thip_status_t s = literalInput(c.input2, "torq_hl.matmul input2", &bRef)) return s;
        for (int64_t r = 0; r < wcount; r++) {
            DescRef t = newTemp((uint64_t)(N * K) * 2);
            DescRef src = bRef;
            src.offset += (uint64_t)(r * K * N) * 2;
            emitTranspose(src, t, 1, K, N, 2);
            wrefs.push_back(t);
        }
    }
    // one record per batch, or a single one over all rows when input2 is shared
    const bool merge = Bb == 1;
    for (int64_t r = 0; r < (merge ? 1 : B); r++) {
        DescOp op;
        memset(&op, 0, sizeof(op));
        op.kind = kKindFcBf16;
        op.out_dtype = THIP_DTYPE_BF16;
        op.output_min = c.output_min;
        op.output_max = c.output_max;
        const int64_t rows = merge ? (Ba == 1 ? M : B * M) : M;
        op.M = (int32_t)rows; op.K = (int32_t)K; op.Kp = (int32_t)K; op.Nn = (int32_t)N; op.Np = (int32_t)N;
        op.in0 = aRef;
        op.in0.offset += (uint64_t)(Ba == 1 ? 0 : r * M * K) * 2;
        op.out = outRef;
        op.out.offset += (uint64_t)(r * M * N) * 2;
        if (q8) {
            const int steps = (int)((K + 63) / 64);
            const int64_t cols = roundUp(N, 32);
            const int8_t *wd = (const int8_t *)ex.w->data.data();
            std::vector<int8_t> packed((size_t)cols * (size_t)steps * 64, 0);
            for (int64_t k = 0; k < K; k++) {
                for (int64_t n = 0; n < N; n++) packed[fcBf16Q8FragmentOffset((int)n, (int)k, steps)] = wd[k * N + n];
            }
            std::vector<uint16_t> sc((size_t)(ex.G * cols), 0);
            std::vector<float> bi((size_t)(ex.G * cols), 0.0f);
            for (int64_t g = 0; g < ex.G; g++) {
                memcpy(&sc[(size_t)(g * cols)], (const uint16_t *)ex.scale->data.data() + g * N, (size_t)N * 2);
                memcpy(&bi[(size_t)(g * cols)], (const float *)ex.bias->data.data() + g * ex.biasCols, (size_t)N * 4);
            }
            op.loader = 2;
            op.weights = newConst(packed);
            op.scale = newConst(sc);
            op.table = newConst(bi);
            op.gran = (uint32_t)ex.block;
            op.Np = (int32_t)cols;
            op.bias0 = folded->second->output_min;
            op.scale0 = folded->second->output_max;
        } else if (!wconst.empty()) {
            packBf16Weights(&op, wconst[(size_t)(merge ? 0 : r)].data(), N, K);
        } else {
            op.weights = wrefs[(size_t)(merge ? 0 : r)];
        }
        op.bias = biasRef;
        planFcBf16Split(&op);
        ops_.push_back(op);
    }
    return THIP_OK;
}

thip_status_t Emitter::emitMaxPool(const thip_hl_maxpool2d_t &c) {
    const char *what = "torq_hl.maxpool2d";
    if (c.segment_output) return fail(THIP_UNIMPLEMENTED, "%s: segment_output is an NPU memory layout", what);
    if (c.input_zp < -128 || c.input_zp > 127) return fail(THIP_INVALID_ARGUMENT, "%s: input_zp outside int8", what);
    if (c.output_min > c.output_max || c.output_min < -128 || c.output_max > 127) return fail(THIP_INVALID_ARGUMENT, "%s: clamp outside int8", what);
    Dims4 d;
    DescRef in;
    if (thip_status_t s = nhwcInput(c.input, c.nhwc_input != 0, "torq_hl.maxpool2d input", &d, &in)) return s;
    int64_t OH, OW;
    if (thip_status_t s = windowGeometry(what, d.H, d.W, c.kernel[0], c.kernel[1], c.pad, c.stride, &OH, &OW)) return s;
    const int64_t Cp = physC(c.input, d.C);  // input and output are padded alike
    if (!fitsInt32(d.N * d.H * d.W * Cp)) return fail(THIP_UNIMPLEMENTED, "%s: tensor too large for 32-bit indexing", what);
    DescOp op;
    memset(&op, 0, sizeof(op));
    DescRef out;
    Pending post;
    if (thip_status_t s = nhwcOutput(c.init, c.nhwc_input != 0, "torq_hl.maxpool2d init", THIP_DTYPE_I8, d.N, d.C, OH, OW, &out, &post)) return s;
    op.kind = kKindMaxPool;
    op.out_dtype = THIP_DTYPE_I8;
    op.input_zp = c.input_zp;
    op.output_min = c.output_min;
    op.output_max = c.output_max;
    op.N = (int32_t)d.N; op.H = (int32_t)d.H; op.W = (int32_t)d.W; op.C = (int32_t)Cp;
    op.OH = (int32_t)OH; op.OW = (int32_t)OW; op.OC = (int32_t)Cp;
    op.KH = (int32_t)c.kernel[0]; op.KW = (int32_t)c.kernel[1]; op.SH = (int32_t)c.stride[0]; op.SW = (int32_t)c.stride[1];
    op.PL = (int32_t)c.pad[0]; op.PR = (int32_t)c.pad[1]; op.PT = (int32_t)c.pad[2]; op.PB = (int32_t)c.pad[3];
    op.in0 = in;
    op.out = out;
    ops_.push_back(op);
    finishOutput(post);
    return THIP_OK;
}

thip_status_t Emitter::emitAvgPool(const thip_hl_avg_pool2d_t &c) {
    const char *what = "torq_hl.avg_pool2d";
    const Value *x, *w, *sb;
    if (thip_status_t s = checkValue(c.input, "torq_hl.avg_pool2d input", &x)) return s;
    if (x->dtype == THIP_DTYPE_BF16) return emitAvgPoolBf16(c);
    if (x->rank != 4 || x->dtype != THIP_DTYPE_I8) return fail(THIP_INVALID_ARGUMENT, "%s: input must be an int8 N,H,W,C tensor", what);
    if (state_[c.input].nhwcOfNchw) return fail(THIP_INVALID_ARGUMENT, "%s: input %d is declared N,C,H,W; insert torq_hl.transpose [0,2,3,1]", what, (int)c.input);
    if (thip_status_t s = constantData(c.weights, "torq_hl.avg_pool2d weights", THIP_DTYPE_I8, &w)) return s;
    if (thip_status_t s = constantData(c.scale_bias, "torq_hl.avg_pool2d scale_bias", THIP_DTYPE_I32, &sb)) return s;
    if (w->numel() < 1 || sb->numel() < 2) return fail(THIP_INVALID_ARGUMENT, "%s: weights / scale_bias too short", what);
    if (thip_status_t s = checkRequant(what, c.shift_factor, c.output_zp, c.output_min, c.output_max, THIP_DTYPE_I8)) return s;
    const int64_t N = x->shape[0], H = x->shape[1], W = x->shape[2], C = x->shape[3];
    if (!fitsInt32(N * H * W * C)) return fail(THIP_UNIMPLEMENTED, "%s: tensor too large for 32-bit indexing", what);
    DescOp op;
    memset(&op, 0, sizeof(op));
    if (thip_status_t s = literalInput(c.input, "torq_hl.avg_pool2d input", &op.in0)) return s;
    if (thip_status_t s = literalOutput(c.init, "torq_hl.avg_pool2d init", THIP_DTYPE_I8, N * C, &op.out)) return s;
    op.kind = kKindAvgPool;
    op.out_dtype = THIP_DTYPE_I8;
    op.output_zp = c.output_zp;
    op.output_min = c.output_min;
    op.output_max = c.output_max;
    op.shift = c.shift_factor;
    op.N = (int32_t)N; op.H = (int32_t)H; op.W = (int32_t)W; op.C = (int32_t)C;
    op.w0 = ((const int8_t *)w->data.data())[0];
    op.bias0 = ((const int32_t *)sb->data.data())[0];
    op.scale0 = ((const int32_t *)sb->data.data())[1];
    ops_.push_back(op);
    return THIP_OK;
}

thip_status_t Emitter::emitAvgPoolBf16(const thip_hl_avg_pool2d_t &c) {
    // one bf16 weight and one float bias for every channel, no rescale
    // (compiler/torq/Conversions/LinalgToTorqHL/PoolingPattern.cpp:448-457)
    const char *what = "torq_hl.avg_pool2d (bf16)";
    if (thip_status_t s = checkFloatAct(what, c.shift_factor, c.input_zp, 0, c.output_zp)) return s;
    const Value *x, *w, *sb, *init;
    if (thip_status_t s = checkValue(c.input, "torq_hl.avg_pool2d input", &x)) return s;
    if (thip_status_t s = checkValue(c.init, "torq_hl.avg_pool2d init", &init)) return s;
    if (x->rank != 4 || init->dtype != THIP_DTYPE_BF16) return fail(THIP_INVALID_ARGUMENT, "%s: input must be N,H,W,C and init bf16", what);
    if (state_[c.input].nhwcOfNchw) return fail(THIP_INVALID_ARGUMENT, "%s: input %d is declared N,C,H,W; insert torq_hl.transpose [0,2,3,1]", what, (int)c.input);
    if (thip_status_t s = constantData(c.weights, "torq_hl.avg_pool2d weights", THIP_DTYPE_BF16, &w)) return s;
    if (thip_status_t s = constantData(c.scale_bias, "torq_hl.avg_pool2d scale_bias", THIP_DTYPE_F32, &sb)) return s;
    if (w->numel() < 1 || sb->numel() < 1) return fail(THIP_INVALID_ARGUMENT, "%s: weights / scale_bias too short", what);
    const int64_t N = x->shape[0], H = x->shape[1], W = x->shape[2], C = x->shape[3];
    if (!fitsInt32(N * H * W * C)) return fail(THIP_UNIMPLEMENTED, "%s: tensor too large for 32-bit indexing", what);
    DescOp op;
    memset(&op, 0, sizeof(op));
    if (thip_status_t s = literalInput(c.input, "torq_hl.avg_pool2d input", &op.in0)) return s;
    if (thip_status_t s = literalOutput(c.init, "torq_hl.avg_pool2d init", THIP_DTYPE_BF16, N * C, &op.out)) return s;
    op.kind = kKindAvgPoolBf16;
    op.out_dtype = THIP_DTYPE_BF16;
    op.output_min = c.output_min;
    op.output_max = c.output_max;
    op.N = (int32_t)N; op.H = (int32_t)H; op.W = (int32_t)W; op.C = (int32_t)C;
    op.w0 = ((const uint16_t *)w->data.data())[0];
    memcpy(&op.bias0, sb->data.data(), 4);
    ops_.push_back(op);
    return THIP_OK;
}

thip_status_t Emitter::checkExpandWeights(const thip_hl_expand_weights_t &c, ExpandShape *out) {
    const char *what = "torq_hl.expand_weights";
    ExpandShape e;
    if (thip_status_t s = checkValue(c.input, "torq_hl.expand_weights input", &e.w)) return s;
    if (thip_status_t s = checkValue(c.scale, "torq_hl.expand_weights scale", &e.scale)) return s;
    if (thip_status_t s = checkValue(c.scale_bias, "torq_hl.expand_weights scale_bias", &e.bias)) return s;
    if (thip_status_t s = checkValue(c.init, "torq_hl.expand_weights init", &e.init)) return s;
    if (e.w->dtype != THIP_DTYPE_I8) return fail(THIP_UNIMPLEMENTED, "%s: only int8 weights (4-bit and fp8 inputs are not on this path)", what);
    if (e.scale->dtype != THIP_DTYPE_BF16 || e.bias->dtype != THIP_DTYPE_F32 || e.init->dtype != THIP_DTYPE_BF16) {
        return fail(THIP_UNIMPLEMENTED, "%s: scale and init must be bf16 and scale_bias float32", what);
    }
    if (e.w->rank != 2) return fail(THIP_INVALID_ARGUMENT, "%s: input must be K,N", what);
    e.K = e.w->shape[0];
    e.N = e.w->shape[1];
    e.block = c.block_size;
    if (e.block <= 0 || e.K % e.block != 0) return fail(THIP_INVALID_ARGUMENT, "%s: block_size %lld does not divide K=%lld", what, (long long)e.block, (long long)e.K);
    e.G = e.K / e.block;
    const bool initOk = (e.init->rank == 2 && e.init->shape[0] == e.K && e.init->shape[1] == e.N) ||
                        (e.init->rank == 3 && e.init->shape[0] == 1 && e.init->shape[1] == e.K && e.init->shape[2] == e.N);
    if (!initOk) return fail(THIP_INVALID_ARGUMENT, "%s: init must be K,N or 1,K,N", what);
    if (e.scale->numel() != e.G * e.N) return fail(THIP_INVALID_ARGUMENT, "%s: scale must hold K/block_size x N values", what);
    if (e.bias->numel() % e.G != 0 || e.bias->numel() / e.G < e.N) return fail(THIP_INVALID_ARGUMENT, "%s: scale_bias must hold K/block_size rows of at least N values", what);
    e.biasCols = e.bias->numel() / e.G;
    if (!fitsInt32(e.K * e.N)) return fail(THIP_UNIMPLEMENTED, "%s: tensor too large for 32-bit indexing", what);
    *out = e;
    return THIP_OK;
}

thip_status_t Emitter::emitExpandWeights(const thip_hl_expand_weights_t &c) {
    ExpandShape e;
    if (thip_status_t s = checkExpandWeights(c, &e)) return s;
    if (foldedExpand_.count(c.init)) return THIP_OK;  // the matmul that reads it takes the quantized weights
    DescOp op;
    memset(&op, 0, sizeof(op));
    op.kind = kKindExpandWeights;
    op.out_dtype = THIP_DTYPE_BF16;
    op.output_min = c.output_min;
    op.output_max = c.output_max;
    op.K = (int32_t)e.K; op.Nn = (int32_t)e.N; op.Np = (int32_t)e.biasCols; op.gran = (uint32_t)e.block;
    op.M = 1; op.Kp = (int32_t)e.K;
    if (thip_status_t s = literalInput(c.input, "torq_hl.expand_weights input", &op.in0)) return s;
    if (thip_status_t s = literalInput(c.scale, "torq_hl.expand_weights scale", &op.scale)) return s;
    if (thip_status_t s = literalInput(c.scale_bias, "torq_hl.expand_weights scale_bias", &op.bias)) return s;
    if (thip_status_t s = literalOutput(c.init, "torq_hl.expand_weights init", THIP_DTYPE_BF16, e.K * e.N, &op.out)) return s;
    ops_.push_back(op);
    return THIP_OK;
}

static bool isIntDtype(int32_t d) { return d == THIP_DTYPE_I8 || d == THIP_DTYPE_I16 || d == THIP_DTYPE_I32; }

thip_status_t Emitter::eltwiseCommon(const char *what, thip_value_t input, thip_value_t init, DescOp *op) {
    const Value *x, *o;
    if (thip_status_t s = checkValue(input, what, &x)) return s;
    if (thip_status_t s = checkValue(init, what, &o)) return s;
    auto carried = [](int32_t d) { return isIntDtype(d) || d == THIP_DTYPE_I1; };
    if (!carried(x->dtype) || !carried(o->dtype)) return fail(THIP_UNIMPLEMENTED, "%s: int8 / int16 / int32 / i1 tensors only", what);
    if (x->numel() != o->numel() || x->numel() <= 0) return fail(THIP_INVALID_ARGUMENT, "%s: input and init differ in element count", what);
    if (state_[input].nhwcOfNchw) return fail(THIP_UNIMPLEMENTED, "%s: N,C,H,W intermediates are not accepted", what);
    if (!fitsInt32(x->numel())) return fail(THIP_UNIMPLEMENTED, "%s: tensor too large for 32-bit indexing", what);
    memset(op, 0, sizeof(*op));
    op->kind = kKindEltwise;
    op->gran = (uint32_t)elemSize(x->dtype);
    op->out_dtype = o->dtype == THIP_DTYPE_I1 ? THIP_DTYPE_I8 : o->dtype;  // a truth value is a byte to the kernel
    op->N = 1; op->H = 1; op->W = 1;
    op->C = (int32_t)x->numel();
    if (thip_status_t s = literalInput(input, what, &op->in0)) return s;
    return literalOutput(init, what, o->dtype, x->numel(), &op->out);
}

thip_status_t Emitter::emitFma(const thip_hl_fma_t &c) {
    const char *what = "torq_hl.fma";
    const Value *w, *sb, *init;
    if (thip_status_t s = checkValue(c.init, what, &init)) return s;
    if (thip_status_t s = checkRequant(what, c.shift_factor, c.output_zp, c.output_min, c.output_max, init->dtype)) return s;
    if (thip_status_t s = checkValue(c.weights, "torq_hl.fma weights", &w)) return s;
    if (w->kind != kValueConstant || (w->dtype != THIP_DTYPE_I8 && w->dtype != THIP_DTYPE_I16) || w->numel() < 1) {
        return fail(THIP_UNIMPLEMENTED, "%s: weights must be a constant int8 / int16 scalar", what);
    }
    if (thip_status_t s = constantData(c.scale_bias, "torq_hl.fma scale_bias", THIP_DTYPE_I32, &sb)) return s;
    if (sb->numel() < 2) return fail(THIP_INVALID_ARGUMENT, "%s: scale_bias too short", what);
    DescOp op;
    if (thip_status_t s = eltwiseCommon(what, c.input, c.init, &op)) return s;
    op.variant = kEltFma;
    op.w0 = w->dtype == THIP_DTYPE_I8 ? (int32_t)((const int8_t *)w->data.data())[0] : (int32_t)((const int16_t *)w->data.data())[0];
    op.bias0 = ((const int32_t *)sb->data.data())[0];
    op.scale0 = ((const int32_t *)sb->data.data())[1];
    op.shift = c.shift_factor;
    op.output_zp = c.output_zp;
    op.output_min = c.output_min;
    op.output_max = c.output_max;
    ops_.push_back(op);
    return THIP_OK;
}

thip_status_t Emitter::emitMul(const thip_hl_mul_t &c) {
    const char *what = "torq_hl.mul";
    const Value *a, *b, *init, *sb;
    if (thip_status_t s = checkValue(c.input1, "torq_hl.mul input1", &a)) return s;
    if (thip_status_t s = checkValue(c.input2, "torq_hl.mul input2", &b)) return s;
    if (thip_status_t s = checkValue(c.init, "torq_hl.mul init", &init)) return s;
    if (a->dtype != b->dtype || (a->dtype != THIP_DTYPE_I8 && a->dtype != THIP_DTYPE_I16)) {
        return fail(THIP_UNIMPLEMENTED, "%s: inputs must both be int8 or both int16 (the bf16 form is not on this path)", what);
    }
    if (!isIntDtype(init->dtype)) return fail(THIP_UNIMPLEMENTED, "%s: init must be int8 / int16 / int32", what);
    if (thip_status_t s = checkRequant(what, c.shift, c.output_zp, c.output_min, c.output_max, init->dtype)) return s;
    const int64_t count = init->numel();
    if ((a->numel() != count && a->numel() != 1) || (b->numel() != count && b->numel() != 1) || count <= 0) {
        return fail(THIP_UNIMPLEMENTED, "%s: an input must have init's element count or one element", what);
    }
    if (state_[c.input1].nhwcOfNchw || state_[c.input2].nhwcOfNchw) return fail(THIP_UNIMPLEMENTED, "%s: N,C,H,W intermediates are not accepted", what);
    if (!fitsInt32(count)) return fail(THIP_UNIMPLEMENTED, "%s: tensor too large for 32-bit indexing", what);
    if (thip_status_t s = constantData(c.scale_bias, "torq_hl.mul scale_bias", THIP_DTYPE_I32, &sb)) return s;
    if (sb->numel() < 2) return fail(THIP_INVALID_ARGUMENT, "%s: scale_bias too short", what);
    DescOp op;
    memset(&op, 0, sizeof(op));
    op.kind = kKindEltwise;
    op.variant = kEltMul;
    op.gran = (uint32_t)elemSize(a->dtype);
    op.out_dtype = init->dtype;
    op.N = 1; op.H = 1; op.W = 1;
    op.C = (int32_t)count;
    op.w1 = count == 1 ? 0 : a->numel() == 1 ? 1 : b->numel() == 1 ? 2 : 0;
    if (thip_status_t s = literalInput(c.input1, "torq_hl.mul input1", &op.in0)) return s;
    if (thip_status_t s = literalInput(c.input2, "torq_hl.mul input2", &op.in1)) return s;
    if (thip_status_t s = literalOutput(c.init, "torq_hl.mul init", init->dtype, count, &op.out)) return s;
    op.bias0 = ((const int32_t *)sb->data.data())[0];
    op.scale0 = ((const int32_t *)sb->data.data())[1];
    op.shift = c.shift;
    op.output_zp = c.output_zp;
    op.output_min = c.output_min;
    op.output_max = c.output_max;
    ops_.push_back(op);
    return THIP_OK;
}

thip_status_t Emitter::emitBinary(const thip_hl_elementwisebinary_t &c) {
    const char *what = "torq_hl.elementwisebinary";
    uint32_t variant;
    switch (c.op_type) {  // ElementwiseOpEnum, compiler/torq/Dialect/TorqHL/TorqHLAttrs.td:219-235
    case 0: variant = kEltAnd; break;
    case 1: variant = kEltOr; break;
    case 2: variant = kEltXor; break;
    case 4: variant = kEltMin; break;
    case 5: variant = kEltMax; break;
    case 6: variant = kEltGreater; break;
    case 7: variant = kEltGreaterEqual; break;
    case 8: variant = kEltEqual; break;
    case 9: variant = kEltLogicalAnd; break;
    case 10: variant = kEltLogicalOr; break;
    case 11: variant = kEltLogicalXor; break;
    default: return fail(THIP_UNIMPLEMENTED, "%s: op_type %d is not on this path (bitwise, minimum / maximum, comparisons and logical ops are)", what, (int)c.op_type);
    }
    const Value *a, *b, *init;
    if (thip_status_t s = checkValue(c.input1, "torq_hl.elementwisebinary input1", &a)) return s;
    if (thip_status_t s = checkValue(c.input2, "torq_hl.elementwisebinary input2", &b)) return s;
    if (thip_status_t s = checkValue(c.init, "torq_hl.elementwisebinary init", &init)) return s;
    const bool compares = variant >= kEltGreater && variant <= kEltEqual, logical = variant >= kEltLogicalAnd;
    if (a->dtype != b->dtype) return fail(THIP_UNIMPLEMENTED, "%s: the inputs must share one type", what);
    if (logical) {
        if (a->dtype != THIP_DTYPE_I1 || init->dtype != THIP_DTYPE_I1) return fail(THIP_UNIMPLEMENTED, "%s: logical ops take and give i1 tensors", what);
    } else if (compares) {
        if (!isIntDtype(a->dtype) || init->dtype != THIP_DTYPE_I1) return fail(THIP_UNIMPLEMENTED, "%s: a comparison takes int8 / int16 / int32 tensors and gives an i1 tensor", what);
    } else if (!isIntDtype(a->dtype) || a->dtype != init->dtype) {
        return fail(THIP_UNIMPLEMENTED, "%s: inputs and init must share one integer type", what);
    }
    if (a->numel() != b->numel() || a->numel() != init->numel()) return fail(THIP_INVALID_ARGUMENT, "%s: operand shapes differ (broadcast is materialised by the patterns)", what);
    if (c.is_unsigned && (a->dtype != THIP_DTYPE_I16 || logical || variant <= kEltXor)) return fail(THIP_UNIMPLEMENTED, "%s: is_unsigned applies to 16-bit minimum / maximum / comparisons only", what);
    if (state_[c.input2].nhwcOfNchw) return fail(THIP_UNIMPLEMENTED, "%s: N,C,H,W intermediates are not accepted", what);
    DescOp op;
    if (thip_status_t s = eltwiseCommon(what, c.input1, c.init, &op)) return s;
    if (thip_status_t s = literalInput(c.input2, "torq_hl.elementwisebinary input2", &op.in1)) return s;
    op.variant = variant;
    op.w0 = c.is_unsigned ? 1 : 0;
    ops_.push_back(op);
    return THIP_OK;
}

thip_status_t Emitter::emitUnary(const thip_hl_elementwiseunary_t &c) {
    const char *what = "torq_hl.elementwiseunary";
    if (c.op_type != 3 && c.op_type != 12) return fail(THIP_UNIMPLEMENTED, "%s: op_type %d is not a unary mode (BITWISE_NOT 3 and LOGICAL_NOT 12 are)", what, (int)c.op_type);
    const Value *x, *init;
    if (thip_status_t s = checkValue(c.input, "torq_hl.elementwiseunary input", &x)) return s;
    if (thip_status_t s = checkValue(c.init, "torq_hl.elementwiseunary init", &init)) return s;
    if (x->dtype != init->dtype) return fail(THIP_UNIMPLEMENTED, "%s: input and init must share one type", what);
    if (c.op_type == 3 ? !isIntDtype(x->dtype) : x->dtype != THIP_DTYPE_I1) return fail(THIP_UNIMPLEMENTED, "%s: BITWISE_NOT takes integers, LOGICAL_NOT i1", what);
    DescOp op;
    if (thip_status_t s = eltwiseCommon(what, c.input, c.init, &op)) return s;
    op.variant = c.op_type == 3 ? kEltNot : kEltLogicalNot;
    ops_.push_back(op);
    return THIP_OK;
}

thip_status_t Emitter::emitShift(const thip_hl_elementwiseshift_t &c) {
    const char *what = "torq_hl.elementwiseshift";
    uint32_t variant;
    switch (c.op_type) {  // ShiftModeEnum, compiler/torq/Dialect/TorqHL/TorqHLAttrs.td:239-246
    case 0: variant = kEltLsr; break;
    case 1: variant = kEltLsl; break;
    case 2: variant = kEltAsr; break;
    default: return fail(THIP_UNIMPLEMENTED, "%s: shift mode %d is not lowered (LSR 0, LSL 1 and ASR 2 are)", what, (int)c.op_type);
    }
    const Value *a, *b, *init;
    if (thip_status_t s = checkValue(c.input1, "torq_hl.elementwiseshift input1", &a)) return s;
    if (thip_status_t s = checkValue(c.input2, "torq_hl.elementwiseshift input2", &b)) return s;
    if (thip_status_t s = checkValue(c.init, "torq_hl.elementwiseshift init", &init)) return s;
    if (!isIntDtype(a->dtype) || a->dtype != b->dtype || a->dtype != init->dtype) return fail(THIP_UNIMPLEMENTED, "%s: inputs and init must share one integer type", what);
    if (a->numel() != b->numel() || a->numel() != init->numel()) return fail(THIP_INVALID_ARGUMENT, "%s: operand shapes differ", what);
    if (state_[c.input2].nhwcOfNchw) return fail(THIP_UNIMPLEMENTED, "%s: N,C,H,W intermediates are not accepted", what);
    DescOp op;
    if (thip_status_t s = eltwiseCommon(what, c.input1, c.init, &op)) return s;
    if (thip_status_t s = literalInput(c.input2, "torq_hl.elementwiseshift input2", &op.in1)) return s;
    op.variant = variant;
    op.w0 = c.round ? 1 : 0;
    ops_.push_back(op);
    return THIP_OK;
}

// torq_hl.table in the forms the lookup patterns produce (compiler/torq/Conversions/LinalgToTorqHL/
// ExtractPattern.cpp:30-62,285-298,432-545): scale_bias = [-128, 128] turns the input into a 9.7 fixed-point index
// with a zero fraction (compiler/torq/Conversions/TorqHLToTorqHW/TablePattern.cpp:20-27), so only the base half of a
// segment word is ever used and the op is out = lut[int8(x) + 128], the statement of the program it replaced.  The
// record carries the 256 values in the output's type.
thip_status_t Emitter::emitTable(const thip_hl_table_t &c, const std::vector<int32_t> &staticTable) {
    const char *what = "torq_hl.table";
    const Value *x, *init, *sb;
    if (thip_status_t s = checkValue(c.input, "torq_hl.table input", &x)) return s;
    if (thip_status_t s = checkValue(c.init, "torq_hl.table init", &init)) return s;
    if (thip_status_t s = constantData(c.scale_bias, "torq_hl.table scale_bias", THIP_DTYPE_I32, &sb)) return s;
    if (sb->numel() < 2) return fail(THIP_INVALID_ARGUMENT, "%s: scale_bias too short", what);
    const int32_t *sbd = (const int32_t *)sb->data.data();
    if (sbd[0] != -128 || sbd[1] != 128) {
        return fail(THIP_UNIMPLEMENTED, "%s: scale_bias [%d, %d] asks for an interpolated lookup; only the plain lookup [-128, 128] is on this path", what, (int)sbd[0], (int)sbd[1]);
    }
    const bool out8 = init->dtype == THIP_DTYPE_I8, out16 = init->dtype == THIP_DTYPE_I16;
    if (!(out8 && x->dtype == THIP_DTYPE_I8) && !(out16 && (x->dtype == THIP_DTYPE_I8 || x->dtype == THIP_DTYPE_I16))) {
        return fail(THIP_UNIMPLEMENTED, "%s: int8 -> int8, int8 -> int16 and int16 -> int16 lookups only", what);
    }
    const int32_t *words = nullptr;
    int64_t count = 0;
    if (c.static_table_count > 0) {
        if (c.dynamic_table != THIP_NO_VALUE) return fail(THIP_INVALID_ARGUMENT, "%s: both static_table and dynamic_table given", what);
        words = staticTable.data();
        count = (int64_t)staticTable.size();
    } else {
        const Value *t;
        if (thip_status_t s = checkValue(c.dynamic_table, "torq_hl.table dynamic_table", &t)) return s;
        if (t->kind != kValueConstant) return fail(THIP_UNIMPLEMENTED, "%s: a run-time table is torq_hl.gather in the reference and is not on this path", what);
        if (t->dtype != THIP_DTYPE_I32) return fail(THIP_INVALID_ARGUMENT, "%s: the table must be int32 segment words", what);
        words = (const int32_t *)t->data.data();
        count = t->numel();
    }
    if (count != 256) return fail(THIP_UNIMPLEMENTED, "%s: the lookup patterns produce 256 entries, this table has %lld", what, (long long)count);
    std::vector<uint8_t> lut(out8 ? 256 : 512);
    for (int i = 0; i < 256; i++) {
        const int16_t base = (int16_t)(uint16_t)((uint32_t)words[i] & 0xffffu);
        if (out8) {
            if (base & 0xff) return fail(THIP_UNIMPLEMENTED, "%s: entry %d has a base that is not an int8 value shifted left by 8", what, i);
            lut[(size_t)i] = (uint8_t)(int8_t)(base >> 8);
        } else {
            memcpy(&lut[(size_t)i * 2], &base, 2);
        }
    }
    DescOp op;
    if (thip_status_t s = eltwiseCommon(what, c.input, c.init, &op)) return s;
    op.variant = kEltTable;
    op.in1 = newConst(lut);
    ops_.push_back(op);
    return THIP_OK;
}

thip_status_t Emitter::emitAct(const thip_hl_act_t &c, const std::string &name) {
    const char *what = "torq_hl.act";
    if (c.weights != THIP_NO_VALUE) return fail(THIP_UNIMPLEMENTED, "%s: weights (the unsigned cast) are not on this path", what);
    const Value *init;
    if (thip_status_t s = checkValue(c.init, what, &init)) return s;
    int64_t lo, hi;
    switch (init->dtype) {
    case THIP_DTYPE_I8: lo = -128; hi = 127; break;
    case THIP_DTYPE_I16: lo = -32768; hi = 32767; break;
    default: lo = INT32_MIN; hi = INT32_MAX; break;
    }
    uint32_t variant;
    if (name == "clamp") {
        variant = kEltClamp;
        if (c.min_int > c.max_int) return fail(THIP_INVALID_ARGUMENT, "%s: min_int > max_int", what);
        // a clip range beyond the output type would leave the order of clip and truncation to decide the result
        if (c.min_int < lo || c.max_int > hi) return fail(THIP_INVALID_ARGUMENT, "%s: clamp range exceeds the output element type", what);
        lo = c.min_int;
        hi = c.max_int;
    } else if (name == "abs") {
        variant = kEltAbs;
    } else if (name == "negate") {
        variant = kEltNegate;
    } else if (name == "i2i") {
        variant = kEltCast;
        lo = INT32_MIN;
        hi = INT32_MAX;
    } else {
        return fail(THIP_UNIMPLEMENTED, "%s: \"%s\" is not on this path (clamp, abs, negate, i2i on integers are)", what, name.c_str());
    }
    DescOp op;
    if (thip_status_t s = eltwiseCommon(what, c.input, c.init, &op)) return s;
    op.variant = variant;
    op.output_min = (int32_t)lo;
    op.output_max = (int32_t)hi;
    ops_.push_back(op);
    return THIP_OK;
}

thip_status_t Emitter::emitAdd(const thip_hl_add_t &c) {
    const char *what = "torq_hl.add";
    if (c.segment_output) return fail(THIP_UNIMPLEMENTED, "%s: segment_output is an NPU memory layout", what);
    if (c.rhs_is_scalar) return fail(THIP_UNIMPLEMENTED, "%s: rhs_is_scalar (tensor + scalar) is not on this path", what);
    const Value *a, *b, *init, *w, *sb;
    if (thip_status_t s = checkValue(c.input1, "torq_hl.add input1", &a)) return s;
    if (thip_status_t s = checkValue(c.input2, "torq_hl.add input2", &b)) return s;
    if (thip_status_t s = checkValue(c.init, "torq_hl.add init", &init)) return s;
    const bool bf16 = a->dtype == THIP_DTYPE_BF16;
    if (bf16 ? (b->dtype != THIP_DTYPE_BF16 || init->dtype != THIP_DTYPE_BF16)
             : (a->dtype != THIP_DTYPE_I8 || b->dtype != THIP_DTYPE_I8 || init->dtype != THIP_DTYPE_I8)) {
        return fail(THIP_UNIMPLEMENTED, "%s: int8 tensors, or bf16 tensors, only", what);
    }
    if (a->rank != b->rank || a->rank != init->rank) return fail(THIP_INVALID_ARGUMENT, "%s: operand ranks differ (broadcast is materialised by the patterns)", what);
    for (int i = 0; i < a->rank; i++) {
        if (a->shape[i] != b->shape[i] || a->shape[i] != init->shape[i]) return fail(THIP_INVALID_ARGUMENT, "%s: operand shapes differ", what);
    }
    if (bf16) {
        // floating-point partials: two bf16 weights, one float bias, no rescale
        // (compiler/torq/Conversions/TorqHLToTorqHW/AddPattern.cpp:118-121,262-281)
        if (thip_status_t s = checkFloatAct(what, c.shift_factor, c.input_zp, 0, c.output_zp)) return s;
        if (thip_status_t s = constantData(c.weights, "torq_hl.add weights", THIP_DTYPE_BF16, &w)) return s;
        if (thip_status_t s = constantData(c.scale_bias, "torq_hl.add scale_bias", THIP_DTYPE_F32, &sb)) return s;
        if (w->numel() < 2 || sb->numel() < 1) return fail(THIP_INVALID_ARGUMENT, "%s: weights / scale_bias too short", what);
        if (state_[c.input1].nhwcOfNchw || state_[c.input2].nhwcOfNchw) return fail(THIP_UNIMPLEMENTED, "%s: N,C,H,W intermediates are not accepted", what);
        if (!fitsInt32(a->numel())) return fail(THIP_UNIMPLEMENTED, "%s: tensor too large for 32-bit indexing", what);
        DescOp op;
        memset(&op, 0, sizeof(op));
        op.kind = kKindAddBf16;
        op.out_dtype = THIP_DTYPE_BF16;
        op.output_min = c.output_min;
        op.output_max = c.output_max;
        op.w0 = ((const uint16_t *)w->data.data())[0];
        op.w1 = ((const uint16_t *)w->data.data())[1];
        memcpy(&op.bias0, sb->data.data(), 4);
        if (thip_status_t s = literalInput(c.input1, "torq_hl.add input1", &op.in0)) return s;
        if (thip_status_t s = literalInput(c.input2, "torq_hl.add input2", &op.in1)) return s;
        if (thip_status_t s = literalOutput(c.init, "torq_hl.add init", THIP_DTYPE_BF16, a->numel(), &op.out)) return s;
        op.N = 1; op.H = 1; op.W = 1;
        op.C = (int32_t)a->numel();
        ops_.push_back(op);
        return THIP_OK;
    }
    if (thip_status_t s = constantData(c.weights, "torq_hl.add weights", THIP_DTYPE_I16, &w)) return s;
    if (thip_status_t s = constantData(c.scale_bias, "torq_hl.add scale_bias", THIP_DTYPE_I32, &sb)) return s;
    if (w->numel() < 2 || sb->numel() < 2) return fail(THIP_INVALID_ARGUMENT, "%s: weights / scale_bias too short", what);
    if (thip_status_t s = checkRequant(what, c.shift_factor, c.output_zp, c.output_min, c.output_max, THIP_DTYPE_I8)) return s;
    DescOp op;
    memset(&op, 0, sizeof(op));
    op.kind = kKindAdd;
    op.out_dtype = THIP_DTYPE_I8;
    op.output_zp = c.output_zp;
    op.output_min = c.output_min;
    op.output_max = c.output_max;
    op.shift = c.shift_factor;
    op.w0 = ((const int16_t *)w->data.data())[0];
    op.w1 = ((const int16_t *)w->data.data())[1];
    op.bias0 = ((const int32_t *)sb->data.data())[0];
    op.scale0 = ((const int32_t *)sb->data.data())[1];
    // elements in memory: the three operands of an add are padded alike (padded channels hold
    // values nobody reads)
    const int64_t count = physNumel(c.init);
    if (!fitsInt32(count)) return fail(THIP_UNIMPLEMENTED, "%s: tensor too large for 32-bit indexing", what);
    Pending post;
    // Elementwise: any memory order works as long as all three agree.  If one
    // operand is an N,C,H,W intermediate kept as NHWC, bring the others to it.
    const bool anyNhwc = state_[c.input1].nhwcOfNchw || state_[c.input2].nhwcOfNchw;
    if (anyNhwc && a->rank == 4) {
        Dims4 d;
        if (thip_status_t s = nhwcInput(c.input1, false, "torq_hl.add input1", &d, &op.in0)) return s;
        if (thip_status_t s = nhwcInput(c.input2, false, "torq_hl.add input2", &d, &op.in1)) return s;
        if (thip_status_t s = nhwcOutput(c.init, false, "torq_hl.add init", THIP_DTYPE_I8, d.N, d.C, d.H, d.W, &op.out, &post)) return s;
    } else {
        if (thip_status_t s = literalInput(c.input1, "torq_hl.add input1", &op.in0)) return s;
        if (thip_status_t s = literalInput(c.input2, "torq_hl.add input2", &op.in1)) return s;
        if (thip_status_t s = literalOutput(c.init, "torq_hl.add init", THIP_DTYPE_I8, a->numel(), &op.out, count)) return s;
    }
    op.N = 1; op.H = 1; op.W = 1;
    op.C = (int32_t)count;
    ops_.push_back(op);
    finishOutput(post);
    return THIP_OK;
}

thip_status_t Emitter::emitTransposeOp(const thip_hl_transpose_t &c) {
    const char *what = "torq_hl.transpose";
    const Value *x, *init;
    if (thip_status_t s = checkValue(c.input, "torq_hl.transpose input", &x)) return s;
    if (thip_status_t s = checkValue(c.init, "torq_hl.transpose init", &init)) return s;
    const uint32_t elem = (uint32_t)elemSize(x->dtype);
    if (x->dtype != init->dtype || (elem != 1 && elem != 2)) return fail(THIP_UNIMPLEMENTED, "%s: 8- and 16-bit tensors of one type only", what);
    const int32_t dt = x->dtype;
    if (c.rank != x->rank || c.rank != init->rank) return fail(THIP_INVALID_ARGUMENT, "%s: rank mismatch", what);
    for (int i = 0; i < c.rank; i++) {
        if (c.perm[i] < 0 || c.perm[i] >= c.rank || init->shape[i] != x->shape[c.perm[i]]) {
            return fail(THIP_INVALID_ARGUMENT, "%s: init shape is not the permuted input shape", what);
        }
    }
    int64_t B = 1, R = 0, S = 0;
    bool toNhwc = false, toNchw = false;
    if (c.rank == 4 && c.perm[0] == 0 && c.perm[1] == 2 && c.perm[2] == 3 && c.perm[3] == 1) {
        toNhwc = true;  // N,C,H,W -> N,H,W,C
        B = x->shape[0]; R = x->shape[1]; S = x->shape[2] * x->shape[3];
    } else if (c.rank == 4 && c.perm[0] == 0 && c.perm[1] == 3 && c.perm[2] == 1 && c.perm[3] == 2) {
        toNchw = true;  // N,H,W,C -> N,C,H,W
        B = x->shape[0]; R = x->shape[1] * x->shape[2]; S = x->shape[3];
    } else if (c.rank == 2 && c.perm[0] == 1 && c.perm[1] == 0) {
        R = x->shape[0]; S = x->shape[1];
    } else if (c.rank == 3 && c.perm[0] == 0 && c.perm[1] == 2 && c.perm[2] == 1) {
        B = x->shape[0]; R = x->shape[1]; S = x->shape[2];
    } else {
        return fail(THIP_UNIMPLEMENTED, "%s: unsupported permutation", what);
    }
    if (!fitsInt32(x->numel())) return fail(THIP_UNIMPLEMENTED, "%s: tensor too large for 32-bit indexing", what);
    DescRef in;
    if (thip_status_t s = literalInput(c.input, "torq_hl.transpose input", &in)) return s;
    const bool inNhwcOfNchw = state_[c.input].nhwcOfNchw;
    if (init->kind == kValueTensor) {
        // Fold with the layout the producer already wrote.
        if (toNhwc && inNhwcOfNchw) {
            state_[c.init] = state_[c.input];
            state_[c.init].nhwcOfNchw = false;  // literal N,H,W,C now
            return THIP_OK;
        }
        if (toNchw && !inNhwcOfNchw) {
            state_[c.init].ref = in;
            state_[c.init].defined = true;
            state_[c.init].nhwcOfNchw = !(S == 1 || R == 1);
            return THIP_OK;
        }
    }
    if (inNhwcOfNchw) {
        if (toNhwc) {
            // bytes are already N,H,W,C: copy through a double transpose is wasteful, but
            // a binding destination needs its own bytes; use add-free copy = transpose with R == 1
            DescRef out;
            if (thip_status_t s = literalOutput(c.init, "torq_hl.transpose init", dt, x->numel(), &out)) return s;
            emitTranspose(in, out, 1, 1, x->numel(), elem);
            return THIP_OK;
        }
        return fail(THIP_UNIMPLEMENTED, "%s: permutation of an N,C,H,W intermediate other than [0,2,3,1]", what);
    }
    DescRef out;
    if (thip_status_t s = literalOutput(c.init, "torq_hl.transpose init", dt, x->numel(), &out)) return s;
    emitTranspose(in, out, B, R, S, elem);
    return THIP_OK;
}

// ---- decode-shaped programs ------------------------------------------------------------------------------------
// A decoder's step is a chain of some hundred small dependent ops on one to 32 rows: what it costs is the number of
// launches and the memory round trips inside each.  The ops are therefore grouped: linears that read the same rows
// become one record (query, key and value projections), two linears whose results meet in an add become one record
// that computes both and adds (gate and up), the add behind a linear moves into its epilogue (residual connections),
// and a transpose in front of a matmul's input2 is read in place.  THIP_NO_DECODE_FUSION leaves every op its own record.

void Emitter::planDecodeFolding() {
    foldedTranspose_.clear();
    consumed_.assign(prog_.ops.size(), 0);
    if (getenv("THIP_NO_DECODE_FUSION")) return;
    const size_t n = prog_.values.size();
    auto valid = [&](thip_value_t v) { return v >= 0 && (size_t)v < n; };
    for (size_t t = 0; t < prog_.ops.size(); t++) {
        if (prog_.ops[t].kind != kHlTranspose) continue;
        const thip_hl_transpose_t &tr = prog_.ops[t].u.tr;
        if (!valid(tr.init) || !valid(tr.input)) continue;
        const Value &res = prog_.values[(size_t)tr.init], &src = prog_.values[(size_t)tr.input];
        if (res.kind != kValueTensor || res.dtype != THIP_DTYPE_BF16 || src.dtype != THIP_DTYPE_BF16 || src.kind == kValueConstant) continue;
        const bool swap2 = tr.rank == 2 && tr.perm[0] == 1 && tr.perm[1] == 0;
        const bool swap3 = tr.rank == 3 && tr.perm[0] == 0 && tr.perm[1] == 2 && tr.perm[2] == 1;
        if ((!swap2 && !swap3) || src.rank != tr.rank || res.rank != tr.rank || valueReads_[(size_t)tr.init] != 1) continue;
        bool shapeOk = true;
        for (int i = 0; i < tr.rank; i++) shapeOk = shapeOk && res.shape[i] == src.shape[tr.perm[i]];
        if (!shapeOk) continue;  // emitTransposeOp reports it
        for (size_t m = t + 1; m < prog_.ops.size(); m++) {
            if (prog_.ops[m].kind != kHlMatmul || prog_.ops[m].u.mm.input2 != tr.init) continue;
            const thip_hl_matmul_t &mm = prog_.ops[m].u.mm;
            if (!valid(mm.input1) || !valid(mm.init) || mm.input1 == tr.init) break;
            const Value &a = prog_.values[(size_t)mm.input1];
            if (a.dtype != THIP_DTYPE_BF16 || a.rank < 2 || a.rank > 3 || a.shape[a.rank - 2] > kDecMaxRows) break;
            const int64_t batches = std::max<int64_t>(a.rank == 3 ? a.shape[0] : 1, res.rank == 3 ? res.shape[0] : 1);
            if (batches > 65535 || a.shape[a.rank - 1] % 8 != 0) break;
            foldedTranspose_[tr.init] = t;
            break;
        }
    }
}

thip_status_t Emitter::emitDecodeMatmul(const thip_hl_matmul_t &c, size_t transposeAt) {
    const char *what = "torq_hl.matmul (bf16, transposed input2 read in place)";
    const thip_hl_transpose_t &tr = prog_.ops[transposeAt].u.tr;
    const Value *a, *w, *init, *bv;
    if (thip_status_t s = checkValue(c.input1, "torq_hl.matmul input1", &a)) return s;
    if (thip_status_t s = checkValue(tr.input, "torq_hl.transpose input", &w)) return s;
    if (thip_status_t s = checkValue(c.init, "torq_hl.matmul init", &init)) return s;
    if (init->dtype != THIP_DTYPE_BF16) return fail(THIP_INVALID_ARGUMENT, "%s: init must be bf16", what);
    if (state_[c.input1].nhwcOfNchw || state_[tr.input].nhwcOfNchw) return fail(THIP_UNIMPLEMENTED, "%s: N,C,H,W intermediates are not accepted", what);
    const int64_t Ba = a->rank == 3 ? a->shape[0] : 1, Bw = w->rank == 3 ? w->shape[0] : 1;
    const int64_t M = a->shape[a->rank - 2], K = a->shape[a->rank - 1];
    const int64_t N = w->shape[w->rank - 2], K2 = w->shape[w->rank - 1];  // the transpose's input: [N][K]
    if (K != K2) return fail(THIP_INVALID_ARGUMENT, "%s: inner dimensions differ (%lld vs %lld)", what, (long long)K, (long long)K2);
    const int64_t B = std::max(Ba, Bw);
    if ((Ba != B && Ba != 1) || (Bw != B && Bw != 1)) return fail(THIP_INVALID_ARGUMENT, "%s: batch dimensions do not broadcast", what);
    if (thip_status_t s = constantData(c.scale_bias, "torq_hl.matmul scale_bias", THIP_DTYPE_F32, &bv)) return s;
    if (bv->numel() < 1) return fail(THIP_INVALID_ARGUMENT, "%s: scale_bias is empty", what);
    if (!fitsInt32(B * M * N) || !fitsInt32(B * M * K) || !fitsInt32(B * K * N)) return fail(THIP_UNIMPLEMENTED, "%s: tensor too large for 32-bit indexing", what);
    DescOp op;
    memset(&op, 0, sizeof(op));
    op.kind = kKindDecMatmul;
    op.out_dtype = THIP_DTYPE_BF16;
    op.output_min = c.output_min;
    op.output_max = c.output_max;
    memcpy(&op.bias0, bv->data.data(), 4);
    op.TB = (int32_t)B; op.M = (int32_t)M; op.K = (int32_t)K; op.Kp = (int32_t)K; op.Nn = (int32_t)N; op.Np = (int32_t)N;
    op.w0 = (Ba == 1 && B > 1) ? 1 : 0;
    op.w1 = (Bw == 1 && B > 1) ? 1 : 0;
    if (thip_status_t s = literalInput(c.input1, "torq_hl.matmul input1", &op.in0)) return s;
    if (thip_status_t s = literalInput(tr.input, "torq_hl.transpose input", &op.weights)) return s;
    if (thip_status_t s = literalOutput(c.init, "torq_hl.matmul init", THIP_DTYPE_BF16, B * M * N, &op.out)) return s;
    if ((op.in0.offset & 15) || (op.weights.offset & 15) || (op.out.offset & 7)) return fail(THIP_UNIMPLEMENTED, "%s: a view at an offset that is no multiple of 16 bytes", what);
    ops_.push_back(op);
    return THIP_OK;
}

size_t Emitter::nextLiveOp(size_t at) const {
    for (size_t i = at + 1; i < prog_.ops.size(); i++) {
        const HlOp &op = prog_.ops[i];
        if (consumed_[i]) continue;
        if (op.kind == kHlExpandWeights && foldedExpand_.count(op.u.ew.init)) continue;
        if (op.kind == kHlTranspose && foldedTranspose_.count(op.u.tr.init)) continue;
        return i;
    }
    return prog_.ops.size();
}

// LDS a workgroup of the grouped linear kernel needs for its share of ONE matrix: 16 columns of the whole K, in whole
// k-blocks per wave.
static int64_t decLinearShare(int64_t K) {
    const int64_t kblocks = K / 128, waves = kblocks < 8 ? 8 : (kblocks > 16 ? 16 : kblocks);
    return waves * ((kblocks + waves - 1) / waves) * (2048 + 128);
}

bool Emitter::decodeCandidate(size_t at, DecCandidate *out) {
    if (at >= prog_.ops.size() || prog_.ops[at].kind != kHlMatmul || consumed_[at]) return false;
    const thip_hl_matmul_t &c = prog_.ops[at].u.mm;
    const size_t n = prog_.values.size();
    if (c.input1 < 0 || (size_t)c.input1 >= n || c.input2 < 0 || (size_t)c.input2 >= n || c.init < 0 || (size_t)c.init >= n || c.scale_bias < 0 || (size_t)c.scale_bias >= n) return false;
    const auto folded = foldedExpand_.find(c.input2);
    if (folded == foldedExpand_.end() || c.shift != 0 || c.output_zp != 0) return false;
    const Value &a = prog_.values[(size_t)c.input1], &init = prog_.values[(size_t)c.init], &bv = prog_.values[(size_t)c.scale_bias];
    if (a.dtype != THIP_DTYPE_BF16 || init.dtype != THIP_DTYPE_BF16 || a.rank != 2 || state_[c.input1].nhwcOfNchw) return false;
    if (bv.kind != kValueConstant || bv.dtype != THIP_DTYPE_F32 || bv.numel() < 1) return false;
    const thip_hl_expand_weights_t &ew = *folded->second;
    if (ew.input < 0 || (size_t)ew.input >= n || ew.scale < 0 || (size_t)ew.scale >= n || ew.scale_bias < 0 || (size_t)ew.scale_bias >= n) return false;
    const Value &w = prog_.values[(size_t)ew.input], &sc = prog_.values[(size_t)ew.scale], &qb = prog_.values[(size_t)ew.scale_bias];
    if (w.dtype != THIP_DTYPE_I8 || w.rank != 2 || sc.dtype != THIP_DTYPE_BF16 || qb.dtype != THIP_DTYPE_F32) return false;
    const int64_t M = a.shape[0], K = a.shape[1], N = w.shape[1], block = ew.block_size;
    if (w.shape[0] != K || M > kDecMaxRows || K % 128 != 0 || N % 16 != 0 || N / 16 > 1024 || block <= 0 || block % 128 != 0 || K % block != 0) return false;
    const int64_t G = K / block;
    if (sc.numel() != G * N || qb.numel() % G != 0 || qb.numel() / G < N || init.numel() != M * N) return false;
    if (decLinearShare(K) > 152 * 1024) return false;  // a workgroup's share of the weights (16 columns of the whole K) must fit a CU's LDS
    out->mm = &c;
    out->ew = &ew;
    out->M = M; out->K = K; out->N = N; out->block = block;
    memcpy(&out->bias, bv.data.data(), 4);
    return true;
}

thip_status_t Emitter::tryEmitDecodeLinear(size_t at, bool *handled) {
    *handled = false;
    if (getenv("THIP_NO_DECODE_FUSION")) return THIP_OK;
    DecCandidate c0;
    if (!decodeCandidate(at, &c0)) return THIP_OK;
    const size_t end = prog_.ops.size();
    const size_t j1 = nextLiveOp(at), j2 = j1 < end ? nextLiveOp(j1) : end;
    auto sameGroup = [&](const DecCandidate &a, const DecCandidate &b) {
        return a.mm->input1 == b.mm->input1 && a.K == b.K && a.M == b.M && a.block == b.block && a.mm->output_min == b.mm->output_min &&
               a.mm->output_max == b.mm->output_max && a.ew->output_min == b.ew->output_min && a.ew->output_max == b.ew->output_max &&
               a.mm->init != b.mm->init;
    };
    auto bf16Add = [&](size_t i, const thip_hl_add_t **out) {
        if (i >= end || prog_.ops[i].kind != kHlAdd) return false;
        const thip_hl_add_t &ad = prog_.ops[i].u.add;
        const size_t n = prog_.values.size();
        if (ad.input1 < 0 || (size_t)ad.input1 >= n || ad.input2 < 0 || (size_t)ad.input2 >= n || ad.init < 0 || (size_t)ad.init >= n ||
            ad.weights < 0 || (size_t)ad.weights >= n || ad.scale_bias < 0 || (size_t)ad.scale_bias >= n) return false;
        const Value &x = prog_.values[(size_t)ad.input1], &y = prog_.values[(size_t)ad.input2], &z = prog_.values[(size_t)ad.init];
        const Value &w = prog_.values[(size_t)ad.weights], &sb = prog_.values[(size_t)ad.scale_bias];
        if (x.dtype != THIP_DTYPE_BF16 || y.dtype != THIP_DTYPE_BF16 || z.dtype != THIP_DTYPE_BF16 || ad.segment_output || ad.rhs_is_scalar) return false;
        if (ad.shift_factor != 0 || ad.input_zp != 0 || ad.output_zp != 0) return false;
        if (w.kind != kValueConstant || w.dtype != THIP_DTYPE_BF16 || w.numel() < 2 || sb.kind != kValueConstant || sb.dtype != THIP_DTYPE_F32 || sb.numel() < 1) return false;
        if (x.numel() != y.numel() || x.numel() != z.numel()) return false;
        *out = &ad;
        return true;
    };
    // the matrices of the record, and the add folded into it
    std::vector<DecCandidate> mats{c0};
    std::vector<size_t> members{at};
    const thip_hl_add_t *add = nullptr;
    int flags = 0;
    DecCandidate c1, c2;
    const thip_hl_add_t *ad = nullptr;
    const bool pairFits = 2 * decLinearShare(c0.K) <= 152 * 1024;  // twice the share of one matrix
    if (pairFits && j1 < end && decodeCandidate(j1, &c1) && sameGroup(c0, c1) && c0.N == c1.N && bf16Add(j2, &ad) &&
        ((ad->input1 == c0.mm->init && ad->input2 == c1.mm->init) || (ad->input1 == c1.mm->init && ad->input2 == c0.mm->init)) &&
        ad->init != c0.mm->init && ad->init != c1.mm->init) {
        // gate and up: matrix 0 is the producer of the add's input1
        if (ad->input1 == c0.mm->init) mats = {c0, c1};
        else mats = {c1, c0};
        members = {at, j1, j2};
        add = ad;
        flags = kDecPair | kDecAddPair;
    } else if (j1 < end && decodeCandidate(j1, &c1) && sameGroup(c0, c1)) {
        mats.push_back(c1);
        members.push_back(j1);
        if (j2 < end && decodeCandidate(j2, &c2) && sameGroup(c0, c2) && c1.mm->init != c2.mm->init) {
            mats.push_back(c2);
            members.push_back(j2);
        }
    } else if (bf16Add(j1, &ad) && ((ad->input1 == c0.mm->init) != (ad->input2 == c0.mm->init)) && ad->init != c0.mm->init) {
        const thip_value_t other = ad->input1 == c0.mm->init ? ad->input2 : ad->input1;
        // the other operand must exist already: a binding, or an intermediate some earlier record wrote
        const Value &ov = prog_.values[(size_t)other];
        const bool ready = ov.kind == kValueBinding || (ov.kind == kValueView ? (prog_.values[(size_t)ov.base].kind == kValueBinding || state_[ov.base].defined) : state_[other].defined);
        if (ready && !state_[other].nhwcOfNchw && ov.numel() == c0.M * c0.N) {
            members = {at, j1};
            add = ad;
            flags = kDecAddResidual | (ad->input1 == c0.mm->init ? 0 : kDecResFirst);
        }
    }
    const char *what = "torq_hl.matmul (bf16, grouped)";
    DescOp op;
    memset(&op, 0, sizeof(op));
    op.kind = kKindDecLinear;
    op.out_dtype = THIP_DTYPE_BF16;
    op.output_min = c0.mm->output_min;
    op.output_max = c0.mm->output_max;
    op.bias0 = c0.ew->output_min;
    op.scale0 = c0.ew->output_max;
    op.M = (int32_t)c0.M; op.K = (int32_t)c0.K; op.Kp = (int32_t)c0.K;
    op.gran = (uint32_t)c0.block;
    op.w0 = (int32_t)mats.size();
    op.w1 = flags;
    if (thip_status_t s = literalInput(c0.mm->input1, "torq_hl.matmul input1", &op.in0)) return s;
    if (op.in0.offset & 15) return THIP_OK;  // a view at an odd offset: the ungrouped path takes it
    DecLinearExt x;
    memset(&x, 0, sizeof(x));
    const int kblocks = (int)(c0.K / 128);
    // block biases: stored only if any of them is non-zero in any matrix of the record
    bool anyBias = false;
    for (const DecCandidate &m : mats) {
        const Value &qb = prog_.values[(size_t)m.ew->scale_bias];
        const float *bd = (const float *)qb.data.data();
        const int64_t cols = qb.numel() / (m.K / m.block);
        for (int64_t g = 0; g < m.K / m.block && !anyBias; g++) {
            for (int64_t n = 0; n < m.N && !anyBias; n++) anyBias = bd[g * cols + n] != 0.0f;
        }
    }
    x.has_qbias = anyBias ? 1 : 0;
    for (size_t mi = 0; mi < mats.size(); mi++) {
        const DecCandidate &m = mats[mi];
        const Value &w = prog_.values[(size_t)m.ew->input], &sc = prog_.values[(size_t)m.ew->scale], &qb = prog_.values[(size_t)m.ew->scale_bias];
        const int8_t *wd = (const int8_t *)w.data.data();
        std::vector<int8_t> packed(decWeightBytes((int)m.N, (int)m.K, anyBias), 0);
        const int slot = decSlotBytes(anyBias);
        for (int64_t k = 0; k < m.K; k++) {
            const int8_t *row = wd + k * m.N;
            // decWeightOffset(n, k) with the parts that depend on k only taken out of the inner loop
            const int b = (int)(k >> 7), kk = (int)(k & 127), j = kk >> 5, g = (kk & 31) >> 3, e = kk & 7;
            const size_t inSlot = ((size_t)(j >> 1) * 64 + (size_t)g * 16) * 16 + (size_t)((j & 1) * 8 + e);
            for (int64_t n = 0; n < m.N; n++) packed[((size_t)(n >> 4) * kblocks + b) * slot + inSlot + (size_t)(n & 15) * 16] = row[n];
        }
        const int64_t G = m.K / m.block, cols = qb.numel() / G;
        const uint16_t *sd = (const uint16_t *)sc.data.data();
        const float *bd = (const float *)qb.data.data();
        for (int b = 0; b < kblocks; b++) {
            const int64_t g = (int64_t)b * 128 / m.block;
            for (int64_t n = 0; n < m.N; n++) {
                const float sv = floatFromBf16(sd[g * m.N + n]);
                memcpy(&packed[decScaleOffset((int)n, b, kblocks, anyBias, 0)], &sv, 4);
                if (anyBias) memcpy(&packed[decScaleOffset((int)n, b, kblocks, anyBias, 1)], &bd[g * cols + n], 4);
            }
        }
        x.weights[mi] = newConst(packed);
        x.bias[mi] = newConst(std::vector<float>((size_t)m.N, m.bias));
        x.N[mi] = (int32_t)m.N;
        // the result is stored unless its only reader is the add folded into this record
        const Value &iv = prog_.values[(size_t)m.mm->init];
        const bool onlyTheAdd = add && iv.kind == kValueTensor && valueReads_[(size_t)m.mm->init] == 1;
        if (!onlyTheAdd) {
            if (thip_status_t s = literalOutput(m.mm->init, "torq_hl.matmul init", THIP_DTYPE_BF16, m.M * m.N, &x.out[mi])) return s;
            if (x.out[mi].offset & 7) return fail(THIP_UNIMPLEMENTED, "%s: init is a view at an offset that is no multiple of 8 bytes", what);
        }
    }
    if (add) {
        const Value &w = prog_.values[(size_t)add->weights], &sb = prog_.values[(size_t)add->scale_bias];
        x.aw0 = ((const uint16_t *)w.data.data())[0];
        x.aw1 = ((const uint16_t *)w.data.data())[1];
        memcpy(&x.abias, sb.data.data(), 4);
        x.alo = add->output_min;
        x.ahi = add->output_max;
        if (flags & kDecAddResidual) {
            const thip_value_t other = add->input1 == c0.mm->init ? add->input2 : add->input1;
            if (thip_status_t s = literalInput(other, "torq_hl.add operand", &x.res)) return s;
        }
        if (thip_status_t s = literalOutput(add->init, "torq_hl.add init", THIP_DTYPE_BF16, c0.M * c0.N, &x.add_out)) return s;
        if ((x.res.offset & 7) || (x.add_out.offset & 7)) return fail(THIP_UNIMPLEMENTED, "%s: the add behind it works on a view at an offset that is no multiple of 8 bytes", what);
    }
    std::vector<uint8_t> blob(sizeof(x));
    memcpy(blob.data(), &x, sizeof(x));
    op.table = newConst(blob);
    op.out = add ? x.add_out : x.out[0];
    op.Nn = (int32_t)mats[0].N; op.Np = (int32_t)mats[0].N;
    ops_.push_back(op);
    for (size_t mbr : members) consumed_[mbr] = 1;
    *handled = true;
    return THIP_OK;
}

// Decides which intermediates are stored with their channel axis padded to a multiple of 16.
// A pointwise convolution over such a tensor streams it with 16-byte loads (the dense loader)
// instead of gathering 8-byte pieces, which is what the 24-channel bottlenecks of mobile
// networks otherwise cost.  Padded channels are produced with zero weights, bias and scale and
// met with zero weights by every consumer, so their values never reach a result.  Ops that do
// not look at single channels (depthwise, max pool, add) tie their operands together: all of
// them are padded or none.  Anything that reads a tensor in its declared order (bindings,
// fully_connected, matmul, avg_pool2d, transpose) keeps the whole group unpadded.
// THIP_NO_CHANNEL_PAD switches the pass off.
void Emitter::planChannelPadding() {
    const size_t n = prog_.values.size();
    cpad_.assign(n, 0);
    cdeclared_.assign(n, 0);
    if (getenv("THIP_NO_CHANNEL_PAD")) return;
    std::vector<size_t> parent(n);
    for (size_t i = 0; i < n; i++) parent[i] = i;
    std::vector<int64_t> chan(n, 0);  // channel count seen at the uses; -1 = must stay as declared
    std::vector<char> touched(n, 0);
    auto valid = [&](thip_value_t v) { return v >= 0 && (size_t)v < n; };
    auto find = [&](size_t v) {
        while (parent[v] != v) v = parent[v] = parent[parent[v]];
        return v;
    };
    auto tie = [&](thip_value_t a, thip_value_t b) {
        if (!valid(a) || !valid(b)) return;
        parent[find((size_t)a)] = find((size_t)b);
        touched[a] = touched[b] = 1;
    };
    auto bar = [&](thip_value_t v) {
        if (!valid(v)) return;
        chan[v] = -1;
        touched[v] = 1;
    };
    auto use = [&](thip_value_t v, bool nhwc) {
        if (!valid(v)) return;
        const Value &val = prog_.values[v];
        touched[v] = 1;
        const int64_t C = val.rank == 4 ? val.shape[nhwc ? 3 : 1] : -1;
        if (chan[v] == 0) chan[v] = C;
        else if (chan[v] != C) chan[v] = -1;
    };
    for (size_t v = 0; v < n; v++) {
        if (prog_.values[v].kind == kValueView) {
            bar((thip_value_t)v);
            bar(prog_.values[v].base);
        }
    }
    for (const HlOp &op : prog_.ops) {
        switch (op.kind) {
        case kHlConv2d:
            use(op.u.conv.input, op.u.conv.nhwc_input != 0);
            use(op.u.conv.init, op.u.conv.nhwc_input != 0);
            break;
        case kHlDepthwise:
            use(op.u.dw.input, op.u.dw.nhwc_input != 0);
            use(op.u.dw.init, op.u.dw.nhwc_input != 0);
            tie(op.u.dw.input, op.u.dw.init);
            break;
        case kHlMaxPool:
            use(op.u.mp.input, op.u.mp.nhwc_input != 0);
            use(op.u.mp.init, op.u.mp.nhwc_input != 0);
            tie(op.u.mp.input, op.u.mp.init);
            break;
        case kHlAdd:
            tie(op.u.add.input1, op.u.add.input2);
            tie(op.u.add.input1, op.u.add.init);
            break;
        case kHlFullyConnected: bar(op.u.fc.input); bar(op.u.fc.init); break;
        case kHlMatmul: bar(op.u.mm.input1); bar(op.u.mm.input2); bar(op.u.mm.init); break;
        case kHlAvgPool: bar(op.u.ap.input); bar(op.u.ap.init); break;
        case kHlTranspose: bar(op.u.tr.input); bar(op.u.tr.init); break;
        case kHlExpandWeights: bar(op.u.ew.input); bar(op.u.ew.init); break;
        case kHlFma: bar(op.u.fma.input); bar(op.u.fma.init); break;
        case kHlMul: bar(op.u.mul.input1); bar(op.u.mul.input2); bar(op.u.mul.init); break;
        case kHlAct: bar(op.u.act.input); bar(op.u.act.init); break;
        case kHlBinary: bar(op.u.bin.input1); bar(op.u.bin.input2); bar(op.u.bin.init); break;
        case kHlUnary: bar(op.u.un.input); bar(op.u.un.init); break;
        case kHlShift: bar(op.u.sh.input1); bar(op.u.sh.input2); bar(op.u.sh.init); break;
        case kHlTable: bar(op.u.tab.input); bar(op.u.tab.init); break;
        }
    }
    // one verdict per group: every member an int8 rank-4 intermediate, all uses agreeing on C
    std::vector<int64_t> groupC(n, 0);
    for (size_t v = 0; v < n; v++) {
        const size_t g = find(v);
        const Value &val = prog_.values[v];
        if (!touched[v]) continue;  // weights and other values no activation op touches
        const bool plain = val.kind == kValueTensor && val.rank == 4 && val.dtype == THIP_DTYPE_I8;
        if (!plain || chan[v] < 0) groupC[g] = -1;
        else if (chan[v] > 0 && groupC[g] == 0) groupC[g] = chan[v];
        else if (chan[v] > 0 && groupC[g] != chan[v]) groupC[g] = -1;
    }
    for (size_t v = 0; v < n; v++) {
        const int64_t C = groupC[find(v)];
        if (C > 16 && C % 16 != 0 && prog_.values[v].kind == kValueTensor) {
            cpad_[v] = roundUp(C, 16);
            cdeclared_[v] = C;
        }
    }
}

void Emitter::planExpandFolding() {
    foldedExpand_.clear();
    const size_t n = prog_.values.size();
    std::vector<int> reads(n, 0), asMatmulRhs(n, 0);
    auto read = [&](thip_value_t v) {
        if (v < 0 || (size_t)v >= n) return;
        reads[(size_t)v]++;
        if (prog_.values[(size_t)v].kind == kValueView) reads[(size_t)prog_.values[(size_t)v].base]++;  // a read of a view reads its base
    };
    for (const HlOp &op : prog_.ops) {
        switch (op.kind) {
        case kHlConv2d: read(op.u.conv.input); break;
        case kHlDepthwise: read(op.u.dw.input); break;
        case kHlFullyConnected: read(op.u.fc.input); break;
        case kHlMatmul:
            read(op.u.mm.input1);
            read(op.u.mm.input2);
            if (op.u.mm.input2 >= 0 && (size_t)op.u.mm.input2 < n && op.u.mm.input1 >= 0 && (size_t)op.u.mm.input1 < n &&
                prog_.values[(size_t)op.u.mm.input1].dtype == THIP_DTYPE_BF16) {
                asMatmulRhs[(size_t)op.u.mm.input2]++;
            }
            break;
        case kHlMaxPool: read(op.u.mp.input); break;
        case kHlAvgPool: read(op.u.ap.input); break;
        case kHlAdd: read(op.u.add.input1); read(op.u.add.input2); break;
        case kHlTranspose: read(op.u.tr.input); break;
        case kHlExpandWeights: read(op.u.ew.input); read(op.u.ew.scale); read(op.u.ew.scale_bias); break;
        case kHlFma: read(op.u.fma.input); break;
        case kHlMul: read(op.u.mul.input1); read(op.u.mul.input2); break;
        case kHlAct: read(op.u.act.input); break;
        case kHlBinary: read(op.u.bin.input1); read(op.u.bin.input2); break;
        case kHlUnary: read(op.u.un.input); break;
        case kHlShift: read(op.u.sh.input1); read(op.u.sh.input2); break;
        case kHlTable: read(op.u.tab.input); break;
        }
    }
    valueReads_ = reads;
    if (getenv("THIP_NO_EXPAND_FOLD")) return;
    auto constant = [&](thip_value_t v) { return v >= 0 && (size_t)v < n && prog_.values[(size_t)v].kind == kValueConstant; };
    for (const HlOp &op : prog_.ops) {
        if (op.kind != kHlExpandWeights) continue;
        const thip_hl_expand_weights_t &c = op.u.ew;
        if (c.init < 0 || (size_t)c.init >= n || prog_.values[(size_t)c.init].kind != kValueTensor) continue;
        if (!constant(c.input) || !constant(c.scale) || !constant(c.scale_bias)) continue;
        if (reads[(size_t)c.init] == 1 && asMatmulRhs[(size_t)c.init] == 1) foldedExpand_[c.init] = &c;
    }
}

void Emitter::fuseResidualAdd() {
    if (getenv("THIP_NO_ADD_FUSION")) return;
    auto same = [](const DescRef &a, const DescRef &b) { return a.space == b.space && a.index == b.index && a.offset == b.offset; };
    for (size_t i = 0; i + 1 < ops_.size(); i++) {
        const DescOp conv = ops_[i], add = ops_[i + 1];
        if (conv.kind != kKindIgemm || conv.loader != kLoaderDense || conv.out_dtype != THIP_DTYPE_I8) continue;
        // the pixel-streaming kernel, or the small dense tile when it will run its in-register epilogue
        const bool inRegister = conv.variant == kIgemmDense64x64 && conv.Nn % 16 == 0 && conv.shift >= 33 && conv.shift <= 45 &&
                                conv.pre_shift == 0 && conv.t0_clamp == 0 && conv.output_min <= conv.output_max && !getenv("THIP_NO_DIRECT_EPILOGUE");
        if (conv.variant != kIgemmStream && !inRegister) continue;
        if (conv.in1.space != kSpaceNone || conv.out.space != kSpaceTemp || conv.out.offset != 0 || add.kind != kKindAdd) continue;
        const bool first = same(add.in0, conv.out), second = same(add.in1, conv.out);
        if (first == second || add.C != (int64_t)conv.M * conv.Nn) continue;
        // nobody else may touch the convolution's result
        bool shared = false;
        for (size_t k = 0; k < ops_.size() && !shared; k++) {
            if (k == i || k == i + 1) continue;
            const DescRef *refs[] = {&ops_[k].in0, &ops_[k].in1, &ops_[k].weights, &ops_[k].bias, &ops_[k].scale, &ops_[k].table, &ops_[k].out};
            for (const DescRef *r : refs) shared = shared || (r->space == kSpaceTemp && r->index == conv.out.index);
        }
        if (shared) continue;
        ResidualAddParams ap;
        memset(&ap, 0, sizeof(ap));
        ap.w0 = add.w0; ap.w1 = add.w1; ap.bias = add.bias0; ap.scale = add.scale0;
        ap.shift = add.shift; ap.output_zp = add.output_zp; ap.output_min = add.output_min; ap.output_max = add.output_max;
        ap.other_first = second;  // the convolution's result is input2: the operand read from memory is input1
        std::vector<uint8_t> blob(sizeof(ap));
        memcpy(blob.data(), &ap, sizeof(ap));
        DescOp f = conv;
        f.in1 = second ? add.in0 : add.in1;
        f.table = newConst(blob);
        f.out = add.out;
        temps_[conv.out.index] = 0;  // never materialised
        ops_[i] = f;
        ops_.erase(ops_.begin() + (long)i + 1);
    }
}

thip_status_t Emitter::run(void **outBlob, size_t *outSize) {
    planChannelPadding();
    planExpandFolding();
    planDecodeFolding();
    for (size_t at = 0; at < prog_.ops.size(); at++) {
        const HlOp &op = prog_.ops[at];
        thip_status_t s = THIP_OK;
        addFollows_ = false;
        if (consumed_[at]) continue;
        if (op.kind == kHlTranspose && foldedTranspose_.count(op.u.tr.init)) continue;  // read in place by its matmul
        if (op.kind == kHlMatmul) {
            bool handled = false;
            if ((s = tryEmitDecodeLinear(at, &handled))) return s;
            if (handled) continue;
        }
        if (op.kind == kHlConv2d && at + 1 < prog_.ops.size() && prog_.ops[at + 1].kind == kHlAdd && !getenv("THIP_NO_ADD_FUSION")) {
            const thip_value_t y = op.u.conv.init;
            const thip_hl_add_t &next = prog_.ops[at + 1].u.add;
            addFollows_ = y >= 0 && (size_t)y < valueReads_.size() && valueReads_[(size_t)y] == 1 && ((next.input1 == y) != (next.input2 == y));
        }
        switch (op.kind) {
        case kHlConv2d: s = emitConv2d(op.u.conv); break;
        case kHlDepthwise: s = emitDepthwise(op.u.dw); break;
        case kHlFullyConnected: s = emitFullyConnected(op.u.fc); break;
        case kHlMatmul: s = emitMatmul(op.u.mm); break;
        case kHlMaxPool: s = emitMaxPool(op.u.mp); break;
        case kHlAvgPool: s = emitAvgPool(op.u.ap); break;
        case kHlAdd: s = emitAdd(op.u.add); break;
        case kHlTranspose: s = emitTransposeOp(op.u.tr); break;
        case kHlExpandWeights: s = emitExpandWeights(op.u.ew); break;
        case kHlFma: s = emitFma(op.u.fma); break;
        case kHlMul: s = emitMul(op.u.mul); break;
        case kHlAct: s = emitAct(op.u.act, op.name); break;
        case kHlBinary: s = emitBinary(op.u.bin); break;
        case kHlUnary: s = emitUnary(op.u.un); break;
        case kHlShift: s = emitShift(op.u.sh); break;
        case kHlTable: s = emitTable(op.u.tab, op.staticTable); break;
        }
        if (s != THIP_OK) return s;
    }
    if (ops_.empty()) return fail(THIP_INVALID_ARGUMENT, "program has no ops");
    fuseResidualAdd();

    // Binding ids must be dense 0..n-1 so the dispatch's binding table indexes directly.
    uint32_t bindingCount = 0;
    for (auto &kv : bindings_) bindingCount = std::max(bindingCount, kv.first + 1);
    std::vector<DescBinding> btable(bindingCount);
    for (uint32_t i = 0; i < bindingCount; i++) btable[i] = DescBinding{i, 0, 0};
    for (auto &kv : bindings_) btable[kv.first] = kv.second;

    DescHeader h;
    memset(&h, 0, sizeof(h));
    h.magic = kMagic;
    h.version = kDescriptorVersion;
    h.arch = kArchGfx950;
    h.op_count = (uint32_t)ops_.size();
    h.binding_count = bindingCount;
    h.temp_count = (uint32_t)temps_.size();
    h.const_count = (uint32_t)consts_.size();
    snprintf(h.name, sizeof(h.name), "%s", prog_.name.c_str());
    uint64_t off = sizeof(DescHeader);
    h.ops_offset = off;
    off += sizeof(DescOp) * ops_.size();
    h.bindings_offset = off;
    off += sizeof(DescBinding) * btable.size();
    h.temps_offset = off;
    off += sizeof(DescTemp) * temps_.size();
    h.consts_offset = off;
    off += sizeof(DescConst) * consts_.size();
    off = (uint64_t)roundUp((int64_t)off, (int64_t)kDataAlign);
    h.data_offset = off;
    std::vector<DescConst> ctable(consts_.size());
    uint64_t dataOff = 0;
    for (size_t i = 0; i < consts_.size(); i++) {
        ctable[i].offset = dataOff;
        ctable[i].size = consts_[i].size();
        dataOff = (uint64_t)roundUp((int64_t)(dataOff + consts_[i].size()), (int64_t)kDataAlign);
    }
    h.total_size = h.data_offset + dataOff;

    uint8_t *blob = (uint8_t *)calloc(1, (size_t)h.total_size);
    if (!blob) return fail(THIP_RESOURCE_EXHAUSTED, "out of memory serialising %llu bytes", (unsigned long long)h.total_size);
    memcpy(blob, &h, sizeof(h));
    memcpy(blob + h.ops_offset, ops_.data(), sizeof(DescOp) * ops_.size());
    if (!btable.empty()) memcpy(blob + h.bindings_offset, btable.data(), sizeof(DescBinding) * btable.size());
    for (size_t i = 0; i < temps_.size(); i++) {
        DescTemp t{temps_[i]};
        memcpy(blob + h.temps_offset + i * sizeof(DescTemp), &t, sizeof(t));
    }
    if (!ctable.empty()) memcpy(blob + h.consts_offset, ctable.data(), sizeof(DescConst) * ctable.size());
    for (size_t i = 0; i < consts_.size(); i++) {
        if (!consts_[i].empty()) memcpy(blob + h.data_offset + ctable[i].offset, consts_[i].data(), consts_[i].size());
    }
    *outBlob = blob;
    *outSize = (size_t)h.total_size;
    return THIP_OK;
}

static thip_status_t addValue(thip_program_t *p, ValueKind kind, uint32_t binding, int32_t dtype, int32_t rank,
                              const int64_t *shape, const void *data, size_t dataSize, thip_value_t *out) {
    if (!p || !out) return fail(THIP_INVALID_ARGUMENT, "null program or result pointer");
    if (elemSize(dtype) == 0) return fail(THIP_INVALID_ARGUMENT, "unknown element type %d", dtype);
    if (rank < 1 || rank > THIP_MAX_RANK || !shape) return fail(THIP_INVALID_ARGUMENT, "rank %d is outside 1..%d", rank, THIP_MAX_RANK);
    Value v;
    v.kind = kind;
    v.dtype = dtype;
    v.rank = rank;
    v.binding = binding;
    for (int i = 0; i < THIP_MAX_RANK; i++) v.shape[i] = i < rank ? shape[i] : 1;
    for (int i = 0; i < rank; i++) {
        if (shape[i] <= 0) return fail(THIP_INVALID_ARGUMENT, "dimension %d is %lld", i, (long long)shape[i]);
    }
    if (kind == kValueConstant) {
        const size_t need = (size_t)v.numel() * elemSize(dtype);
        if (!data || dataSize != need) return fail(THIP_INVALID_ARGUMENT, "constant carries %zu bytes, its shape needs %zu", dataSize, need);
        v.data.assign((const uint8_t *)data, (const uint8_t *)data + need);
    }
    p->values.push_back(std::move(v));
    *out = (thip_value_t)(p->values.size() - 1);
    return THIP_OK;
}

}  // namespace thip

using namespace thip;

extern "C" {

thip_status_t thip_program_create(thip_program_t **out_program) {
    if (!out_program) return fail(THIP_INVALID_ARGUMENT, "null result pointer");
    *out_program = new (std::nothrow) thip_program_t();
    if (!*out_program) return fail(THIP_RESOURCE_EXHAUSTED, "out of memory");
    return THIP_OK;
}

void thip_program_destroy(thip_program_t *program) { delete program; }

thip_status_t thip_program_set_name(thip_program_t *program, const char *name) {
    if (!program || !name) return fail(THIP_INVALID_ARGUMENT, "null argument");
    const size_t n = strlen(name);
    if (n == 0 || n >= sizeof(DescHeader::name)) return fail(THIP_INVALID_ARGUMENT, "an executable name has 1..%zu characters", sizeof(DescHeader::name) - 1);
    for (size_t i = 0; i < n; i++) {
        const char c = name[i];
        // the name becomes a directory of the dumps and a CSV column: keep it to what is safe in both
        if (!((c >= 'a' && c <= 'z') || (c >= 'A' && c <= 'Z') || (c >= '0' && c <= '9') || c == '_' || c == '-' || c == '.' || c == '$') || (i == 0 && c == '.')) {
            return fail(THIP_INVALID_ARGUMENT, "executable name has a character outside [A-Za-z0-9_.$-]");
        }
    }
    program->name = name;
    return THIP_OK;
}

thip_status_t thip_program_binding(thip_program_t *program, uint32_t binding, int32_t dtype, int32_t rank,
                                   const int64_t *shape, thip_value_t *out_value) {
    if (binding >= 64) return fail(THIP_INVALID_ARGUMENT, "binding %u exceeds the maximum binding count", binding);
    return addValue(program, kValueBinding, binding, dtype, rank, shape, nullptr, 0, out_value);
}

thip_status_t thip_program_constant(thip_program_t *program, int32_t dtype, int32_t rank, const int64_t *shape,
                                    const void *data, size_t data_size, thip_value_t *out_value) {
    return addValue(program, kValueConstant, 0, dtype, rank, shape, data, data_size, out_value);
}

thip_status_t thip_program_tensor(thip_program_t *program, int32_t dtype, int32_t rank, const int64_t *shape,
                                  thip_value_t *out_value) {
    return addValue(program, kValueTensor, 0, dtype, rank, shape, nullptr, 0, out_value);
}

thip_status_t thip_program_view(thip_program_t *program, thip_value_t base, int64_t element_offset, int32_t rank,
                                const int64_t *shape, thip_value_t *out_value) {
    if (!program || !out_value) return fail(THIP_INVALID_ARGUMENT, "null program or result pointer");
    if (base < 0 || (size_t)base >= program->values.size()) return fail(THIP_INVALID_ARGUMENT, "thip_program_view: value %d does not exist", (int)base);
    // a view of a view names the underlying value directly
    const Value b = program->values[(size_t)base];
    const thip_value_t root = b.kind == kValueView ? b.base : base;
    const int64_t rootOffset = b.kind == kValueView ? b.viewOffset : 0;
    if (b.kind == kValueConstant) return fail(THIP_UNIMPLEMENTED, "thip_program_view: a view of a constant (declare the constant in the shape it is used in)");
    if (thip_status_t s = addValue(program, kValueView, 0, b.dtype, rank, shape, nullptr, 0, out_value)) return s;
    Value &v = program->values.back();
    if (element_offset < 0 || element_offset > b.numel() || v.numel() > b.numel() - element_offset) {
        program->values.pop_back();
        return fail(THIP_INVALID_ARGUMENT, "thip_program_view: elements %lld .. %lld lie outside the %lld of value %d", (long long)element_offset,
                    (long long)(element_offset + v.numel()), (long long)b.numel(), (int)base);
    }
    v.base = root;
    v.viewOffset = rootOffset + element_offset;
    v.binding = program->values[(size_t)root].binding;
    return THIP_OK;
}

thip_status_t thip_gemm_tile_choice(int32_t addressing, int64_t M, int64_t N, int64_t K, int64_t C, int32_t out_dtype, int32_t add_follows,
                                    uint32_t *out_variant, char *name, size_t capacity) {
    if (!out_variant) return fail(THIP_INVALID_ARGUMENT, "thip_gemm_tile_choice: null result pointer");
    if (addressing < (int32_t)kLoaderDense || addressing > (int32_t)kLoaderWindow) return fail(THIP_INVALID_ARGUMENT, "thip_gemm_tile_choice: addressing %d is none of 0 .. 3", (int)addressing);
    if (M < 1 || N < 1 || K < 1 || C < 1) return fail(THIP_INVALID_ARGUMENT, "thip_gemm_tile_choice: M, N, K and C must be positive");
    const uint32_t v = Emitter::tileChoice((uint32_t)addressing, M, N, K, C, (int32_t)out_dtype, add_follows != 0);
    *out_variant = v;
    if (name && capacity) snprintf(name, capacity, "%s", igemmTile(v).name);
    return THIP_OK;
}

#define THIP_DEFINE_HL(fn, type, kindEnum, member)                                        \
    thip_status_t fn(thip_program_t *program, const type *op) {                            \
        if (!program || !op) return fail(THIP_INVALID_ARGUMENT, #fn ": null argument");   \
        HlOp h;                                                                            \
        memset((void *)&h.u, 0, sizeof(h.u));                                              \
        h.kind = kindEnum;                                                                 \
        h.u.member = *op;                                                                  \
        program->ops.push_back(h);                                                         \
        return THIP_OK;                                                                    \
    }

THIP_DEFINE_HL(thip_hl_conv2d, thip_hl_conv2d_t, kHlConv2d, conv)
THIP_DEFINE_HL(thip_hl_depthwise_conv2d, thip_hl_depthwise_conv2d_t, kHlDepthwise, dw)
THIP_DEFINE_HL(thip_hl_fully_connected, thip_hl_fully_connected_t, kHlFullyConnected, fc)
THIP_DEFINE_HL(thip_hl_matmul, thip_hl_matmul_t, kHlMatmul, mm)
THIP_DEFINE_HL(thip_hl_maxpool2d, thip_hl_maxpool2d_t, kHlMaxPool, mp)
THIP_DEFINE_HL(thip_hl_avg_pool2d, thip_hl_avg_pool2d_t, kHlAvgPool, ap)
THIP_DEFINE_HL(thip_hl_transpose, thip_hl_transpose_t, kHlTranspose, tr)
THIP_DEFINE_HL(thip_hl_expand_weights, thip_hl_expand_weights_t, kHlExpandWeights, ew)
THIP_DEFINE_HL(thip_hl_fma, thip_hl_fma_t, kHlFma, fma)
THIP_DEFINE_HL(thip_hl_mul, thip_hl_mul_t, kHlMul, mul)
THIP_DEFINE_HL(thip_hl_elementwisebinary, thip_hl_elementwisebinary_t, kHlBinary, bin)
THIP_DEFINE_HL(thip_hl_elementwiseunary, thip_hl_elementwiseunary_t, kHlUnary, un)
THIP_DEFINE_HL(thip_hl_elementwiseshift, thip_hl_elementwiseshift_t, kHlShift, sh)

thip_status_t thip_hl_table(thip_program_t *program, const thip_hl_table_t *op) {
    if (!program || !op) return fail(THIP_INVALID_ARGUMENT, "thip_hl_table: null argument");
    if (op->static_table_count < 0 || (op->static_table_count > 0 && !op->static_table) || op->static_table_count > 65536) {
        return fail(THIP_INVALID_ARGUMENT, "thip_hl_table: bad static_table");
    }
    HlOp h;
    memset((void *)&h.u, 0, sizeof(h.u));
    h.kind = kHlTable;
    h.u.tab = *op;
    if (op->static_table_count > 0) h.staticTable.assign(op->static_table, op->static_table + op->static_table_count);
    h.u.tab.static_table = nullptr;  // the copy is what the serialiser reads
    program->ops.push_back(h);
    return THIP_OK;
}

thip_status_t thip_hl_act(thip_program_t *program, const thip_hl_act_t *op) {
    if (!program || !op || !op->name) return fail(THIP_INVALID_ARGUMENT, "thip_hl_act: null argument");
    HlOp h;
    memset((void *)&h.u, 0, sizeof(h.u));
    h.kind = kHlAct;
    h.u.act = *op;
    h.name = op->name;  // the caller's string need not outlive this call
    h.u.act.name = nullptr;
    program->ops.push_back(h);
    return THIP_OK;
}

thip_status_t thip_hl_add(thip_program_t *program, const thip_hl_add_t *op) {
    if (!program || !op) return fail(THIP_INVALID_ARGUMENT, "thip_hl_add: null argument");
    HlOp h;
    memset((void *)&h.u, 0, sizeof(h.u));
    h.kind = kHlAdd;
    h.u.add = *op;
    h.name = op->name ? op->name : "add";
    h.u.add.name = nullptr;  // the caller's string is not kept
    program->ops.push_back(h);
    return THIP_OK;
}

thip_status_t thip_program_serialize(thip_program_t *program, void **out_blob, size_t *out_size) {
    if (!program || !out_blob || !out_size) return fail(THIP_INVALID_ARGUMENT, "thip_program_serialize: null argument");
    *out_blob = nullptr;
    *out_size = 0;
    Emitter e(*program);
    return e.run(out_blob, out_size);
}

void thip_blob_free(void *blob) { free(blob); }

}  // extern "C"
