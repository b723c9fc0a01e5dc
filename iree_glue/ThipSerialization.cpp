// Compile side of the MI355X backend inside the torq compiler plugin: walks the TorqHL ops of one dispatch function
// exactly as they leave LinalgToTorqHL*Conversion (compiler/torq/Codegen/TORQLowerExecutableTargetPass.cpp:125,142)
// and hands each one to the emitter behind include/thip.h, field for field.  It takes the place that
// serializeTorqHW (compiler/torq/Serialization/Serialization.cpp:265-302) has for the NPU target: the NPU-only passes
// between the pattern set and serialisation (kernel selection, tensor encoding, slicing, address assignment) are not
// run for this target, the emitter does their job for the GPU.
//
// This file needs MLIR, IREE and the plugin's TorqHL dialect headers; none of them exists in the image this
// repository is built and tested in, so it is compiled only inside the reference's tree (see README.md here).
#include "ThipSerialization.h"

#include "thip.h"

#include "torq/Dialect/TorqHL/TorqHLOps.h"
#include "torq/Utils/ComputeConstants.h"

#include "iree/compiler/Dialect/HAL/IR/HALOps.h"
#include "mlir/Dialect/Arith/IR/Arith.h"
#include "mlir/Dialect/Func/IR/FuncOps.h"
#include "mlir/Dialect/Tensor/IR/Tensor.h"
#include "mlir/IR/BuiltinAttributes.h"
#include "mlir/IR/BuiltinTypes.h"
#include "llvm/ADT/DenseMap.h"
#include "llvm/ADT/TypeSwitch.h"

using namespace mlir;
using namespace mlir::iree_compiler;

namespace mlir::syna::thip {

namespace {

// Element type of a tensor / memref in the C-ABI's numbering; -1 when the path does not carry it.
int32_t dtypeOf(Type elementType) {
    if (elementType.isInteger(1)) return THIP_DTYPE_I1;  // stored as one byte of 0 / 1
    if (elementType.isInteger(8)) return THIP_DTYPE_I8;
    if (elementType.isInteger(16)) return THIP_DTYPE_I16;
    if (elementType.isInteger(32)) return THIP_DTYPE_I32;
    if (elementType.isBF16()) return THIP_DTYPE_BF16;
    if (elementType.isF32()) return THIP_DTYPE_F32;
    return -1;
}

class ProgramBuilder {
  public:
    explicit ProgramBuilder(func::FuncOp funcOp) : funcOp_(funcOp) {}
    ~ProgramBuilder() { thip_program_destroy(program_); }

    LogicalResult build(StringRef name, std::vector<uint8_t> &blob) {
        if (thip_program_create(&program_) != THIP_OK) return funcOp_.emitError() << thip_status_message();
        if (check(funcOp_, thip_program_set_name(program_, name.str().c_str())).failed()) return failure();
        WalkResult walked = funcOp_.walk([&](Operation *op) {
            if (!isa<torq_hl::TorqHLDialect>(op->getDialect())) return WalkResult::advance();
            return failed(emit(op)) ? WalkResult::interrupt() : WalkResult::advance();
        });
        if (walked.wasInterrupted()) return failure();
        void *data = nullptr;
        size_t size = 0;
        if (check(funcOp_, thip_program_serialize(program_, &data, &size)).failed()) return failure();
        blob.assign((const uint8_t *)data, (const uint8_t *)data + size);
        thip_blob_free(data);
        return success();
    }

  private:
    func::FuncOp funcOp_;
    thip_program_t *program_ = nullptr;
    llvm::DenseMap<Value, thip_value_t> values_;

    LogicalResult check(Operation *at, thip_status_t status) {
        if (status == THIP_OK) return success();
        return at->emitError() << "MI355X backend: " << thip_status_message();
    }

    // A value of the dispatch function as the emitter knows it: a binding (hal.interface.binding.subspan, through
    // any tensor-import / cast chain), a compile-time constant (anything ComputeConstants can fold: arith.constant,
    // torq_hl.const, constant linalg chains), or the intermediate a previous TorqHL op produced.
    FailureOr<thip_value_t> lookup(Operation *user, Value v) {
        if (auto it = values_.find(v); it != values_.end()) return it->second;
        auto shaped = dyn_cast<ShapedType>(v.getType());
        if (!shaped || !shaped.hasStaticShape() || shaped.getRank() < 1 || shaped.getRank() > THIP_MAX_RANK) {
            return user->emitError("MI355X backend: operands need a static shape of rank 1..4");
        }
        const int32_t dtype = dtypeOf(shaped.getElementType());
        if (dtype < 0) return user->emitError("MI355X backend: element type not carried by this path");
        SmallVector<int64_t> shape(shaped.getShape());
        thip_value_t id = THIP_NO_VALUE;

        Value root = v;
        while (Operation *def = root.getDefiningOp()) {
            if (isa<IREE::HAL::InterfaceBindingSubspanOp>(def)) break;
            if (isa<tensor::CastOp, IREE::TensorExt::DispatchTensorLoadOp>(def) && def->getNumOperands() >= 1) {
                root = def->getOperand(0);
                continue;
            }
            break;
        }
        if (auto subspan = root.getDefiningOp<IREE::HAL::InterfaceBindingSubspanOp>()) {
            const uint32_t binding = (uint32_t)subspan.getBinding().getZExtValue();
            if (failed(check(user, thip_program_binding(program_, binding, dtype, (int32_t)shape.size(), shape.data(), &id)))) return failure();
        } else if (auto folded = torq::computeConstant(v)) {
            // dense bytes in row-major order, element type as declared
            ArrayRef<char> raw = cast<DenseElementsAttr>(*folded).getRawData();
            std::vector<char> bytes(raw.begin(), raw.end());
            if (cast<DenseElementsAttr>(*folded).isSplat()) {
                // a splat stores one element: expand it
                const size_t elem = raw.size();
                bytes.resize(elem * (size_t)shaped.getNumElements());
                for (size_t i = elem; i < bytes.size(); i++) bytes[i] = raw[i % elem];
            }
            if (failed(check(user, thip_program_constant(program_, dtype, (int32_t)shape.size(), shape.data(), bytes.data(), bytes.size(), &id)))) return failure();
        } else if (v.getDefiningOp<tensor::EmptyOp>() || isa<BlockArgument>(v)) {
            // the init of an op whose result stays inside the dispatch
            if (failed(check(user, thip_program_tensor(program_, dtype, (int32_t)shape.size(), shape.data(), &id)))) return failure();
        } else {
            return user->emitError("MI355X backend: operand is neither a binding, a constant nor the result of a TorqHL op");
        }
        values_[v] = id;
        return id;
    }

    // The result of a DPS op is its init under another SSA name.
    void aliasResult(Operation *op, thip_value_t init) {
        if (op->getNumResults() == 1) values_[op->getResult(0)] = init;
    }

    template <typename Fill>
    LogicalResult withOperands(Operation *op, ArrayRef<std::pair<Value, thip_value_t *>> operands, Fill &&call) {
        for (auto &[value, slot] : operands) {
            if (!value) {
                *slot = THIP_NO_VALUE;
                continue;
            }
            auto id = lookup(op, value);
            if (failed(id)) return failure();
            *slot = *id;
        }
        return check(op, call());
    }

    static void copy4(int64_t (&dst)[4], ArrayRef<int64_t> src) {
        for (int i = 0; i < 4; i++) dst[i] = i < (int)src.size() ? src[i] : 0;
    }
    static void copy2(int64_t (&dst)[2], ArrayRef<int64_t> src) {
        for (int i = 0; i < 2; i++) dst[i] = i < (int)src.size() ? src[i] : 1;
    }

    LogicalResult emit(Operation *op) {
        return llvm::TypeSwitch<Operation *, LogicalResult>(op)
            .Case<torq_hl::Conv2DOp>([&](torq_hl::Conv2DOp c) {
                thip_hl_conv2d_t s = {};
                s.input_zp = c.getInputZp(); s.weight_zp = c.getWeightZp(); s.output_zp = c.getOutputZp();
                s.output_min = c.getOutputMin(); s.output_max = c.getOutputMax(); s.shift_factor = c.getShiftFactor();
                s.groups = c.getGroups();
                copy4(s.pad, c.getPad()); copy2(s.stride, c.getStride()); copy2(s.dilation, c.getDilation());
                s.vectorization_mode = (int32_t)c.getVectorizationMode();
                s.nhwc_input = c.getNhwcInput(); s.segment_output = c.getSegmentOutput();
                LogicalResult r = withOperands(op, {{c.getInit(), &s.init}, {c.getWeights(), &s.weights}, {c.getScaleBias(), &s.scale_bias}, {c.getInput(), &s.input}},
                                               [&] { return thip_hl_conv2d(program_, &s); });
                aliasResult(op, s.init);
                return r;
            })
            .Case<torq_hl::DepthwiseConv2DOp>([&](torq_hl::DepthwiseConv2DOp c) {
                thip_hl_depthwise_conv2d_t s = {};
                s.input_zp = c.getInputZp(); s.weight_zp = c.getWeightZp(); s.output_zp = c.getOutputZp();
                s.output_min = c.getOutputMin(); s.output_max = c.getOutputMax(); s.shift_factor = c.getShiftFactor();
                s.groups = c.getGroups();
                copy4(s.pad, c.getPad()); copy2(s.stride, c.getStride()); copy2(s.dilation, c.getDilation());
                s.vectorization_mode = (int32_t)c.getVectorizationMode();
                s.nhwc_input = c.getNhwcInput(); s.segment_output = c.getSegmentOutput(); s.is_dw1d_stride1 = c.getIsDw1dStride1();
                LogicalResult r = withOperands(op, {{c.getInit(), &s.init}, {c.getWeights(), &s.weights}, {c.getScaleBias(), &s.scale_bias}, {c.getInput(), &s.input}},
                                               [&] { return thip_hl_depthwise_conv2d(program_, &s); });
                aliasResult(op, s.init);
                return r;
            })
            .Case<torq_hl::FullyConnectedOp>([&](torq_hl::FullyConnectedOp c) {
                thip_hl_fully_connected_t s = {};
                s.input_zp = c.getInputZp(); s.weight_zp = c.getWeightZp(); s.output_zp = c.getOutputZp();
                s.output_min = c.getOutputMin(); s.output_max = c.getOutputMax(); s.shift_factor = c.getShiftFactor();
                s.vectorization_mode = (int32_t)c.getVectorizationMode();
                LogicalResult r = withOperands(op, {{c.getInit(), &s.init}, {c.getWeights(), &s.weights}, {c.getScaleBias(), &s.scale_bias}, {c.getInput(), &s.input}},
                                               [&] { return thip_hl_fully_connected(program_, &s); });
                aliasResult(op, s.init);
                return r;
            })
            .Case<torq_hl::MatMulOp>([&](torq_hl::MatMulOp c) {
                thip_hl_matmul_t s = {};
                s.output_zp = c.getOutputZp(); s.output_min = c.getOutputMin(); s.output_max = c.getOutputMax(); s.shift = c.getShift();
                LogicalResult r = withOperands(op, {{c.getInit(), &s.init}, {c.getScaleBias(), &s.scale_bias}, {c.getInput1(), &s.input1}, {c.getInput2(), &s.input2}},
                                               [&] { return thip_hl_matmul(program_, &s); });
                aliasResult(op, s.init);
                return r;
            })
            .Case<torq_hl::MaxPool2dOp>([&](torq_hl::MaxPool2dOp c) {
                thip_hl_maxpool2d_t s = {};
                s.input_zp = c.getInputZp(); s.output_min = c.getOutputMin(); s.output_max = c.getOutputMax();
                copy2(s.stride, c.getStride()); copy4(s.pad, c.getPad()); copy2(s.kernel, c.getKernel());
                s.segment_output = c.getSegmentOutput(); s.nhwc_input = c.getNhwcInput();
                LogicalResult r = withOperands(op, {{c.getInit(), &s.init}, {c.getWeights(), &s.weights}, {c.getScaleBias(), &s.scale_bias}, {c.getInput(), &s.input}},
                                               [&] { return thip_hl_maxpool2d(program_, &s); });
                aliasResult(op, s.init);
                return r;
            })
            .Case<torq_hl::AvgPool2DOp>([&](torq_hl::AvgPool2DOp c) {
                thip_hl_avg_pool2d_t s = {};
                s.input_zp = c.getInputZp(); s.output_zp = c.getOutputZp(); s.output_min = c.getOutputMin(); s.output_max = c.getOutputMax();
                s.shift_factor = c.getShiftFactor();
                LogicalResult r = withOperands(op, {{c.getInit(), &s.init}, {c.getWeights(), &s.weights}, {c.getScaleBias(), &s.scale_bias}, {c.getInput(), &s.input}},
                                               [&] { return thip_hl_avg_pool2d(program_, &s); });
                aliasResult(op, s.init);
                return r;
            })
            .Case<torq_hl::AddOp>([&](torq_hl::AddOp c) {
                thip_hl_add_t s = {};
                const std::string name = c.getName().str();  // "add" or "sub": the sign is already in the weights
                s.name = name.c_str();
                s.input_zp = c.getInputZp(); s.output_zp = c.getOutputZp(); s.output_min = c.getOutputMin(); s.output_max = c.getOutputMax();
                s.shift_factor = c.getShiftFactor(); s.segment_output = c.getSegmentOutput(); s.rhs_is_scalar = c.getRhsIsScalar();
                LogicalResult r = withOperands(op, {{c.getInit(), &s.init}, {c.getWeights(), &s.weights}, {c.getScaleBias(), &s.scale_bias},
                                                    {c.getInput1(), &s.input1}, {c.getInput2(), &s.input2}},
                                               [&] { return thip_hl_add(program_, &s); });
                aliasResult(op, s.init);
                return r;
            })
            .Case<torq_hl::TransposeOp>([&](torq_hl::TransposeOp c) {
                thip_hl_transpose_t s = {};
                ArrayRef<int64_t> perm = c.getPerm();
                if (perm.size() > THIP_MAX_RANK) return LogicalResult(op->emitError("MI355X backend: transpose rank above 4"));
                s.rank = (int32_t)perm.size();
                for (size_t i = 0; i < perm.size(); i++) s.perm[i] = perm[i];
                LogicalResult r = withOperands(op, {{c.getInit(), &s.init}, {c.getInput(), &s.input}}, [&] { return thip_hl_transpose(program_, &s); });
                aliasResult(op, s.init);
                return r;
            })
            .Case<torq_hl::ExpandWeightsOp>([&](torq_hl::ExpandWeightsOp c) {
                thip_hl_expand_weights_t s = {};
                s.output_min = c.getOutputMin(); s.output_max = c.getOutputMax(); s.block_size = c.getBlockSize();
                LogicalResult r = withOperands(op, {{c.getInit(), &s.init}, {c.getScaleBias(), &s.scale_bias}, {c.getScale(), &s.scale}, {c.getInput(), &s.input}},
                                               [&] { return thip_hl_expand_weights(program_, &s); });
                aliasResult(op, s.init);
                return r;
            })
            .Case<torq_hl::FMAOp>([&](torq_hl::FMAOp c) {
                thip_hl_fma_t s = {};
                s.output_zp = c.getOutputZp(); s.output_min = c.getOutputMin(); s.output_max = c.getOutputMax(); s.shift_factor = c.getShiftFactor();
                LogicalResult r = withOperands(op, {{c.getInit(), &s.init}, {c.getWeights(), &s.weights}, {c.getScaleBias(), &s.scale_bias}, {c.getInput(), &s.input}},
                                               [&] { return thip_hl_fma(program_, &s); });
                aliasResult(op, s.init);
                return r;
            })
            .Case<torq_hl::MulOp>([&](torq_hl::MulOp c) {
                thip_hl_mul_t s = {};
                s.output_zp = c.getOutputZp(); s.output_min = c.getOutputMin(); s.output_max = c.getOutputMax(); s.shift = c.getShift();
                LogicalResult r = withOperands(op, {{c.getInit(), &s.init}, {c.getScaleBias(), &s.scale_bias}, {c.getInput1(), &s.input1}, {c.getInput2(), &s.input2}},
                                               [&] { return thip_hl_mul(program_, &s); });
                aliasResult(op, s.init);
                return r;
            })
            .Case<torq_hl::ActOp>([&](torq_hl::ActOp c) {
                thip_hl_act_t s = {};
                const std::string name = c.getName().str();
                s.name = name.c_str();
                s.input_zp = c.getInputZp(); s.output_zp = c.getOutputZp(); s.min_int = c.getMinInt(); s.max_int = c.getMaxInt();
                s.min_fp = c.getMinFp().convertToFloat(); s.max_fp = c.getMaxFp().convertToFloat();
                LogicalResult r = withOperands(op, {{c.getInit(), &s.init}, {c.getInput(), &s.input}, {c.getWeights(), &s.weights}}, [&] { return thip_hl_act(program_, &s); });
                aliasResult(op, s.init);
                return r;
            })
            .Case<torq_hl::ElementWiseBinaryOp>([&](torq_hl::ElementWiseBinaryOp c) {
                thip_hl_elementwisebinary_t s = {};
                s.op_type = (int32_t)c.getOpType(); s.is_unsigned = c.getIsUnsigned();
                LogicalResult r = withOperands(op, {{c.getInit(), &s.init}, {c.getInput1(), &s.input1}, {c.getInput2(), &s.input2}},
                                               [&] { return thip_hl_elementwisebinary(program_, &s); });
                aliasResult(op, s.init);
                return r;
            })
            .Case<torq_hl::ElementWiseUnaryOp>([&](torq_hl::ElementWiseUnaryOp c) {
                thip_hl_elementwiseunary_t s = {};
                s.op_type = (int32_t)c.getOpType();
                LogicalResult r = withOperands(op, {{c.getInit(), &s.init}, {c.getInput(), &s.input}}, [&] { return thip_hl_elementwiseunary(program_, &s); });
                aliasResult(op, s.init);
                return r;
            })
            .Case<torq_hl::ElementWiseShiftOp>([&](torq_hl::ElementWiseShiftOp c) {
                thip_hl_elementwiseshift_t s = {};
                s.op_type = (int32_t)c.getOpType(); s.round = c.getRound();
                LogicalResult r = withOperands(op, {{c.getInit(), &s.init}, {c.getInput1(), &s.input1}, {c.getInput2(), &s.input2}},
                                               [&] { return thip_hl_elementwiseshift(program_, &s); });
                aliasResult(op, s.init);
                return r;
            })
            .Case<torq_hl::TableOp>([&](torq_hl::TableOp c) {
                // the plain lookups only (scale_bias = [-128, 128]); the interpolating tables of the bf16 activation
                // functions come back as THIP_UNIMPLEMENTED and stay on the NPU target
                thip_hl_table_t s = {};
                SmallVector<int32_t> words;
                if (auto attr = c.getStaticTableAttr()) {
                    words.assign(attr.asArrayRef().begin(), attr.asArrayRef().end());
                    s.static_table = words.data();
                    s.static_table_count = (int32_t)words.size();
                }
                LogicalResult r = withOperands(op, {{c.getInit(), &s.init}, {c.getScaleBias(), &s.scale_bias}, {c.getInput(), &s.input},
                                                    {c.getDynamicTable(), &s.dynamic_table}},
                                               [&] { return thip_hl_table(program_, &s); });
                aliasResult(op, s.init);
                return r;
            })
            .Default([&](Operation *other) {
                // everything else the pattern set can produce (reduce, gather, argmax, ...) stays on the NPU target
                return LogicalResult(other->emitError("MI355X backend: ") << other->getName() << " is outside the quantized operator path this target covers");
            });
    }
};

}  // namespace

LogicalResult serializeThipExecutable(ModuleOp innerModule, StringRef executableName, DenseIntElementsAttr &binaryAttr) {
    func::FuncOp entry;
    for (auto funcOp : innerModule.getOps<func::FuncOp>()) {
        if (entry) return innerModule.emitError("MI355X backend: one dispatch function per executable");
        entry = funcOp;
    }
    if (!entry) return innerModule.emitError("MI355X backend: no dispatch function");
    std::vector<uint8_t> blob;
    ProgramBuilder builder(entry);
    if (failed(builder.build(executableName, blob))) return failure();
    // what the driver would refuse is refused here, at compile time
    if (thip_descriptor_validate(blob.data(), blob.size()) != THIP_OK) {
        return entry.emitError() << "MI355X backend: emitted descriptor does not validate: " << thip_status_message();
    }
    auto type = RankedTensorType::get({(int64_t)blob.size()}, IntegerType::get(innerModule.getContext(), 8));
    binaryAttr = cast<DenseIntElementsAttr>(DenseElementsAttr::getFromRawBuffer(type, ArrayRef<char>((const char *)blob.data(), blob.size())));
    return success();
}

}  // namespace mlir::syna::thip
