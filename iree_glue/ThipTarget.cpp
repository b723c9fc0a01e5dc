// HAL target backend "thip" of the torq compiler plugin: the same input conversion and Linalg -> TorqHL pattern set
// as the NPU target, then the MI355X emitter instead of the NPU lowering.  Counterpart of
// compiler/torq/Target/TorqTarget.cpp:72-154 (device id, executable format, translation pipeline,
// serializeExecutable) and registered next to it from the plugin session
// (compiler/torq/PluginRegistration.cpp:270-276: populateHALTargetDevices / populateHALTargetBackends).
//
// Needs MLIR / IREE; compiled only inside the reference's tree (README.md in this directory).
#include "ThipSerialization.h"

#include "torq/Codegen/Passes.h"
#include "torq/Conversions/LinalgToTorqHL/Passes.h"
#include "torq/Dialect/TorqHL/TorqHLDialect.h"

#include "iree/compiler/Codegen/Dialect/Codegen/IR/IREECodegenDialect.h"
#include "iree/compiler/Dialect/HAL/Target/TargetRegistry.h"
#include "mlir/Dialect/Func/IR/FuncOps.h"
#include "mlir/Pass/PassManager.h"

using namespace mlir;
using namespace mlir::iree_compiler;

namespace mlir::syna::thip {

namespace {

constexpr const char *kDeviceId = "thip";
constexpr const char *kExecutableFormat = "thip-gfx950";  // what thip_infer_format answers

class ThipTargetDevice : public IREE::HAL::TargetDevice {
  public:
    IREE::HAL::DeviceTargetAttr getDefaultDeviceTarget(MLIRContext *context, const IREE::HAL::TargetRegistry &registry) const override {
        Builder b(context);
        SmallVector<IREE::HAL::ExecutableTargetAttr> executableTargets;
        registry.getTargetBackend(kDeviceId)->getDefaultExecutableTargets(context, kDeviceId, b.getDictionaryAttr({}), executableTargets);
        return IREE::HAL::DeviceTargetAttr::get(context, b.getStringAttr(kDeviceId), b.getDictionaryAttr({}), executableTargets);
    }
};

class ThipTargetBackend : public IREE::HAL::TargetBackend {
  public:
    std::string getLegacyDefaultDeviceID() const override { return kDeviceId; }

    void getDefaultExecutableTargets(MLIRContext *context, StringRef, DictionaryAttr,
                                     SmallVectorImpl<IREE::HAL::ExecutableTargetAttr> &executableTargetAttrs) const override {
        Builder b(context);
        executableTargetAttrs.push_back(
            IREE::HAL::ExecutableTargetAttr::get(context, b.getStringAttr(kDeviceId), b.getStringAttr(kExecutableFormat), b.getDictionaryAttr({})));
    }

    void getDependentDialects(DialectRegistry &registry) const override {
        registry.insert<torq_hl::TorqHLDialect, IREE::Codegen::IREECodegenDialect>();
    }

    void buildConfigurationPassPipeline(IREE::HAL::ExecutableTargetAttr, OpPassManager &) override {}

    // The NPU target's pipeline up to and including the Linalg -> TorqHL conversions
    // (compiler/torq/Codegen/TORQLowerExecutableTargetPass.cpp:117-142) and nothing after them: ValidToSamePad,
    // KernelSelection, segmentation, tensor encoding, slicing and address assignment rewrite the ops for the NPU's
    // memories and would only have to be undone.
    void buildTranslationPassPipeline(IREE::HAL::ExecutableTargetAttr, OpPassManager &passManager) override {
        OpPassManager &modulePm = passManager.nest<ModuleOp>();
        OpPassManager &funcPm = modulePm.nest<func::FuncOp>();
        torq::buildLinalgNormalizationPipeline(funcPm);           // the transforms of :323-356
        funcPm.addPass(torq::createLinalgToTorqHLPreConversionPass());
        funcPm.addPass(torq::createLinalgToTorqHLConversionPass());
    }

    void buildLinkingPassPipeline(OpPassManager &) override {}

    LogicalResult serializeExecutable(const SerializationOptions &, IREE::HAL::ExecutableVariantOp variantOp, OpBuilder &executableBuilder) override {
        auto exportOps = llvm::to_vector(variantOp.getOps<IREE::HAL::ExecutableExportOp>());
        if (exportOps.size() != 1) return variantOp.emitError() << "exactly one hal.executable.export op is supported";
        ModuleOp innerModuleOp = variantOp.getInnerModule();
        if (!innerModuleOp) return variantOp.emitError("expected a non-empty inner module");
        DenseIntElementsAttr binaryAttr;
        if (failed(serializeThipExecutable(innerModuleOp, exportOps.front().getSymName(), binaryAttr))) {
            return innerModuleOp.emitError("failed to serialize for the MI355X backend");
        }
        auto binaryOp = IREE::HAL::ExecutableBinaryOp::create(executableBuilder, variantOp.getLoc(), variantOp.getSymName(),
                                                              variantOp.getTarget().getFormat(), binaryAttr);
        binaryOp.setMimeTypeAttr(executableBuilder.getStringAttr("application/octet-stream"));
        return success();
    }
};

}  // namespace

// Called from the plugin session next to the NPU target's registration.
void populateHALTargetDevices(IREE::HAL::TargetDeviceList &targets) {
    targets.add(kDeviceId, [] { return std::make_shared<ThipTargetDevice>(); });
}
void populateHALTargetBackends(IREE::HAL::TargetBackendList &targets) {
    targets.add(kDeviceId, [] { return std::make_shared<ThipTargetBackend>(); });
}

}  // namespace mlir::syna::thip
