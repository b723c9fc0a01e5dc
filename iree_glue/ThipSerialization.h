// Serialises the TorqHL ops of one dispatch into a descriptor for the MI355X backend (see ThipSerialization.cpp).
#pragma once

#include "mlir/IR/BuiltinAttributes.h"
#include "mlir/IR/BuiltinOps.h"
#include "mlir/Support/LogicalResult.h"

namespace mlir::syna::thip {

// `innerModule` holds the dispatch function after the LinalgToTorqHL conversions; `binaryAttr` receives the blob
// (an i8 tensor attribute, what hal.executable.binary carries).
LogicalResult serializeThipExecutable(ModuleOp innerModule, StringRef executableName, DenseIntElementsAttr &binaryAttr);

}  // namespace mlir::syna::thip
