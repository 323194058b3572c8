//===- IndexTreeToHipRuntime.h - index trees of the hot-path shapes -> HIP runtime calls -*- C++ -*-===//
//
// Goes into pnnl/COMET as include/comet/Conversion/IndexTreeToHipRuntime/IndexTreeToHipRuntime.h, next to
// include/comet/Conversion/IndexTreeToSCF/IndexTreeToSCF.h, whose layout it follows.
//
//===----------------------------------------------------------------------------------------------===//
#ifndef COMET_CONVERSION_INDEXTREETOHIPRUNTIME_H
#define COMET_CONVERSION_INDEXTREETOHIPRUNTIME_H

#include <memory>

#include "mlir/Support/LLVM.h"

namespace mlir
{
    class Pass;

    namespace comet
    {
        /// Replaces every index tree whose shape is one of SpMV, SpMM, SpGEMM (with or without a mask and
        /// with any semiring the runtime knows), dense-times-CSR and CSR .* CSR by calls into
        /// libcomet_hip_rt.so; every other tree is left for createLowerIndexTreeToSCFPass().
        /// indexBitwidth: 32 with --target=GPU (the front end then emits i32 index tensors), else 64.
        std::unique_ptr<Pass> createLowerIndexTreeToHipRuntimePass(unsigned indexBitwidth = 64);
    }
} // namespace mlir

#endif // COMET_CONVERSION_INDEXTREETOHIPRUNTIME_H
