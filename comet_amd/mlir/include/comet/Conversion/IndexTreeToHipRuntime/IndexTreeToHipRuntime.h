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
        /// Replaces every index tree whose shape is one of SpMV, SpMM (plus-times) and SpGEMM (with or
        /// without a mask, with any semiring the runtime knows) by calls into libcomet_hip_rt.so; every
        /// other tree is left for createLowerIndexTreeToSCFPass().
        /// indexBitwidth: 32 with --target=GPU (the front end then emits i32 index tensors), else 64.
        std::unique_ptr<Pass> createLowerIndexTreeToHipRuntimePass(unsigned indexBitwidth = 64);

        /// Replaces ta.mul on dense f64 tensors of rank <= 8 by one call to comet_hip_ttgt_contract_f64
        /// (upload, plan, transposes, GEMM, download); runs in place of createLoweringTTGTPass().
        std::unique_ptr<Pass> createLowerDenseContractionToHipRuntimePass();
    }
} // namespace mlir

#endif // COMET_CONVERSION_INDEXTREETOHIPRUNTIME_H
