//===- IndexTreeToHipRuntime.cpp - index trees of the hot-path shapes -> HIP runtime calls ----===//
//
// Goes into pnnl/COMET as lib/Conversion/IndexTreeToHipRuntime/IndexTreeToHipRuntime.cpp.  It is source for
// the COMET build (needs its MLIR tree); nothing in this repository compiles or runs it.
//
// Where it runs: in frontends/comet_dsl/comet.cpp, inside the `IsLoweringtoSCF || emitLoops || ...` block,
// after createLowerTensorAlgebraToSCFPass() and BEFORE createIndexTreeSymbolicComputePass() (:529-533), under
//     if (CodegenTarget == TargetDevice::GPU && GpuRuntime == "hip-rt")
//       optPM.addPass(mlir::comet::createLowerIndexTreeToHipRuntimePass(/*indexBitwidth=*/32));
// so that a product it takes over never gets a symbolic tree, and every tree it leaves alone goes on to
// createLowerIndexTreeToSCFPass() exactly as before.  At that point tensor declarations are lowered: a sparse
// operand is the result of a ta.spTensor_construct (TensorDeclLowering.cpp:1096-1118), a dense one a tensor
// backed by a memref.alloc, and a tree is one it.itree region holding a chain of it.IndexOp, the operand ops
// and ONE it.ComputeOp (TensorAlgebraToIndexTree.cpp:225-443).
//
// What it matches (formats per dimension as SparseTensorType::getFormat() holds them, D = dense,
// CU = compressed unique; CSR = {D, CU}):
//
//   shape                                    indices   call (suffix _i32 or _i64 by the index tensors' width)
//   C[a]   = A[a,b] * B[b]     A CSR          a, b      comet_hip_spmv_csr_f64
//   C[a,c] = A[a,b] * B[b,c]   A CSR, B dense a, b, c   comet_hip_spmm_csr_f64
//   C[a,c] = A[a,b] * B[b,c]   all CSR        a, b, c   comet_hip_spgemm_csr_sizes_f64 + comet_hip_spgemm_csr_fill_f64
//            (+ optional mask operand of the compute op: its pos/crd are passed, else two empty memrefs)
//
//   C[a,c] = A[a,b] @(r,m) B[b,c] all CSR     a, b, c   comet_hip_spgemm_csr_sizes_semiring_f64 + ..._fill_semiring_f64
//            (the compute op's semiring attribute "<reduce>_<mult>", frontends/comet_dsl/mlir/MLIRGen.cpp:101-147,
//             turned into the runtime's operator codes; SpMV and SpMM are taken for plus-times only)
//
// A second pass in this file, createLowerDenseContractionToHipRuntimePass(), takes ta.mul on dense tensors of
// rank <= 8 - what --convert-tc-to-ttgt rewrites into transpose/collapse/matmul/expand/transpose
// (lib/Dialect/TensorAlgebra/Transforms/TCtoTTGTDyn.cpp:153-723) - and emits one call to
// comet_hip_ttgt_contract_f64 with the three tensors as unranked memrefs and their index labels (the positions of
// the affine maps' results) as constant index memrefs.  It runs where createLoweringTTGTPass() would
// (frontends/comet_dsl/comet.cpp:447-470), under the same GpuRuntime == "hip-rt" switch.
//
// The callee declarations follow declare_vendor_funcs (lib/Conversion/GpuUtils/GpuUtils.cpp:307-411): private
// func.func added to the module, here with llvm.emit_c_interface so that the symbol resolved at link time is
// _mlir_ciface_<name> and every memref arrives as a pointer to its descriptor (include/comet_hip_rt.h).
//
//===------------------------------------------------------------------------------------------===//

#include "comet/Conversion/IndexTreeToHipRuntime/IndexTreeToHipRuntime.h"
#include "comet/Dialect/IndexTree/IR/IndexTreeDialect.h"
#include "comet/Dialect/TensorAlgebra/IR/TADialect.h"
#include "comet/Dialect/Utils/Utils.h"

#include "llvm/ADT/StringSwitch.h"
#include "mlir/Dialect/Arith/IR/Arith.h"
#include "mlir/Dialect/Bufferization/IR/Bufferization.h"
#include "mlir/Dialect/Func/IR/FuncOps.h"
#include "mlir/Dialect/MemRef/IR/MemRef.h"
#include "mlir/Dialect/Tensor/IR/Tensor.h"
#include "mlir/IR/AffineExpr.h"
#include "mlir/IR/AffineMap.h"
#include "mlir/IR/BuiltinOps.h"
#include "mlir/IR/PatternMatch.h"
#include "mlir/Pass/Pass.h"

using namespace mlir;
using namespace mlir::indexTree;
using namespace mlir::tensorAlgebra;

namespace
{
  enum class Shape
  {
    None,
    SpMV,
    SpMM,
    SpGEMM
  };

  /// One matched tree: the compute op and its tensors as the enclosing function sees them.
  struct Match
  {
    Shape shape = Shape::None;
    IndexTreeComputeOp compute;
    Value lhs, a, b, mask;
    int reduceOp = 0, multOp = 0; /// COMET_SR_* / COMET_OP_* of include/comet_hip_rt.h
  };

  /// "<reduce>_<mult>" with the DSL's operator names -> the runtime's codes; false if either is unknown to it
  /// (lor, land, noop: those trees stay with the loop lowering).
  bool semiringCodes(StringRef semiring, int &reduceOp, int &multOp)
  {
    auto parts = semiring.split('_');
    int r = llvm::StringSwitch<int>(parts.first).Case("plusxy", 0).Case("minxy", 1).Case("any", 3).Default(-1);
    int m = llvm::StringSwitch<int>(parts.second)
                .Case("times", 0)
                .Case("first", 1)
                .Case("second", 2)
                .Case("pairxy", 3)
                .Case("plusxy", 4)
                .Case("minus", 5)
                .Default(-1);
    if (r < 0 || m < 0)
      return false;
    reduceOp = r;
    multOp = m;
    return true;
  }

  bool isCSR(Type t)
  {
    auto st = dyn_cast<SparseTensorType>(t);
    if (!st || st.getDims().size() != 2)
      return false;
    auto f = st.getFormat(); /// two entries per dimension: format, tile format
    return (TensorFormatEnum)f[0] == TensorFormatEnum::D && (TensorFormatEnum)f[2] == TensorFormatEnum::CU;
  }

  bool isDenseOfRank(Type t, int64_t rank)
  {
    auto rt = dyn_cast<RankedTensorType>(t);
    return rt && rt.getRank() == rank && rt.getElementType().isF64();
  }

  /// A tensor used inside the tree is either defined outside it or is the region argument that stands for
  /// the tree's input (generalIndexOperationRewrite passes the output tensor in that way).
  Value outsideValue(IndexTreeOp tree, Value v)
  {
    if (auto arg = dyn_cast<BlockArgument>(v))
      if (arg.getOwner()->getParentOp() == tree.getOperation())
        return tree.getInputs()[arg.getArgNumber()];
    return v;
  }

  Match classify(IndexTreeOp tree)
  {
    Match m;
    SmallVector<IndexTreeComputeOp> computes;
    unsigned nIndices = 0;
    tree.getRegion().walk([&](Operation *op)
                          {
      if (auto c = dyn_cast<IndexTreeComputeOp>(op))
        computes.push_back(c);
      else if (isa<IndexTreeIndicesOp>(op))
        ++nIndices; });
    if (computes.size() != 1 || tree->getNumResults() != 1)
      return m; /// fused trees and workspace forms go to the loop lowering
    IndexTreeComputeOp c = computes.front();
    if (!semiringCodes(c.getSemiring(), m.reduceOp, m.multOp) || c.getRhs().size() != 2 || c.getComputeMissing())
      return m;
    const bool plusTimes = m.reduceOp == 0 && m.multOp == 0;
    auto lhsOp = c.getLhs().getDefiningOp<IndexTreeLHSOperandOp>();
    auto aOp = c.getRhs()[0].getDefiningOp<IndexTreeOperandOp>();
    auto bOp = c.getRhs()[1].getDefiningOp<IndexTreeOperandOp>();
    if (!lhsOp || !aOp || !bOp)
      return m;
    m.compute = c;
    m.lhs = outsideValue(tree, lhsOp.getTensor());
    m.a = outsideValue(tree, aOp.getTensor());
    m.b = outsideValue(tree, bOp.getTensor());
    if (c.getMask())
      if (auto mOp = c.getMask().getDefiningOp<IndexTreeOperandOp>())
        m.mask = outsideValue(tree, mOp.getTensor());

    Type tl = m.lhs.getType(), ta = m.a.getType(), tb = m.b.getType();
    if (!isCSR(ta))
      return m;
    if (nIndices == 2 && isDenseOfRank(tb, 1) && isDenseOfRank(tl, 1) && !m.mask && plusTimes)
      m.shape = Shape::SpMV;
    else if (nIndices == 3 && isDenseOfRank(tb, 2) && isDenseOfRank(tl, 2) && !m.mask && plusTimes)
      m.shape = Shape::SpMM;
    else if (nIndices == 3 && isCSR(tb) && isCSR(tl) && (!m.mask || isCSR(m.mask.getType())))
      m.shape = Shape::SpGEMM;
    return m;
  }

  struct Lowering
  {
    OpBuilder &b;
    ModuleOp module;
    unsigned width;

    Type idxElem() { return b.getIntegerType(width); }
    MemRefType idxMemref() { return MemRefType::get({ShapedType::kDynamic}, idxElem()); }
    MemRefType f64Memref(unsigned rank)
    {
      return MemRefType::get(SmallVector<int64_t>(rank, ShapedType::kDynamic), b.getF64Type());
    }
    std::string name(StringRef stem) { return ("comet_hip_" + stem + "_f64_i" + Twine(width)).str(); }

    /// private func.func with llvm.emit_c_interface, once per module (cf. declare_vendor_funcs)
    void declare(StringRef fn, TypeRange args, TypeRange results)
    {
      if (module.lookupSymbol<func::FuncOp>(fn))
        return;
      OpBuilder::InsertionGuard g(b);
      b.clearInsertionPoint();
      auto f = b.create<func::FuncOp>(b.getUnknownLoc(), fn, b.getFunctionType(args, results));
      f.setVisibility(SymbolTable::Visibility::Private);
      f->setAttr("llvm.emit_c_interface", b.getUnitAttr());
      module.push_back(f);
    }

    /// tensor<?x..> -> memref<?x..> of the same element type (the tensors here are to_tensor views of
    /// allocations, so this folds back to the allocation during bufferisation)
    Value buffer(Location loc, Value tensor)
    {
      auto tt = cast<RankedTensorType>(tensor.getType());
      return b.create<bufferization::ToMemrefOp>(loc, MemRefType::get(tt.getShape(), tt.getElementType()), tensor);
    }
    Value pos(Location loc, Value sp) { return buffer(loc, b.create<SpTensorGetDimPos>(loc, sp, b.getI32IntegerAttr(1))); }
    Value crd(Location loc, Value sp) { return buffer(loc, b.create<SpTensorGetDimCrd>(loc, sp, b.getI32IntegerAttr(1))); }
    Value vals(Location loc, Value sp) { return buffer(loc, b.create<SpTensorGetVals>(loc, sp)); }
    Value dim(Location loc, Value sp, int d) { return b.create<SpTensorGetDimSize>(loc, sp, b.getI32IntegerAttr(d)); }
    Value i64(Location loc, Value index) { return b.create<arith::IndexCastOp>(loc, b.getI64Type(), index); }

    /// y (+)= A x  and  C (+)= A B: the runtime adds into the output it is given, like the loop nest it
    /// replaces (IndexTreeToSCF.cpp:1247-1284), so the fill that precedes the statement stays valid.
    void lowerDense(IndexTreeOp tree, Match &m, StringRef stem, unsigned rank)
    {
      Location loc = tree.getLoc();
      declare(name(stem), {idxMemref(), idxMemref(), f64Memref(1), f64Memref(rank), f64Memref(rank)}, {});
      b.setInsertionPoint(tree);
      Value out = buffer(loc, m.lhs);
      b.create<func::CallOp>(loc, name(stem), TypeRange{},
                             ValueRange{pos(loc, m.a), crd(loc, m.a), vals(loc, m.a), buffer(loc, m.b), out});
      /// the call wrote through `out`: the tree's result is the same tensor again
      Value res = b.create<bufferization::ToTensorOp>(loc, out, b.getUnitAttr(), b.getUnitAttr());
      tree->getResult(0).replaceAllUsesWith(res);
      tree.erase();
    }

    /// CSR x CSR -> CSR in the reader's two-call style (TensorDeclLowering.cpp:994-1118): sizes, allocate
    /// pos/crd/val, fill, spTensor_construct.
    void lowerSpGEMM(IndexTreeOp tree, Match &m)
    {
      Location loc = tree.getLoc();
      auto indexMemref = MemRefType::get({ShapedType::kDynamic}, b.getIndexType());
      SmallVector<Type> sizesArgs = {b.getI64Type(), b.getI64Type()};
      for (int k = 0; k < 2; ++k)
        sizesArgs.append({idxMemref(), idxMemref(), f64Memref(1)}); /// A, B
      sizesArgs.append({idxMemref(), idxMemref(), indexMemref});       /// mask pos/crd, sizes
      const bool semi = m.reduceOp != 0 || m.multOp != 0;
      if (semi)
        sizesArgs.append({b.getI32Type(), b.getI32Type()}); /// reduce and mult operator codes
      const std::string sizesFn = name(semi ? "spgemm_csr_sizes_semiring" : "spgemm_csr_sizes");
      const std::string fillFn = name(semi ? "spgemm_csr_fill_semiring" : "spgemm_csr_fill");
      declare(sizesFn, sizesArgs, {});
      declare(fillFn, {idxMemref(), idxMemref(), f64Memref(1)}, {});

      b.setInsertionPoint(tree);
      Value zero = b.create<arith::ConstantIndexOp>(loc, 0);
      Value one = b.create<arith::ConstantIndexOp>(loc, 1);
      Value nrows = dim(loc, m.a, 0), ncols = dim(loc, m.b, 1);
      Value sizes = b.create<memref::AllocOp>(loc, indexMemref, ValueRange{one});
      Value mpos, mcrd;
      if (m.mask)
      {
        mpos = pos(loc, m.mask);
        mcrd = crd(loc, m.mask);
      }
      else
      { /// no mask: two memrefs of size 0
        mpos = b.create<memref::AllocOp>(loc, idxMemref(), ValueRange{zero});
        mcrd = b.create<memref::AllocOp>(loc, idxMemref(), ValueRange{zero});
      }
      SmallVector<Value> sizesOperands = {i64(loc, nrows), i64(loc, ncols), pos(loc, m.a), crd(loc, m.a), vals(loc, m.a),
                                          pos(loc, m.b), crd(loc, m.b), vals(loc, m.b), mpos, mcrd, sizes};
      if (semi)
      {
        sizesOperands.push_back(b.create<arith::ConstantIntOp>(loc, m.reduceOp, 32));
        sizesOperands.push_back(b.create<arith::ConstantIntOp>(loc, m.multOp, 32));
      }
      b.create<func::CallOp>(loc, sizesFn, TypeRange{}, sizesOperands);
      Value nnz = b.create<memref::LoadOp>(loc, sizes, ValueRange{zero});
      Value npos = b.create<arith::AddIOp>(loc, nrows, one);
      Value cpos = b.create<memref::AllocOp>(loc, idxMemref(), ValueRange{npos});
      Value ccrd = b.create<memref::AllocOp>(loc, idxMemref(), ValueRange{nnz});
      Value cval = b.create<memref::AllocOp>(loc, f64Memref(1), ValueRange{nnz});
      b.create<func::CallOp>(loc, fillFn, TypeRange{}, ValueRange{cpos, ccrd, cval});

      /// the remaining arrays of the CSR tuple: A1pos = [nrows], A1crd and the tile arrays = [-1]
      /// (what read_input_2D leaves in them, SparseUtils.cpp:1840-1848, 1898-1936)
      auto small = [&](Value v) -> Value
      {
        Value mem = b.create<memref::AllocOp>(loc, idxMemref(), ValueRange{one});
        b.create<memref::StoreOp>(loc, v, mem, ValueRange{zero});
        return b.create<bufferization::ToTensorOp>(loc, mem, b.getUnitAttr(), b.getUnitAttr());
      };
      Value minus1 = b.create<arith::ConstantOp>(loc, idxElem(), b.getIntegerAttr(idxElem(), -1));
      Value nrowsIdx = b.create<arith::IndexCastOp>(loc, idxElem(), nrows);
      auto tensorOf = [&](Value mem) -> Value
      { return b.create<bufferization::ToTensorOp>(loc, mem, b.getUnitAttr(), b.getUnitAttr()); };
      Value dims = b.create<tensor::FromElementsOp>(loc, ValueRange{nrows, ncols});
      auto lhsType = cast<SparseTensorType>(m.lhs.getType());
      Value c = b.create<SparseTensorConstructOp>(
          loc, lhsType, dims,
          ValueRange{small(nrowsIdx), tensorOf(cpos)}, /// A1pos, A2pos
          ValueRange{small(minus1), tensorOf(ccrd)},   /// A1crd, A2crd
          ValueRange{small(minus1), small(minus1)},    /// tile pos
          ValueRange{small(minus1), small(minus1)},    /// tile crd
          tensorOf(cval), 2, m.lhs.getDefiningOp() ? m.lhs.getDefiningOp()->getAttr("dimension_formats") : Attribute());
      tree->getResult(0).replaceAllUsesWith(c);
      tree.erase();
    }
  };

  struct LowerIndexTreeToHipRuntimePass
      : public PassWrapper<LowerIndexTreeToHipRuntimePass, OperationPass<ModuleOp>>
  {
    MLIR_DEFINE_EXPLICIT_INTERNAL_INLINE_TYPE_ID(LowerIndexTreeToHipRuntimePass)
    unsigned width;
    explicit LowerIndexTreeToHipRuntimePass(unsigned w) : width(w) {}

    StringRef getArgument() const final { return "convert-it-to-hip-runtime"; }
    StringRef getDescription() const final
    {
      return "Replace index trees of the SpMV, SpMM and SpGEMM shapes by calls into libcomet_hip_rt";
    }
    void getDependentDialects(DialectRegistry &registry) const override
    {
      registry.insert<func::FuncDialect, memref::MemRefDialect, arith::ArithDialect, tensor::TensorDialect,
                      bufferization::BufferizationDialect>();
    }

    void runOnOperation() override
    {
      ModuleOp module = getOperation();
      SmallVector<IndexTreeOp> trees;
      module.walk([&](IndexTreeOp t) { trees.push_back(t); });
      OpBuilder builder(module.getContext());
      Lowering low{builder, module, width};
      for (IndexTreeOp tree : trees)
      {
        Match m = classify(tree);
        /// the index tensors of the operands must have the width the callee was declared with
        if (m.shape != Shape::None &&
            cast<SparseTensorType>(m.a.getType()).getIndicesType().getIntOrFloatBitWidth() != width)
          m.shape = Shape::None;
        switch (m.shape)
        {
        case Shape::SpMV:
          low.lowerDense(tree, m, "spmv_csr", 1);
          break;
        case Shape::SpMM:
          low.lowerDense(tree, m, "spmm_csr", 2);
          break;
        case Shape::SpGEMM:
          low.lowerSpGEMM(tree, m);
          break;
        case Shape::None:
          break; /// stays an index tree: createLowerIndexTreeToSCFPass() takes it
        }
      }
    }
  };

  /// ta.mul on dense f64 tensors -> one call to comet_hip_ttgt_contract_f64.
  struct LowerDenseContractionToHipRuntimePass
      : public PassWrapper<LowerDenseContractionToHipRuntimePass, OperationPass<ModuleOp>>
  {
    MLIR_DEFINE_EXPLICIT_INTERNAL_INLINE_TYPE_ID(LowerDenseContractionToHipRuntimePass)
    StringRef getArgument() const final { return "convert-tc-to-hip-runtime"; }
    StringRef getDescription() const final
    {
      return "Replace dense tensor contractions (ta.mul) by a call to comet_hip_ttgt_contract_f64 of libcomet_hip_rt";
    }
    void getDependentDialects(DialectRegistry &registry) const override
    {
      registry.insert<func::FuncDialect, memref::MemRefDialect, arith::ArithDialect, bufferization::BufferizationDialect>();
    }

    void runOnOperation() override
    {
      ModuleOp module = getOperation();
      OpBuilder b(module.getContext());
      const char *fn = "comet_hip_ttgt_contract_f64";
      auto unrankedF64 = UnrankedMemRefType::get(b.getF64Type(), 0);
      auto labels = MemRefType::get({ShapedType::kDynamic}, b.getIndexType());
      SmallVector<TensorMultOp> mults;
      module.walk([&](TensorMultOp op) { mults.push_back(op); });
      for (TensorMultOp op : mults)
      {
        /// operands as TCtoTTGTDyn.cpp:161-231 reads them: rhs1, rhs2, and the tensor the result is set into
        Value a = op->getOperand(0), c2 = op->getOperand(1), dst;
        TensorSetOp set;
        for (Operation *u : op->getResult(0).getUsers())
          if ((set = dyn_cast<TensorSetOp>(u)))
            dst = set->getOperand(1);
        auto ta = dyn_cast<RankedTensorType>(a.getType()), tb = dyn_cast<RankedTensorType>(c2.getType());
        auto tc = dst ? dyn_cast<RankedTensorType>(dst.getType()) : RankedTensorType();
        if (!ta || !tb || !tc || !ta.getElementType().isF64() || ta.getRank() > 8 || tb.getRank() > 8 || tc.getRank() > 8)
          continue; /// sparse operands and other element types go the reference's way
        if (!module.lookupSymbol<func::FuncOp>(fn))
        {
          OpBuilder::InsertionGuard g(b);
          b.clearInsertionPoint();
          auto f = b.create<func::FuncOp>(
              b.getUnknownLoc(), fn,
              b.getFunctionType({unrankedF64, unrankedF64, unrankedF64, labels, labels, labels, b.getF64Type()}, {}));
          f.setVisibility(SymbolTable::Visibility::Private);
          f->setAttr("llvm.emit_c_interface", b.getUnitAttr());
          module.push_back(f);
        }
        Location loc = op.getLoc();
        b.setInsertionPoint(op);
        auto asUnranked = [&](Value tensor)
        {
          auto tt = cast<RankedTensorType>(tensor.getType());
          Value mem = b.create<bufferization::ToMemrefOp>(loc, MemRefType::get(tt.getShape(), tt.getElementType()), tensor);
          return b.create<memref::CastOp>(loc, unrankedF64, mem).getResult();
        };
        /// the labels of an operand: the dimension positions its indexing map names, as index constants
        auto labelMemref = [&](AffineMap map)
        {
          Value n = b.create<arith::ConstantIndexOp>(loc, map.getNumResults());
          Value mem = b.create<memref::AllocOp>(loc, labels, ValueRange{n});
          for (unsigned i = 0; i < map.getNumResults(); ++i)
          {
            Value at = b.create<arith::ConstantIndexOp>(loc, i);
            Value lab = b.create<arith::ConstantIndexOp>(loc, cast<AffineDimExpr>(map.getResult(i)).getPosition());
            b.create<memref::StoreOp>(loc, lab, mem, ValueRange{at});
          }
          return mem;
        };
        ArrayAttr maps = op.getIndexingMaps();
        Value la = labelMemref(cast<AffineMapAttr>(maps[0]).getValue());
        Value lb = labelMemref(cast<AffineMapAttr>(maps[1]).getValue());
        Value lc = labelMemref(cast<AffineMapAttr>(maps[2]).getValue());
        double betaValue = 0.0;
        if (auto betaAttr = op->getAttrOfType<FloatAttr>("__beta__"))
          betaValue = betaAttr.getValueAsDouble();
        Value beta = b.create<arith::ConstantFloatOp>(loc, APFloat(betaValue), b.getF64Type());
        Value cm = asUnranked(dst);
        b.create<func::CallOp>(loc, fn, TypeRange{}, ValueRange{asUnranked(a), asUnranked(c2), cm, la, lb, lc, beta});
        /// the call wrote through dst's buffer: the set op that copied the product into it has nothing left to do
        op->getResult(0).replaceAllUsesWith(dst);
        set.erase();
        op.erase();
      }
    }
  };
} // namespace

std::unique_ptr<Pass> mlir::comet::createLowerIndexTreeToHipRuntimePass(unsigned indexBitwidth)
{
  return std::make_unique<LowerIndexTreeToHipRuntimePass>(indexBitwidth);
}

std::unique_ptr<Pass> mlir::comet::createLowerDenseContractionToHipRuntimePass()
{
  return std::make_unique<LowerDenseContractionToHipRuntimePass>();
}
