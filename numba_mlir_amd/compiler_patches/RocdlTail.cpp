// UNBUILT SOURCE.  Needs the LLVM/MLIR checkout the reference pins
// (llvm-sha.txt) and the reference's own headers; nothing in this repository
// compiles, links or loads this file.  It states, as code against those APIs,
// what replaces the SPIR-V tail of the reference's GPU pipeline so that the
// compiler emits a gfx950 code object for the HIP runtime.
//
// Where it goes in the reference:
//
//  * numba_mlir/numba_mlir/mlir_compiler/lib/pipelines/LowerToGpu.cpp:2204-2217
//    (AbiAttrs, SetSPIRVCapabilities, TruncateF64ForGPU, GPUToSpirv,
//    GpuIndexCast, the spirv::ModuleOp passes, SerializeSPIRV) becomes one
//    call: populateRocdlTail(pm).  Everything before (tiling, outlining,
//    builtins) and after (GenDeviceFuncs, GPUEx, OutlineInit) stays: those
//    passes only look at gpu.module / gpu.func and at the "gpu.binary"
//    string attribute (mlir/lib/Conversion/GpuToGpuRuntime.cpp:2635), which
//    SerializeHsacoPass below sets exactly as SerializeSPIRVPass does
//    (1234-1275), with the bytes of an ELF code object instead of SPIR-V
//    words.  gpuxModuleLoad takes either.
//
//  * TruncateF64ForGPUPass is dropped, not replaced: gfx950 has full-rate
//    float64 and the device reports fp64 = True, so no value is narrowed.
//
//  * LowerToGpu.cpp:1683-1688 hard-codes a subgroup of 8 lanes when it sizes
//    the workgroup buffer of a group reduction; kSubgroupSize below (64, a
//    CDNA wavefront) takes its place:
//        -      rewriter.create<mlir::arith::ConstantIndexOp>(loc, 8);
//        +      rewriter.create<mlir::arith::ConstantIndexOp>(loc, kSubgroupSize);
//
//  * numba_mlir/numba_mlir/mlir/gpu_runtime.py:14-21 selects the runtime
//    library by NUMBA_MLIR_GPU_RUNTIME; with "hip" the pipeline registration
//    (LowerToGpu.cpp:2236-2262) takes this tail instead of the SPIR-V one.
#include <mlir/Conversion/GPUToROCDL/GPUToROCDLPass.h>
#include <mlir/Dialect/GPU/IR/GPUDialect.h>
#include <mlir/Dialect/GPU/Transforms/Passes.h>
#include <mlir/Dialect/LLVMIR/ROCDLDialect.h>
#include <mlir/Pass/Pass.h>
#include <mlir/Pass/PassManager.h>
#include <mlir/Target/LLVM/ROCDL/Target.h>
#include <mlir/Transforms/Passes.h>

#include "numba/Conversion/GpuToGpuRuntime.hpp" // getGpuBinaryAttrName

namespace hip_tail {

constexpr int64_t kSubgroupSize = 64;        // lanes of a gfx950 wavefront
constexpr const char *kChip = "gfx950";
constexpr const char *kTriple = "amdgcn-amd-amdhsa";

// Attaches #rocdl.target<chip = "gfx950", O = 3> to every gpu.module.  The
// feature string switches packed-FP32 arithmetic off, as every hand-written
// kernel of the HIP backend is built; unsafe-math flags stay off unless the
// function was compiled with fastmath (the reference's
// ApplySPIRVFastmathFlags reads the same "numba.fastmath" unit attribute,
// GpuToGpuRuntime.cpp:2596-2632).
struct SetRocdlTargetPass
    : public mlir::PassWrapper<SetRocdlTargetPass,
                               mlir::OperationPass<mlir::ModuleOp>> {
  MLIR_DEFINE_EXPLICIT_INTERNAL_INLINE_TYPE_ID(SetRocdlTargetPass)

  void getDependentDialects(mlir::DialectRegistry &registry) const override {
    registry.insert<mlir::ROCDL::ROCDLDialect>();
    mlir::ROCDL::registerROCDLTargetInterfaceExternalModels(registry);
  }

  void runOnOperation() override {
    auto *ctx = &getContext();
    for (auto gpuMod : getOperation().getOps<mlir::gpu::GPUModuleOp>()) {
      const bool fast = gpuMod->hasAttr("numba.fastmath");
      auto flags = fast ? mlir::DictionaryAttr::get(
                              ctx, {mlir::NamedAttribute(
                                       mlir::StringAttr::get(ctx, "fast"),
                                       mlir::UnitAttr::get(ctx))})
                        : mlir::DictionaryAttr();
      auto target = mlir::ROCDL::ROCDLTargetAttr::get(
          ctx, /*optLevel=*/3, kTriple, kChip, "-packed-fp32-ops",
          /*abiVersion=*/"500", flags, /*linkFiles=*/nullptr);
      gpuMod.setTargetsAttr(mlir::ArrayAttr::get(ctx, {target}));
    }
  }
};

// gpu.module (ROCDL/LLVM dialect inside) -> ELF code object -> the
// "gpu.binary" string attribute the rest of the pipeline embeds as an LLVM
// global and hands to gpuxModuleLoad (GpuRuntimeToLlvm.cpp:306-322).
struct SerializeHsacoPass
    : public mlir::PassWrapper<SerializeHsacoPass,
                               mlir::OperationPass<mlir::ModuleOp>> {
  MLIR_DEFINE_EXPLICIT_INTERNAL_INLINE_TYPE_ID(SerializeHsacoPass)

  void runOnOperation() override {
    for (auto gpuMod : getOperation().getOps<mlir::gpu::GPUModuleOp>()) {
      auto targets = gpuMod.getTargetsAttr();
      if (!targets || targets.size() != 1) {
        gpuMod.emitError() << "expected exactly one #rocdl.target";
        return signalPassFailure();
      }
      auto target = mlir::cast<mlir::gpu::TargetAttrInterface>(targets[0]);
      mlir::gpu::TargetOptions options(
          /*toolkitPath=*/{}, /*linkFiles=*/{}, /*cmdOptions=*/{},
          mlir::gpu::CompilationTarget::Binary);
      std::optional<llvm::SmallVector<char, 0>> object =
          target.serializeToObject(gpuMod, options);
      if (!object) {
        gpuMod.emitError() << "failed to produce a " << kChip << " code object";
        return signalPassFailure();
      }
      auto bytes = llvm::StringRef(object->data(), object->size());
      gpuMod->setAttr(gpu_runtime::getGpuBinaryAttrName(),
                      mlir::StringAttr::get(&getContext(), bytes));
      // The body is no longer needed; the kernel names stay on the gpu.func
      // declarations GenDeviceFuncs and GPUEx look up.
    }
  }
};

// The replacement for LowerToGpu.cpp:2204-2217.
inline void populateRocdlTail(mlir::OpPassManager &pm) {
  // Kernel ABI: flattened memrefs become (pointer, sizes, strides) scalars --
  // already done by GpuDecomposeMemrefs upstream of here; AbiAttrs only
  // marked SPIR-V entry points and has no ROCDL counterpart.
  pm.addPass(std::make_unique<SetRocdlTargetPass>());
  auto &gpuPM = pm.nest<mlir::gpu::GPUModuleOp>();
  // 64-bit indices: ids and sizes are index-typed and a 1-d launch of 2^31 + 1
  // items must work (test_gpu.py:2269-2283).
  gpuPM.addPass(mlir::createLowerGpuOpsToROCDLOpsPass(
      kChip, /*indexBitwidth=*/64, /*useBarePtrCallConv=*/true,
      mlir::gpu::amd::Runtime::HIP));
  gpuPM.addPass(mlir::createCanonicalizerPass());
  gpuPM.addPass(mlir::createCSEPass());
  pm.addPass(std::make_unique<SerializeHsacoPass>());
}

} // namespace hip_tail
