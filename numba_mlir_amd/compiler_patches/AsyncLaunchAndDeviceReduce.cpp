// UNBUILT SOURCE.  Needs the LLVM/MLIR checkout the reference pins
// (llvm-sha.txt) and the reference's own headers; nothing in this repository
// compiles, links or loads this file.  The runtime and kernel halves of both
// changes exist and are tested here (gpuxLaunchKernel returns an event that
// later launches and gpuxWait accept; csrc/kernels/reduce.hip finishes a
// reduction on the device); this file states the compiler half.
//
// 1. Launches without a host wait in between.
//    mlir/lib/Conversion/GpuRuntimeToLlvm.cpp:619-625 already returns the
//    event of a launch that carries an async token and only waits + destroys
//    when it has none; no producer ever gives one.  ChainLaunchesPass gives
//    every gpu_runtime.launch_gpu_kernel of a block a token, makes each launch
//    depend on the previous one's token (the HIP queue is in order, so the
//    dependency costs nothing at run time) and places one gpu.wait on the last
//    token before the first host use of a buffer the launches wrote, or at
//    the end of the block.  ConvertGpuWaitPattern lowers that gpu.wait to
//    gpuxWait + gpuxDestroyEvent per token.
//
// 2. Reductions finished on the device.
//    LowerGPUGlobalReduce (mlir/lib/Conversion/GpuToGpuRuntime.cpp:2161-2277)
//    allocates a host-shared array of one partial result per workgroup,
//    launches, waits and folds the array in a host loop.  finishOnDevice()
//    keeps the per-workgroup gpu.all_reduce, stores the partial in a DEVICE
//    array and lets the workgroup that arrives last -- counted with one
//    atomic increment of a zero-initialised ticket -- fold the partials in
//    workgroup order and store the result: one launch, no host-shared
//    memory, no host loop, bit-identical from run to run.
#include <mlir/Dialect/Arith/IR/Arith.h>
#include <mlir/Dialect/GPU/IR/GPUDialect.h>
#include <mlir/Dialect/LLVMIR/LLVMDialect.h>
#include <mlir/IR/IRMapping.h>
#include <mlir/Dialect/MemRef/IR/MemRef.h>
#include <mlir/Dialect/SCF/IR/SCF.h>
#include <mlir/Pass/Pass.h>
#include <mlir/Transforms/DialectConversion.h>

#include "numba/Dialect/gpu_runtime/IR/GpuRuntimeOps.hpp"

namespace hip_async {

// ---- 1. one wait per chain of launches --------------------------------------
struct ChainLaunchesPass
    : public mlir::PassWrapper<ChainLaunchesPass, mlir::OperationPass<void>> {
  MLIR_DEFINE_EXPLICIT_INTERNAL_INLINE_TYPE_ID(ChainLaunchesPass)

  void runOnOperation() override {
    getOperation()->walk([&](mlir::Block *block) { chain(*block); });
  }

  static bool readsOnHost(mlir::Operation &op,
                          llvm::ArrayRef<mlir::Value> written) {
    if (mlir::isa<gpu_runtime::LaunchGpuKernelOp>(op))
      return false;
    // Conservative: any other op that takes one of the written buffers, or
    // has regions / unknown effects, ends the chain.
    if (op.getNumRegions() != 0 || !mlir::isMemoryEffectFree(&op))
      for (mlir::Value v : op.getOperands())
        if (llvm::is_contained(written, v))
          return true;
    return op.hasTrait<mlir::OpTrait::IsTerminator>();
  }

  void chain(mlir::Block &block) {
    mlir::OpBuilder builder(block.getParent()->getContext());
    auto tokenType = mlir::gpu::AsyncTokenType::get(builder.getContext());
    mlir::Value last;                       // token of the previous launch
    llvm::SmallVector<mlir::Value> written; // kernel operands since the wait
    auto flush = [&](mlir::Operation *before) {
      if (!last)
        return;
      builder.setInsertionPoint(before);
      builder.create<mlir::gpu::WaitOp>(before->getLoc(), mlir::Type(),
                                        mlir::ValueRange(last));
      last = nullptr;
      written.clear();
    };
    for (mlir::Operation &op : llvm::make_early_inc_range(block)) {
      if (auto launch = mlir::dyn_cast<gpu_runtime::LaunchGpuKernelOp>(op)) {
        if (launch.getAsyncToken())
          continue; // someone else already manages it
        builder.setInsertionPoint(launch);
        llvm::SmallVector<mlir::Value> deps(launch.getAsyncDependencies());
        if (last)
          deps.push_back(last);
        auto chained = builder.create<gpu_runtime::LaunchGpuKernelOp>(
            launch.getLoc(), tokenType, deps, launch.getQueue(),
            launch.getKernel(), launch.getGridSize(), launch.getBlockSize(),
            launch.getKernelOperands());
        last = chained.getAsyncToken();
        llvm::append_range(written, launch.getKernelOperands());
        launch.erase();
        continue;
      }
      if (readsOnHost(op, written))
        flush(&op);
    }
  }
};

// gpu.wait [tokens] -> gpuxWait(queue, t); gpuxDestroyEvent(queue, t) for each
// token.  Sits beside ConvertGpuKernelLaunchPattern
// (GpuRuntimeToLlvm.cpp:444-628) and uses its call builders; the queue is the
// one of the launch that produced the token.
template <typename Base> struct ConvertGpuWaitPattern : public Base {
  using Base::Base;
  mlir::LogicalResult
  matchAndRewrite(mlir::gpu::WaitOp op, typename mlir::gpu::WaitOp::Adaptor adaptor,
                  mlir::ConversionPatternRewriter &rewriter) const override {
    if (op.getAsyncToken())
      return mlir::failure(); // only the blocking form is produced above
    auto loc = op.getLoc();
    for (auto [token, event] :
         llvm::zip(op.getAsyncDependencies(), adaptor.getAsyncDependencies())) {
      auto launch = token.template getDefiningOp<gpu_runtime::LaunchGpuKernelOp>();
      if (!launch)
        return mlir::failure();
      mlir::Value queue = rewriter.getRemappedValue(launch.getQueue());
      this->waitEventCallBuilder.create(loc, rewriter, {queue, event});
      this->destroyEventCallBuilder.create(loc, rewriter, {queue, event});
    }
    rewriter.eraseOp(op);
    return mlir::success();
  }
};

// ---- 2. the last workgroup finishes the reduction -----------------------------
// Replaces the body of LowerGPUGlobalReduce::matchAndRewrite from the
// allocation on (GpuToGpuRuntime.cpp:2187-2277); `neutral` is what
// getNeutralValue() returned for the reduction region.
//
// Ordering.  The partial of a workgroup must be visible device-wide before
// its ticket is, and the last workgroup must not read partials it fetched
// before it drew the last ticket: an agent-scope release fence ahead of the
// increment and an agent-scope acquire fence behind the last draw (LLVM
// dialect fences, which pass through the ROCDL tail unchanged and become
// buffer_wbl2 / buffer_inv around the global_atomic_add).

// Workgroup (bx, by, bz) of a (gx, gy, gz) grid -> bx + gx * (by + gy * bz).
inline mlir::Value linearGroupId(mlir::OpBuilder &b, mlir::Location loc,
                                 const mlir::gpu::KernelDim3 &grid,
                                 const mlir::gpu::KernelDim3 &id) {
  mlir::Value yz = b.create<mlir::arith::AddIOp>(
      loc, id.y, b.create<mlir::arith::MulIOp>(loc, grid.y, id.z));
  return b.create<mlir::arith::AddIOp>(loc, id.x,
                                       b.create<mlir::arith::MulIOp>(loc, grid.x, yz));
}

// True in the work-item whose three local ids are all zero.
inline mlir::Value isFirstItem(mlir::OpBuilder &b, mlir::Location loc,
                               const mlir::gpu::KernelDim3 &tid) {
  mlir::Value zero = b.create<mlir::arith::ConstantIndexOp>(loc, 0);
  mlir::Value any = b.create<mlir::arith::OrIOp>(
      loc, tid.x, b.create<mlir::arith::OrIOp>(loc, tid.y, tid.z));
  return b.create<mlir::arith::CmpIOp>(loc, mlir::arith::CmpIPredicate::eq, any, zero);
}

// acc (x) value by a clone of the reduction block `body` (two arguments, a
// gpu.yield of the combined value), placed at b's insertion point.
inline mlir::Value combineBy(mlir::OpBuilder &b, mlir::Block &body, mlir::Value acc,
                             mlir::Value value) {
  mlir::IRMapping map;
  map.map(body.getArgument(0), acc);
  map.map(body.getArgument(1), value);
  for (mlir::Operation &inner : body.without_terminator())
    b.clone(inner, map);
  auto yield = mlir::cast<mlir::gpu::YieldOp>(body.getTerminator());
  return map.lookupOrDefault(yield.getValues().front());
}

inline void finishOnDevice(mlir::PatternRewriter &rewriter, mlir::gpu::LaunchOp launch,
                           gpu_runtime::GPUGlobalReduceOp op, mlir::TypedAttr neutral) {
  auto loc = op.getLoc();
  auto launchLoc = launch.getLoc();
  auto elemType = op.getValue().getType();
  auto i32 = rewriter.getI32Type();
  mlir::OpBuilder::InsertionGuard g(rewriter);

  // Before the launch: device arrays for the partials and the ticket.
  rewriter.setInsertionPoint(launch);
  mlir::Value groups = rewriter.create<mlir::arith::MulIOp>(
      launchLoc,
      rewriter.create<mlir::arith::MulIOp>(launchLoc, launch.getGridSizeX(),
                                           launch.getGridSizeY()),
      launch.getGridSizeZ());
  auto partialsType = mlir::MemRefType::get({mlir::ShapedType::kDynamic}, elemType);
  auto ticketType = mlir::MemRefType::get({1}, i32);
  mlir::Value partials =
      rewriter
          .create<mlir::gpu::AllocOp>(launchLoc, partialsType, /*asyncToken*/ nullptr,
                                      /*asyncDeps*/ std::nullopt, groups,
                                      /*symbols*/ std::nullopt, /*hostShared*/ false)
          .getMemref();
  mlir::Value ticket =
      rewriter
          .create<mlir::gpu::AllocOp>(launchLoc, ticketType, nullptr, std::nullopt,
                                      std::nullopt, std::nullopt, false)
          .getMemref();
  rewriter.create<mlir::gpu::MemsetOp>(
      launchLoc, mlir::Type(), mlir::ValueRange(), ticket,
      rewriter.create<mlir::arith::ConstantIntOp>(launchLoc, 0, i32));

  // Inside the launch, in place of the global reduce: the workgroup's own
  // reduction with the op's region as its body (2200-2215).
  rewriter.setInsertionPoint(op);
  auto inGroup = rewriter.create<mlir::gpu::AllReduceOp>(
      loc, op.getValue(), mlir::gpu::AllReduceOperationAttr{}, /*uniform*/ true);
  auto &region = inGroup.getRegion();
  rewriter.inlineRegionBefore(op.getRegion(), region, region.end());
  mlir::Block &body = region.front();
  {
    mlir::OpBuilder::InsertionGuard g1(rewriter);
    auto term = mlir::cast<gpu_runtime::GPUGlobalReduceYieldOp>(body.getTerminator());
    rewriter.setInsertionPoint(term);
    rewriter.replaceOpWithNewOp<mlir::gpu::YieldOp>(term, term.getResult());
  }

  mlir::Value zero = rewriter.create<mlir::arith::ConstantIndexOp>(loc, 0);
  mlir::Value one = rewriter.create<mlir::arith::ConstantIndexOp>(loc, 1);
  mlir::Value gid = linearGroupId(rewriter, loc, launch.getGridSize(), launch.getBlockIds());
  mlir::Value first = isFirstItem(rewriter, loc, launch.getThreadIds());

  // One work-item a workgroup publishes the partial and draws a ticket.
  auto ifFirst = rewriter.create<mlir::scf::IfOp>(loc, first, /*withElse*/ false);
  rewriter.setInsertionPointToStart(ifFirst.thenBlock());
  rewriter.create<mlir::memref::StoreOp>(loc, inGroup.getResult(), partials, gid);
  rewriter.create<mlir::LLVM::FenceOp>(loc, mlir::LLVM::AtomicOrdering::release, "agent");
  mlir::Value taken = rewriter.create<mlir::memref::AtomicRMWOp>(
      loc, mlir::arith::AtomicRMWKind::addi,
      rewriter.create<mlir::arith::ConstantIntOp>(loc, 1, i32), ticket,
      mlir::ValueRange(zero));
  mlir::Value lastGroup = rewriter.create<mlir::arith::CmpIOp>(
      loc, mlir::arith::CmpIPredicate::eq,
      rewriter.create<mlir::arith::IndexCastOp>(loc, rewriter.getIndexType(), taken),
      rewriter.create<mlir::arith::SubIOp>(loc, groups, one));

  // The workgroup that drew the last ticket: every other one has published.
  auto ifLast = rewriter.create<mlir::scf::IfOp>(loc, lastGroup, /*withElse*/ false);
  rewriter.setInsertionPointToStart(ifLast.thenBlock());
  rewriter.create<mlir::LLVM::FenceOp>(loc, mlir::LLVM::AtomicOrdering::acquire, "agent");
  mlir::Value init = rewriter.create<mlir::arith::ConstantOp>(loc, neutral);
  auto fold = rewriter.create<mlir::scf::ForOp>(
      loc, zero, groups, one, mlir::ValueRange(init),
      [&](mlir::OpBuilder &b, mlir::Location l, mlir::Value i, mlir::ValueRange acc) {
        mlir::Value p = b.create<mlir::memref::LoadOp>(l, partials, i);
        b.create<mlir::scf::YieldOp>(l, combineBy(b, body, acc.front(), p));
      });
  rewriter.create<mlir::memref::StoreOp>(loc, fold.getResult(0), op.getTarget(),
                                         mlir::ValueRange());

  // After the launch: the two device arrays are released (in-order queue: no
  // wait needed before gpu.dealloc); the host loop of 2240-2270 is gone.
  rewriter.setInsertionPointAfter(launch);
  rewriter.create<mlir::gpu::DeallocOp>(launchLoc, mlir::Type(), mlir::ValueRange(), partials);
  rewriter.create<mlir::gpu::DeallocOp>(launchLoc, mlir::Type(), mlir::ValueRange(), ticket);
  rewriter.eraseOp(op);
}

} // namespace hip_async
