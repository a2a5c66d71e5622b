; A kernel with a workgroup-memory argument and a barrier, as the ROCDL
; lowering gives it for the HIP runtime: the memref in workgroup memory that
; the reference passes as a ptr param with no data
; (mlir/lib/Conversion/GpuRuntimeToLlvm.cpp:507-536) arrives as a byte offset
; into the launch's dynamic LDS block.  Each work-item puts its element into
; workgroup memory; after the barrier, work-item 0 adds the group's elements
; in index order and stores the sum for its group.
@__dynamic_shmem = external addrspace(3) global [0 x i8], align 16

define amdgpu_kernel void @group_sum_f32(ptr %in, ptr %out, i64 %scratch_offset) #0 {
entry:
  %tid = call i32 @llvm.amdgcn.workitem.id.x()
  %bid = call i32 @llvm.amdgcn.workgroup.id.x()
  %tid64 = zext i32 %tid to i64
  %bid64 = zext i32 %bid to i64
  %first = mul i64 %bid64, 256
  %gi = add i64 %first, %tid64
  %pin = getelementptr float, ptr %in, i64 %gi
  %v = load float, ptr %pin, align 4
  %off = trunc i64 %scratch_offset to i32
  %scratch = getelementptr i8, ptr addrspace(3) @__dynamic_shmem, i32 %off
  %slot = getelementptr float, ptr addrspace(3) %scratch, i32 %tid
  store float %v, ptr addrspace(3) %slot, align 4
  fence syncscope("workgroup") release
  call void @llvm.amdgcn.s.barrier()
  fence syncscope("workgroup") acquire
  %leader = icmp eq i32 %tid, 0
  br i1 %leader, label %loop, label %done

loop:
  %k = phi i32 [ 0, %entry ], [ %k1, %loop ]
  %acc = phi float [ 0.0, %entry ], [ %acc1, %loop ]
  %pk = getelementptr float, ptr addrspace(3) %scratch, i32 %k
  %x = load float, ptr addrspace(3) %pk, align 4
  %acc1 = fadd float %acc, %x
  %k1 = add i32 %k, 1
  %more = icmp ult i32 %k1, 256
  br i1 %more, label %loop, label %store

store:
  %po = getelementptr float, ptr %out, i64 %bid64
  store float %acc1, ptr %po, align 4
  br label %done

done:
  ret void
}

declare i32 @llvm.amdgcn.workitem.id.x()
declare i32 @llvm.amdgcn.workgroup.id.x()
declare void @llvm.amdgcn.s.barrier()

attributes #0 = { "amdgpu-flat-work-group-size"="256,256" "uniform-work-group-size"="true" }
