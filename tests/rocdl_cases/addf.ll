; The gpu.module of mlir/test/L0_RUNNER/addf.mlir:21-28 after gpu outlining,
; bare-pointer kernel arguments and convert-gpu-to-rocdl, as LLVM IR:
; gpu.launch blocks (8,1,1) threads (1,1,1), c[bx] = a[bx] + b[bx].
define amdgpu_kernel void @main_kernel(ptr %a, ptr %b, ptr %c) #0 {
  %bx32 = call i32 @llvm.amdgcn.workgroup.id.x()
  %bx = sext i32 %bx32 to i64
  %pa = getelementptr float, ptr %a, i64 %bx
  %pb = getelementptr float, ptr %b, i64 %bx
  %pc = getelementptr float, ptr %c, i64 %bx
  %x = load float, ptr %pa, align 4
  %y = load float, ptr %pb, align 4
  %z = fadd float %x, %y
  store float %z, ptr %pc, align 4
  ret void
}

declare i32 @llvm.amdgcn.workgroup.id.x()

attributes #0 = { "amdgpu-flat-work-group-size"="1,1" "uniform-work-group-size"="true" }
