; @foo of mlir/test/L0_RUNNER/linalg_test_f32.mlir:7-123 (and _f64) with its
; one-op linalg.generic steps fused into one parallel loop over the 500
; elements, that loop mapped to blocks of one work-item (the runner's
; pipeline, mlir/tools/level_zero_runner/LevelZeroRunner.cpp:39-104), after
; convert-gpu-to-rocdl: math.exp is a call into the device library, every
; arithmetic op stays an op of its own (no contraction).
;   v11 = s0 + s1; v13 = s4 - s3; v15 = -s2
;   t19 = a - s0; t27 = exp(v15 * t19) + a; t35 = s3 + v13 / t27
;   out = v11 + t35 * (a - s0)
define amdgpu_kernel void @foo_kernel_f32(ptr %a, ptr %s, ptr %out) #0 {
  %bx32 = call i32 @llvm.amdgcn.workgroup.id.x()
  %i = sext i32 %bx32 to i64
  %s1p = getelementptr float, ptr %s, i64 1
  %s2p = getelementptr float, ptr %s, i64 2
  %s3p = getelementptr float, ptr %s, i64 3
  %s4p = getelementptr float, ptr %s, i64 4
  %s0 = load float, ptr %s, align 4
  %s1 = load float, ptr %s1p, align 4
  %s2 = load float, ptr %s2p, align 4
  %s3 = load float, ptr %s3p, align 4
  %s4 = load float, ptr %s4p, align 4
  %pa = getelementptr float, ptr %a, i64 %i
  %x = load float, ptr %pa, align 4
  %v11 = fadd float %s0, %s1
  %v13 = fsub float %s4, %s3
  %v15 = fneg float %s2
  %t19 = fsub float %x, %s0
  %t21 = fmul float %v15, %t19
  %t23 = call float @__ocml_exp_f32(float %t21)
  %t27 = fadd float %t23, %x
  %t31 = fdiv float %v13, %t27
  %t35 = fadd float %s3, %t31
  %t39 = fsub float %x, %s0
  %t41 = fmul float %t35, %t39
  %r = fadd float %v11, %t41
  %po = getelementptr float, ptr %out, i64 %i
  store float %r, ptr %po, align 4
  ret void
}

define amdgpu_kernel void @foo_kernel_f64(ptr %a, ptr %s, ptr %out) #0 {
  %bx32 = call i32 @llvm.amdgcn.workgroup.id.x()
  %i = sext i32 %bx32 to i64
  %s1p = getelementptr double, ptr %s, i64 1
  %s2p = getelementptr double, ptr %s, i64 2
  %s3p = getelementptr double, ptr %s, i64 3
  %s4p = getelementptr double, ptr %s, i64 4
  %s0 = load double, ptr %s, align 8
  %s1 = load double, ptr %s1p, align 8
  %s2 = load double, ptr %s2p, align 8
  %s3 = load double, ptr %s3p, align 8
  %s4 = load double, ptr %s4p, align 8
  %pa = getelementptr double, ptr %a, i64 %i
  %x = load double, ptr %pa, align 8
  %v11 = fadd double %s0, %s1
  %v13 = fsub double %s4, %s3
  %v15 = fneg double %s2
  %t19 = fsub double %x, %s0
  %t21 = fmul double %v15, %t19
  %t23 = call double @__ocml_exp_f64(double %t21)
  %t27 = fadd double %t23, %x
  %t31 = fdiv double %v13, %t27
  %t35 = fadd double %s3, %t31
  %t39 = fsub double %x, %s0
  %t41 = fmul double %t35, %t39
  %r = fadd double %v11, %t41
  %po = getelementptr double, ptr %out, i64 %i
  store double %r, ptr %po, align 8
  ret void
}

declare i32 @llvm.amdgcn.workgroup.id.x()
declare float @__ocml_exp_f32(float)
declare double @__ocml_exp_f64(double)

attributes #0 = { "amdgpu-flat-work-group-size"="1,1" "uniform-work-group-size"="true" }
