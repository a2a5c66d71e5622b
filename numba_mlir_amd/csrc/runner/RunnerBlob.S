// Embeds the gfx950 code object of the runner's kernels into the runner.
// The assembler finds it through -Wa,-I<build dir>.
	.section .rodata
	.balign 4096
	.global hip_runner_blob
	.global hip_runner_blob_end
hip_runner_blob:
	.incbin "runner_kernels.hsaco"
hip_runner_blob_end:
	.section .note.GNU-stack,"",@progbits
