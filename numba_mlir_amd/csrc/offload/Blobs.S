// Embeds the gfx950 code objects of the kernel families into the offload
// library.  The assembler finds the .hsaco files through -Wa,-I<build dir>.
	.section .rodata
	.balign 4096
	.global nmhip_blob_maps
	.global nmhip_blob_maps_end
nmhip_blob_maps:
	.incbin "maps.hsaco"
nmhip_blob_maps_end:
	.balign 4096
	.global nmhip_blob_reduce
	.global nmhip_blob_reduce_end
nmhip_blob_reduce:
	.incbin "reduce.hsaco"
nmhip_blob_reduce_end:
	.balign 4096
	.global nmhip_blob_reduce_release
	.global nmhip_blob_reduce_release_end
nmhip_blob_reduce_release:
	.incbin "reduce_release.hsaco"
nmhip_blob_reduce_release_end:
	.balign 4096
	.global nmhip_blob_twins
	.global nmhip_blob_twins_end
nmhip_blob_twins:
	.incbin "twins.hsaco"
nmhip_blob_twins_end:
	.section .note.GNU-stack,"",@progbits
