/* The gfx950 code object, embedded verbatim; loaded with hipModuleLoadData at first use. */
    .section .rodata
    .balign 4096
    .global rlx_kernels_blob
    .global rlx_kernels_blob_end
rlx_kernels_blob:
    .incbin "build/rlx_kernels.co"
rlx_kernels_blob_end:
    .byte 0
    .section .note.GNU-stack,"",@progbits
