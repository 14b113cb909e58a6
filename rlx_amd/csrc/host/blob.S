/* The gfx950 code objects, one per kernel source, embedded verbatim; loaded with hipModuleLoadData at first use. */
    .section .rodata
.macro blob name
    .balign 4096
    .global rlx_blob_\name
rlx_blob_\name:
    .incbin "build/\name\().co"
    .byte 0
.endm
    blob dequant
    blob fakequant
    blob gemm
    blob gemm_big
    blob gemv
    blob gemv_wide
    blob moe
    blob rowops
    blob topk
    .section .note.GNU-stack,"",@progbits
