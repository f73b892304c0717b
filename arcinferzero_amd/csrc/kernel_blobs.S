/* The gfx950 code objects, one per kernel module, as read-only data of the host library. */
    .section .rodata
    .macro BLOB name, file
    .balign 4096
    .global \name
\name:
    .incbin "\file"
    .balign 8
    .endm
    BLOB arcz_blob_ops, "build/ops.hsaco"
    BLOB arcz_blob_decode, "build/decode.hsaco"
    BLOB arcz_blob_decode_q80, "build/decode_q80.hsaco"
    BLOB arcz_blob_decode_q4k, "build/decode_q4k.hsaco"
    BLOB arcz_blob_decode_q6k, "build/decode_q6k.hsaco"
    BLOB arcz_blob_gemm, "build/gemm.hsaco"
    BLOB arcz_blob_moe, "build/moe.hsaco"
    .section .note.GNU-stack,"",@progbits
