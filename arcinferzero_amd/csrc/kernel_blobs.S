/* The gfx950 code objects, one per kernel module, as read-only data of the host library
   (found through the assembler's include path: the build directory). */
    .section .rodata
    .macro BLOB name, file
    .balign 4096
    .global \name
\name:
    .incbin "\file"
    .balign 8
    .endm
    BLOB arcz_blob_ops, "ops.hsaco"
    BLOB arcz_blob_decode, "decode.hsaco"
    BLOB arcz_blob_decode_q80, "decode_q80.hsaco"
    BLOB arcz_blob_decode_q40, "decode_q40.hsaco"
    BLOB arcz_blob_decode_q4k, "decode_q4k.hsaco"
    BLOB arcz_blob_decode_q5k, "decode_q5k.hsaco"
    BLOB arcz_blob_decode_q6k, "decode_q6k.hsaco"
    BLOB arcz_blob_decode_iq4xs, "decode_iq4xs.hsaco"
    BLOB arcz_blob_decode_iq3s, "decode_iq3s.hsaco"
    BLOB arcz_blob_decode_iq4nl, "decode_iq4nl.hsaco"
    BLOB arcz_blob_decode_mxfp4, "decode_mxfp4.hsaco"
    BLOB arcz_blob_decode_q3k, "decode_q3k.hsaco"
    BLOB arcz_blob_decode_iq3xxs, "decode_iq3xxs.hsaco"
    BLOB arcz_blob_decode_mm, "decode_mm.hsaco"
    BLOB arcz_blob_gemm, "gemm.hsaco"
    BLOB arcz_blob_moe, "moe.hsaco"
    .section .note.GNU-stack,"",@progbits
