/* Places each compiled gfx950 code object in .rodata between a start and an
 * end symbol.  Assembled with -I <directory holding the .hsaco files>. */
    .macro ROCK_BLOB n
    .global rock_hsaco_\n\()_start
    .global rock_hsaco_\n\()_end
    .balign 4096
rock_hsaco_\n\()_start:
    .incbin "\n\().hsaco"
rock_hsaco_\n\()_end:
    .byte 0
    .endm

    .section .rodata
    ROCK_BLOB gemm_f32
    ROCK_BLOB gemm_f16
    ROCK_BLOB gemm_bf16
    ROCK_BLOB gemm_i8
    ROCK_BLOB gemm_fp8
    ROCK_BLOB gemm_bf8
    ROCK_BLOB gemm_fp8_bf8
    ROCK_BLOB gemm_bf8_fp8
    ROCK_BLOB attention
    ROCK_BLOB relayout
    ROCK_BLOB probe
    .section .note.GNU-stack,"",@progbits
