/* Places each compiled gfx950 code object in .rodata between a start and an
 * end symbol.  Assembled with -I <build directory>, which holds the .hsaco
 * files and blobs_list.S, the generated list of "ROCK_BLOB <kernel name>"
 * lines (one code object per kernel). */
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
#include "blobs_list.S"
    .section .note.GNU-stack,"",@progbits
