/* Embeds the gfx950 code object into the shared library's read-only data. */
    .section .rodata
    .balign 4096
    .global cogni_hsaco_begin
    .type cogni_hsaco_begin, @object
cogni_hsaco_begin:
    .incbin HSACO_PATH
    .global cogni_hsaco_end
    .type cogni_hsaco_end, @object
cogni_hsaco_end:
    .byte 0
    .section .note.GNU-stack,"",@progbits
