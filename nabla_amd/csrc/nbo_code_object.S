/* Embeds the device-only gfx950 code object into the host library, so that the
 * shared object is self-contained: hipModuleLoadData reads it from here. */
    .section .rodata
    .global nbo_code_object
    .global nbo_code_object_end
    .balign 4096
nbo_code_object:
    .incbin NBO_CODE_OBJECT_PATH
nbo_code_object_end:
    .byte 0
    .section .note.GNU-stack,"",@progbits
