/* Embeds a device-only gfx950 code object into the host library, so that the shared object
 * is self-contained: hipModuleLoadData reads it from here.  Assembled once per code object
 * with NBO_CODE_OBJECT_PATH and NBO_CODE_OBJECT_SYMBOL set. */
    .section .rodata
    .global NBO_CODE_OBJECT_SYMBOL
    .balign 4096
NBO_CODE_OBJECT_SYMBOL:
    .incbin NBO_CODE_OBJECT_PATH
    .byte 0
    .section .note.GNU-stack,"",@progbits
