/* Embeds the gfx950 code object into libmaize_hip.so. */
    .section .rodata
    .balign 4096
    .global maize_embedded_hsaco
    .type maize_embedded_hsaco, @object
maize_embedded_hsaco:
    .incbin MAIZE_HSACO_PATH
    .global maize_embedded_hsaco_end
    .type maize_embedded_hsaco_end, @object
maize_embedded_hsaco_end:
    .byte 0
    .size maize_embedded_hsaco, maize_embedded_hsaco_end - maize_embedded_hsaco
    .section .note.GNU-stack,"",@progbits
