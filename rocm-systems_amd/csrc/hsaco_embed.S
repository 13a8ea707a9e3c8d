/* Links the gfx950 code object into the library as read-only data (the
 * reference turns its shader binaries into a C array with xxd,
 * blit_shaders/create_blit_shader_header.sh:44-77).  HSACO_PATH is given on
 * the command line. */
    .section .rodata
    .balign 4096
    .global mi355_blit_hsaco
    .global mi355_blit_hsaco_end
mi355_blit_hsaco:
    .incbin HSACO_PATH
mi355_blit_hsaco_end:
    .section .note.GNU-stack,"",@progbits
