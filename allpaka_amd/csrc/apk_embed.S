/* Embeds the gfx950 code object built from apk_kernels.hip into libapk_hip.so;
 * the host loads it with hipModuleLoadData(apk_kernels_co). */
    .section .rodata
    .global apk_kernels_co
    .global apk_kernels_co_end
    .balign 4096
apk_kernels_co:
    .incbin "apk_kernels.hsaco"
apk_kernels_co_end:
    .byte 0
    .section .note.GNU-stack,"",@progbits
