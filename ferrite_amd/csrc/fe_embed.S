/* The gfx950 code objects, linked into the library as read-only data (the reference embeds its cubins with
 * include_bytes!, crates/fe-exl3/src/gpu/mod.rs:12-13). Paths are relative to the build directory. */
    .section .rodata
    .balign 4096
    .global fe_k_exl3_hsaco
fe_k_exl3_hsaco:
    .incbin "k_exl3.hsaco"
    .global fe_k_exl3_hsaco_end
fe_k_exl3_hsaco_end:
    .balign 4096
    .global fe_k_fp4_hsaco
fe_k_fp4_hsaco:
    .incbin "k_fp4.hsaco"
    .global fe_k_fp4_hsaco_end
fe_k_fp4_hsaco_end:
    .balign 4096
    .global fe_k_route_hsaco
fe_k_route_hsaco:
    .incbin "k_route.hsaco"
    .global fe_k_route_hsaco_end
fe_k_route_hsaco_end:
    .balign 4096
    .global fe_k_bf16_hsaco
fe_k_bf16_hsaco:
    .incbin "k_bf16.hsaco"
    .global fe_k_bf16_hsaco_end
fe_k_bf16_hsaco_end:
    .section .note.GNU-stack,"",@progbits
