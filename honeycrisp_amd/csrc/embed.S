/* Embeds the gfx950 code objects (built by `hipcc --genco`, see build.py) into libhchip.so
 * as read-only data; hchip.cpp hands them to hipModuleLoadData. The assembler's include
 * path (-Wa,-I) points at the directory holding the .hsaco files. */
    .section .rodata
    .macro EMBED sym, file
    .balign 4096
    .global \sym
    .type \sym, @object
\sym:
    .incbin "\file"
    .global \sym\()_end
\sym\()_end:
    .byte 0
    .endm

    EMBED hc_image_elementwise, "elementwise.hsaco"
    EMBED hc_image_reduce, "reduce.hsaco"
    EMBED hc_image_gather, "gather.hsaco"
    EMBED hc_image_scan, "scan.hsaco"
    EMBED hc_image_attention, "attention.hsaco"
    EMBED hc_image_gemm, "gemm.hsaco"
    EMBED hc_image_gemm_f16_fast, "gemm_f16_fast.hsaco"
    EMBED hc_image_gemm_dma, "gemm_dma.hsaco"
    EMBED hc_image_gemm_dma2, "gemm_dma2.hsaco"
    EMBED hc_image_gemm_mi16, "gemm_mi16.hsaco"
    EMBED hc_image_gemm_dma_m, "gemm_dma_m.hsaco"
    EMBED hc_image_gemm_dma2_m_f16, "gemm_dma2_m_f16.hsaco"
    EMBED hc_image_gemm_dma2_m_f32, "gemm_dma2_m_f32.hsaco"
    EMBED hc_image_gemm_mi16_m, "gemm_mi16_m.hsaco"

    .section .note.GNU-stack,"",@progbits
