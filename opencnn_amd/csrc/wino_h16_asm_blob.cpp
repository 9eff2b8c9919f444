// The assembled code object of the hand-scheduled fp16 / bf16 fused kernels
// (gen_wino_h16_asm.py -> wino_h16_asm.s -> wino_h16_asm.hsaco), embedded in the library as a
// byte array.  Host-only translation unit, like wino_f32_asm_blob.cpp.
#ifndef OPENCNN_H16_HSACO
#define OPENCNN_H16_HSACO "wino_h16_asm.hsaco"  // (make diagnostic embeds other builds of the same kernels)
#endif
asm(".section .rodata\n"
    ".balign 4096\n"
    ".global opencnn_wino_h16_asm_hsaco\n"
    ".hidden opencnn_wino_h16_asm_hsaco\n"
    "opencnn_wino_h16_asm_hsaco:\n"
    ".incbin \"" OPENCNN_H16_HSACO "\"\n"
    ".global opencnn_wino_h16_asm_hsaco_end\n"
    ".hidden opencnn_wino_h16_asm_hsaco_end\n"
    "opencnn_wino_h16_asm_hsaco_end:\n"
    ".byte 0\n"
    ".previous\n");
