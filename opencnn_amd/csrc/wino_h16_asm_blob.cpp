// The assembled code object of the hand-scheduled fp16 / bf16 fused kernels
// (gen_wino_h16_asm.py -> wino_h16_asm.s -> wino_h16_asm.hsaco), embedded in the library as a
// byte array.  Host-only translation unit, like wino_f32_asm_blob.cpp.
asm(".section .rodata\n"
    ".balign 4096\n"
    ".global opencnn_wino_h16_asm_hsaco\n"
    ".hidden opencnn_wino_h16_asm_hsaco\n"
    "opencnn_wino_h16_asm_hsaco:\n"
    ".incbin \"wino_h16_asm.hsaco\"\n"
    ".global opencnn_wino_h16_asm_hsaco_end\n"
    ".hidden opencnn_wino_h16_asm_hsaco_end\n"
    "opencnn_wino_h16_asm_hsaco_end:\n"
    ".byte 0\n"
    ".previous\n");
