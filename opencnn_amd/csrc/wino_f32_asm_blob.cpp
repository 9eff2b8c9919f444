// The assembled code object of the hand-scheduled fused kernels (gen_wino_f32_asm.py ->
// wino_f32_asm.s -> wino_f32_asm.hsaco), embedded in the library as a byte array.
// Host-only translation unit: a file-scope asm in a HIP source would also reach the device pass.
asm(".section .rodata\n"
    ".balign 4096\n"
    ".global opencnn_wino_f32_asm_hsaco\n"
    ".hidden opencnn_wino_f32_asm_hsaco\n"
    "opencnn_wino_f32_asm_hsaco:\n"
    ".incbin \"wino_f32_asm.hsaco\"\n"
    ".global opencnn_wino_f32_asm_hsaco_end\n"
    ".hidden opencnn_wino_f32_asm_hsaco_end\n"
    "opencnn_wino_f32_asm_hsaco_end:\n"
    ".byte 0\n"
    ".previous\n");
