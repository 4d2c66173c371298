// The operator kernels as plain gfx950 code objects (built from the same ops_*.hip sources with
// --cuda-device-only), embedded for the HSA loader used by direct dispatch.  PAELLA_HSACO_DIR is set by the
// build to the directory that holds them.
#define PAELLA_STR2(x) #x
#define PAELLA_STR(x) PAELLA_STR2(x)

__asm__(
    ".section .rodata\n"
    ".balign 4096\n"
    ".global paella_hsaco_conv_begin\n"
    "paella_hsaco_conv_begin:\n"
    ".incbin \"" PAELLA_STR(PAELLA_HSACO_DIR) "/ops_conv.hsaco\"\n"
    ".global paella_hsaco_conv_end\n"
    "paella_hsaco_conv_end:\n"
    ".balign 4096\n"
    ".global paella_hsaco_misc_begin\n"
    "paella_hsaco_misc_begin:\n"
    ".incbin \"" PAELLA_STR(PAELLA_HSACO_DIR) "/ops_misc.hsaco\"\n"
    ".global paella_hsaco_misc_end\n"
    "paella_hsaco_misc_end:\n"
    ".previous\n");
