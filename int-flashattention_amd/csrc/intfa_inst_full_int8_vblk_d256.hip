#define INTFA_INST_D 256
#define INTFA_INST_VBLK 1
#include "intfa_inst_full_int8.inc"
