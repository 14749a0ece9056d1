#define INTFA_INST_D 64
#define INTFA_INST_VBLK 2
#include "intfa_inst_full_int8.inc"
