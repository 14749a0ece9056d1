#define INTFA_INST_D 64
#include "intfa_inst_decode.inc"
