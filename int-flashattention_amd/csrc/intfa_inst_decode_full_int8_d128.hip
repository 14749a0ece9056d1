#define INTFA_INST_D 128
#include "intfa_inst_decode.inc"
