#define INTFA_INST_D 256
#include "intfa_inst_decode.inc"
