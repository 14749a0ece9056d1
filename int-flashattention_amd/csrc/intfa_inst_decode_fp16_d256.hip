#define INTFA_INST_D 256
#define INTFA_INST_QK_INT8 0
#include "intfa_inst_decode_f16pv.inc"
