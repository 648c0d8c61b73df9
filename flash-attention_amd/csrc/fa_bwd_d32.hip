#define FA_HEAD_DIM 32
#include "fa_bwd_inst.inc"
