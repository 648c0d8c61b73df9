#define FA_HEAD_DIM 64
#include "fa_bwd_inst.inc"
