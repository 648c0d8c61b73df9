#define FA_HEAD_DIM 128
#include "fa_bwd_inst.inc"
