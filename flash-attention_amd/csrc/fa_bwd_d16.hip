#define FA_HEAD_DIM 16
#include "fa_bwd_inst.inc"
