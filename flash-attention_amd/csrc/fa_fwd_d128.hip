#define FA_HEAD_DIM 128
#include "fa_fwd_inst.inc"
