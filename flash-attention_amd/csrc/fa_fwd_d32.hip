#define FA_HEAD_DIM 32
#include "fa_fwd_inst.inc"
