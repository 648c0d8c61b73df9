#define FA_HEAD_DIM 64
#include "fa_fwd_inst.inc"
