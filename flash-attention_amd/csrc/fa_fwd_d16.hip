#define FA_HEAD_DIM 16
#include "fa_fwd_inst.inc"
