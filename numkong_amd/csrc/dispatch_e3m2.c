/**
 *  @brief Dispatch for the E3M2 kinds: binds the table slots and `nk_find_kernel_punned` to gfx950.
 *  @file numkong_amd/csrc/dispatch_e3m2.c
 *
 *  Counterpart of the reference's c/dispatch_e3m2.c (`nk_dispatch_e3m2_find_`, `nk_dispatch_e3m2_init_`), for the kinds
 *  this backend serves: the packed dots (size, pack, product), the packed distances and the symmetric kinds.
 */
#include "dispatch.h"

NK_AMD_DEFINE_DISPATCH_(e3m2)
