/**
 *  @brief Dispatch for E5M2 packed dots: binds the table slots and `nk_find_kernel_punned` to gfx950.
 *  @file numkong_amd/csrc/dispatch_e5m2.c
 *
 *  Counterpart of the reference's c/dispatch_e5m2.c (`nk_dispatch_e5m2_find_`, `nk_dispatch_e5m2_init_`),
 *  for the kinds nk_kernel_dots_packed_size_k, nk_kernel_dots_pack_k, nk_kernel_dots_packed_k only.
 */
#include "dispatch.h"

NK_AMD_DEFINE_DISPATCH_(e5m2)
