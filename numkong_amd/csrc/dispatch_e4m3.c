/**
 *  @brief Dispatch for E4M3 packed dots: binds the table slots and `nk_find_kernel_punned` to gfx950.
 *  @file numkong_amd/csrc/dispatch_e4m3.c
 *
 *  Counterpart of the reference's c/dispatch_e4m3.c (`nk_dispatch_e4m3_find_`, `nk_dispatch_e4m3_init_`),
 *  for the kinds nk_kernel_dots_packed_size_k, nk_kernel_dots_pack_k, nk_kernel_dots_packed_k only.
 */
#include "dispatch.h"

NK_AMD_DEFINE_DISPATCH_(e4m3)
