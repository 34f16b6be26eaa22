/**
 *  @brief Dispatch for the F32 kinds: binds the table slots and `nk_find_kernel_punned` to gfx950.
 *  @file numkong_amd/csrc/dispatch_f32.c
 *
 *  Counterpart of the reference's c/dispatch_f32.c (`nk_dispatch_f32_find_`, `nk_dispatch_f32_init_`), for the kinds
 *  this backend serves: the packed dots (size, pack, product), the packed distances and the symmetric kinds.
 */
#include "dispatch.h"

NK_AMD_DEFINE_DISPATCH_WIDE_(f32)
