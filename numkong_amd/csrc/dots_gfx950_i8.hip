/**
 *  @brief The i8 product kernels of the gfx950 backend, every tile shape.
 *  @file numkong_amd/csrc/dots_gfx950_i8.hip
 */
#include "dots_gfx950.hpp"

namespace nk_gfx950 {
hipError_t launch_i8(GemmArgs &g, hipStream_t stream, TriangleScratch const *triangle) {
    return launch_typed<I8>(g, stream, triangle);
}
} // namespace nk_gfx950

#ifdef NK_TUNE // the clocks the instrumented i8 kernel of a tuning build leaves behind
extern "C" __attribute__((visibility("default"))) void nk_hip_debug_clocks(unsigned long long *out) {
    (void)hipMemcpyFromSymbol(out, HIP_SYMBOL(g_debug_clocks), sizeof(unsigned long long) * 8);
}
#endif
