/**
 *  @brief The e2m3 product kernels of the gfx950 backend, every tile shape.
 *  @file numkong_amd/csrc/dots_gfx950_e2m3.hip
 */
#include "dots_gfx950.hpp"

namespace nk_gfx950 {
hipError_t launch_e2m3(GemmArgs &g, hipStream_t stream, TriangleScratch const *triangle) {
    return launch_typed<E2M3>(g, stream, triangle);
}
} // namespace nk_gfx950
