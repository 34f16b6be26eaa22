/**
 *  @brief The e3m2 product kernels of the gfx950 backend, every tile shape.
 *  @file numkong_amd/csrc/dots_gfx950_e3m2.hip
 */
#include "dots_gfx950.hpp"

namespace nk_gfx950 {
hipError_t launch_e3m2(GemmArgs &g, hipStream_t stream, TriangleScratch const *triangle) {
    return launch_typed<E3M2>(g, stream, triangle);
}
} // namespace nk_gfx950
