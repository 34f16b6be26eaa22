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
