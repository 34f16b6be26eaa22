/**
 *  @brief The f16 product kernels of the gfx950 backend, every tile shape.
 *  @file numkong_amd/csrc/dots_gfx950_f16.hip
 */
#include "dots_gfx950.hpp"

namespace nk_gfx950 {
hipError_t launch_f16(GemmArgs &g, hipStream_t stream, TriangleScratch const *triangle) {
    return launch_typed<F16>(g, stream, triangle);
}
} // namespace nk_gfx950
