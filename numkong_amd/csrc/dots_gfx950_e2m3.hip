/**
 *  @brief The e2m3 product kernels of the gfx950 backend, every tile shape.
 *  @file numkong_amd/csrc/dots_gfx950_e2m3.hip
 */
#include "dots_gfx950.hpp"

namespace nk_gfx950 {
hipError_t launch_e2m3(GemmArgs &g, hipStream_t stream, TriangleScratch const *triangle) {
    // (rows too deep for exact i32 sums of the integer route run as f16)
    return e2m3_as_integers(g.k) ? launch_typed<E2M3>(g, stream, triangle) : launch_typed<E2M3Deep>(g, stream, triangle);
}
} // namespace nk_gfx950
