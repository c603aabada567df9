// placeholder until the LDS-tiled family lands
#include "common.hpp"
namespace moe_i8 {
bool gemm_tile_supports(const GemmArgs&) { return false; }
hipError_t launch_gemm_tile(const GemmArgs&, hipStream_t) { return hipErrorNotSupported; }
}  // namespace moe_i8
