// Prepacked-B tile GEMM instances: half operands.
#include "tile_gemm_packed_launch.h"
namespace vecops_hip {
hipError_t launch_packed_f16(const TileGemmParams& p, int tile_m, int tile_n, int vector_a, hipStream_t stream) {
  return launch_packed_class<SRC_F16>(p, tile_m, tile_n, vector_a, stream);
}
}  // namespace vecops_hip
