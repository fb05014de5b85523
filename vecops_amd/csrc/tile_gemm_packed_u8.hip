// Prepacked-B tile GEMM instances: 8-bit operands with an unsigned A.
#include "tile_gemm_packed_launch.h"
namespace vecops_hip {
hipError_t launch_packed_i8_flip(const TileGemmParams& p, int tile_m, int tile_n, int vector_a, hipStream_t stream) {
  return launch_packed_class<SRC_I8_FLIP>(p, tile_m, tile_n, vector_a, stream);
}
}  // namespace vecops_hip
