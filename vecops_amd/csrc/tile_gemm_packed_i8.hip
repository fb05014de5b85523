// Prepacked-B tile GEMM instances: signed 8-bit operands.
#include "tile_gemm_packed_launch.h"
namespace vecops_hip {
hipError_t launch_packed_i8(const TileGemmParams& p, int tile_m, int tile_n, int vector_a, hipStream_t stream) {
  return launch_packed_class<SRC_I8>(p, tile_m, tile_n, vector_a, stream);
}
}  // namespace vecops_hip
