// Prepacked-B tile GEMM instances: bf16 operands.
#include "tile_gemm_packed_launch.h"
namespace vecops_hip {
hipError_t launch_packed_bf16(const TileGemmParams& p, int tile_m, int tile_n, int vector_a, hipStream_t stream) {
  return launch_packed_class<SRC_BF16>(p, tile_m, tile_n, vector_a, stream);
}
}  // namespace vecops_hip
