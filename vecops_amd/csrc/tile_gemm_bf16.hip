// bf16 x bf16 tile GEMM instances.
#include "tile_gemm_launch.h"
namespace vecops_hip {
hipError_t launch_tile_gemm_bf16(const TileGemmParams& p, int tile_m, int tile_n, int mode, hipStream_t stream) {
  return launch_tile_class<SRC_BF16>(p, tile_m, tile_n, mode, stream);
}
}  // namespace vecops_hip
