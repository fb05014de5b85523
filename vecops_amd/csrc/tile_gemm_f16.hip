// f16 x f16 tile GEMM instances.
#include "tile_gemm_launch.h"
namespace vecops_hip {
hipError_t launch_tile_gemm_f16(const TileGemmParams& p, int tile_m, int tile_n, int mode, hipStream_t stream) {
  return launch_tile_class<SRC_F16>(p, tile_m, tile_n, mode, stream);
}
}  // namespace vecops_hip
