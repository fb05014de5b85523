// fp32 operands multiplied in fp32 (v_mfma_f32_32x32x2_f32): tile GEMM instances.
#include "tile_gemm_launch.h"
namespace vecops_hip {
hipError_t launch_tile_gemm_f32(const TileGemmParams& p, int tile_m, int tile_n, int mode, hipStream_t stream) {
  return launch_tile_class<SRC_F32>(p, tile_m, tile_n, mode, stream);
}
}  // namespace vecops_hip
