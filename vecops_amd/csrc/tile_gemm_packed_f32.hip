// Prepacked-B tile GEMM instances: fp32 operands (rounded to bf16 on load, or multiplied in fp32).
#include "tile_gemm_packed_launch.h"
namespace vecops_hip {
hipError_t launch_packed_f32_as_bf16(const TileGemmParams& p, int tile_m, int tile_n, int vector_a, hipStream_t stream) {
  return launch_packed_class<SRC_F32_AS_BF16>(p, tile_m, tile_n, vector_a, stream);
}
hipError_t launch_packed_f32(const TileGemmParams& p, int tile_m, int tile_n, int vector_a, hipStream_t stream) {
  return launch_packed_class<SRC_F32>(p, tile_m, tile_n, vector_a, stream);
}
}  // namespace vecops_hip
