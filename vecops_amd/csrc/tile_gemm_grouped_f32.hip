// fp32 operands rounded to bf16 while staged: tile GEMM instances of the grouped launch.
#include "tile_gemm_launch.h"
namespace vecops_hip {
hipError_t launch_tile_gemm_grouped_f32_as_bf16(const GroupedTables& t, int tile, int mode, hipStream_t stream) {
  return launch_grouped_class<SRC_F32_AS_BF16>(t, tile, mode, stream);
}
}  // namespace vecops_hip
