// Tile GEMM instances of the grouped launch for 8-bit integer operands with an unsigned side.
#include "tile_gemm_launch.h"
namespace vecops_hip {
hipError_t launch_tile_gemm_grouped_i8_flip(const GroupedTables& t, int tile, int mode, hipStream_t stream) {
  return launch_grouped_class<SRC_I8_FLIP>(t, tile, mode, stream);
}
}  // namespace vecops_hip
