// int8 x int8 -> int32 tile GEMM instances and the split-K reduction kernels.
#include "tile_gemm_launch.h"
namespace vecops_hip {
hipError_t launch_tile_gemm_i8(const TileGemmParams& p, int tile_m, int tile_n, int mode, hipStream_t stream) {
  return launch_tile_class<SRC_I8>(p, tile_m, tile_n, mode, stream);
}

hipError_t launch_splitk_reduce(const TileGemmParams& p, bool is_int, hipStream_t stream) {
  const int64_t total = static_cast<int64_t>(p.m) * p.n * p.batch;
  int64_t blocks = (total + 255) / 256;
  if (blocks > 256 * 16) blocks = 256 * 16;
  if (blocks < 1) blocks = 1;
  if (is_int)
    hipLaunchKernelGGL(splitk_reduce_kernel<true>, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, p);
  else
    hipLaunchKernelGGL(splitk_reduce_kernel<false>, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, p);
  return hipGetLastError();
}
}  // namespace vecops_hip
