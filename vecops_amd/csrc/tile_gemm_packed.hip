// Tile GEMM instances that take a prepacked B operand, and the packing kernel.
#include "tile_gemm_packed.h"

#include "tile_gemm_launch.h"
namespace vecops_hip {
namespace {

template <int SRC, int WAVES_M, int WAVES_N, int WM, int WN, int LA>
hipError_t launch_packed_instance(const TileGemmParams& p, hipStream_t stream) {
  constexpr int kStages = 2 * (32 * WAVES_M * WM) * 128;
  constexpr int kEpilogue = kEpilogueLdsBytes<WAVES_M, WAVES_N, WM, WN>();
  constexpr int kLds = kStages > kEpilogue ? kStages : kEpilogue;
  auto kernel = tile_gemm_packed_b_kernel<SRC, WAVES_M, WAVES_N, WM, WN, LA>;
  static thread_local int configured_device = -1;
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return e;
  if (configured_device != device) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
    if (e != hipSuccess) return e;
    configured_device = device;
  }
  const int64_t grid = static_cast<int64_t>(p.tiles_m) * p.tiles_n * p.batch * p.split_k;
  if (grid <= 0 || grid > INT32_MAX) return hipErrorInvalidConfiguration;
  hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(grid)), dim3(64 * WAVES_M * WAVES_N), kLds, stream, p);
  return hipGetLastError();
}

template <int SRC, int LA>
hipError_t launch_packed_tile(const TileGemmParams& p, int tile_m, int tile_n, hipStream_t stream) {
  // (for 256x256, 1 x 4 wavefronts of 256x64, which load no B fragment twice but read A from LDS twice as
  // often, measured the same as 2 x 2 of 128x128)
  if (tile_m == 256 && tile_n == 256) return launch_packed_instance<SRC, 2, 2, 4, 4, LA>(p, stream);
  if (tile_m == 256 && tile_n == 128) return launch_packed_instance<SRC, 2, 2, 4, 2, LA>(p, stream);
  if (tile_m == 128 && tile_n == 256) return launch_packed_instance<SRC, 2, 2, 2, 4, LA>(p, stream);
  if (tile_m == 128 && tile_n == 128) return launch_packed_instance<SRC, 2, 2, 2, 2, LA>(p, stream);
  return launch_packed_instance<SRC, 2, 2, 1, 1, LA>(p, stream);
}

template <int SRC>
hipError_t launch_packed_class(const TileGemmParams& p, int tile_m, int tile_n, int vector_a, hipStream_t stream) {
  // vector_a: 0 element loads, 1 16-byte loads, 2 16-byte loads that write LDS themselves (aligned bf16 / int8 A,
  // the three big tiles)
  if constexpr (SRC == SRC_BF16 || SRC == SRC_I8) {
    if (vector_a == 2 && tile_m * tile_n >= 256 * 128) {
      if (tile_m == 256 && tile_n == 256) return launch_packed_instance<SRC, 2, 2, 4, 4, LOAD_KDMA>(p, stream);
      if (tile_m == 256 && tile_n == 128) return launch_packed_instance<SRC, 2, 2, 4, 2, LOAD_KDMA>(p, stream);
      return launch_packed_instance<SRC, 2, 2, 2, 4, LOAD_KDMA>(p, stream);
    }
  }
  return vector_a ? launch_packed_tile<SRC, LOAD_KVEC>(p, tile_m, tile_n, stream)
                  : launch_packed_tile<SRC, LOAD_GENERIC>(p, tile_m, tile_n, stream);
}

}  // namespace

hipError_t launch_tile_gemm_packed_b(int src, const TileGemmParams& p, int tile_m, int tile_n, int vector_a,
                                     hipStream_t stream) {
  switch (src) {
    case SRC_BF16: return launch_packed_class<SRC_BF16>(p, tile_m, tile_n, vector_a, stream);
    case SRC_F32_AS_BF16: return launch_packed_class<SRC_F32_AS_BF16>(p, tile_m, tile_n, vector_a, stream);
    case SRC_I8: return launch_packed_class<SRC_I8>(p, tile_m, tile_n, vector_a, stream);
    default: return hipErrorInvalidValue;
  }
}

hipError_t launch_pack_b(int src, const PackBParams& p, hipStream_t stream) {
  const int epc = src == SRC_I8 ? 16 : 8;
  const int64_t chunks = packed_b_bytes(p.n, p.k, epc) / 16;
  if (chunks == 0) return hipSuccess;
  int64_t blocks = (chunks + 255) / 256;
  if (blocks > 256 * 64) blocks = 256 * 64;
  const dim3 grid(static_cast<unsigned>(blocks)), block(256);
  switch (src) {
    case SRC_BF16: hipLaunchKernelGGL(pack_b_kernel<SRC_BF16>, grid, block, 0, stream, p); break;
    case SRC_F32_AS_BF16: hipLaunchKernelGGL(pack_b_kernel<SRC_F32_AS_BF16>, grid, block, 0, stream, p); break;
    case SRC_I8: hipLaunchKernelGGL(pack_b_kernel<SRC_I8>, grid, block, 0, stream, p); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

}  // namespace vecops_hip
