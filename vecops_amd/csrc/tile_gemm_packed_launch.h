// Launchers of the prepacked-B tile kernels, one translation unit per operand class (tile_gemm_packed_*.hip).
#ifndef VECOPS_HIP_TILE_GEMM_PACKED_LAUNCH_H
#define VECOPS_HIP_TILE_GEMM_PACKED_LAUNCH_H

#include "tile_gemm_packed.h"

#include "tile_gemm_launch.h"
namespace vecops_hip {

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
  if constexpr (SRC == SRC_BF16 || SRC == SRC_F16 || SRC == SRC_I8) {
    if (vector_a == 2 && tile_m * tile_n >= 256 * 128) {
      if (tile_m == 256 && tile_n == 256) return launch_packed_instance<SRC, 2, 2, 4, 4, LOAD_KDMA>(p, stream);
      if (tile_m == 256 && tile_n == 128) return launch_packed_instance<SRC, 2, 2, 4, 2, LOAD_KDMA>(p, stream);
      return launch_packed_instance<SRC, 2, 2, 2, 4, LOAD_KDMA>(p, stream);
    }
  }
  return vector_a ? launch_packed_tile<SRC, LOAD_KVEC>(p, tile_m, tile_n, stream)
                  : launch_packed_tile<SRC, LOAD_GENERIC>(p, tile_m, tile_n, stream);
}


// vector_a: 0 element loads, 1 16-byte loads, 2 16-byte loads that write LDS themselves
hipError_t launch_packed_bf16(const TileGemmParams& p, int tile_m, int tile_n, int vector_a, hipStream_t stream);
hipError_t launch_packed_f16(const TileGemmParams& p, int tile_m, int tile_n, int vector_a, hipStream_t stream);
hipError_t launch_packed_f32_as_bf16(const TileGemmParams& p, int tile_m, int tile_n, int vector_a, hipStream_t stream);
hipError_t launch_packed_f32(const TileGemmParams& p, int tile_m, int tile_n, int vector_a, hipStream_t stream);
hipError_t launch_packed_i8(const TileGemmParams& p, int tile_m, int tile_n, int vector_a, hipStream_t stream);
hipError_t launch_packed_i8_flip(const TileGemmParams& p, int tile_m, int tile_n, int vector_a, hipStream_t stream);

}  // namespace vecops_hip
#endif
