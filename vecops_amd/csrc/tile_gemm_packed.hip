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

}  // namespace

hipError_t launch_tile_gemm_packed_b(int src, const TileGemmParams& p, int tile_m, int tile_n, int vector_a,
                                     hipStream_t stream) {
  switch (src) {
    case SRC_BF16: return launch_packed_class<SRC_BF16>(p, tile_m, tile_n, vector_a, stream);
    case SRC_F16: return launch_packed_class<SRC_F16>(p, tile_m, tile_n, vector_a, stream);
    case SRC_F32_AS_BF16: return launch_packed_class<SRC_F32_AS_BF16>(p, tile_m, tile_n, vector_a, stream);
    case SRC_F32: return launch_packed_class<SRC_F32>(p, tile_m, tile_n, vector_a, stream);
    case SRC_I8: return launch_packed_class<SRC_I8>(p, tile_m, tile_n, vector_a, stream);
    // unsigned A: xored on its way into LDS, so never by the loads that write LDS themselves
    case SRC_I8_FLIP: return launch_packed_class<SRC_I8_FLIP>(p, tile_m, tile_n, vector_a ? 1 : 0, stream);
    default: return hipErrorInvalidValue;
  }
}

// out[b][n] = scale * sum_k B[n,k] (+ add[n], may be null) for an int8 packed operand, once per batch b: the per-column term of an
// unsigned A (a xor 0x80 is multiplied, 128 * sum_k B[n,k] comes back here; wrapping).  One wavefront per
// 32-row block walks its k-steps as one contiguous stream; lanes l and l + 32 hold the two halves of a row.
__global__ __launch_bounds__(256) void packed_row_sums_kernel(const void* packed, int32_t n, int32_t k, int32_t batch,
                                                              uint32_t scale, const int32_t* add, int32_t* out) {
  const int lane = threadIdx.x & 63;
  const int64_t nb = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (nb * 32 >= n) return;
  const int64_t ks_total = packed_k_steps(k, 16);
  const u32x4* src = static_cast<const u32x4*>(packed) + nb * ks_total * 64 + lane;
  int32_t sum = 0;
  for (int64_t ks = 0; ks < ks_total; ++ks) {
    const u32x4 v = src[ks * 64];
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const int32_t x = static_cast<int32_t>(v[w]);
      sum += (x << 24 >> 24) + (x << 16 >> 24) + (x << 8 >> 24) + (x >> 24);
    }
  }
  sum += __shfl_xor(sum, 32, 64);
  const int64_t row = nb * 32 + lane;
  if (lane < 32 && row < n) {
    const int32_t term = static_cast<int32_t>(static_cast<uint32_t>(sum) * scale + (add ? static_cast<uint32_t>(add[row]) : 0u));
    for (int32_t b = 0; b < batch; ++b) out[static_cast<int64_t>(b) * n + row] = term;
  }
}

hipError_t launch_packed_row_sums(const void* packed, int32_t n, int32_t k, int32_t batch, uint32_t scale,
                                  const int32_t* add, int32_t* out, hipStream_t stream) {
  if (n <= 0 || batch <= 0) return hipSuccess;
  const int64_t blocks = ((static_cast<int64_t>(n) + 31) / 32 + 3) / 4;
  hipLaunchKernelGGL(packed_row_sums_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, packed, n, k, batch,
                     scale, add, out);
  return hipGetLastError();
}

hipError_t launch_pack_b(int src, const PackBParams& p, hipStream_t stream) {
  const int epc = src == SRC_I8 ? 16 : src == SRC_F32 ? 4 : 8;
  const int64_t chunks = packed_b_bytes(p.n, p.k, epc) / 16;
  if (chunks == 0) return hipSuccess;
  int64_t blocks = (chunks + 255) / 256;
  if (blocks > 256 * 64) blocks = 256 * 64;
  const dim3 grid(static_cast<unsigned>(blocks)), block(256);
  switch (src) {
    case SRC_BF16: hipLaunchKernelGGL(pack_b_kernel<SRC_BF16>, grid, block, 0, stream, p); break;
    case SRC_F32_AS_BF16: hipLaunchKernelGGL(pack_b_kernel<SRC_F32_AS_BF16>, grid, block, 0, stream, p); break;
    case SRC_F32: hipLaunchKernelGGL(pack_b_kernel<SRC_F32>, grid, block, 0, stream, p); break;
    case SRC_I8: hipLaunchKernelGGL(pack_b_kernel<SRC_I8>, grid, block, 0, stream, p); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

hipError_t launch_unpack_b(int src, const PackBParams& p, hipStream_t stream) {
  const int epc = src == SRC_I8 ? 16 : src == SRC_F32 ? 4 : 8;
  const int64_t chunks = packed_b_bytes(p.n, p.k, epc) / 16;
  if (chunks == 0) return hipSuccess;
  int64_t blocks = (chunks + 255) / 256;
  if (blocks > 256 * 64) blocks = 256 * 64;
  const dim3 grid(static_cast<unsigned>(blocks)), block(256);
  switch (src) {
    case SRC_BF16: hipLaunchKernelGGL(unpack_b_kernel<SRC_BF16>, grid, block, 0, stream, p); break;
    case SRC_F32: hipLaunchKernelGGL(unpack_b_kernel<SRC_F32>, grid, block, 0, stream, p); break;
    case SRC_I8: hipLaunchKernelGGL(unpack_b_kernel<SRC_I8>, grid, block, 0, stream, p); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

}  // namespace vecops_hip
