// Tile GEMM instances that take a prepacked B operand, and the packing kernel.
#include "tile_gemm_packed_launch.h"
namespace vecops_hip {
hipError_t launch_tile_gemm_packed_b(int src, const TileGemmParams& p, int tile_m, int tile_n, int vector_a,
                                     hipStream_t stream) {
  switch (src) {
    case SRC_BF16: return launch_packed_bf16(p, tile_m, tile_n, vector_a, stream);
    case SRC_F16: return launch_packed_f16(p, tile_m, tile_n, vector_a, stream);
    case SRC_F32_AS_BF16: return launch_packed_f32_as_bf16(p, tile_m, tile_n, vector_a, stream);
    case SRC_F32: return launch_packed_f32(p, tile_m, tile_n, vector_a, stream);
    case SRC_I8: return launch_packed_i8(p, tile_m, tile_n, vector_a, stream);
    // unsigned A: xored on its way into LDS, so never by the loads that write LDS themselves
    case SRC_I8_FLIP: return launch_packed_i8_flip(p, tile_m, tile_n, vector_a ? 1 : 0, stream);
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
