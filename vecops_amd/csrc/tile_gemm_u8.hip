// Tile GEMM instances for 8-bit integer operands with an unsigned side, and the
// row-sum kernel that produces their epilogue terms.
#include "tile_gemm_launch.h"
namespace vecops_hip {
hipError_t launch_tile_gemm_i8_flip(const TileGemmParams& p, int tile_m, int tile_n, int mode, hipStream_t stream) {
  return launch_tile_class<SRC_I8_FLIP>(p, tile_m, tile_n, mode, stream);
}

// out[b][r] = scale * sum_k int8(x[b][r][k] xor flip)  (wrapping): the per-row and
// per-column terms of SRC_I8_FLIP.  One wavefront per row, any strides.
__global__ __launch_bounds__(256) void byte_row_sums_kernel(const uint8_t* x, int32_t batch, int32_t rows, int32_t k,
                                                            int64_t bs, int64_t rs, int64_t ks, uint32_t flip,
                                                            uint32_t scale, int32_t* out) {
  const int lane = threadIdx.x & 63;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (row >= static_cast<int64_t>(batch) * rows) return;
  const int64_t b = row / rows, r = row - b * rows;
  const uint8_t* src = x + b * bs + r * rs;
  int32_t sum = 0;
  for (int kk = lane; kk < k; kk += 64) sum += static_cast<int8_t>(src[kk * ks] ^ static_cast<uint8_t>(flip));
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) sum += __shfl_xor(sum, off, 64);
  if (lane == 0) out[row] = static_cast<int32_t>(static_cast<uint32_t>(sum) * scale);
}

hipError_t launch_byte_row_sums(const void* x, int32_t batch, int32_t rows, int32_t k, int64_t bs, int64_t rs,
                                int64_t ks, uint32_t flip, uint32_t scale, int32_t* out, hipStream_t stream) {
  const int64_t total = static_cast<int64_t>(batch) * rows;
  if (total <= 0) return hipSuccess;
  const int64_t blocks = (total + 3) / 4;
  if (blocks > INT32_MAX) return hipErrorInvalidConfiguration;
  hipLaunchKernelGGL(byte_row_sums_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream,
                     static_cast<const uint8_t*>(x), batch, rows, k, bs, rs, ks, flip, scale, out);
  return hipGetLastError();
}
}  // namespace vecops_hip
