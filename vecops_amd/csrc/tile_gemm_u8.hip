// Tile GEMM instances for 8-bit integer operands with an unsigned side, and the
// row-sum kernel that produces their epilogue terms.
#include "tile_gemm_launch.h"
namespace vecops_hip {
hipError_t launch_tile_gemm_i8_flip(const TileGemmParams& p, int tile_m, int tile_n, int mode, hipStream_t stream) {
  return launch_tile_class<SRC_I8_FLIP>(p, tile_m, tile_n, mode, stream);
}

// out[b][r] = scale * sum_k int8(x[b][r][k] xor flip) (+ add[b * add_bs + r])  (wrapping): the per-row and
// per-column terms of SRC_I8_FLIP.  One wavefront per row, any strides; 16 bytes per lane and step
// when the row is contiguous and aligned.
__global__ __launch_bounds__(256) void byte_row_sums_kernel(const uint8_t* x, int32_t batch, int32_t rows, int32_t k,
                                                            int64_t bs, int64_t rs, int64_t ks, uint32_t flip,
                                                            uint32_t scale, const int32_t* add, int64_t add_bs,
                                                            int32_t* out) {
  const int lane = threadIdx.x & 63;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (row >= static_cast<int64_t>(batch) * rows) return;
  const int64_t b = row / rows, r = row - b * rows;
  const uint8_t* src = x + b * bs + r * rs;
  int32_t sum = 0;
  int done = 0;
  if (ks == 1 && (reinterpret_cast<uintptr_t>(src) & 15u) == 0) {
    const int chunks = k / 16;
    for (int ch = lane; ch < chunks; ch += 64) {
      const u32x4 v = reinterpret_cast<const u32x4*>(src)[ch];
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const int32_t word = static_cast<int32_t>(v[w] ^ flip);
        sum += (word << 24 >> 24) + (word << 16 >> 24) + (word << 8 >> 24) + (word >> 24);
      }
    }
    done = chunks * 16;
  }
  for (int kk = done + lane; kk < k; kk += 64) sum += static_cast<int8_t>(src[kk * ks] ^ static_cast<uint8_t>(flip));
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) sum += __shfl_xor(sum, off, 64);
  if (lane == 0) out[row] = static_cast<int32_t>(static_cast<uint32_t>(sum) * scale + (add ? static_cast<uint32_t>(add[b * add_bs + r]) : 0u));
}

// q[b][r][k] = u8(x[b][r][k] * multipliers[b * mult_bs + r] + float(zero_point)): vecops'
// RuntimePerRowAsymmetricQuantizeTransform (matmul/Quantization.h:91-146) and the conversion of its fp32
// result to the uint8 compute type - a multiply and an add, each rounded (the file is compiled without
// contraction), truncation toward zero, NaN and values outside int32 to INT32_MIN, saturation to 0..255.
// One thread per four consecutive k: one 16-byte load when x is K-contiguous and the quad is aligned, one
// 4-byte store when q is.  flip (0 or 0x80) is xored into every byte.
__global__ __launch_bounds__(256) void quantize_rows_kernel(const float* x, int32_t batch, int32_t rows, int32_t k,
                                                            int64_t xbs, int64_t xrs, int64_t xks,
                                                            const float* multipliers, int64_t mult_bs, float zero_point,
                                                            uint32_t flip, uint8_t* q, int64_t qbs, int64_t qrs,
                                                            int64_t qks) {
  const int64_t quads_per_row = (static_cast<int64_t>(k) + 3) / 4;
  const int64_t total = static_cast<int64_t>(batch) * rows * quads_per_row;
  for (int64_t idx = blockIdx.x * 256ll + threadIdx.x; idx < total; idx += gridDim.x * 256ll) {
    const int64_t row = idx / quads_per_row;                 // batch * rows + r
    const int k0 = static_cast<int>(idx - row * quads_per_row) * 4;
    const int64_t b = row / rows, r = row - b * rows;
    const float* src = x + b * xbs + r * xrs + k0 * xks;
    uint8_t* dst = q + b * qbs + r * qrs + k0 * qks;
    const float mult = multipliers[b * mult_bs + r];
    const int left = min(4, k - k0);
    float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (left == 4 && xks == 1 && (reinterpret_cast<uintptr_t>(src) & 15u) == 0) {
      const f32x4 quad = *reinterpret_cast<const f32x4*>(src);
      v[0] = quad[0]; v[1] = quad[1]; v[2] = quad[2]; v[3] = quad[3];
    } else {
      for (int e = 0; e < left; ++e) v[e] = src[e * xks];
    }
    uint32_t bytes[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float scaled = v[e] * mult;
      bytes[e] = narrow_to_byte(scaled + zero_point, false) ^ flip;  // flip 0x80: the byte as q - 128 in int8
    }
    if (left == 4 && qks == 1 && (reinterpret_cast<uintptr_t>(dst) & 3u) == 0) {
      *reinterpret_cast<uint32_t*>(dst) = bytes[0] | (bytes[1] << 8) | (bytes[2] << 16) | (bytes[3] << 24);
    } else {
      for (int e = 0; e < left; ++e) dst[e * qks] = static_cast<uint8_t>(bytes[e]);
    }
  }
}

hipError_t launch_quantize_rows(const float* x, int32_t batch, int32_t rows, int32_t k, int64_t xbs, int64_t xrs,
                                int64_t xks, const float* multipliers, int64_t mult_bs, int32_t zero_point, uint32_t flip,
                                uint8_t* q, int64_t qbs, int64_t qrs, int64_t qks, hipStream_t stream) {
  const int64_t total = static_cast<int64_t>(batch) * rows * ((static_cast<int64_t>(k) + 3) / 4);
  if (total <= 0) return hipSuccess;
  int64_t blocks = (total + 255) / 256;
  if (blocks > 256 * 32) blocks = 256 * 32;
  hipLaunchKernelGGL(quantize_rows_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, x, batch, rows, k,
                     xbs, xrs, xks, multipliers, mult_bs, static_cast<float>(zero_point), flip & 0xffu, q, qbs, qrs, qks);
  return hipGetLastError();
}

hipError_t launch_byte_row_sums(const void* x, int32_t batch, int32_t rows, int32_t k, int64_t bs, int64_t rs,
                                int64_t ks, uint32_t flip, uint32_t scale, const int32_t* add, int64_t add_bs, int32_t* out,
                                hipStream_t stream) {
  const int64_t total = static_cast<int64_t>(batch) * rows;
  if (total <= 0) return hipSuccess;
  const int64_t blocks = (total + 3) / 4;
  if (blocks > INT32_MAX) return hipErrorInvalidConfiguration;
  hipLaunchKernelGGL(byte_row_sums_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream,
                     static_cast<const uint8_t*>(x), batch, rows, k, bs, rs, ks, flip, scale, add, add_bs, out);
  return hipGetLastError();
}
}  // namespace vecops_hip
