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
struct ByteRowSums {
  const uint8_t* x;
  int32_t batch, rows, k;
  int64_t bs, rs, ks;
  uint32_t flip, scale;
  const int32_t* add;
  int64_t add_bs;
  int32_t* out;
};

// (block: the workgroup's number among those that sum rows)
__device__ __forceinline__ void byte_row_sums(const ByteRowSums& a, int64_t block) {
  const uint8_t* x = a.x;
  const int32_t batch = a.batch, rows = a.rows, k = a.k;
  const int64_t bs = a.bs, rs = a.rs, ks = a.ks, add_bs = a.add_bs;
  const uint32_t flip = a.flip, scale = a.scale;
  const int32_t* add = a.add;
  int32_t* out = a.out;
  const int lane = threadIdx.x & 63;
  const int64_t row = block * 4 + (threadIdx.x >> 6);
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

__global__ __launch_bounds__(256) void byte_row_sums_kernel(const ByteRowSums a) { byte_row_sums(a, blockIdx.x); }

// q[b][r][k] = u8(x[b][r][k] * multipliers[b * mult_bs + r] + float(zero_point)): vecops'
// RuntimePerRowAsymmetricQuantizeTransform (matmul/Quantization.h:91-146) and the conversion of its fp32
// result to the uint8 compute type - a multiply and an add, each rounded (the file is compiled without
// contraction), truncation toward zero, NaN and values outside int32 to INT32_MIN, saturation to 0..255.
// One thread per four consecutive k: one 16-byte load when x is K-contiguous and the quad is aligned, one
// 4-byte store when q is.  flip (0 or 0x80) is xored into every byte.
struct QuantizeRows {
  const float* x;
  int32_t batch, rows, k;
  int64_t xbs, xrs, xks;
  const float* multipliers;
  int64_t mult_bs;
  float zero_point;
  uint32_t flip;
  uint8_t* q;
  int64_t qbs, qrs, qks;
};

// (block of blocks: the workgroup's number among those that quantise, and how many they are)
__device__ __forceinline__ void quantize_rows(const QuantizeRows& a, int64_t block, int64_t blocks) {
  const float* x = a.x;
  const int32_t batch = a.batch, rows = a.rows, k = a.k;
  const int64_t xbs = a.xbs, xrs = a.xrs, xks = a.xks, mult_bs = a.mult_bs, qbs = a.qbs, qrs = a.qrs, qks = a.qks;
  const float* multipliers = a.multipliers;
  const float zero_point = a.zero_point;
  const uint32_t flip = a.flip;
  uint8_t* q = a.q;
  const int64_t quads_per_row = (static_cast<int64_t>(k) + 3) / 4;
  const int64_t total = static_cast<int64_t>(batch) * rows * quads_per_row;
  for (int64_t idx = block * 256ll + threadIdx.x; idx < total; idx += blocks * 256ll) {
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

__global__ __launch_bounds__(256) void quantize_rows_kernel(const QuantizeRows a) { quantize_rows(a, blockIdx.x, gridDim.x); }

// Both preparations of a runtime-quantised product in one launch: the first quantize_blocks workgroups quantise the
// activations, the others sum the weight rows (two memory-bound kernels of about 10 us each, neither of which needs the
// other: one launch saves a launch gap and lets their tails overlap).
__global__ __launch_bounds__(256) void quantize_and_row_sums_kernel(const QuantizeRows qa, const ByteRowSums sa, uint32_t quantize_blocks) {
  if (blockIdx.x < quantize_blocks) quantize_rows(qa, blockIdx.x, quantize_blocks);
  else byte_row_sums(sa, blockIdx.x - quantize_blocks);
}

namespace {
int64_t quantize_blocks_for(int64_t total_quads) {
  int64_t blocks = (total_quads + 255) / 256;
  return blocks > 256 * 32 ? 256 * 32 : blocks;
}
}  // namespace

hipError_t launch_quantize_rows(const float* x, int32_t batch, int32_t rows, int32_t k, int64_t xbs, int64_t xrs,
                                int64_t xks, const float* multipliers, int64_t mult_bs, int32_t zero_point, uint32_t flip,
                                uint8_t* q, int64_t qbs, int64_t qrs, int64_t qks, hipStream_t stream) {
  const int64_t total = static_cast<int64_t>(batch) * rows * ((static_cast<int64_t>(k) + 3) / 4);
  if (total <= 0) return hipSuccess;
  const QuantizeRows a{x, batch, rows, k, xbs, xrs, xks, multipliers, mult_bs, static_cast<float>(zero_point), flip & 0xffu, q, qbs, qrs, qks};
  hipLaunchKernelGGL(quantize_rows_kernel, dim3(static_cast<unsigned>(quantize_blocks_for(total))), dim3(256), 0, stream, a);
  return hipGetLastError();
}

hipError_t launch_byte_row_sums(const void* x, int32_t batch, int32_t rows, int32_t k, int64_t bs, int64_t rs,
                                int64_t ks, uint32_t flip, uint32_t scale, const int32_t* add, int64_t add_bs, int32_t* out,
                                hipStream_t stream) {
  const int64_t total = static_cast<int64_t>(batch) * rows;
  if (total <= 0) return hipSuccess;
  const int64_t blocks = (total + 3) / 4;
  if (blocks > INT32_MAX) return hipErrorInvalidConfiguration;
  const ByteRowSums a{static_cast<const uint8_t*>(x), batch, rows, k, bs, rs, ks, flip, scale, add, add_bs, out};
  hipLaunchKernelGGL(byte_row_sums_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, a);
  return hipGetLastError();
}

// launch_quantize_rows and launch_byte_row_sums as one launch (both must have work: the caller checks).
hipError_t launch_quantize_and_row_sums(const float* x, int32_t batch, int32_t rows, int32_t k, int64_t xbs, int64_t xrs,
                                        int64_t xks, const float* multipliers, int64_t mult_bs, int32_t zero_point, uint32_t flip,
                                        uint8_t* q, int64_t qbs, int64_t qrs, int64_t qks, const void* w, int32_t w_batch,
                                        int32_t w_rows, int64_t w_bs, int64_t w_rs, int64_t w_ks, uint32_t w_flip, uint32_t scale,
                                        const int32_t* add, int64_t add_bs, int32_t* out, hipStream_t stream) {
  const int64_t total = static_cast<int64_t>(batch) * rows * ((static_cast<int64_t>(k) + 3) / 4);
  const int64_t sums = static_cast<int64_t>(w_batch) * w_rows;
  if (total <= 0 || sums <= 0) return hipErrorInvalidValue;
  const int64_t q_blocks = quantize_blocks_for(total), s_blocks = (sums + 3) / 4;
  if (q_blocks + s_blocks > INT32_MAX) return hipErrorInvalidConfiguration;
  const QuantizeRows qa{x, batch, rows, k, xbs, xrs, xks, multipliers, mult_bs, static_cast<float>(zero_point), flip & 0xffu, q, qbs, qrs, qks};
  const ByteRowSums sa{static_cast<const uint8_t*>(w), w_batch, w_rows, k, w_bs, w_rs, w_ks, w_flip, scale, add, add_bs, out};
  hipLaunchKernelGGL(quantize_and_row_sums_kernel, dim3(static_cast<unsigned>(q_blocks + s_blocks)), dim3(256), 0, stream, qa, sa,
                     static_cast<uint32_t>(q_blocks));
  return hipGetLastError();
}
}  // namespace vecops_hip
