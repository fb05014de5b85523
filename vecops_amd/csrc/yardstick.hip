// Measurement yardsticks (declared in include/vecops_hip.h): kernels that do nothing but the matrix-core
// instruction stream of the tile kernels, on operand values the caller supplies.  What they sustain is the
// ceiling a GEMM can reach on this machine with these operand values (the clocks follow the power the
// multipliers draw, which depends on the data), to be quoted beside the nominal peak.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "vecops_hip.h"

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(16))) int i32x16;
typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

// One wavefront per SIMD (256 threads per workgroup, one workgroup per compute unit and launch slot), 4 x 4
// accumulator tiles of 32x32 per wavefront as in the 256x256 tile kernel; two fragment sets (2 x (4 + 4)
// operand registers of 16 bytes) taken from `operands` and used alternately, so consecutive instructions see
// different operand values as the k-steps of a GEMM do.  `iters` x 32 matrix instructions per wavefront.
template <bool INT>
__global__ __launch_bounds__(256) void mfma_stream_kernel(const u32x4* __restrict__ operands, uint32_t chunks,
                                                         int iters, uint32_t* __restrict__ out) {
  const uint32_t tid = blockIdx.x * 256u + threadIdx.x;
  u32x4 a[2][4], b[2][4];
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      a[s][i] = operands[(tid * 16u + s * 8 + i) % chunks];
      b[s][i] = operands[(tid * 16u + s * 8 + 4 + i) % chunks];
    }
  using Acc = typename std::conditional<INT, i32x16, f32x16>::type;
  Acc acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if constexpr (INT)
            acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, b[s][j]),
                                                              __builtin_bit_cast(i32x4, a[s][i]), acc[i][j], 0, 0, 0);
          else
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, b[s][j]),
                                                                __builtin_bit_cast(bf16x8, a[s][i]), acc[i][j], 0, 0, 0);
        }
  }
  uint32_t folded = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        if constexpr (INT) folded += static_cast<uint32_t>(acc[i][j][e]);
        else folded += __float_as_uint(acc[i][j][e]);
      }
  out[tid] = folded;
}

// The same stream on the 16x16 shapes: 4 x 4 accumulator quads per wavefront, the fragment sets used alternately.
template <bool INT>
__global__ __launch_bounds__(256) void mfma_stream16_kernel(const u32x4* __restrict__ operands, uint32_t chunks,
                                                           int iters, uint32_t* __restrict__ out) {
  typedef __attribute__((ext_vector_type(4))) float f32x4;
  const uint32_t tid = blockIdx.x * 256u + threadIdx.x;
  u32x4 a[2][4], b[2][4];
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      a[s][i] = operands[(tid * 16u + s * 8 + i) % chunks];
      b[s][i] = operands[(tid * 16u + s * 8 + 4 + i) % chunks];
    }
  using Acc = typename std::conditional<INT, i32x4, f32x4>::type;
  Acc acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[i][j][e] = 0;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if constexpr (INT)
            acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(i32x4, b[s][j]),
                                                              __builtin_bit_cast(i32x4, a[s][i]), acc[i][j], 0, 0, 0);
          else
            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, b[s][j]),
                                                                __builtin_bit_cast(bf16x8, a[s][i]), acc[i][j], 0, 0, 0);
        }
  }
  uint32_t folded = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if constexpr (INT) folded += static_cast<uint32_t>(acc[i][j][e]);
        else folded += __float_as_uint(acc[i][j][e]);
      }
  out[tid] = folded;
}

}  // namespace

extern "C" {

uint64_t vecops_hip_mfma_stream_shape_ops(uint32_t dtype, uint32_t shape, int32_t workgroups, int32_t iters) {
  if (shape == 0) return vecops_hip_mfma_stream_ops(dtype, workgroups, iters);
  if (shape != 1 || workgroups <= 0 || iters <= 0) return 0;
  const uint64_t per_instruction = dtype == 2 ? 2ull * 16 * 16 * 64 : 2ull * 16 * 16 * 32;
  return per_instruction * 32ull * static_cast<uint64_t>(iters) * 4ull * static_cast<uint64_t>(workgroups);
}

int32_t vecops_hip_mfma_stream_shape(uint32_t dtype, uint32_t shape, const void* operands, uint64_t operand_bytes,
                                     int32_t workgroups, int32_t iters, void* out, void* stream) {
  if (shape == 0) return vecops_hip_mfma_stream(dtype, operands, operand_bytes, workgroups, iters, out, stream);
  if (shape != 1 || (dtype != 2 && dtype != 11) || operands == nullptr || out == nullptr || operand_bytes < 16 ||
      workgroups <= 0 || iters <= 0 || (reinterpret_cast<uintptr_t>(operands) & 15u) != 0)
    return 1;
  const uint32_t chunks = static_cast<uint32_t>(operand_bytes / 16 > 0xffffffffull ? 0xffffffffull : operand_bytes / 16);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == 2)
    hipLaunchKernelGGL(mfma_stream16_kernel<true>, dim3(workgroups), dim3(256), 0, s, static_cast<const u32x4*>(operands),
                       chunks, iters, static_cast<uint32_t*>(out));
  else
    hipLaunchKernelGGL(mfma_stream16_kernel<false>, dim3(workgroups), dim3(256), 0, s, static_cast<const u32x4*>(operands),
                       chunks, iters, static_cast<uint32_t*>(out));
  return hipGetLastError() == hipSuccess ? 0 : 6;
}

uint64_t vecops_hip_mfma_stream_ops(uint32_t dtype, int32_t workgroups, int32_t iters) {
  if (workgroups <= 0 || iters <= 0) return 0;
  const uint64_t per_instruction = dtype == 2 ? 2ull * 32 * 32 * 32 : 2ull * 32 * 32 * 16;
  return per_instruction * 32ull * static_cast<uint64_t>(iters) * 4ull * static_cast<uint64_t>(workgroups);
}

int32_t vecops_hip_mfma_stream(uint32_t dtype, const void* operands, uint64_t operand_bytes, int32_t workgroups,
                               int32_t iters, void* out, void* stream) {
  if ((dtype != 2 && dtype != 11) || operands == nullptr || out == nullptr || operand_bytes < 16 || workgroups <= 0 ||
      iters <= 0 || (reinterpret_cast<uintptr_t>(operands) & 15u) != 0)
    return 1;
  const uint32_t chunks = static_cast<uint32_t>(operand_bytes / 16 > 0xffffffffull ? 0xffffffffull : operand_bytes / 16);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == 2)
    hipLaunchKernelGGL(mfma_stream_kernel<true>, dim3(workgroups), dim3(256), 0, s, static_cast<const u32x4*>(operands),
                       chunks, iters, static_cast<uint32_t*>(out));
  else
    hipLaunchKernelGGL(mfma_stream_kernel<false>, dim3(workgroups), dim3(256), 0, s, static_cast<const u32x4*>(operands),
                       chunks, iters, static_cast<uint32_t*>(out));
  return hipGetLastError() == hipSuccess ? 0 : 6;
}

}  // extern "C"
