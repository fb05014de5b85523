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
// The 32 instructions of a trip are ONE asm statement whose accumulators are tied operands in the accumulation
// registers: written with the builtins the loop came out with three register copies per matrix instruction
// (a new accumulator on every trip, copied back at the loop's head) and measured 30 % below the pipe's rate.
#define VECOPS_Y16(INSTR, i, j, s) INSTR " %[c" #i #j "], %[b" #s #j "], %[a" #s #i "], %[c" #i #j "]\n\t"
#define VECOPS_Y16_ROW(INSTR, i, s) \
  VECOPS_Y16(INSTR, i, 0, s) VECOPS_Y16(INSTR, i, 1, s) VECOPS_Y16(INSTR, i, 2, s) VECOPS_Y16(INSTR, i, 3, s)
#define VECOPS_Y16_SET(INSTR, s) \
  VECOPS_Y16_ROW(INSTR, 0, s) VECOPS_Y16_ROW(INSTR, 1, s) VECOPS_Y16_ROW(INSTR, 2, s) VECOPS_Y16_ROW(INSTR, 3, s)
#define VECOPS_Y16_ACC(i) \
  [c##i##0] "+a"(acc[i][0]), [c##i##1] "+a"(acc[i][1]), [c##i##2] "+a"(acc[i][2]), [c##i##3] "+a"(acc[i][3])
#define VECOPS_Y16_FRAGS(s)                                                                                   \
  [a##s##0] "v"(a[s][0]), [a##s##1] "v"(a[s][1]), [a##s##2] "v"(a[s][2]), [a##s##3] "v"(a[s][3]),          \
  [b##s##0] "v"(b[s][0]), [b##s##1] "v"(b[s][1]), [b##s##2] "v"(b[s][2]), [b##s##3] "v"(b[s][3])
#define VECOPS_Y16_TRIP(INSTR)                                                                               \
  asm volatile(VECOPS_Y16_SET(INSTR, 0) VECOPS_Y16_SET(INSTR, 1)                                             \
               : VECOPS_Y16_ACC(0), VECOPS_Y16_ACC(1), VECOPS_Y16_ACC(2), VECOPS_Y16_ACC(3)                  \
               : VECOPS_Y16_FRAGS(0), VECOPS_Y16_FRAGS(1))

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
    if constexpr (INT) VECOPS_Y16_TRIP("v_mfma_i32_16x16x64_i8");
    else VECOPS_Y16_TRIP("v_mfma_f32_16x16x32_bf16");
  }
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");  // the last results are in their registers before they are read
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

// Read-only yardstick of the skinny kernels: every workgroup streams its share of `chunks` 16-byte pieces with eight
// loads in flight per lane and folds them into one word per lane.  Nothing is computed and 1 KiB per workgroup is
// written: what it sustains on a buffer of the GEMV's size is the rate at which this machine delivers that many bytes
// to a kernel launched back to back, launch and ramp included.
__global__ __launch_bounds__(256) void read_stream_kernel(const u32x4* __restrict__ src, uint64_t chunks,
                                                         uint32_t* __restrict__ out) {
  const uint64_t stride = static_cast<uint64_t>(gridDim.x) * 256u;
  uint64_t i = static_cast<uint64_t>(blockIdx.x) * 256u + threadIdx.x;
  u32x4 f = {0u, 0u, 0u, 0u};
  for (; i + 7 * stride < chunks; i += 8 * stride) {
    u32x4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = __builtin_nontemporal_load(src + i + u * stride);
#pragma unroll
    for (int u = 0; u < 8; ++u) f ^= v[u];
  }
  for (; i < chunks; i += stride) f ^= __builtin_nontemporal_load(src + i);
  out[blockIdx.x * 256u + threadIdx.x] = f.x ^ f.y ^ f.z ^ f.w;
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

int32_t vecops_hip_read_stream(const void* src, uint64_t bytes, int32_t workgroups, void* out, void* stream) {
  if (src == nullptr || out == nullptr || bytes < 16 || workgroups <= 0 || (reinterpret_cast<uintptr_t>(src) & 15u) != 0)
    return 1;
  hipLaunchKernelGGL(read_stream_kernel, dim3(workgroups), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const u32x4*>(src), bytes / 16, static_cast<uint32_t*>(out));
  return hipGetLastError() == hipSuccess ? 0 : 6;
}

}  // extern "C"
