// Skinny bf16 matmul for gfx950 (HBM-bound): one operand has at most 16 rows.
//   y[s, r] = sum_k x[s, k] * w[r, k]      w: the wide operand [R, K], x: the narrow one [S <= 16, K]
// fp32 accumulation, both operands bf16 with K contiguous.  This is the GPU
// counterpart of vecops' small-vector leaves (small_vector_dense_matmul /
// small_vector_tall_matmul, matmul/details/kernel/amx/Backend.h:767-1151): the wide
// operand is read exactly once, the narrow one is kept in registers.
//
// One v_mfma_f32_16x16x32_bf16 multiplies 16 wide rows x 32 k by 32 k x 16 narrow rows
// (S padded to 16 with zeros).  Lane l holds wide row l % 16 and the 8 consecutive k
// of quarter l / 16 of a 32-element step (one 16-byte load); the narrow operand uses the
// same k order.  A workgroup of 8 wavefronts owns PASSES x TILES blocks of 16 wide
// rows; its wavefronts split K step by step (step t belongs to wavefront t % 8), so K
// need only be a multiple of 8.  K is walked in blocks of 4096: a wavefront loads the
// narrow fragments of its 16 steps of the block once (64 registers) and reuses them
// for every row block.  Loads of the wide operand run D = 4 steps ahead.  The K
// slices are summed through LDS at the end.
#ifndef VECOPS_HIP_SKINNY_DENSE_H
#define VECOPS_HIP_SKINNY_DENSE_H

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "tile_gemm.h"

namespace vecops_hip {

struct SkinnyDenseParams {
  const uint16_t* w;  // wide operand, bf16 bits
  const uint16_t* x;  // narrow operand, bf16 bits
  void* y;            // fp32 or bf16
  int64_t ldw, ldx;   // row strides in elements
  int64_t w_bs, x_bs, y_bs;  // batch strides in elements (0 broadcasts an operand)
  int64_t y_stride_r;  // elements between consecutive wide rows in y
  int64_t y_stride_s;  // elements between consecutive narrow rows in y
  int32_t rows;        // R
  int32_t s;           // S, 1..16
  int32_t k;           // multiple of 8
  int32_t out_bf16;
};

template <int PASSES, int TILES>
__global__ __launch_bounds__(512) void skinny_dense_kernel(const SkinnyDenseParams p) {
  constexpr int WAVES = 8, XS = 16, D = 4;  // XS steps of 32 k per wavefront and K block
  constexpr int BLOCKS = PASSES * TILES;    // 16-row blocks of this workgroup
  __shared__ float red[WAVES][BLOCKS][16 * 16];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int row = lane & 15, quarter = lane >> 4;
  const int batch = blockIdx.y;
  const int64_t row0 = static_cast<int64_t>(blockIdx.x) * (16 * BLOCKS);
  const int64_t last_row = static_cast<int64_t>(p.rows) - 1;
  const VECOPS_GLOBAL uint16_t* wbase = (const VECOPS_GLOBAL uint16_t*)p.w + batch * p.w_bs;
  const VECOPS_GLOBAL uint16_t* xrow =
      (const VECOPS_GLOBAL uint16_t*)p.x + batch * p.x_bs + static_cast<int64_t>(min(row, p.s - 1)) * p.ldx;
  // rows past R are clamped: computed, never stored
  const VECOPS_GLOBAL uint16_t* wrow[BLOCKS];
#pragma unroll
  for (int b = 0; b < BLOCKS; ++b) wrow[b] = wbase + min(row0 + b * 16 + row, last_row) * p.ldw;

  f32x4 acc[BLOCKS];
#pragma unroll
  for (int b = 0; b < BLOCKS; ++b) acc[b] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int k_blocks = (p.k + 4095) / 4096;
  for (int kb = 0; kb < k_blocks; ++kb) {
    // k of (step s of this wavefront, this lane's quarter) in this K block
    auto k_of = [&](int s) { return (kb * 128 + s * WAVES + wave) * 32 + quarter * 8; };
    u32x4 xq[XS];
#pragma unroll
    for (int s = 0; s < XS; ++s) {
      const int k0 = k_of(s);
      xq[s] = u32x4{0u, 0u, 0u, 0u};
      if (row < p.s && k0 < p.k) xq[s] = *(const VECOPS_GLOBAL u32x4*)(xrow + k0);
    }
    // flat sequence of (block, step) with the wide loads D ahead; a load past K reads as zero
    u32x4 wq[D];
    auto issue = [&](auto slot_tag, auto b_tag, auto s_tag) {
      constexpr int slot = decltype(slot_tag)::value, b = decltype(b_tag)::value, s = decltype(s_tag)::value;
      if constexpr (b < BLOCKS) {
        const int k0 = k_of(s);
        wq[slot] = u32x4{0u, 0u, 0u, 0u};
        if (k0 < p.k) wq[slot] = *(const VECOPS_GLOBAL u32x4*)(wrow[b] + k0);
      }
    };
    static_for<D>([&](auto u) { issue(u, std::integral_constant<int, 0>{}, u); });
    static_for<BLOCKS>([&](auto cb) {
      constexpr int b = decltype(cb)::value;
      static_for<XS>([&](auto cs) {
        constexpr int s = decltype(cs)::value, slot = s % D;
        acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wq[slot]),
                                                         __builtin_bit_cast(bf16x8, xq[s]), acc[b], 0, 0, 0);
        constexpr int ns = s + D;  // the step that takes over this slot
        issue(std::integral_constant<int, slot>{}, std::integral_constant<int, b + ns / XS>{},
              std::integral_constant<int, ns % XS>{});
      });
    });
  }

  // Sum the K slices through LDS.  Accumulator register r of lane l is output
  // (wide row quarter*4 + r, narrow row l % 16) of its 16x16 block.
#pragma unroll
  for (int b = 0; b < BLOCKS; ++b)
#pragma unroll
    for (int r = 0; r < 4; ++r) red[wave][b][(quarter * 4 + r) * 16 + row] = acc[b][r];
  __syncthreads();
  for (int b = wave; b < BLOCKS; b += WAVES) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float total = 0.0f;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) total += red[w][b][(quarter * 4 + r) * 16 + row];
      const int64_t n = row0 + b * 16 + quarter * 4 + r;
      if (row < p.s && n < p.rows) {
        const int64_t at = batch * p.y_bs + n * p.y_stride_r + row * p.y_stride_s;
        if (p.out_bf16) static_cast<uint16_t*>(p.y)[at] = static_cast<uint16_t>(bf16_bits_rne(total));
        else static_cast<float*>(p.y)[at] = total;
      }
    }
  }
}

}  // namespace vecops_hip
#endif
