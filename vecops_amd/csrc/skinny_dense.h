// Skinny matmul for gfx950 (HBM-bound): one operand has at most 16 rows.
//   y[s, r] = sum_k x[s, k] * w[r, k]      w: the wide operand [R, K], x: the narrow one [S <= 16, K]
// bf16 x bf16 (f16 x f16) with fp32 accumulation, fp32 operands rounded to bf16 on their way into the registers or
// multiplied in fp32, or int8 x int8 with wrapping int32 accumulation (optionally followed by the per-row x
// per-column dequantisation); both operands K contiguous.  This is the GPU counterpart of vecops' small-vector leaves
// (small_vector_dense_matmul / small_vector_tall_matmul,
// matmul/details/kernel/amx/Backend.h:767-1151): the wide operand is read exactly
// once, the narrow one is kept in registers.
//
// One v_mfma_f32_16x16x32_bf16 (_f16 for half operands; v_mfma_i32_16x16x64_i8) multiplies 16 wide rows by 16
// narrow rows (S padded to 16 with zeros) over a step of 32 (64) k.  Lane l holds wide
// row l % 16 and the 16 consecutive bytes of quarter l / 16 of the step (one 16-byte
// load; fp32 memory rounded to bf16: two loads, eight floats, converted in front of the MFMA);
// the narrow operand uses the same k order.  fp32 compute: a step is 16 k, a lane's 16-byte load holds four
// floats, and four v_mfma_f32_16x16x4_f32 each take one of them (k = 4 * quarter + e for MFMA e on both sides).  A workgroup of 8 wavefronts owns
// PASSES x TILES blocks of 16 wide rows; its wavefronts split K step by step (step t
// belongs to wavefront t % 8), so K need only be a multiple of 16 bytes.  K is walked
// in blocks of 128 steps: a wavefront loads the narrow fragments of its 16 steps of the
// block once (64 registers) and reuses them for every row block.  Loads of the wide
// operand run D = 4 steps ahead.  The K slices are summed through LDS at the end.
#ifndef VECOPS_HIP_SKINNY_DENSE_H
#define VECOPS_HIP_SKINNY_DENSE_H

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "tile_gemm.h"

namespace vecops_hip {

enum SkinnyOut : int { SKINNY_OUT_F32 = 0, SKINNY_OUT_BF16 = 1, SKINNY_OUT_I32 = 2, SKINNY_OUT_DEQUANT_F32 = 3, SKINNY_OUT_F16 = 4 };

struct SkinnyDenseParams {
  const void* w;      // wide operand (bf16 bits or int8)
  const void* x;      // narrow operand
  void* y;            // fp32, bf16 or int32
  int64_t ldw, ldx;   // row strides in elements
  int64_t w_bs, x_bs, y_bs;  // batch strides in elements (0 broadcasts an operand)
  int64_t y_stride_r;  // elements between consecutive wide rows in y
  int64_t y_stride_s;  // elements between consecutive narrow rows in y
  // dequantisation (SKINNY_OUT_DEQUANT_F32): y = (float(acc + wide_term[r]) * narrow_scales[s]) * wide_scales[r]
  const float* narrow_scales;
  const float* wide_scales;
  const int32_t* wide_term;  // null = none
  int32_t rows;        // R
  int32_t s;           // S, 1..16
  int32_t k;           // multiple of 16 bytes of elements
  int32_t out_kind;    // SkinnyOut
};

template <int SRC, int PASSES, int TILES>
__global__ __launch_bounds__(512) void skinny_dense_kernel(const SkinnyDenseParams p) {
  constexpr bool INT = SrcTraits<SRC>::kInt;
  constexpr int EPL = SrcTraits<SRC>::kElemsPerChunk;  // elements per lane and step
  constexpr int EPS = 4 * EPL;                         // elements per step
  constexpr int EB = SrcTraits<SRC>::kSrcBytes;
  constexpr int LOADS = EPL * EB / 16;                 // 16-byte loads per lane and step (2: fp32 memory, bf16 compute)
  struct Loaded { u32x4 v[LOADS]; };
  // the lane's elements of one step as they lie in memory -> the MFMA operand
  auto operand_of = [](const Loaded& raw) {
    if constexpr (SRC == SRC_F32_AS_BF16) {
      return u32x4{cvt_pk_bf16(__uint_as_float(raw.v[0][0]), __uint_as_float(raw.v[0][1])),
                   cvt_pk_bf16(__uint_as_float(raw.v[0][2]), __uint_as_float(raw.v[0][3])),
                   cvt_pk_bf16(__uint_as_float(raw.v[1][0]), __uint_as_float(raw.v[1][1])),
                   cvt_pk_bf16(__uint_as_float(raw.v[1][2]), __uint_as_float(raw.v[1][3]))};
    } else {
      return raw.v[0];
    }
  };
  auto load_of = [](const VECOPS_GLOBAL char* at, Loaded& out) {
#pragma unroll
    for (int i = 0; i < LOADS; ++i) out.v[i] = *(const VECOPS_GLOBAL u32x4*)(at + 16 * i);
  };
  using AccScalar = typename std::conditional<INT, int32_t, float>::type;
  using Acc4 = typename std::conditional<INT, i32x4, f32x4>::type;
  constexpr int WAVES = 8, XS = 16, D = 4;  // XS steps per wavefront and K block
  constexpr int BLOCKS = PASSES * TILES;    // 16-row blocks of this workgroup
  __shared__ AccScalar red[WAVES][BLOCKS][16 * 16];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int row = lane & 15, quarter = lane >> 4;
  const int batch = blockIdx.y;
  const int64_t row0 = static_cast<int64_t>(blockIdx.x) * (16 * BLOCKS);
  const int64_t last_row = static_cast<int64_t>(p.rows) - 1;
  const VECOPS_GLOBAL char* wbase = (const VECOPS_GLOBAL char*)p.w + batch * p.w_bs * EB;
  const VECOPS_GLOBAL char* xrow =
      (const VECOPS_GLOBAL char*)p.x + (batch * p.x_bs + static_cast<int64_t>(min(row, p.s - 1)) * p.ldx) * EB;
  // rows past R are clamped: computed, never stored
  const VECOPS_GLOBAL char* wrow[BLOCKS];
#pragma unroll
  for (int b = 0; b < BLOCKS; ++b) wrow[b] = wbase + min(row0 + b * 16 + row, last_row) * p.ldw * EB;

  Acc4 acc[BLOCKS];
#pragma unroll
  for (int b = 0; b < BLOCKS; ++b) acc[b] = Acc4{0, 0, 0, 0};

  const int k_blocks = (p.k + 128 * EPS - 1) / (128 * EPS);
  for (int kb = 0; kb < k_blocks; ++kb) {
    // k of (step s of this wavefront, this lane's quarter) in this K block
    auto k_of = [&](int s) { return (kb * 128 + s * WAVES + wave) * EPS + quarter * EPL; };
    u32x4 xq[XS];
#pragma unroll
    for (int s = 0; s < XS; ++s) {
      const int k0 = k_of(s);
      xq[s] = u32x4{0u, 0u, 0u, 0u};
      if (row < p.s && k0 < p.k) {
        Loaded raw;
        load_of(xrow + static_cast<int64_t>(k0) * EB, raw);
        xq[s] = operand_of(raw);
      }
    }
    // flat sequence of (block, step) with the wide loads D ahead; a load past K reads as zero
    Loaded wq[D];
    auto issue = [&](auto slot_tag, auto b_tag, auto s_tag) {
      constexpr int slot = decltype(slot_tag)::value, b = decltype(b_tag)::value, s = decltype(s_tag)::value;
      if constexpr (b < BLOCKS) {
        const int k0 = k_of(s);
#pragma unroll
        for (int i = 0; i < LOADS; ++i) wq[slot].v[i] = u32x4{0u, 0u, 0u, 0u};
        if (k0 < p.k) load_of(wrow[b] + static_cast<int64_t>(k0) * EB, wq[slot]);
      }
    };
    static_for<D>([&](auto u) { issue(u, std::integral_constant<int, 0>{}, u); });
    static_for<BLOCKS>([&](auto cb) {
      constexpr int b = decltype(cb)::value;
      static_for<XS>([&](auto cs) {
        constexpr int s = decltype(cs)::value, slot = s % D;
        const u32x4 wv = operand_of(wq[slot]);
        if constexpr (INT)
          acc[b] = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(i32x4, wv),
                                                         __builtin_bit_cast(i32x4, xq[s]), acc[b], 0, 0, 0);
        else if constexpr (SRC == SRC_F16) {
          typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
          acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, wv),
                                                          __builtin_bit_cast(f16x8, xq[s]), acc[b], 0, 0, 0);
        } else if constexpr (SRC == SRC_F32) {
          // four floats per lane: MFMA e multiplies element e of every lane (the same k on both sides)
          acc[b] = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(wv[0]), __uint_as_float(xq[s][0]), acc[b], 0, 0, 0);
          acc[b] = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(wv[1]), __uint_as_float(xq[s][1]), acc[b], 0, 0, 0);
          acc[b] = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(wv[2]), __uint_as_float(xq[s][2]), acc[b], 0, 0, 0);
          acc[b] = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(wv[3]), __uint_as_float(xq[s][3]), acc[b], 0, 0, 0);
        } else
          acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wv),
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
      AccScalar total = 0;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) {
        if constexpr (INT) total = static_cast<int32_t>(static_cast<uint32_t>(total) + static_cast<uint32_t>(red[w][b][(quarter * 4 + r) * 16 + row]));
        else total += red[w][b][(quarter * 4 + r) * 16 + row];
      }
      const int64_t n = row0 + b * 16 + quarter * 4 + r;
      if (row < p.s && n < p.rows) {
        const int64_t at = batch * p.y_bs + n * p.y_stride_r + row * p.y_stride_s;
        if constexpr (INT) {
          if (p.out_kind == SKINNY_OUT_DEQUANT_F32) {
            const uint32_t term = p.wide_term ? static_cast<uint32_t>(p.wide_term[n]) : 0u;
            const float t = static_cast<float>(static_cast<int32_t>(static_cast<uint32_t>(total) + term)) * p.narrow_scales[row];
            static_cast<float*>(p.y)[at] = t * p.wide_scales[n];  // two separately rounded multiplies, row scale first
          } else {
            static_cast<int32_t*>(p.y)[at] = total;
          }
        } else {
          if (p.out_kind == SKINNY_OUT_BF16) static_cast<uint16_t*>(p.y)[at] = static_cast<uint16_t>(bf16_bits_rne(total));
          else if (p.out_kind == SKINNY_OUT_F16) static_cast<uint16_t*>(p.y)[at] = static_cast<uint16_t>(f16_bits_rne(total));
          else static_cast<float*>(p.y)[at] = total;
        }
      }
    }
  }
}

}  // namespace vecops_hip
#endif
