// Decode-shaped weight-only int8 matmul for gfx950 (HBM-bound):
//   y[m,n] = bf16( sum_g S[n,g] * sum_{k in g} float(x[m,k]) * float(W[n,k]) ),  M <= 16.
//
// The weight matrix is read exactly once, 16 bytes per lane per load, a whole
// wavefront reading 1 KiB contiguous of one weight row.  A wavefront owns ROWS
// consecutive weight rows and walks K in steps of 1024 elements; the activation
// chunk a lane needs (the same k range for every row) is loaded once per step
// and reused for all ROWS rows, so activations cost 1/ROWS of the weight
// traffic from cache.  Products and sums are fp32 (fmaf); the group scale
// multiplies the 16-element partial sum of a lane, which never straddles a group
// because the group size is a multiple of 16.  The per-lane sums are reduced
// across the wavefront with DPP-free shuffles at the end.
#ifndef VECOPS_HIP_SKINNY_W8A16_H
#define VECOPS_HIP_SKINNY_W8A16_H

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "tile_gemm.h"

namespace vecops_hip {

struct SkinnyW8A16Params {
  const uint16_t* x;  // bf16 bits
  const int8_t* w;
  const float* scales;
  uint16_t* y;
  int64_t ldx, ldw, ldy;
  int32_t m, n, k, group;
  int32_t groups;  // k / group
};

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

template <int MB, int ROWS>
__global__ __launch_bounds__(256) void skinny_w8a16_kernel(const SkinnyW8A16Params p) {
  const int lane = threadIdx.x & 63;
  const int wave_in_block = threadIdx.x >> 6;
  const int64_t wave_id = static_cast<int64_t>(blockIdx.x) * 4 + wave_in_block;
  const int64_t n0 = wave_id * ROWS;
  if (n0 >= p.n) return;

  float acc[ROWS][MB];
#pragma unroll
  for (int r = 0; r < ROWS; ++r)
#pragma unroll
    for (int mm = 0; mm < MB; ++mm) acc[r][mm] = 0.0f;

  const int chunks = p.k >> 4;
  for (int c0 = 0; c0 < chunks; c0 += 64) {
    const int c = c0 + lane;
    const bool active = c < chunks;
    const int k0 = c << 4;
    // weights first: ROWS independent 16-byte loads in flight per lane
    u32x4 wq[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      const int64_t n = n0 + r;
      wq[r] = u32x4{0u, 0u, 0u, 0u};
      if (active && n < p.n) wq[r] = *reinterpret_cast<const u32x4*>(p.w + n * p.ldw + k0);
    }
    const int g = active ? k0 / p.group : 0;
    float sc[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      const int64_t n = n0 + r;
      sc[r] = (active && n < p.n) ? p.scales[n * p.groups + g] : 0.0f;
    }
    // activations: 16 bf16 per row of x, widened to fp32
    float xf[MB][16];
#pragma unroll
    for (int mm = 0; mm < MB; ++mm) {
      u32x4 lo = {0u, 0u, 0u, 0u}, hi = {0u, 0u, 0u, 0u};
      if (active && mm < p.m) {
        const u32x4* px = reinterpret_cast<const u32x4*>(p.x + mm * p.ldx + k0);
        lo = px[0];
        hi = px[1];
      }
      const uint32_t words[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        xf[mm][2 * e] = __uint_as_float(words[e] << 16);
        xf[mm][2 * e + 1] = __uint_as_float(words[e] & 0xffff0000u);
      }
    }
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
      const uint32_t words[4] = {wq[r].x, wq[r].y, wq[r].z, wq[r].w};
      float wf[16];
#pragma unroll
      for (int e = 0; e < 16; ++e)
        wf[e] = static_cast<float>(static_cast<int8_t>((words[e >> 2] >> ((e & 3) * 8)) & 0xffu));
#pragma unroll
      for (int mm = 0; mm < MB; ++mm) {
        float part = 0.0f;
#pragma unroll
        for (int e = 0; e < 16; ++e) part = fmaf(xf[mm][e], wf[e], part);
        acc[r][mm] = fmaf(sc[r], part, acc[r][mm]);
      }
    }
  }

#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
#pragma unroll
    for (int mm = 0; mm < MB; ++mm) {
      const float total = wave_sum(acc[r][mm]);
      const int64_t n = n0 + r;
      if (lane == 0 && mm < p.m && n < p.n) p.y[mm * p.ldy + n] = static_cast<uint16_t>(bf16_bits_rne(total));
    }
  }
}

}  // namespace vecops_hip
#endif
