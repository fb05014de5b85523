// Decode-shaped weight-only int8 matmul for gfx950 (HBM-bound):
//   y[m,n] = bf16( sum_g S[n,g] * sum_{k in g} float(x[m,k]) * float(W[n,k]) ),  M <= 16.
//
// The weight matrix is read exactly once.  Two kernel families:
//  * dot-product (M <= 2, or group sizes that are not multiples of 64): a
//    wavefront owns ROWS consecutive weight rows and reads 1 KiB contiguous of one
//    row per load instruction (16 bytes per lane); products and sums in fp32 on the
//    vector ALU.
//  * matrix-core (M = 3..16): 16 weight rows x 16 activation rows per
//    v_mfma_f32_16x16x32_bf16, so the cost of widening a weight byte is paid once
//    for all activation rows.
// Both widen weights with the unsigned-byte converter, u = w xor 0x80 = w + 128, and
// use  sum_k x_k*w_k = sum_k x_k*u_k - 128 * sum_k x_k  per scale group; a lane's
// 16-element chunk never straddles a group because group sizes are multiples of 16.
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

// ---- dot-product family (VALU): one wavefront owns ROWS consecutive weight rows ----------
template <int MB, int ROWS, int UNROLL>
__global__ __launch_bounds__(256) void skinny_w8a16_kernel(const SkinnyW8A16Params p) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int64_t n0 = (static_cast<int64_t>(blockIdx.x) * 4 + wave) * ROWS;
  if (n0 >= p.n) return;
  const int chunks = p.k >> 4;  // 16-element chunks per row
  const VECOPS_GLOBAL char* wbase = (const VECOPS_GLOBAL char*)p.w;
  const VECOPS_GLOBAL uint16_t* xbase = (const VECOPS_GLOBAL uint16_t*)p.x;
  const VECOPS_GLOBAL float* sbase = (const VECOPS_GLOBAL float*)p.scales;

  float acc[ROWS][MB];
#pragma unroll
  for (int r = 0; r < ROWS; ++r)
#pragma unroll
    for (int mm = 0; mm < MB; ++mm) acc[r][mm] = 0.0f;

  for (int c0 = 0; c0 < chunks; c0 += 64 * UNROLL) {
    // all weight loads of this step first
    u32x4 wq[UNROLL][ROWS];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int c = c0 + u * 64 + lane;
#pragma unroll
      for (int r = 0; r < ROWS; ++r) {
        const int64_t n = n0 + r;
        wq[u][r] = u32x4{0x80808080u, 0x80808080u, 0x80808080u, 0x80808080u};  // reads as w == 0
        if (c < chunks && n < p.n)
          wq[u][r] = *(const VECOPS_GLOBAL u32x4*)(wbase + n * p.ldw + (static_cast<int64_t>(c) << 4));
      }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int c = c0 + u * 64 + lane;
      const bool active = c < chunks;
      const int k0 = c << 4;
      const int g = active ? k0 / p.group : 0;
      float sc[ROWS];
#pragma unroll
      for (int r = 0; r < ROWS; ++r) {
        const int64_t n = n0 + r;
        sc[r] = (active && n < p.n) ? sbase[n * p.groups + g] : 0.0f;
      }
      // activations: 16 bf16 per row of x, widened to fp32, and their sum
      float xf[MB][16], xsum[MB];
#pragma unroll
      for (int mm = 0; mm < MB; ++mm) {
        u32x4 lo = {0u, 0u, 0u, 0u}, hi = {0u, 0u, 0u, 0u};
        if (active && mm < p.m) {
          const VECOPS_GLOBAL u32x4* px = (const VECOPS_GLOBAL u32x4*)(xbase + mm * p.ldx + k0);
          lo = px[0];
          hi = px[1];
        }
        const uint32_t words[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
        float s = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          xf[mm][2 * e] = __uint_as_float(words[e] << 16);
          xf[mm][2 * e + 1] = __uint_as_float(words[e] & 0xffff0000u);
          s += xf[mm][2 * e];
          s += xf[mm][2 * e + 1];
        }
        xsum[mm] = s;
      }
#pragma unroll
      for (int r = 0; r < ROWS; ++r) {
        const uint32_t words[4] = {wq[u][r].x ^ 0x80808080u, wq[u][r].y ^ 0x80808080u, wq[u][r].z ^ 0x80808080u,
                                   wq[u][r].w ^ 0x80808080u};
        float wf[16];
#pragma unroll
        for (int e = 0; e < 16; ++e) wf[e] = static_cast<float>((words[e >> 2] >> ((e & 3) * 8)) & 0xffu);
#pragma unroll
        for (int mm = 0; mm < MB; ++mm) {
          float part = -128.0f * xsum[mm];
#pragma unroll
          for (int e = 0; e < 16; ++e) part = fmaf(xf[mm][e], wf[e], part);
          acc[r][mm] = fmaf(sc[r], part, acc[r][mm]);
        }
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

// ---- M = 1, streaming: a wavefront walks many weight rows with the next row's loads in flight --------
// K = CH x 1024: lane l owns the 16-element chunks u * 64 + l (u < CH) of every row, exactly as in the
// dot-product kernel above, so the sums are taken in the same order and the results are the same
// bits.  The activations of the lane's chunks (widened to fp32) and their sums stay in registers for
// the whole kernel; wavefront w takes rows w, w + W, w + 2W, ... (W wavefronts in the grid), so that at
// any moment the grid reads one contiguous run of rows; a row's CH weight loads and CH scale loads are
// issued one row ahead of its arithmetic (two rows ahead measured 10 % slower).  The dot-product
// kernel's grid starts every wavefront at the same moment - all of them load, then all of them
// compute; here each wavefront overlaps the two.
template <int CH>
__global__ __launch_bounds__(256) void skinny_w8a16_stream_kernel(const SkinnyW8A16Params p) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  const int64_t waves = static_cast<int64_t>(gridDim.x) * 4;
  const VECOPS_GLOBAL char* wbase = (const VECOPS_GLOBAL char*)p.w;
  const VECOPS_GLOBAL uint16_t* xbase = (const VECOPS_GLOBAL uint16_t*)p.x;
  const VECOPS_GLOBAL float* sbase = (const VECOPS_GLOBAL float*)p.scales;

  int group_of[CH];
#pragma unroll
  for (int u = 0; u < CH; ++u) group_of[u] = ((u * 64 + lane) << 4) / p.group;

  u32x4 wq[2][CH];
  float sc[2][CH];
  auto fetch = [&](int set, int64_t n) {
    // rows past N are clamped: computed, never stored
    const int64_t row = n < p.n ? n : p.n - 1;
#pragma unroll
    for (int u = 0; u < CH; ++u) {
      wq[set][u] = *(const VECOPS_GLOBAL u32x4*)(wbase + row * p.ldw + (static_cast<int64_t>(u * 64 + lane) << 4));
      sc[set][u] = sbase[row * p.groups + group_of[u]];
    }
  };
  if (wave >= p.n) return;
  // the first row's weights are requested before the activations: they arrive while those are fetched and widened
  fetch(0, wave);

  float xf[CH][16], xsum[CH];
#pragma unroll
  for (int u = 0; u < CH; ++u) {
    const int k0 = (u * 64 + lane) << 4;
    const VECOPS_GLOBAL u32x4* px = (const VECOPS_GLOBAL u32x4*)(xbase + k0);
    const u32x4 lo = px[0], hi = px[1];
    const uint32_t words[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    float s = 0.0f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      xf[u][2 * e] = __uint_as_float(words[e] << 16);
      xf[u][2 * e + 1] = __uint_as_float(words[e] & 0xffff0000u);
      s += xf[u][2 * e];
      s += xf[u][2 * e + 1];
    }
    xsum[u] = s;
  }

  auto finish = [&](int set, int64_t n) {
    float acc = 0.0f;
#pragma unroll
    for (int u = 0; u < CH; ++u) {
      const uint32_t words[4] = {wq[set][u].x ^ 0x80808080u, wq[set][u].y ^ 0x80808080u, wq[set][u].z ^ 0x80808080u,
                                 wq[set][u].w ^ 0x80808080u};
      float part = -128.0f * xsum[u];
#pragma unroll
      for (int e = 0; e < 16; ++e)
        part = fmaf(xf[u][e], static_cast<float>((words[e >> 2] >> ((e & 3) * 8)) & 0xffu), part);
      acc = fmaf(sc[set][u], part, acc);
    }
    const float total = wave_sum(acc);
    if (lane == 0 && n < p.n) p.y[n] = static_cast<uint16_t>(bf16_bits_rne(total));
  };

  int64_t n = wave;
  // two rows per trip so that the register set of a row is a compile-time choice
  for (; n + waves < p.n; n += 2 * waves) {
    fetch(1, n + waves);
    finish(0, n);
    fetch(0, n + 2 * waves);
    finish(1, n + waves);
  }
  if (n < p.n) finish(0, n);
}

// ---- M = 2, streaming: the M = 1 walk over the weight rows with MT activation rows resident ----------
// K = CH x 1024.  The activations of a lane's chunks, widened to fp32, take MT x CH x 16 registers, which
// is what limits MT to 2 at two wavefronts per SIMD.  A weight byte is widened once (u = w + 128,
// -128 * sum_k x per 16-element chunk, as in the M = 1 kernel) and multiplied into MT sums.  More rows run
// into the vector ALU: at N = 14336 one row takes 12.2 us, two 13.9; four rows - K shared between two
// wavefronts that meet in LDS - took 25 us, and v_dot2c_f32_bf16 on packed activations 19.7 (it issues at
// a quarter of the rate), so three rows and more stay with the matrix-core kernels below.  The code the
// compiler makes of this loop is touchy: with the wavefront's number in a vector register (row addresses
// as vector arithmetic) two rows took 20.4 us, and with a trip count shared by all wavefronts (an eighth,
// clamped row for each at N = 14336) 15.8.
template <int MT, int CH>
__global__ __launch_bounds__(256) void skinny_w8a16_stream_rows_kernel(const SkinnyW8A16Params p) {
  const int lane = threadIdx.x & 63;
  // (the wavefront's number in a scalar register: row addresses are then scalar arithmetic)
  const int64_t wave = static_cast<int64_t>(blockIdx.x) * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t waves = static_cast<int64_t>(gridDim.x) * 4;
  const VECOPS_GLOBAL char* wbase = (const VECOPS_GLOBAL char*)p.w;
  const VECOPS_GLOBAL float* sbase = (const VECOPS_GLOBAL float*)p.scales;

  float xf[MT][CH][16], xsum[MT][CH];
  int group_of[CH];
#pragma unroll
  for (int u = 0; u < CH; ++u) {
    const int k0 = (u * 64 + lane) << 4;
    group_of[u] = k0 / p.group;
#pragma unroll
    for (int mm = 0; mm < MT; ++mm) {
      const VECOPS_GLOBAL uint16_t* xrow = (const VECOPS_GLOBAL uint16_t*)p.x + static_cast<int64_t>(min(mm, p.m - 1)) * p.ldx;
      const VECOPS_GLOBAL u32x4* px = (const VECOPS_GLOBAL u32x4*)(xrow + k0);
      const u32x4 lo = px[0], hi = px[1];
      const uint32_t words[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
      float sum = 0.0f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        xf[mm][u][2 * e] = __uint_as_float(words[e] << 16);
        xf[mm][u][2 * e + 1] = __uint_as_float(words[e] & 0xffff0000u);
        sum += xf[mm][u][2 * e];
        sum += xf[mm][u][2 * e + 1];
      }
      xsum[mm][u] = sum;
    }
  }

  u32x4 wq[2][CH];
  float sc[2][CH];
  auto fetch = [&](int set, int64_t n) {
    const int64_t row = n < p.n ? n : p.n - 1;  // rows past N are clamped: computed, never stored
#pragma unroll
    for (int u = 0; u < CH; ++u) {
      wq[set][u] = *(const VECOPS_GLOBAL u32x4*)(wbase + row * p.ldw + (static_cast<int64_t>(u * 64 + lane) << 4));
      sc[set][u] = sbase[row * p.groups + group_of[u]];
    }
  };
  auto finish = [&](int set, int64_t n) {
    float acc[MT];
#pragma unroll
    for (int mm = 0; mm < MT; ++mm) acc[mm] = 0.0f;
#pragma unroll
    for (int u = 0; u < CH; ++u) {
      const uint32_t words[4] = {wq[set][u].x ^ 0x80808080u, wq[set][u].y ^ 0x80808080u, wq[set][u].z ^ 0x80808080u,
                                 wq[set][u].w ^ 0x80808080u};
      float part[MT];
#pragma unroll
      for (int mm = 0; mm < MT; ++mm) part[mm] = -128.0f * xsum[mm][u];
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const float wf = static_cast<float>((words[e >> 2] >> ((e & 3) * 8)) & 0xffu);
#pragma unroll
        for (int mm = 0; mm < MT; ++mm) part[mm] = fmaf(xf[mm][u][e], wf, part[mm]);
      }
#pragma unroll
      for (int mm = 0; mm < MT; ++mm) acc[mm] = fmaf(sc[set][u], part[mm], acc[mm]);
    }
#pragma unroll
    for (int mm = 0; mm < MT; ++mm) {
      const float total = wave_sum(acc[mm]);
      if (lane == 0 && mm < p.m && n < p.n)
        p.y[static_cast<int64_t>(mm) * p.ldy + n] = static_cast<uint16_t>(bf16_bits_rne(total));
    }
  };

  if (wave >= p.n) return;
  fetch(0, wave);
  int64_t n = wave;
  // two rows per trip so that the register set of a row is a compile-time choice
  for (; n + waves < p.n; n += 2 * waves) {
    fetch(1, n + waves);
    finish(0, n);
    fetch(0, n + 2 * waves);
    finish(1, n + waves);
  }
  if (n < p.n) finish(0, n);
}

// ---- matrix-core family: a workgroup owns TILES x 16 weight rows, its WAVES wavefronts
// split K by scale groups --------------------------------------------------------------------
// One v_mfma_f32_16x16x32_bf16 multiplies 16 weight rows x 32 k by 32 k x 16
// activation rows (M padded to 16 with zeros).  Lane l holds weight row l % 16 and
// the 16 consecutive k of quarter l / 16 of a 64-element step (one 16-byte load),
// which feed two MFMAs; the activation operand uses the same k order.  Weights are
// widened byte -> fp32 -> bf16 (exact for 0..255) as u = w + 128, and a second
// MFMA against an all-ones operand accumulates sum_k x[m,k] of the group, so that
//   acc += S[n,g] * (sum_k u*x - 128 * sum_k x).
// Loads run D = 4 steps ahead of their use (flat software pipeline across groups).
// SPG = 64-element steps per scale group (group size / 64).
template <int WAVES, int SPG, int TILES>
__global__ __launch_bounds__(64 * WAVES) void skinny_w8a16_mfma_kernel(const SkinnyW8A16Params p) {
  constexpr int D = 4;
  static_assert(D % SPG == 0, "pipeline depth must hold whole groups");
  __shared__ float red[WAVES][TILES][16 * 16];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int64_t n0 = static_cast<int64_t>(blockIdx.x) * (16 * TILES);
  const int row = lane & 15, quarter = lane >> 4;
  const int gpw = (p.groups + WAVES - 1) / WAVES;
  const int g_begin = min(p.groups, wave * gpw), g_end = min(p.groups, g_begin + gpw);
  const int total = (g_end - g_begin) * SPG;  // steps of this wavefront
  // rows past N are clamped: computed, never stored
  const VECOPS_GLOBAL char* wrow[TILES];
  const VECOPS_GLOBAL float* srow[TILES][4];
#pragma unroll
  for (int t = 0; t < TILES; ++t) {
    const int64_t n = min(n0 + t * 16 + row, static_cast<int64_t>(p.n) - 1);
    wrow[t] = (const VECOPS_GLOBAL char*)p.w + n * p.ldw + quarter * 16 + static_cast<int64_t>(g_begin) * SPG * 64;
#pragma unroll
    for (int r = 0; r < 4; ++r)
      srow[t][r] = (const VECOPS_GLOBAL float*)p.scales +
                   min(n0 + t * 16 + quarter * 4 + r, static_cast<int64_t>(p.n) - 1) * p.groups + g_begin;
  }
  const VECOPS_GLOBAL char* xrow = (const VECOPS_GLOBAL char*)(p.x + static_cast<int64_t>(min(row, p.m - 1)) * p.ldx) +
                                   quarter * 32 + static_cast<int64_t>(g_begin) * SPG * 128;
  const bool x_ok = row < p.m;

  f32x4 acc[TILES], dot[TILES], xs = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int t = 0; t < TILES; ++t) {
    acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    dot[t] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  const u32x4 ones = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};  // eight bf16 1.0
  u32x4 wq[D][TILES], x1[D], x2[D];
  float sc[D / SPG][TILES][4];

  auto issue = [&](auto slot_tag, int step) {
    constexpr int slot = decltype(slot_tag)::value;
    if (step < total) {
#pragma unroll
      for (int t = 0; t < TILES; ++t) wq[slot][t] = *(const VECOPS_GLOBAL u32x4*)(wrow[t] + static_cast<int64_t>(step) * 64);
      x1[slot] = u32x4{0u, 0u, 0u, 0u};
      x2[slot] = u32x4{0u, 0u, 0u, 0u};
      if (x_ok) {
        const VECOPS_GLOBAL u32x4* px = (const VECOPS_GLOBAL u32x4*)(xrow + static_cast<int64_t>(step) * 128);
        x1[slot] = px[0];
        x2[slot] = px[1];
      }
      // the group's scales ride with its last step: consumed there, free when the slot is reissued
      if constexpr (slot % SPG == SPG - 1) {
#pragma unroll
        for (int t = 0; t < TILES; ++t)
#pragma unroll
          for (int r = 0; r < 4; ++r) sc[slot / SPG][t][r] = srow[t][r][step / SPG];
      }
    }
  };
  auto consume = [&](auto slot_tag, int step) {
    constexpr int slot = decltype(slot_tag)::value;
    if (step < total) {
      const bf16x8 b1 = __builtin_bit_cast(bf16x8, x1[slot]), b2 = __builtin_bit_cast(bf16x8, x2[slot]);
#pragma unroll
      for (int t = 0; t < TILES; ++t) {
        uint32_t a[8];
        const uint32_t wd[4] = {wq[slot][t].x ^ 0x80808080u, wq[slot][t].y ^ 0x80808080u, wq[slot][t].z ^ 0x80808080u,
                                wq[slot][t].w ^ 0x80808080u};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float f0 = static_cast<float>(wd[q] & 0xffu), f1 = static_cast<float>((wd[q] >> 8) & 0xffu);
          const float f2 = static_cast<float>((wd[q] >> 16) & 0xffu), f3 = static_cast<float>(wd[q] >> 24);
          // upper halves of two fp32 = two bf16 (exact: the values are integers below 256)
          a[2 * q] = __builtin_amdgcn_perm(__float_as_uint(f1), __float_as_uint(f0), 0x07060302u);
          a[2 * q + 1] = __builtin_amdgcn_perm(__float_as_uint(f3), __float_as_uint(f2), 0x07060302u);
        }
        const u32x4 a1 = {a[0], a[1], a[2], a[3]}, a2 = {a[4], a[5], a[6], a[7]};
        dot[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a1), b1, dot[t], 0, 0, 0);
        dot[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a2), b2, dot[t], 0, 0, 0);
      }
      xs = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, ones), b1, xs, 0, 0, 0);
      xs = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, ones), b2, xs, 0, 0, 0);
      if constexpr (slot % SPG == SPG - 1) {
#pragma unroll
        for (int t = 0; t < TILES; ++t)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            acc[t][r] = fmaf(sc[slot / SPG][t][r], fmaf(-128.0f, xs[r], dot[t][r]), acc[t][r]);
            dot[t][r] = 0.0f;
          }
#pragma unroll
        for (int r = 0; r < 4; ++r) xs[r] = 0.0f;
      }
    }
  };

  static_for<D>([&](auto u) { issue(u, decltype(u)::value); });
  for (int s = 0; s < total; s += D) {
    static_for<D>([&](auto u) {
      consume(u, s + decltype(u)::value);
      issue(u, s + D + decltype(u)::value);
    });
  }

  // Sum the K slices through LDS.  Accumulator register r of lane l is output
  // (weight row quarter*4 + r, activation row l % 16) of its 16x16 tile.
#pragma unroll
  for (int t = 0; t < TILES; ++t)
#pragma unroll
    for (int r = 0; r < 4; ++r) red[wave][t][(quarter * 4 + r) * 16 + row] = acc[t][r];
  __syncthreads();
  if (wave == 0) {
#pragma unroll
    for (int t = 0; t < TILES; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float total_sum = 0.0f;
        for (int w = 0; w < WAVES; ++w) total_sum += red[w][t][(quarter * 4 + r) * 16 + row];
        const int64_t n = n0 + t * 16 + quarter * 4 + r;
        if (row < p.m && n < p.n)
          p.y[static_cast<int64_t>(row) * p.ldy + n] = static_cast<uint16_t>(bf16_bits_rne(total_sum));
      }
  }
}

// ---- matrix-core family, activations resident in registers -------------------------------------
// Same arithmetic and operand layout as skinny_w8a16_mfma_kernel, for K = 8 wavefronts
// x 8 steps x 64 (4096).  In that kernel every step carries, besides its weight loads,
// two activation loads and its share of the scale loads - four of five memory
// instructions fetch data that is not weights.  Here a wavefront fetches the activation
// rows of its K slice once - one load instruction per row, 1 KiB contiguous, written
// straight into LDS, from where they come back as matrix-core fragments (64 registers;
// fetching the fragments themselves, 64 bytes of each of 16 rows per instruction, cost
// 3 us of 18 at M = 16: twice the cache lines per byte, in a memory pipeline that the
// weights keep full) - and keeps them while the workgroup walks PASSES consecutive blocks
// of TILES x 16 weight rows; the scales of a block arrive as one coalesced 4-byte load per
// lane (lane = row + 16 * group) and are handed to the lanes that need them with lane
// permutes.  The steps of all passes form one flat sequence with loads D = 4 steps ahead.
// The K slices of every pass wait in LDS (in the wavefront's own activation rows, which are
// dead by then) and are summed behind ONE barrier at the end: with a barrier per pass every
// wavefront waited for the slowest of its workgroup, 1.7 us per pass measured inside the
// kernel, with no new loads going out meanwhile.
template <int SPG, int TILES, int PASSES>
__global__ __launch_bounds__(512) void skinny_w8a16_mfma_resident_kernel(const SkinnyW8A16Params p) {
  constexpr int WAVES = 8, S = 8, D = 4;  // a deeper pipeline (D = 8) measured no faster
  constexpr int GPW = S / SPG;                      // scale groups of a wavefront's K slice
  constexpr int NSC = (16 * GPW + 63) / 64;         // scale registers per tile
  static_assert(S % SPG == 0 && D % SPG == 0, "whole groups per pipeline round");
  constexpr int XPITCH = 1024 + 16;   // bytes between the activation rows of a wavefront's K slice in LDS
  __shared__ __attribute__((aligned(16))) char xlds[WAVES][16 * XPITCH];
  static_assert(PASSES * TILES * 1024 <= 16 * XPITCH, "a wavefront's partial sums reuse its own staging rows");
  constexpr int passes = PASSES;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int row = lane & 15, quarter = lane >> 4;
  const int64_t wg_row0 = static_cast<int64_t>(blockIdx.x) * passes * (16 * TILES);
  const int64_t last_row = static_cast<int64_t>(p.n) - 1;
  const int g_begin = wave * GPW;
  // Weight loads: lanes 4r .. 4r + 3 fetch the four 16-byte quarters of row r's 64-byte step - one contiguous 64-byte
  // request per group of four lanes instead of four lines touched by it - and a lane permute
  // puts the quarters where the matrix cores want them (lane i + 16q: row i, quarter q).
  const int load_row = lane >> 2;
  const VECOPS_GLOBAL char* wbase = (const VECOPS_GLOBAL char*)p.w + (lane & 3) * 16 + static_cast<int64_t>(wave) * S * 64;
  const int from_lane_bytes = (4 * row + quarter) * 4;  // ds_bpermute address of the lane that loaded (row, quarter)
  const VECOPS_GLOBAL float* sbase = (const VECOPS_GLOBAL float*)p.scales;

  // activation fragments of this K slice, resident for the whole kernel
  u32x4 x1[S], x2[S];

  const u32x4 ones = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};  // eight bf16 1.0
  u32x4 wq[D][TILES];
  float sc_cur[TILES][NSC], sc_nxt[TILES][NSC] = {};
  f32x4 acc[TILES], dot[TILES], xs = {0.f, 0.f, 0.f, 0.f};
  const int total = passes * S;

  // rows past N are clamped: computed, never stored
  auto weight_row = [&](int pass, int t) { return min(wg_row0 + (pass * TILES + t) * 16 + row, last_row); };
  auto loaded_row = [&](int pass, int t) { return min(wg_row0 + (pass * TILES + t) * 16 + load_row, last_row); };
  auto load_scales = [&](float (&dst)[TILES][NSC], int pass) {
#pragma unroll
    for (int t = 0; t < TILES; ++t)
#pragma unroll
      for (int i = 0; i < NSC; ++i) {
        const int h = i * 64 + lane;  // holder index = row + 16 * group
        const int g = min(h >> 4, GPW - 1);
        dst[t][i] = sbase[weight_row(pass, t) * p.groups + g_begin + g];
      }
  };
  auto issue = [&](auto slot_tag, int step) {
    constexpr int slot = decltype(slot_tag)::value;
    if (step < total) {
      const int pass = step / S, s = step - pass * S;
#pragma unroll
      for (int t = 0; t < TILES; ++t)
        wq[slot][t] = *(const VECOPS_GLOBAL u32x4*)(wbase + loaded_row(pass, t) * p.ldw + s * 64);
    }
  };
  // S is a multiple of D: slot `slot` always holds step s = slot or slot + D of its pass
  auto consume = [&](auto slot_tag, auto s_tag, int pass) {
    constexpr int slot = decltype(slot_tag)::value, s = decltype(s_tag)::value;
    const bf16x8 b1 = __builtin_bit_cast(bf16x8, x1[s]), b2 = __builtin_bit_cast(bf16x8, x2[s]);
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
      uint32_t a[8];
      const uint32_t raw[4] = {wq[slot][t].x, wq[slot][t].y, wq[slot][t].z, wq[slot][t].w};
      uint32_t wd[4];
#pragma unroll
      for (int q = 0; q < 4; ++q)
        wd[q] = static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(from_lane_bytes, static_cast<int>(raw[q]))) ^ 0x80808080u;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const float f0 = static_cast<float>(wd[q] & 0xffu), f1 = static_cast<float>((wd[q] >> 8) & 0xffu);
        const float f2 = static_cast<float>((wd[q] >> 16) & 0xffu), f3 = static_cast<float>(wd[q] >> 24);
        // upper halves of two fp32 = two bf16 (exact: the values are integers below 256)
        a[2 * q] = __builtin_amdgcn_perm(__float_as_uint(f1), __float_as_uint(f0), 0x07060302u);
        a[2 * q + 1] = __builtin_amdgcn_perm(__float_as_uint(f3), __float_as_uint(f2), 0x07060302u);
      }
      const u32x4 a1 = {a[0], a[1], a[2], a[3]}, a2 = {a[4], a[5], a[6], a[7]};
      dot[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a1), b1, dot[t], 0, 0, 0);
      dot[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a2), b2, dot[t], 0, 0, 0);
    }
    xs = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, ones), b1, xs, 0, 0, 0);
    xs = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, ones), b2, xs, 0, 0, 0);
    if constexpr (s % SPG == SPG - 1) {
      constexpr int g = s / SPG;
#pragma unroll
      for (int t = 0; t < TILES; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          // the scale of (weight row quarter*4 + r, group g) sits in lane (quarter*4 + r) + 16*g of its register
          const int h = quarter * 4 + r + 16 * g;
          const float scale = __shfl(sc_cur[t][(16 * g) / 64], h & 63, 64);
          acc[t][r] = fmaf(scale, fmaf(-128.0f, xs[r], dot[t][r]), acc[t][r]);
          dot[t][r] = 0.0f;
        }
#pragma unroll
      for (int r = 0; r < 4; ++r) xs[r] = 0.0f;
    }
    (void)pass;
  };

  // the first weights are requested before the activations: they arrive while those are fetched
  // start-up: the wavefront's K slice of every activation row goes into LDS by loads that write LDS themselves - one
  // instruction per row, 1 KiB contiguous - and comes back as matrix-core fragments (lane = row + 16 * quarter)
  {
    const __amdgpu_buffer_rsrc_t xbuf = tile_buffer((const VECOPS_GLOBAL char*)p.x);
    char* mine = xlds[wave];
#pragma unroll
    for (int r = 0; r < 16; ++r)
      if (r < p.m)
        load_16_bytes_into_lds_counted(xbuf, (lds_void_ptr)(mine + r * XPITCH), static_cast<uint32_t>(lane * 16),
                                       __builtin_amdgcn_readfirstlane(static_cast<uint32_t>((r * p.ldx + wave * S * 64) * 2)));
  }
  asm volatile("" ::: "memory");  // (the weight loads stay behind the loads above)
  static_for<D>([&](auto u) {
    issue(u, decltype(u)::value);
    if constexpr (decltype(u)::value == 0) load_scales(sc_cur, 0);
  });
  {
    // The loads that write LDS are counted with the loads issued behind them, in order: at least D * TILES weight
    // loads follow, so "at most D * TILES - TILES still in flight" means the activations (and the first step's
    // weights) have landed.  Through a statement the compiler moves no memory access across.
    static_assert(D * TILES - TILES == 6, "the wait below is written for six");
    asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
    const char* mine = xlds[wave] + row * XPITCH + quarter * 32;
#pragma unroll
    for (int s = 0; s < S; ++s) {
      const u32x4 a = *reinterpret_cast<const u32x4*>(mine + s * 128), b = *reinterpret_cast<const u32x4*>(mine + s * 128 + 16);
      x1[s] = row < p.m ? a : u32x4{0u, 0u, 0u, 0u};
      x2[s] = row < p.m ? b : u32x4{0u, 0u, 0u, 0u};
    }
  }
  for (int pass = 0; pass < passes; ++pass) {
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
      acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
      dot[t] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    if (pass + 1 < passes) load_scales(sc_nxt, pass + 1);
    static_for<S>([&](auto cs) {
      constexpr int s = decltype(cs)::value;
      consume(std::integral_constant<int, s % D>{}, cs, pass);
      issue(std::integral_constant<int, s % D>{}, pass * S + s + D);
    });
    // Sum the K slices through LDS.  Accumulator register r of lane l is output
    // (weight row quarter*4 + r, activation row l % 16) of its 16x16 tile.
    float (*mine)[16 * 16] = reinterpret_cast<float (*)[16 * 16]>(xlds[wave]) + pass * TILES;
#pragma unroll
    for (int t = 0; t < TILES; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) mine[t][(quarter * 4 + r) * 16 + row] = acc[t][r];
#pragma unroll
    for (int t = 0; t < TILES; ++t)
#pragma unroll
      for (int i = 0; i < NSC; ++i) sc_cur[t][i] = sc_nxt[t][i];
  }
  // One barrier for the whole kernel: the K slices of every pass wait in LDS and are summed at the end (a barrier per
  // pass held every wavefront until the slowest had finished the pass, with no new loads going out meanwhile).
  __syncthreads();
  for (int job = wave; job < passes * TILES; job += WAVES) {
    const int pass = job / TILES, t = job - pass * TILES;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float total_sum = 0.0f;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) total_sum += (reinterpret_cast<const float (*)[16 * 16]>(xlds[w]) + pass * TILES)[t][(quarter * 4 + r) * 16 + row];
      const int64_t n = wg_row0 + (pass * TILES + t) * 16 + quarter * 4 + r;
      if (row < p.m && n < p.n)
        p.y[static_cast<int64_t>(row) * p.ldy + n] = static_cast<uint16_t>(bf16_bits_rne(total_sum));
    }
  }
}


}  // namespace vecops_hip
#endif
