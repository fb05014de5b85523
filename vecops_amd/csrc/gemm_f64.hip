// fp64 x fp64 -> fp64 tile GEMM for gfx950: the GPU form of vecops' SME_F64F64 atom
// (matmul/details/kernel/sme/Atoms.h:108-112: FMOPA .d, fp64 operands, fp64 accumulate).
//   C[..,M,N] = C_in + A[..,M,K] . B[..,N,K]^T, any element strides, rank-3 batches on blockIdx.z.
// One v_mfma_f64_16x16x4_f64 multiplies 16 rows x 4 k by 4 k x 16 columns: lane l supplies A[row l % 16][k l / 16]
// and B[column l % 16][k l / 16] and receives D[4 r + l / 16][l % 16] in register r.  A workgroup of four
// wavefronts (2 x 2) owns a 128 x 128 tile of C, a wavefront 64 x 64 = 4 x 4 accumulator tiles (128 registers);
// K is walked in tiles of 8 (two MFMA steps) through two LDS stages: the global loads of tile t + 1 are in
// flight while tile t is multiplied.  A lane stages four consecutive k of one row per operand (32 bytes when K
// is contiguous); rows past the extents and k past K are staged as zeros.  LDS rows are 9 doubles apart, so the
// sixteen rows of an operand read fall into different banks.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "gemm_f64.h"

namespace vecops_hip {
namespace {

typedef __attribute__((ext_vector_type(4))) double f64x4;
// loads through generic pointers count against the LDS counter too: every wait for a fragment read would then wait
// for the prefetch of the next K tile as well
#define GLOBAL_F64 __attribute__((address_space(1))) double

constexpr int kTile = 128, kK = 8, kPitch = kK + 1;

__global__ __launch_bounds__(256) void gemm_f64_kernel(const GemmF64Params p) {
  __shared__ double lds[2][2][kTile * kPitch];  // [stage][operand][row * pitch + k]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int tiles_n = (p.n + kTile - 1) / kTile;
  const int tm = blockIdx.x / tiles_n, tn = blockIdx.x % tiles_n;
  const int batch = blockIdx.y;
  const int m0 = tm * kTile, n0 = tn * kTile;
  const double* a = p.a + batch * p.a_bs;
  const double* b = p.b + batch * p.b_bs;

  // staging: thread t holds k half (t & 1) of row t >> 1 of both operand tiles (4 doubles each)
  const int s_row = tid >> 1, s_k = (tid & 1) * 4;
  const bool a_row_ok = m0 + s_row < p.m, b_row_ok = n0 + s_row < p.n;
  const GLOBAL_F64* a_src = (const GLOBAL_F64*)(a + static_cast<int64_t>(a_row_ok ? m0 + s_row : 0) * p.a_rs);
  const GLOBAL_F64* b_src = (const GLOBAL_F64*)(b + static_cast<int64_t>(b_row_ok ? n0 + s_row : 0) * p.b_rs);
  double ra[4], rb[4];
  auto fetch = [&](int kt) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int k = kt * kK + s_k + e;
      ra[e] = (a_row_ok && k < p.k) ? a_src[static_cast<int64_t>(k) * p.a_ks] : 0.0;
      rb[e] = (b_row_ok && k < p.k) ? b_src[static_cast<int64_t>(k) * p.b_ks] : 0.0;
    }
  };
  auto commit = [&](int stage) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      lds[stage][0][s_row * kPitch + s_k + e] = ra[e];
      lds[stage][1][s_row * kPitch + s_k + e] = rb[e];
    }
  };

  f64x4 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = f64x4{0.0, 0.0, 0.0, 0.0};

  const int k_tiles = (p.k + kK - 1) / kK;
  const int frag_row = lane & 15, frag_k = lane >> 4;
  if (k_tiles > 0) {
    fetch(0);
    commit(0);
    __syncthreads();
    for (int kt = 0; kt < k_tiles; ++kt) {
      const int stage = kt & 1;
      if (kt + 1 < k_tiles) fetch(kt + 1);
      const double* ta = &lds[stage][0][(wm * 64 + frag_row) * kPitch + frag_k];
      const double* tb = &lds[stage][1][(wn * 64 + frag_row) * kPitch + frag_k];
#pragma unroll
      for (int ks = 0; ks < kK / 4; ++ks) {
        double fa[4], fb[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) fa[i] = ta[i * 16 * kPitch + ks * 4];
#pragma unroll
        for (int j = 0; j < 4; ++j) fb[j] = tb[j * 16 * kPitch + ks * 4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(fa[i], fb[j], acc[i][j], 0, 0, 0);
      }
      if (kt + 1 < k_tiles) commit(stage ^ 1);  // the other stage was read in iteration kt - 1, behind its barrier
      __syncthreads();
    }
  }

  // register r of lane l: row 4 r + l / 16, column l % 16 of its 16 x 16 tile
  const double* cin = p.cin ? p.cin + batch * p.cin_bs : nullptr;
  double* c = p.c + batch * p.c_bs;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = m0 + wm * 64 + i * 16 + r * 4 + frag_k, col = n0 + wn * 64 + j * 16 + frag_row;
        if (row < p.m && col < p.n) {
          double v = acc[i][j][r];
          if (cin) v += cin[static_cast<int64_t>(row) * p.cin_rs + static_cast<int64_t>(col) * p.cin_cs];
          c[static_cast<int64_t>(row) * p.c_rs + static_cast<int64_t>(col) * p.c_cs] = v;
        }
      }
}

}  // namespace

hipError_t launch_gemm_f64(const GemmF64Params& p, hipStream_t stream) {
  const int64_t tiles = static_cast<int64_t>((p.m + kTile - 1) / kTile) * ((p.n + kTile - 1) / kTile);
  if (tiles <= 0 || p.batch <= 0) return hipSuccess;
  if (tiles > INT32_MAX || p.batch > 65535) return hipErrorInvalidConfiguration;
  hipLaunchKernelGGL(gemm_f64_kernel, dim3(static_cast<unsigned>(tiles), static_cast<unsigned>(p.batch)), dim3(256), 0,
                     stream, p);
  return hipGetLastError();
}

}  // namespace vecops_hip
