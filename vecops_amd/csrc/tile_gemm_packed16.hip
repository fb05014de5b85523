// Prepacked B on the 256 x 256 workgroup tile with the 16x16 matrix instructions and the written-out K loop
// (VECOPS_LOOP256_PK of tile_loop_asm.inc): the packed operand keeps its own order in LDS.  A load instruction of a
// wavefront moves one whole (panel of 32 rows, k-step of two chunks) block of the pack - 1 KiB contiguous in memory and
// in LDS - and a fragment read is the stage's one per-lane base plus a constant:
//   LDS, B part of a stage: [panel 0..7 of the tile][k-step 0..3 of the K tile][chunk half][row 0..31][16 bytes]
//   column block j (16 columns) of a wavefront = its panel j / 2, rows 16 (j % 2) .. + 15; matrix k-step ks reads the
//   pack's k-steps 2 ks and 2 ks + 1 (the lane's chunk c: k-step 2 ks + c / 2, half c % 2)
// A travels as in tile_gemm_kernel's written-out loop (swizzled rows of 128 bytes, loads that write LDS themselves).
// The other prepacked kernel (tile_gemm_packed_b_kernel: B straight into registers, 32x32 instructions, a loop the
// compiler schedules) serves whatever this one does not.
//
// What it serves (launch_tile_gemm_packed16_serves): bf16, f16 or signed 8-bit operands; A K-contiguous with 16-byte
// aligned base, rows and batches; K a whole number of K tiles (128 bytes of a row); K unsplit.  Any M, N, batch count,
// C input and output type of the class: start-up and epilogue are tile_gemm_kernel's.
#include "tile_gemm_packed.h"

#include "tile_gemm_launch.h"

namespace vecops_hip {

namespace {

constexpr int kStage = 65536;   // 256 rows of A and 8 panels of B, 128 bytes of K each
constexpr int kBTile = 32768;   // the B part lies behind the A part

template <int SRC>
__global__ __launch_bounds__(256, 1) void tile_gemm_packed16_kernel(const TileGemmParams p) {
  using T = SrcTraits<SRC>;
  constexpr bool INT = T::kInt;
  constexpr int KTILE = 8 * T::kElemsPerChunk;
  constexpr int kEpilogue = kEpilogueLdsBytes<2, 2, 4, 4>();
  constexpr int kLdsBytes = 2 * kStage > kEpilogue ? 2 * kStage : kEpilogue;
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  int batch, split, tm, tn;
  map_workgroup(p, blockIdx.x, gridDim.x, batch, split, tm, tn);
  batch = __builtin_amdgcn_readfirstlane(batch);
  split = __builtin_amdgcn_readfirstlane(split);
  tm = __builtin_amdgcn_readfirstlane(tm);
  tn = __builtin_amdgcn_readfirstlane(tn);
  const int m0 = tm * 256, n0 = tn * 256;
  const int nk = __builtin_amdgcn_readfirstlane(p.k / KTILE);

  // Loads of A: instruction i of a K tile fills rows 32 i .. 32 i + 31 of the tile, this wavefront eight of them; lane l
  // fetches the chunk of row l / 8 whose swizzled slot is l % 8.  Rows past M are clamped onto the last row: loaded,
  // multiplied, never stored.
  uint32_t rows_a[8], rows_b[8];
  {
    const int load_row = tid >> 3;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int tile_row = load_row + 32 * i;
      const int chunk = ((tid & 7) ^ tile_row ^ (tile_row >> 3)) & 7;
      const int row = min(m0 + tile_row, p.m - 1) - m0;
      rows_a[i] = static_cast<uint32_t>(static_cast<int64_t>(row) * p.a_rs * T::kSrcBytes + chunk * 16);
    }
    // Loads of B: instruction i moves the tile's panel i (clamped onto the operand's last panel), this wavefront the
    // pack's k-step number `wave` of the K tile's four
    const int64_t ks_total = static_cast<int64_t>(nk) * 4;
    const int nb0 = n0 / 32, nb_last = (p.n + 31) / 32 - 1;
#pragma unroll
    for (int i = 0; i < 8; ++i)
      rows_b[i] = static_cast<uint32_t>(((min(nb0 + i, nb_last) - nb0) * ks_total + wave) * 1024 + lane * 16);
  }
  const u32x4 desc_a = tile_buffer_words((const VECOPS_GLOBAL char*)p.a +
                                         (static_cast<int64_t>(batch) * p.a_bs + static_cast<int64_t>(m0) * p.a_rs) * T::kSrcBytes);
  const u32x4 desc_b = tile_buffer_words((const VECOPS_GLOBAL char*)p.b + static_cast<int64_t>(n0 / 32) * nk * 4096);
  const uint32_t lds0 = lds_address_of(lds);
  const uint32_t m0_wave = lds0 + static_cast<uint32_t>(wave) * 1024u;

  auto fill = [&](int kt, int stage) {
#pragma unroll
    for (int i = 0; i < 8; ++i)
      load_16_bytes_into_lds(desc_a, m0_wave, static_cast<uint32_t>(stage * kStage + i * 4096), rows_a[i],
                             static_cast<uint32_t>(kt) * 128u);
#pragma unroll
    for (int i = 0; i < 8; ++i)
      load_16_bytes_into_lds(desc_b, m0_wave, static_cast<uint32_t>(stage * kStage + kBTile + i * 4096), rows_b[i],
                             static_cast<uint32_t>(kt) * 4096u);
  };
  if (nk > 1) fill(1, 1);
  fill(0, 0);

  // Fragment reads: lane l supplies row l % 16 of a block and one of the four chunks of the matrix k-step (the 16-lane
  // groups in the order 0, 2, 1, 3, as in tile_gemm_kernel: which k a group multiplies is free as long as A and B agree)
  const int frag_row = lane & 15;
  const int frag_chunk = ((lane >> 4) & 1) << 1 | (lane >> 5);
  uint32_t base_a[2][4], base_b[2][4];
  {
    const int slot = frag_chunk ^ frag_row ^ (frag_row >> 3);
#pragma unroll
    for (int st = 0; st < 2; ++st)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        base_a[st][q] = lds0 + st * kStage + (wm * 128 + frag_row) * 128 + (((slot ^ (2 * q)) & 7) << 4);
        base_b[st][q] = lds0 + st * kStage + kBTile + wn * 4 * 4096 + (frag_chunk >> 1) * 1024 + (frag_chunk & 1) * 512 +
                        frag_row * 16;
      }
  }

  Accumulators<INT, 4, 4, true> acc;
  acc.clear();
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm_k_loop<SRC, 2>(acc, base_a, base_b, rows_a, rows_b, desc_a, desc_b, m0_wave, 256u, 8192u, 4096u, 0u, nk);
  store_accumulators<SRC, 2, 2, 4, 4, kLdsBytes, true>(p, lds, acc, batch, split, m0, n0, wm, wn, wave, lane);
}

template <int SRC>
hipError_t launch(const TileGemmParams& p, hipStream_t stream) {
  constexpr int kEpilogue = kEpilogueLdsBytes<2, 2, 4, 4>();
  constexpr int kLds = 2 * kStage > kEpilogue ? 2 * kStage : kEpilogue;
  auto kernel = tile_gemm_packed16_kernel<SRC>;
  static thread_local int configured_device = -1;
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return e;
  if (configured_device != device) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
    if (e != hipSuccess) return e;
    configured_device = device;
  }
  const int64_t grid = static_cast<int64_t>(p.tiles_m) * p.tiles_n * p.batch;
  if (grid <= 0 || grid > INT32_MAX) return hipErrorInvalidConfiguration;
  hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(grid)), dim3(256), kLds, stream, p);
  return hipGetLastError();
}

}  // namespace

bool launch_tile_gemm_packed16_serves(int src, const TileGemmParams& p, int tile_m, int tile_n) {
  if (src != SRC_BF16 && src != SRC_F16 && src != SRC_I8) return false;
  if (tile_m != 256 || tile_n != 256 || p.split_k != 1 || p.m <= 0 || p.n <= 0) return false;
  const int elem = src == SRC_I8 ? 1 : 2, ktile = 128 / elem;
  if (p.k < ktile || p.k % ktile != 0 || p.a_ks != 1) return false;
  // A: loads that write LDS need 16-byte aligned addresses; 32-bit byte offsets inside a tile's 256 rows
  if ((reinterpret_cast<uintptr_t>(p.a) & 15u) != 0 || (p.a_rs * elem) % 16 != 0 || (p.a_bs * elem) % 16 != 0) return false;
  if (256 * p.a_rs * elem + static_cast<int64_t>(p.k) * elem >= (int64_t{1} << 31)) return false;
  // B: 32-bit byte offsets inside the tile's eight panels of the pack
  if (8 * static_cast<int64_t>(p.k / ktile) * 4096 >= (int64_t{1} << 31)) return false;
  return (reinterpret_cast<uintptr_t>(p.b) & 15u) == 0;
}

hipError_t launch_tile_gemm_packed16(int src, const TileGemmParams& p, hipStream_t stream) {
  switch (src) {
    case SRC_BF16: return launch<SRC_BF16>(p, stream);
    case SRC_F16: return launch<SRC_F16>(p, stream);
    case SRC_I8: return launch<SRC_I8>(p, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace vecops_hip
