// The 128 x 128 workgroup tile for products that give a compute unit at most one workgroup (256 tiles or fewer): four
// LDS stages instead of two, the loads three K tiles ahead, and the K loop a written-out instruction stream
// (VECOPS_LOOP128_DEEP of tile_loop_asm.inc; gen_tile_loop.py describes its schedule).  tile_gemm_kernel's 128 x 128
// instance is built for two workgroups per unit, each hiding the other's waits; alone on a unit it waits out every K
// tile's loads (0.67 us per K tile of 0.25 us of matrix instructions at 1024 x 4096 x 4096).
//
// What it serves (launch_tile_gemm_deep128_serves): bf16, f16 or signed 8-bit operands, both K-contiguous with 16-byte
// aligned bases, rows and batches (the loads write LDS themselves), or - 16-bit operands - B handed over as [K,N]
// (TR: the tile lies [k][n] in LDS, 64 rows of 256 bytes, swizzled as tile_gemm_kernel's, and the fragment reads
// transpose); K a whole number of K tiles.  Any M, N, batch count, K split, C input and output type of the class: the
// epilogue is tile_gemm_kernel's.  PK: B prepacked by vecops_hip_pack_b and kept in its pack order in LDS - a load
// instruction of a wavefront moves one whole (panel of 32 rows, k-step of two chunks) block, 1 KiB contiguous on both
// sides, and a fragment read is the stage pair's one per-lane base plus a constant (as in tile_gemm_packed16.hip).
#include "tile_gemm_launch.h"

namespace vecops_hip {

namespace {

constexpr int kDeepStage = 32768;  // 128 rows of A, then 128 of B, 128 bytes of K each
constexpr int kDeepStages = 4;

template <int SRC, bool TR, bool PK>
__global__ __launch_bounds__(256, 1) void tile_gemm_deep128_kernel(const TileGemmParams p) {
  static_assert(!(TR && PK), "one layout of B");
  using T = SrcTraits<SRC>;
  constexpr bool INT = T::kInt;
  constexpr int KTILE = 8 * T::kElemsPerChunk;
  constexpr int kEpilogue = kEpilogueLdsBytes<2, 2, 2, 2>();
  constexpr int kLdsBytes = kDeepStages * kDeepStage > kEpilogue ? kDeepStages * kDeepStage : kEpilogue;
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
  const int m0 = tm * 128, n0 = tn * 128;
  const int total_k_tiles = p.k / KTILE;
  const int kt_begin = split * p.k_tiles_per_split;
  const int kt_end = min(total_k_tiles, kt_begin + p.k_tiles_per_split);
  const int nk = __builtin_amdgcn_readfirstlane(max(kt_end - kt_begin, 0));

  // Loads: instruction i of an operand's K tile fills its rows 32 i .. 32 i + 31, this wavefront eight of them; lane l
  // fetches the chunk of row l / 8 whose swizzled slot is l % 8.  Rows past the operand's extent are clamped onto its
  // last row: loaded, multiplied, never stored.
  uint32_t rows_a[4], rows_b[4];
  {
    const int load_row = tid >> 3;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int tile_row = load_row + 32 * i;
      const int chunk = ((tid & 7) ^ tile_row ^ (tile_row >> 3)) & 7;
      rows_a[i] = static_cast<uint32_t>(static_cast<int64_t>(min(m0 + tile_row, p.m - 1) - m0) * p.a_rs * T::kSrcBytes + chunk * 16);
      rows_b[i] = static_cast<uint32_t>(static_cast<int64_t>(min(n0 + tile_row, p.n - 1) - n0) * p.b_rs * T::kSrcBytes + chunk * 16);
    }
    if constexpr (TR) {
      // B as [K,N]: a load instruction of the workgroup fills sixteen k rows of 256 bytes; lane t fetches, of k row
      // t / 16, the chunk of eight columns whose swizzled slot is t % 16 (slot = chunk xor 4 * (k row % 4): the four
      // rows a transposing read touches lie in different bank groups).  N is a multiple of eight on this path: a chunk
      // past it is clamped onto the last one.
      const int krow = tid >> 4, slot = tid & 15;
      const int chunk = slot ^ ((krow & 3) << 2);
      const int col = min(n0 + chunk * 8, p.n - 8) - n0;
      rows_b[0] = static_cast<uint32_t>((static_cast<int64_t>(krow) * p.b_ks + col) * T::kSrcBytes);
    }
    if constexpr (PK) {
      // B prepacked: instruction i moves the tile's panel i (clamped onto the operand's last panel), this wavefront the
      // pack's k-step number `wave` of the K tile's four
      const int64_t ks_total = static_cast<int64_t>(total_k_tiles) * 4;
      const int nb0 = n0 / 32, nb_last = (p.n + 31) / 32 - 1;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        rows_b[i] = static_cast<uint32_t>(((min(nb0 + i, nb_last) - nb0) * ks_total + wave) * 1024 + lane * 16);
    }
  }
  // bytes from one K tile of B to the next, and (TR) from one of its four loads to the next
  const uint32_t step_b = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(TR ? 64 * p.b_ks * T::kSrcBytes : PK ? 4096 : 128));
  const uint32_t part_b = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(TR ? 16 * p.b_ks * T::kSrcBytes : 0));
  const u32x4 desc_a = tile_buffer_words((const VECOPS_GLOBAL char*)p.a +
                                         (static_cast<int64_t>(batch) * p.a_bs + static_cast<int64_t>(m0) * p.a_rs) * T::kSrcBytes);
  // (TR: the rows of the [N,K] view are one element apart)
  // (PK: one packed operand for every batch; a panel's K tiles lie 4 KiB apart)
  const u32x4 desc_b = tile_buffer_words((const VECOPS_GLOBAL char*)p.b +
                                         (PK ? static_cast<int64_t>(n0 / 32) * total_k_tiles * 4096
                                             : (static_cast<int64_t>(batch) * p.b_bs + static_cast<int64_t>(n0) * p.b_rs) * T::kSrcBytes));
  const uint32_t lds0 = lds_address_of(lds);
  const uint32_t m0_wave = lds0 + static_cast<uint32_t>(wave) * 1024u;

  // K tiles 0, 1, 2 of the range into stages 0, 1, 2 (a tile the range does not have: loads that fetch nothing, so that
  // the loop's count of loads in flight holds)
  auto fill = [&](int t) {
    u32x4 da = desc_a, db = desc_b;
    if (t >= nk) da[2] = db[2] = 0u;
    // (wavefront-uniform by construction; said so, or the compiler may carry them in vector registers, which the
    //  load's scalar offset does not take)
    const uint32_t k_tile = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(kt_begin + t));
    const uint32_t k_bytes = k_tile * 128u;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      load_16_bytes_into_lds(da, m0_wave, static_cast<uint32_t>(t * kDeepStage + i * 4096), rows_a[i], k_bytes);
#pragma unroll
    for (int i = 0; i < 4; ++i)
      load_16_bytes_into_lds(db, m0_wave, static_cast<uint32_t>(t * kDeepStage + 16384 + i * 4096), rows_b[TR ? 0 : i],
                             TR ? k_tile * step_b + static_cast<uint32_t>(i) * part_b : PK ? k_tile * step_b : k_bytes);
  };
  fill(0);
  fill(1);
  fill(2);

  // Fragment reads: lane l supplies row l % 16 of a block and one of the four chunks of the matrix k-step (the 16-lane
  // groups in the order 0, 2, 1, 3, as in tile_gemm_kernel).  [stage pair][q]: the odd stage lies 32 KiB up.
  const int frag_row = lane & 15;
  const int frag_chunk = ((lane >> 4) & 1) << 1 | (lane >> 5);
  uint32_t base_a[2][4], base_b[2][4];
  {
    const int slot = frag_chunk ^ frag_row ^ (frag_row >> 3);
#pragma unroll
    for (int pair = 0; pair < 2; ++pair)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        base_a[pair][q] = lds0 + pair * 2 * kDeepStage + (wm * 64 + frag_row) * 128 + (((slot ^ (2 * q)) & 7) << 4);
        if constexpr (TR) {
          // transposing read: lane s of the 16-lane group addresses row s / 4 of a block of four k rows, columns
          // 4 (s % 4) .. + 3 of the column block pair q, and receives column s of the block's 16; the group reads
          // chunk frag_chunk of k.  The 64-byte group is swizzled with the row's low two bits, which are s / 4.
          int col_bytes = ((wn * 4 + 2 * q) * 16 + (frag_row & 3) * 4) * 2;
          col_bytes ^= ((frag_row >> 2) & 3) << 6;
          base_b[pair][q] = lds0 + pair * 2 * kDeepStage + 16384 + (frag_chunk * 8 + (frag_row >> 2)) * 256 + col_bytes;
        } else if constexpr (PK) {
          // [panel][k-step of the pack: chunk / 2][half: chunk % 2][row of the panel][16 bytes]: the wavefront's two panels
          base_b[pair][q] = lds0 + pair * 2 * kDeepStage + 16384 + wn * 2 * 4096 + (frag_chunk >> 1) * 1024 +
                            (frag_chunk & 1) * 512 + frag_row * 16;
        } else {
          base_b[pair][q] = lds0 + pair * 2 * kDeepStage + 16384 + (wn * 64 + frag_row) * 128 + (((slot ^ (2 * q)) & 7) << 4);
        }
      }
  }

  Accumulators<INT, 2, 2, true> acc;
  acc.clear();
  if (nk > 0) {
    asm volatile("s_waitcnt vmcnt(16)" ::: "memory");   // tile 0 has landed
    __builtin_amdgcn_s_barrier();
#if defined(__HIP_DEVICE_COMPILE__)
    auto uniform = [](uint32_t v) { return static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(v)); };
    int left = nk - 3, n = nk;
    uint32_t k_a = uniform(static_cast<uint32_t>(kt_begin + 3) * 128u);   // the loop fetches tile 3 of the range first
    uint32_t k_b = uniform(static_cast<uint32_t>(kt_begin + 3) * step_b);
    const uint32_t sb = uniform(step_b), pb = uniform(part_b);
    const uint32_t da[4] = {uniform(desc_a[0]), uniform(desc_a[1]), uniform(desc_a[2]), uniform(desc_a[3])};
    const uint32_t db[4] = {uniform(desc_b[0]), uniform(desc_b[1]), uniform(desc_b[2]), uniform(desc_b[3])};
    const uint32_t m0w = uniform(m0_wave);
#define VECOPS_DEEP_STATEMENT(TEXT)                                                                                  \
    asm volatile(TEXT                                                                                                 \
                 : VECOPS_LOOP128_ACCUMULATORS(acc.t), [ka] "+s"(k_a), [kb] "+s"(k_b), [left] "+s"(left), [n] "+s"(n)  \
                 : [la00] "v"(base_a[0][0]), [la01] "v"(base_a[0][1]), [la02] "v"(base_a[0][2]), [la03] "v"(base_a[0][3]), \
                   [la10] "v"(base_a[1][0]), [la11] "v"(base_a[1][1]), [la12] "v"(base_a[1][2]), [la13] "v"(base_a[1][3]), \
                   [lb00] "v"(base_b[0][0]), [lb01] "v"(base_b[0][1]), [lb02] "v"(base_b[0][2]), [lb03] "v"(base_b[0][3]), \
                   [lb10] "v"(base_b[1][0]), [lb11] "v"(base_b[1][1]), [lb12] "v"(base_b[1][2]), [lb13] "v"(base_b[1][3]), \
                   [ra0] "v"(rows_a[0]), [ra1] "v"(rows_a[1]), [ra2] "v"(rows_a[2]), [ra3] "v"(rows_a[3]),            \
                   [rb0] "v"(rows_b[0]), [rb1] "v"(rows_b[1]), [rb2] "v"(rows_b[2]), [rb3] "v"(rows_b[3]),            \
                   [da0] "s"(da[0]), [da1] "s"(da[1]), [da2] "s"(da[2]), [da3] "s"(da[3]),                            \
                   [db0] "s"(db[0]), [db1] "s"(db[1]), [db2] "s"(db[2]), [db3] "s"(db[3]), [m0w] "s"(m0w),            \
                   [sb] "s"(sb), [pb] "s"(pb)                                                                         \
                 : "memory", "m0", "scc", VECOPS_LOOP128_CLOBBERS)
    if constexpr (PK) {
      if constexpr (SRC == SRC_F16) VECOPS_DEEP_STATEMENT(VECOPS_LOOP128_DEEP_PK("v_mfma_f32_16x16x32_f16"));
      else if constexpr (INT) VECOPS_DEEP_STATEMENT(VECOPS_LOOP128_DEEP_PK("v_mfma_i32_16x16x64_i8"));
      else VECOPS_DEEP_STATEMENT(VECOPS_LOOP128_DEEP_PK("v_mfma_f32_16x16x32_bf16"));
    } else if constexpr (TR) {
      static_assert(SRC == SRC_BF16 || SRC == SRC_F16, "transposing LDS reads move 16-bit elements");
      if constexpr (SRC == SRC_F16) VECOPS_DEEP_STATEMENT(VECOPS_LOOP128_DEEP_TR("v_mfma_f32_16x16x32_f16"));
      else VECOPS_DEEP_STATEMENT(VECOPS_LOOP128_DEEP_TR("v_mfma_f32_16x16x32_bf16"));
    } else if constexpr (SRC == SRC_F16) VECOPS_DEEP_STATEMENT(VECOPS_LOOP128_DEEP("v_mfma_f32_16x16x32_f16"));
    else if constexpr (INT) VECOPS_DEEP_STATEMENT(VECOPS_LOOP128_DEEP("v_mfma_i32_16x16x64_i8"));
    else VECOPS_DEEP_STATEMENT(VECOPS_LOOP128_DEEP("v_mfma_f32_16x16x32_bf16"));
#undef VECOPS_DEEP_STATEMENT
#endif
  } else {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  }
  __builtin_amdgcn_s_barrier();   // every wavefront has left the loop before the epilogue lays C out in LDS
  store_accumulators<SRC, 2, 2, 2, 2, kLdsBytes, true>(p, lds, acc, batch, split, m0, n0, wm, wn, wave, lane);
}

template <int SRC, bool TR, bool PK>
hipError_t launch(const TileGemmParams& p, hipStream_t stream) {
  constexpr int kEpilogue = kEpilogueLdsBytes<2, 2, 2, 2>();
  constexpr int kLds = kDeepStages * kDeepStage > kEpilogue ? kDeepStages * kDeepStage : kEpilogue;
  auto kernel = tile_gemm_deep128_kernel<SRC, TR, PK>;
  static thread_local int configured_device = -1;
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return e;
  if (configured_device != device) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
    if (e != hipSuccess) return e;
    configured_device = device;
  }
  const int64_t grid = static_cast<int64_t>(p.tiles_m) * p.tiles_n * p.batch * p.split_k;
  if (grid <= 0 || grid > INT32_MAX) return hipErrorInvalidConfiguration;
  hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(grid)), dim3(256), kLds, stream, p);
  return hipGetLastError();
}

}  // namespace

bool launch_tile_gemm_deep128_serves(int src, const TileGemmParams& p, int mode, bool packed_b) {
  if (src != SRC_BF16 && src != SRC_F16 && src != SRC_I8) return false;
  const bool tr = !packed_b && mode == MODE_NVEC_B_DMA;
  if (p.m <= 0 || p.n <= 0 || p.split_k < 1) return false;
  const int elem = src == SRC_I8 ? 1 : 2, ktile = 128 / elem;
  if (p.k < ktile || p.k % ktile != 0) return false;
  // 32-bit byte offsets inside a tile's 128 rows
  if (128 * p.a_rs * elem + static_cast<int64_t>(p.k) * elem >= (int64_t{1} << 31)) return false;
  if (packed_b) {
    // A: loads that write LDS need 16-byte aligned addresses; B: 32-bit byte offsets inside the tile's four panels
    if (p.a_ks != 1 || (reinterpret_cast<uintptr_t>(p.a) & 15u) != 0 || (p.a_rs * elem) % 16 != 0 || (p.a_bs * elem) % 16 != 0) return false;
    return (reinterpret_cast<uintptr_t>(p.b) & 15u) == 0 && 4 * static_cast<int64_t>(p.k / ktile) * 4096 < (int64_t{1} << 31);
  }
  if ((mode != MODE_KVEC_DMA && !tr) || (tr && src == SRC_I8)) return false;
  if (tr) return p.n % 8 == 0 && p.n >= 8 && p.b_rs == 1 && static_cast<int64_t>(p.k) * p.b_ks * elem + 256 < (int64_t{1} << 31);
  return 128 * p.b_rs * elem + static_cast<int64_t>(p.k) * elem < (int64_t{1} << 31);
}

hipError_t launch_tile_gemm_deep128(int src, const TileGemmParams& p, int mode, bool packed_b, hipStream_t stream) {
  const bool tr = !packed_b && mode == MODE_NVEC_B_DMA;
  if (packed_b) {
    switch (src) {
      case SRC_BF16: return launch<SRC_BF16, false, true>(p, stream);
      case SRC_F16: return launch<SRC_F16, false, true>(p, stream);
      case SRC_I8: return launch<SRC_I8, false, true>(p, stream);
      default: return hipErrorInvalidValue;
    }
  }
  switch (src) {
    case SRC_BF16: return tr ? launch<SRC_BF16, true, false>(p, stream) : launch<SRC_BF16, false, false>(p, stream);
    case SRC_F16: return tr ? launch<SRC_F16, true, false>(p, stream) : launch<SRC_F16, false, false>(p, stream);
    case SRC_I8: return launch<SRC_I8, false, false>(p, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace vecops_hip
