// fp32 operands multiplied in fp32 (v_mfma_f32_32x32x2_f32) when a product gives a compute unit at most ONE workgroup:
// 64 x 64 or 128 x 128 tiles, 128 KiB of LDS as a ring of stages (eight of 16 KiB, four of 32 KiB) that loads which
// write LDS themselves fill several K tiles ahead.  tile_gemm_kernel's fp32 instances stage one K tile ahead through
// registers and wait out every tile's loads when no second workgroup shares the unit (1024^3: 1780 cycles per K tile of
// 1024 of matrix instructions).  Here a K tile (32 floats of every row) is in flight for the time of stages - 2 tiles:
//   tile t lies in stage t mod S.  k-steps 0..2 of tile t multiply and read the next k-step's fragments; then
//   s_waitcnt vmcnt((S - 3) L) - tile t + 1 has landed, L loads a tile and wavefront - and the one barrier of the tile
//   (every wavefront has read stage (t - 1) mod S for the last time); the loads of tile t + S - 1 go into that stage;
//   k-step 3 multiplies under the reads of tile t + 1's first fragments.
// Tiles past the end are fetched against a descriptor of no records, so the count the wait relies on holds to the end.
// The matrix instructions run in tile_gemm_kernel's order (a k-step of eight: pairs (k_e, k_4+e), e = 0..3, B fragment
// first), so sums equal that kernel's bit for bit; start-up and epilogue (store_accumulators: every output, C input,
// split-K partials) are its own.
//
// LDS, a stage: A as BM rows of 128 bytes, chunks swizzled (lds_chunk_offset); B likewise when it is K-contiguous, or -
// handed over as [K,N] - as it lies in memory: 32 k rows of BN floats, neighbouring 128-byte pieces of a row swapped
// in the k rows 4-7 of each eight, so that the two half-wavefronts of a fragment read (k rows four apart) use different
// banks.
//
// What it serves (launch_tile_gemm_deep_f32_serves): fp32 compute, A K-contiguous, B K-contiguous or [K,N] with N a
// multiple of four, 16-byte aligned bases, rows and batches, K a whole number of K tiles, at most 256 workgroups.
#include "tile_gemm_launch.h"

namespace vecops_hip {

namespace {

constexpr int kRingBytes = 131072;

template <int WB, bool KN>
__global__ __launch_bounds__(256, 1) void tile_gemm_deep_f32_kernel(const TileGemmParams p) {
  constexpr int BM = 64 * WB, BN = 64 * WB;
  constexpr int kTileA = BM * 128, kTileB = BN * 128, kStage = kTileA + kTileB;
  constexpr int S = kRingBytes / kStage;           // stages
  constexpr int LA = BM / 32, LB = BN / 32, L = LA + LB;   // load instructions a K tile and wavefront
  constexpr int kEpilogue = kEpilogueLdsBytes<2, 2, WB, WB>();
  constexpr int kLdsBytes = kRingBytes > kEpilogue ? kRingBytes : kEpilogue;
  constexpr int kPitchKN = BN * 4;                 // bytes between the k rows of a [k][n] tile
  static_assert(S >= 4 && (S - 2) * L <= 63, "the waits count at most 63 loads");
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
  const int m0 = tm * BM, n0 = tn * BN;
  const int total_k_tiles = p.k / 32;
  const int kt_begin = split * p.k_tiles_per_split;
  const int kt_end = min(total_k_tiles, kt_begin + p.k_tiles_per_split);
  const int nk = __builtin_amdgcn_readfirstlane(max(kt_end - kt_begin, 0));

  // Loads: instruction i of a K-contiguous operand's K tile fills its rows 32 i .. 32 i + 31, this wavefront eight of
  // them; lane l fetches the chunk of row l / 8 whose swizzled slot is l % 8.  Rows past the extent are clamped onto
  // the last row: loaded, multiplied, never stored.
  uint32_t rows_a[LA], rows_b[LB];
  {
    const int load_row = tid >> 3;
#pragma unroll
    for (int i = 0; i < LA; ++i) {
      const int tile_row = load_row + 32 * i;
      const int chunk = ((tid & 7) ^ tile_row ^ (tile_row >> 3)) & 7;
      rows_a[i] = static_cast<uint32_t>((static_cast<int64_t>(min(m0 + tile_row, p.m - 1) - m0) * p.a_rs + chunk * 4) * 4);
    }
#pragma unroll
    for (int i = 0; i < LB; ++i) {
      const int tile_row = load_row + 32 * i;
      const int chunk = ((tid & 7) ^ tile_row ^ (tile_row >> 3)) & 7;
      rows_b[i] = static_cast<uint32_t>((static_cast<int64_t>(min(n0 + tile_row, p.n - 1) - n0) * p.b_rs + chunk * 4) * 4);
    }
    if constexpr (KN) {
      // B as [K,N]: an instruction of the workgroup fills 4 KiB = 4096 / kPitchKN k rows; lane t's 16 bytes are slot
      // (16 t % pitch) / 16 of k row 16 t / pitch, and it fetches the chunk of four columns whose slot that is (chunk
      // xor 8 in the k rows 4-7 of each eight).  N is a multiple of four here: a chunk past it is clamped onto the last.
      const int krow = tid * 16 / kPitchKN, slot = (tid * 16 % kPitchKN) / 16;
      const int chunk = slot ^ (((krow >> 2) & 1) << 3);
      const int col = min(n0 + chunk * 4, p.n - 4) - n0;
      rows_b[0] = static_cast<uint32_t>((static_cast<int64_t>(krow) * p.b_ks + col) * 4);
    }
  }
  // bytes from one K tile of B to the next, and ([K,N]) from one of its load instructions to the next
  const uint32_t step_b = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(KN ? 32 * p.b_ks * 4 : 128));
  const uint32_t part_b = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(KN ? (4096 / kPitchKN) * p.b_ks * 4 : 0));
  const u32x4 desc_a = tile_buffer_words((const VECOPS_GLOBAL char*)p.a +
                                         (static_cast<int64_t>(batch) * p.a_bs + static_cast<int64_t>(m0) * p.a_rs) * 4);
  // ([K,N]: the rows of the [N,K] view are one element apart)
  const u32x4 desc_b = tile_buffer_words((const VECOPS_GLOBAL char*)p.b +
                                         (static_cast<int64_t>(batch) * p.b_bs + static_cast<int64_t>(n0) * p.b_rs) * 4);
  const uint32_t lds0 = lds_address_of(lds);
  const uint32_t m0_wave = lds0 + static_cast<uint32_t>(wave) * 1024u;

  // K tile t of the range into its stage (a tile the range does not have: loads that fetch nothing)
  auto fill = [&](int t) {
    u32x4 da = desc_a, db = desc_b;
    if (t >= nk) da[2] = db[2] = 0u;
    // (wavefront-uniform numbers, said so: the instruction takes them from scalar registers)
    auto uniform = [](uint32_t v) { return static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(v)); };
    const uint32_t stage = uniform(static_cast<uint32_t>(t % S) * kStage);
    const uint32_t kt = uniform(static_cast<uint32_t>(kt_begin + min(t, max(nk - 1, 0))));
#pragma unroll
    for (int i = 0; i < LA; ++i) load_16_bytes_into_lds(da, m0_wave, stage + i * 4096, rows_a[i], uniform(kt * 128u));
#pragma unroll
    for (int i = 0; i < LB; ++i)
      load_16_bytes_into_lds(db, m0_wave, stage + kTileA + i * 4096, rows_b[KN ? 0 : i],
                             uniform(KN ? kt * step_b + static_cast<uint32_t>(i) * part_b : kt * 128u));
  };
#pragma unroll
  for (int t = 0; t < S - 1; ++t) fill(t);

  // Fragment reads.  K-contiguous: lane l supplies the chunk 2 ks + l / 32 (k 0-3 or 4-7 of the k-step's eight) of row
  // l % 32 of a block.  [K,N]: the same k, one float per read, from the rows 8 ks + 4 (l / 32) + e of column l % 32.
  const int frag_row = lane & 31, frag_half = lane >> 5;
  uint32_t off_a[WB], off_b[WB];
#pragma unroll
  for (int i = 0; i < WB; ++i) off_a[i] = static_cast<uint32_t>(lds_chunk_offset((wm * WB + i) * 32 + frag_row, frag_half));
#pragma unroll
  for (int j = 0; j < WB; ++j) {
    if constexpr (KN)
      off_b[j] = static_cast<uint32_t>(kTileA + 4 * frag_half * kPitchKN + ((((wn * WB + j) * 32 + frag_row) * 4) ^ (frag_half << 7)));
    else
      off_b[j] = static_cast<uint32_t>(kTileA + lds_chunk_offset((wn * WB + j) * 32 + frag_row, frag_half));
  }
  auto read_a = [&](const char* stage, int ks, int i) -> u32x4 {
    return *reinterpret_cast<const u32x4*>(stage + (off_a[i] ^ static_cast<uint32_t>(ks << 5)));
  };
  auto read_b = [&](const char* stage, int ks, int j) -> u32x4 {
    if constexpr (KN) {
      const char* at = stage + off_b[j] + ks * 8 * kPitchKN;
      return u32x4{*reinterpret_cast<const uint32_t*>(at), *reinterpret_cast<const uint32_t*>(at + kPitchKN),
                   *reinterpret_cast<const uint32_t*>(at + 2 * kPitchKN), *reinterpret_cast<const uint32_t*>(at + 3 * kPitchKN)};
    } else {
      return *reinterpret_cast<const u32x4*>(stage + (off_b[j] ^ static_cast<uint32_t>(ks << 5)));
    }
  };

  Accumulators<false, WB, WB, false> acc;
  acc.clear();
  u32x4 fa[2][WB], fb[2][WB];
  auto read_frags = [&](int set, const char* stage, int ks) {
#pragma unroll
    for (int i = 0; i < WB; ++i) fa[set][i] = read_a(stage, ks, i);
#pragma unroll
    for (int j = 0; j < WB; ++j) fb[set][j] = read_b(stage, ks, j);
    // (the reads are issued here, ahead of the matrix instructions that follow in the text, which then cover their
    // latency: left free, the scheduler hoists those instructions over the reads and every k-step waits for LDS)
    __builtin_amdgcn_sched_barrier(0);
  };
  // (the four instructions of a k-step and block - pairs (k_e, k_4+e), e = 0..3 - go round the blocks: consecutive
  // matrix instructions accumulate into different registers; every block still sums its k in order)
  auto multiply = [&](int set) {
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
      for (int i = 0; i < WB; ++i)
#pragma unroll
        for (int j = 0; j < WB; ++j)
          acc.t[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(fb[set][j][e]), __uint_as_float(fa[set][i][e]),
                                                             acc.t[i][j], 0, 0, 0);
  };

  if (nk > 0) {
    // tile 0 has landed (S - 2 later tiles may be in flight)
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"((S - 2) * L) : "memory");
    read_frags(0, lds, 0);
    int stage = 0;   // of tile t
    for (int t = 0; t < nk; ++t) {
      const char* here = lds + stage * kStage;
      const int next_stage = stage + 1 == S ? 0 : stage + 1;
      read_frags(1, here, 1);
      multiply(0);
      read_frags(0, here, 2);
      multiply(1);
      read_frags(1, here, 3);
      multiply(0);
      // tile t + 1 has landed; every wavefront has read the stage of tile t - 1 for the last time
      asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"((S - 3) * L) : "memory");
      fill(t + S - 1);
      read_frags(0, lds + next_stage * kStage, 0);
      multiply(1);
      stage = next_stage;
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();   // every wavefront has left the loop before the epilogue lays C out in LDS
  store_accumulators<SRC_F32, 2, 2, WB, WB, kLdsBytes, false>(p, lds, acc, batch, split, m0, n0, wm, wn, wave, lane);
}

template <int WB, bool KN>
hipError_t launch(const TileGemmParams& p, hipStream_t stream) {
  constexpr int kEpilogue = kEpilogueLdsBytes<2, 2, WB, WB>();
  constexpr int kLds = kRingBytes > kEpilogue ? kRingBytes : kEpilogue;
  auto kernel = tile_gemm_deep_f32_kernel<WB, KN>;
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

bool launch_tile_gemm_deep_f32_serves(const TileGemmParams& p, int tile, bool b_as_kn) {
  auto aligned = [](const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; };
  if ((tile != 64 && tile != 128) || p.m <= 0 || p.n <= 0 || p.split_k < 1 || p.k < 32 || p.k % 32 != 0) return false;
  if (!aligned(p.a) || !aligned(p.b) || p.a_ks != 1 || p.a_rs % 4 != 0 || p.a_bs % 4 != 0 || p.b_bs % 4 != 0) return false;
  if (p.a_flip != 0u || p.b_flip != 0u) return false;
  // 32-bit byte offsets inside a tile's rows
  if ((tile * p.a_rs + p.k) * 4 >= (int64_t{1} << 31)) return false;
  if (b_as_kn)
    return p.b_rs == 1 && p.b_ks % 4 == 0 && p.n % 4 == 0 && p.n >= 4 && (static_cast<int64_t>(p.k) * p.b_ks + tile) * 4 < (int64_t{1} << 31);
  return p.b_ks == 1 && p.b_rs % 4 == 0 && (tile * p.b_rs + p.k) * 4 < (int64_t{1} << 31);
}

hipError_t launch_tile_gemm_deep_f32(const TileGemmParams& p, int tile, bool b_as_kn, hipStream_t stream) {
  if (tile == 64) return b_as_kn ? launch<1, true>(p, stream) : launch<1, false>(p, stream);
  if (tile == 128) return b_as_kn ? launch<2, true>(p, stream) : launch<2, false>(p, stream);
  return hipErrorInvalidValue;
}

}  // namespace vecops_hip
