// Products one matrix instruction deep (8 <= K <= 32) on 16-bit compute: a kernel whose life is writing C.
//
// The tile kernels stage operands through LDS in K tiles of 64 and hold two 32 KiB stages and 244 registers a lane:
// two workgroups on a compute unit, each of which loads, waits, multiplies once and then writes 64 KiB - batch 8 of
// 3000 x 3000 x 17 to fp32 wrote its 288 MB at 4.2 TB/s.  Here a wavefront owns 32 x 64 of C, loads its operand
// fragments from memory straight into the registers the matrix instruction reads (six 16-byte loads a lane per tile),
// multiplies with B as the first operand - so a lane's four results are four consecutive columns of one row of C -
// lays sixteen rows at a time row-major into its own 4 KiB of LDS, and writes them as whole 256-byte row segments,
// four rows per store instruction.  No workgroup barrier, 17 KiB of LDS a workgroup and at most 128 registers: a
// compute unit holds four workgroups, each of which walks tiles with the next tile's loads in flight behind the
// stores of the tile at hand (5.4 TB/s on that shape).
#include "tile_gemm_launch.h"
namespace vecops_hip {
namespace {

constexpr int kWaveRows = 32, kWaveCols = 64;    // one wavefront's part of C
constexpr int kTileRows = 32, kTileCols = 256;   // a workgroup: four wavefronts side by side along N (1 KiB of a row of fp32 C)
constexpr int kStageRows = 16;                   // rows of C a wavefront lays out in LDS at a time
constexpr int kPitch = kWaveCols + 4;            // 32-bit words per staged row: rows start 16 bytes apart in the bank period

// Eight compute elements of a K-contiguous row of at least eight elements as one 16-byte chunk: elements k0 .. k0+7
// where they lie inside the row, else the row's last eight with those below k0 zeroed - the sum over k takes its
// terms in any order, so a chunk may hold any eight elements as long as both operands' chunks hold the same ones and
// every element turns up once.  One load and no branch whatever k0 (a chunk past the row's end comes out all zeros).
// The load and the zeroing are separate steps: what is loaded for the next tile is not touched before that tile's turn.
__device__ __forceinline__ int fragment_start(int k0, int k) { return min(k0, k - 8); }

__device__ __forceinline__ u32x4 fragment_zeroed(u32x4 w, int k0, int k) {
  const int zeroed = min(k0 - fragment_start(k0, k), 8);   // elements at the chunk's low end that an earlier chunk holds
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const int n = zeroed - 2 * d;
    w[d] &= n >= 2 ? 0u : n == 1 ? 0xffff0000u : 0xffffffffu;
  }
  return w;
}

// One wavefront's place in a tile of the launch: tiles are numbered along N first, then M, then the batch.
struct ShortKPlace {
  int batch, m0, n0;
};
__device__ __forceinline__ ShortKPlace short_k_place(const TileGemmParams& p, int tile, int wave) {
  const int per_batch = p.tiles_m * p.tiles_n;
  const int batch = tile / per_batch, in_batch = tile - batch * per_batch;
  const int tm = in_batch / p.tiles_n, tn = in_batch - tm * p.tiles_n;
  return ShortKPlace{batch, tm * kTileRows, tn * kTileCols + wave * kWaveCols};
}

// The wavefront's operand fragments of one step of 32 along K, as loaded (rows past the operand read its last row:
// what they produce is not stored).
template <int SRC>
struct ShortKFragments {
  Staged<SRC> a[2], b[4];
  __device__ __forceinline__ void load(const TileGemmParams& p, const ShortKPlace& at, int lane, int k0) {
    const int frag_row = lane & 15, start = fragment_start(k0 + (lane >> 4) * 8, p.k);
#pragma unroll
    for (int i = 0; i < 2; ++i)
      a[i] = load_chunk_whole<SRC>(p.a, at.batch * p.a_bs + static_cast<int64_t>(min(at.m0 + i * 16 + frag_row, p.m - 1)) * p.a_rs + start);
#pragma unroll
    for (int j = 0; j < 4; ++j)
      b[j] = load_chunk_whole<SRC>(p.b, at.batch * p.b_bs + static_cast<int64_t>(min(at.n0 + j * 16 + frag_row, p.n - 1)) * p.b_rs + start);
  }
  // acc[i][j] += the 16 x 16 products of this step.  B's rows are the instruction's first operand: lane l ends up with
  // C[m0 + 16 i + l % 16][n0 + 16 j + 4 (l / 16) + 0..3], four consecutive columns of one row.
  __device__ __forceinline__ void multiply(f32x4 (&acc)[2][4], int lane, int k0, int k) const {
    u32x4 fa[2], fb[4];
#pragma unroll
    for (int i = 0; i < 2; ++i) fa[i] = fragment_zeroed(a[i].chunk(), k0 + (lane >> 4) * 8, k);
#pragma unroll
    for (int j = 0; j < 4; ++j) fb[j] = fragment_zeroed(b[j].chunk(), k0 + (lane >> 4) * 8, k);
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) mfma_step16<SRC>(acc[i][j], fb[j], fa[i]);
  }
};

// How a launch's results leave: as they are, 32 bits each, in 16-byte runs, or narrowed to 16 bits, eight to a 16-byte
// run.  Both: no fused transform, C's rows contiguous and every run inside C and aligned, a C input (if any) laid out
// like C and of its type - anything else is the two-stage tile kernel's.
enum ShortKStore : int { STORE_PLAIN32 = 0, STORE_PLAIN_BF16 = 1, STORE_PLAIN_F16 = 2, STORE_NONE = -1 };

// A workgroup walks tiles blockIdx.x, blockIdx.x + gridDim.x, ...: the fragments of its next tile are on their way
// while it lays out and stores the tile at hand (a tile's loads and its stores are each a memory round trip, and a
// compute unit holds four workgroups: without the overlap a wavefront's life was 6 us for 8 KiB written).  The plain
// stores go through a buffer descriptor and switch a lane off by an offset beyond its range: every tile issues the
// same stores on every path, so the wait for the next tile's fragments can leave exactly them outstanding.
// CIN: a C input of C's own element type with contiguous, aligned rows (or one row for all: row stride 0) is added to the
// sums.  Its loads for the whole tile go out behind the next tile's fragment loads and are waited for before the first
// store: a tile's loads are then one round trip, at the price of the stores of the tile before having to land first
// (loads and stores complete in the order of their issue) - the other wavefronts of the unit cover that.
template <int SRC, int STORE, bool CIN>
__global__ __launch_bounds__(256) void tile_gemm_short_k_kernel(const TileGemmParams p) {
  __shared__ uint32_t staged[4][kStageRows * kPitch];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int frag_row = lane & 15, group = lane >> 4;
  const int total = p.tiles_m * p.tiles_n * p.batch;
  int tile = blockIdx.x;
  if (tile >= total) return;
  ShortKPlace at = short_k_place(p, tile, wave);
  ShortKFragments<SRC> frags;
  frags.load(p, at, lane, 0);
  uint32_t* mine = staged[wave];
  constexpr bool kNarrow = STORE == STORE_PLAIN_BF16 || STORE == STORE_PLAIN_F16;
  constexpr int kOutBytes = kNarrow ? 2 : 4;
  constexpr int kRun = 16 / kOutBytes;                        // elements of C a lane stores at once (plain paths)
  constexpr int kLanesPerRow = kWaveCols / kRun, kRowsPerStep = 64 / kLanesPerRow;
  const int my_row = lane / kLanesPerRow, my_col = (lane % kLanesPerRow) * kRun;
  const uint32_t row_bytes = static_cast<uint32_t>(p.c_rs) * kOutBytes;
  const uint32_t cin_row_bytes = static_cast<uint32_t>(p.cin_rs) * kOutBytes;
  constexpr int kSteps = kStageRows / kRowsPerStep;           // store instructions a block of sixteen rows takes
  {
    // As many stores as a tile issues, every lane switched off: the first pass of the loop then meets what every
    // later one does - its fragments' loads with one tile's stores behind them - and the wait the compiler places
    // at the loop's head is for the loads alone on every pass.
    const __amdgpu_buffer_rsrc_t out = tile_buffer((const VECOPS_GLOBAL char*)p.c);
#pragma unroll
    for (int st = 0; st < 2 * kStageRows / kRowsPerStep; ++st)
      __builtin_amdgcn_raw_buffer_store_b128(u32x4{0u, 0u, 0u, 0u}, out, 0x80000000u + 16u * st, 0, 0);   // (distinct: none is dead)
  }

  while (true) {
    f32x4 acc[2][4];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};
    frags.multiply(acc, lane, 0, p.k);
    for (int k0 = 32; k0 < p.k; k0 += 32) {
      frags.load(p, at, lane, k0);
      frags.multiply(acc, lane, k0, p.k);
    }
    const int batch = at.batch, m0 = at.m0, n0 = at.n0;
    tile += gridDim.x;
    const bool more = tile < total;
    at = short_k_place(p, min(tile, total - 1), wave);   // (past the last tile: that tile's fragments again, unused)
    frags.load(p, at, lane, 0);
    u32x4 cin[2][kSteps];
    if constexpr (CIN) {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int row0 = m0 + i * kStageRows;
        const __amdgpu_buffer_rsrc_t in = tile_buffer(
            (const VECOPS_GLOBAL char*)p.cin + (batch * p.cin_bs + static_cast<int64_t>(row0) * p.cin_rs + n0) * kOutBytes);
#pragma unroll
        for (int step = 0; step < kSteps; ++step) {
          const int r = step * kRowsPerStep + my_row;
          const uint32_t offset = (n0 + my_col < p.n && row0 + r < p.m) ? static_cast<uint32_t>(r) * cin_row_bytes + my_col * kOutBytes : 0x80000000u;
          cin[i][step] = __builtin_amdgcn_raw_buffer_load_b128(in, offset, 0, 0);   // (a lane switched off reads zeros)
        }
      }
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int row0 = m0 + i * kStageRows;
      __builtin_amdgcn_wave_barrier();   // the reads of the block before are issued: LDS serves one wavefront in order
#pragma unroll
      for (int j = 0; j < 4; ++j)
        *reinterpret_cast<u32x4*>(mine + frag_row * kPitch + j * 16 + group * 4) = __builtin_bit_cast(u32x4, acc[i][j]);
      __builtin_amdgcn_wave_barrier();
      // descriptor at C[batch][row0][n0]: a lane's offset is its row and column inside the block
      const __amdgpu_buffer_rsrc_t out = tile_buffer(
          (const VECOPS_GLOBAL char*)p.c + (batch * p.c_bs + static_cast<int64_t>(row0) * p.c_rs + n0) * kOutBytes);
      const bool col_ok = n0 + my_col < p.n;    // N is a multiple of the run: a run lies inside C or outside
#pragma unroll
      for (int step = 0; step < kSteps; ++step) {
        const int r = step * kRowsPerStep + my_row;
        u32x4 v = *reinterpret_cast<const u32x4*>(mine + r * kPitch + my_col);
        if constexpr (kNarrow) {
          constexpr int kKind = STORE == STORE_PLAIN_BF16 ? OUT_BF16 : OUT_F16;
          const u32x4 hi = *reinterpret_cast<const u32x4*>(mine + r * kPitch + my_col + 4);
          float f[8];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            f[e] = __uint_as_float(v[e]);
            f[4 + e] = __uint_as_float(hi[e]);
          }
          if constexpr (CIN) {   // acc + float(cin), then the one rounding to C's type
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              const uint32_t bits = (cin[i][step][e >> 1] >> ((e & 1) * 16)) & 0xffffu;
              f[e] += kKind == OUT_BF16 ? bf16_bits_to_f32(bits) : f16_bits_to_f32(bits);
            }
          }
          uint32_t h[8];
#pragma unroll
          for (int e = 0; e < 8; ++e) h[e] = float_output_bits(kKind, f[e]);
          v = u32x4{h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16)};
        } else if constexpr (CIN) {
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = __float_as_uint(__uint_as_float(v[e]) + __uint_as_float(cin[i][step][e]));
        }
        const uint32_t offset = (col_ok && row0 + r < p.m) ? static_cast<uint32_t>(r) * row_bytes + my_col * kOutBytes : 0x80000000u;
        __builtin_amdgcn_raw_buffer_store_b128(v, out, offset, 0, 0);
      }
    }
    if (!more) break;
  }
}

// Launches one instance on as many workgroups as the device holds at once (every workgroup then starts at time zero
// and walks its share of the tiles: the instances use 104 to 164 registers a lane, three or four workgroups a unit).
template <auto KERNEL>
hipError_t launch_resident(const TileGemmParams& p, int64_t tiles, hipStream_t stream) {
  static thread_local int resident = 0, resident_device = -1;
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return e;
  if (resident_device != device) {
    int per_unit = 0, units = 0;
    e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_unit, KERNEL, 256, 0);
    if (e != hipSuccess) return e;
    e = hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, device);
    if (e != hipSuccess) return e;
    resident = (per_unit > 0 ? per_unit : 1) * (units > 0 ? units : 1);
    resident_device = device;
  }
  const dim3 grid(static_cast<unsigned>(tiles < resident ? tiles : resident)), block(256);
  hipLaunchKernelGGL(KERNEL, grid, block, 0, stream, p);
  return hipGetLastError();
}

// Which of the store forms a launch's C takes (STORE_NONE: none of them).
int store_kind(const TileGemmParams& p) {
  if (p.fused != 0) return STORE_NONE;
  const int out_bytes = (p.out_kind == OUT_BF16 || p.out_kind == OUT_F16) ? 2 : (p.out_kind == OUT_F32) ? 4 : 0;
  if (out_bytes == 0) return STORE_NONE;
  // every run of 16 bytes lies inside C or outside and starts on a 16-byte boundary; the offsets inside a block of
  // sixteen rows fit the descriptor's range
  const int64_t run = 16 / out_bytes;
  if (p.c_cs != 1 || p.n % run != 0 || p.c_rs % run != 0 || p.c_bs % run != 0 || (reinterpret_cast<uintptr_t>(p.c) & 15u) != 0 ||
      p.c_rs <= 0 || (kStageRows * p.c_rs + kWaveCols) * out_bytes >= (int64_t{1} << 31))
    return STORE_NONE;
  // a C input: C's own element type, rows as C's (a row stride of 0 is one row for all)
  if (p.cin != nullptr && (p.cin_kind != p.out_kind || p.cin_cs != 1 || p.cin_rs < 0 || p.cin_rs % run != 0 || p.cin_bs % run != 0 ||
                           (reinterpret_cast<uintptr_t>(p.cin) & 15u) != 0 ||
                           (kStageRows * p.cin_rs + kWaveCols) * out_bytes >= (int64_t{1} << 31)))
    return STORE_NONE;
  return p.out_kind == OUT_F32 ? STORE_PLAIN32 : p.out_kind == OUT_BF16 ? STORE_PLAIN_BF16 : STORE_PLAIN_F16;
}

template <int SRC>
hipError_t launch(const TileGemmParams& p, hipStream_t stream) {
  const int64_t tiles = static_cast<int64_t>(p.tiles_m) * p.tiles_n * p.batch;
  if (tiles <= 0 || tiles > INT32_MAX) return hipErrorInvalidConfiguration;
  auto go = [&](auto store_tag) {
    constexpr int STORE = decltype(store_tag)::value;
    return p.cin != nullptr ? launch_resident<tile_gemm_short_k_kernel<SRC, STORE, true>>(p, tiles, stream)
                            : launch_resident<tile_gemm_short_k_kernel<SRC, STORE, false>>(p, tiles, stream);
  };
  switch (store_kind(p)) {
    case STORE_PLAIN32: return go(std::integral_constant<int, STORE_PLAIN32>{});
    case STORE_PLAIN_BF16: return go(std::integral_constant<int, STORE_PLAIN_BF16>{});
    case STORE_PLAIN_F16: return go(std::integral_constant<int, STORE_PLAIN_F16>{});
    default: return hipErrorInvalidConfiguration;
  }
}

}  // namespace

// What the kernel takes: 16-bit compute (bf16, f16, fp32 operands multiplied as bf16), both operands K-contiguous with at
// least eight elements a row (any extents, row strides and alignment), no K split; fp32, bf16 or f16 results into a C
// with contiguous, 16-byte aligned rows and N a multiple of four (fp32) or eight, no fused transform; a C input of C's
// type with rows like C's (or one row for all).
bool launch_tile_gemm_short_k_serves(int src, const TileGemmParams& p) {
  if (src != SRC_BF16 && src != SRC_F16 && src != SRC_F32_AS_BF16) return false;
  return p.m > 0 && p.n > 0 && p.k >= 8 && p.split_k == 1 && p.a_ks == 1 && p.b_ks == 1 && store_kind(p) != STORE_NONE;
}

// (sets the tile counts of its own 32 x 256 tile in its copy of the parameters)
hipError_t launch_tile_gemm_short_k(int src, TileGemmParams p, hipStream_t stream) {
  p.tiles_m = (p.m + kTileRows - 1) / kTileRows;
  p.tiles_n = (p.n + kTileCols - 1) / kTileCols;
  switch (src) {
    case SRC_BF16: return launch<SRC_BF16>(p, stream);
    case SRC_F16: return launch<SRC_F16>(p, stream);
    case SRC_F32_AS_BF16: return launch<SRC_F32_AS_BF16>(p, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace vecops_hip
