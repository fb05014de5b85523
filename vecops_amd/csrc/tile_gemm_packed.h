// Tile GEMM with a prepacked B operand for gfx950, and the kernel that packs it.
//
// The counterpart of vecops' ops::matmul_pack / matmul::packed_layout
// (ops/MatmulPack.h:9-117; AMX format packing/amx/Format.h:27-58,158-182): weights
// that are multiplied many times are shuffled once into the order the matrix cores
// consume, so that the multiplication can fetch them straight from global memory
// into MFMA operand registers.  B then bypasses LDS entirely: the LDS pipe, which
// the plain kernel keeps three quarters busy, carries only A.
//
// Packed layout (bytes; EPC = elements per 16-byte chunk: 8 for bf16 and f16, 16 for int8, 4 for fp32 kept as fp32 -
// the fp32-compute atom, whose matrix instruction takes one float per lane: a lane's chunk feeds four of them).
// B[N, K] is cut into blocks of 32 rows (n) x one MFMA k-step (2 * EPC elements of
// k); block (nb, ks) is 1 KiB at ((nb * KS) + ks) * 1024, KS = k-steps of K rounded
// up to whole K tiles (4 k-steps); inside it lane l of a wavefront owns the 16 bytes
// at l * 16: row nb * 32 + l % 32, k = (ks * 2 + l / 32) * EPC .. + EPC - 1.  Rows
// past N and k past K are zero.  A wavefront walking K for one fragment therefore
// reads one contiguous stream.
#ifndef VECOPS_HIP_TILE_GEMM_PACKED_H
#define VECOPS_HIP_TILE_GEMM_PACKED_H

#include "tile_gemm.h"

namespace vecops_hip {

// k-steps of the packed layout for a K extent (whole K tiles)
__host__ __device__ inline int64_t packed_k_steps(int64_t k, int elems_per_chunk) {
  const int64_t ktile = 8 * elems_per_chunk;
  return (k + ktile - 1) / ktile * 4;
}
__host__ __device__ inline int64_t packed_b_bytes(int64_t n, int64_t k, int elems_per_chunk) {
  return (n + 31) / 32 * packed_k_steps(k, elems_per_chunk) * 1024;
}

struct PackBParams {
  const void* b;   // [N, K] with element strides rs, ks (unpacking: the destination)
  void* packed;
  int64_t rs, ks;
  int32_t n, k;
  uint32_t flip;   // bytes only: 0x80 packs an unsigned operand as the signed b - 128 (padding stays zero)
};

// One thread per 16-byte chunk of the packed operand.  SRC_BF16: bf16 in, bf16
// packed; SRC_F32_AS_BF16: fp32 in, rounded to bf16 (nearest even); SRC_F32: fp32 in, fp32 packed; SRC_I8: bytes.
template <int SRC>
__global__ __launch_bounds__(256) void pack_b_kernel(const PackBParams p) {
  constexpr int EPC = SrcTraits<SRC>::kElemsPerChunk;
  const int64_t ks_total = packed_k_steps(p.k, EPC);
  const int64_t chunks = (static_cast<int64_t>(p.n) + 31) / 32 * ks_total * 64;
  for (int64_t idx = blockIdx.x * 256ll + threadIdx.x; idx < chunks; idx += gridDim.x * 256ll) {
    const int lane = static_cast<int>(idx & 63);
    const int64_t block = idx >> 6;
    const int64_t nb = block / ks_total, ks = block - nb * ks_total;
    const int64_t n = nb * 32 + (lane & 31);
    const int64_t k0 = (ks * 2 + (lane >> 5)) * EPC;
    uint32_t w[4] = {0u, 0u, 0u, 0u};
    if (n < p.n) {
#pragma unroll
      for (int e = 0; e < EPC; ++e) {
        const int64_t k = k0 + e;
        if (k < p.k) {
          const int64_t at = n * p.rs + k * p.ks;
          uint32_t v;
          if constexpr (SRC == SRC_BF16) v = static_cast<const uint16_t*>(p.b)[at];
          else if constexpr (SRC == SRC_F32_AS_BF16) v = cvt_pk_bf16(static_cast<const float*>(p.b)[at], 0.0f) & 0xffffu;
          else if constexpr (SRC == SRC_F32) v = static_cast<const uint32_t*>(p.b)[at];
          else v = static_cast<const uint8_t*>(p.b)[at] ^ p.flip;
          constexpr int per_word = EPC / 4;
          w[e / per_word] |= v << ((e % per_word) * (32 / per_word));
        }
      }
    }
    static_cast<u32x4*>(p.packed)[idx] = u32x4{w[0], w[1], w[2], w[3]};
  }
}

// The inverse: the dense [N, K] operand (element strides rs, ks) back out of its packed form; 16-bit elements,
// bytes or fp32 (SRC_BF16 / SRC_I8 / SRC_F32), p.flip undone.  Used when both operands of a product arrive packed.
template <int SRC>
__global__ __launch_bounds__(256) void unpack_b_kernel(const PackBParams p) {
  constexpr int EPC = SrcTraits<SRC>::kElemsPerChunk;
  const int64_t ks_total = packed_k_steps(p.k, EPC);
  const int64_t chunks = (static_cast<int64_t>(p.n) + 31) / 32 * ks_total * 64;
  for (int64_t idx = blockIdx.x * 256ll + threadIdx.x; idx < chunks; idx += gridDim.x * 256ll) {
    const int lane = static_cast<int>(idx & 63);
    const int64_t block = idx >> 6;
    const int64_t nb = block / ks_total, ks = block - nb * ks_total;
    const int64_t n = nb * 32 + (lane & 31);
    const int64_t k0 = (ks * 2 + (lane >> 5)) * EPC;
    if (n >= p.n || k0 >= p.k) continue;
    const u32x4 v = static_cast<const u32x4*>(p.packed)[idx];
    const uint32_t w[4] = {v[0], v[1], v[2], v[3]};
    constexpr int per_word = EPC / 4;
#pragma unroll
    for (int e = 0; e < EPC; ++e) {
      const int64_t k = k0 + e;
      if (k < p.k) {
        const uint32_t bits = w[e / per_word] >> ((e % per_word) * (32 / per_word));
        const int64_t at = n * p.rs + k * p.ks;
        if constexpr (SRC == SRC_BF16) static_cast<uint16_t*>(const_cast<void*>(p.b))[at] = static_cast<uint16_t>(bits);
        else if constexpr (SRC == SRC_F32) static_cast<uint32_t*>(const_cast<void*>(p.b))[at] = bits;
        else static_cast<uint8_t*>(const_cast<void*>(p.b))[at] = static_cast<uint8_t>(bits ^ p.flip);
      }
    }
  }
}

// C = C_in + A . B^T with B prepacked.  Workgroup = 2 x 2 wavefronts of WM x WN
// accumulator tiles; p.b addresses the packed operand (p.b_rs / b_ks / b_bs unused:
// a packed B has no batch dimension and is shared by every batch, as in vecops).
// A goes through LDS exactly as in tile_gemm_kernel (two stages, staging registers
// stored and refilled part by part).  The B fragments of a whole K tile live in
// registers; the MFMAs of a k-step run fragment by fragment (all A rows against B
// fragment 0, then fragment 1, ...), and as soon as the last MFMA that reads a
// fragment register has issued, the same register is refilled with that fragment
// of the next K tile - a whole K tile of MFMA work ahead of its use.
template <int SRC, int WAVES_M, int WAVES_N, int WM, int WN, int LOAD_A>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N) void tile_gemm_packed_b_kernel(const TileGemmParams p) {
  using T = SrcTraits<SRC>;
  constexpr bool INT = T::kInt;
  using Acc = typename AccTile<INT>::type;
  constexpr int EPC = T::kElemsPerChunk;
  constexpr int KTILE = 8 * EPC;
  constexpr int THREADS = 64 * WAVES_M * WAVES_N;
  constexpr int BM = 32 * WAVES_M * WM, BN = 32 * WAVES_N * WN;
  constexpr int STAGE_BYTES = BM * 128;
  constexpr int N_MFMA = WM * WN;
  constexpr int kEpilogueBytes = kEpilogueLdsBytes<WAVES_M, WAVES_N, WM, WN>();
  constexpr int kLdsBytes = 2 * STAGE_BYTES > kEpilogueBytes ? 2 * STAGE_BYTES : kEpilogueBytes;

  extern __shared__ __attribute__((aligned(16))) char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;

  int batch, split, tm, tn;
  map_workgroup(p, blockIdx.x, gridDim.x, batch, split, tm, tn);
  batch = __builtin_amdgcn_readfirstlane(batch);
  split = __builtin_amdgcn_readfirstlane(split);
  tm = __builtin_amdgcn_readfirstlane(tm);
  tn = __builtin_amdgcn_readfirstlane(tn);
  const int m0 = tm * BM, n0 = tn * BN;

  const int total_k_tiles = (p.k + KTILE - 1) / KTILE;
  const int full_k_tiles = p.k / KTILE;
  const int kt_begin = split * p.k_tiles_per_split;
  const int kt_end = min(total_k_tiles, kt_begin + p.k_tiles_per_split);
  const int nk = __builtin_amdgcn_readfirstlane(kt_end - kt_begin);
  const int has_tail = __builtin_amdgcn_readfirstlane((nk > 0 && kt_end > full_k_tiles) ? 1 : 0);
  // the partial last K tile (if this split owns it) comes first: see tile_gemm_kernel
  auto seq = [&](int j) { return (has_tail && j == 0) ? kt_end - 1 : kt_begin + j - has_tail; };

  Stager<SRC, LOAD_A, BM, THREADS> stager_a;
  stager_a.init(static_cast<const char*>(p.a) + batch * p.a_bs * T::kSrcBytes, p.a_rs, p.a_ks, m0, p.m, p.k, tid, p.a_flip);
  using SA = decltype(stager_a);

  // packed B: descriptor at the first 32-row block of this tile; the lane offset picks block row and lane
  const int64_t ks_total = static_cast<int64_t>(total_k_tiles) * 4;
  const int nb0 = n0 / 32, nb_last = (p.n + 31) / 32 - 1;
  const __amdgpu_buffer_rsrc_t b_buf =
      tile_buffer((const VECOPS_GLOBAL char*)p.b + static_cast<int64_t>(nb0) * ks_total * 1024);
  uint32_t b_off[WN];
#pragma unroll
  for (int j = 0; j < WN; ++j)  // blocks past N are clamped: computed, never stored
    b_off[j] = static_cast<uint32_t>((min(nb0 + wn * WN + j, nb_last) - nb0) * ks_total * 1024 + lane * 16);

  const int frag_row = lane & 31;
  const int frag_half = lane >> 5;
  int off_a[WM];
#pragma unroll
  for (int i = 0; i < WM; ++i) off_a[i] = lds_chunk_offset((wm * WM + i) * 32 + frag_row, frag_half);

  u32x4 fa[2][WM];
  u32x4 bq[4][WN];
  auto read_a = [&](int set, const char* tile, int ks, auto i_tag) {
    constexpr int i = decltype(i_tag)::value;
    fa[set][i] = *reinterpret_cast<const u32x4*>(tile + (off_a[i] ^ (ks << 5)));
  };
  auto load_b = [&](auto ks_tag, auto j_tag, int kt) {
    constexpr int ks = decltype(ks_tag)::value, j = decltype(j_tag)::value;
    bq[ks][j] = __builtin_amdgcn_raw_buffer_load_b128(b_buf, b_off[j], (kt * 4 + ks) * 1024, 0);
  };
  auto lds_barrier = [&]() {
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0), vmcnt / expcnt untouched
    __builtin_amdgcn_s_barrier();
  };

  // LOAD_KDMA: A's loads write LDS themselves (the counted form: B's register loads are in flight beside them)
  constexpr bool DMA_A = LOAD_A == LOAD_KDMA;
  // Start: A tiles 0 and 1 as in tile_gemm_kernel; the B fragments of tile 0.
  if constexpr (DMA_A) {
    if (nk > 0) {
      const int first = __builtin_amdgcn_readfirstlane(seq(0));
      if (first < full_k_tiles) static_for<SA::kParts>([&](auto ci) { stager_a.dma_part_counted(decltype(ci)::value, first, lds); });
      else stager_a.stage_checked(first, lds);
      static_for<4>([&](auto cks) { static_for<WN>([&](auto cj) { load_b(cks, cj, first); }); });
    }
  } else if constexpr (!DMA_A) {
   if (nk > 0) {
    const int first = __builtin_amdgcn_readfirstlane(seq(0));
    const int second = __builtin_amdgcn_readfirstlane(seq(nk > 1 ? 1 : 0));
    const bool tail_first = first >= full_k_tiles;
    if (!tail_first) stager_a.fetch_full(first);
    else if constexpr (SA::kStagesChecked) stager_a.stage_checked(first, lds);
    else stager_a.fetch_checked(first);
    static_for<4>([&](auto cks) { static_for<WN>([&](auto cj) { load_b(cks, cj, first); }); });
    typename SA::Spare spare_a;
    if (nk > 1) {
      if constexpr (SA::kHasSpare) stager_a.fetch_full_spare(spare_a, second);
    }
    if (!(SA::kStagesChecked && tail_first)) stager_a.commit(lds);
    if (nk > 1) {
      if constexpr (SA::kHasSpare) stager_a.take_spare(spare_a);
      else stager_a.fetch_full(second);
    }
   }
  }

  Accumulators<INT, WM, WN, false> accumulators;  // prepacked fragments are those of the 32x32 shapes
  auto& acc = accumulators.t;
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

  if (nk > 0) {
    const int full_in_range = nk - has_tail;
    // Every load of the start-up has landed before the loop is entered.  Without this the compiler's
    // wait insertion, which does not know that both start-up branches test the same condition, carries
    // "spare tile still in flight" into the loop and waits for nearly all loads in every iteration.
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
    lds_barrier();  // tile 0 is in LDS
    static_for<WM>([&](auto ci) { read_a(0, lds, 0, ci); });

    // Per k-step: 16 slots of one MFMA plus the memory operations dealt to the slot -
    // A fragment reads of the next k-step, this step's share of A's staging stores and
    // refills, and the refill of each B fragment register behind its last reader.
    auto main_loop = [&](auto prefetch_tag) {
      constexpr bool PREFETCH = decltype(prefetch_tag)::value;
      constexpr int PARTS = SA::kParts;
      for (int it = 0; it < nk; ++it) {
        const char* tile = lds + (it & 1) * STAGE_BYTES;
        char* other = lds + ((it & 1) ^ 1) * STAGE_BYTES;
        // K tiles to prefetch, clamped to the last one, never the tail tile (position 0)
        const int t1 = __builtin_amdgcn_readfirstlane(kt_begin - has_tail + max(has_tail, min(it + 1, nk - 1)));
        const int t2 = __builtin_amdgcn_readfirstlane(kt_begin - has_tail + max(has_tail, min(it + 2, nk - 1)));
        auto slots = [&](auto ks_tag, auto s0_tag, auto s1_tag, auto reads_tag, auto stage_tag) {
          constexpr int KS = decltype(ks_tag)::value, S0 = decltype(s0_tag)::value, S1 = decltype(s1_tag)::value;
          constexpr int NS = S1 - S0;
          constexpr bool READS = decltype(reads_tag)::value, STAGE = decltype(stage_tag)::value;
          // the staging parts of this k-step: stores, then refills (k-step 3 has the barrier behind its stores)
          // (loads that write LDS: no stores; the parts of tile it + 1 go into the other stage in k-steps 0 and 1)
          constexpr int P0 = DMA_A ? (KS < 2 ? KS * PARTS / 2 : PARTS) : (KS * PARTS + 3) / 4;
          constexpr int P1 = DMA_A ? (KS < 2 ? (KS + 1) * PARTS / 2 : PARTS) : ((KS + 1) * PARTS + 3) / 4;
          constexpr int NP = STAGE ? P1 - P0 : 0;
          constexpr int OPS = DMA_A ? NP : NP * 2;
          auto stage_op = [&](auto cg) {
            constexpr int g = decltype(cg)::value;
            if constexpr (DMA_A) {
              if constexpr (PREFETCH) stager_a.dma_part_counted(P0 + g, t1, other);
            } else {
              if constexpr (g < NP) stager_a.template store_op<P0 + g, 0>(other);
              else if constexpr (PREFETCH) stager_a.template load_op<P0 + g - NP, 0>(t2, 0u);
            }
          };
          if constexpr (NS == 0) static_for<OPS>(stage_op);
          static_for<NS>([&](auto cs) {
            constexpr int s = decltype(cs)::value, x = S0 + s;
            constexpr int i = x % WM, j = x / WM;
            mfma_step<SRC>(acc[i][j], bq[KS][j], fa[KS & 1][i]);  // B rows first: see the epilogue
            if constexpr (i == WM - 1) load_b(ks_tag, std::integral_constant<int, j>{}, t1);
            if constexpr (READS) {
              constexpr int r0 = (s * WM + NS - 1) / NS, r1 = ((s + 1) * WM + NS - 1) / NS;
              static_for<r1 - r0>([&](auto cr) {
                constexpr int r = r0 + decltype(cr)::value;
                if constexpr (KS < 3) read_a((KS + 1) & 1, tile, KS + 1, std::integral_constant<int, r>{});
                else read_a(0, other, 0, std::integral_constant<int, r>{});
              });
            }
            constexpr int g0 = s * OPS / NS, g1 = (s + 1) * OPS / NS;
            static_for<g1 - g0>([&](auto cg) { stage_op(std::integral_constant<int, g0 + decltype(cg)::value>{}); });
            __builtin_amdgcn_sched_barrier(0);
          });
        };
        using I0 = std::integral_constant<int, 0>;
        using All = std::integral_constant<int, N_MFMA>;
        using Half = std::integral_constant<int, N_MFMA / 2>;
        slots(std::integral_constant<int, 0>{}, I0{}, All{}, std::true_type{}, std::true_type{});
        slots(std::integral_constant<int, 1>{}, I0{}, All{}, std::true_type{}, std::true_type{});
        slots(std::integral_constant<int, 2>{}, I0{}, All{}, std::true_type{}, std::true_type{});
        slots(std::integral_constant<int, 3>{}, I0{}, Half{}, std::false_type{}, std::true_type{});
        // A's loads of the next tile have landed once no more loads are in flight than the B fragment loads
        // issued after them (those of k-step 2 and of the first half of k-step 3)
        if constexpr (DMA_A) __builtin_amdgcn_s_waitcnt(0x0f70 | (WN + WN / 2));
        lds_barrier();
        slots(std::integral_constant<int, 3>{}, Half{}, All{}, std::true_type{}, std::false_type{});
      }
    };
    if (full_in_range > 0) main_loop(std::true_type{});
    else main_loop(std::false_type{});
  }

  store_accumulators<SRC, WAVES_M, WAVES_N, WM, WN, kLdsBytes, false>(p, lds, accumulators, batch, split, m0, n0, wm, wn, wave,
                                                                      lane);
}

}  // namespace vecops_hip
#endif
