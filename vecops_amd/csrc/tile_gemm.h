// MFMA workgroup-tile GEMM for gfx950: C[M,N] (+)= A[M,K] . B[N,K]^T.
//
// Geometry (identical in bytes for every operand type):
//   * a K tile is 128 bytes of operand per row = eight 16-byte chunks
//     (64 bf16 or 128 int8 elements);
//   * one MFMA k-step consumes two chunks: lanes 0-31 take the even chunk,
//     lanes 32-63 the odd one, each lane holding 16 contiguous bytes of its row
//     (v_mfma_f32_32x32x16_bf16: 8 bf16; v_mfma_i32_32x32x32_i8: 16 int8);
//   * a workgroup is WAVES_M x WAVES_N wavefronts; each wavefront owns
//     WM x WN accumulator tiles of 32x32, so the workgroup tile is
//     (32*WAVES_M*WM) x (32*WAVES_N*WN);
//   * LDS holds two stages of (BM + BN) rows x 128 bytes; chunk c of row r lives
//     at r*128 + (((c ^ r ^ r/8) & 7) * 16), which makes the 16-byte reads of eight
//     consecutive rows hit eight different bank groups.
//
// fp32 operands in "bf16 compute" mode are rounded to bf16 (nearest even) while
// they are staged into LDS, so the inner loop is the bf16 one.
#ifndef VECOPS_HIP_TILE_GEMM_H
#define VECOPS_HIP_TILE_GEMM_H


#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

namespace vecops_hip {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(16))) int i32x16;
typedef __attribute__((ext_vector_type(4))) unsigned u32x4;
typedef __attribute__((ext_vector_type(2))) unsigned u32x2;

// SRC_I8_FLIP: 8-bit integer operands of which at least one is unsigned.  The
// matrix cores multiply signed bytes only, so an unsigned operand is staged as
// s = u xor 0x80 = u - 128 and the difference is added back in the epilogue:
//   sum_k ua*b  = sum_k sa*b  + 128 * sum_k b          (per output column)
//   sum_k a*ub  = sum_k a*sb  + 128 * sum_k a          (per output row)
//   sum_k ua*ub = sum_k sa*sb + 128 * sum_k sb + 128 * sum_k sa + 16384 * K
// all in wrapping 32-bit arithmetic, like the accumulators themselves.
// SRC_F32: fp32 operands multiplied in fp32 on the fp32 matrix cores
// (v_mfma_f32_32x32x2_f32); a 16-byte chunk holds four k, a k-step (two chunks)
// feeds four MFMAs per accumulator tile, a K tile is 32 elements.
enum SrcKind : int { SRC_BF16 = 0, SRC_F32_AS_BF16 = 1, SRC_I8 = 2, SRC_I8_FLIP = 3, SRC_F32 = 4, SRC_F16 = 5 };
enum OutKind : int { OUT_F32 = 0, OUT_BF16 = 1, OUT_I32 = 2, OUT_U8 = 3, OUT_I8 = 4, OUT_F16 = 5 };
enum Activation : int { ACT_NONE = 0, ACT_RELU = 1, ACT_CLAMP = 2, ACT_SIGMOID = 3, ACT_SILU = 4 };
// How an operand tile is fetched from global memory.
enum LoadKind : int {
  LOAD_KVEC = 0,     // K contiguous (rows at any element alignment): one 16-byte load per chunk
  LOAD_GENERIC = 1,  // any strides: one load per element
  LOAD_NTR = 3,      // spatial index contiguous (B given as [K,N] row-major), 16-bit compute elements: stored in
                     // LDS as it lies in memory ([k][n]) and transposed by the LDS read (ds_read_b64_tr_b16)
  LOAD_KDMA = 4,     // LOAD_KVEC with the loads writing LDS themselves (buffer_load ... lds): no staging
                     // registers, no LDS store instructions
  LOAD_NTR_DMA = 5,  // LOAD_NTR likewise; rows of the [k][n] tile are packed (no pad) and swizzled instead
  LOAD_KN32 = 6      // the same operand layout for 32-bit compute elements (fp32 on the fp32 matrix cores): stored in LDS
                     // as it lies in memory ([k][n]); a matrix instruction's operand is one 4-byte LDS read per lane
};
constexpr bool load_is_dma(int load) { return load == LOAD_KDMA || load == LOAD_NTR_DMA; }
constexpr bool load_is_ntr(int load) { return load == LOAD_NTR || load == LOAD_NTR_DMA; }

struct TileGemmParams {
  const void* a;
  const void* b;
  const void* cin;  // null = zero accumulator
  void* c;
  void* partial;    // split-K partial sums [split][batch][M][N] in accumulator type
  const float* row_scales;     // int8 dequant epilogue (null = none); batch b reads row_scales[b * row_scales_bs + row]
  const float* column_scales;
  const int32_t* correction;   // int32 row added to every accumulator row (null = none): correction[b * correction_bs + col]
  int64_t row_scales_bs, correction_bs;  // 0 = one set for every batch
  // unsigned-operand terms (SRC_I8_FLIP; null / zero = none), added to the accumulator first
  const int32_t* row_term;     // [batch][M]
  const int32_t* col_term;     // [batch][N]
  uint32_t const_term;
  uint32_t a_flip, b_flip;     // 0x80808080 for an unsigned operand, else 0
  int32_t m, n, k;
  int32_t batch;
  int32_t tiles_m, tiles_n;
  int32_t split_k;
  int32_t k_tiles_per_split;
  int32_t out_kind;
  int32_t cin_kind;
  int64_t a_rs, a_ks, a_bs;  // row, k and batch strides in elements
  int64_t b_rs, b_ks, b_bs;
  int64_t c_rs, c_cs, c_bs;
  int64_t cin_rs, cin_cs, cin_bs;
  // Fused output transform (fused != 0), applied once the accumulator (+ C-input, + the dequantisation
  // above) is a float:  v * ep_row_scales[row] * ep_column_scales[col] * ep_scale + ep_shift, then the
  // activation, then the conversion to the memory dtype of C.
  const float* ep_row_scales;     // [batch][M]; null = none
  const float* ep_column_scales;  // null = none
  float ep_scale, ep_shift;       // used when ep_flags has bit 0 / bit 1
  float ep_lo, ep_hi;             // ACT_CLAMP bounds
  uint32_t ep_flags;
  int32_t ep_act;
  int32_t fused;
};

template <int SRC>
struct SrcTraits;
template <>
struct SrcTraits<SRC_BF16> {
  static constexpr int kElemsPerChunk = 8;
  static constexpr int kSrcBytes = 2;
  static constexpr bool kInt = false;
};
template <>
struct SrcTraits<SRC_F16> : SrcTraits<SRC_BF16> {};  // IEEE half: same 16-bit chunks, its own MFMA
template <>
struct SrcTraits<SRC_F32_AS_BF16> {
  static constexpr int kElemsPerChunk = 8;
  static constexpr int kSrcBytes = 4;
  static constexpr bool kInt = false;
};
template <>
struct SrcTraits<SRC_I8> {
  static constexpr int kElemsPerChunk = 16;
  static constexpr int kSrcBytes = 1;
  static constexpr bool kInt = true;
};
template <>
struct SrcTraits<SRC_I8_FLIP> : SrcTraits<SRC_I8> {};
template <>
struct SrcTraits<SRC_F32> {
  static constexpr int kElemsPerChunk = 4;
  static constexpr int kSrcBytes = 4;
  static constexpr bool kInt = false;
};

// fp32 -> bf16 bits, round to nearest even; NaN -> 0x7fc0 (vecops util/BFloat16.h:25-37).
__device__ __forceinline__ uint32_t bf16_bits_rne(float x) {
  uint32_t bits = __float_as_uint(x);
  uint32_t rounded = (bits + (((bits >> 16) & 1u) + 0x7fffu)) >> 16;
  return (x != x) ? 0x7fc0u : rounded;
}

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  return bf16_bits_rne(lo) | (bf16_bits_rne(hi) << 16);
}

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

// IEEE binary16 <-> fp32 with the hardware converters (to half: round to nearest even, overflow to infinity -
// what vecops' Float16 does through F16C, util/Float16.h).
__device__ __forceinline__ uint32_t f16_bits_rne(float x) {
  return __builtin_bit_cast(uint16_t, static_cast<_Float16>(x));
}
__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) {
  return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(h)));
}

// LDS byte offset of 16-byte chunk `chunk` (0..7) of tile row `row`.  The chunk
// slot is XOR-swizzled with (row ^ row/8): eight consecutive rows at one logical
// chunk (the MFMA fragment read), the eight chunks of one row (the K-contiguous
// staging write) and eight rows 8 apart at one chunk (the transposing staging
// write) all land in eight different 16-byte slots of the 128-byte bank period.
__device__ __forceinline__ int lds_chunk_offset(int row, int chunk) {
  return row * 128 + (((chunk ^ row ^ (row >> 3)) & 7) << 4);
}

typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;

// Two fp32 -> packed bf16 pair with the hardware converter (round to nearest even).
__device__ __forceinline__ uint32_t cvt_pk_bf16(float lo, float hi) {
  f32x2 v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}

#define VECOPS_GLOBAL __attribute__((address_space(1)))

// Tells the compiler that a global pointer is the same in every lane, so that it is
// kept in scalar registers.
__device__ __forceinline__ const VECOPS_GLOBAL char* uniform_ptr(const VECOPS_GLOBAL char* p) {
  const uint64_t bits = reinterpret_cast<uint64_t>(p);
  const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(bits));
  const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(bits >> 32));
  return reinterpret_cast<const VECOPS_GLOBAL char*>((static_cast<uint64_t>(hi) << 32) | lo);
}

// Buffer descriptor over [base, base + 4 GiB): loads through it take the base from
// four scalar registers, a 32-bit per-lane byte offset and a scalar byte offset,
// so a load costs no vector ALU work for its address.  `base` must be the same in
// every lane.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t tile_buffer(const VECOPS_GLOBAL char* base) {
  return __builtin_amdgcn_make_buffer_rsrc((void*)uniform_ptr(base), 0, 0x7fffffff, 0x00020000);
}

// What the staging registers hold for one 16-byte chunk of compute elements between
// its global load and its LDS store.  fp32 operands that are multiplied as bf16 are
// held as loaded (32 bytes) and rounded only when they are stored: a conversion right
// behind the load would wait for the load and expose the memory latency of every chunk.
template <int SRC>
struct Staged {
  u32x4 v;
  __device__ __forceinline__ u32x4 chunk() const { return v; }
};
template <>
struct Staged<SRC_F32_AS_BF16> {
  u32x4 lo, hi;  // eight fp32 values
  __device__ __forceinline__ u32x4 chunk() const {
    u32x4 out;
    out.x = cvt_pk_bf16(__uint_as_float(lo.x), __uint_as_float(lo.y));
    out.y = cvt_pk_bf16(__uint_as_float(lo.z), __uint_as_float(lo.w));
    out.z = cvt_pk_bf16(__uint_as_float(hi.x), __uint_as_float(hi.y));
    out.w = cvt_pk_bf16(__uint_as_float(hi.z), __uint_as_float(hi.w));
    return out;
  }
};

// Fast path: one whole 16-byte chunk, no bounds checks (the caller guarantees
// that the row exists and that the chunk lies inside K).  `uniform_offset` (same in
// every lane) and `lane_offset` are byte offsets from the descriptor's base; their
// sum stays below 2^31.
template <int SRC>
__device__ __forceinline__ Staged<SRC> load_chunk_fast(__amdgpu_buffer_rsrc_t buffer, uint32_t lane_offset,
                                                       uint32_t uniform_offset) {
  if constexpr (SRC == SRC_F32_AS_BF16) {
    Staged<SRC> out;
    out.lo = __builtin_amdgcn_raw_buffer_load_b128(buffer, lane_offset, uniform_offset, 0);
    out.hi = __builtin_amdgcn_raw_buffer_load_b128(buffer, lane_offset + 16, uniform_offset, 0);
    return out;
  } else {
    return Staged<SRC>{__builtin_amdgcn_raw_buffer_load_b128(buffer, lane_offset, uniform_offset, 0)};
  }
}

// A whole chunk of K-contiguous source elements that lies inside its row, at any alignment (element-aligned
// addresses: the memory system takes 16-byte loads at any byte address).
template <int SRC>
__device__ __forceinline__ Staged<SRC> load_chunk_whole(const void* base, int64_t first_element) {
  Staged<SRC> out;  // (operands live in global memory: a global load, which LDS traffic does not wait for)
  __builtin_memcpy(&out, (const VECOPS_GLOBAL char*)base + first_element * SrcTraits<SRC>::kSrcBytes, sizeof(out));
  return out;
}

// Slow path: bounds checks and arbitrary K stride; used for the K tail of the vector path and for every chunk
// of the generic path.  A chunk that lies wholly inside a K-contiguous row is still one load; only the chunk
// that straddles the end of K (and every chunk of an operand whose K stride is not 1) goes element by element.
template <int SRC>
__device__ __noinline__ Staged<SRC> load_chunk_checked(const void* base, int64_t row_off, int64_t kstep, int k0,
                                                       int k_end, bool row_ok, uint32_t pad) {
  // `pad` is what an element outside the operand reads as: 0, or for an operand
  // that is xor-flipped on its way into LDS the flip byte, so that it ends up 0
  constexpr int EPC = SrcTraits<SRC>::kElemsPerChunk;
  if (kstep == 1 && row_ok && k0 + EPC <= k_end) return load_chunk_whole<SRC>(base, row_off + k0);
  if constexpr (SRC == SRC_F32_AS_BF16) {
    uint32_t w[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int k = k0 + e;
      w[e] = (row_ok && k < k_end) ? __float_as_uint(static_cast<const float*>(base)[row_off + k * kstep]) : 0u;
    }
    return Staged<SRC>{u32x4{w[0], w[1], w[2], w[3]}, u32x4{w[4], w[5], w[6], w[7]}};
  } else {
    uint32_t w0 = 0u, w1 = 0u, w2 = 0u, w3 = 0u;
#pragma unroll
    for (int e = 0; e < EPC; ++e) {
      const int k = k0 + e;
      uint32_t v = pad;
      if (row_ok && k < k_end) {
        if constexpr (SRC == SRC_BF16 || SRC == SRC_F16) v = static_cast<const uint16_t*>(base)[row_off + k * kstep];
        else if constexpr (SRC == SRC_F32) v = __float_as_uint(static_cast<const float*>(base)[row_off + k * kstep]);
        else v = static_cast<const uint8_t*>(base)[row_off + k * kstep];
      }
      constexpr int per_word = EPC / 4;
      const uint32_t shifted = v << ((e % per_word) * (32 / per_word));
      const int word = e / per_word;
      if (word == 0) w0 |= shifted;
      else if (word == 1) w1 |= shifted;
      else if (word == 2) w2 |= shifted;
      else w3 |= shifted;
    }
    return Staged<SRC>{u32x4{w0, w1, w2, w3}};
  }
}

// A whole operand tile (rows x eight chunks), bounds-checked (chunk by chunk where the rows are K-contiguous,
// element by element otherwise), straight into its LDS tile: the partial last K tile.  Out of line and rolled - it runs once per workgroup - and
// one call per operand: a call has to wait for its loads before it returns, so chunk-by-chunk calls
// would pay one memory round trip each.
template <int SRC>
__device__ __noinline__ void stage_rows_checked(const void* base, int64_t rs, int64_t kstep, int first_row, int extent,
                                                int rows, int k0_tile, int k_end, char* lds_tile, int tid,
                                                int threads, uint32_t flip) {
  constexpr int EPC = SrcTraits<SRC>::kElemsPerChunk;
  if (kstep == 1 && k_end >= EPC) {
    // K-contiguous rows of at least one chunk: every chunk is ONE load and no branch.  A chunk that straddles the
    // end of K (or lies beyond it) loads the row's last EPC elements instead and shifts them down, so that zeros
    // fill what lies past the end; a row past the operand loads the last row and shifts everything out.  (Element
    // loads under per-element conditions, as below, came out as one memory round trip per two elements: batch 8 of
    // 3000 x 3000 x 17, whose only K tile is a partial one, took 83 us that way and takes 67.)
    constexpr int ELEM_BITS = 128 / EPC;  // of the compute chunk: 16, 8 (bytes) or 32 (fp32 compute)
    constexpr int BATCH = 4;              // loads in flight before the first is used
    const int chunks = rows * 8;
    for (int idx0 = tid; idx0 < chunks; idx0 += threads * BATCH) {
      u32x4 v[BATCH];
#pragma unroll
      for (int j = 0; j < BATCH; ++j) {
        const int idx = min(idx0 + j * threads, chunks - 1);
        const int row_c = min(first_row + (idx >> 3), extent - 1);
        const int start = min(k0_tile + (idx & 7) * EPC, k_end - EPC);
        v[j] = load_chunk_whole<SRC>(base, static_cast<int64_t>(row_c) * rs + start).chunk();
      }
#pragma unroll
      for (int j = 0; j < BATCH; ++j) {
        const int idx = idx0 + j * threads;
        const int row = idx >> 3, chunk = idx & 7;
        const int k0 = k0_tile + chunk * EPC;
        u32x4 w = v[j];
        if constexpr (SRC == SRC_I8_FLIP) w ^= u32x4{flip, flip, flip, flip};
        const int shift = (first_row + row < extent) ? min(k0 - min(k0, k_end - EPC), EPC) : EPC;  // in elements
        const uint32_t bits = static_cast<uint32_t>(shift * ELEM_BITS);                            // 0 .. 128
        const uint64_t lo = (static_cast<uint64_t>(w.y) << 32) | w.x, hi = (static_cast<uint64_t>(w.w) << 32) | w.z;
        // (shifts by bits & 63 with the carried half masked out where the count is 0: no branch)
        const uint32_t b = bits & 63u;
        const uint64_t carry = b ? hi << (64u - b) : 0;
        const uint64_t lo_small = (lo >> b) | carry, hi_small = hi >> b;  // bits < 64
        const uint64_t out_lo = bits >= 128u ? 0 : bits >= 64u ? hi >> b : lo_small;
        const uint64_t out_hi = bits >= 64u ? 0 : hi_small;
        if (idx < chunks)
          *reinterpret_cast<u32x4*>(lds_tile + lds_chunk_offset(row, chunk)) =
              u32x4{static_cast<uint32_t>(out_lo), static_cast<uint32_t>(out_lo >> 32), static_cast<uint32_t>(out_hi),
                    static_cast<uint32_t>(out_hi >> 32)};
      }
    }
    return;
  }
#pragma unroll 2
  for (int idx = tid; idx < rows * 8; idx += threads) {
    const int row = idx >> 3, chunk = idx & 7;
    const int k0 = k0_tile + chunk * EPC;
    const bool row_ok = first_row + row < extent;
    const int64_t row_off = static_cast<int64_t>(first_row + row) * rs;
    u32x4 out;
    if (kstep == 1 && row_ok && k0 + EPC <= k_end) {  // a whole chunk inside the row: one load (two for fp32 pairs)
      out = load_chunk_whole<SRC>(base, row_off + k0).chunk();
      if constexpr (SRC == SRC_I8_FLIP) out ^= u32x4{flip, flip, flip, flip};
    } else if constexpr (SRC == SRC_F32_AS_BF16) {
      float f[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int k = k0 + e;
        f[e] = (row_ok && k < k_end) ? static_cast<const float*>(base)[row_off + k * kstep] : 0.0f;
      }
      out = u32x4{cvt_pk_bf16(f[0], f[1]), cvt_pk_bf16(f[2], f[3]), cvt_pk_bf16(f[4], f[5]), cvt_pk_bf16(f[6], f[7])};
    } else {
      uint32_t w[4] = {0u, 0u, 0u, 0u};
#pragma unroll
      for (int e = 0; e < EPC; ++e) {
        const int k = k0 + e;
        uint32_t v = flip & 0xffu;  // an element outside the operand: the flip byte, which the xor below turns into 0
        if (row_ok && k < k_end) {
          if constexpr (SRC == SRC_BF16 || SRC == SRC_F16) v = static_cast<const uint16_t*>(base)[row_off + k * kstep];
          else if constexpr (SRC == SRC_F32) v = __float_as_uint(static_cast<const float*>(base)[row_off + k * kstep]);
          else v = static_cast<const uint8_t*>(base)[row_off + k * kstep];
        }
        constexpr int per_word = EPC / 4;
        w[e / per_word] |= v << ((e % per_word) * (32 / per_word));
      }
      out = u32x4{w[0], w[1], w[2], w[3]};
      if constexpr (SRC == SRC_I8_FLIP) out ^= u32x4{flip, flip, flip, flip};
    }
    *reinterpret_cast<u32x4*>(lds_tile + lds_chunk_offset(row, chunk)) = out;
  }
}

template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (N > 0) {
    static_for<N - 1>(f);
    f(std::integral_constant<int, N - 1>{});
  }
}

// Accumulator tile type per operand class.
template <bool INT>
struct AccTile {
  using type = f32x16;
};
template <>
struct AccTile<true> {
  using type = i32x16;
};

template <bool INT>
struct AccQuad {
  using type = f32x4;
};
template <>
struct AccQuad<true> {
  using type = i32x4;
};

template <int SRC>
__device__ __forceinline__ void mfma_step(typename AccTile<SrcTraits<SRC>::kInt>::type& acc, const u32x4& a,
                                          const u32x4& b) {
  if constexpr (SRC == SRC_F32) {
    // lanes 0-31 hold k0..k3 of their row, lanes 32-63 k4..k7: MFMA e multiplies the pair (k_e, k_{4+e})
#pragma unroll
    for (int e = 0; e < 4; ++e)
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a[e]), __uint_as_float(b[e]), acc, 0, 0, 0);
  } else if constexpr (SRC == SRC_F16) {
    typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), acc, 0, 0, 0);
  } else if constexpr (SrcTraits<SRC>::kInt) {
    acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4, a), __builtin_bit_cast(i32x4, b), acc, 0, 0,
                                                0);
  } else {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), acc,
                                                  0, 0, 0);
  }
}

// The same product on the 16x16 shapes (v_mfma_f32_16x16x32_bf16 / _f16, v_mfma_i32_16x16x64_i8): lane l
// supplies 16 bytes of row l % 16, chunk l / 16 of the four 16-byte chunks the instruction consumes along k.
// On operands with real bit patterns the matrix cores sustain a tenth to a sixth more with this shape than
// with 32x32 (measured with loops of nothing but independent MFMAs: half the accumulator traffic per
// multiply-add, and the chip runs against its power limit).
template <int SRC>
__device__ __forceinline__ void mfma_step16(typename AccQuad<SrcTraits<SRC>::kInt>::type& acc, const u32x4& a,
                                            const u32x4& b) {
  static_assert(SRC != SRC_F32, "the fp32 class stays on 32x32x2");
  if constexpr (SRC == SRC_F16) {
    typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), acc, 0, 0, 0);
  } else if constexpr (SrcTraits<SRC>::kInt) {
    acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(i32x4, a), __builtin_bit_cast(i32x4, b), acc, 0, 0,
                                                0);
  } else {
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), acc,
                                                  0, 0, 0);
  }
}

// Which tile kernels multiply on the 16x16 shapes: the 128x128 and 64x64 tiles of every class that has them.
// Measured against the 32x32 shapes in one process on one box (launch to launch, K-contiguous operands): 128x128
// tiles 1024 x 4096 x 4096 bf16 45.6 against 49.5 us, int8 28.9 against 31.8, int8 2048 x 11008 x 4096 97.6 against
// 104.7, bf16 2048^3 26.6 against 28.4; 64x64 tiles 512 x 4096 x 4096 33.2 against 36.9 - the short shape draws less
// power per multiply-add (a loop of nothing but MFMAs sustains 2.06 against 1.75 PFLOP/s on real operands) and its
// loop below has no address arithmetic.  The rectangular tiles (256x128, 128x256: 32 quads a wavefront) take the
// short shape too: bf16 4096^3 required of them 119 against 132 us, 1536 x 11008 x 4096 164 against 182, 768 x 4096 x
// 4096 53 against 59.  The 256x256 tile's 256 accumulator registers need the accumulation half of the register file,
// where the compiler does not tie an MFMA's result to its addend and permutes the accumulators back at the loop's
// head (a hundred copies per K tile): on the compiler's loop it stays on 32x32, and takes the 16x16 shapes only under
// the written-out loop (asm_k_loop).  A tile of at most 128x128 fits two wavefronts per SIMD, where MFMAs accumulate
// in place in vector registers.
template <int SRC, int WM, int WN>
constexpr bool kShortMfma = SRC != SRC_F32 && WM * WN <= 8;

// The accumulators of one wavefront: WM x WN blocks of 32x32 elements of C, held either as one 32x32 MFMA
// result per block (M16 = false) or as its four 16x16 quadrants (M16 = true).  Both shapes are issued with the
// B fragment as first operand, so a lane holds runs of four consecutive columns of one row of C: quad q of a
// block is the four values at row(lane, q), columns col(lane, q) .. + 3 of the block.
//   32x32: register r of lane l is C[l % 32][(r / 4) * 8 + (l / 32) * 4 + r % 4], quad q = registers 4q .. 4q + 3
//   16x16: quadrant (q / 2, q % 2); register r of lane l is C[l % 16][(l / 16) * 4 + r] of the quadrant
template <bool INT, int WM, int WN, bool M16>
struct Accumulators {
  using Quad = typename AccQuad<INT>::type;
  using Frag = typename std::conditional<M16, Quad, typename AccTile<INT>::type>::type;
  static constexpr int FM = M16 ? 2 * WM : WM, FN = M16 ? 2 * WN : WN;  // fragments per wavefront tile
  Frag t[FM][FN];
  __device__ __forceinline__ void clear() {
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
      for (int j = 0; j < FN; ++j)
#pragma unroll
        for (int r = 0; r < (M16 ? 4 : 16); ++r) t[i][j][r] = 0;
  }
  // The 64 quads of the 256x256 tile's 16x16 form come out of its written-out K loop in the accumulation registers
  // and stay there until the epilogue takes them one by one: left to itself the compiler copies all 256 values into
  // vector registers ahead of the branch between the epilogue's paths, spills what does not fit, and reloaded one
  // spilled value wrongly (ROCm 7.2).  The empty statement pins a quad to its accumulation registers at its use.
  static constexpr bool kPinned = M16 && WM * WN > 8;
  template <int I, int J, int Q>
  __device__ __forceinline__ Quad quad() const {
    if constexpr (M16) {
#if defined(__HIP_DEVICE_COMPILE__)
      if constexpr (kPinned) asm volatile("" : "+a"(const_cast<Frag&>(t[2 * I + (Q >> 1)][2 * J + (Q & 1)])));
#endif
      return t[2 * I + (Q >> 1)][2 * J + (Q & 1)];
    } else {
      return __builtin_shufflevector(t[I][J], t[I][J], 4 * Q, 4 * Q + 1, 4 * Q + 2, 4 * Q + 3);
    }
  }
  static __device__ __forceinline__ int row(int lane, int q) { return M16 ? (q >> 1) * 16 + (lane & 15) : (lane & 31); }
  static __device__ __forceinline__ int col(int lane, int q) {
    return M16 ? (q & 1) * 16 + (lane >> 4) * 4 : q * 8 + (lane >> 5) * 4;
  }
  // which of the (at most two) different rows a lane has in a block quad q lies in
  static constexpr int row_slot(int q) { return M16 ? (q >> 1) : 0; }
  static constexpr int kRowSlots = M16 ? 2 : 1;
};

// The fused output transform in the order the header states.  Every step is its own fp32
// operation (the file is compiled without contraction), as vecops' transforms are separate
// vector instructions (tests/ops/MatmulConversionTestCommon.h:652-660, 735-740, 1047-1057,
// 1121-1128, 1222-1234).
__device__ __forceinline__ float apply_activation(const TileGemmParams& p, float v) {
  switch (p.ep_act) {
    // x86 max_ps(a, b) = a > b ? a : b and min_ps(a, b) = a < b ? a : b: NaN and equal zeros give b
    case ACT_RELU: return v > 0.0f ? v : 0.0f;
    case ACT_CLAMP: {
      const float t = v > p.ep_lo ? v : p.ep_lo;
      return t < p.ep_hi ? t : p.ep_hi;
    }
    case ACT_SIGMOID: return __builtin_amdgcn_rcpf(1.0f + __expf(-v));
    case ACT_SILU: return v * __builtin_amdgcn_rcpf(1.0f + __expf(-v));
    default: return v;
  }
}

__device__ __forceinline__ float finish_value(const TileGemmParams& p, float v, int batch, int row, int col) {
  if (p.ep_row_scales) v *= p.ep_row_scales[static_cast<int64_t>(batch) * p.m + row];
  if (p.ep_column_scales) v *= p.ep_column_scales[col];
  if (p.ep_flags & 1u) v *= p.ep_scale;
  if (p.ep_flags & 2u) v += p.ep_shift;
  return apply_activation(p, v);
}

// fp32 -> 8-bit integer as vecops' x86 store path does it (vec/details/x86/Conversion.h:522-528:
// a truncating convert to int32 - NaN and anything outside int32 give INT32_MIN - then a saturating
// narrow).
__device__ __forceinline__ uint32_t narrow_to_byte(float v, bool is_signed) {
  const int32_t t = (v >= -2147483648.0f && v < 2147483648.0f) ? static_cast<int32_t>(v) : INT32_MIN;
  return is_signed ? static_cast<uint32_t>(min(max(t, -128), 127)) & 0xffu : static_cast<uint32_t>(min(max(t, 0), 255));
}

// A finished fp32 value as the bits of one element of C (fp32, bf16, or an 8-bit integer).
__device__ __forceinline__ uint32_t float_output_bits(int out_kind, float v) {
  switch (out_kind) {
    case OUT_BF16: return bf16_bits_rne(v);
    case OUT_F16: return f16_bits_rne(v);
    case OUT_U8: return narrow_to_byte(v, false);
    case OUT_I8: return narrow_to_byte(v, true);
    default: return __float_as_uint(v);
  }
}

__device__ __forceinline__ int output_element_bytes(int out_kind) {
  return (out_kind == OUT_BF16 || out_kind == OUT_F16) ? 2 : (out_kind == OUT_U8 || out_kind == OUT_I8) ? 1 : 4;
}

// Final value of one output element: accumulator (+ correction) (+ Cin), then
// the optional dequantisation, then conversion to the memory dtype of C.
//   fp :  c = convert(acc + cin)
//   int:  v = acc + correction[col] + cin  (wrapping);  c = v  or
//         c = (float(v) * row_scales[row]) * column_scales[col]
//         (vecops matmul/Quantization.h:224-231: two multiplies, row first).
// Returns the 32-bit pattern of the output element (fp32 or int32), or its bf16 bits.
template <bool INT, typename AccScalar>
__device__ __forceinline__ uint32_t output_bits(const TileGemmParams& p, int batch, int row, int col, AccScalar acc) {
  if constexpr (INT) {
    uint32_t v = static_cast<uint32_t>(acc) + p.const_term;
    if (p.row_term) v += static_cast<uint32_t>(p.row_term[static_cast<int64_t>(batch) * p.m + row]);
    if (p.col_term) v += static_cast<uint32_t>(p.col_term[static_cast<int64_t>(batch) * p.n + col]);
    if (p.correction) v += static_cast<uint32_t>(p.correction[batch * p.correction_bs + col]);
    if (p.cin) v += static_cast<uint32_t>(
                 static_cast<const int32_t*>(p.cin)[batch * p.cin_bs + row * p.cin_rs + col * p.cin_cs]);
    const int32_t s = static_cast<int32_t>(v);
    float f = static_cast<float>(s);
    if (p.row_scales) {
      const float t = f * p.row_scales[batch * p.row_scales_bs + row];
      f = t * p.column_scales[col];
    } else if (p.out_kind == OUT_I32) {
      return v;
    }
    if (p.fused) f = finish_value(p, f, batch, row, col);
    return float_output_bits(p.out_kind, f);
  } else {
    float v = acc;
    if (p.cin) {
      const int64_t ci = batch * p.cin_bs + row * p.cin_rs + col * p.cin_cs;
      v += (p.cin_kind == OUT_BF16)  ? bf16_bits_to_f32(static_cast<const uint16_t*>(p.cin)[ci])
           : (p.cin_kind == OUT_F16) ? f16_bits_to_f32(static_cast<const uint16_t*>(p.cin)[ci])
                                     : static_cast<const float*>(p.cin)[ci];
    }
    if (p.fused) v = finish_value(p, v, batch, row, col);
    return float_output_bits(p.out_kind, v);
  }
}

template <bool INT, typename AccScalar>
__device__ __forceinline__ void store_output(const TileGemmParams& p, int batch, int row, int col, AccScalar acc) {
  const int64_t c_off = batch * p.c_bs + row * p.c_rs + col * p.c_cs;
  const uint32_t bits = output_bits<INT, AccScalar>(p, batch, row, col, acc);
  const int bytes = output_element_bytes(p.out_kind);
  if (bytes == 2) static_cast<uint16_t*>(p.c)[c_off] = static_cast<uint16_t>(bits);
  else if (bytes == 1) static_cast<uint8_t*>(p.c)[c_off] = static_cast<uint8_t>(bits);
  else static_cast<uint32_t*>(p.c)[c_off] = bits;
}

// Whether four consecutive elements of a row of C can leave as one store: contiguous columns and
// row / batch strides and base that keep every quad aligned to its own size.
__device__ __forceinline__ bool c_takes_quads(const TileGemmParams& p) {
  const uintptr_t quad_bytes = 4u * output_element_bytes(p.out_kind);
  return p.c_cs == 1 && (p.c_rs & 3) == 0 && (p.c_bs & 3) == 0 && (reinterpret_cast<uintptr_t>(p.c) & (quad_bytes - 1)) == 0;
}

__device__ __forceinline__ void store_quad_bits(const TileGemmParams& p, int64_t c_off, const uint32_t (&bits)[4]) {
  switch (output_element_bytes(p.out_kind)) {
    case 2:
      *reinterpret_cast<u32x2*>(static_cast<uint16_t*>(p.c) + c_off) = u32x2{bits[0] | (bits[1] << 16), bits[2] | (bits[3] << 16)};
      break;
    case 1:
      *reinterpret_cast<uint32_t*>(static_cast<uint8_t*>(p.c) + c_off) = bits[0] | (bits[1] << 8) | (bits[2] << 16) | (bits[3] << 24);
      break;
    default:
      *reinterpret_cast<u32x4*>(static_cast<uint32_t*>(p.c) + c_off) = u32x4{bits[0], bits[1], bits[2], bits[3]};
  }
}

// The staged fast path's view of the output transform: the same operations in the same order as
// output_bits, with every optional step turned into an operation that is exact when the step is absent
// (x * 1.0f and x + -0.0f return x bit for bit; relu is clamp(0, +inf)), so that the per-element code has
// no branches.  Built once per kernel from uniform parameters.
struct Finisher {
  float scale, shift, lo, hi;
  bool clamps, smooth, silu, row_scaled;
  bool int_sums, int_out;  // the staged values are int32 sums; they leave as int32
  int out_kind;
};

template <bool INT>
__device__ __forceinline__ Finisher make_finisher(const TileGemmParams& p, bool dequantised) {
  Finisher f;
  const bool on = p.fused != 0;
  f.scale = (on && (p.ep_flags & 1u)) ? p.ep_scale : 1.0f;
  f.shift = (on && (p.ep_flags & 2u)) ? p.ep_shift : -0.0f;
  f.clamps = on && (p.ep_act == ACT_RELU || p.ep_act == ACT_CLAMP);
  f.lo = p.ep_act == ACT_RELU ? 0.0f : p.ep_lo;
  f.hi = p.ep_act == ACT_RELU ? __builtin_inff() : p.ep_hi;
  f.smooth = on && (p.ep_act == ACT_SIGMOID || p.ep_act == ACT_SILU);
  f.silu = p.ep_act == ACT_SILU;
  f.row_scaled = on && p.ep_row_scales != nullptr;
  f.int_sums = INT && !dequantised;
  f.int_out = f.int_sums && p.out_kind == OUT_I32;
  f.out_kind = p.out_kind;
  return f;
}

// Four consecutive columns of one output row from their staged 32-bit values (int32 sums with the
// correction added, dequantised fp32, or fp32 sums) to the bits of C.  C-input rows are contiguous and
// need no alignment; `ecs` are the lane's four fused column scales (ones when there are none).
typedef uint32_t u32x4_align4 __attribute__((ext_vector_type(4), aligned(4)));
typedef uint32_t u32x2_align2 __attribute__((ext_vector_type(2), aligned(2)));
__device__ __forceinline__ void finish_quad(const TileGemmParams& p, const Finisher& fin, const u32x4& v, int batch,
                                            int row, int col0, int cols_left, const f32x4& ecs, uint32_t (&bits)[4]) {
  const uint32_t none = fin.int_sums ? 0u : 0x80000000u;  // adding int 0 or fp32 -0.0 changes nothing
  u32x4 cin = {none, none, none, none};                   // int32, or fp32 bits (bf16 widened)
  if (p.cin) {
    const int64_t ci = batch * p.cin_bs + static_cast<int64_t>(row) * p.cin_rs + col0;
    if (p.cin_kind == OUT_BF16 || p.cin_kind == OUT_F16) {
      const uint16_t* src = static_cast<const uint16_t*>(p.cin) + ci;
      uint32_t h[4] = {0u, 0u, 0u, 0u};  // the four 16-bit patterns
      if (cols_left >= 4) {
        const u32x2_align2 pair = *reinterpret_cast<const u32x2_align2*>(src);
        h[0] = pair.x & 0xffffu; h[1] = pair.x >> 16; h[2] = pair.y & 0xffffu; h[3] = pair.y >> 16;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (e < cols_left) h[e] = src[e];
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (e < cols_left) cin[e] = p.cin_kind == OUT_BF16 ? (h[e] << 16) : __float_as_uint(f16_bits_to_f32(h[e]));
      }
    } else {
      const uint32_t* src = static_cast<const uint32_t*>(p.cin) + ci;
      if (cols_left >= 4) {
        cin = *reinterpret_cast<const u32x4_align4*>(src);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (e < cols_left) cin[e] = src[e];
      }
    }
  }
  float f[4];
  if (fin.int_sums) {
    const u32x4 sum = v + cin;
    if (fin.int_out) {
#pragma unroll
      for (int e = 0; e < 4; ++e) bits[e] = sum[e];
      return;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) f[e] = static_cast<float>(static_cast<int32_t>(sum[e]));
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) f[e] = __uint_as_float(v[e]) + __uint_as_float(cin[e]);
  }
  const float row_scale = fin.row_scaled ? p.ep_row_scales[static_cast<int64_t>(batch) * p.m + row] : 1.0f;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    float x = ((f[e] * row_scale) * ecs[e]) * fin.scale + fin.shift;
    // x86 max_ps(a, b) = a > b ? a : b, min_ps(a, b) = a < b ? a : b
    float t = x > fin.lo ? x : fin.lo;
    t = t < fin.hi ? t : fin.hi;
    f[e] = fin.clamps ? t : x;
  }
  if (fin.smooth) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float sg = __builtin_amdgcn_rcpf(1.0f + __expf(-f[e]));
      f[e] = fin.silu ? f[e] * sg : sg;
    }
  }
  switch (fin.out_kind) {
    case OUT_BF16:
#pragma unroll
      for (int e = 0; e < 4; ++e) bits[e] = bf16_bits_rne(f[e]);
      break;
    case OUT_F16:
#pragma unroll
      for (int e = 0; e < 4; ++e) bits[e] = f16_bits_rne(f[e]);
      break;
    case OUT_U8:
#pragma unroll
      for (int e = 0; e < 4; ++e) bits[e] = narrow_to_byte(f[e], false);
      break;
    case OUT_I8:
#pragma unroll
      for (int e = 0; e < 4; ++e) bits[e] = narrow_to_byte(f[e], true);
      break;
    default:
#pragma unroll
      for (int e = 0; e < 4; ++e) bits[e] = __float_as_uint(f[e]);
  }
}

// Four consecutive columns of one output row through the full epilogue, with bounds
// checks (edge tiles, split-K partials, C-input and strided C): `raw` holds the four
// accumulators (fp32 or int32 bit patterns) of C[row][col .. col+3].  One 16-byte
// (bf16: 8-byte) store when the run lies inside C and C's rows are contiguous and
// aligned, else element by element.
template <bool INT>
__device__ __forceinline__ void store_quad_general(const TileGemmParams& p, int batch, int split, int row, int col,
                                                   const u32x4& raw, bool vec_c, bool vec_partial) {
  using AccScalar = typename std::conditional<INT, int32_t, float>::type;
  if (row >= p.m || col >= p.n) return;
  auto value = [&](int e) {
    if constexpr (INT) return static_cast<int32_t>(raw[e]);
    else return __uint_as_float(raw[e]);
  };
  if (p.split_k > 1) {
    uint32_t* part = static_cast<uint32_t*>(p.partial) +
                     ((static_cast<int64_t>(split) * p.batch + batch) * p.m + row) * p.n + col;
    if (vec_partial && col + 3 < p.n) {
      *reinterpret_cast<u32x4*>(part) = raw;
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (col + e < p.n) part[e] = raw[e];
    }
    return;
  }
  if (vec_c && col + 3 < p.n) {
    uint32_t bits[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) bits[e] = output_bits<INT, AccScalar>(p, batch, row, col + e, value(e));
    store_quad_bits(p, batch * p.c_bs + static_cast<int64_t>(row) * p.c_rs + col, bits);
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (col + e < p.n) store_output<INT, AccScalar>(p, batch, row, col + e, value(e));
  }
}

// Workgroup id -> (batch, split, tile_m, tile_n).  Workgroups are dealt to the
// eight XCDs round-robin, each XCD with its own L2: renumber so that an XCD
// receives a contiguous run of tiles, then walk tiles in bands of 8 tile rows so
// that a run shares A rows and B columns.
// `pid` of `total`: the workgroup's number within its launch (or within its group's run of a grouped launch).
__device__ __forceinline__ void map_workgroup(const TileGemmParams& p, int pid, int total, int& batch, int& split, int& tm,
                                              int& tn) {
  {
    // XCD x = pid & 7 serves the tiles [start(x), start(x + 1)): total / 8 each, one more on the first total % 8
    // (without the remainder's share, a launch of 1020 tiles ran unrenumbered: 182 us where 1032 tiles took 139)
    const int xcd = pid & 7, share = total >> 3, extra = total & 7;
    pid = xcd * share + min(xcd, extra) + (pid >> 3);
  }
  const int tiles = p.tiles_m * p.tiles_n;
  const int tile = pid % tiles;
  const int rest = pid / tiles;
  split = rest % p.split_k;
  batch = rest / p.split_k;
  constexpr int kBand = 8;
  const int band_size = kBand * p.tiles_n;
  const int band = tile / band_size;
  const int first_m = band * kBand;
  const int rows_in_band = min(p.tiles_m - first_m, kBand);
  const int in_band = tile - band * band_size;
  tm = first_m + in_band % rows_in_band;
  tn = in_band / rows_in_band;
}

// Staging of one operand tile (ROWS rows x 128 bytes) from global memory into
// LDS.  A stager owns the registers that hold a fetched tile between fetch and
// commit.  The registers form kParts groups that are stored and refilled
// independently, so the main loop can spread a tile's LDS writes (the scarce
// resource: a 16-byte LDS write costs about three times a 16-byte read) evenly
// over its k-steps and refill each group right after it has been stored.  Rows
// past the operand's extent are clamped to its last row on the fast paths: they
// are loaded but only feed accumulator rows/columns that are never stored.
//
// LOAD_KVEC / LOAD_GENERIC: thread t stages chunk (t & 7) of rows (t >> 3) + (THREADS/8)*i;
// part i is that one chunk.
template <int SRC, int LOAD, int ROWS, int THREADS>
struct Stager {
  using T = SrcTraits<SRC>;
  static constexpr int ROWS_PER_PASS = THREADS / 8;  // eight threads stage one 128-byte row
  static constexpr int CHUNKS = ROWS / ROWS_PER_PASS;
  static_assert(CHUNKS >= 1, "tile too small for this many threads");
  static constexpr int kParts = CHUNKS;
  static constexpr int kStoreOps = 1;  // schedulable operations per part: one LDS write,
  static constexpr int kLoadOps = 1;   // one refill (one or two load instructions)
  // a second register set for the start of the pipeline (fp32 held as loaded is twice the registers: no room)
  static constexpr bool kHasSpare = LOAD == LOAD_KVEC && SRC != SRC_F32_AS_BF16;
  const char* base;
  __amdgpu_buffer_rsrc_t tile_buf;  // descriptor based at the first row of the tile, k = 0 (fast path)
  uint32_t row_bytes[CHUNKS];  // byte offset of each staged row from that base, chunk included (fast path)
  int64_t rs, ks;              // element strides (checked path)
  int first_row, extent, k_end, ld_row, ld_chunk;
  uint32_t flip;  // SRC_I8_FLIP: xor mask applied on the way into LDS
  Staged<SRC> regs[CHUNKS];

  __device__ __forceinline__ void init(const void* base_, int64_t rs_, int64_t ks_, int first_row_, int extent_,
                                       int k_end_, int tid, uint32_t flip_) {
    base = static_cast<const char*>(base_);
    rs = rs_;
    ks = ks_;
    first_row = first_row_;
    extent = extent_;
    k_end = k_end_;
    flip = flip_;
    ld_chunk = tid & 7;
    ld_row = tid >> 3;
    tile_buf = tile_buffer((const VECOPS_GLOBAL char*)(base + static_cast<int64_t>(first_row) * rs * T::kSrcBytes));
#pragma unroll
    for (int i = 0; i < CHUNKS; ++i) {
      const int row = min(first_row + ld_row + i * ROWS_PER_PASS, extent - 1) - first_row;
      // the launcher admits this path only when a tile's rows plus one row's K span less than 2 GiB
      row_bytes[i] = static_cast<uint32_t>((static_cast<int64_t>(row) * rs + ld_chunk * T::kElemsPerChunk) * T::kSrcBytes);
    }
  }

  // Part PART of K tile kt, which lies wholly inside [0, K): an unconditional
  // 16-byte load on the vector path (the generic path checks every element).
  template <int PART>
  __device__ __forceinline__ void fetch_part(int kt) {
    if constexpr (LOAD == LOAD_KVEC) {
      regs[PART] = load_chunk_fast<SRC>(tile_buf, row_bytes[PART], kt * (8 * T::kElemsPerChunk * T::kSrcBytes));
    } else {
      const int k0 = kt * 8 * T::kElemsPerChunk + ld_chunk * T::kElemsPerChunk;
      const int row = first_row + ld_row + PART * ROWS_PER_PASS;
      regs[PART] = load_chunk_checked<SRC>(base, static_cast<int64_t>(row) * rs, ks, k0, k_end, row < extent, flip & 0xffu);
    }
  }

  // Whole tile kt, which lies wholly inside [0, K).
  __device__ __forceinline__ void fetch_full(int kt) {
    static_for<CHUNKS>([&](auto ci) { fetch_part<decltype(ci)::value>(kt); });
  }

  // A second register set for the start of the pipeline: the tile after the first
  // one is requested while the first is still in flight, and moved into the
  // staging registers once the first has been stored.
  struct Spare {
    Staged<SRC> regs[kHasSpare ? CHUNKS : 1];
  };
  __device__ __forceinline__ void fetch_full_spare(Spare& spare, int kt) {
    if constexpr (kHasSpare) {
#pragma unroll
      for (int i = 0; i < CHUNKS; ++i)
        spare.regs[i] = load_chunk_fast<SRC>(tile_buf, row_bytes[i], kt * (8 * T::kElemsPerChunk * T::kSrcBytes));
    }
  }
  __device__ __forceinline__ void take_spare(const Spare& spare) {
    if constexpr (kHasSpare) {
#pragma unroll
      for (int i = 0; i < CHUNKS; ++i) regs[i] = spare.regs[i];
    }
  }

  // The partial last K tile, bounds-checked, straight into its LDS tile (no registers involved).
  // (not for fp32 held as loaded: its 256x256 instances have no register to spare for the extra path)
  static constexpr bool kStagesChecked = SRC != SRC_F32_AS_BF16;
  __device__ __forceinline__ void stage_checked(int kt, char* lds_tile) const {
    stage_rows_checked<SRC>(base, rs, ks, first_row, extent, ROWS, kt * 8 * T::kElemsPerChunk, k_end, lds_tile,
                            ld_row * 8 + ld_chunk, THREADS, flip);
  }

  // Whole tile, every element bounds-checked, into the staging registers.
  __device__ __forceinline__ void fetch_checked(int kt) {
    const int k0 = kt * 8 * T::kElemsPerChunk + ld_chunk * T::kElemsPerChunk;
#pragma unroll
    for (int i = 0; i < CHUNKS; ++i) {
      const int row = first_row + ld_row + i * ROWS_PER_PASS;
      regs[i] = load_chunk_checked<SRC>(base, static_cast<int64_t>(row) * rs, ks, k0, k_end, row < extent, flip & 0xffu);
    }
  }

  template <int PART>
  __device__ __forceinline__ void commit_part(char* lds_tile) const {
    u32x4 v = regs[PART].chunk();
    if constexpr (SRC == SRC_I8_FLIP) v ^= u32x4{flip, flip, flip, flip};
    *reinterpret_cast<u32x4*>(lds_tile + lds_chunk_offset(ld_row + PART * ROWS_PER_PASS, ld_chunk)) = v;
  }

  // the main loop's view: part PART as numbered store / load operations
  template <int PART, int OP>
  __device__ __forceinline__ void store_op(char* lds_tile) const {
    commit_part<PART>(lds_tile);
  }
  template <int PART, int OP>
  __device__ __forceinline__ void load_op(int kt, uint32_t /*lds_tile*/) {
    fetch_part<PART>(kt);
  }

  __device__ __forceinline__ void commit(char* lds_tile) const {
    static_for<CHUNKS>([&](auto ci) { commit_part<decltype(ci)::value>(lds_tile); });
  }
};

// LOAD_NTR: the operand is stored with its spatial index contiguous (B handed over
// as [K,N] row-major) and goes into LDS untransposed: row k of the K tile holds the
// tile's ROWS spatial positions, kPitch bytes apart.  Thread t stages 16-byte chunk
// idx % (ROWS/8) of k row idx / (ROWS/8), idx = t + THREADS * i; part i is that one
// chunk, exactly like the K-contiguous stager.  16-bit compute elements (bf16, or
// fp32 rounded to bf16 on load).  The matching fragment read is ds_read_b64_tr_b16:
// within 16 lanes, lane s supplies the address of four consecutive n of row
// k0 + s/4 at column n0 + 4*(s%4), and lane j receives column n0 + j of rows
// k0 .. k0+3 - four consecutive k of one spatial position, half an MFMA operand.
// The pitch is 64 bytes more than a row so that the four rows of such a read fall
// into different bank groups.
template <int SRC, int ROWS, int THREADS>
struct Stager<SRC, LOAD_NTR, ROWS, THREADS> {
  using T = SrcTraits<SRC>;
  static_assert(T::kElemsPerChunk == 8, "transposing LDS reads handle 16-bit compute elements");
  static constexpr int kPitch = ROWS * 2 + 64;
  static constexpr int CHUNKS_PER_ROW = ROWS / 8;
  static constexpr int CHUNKS = 64 * CHUNKS_PER_ROW / THREADS;
  static_assert(CHUNKS >= 1 && 64 * CHUNKS_PER_ROW % THREADS == 0, "whole chunks per thread");
  static constexpr int kParts = CHUNKS;
  static constexpr int kStoreOps = 1;
  static constexpr int kLoadOps = 1;
  static constexpr bool kHasSpare = SRC != SRC_F32_AS_BF16;
  static constexpr bool kStagesChecked = false;
  __device__ __forceinline__ void stage_checked(int, char*) const {}
  const char* base;
  const VECOPS_GLOBAL char* tile_base;  // (k = 0, first n of the tile), wavefront-uniform
  static_assert(THREADS % CHUNKS_PER_ROW == 0, "every part of a thread is the same chunk, THREADS / CHUNKS_PER_ROW k rows on");
  static constexpr int K_ROWS_PER_PART = THREADS / CHUNKS_PER_ROW;
  uint32_t chunk_bytes;  // byte offset of (k row of part 0, first n of the chunk) from tile_base
  int64_t rs, ks;                // rs == 1; ks = elements between consecutive k
  int first_row, extent, k_end, tid_;
  Staged<SRC> regs[CHUNKS];
  struct Spare {
    Staged<SRC> regs[kHasSpare ? CHUNKS : 1];
  };

  __device__ __forceinline__ static int k_row(int part, int tid) { return (part * THREADS + tid) / CHUNKS_PER_ROW; }
  __device__ __forceinline__ static int chunk(int part, int tid) { return (part * THREADS + tid) % CHUNKS_PER_ROW; }

  __device__ __forceinline__ void init(const void* base_, int64_t rs_, int64_t ks_, int first_row_, int extent_,
                                       int k_end_, int tid, uint32_t /*flip*/) {
    base = static_cast<const char*>(base_);
    rs = rs_;
    ks = ks_;
    first_row = first_row_;
    extent = extent_;
    k_end = k_end_;
    tid_ = tid;
    tile_base = uniform_ptr((const VECOPS_GLOBAL char*)(base + static_cast<int64_t>(first_row) * T::kSrcBytes));
    // extent is a multiple of 8 on this path: a chunk past it is clamped onto the last one
    const int n = min(first_row + chunk(0, tid) * 8, extent - 8) - first_row;
    // the launcher admits this path only when a K tile's 64 rows span less than 2 GiB
    chunk_bytes = static_cast<uint32_t>((static_cast<int64_t>(k_row(0, tid)) * ks + n) * T::kSrcBytes);
  }
  // byte offset of part PART's k rows from part 0's (wavefront-uniform)
  __device__ __forceinline__ uint32_t part_offset(int part) const {
    return __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(part * K_ROWS_PER_PART * ks * T::kSrcBytes));
  }

  // descriptor based at row 0 of K tile kt (scalar arithmetic: every term is wavefront-uniform)
  __device__ __forceinline__ __amdgpu_buffer_rsrc_t k_tile_buffer(int kt) const {
    return tile_buffer(tile_base + static_cast<int64_t>(kt) * 64 * ks * T::kSrcBytes);
  }
  template <int PART>
  __device__ __forceinline__ void fetch_part(int kt) {
    regs[PART] = load_chunk_fast<SRC>(k_tile_buffer(kt), chunk_bytes, part_offset(PART));
  }
  __device__ __forceinline__ void fetch_full(int kt) {
    static_for<CHUNKS>([&](auto ci) { fetch_part<decltype(ci)::value>(kt); });
  }
  __device__ __forceinline__ void fetch_full_spare(Spare& spare, int kt) {
    if constexpr (kHasSpare) {
      const __amdgpu_buffer_rsrc_t k_buf = k_tile_buffer(kt);
#pragma unroll
      for (int i = 0; i < CHUNKS; ++i) spare.regs[i] = load_chunk_fast<SRC>(k_buf, chunk_bytes, part_offset(i));
    }
  }
  __device__ __forceinline__ void take_spare(const Spare& spare) {
    if constexpr (kHasSpare) {
#pragma unroll
      for (int i = 0; i < CHUNKS; ++i) regs[i] = spare.regs[i];
    }
  }

  // Whole tile with bounds checks (the partial last K tile): rows k >= K read as
  // zero, columns n >= N as zero.
  __device__ __forceinline__ void fetch_checked(int kt) {
#pragma unroll
    for (int i = 0; i < CHUNKS; ++i) {
      const int k = kt * 64 + k_row(i, tid_);
      if constexpr (SRC == SRC_BF16 || SRC == SRC_F16) {
        uint32_t w[4] = {0u, 0u, 0u, 0u};
        if (k < k_end) {
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const int n = first_row + chunk(i, tid_) * 8 + e;
            if (n < extent) w[e >> 1] |= static_cast<uint32_t>(reinterpret_cast<const uint16_t*>(base)[k * ks + n]) << ((e & 1) * 16);
          }
        }
        regs[i] = Staged<SRC>{u32x4{w[0], w[1], w[2], w[3]}};
      } else {
        uint32_t w[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int n = first_row + chunk(i, tid_) * 8 + e;
          w[e] = (k < k_end && n < extent) ? __float_as_uint(reinterpret_cast<const float*>(base)[k * ks + n]) : 0u;
        }
        regs[i] = Staged<SRC>{u32x4{w[0], w[1], w[2], w[3]}, u32x4{w[4], w[5], w[6], w[7]}};
      }
    }
  }

  template <int PART>
  __device__ __forceinline__ void commit_part(char* lds_tile) const {
    *reinterpret_cast<u32x4*>(lds_tile + k_row(PART, tid_) * kPitch + chunk(PART, tid_) * 16) = regs[PART].chunk();
  }
  __device__ __forceinline__ void commit(char* lds_tile) const {
    static_for<CHUNKS>([&](auto ci) { commit_part<decltype(ci)::value>(lds_tile); });
  }
  template <int PART, int OP>
  __device__ __forceinline__ void store_op(char* lds_tile) const {
    commit_part<PART>(lds_tile);
  }
  template <int PART, int OP>
  __device__ __forceinline__ void load_op(int kt, uint32_t /*lds_tile*/) {
    fetch_part<PART>(kt);
  }
};

// The partial last K tile of an operand stored [k][n] (bf16), bounds-checked, straight into the packed and
// swizzled LDS tile of the LOAD_NTR_DMA stager: rows k >= K and columns n >= N read as zero.
// Where chunk `chunk` (16 bytes, 8 columns) of k row `krow` lies in its row of a [k][n] tile filled by loads that
// write LDS (rows packed, cols * 2 bytes apart): the four rows a transposing read touches must lie in different
// 64-byte groups of the bank period.  A power-of-two count of chunk slots: bits 2-3 of the slot xored with the row's
// low two bits (rows 512 bytes apart would all start in one bank).  192 columns (24 slots, rows 384 bytes apart): the
// row's chunks rotated by four slots per row of the four.
__device__ __forceinline__ int ntr_dma_slot(int cols, int krow, int chunk) {
  if (cols == 192) {
    const int slot = chunk + ((krow & 3) << 2);
    return slot >= 24 ? slot - 24 : slot;
  }
  return chunk ^ ((krow & 3) << 2);
}

__device__ __noinline__ void stage_kn_checked(const void* base, int64_t ks, int first_n, int extent, int cols,
                                              int k0_tile, int k_end, char* lds_tile, int tid, int threads) {
  const int chunks_per_row = cols / 8;
#pragma unroll 2
  for (int idx = tid; idx < 64 * chunks_per_row; idx += threads) {
    const int krow = idx / chunks_per_row, chunk = idx % chunks_per_row;
    const int k = k0_tile + krow;
    uint32_t w[4] = {0u, 0u, 0u, 0u};
    if (k < k_end) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int n = first_n + chunk * 8 + e;
        if (n < extent)
          w[e >> 1] |= static_cast<uint32_t>(static_cast<const uint16_t*>(base)[k * ks + n]) << ((e & 1) * 16);
      }
    }
    *reinterpret_cast<u32x4*>(lds_tile + krow * (cols * 2) + (ntr_dma_slot(cols, krow, chunk) << 4)) = u32x4{w[0], w[1], w[2], w[3]};
  }
}

typedef __attribute__((address_space(3))) void* lds_void_ptr;

// The four words of a raw buffer descriptor over [base, base + 2 GiB): what tile_buffer() builds, as scalars.
__device__ __forceinline__ u32x4 tile_buffer_words(const VECOPS_GLOBAL char* base) {
  const uint64_t bits = reinterpret_cast<uint64_t>(base);
  return u32x4{static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<uint32_t>(bits))),
               static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<uint32_t>(bits >> 32) & 0xffffu)),
               0x7fffffffu, 0x00020000u};
}

// One buffer load of 16 bytes per lane that writes LDS itself: lane l's bytes land at tile_address + tile_offset +
// 16 * l (both wavefront-uniform numbers; the low half of a generic pointer into LDS is the LDS address).  Written
// as an instruction rather than through the compiler's builtin: the compiler orders every later LDS read it cannot
// tell apart behind such a load - it would wait for the load in front of each transposing fragment read of the
// tile being multiplied, which lies in the other stage.  The kernel orders them itself: vmcnt(0) and a barrier
// before a stage filled this way is read.  The LDS address goes into M0 by the one scalar add; handing a pointer
// over instead cost four more scalar instructions per load (a 64-bit add and the null check of the pointer
// conversion), and sixteen such sequences per K tile were 3-7 % of the kernel's time.
// (The instruction exists only in the device pass of the compiler.)
__device__ __forceinline__ void load_16_bytes_into_lds(const u32x4& descriptor, uint32_t tile_address, uint32_t tile_offset,
                                                       uint32_t lane_offset, uint32_t uniform_offset) {
#if defined(__HIP_DEVICE_COMPILE__)
  asm volatile("s_add_u32 m0, %0, %1\n\ts_nop 0\n\tbuffer_load_dwordx4 %2, %3, %4 offen lds"
               :
               : "s"(tile_address), "s"(tile_offset), "v"(lane_offset), "s"(descriptor), "s"(uniform_offset)
               : "memory", "m0", "scc");
#else
  (void)descriptor; (void)tile_address; (void)tile_offset; (void)lane_offset; (void)uniform_offset;
#endif
}

// LDS address of a generic pointer into LDS as a wavefront-uniform number: the low half of the pointer.
__device__ __forceinline__ uint32_t lds_address_of(const char* lds_pointer) {
  return __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds_pointer)));
}

// The same load through the compiler's builtin, for a kernel that has other loads in flight: the compiler
// counts it among them (it derives its vmcnt waits from the order of the loads it knows of), at the price
// described above - fit for loops without transposing reads.
__device__ __forceinline__ void load_16_bytes_into_lds_counted(__amdgpu_buffer_rsrc_t buffer, lds_void_ptr dst,
                                                               uint32_t lane_offset, uint32_t uniform_offset) {
#if defined(__HIP_DEVICE_COMPILE__)
  __builtin_amdgcn_raw_ptr_buffer_load_lds(buffer, dst, 16, lane_offset, uniform_offset, 0, 0);
#else
  (void)buffer; (void)dst; (void)lane_offset; (void)uniform_offset;
#endif
}

// LOAD_KDMA: the K-contiguous stager whose loads write LDS themselves.  A load instruction of a
// wavefront fills 1 KiB of LDS in lane order, which is eight rows of the tile; the swizzle of
// lds_chunk_offset is kept by permuting which chunk of its row a lane fetches (the eight lanes of a row
// still cover one contiguous 128 bytes of memory).  Part i is the wavefront's eight rows of pass i.
template <int SRC, int ROWS, int THREADS>
struct Stager<SRC, LOAD_KDMA, ROWS, THREADS> {
  using T = SrcTraits<SRC>;
  static_assert(SRC == SRC_BF16 || SRC == SRC_F16 || SRC == SRC_I8, "operands that go into LDS as they are");
  static constexpr int ROWS_PER_PASS = THREADS / 8;
  static constexpr int CHUNKS = ROWS / ROWS_PER_PASS;
  static_assert(CHUNKS >= 1, "tile too small for this many threads");
  static constexpr int kParts = CHUNKS;
  static constexpr int kStoreOps = 0;
  static constexpr int kLoadOps = 1;
  static constexpr bool kHasSpare = false;
  static constexpr bool kStagesChecked = true;
  struct Spare {};
  const char* base;
  u32x4 tile_buf;  // descriptor words, based at the first row of the tile, k = 0
  __amdgpu_buffer_rsrc_t tile_rsrc;  // the same descriptor for the counted form of the load
  uint32_t row_bytes[CHUNKS];
  int64_t rs, ks;
  int first_row, extent, k_end, tid_, wave_;

  __device__ __forceinline__ void init(const void* base_, int64_t rs_, int64_t ks_, int first_row_, int extent_,
                                       int k_end_, int tid, uint32_t /*flip*/) {
    base = static_cast<const char*>(base_);
    rs = rs_;
    ks = ks_;
    first_row = first_row_;
    extent = extent_;
    k_end = k_end_;
    tid_ = tid;
    wave_ = __builtin_amdgcn_readfirstlane(tid >> 6);
    tile_buf = tile_buffer_words((const VECOPS_GLOBAL char*)(base + static_cast<int64_t>(first_row) * rs * T::kSrcBytes));
    tile_rsrc = tile_buffer((const VECOPS_GLOBAL char*)(base + static_cast<int64_t>(first_row) * rs * T::kSrcBytes));
#pragma unroll
    for (int i = 0; i < CHUNKS; ++i) {
      const int tile_row = (tid >> 3) + i * ROWS_PER_PASS;
      const int chunk = ((tid & 7) ^ tile_row ^ (tile_row >> 3)) & 7;  // the chunk whose swizzled slot is tid & 7
      const int row = min(first_row + tile_row, extent - 1) - first_row;
      row_bytes[i] = static_cast<uint32_t>((static_cast<int64_t>(row) * rs + chunk * T::kElemsPerChunk) * T::kSrcBytes);
    }
  }
  // lds_tile: LDS address of the operand's tile (lds_address_of).  kt < 0: a load that fetches nothing (a buffer of
  // no records: every lane is out of range, zeros land in LDS and no memory is touched) - for the trips of a loop
  // that loads ahead of the last tile.
  __device__ __forceinline__ void dma_part(int part, int kt, uint32_t lds_tile) const {
    u32x4 buf = tile_buf;
    buf[2] = kt < 0 ? 0u : buf[2];
    load_16_bytes_into_lds(buf, lds_tile, __builtin_amdgcn_readfirstlane((part * ROWS_PER_PASS + wave_ * 8) * 128),
                           row_bytes[part], max(kt, 0) * (8 * T::kElemsPerChunk * T::kSrcBytes));
  }
  __device__ __forceinline__ void dma_full(int kt, char* lds_tile) const {
    const uint32_t address = lds_address_of(lds_tile);
    static_for<CHUNKS>([&](auto ci) { dma_part(decltype(ci)::value, kt, address); });
  }
  __device__ __forceinline__ void dma_part_counted(int part, int kt, char* lds_tile) const {
    load_16_bytes_into_lds_counted(tile_rsrc, (lds_void_ptr)(lds_tile + (part * ROWS_PER_PASS + wave_ * 8) * 128),
                                   row_bytes[part], kt * (8 * T::kElemsPerChunk * T::kSrcBytes));
  }
  __device__ __forceinline__ void stage_checked(int kt, char* lds_tile) const {
    stage_rows_checked<SRC>(base, rs, ks, first_row, extent, ROWS, kt * 8 * T::kElemsPerChunk, k_end, lds_tile, tid_,
                            THREADS, 0u);
  }
  template <int PART, int OP>
  __device__ __forceinline__ void store_op(char*) const {}
  template <int PART, int OP>
  __device__ __forceinline__ void load_op(int kt, uint32_t lds_tile) const {
    dma_part(PART, kt, lds_tile);
  }
};

// LOAD_NTR_DMA: the [k][n] stager whose loads write LDS themselves.  The 64 k rows of a tile lie
// ROWS * 2 bytes apart with no pad, so that the 64 chunks a wavefront's load instruction fills are
// contiguous; the four rows a transposing read touches are kept in different bank groups by ntr_dma_slot.
// bf16 / f16 only; tiles of 128 or more columns.  Part i is chunks i * THREADS .. of the tile's 64 * ROWS / 8, in
// LDS order: where a row's chunk count divides the thread count a thread keeps its slot and moves
// THREADS / CHUNKS_PER_ROW k rows on per part (one offset register and a uniform step); else (192 columns: 24 chunks
// a row) each part has its own row and slot.
template <int SRC, int ROWS, int THREADS>
struct Stager<SRC, LOAD_NTR_DMA, ROWS, THREADS> {
  using T = SrcTraits<SRC>;
  static_assert(SRC == SRC_BF16 || SRC == SRC_F16, "operands that go into LDS as they are");
  static constexpr int kPitch = ROWS * 2;
  static constexpr int CHUNKS_PER_ROW = ROWS / 8;
  static_assert(CHUNKS_PER_ROW >= 16, "the swizzle needs sixteen chunk slots per row");
  static constexpr int CHUNKS = 64 * CHUNKS_PER_ROW / THREADS;
  static_assert(CHUNKS >= 1 && 64 * CHUNKS_PER_ROW % THREADS == 0, "whole chunks per thread");
  static constexpr bool kRegular = THREADS % CHUNKS_PER_ROW == 0 && (THREADS / CHUNKS_PER_ROW) % 4 == 0;  // a thread keeps its row's low bits
  static_assert(kRegular || ROWS == 192, "a row's chunks divide the threads, or the 192-column tile");
  static constexpr int K_ROWS_PER_PART = THREADS / CHUNKS_PER_ROW;
  static constexpr int kParts = CHUNKS;
  static constexpr int kStoreOps = 0;
  static constexpr int kLoadOps = 1;
  static constexpr bool kHasSpare = false;
  static constexpr bool kStagesChecked = true;
  struct Spare {};
  const char* base;
  const VECOPS_GLOBAL char* tile_base;
  uint32_t chunk_bytes;                           // (regular) the part-0 chunk's byte offset from tile_base
  uint32_t part_bytes[kRegular ? 1 : CHUNKS];     // (else) every part's
  int64_t ks;
  int first_row, extent, k_end, tid_, wave_;

  // byte offset from tile_base of the chunk whose LDS place is number `place` of the tile's (k row, slot) places
  __device__ __forceinline__ uint32_t offset_of_place(int place) const {
    const int krow = place / CHUNKS_PER_ROW, slot = place % CHUNKS_PER_ROW;
    int chunk;  // the chunk whose swizzled slot this is
    if constexpr (ROWS == 192) {
      chunk = slot - ((krow & 3) << 2);
      chunk = chunk < 0 ? chunk + CHUNKS_PER_ROW : chunk;
    } else {
      chunk = slot ^ ((krow & 3) << 2);
    }
    // extent is a multiple of 8 on this path: a chunk past it is clamped onto the last one
    const int n = min(first_row + chunk * 8, extent - 8) - first_row;
    return static_cast<uint32_t>((static_cast<int64_t>(krow) * ks + n) * T::kSrcBytes);
  }
  __device__ __forceinline__ void init(const void* base_, int64_t /*rs*/, int64_t ks_, int first_row_, int extent_,
                                       int k_end_, int tid, uint32_t /*flip*/) {
    base = static_cast<const char*>(base_);
    ks = ks_;
    first_row = first_row_;
    extent = extent_;
    k_end = k_end_;
    tid_ = tid;
    wave_ = __builtin_amdgcn_readfirstlane(tid >> 6);
    tile_base = uniform_ptr((const VECOPS_GLOBAL char*)(base + static_cast<int64_t>(first_row) * T::kSrcBytes));
    chunk_bytes = offset_of_place(tid);
    if constexpr (!kRegular) {
#pragma unroll
      for (int part = 0; part < CHUNKS; ++part) part_bytes[part] = offset_of_place(part * THREADS + tid);
    } else {
      part_bytes[0] = chunk_bytes;
    }
  }
  __device__ __forceinline__ uint32_t part_offset(int part) const {
    return __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(part * K_ROWS_PER_PART * ks * T::kSrcBytes));
  }
  // (kt < 0: a load that fetches nothing, as in the K-contiguous stager)
  __device__ __forceinline__ void dma_part(int part, int kt, uint32_t lds_tile) const {
    u32x4 buf = tile_buffer_words(tile_base + static_cast<int64_t>(max(kt, 0)) * 64 * ks * T::kSrcBytes);
    buf[2] = kt < 0 ? 0u : buf[2];
    if constexpr (kRegular) {
      load_16_bytes_into_lds(buf, lds_tile, __builtin_amdgcn_readfirstlane((part * THREADS + wave_ * 64) * 16), chunk_bytes,
                             part_offset(part));
    } else {
      load_16_bytes_into_lds(buf, lds_tile, __builtin_amdgcn_readfirstlane((part * THREADS + wave_ * 64) * 16), part_bytes[part], 0u);
    }
  }
  __device__ __forceinline__ void dma_full(int kt, char* lds_tile) const {
    const uint32_t address = lds_address_of(lds_tile);
    static_for<CHUNKS>([&](auto ci) { dma_part(decltype(ci)::value, kt, address); });
  }
  __device__ __forceinline__ void stage_checked(int kt, char* lds_tile) const {
    stage_kn_checked(base, ks, first_row, extent, ROWS, kt * 64, k_end, lds_tile, tid_, THREADS);
  }
  template <int PART, int OP>
  __device__ __forceinline__ void store_op(char*) const {}
  template <int PART, int OP>
  __device__ __forceinline__ void load_op(int kt, uint32_t lds_tile) const {
    dma_part(PART, kt, lds_tile);
  }
};

// LOAD_KN32: fp32 operands multiplied in fp32, stored with the spatial index contiguous (B handed over as [K,N]
// row-major).  The K tile (32 k rows of ROWS floats) goes into LDS as it lies in memory, kPitch bytes between k rows:
// 16-byte loads along n, 16-byte LDS writes, no shuffling.  v_mfma_f32_32x32x2_f32 takes ONE float per lane and
// operand - lane l supplies column l % 32 at k = e (lanes 0-31) or 4 + e (lanes 32-63) of the k-step for instruction
// e - which is a 4-byte LDS read of 128 contiguous bytes per half wavefront; the pitch (a row plus 32 bytes) puts the
// two halves' rows, four k rows apart, into different halves of the banks.  (Transposing 4 x 4 units in registers
// on the way into a K-contiguous tile, four loads and four 16-byte LDS writes per unit with half the threads idle,
// made the 1024^3 product take 39 us where K-contiguous operands take 23.)
template <int ROWS, int THREADS>
struct Stager<SRC_F32, LOAD_KN32, ROWS, THREADS> {
  using T = SrcTraits<SRC_F32>;
  static constexpr int kPitch = ROWS * 4 + 32;
  static constexpr int CHUNKS_PER_ROW = ROWS / 4;
  static constexpr int CHUNKS = 32 * CHUNKS_PER_ROW / THREADS;
  static_assert(CHUNKS >= 1 && 32 * CHUNKS_PER_ROW % THREADS == 0, "whole chunks per thread");
  static_assert(THREADS % CHUNKS_PER_ROW == 0, "every part of a thread is the same chunk, THREADS / CHUNKS_PER_ROW k rows on");
  static constexpr int K_ROWS_PER_PART = THREADS / CHUNKS_PER_ROW;
  static constexpr int kParts = CHUNKS;
  static constexpr int kStoreOps = 1;
  static constexpr int kLoadOps = 1;
  static constexpr bool kHasSpare = false;
  static constexpr bool kStagesChecked = false;
  struct Spare {};
  __device__ __forceinline__ void stage_checked(int, char*) const {}
  const char* base;
  const VECOPS_GLOBAL char* tile_base;  // (k = 0, first n of the tile), wavefront-uniform
  uint32_t chunk_bytes;                 // byte offset of (k row of part 0, first n of the chunk) from tile_base
  int64_t ks;                           // elements between consecutive k
  int first_row, extent, k_end, tid_;
  u32x4 regs[CHUNKS];

  __device__ __forceinline__ static int k_row(int part, int tid) { return (part * THREADS + tid) / CHUNKS_PER_ROW; }
  __device__ __forceinline__ static int chunk(int part, int tid) { return (part * THREADS + tid) % CHUNKS_PER_ROW; }

  __device__ __forceinline__ void init(const void* base_, int64_t /*rs*/, int64_t ks_, int first_row_, int extent_,
                                       int k_end_, int tid, uint32_t /*flip*/) {
    base = static_cast<const char*>(base_);
    ks = ks_;
    first_row = first_row_;
    extent = extent_;
    k_end = k_end_;
    tid_ = tid;
    tile_base = uniform_ptr((const VECOPS_GLOBAL char*)(base + static_cast<int64_t>(first_row) * 4));
    // extent is a multiple of 8 on this path: a chunk past it is clamped onto the last one
    const int n = min(first_row + chunk(0, tid) * 4, extent - 4) - first_row;
    chunk_bytes = static_cast<uint32_t>((static_cast<int64_t>(k_row(0, tid)) * ks + n) * 4);
  }
  __device__ __forceinline__ uint32_t part_offset(int part) const {
    return __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(part * K_ROWS_PER_PART * ks * 4));
  }
  __device__ __forceinline__ __amdgpu_buffer_rsrc_t k_tile_buffer(int kt) const {
    return tile_buffer(tile_base + static_cast<int64_t>(kt) * 32 * ks * 4);
  }
  template <int PART>
  __device__ __forceinline__ void fetch_part(int kt) {
    regs[PART] = __builtin_amdgcn_raw_buffer_load_b128(k_tile_buffer(kt), chunk_bytes, part_offset(PART), 0);
  }
  __device__ __forceinline__ void fetch_full(int kt) {
    static_for<CHUNKS>([&](auto ci) { fetch_part<decltype(ci)::value>(kt); });
  }
  __device__ __forceinline__ void fetch_full_spare(Spare&, int) {}
  __device__ __forceinline__ void take_spare(const Spare&) {}
  // Whole tile with bounds checks (the partial last K tile): rows k >= K and columns n >= N read as zero.
  __device__ __forceinline__ void fetch_checked(int kt) {
#pragma unroll
    for (int i = 0; i < CHUNKS; ++i) {
      const int k = kt * 32 + k_row(i, tid_);
      uint32_t w[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int n = first_row + chunk(i, tid_) * 4 + e;
        w[e] = (k < k_end && n < extent) ? __float_as_uint(reinterpret_cast<const float*>(base)[k * ks + n]) : 0u;
      }
      regs[i] = u32x4{w[0], w[1], w[2], w[3]};
    }
  }
  template <int PART>
  __device__ __forceinline__ void commit_part(char* lds_tile) const {
    *reinterpret_cast<u32x4*>(lds_tile + k_row(PART, tid_) * kPitch + chunk(PART, tid_) * 16) = regs[PART];
  }
  __device__ __forceinline__ void commit(char* lds_tile) const {
    static_for<CHUNKS>([&](auto ci) { commit_part<decltype(ci)::value>(lds_tile); });
  }
  template <int PART, int OP>
  __device__ __forceinline__ void store_op(char* lds_tile) const {
    commit_part<PART>(lds_tile);
  }
  template <int PART, int OP>
  __device__ __forceinline__ void load_op(int kt, uint32_t /*lds_tile*/) {
    fetch_part<PART>(kt);
  }
};

// One schedulable staging operation: store operation `op` or load operation `op`
// of part `part` of operand A (0) or B (1); operand -1 = none.
struct StagingOp {
  int operand, part, is_load, op;
};

// Which of the four k-steps of a K tile stores (and then refills) which staging
// parts, and in what order.  A part is one LDS write and one refill; they are dealt
// out evenly, A's first.
//
// LATE (loads that write LDS, under the loop of the 16x16 shapes, whose barrier stands in the middle of the K
// tile): the loads are those of the tile after the next, into the stage the barrier has just freed, in phases
// 4 and 5 = the two quarters of the K tile behind the barrier; a load has half a K tile and more to land.
template <typename SA, typename SB, bool LATE = false>
struct StagingSchedule {
  static constexpr int PARTS_A = SA::kParts, PARTS_B = SB::kParts;
  static constexpr bool DMA = SA::kStoreOps == 0;  // loads that write LDS: all of them early, in k-steps 0 and 1
  static_assert(DMA || !LATE, "only loads that write LDS can run a tile ahead of the stores");
  static constexpr int step_a(int part) {
    if constexpr (LATE) return 4 + part * 2 / (PARTS_A + PARTS_B);
    else if constexpr (DMA) return part * 2 / (PARTS_A + PARTS_B);
    else return part * 4 / (PARTS_A + PARTS_B);
  }
  static constexpr int step_b(int part) {
    if constexpr (LATE) return 4 + (PARTS_A + part) * 2 / (PARTS_A + PARTS_B);
    else if constexpr (DMA) return (PARTS_A + part) * 2 / (PARTS_A + PARTS_B);
    else return (PARTS_A + part) * 4 / (PARTS_A + PARTS_B);
  }
  // number of operations of k-step `step`
  static constexpr int ops(int step) {
    int n = 0;
    for (int q = 0; q < PARTS_A; ++q) n += step_a(q) == step ? SA::kStoreOps + SA::kLoadOps : 0;
    for (int q = 0; q < PARTS_B; ++q) n += step_b(q) == step ? SB::kStoreOps + SB::kLoadOps : 0;
    return n;
  }
  // Operation number g of k-step `step`.  Part by part (a part's stores, then its
  // loads), or, with stores_first, every store of the step before any load: the
  // order for the k-step whose stores are followed by the barrier.
  static constexpr StagingOp op(int step, int g, bool stores_first) {
    int n = 0;
    for (int pass = 0; pass < (stores_first ? 2 : 1); ++pass) {
      for (int operand = 0; operand < 2; ++operand) {
        const int parts = operand == 0 ? PARTS_A : PARTS_B;
        const int n_st = operand == 0 ? SA::kStoreOps : SB::kStoreOps;
        const int n_ld = operand == 0 ? SA::kLoadOps : SB::kLoadOps;
        for (int q = 0; q < parts; ++q) {
          if ((operand == 0 ? step_a(q) : step_b(q)) != step) continue;
          if (!stores_first || pass == 0)
            for (int e = 0; e < n_st; ++e)
              if (n++ == g) return StagingOp{operand, q, 0, e};
          if (!stores_first || pass == 1)
            for (int r = 0; r < n_ld; ++r)
              if (n++ == g) return StagingOp{operand, q, 1, r};
        }
      }
    }
    return StagingOp{-1, 0, 0, 0};
  }
};

// Bytes of one LDS stage: the A tile (rows x 128) and the B tile, which in its
// untransposed form is 64 k rows of (columns x 2 + 64) bytes.
template <int WAVES_M, int WAVES_N, int WM, int WN, int LOAD_B>
constexpr int kStageBytes() {
  const int bm = 32 * WAVES_M * WM, bn = 32 * WAVES_N * WN;
  if (LOAD_B == LOAD_KN32) return bm * 128 + 32 * (bn * 4 + 32);  // 32 k rows of bn floats and 32 bytes
  return bm * 128 + (LOAD_B == LOAD_NTR ? 64 * (bn * 2 + 64) : bn * 128);  // LOAD_NTR_DMA: 64 rows of bn * 2 bytes
}

// Dynamic LDS one workgroup is launched with: two staging stages, or the bf16
// epilogue's row-major tiles if those are larger.
// LDS the epilogues lay accumulators out in: the bf16 path's row-major tiles, and one 32-row block of
// 32-bit values per wavefront for the general path.
template <int WAVES_M, int WAVES_N, int WM, int WN>
constexpr int kEpilogueLdsBytes() {
  const int bf16_tiles = (WN * 32 * 2 + 16) * (WM * 32) * WAVES_M * WAVES_N;
  const int general = 32 * (WN * 32 + 4) * 4 * WAVES_M * WAVES_N;
  const int columns32 = WM * 32 * 36 * 4 * WAVES_M * WAVES_N;
  const int most = bf16_tiles > general ? bf16_tiles : general;
  return most > columns32 ? most : columns32;
}

template <int WAVES_M, int WAVES_N, int WM, int WN, int LOAD_B>
constexpr int kTileLdsBytes() {
  const int stages = 2 * kStageBytes<WAVES_M, WAVES_N, WM, WN, LOAD_B>();
  const int epilogue = kEpilogueLdsBytes<WAVES_M, WAVES_N, WM, WN>();
  return stages > epilogue ? stages : epilogue;
}

// Epilogue of the tile kernels: the accumulators of one wavefront to C.
template <int SRC, int WAVES_M, int WAVES_N, int WM, int WN, int LDS_BYTES, bool M16>
__device__ __forceinline__ void store_accumulators(const TileGemmParams& p, char* lds,
                                                   const Accumulators<SrcTraits<SRC>::kInt, WM, WN, M16>& acc, int batch,
                                                   int split, int m0, int n0, int wm, int wn, int wave, int lane) {
  constexpr bool INT = SrcTraits<SRC>::kInt;
  constexpr int BM = 32 * WAVES_M * WM, BN = 32 * WAVES_N * WN;
  using ACC = Accumulators<INT, WM, WN, M16>;
  // Epilogue.  The MFMAs were issued with the B tile as first operand, so the
  // accumulators hold C transposed: a lane holds quads of four consecutive columns
  // of one row of C (Accumulators::row / col), which
  // become one 8-byte (bf16) or 16-byte (fp32 / int32) store.  Tiles that lie
  // wholly inside C, need no C-input or split-K and have 16-byte aligned rows take
  // one of three inline store loops; everything else goes through the general
  // out-of-line routine.
  const bool interior = m0 + BM <= p.m && n0 + BN <= p.n;
  const bool aligned = (p.c_rs & 3) == 0 && (p.c_bs & 3) == 0 && (reinterpret_cast<uintptr_t>(p.c) & 15) == 0;
  // the two fast paths take edge tiles too: their stores (and scale loads) are guarded per row and per run
  // of columns, which costs an interior tile a few compares
  const bool dequant = INT && p.row_scales != nullptr;
  // work that happens on the row-major side of the 32-bit staging: C-input, int32 sums leaving as floats,
  // the fused output transform, outputs narrower than 32 bits
  const bool finishing = p.cin != nullptr || p.fused != 0 || (INT ? (!dequant && p.out_kind != OUT_I32) : p.out_kind != OUT_F32);
  // (an unsigned operand's terms go through the general path, unless the launcher has folded them into the
  // per-column correction: unsigned A, one batch)
  const bool flip_terms = SRC == SRC_I8_FLIP && (p.row_term != nullptr || p.col_term != nullptr || p.const_term != 0u);
  const bool simple = aligned && p.split_k == 1 && p.c_cs == 1 && !flip_terms &&
                      (p.cin == nullptr || (p.cin_cs == 1 && !dequant));
  char* c_base = static_cast<char*>(p.c);
  if (simple && !INT && p.out_kind == OUT_BF16 && p.cin == nullptr && p.fused == 0) {
    // bf16: 8-byte pieces scattered over 32 rows would waste most of every memory
    // transaction, so each wavefront first lays its tile out row-major in LDS (the
    // staging buffers are dead by now) and then stores whole 16-byte row segments.
    constexpr int TILE_COLS = WN * 32, TILE_ROWS = WM * 32;
    constexpr int PITCH = TILE_COLS * 2 + 16;  // bytes; the pad staggers rows across banks
    static_assert(PITCH * TILE_ROWS * WAVES_M * WAVES_N <= LDS_BYTES,
                  "epilogue staging must fit the launch's LDS");
    __syncthreads();  // every wavefront is done reading fragments
    char* mine = lds + wave * (PITCH * TILE_ROWS);
    static_for<WM>([&](auto ci) {
      constexpr int i = decltype(ci)::value;
      static_for<WN>([&](auto cj) {
        constexpr int j = decltype(cj)::value;
        static_for<4>([&](auto cq) {
          constexpr int q = decltype(cq)::value;
          if constexpr (!INT) {
            const auto a4 = acc.template quad<i, j, q>();
            u32x2 v;
            v.x = cvt_pk_bf16(a4[0], a4[1]);
            v.y = cvt_pk_bf16(a4[2], a4[3]);
            *reinterpret_cast<u32x2*>(mine + (i * 32 + ACC::row(lane, q)) * PITCH + (j * 32 + ACC::col(lane, q)) * 2) = v;
          }
        });
      });
    });
    // the wavefront reads back only what it wrote itself: its own LDS traffic is ordered
    constexpr int SEGS = TILE_COLS / 8;        // 16-byte segments per row
    constexpr int TOTAL = TILE_ROWS * SEGS;    // 16-byte segments of this wavefront's tile
    static_assert(TOTAL % 64 == 0, "whole store instructions");
    uint16_t* out = reinterpret_cast<uint16_t*>(c_base) + batch * p.c_bs +
                    static_cast<int64_t>(m0 + wm * TILE_ROWS) * p.c_rs + n0 + wn * TILE_COLS;
#pragma unroll
    for (int base = 0; base < TOTAL; base += 64) {
      const int idx = base + lane, r = idx / SEGS, seg = idx % SEGS;
      const u32x4 v = *reinterpret_cast<const u32x4*>(mine + r * PITCH + seg * 16);
      // (the non-temporal hint was measured on these whole-line stores: no gain at 4096^3, and 13 % slower
      // when the output dominates, 8192 x 8192 x 64)
      uint16_t* dst = out + static_cast<int64_t>(r) * p.c_rs + seg * 8;
      const int cols_left = p.n - (n0 + wn * TILE_COLS + seg * 8);
      if (m0 + wm * TILE_ROWS + r < p.m) {
        if (cols_left >= 8) {
          *reinterpret_cast<u32x4*>(dst) = v;
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (e < cols_left) dst[e] = static_cast<uint16_t>(v[e >> 1] >> ((e & 1) * 16));
        }
      }
    }
  } else if (simple) {
    // 32-bit outputs: one 32-column block of the wavefront's tile at a time goes row-major through LDS
    // (128 rows x 128 bytes) and leaves as whole cache lines (16-byte pieces scattered over 32 rows, straight
    // from the accumulator layout, wrote 8192 x 8192 fp32 at 3.9 TB/s; whole lines at 4.9 TB/s).
    constexpr int ROWS = WM * 32, PITCH = 36;  // words
    static_assert(ROWS * PITCH * 4 * WAVES_M * WAVES_N <= LDS_BYTES, "32-bit epilogue staging must fit the launch's LDS");
    __syncthreads();  // every wavefront is done reading fragments
    uint32_t* mine = reinterpret_cast<uint32_t*>(lds) + wave * (ROWS * PITCH);
    float rs[WM][ACC::kRowSlots];
    static_for<WM>([&](auto ci) {
      static_for<ACC::kRowSlots>([&](auto ch) {
        const int row = m0 + (wm * WM + decltype(ci)::value) * 32 + ACC::row(lane, 2 * decltype(ch)::value);
        rs[decltype(ci)::value][decltype(ch)::value] =
            (dequant && row < p.m) ? p.row_scales[batch * p.row_scales_bs + row] : 1.0f;
      });
    });
    uint32_t* out = reinterpret_cast<uint32_t*>(c_base) + batch * p.c_bs + static_cast<int64_t>(m0 + wm * ROWS) * p.c_rs;
    const int out_bytes = output_element_bytes(p.out_kind);
    const Finisher fin = make_finisher<INT>(p, dequant);
    static_for<WN>([&](auto cj) {
      constexpr int j = decltype(cj)::value;
      const int col_block = n0 + (wn * WN + j) * 32;
      f32x4 cs[4];
      i32x4 corr[4];
      static_for<4>([&](auto cq) {
        constexpr int q = decltype(cq)::value;
        const int col0 = col_block + ACC::col(lane, q);
        cs[q] = f32x4{1.f, 1.f, 1.f, 1.f};
        corr[q] = i32x4{0, 0, 0, 0};
        if (col0 + 3 < p.n) {
          if (dequant) cs[q] = *reinterpret_cast<const f32x4*>(p.column_scales + col0);
          if (INT && p.correction) corr[q] = *reinterpret_cast<const i32x4*>(p.correction + batch * p.correction_bs + col0);
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if (col0 + e < p.n) {
              if (dequant) cs[q][e] = p.column_scales[col0 + e];
              if (INT && p.correction) corr[q][e] = p.correction[batch * p.correction_bs + col0 + e];
            }
          }
        }
      });
      static_for<WM>([&](auto ci) {
        constexpr int i = decltype(ci)::value;
        static_for<4>([&](auto cq) {
          constexpr int q = decltype(cq)::value;
          const auto a4 = acc.template quad<i, j, q>();
          u32x4 bits = __builtin_bit_cast(u32x4, a4);
          if constexpr (INT) {
            bits += __builtin_bit_cast(u32x4, corr[q]);
            if (dequant) {
              f32x4 o;
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                const float t = static_cast<float>(static_cast<int32_t>(bits[e])) * rs[i][ACC::row_slot(q)];  // row scale first, then
                o[e] = t * cs[q][e];                                                         // column scale
              }
              bits = __builtin_bit_cast(u32x4, o);
            }
          }
          *reinterpret_cast<u32x4*>(mine + (i * 32 + ACC::row(lane, q)) * PITCH + ACC::col(lane, q)) = bits;
        });
      });
      // the wavefront reads back only what it wrote itself: its own LDS traffic is ordered
      if (!finishing) {
#pragma unroll
        for (int base = 0; base < ROWS * 8; base += 64) {
          const int idx = base + lane, r = idx >> 3, cq = idx & 7;
          const u32x4 v = *reinterpret_cast<const u32x4*>(mine + r * PITCH + cq * 4);
          uint32_t* dst = out + static_cast<int64_t>(r) * p.c_rs + col_block + cq * 4;
          const int cols_left = p.n - (col_block + cq * 4);
          if (m0 + wm * ROWS + r < p.m) {
            if (cols_left >= 4) {
              *reinterpret_cast<u32x4*>(dst) = v;
            } else {
#pragma unroll
              for (int e = 0; e < 4; ++e)
                if (e < cols_left) dst[e] = v[e];
            }
          }
        }
      } else {
        // a lane keeps its four columns through the whole block: their fused scales are loaded once
        const int col0 = col_block + (lane & 7) * 4, cols_left = p.n - col0;
        f32x4 ecs = {1.f, 1.f, 1.f, 1.f};
        if (p.fused && p.ep_column_scales) {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (e < cols_left) ecs[e] = p.ep_column_scales[col0 + e];
        }
#pragma unroll 4
        for (int base = 0; base < ROWS * 8; base += 64) {
          const int r = (base + lane) >> 3, row = m0 + wm * ROWS + r;
          const u32x4 v = *reinterpret_cast<const u32x4*>(mine + r * PITCH + (lane & 7) * 4);
          if (row < p.m && cols_left > 0) {
            uint32_t bits[4];
            finish_quad(p, fin, v, batch, row, col0, cols_left, ecs, bits);
            const int64_t c_off = batch * p.c_bs + static_cast<int64_t>(row) * p.c_rs + col0;
            if (cols_left >= 4) {
              store_quad_bits(p, c_off, bits);
            } else {
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                if (e < cols_left) {
                  if (out_bytes == 2) reinterpret_cast<uint16_t*>(c_base)[c_off + e] = static_cast<uint16_t>(bits[e]);
                  else if (out_bytes == 1) reinterpret_cast<uint8_t*>(c_base)[c_off + e] = static_cast<uint8_t>(bits[e]);
                  else reinterpret_cast<uint32_t*>(c_base)[c_off + e] = bits[e];
                }
              }
            }
          }
        }
      }
    });
  } else if (interior && p.split_k > 1 && (p.n & 3) == 0 && (reinterpret_cast<uintptr_t>(p.partial) & 15) == 0) {
    // split-K partial sums of an interior tile: raw accumulators, 16 bytes per store
    uint32_t* partial = static_cast<uint32_t*>(p.partial) + (static_cast<int64_t>(split) * p.batch + batch) * p.m * p.n;
    static_for<WM>([&](auto ci) {
      constexpr int i = decltype(ci)::value;
      static_for<WN>([&](auto cj) {
        constexpr int j = decltype(cj)::value;
        static_for<4>([&](auto cq) {
          constexpr int q = decltype(cq)::value;
          const int row = m0 + (wm * WM + i) * 32 + ACC::row(lane, q);
          const auto v = acc.template quad<i, j, q>();
          *reinterpret_cast<typename std::remove_const<decltype(v)>::type*>(
              partial + static_cast<int64_t>(row) * p.n + n0 + (wn * WN + j) * 32 + ACC::col(lane, q)) = v;
        });
      });
    });
  } else {
    // Everything else (edge tiles, C-input, split-K partials, strided or unaligned C, unsigned-operand
    // terms): each wavefront lays one 32-row block of its accumulators out row-major in LDS and walks it
    // in a rolled loop, a lane taking four consecutive columns of one row per step - one copy of the
    // general store code, and stores that run along rows.
    constexpr int COLS = WN * 32, QUADS = COLS / 4;
    constexpr int PITCH = COLS + 4;  // 32-bit words; the pad staggers rows across banks
    static_assert(32 * PITCH * 4 * WAVES_M * WAVES_N <= LDS_BYTES, "general epilogue staging must fit the launch's LDS");
    __syncthreads();  // every wavefront is done reading fragments
    uint32_t* mine = reinterpret_cast<uint32_t*>(lds) + wave * (32 * PITCH);
    const bool vec_c = c_takes_quads(p);
    const bool vec_partial = (p.n & 3) == 0 && (reinterpret_cast<uintptr_t>(p.partial) & 15) == 0;
    static_for<WM>([&](auto ci) {
      constexpr int i = decltype(ci)::value;
      static_for<WN>([&](auto cj) {
        constexpr int j = decltype(cj)::value;
        static_for<4>([&](auto cq) {
          constexpr int q = decltype(cq)::value;
          const auto v = acc.template quad<i, j, q>();
          *reinterpret_cast<u32x4*>(mine + ACC::row(lane, q) * PITCH + j * 32 + ACC::col(lane, q)) = __builtin_bit_cast(u32x4, v);
        });
      });
      // the wavefront reads back only what it wrote itself: its own LDS traffic is ordered
      const int row_base = m0 + (wm * WM + i) * 32, col_base = n0 + wn * COLS;
#pragma unroll 1
      for (int idx = lane; idx < 32 * QUADS; idx += 64) {
        const int r = idx / QUADS, cq = idx % QUADS;
        const u32x4 raw = *reinterpret_cast<const u32x4*>(mine + r * PITCH + cq * 4);
        store_quad_general<INT>(p, batch, split, row_base + r, col_base + cq * 4, raw, vec_c, vec_partial);
      }
    });
  }
}

// The K loop of the 256x256 tile on the 16x16 matrix instructions, as one written-out instruction stream
// (tile_loop_asm.inc, generated by gen_tile_loop.py, which describes the schedule).  On entry tile 0 lies in LDS
// stage 0 and tile 1 (if any) in stage 1, and a barrier has been passed.  Operands:
//   acc               the 64 accumulator quads (accumulation registers)
//   lds_a, lds_b      per-lane LDS addresses of the fragment reads, [stage][q] (see tile_gemm_workgroup)
//   rows_a, rows_b    per-lane byte offsets of the eight loads of a K tile of A and of B (TR: B's one offset)
//   desc_a, desc_b    buffer descriptors of the operands' tiles (K tile 0)
//   m0_wave           LDS address of the wavefront's 1 KiB slice of a load's 4 KiB (stage 0, A tile)
//   k_a, k_b          byte offset of the first K tile the loop fetches (tile 2 of the walk), step_b B's per K tile
//                     (A's is 128), part_b (TR) the offset between B's eight loads of a K tile
//   nk                K tiles to multiply
#include "tile_loop_asm.inc"
// B_MODE: 0 B K-contiguous in LDS, 1 B as [k][n] (transposing reads), 2 B prepacked and kept in its pack order.
template <int SRC, int B_MODE, typename ACC>
__device__ __forceinline__ void asm_k_loop(ACC& acc, const uint32_t (&lds_a)[2][4], const uint32_t (&lds_b)[2][4],
                                           const uint32_t (&rows_a)[8], const uint32_t (&rows_b)[8], const u32x4& desc_a,
                                           const u32x4& desc_b, uint32_t m0_wave, uint32_t k_a, uint32_t k_b, uint32_t step_b,
                                           uint32_t part_b, int nk) {
#if defined(__HIP_DEVICE_COMPILE__)
  // (wavefront-uniform by construction; said again here, so that each lives in a scalar register)
  auto uniform = [](uint32_t v) { return static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(v)); };
  int left = uniform(nk) - 2, n = uniform(nk);
  k_a = uniform(k_a);
  k_b = uniform(k_b);
  const uint32_t da[4] = {uniform(desc_a[0]), uniform(desc_a[1]), uniform(desc_a[2]), uniform(desc_a[3])};
  const uint32_t db[4] = {uniform(desc_b[0]), uniform(desc_b[1]), uniform(desc_b[2]), uniform(desc_b[3])};
  m0_wave = uniform(m0_wave);
  step_b = uniform(step_b);
  part_b = uniform(part_b);
#define VECOPS_LOOP256_STATEMENT(TEXT)                                                                                  \
  asm volatile(TEXT                                                                                                     \
               : VECOPS_LOOP256_ACCUMULATORS(acc.t), [ka] "+s"(k_a), [kb] "+s"(k_b), [left] "+s"(left), [n] "+s"(n)       \
               : [la00] "v"(lds_a[0][0]), [la01] "v"(lds_a[0][1]), [la02] "v"(lds_a[0][2]), [la03] "v"(lds_a[0][3]),    \
                 [la10] "v"(lds_a[1][0]), [la11] "v"(lds_a[1][1]), [la12] "v"(lds_a[1][2]), [la13] "v"(lds_a[1][3]),    \
                 [lb00] "v"(lds_b[0][0]), [lb01] "v"(lds_b[0][1]), [lb02] "v"(lds_b[0][2]), [lb03] "v"(lds_b[0][3]),    \
                 [lb10] "v"(lds_b[1][0]), [lb11] "v"(lds_b[1][1]), [lb12] "v"(lds_b[1][2]), [lb13] "v"(lds_b[1][3]),    \
                 [ra0] "v"(rows_a[0]), [ra1] "v"(rows_a[1]), [ra2] "v"(rows_a[2]), [ra3] "v"(rows_a[3]),                \
                 [ra4] "v"(rows_a[4]), [ra5] "v"(rows_a[5]), [ra6] "v"(rows_a[6]), [ra7] "v"(rows_a[7]),                \
                 [rb0] "v"(rows_b[0]), [rb1] "v"(rows_b[1]), [rb2] "v"(rows_b[2]), [rb3] "v"(rows_b[3]),                \
                 [rb4] "v"(rows_b[4]), [rb5] "v"(rows_b[5]), [rb6] "v"(rows_b[6]), [rb7] "v"(rows_b[7]),                \
                 [da0] "s"(da[0]), [da1] "s"(da[1]), [da2] "s"(da[2]), [da3] "s"(da[3]),                                \
                 [db0] "s"(db[0]), [db1] "s"(db[1]), [db2] "s"(db[2]), [db3] "s"(db[3]),                                \
                 [m0w] "s"(m0_wave), [sb] "s"(step_b), [pb] "s"(part_b)                                                 \
               : "memory", "m0", "scc", VECOPS_LOOP256_CLOBBERS)
  if constexpr (B_MODE == 2) {
    if constexpr (SRC == SRC_F16) VECOPS_LOOP256_STATEMENT(VECOPS_LOOP256_PK("v_mfma_f32_16x16x32_f16"));
    else if constexpr (SrcTraits<SRC>::kInt) VECOPS_LOOP256_STATEMENT(VECOPS_LOOP256_PK("v_mfma_i32_16x16x64_i8"));
    else VECOPS_LOOP256_STATEMENT(VECOPS_LOOP256_PK("v_mfma_f32_16x16x32_bf16"));
  } else if constexpr (B_MODE == 1) {
    static_assert(SRC == SRC_BF16 || SRC == SRC_F16, "transposing LDS reads move 16-bit elements");
    if constexpr (SRC == SRC_F16) VECOPS_LOOP256_STATEMENT(VECOPS_LOOP256_TR("v_mfma_f32_16x16x32_f16"));
    else VECOPS_LOOP256_STATEMENT(VECOPS_LOOP256_TR("v_mfma_f32_16x16x32_bf16"));
  } else {
    if constexpr (SRC == SRC_F16) VECOPS_LOOP256_STATEMENT(VECOPS_LOOP256_K("v_mfma_f32_16x16x32_f16"));
    else if constexpr (SrcTraits<SRC>::kInt) VECOPS_LOOP256_STATEMENT(VECOPS_LOOP256_K("v_mfma_i32_16x16x64_i8"));
    else VECOPS_LOOP256_STATEMENT(VECOPS_LOOP256_K("v_mfma_f32_16x16x32_bf16"));
  }
#undef VECOPS_LOOP256_STATEMENT
#else
  (void)acc; (void)lds_a; (void)lds_b; (void)rows_a; (void)rows_b; (void)desc_a; (void)desc_b; (void)m0_wave;
  (void)k_a; (void)k_b; (void)step_b; (void)part_b; (void)nk;
#endif
}

// Bytes between the k rows of a B tile kept untransposed in LDS (0 for the other layouts).
template <int SRC, int LOAD_B, int ROWS, int THREADS>
constexpr int ntr_pitch() {
  if constexpr (load_is_ntr(LOAD_B)) return Stager<SRC, LOAD_B, ROWS, THREADS>::kPitch;
  else return 0;
}

// Workgroup shapes: WAVES_M x WAVES_N wavefronts, each owning WM x WN accumulator
// tiles of 32x32.  Every shape in use runs 4 wavefronts, one per SIMD: the 256x256
// tile with 128x128 per wavefront (256 accumulator registers in the AGPR half of
// the unified file), the small tiles with 64x64 or 32x32.
//
// The work of one workgroup: number `pid` of the `total` that serve the problem `p`.
// M16: multiply on the 16x16 MFMA shapes (the default: where kShortMfma says so).
template <int SRC, int WAVES_M, int WAVES_N, int WM, int WN, int LOAD_A, int LOAD_B, bool M16 = kShortMfma<SRC, WM, WN>>
__device__ __forceinline__ void tile_gemm_workgroup(const TileGemmParams& p, int pid, int total) {
  using T = SrcTraits<SRC>;
  constexpr bool INT = T::kInt;
  using Acc = typename AccTile<INT>::type;
  constexpr int EPC = T::kElemsPerChunk;
  constexpr int KTILE = 8 * EPC;  // elements per K tile
  constexpr int THREADS = 64 * WAVES_M * WAVES_N;
  constexpr int BM = 32 * WAVES_M * WM, BN = 32 * WAVES_N * WN;
  constexpr int STAGE_BYTES = kStageBytes<WAVES_M, WAVES_N, WM, WN, LOAD_B>();
  // The 16x16 MFMA shapes: a K tile is then two k-steps of four 16-byte chunks, and a 32-row block of a
  // wavefront's tile two fragments
  static_assert(!M16 || SRC != SRC_F32, "the fp32 MFMA has one shape here");
  constexpr int FM = M16 ? 2 * WM : WM, FN = M16 ? 2 * WN : WN;
  // The 256x256 tile on the 16x16 shapes runs its K loop as a written-out instruction stream (asm_k_loop): its 64
  // accumulator quads fill the accumulation registers, where the compiler's own loop copies them about.
  constexpr bool ASM_LOOP = M16 && WM == 4 && WN == 4;
  // (the 192x192 tile's 36 quads a wavefront: the compiler's loop copies accumulators about there too, and is still
  // a tenth ahead of the 32x32 shapes - 3072 x 3072 x 4096 bf16 66.9 us against 75.0)
  static_assert(!M16 || WM * WN <= 9 || (ASM_LOOP && load_is_dma(LOAD_A) && load_is_dma(LOAD_B) && WAVES_M == 2 && WAVES_N == 2),
                "the 16x16 shapes: tiles up to 256x128 and 192x192, or the 256x256 tile fed by loads that write LDS");

  extern __shared__ __attribute__((aligned(16))) char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;

  int batch, split, tm, tn;
  map_workgroup(p, pid, total, batch, split, tm, tn);
  // workgroup-uniform by construction; say so, or every loop bound derived from
  // them is treated as divergent
  batch = __builtin_amdgcn_readfirstlane(batch);
  if (batch >= p.batch) return;  // a grouped launch rounds each group's run of workgroups up to a multiple of eight
  split = __builtin_amdgcn_readfirstlane(split);
  tm = __builtin_amdgcn_readfirstlane(tm);
  tn = __builtin_amdgcn_readfirstlane(tn);
  const int m0 = tm * BM, n0 = tn * BN;

  const int total_k_tiles = (p.k + KTILE - 1) / KTILE;
  const int full_k_tiles = p.k / KTILE;
  const int kt_begin = split * p.k_tiles_per_split;
  const int kt_end = min(total_k_tiles, kt_begin + p.k_tiles_per_split);

  Stager<SRC, LOAD_A, BM, THREADS> stager_a;
  Stager<SRC, LOAD_B, BN, THREADS> stager_b;
  stager_a.init(static_cast<const char*>(p.a) + batch * p.a_bs * T::kSrcBytes, p.a_rs, p.a_ks, m0, p.m, p.k, tid, p.a_flip);
  stager_b.init(static_cast<const char*>(p.b) + batch * p.b_bs * T::kSrcBytes, p.b_rs, p.b_ks, n0, p.n, p.k, tid, p.b_flip);

  // a lane's row of a fragment and its 16-byte chunk within the k-step
  const int frag_row = M16 ? (lane & 15) : (lane & 31);
  // (16x16: the four 16-lane groups take the chunks in the order 0, 2, 1, 3 - which k a group multiplies is free as
  // long as A and B agree, and an LDS read serves lanes l and l + 32 together: their chunks must differ in the
  // low bit, as they do for the 32x32 shapes, or every fragment read is a two-way bank conflict)
  const int frag_chunk = M16 ? (((lane >> 4) & 1) << 1 | (lane >> 5)) : (lane >> 5);
  // 32x32: LDS offsets of this lane's fragments at k-step 0; k-step ks flips chunk bits: off ^ (ks << 5)
  int off_a[M16 ? 1 : FM], off_b[M16 ? 1 : FN];
  // 16x16: every fragment read is one of a few per-lane base addresses (per stage) plus a constant, so that a
  // read costs no vector ALU instruction - with MFMAs of 16 cycles the address arithmetic of the 32x32 loop
  // (two dependent instructions in front of every read) no longer hides behind the matrix pipe.
  //   K-contiguous tiles: fragment f, k-step ks lies at row (first + 16 f + lane % 16), chunk slot
  //   ((4 ks + chunk) ^ row ^ row / 8) & 7 = lane_slot ^ (4 ks ^ 2 f) & 7: four bases by the constant's bits 1-2
  //   B as k rows: column block j lies (j & 1) * 32 bytes into the 64-byte group ((j >> 1) ^ swizzle)
  constexpr int PITCH_NTR = ntr_pitch<SRC, LOAD_B, BN, THREADS>();
  constexpr int PITCH_KN32 = BN * 4 + 32;  // (LOAD_KN32: bytes between the k rows of the fp32 B tile)
  uint32_t base_a[2][4], base_b[2][4];
  if constexpr (M16) {
    const uint32_t lds0 = lds_address_of(lds);
    const int row_a = wm * FM * 16, row_b = wn * FN * 16;
    const int slot_a = frag_chunk ^ frag_row ^ (frag_row >> 3) ^ (row_a >> 3);
    const int slot_b = frag_chunk ^ frag_row ^ (frag_row >> 3) ^ (row_b >> 3);
#pragma unroll
    for (int st = 0; st < 2; ++st)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        base_a[st][q] = lds0 + st * STAGE_BYTES + (row_a + frag_row) * 128 + (((slot_a ^ (2 * q)) & 7) << 4);
        if constexpr (load_is_ntr(LOAD_B)) {
          // transposing read: lane s of the 16-lane group addresses row s / 4 of a block of four k rows, columns
          // 4 * (s % 4) .. + 3, and receives column s of the block's 16; the group reads chunk frag_chunk of k
          const int s16 = lane & 15;
          int col_bytes = ((wn * FN + 2 * q) * 16 + (s16 & 3) * 4) * 2;
          // packed rows: the 64-byte group is swizzled with the row's low two bits, which are s / 4 for both reads
          // of every k-step
          if constexpr (LOAD_B == LOAD_NTR_DMA) {
            if constexpr (BN == 192) {  // (ntr_dma_slot: the row's 64-byte groups rotated by one per row of the four)
              const int turned = (col_bytes & ~63) + (((s16 >> 2) & 3) << 6);
              col_bytes = (turned >= 384 ? turned - 384 : turned) | (col_bytes & 63);
            } else {
              col_bytes ^= ((s16 >> 2) & 3) << 6;
            }
          }
          base_b[st][q] = lds0 + st * STAGE_BYTES + BM * 128 + (frag_chunk * 8 + (s16 >> 2)) * PITCH_NTR + col_bytes;
        } else {
          base_b[st][q] = lds0 + st * STAGE_BYTES + BM * 128 + (row_b + frag_row) * 128 + (((slot_b ^ (2 * q)) & 7) << 4);
        }
      }
  } else {
#pragma unroll
    for (int i = 0; i < FM; ++i) off_a[i] = lds_chunk_offset((wm * FM + i) * 32 + frag_row, frag_chunk);
#pragma unroll
    for (int j = 0; j < FN; ++j) {
      if constexpr (load_is_ntr(LOAD_B)) {
        // transposing read: 16-lane group g = lane / 16 serves columns (g & 1) * 16 .. + 15 of the fragment and
        // the k half g / 2; lane s of the group addresses row s / 4, columns 4 * (s % 4) .. + 3
        const int s16 = lane & 15, g = lane >> 4;
        int col_bytes = ((wn * FN + j) * 32 + (g & 1) * 16 + (s16 & 3) * 4) * 2;
        static_assert(!(LOAD_B == LOAD_NTR_DMA && BN == 192), "the 192-column [k][n] tile: the 16x16 shapes' reads only");
        if constexpr (LOAD_B == LOAD_NTR_DMA) col_bytes ^= ((s16 >> 2) & 3) << 6;
        off_b[j] = BM * 128 + ((g >> 1) * 8 + (s16 >> 2)) * PITCH_NTR + col_bytes;
      } else if constexpr (LOAD_B == LOAD_KN32) {
        // one float per lane and matrix instruction: column lane % 32 of the block, k row e (+ 4 for the upper lanes)
        off_b[j] = BM * 128 + 4 * (lane >> 5) * PITCH_KN32 + ((wn * FN + j) * 32 + (lane & 31)) * 4;
      } else {
        off_b[j] = BM * 128 + lds_chunk_offset((wn * FN + j) * 32 + frag_row, frag_chunk);
      }
    }
  }

  // The K tiles of this workgroup are walked as a sequence seq(0..nk-1): a partial
  // last tile of K (if this split owns it) comes FIRST, so that only the prologue
  // needs bounds-checked loads and the steady-state loop issues nothing but whole
  // 16-byte loads (sums may be taken in any order).
  const int nk = __builtin_amdgcn_readfirstlane(kt_end - kt_begin);
  const int has_tail = __builtin_amdgcn_readfirstlane((nk > 0 && kt_end > full_k_tiles) ? 1 : 0);
  auto seq = [&](int j) { return (has_tail && j == 0) ? kt_end - 1 : kt_begin + j - has_tail; };

  // Software pipeline over K tiles, two LDS stages, two fragment register sets.
  // (32x32 shapes; the 16x16 shapes' two k-steps follow the same plan, see the loop.)
  // K tile `it` is multiplied in four k-steps; k-step s
  //   * reads the fragments of k-step s+1 (for s = 3: of k-step 0 of tile it+1, from
  //     the other stage, after the barrier),
  //   * stores its share of the staging registers (tile it+1) into the other stage
  //     and refills them with global loads of tile it+2,
  //   * issues the MFMAs of k-step s.
  // A k-step is written out as slots: one MFMA followed by the memory operations
  // dealt to that slot, each slot fenced against reordering, so that every memory
  // instruction issues in the shadow of an MFMA and the LDS pipe sees an even
  // stream instead of bursts (all wavefronts of a workgroup run in step).  The
  // barrier sits in the middle of k-step 3: its stores and a first half of its
  // MFMAs before, the fragment reads and the other half after.  A global load has a
  // whole K tile of MFMA work to land before its registers are stored; an LDS read
  // has most of a k-step.
  u32x4 fa[2][FM], fb[2][FN];
  constexpr int N_MFMA = FM * FN, N_READ = FM + FN;
  // fragment reads in the order the MFMAs consume them: A fragment 0, every B fragment, the other A fragments;
  // stage and k-step are compile-time constants
  typedef __attribute__((ext_vector_type(4))) short s16x4;
  typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
  typedef __attribute__((address_space(3))) u32x4 lds_u32x4;
  // (the stage is a compile-time constant under the 16x16 shapes, whose loop is written out for both stages, and a
  // run-time number otherwise)
  auto read_a = [&](auto st, auto ks_tag, auto f_tag) -> u32x4 {
    constexpr int KS = decltype(ks_tag)::value, F = decltype(f_tag)::value;
    if constexpr (M16) {
      constexpr int ST = decltype(st)::value;
      return *reinterpret_cast<const lds_u32x4*>(static_cast<uintptr_t>(base_a[ST][((4 * KS) ^ (2 * F)) >> 1 & 3] + F * 2048));
    } else {
      return *reinterpret_cast<const u32x4*>(lds + static_cast<int>(st) * STAGE_BYTES + (off_a[F] ^ (KS << 5)));
    }
  };
  auto read_b = [&](auto st, auto ks_tag, auto f_tag) -> u32x4 {
    constexpr int KS = decltype(ks_tag)::value, F = decltype(f_tag)::value;
    if constexpr (load_is_ntr(LOAD_B)) {
      // k-step KS covers rows 16 KS .. + 15 (16x16: 32 KS .. + 31) of the tile; the two reads give k 0-3 and
      // 4-7 of the lane's chunk
      if constexpr (M16) {
        constexpr int ST = decltype(st)::value;
        const uint32_t at = base_b[ST][F >> 1] + (F & 1) * 32 + KS * 32 * PITCH_NTR;
        const u32x2 lo = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<lds_s16x4*>(static_cast<uintptr_t>(at))));
        const u32x2 hi = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<lds_s16x4*>(static_cast<uintptr_t>(at + 4 * PITCH_NTR))));
        return u32x4{lo.x, lo.y, hi.x, hi.y};
      } else {
        const char* at = lds + static_cast<int>(st) * STAGE_BYTES + off_b[F] + KS * 16 * PITCH_NTR;
        const u32x2 lo = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(at)));
        const u32x2 hi = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(at + 4 * PITCH_NTR)));
        return u32x4{lo.x, lo.y, hi.x, hi.y};
      }
    } else if constexpr (LOAD_B == LOAD_KN32) {
      // k-step KS covers rows 8 KS .. + 7 of the tile: instruction e takes rows e and 4 + e
      const char* at = lds + static_cast<int>(st) * STAGE_BYTES + off_b[F] + KS * 8 * PITCH_KN32;
      return u32x4{*reinterpret_cast<const uint32_t*>(at), *reinterpret_cast<const uint32_t*>(at + PITCH_KN32),
                   *reinterpret_cast<const uint32_t*>(at + 2 * PITCH_KN32), *reinterpret_cast<const uint32_t*>(at + 3 * PITCH_KN32)};
    } else if constexpr (M16) {
      constexpr int ST = decltype(st)::value;
      return *reinterpret_cast<const lds_u32x4*>(static_cast<uintptr_t>(base_b[ST][((4 * KS) ^ (2 * F)) >> 1 & 3] + F * 2048));
    } else {
      return *reinterpret_cast<const u32x4*>(lds + static_cast<int>(st) * STAGE_BYTES + (off_b[F] ^ (KS << 5)));
    }
  };
  auto read_frag = [&](int set, auto st_tag, auto ks_tag, auto r_tag) {
    constexpr int r = decltype(r_tag)::value;
    if constexpr (r == 0) fa[set][0] = read_a(st_tag, ks_tag, std::integral_constant<int, 0>{});
    else if constexpr (r <= FN) fb[set][r - 1] = read_b(st_tag, ks_tag, std::integral_constant<int, r - 1>{});
    else fa[set][r - FN] = read_a(st_tag, ks_tag, std::integral_constant<int, r - FN>{});
  };
  auto read_frags = [&](int set, auto st_tag, auto ks_tag) {
    static_for<N_READ>([&](auto cr) { read_frag(set, st_tag, ks_tag, cr); });
  };
  // workgroup barrier that waits only for this wave's LDS traffic, not for the
  // global prefetch in flight
  auto lds_barrier = [&]() {
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0), vmcnt / expcnt untouched
    __builtin_amdgcn_s_barrier();
  };

  using SA = decltype(stager_a);
  using SB = decltype(stager_b);
  using Sched = StagingSchedule<SA, SB, M16 && load_is_dma(LOAD_A)>;

  // Start of the pipeline: tile 0 into the staging registers and, without waiting
  // for it, tile 1 into a spare set (position 1 is never the partial tile: one
  // straight path also keeps the count of loads in flight, which the waits of the
  // loop are derived from, exact); tile 0 to LDS; tile 1 into the staging registers.
  constexpr bool DMA = load_is_dma(LOAD_A);
  static_assert(load_is_dma(LOAD_A) == load_is_dma(LOAD_B), "both operands by loads into LDS, or neither");
  if constexpr (DMA) {
    // loads that write LDS: tile 0 goes straight into stage 0 (the partial tile through ordinary stores)
    if (nk > 0) {
      const int first = __builtin_amdgcn_readfirstlane(seq(0));
      if constexpr (M16) {
        // the loop of the 16x16 shapes loads two tiles ahead: the second tile (never the partial one) goes into
        // stage 1 here - ahead of a partial first tile, whose out-of-line staging waits for its own loads twice
        if (nk > 1) {
          const int second = __builtin_amdgcn_readfirstlane(kt_begin - has_tail + 1);
          stager_a.dma_full(second, lds + STAGE_BYTES);
          stager_b.dma_full(second, lds + STAGE_BYTES + BM * 128);
        }
      }
      if (first < full_k_tiles) {
        stager_a.dma_full(first, lds);
        stager_b.dma_full(first, lds + BM * 128);
      } else {
        stager_a.stage_checked(first, lds);
        stager_b.stage_checked(first, lds + BM * 128);
      }
    }
  } else if constexpr (!DMA) {
   if (nk > 0) {
    // one branch for both operands: a wait in front of the out-of-line checked
    // loader must not separate A's loads from B's
    // (scalar tile indices: a load whose uniform offset sits in a vector register is wrapped in a loop)
    const int first = __builtin_amdgcn_readfirstlane(seq(0));
    const int second = __builtin_amdgcn_readfirstlane(seq(nk > 1 ? 1 : 0));
    const bool tail_first = first >= full_k_tiles;
    if (!tail_first) {
      stager_a.fetch_full(first);
      stager_b.fetch_full(first);
    } else {
      if constexpr (SA::kStagesChecked) stager_a.stage_checked(first, lds);
      else stager_a.fetch_checked(first);
      if constexpr (SB::kStagesChecked) stager_b.stage_checked(first, lds + BM * 128);
      else stager_b.fetch_checked(first);
    }
    typename SA::Spare spare_a;
    typename SB::Spare spare_b;
    if (nk > 1) {
      if constexpr (SA::kHasSpare) stager_a.fetch_full_spare(spare_a, second);
      if constexpr (SB::kHasSpare) stager_b.fetch_full_spare(spare_b, second);
    }
    if (!(SA::kStagesChecked && tail_first)) stager_a.commit(lds);
    if (!(SB::kStagesChecked && tail_first)) stager_b.commit(lds + BM * 128);
    if (nk > 1) {
      if constexpr (SA::kHasSpare) stager_a.take_spare(spare_a);
      else stager_a.fetch_full(second);
      if constexpr (SB::kHasSpare) stager_b.take_spare(spare_b);
      else stager_b.fetch_full(second);
    }
   }
  }

  Accumulators<INT, WM, WN, M16> acc;
  acc.clear();

  if (nk > 0) {
    const int full_in_range = nk - has_tail;  // whole K tiles this workgroup owns
    // Every load of the start-up has landed before the loop is entered: the compiler's wait insertion
    // merges the start-up's branches without knowing which conditions coincide, and would otherwise
    // carry loads "still in flight" into the loop and wait for them in every iteration.
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
    lds_barrier();  // tile 0 is in LDS (and tile 1, where the loop loads two tiles ahead)
    if constexpr (ASM_LOOP) {
      // the loop fetches tile 2 of the walk first (positions 1, 2, ... of the walk are consecutive K tiles)
      const uint32_t kt2 = static_cast<uint32_t>(kt_begin - has_tail + 2);
      const uint32_t m0_wave = lds_address_of(lds) + static_cast<uint32_t>(wave) * 1024u;
      if constexpr (load_is_ntr(LOAD_B)) {
        const uint32_t step_b = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(64 * stager_b.ks * T::kSrcBytes));
        const uint32_t rows_b[8] = {stager_b.chunk_bytes, 0, 0, 0, 0, 0, 0, 0};
        asm_k_loop<SRC, 1>(acc, base_a, base_b, stager_a.row_bytes, rows_b, stager_a.tile_buf,
                              tile_buffer_words(stager_b.tile_base), m0_wave, kt2 * 128u, kt2 * step_b, step_b,
                              stager_b.part_offset(1), nk);
      } else {
        asm_k_loop<SRC, 0>(acc, base_a, base_b, stager_a.row_bytes, stager_b.row_bytes, stager_a.tile_buf,
                               stager_b.tile_buf, m0_wave, kt2 * 128u, kt2 * 128u, 128u, 0u, nk);
      }
    } else {
    read_frags(0, std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{});

    // The loop body is one straight-line block: stores into the other stage,
    // prefetches (tile index clamped to the last one) and the fragment reads of the
    // next tile are issued unconditionally; the surplus ones of the final
    // iterations touch valid memory and are never consumed.
    const uint32_t lds_address = lds_address_of(lds);
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    using I3 = std::integral_constant<int, 3>;
    auto main_loop = [&](auto prefetch_tag) {
      constexpr bool PREFETCH = decltype(prefetch_tag)::value;
      // One K tile, which lies in stage `this_stage`: an integral constant under the 16x16 shapes (the loop below is
      // written out for both stages, which makes every fragment address a register plus a constant) and it & 1
      // otherwise (written out twice, the 32x32 loop loses more to the copies the register allocator then makes
      // between its two sets of accumulator registers: int8 4096^3 86 us against 70)
      auto k_tile = [&](auto this_stage, int it) {
        const int ST = this_stage;
        auto other_stage = [&]() {
          if constexpr (std::is_integral<decltype(this_stage)>::value) return this_stage ^ 1;
          else return std::integral_constant<int, decltype(this_stage)::value ^ 1>{};
        }();
        char* other = lds + (ST ^ 1) * STAGE_BYTES;
        const uint32_t other_address = lds_address + (ST ^ 1) * STAGE_BYTES;  // what the loads that write LDS put into M0
        // K tile to prefetch: seq(min(it + 2, nk - 1)), never the tail tile (position 0)
        // (loads that write LDS fetch the next tile, into the other stage)
        // (the 16x16 loop's loads that write LDS fetch the tile after the next, behind the barrier, into this stage;
        // on the last trips of either loop there is no such tile, and loads that write LDS fetch nothing)
        constexpr int AHEAD = DMA && !M16 ? 1 : 2;
        const int t2 = (DMA && it + AHEAD >= nk)
                           ? -1
                           : __builtin_amdgcn_readfirstlane(kt_begin - has_tail + max(has_tail, min(it + AHEAD, nk - 1)));
        const uint32_t load_address = (DMA && M16) ? lds_address + ST * STAGE_BYTES : other_address;

        auto stage_op = [&](auto step_tag, auto g_tag, auto order_tag) {
          constexpr StagingOp o = Sched::op(decltype(step_tag)::value, decltype(g_tag)::value, decltype(order_tag)::value);
          // (a stager whose loads write LDS has no store operations; the others ignore the load's LDS address)
          if constexpr (o.operand == 0 && o.is_load == 0) stager_a.template store_op<o.part, o.op>(other);
          if constexpr (o.operand == 0 && o.is_load == 1 && PREFETCH) stager_a.template load_op<o.part, o.op>(t2, load_address);
          if constexpr (o.operand == 1 && o.is_load == 0) stager_b.template store_op<o.part, o.op>(other + BM * 128);
          if constexpr (o.operand == 1 && o.is_load == 1 && PREFETCH) stager_b.template load_op<o.part, o.op>(t2, load_address + BM * 128);
        };
        // Slots [S0, S1) of a k-step: MFMA x on fragment set mfma_set, then this
        // slot's share of the fragment reads RD0 .. RD0 + N_RD - 1 (k-step read_ks of
        // stage read_st into the other set; dealt front-biased) and of the staging
        // operations of phase STEP of the K tile (if STAGE).
        auto slots = [&](auto step_tag, auto s0_tag, auto s1_tag, auto rd0_tag, auto nrd_tag, auto stage_tag,
                         auto order_tag, int mfma_set, auto read_st, auto read_ks) {
          constexpr int STEP = decltype(step_tag)::value, S0 = decltype(s0_tag)::value, S1 = decltype(s1_tag)::value;
          constexpr int NS = S1 - S0, RD0 = decltype(rd0_tag)::value, N_RD = decltype(nrd_tag)::value;
          constexpr int G = decltype(stage_tag)::value ? Sched::ops(STEP) : 0;
          if constexpr (NS == 0) {
            static_for<G>([&](auto cg) { stage_op(step_tag, cg, order_tag); });
          }
          static_for<NS>([&](auto ci) {
            constexpr int i = decltype(ci)::value, x = S0 + i;
            // B rows first: see the epilogue
            if constexpr (M16) mfma_step16<SRC>(acc.t[x / FN][x % FN], fb[mfma_set][x % FN], fa[mfma_set][x / FN]);
            else mfma_step<SRC>(acc.t[x / FN][x % FN], fb[mfma_set][x % FN], fa[mfma_set][x / FN]);
            constexpr int r0 = (i * N_RD + NS - 1) / NS, r1 = ((i + 1) * N_RD + NS - 1) / NS;
            static_for<r1 - r0>([&](auto cr) {
              read_frag(mfma_set ^ 1, read_st, read_ks, std::integral_constant<int, RD0 + r0 + decltype(cr)::value>{});
            });
            constexpr int g0 = i * G / NS, g1 = (i + 1) * G / NS;
            static_for<g1 - g0>([&](auto cg) {
              stage_op(step_tag, std::integral_constant<int, g0 + decltype(cg)::value>{}, order_tag);
            });
            __builtin_amdgcn_sched_barrier(0);
          });
        };
        using All = std::integral_constant<int, N_MFMA>;
        using Half = std::integral_constant<int, N_MFMA / 2>;
        using Reads = std::integral_constant<int, N_READ>;

        if constexpr (!M16) {
          slots(I0{}, I0{}, All{}, I0{}, Reads{}, std::true_type{}, std::false_type{}, 0, this_stage, I1{});
          slots(I1{}, I0{}, All{}, I0{}, Reads{}, std::true_type{}, std::false_type{}, 1, this_stage, I2{});
          slots(I2{}, I0{}, All{}, I0{}, Reads{}, std::true_type{}, std::false_type{}, 0, this_stage, I3{});
          slots(I3{}, I0{}, Half{}, I0{}, I0{}, std::true_type{}, std::true_type{}, 1, this_stage, I0{});
          if constexpr (DMA) __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): the next tile has landed in the other stage
          lds_barrier();
          slots(I3{}, Half{}, All{}, I0{}, Reads{}, std::false_type{}, std::false_type{}, 1, other_stage, I0{});
        } else if constexpr (DMA) {
          // Two k-steps of N_MFMA short MFMAs.  Every fragment of the tile's second k-step is read during the
          // first, so the barrier stands between the two: behind it this stage is free for the loads of the tile
          // after the next, and the other stage, complete since those loads were issued half a K tile ago, gives
          // the next tile's first fragments.
          using ReadsLo = std::integral_constant<int, N_READ / 2>;
          using ReadsHi = std::integral_constant<int, N_READ - N_READ / 2>;
          using I4 = std::integral_constant<int, 4>;
          using I5 = std::integral_constant<int, 5>;
          slots(I0{}, I0{}, Half{}, I0{}, ReadsLo{}, std::false_type{}, std::false_type{}, 0, this_stage, I1{});
          slots(I1{}, Half{}, All{}, ReadsLo{}, ReadsHi{}, std::false_type{}, std::false_type{}, 0, this_stage, I1{});
          __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): the next tile has landed in the other stage
          lds_barrier();
          slots(I4{}, I0{}, Half{}, I0{}, ReadsLo{}, std::true_type{}, std::false_type{}, 1, other_stage, I0{});
          slots(I5{}, Half{}, All{}, ReadsLo{}, ReadsHi{}, std::true_type{}, std::false_type{}, 1, other_stage, I0{});
        } else {
          // Register staging under the 16x16 shapes: the four phases of the staging schedule are the halves of
          // the two k-steps, and the barrier stands behind the last phase's stores.
          using ReadsLo = std::integral_constant<int, N_READ / 2>;
          using ReadsHi = std::integral_constant<int, N_READ - N_READ / 2>;
          using Late = std::integral_constant<int, N_MFMA / 2 + N_MFMA / 4>;
          slots(I0{}, I0{}, Half{}, I0{}, ReadsLo{}, std::true_type{}, std::false_type{}, 0, this_stage, I1{});
          slots(I1{}, Half{}, All{}, ReadsLo{}, ReadsHi{}, std::true_type{}, std::false_type{}, 0, this_stage, I1{});
          slots(I2{}, I0{}, Half{}, I0{}, I0{}, std::true_type{}, std::false_type{}, 1, this_stage, I0{});
          slots(I3{}, Half{}, Late{}, I0{}, I0{}, std::true_type{}, std::true_type{}, 1, this_stage, I0{});
          lds_barrier();
          slots(I3{}, Late{}, All{}, I0{}, Reads{}, std::false_type{}, std::false_type{}, 1, other_stage, I0{});
        }
      };
      if constexpr (M16) {
        int it = 0;
        for (; it + 1 < nk; it += 2) {
          k_tile(I0{}, it);
          k_tile(I1{}, it + 1);
        }
        if (it < nk) k_tile(I0{}, it);
      } else {
        for (int it = 0; it < nk; ++it) k_tile(it & 1, it);
      }
    };
    if (full_in_range > 0) main_loop(std::true_type{});
    else main_loop(std::false_type{});
    }
    // (the last trips' surplus loads into LDS must have landed before the epilogue lays C out there)
    if constexpr (DMA && M16) __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
  }

  store_accumulators<SRC, WAVES_M, WAVES_N, WM, WN, kTileLdsBytes<WAVES_M, WAVES_N, WM, WN, LOAD_B>(), M16>(
      p, lds, acc, batch, split, m0, n0, wm, wn, wave, lane);
}

template <int SRC, int WAVES_M, int WAVES_N, int WM, int WN, int LOAD_A, int LOAD_B, bool M16 = kShortMfma<SRC, WM, WN>>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N, (M16 && WM * WN <= 4 ? 2 : 1)) void tile_gemm_kernel(const TileGemmParams p) {
  tile_gemm_workgroup<SRC, WAVES_M, WAVES_N, WM, WN, LOAD_A, LOAD_B, M16>(p, blockIdx.x, gridDim.x);
}

// Several independent problems in one launch (irregular batches: every group has its own extents, strides and
// pointers; all share the operand class, the workgroup tile and the loaders).  Workgroups first[g] .. first[g + 1] - 1
// serve group g (each run a multiple of eight long, so that a group's workgroups are dealt to the XCDs like a
// launch of its own); group_of[w] names the group of workgroup w.  No group splits K.
template <int SRC, int WAVES_M, int WAVES_N, int WM, int WN, int LOAD_A, int LOAD_B, bool M16 = kShortMfma<SRC, WM, WN>>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N, (M16 && WM * WN <= 4 ? 2 : 1)) void tile_gemm_grouped_kernel(
    const int32_t* __restrict__ group_of, const int32_t* __restrict__ first, const TileGemmParams* __restrict__ groups) {
  const int g = __builtin_amdgcn_readfirstlane(group_of[blockIdx.x]);
  const TileGemmParams p = groups[g];
  const int begin = __builtin_amdgcn_readfirstlane(first[g]);
  const int end = __builtin_amdgcn_readfirstlane(first[g + 1]);
  tile_gemm_workgroup<SRC, WAVES_M, WAVES_N, WM, WN, LOAD_A, LOAD_B, M16>(p, static_cast<int>(blockIdx.x) - begin, end - begin);
}

// Table set-up of a grouped launch is fed through kernel arguments, so that no host buffer has to outlive the
// call: one chunk carries up to kGroupChunk problem records and their first workgroups.
constexpr int kGroupChunk = 12;
struct GroupChunk {
  TileGemmParams params[kGroupChunk];
  int32_t first[kGroupChunk + 1];  // first[count] = end of the last group of this chunk
  int32_t count, offset;           // groups in this chunk, index of its first group
};
static_assert(sizeof(GroupChunk) <= 4096, "a chunk travels as kernel arguments");
static_assert(sizeof(TileGemmParams) % 8 == 0, "records are copied word by word and stored back to back");

// Sums the split-K partials and applies the same epilogue as the tile kernel.
constexpr int kReduceBatch = 8;  // partials loaded before the first is added
template <bool INT>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const TileGemmParams p) {
  using AccScalar = typename std::conditional<INT, int32_t, float>::type;
  const int64_t per_batch = static_cast<int64_t>(p.m) * p.n;
  const int64_t total = per_batch * p.batch;
  const AccScalar* part = static_cast<const AccScalar*>(p.partial);
  // four consecutive columns of a row per thread when rows hold whole quads (16-byte loads of the
  // partials, one 16-byte or 8-byte store), else element by element
  const bool quads = (p.n & 3) == 0 && (reinterpret_cast<uintptr_t>(p.partial) & 15) == 0;
  if (quads) {
    const bool vec_c = c_takes_quads(p);
    typedef AccScalar Vec4 __attribute__((ext_vector_type(4)));
    TileGemmParams q = p;  // split_k is > 1 here, or 0 (the empty sum): the sums leave through the final epilogue
    q.split_k = 1;
    for (int64_t idx = (blockIdx.x * 256ll + threadIdx.x) * 4; idx < total; idx += gridDim.x * 1024ll) {
      const int batch = static_cast<int>(idx / per_batch);
      const int64_t rem = idx - batch * per_batch;
      const int row = static_cast<int>(rem / p.n), col = static_cast<int>(rem - static_cast<int64_t>(row) * p.n);
      Vec4 sum = {0, 0, 0, 0};
      auto add = [&](const Vec4 v) {
        if constexpr (INT) sum = __builtin_bit_cast(Vec4, __builtin_bit_cast(u32x4, sum) + __builtin_bit_cast(u32x4, v));
        else sum += v;
      };
      // eight partials in flight at a time (one after the other, every load would cost a memory round trip: the
      // kernel took 0.4 us per split), added in the order of the splits
      int s = 0;
      for (; s + kReduceBatch <= p.split_k; s += kReduceBatch) {
        Vec4 v[kReduceBatch];
#pragma unroll
        for (int j = 0; j < kReduceBatch; ++j) v[j] = *reinterpret_cast<const Vec4*>(part + (s + j) * total + idx);
#pragma unroll
        for (int j = 0; j < kReduceBatch; ++j) add(v[j]);
      }
      for (; s < p.split_k; ++s) add(*reinterpret_cast<const Vec4*>(part + s * total + idx));
      store_quad_general<INT>(q, batch, 0, row, col, __builtin_bit_cast(u32x4, sum), vec_c, false);
    }
    return;
  }
  for (int64_t idx = blockIdx.x * 256ll + threadIdx.x; idx < total; idx += gridDim.x * 256ll) {
    const int batch = static_cast<int>(idx / per_batch);
    const int64_t rem = idx - batch * per_batch;
    const int row = static_cast<int>(rem / p.n), col = static_cast<int>(rem - static_cast<int64_t>(row) * p.n);
    AccScalar sum = 0;
    auto add = [&](const AccScalar v) {
      if constexpr (INT) sum = static_cast<int32_t>(static_cast<uint32_t>(sum) + static_cast<uint32_t>(v));
      else sum += v;
    };
    int s = 0;
    for (; s + kReduceBatch <= p.split_k; s += kReduceBatch) {
      AccScalar v[kReduceBatch];
#pragma unroll
      for (int j = 0; j < kReduceBatch; ++j) v[j] = part[(s + j) * total + idx];
#pragma unroll
      for (int j = 0; j < kReduceBatch; ++j) add(v[j]);
    }
    for (; s < p.split_k; ++s) add(part[s * total + idx]);
    store_output<INT, AccScalar>(p, batch, row, col, sum);
  }
}

}  // namespace vecops_hip
#endif
