// Host-side launchers of the tile GEMM kernels, one translation unit per operand
// class so the kernels compile in parallel.
#ifndef VECOPS_HIP_TILE_GEMM_LAUNCH_H
#define VECOPS_HIP_TILE_GEMM_LAUNCH_H

#include <hip/hip_runtime.h>

#include <type_traits>

#include "tile_gemm.h"

namespace vecops_hip {

// How the operand pair is fetched.
enum LoadMode : int {
  MODE_GENERIC = 0,  // element loads, any strides
  MODE_KVEC = 1,     // A and B K-contiguous and 16-byte aligned
  MODE_NVEC_B = 2,   // A K-contiguous; B stored [K,N] row-major, 16-byte aligned (16- and 32-bit compute types)
  MODE_KVEC_DMA = 3,   // MODE_KVEC with 16-byte aligned rows and bases: loads that write LDS themselves
  MODE_NVEC_B_DMA = 4  // MODE_NVEC_B likewise
};

// tile_m x tile_n: 256x256, 256x128, 128x256, 192x192, 128x128 or 64x64 (the workgroup tile).  Returns the HIP
// error of the launch (hipSuccess when enqueued).
hipError_t launch_tile_gemm_bf16(const TileGemmParams& p, int tile_m, int tile_n, int mode, hipStream_t stream);
hipError_t launch_tile_gemm_f16(const TileGemmParams& p, int tile_m, int tile_n, int mode, hipStream_t stream);
hipError_t launch_tile_gemm_f32_as_bf16(const TileGemmParams& p, int tile_m, int tile_n, int mode, hipStream_t stream);
hipError_t launch_tile_gemm_f32(const TileGemmParams& p, int tile_m, int tile_n, int mode, hipStream_t stream);  // fp32 compute
hipError_t launch_tile_gemm_i8(const TileGemmParams& p, int tile_m, int tile_n, int mode, hipStream_t stream);
// 8-bit operands of which at least one is unsigned (p.a_flip / p.b_flip and the epilogue terms set)
hipError_t launch_tile_gemm_i8_flip(const TileGemmParams& p, int tile_m, int tile_n, int mode, hipStream_t stream);
// out[b][r] = scale * sum_k int8(x[b][r][k] xor flip) (+ add[b * add_bs + r], add may be null): the epilogue terms of an
// unsigned operand
hipError_t launch_byte_row_sums(const void* x, int32_t batch, int32_t rows, int32_t k, int64_t bs, int64_t rs,
                                int64_t ks, uint32_t flip, uint32_t scale, const int32_t* add, int64_t add_bs, int32_t* out,
                                hipStream_t stream);
// q = u8(x * multipliers[batch * mult_bs + row] + zero_point) xor flip: the per-row asymmetric quantisation of fp32
// activations (flip 0x80 stores the byte as the int8 q - 128)
hipError_t launch_quantize_rows(const float* x, int32_t batch, int32_t rows, int32_t k, int64_t xbs, int64_t xrs,
                                int64_t xks, const float* multipliers, int64_t mult_bs, int32_t zero_point, uint32_t flip,
                                uint8_t* q, int64_t qbs, int64_t qrs, int64_t qks, hipStream_t stream);
// both of the above as one launch (each must have work to do): what a runtime-quantised product prepares
hipError_t launch_quantize_and_row_sums(const float* x, int32_t batch, int32_t rows, int32_t k, int64_t xbs, int64_t xrs,
                                        int64_t xks, const float* multipliers, int64_t mult_bs, int32_t zero_point, uint32_t flip,
                                        uint8_t* q, int64_t qbs, int64_t qrs, int64_t qks, const void* w, int32_t w_batch,
                                        int32_t w_rows, int64_t w_bs, int64_t w_rs, int64_t w_ks, uint32_t w_flip, uint32_t scale,
                                        const int32_t* add, int64_t add_bs, int32_t* out, hipStream_t stream);
// the 256 x 352 tile of signed 8-bit operands (tile_gemm_wide_i8.hip): p.tiles_m / p.tiles_n count its tiles; `serves`
// says whether it can run the problem (mode: the operands' LoadMode)
// (packed_b: p.b is the operand as launch_pack_b lays it out)
bool launch_tile_gemm_wide_serves(int src, const TileGemmParams& p, int mode, bool packed_b);
hipError_t launch_tile_gemm_wide(int src, const TileGemmParams& p, bool packed_b, hipStream_t stream);
hipError_t launch_splitk_reduce(const TileGemmParams& p, bool is_int, hipStream_t stream);
// B prepacked by launch_pack_b (src: SRC_BF16, SRC_F32_AS_BF16 = fp32 A against bf16-packed B, SRC_I8,
// SRC_I8_FLIP = unsigned A against int8-packed B with p.a_flip and p.col_term set);
// vector_a: 0 = any strides, 1 = A is K-contiguous, 2 = and its base, rows and batches are 16-byte aligned
hipError_t launch_tile_gemm_packed_b(int src, const TileGemmParams& p, int tile_m, int tile_n, int vector_a,
                                     hipStream_t stream);
// out[b][n] = scale * sum_k B[n,k] (+ add[n], may be null) of an int8-packed operand, for b < batch
hipError_t launch_packed_row_sums(const void* packed, int32_t n, int32_t k, int32_t batch, uint32_t scale,
                                  const int32_t* add, int32_t* out, hipStream_t stream);
struct PackBParams;
hipError_t launch_pack_b(int src, const PackBParams& p, hipStream_t stream);
// the dense operand back out of its packed form (src: SRC_BF16 for 16-bit elements, SRC_I8 for bytes)
hipError_t launch_unpack_b(int src, const PackBParams& p, hipStream_t stream);

// Shared by the per-class translation units.
template <int SRC, int WAVES_M, int WAVES_N, int WM, int WN, int LA, int LB, bool M16>
hipError_t launch_tile_instance(const TileGemmParams& p, hipStream_t stream) {
  constexpr int kLds = kTileLdsBytes<WAVES_M, WAVES_N, WM, WN, LB>();
  constexpr int kThreads = 64 * WAVES_M * WAVES_N;
  auto kernel = tile_gemm_kernel<SRC, WAVES_M, WAVES_N, WM, WN, LA, LB, M16>;
  // > 64 KiB of dynamic LDS has to be enabled once per device; cheap enough to repeat per thread.
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
  hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(grid)), dim3(kThreads), kLds, stream, p);
  return hipGetLastError();
}

// Calls f(load of A, load of B) with the loader pair of a fetch mode, as integral constants.
template <int SRC, int WAVES_M, int WAVES_N, int WM, int WN, typename F>
hipError_t with_loaders(int mode, F&& f) {
  auto pair = [&](auto la, auto lb) { return f(la, lb); };
  using std::integral_constant;
  // loads into LDS: bf16 and int8 operands on the tiles of 128 or more columns
  if constexpr ((SRC == SRC_BF16 || SRC == SRC_F16 || SRC == SRC_I8) && WAVES_N * WN * 32 >= 128) {
    if (mode == MODE_KVEC_DMA) return pair(integral_constant<int, LOAD_KDMA>{}, integral_constant<int, LOAD_KDMA>{});
    if constexpr (SRC == SRC_BF16 || SRC == SRC_F16) {
      if (mode == MODE_NVEC_B_DMA) return pair(integral_constant<int, LOAD_KDMA>{}, integral_constant<int, LOAD_NTR_DMA>{});
    }
  }
  if (mode == MODE_KVEC_DMA) mode = MODE_KVEC;
  if (mode == MODE_NVEC_B_DMA) mode = MODE_NVEC_B;
  if (mode == MODE_KVEC) return pair(integral_constant<int, LOAD_KVEC>{}, integral_constant<int, LOAD_KVEC>{});
  if constexpr (SrcTraits<SRC>::kElemsPerChunk == 8) {  // 16-bit compute: B untransposed in LDS, transposing reads
    if (mode == MODE_NVEC_B) return pair(integral_constant<int, LOAD_KVEC>{}, integral_constant<int, LOAD_NTR>{});
  } else if constexpr (SRC == SRC_F32) {                // 32-bit compute: B untransposed in LDS, one 4-byte read per operand
    if (mode == MODE_NVEC_B) return pair(integral_constant<int, LOAD_KVEC>{}, integral_constant<int, LOAD_KN32>{});
  }
  return pair(integral_constant<int, LOAD_GENERIC>{}, integral_constant<int, LOAD_GENERIC>{});
}

template <int SRC, int WAVES_M, int WAVES_N, int WM, int WN, bool M16 = kShortMfma<SRC, WM, WN>>
hipError_t launch_tile_mode(const TileGemmParams& p, int mode, hipStream_t stream) {
  return with_loaders<SRC, WAVES_M, WAVES_N, WM, WN>(mode, [&](auto la, auto lb) {
    return launch_tile_instance<SRC, WAVES_M, WAVES_N, WM, WN, decltype(la)::value, decltype(lb)::value, M16>(p, stream);
  });
}

// 128 x 128 tiles of 16-bit operands with at most four K tiles multiply on the 32x32 shape after all: to fp32
// outputs the 16x16 instance's workgroups live about 1 us longer there (3072 x 3072 x 64 15.0 us against 12.8,
// x 256 19.1 against 17.1, 8192 x 8192 x 128 73 against 62; 5 % at K = 512, level at 1024, and from there on the
// 16x16 shape is ahead), and to bf16 outputs the two are level up to K = 256 (from K = 512 the 16x16 shape is
// ahead, as it is at every K for int32 outputs).  The rule does not look at the output type: a product's bf16
// output stays the rounded fp32 output of the same call sequence.
template <int SRC>
bool long_shape_pays(const TileGemmParams& p) {
  return !SrcTraits<SRC>::kInt && p.split_k == 1 && p.k_tiles_per_split <= 4;
}

template <int SRC>
hipError_t launch_tile_class(const TileGemmParams& p, int tile_m, int tile_n, int mode, hipStream_t stream) {
  // Every shape runs 4 wavefronts (2 x 2), one per SIMD.  256x256: 128x128 per wavefront - a third less LDS
  // read traffic than 8 wavefronts of 128x64, which matters because the LDS pipe, not the MFMA pipe, is
  // what the 8-wavefront shape saturates.
  if (tile_m == 256 && tile_n == 256) {
    // operands whose loads write LDS themselves: the 16x16 shapes under the written-out K loop (asm_k_loop), whose
    // scalar K offsets are 32-bit
    if constexpr (SRC == SRC_BF16 || SRC == SRC_F16 || SRC == SRC_I8) {
      if (mode == MODE_KVEC_DMA) return launch_tile_instance<SRC, 2, 2, 4, 4, LOAD_KDMA, LOAD_KDMA, true>(p, stream);
      if constexpr (SRC != SRC_I8) {
        if (mode == MODE_NVEC_B_DMA && static_cast<int64_t>(p.k) * p.b_ks * 2 < (1ll << 31))
          return launch_tile_instance<SRC, 2, 2, 4, 4, LOAD_KDMA, LOAD_NTR_DMA, true>(p, stream);
      }
    }
    return launch_tile_mode<SRC, 2, 2, 4, 4>(p, mode, stream);
  }
  if (tile_m == 192 && tile_n == 192) {
    // 96 x 96 a wavefront on the 16x16 shapes: only for operands whose loads write LDS themselves (what the rule table
    // plans it for, and what a request for it is checked against)
    if constexpr (SRC == SRC_BF16 || SRC == SRC_F16 || SRC == SRC_I8) {
      if (mode == MODE_KVEC_DMA) return launch_tile_instance<SRC, 2, 2, 3, 3, LOAD_KDMA, LOAD_KDMA, true>(p, stream);
      if constexpr (SRC != SRC_I8) {
        if (mode == MODE_NVEC_B_DMA) return launch_tile_instance<SRC, 2, 2, 3, 3, LOAD_KDMA, LOAD_NTR_DMA, true>(p, stream);
      }
    }
    return hipErrorInvalidConfiguration;
  }
  if (tile_m == 256 && tile_n == 128) return launch_tile_mode<SRC, 2, 2, 4, 2>(p, mode, stream);
  if (tile_m == 128 && tile_n == 256) return launch_tile_mode<SRC, 2, 2, 2, 4>(p, mode, stream);
  if (tile_m == 128 && tile_n == 128) {
    if constexpr (kShortMfma<SRC, 2, 2> && !SrcTraits<SRC>::kInt) {
      if (long_shape_pays<SRC>(p)) return launch_tile_mode<SRC, 2, 2, 2, 2, false>(p, mode, stream);
    }
    return launch_tile_mode<SRC, 2, 2, 2, 2>(p, mode, stream);
  }
  return launch_tile_mode<SRC, 2, 2, 1, 1>(p, mode, stream);
}

// A grouped launch: the device tables written by launch_group_tables, `workgroups` = first[groups].
struct GroupedTables {
  const int32_t* group_of;
  const int32_t* first;
  const TileGemmParams* groups;
  int32_t workgroups;
};

template <int SRC, int WAVES_M, int WAVES_N, int WM, int WN, int LA, int LB, bool M16 = kShortMfma<SRC, WM, WN>>
hipError_t launch_grouped_instance(const GroupedTables& t, hipStream_t stream) {
  constexpr int kLds = kTileLdsBytes<WAVES_M, WAVES_N, WM, WN, LB>();
  constexpr int kThreads = 64 * WAVES_M * WAVES_N;
  auto kernel = tile_gemm_grouped_kernel<SRC, WAVES_M, WAVES_N, WM, WN, LA, LB, M16>;
  static thread_local int configured_device = -1;
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return e;
  if (configured_device != device) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
    if (e != hipSuccess) return e;
    configured_device = device;
  }
  if (t.workgroups <= 0) return hipErrorInvalidConfiguration;
  hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(t.workgroups)), dim3(kThreads), kLds, stream, t.group_of, t.first,
                     t.groups);
  return hipGetLastError();
}

// Square tiles of 256, 128 or 64.
template <int SRC>
hipError_t launch_grouped_class(const GroupedTables& t, int tile, int mode, hipStream_t stream) {
  auto go = [&](auto wm_tag) {
    constexpr int W = decltype(wm_tag)::value;
    return with_loaders<SRC, 2, 2, W, W>(mode, [&](auto la, auto lb) {
      return launch_grouped_instance<SRC, 2, 2, W, W, decltype(la)::value, decltype(lb)::value>(t, stream);
    });
  };
  if (tile == 256) {
    // as a single product's 256 x 256 tiles: the written-out K loop where the loads write LDS themselves (the table's
    // mode is that of its weakest group, and none of them then needs more than 32-bit K offsets)
    if constexpr (SRC == SRC_BF16 || SRC == SRC_F16 || SRC == SRC_I8) {
      if (mode == MODE_KVEC_DMA) return launch_grouped_instance<SRC, 2, 2, 4, 4, LOAD_KDMA, LOAD_KDMA, true>(t, stream);
      if constexpr (SRC != SRC_I8) {
        if (mode == MODE_NVEC_B_DMA) return launch_grouped_instance<SRC, 2, 2, 4, 4, LOAD_KDMA, LOAD_NTR_DMA, true>(t, stream);
      }
    }
    return go(std::integral_constant<int, 4>{});
  }
  if (tile == 128) return go(std::integral_constant<int, 2>{});
  return go(std::integral_constant<int, 1>{});
}
// The 256 x 256 tile on a prepacked B with the written-out K loop (tile_gemm_packed16.hip): whether it serves a
// launch that the plan gave these tile extents, and the launch.
bool launch_tile_gemm_packed16_serves(int src, const TileGemmParams& p, int tile_m, int tile_n);
hipError_t launch_tile_gemm_packed16(int src, const TileGemmParams& p, hipStream_t stream);
// The 128 x 128 tile on four LDS stages for launches of at most one workgroup per compute unit (tile_gemm_deep128.hip).
// packed_b: p.b is vecops_hip_pack_b's layout (mode is then not consulted).
bool launch_tile_gemm_deep128_serves(int src, const TileGemmParams& p, int mode, bool packed_b);
hipError_t launch_tile_gemm_deep128(int src, const TileGemmParams& p, int mode, bool packed_b, hipStream_t stream);
// fp32 compute on 64 x 64 (tile = 64) or 128 x 128 tiles with a ring of LDS stages, for launches of at most one workgroup
// per compute unit (tile_gemm_deep_f32.hip); b_as_kn: B handed over as [K,N].
bool launch_tile_gemm_deep_f32_serves(const TileGemmParams& p, int tile, bool b_as_kn);
hipError_t launch_tile_gemm_deep_f32(const TileGemmParams& p, int tile, bool b_as_kn, hipStream_t stream);
// Very short K on 16-bit compute, operands K-contiguous: fragments loaded straight from memory, 64 x 128 of C a workgroup
// (tile_gemm_short_k.hip).
bool launch_tile_gemm_short_k_serves(int src, const TileGemmParams& p);
hipError_t launch_tile_gemm_short_k(int src, TileGemmParams p, hipStream_t stream);
hipError_t launch_tile_gemm_grouped_bf16(const GroupedTables& t, int tile, int mode, hipStream_t stream);
hipError_t launch_tile_gemm_grouped_i8(const GroupedTables& t, int tile, int mode, hipStream_t stream);
hipError_t launch_tile_gemm_grouped_i8_flip(const GroupedTables& t, int tile, int mode, hipStream_t stream);
hipError_t launch_tile_gemm_grouped_f16(const GroupedTables& t, int tile, int mode, hipStream_t stream);
hipError_t launch_tile_gemm_grouped_f32_as_bf16(const GroupedTables& t, int tile, int mode, hipStream_t stream);
hipError_t launch_tile_gemm_grouped_f32(const GroupedTables& t, int tile, int mode, hipStream_t stream);

}  // namespace vecops_hip
#endif
