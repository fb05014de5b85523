// TEST INFRASTRUCTURE ONLY.  A caller of the real vecops CPU matmul
// (ops::matmul, include/vecops/ops/Matmul.h:530-586) exposed through a C ABI so
// the Python tests can hold the oracle restatement and the gfx950 kernels
// against the reference itself.  It is compiled by oracle/Makefile from the
// vecops sources where they lie (never copied) into oracle/_ref/, and needs an
// x86 host with AMX (the only x86 matmul backend,
// include/vecops/matmul/details/kernel/Backend.h:57-72).
//
// Every tensor is passed with fully dynamic extents and strides (meta::Any), the
// most general form the reference accepts (tests/ops/MatmulTest.cpp:220-279).
#include <cpuid.h>
#include <sys/syscall.h>
#include <unistd.h>

#include <cstdint>
#include <vector>

#include "vecops/matmul/Quantization.h"
#include "vecops/ops/Matmul.h"

using namespace vecops;
using namespace vecops::meta;
using namespace vecops::tensor;

namespace {

bool g_amx_ready = false;

// tests/ops/MatmulTestArch.h:22-27: AMX tile data must be requested from the
// kernel before the first tile instruction.
bool enable_amx() {
  if (g_amx_ready) return true;
  unsigned eax = 0, ebx = 0, ecx = 0, edx = 0;
  if (!__get_cpuid_count(7, 0, &eax, &ebx, &ecx, &edx)) return false;
  const bool amx_bf16 = (edx >> 22) & 1, amx_tile = (edx >> 24) & 1, amx_int8 = (edx >> 25) & 1;
  const bool avx512f = (ebx >> 16) & 1;
  if (!(amx_bf16 && amx_tile && amx_int8 && avx512f)) return false;
  if (syscall(SYS_arch_prctl, 0x1023, 18) != 0) return false;
  g_amx_ready = true;
  return true;
}

template <typename T>
auto view2(T* p, int64_t rows, int64_t cols, int64_t s0, int64_t s1) {
  return make_tensor(p, make_layout(make_shape(Any{rows}, Any{cols}), make_strides(Any{s0}, Any{s1})));
}

template <typename T>
auto view3(T* p, int64_t batch, int64_t rows, int64_t cols, int64_t sb, int64_t s0, int64_t s1) {
  return make_tensor(
    p, make_layout(make_shape(Any{batch}, Any{rows}, Any{cols}), make_strides(Any{sb}, Any{s0}, Any{s1})));
}

template <typename Atom, typename TA, typename TB, typename TC>
int run2(const TA* a, const TB* b, TC* c, const TC* cin, int64_t m, int64_t n, int64_t k, const int64_t* sa,
         const int64_t* sb, const int64_t* sc) {
  if (!enable_amx()) return -1;
  auto at = view2(const_cast<TA*>(a), m, k, sa[0], sa[1]);
  auto bt = view2(const_cast<TB*>(b), n, k, sb[0], sb[1]);
  auto ct = view2(c, m, n, sc[0], sc[1]);
  auto op = ops::matmul(ops::MatmulConfig<Atom>{});
  if (cin) {
    auto cit = view2(const_cast<TC*>(cin), m, n, sc[0], sc[1]);
    const nint_t bytes = op.required_workspace(Any{m}, Any{n}, Any{k}, at, bt, cit, ct);
    kernel::Workspace ws(bytes);
    auto v = ws.view();
    op(v, Any{m}, Any{n}, Any{k}, at, bt, cit, ct);
  } else {
    const nint_t bytes = op.required_workspace(Any{m}, Any{n}, Any{k}, at, bt, ct);
    kernel::Workspace ws(bytes);
    auto v = ws.view();
    op(v, Any{m}, Any{n}, Any{k}, at, bt, ct);
  }
  return 0;
}

template <typename Atom, typename TA, typename TB, typename TC>
int run3(const TA* a, const TB* b, TC* c, int64_t batch, int64_t m, int64_t n, int64_t k, const int64_t* sa,
         const int64_t* sb, const int64_t* sc) {
  if (!enable_amx()) return -1;
  auto at = view3(const_cast<TA*>(a), batch, m, k, sa[0], sa[1], sa[2]);
  auto bt = view3(const_cast<TB*>(b), batch, n, k, sb[0], sb[1], sb[2]);
  auto ct = view3(c, batch, m, n, sc[0], sc[1], sc[2]);
  auto op = ops::matmul(ops::MatmulConfig<Atom>{});
  const nint_t bytes = op.required_workspace(Any{m}, Any{n}, Any{k}, at, bt, ct);
  kernel::Workspace ws(bytes);
  auto v = ws.view();
  op(v, Any{m}, Any{n}, Any{k}, at, bt, ct);
  return 0;
}

// Fused output transforms, built the way the reference's own tests build them
// (tests/ops/MatmulConversionTestCommon.h: per-column scale :652-660, clamp :735-740,
// relu :1047-1050, sigmoid :1051-1057, silu :1121-1128, requantisation :1222-1234):
//   v = A.B^T + bias[col]                (bias = stride-0 C-input row, may be null)
//   v = float(v)                         (int32 accumulators only)
//   v = v * scale                        (flags & 1)
//   v = v * column_scales[col]           (column_scales != null; readable 64 floats past n)
//   v = v + shift                        (flags & 2)
//   v = act(v)                           0 none, 1 relu, 2 clamp(lo, hi), 3 sigmoid, 4 silu
//   c = convert<memory dtype of C>(v)
struct FusedSpec {
  int32_t activation;
  uint32_t flags;
  float scale, shift, lo, hi;
  const float* column_scales;
};

template <typename Domain>
auto fused_transform(const FusedSpec* spec) {
  return tensor::make_lane_local_vec_transform<Domain, Domain>(
    [spec](auto tag, auto value, const auto& context) VECOPS_KERNEL_LAMBDA {
      const auto coordinate = context.lane_coord(0);
      const nint_t column = coordinate[coordinate.size() - 1];
      auto v = value;
      if (spec->flags & 1u) v = vec::mul(tag, v, vec::fill(tag, Domain{spec->scale}));
      if (spec->column_scales) v = vec::mul(tag, v, vec::load(tag, spec->column_scales + column));
      if (spec->flags & 2u) v = vec::add(tag, v, vec::fill(tag, Domain{spec->shift}));
      const auto one = vec::fill(tag, Domain{1});
      switch (spec->activation) {
        case 1: v = vec::max(tag, v, vec::zeros(tag)); break;
        case 2: v = vec::min(tag, vec::max(tag, v, vec::fill(tag, Domain{spec->lo})), vec::fill(tag, Domain{spec->hi})); break;
        case 3: v = vec::div(tag, one, vec::add(tag, one, vec::exp(tag, vec::neg(tag, v)))); break;
        case 4: v = vec::mul(tag, v, vec::div(tag, one, vec::add(tag, one, vec::exp(tag, vec::neg(tag, v))))); break;
        default: break;
      }
      return v;
    });
}

template <typename Atom, typename TA, typename TB, typename TBias, typename TC>
int run_fused(const TA* a, const TB* b, const TBias* bias, TC* c, int64_t m, int64_t n, int64_t k,
              const FusedSpec* spec) {
  if (!enable_amx()) return -1;
  using Acc = typename Atom::TAcc;
  auto at = view2(const_cast<TA*>(a), m, k, k, 1);
  auto bt = view2(const_cast<TB*>(b), n, k, k, 1);
  auto ct = view2(c, m, n, n, 1);
  auto cout = tensor::output<Acc>(ct, fused_transform<float32_t>(spec));
  auto op = ops::matmul(ops::MatmulConfig<Atom>{});
  if (bias) {
    auto bias_t = tensor::input<Acc>(view2(const_cast<TBias*>(bias), m, n, 0, 1));
    const nint_t bytes = op.required_workspace(Any{m}, Any{n}, Any{k}, at, bt, bias_t, cout);
    kernel::Workspace ws(bytes);
    auto v = ws.view();
    op(v, Any{m}, Any{n}, Any{k}, at, bt, bias_t, cout);
  } else {
    const nint_t bytes = op.required_workspace(Any{m}, Any{n}, Any{k}, at, bt, cout);
    kernel::Workspace ws(bytes);
    auto v = ws.view();
    op(v, Any{m}, Any{n}, Any{k}, at, bt, cout);
  }
  return 0;
}

// ---- dense forms, for timing the reference at its best ----------------------------------------------
// The entry points above describe every tensor with run-time strides, the most general form; vecops plans its
// kernels from the layout types, and a dense row-major layout (unit inner stride known at compile time) is the
// form its own benchmarks use (benchmarks/ops/MatmulBenchCommon.h:133-190).  A conventional B[K,N] is the
// transposed view of a dense [K,N] tensor (tests/ops/MatmulOrientationTest.cpp:65-70).
template <typename T>
auto dense2(T* p, int64_t rows, int64_t cols) {
  return make_tensor(p, make_layout(make_shape(Any{rows}, Any{cols})));
}
template <typename T>
auto dense3(T* p, int64_t batch, int64_t rows, int64_t cols) {
  return make_tensor(p, make_layout(make_shape(Any{batch}, Any{rows}, Any{cols})));
}
template <typename Atom, typename A, typename B, typename Cc>
int run_dense(A at, B bt, Cc ct, int64_t m, int64_t n, int64_t k) {
  if (!enable_amx()) return -1;
  auto op = ops::matmul(ops::MatmulConfig<Atom>{});
  const nint_t bytes = op.required_workspace(Any{m}, Any{n}, Any{k}, at, bt, ct);
  kernel::Workspace ws(bytes);
  auto v = ws.view();
  op(v, Any{m}, Any{n}, Any{k}, at, bt, ct);
  return 0;
}

}  // namespace

extern "C" {

#define VREF_EXPORT __attribute__((visibility("default")))

VREF_EXPORT int vref_available(void) { return enable_amx() ? 1 : 0; }

// bf16 x bf16 -> fp32 / bf16, fp32 memory -> bf16 compute -> fp32 / bf16 (AMX_BF16F32).
VREF_EXPORT int vref_matmul_bf16_f32(const uint16_t* a, const uint16_t* b, float* c, const float* cin, int64_t m,
                                     int64_t n, int64_t k, const int64_t* sa, const int64_t* sb, const int64_t* sc) {
  return run2<matmul::AMX_BF16F32>(reinterpret_cast<const bfloat16_t*>(a), reinterpret_cast<const bfloat16_t*>(b), c,
                                   cin, m, n, k, sa, sb, sc);
}
VREF_EXPORT int vref_matmul_bf16_bf16(const uint16_t* a, const uint16_t* b, uint16_t* c, int64_t m, int64_t n,
                                      int64_t k, const int64_t* sa, const int64_t* sb, const int64_t* sc) {
  return run2<matmul::AMX_BF16F32>(reinterpret_cast<const bfloat16_t*>(a), reinterpret_cast<const bfloat16_t*>(b),
                                   reinterpret_cast<bfloat16_t*>(c), static_cast<const bfloat16_t*>(nullptr), m, n, k,
                                   sa, sb, sc);
}
VREF_EXPORT int vref_matmul_f32_f32(const float* a, const float* b, float* c, const float* cin, int64_t m, int64_t n,
                                    int64_t k, const int64_t* sa, const int64_t* sb, const int64_t* sc) {
  return run2<matmul::AMX_BF16F32>(a, b, c, cin, m, n, k, sa, sb, sc);
}
VREF_EXPORT int vref_matmul_f32_bf16(const float* a, const float* b, uint16_t* c, int64_t m, int64_t n, int64_t k,
                                     const int64_t* sa, const int64_t* sb, const int64_t* sc) {
  return run2<matmul::AMX_BF16F32>(a, b, reinterpret_cast<bfloat16_t*>(c), static_cast<const bfloat16_t*>(nullptr), m,
                                   n, k, sa, sb, sc);
}
// Rank-3 batch (stride 0 on the batch axis = broadcast operand).
VREF_EXPORT int vref_matmul_bf16_f32_batched(const uint16_t* a, const uint16_t* b, float* c, int64_t batch, int64_t m,
                                             int64_t n, int64_t k, const int64_t* sa, const int64_t* sb,
                                             const int64_t* sc) {
  return run3<matmul::AMX_BF16F32>(reinterpret_cast<const bfloat16_t*>(a), reinterpret_cast<const bfloat16_t*>(b), c,
                                   batch, m, n, k, sa, sb, sc);
}
// int8 x int8 -> int32 (wraps) and u8 x i8 -> int32.
VREF_EXPORT int vref_matmul_i8_i32(const int8_t* a, const int8_t* b, int32_t* c, const int32_t* cin, int64_t m,
                                   int64_t n, int64_t k, const int64_t* sa, const int64_t* sb, const int64_t* sc) {
  return run2<matmul::AMX_I8I32<int8_t, int8_t>>(a, b, c, cin, m, n, k, sa, sb, sc);
}
VREF_EXPORT int vref_matmul_u8i8_i32(const uint8_t* a, const int8_t* b, int32_t* c, int64_t m, int64_t n, int64_t k,
                                     const int64_t* sa, const int64_t* sb, const int64_t* sc) {
  return run2<matmul::AMX_I8I32<uint8_t, int8_t>>(a, b, c, static_cast<const int32_t*>(nullptr), m, n, k, sa, sb, sc);
}

// int8 x int8 with the fused per-row x per-column dequantisation epilogue
// (matmul/Quantization.h:195-250).  column_scales must be readable 64 floats
// past n (unmasked vector load, Quantization.h:229-231).  correction (may be
// null) is the stride-0 int32 C-input row of
// tests/ops/MatmulConversionTestCommon.h:1467-1472.
VREF_EXPORT int vref_matmul_i8_dequant(const int8_t* a, const int8_t* b, const float* row_scales,
                                       const float* column_scales, const int32_t* correction, float* c, int64_t m,
                                       int64_t n, int64_t k) {
  if (!enable_amx()) return -1;
  using Atom = matmul::AMX_I8I32<int8_t, int8_t>;
  auto at = view2(const_cast<int8_t*>(a), m, k, k, 1);
  auto bt = view2(const_cast<int8_t*>(b), n, k, k, 1);
  auto ct = view2(c, m, n, n, 1);
  auto deq = matmul::make_runtime_per_row_column_dequantize_transform({row_scales, column_scales, 0});
  auto cout = tensor::output<int32_t>(ct, deq);
  auto op = ops::matmul(ops::MatmulConfig<Atom>{});
  if (correction) {
    auto cit = view2(const_cast<int32_t*>(correction), m, n, 0, 1);
    const nint_t bytes = op.required_workspace(Any{m}, Any{n}, Any{k}, at, bt, cit, cout);
    kernel::Workspace ws(bytes);
    auto v = ws.view();
    op(v, Any{m}, Any{n}, Any{k}, at, bt, cit, cout);
  } else {
    const nint_t bytes = op.required_workspace(Any{m}, Any{n}, Any{k}, at, bt, cout);
    kernel::Workspace ws(bytes);
    auto v = ws.view();
    op(v, Any{m}, Any{n}, Any{k}, at, bt, cout);
  }
  return 0;
}

// fp32 activations quantised on their way in by RuntimePerRowAsymmetricQuantizeTransform
// (matmul/Quantization.h:91-146: q = x * multipliers[row] + float(zero_point), converted to the
// atom's uint8), int8 weights, the stride-0 int32 correction row as C input, and either the
// plain int32 sums (row_scales == null: c is int32) or the per-row x per-column dequantisation
// (c is fp32) - the pipeline of tests/ops/MatmulConversionTestCommon.h:1437-1540 with B unpacked.
VREF_EXPORT int vref_matmul_runtime_quant(const float* a, const int8_t* b, const float* multipliers,
                                          int32_t zero_point, const float* row_scales, const float* column_scales,
                                          const int32_t* correction, void* c, int64_t m, int64_t n, int64_t k) {
  if (!enable_amx()) return -1;
  using Atom = matmul::AMX_I8I32<uint8_t, int8_t>;
  auto at = view2(const_cast<float*>(a), m, k, k, 1);
  auto bt = view2(const_cast<int8_t*>(b), n, k, k, 1);
  auto cit = view2(const_cast<int32_t*>(correction), m, n, 0, 1);
  auto quantize = matmul::make_runtime_per_row_asymmetric_quantize_transform({multipliers, &zero_point, 0});
  auto ain = tensor::input<uint8_t>(at, quantize);
  auto cin = tensor::input<int32_t>(cit);
  auto op = ops::matmul(ops::MatmulConfig<Atom>{});
  if (row_scales != nullptr) {
    auto ct = view2(static_cast<float*>(c), m, n, n, 1);
    auto deq = matmul::make_runtime_per_row_column_dequantize_transform({row_scales, column_scales, 0});
    auto cout = tensor::output<int32_t>(ct, deq);
    kernel::Workspace ws(op.required_workspace(Any{m}, Any{n}, Any{k}, ain, bt, cin, cout));
    auto v = ws.view();
    op(v, Any{m}, Any{n}, Any{k}, ain, bt, cin, cout);
  } else {
    auto ct = view2(static_cast<int32_t*>(c), m, n, n, 1);
    kernel::Workspace ws(op.required_workspace(Any{m}, Any{n}, Any{k}, ain, bt, cin, ct));
    auto v = ws.view();
    op(v, Any{m}, Any{n}, Any{k}, ain, bt, cin, ct);
  }
  return 0;
}

// The batched form of the same pipeline (tests/ops/MatmulConversionTestCommon.h:1277-1434): a [batch,M,K] (batch
// stride 0 when broadcast_a), b [batch,N,K] (0 when broadcast_b), the correction rows as a C input of strides
// {N or 0, 0, 1}, multipliers and row_scales with batch stride M or 0, c fp32 [batch,M,N] dense.
VREF_EXPORT int vref_matmul_runtime_quant_batched(const float* a, const int8_t* b, const float* multipliers,
                                                  int32_t zero_point, const float* row_scales, const float* column_scales,
                                                  const int32_t* correction, float* c, int64_t batch, int64_t m, int64_t n,
                                                  int64_t k, int broadcast_a, int broadcast_b) {
  if (!enable_amx()) return -1;
  using Atom = matmul::AMX_I8I32<uint8_t, int8_t>;
  auto at = view3(const_cast<float*>(a), batch, m, k, broadcast_a ? 0 : m * k, k, 1);
  auto bt = view3(const_cast<int8_t*>(b), batch, n, k, broadcast_b ? 0 : n * k, k, 1);
  auto cit = view3(const_cast<int32_t*>(correction), batch, m, n, broadcast_b ? 0 : n, 0, 1);
  auto ct = view3(c, batch, m, n, m * n, n, 1);
  const nint_t scale_stride = broadcast_a ? 0 : m;
  auto quantize = matmul::make_runtime_per_row_asymmetric_quantize_transform({multipliers, &zero_point, scale_stride});
  auto deq = matmul::make_runtime_per_row_column_dequantize_transform({row_scales, column_scales, scale_stride});
  auto ain = tensor::input<uint8_t>(at, quantize);
  auto bin = tensor::input<int8_t>(bt);
  auto cin = tensor::input<int32_t>(cit);
  auto cout = tensor::output<int32_t>(ct, deq);
  auto op = ops::matmul(ops::MatmulConfig<Atom>{});
  kernel::Workspace ws(op.required_workspace(Any{m}, Any{n}, Any{k}, ain, bin, cin, cout));
  auto v = ws.view();
  op(v, Any{m}, Any{n}, Any{k}, ain, bin, cin, cout);
  return 0;
}

// c_kind: 0 fp32, 1 bf16, 3 uint8, 4 int8 (the dtype codes of include/vecops_hip.h are not used here).
VREF_EXPORT int vref_matmul_bf16_fused(const uint16_t* a, const uint16_t* b, const float* bias, void* c, int c_kind,
                                       int64_t m, int64_t n, int64_t k, const FusedSpec* spec) {
  const auto* ab = reinterpret_cast<const bfloat16_t*>(a);
  const auto* bb = reinterpret_cast<const bfloat16_t*>(b);
  using Atom = matmul::AMX_BF16F32;
  if (c_kind == 0) return run_fused<Atom>(ab, bb, bias, static_cast<float*>(c), m, n, k, spec);
  if (c_kind == 1) return run_fused<Atom>(ab, bb, bias, static_cast<bfloat16_t*>(c), m, n, k, spec);
  return -2;
}
VREF_EXPORT int vref_matmul_i8_fused(const int8_t* a, const int8_t* b, const int32_t* bias, void* c, int c_kind,
                                     int64_t m, int64_t n, int64_t k, const FusedSpec* spec) {
  using Atom = matmul::AMX_I8I32<int8_t, int8_t>;
  if (c_kind == 0) return run_fused<Atom>(a, b, bias, static_cast<float*>(c), m, n, k, spec);
  if (c_kind == 3) return run_fused<Atom>(a, b, bias, static_cast<uint8_t*>(c), m, n, k, spec);
  if (c_kind == 4) return run_fused<Atom>(a, b, bias, static_cast<int8_t*>(c), m, n, k, spec);
  return -2;
}

// The non-inline dispatch predicates of src/MatmulRuntimeDispatch.cpp:12-32.
VREF_EXPORT int vref_dense_bf16_bf16(const uint16_t* a, const uint16_t* b, uint16_t* c, int64_t m, int64_t n, int64_t k,
                                     int b_is_kn) {
  auto at = dense2(reinterpret_cast<bfloat16_t*>(const_cast<uint16_t*>(a)), m, k);
  auto ct = dense2(reinterpret_cast<bfloat16_t*>(c), m, n);
  bfloat16_t* bp = reinterpret_cast<bfloat16_t*>(const_cast<uint16_t*>(b));
  if (b_is_kn) return run_dense<matmul::AMX_BF16F32>(at, tensor::transpose_view<0, 1>(dense2(bp, k, n)), ct, m, n, k);
  return run_dense<matmul::AMX_BF16F32>(at, dense2(bp, n, k), ct, m, n, k);
}

VREF_EXPORT int vref_dense_f32_f32(const float* a, const float* b, float* c, int64_t m, int64_t n, int64_t k, int b_is_kn) {
  auto at = dense2(const_cast<float*>(a), m, k);
  auto ct = dense2(c, m, n);
  float* bp = const_cast<float*>(b);
  if (b_is_kn) return run_dense<matmul::AMX_BF16F32>(at, tensor::transpose_view<0, 1>(dense2(bp, k, n)), ct, m, n, k);
  return run_dense<matmul::AMX_BF16F32>(at, dense2(bp, n, k), ct, m, n, k);
}

VREF_EXPORT int vref_dense_bf16_f32_batched(const uint16_t* a, const uint16_t* b, float* c, int64_t batch, int64_t m,
                                            int64_t n, int64_t k) {
  return run_dense<matmul::AMX_BF16F32>(dense3(reinterpret_cast<bfloat16_t*>(const_cast<uint16_t*>(a)), batch, m, k),
                                        dense3(reinterpret_cast<bfloat16_t*>(const_cast<uint16_t*>(b)), batch, n, k),
                                        dense3(c, batch, m, n), m, n, k);
}

VREF_EXPORT int vref_dense_i8_dequant(const int8_t* a, const int8_t* b, const float* row_scales, const float* column_scales,
                                      float* c, int64_t m, int64_t n, int64_t k) {
  auto deq = matmul::make_runtime_per_row_column_dequantize_transform({row_scales, column_scales, 0});
  return run_dense<matmul::AMX_I8I32<int8_t, int8_t>>(dense2(const_cast<int8_t*>(a), m, k), dense2(const_cast<int8_t*>(b), n, k),
                                                      tensor::output<int32_t>(dense2(c, m, n), deq), m, n, k);
}

VREF_EXPORT int vref_amx_small_vector_profitable(int shape, int64_t m, int64_t n, int64_t k) {
  return kernel::matmul_details::runtime_amx_small_vector_profitable(
    static_cast<kernel::matmul_details::SmallVectorShape>(shape), m, n, k);
}
VREF_EXPORT int vref_sme_small_vector_profitable(int shape, int64_t m, int64_t n, int64_t k) {
  return kernel::matmul_details::runtime_sme_small_vector_profitable(
    static_cast<kernel::matmul_details::SmallVectorShape>(shape), m, n, k);
}
VREF_EXPORT int vref_small_area_profitable(int64_t m, int64_t n, int64_t k, int64_t limit) {
  return kernel::matmul_details::runtime_small_area_profitable(m, n, k, limit);
}
VREF_EXPORT int vref_amx_residual_split_profitable(int64_t m, int64_t n, int64_t k) {
  return kernel::matmul_details::runtime_amx_residual_split_profitable(m, n, k);
}

}  // extern "C"
