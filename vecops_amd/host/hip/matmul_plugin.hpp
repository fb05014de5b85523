// The MI355X drop-in for the vecops matmul path: operator schemas, kernel
// recipes, the shape-class dispatch policy and the executable provider that
// hands out ahead-of-time built HIP artifact DSOs.  Everything here implements
// vecops' own plug-in interfaces (runtime/Operator.h:67-191); an application
// builds `Operator(schema, recipes, policy, provider)` exactly as it would for
// any other vecops backend.
//
// Logical operators (vecops ships no matmul OperatorSchema; at its C++ level the
// scales ride on tensor specs as functor transforms, matmul/Quantization.h:91-250,
// which cannot cross the C ABI, so they are positional tensors here; outputs
// last and caller-allocated, runtime/KernelDefinition.h:217-229):
//
//   vecops::matmul              (a[..,M,K], b[..,N,K], c_in?[..,M,N], c[..,M,N] out)
//       specialization value  ComputeType : DType   (BFloat16 default, Float32)
//   vecops::matmul_i8_dequant   (a i8[M,K], b i8[N,K], row_scales f32[M],
//                                column_scales f32[N], correction? i32[N], c f32[M,N] out)
//   vecops::matmul_w8a16_group  (x bf16[M,K], w i8[N,K], scales f32[N,K/G], y bf16[M,N] out)
//       specialization value  G : ConstInt          (128 default)
//   vecops::matmul_pack_b       (b[N,K], a_zero_point scalar, packed u8[bytes] out, compensation? i32[N] out)
//       specialization value  PackedType : DType    (the source's own class by default)
//   vecops::matmul_packed_b     (a[..,M,K], packed_b u8[bytes], c_in?[..,M,N], c[..,M,N] out)
//   vecops::matmul_runtime_quant (a f32[M,K], b i8[N,K], multipliers f32[M], zero_point scalar,
//                                row_scales f32[M], column_scales f32[N], correction? i32[N], c f32[M,N] out)
#ifndef VECOPS_HIP_MATMUL_PLUGIN_HPP
#define VECOPS_HIP_MATMUL_PLUGIN_HPP

#include <condition_variable>
#include <filesystem>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "vecops_rt/surface.hpp"

namespace vecops::hip {

namespace rt = ::vecops::runtime;

inline constexpr const char* kMatmulName = "vecops::matmul";
inline constexpr const char* kMatmulI8DequantName = "vecops::matmul_i8_dequant";
inline constexpr const char* kMatmulW8A16GroupName = "vecops::matmul_w8a16_group";
inline constexpr const char* kMatmulFusedName = "vecops::matmul_fused";
inline constexpr const char* kMatmulPackBName = "vecops::matmul_pack_b";
inline constexpr const char* kMatmulPackedBName = "vecops::matmul_packed_b";
inline constexpr const char* kMatmulPackAName = "vecops::matmul_pack_a";
inline constexpr const char* kMatmulPackedAName = "vecops::matmul_packed_a";
inline constexpr const char* kMatmulRuntimeQuantName = "vecops::matmul_runtime_quant";

// Operand classes of vecops::matmul, one artifact each (U8: packs of unsigned bytes only).
enum class OperandClass { BF16, F32, I8, F16, U8 };
// The side a packed operand was packed for (ops::matmul_pack's Operand::A / Operand::B, ops/MatmulPack.h:63-65).
enum class PackSide { A, B };

// Schemas.  Ranks are left open on vecops::matmul (rank 2 and rank 3 go through
// one operator); the relation validator enforces what the CPU path asserts in
// validate() (planning/families/ArchitectureFamily.h:1590-1652,
// planning/families/GenericTiled.h:100-154): equal ranks, A=[..,M,K], B=[..,N,K],
// C=[..,M,N], equal batch extents.
rt::OperatorSchema make_matmul_schema();
rt::OperatorSchema make_matmul_i8_dequant_schema();
rt::OperatorSchema make_matmul_w8a16_group_schema();
// vecops::matmul_fused (a, b, c_in?, row_scales?, column_scales?, activation, scale, shift, clamp_lo, clamp_hi,
// c out): vecops::matmul with a fused output transform, the catalogue that vecops' tests build from
// tensor::output transforms (tests/ops/MatmulFusionTest.cpp:29-112).  The five scalars are always present
// (the call ABI has no optional scalars): activation 0 none, 1 relu, 2 clamp, 3 sigmoid, 4 silu; scale 1.0 and
// shift 0.0 mean "no such step".
rt::OperatorSchema make_matmul_fused_schema();
// vecops::matmul_pack_b (b, a_zero_point, packed out, compensation? out): the B side of ops::matmul_pack
// (ops/MatmulPack.h:9-117).  `packed` is an opaque byte tensor of at least vecops_hip_packed_b_bytes(dtype, N, K) bytes; with a
// compensation tensor (int8 only) the pack also writes -a_zero_point * sum_k b[n,k], the sidecar of
// MatmulPackBCompensated.  vecops::matmul_packed_b (a, packed_b, c_in?, c out) multiplies by such a tensor: N
// comes from c, K from a, and one packed operand serves every batch of a rank-3 a (ops/MatmulPack.h:22-24).
rt::OperatorSchema make_matmul_pack_b_schema();
rt::OperatorSchema make_matmul_packed_b_schema();
// Side A (ops::MatmulPack<MatmulPackConfig<Atom, Operand::A>>, ops/MatmulPack.h:81-96; tests/ops/MatmulMixedPackingTest.cpp:24-28):
// vecops::matmul_pack_a (a[M,K], packed out) and vecops::matmul_packed_a (packed_a, b[..,N,K], c_in?, c out) - M comes
// from c, K from b, and the one packed a serves every batch of a rank-3 b.
// Unsigned weights (AMX_I8I32<int8_t, uint8_t>, <uint8_t, uint8_t>): a uint8 source packs like any other; the product
// is told by the specialization value `PackedType` = UInt8 that its packed operand holds unsigned bytes (a packed
// tensor is opaque bytes here, where vecops' packed Tensor carries its dtype).  Absent, the packed operand has the
// class's own type (int8 for the 8-bit class).
rt::OperatorSchema make_matmul_pack_a_schema();
rt::OperatorSchema make_matmul_packed_a_schema();
// vecops::matmul_runtime_quant: fp32 activations quantised on the way in by vecops'
// RuntimePerRowAsymmetricQuantizeTransform (q = u8(a * multipliers[row] + zero_point), matmul/Quantization.h:91-146),
// int8 weights, the int32 correction row as C input and the per-row x per-column dequantisation on the way out -
// the pipeline of tests/ops/MatmulConversionTestCommon.h:1437-1540 with the transforms' arrays as positional tensors.
rt::OperatorSchema make_matmul_runtime_quant_schema();

// Kernel families a recipe stands for: the MFMA workgroup-tile kernels or the
// wavefront split-K dot-product kernels for skinny shapes.
enum class KernelFamily { Tile, Skinny };

// Where the tensors of a call live.  Host tensors are staged through device
// memory inside the artifact; device tensors (VECOPS_DEVICE_PRIVATE carrying HIP
// device pointers) are used in place.
enum class Placement { Host, Device };

// Recipe of vecops::matmul for one operand class.  match() is metadata-only:
// dtype class, ComputeType, uniform placement.  bind() yields
//   vecops::matmul;operands=<bf16|f16|f32|i8>;compute=<bf16|f16|f32|i32>;memory=<host|device>;backend=hip-gfx950
class MatmulRecipe final : public rt::KernelRecipe {
public:
  explicit MatmulRecipe(OperandClass operands);
  [[nodiscard]] std::string_view id() const override { return id_; }
  [[nodiscard]] rt::Status match(const rt::KernelCall& call) const override;
  [[nodiscard]] rt::Result<rt::BoundKernelRecipe> bind(const rt::KernelCall& call) const override;
  [[nodiscard]] OperandClass operands() const { return operands_; }

private:
  OperandClass operands_;
  std::string id_;
};

// vecops::matmul_i8_dequant:  ...;operands=i8;epilogue=row_col_dequant;memory=..;backend=hip-gfx950
class MatmulI8DequantRecipe final : public rt::KernelRecipe {
public:
  [[nodiscard]] std::string_view id() const override { return "hip.matmul_i8_dequant.tile"; }
  [[nodiscard]] rt::Status match(const rt::KernelCall& call) const override;
  [[nodiscard]] rt::Result<rt::BoundKernelRecipe> bind(const rt::KernelCall& call) const override;
};

// vecops::matmul_fused for one operand class (fp32 operands multiply in bf16):
//   vecops::matmul_fused;operands=<bf16|f16|f32|i8>;memory=<host|device>;backend=hip-gfx950
class MatmulFusedRecipe final : public rt::KernelRecipe {
public:
  explicit MatmulFusedRecipe(OperandClass operands);
  [[nodiscard]] std::string_view id() const override { return id_; }
  [[nodiscard]] rt::Status match(const rt::KernelCall& call) const override;
  [[nodiscard]] rt::Result<rt::BoundKernelRecipe> bind(const rt::KernelCall& call) const override;
  [[nodiscard]] OperandClass operands() const { return operands_; }

private:
  OperandClass operands_;
  std::string id_;
};

// vecops::matmul_w8a16_group, skinny family (M <= 16):  ...;G=<group>;memory=..;backend=hip-gfx950
class MatmulW8A16GroupRecipe final : public rt::KernelRecipe {
public:
  [[nodiscard]] std::string_view id() const override { return "hip.matmul_w8a16_group.skinny"; }
  [[nodiscard]] rt::Status match(const rt::KernelCall& call) const override;
  [[nodiscard]] rt::Result<rt::BoundKernelRecipe> bind(const rt::KernelCall& call) const override;
};

// vecops::matmul_pack_b / vecops::matmul_pack_a for one packed class (BF16 takes bf16 and fp32 sources, I8 int8,
// U8 uint8, F16 half; F32 takes fp32 sources when the call's ComputeType is Float32 and keeps their elements fp32 - the
// pack of the fp32-compute atom):
//   vecops::matmul_pack_<a|b>;operands=<bf16|f16|f32|i8|u8>;memory=<host|device>;backend=hip-gfx950
class MatmulPackBRecipe final : public rt::KernelRecipe {
public:
  explicit MatmulPackBRecipe(OperandClass packed, PackSide side = PackSide::B);
  [[nodiscard]] std::string_view id() const override { return id_; }
  [[nodiscard]] rt::Status match(const rt::KernelCall& call) const override;
  [[nodiscard]] rt::Result<rt::BoundKernelRecipe> bind(const rt::KernelCall& call) const override;
  [[nodiscard]] OperandClass operands() const { return packed_; }
  [[nodiscard]] PackSide side() const { return side_; }

private:
  OperandClass packed_;
  PackSide side_;
  std::string id_;
};

// vecops::matmul_packed_b for one class of a (fp32 rows are rounded to bf16 against a bf16 pack; the i8 class
// takes signed and unsigned bytes, AMX_I8I32<uint8_t, int8_t> being what the compensated pack is for):
//   vecops::matmul_packed_b;operands=<bf16|f32|i8>;memory=<host|device>;backend=hip-gfx950
// With side A the same for vecops::matmul_packed_a and the class of b; `packed_unsigned` marks the recipe of the 8-bit
// class that serves PackedType = UInt8:  ...;operands=i8;packed=u8;memory=...; `f32_compute` the recipe of the fp32
// class that serves ComputeType = Float32 (an fp32-packed operand, products in fp32):  ...;operands=f32;compute=f32;...
class MatmulPackedBRecipe final : public rt::KernelRecipe {
public:
  explicit MatmulPackedBRecipe(OperandClass operands, PackSide side = PackSide::B, bool packed_unsigned = false,
                               bool f32_compute = false);
  [[nodiscard]] std::string_view id() const override { return id_; }
  [[nodiscard]] rt::Status match(const rt::KernelCall& call) const override;
  [[nodiscard]] rt::Result<rt::BoundKernelRecipe> bind(const rt::KernelCall& call) const override;
  [[nodiscard]] OperandClass operands() const { return operands_; }
  [[nodiscard]] PackSide side() const { return side_; }
  [[nodiscard]] bool packed_unsigned() const { return packed_unsigned_; }
  [[nodiscard]] bool f32_compute() const { return f32_compute_; }

private:
  OperandClass operands_;
  PackSide side_;
  bool packed_unsigned_;
  bool f32_compute_;
  std::string id_;
};

// vecops::matmul_runtime_quant:  ...;operands=f32_i8;epilogue=row_col_dequant;memory=..;backend=hip-gfx950
class MatmulRuntimeQuantRecipe final : public rt::KernelRecipe {
public:
  [[nodiscard]] std::string_view id() const override { return "hip.matmul_runtime_quant.tile"; }
  [[nodiscard]] rt::Status match(const rt::KernelCall& call) const override;
  [[nodiscard]] rt::Result<rt::BoundKernelRecipe> bind(const rt::KernelCall& call) const override;
};

// GPU counterpart of the call sites of vecops' runtime shape predicates
// (matmul/details/kernel/amx/Backend.h:2724-2757 consulting
// src/MatmulRuntimeDispatch.cpp:12-32): orders the recipes of an operator for
// one call.  Recipes whose operand class cannot take the call are dropped (they
// would answer NotApplicable anyway); the rest keep declaration order.
class MatmulDispatchPolicy final : public rt::DispatchPolicy {
public:
  [[nodiscard]] rt::Result<std::vector<std::size_t>>
  candidates(const rt::KernelCall& call, std::span<const std::shared_ptr<const rt::KernelRecipe>> recipes) const override;
};

// Resolves bound recipes to artifact DSOs found in one directory
// (<directory>/<file name derived from the specialization key>.so).  Never
// builds: a missing artifact is NotFound, like vecops' provider in CacheOnly
// mode (src/runtime/Provider.cpp:175-236).  Thread-safe; identical concurrent
// requests load the DSO once.
class HipExecutableProvider final : public rt::ExecutableProvider {
public:
  explicit HipExecutableProvider(std::filesystem::path artifact_directory);
  [[nodiscard]] rt::Result<std::shared_ptr<rt::Executable>> resolve(const rt::BoundKernelRecipe& recipe) override;
  // File an artifact with this key is expected under.
  [[nodiscard]] std::filesystem::path artifact_path(std::string_view specialization_key) const;
  [[nodiscard]] std::size_t loads() const;  // DSOs actually loaded so far (tests)

private:
  struct Pending {
    std::condition_variable ready;
    bool done = false;
  };
  std::filesystem::path directory_;
  mutable std::mutex mutex_;
  std::map<std::string, std::shared_ptr<rt::Executable>, std::less<>> loaded_;
  std::map<std::string, std::shared_ptr<Pending>, std::less<>> pending_;
  std::size_t loads_ = 0;
};

// File name (without directory) of the artifact for a specialization key:
// characters outside [A-Za-z0-9_.=-] become '_', plus ".so".
std::string artifact_file_name(std::string_view specialization_key);

// Ready-made operators over one artifact directory.
std::shared_ptr<rt::Operator> make_matmul_operator(const std::filesystem::path& artifact_directory);
std::shared_ptr<rt::Operator> make_matmul_i8_dequant_operator(const std::filesystem::path& artifact_directory);
std::shared_ptr<rt::Operator> make_matmul_w8a16_group_operator(const std::filesystem::path& artifact_directory);
std::shared_ptr<rt::Operator> make_matmul_fused_operator(const std::filesystem::path& artifact_directory);
std::shared_ptr<rt::Operator> make_matmul_pack_b_operator(const std::filesystem::path& artifact_directory);
std::shared_ptr<rt::Operator> make_matmul_packed_b_operator(const std::filesystem::path& artifact_directory);
std::shared_ptr<rt::Operator> make_matmul_pack_a_operator(const std::filesystem::path& artifact_directory);
std::shared_ptr<rt::Operator> make_matmul_packed_a_operator(const std::filesystem::path& artifact_directory);
std::shared_ptr<rt::Operator> make_matmul_runtime_quant_operator(const std::filesystem::path& artifact_directory);

}  // namespace vecops::hip
#endif
