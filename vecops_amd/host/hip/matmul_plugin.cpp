#include "matmul_plugin.hpp"

#include <algorithm>

namespace vecops::hip {

namespace {

using rt::DType;
using rt::Status;
using rt::StatusCode;
using rt::TensorView;
using rt::Value;

Status invalid(std::string m) { return Status(StatusCode::InvalidArgument, std::move(m)); }
Status not_applicable(std::string m) { return Status(StatusCode::NotApplicable, std::move(m)); }

const TensorView* tensor_at(std::span<const Value> values, std::size_t i) {
  return i < values.size() ? std::get_if<TensorView>(&values[i]) : nullptr;
}

rt::ParameterSchema tensor_param(std::string name, std::uint64_t dtypes, std::optional<std::uint32_t> rank,
                                 std::uint64_t flags, bool optional = false) {
  rt::TensorConstraint c;
  c.dtype_mask = dtypes;
  c.rank = rank;
  c.required_flags = flags;
  c.optional = optional;
  return rt::ParameterSchema{std::move(name), std::move(c)};
}

std::int64_t rows(const TensorView& t) { return t.sizes[t.sizes.size() - 2]; }
std::int64_t cols(const TensorView& t) { return t.sizes[t.sizes.size() - 1]; }

// A = [..,M,K], B = [..,N,K], C_in / C = [..,M,N]; ranks 2 or 3 and all equal;
// batch extents equal (planning/families/ArchitectureFamily.h:1590-1652).
Status matmul_relations(std::span<const Value> v) {
  const TensorView* a = tensor_at(v, 0);
  const TensorView* b = tensor_at(v, 1);
  const TensorView* cin = tensor_at(v, 2);
  const TensorView* c = tensor_at(v, 3);
  if (a == nullptr || b == nullptr || c == nullptr) return invalid("vecops::matmul needs a, b and c tensors");
  const std::size_t rank = a->sizes.size();
  if (rank != 2 && rank != 3) return invalid("a must have rank 2 or 3");
  if (b->sizes.size() != rank || c->sizes.size() != rank || (cin && cin->sizes.size() != rank))
    return invalid("a, b, c_in and c must have the same rank");
  if (cols(*a) != cols(*b)) return invalid("a and b disagree on K");
  if (rows(*c) != rows(*a) || cols(*c) != rows(*b)) return invalid("c must be [.., M, N]");
  if (cin && (rows(*cin) != rows(*c) || cols(*cin) != cols(*c))) return invalid("c_in must be [.., M, N]");
  if (rank == 3) {
    if (a->sizes[0] != b->sizes[0] || a->sizes[0] != c->sizes[0] || (cin && cin->sizes[0] != c->sizes[0]))
      return invalid("batch extents differ");
  }
  return Status::success();
}

Status dequant_relations(std::span<const Value> v) {
  const TensorView* a = tensor_at(v, 0);
  const TensorView* b = tensor_at(v, 1);
  const TensorView* rs = tensor_at(v, 2);
  const TensorView* cs = tensor_at(v, 3);
  const TensorView* corr = tensor_at(v, 4);
  const TensorView* c = tensor_at(v, 5);
  if (!a || !b || !rs || !cs || !c) return invalid("vecops::matmul_i8_dequant needs a, b, both scale vectors and c");
  if (a->sizes[1] != b->sizes[1]) return invalid("a and b disagree on K");
  if (c->sizes[0] != a->sizes[0] || c->sizes[1] != b->sizes[0]) return invalid("c must be [M, N]");
  if (rs->sizes[0] != a->sizes[0]) return invalid("row_scales must have M entries");
  if (cs->sizes[0] != b->sizes[0]) return invalid("column_scales must have N entries");
  if (corr && corr->sizes[0] != b->sizes[0]) return invalid("correction must have N entries");
  return Status::success();
}

// vecops::matmul_fused: the matmul relations on (a, b, c_in, c = value 10) plus the scale vectors.
Status fused_relations(std::span<const Value> v) {
  const TensorView* a = tensor_at(v, 0);
  const TensorView* b = tensor_at(v, 1);
  const TensorView* cin = tensor_at(v, 2);
  const TensorView* rs = tensor_at(v, 3);
  const TensorView* cs = tensor_at(v, 4);
  const TensorView* c = tensor_at(v, 10);
  if (a == nullptr || b == nullptr || c == nullptr) return invalid("vecops::matmul_fused needs a, b and c tensors");
  const std::size_t rank = a->sizes.size();
  if (rank != 2 && rank != 3) return invalid("a must have rank 2 or 3");
  if (b->sizes.size() != rank || c->sizes.size() != rank || (cin && cin->sizes.size() != rank))
    return invalid("a, b, c_in and c must have the same rank");
  if (cols(*a) != cols(*b)) return invalid("a and b disagree on K");
  if (rows(*c) != rows(*a) || cols(*c) != rows(*b)) return invalid("c must be [.., M, N]");
  if (cin && (rows(*cin) != rows(*c) || cols(*cin) != cols(*c))) return invalid("c_in must be [.., M, N]");
  if (rank == 3 && (a->sizes[0] != b->sizes[0] || a->sizes[0] != c->sizes[0] || (cin && cin->sizes[0] != c->sizes[0])))
    return invalid("batch extents differ");
  const std::int64_t batch = rank == 3 ? a->sizes[0] : 1;
  if (rs && rs->sizes[0] != batch * rows(*a)) return invalid("row_scales must have one entry per row of a");
  if (cs && cs->sizes[0] != rows(*b)) return invalid("column_scales must have N entries");
  const auto* act = std::get_if<rt::Scalar>(&v[5]);
  if (act == nullptr || act->value.i64 < 0 || act->value.i64 > 4) return invalid("activation must be 0..4");
  return Status::success();
}

Status w8a16_relations(std::span<const Value> v) {
  const TensorView* x = tensor_at(v, 0);
  const TensorView* w = tensor_at(v, 1);
  const TensorView* s = tensor_at(v, 2);
  const TensorView* y = tensor_at(v, 3);
  if (!x || !w || !s || !y) return invalid("vecops::matmul_w8a16_group needs x, w, scales and y");
  if (x->sizes[1] != w->sizes[1]) return invalid("x and w disagree on K");
  if (y->sizes[0] != x->sizes[0] || y->sizes[1] != w->sizes[0]) return invalid("y must be [M, N]");
  if (s->sizes[0] != w->sizes[0]) return invalid("scales must have N rows");
  return Status::success();
}

// vecops::matmul_pack_b (b, a_zero_point, packed, compensation?)
Status pack_b_relations(std::span<const Value> v) {
  const TensorView* b = tensor_at(v, 0);
  const TensorView* packed = tensor_at(v, 2);
  const TensorView* comp = tensor_at(v, 3);
  if (b == nullptr || packed == nullptr) return invalid("vecops::matmul_pack_b needs b and packed tensors");
  if (v.size() < 2 || std::get_if<rt::Scalar>(&v[1]) == nullptr) return invalid("a_zero_point must be a scalar");
  if (comp != nullptr && b->dtype != DType::Int8) return invalid("compensation goes with an int8 b");
  if (comp != nullptr && comp->sizes[0] != b->sizes[0]) return invalid("compensation must have N entries");
  return Status::success();
}

// vecops::matmul_pack_a (a, packed)
Status pack_a_relations(std::span<const Value> v) {
  if (tensor_at(v, 0) == nullptr || tensor_at(v, 1) == nullptr) return invalid("vecops::matmul_pack_a needs a and packed tensors");
  return Status::success();
}

// vecops::matmul_packed_a (packed_a, b, c_in?, c): M is c's second-to-last extent, K is b's last.
Status packed_a_relations(std::span<const Value> v) {
  const TensorView* packed = tensor_at(v, 0);
  const TensorView* b = tensor_at(v, 1);
  const TensorView* cin = tensor_at(v, 2);
  const TensorView* c = tensor_at(v, 3);
  if (packed == nullptr || b == nullptr || c == nullptr) return invalid("vecops::matmul_packed_a needs packed_a, b and c");
  const std::size_t rank = b->sizes.size();
  if (rank != 2 && rank != 3) return invalid("b must have rank 2 or 3");
  if (c->sizes.size() != rank || (cin && cin->sizes.size() != rank)) return invalid("b, c_in and c must have the same rank");
  if (cols(*c) != rows(*b)) return invalid("c must be [.., M, N]");
  if (cin && (rows(*cin) != rows(*c) || cols(*cin) != cols(*c))) return invalid("c_in must be [.., M, N]");
  if (rank == 3 && (b->sizes[0] != c->sizes[0] || (cin && cin->sizes[0] != c->sizes[0]))) return invalid("batch extents differ");
  return Status::success();
}

// vecops::matmul_packed_b (a, packed_b, c_in?, c): N is c's last extent, K is a's.
Status packed_b_relations(std::span<const Value> v) {
  const TensorView* a = tensor_at(v, 0);
  const TensorView* packed = tensor_at(v, 1);
  const TensorView* cin = tensor_at(v, 2);
  const TensorView* c = tensor_at(v, 3);
  if (a == nullptr || packed == nullptr || c == nullptr) return invalid("vecops::matmul_packed_b needs a, packed_b and c");
  const std::size_t rank = a->sizes.size();
  if (rank != 2 && rank != 3) return invalid("a must have rank 2 or 3");
  if (c->sizes.size() != rank || (cin && cin->sizes.size() != rank)) return invalid("a, c_in and c must have the same rank");
  if (rows(*c) != rows(*a)) return invalid("c must be [.., M, N]");
  if (cin && (rows(*cin) != rows(*c) || cols(*cin) != cols(*c))) return invalid("c_in must be [.., M, N]");
  if (rank == 3 && (a->sizes[0] != c->sizes[0] || (cin && cin->sizes[0] != c->sizes[0]))) return invalid("batch extents differ");
  return Status::success();
}

// vecops::matmul_runtime_quant (a, b, multipliers, zero_point, row_scales, column_scales, correction?, c)
Status runtime_quant_relations(std::span<const Value> v) {
  const TensorView* a = tensor_at(v, 0);
  const TensorView* b = tensor_at(v, 1);
  const TensorView* mult = tensor_at(v, 2);
  const TensorView* rs = tensor_at(v, 4);
  const TensorView* cs = tensor_at(v, 5);
  const TensorView* corr = tensor_at(v, 6);
  const TensorView* c = tensor_at(v, 7);
  if (!a || !b || !mult || !rs || !cs || !c)
    return invalid("vecops::matmul_runtime_quant needs a, b, multipliers, both scale vectors and c");
  if (v.size() < 4 || std::get_if<rt::Scalar>(&v[3]) == nullptr) return invalid("zero_point must be a scalar");
  if (a->sizes[1] != b->sizes[1]) return invalid("a and b disagree on K");
  if (c->sizes[0] != a->sizes[0] || c->sizes[1] != b->sizes[0]) return invalid("c must be [M, N]");
  if (mult->sizes[0] != a->sizes[0]) return invalid("multipliers must have M entries");
  if (rs->sizes[0] != a->sizes[0]) return invalid("row_scales must have M entries");
  if (cs->sizes[0] != b->sizes[0]) return invalid("column_scales must have N entries");
  if (corr && corr->sizes[0] != b->sizes[0]) return invalid("correction must have N entries");
  return Status::success();
}

// Placement of a call: all tensors on the host, or all on the device.
rt::Result<Placement> placement_of(const rt::KernelCall& call) {
  bool host = false, device = false;
  for (const Value& v : call.arguments().values()) {
    if (const auto* t = std::get_if<TensorView>(&v)) {
      if (t->device_type == VECOPS_DEVICE_CPU) host = true;
      else if (t->device_type == VECOPS_DEVICE_PRIVATE) device = true;
      else return not_applicable("tensors must be host (CPU) or HIP device (PRIVATE) memory");
    }
  }
  if (host && device) return not_applicable("tensors of one call must all be host or all be device memory");
  return device ? Placement::Device : Placement::Host;
}

const char* placement_name(Placement p) { return p == Placement::Device ? "device" : "host"; }

rt::Result<DType> compute_type(const rt::KernelCall& call) {
  auto it = call.values().find("ComputeType");
  if (it == call.values().end()) return DType::BFloat16;
  if (const auto* d = std::get_if<DType>(&it->second)) return *d;
  return invalid("ComputeType must be a DType");
}

// The `PackedType` specialization value of vecops::matmul_packed_a / _b: the element type of the packed operand where the
// dense operand does not fix it - UInt8 for packs of unsigned bytes; absent (or the class's own type) otherwise.
rt::Result<bool> packed_is_unsigned(const rt::KernelCall& call) {
  auto it = call.values().find("PackedType");
  if (it == call.values().end()) return false;
  if (const auto* d = std::get_if<DType>(&it->second)) return *d == DType::UInt8;
  return invalid("PackedType must be a DType");
}

// The `Family` specialization value of vecops::matmul: the number of a kernel family the call requires (vecops'
// family_selection::Require<F>, matmul/Family.h:234-239), or absent / 0 for the automatic choice.  Returns the
// family's name in the specialization key ("" for automatic).
rt::Result<std::string> required_family(const rt::KernelCall& call) {
  auto it = call.values().find("Family");
  if (it == call.values().end()) return std::string();
  const auto* f = std::get_if<std::int64_t>(&it->second);
  if (f == nullptr) return invalid("Family must be an integer (a VecopsHipKernelFamily number)");
  switch (*f) {
    case 0: return std::string();
    case 1: return std::string("tile_256");
    case 2: return std::string("tile_128");
    case 3: return std::string("tile_64");
    case 4: return std::string("skinny");
    case 6: return std::string("tile_256x128");
    case 7: return std::string("tile_128x256");
    case 8: return std::string("tile_256x352");
    case 9: return std::string("tile_192");
    default: return invalid("Family names no kernel family a caller can require");
  }
}

rt::Result<std::int64_t> group_size(const rt::KernelCall& call) {
  auto it = call.values().find("G");
  if (it == call.values().end()) return std::int64_t{128};
  if (const auto* g = std::get_if<std::int64_t>(&it->second)) return *g;
  return invalid("G must be an integer");
}

constexpr const char* kBackend = "backend=hip-gfx950";

std::shared_ptr<rt::Operator> assemble(rt::OperatorSchema schema,
                                       std::vector<std::shared_ptr<const rt::KernelRecipe>> recipes,
                                       const std::filesystem::path& dir) {
  return std::make_shared<rt::Operator>(std::move(schema), std::move(recipes),
                                        std::make_shared<MatmulDispatchPolicy>(),
                                        std::make_shared<HipExecutableProvider>(dir));
}

}  // namespace

// ---- schemas -----------------------------------------------------------------------------------

rt::OperatorSchema make_matmul_schema() {
  using rt::dtype_bit;
  const std::uint64_t in = dtype_bit(DType::BFloat16) | dtype_bit(DType::Float16) | dtype_bit(DType::Float32) |
                           dtype_bit(DType::Int8) | dtype_bit(DType::UInt8);
  const std::uint64_t out = dtype_bit(DType::BFloat16) | dtype_bit(DType::Float16) | dtype_bit(DType::Float32) |
                            dtype_bit(DType::Int32);
  std::vector<rt::ParameterSchema> params;
  params.push_back(tensor_param("a", in, std::nullopt, VECOPS_TENSOR_READ));
  params.push_back(tensor_param("b", in, std::nullopt, VECOPS_TENSOR_READ));
  params.push_back(tensor_param("c_in", out, std::nullopt, VECOPS_TENSOR_READ, /*optional=*/true));
  params.push_back(tensor_param("c", out, std::nullopt, VECOPS_TENSOR_WRITE));
  return rt::OperatorSchema(kMatmulName, std::move(params), matmul_relations);
}

rt::OperatorSchema make_matmul_i8_dequant_schema() {
  using rt::dtype_bit;
  std::vector<rt::ParameterSchema> params;
  params.push_back(tensor_param("a", dtype_bit(DType::Int8), 2u, VECOPS_TENSOR_READ));
  params.push_back(tensor_param("b", dtype_bit(DType::Int8), 2u, VECOPS_TENSOR_READ));
  params.push_back(tensor_param("row_scales", dtype_bit(DType::Float32), 1u, VECOPS_TENSOR_READ));
  params.push_back(tensor_param("column_scales", dtype_bit(DType::Float32), 1u, VECOPS_TENSOR_READ));
  params.push_back(tensor_param("correction", dtype_bit(DType::Int32), 1u, VECOPS_TENSOR_READ, /*optional=*/true));
  params.push_back(tensor_param("c", dtype_bit(DType::Float32), 2u, VECOPS_TENSOR_WRITE));
  return rt::OperatorSchema(kMatmulI8DequantName, std::move(params), dequant_relations);
}

rt::OperatorSchema make_matmul_fused_schema() {
  using rt::dtype_bit;
  const std::uint64_t in = dtype_bit(DType::BFloat16) | dtype_bit(DType::Float16) | dtype_bit(DType::Float32) |
                           dtype_bit(DType::Int8) | dtype_bit(DType::UInt8);
  const std::uint64_t cin = dtype_bit(DType::BFloat16) | dtype_bit(DType::Float16) | dtype_bit(DType::Float32) |
                            dtype_bit(DType::Int32);
  const std::uint64_t out = dtype_bit(DType::BFloat16) | dtype_bit(DType::Float16) | dtype_bit(DType::Float32) |
                            dtype_bit(DType::UInt8) | dtype_bit(DType::Int8);
  const std::uint64_t real = dtype_bit(DType::Float32) | dtype_bit(DType::Float64);
  std::vector<rt::ParameterSchema> params;
  params.push_back(tensor_param("a", in, std::nullopt, VECOPS_TENSOR_READ));
  params.push_back(tensor_param("b", in, std::nullopt, VECOPS_TENSOR_READ));
  params.push_back(tensor_param("c_in", cin, std::nullopt, VECOPS_TENSOR_READ, /*optional=*/true));
  params.push_back(tensor_param("row_scales", dtype_bit(DType::Float32), 1u, VECOPS_TENSOR_READ, /*optional=*/true));
  params.push_back(tensor_param("column_scales", dtype_bit(DType::Float32), 1u, VECOPS_TENSOR_READ, /*optional=*/true));
  params.push_back(rt::ParameterSchema{"activation", rt::ScalarConstraint{dtype_bit(DType::Int64) | dtype_bit(DType::Int32)}});
  for (const char* name : {"scale", "shift", "clamp_lo", "clamp_hi"})
    params.push_back(rt::ParameterSchema{name, rt::ScalarConstraint{real}});
  params.push_back(tensor_param("c", out, std::nullopt, VECOPS_TENSOR_WRITE));
  return rt::OperatorSchema(kMatmulFusedName, std::move(params), fused_relations);
}

rt::OperatorSchema make_matmul_w8a16_group_schema() {
  using rt::dtype_bit;
  std::vector<rt::ParameterSchema> params;
  params.push_back(tensor_param("x", dtype_bit(DType::BFloat16), 2u, VECOPS_TENSOR_READ));
  params.push_back(tensor_param("w", dtype_bit(DType::Int8), 2u, VECOPS_TENSOR_READ));
  params.push_back(tensor_param("scales", dtype_bit(DType::Float32), 2u, VECOPS_TENSOR_READ));
  params.push_back(tensor_param("y", dtype_bit(DType::BFloat16), 2u, VECOPS_TENSOR_WRITE));
  return rt::OperatorSchema(kMatmulW8A16GroupName, std::move(params), w8a16_relations);
}

rt::OperatorSchema make_matmul_pack_b_schema() {
  using rt::dtype_bit;
  std::vector<rt::ParameterSchema> params;
  params.push_back(tensor_param("b", dtype_bit(DType::BFloat16) | dtype_bit(DType::Float16) | dtype_bit(DType::Float32) |
                                       dtype_bit(DType::Int8) | dtype_bit(DType::UInt8), 2u, VECOPS_TENSOR_READ));
  params.push_back(rt::ParameterSchema{"a_zero_point", rt::ScalarConstraint{dtype_bit(DType::Int64) | dtype_bit(DType::Int32)}});
  params.push_back(tensor_param("packed", dtype_bit(DType::UInt8), 1u, VECOPS_TENSOR_WRITE));
  params.push_back(tensor_param("compensation", dtype_bit(DType::Int32), 1u, VECOPS_TENSOR_WRITE, /*optional=*/true));
  return rt::OperatorSchema(kMatmulPackBName, std::move(params), pack_b_relations);
}

rt::OperatorSchema make_matmul_packed_b_schema() {
  using rt::dtype_bit;
  const std::uint64_t in = dtype_bit(DType::BFloat16) | dtype_bit(DType::Float16) | dtype_bit(DType::Float32) |
                           dtype_bit(DType::Int8) | dtype_bit(DType::UInt8);
  const std::uint64_t out = dtype_bit(DType::BFloat16) | dtype_bit(DType::Float16) | dtype_bit(DType::Float32) |
                            dtype_bit(DType::Int32);
  std::vector<rt::ParameterSchema> params;
  params.push_back(tensor_param("a", in, std::nullopt, VECOPS_TENSOR_READ));
  params.push_back(tensor_param("packed_b", dtype_bit(DType::UInt8), 1u, VECOPS_TENSOR_READ));
  params.push_back(tensor_param("c_in", out, std::nullopt, VECOPS_TENSOR_READ, /*optional=*/true));
  params.push_back(tensor_param("c", out, std::nullopt, VECOPS_TENSOR_WRITE));
  return rt::OperatorSchema(kMatmulPackedBName, std::move(params), packed_b_relations);
}

rt::OperatorSchema make_matmul_pack_a_schema() {
  using rt::dtype_bit;
  std::vector<rt::ParameterSchema> params;
  params.push_back(tensor_param("a", dtype_bit(DType::BFloat16) | dtype_bit(DType::Float16) | dtype_bit(DType::Float32) |
                                       dtype_bit(DType::Int8) | dtype_bit(DType::UInt8), 2u, VECOPS_TENSOR_READ));
  params.push_back(tensor_param("packed", dtype_bit(DType::UInt8), 1u, VECOPS_TENSOR_WRITE));
  return rt::OperatorSchema(kMatmulPackAName, std::move(params), pack_a_relations);
}

rt::OperatorSchema make_matmul_packed_a_schema() {
  using rt::dtype_bit;
  const std::uint64_t in = dtype_bit(DType::BFloat16) | dtype_bit(DType::Float16) | dtype_bit(DType::Float32) |
                           dtype_bit(DType::Int8) | dtype_bit(DType::UInt8);
  const std::uint64_t out = dtype_bit(DType::BFloat16) | dtype_bit(DType::Float16) | dtype_bit(DType::Float32) |
                            dtype_bit(DType::Int32);
  std::vector<rt::ParameterSchema> params;
  params.push_back(tensor_param("packed_a", dtype_bit(DType::UInt8), 1u, VECOPS_TENSOR_READ));
  params.push_back(tensor_param("b", in, std::nullopt, VECOPS_TENSOR_READ));
  params.push_back(tensor_param("c_in", out, std::nullopt, VECOPS_TENSOR_READ, /*optional=*/true));
  params.push_back(tensor_param("c", out, std::nullopt, VECOPS_TENSOR_WRITE));
  return rt::OperatorSchema(kMatmulPackedAName, std::move(params), packed_a_relations);
}

rt::OperatorSchema make_matmul_runtime_quant_schema() {
  using rt::dtype_bit;
  std::vector<rt::ParameterSchema> params;
  params.push_back(tensor_param("a", dtype_bit(DType::Float32), 2u, VECOPS_TENSOR_READ));
  params.push_back(tensor_param("b", dtype_bit(DType::Int8), 2u, VECOPS_TENSOR_READ));
  params.push_back(tensor_param("multipliers", dtype_bit(DType::Float32), 1u, VECOPS_TENSOR_READ));
  params.push_back(rt::ParameterSchema{"zero_point", rt::ScalarConstraint{dtype_bit(DType::Int64) | dtype_bit(DType::Int32)}});
  params.push_back(tensor_param("row_scales", dtype_bit(DType::Float32), 1u, VECOPS_TENSOR_READ));
  params.push_back(tensor_param("column_scales", dtype_bit(DType::Float32), 1u, VECOPS_TENSOR_READ));
  params.push_back(tensor_param("correction", dtype_bit(DType::Int32), 1u, VECOPS_TENSOR_READ, /*optional=*/true));
  params.push_back(tensor_param("c", dtype_bit(DType::Float32), 2u, VECOPS_TENSOR_WRITE));
  return rt::OperatorSchema(kMatmulRuntimeQuantName, std::move(params), runtime_quant_relations);
}

// ---- recipes ------------------------------------------------------------------------------------

// Operand dtypes of a class: the 8-bit integer class takes signed and unsigned
// bytes on either side (AMX_I8I32<A, B>, matmul/details/kernel/amx/Atoms.h:73-86).
static bool takes(OperandClass operands, DType dtype) {
  switch (operands) {
    case OperandClass::BF16: return dtype == DType::BFloat16;
    case OperandClass::F16: return dtype == DType::Float16;
    case OperandClass::F32: return dtype == DType::Float32;
    default: return dtype == DType::Int8 || dtype == DType::UInt8;
  }
}

MatmulRecipe::MatmulRecipe(OperandClass operands) : operands_(operands) {
  id_ = operands == OperandClass::BF16 ? "hip.matmul.bf16.tile"
        : operands == OperandClass::F16 ? "hip.matmul.f16.tile"
        : operands == OperandClass::F32 ? "hip.matmul.f32.tile"
                                        : "hip.matmul.i8.tile";
}

Status MatmulRecipe::match(const rt::KernelCall& call) const {
  const auto values = call.arguments().values();
  const TensorView* a = tensor_at(values, 0);
  const TensorView* b = tensor_at(values, 1);
  const TensorView* cin = tensor_at(values, 2);
  const TensorView* c = tensor_at(values, 3);
  if (a == nullptr || b == nullptr || c == nullptr) return invalid("vecops::matmul needs a, b and c tensors");
  if (!takes(operands_, a->dtype) || !takes(operands_, b->dtype))
    return not_applicable("operand dtypes belong to another recipe");
  const bool int_out = operands_ == OperandClass::I8;
  // floating sums leave as fp32 or in the operands' own 16-bit type (fp32 operands: bf16)
  const DType narrow = operands_ == OperandClass::F16 ? DType::Float16 : DType::BFloat16;
  if (int_out ? c->dtype != DType::Int32 : (c->dtype != DType::Float32 && c->dtype != narrow))
    return not_applicable("output dtype does not fit these operands");
  if (cin != nullptr && (int_out ? cin->dtype != DType::Int32 : (cin->dtype != DType::Float32 && cin->dtype != narrow)))
    return not_applicable("c_in dtype does not fit these operands");
  auto compute = compute_type(call);
  if (!compute) return compute.status();
  if (operands_ == OperandClass::F32) {
    // fp32 memory: bf16 compute (what vecops' x86 path does, AMX_BF16F32 on converted operands) or
    // fp32 compute (the SME_F32F32 atom, matmul/details/kernel/sme/Atoms.h:65-76)
    if (compute.value() != DType::BFloat16 && compute.value() != DType::Float32)
      return not_applicable("ComputeType must be BFloat16 or Float32 for fp32 operands");
  } else if (operands_ == OperandClass::BF16 && compute.value() != DType::BFloat16) {
    return not_applicable("bf16 operands are multiplied in bf16");
  } else if (operands_ == OperandClass::F16 && compute.value() != DType::BFloat16 && compute.value() != DType::Float16) {
    return not_applicable("half operands are multiplied in half");  // (BFloat16 is the default of an absent ComputeType)
  }
  auto family = required_family(call);
  if (!family) return family.status();
  // artifacts that require a family exist for the bf16 and the 8-bit integer class
  if (!family.value().empty() && operands_ != OperandClass::BF16 && operands_ != OperandClass::I8)
    return not_applicable("a required kernel family is served for bf16 and 8-bit integer operands");
  auto place = placement_of(call);
  if (!place) return place.status();
  return Status::success();
}

rt::Result<rt::BoundKernelRecipe> MatmulRecipe::bind(const rt::KernelCall& call) const {
  if (Status st = match(call); !st.ok()) return st;
  const Placement place = placement_of(call).value();
  const char* operands = operands_ == OperandClass::BF16 ? "bf16" : operands_ == OperandClass::F16 ? "f16"
                         : operands_ == OperandClass::F32 ? "f32" : "i8";
  const bool f32_compute = operands_ == OperandClass::F32 && compute_type(call).value() == DType::Float32;
  const char* compute = operands_ == OperandClass::I8 ? "i32" : operands_ == OperandClass::F16 ? "f16"
                        : f32_compute ? "f32" : "bf16";
  rt::BoundKernelRecipe bound;
  bound.recipe_id = id_;
  const std::string family = required_family(call).value();
  bound.specialization_key = std::string(kMatmulName) + ";operands=" + operands + ";compute=" + compute +
                             (family.empty() ? std::string() : ";family=" + family) +
                             ";memory=" + placement_name(place) + ";" + kBackend;
  bound.artifact_key = id_ + ";" + bound.specialization_key;
  return bound;
}

Status MatmulI8DequantRecipe::match(const rt::KernelCall& call) const {
  auto place = placement_of(call);
  if (!place) return place.status();
  const auto values = call.arguments().values();
  for (std::size_t i : {std::size_t{0}, std::size_t{1}, std::size_t{5}}) {
    const TensorView* t = tensor_at(values, i);
    if (t == nullptr) return invalid("vecops::matmul_i8_dequant needs a, b and c tensors");
    if (t->strides.size() != 2 || (t->sizes[1] > 1 && t->strides[1] != 1))
      return not_applicable("a, b and c must be contiguous along their last axis");
  }
  return Status::success();
}

rt::Result<rt::BoundKernelRecipe> MatmulI8DequantRecipe::bind(const rt::KernelCall& call) const {
  if (Status st = match(call); !st.ok()) return st;
  rt::BoundKernelRecipe bound;
  bound.recipe_id = std::string(id());
  bound.specialization_key = std::string(kMatmulI8DequantName) + ";operands=i8;epilogue=row_col_dequant;memory=" +
                             placement_name(placement_of(call).value()) + ";" + kBackend;
  bound.artifact_key = bound.recipe_id + ";" + bound.specialization_key;
  return bound;
}

MatmulFusedRecipe::MatmulFusedRecipe(OperandClass operands) : operands_(operands) {
  id_ = operands == OperandClass::BF16 ? "hip.matmul_fused.bf16.tile"
        : operands == OperandClass::F16 ? "hip.matmul_fused.f16.tile"
        : operands == OperandClass::F32 ? "hip.matmul_fused.f32.tile"
                                        : "hip.matmul_fused.i8.tile";
}

Status MatmulFusedRecipe::match(const rt::KernelCall& call) const {
  const auto values = call.arguments().values();
  const TensorView* a = tensor_at(values, 0);
  const TensorView* b = tensor_at(values, 1);
  const TensorView* cin = tensor_at(values, 2);
  const TensorView* c = tensor_at(values, 10);
  if (a == nullptr || b == nullptr || c == nullptr) return invalid("vecops::matmul_fused needs a, b and c tensors");
  if (!takes(operands_, a->dtype) || !takes(operands_, b->dtype))
    return not_applicable("operand dtypes belong to another recipe");
  // int32 sums leave as fp32 or as requantised bytes; floating sums as fp32 or bf16
  const bool integer = operands_ == OperandClass::I8;
  const DType narrow = operands_ == OperandClass::F16 ? DType::Float16 : DType::BFloat16;
  const bool out_ok = integer ? (c->dtype == DType::Float32 || c->dtype == DType::UInt8 || c->dtype == DType::Int8)
                              : (c->dtype == DType::Float32 || c->dtype == narrow);
  if (!out_ok) return not_applicable("output dtype does not fit these operands");
  if (cin != nullptr && (integer ? cin->dtype != DType::Int32 : (cin->dtype != DType::Float32 && cin->dtype != narrow)))
    return not_applicable("c_in dtype does not fit these operands");
  auto place = placement_of(call);
  if (!place) return place.status();
  return Status::success();
}

rt::Result<rt::BoundKernelRecipe> MatmulFusedRecipe::bind(const rt::KernelCall& call) const {
  if (Status st = match(call); !st.ok()) return st;
  const char* operands = operands_ == OperandClass::BF16 ? "bf16" : operands_ == OperandClass::F16 ? "f16"
                         : operands_ == OperandClass::F32 ? "f32" : "i8";
  rt::BoundKernelRecipe bound;
  bound.recipe_id = id_;
  bound.specialization_key = std::string(kMatmulFusedName) + ";operands=" + operands + ";memory=" +
                             placement_name(placement_of(call).value()) + ";" + kBackend;
  bound.artifact_key = id_ + ";" + bound.specialization_key;
  return bound;
}

Status MatmulW8A16GroupRecipe::match(const rt::KernelCall& call) const {
  auto place = placement_of(call);
  if (!place) return place.status();
  auto g = group_size(call);
  if (!g) return g.status();
  const auto values = call.arguments().values();
  const TensorView* x = tensor_at(values, 0);
  const TensorView* w = tensor_at(values, 1);
  const TensorView* s = tensor_at(values, 2);
  if (x == nullptr || w == nullptr || s == nullptr) return invalid("vecops::matmul_w8a16_group needs x, w and scales");
  if (g.value() <= 0 || g.value() % 16 != 0) return invalid("G must be a positive multiple of 16");
  if (x->sizes[1] % g.value() != 0) return invalid("K must be a multiple of G");
  if (s->sizes[1] != x->sizes[1] / g.value()) return invalid("scales must be [N, K/G]");
  if (x->sizes[0] > 16) return not_applicable("the skinny family takes at most 16 activation rows");
  return Status::success();
}

rt::Result<rt::BoundKernelRecipe> MatmulW8A16GroupRecipe::bind(const rt::KernelCall& call) const {
  if (Status st = match(call); !st.ok()) return st;
  rt::BoundKernelRecipe bound;
  bound.recipe_id = std::string(id());
  bound.specialization_key = std::string(kMatmulW8A16GroupName) + ";G=" + std::to_string(group_size(call).value()) +
                             ";memory=" + placement_name(placement_of(call).value()) + ";" + kBackend;
  bound.artifact_key = bound.recipe_id + ";" + bound.specialization_key;
  return bound;
}

namespace {
const char* class_name(OperandClass c) {
  switch (c) {
    case OperandClass::BF16: return "bf16";
    case OperandClass::F16: return "f16";
    case OperandClass::F32: return "f32";
    case OperandClass::I8: return "i8";
    case OperandClass::U8: return "u8";
  }
  return "";
}
}  // namespace

MatmulPackBRecipe::MatmulPackBRecipe(OperandClass packed, PackSide side) : packed_(packed), side_(side) {
  id_ = std::string(side == PackSide::A ? "hip.matmul_pack_a." : "hip.matmul_pack_b.") + class_name(packed);
}

Status MatmulPackBRecipe::match(const rt::KernelCall& call) const {
  const auto values = call.arguments().values();
  const TensorView* src = tensor_at(values, 0);
  if (src == nullptr) return invalid(std::string(side_ == PackSide::A ? kMatmulPackAName : kMatmulPackBName) + " needs a source tensor");
  auto compute = compute_type(call);
  if (!compute) return compute.status();
  const bool keep_f32 = src->dtype == DType::Float32 && compute.value() == DType::Float32;  // the fp32-compute atom's pack
  const bool mine = packed_ == OperandClass::I8    ? src->dtype == DType::Int8
                    : packed_ == OperandClass::U8  ? src->dtype == DType::UInt8
                    : packed_ == OperandClass::F16 ? src->dtype == DType::Float16
                    : packed_ == OperandClass::F32 ? keep_f32
                                                   : (src->dtype == DType::BFloat16 || (src->dtype == DType::Float32 && !keep_f32));
  if (!mine) return not_applicable("source dtype belongs to another recipe");
  auto place = placement_of(call);
  if (!place) return place.status();
  return Status::success();
}

rt::Result<rt::BoundKernelRecipe> MatmulPackBRecipe::bind(const rt::KernelCall& call) const {
  if (Status st = match(call); !st.ok()) return st;
  rt::BoundKernelRecipe bound;
  bound.recipe_id = id_;
  bound.specialization_key = std::string(side_ == PackSide::A ? kMatmulPackAName : kMatmulPackBName) + ";operands=" +
                             class_name(packed_) + ";memory=" + placement_name(placement_of(call).value()) + ";" + kBackend;
  bound.artifact_key = id_ + ";" + bound.specialization_key;
  return bound;
}

MatmulPackedBRecipe::MatmulPackedBRecipe(OperandClass operands, PackSide side, bool packed_unsigned, bool f32_compute)
  : operands_(operands), side_(side), packed_unsigned_(packed_unsigned), f32_compute_(f32_compute) {
  id_ = std::string(side == PackSide::A ? "hip.matmul_packed_a." : "hip.matmul_packed_b.") + class_name(operands) +
        (packed_unsigned ? ".packed_u8" : "") + (f32_compute ? ".f32_compute" : "") + ".tile";
}

Status MatmulPackedBRecipe::match(const rt::KernelCall& call) const {
  const auto values = call.arguments().values();
  const char* op = side_ == PackSide::A ? kMatmulPackedAName : kMatmulPackedBName;
  const TensorView* dense = tensor_at(values, side_ == PackSide::A ? 1 : 0);
  const TensorView* cin = tensor_at(values, 2);
  const TensorView* c = tensor_at(values, 3);
  if (dense == nullptr || c == nullptr) return invalid(std::string(op) + " needs its dense operand and c");
  const bool mine = operands_ == OperandClass::I8 ? (dense->dtype == DType::Int8 || dense->dtype == DType::UInt8)
                    : operands_ == OperandClass::F32 ? dense->dtype == DType::Float32
                    : operands_ == OperandClass::F16 ? dense->dtype == DType::Float16
                                                     : dense->dtype == DType::BFloat16;
  if (!mine) return not_applicable("operand dtype belongs to another recipe");
  auto unsigned_pack = packed_is_unsigned(call);
  if (!unsigned_pack) return unsigned_pack.status();
  if (unsigned_pack.value() && operands_ != OperandClass::I8) return invalid("PackedType UInt8 goes with 8-bit integer operands");
  if (unsigned_pack.value() != packed_unsigned_) return not_applicable("the packed operand's signedness belongs to another recipe");
  auto compute = compute_type(call);
  if (!compute) return compute.status();
  const bool wants_f32 = operands_ == OperandClass::F32 && compute.value() == DType::Float32;
  if (wants_f32 != f32_compute_) return not_applicable("the compute type belongs to another recipe");
  if (f32_compute_ && c->dtype != DType::Float32) return not_applicable("fp32 products leave as fp32");
  const bool int_out = operands_ == OperandClass::I8;
  const DType narrow = operands_ == OperandClass::F16 ? DType::Float16 : DType::BFloat16;  // the operands' own 16-bit type
  if (int_out ? c->dtype != DType::Int32 : (c->dtype != DType::Float32 && c->dtype != narrow))
    return not_applicable("output dtype does not fit these operands");
  if (cin != nullptr && (int_out ? cin->dtype != DType::Int32 : (cin->dtype != DType::Float32 && cin->dtype != narrow)))
    return not_applicable("c_in dtype does not fit these operands");
  auto place = placement_of(call);
  if (!place) return place.status();
  return Status::success();
}

rt::Result<rt::BoundKernelRecipe> MatmulPackedBRecipe::bind(const rt::KernelCall& call) const {
  if (Status st = match(call); !st.ok()) return st;
  rt::BoundKernelRecipe bound;
  bound.recipe_id = id_;
  bound.specialization_key = std::string(side_ == PackSide::A ? kMatmulPackedAName : kMatmulPackedBName) + ";operands=" +
                             class_name(operands_) + (packed_unsigned_ ? ";packed=u8" : "") +
                             (f32_compute_ ? ";compute=f32" : "") + ";memory=" +
                             placement_name(placement_of(call).value()) + ";" + kBackend;
  bound.artifact_key = id_ + ";" + bound.specialization_key;
  return bound;
}

Status MatmulRuntimeQuantRecipe::match(const rt::KernelCall& call) const {
  auto place = placement_of(call);
  if (!place) return place.status();
  const auto values = call.arguments().values();
  for (std::size_t i : {std::size_t{2}, std::size_t{4}, std::size_t{5}, std::size_t{6}}) {
    const TensorView* t = tensor_at(values, i);
    if (t != nullptr && t->sizes[0] > 1 && t->strides[0] != 1) return not_applicable("the vectors must be contiguous");
  }
  return Status::success();
}

rt::Result<rt::BoundKernelRecipe> MatmulRuntimeQuantRecipe::bind(const rt::KernelCall& call) const {
  if (Status st = match(call); !st.ok()) return st;
  rt::BoundKernelRecipe bound;
  bound.recipe_id = std::string(id());
  bound.specialization_key = std::string(kMatmulRuntimeQuantName) + ";operands=f32_i8;epilogue=row_col_dequant;memory=" +
                             placement_name(placement_of(call).value()) + ";" + kBackend;
  bound.artifact_key = bound.recipe_id + ";" + bound.specialization_key;
  return bound;
}

// ---- dispatch policy --------------------------------------------------------------------------------

rt::Result<std::vector<std::size_t>>
MatmulDispatchPolicy::candidates(const rt::KernelCall& call,
                                 std::span<const std::shared_ptr<const rt::KernelRecipe>> recipes) const {
  std::vector<std::size_t> order;
  const auto values = call.arguments().values();
  const TensorView* a = tensor_at(values, 0);
  for (std::size_t i = 0; i < recipes.size(); ++i) {
    if (recipes[i] == nullptr) continue;
    if (const auto* mm = dynamic_cast<const MatmulRecipe*>(recipes[i].get()); mm != nullptr && a != nullptr) {
      if (!takes(mm->operands(), a->dtype)) continue;
    }
    if (const auto* mf = dynamic_cast<const MatmulFusedRecipe*>(recipes[i].get()); mf != nullptr && a != nullptr) {
      if (!takes(mf->operands(), a->dtype)) continue;
    }
    if (const auto* mp = dynamic_cast<const MatmulPackedBRecipe*>(recipes[i].get()); mp != nullptr) {
      const TensorView* dense = tensor_at(values, mp->side() == PackSide::A ? 1 : 0);   // (packed_a, b, ..) / (a, packed_b, ..)
      if (dense != nullptr &&
          (mp->operands() == OperandClass::I8 ? (dense->dtype != DType::Int8 && dense->dtype != DType::UInt8)
           : mp->operands() == OperandClass::F32 ? dense->dtype != DType::Float32
           : mp->operands() == OperandClass::F16 ? dense->dtype != DType::Float16
                                                 : dense->dtype != DType::BFloat16)) continue;
    }
    if (const auto* pk = dynamic_cast<const MatmulPackBRecipe*>(recipes[i].get()); pk != nullptr && a != nullptr) {
      if ((pk->operands() == OperandClass::I8) != (a->dtype == DType::Int8) ||
          (pk->operands() == OperandClass::U8) != (a->dtype == DType::UInt8) ||
          (pk->operands() == OperandClass::F16) != (a->dtype == DType::Float16) ||
          (pk->operands() == OperandClass::F32 && a->dtype != DType::Float32)) continue;   // (fp32: match() reads ComputeType)
    }
    order.push_back(i);
  }
  if (order.empty())
    return Status(StatusCode::NotFound, "no recipe of this operator takes operands of this dtype");
  return order;
}

// ---- provider -----------------------------------------------------------------------------------------

std::string artifact_file_name(std::string_view key) {
  std::string name;
  name.reserve(key.size() + 3);
  for (const char ch : key) {
    const bool keep = (ch >= 'A' && ch <= 'Z') || (ch >= 'a' && ch <= 'z') || (ch >= '0' && ch <= '9') || ch == '_' ||
                      ch == '.' || ch == '=' || ch == '-';
    name.push_back(keep ? ch : '_');
  }
  return name + ".so";
}

HipExecutableProvider::HipExecutableProvider(std::filesystem::path artifact_directory)
  : directory_(std::move(artifact_directory)) {}

std::filesystem::path HipExecutableProvider::artifact_path(std::string_view specialization_key) const {
  return directory_ / artifact_file_name(specialization_key);
}

std::size_t HipExecutableProvider::loads() const {
  std::lock_guard<std::mutex> lock(mutex_);
  return loads_;
}

rt::Result<std::shared_ptr<rt::Executable>> HipExecutableProvider::resolve(const rt::BoundKernelRecipe& recipe) {
  const std::string& key = recipe.specialization_key;
  std::shared_ptr<Pending> mine;
  {
    std::unique_lock<std::mutex> lock(mutex_);
    for (;;) {
      if (auto it = loaded_.find(key); it != loaded_.end()) return it->second;
      auto waiting = pending_.find(key);
      if (waiting == pending_.end()) break;
      auto other = waiting->second;  // another thread is loading this key: wait for it
      other->ready.wait(lock, [&] { return other->done; });
    }
    mine = std::make_shared<Pending>();
    pending_.emplace(key, mine);
  }
  auto finish = [&](std::shared_ptr<rt::Executable> executable) {
    std::lock_guard<std::mutex> lock(mutex_);
    if (executable != nullptr) {
      loaded_.emplace(key, std::move(executable));
      ++loads_;
    }
    pending_.erase(key);
    mine->done = true;
    mine->ready.notify_all();
  };
  const std::filesystem::path path = artifact_path(key);
  std::error_code ec;
  if (!std::filesystem::exists(path, ec)) {
    finish(nullptr);
    return Status(StatusCode::NotFound, "no HIP artifact for " + key + " (expected " + path.string() + ")");
  }
  auto executable = rt::Executable::load(path);
  if (!executable) {
    finish(nullptr);
    return executable.status();
  }
  if (executable.value()->specialization_key() != key) {
    finish(nullptr);
    return Status(StatusCode::AbiMismatch, path.string() + " carries specialization key '" +
                                             std::string(executable.value()->specialization_key()) + "', wanted '" +
                                             key + "'");
  }
  finish(executable.value());
  return executable;
}

// ---- operators ---------------------------------------------------------------------------------------------

std::shared_ptr<rt::Operator> make_matmul_operator(const std::filesystem::path& dir) {
  return assemble(make_matmul_schema(),
                  {std::make_shared<MatmulRecipe>(OperandClass::BF16), std::make_shared<MatmulRecipe>(OperandClass::F16),
                   std::make_shared<MatmulRecipe>(OperandClass::F32), std::make_shared<MatmulRecipe>(OperandClass::I8)},
                  dir);
}

std::shared_ptr<rt::Operator> make_matmul_i8_dequant_operator(const std::filesystem::path& dir) {
  return assemble(make_matmul_i8_dequant_schema(), {std::make_shared<MatmulI8DequantRecipe>()}, dir);
}

std::shared_ptr<rt::Operator> make_matmul_fused_operator(const std::filesystem::path& dir) {
  return assemble(make_matmul_fused_schema(),
                  {std::make_shared<MatmulFusedRecipe>(OperandClass::BF16),
                   std::make_shared<MatmulFusedRecipe>(OperandClass::F16),
                   std::make_shared<MatmulFusedRecipe>(OperandClass::F32),
                   std::make_shared<MatmulFusedRecipe>(OperandClass::I8)},
                  dir);
}

std::shared_ptr<rt::Operator> make_matmul_pack_b_operator(const std::filesystem::path& dir) {
  return assemble(make_matmul_pack_b_schema(),
                  {std::make_shared<MatmulPackBRecipe>(OperandClass::BF16), std::make_shared<MatmulPackBRecipe>(OperandClass::F16),
                   std::make_shared<MatmulPackBRecipe>(OperandClass::I8), std::make_shared<MatmulPackBRecipe>(OperandClass::U8),
                   std::make_shared<MatmulPackBRecipe>(OperandClass::F32)},
                  dir);
}

std::shared_ptr<rt::Operator> make_matmul_pack_a_operator(const std::filesystem::path& dir) {
  return assemble(make_matmul_pack_a_schema(),
                  {std::make_shared<MatmulPackBRecipe>(OperandClass::BF16, PackSide::A),
                   std::make_shared<MatmulPackBRecipe>(OperandClass::F16, PackSide::A),
                   std::make_shared<MatmulPackBRecipe>(OperandClass::I8, PackSide::A),
                   std::make_shared<MatmulPackBRecipe>(OperandClass::U8, PackSide::A),
                   std::make_shared<MatmulPackBRecipe>(OperandClass::F32, PackSide::A)},
                  dir);
}

std::shared_ptr<rt::Operator> make_matmul_packed_a_operator(const std::filesystem::path& dir) {
  return assemble(make_matmul_packed_a_schema(),
                  {std::make_shared<MatmulPackedBRecipe>(OperandClass::BF16, PackSide::A),
                   std::make_shared<MatmulPackedBRecipe>(OperandClass::F16, PackSide::A),
                   std::make_shared<MatmulPackedBRecipe>(OperandClass::F32, PackSide::A),
                   std::make_shared<MatmulPackedBRecipe>(OperandClass::I8, PackSide::A),
                   std::make_shared<MatmulPackedBRecipe>(OperandClass::I8, PackSide::A, /*packed_unsigned=*/true),
                   std::make_shared<MatmulPackedBRecipe>(OperandClass::F32, PackSide::A, false, /*f32_compute=*/true)},
                  dir);
}

std::shared_ptr<rt::Operator> make_matmul_packed_b_operator(const std::filesystem::path& dir) {
  return assemble(make_matmul_packed_b_schema(),
                  {std::make_shared<MatmulPackedBRecipe>(OperandClass::BF16),
                   std::make_shared<MatmulPackedBRecipe>(OperandClass::F16),
                   std::make_shared<MatmulPackedBRecipe>(OperandClass::F32),
                   std::make_shared<MatmulPackedBRecipe>(OperandClass::I8),
                   std::make_shared<MatmulPackedBRecipe>(OperandClass::I8, PackSide::B, /*packed_unsigned=*/true),
                   std::make_shared<MatmulPackedBRecipe>(OperandClass::F32, PackSide::B, false, /*f32_compute=*/true)},
                  dir);
}

std::shared_ptr<rt::Operator> make_matmul_runtime_quant_operator(const std::filesystem::path& dir) {
  return assemble(make_matmul_runtime_quant_schema(), {std::make_shared<MatmulRuntimeQuantRecipe>()}, dir);
}

std::shared_ptr<rt::Operator> make_matmul_w8a16_group_operator(const std::filesystem::path& dir) {
  return assemble(make_matmul_w8a16_group_schema(), {std::make_shared<MatmulW8A16GroupRecipe>()}, dir);
}

}  // namespace vecops::hip
