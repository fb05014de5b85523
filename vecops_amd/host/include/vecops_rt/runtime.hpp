// The vecops runtime plug-in surface, restated so the HIP provider of this
// repository builds and is testable without the vecops tree:
//
//   OperatorSchema -> Operator / DispatchPolicy -> KernelRecipe
//                  -> ExecutableProvider -> Executable (a loaded artifact DSO)
//
// Type names, member names, signatures and observable behaviour (status codes,
// validation order, what is checked before a DSO callback is entered) follow
// vecops' include/vecops/runtime/{Status,Argument,Schema,KernelDefinition,
// Operator,Executable}.h and src/runtime/{Schema,Argument,Operator,Executable}.cpp;
// each class cites the lines it mirrors.  Code written against this header (the
// recipes, dispatch policy and provider under vecops_amd/host/hip) compiles
// unchanged against the vecops headers: define VECOPS_HIP_USE_UPSTREAM_RUNTIME
// and put the vecops include directory on the path (see vecops_rt/surface.hpp).
//
// Not restated: KernelDef / bind_kernel_call / SourceKernelRecipe /
// ArtifactExecutableProvider, which exist to compile `__kernel__` C++ sources
// with a host compiler; the HIP artifacts are built ahead of time.
#ifndef VECOPS_RT_RUNTIME_HPP
#define VECOPS_RT_RUNTIME_HPP

#include <cstdint>
#include <filesystem>
#include <functional>
#include <map>
#include <memory>
#include <optional>
#include <span>
#include <string>
#include <string_view>
#include <utility>
#include <variant>
#include <vector>

#include "vecops_rt/abi.h"

namespace vecops {
using nint_t = std::int64_t;  // vecops CoreTypes.h: the library-wide signed extent type
}

namespace vecops::runtime {

// ---- Status / Result (runtime/Status.h:23-146) --------------------------------------------------

enum class StatusCode : int {
  Ok = VECOPS_STATUS_OK,
  InvalidArgument = VECOPS_STATUS_INVALID_ARGUMENT,
  NotApplicable = VECOPS_STATUS_NOT_APPLICABLE,
  NotFound = VECOPS_STATUS_NOT_FOUND,
  AbiMismatch = VECOPS_STATUS_ABI_MISMATCH,
  LoadError = VECOPS_STATUS_LOAD_ERROR,
  ExecutionError = VECOPS_STATUS_EXECUTION_ERROR,
  InternalError = VECOPS_STATUS_INTERNAL_ERROR,
};

class Status {
public:
  Status() = default;
  Status(StatusCode code, std::string message) : code_(code), message_(std::move(message)) {}
  static Status success() { return {}; }
  [[nodiscard]] bool ok() const { return code_ == StatusCode::Ok; }
  [[nodiscard]] StatusCode code() const { return code_; }
  [[nodiscard]] const std::string& message() const { return message_; }

private:
  StatusCode code_ = StatusCode::Ok;
  std::string message_;
};

// A value or the failure that prevented it.  Constructing one from a success
// status is a caller bug and is turned into InternalError.
template <typename T>
class Result {
public:
  Result(T value) : value_(std::move(value)) {}
  Result(Status status)
    : status_(status.ok() ? Status(StatusCode::InternalError, "a value-less Result cannot contain success")
                          : std::move(status)) {}
  [[nodiscard]] bool ok() const { return value_.has_value(); }
  [[nodiscard]] explicit operator bool() const { return ok(); }
  [[nodiscard]] const Status& status() const {
    static const Status success_status;
    return ok() ? success_status : status_;
  }
  [[nodiscard]] T& value() & { return *value_; }
  [[nodiscard]] const T& value() const& { return *value_; }
  [[nodiscard]] T&& value() && { return std::move(*value_); }

private:
  std::optional<T> value_;
  Status status_;
};

// ---- Argument metadata (runtime/Argument.h:33-330, src/runtime/Argument.cpp) -----------------------

enum class DType : std::uint32_t {
  Invalid = VECOPS_DTYPE_INVALID,
  Bool = VECOPS_DTYPE_BOOL,
  Int8 = VECOPS_DTYPE_I8,
  UInt8 = VECOPS_DTYPE_U8,
  Int16 = VECOPS_DTYPE_I16,
  UInt16 = VECOPS_DTYPE_U16,
  Int32 = VECOPS_DTYPE_I32,
  UInt32 = VECOPS_DTYPE_U32,
  Int64 = VECOPS_DTYPE_I64,
  UInt64 = VECOPS_DTYPE_U64,
  Float16 = VECOPS_DTYPE_F16,
  BFloat16 = VECOPS_DTYPE_BF16,
  Float32 = VECOPS_DTYPE_F32,
  Float64 = VECOPS_DTYPE_F64,
};

// Mask bit of one dtype: bit (dtype - 1); zero for values outside Bool..Float64.
constexpr std::uint64_t dtype_bit(DType dtype) {
  const auto v = static_cast<std::uint32_t>(dtype);
  return (v < 1 || v > 13) ? 0 : (std::uint64_t{1} << (v - 1));
}
constexpr std::uint64_t all_dtypes() { return (std::uint64_t{1} << 13) - 1; }

struct TensorView {
  void* data = nullptr;
  std::uint64_t byte_offset = 0;
  std::uint32_t device_type = VECOPS_DEVICE_CPU;
  std::int32_t device_index = 0;
  DType dtype = DType::Invalid;
  std::vector<std::int64_t> sizes;
  std::vector<std::int64_t> strides;
  std::uint64_t flags = VECOPS_TENSOR_READ;
  [[nodiscard]] bool writable() const { return (flags & VECOPS_TENSOR_WRITE) != 0; }
};

struct Scalar {
  DType dtype = DType::Invalid;
  VecopsScalarStorage value{};
  static Scalar signed_integer(std::int64_t value, DType dtype = DType::Int64);
  static Scalar unsigned_integer(std::uint64_t value, DType dtype = DType::UInt64);
  static Scalar floating(double value, DType dtype = DType::Float64);
};

using Value = std::variant<std::monostate, TensorView, Scalar>;

class ArgumentMetadata {
public:
  ArgumentMetadata() = default;
  explicit ArgumentMetadata(std::vector<Value> values) : values_(std::move(values)) {}
  [[nodiscard]] std::span<const Value> values() const { return values_; }
  [[nodiscard]] std::span<Value> values() { return values_; }
  [[nodiscard]] std::size_t size() const { return values_.size(); }
  [[nodiscard]] const Value& operator[](std::size_t index) const { return values_[index]; }

private:
  std::vector<Value> values_;
};

// The C records of one call, built from (and borrowing the size/stride arrays
// of) an ArgumentMetadata that must outlive it.
class CallFrame {
public:
  explicit CallFrame(const ArgumentMetadata& arguments, void* workspace = nullptr, std::uint64_t workspace_size = 0,
                     const VecopsExecutionContext* context = nullptr);
  [[nodiscard]] const VecopsCall& abi() const { return call_; }

private:
  std::vector<VecopsValue> values_;
  VecopsCall call_{};
};

inline Value erase_value(Value value) { return value; }
inline Value erase_value(std::monostate value) { return value; }
inline Value erase_value(TensorView value) { return value; }
inline Value erase_value(Scalar value) { return value; }

template <typename... Values>
ArgumentMetadata make_arguments(Values&&... values) {
  std::vector<Value> erased;
  erased.reserve(sizeof...(Values));
  (erased.push_back(erase_value(std::forward<Values>(values))), ...);
  return ArgumentMetadata(std::move(erased));
}

// ---- Schema (runtime/Schema.h:27-188, src/runtime/Schema.cpp:26-147) ----------------------------------

struct DimensionConstraint {
  enum class Kind { Any, Const, Dynamic };
  Kind kind = Kind::Any;
  std::int64_t value = 0;
  std::int64_t lower_bound = 0;
  std::int64_t upper_bound = INT64_MAX;
  std::int64_t alignment = 1;
  static DimensionConstraint any();
  static DimensionConstraint constant(std::int64_t value);
  static DimensionConstraint dynamic(std::int64_t lower_bound = 0, std::int64_t upper_bound = INT64_MAX,
                                     std::int64_t alignment = 1);
  [[nodiscard]] bool accepts(std::int64_t candidate) const;
};

struct TensorConstraint {
  std::uint64_t dtype_mask = all_dtypes();
  std::uint32_t device_type = 0;   // 0 = any
  std::int32_t device_index = -1;  // -1 = any
  std::optional<std::uint32_t> rank;
  std::vector<DimensionConstraint> sizes;
  std::vector<DimensionConstraint> strides;
  std::uint64_t required_flags = VECOPS_TENSOR_READ;
  bool optional = false;
};

struct ScalarConstraint {
  std::uint64_t dtype_mask = all_dtypes();
};

struct ParameterSchema {
  std::string name;
  std::variant<TensorConstraint, ScalarConstraint> constraint;
};

class OperatorSchema {
public:
  using RelationValidator = std::function<Status(std::span<const Value>)>;
  OperatorSchema(std::string name, std::vector<ParameterSchema> parameters, RelationValidator relation_validator = {});
  [[nodiscard]] const std::string& name() const { return name_; }
  [[nodiscard]] std::span<const ParameterSchema> parameters() const { return parameters_; }
  // Count, kind, per-tensor constraints in positional order, then the relation validator.
  [[nodiscard]] Status validate(const ArgumentMetadata& arguments) const;

private:
  std::string name_;
  std::vector<ParameterSchema> parameters_;
  RelationValidator relation_validator_;
};

Status validate_tensor(const TensorView& tensor, const TensorConstraint& constraint, std::string_view parameter_name);

// ---- Calls with explicit specialization values (runtime/KernelDefinition.h:41-46,340-392) ----------------

using SpecializationValue = std::variant<std::int64_t, DType>;
using SpecializationValues = std::map<std::string, SpecializationValue, std::less<>>;

class KernelCall {
public:
  KernelCall() = default;
  explicit KernelCall(ArgumentMetadata arguments, SpecializationValues values = {})
    : arguments_(std::move(arguments)), values_(std::move(values)) {}
  template <typename... Values>
  static KernelCall from_values(SpecializationValues specialization_values, Values&&... values) {
    return KernelCall(make_arguments(std::forward<Values>(values)...), std::move(specialization_values));
  }
  [[nodiscard]] const ArgumentMetadata& arguments() const { return arguments_; }
  [[nodiscard]] const SpecializationValues& values() const { return values_; }

private:
  ArgumentMetadata arguments_;
  SpecializationValues values_;
};

// ---- Executable (runtime/Executable.h:36-169, src/runtime/Executable.cpp) ------------------------------

// One dlopen'ed artifact and its validated descriptor; unloads on destruction.
class LoadedModule {
public:
  ~LoadedModule();
  LoadedModule(const LoadedModule&) = delete;
  LoadedModule& operator=(const LoadedModule&) = delete;
  // LoadError when the DSO cannot be mapped, AbiMismatch when it lacks
  // vecops_kernel_query_v1 or its descriptor fails validation.
  static Result<std::shared_ptr<LoadedModule>> load(const std::filesystem::path& library_path);
  [[nodiscard]] const VecopsKernelDescriptorV1& descriptor() const { return *descriptor_; }
  [[nodiscard]] const std::filesystem::path& path() const { return path_; }

private:
  LoadedModule(std::filesystem::path path, void* handle, const VecopsKernelDescriptorV1* descriptor)
    : path_(std::move(path)), handle_(handle), descriptor_(descriptor) {}
  std::filesystem::path path_;
  void* handle_ = nullptr;
  const VecopsKernelDescriptorV1* descriptor_ = nullptr;
};

class Executable {
public:
  explicit Executable(std::shared_ptr<LoadedModule> module) : module_(std::move(module)) {}
  static Result<std::shared_ptr<Executable>> load(const std::filesystem::path& library_path);
  [[nodiscard]] std::string_view operator_name() const;
  [[nodiscard]] std::string_view specialization_key() const;
  [[nodiscard]] const std::shared_ptr<LoadedModule>& module() const { return module_; }
  // Arguments against the descriptor: count, optional, dtype mask, device, rank,
  // negative sizes, null data, access flags, size and stride constraints.
  [[nodiscard]] Status can_invoke(const ArgumentMetadata& arguments) const;
  [[nodiscard]] Result<std::uint64_t> workspace_size(const ArgumentMetadata& arguments,
                                                     const VecopsExecutionContext* context = nullptr) const;
  // can_invoke, workspace query, "required <= supplied", then the DSO's run callback.
  [[nodiscard]] Status invoke(const ArgumentMetadata& arguments, void* workspace = nullptr,
                              std::uint64_t workspace_size = 0, const VecopsExecutionContext* context = nullptr) const;
  [[nodiscard]] Status invoke_prevalidated(const VecopsCall& call) const;

private:
  [[nodiscard]] Status invoke_unchecked(const VecopsCall& call) const;
  std::shared_ptr<LoadedModule> module_;
};

// ---- Operator (runtime/Operator.h:34-293, src/runtime/Operator.cpp:157-285) ------------------------------

struct BoundKernelRecipe {
  std::string recipe_id;
  std::string specialization_key;
  std::string artifact_key;
  // Compiler input of source-backed recipes.  Ahead-of-time recipes leave `source`
  // null, which also keeps the runtime from appending a ";$Parallelism=i:P" suffix
  // to the keys (src/runtime/Operator.cpp:97-99).
  struct SourceInstantiation {
    std::filesystem::path kernel_file;
    nint_t parallelism = 1;
  };
  std::shared_ptr<const SourceInstantiation> source;
};

class KernelRecipe {
public:
  virtual ~KernelRecipe() = default;
  [[nodiscard]] virtual std::string_view id() const = 0;
  // Cheap, side-effect free, thread-safe: NotApplicable sends dispatch to the next recipe.
  [[nodiscard]] virtual Status match(const KernelCall& call) const = 0;
  [[nodiscard]] virtual Result<BoundKernelRecipe> bind(const KernelCall& call) const = 0;
};

class DispatchPolicy {
public:
  virtual ~DispatchPolicy() = default;
  [[nodiscard]] virtual Result<std::vector<std::size_t>>
  candidates(const KernelCall& call, std::span<const std::shared_ptr<const KernelRecipe>> recipes) const = 0;
};

class OrderedDispatchPolicy final : public DispatchPolicy {
public:
  [[nodiscard]] Result<std::vector<std::size_t>>
  candidates(const KernelCall& call, std::span<const std::shared_ptr<const KernelRecipe>> recipes) const override;
};

class ExecutableProvider {
public:
  virtual ~ExecutableProvider() = default;
  // May do I/O and load DSOs; the executable's key must equal the request's.
  [[nodiscard]] virtual Result<std::shared_ptr<Executable>> resolve(const BoundKernelRecipe& recipe) = 0;
};

class Operator {
public:
  Operator(OperatorSchema schema, std::vector<std::shared_ptr<const KernelRecipe>> recipes,
           std::shared_ptr<const DispatchPolicy> dispatch_policy, std::shared_ptr<ExecutableProvider> provider);
  [[nodiscard]] const OperatorSchema& schema() const { return schema_; }
  [[nodiscard]] Result<std::shared_ptr<Executable>> resolve(const ArgumentMetadata& arguments) const;
  [[nodiscard]] Result<std::shared_ptr<Executable>> resolve(const KernelCall& call,
                                                            const VecopsExecutionContext* context = nullptr) const;
  [[nodiscard]] Status invoke(const ArgumentMetadata& arguments, void* workspace = nullptr,
                              std::uint64_t workspace_size = 0, const VecopsExecutionContext* context = nullptr) const;
  [[nodiscard]] Status invoke(const KernelCall& call, const VecopsExecutionContext* context = nullptr,
                              void* workspace = nullptr, std::uint64_t workspace_size = 0) const;
  [[nodiscard]] Status operator()(const KernelCall& call) const { return invoke(call); }
  template <typename... Values>
  [[nodiscard]] Status invoke_values(Values&&... values) const {
    return invoke(make_arguments(std::forward<Values>(values)...));
  }

private:
  [[nodiscard]] Result<std::shared_ptr<Executable>> resolve_validated(const KernelCall& call) const;
  OperatorSchema schema_;
  std::vector<std::shared_ptr<const KernelRecipe>> recipes_;
  std::shared_ptr<const DispatchPolicy> dispatch_policy_;
  std::shared_ptr<ExecutableProvider> provider_;
};

}  // namespace vecops::runtime
#endif
