// Implementation of the restated vecops runtime surface (vecops_rt/runtime.hpp).
// Behaviour follows vecops src/runtime/{Argument,Schema,Executable,Operator}.cpp;
// the cited lines say which rule each block reproduces.
#include "vecops_rt/runtime.hpp"

#include <dlfcn.h>

#include <array>
#include <cstddef>
#include <limits>
#include <numeric>

namespace vecops::runtime {

namespace {

Status invalid(std::string message) { return Status(StatusCode::InvalidArgument, std::move(message)); }
Status abi_mismatch(std::string message) { return Status(StatusCode::AbiMismatch, std::move(message)); }

// Descriptor arrays are walked by their declared byte stride so that records
// appended to by a newer ABI minor still read correctly (Executable.cpp:27-33).
template <typename T>
const T& record_at(const T* first, std::uint32_t stride, std::size_t index) {
  return *reinterpret_cast<const T*>(reinterpret_cast<const std::byte*>(first) + std::size_t{stride} * index);
}

bool well_formed(const VecopsDimensionConstraint& c) {
  return c.struct_size >= sizeof(VecopsDimensionConstraint) && c.kind <= VECOPS_DIM_DYNAMIC &&
         !(c.kind == VECOPS_DIM_DYNAMIC && c.alignment <= 0);
}

// What a loader must verify before it trusts a descriptor (Executable.cpp:39-100).
Status check_descriptor(const VecopsKernelDescriptorV1* d) {
  if (d == nullptr) return abi_mismatch("kernel query returned a null descriptor");
  if (d->struct_size < sizeof(VecopsKernelDescriptorV1)) return abi_mismatch("kernel descriptor is smaller than ABI v1");
  if (d->abi_version_major != VECOPS_KERNEL_ABI_VERSION_MAJOR || d->abi_version_minor > VECOPS_KERNEL_ABI_VERSION_MINOR)
    return abi_mismatch("kernel ABI version is not supported by this runtime");
  if (d->operator_name == nullptr || d->specialization_key == nullptr)
    return abi_mismatch("kernel descriptor has no operator or specialization name");
  if (d->num_parameters != 0) {
    if (d->parameters == nullptr) return abi_mismatch("kernel descriptor has no parameter array");
    if (d->parameter_stride < sizeof(VecopsParameterDescriptor) ||
        d->parameter_stride % alignof(VecopsParameterDescriptor) != 0)
      return abi_mismatch("kernel has an invalid parameter stride");
  }
  if (d->run == nullptr) return abi_mismatch("kernel descriptor has no run entry point");
  for (std::uint32_t i = 0; i < d->num_parameters; ++i) {
    const auto& p = record_at(d->parameters, d->parameter_stride, i);
    if (p.struct_size < sizeof(VecopsParameterDescriptor) || p.name == nullptr)
      return abi_mismatch("kernel has an invalid parameter descriptor");
    if (p.kind == VECOPS_VALUE_SCALAR) {
      if (p.constraint.scalar.struct_size < sizeof(VecopsScalarParameter))
        return abi_mismatch("kernel has an invalid scalar constraint");
      continue;
    }
    if (p.kind != VECOPS_VALUE_TENSOR) return abi_mismatch("kernel parameter has an unknown value kind");
    const auto& t = p.constraint.tensor;
    const bool stride_ok = t.dimension_constraint_stride >= sizeof(VecopsDimensionConstraint) &&
                           t.dimension_constraint_stride % alignof(VecopsDimensionConstraint) == 0;
    if (t.struct_size < sizeof(VecopsTensorParameter) || t.rank < -1 || (t.rank > 0 && t.sizes == nullptr) ||
        (t.rank > 0 && !stride_ok) || (t.rank == -1 && (t.sizes != nullptr || t.strides != nullptr)))
      return abi_mismatch("kernel has an invalid tensor constraint");
    for (std::int32_t axis = 0; axis < t.rank; ++axis) {
      if (!well_formed(record_at(t.sizes, t.dimension_constraint_stride, axis)))
        return abi_mismatch("kernel has an invalid size constraint");
      if (t.strides != nullptr && !well_formed(record_at(t.strides, t.dimension_constraint_stride, axis)))
        return abi_mismatch("kernel has an invalid stride constraint");
    }
  }
  return Status::success();
}

bool dimension_accepts(const VecopsDimensionConstraint& c, std::int64_t v) {
  if (c.struct_size < sizeof(VecopsDimensionConstraint)) return false;
  if (c.kind == VECOPS_DIM_ANY) return true;
  if (c.kind == VECOPS_DIM_CONST) return v == c.value;
  if (c.kind == VECOPS_DIM_DYNAMIC)
    return c.alignment > 0 && v >= c.lower_bound && v <= c.upper_bound && v % c.alignment == 0;
  return false;
}

// Arguments against an artifact's own parameter table (Executable.cpp:118-184).
Status check_arguments(const ArgumentMetadata& args, const VecopsKernelDescriptorV1& d) {
  if (args.size() != d.num_parameters) return invalid("argument count does not match the kernel specialization");
  for (std::size_t i = 0; i < args.size(); ++i) {
    const Value& value = args[i];
    const auto& p = record_at(d.parameters, d.parameter_stride, i);
    const std::string name(p.name);
    if (std::holds_alternative<std::monostate>(value)) {
      if (p.kind == VECOPS_VALUE_TENSOR && p.constraint.tensor.optional != 0) continue;
      return invalid(name + " is not optional");
    }
    if (p.kind != VECOPS_VALUE_TENSOR) {
      const auto* scalar = std::get_if<Scalar>(&value);
      if (scalar == nullptr || (dtype_bit(scalar->dtype) & p.constraint.scalar.dtype_mask) == 0)
        return invalid(name + " scalar mismatch");
      continue;
    }
    const auto* t = std::get_if<TensorView>(&value);
    if (t == nullptr) return invalid(name + " must be a tensor");
    const auto& c = p.constraint.tensor;
    if ((dtype_bit(t->dtype) & c.dtype_mask) == 0) return invalid(name + " dtype mismatch");
    if ((c.device_type != 0 && t->device_type != c.device_type) ||
        (c.device_index >= 0 && t->device_index != c.device_index))
      return invalid(name + " device mismatch");
    if (t->sizes.size() != t->strides.size() || t->sizes.size() > std::numeric_limits<std::uint32_t>::max() ||
        (c.rank >= 0 && t->sizes.size() != static_cast<std::size_t>(c.rank)))
      return invalid(name + " rank mismatch");
    bool empty = false;
    for (const auto s : t->sizes) {
      if (s < 0) return invalid(name + " has a negative size");
      empty = empty || s == 0;
    }
    if (!empty && t->data == nullptr) return invalid(name + " has no data");
    const auto need = c.required_flags & (VECOPS_TENSOR_READ | VECOPS_TENSOR_WRITE);
    if ((t->flags & need) != need) return invalid(name + " access mismatch");
    for (std::size_t axis = 0; axis < t->sizes.size(); ++axis) {
      if (c.sizes != nullptr &&
          !dimension_accepts(record_at(c.sizes, c.dimension_constraint_stride, axis), t->sizes[axis]))
        return invalid(name + " shape mismatch");
      if (c.strides != nullptr &&
          !dimension_accepts(record_at(c.strides, c.dimension_constraint_stride, axis), t->strides[axis]))
        return invalid(name + " stride mismatch");
    }
  }
  return Status::success();
}

// Callback result -> Status; a message the callee left wins over the fallback
// and out-of-range codes read as ExecutionError (Executable.cpp:186-197).
Status callback_status(std::int32_t rc, const VecopsError& error, std::string_view fallback) {
  if (rc == VECOPS_STATUS_OK) return Status::success();
  std::string message(fallback);
  if (error.message != nullptr && error.message[0] != '\0') message = error.message;
  const bool known = rc >= VECOPS_STATUS_INVALID_ARGUMENT && rc <= VECOPS_STATUS_INTERNAL_ERROR;
  return Status(known ? static_cast<StatusCode>(rc) : StatusCode::ExecutionError, std::move(message));
}

constexpr std::size_t kMessageBytes = 1024;

}  // namespace

// ---- Argument ---------------------------------------------------------------------------------

Scalar Scalar::signed_integer(std::int64_t value, DType dtype) {
  Scalar s;
  s.dtype = dtype;
  s.value.i64 = value;
  return s;
}
Scalar Scalar::unsigned_integer(std::uint64_t value, DType dtype) {
  Scalar s;
  s.dtype = dtype;
  s.value.u64 = value;
  return s;
}
Scalar Scalar::floating(double value, DType dtype) {
  Scalar s;
  s.dtype = dtype;
  s.value.f64 = value;
  return s;
}

CallFrame::CallFrame(const ArgumentMetadata& arguments, void* workspace, std::uint64_t workspace_size,
                     const VecopsExecutionContext* context) {
  values_.resize(arguments.size());
  for (std::size_t i = 0; i < arguments.size(); ++i) {
    VecopsValue& out = values_[i];
    out = VecopsValue{};
    out.struct_size = sizeof(VecopsValue);
    const Value& in = arguments[i];
    if (const auto* t = std::get_if<TensorView>(&in)) {
      out.kind = VECOPS_VALUE_TENSOR;
      auto& v = out.value.tensor;
      v.struct_size = sizeof(VecopsTensorView);
      v.data = t->data;
      v.byte_offset = t->byte_offset;
      v.device_type = t->device_type;
      v.device_index = t->device_index;
      v.dtype = static_cast<std::uint32_t>(t->dtype);
      v.rank = static_cast<std::uint32_t>(t->sizes.size());
      v.sizes = t->sizes.data();  // borrowed from `arguments`
      v.strides = t->strides.data();
      v.flags = t->flags;
    } else if (const auto* s = std::get_if<Scalar>(&in)) {
      out.kind = VECOPS_VALUE_SCALAR;
      out.value.scalar.struct_size = sizeof(VecopsScalar);
      out.value.scalar.dtype = static_cast<std::uint32_t>(s->dtype);
      out.value.scalar.value = s->value;
    } else {
      out.kind = VECOPS_VALUE_NONE;
    }
  }
  call_.struct_size = sizeof(VecopsCall);
  call_.num_values = static_cast<std::uint32_t>(values_.size());
  call_.values = values_.data();
  call_.workspace = workspace;
  call_.workspace_size = workspace_size;
  call_.context = context;
}

// ---- Schema ---------------------------------------------------------------------------------------

DimensionConstraint DimensionConstraint::any() { return {}; }
DimensionConstraint DimensionConstraint::constant(std::int64_t value) {
  DimensionConstraint c;
  c.kind = Kind::Const;
  c.value = value;
  return c;
}
DimensionConstraint DimensionConstraint::dynamic(std::int64_t lower_bound, std::int64_t upper_bound,
                                                 std::int64_t alignment) {
  DimensionConstraint c;
  c.kind = Kind::Dynamic;
  c.lower_bound = lower_bound;
  c.upper_bound = upper_bound;
  c.alignment = alignment;
  return c;
}
bool DimensionConstraint::accepts(std::int64_t candidate) const {
  if (kind == Kind::Any) return true;
  if (kind == Kind::Const) return candidate == value;
  return candidate >= lower_bound && candidate <= upper_bound && alignment > 0 && candidate % alignment == 0;
}

// Order of checks as in Schema.cpp:56-103: dtype, device, rank consistency,
// negative sizes, rank, constraint arity, sizes, strides, access flags.
Status validate_tensor(const TensorView& t, const TensorConstraint& c, std::string_view parameter_name) {
  const std::string name(parameter_name);
  if ((dtype_bit(t.dtype) & c.dtype_mask) == 0) return invalid(name + " has an unsupported dtype");
  if ((c.device_type != 0 && t.device_type != c.device_type) ||
      (c.device_index >= 0 && t.device_index != c.device_index))
    return invalid(name + " is on the wrong device");
  if (t.sizes.size() != t.strides.size()) return invalid(name + " has different size and stride ranks");
  if (t.sizes.size() > std::numeric_limits<std::uint32_t>::max()) return invalid(name + " rank exceeds the ABI limit");
  for (const auto s : t.sizes)
    if (s < 0) return invalid(name + " has a negative size");
  if (c.rank && t.sizes.size() != *c.rank) return invalid(name + " has the wrong rank");
  if (!c.sizes.empty() && c.sizes.size() != t.sizes.size()) return invalid(name + " has no size constraint for its rank");
  if (!c.strides.empty() && c.strides.size() != t.strides.size())
    return invalid(name + " has no stride constraint for its rank");
  for (std::size_t i = 0; i < c.sizes.size(); ++i)
    if (!c.sizes[i].accepts(t.sizes[i])) return invalid(name + " size[" + std::to_string(i) + "] violates schema");
  for (std::size_t i = 0; i < c.strides.size(); ++i)
    if (!c.strides[i].accepts(t.strides[i])) return invalid(name + " stride[" + std::to_string(i) + "] violates schema");
  if ((t.flags & c.required_flags) != c.required_flags)
    return invalid(name + " does not satisfy the required access flags");
  return Status::success();
}

OperatorSchema::OperatorSchema(std::string name, std::vector<ParameterSchema> parameters,
                               RelationValidator relation_validator)
  : name_(std::move(name)), parameters_(std::move(parameters)), relation_validator_(std::move(relation_validator)) {}

Status OperatorSchema::validate(const ArgumentMetadata& arguments) const {
  if (arguments.size() != parameters_.size())
    return invalid(name_ + " expects " + std::to_string(parameters_.size()) + " arguments, got " +
                   std::to_string(arguments.size()));
  for (std::size_t i = 0; i < parameters_.size(); ++i) {
    const ParameterSchema& p = parameters_[i];
    const Value& v = arguments[i];
    if (const auto* tc = std::get_if<TensorConstraint>(&p.constraint)) {
      if (std::holds_alternative<std::monostate>(v)) {
        if (!tc->optional) return invalid(p.name + " is not optional");
        continue;
      }
      const auto* t = std::get_if<TensorView>(&v);
      if (t == nullptr) return invalid(p.name + " must be a tensor");
      if (auto st = validate_tensor(*t, *tc, p.name); !st.ok()) return st;
    } else {
      const auto* s = std::get_if<Scalar>(&v);
      if (s == nullptr) return invalid(p.name + " must be a scalar");
      if ((dtype_bit(s->dtype) & std::get<ScalarConstraint>(p.constraint).dtype_mask) == 0)
        return invalid(p.name + " has an unsupported scalar dtype");
    }
  }
  return relation_validator_ ? relation_validator_(arguments.values()) : Status::success();
}

// ---- Executable -------------------------------------------------------------------------------------

LoadedModule::~LoadedModule() {
  if (handle_ != nullptr) dlclose(handle_);
}

Result<std::shared_ptr<LoadedModule>> LoadedModule::load(const std::filesystem::path& library_path) {
  dlerror();
  void* handle = dlopen(library_path.c_str(), RTLD_NOW | RTLD_LOCAL);
  if (handle == nullptr) {
    const char* why = dlerror();
    return Status(StatusCode::LoadError,
                  "failed to load " + library_path.string() + ": " + (why ? why : "unknown dynamic-loader error"));
  }
  dlerror();
  auto query = reinterpret_cast<VecopsKernelQueryFnV1>(dlsym(handle, VECOPS_KERNEL_QUERY_SYMBOL_V1));
  const char* why = dlerror();
  if (query == nullptr || why != nullptr) {
    std::string message = std::string("kernel artifact does not export ") + VECOPS_KERNEL_QUERY_SYMBOL_V1;
    if (why != nullptr) message += std::string(": ") + why;
    dlclose(handle);
    return abi_mismatch(std::move(message));
  }
  const VecopsKernelDescriptorV1* descriptor = query();
  if (auto st = check_descriptor(descriptor); !st.ok()) {
    dlclose(handle);
    return st;
  }
  return std::shared_ptr<LoadedModule>(new LoadedModule(library_path, handle, descriptor));
}

Result<std::shared_ptr<Executable>> Executable::load(const std::filesystem::path& library_path) {
  auto module = LoadedModule::load(library_path);
  if (!module) return module.status();
  return std::make_shared<Executable>(std::move(module).value());
}

std::string_view Executable::operator_name() const { return module_->descriptor().operator_name; }
std::string_view Executable::specialization_key() const { return module_->descriptor().specialization_key; }

Status Executable::can_invoke(const ArgumentMetadata& arguments) const {
  return check_arguments(arguments, module_->descriptor());
}

Result<std::uint64_t> Executable::workspace_size(const ArgumentMetadata& arguments,
                                                 const VecopsExecutionContext* context) const {
  if (auto st = can_invoke(arguments); !st.ok()) return st;
  const VecopsWorkspaceFn query = module_->descriptor().workspace;
  if (query == nullptr) return std::uint64_t{0};
  CallFrame frame(arguments, nullptr, 0, context);
  std::array<char, kMessageBytes> text{};
  VecopsError error{};
  error.struct_size = sizeof(VecopsError);
  error.message = text.data();
  error.message_capacity = text.size();
  std::uint64_t bytes = 0;
  const std::int32_t rc = query(&frame.abi(), &bytes, &error);
  text.back() = '\0';
  if (auto st = callback_status(rc, error, "kernel workspace query failed"); !st.ok()) return st;
  return bytes;
}

Status Executable::invoke(const ArgumentMetadata& arguments, void* workspace, std::uint64_t workspace_size,
                          const VecopsExecutionContext* context) const {
  auto required = this->workspace_size(arguments, context);
  if (!required) return required.status();
  if (required.value() > workspace_size || (required.value() != 0 && workspace == nullptr))
    return invalid("kernel requires " + std::to_string(required.value()) + " workspace bytes, but " +
                   std::to_string(workspace_size) + " were supplied");
  CallFrame frame(arguments, workspace, workspace_size, context);
  return invoke_unchecked(frame.abi());
}

Status Executable::invoke_unchecked(const VecopsCall& call) const {
  std::array<char, kMessageBytes> text{};
  VecopsError error{};
  error.struct_size = sizeof(VecopsError);
  error.message = text.data();
  error.message_capacity = text.size();
  const std::int32_t rc = module_->descriptor().run(&call, &error);
  text.back() = '\0';
  return callback_status(rc, error, "kernel execution failed");
}

Status Executable::invoke_prevalidated(const VecopsCall& call) const { return invoke_unchecked(call); }

// ---- Operator ---------------------------------------------------------------------------------------

Result<std::vector<std::size_t>>
OrderedDispatchPolicy::candidates(const KernelCall&, std::span<const std::shared_ptr<const KernelRecipe>> recipes) const {
  std::vector<std::size_t> order(recipes.size());
  std::iota(order.begin(), order.end(), std::size_t{0});
  return order;
}

Operator::Operator(OperatorSchema schema, std::vector<std::shared_ptr<const KernelRecipe>> recipes,
                   std::shared_ptr<const DispatchPolicy> dispatch_policy, std::shared_ptr<ExecutableProvider> provider)
  : schema_(std::move(schema))
  , recipes_(std::move(recipes))
  , dispatch_policy_(std::move(dispatch_policy))
  , provider_(std::move(provider)) {}

// The dispatch loop of Operator.cpp:215-263: candidates in policy order; a
// recipe's NotApplicable, or the provider's NotFound / NotApplicable, moves on to
// the next candidate and is remembered as the failure to report; any other error
// ends dispatch.  A resolved executable must carry this operator's name and
// exactly the requested specialization key.
Result<std::shared_ptr<Executable>> Operator::resolve_validated(const KernelCall& call) const {
  if (dispatch_policy_ == nullptr || provider_ == nullptr)
    return Status(StatusCode::InternalError, "operator has no dispatch policy or executable provider");
  auto order = dispatch_policy_->candidates(call, recipes_);
  if (!order) return order.status();
  Status last(StatusCode::NotFound, "no kernel recipe accepted this invocation");
  for (const std::size_t index : order.value()) {
    if (index >= recipes_.size() || recipes_[index] == nullptr)
      return Status(StatusCode::InternalError, "dispatch policy returned an invalid recipe index");
    const KernelRecipe& recipe = *recipes_[index];
    if (Status st = recipe.match(call); !st.ok()) {
      if (st.code() != StatusCode::NotApplicable) return st;
      last = st;
      continue;
    }
    auto bound = recipe.bind(call);
    if (!bound) {
      if (bound.status().code() != StatusCode::NotApplicable) return bound.status();
      last = bound.status();
      continue;
    }
    if (bound.value().recipe_id.empty()) bound.value().recipe_id = std::string(recipe.id());
    auto executable = provider_->resolve(bound.value());
    if (!executable) {
      const StatusCode code = executable.status().code();
      if (code != StatusCode::NotFound && code != StatusCode::NotApplicable) return executable.status();
      last = executable.status();
      continue;
    }
    if (executable.value() == nullptr)
      return Status(StatusCode::InternalError, "executable provider returned a null executable");
    if (executable.value()->operator_name() != schema_.name())
      return abi_mismatch("resolved executable belongs to a different operator");
    if (executable.value()->specialization_key() != bound.value().specialization_key)
      return abi_mismatch("resolved executable has a different specialization key");
    return executable;
  }
  return last;
}

Result<std::shared_ptr<Executable>> Operator::resolve(const ArgumentMetadata& arguments) const {
  return resolve(KernelCall(arguments), nullptr);
}

Result<std::shared_ptr<Executable>> Operator::resolve(const KernelCall& call, const VecopsExecutionContext*) const {
  if (Status st = schema_.validate(call.arguments()); !st.ok()) return st;
  return resolve_validated(call);
}

Status Operator::invoke(const ArgumentMetadata& arguments, void* workspace, std::uint64_t workspace_size,
                        const VecopsExecutionContext* context) const {
  return invoke(KernelCall(arguments), context, workspace, workspace_size);
}

Status Operator::invoke(const KernelCall& call, const VecopsExecutionContext* context, void* workspace,
                        std::uint64_t workspace_size) const {
  if (Status st = schema_.validate(call.arguments()); !st.ok()) return st;
  auto executable = resolve_validated(call);
  if (!executable) return executable.status();
  return executable.value()->invoke(call.arguments(), workspace, workspace_size, context);
}

}  // namespace vecops::runtime
