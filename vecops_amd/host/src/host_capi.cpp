// C entry points over the Operator objects of the HIP drop-in (include/vecops_hip_host.h).
#include "vecops_hip_host.h"

#include <cstring>
#include <string>

#include "../hip/matmul_plugin.hpp"

namespace {

namespace rt = vecops::runtime;

struct Handle {
  std::shared_ptr<rt::Operator> op;
};

void put(char* dst, size_t cap, std::string_view text) {
  if (dst == nullptr || cap == 0) return;
  const size_t n = text.size() < cap - 1 ? text.size() : cap - 1;
  memcpy(dst, text.data(), n);
  dst[n] = '\0';
}

int32_t finish(const rt::Status& st, char* message, size_t cap) {
  put(message, cap, st.message());
  return static_cast<int32_t>(st.code());
}

rt::KernelCall make_call(const VecopsValue* values, uint32_t n, const VecopsHostSpecialization* specs, uint32_t ns) {
  std::vector<rt::Value> erased;
  erased.reserve(n);
  for (uint32_t i = 0; i < n; ++i) {
    const VecopsValue& v = values[i];
    if (v.kind == VECOPS_VALUE_TENSOR) {
      const VecopsTensorView& t = v.value.tensor;
      rt::TensorView view;
      view.data = t.data;
      view.byte_offset = t.byte_offset;
      view.device_type = t.device_type;
      view.device_index = t.device_index;
      view.dtype = static_cast<rt::DType>(t.dtype);
      view.sizes.assign(t.sizes, t.sizes + t.rank);
      view.strides.assign(t.strides, t.strides + t.rank);
      view.flags = t.flags;
      erased.emplace_back(std::move(view));
    } else if (v.kind == VECOPS_VALUE_SCALAR) {
      rt::Scalar s;
      s.dtype = static_cast<rt::DType>(v.value.scalar.dtype);
      s.value = v.value.scalar.value;
      erased.emplace_back(s);
    } else {
      erased.emplace_back(std::monostate{});
    }
  }
  rt::SpecializationValues sv;
  for (uint32_t i = 0; i < ns; ++i) {
    if (specs[i].kind == 1) sv.emplace(specs[i].name, static_cast<rt::DType>(specs[i].value));
    else sv.emplace(specs[i].name, static_cast<std::int64_t>(specs[i].value));
  }
  return rt::KernelCall(rt::ArgumentMetadata(std::move(erased)), std::move(sv));
}

}  // namespace

extern "C" {

void* vecops_hip_host_operator_create(const char* operator_name, const char* artifact_directory) {
  if (operator_name == nullptr || artifact_directory == nullptr) return nullptr;
  const std::string name(operator_name);
  std::shared_ptr<rt::Operator> op;
  if (name == vecops::hip::kMatmulName) op = vecops::hip::make_matmul_operator(artifact_directory);
  else if (name == vecops::hip::kMatmulI8DequantName) op = vecops::hip::make_matmul_i8_dequant_operator(artifact_directory);
  else if (name == vecops::hip::kMatmulW8A16GroupName) op = vecops::hip::make_matmul_w8a16_group_operator(artifact_directory);
  else if (name == vecops::hip::kMatmulFusedName) op = vecops::hip::make_matmul_fused_operator(artifact_directory);
  else if (name == vecops::hip::kMatmulPackBName) op = vecops::hip::make_matmul_pack_b_operator(artifact_directory);
  else if (name == vecops::hip::kMatmulPackedBName) op = vecops::hip::make_matmul_packed_b_operator(artifact_directory);
  else if (name == vecops::hip::kMatmulRuntimeQuantName) op = vecops::hip::make_matmul_runtime_quant_operator(artifact_directory);
  else return nullptr;
  return new Handle{std::move(op)};
}

void vecops_hip_host_operator_destroy(void* op) { delete static_cast<Handle*>(op); }

const char* vecops_hip_host_runtime_flavor(void) {
#ifdef VECOPS_HIP_USE_UPSTREAM_RUNTIME
  return "upstream";
#else
  return "restated";
#endif
}

int32_t vecops_hip_host_operator_resolve(void* op, const VecopsValue* values, uint32_t num_values,
                                         const VecopsHostSpecialization* specs, uint32_t num_specs, char* key,
                                         size_t key_capacity, char* message, size_t message_capacity) {
  auto* h = static_cast<Handle*>(op);
  if (h == nullptr) return VECOPS_STATUS_INVALID_ARGUMENT;
  const rt::KernelCall call = make_call(values, num_values, specs, num_specs);
  auto executable = h->op->resolve(call, nullptr);
  if (!executable) return finish(executable.status(), message, message_capacity);
  put(key, key_capacity, executable.value()->specialization_key());
  return VECOPS_STATUS_OK;
}

int32_t vecops_hip_host_operator_workspace(void* op, const VecopsValue* values, uint32_t num_values,
                                           const VecopsHostSpecialization* specs, uint32_t num_specs, uint64_t* bytes,
                                           char* message, size_t message_capacity) {
  auto* h = static_cast<Handle*>(op);
  if (h == nullptr || bytes == nullptr) return VECOPS_STATUS_INVALID_ARGUMENT;
  const rt::KernelCall call = make_call(values, num_values, specs, num_specs);
  auto executable = h->op->resolve(call, nullptr);
  if (!executable) return finish(executable.status(), message, message_capacity);
  auto size = executable.value()->workspace_size(call.arguments(), nullptr);
  if (!size) return finish(size.status(), message, message_capacity);
  *bytes = size.value();
  return VECOPS_STATUS_OK;
}

int32_t vecops_hip_host_operator_invoke(void* op, const VecopsValue* values, uint32_t num_values,
                                        const VecopsHostSpecialization* specs, uint32_t num_specs, void* workspace,
                                        uint64_t workspace_size, const VecopsExecutionContext* context, char* message,
                                        size_t message_capacity) {
  auto* h = static_cast<Handle*>(op);
  if (h == nullptr) return VECOPS_STATUS_INVALID_ARGUMENT;
  const rt::KernelCall call = make_call(values, num_values, specs, num_specs);
  return finish(h->op->invoke(call, context, workspace, workspace_size), message, message_capacity);
}

int32_t vecops_hip_host_load_artifact(const char* path, char* operator_name, size_t name_capacity, char* key,
                                      size_t key_capacity, char* message, size_t message_capacity) {
  auto executable = rt::Executable::load(path);
  if (!executable) return finish(executable.status(), message, message_capacity);
  put(operator_name, name_capacity, executable.value()->operator_name());
  put(key, key_capacity, executable.value()->specialization_key());
  return VECOPS_STATUS_OK;
}

}  // extern "C"
