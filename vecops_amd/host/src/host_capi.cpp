// C entry points over the Operator objects of the HIP drop-in (include/vecops_hip_host.h).
#include "vecops_hip_host.h"

#include <dlfcn.h>

#include <atomic>
#include <cstddef>
#include <cstring>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

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

// ---- the process-local bridge (vecops runtime/OperatorBridgeAbi.h) ---------------------------------------------
// Handles are small integers that stay invalid after unregistration (never reused), so a stale handle held by a
// framework extension is refused rather than served by another operator.
std::mutex g_bridge_mutex;
std::unordered_map<std::uint64_t, std::shared_ptr<rt::Operator>> g_bridge_operators;
std::atomic<std::uint64_t> g_next_handle{1};

// Device workspace of bridge calls that bring none: one buffer per host thread and device, grown on demand
// (a bridge call is synchronous, so a thread never has two calls using its buffer).  The HIP runtime is looked up at
// the first need - this library itself does not link it.
struct HipRuntime {
  int (*get_device)(int*) = nullptr;
  int (*malloc_)(void**, size_t) = nullptr;
  int (*free_)(void*) = nullptr;
  bool ok = false;
};
const HipRuntime& hip_runtime() {
  static const HipRuntime runtime = [] {
    HipRuntime r;
    void* lib = dlopen("libamdhip64.so", RTLD_NOW | RTLD_GLOBAL);
    if (lib == nullptr) lib = dlopen("/opt/rocm/lib/libamdhip64.so", RTLD_NOW | RTLD_GLOBAL);
    if (lib == nullptr) return r;
    r.get_device = reinterpret_cast<int (*)(int*)>(dlsym(lib, "hipGetDevice"));
    r.malloc_ = reinterpret_cast<int (*)(void**, size_t)>(dlsym(lib, "hipMalloc"));
    r.free_ = reinterpret_cast<int (*)(void*)>(dlsym(lib, "hipFree"));
    r.ok = r.get_device != nullptr && r.malloc_ != nullptr && r.free_ != nullptr;
    return r;
  }();
  return runtime;
}
// Buffers are never given back to the device: a thread that ends returns its buffers to a process-wide pool for the
// next thread to take (no HIP call runs in a thread's or the process's teardown, when the runtime may be gone).
struct DeviceBuffer {
  void* data = nullptr;
  std::uint64_t size = 0;
};
constexpr int kBridgeDevices = 64;
std::mutex g_pool_mutex;
std::vector<DeviceBuffer> g_buffer_pool[kBridgeDevices];

struct ThreadWorkspace {
  DeviceBuffer mine[kBridgeDevices];
  ~ThreadWorkspace() {
    std::lock_guard<std::mutex> lock(g_pool_mutex);
    for (int d = 0; d < kBridgeDevices; ++d)
      if (mine[d].data != nullptr) g_buffer_pool[d].push_back(mine[d]);
  }
  rt::Status get(std::uint64_t bytes, void** out) {
    const HipRuntime& hip = hip_runtime();
    if (!hip.ok) return rt::Status(rt::StatusCode::ExecutionError, "bridge workspace: the HIP runtime is not available");
    int device = 0;
    if (hip.get_device(&device) != 0 || device < 0 || device >= kBridgeDevices)
      return rt::Status(rt::StatusCode::ExecutionError, "bridge workspace: no current HIP device");
    DeviceBuffer& buffer = mine[device];
    if (buffer.size < bytes) {
      std::lock_guard<std::mutex> lock(g_pool_mutex);
      std::vector<DeviceBuffer>& pool = g_buffer_pool[device];
      // The buffer that is too small for this call goes back to the pool (someone else's next call may fit), unless
      // the pool is full: then it is freed (hipFree waits for the device, so no kernel of an earlier call still
      // uses it).  The pool holds at most kPoolCap buffers per device, which bounds what the bridge keeps.
      constexpr size_t kPoolCap = 8;
      if (buffer.data != nullptr) {
        if (pool.size() < kPoolCap) pool.push_back(buffer);
        else hip.free_(buffer.data);
      }
      buffer = DeviceBuffer{};
      // the smallest pooled buffer that fits: a small request must not take the largest one
      size_t best = pool.size();
      for (size_t i = 0; i < pool.size(); ++i)
        if (pool[i].size >= bytes && (best == pool.size() || pool[i].size < pool[best].size)) best = i;
      if (best != pool.size()) {
        buffer = pool[best];
        pool.erase(pool.begin() + static_cast<std::ptrdiff_t>(best));
      }
      if (buffer.data == nullptr) {
        const std::uint64_t want = (bytes + (std::uint64_t{1} << 20) - 1) & ~((std::uint64_t{1} << 20) - 1);
        if (hip.malloc_(&buffer.data, want) != 0) {
          buffer = DeviceBuffer{};
          return rt::Status(rt::StatusCode::ExecutionError,
                            "bridge workspace: device allocation of " + std::to_string(want) + " bytes failed");
        }
        buffer.size = want;
      }
    }
    *out = buffer.data;
    return rt::Status::success();
  }
};

rt::Status bridge_invoke(std::uint64_t handle, const VecopsCall* call, std::uint32_t num_specs,
                         const VecopsSpecializationArgument* specs) {
  if (call == nullptr || call->struct_size < sizeof(VecopsCall))
    return rt::Status(rt::StatusCode::InvalidArgument, "bridge call record is missing or too short");
  if (call->num_values != 0 && call->values == nullptr)
    return rt::Status(rt::StatusCode::InvalidArgument, "bridge call has values but no array");
  if (num_specs != 0 && specs == nullptr)
    return rt::Status(rt::StatusCode::InvalidArgument, "bridge call has specialization values but no array");
  std::shared_ptr<rt::Operator> op;
  {
    std::lock_guard<std::mutex> lock(g_bridge_mutex);
    auto it = g_bridge_operators.find(handle);
    if (it != g_bridge_operators.end()) op = it->second;  // the call keeps the operator alive
  }
  if (op == nullptr) return rt::Status(rt::StatusCode::InvalidArgument, "bridge handle " + std::to_string(handle) + " names no operator");
  std::vector<VecopsHostSpecialization> converted(num_specs);
  for (std::uint32_t i = 0; i < num_specs; ++i) {
    const VecopsSpecializationArgument& a = specs[i];
    if (a.struct_size < sizeof(VecopsSpecializationArgument) || a.name == nullptr)
      return rt::Status(rt::StatusCode::InvalidArgument, "malformed specialization argument");
    if (a.kind == VECOPS_SPECIALIZATION_CONST_INT) converted[i] = {a.name, 0, a.value.integer};
    else if (a.kind == VECOPS_SPECIALIZATION_DTYPE) converted[i] = {a.name, 1, static_cast<std::int64_t>(a.value.dtype)};
    else return rt::Status(rt::StatusCode::InvalidArgument, "unknown specialization value kind");
  }
  const rt::KernelCall kernel_call = make_call(call->values, call->num_values, converted.data(), num_specs);
  void* workspace = call->workspace;
  std::uint64_t workspace_size = call->workspace_size;
  if (workspace == nullptr) {
    // the bridge owns the scratch of calls that bring none (vecops allocates a host Workspace here,
    // python/bindings/module.cpp:1186-1203; device tensors need device memory)
    auto executable = op->resolve(kernel_call, call->context);
    if (!executable) return executable.status();
    auto need = executable.value()->workspace_size(kernel_call.arguments(), call->context);
    if (!need) return need.status();
    workspace_size = need.value();
    if (workspace_size != 0) {
      thread_local ThreadWorkspace cache;
      if (rt::Status st = cache.get(workspace_size, &workspace); !st.ok()) return st;
      // the thread's buffer serves its next call too: this one has to be over on return, whatever the caller's
      // context says about stream order (bit 0 of flags: VECOPS_HIP_CONTEXT_STREAM_ORDERED)
      if (call->context != nullptr && call->context->struct_size >= offsetof(VecopsExecutionContext, flags) + sizeof(std::uint64_t) &&
          (call->context->flags & 1u) != 0) {
        VecopsExecutionContext waiting;
        memset(&waiting, 0, sizeof(waiting));
        memcpy(&waiting, call->context, call->context->struct_size < sizeof(waiting) ? call->context->struct_size : sizeof(waiting));
        waiting.flags &= ~std::uint64_t{1};
        return op->invoke(kernel_call, &waiting, workspace, workspace_size);
      }
    }
  }
  return op->invoke(kernel_call, call->context, workspace, workspace_size);
}

}  // namespace

extern "C" {

uint64_t vecops_hip_host_bridge_register(void* op) {
  auto* h = static_cast<Handle*>(op);
  if (h == nullptr || h->op == nullptr) return 0;
  const std::uint64_t handle = g_next_handle.fetch_add(1);
  std::lock_guard<std::mutex> lock(g_bridge_mutex);
  g_bridge_operators.emplace(handle, h->op);
  return handle;
}

void vecops_hip_host_bridge_unregister(uint64_t handle) {
  std::lock_guard<std::mutex> lock(g_bridge_mutex);
  g_bridge_operators.erase(handle);
}

int32_t vecops_operator_bridge_invoke_v1(uint64_t handle, const VecopsCall* call, uint32_t num_specialization_values,
                                         const VecopsSpecializationArgument* specialization_values, VecopsError* error) {
  const rt::Status result = bridge_invoke(handle, call, num_specialization_values, specialization_values);
  if (result.ok()) return VECOPS_STATUS_OK;
  if (error != nullptr && error->struct_size >= sizeof(VecopsError)) {
    const std::string_view message = result.message();
    error->code = static_cast<std::int32_t>(result.code());
    error->message_required = message.size() + 1;
    if (error->message != nullptr && error->message_capacity != 0) {
      const size_t copied = message.size() < error->message_capacity - 1 ? message.size() : error->message_capacity - 1;
      memcpy(error->message, message.data(), copied);
      error->message[copied] = '\0';
    }
  }
  return static_cast<std::int32_t>(result.code());
}

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
  else if (name == vecops::hip::kMatmulPackAName) op = vecops::hip::make_matmul_pack_a_operator(artifact_directory);
  else if (name == vecops::hip::kMatmulPackedAName) op = vecops::hip::make_matmul_packed_a_operator(artifact_directory);
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
