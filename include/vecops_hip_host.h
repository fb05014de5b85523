/*
 * vecops_hip_host.h - C access to the vecops Operator objects of the HIP drop-in
 * (libvecops_hip_host.so), for embeddings and tests that are not C++.
 *
 * An operator handle wraps a vecops::runtime::Operator assembled from this
 * repository's schema, recipes, dispatch policy and HipExecutableProvider
 * (vecops_amd/host/hip/matmul_plugin.hpp) - the same objects a C++ embedding
 * passes to `Operator(schema, recipes, policy, provider)`
 * (vecops runtime/Operator.h:210-211).  Calls take the positional
 * VecopsValue records of vecops' call ABI (runtime/CallAbi.h:186-197) and go
 * through Operator::invoke (src/runtime/Operator.cpp:265-285): schema
 * validation, dispatch, provider resolution, descriptor validation, workspace
 * check, then the artifact DSO's run callback.  Status codes are
 * VecopsStatusCode numbers.
 */
#ifndef VECOPS_HIP_HOST_H
#define VECOPS_HIP_HOST_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

struct VecopsValue;
struct VecopsExecutionContext;
struct VecopsCall;
struct VecopsError;
struct VecopsSpecializationArgument;

#define VECOPS_HIP_HOST_EXPORT __attribute__((visibility("default")))

/* Specialization value of a call: kind 0 = integer (ConstInt), 1 = dtype (VecopsDType number). */
typedef struct VecopsHostSpecialization {
  const char* name;
  int32_t kind;
  int64_t value;
} VecopsHostSpecialization;

/* operator_name: "vecops::matmul", "vecops::matmul_fused", "vecops::matmul_i8_dequant",
 * "vecops::matmul_runtime_quant", "vecops::matmul_pack_b", "vecops::matmul_packed_b", "vecops::matmul_pack_a",
 * "vecops::matmul_packed_a" or "vecops::matmul_w8a16_group".  Returns null for an unknown name. */
VECOPS_HIP_HOST_EXPORT void* vecops_hip_host_operator_create(const char* operator_name, const char* artifact_directory);
VECOPS_HIP_HOST_EXPORT void vecops_hip_host_operator_destroy(void* op);

/* Which runtime this library was compiled against: "restated" or "upstream". */
VECOPS_HIP_HOST_EXPORT const char* vecops_hip_host_runtime_flavor(void);

/* Operator::resolve: writes the specialization key of the executable that would run. */
VECOPS_HIP_HOST_EXPORT int32_t vecops_hip_host_operator_resolve(void* op, const struct VecopsValue* values,
                                                                uint32_t num_values,
                                                                const VecopsHostSpecialization* specs,
                                                                uint32_t num_specs, char* key, size_t key_capacity,
                                                                char* message, size_t message_capacity);

/* Executable::workspace_size of the resolved executable. */
VECOPS_HIP_HOST_EXPORT int32_t vecops_hip_host_operator_workspace(void* op, const struct VecopsValue* values,
                                                                  uint32_t num_values,
                                                                  const VecopsHostSpecialization* specs,
                                                                  uint32_t num_specs, uint64_t* bytes, char* message,
                                                                  size_t message_capacity);

/* Operator::invoke(KernelCall, context, workspace, workspace_size). */
VECOPS_HIP_HOST_EXPORT int32_t vecops_hip_host_operator_invoke(void* op, const struct VecopsValue* values,
                                                               uint32_t num_values,
                                                               const VecopsHostSpecialization* specs,
                                                               uint32_t num_specs, void* workspace,
                                                               uint64_t workspace_size,
                                                               const struct VecopsExecutionContext* context,
                                                               char* message, size_t message_capacity);

/*
 * The process-local bridge of vecops' generated framework adapters (runtime/OperatorBridgeAbi.h:69-71;
 * implementation python/bindings/module.cpp:1223-1239): an extension holds an opaque handle and enters the Operator
 * with vecops' own call record.  vecops_operator_bridge_invoke_v1 has the reference's name, signature and error
 * protocol (VecopsCall, VecopsSpecializationArgument and VecopsError are the records of vecops_rt/abi.h, layout
 * identical to vecops' headers): it validates the handle and the records, resolves the executable and invokes it
 * synchronously, in one foreign call that holds no interpreter lock.  A call that brings no workspace gets device
 * scratch from a per-thread buffer of the bridge, grown on demand and kept.  Handles are never reused: after
 * vecops_hip_host_bridge_unregister a stale handle is an InvalidArgument (1), not another operator.
 */
VECOPS_HIP_HOST_EXPORT uint64_t vecops_hip_host_bridge_register(void* op);
VECOPS_HIP_HOST_EXPORT void vecops_hip_host_bridge_unregister(uint64_t handle);
VECOPS_HIP_HOST_EXPORT int32_t vecops_operator_bridge_invoke_v1(uint64_t handle, const struct VecopsCall* call,
                                                                uint32_t num_specialization_values,
                                                                const struct VecopsSpecializationArgument* specialization_values,
                                                                struct VecopsError* error);

/* Executable::load on one file: 0 when it is a valid artifact; writes its operator name and key. */
VECOPS_HIP_HOST_EXPORT int32_t vecops_hip_host_load_artifact(const char* path, char* operator_name, size_t name_capacity,
                                                             char* key, size_t key_capacity, char* message,
                                                             size_t message_capacity);

#ifdef __cplusplus
}
#endif
#endif /* VECOPS_HIP_HOST_H */
