/*
 * Binary contract between a vecops runtime and a kernel artifact DSO, restated
 * for the HIP artifacts of this repository.  Record layouts, enum values and
 * the query symbol are those of vecops' runtime/CallAbi.h:34-400 and
 * runtime/KernelAbi.h:23-176, so a DSO built against this header loads into an
 * unmodified vecops runtime and vice versa; only the records the matmul path
 * touches are restated (the thread-pool, arena-provider and allocation-observer
 * records stay opaque pointers inside VecopsExecutionContext).
 *
 * Rules of the contract (runtime/CallAbi.h:7-16): every record starts with the
 * size its writer knew; readers must not touch fields past that size; nothing
 * passed in is owned by the callee or valid after the call returns; calls are
 * synchronous; sizes and strides count elements, byte_offset and workspace
 * sizes count bytes.
 */
#ifndef VECOPS_RT_ABI_H
#define VECOPS_RT_ABI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define VECOPS_RUNTIME_EXPORT __attribute__((visibility("default")))

/* ---- enumerations (numeric values are the contract) ------------------------- */

typedef enum VecopsStatusCode {
  VECOPS_STATUS_OK = 0,
  VECOPS_STATUS_INVALID_ARGUMENT = 1, /* caller broke a contract */
  VECOPS_STATUS_NOT_APPLICABLE = 2,   /* valid call, but not for this recipe */
  VECOPS_STATUS_NOT_FOUND = 3,        /* no artifact / recipe / specialization */
  VECOPS_STATUS_ABI_MISMATCH = 4,     /* version, record size or key differs */
  VECOPS_STATUS_LOAD_ERROR = 5,       /* dlopen / dlsym failed */
  VECOPS_STATUS_EXECUTION_ERROR = 6,  /* the kernel callback failed */
  VECOPS_STATUS_INTERNAL_ERROR = 7
} VecopsStatusCode;

typedef enum VecopsDeviceType {
  VECOPS_DEVICE_CPU = 1,
  VECOPS_DEVICE_CUDA = 2,
  VECOPS_DEVICE_PRIVATE = 255 /* embedding-defined; the HIP artifacts read it as "HIP device pointer" */
} VecopsDeviceType;

typedef enum VecopsDType {
  VECOPS_DTYPE_INVALID = 0,
  VECOPS_DTYPE_BOOL = 1,
  VECOPS_DTYPE_I8 = 2,
  VECOPS_DTYPE_U8 = 3,
  VECOPS_DTYPE_I16 = 4,
  VECOPS_DTYPE_U16 = 5,
  VECOPS_DTYPE_I32 = 6,
  VECOPS_DTYPE_U32 = 7,
  VECOPS_DTYPE_I64 = 8,
  VECOPS_DTYPE_U64 = 9,
  VECOPS_DTYPE_F16 = 10,
  VECOPS_DTYPE_BF16 = 11,
  VECOPS_DTYPE_F32 = 12,
  VECOPS_DTYPE_F64 = 13
} VecopsDType;

typedef enum VecopsValueKind { VECOPS_VALUE_NONE = 0, VECOPS_VALUE_TENSOR = 1, VECOPS_VALUE_SCALAR = 2 } VecopsValueKind;

typedef enum VecopsTensorFlags {
  VECOPS_TENSOR_READ = UINT64_C(1) << 0,
  VECOPS_TENSOR_WRITE = UINT64_C(1) << 1
} VecopsTensorFlags;

/* ---- call records ---------------------------------------------------------------- */

typedef struct VecopsError {
  uint32_t struct_size;
  int32_t code;             /* written by a failing callee */
  char* message;            /* caller-owned buffer, may be null */
  size_t message_capacity;  /* bytes, terminator included */
  size_t message_required;  /* bytes the full message needs, terminator included */
} VecopsError;

typedef struct VecopsTensorView {
  uint32_t struct_size;
  void* data;            /* base address; logical element zero is data + byte_offset */
  uint64_t byte_offset;
  uint32_t device_type;  /* VecopsDeviceType */
  int32_t device_index;
  uint32_t dtype;        /* VecopsDType */
  uint32_t rank;
  const int64_t* sizes;    /* rank entries */
  const int64_t* strides;  /* rank entries, elements */
  uint64_t flags;          /* VecopsTensorFlags granted by the caller */
} VecopsTensorView;

typedef union VecopsScalarStorage {
  int64_t i64;
  uint64_t u64;
  double f64;
} VecopsScalarStorage;

typedef struct VecopsScalar {
  uint32_t struct_size;
  uint32_t dtype;
  VecopsScalarStorage value;
} VecopsScalar;

typedef struct VecopsValue {
  uint32_t struct_size;
  uint32_t kind; /* VecopsValueKind */
  union {
    VecopsTensorView tensor;
    VecopsScalar scalar;
  } value;
} VecopsValue;

struct VecopsWorkspaceArenaProvider;
struct VecopsThreadPoolV1;
struct VecopsAllocationObserverV1;

typedef struct VecopsExecutionContext {
  uint32_t struct_size;
  uint32_t requested_threads;
  void* stream;     /* forwarded uninterpreted by the runtime; the HIP artifacts read a hipStream_t */
  void* user_data;
  uint64_t flags;
  /* the three extension pointers are absent from older, shorter records */
  const struct VecopsWorkspaceArenaProvider* workspace_provider;
  const struct VecopsThreadPoolV1* thread_pool;
  const struct VecopsAllocationObserverV1* allocation_observer;
} VecopsExecutionContext;

typedef struct VecopsCall {
  uint32_t struct_size;
  uint32_t num_values;
  const VecopsValue* values;  /* positional, descriptor order */
  void* workspace;            /* caller-owned, may be null */
  uint64_t workspace_size;
  const VecopsExecutionContext* context;
} VecopsCall;

/* ---- artifact descriptor ------------------------------------------------------------ */

#define VECOPS_KERNEL_ABI_VERSION_MAJOR 1u
#define VECOPS_KERNEL_ABI_VERSION_MINOR 1u
#define VECOPS_KERNEL_QUERY_SYMBOL_V1 "vecops_kernel_query_v1"

typedef enum VecopsDimensionKind { VECOPS_DIM_ANY = 0, VECOPS_DIM_CONST = 1, VECOPS_DIM_DYNAMIC = 2 } VecopsDimensionKind;

typedef struct VecopsDimensionConstraint {
  uint32_t struct_size;
  uint32_t kind;        /* VecopsDimensionKind */
  int64_t value;        /* CONST */
  int64_t lower_bound;  /* DYNAMIC, inclusive */
  int64_t upper_bound;  /* DYNAMIC, inclusive */
  int64_t alignment;    /* DYNAMIC, positive power of two */
} VecopsDimensionConstraint;

typedef struct VecopsTensorParameter {
  uint32_t struct_size;
  uint64_t dtype_mask;   /* bit (dtype - 1) per accepted dtype */
  uint32_t device_type;  /* 0 = any */
  int32_t device_index;  /* -1 = any */
  int32_t rank;          /* -1 = any */
  uint32_t optional;
  uint32_t dimension_constraint_stride;
  const VecopsDimensionConstraint* sizes;
  const VecopsDimensionConstraint* strides;
  uint64_t required_flags;
} VecopsTensorParameter;

typedef struct VecopsScalarParameter {
  uint32_t struct_size;
  uint64_t dtype_mask;
} VecopsScalarParameter;

typedef struct VecopsParameterDescriptor {
  uint32_t struct_size;
  uint32_t kind; /* VECOPS_VALUE_TENSOR or VECOPS_VALUE_SCALAR */
  const char* name;
  union {
    VecopsTensorParameter tensor;
    VecopsScalarParameter scalar;
  } constraint;
} VecopsParameterDescriptor;

typedef int32_t (*VecopsWorkspaceFn)(const VecopsCall*, uint64_t*, VecopsError*);
typedef int32_t (*VecopsRunFn)(const VecopsCall*, VecopsError*);

typedef struct VecopsKernelDescriptorV1 {
  uint32_t struct_size;
  uint16_t abi_version_major;
  uint16_t abi_version_minor;
  const char* operator_name;
  const char* specialization_key;
  uint32_t num_parameters;
  uint32_t parameter_stride;
  const VecopsParameterDescriptor* parameters;
  VecopsWorkspaceFn workspace; /* null = never needs workspace */
  VecopsRunFn run;
  uint64_t flags; /* must be zero in v1 */
} VecopsKernelDescriptorV1;

typedef const VecopsKernelDescriptorV1* (*VecopsKernelQueryFnV1)(void);

/* The one symbol an artifact DSO exports. */
VECOPS_RUNTIME_EXPORT const VecopsKernelDescriptorV1* vecops_kernel_query_v1(void);

/* ---- process-local operator bridge (vecops runtime/OperatorBridgeAbi.h:29-71) --------- */
/* A framework extension enters an Operator it knows by handle; the records are vecops' own. */

#define VECOPS_OPERATOR_BRIDGE_ABI_VERSION_MAJOR 1u
#define VECOPS_OPERATOR_BRIDGE_ABI_VERSION_MINOR 0u

typedef enum VecopsSpecializationValueKind {
  VECOPS_SPECIALIZATION_CONST_INT = 1,
  VECOPS_SPECIALIZATION_DTYPE = 2
} VecopsSpecializationValueKind;

typedef struct VecopsSpecializationArgument {
  uint32_t struct_size;
  uint32_t kind;      /* VecopsSpecializationValueKind */
  const char* name;   /* caller-owned, nul-terminated */
  union {
    int64_t integer;  /* CONST_INT */
    uint32_t dtype;   /* DTYPE: a VecopsDType number */
  } value;
} VecopsSpecializationArgument;

VECOPS_RUNTIME_EXPORT int32_t vecops_operator_bridge_invoke_v1(uint64_t handle, const VecopsCall* call,
                                                               uint32_t num_specialization_values,
                                                               const VecopsSpecializationArgument* specialization_values,
                                                               VecopsError* error);

#ifdef __cplusplus
}
#endif
#endif /* VECOPS_RT_ABI_H */