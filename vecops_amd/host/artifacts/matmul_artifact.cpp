// Source of the HIP kernel-artifact DSOs for the vecops matmul operators.  One
// DSO per (operator, operand class, memory placement); the build compiles this
// file once per artifact with
//   -DVECOPS_ARTIFACT_KIND=<0..8>   0 matmul bf16, 1 matmul f32 (bf16 compute), 5 matmul f32 (fp32 compute), 2 matmul i8,
//                                   3 matmul_i8_dequant, 4 matmul_w8a16_group, 6 / 7 / 8 / 10 matmul_fused for bf16 /
//                                   f32 / i8 / f16 operands, 9 matmul f16, 11 / 12 matmul_pack_b to bf16 / i8,
//                                   13 / 14 / 15 matmul_packed_b for bf16 / f32 / i8 a, 16 matmul_runtime_quant,
//                                   17 / 18 matmul_pack_b / matmul_packed_b for f16, 19 matmul_pack_b of u8 weights,
//                                   20 matmul_packed_b for i8 a against u8-packed weights, 21..24 matmul_pack_a to
//                                   bf16 / f16 / i8 / u8, 25..28 matmul_packed_a for bf16 / f32 / f16 / i8 b,
//                                   29 matmul_packed_a for i8 b against a u8-packed a, 30 / 31 matmul_pack_b / _a of
//                                   fp32 kept fp32, 32 / 33 matmul_packed_b / _a in fp32 compute
//   -DVECOPS_ARTIFACT_DEVICE=<0|1>  0: tensors are host memory, staged through HBM here
//                                   1: tensors are HIP device pointers, used in place
//   -DVECOPS_ARTIFACT_GROUP=<G>     group size of kind 4
//   -DVECOPS_ARTIFACT_FAMILY=<F>    vecops::matmul only: the kernel family the artifact's callers require (0: none)
//
// Each DSO exports exactly vecops_kernel_query_v1 (vecops runtime/KernelAbi.h:176)
// and follows the callback contract of runtime/KernelAbi.h:129-131: status codes
// out, message into the caller's VecopsError, no exception crosses, everything in
// the call record is borrowed, and run() returns only when the result is visible
// to the caller (the ABI is synchronous, runtime/CallAbi.h:16).  The context's
// `stream` is read as a hipStream_t (null = the default stream).
#include <hip/hip_runtime_api.h>

#include <cstddef>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "vecops_hip.h"
#include "vecops_rt/abi.h"

#ifndef VECOPS_ARTIFACT_KIND
#error "VECOPS_ARTIFACT_KIND must be defined"
#endif
#ifndef VECOPS_ARTIFACT_DEVICE
#error "VECOPS_ARTIFACT_DEVICE must be defined"
#endif
#ifndef VECOPS_ARTIFACT_GROUP
#define VECOPS_ARTIFACT_GROUP 128
#endif

#define VSTR2(x) #x
#define VSTR(x) VSTR2(x)

namespace {

#if VECOPS_ARTIFACT_DEVICE
#define MEMORY_NAME "device"
constexpr uint32_t kDeviceType = VECOPS_DEVICE_PRIVATE;
#else
#define MEMORY_NAME "host"
constexpr uint32_t kDeviceType = VECOPS_DEVICE_CPU;
#endif

constexpr uint64_t bit(uint32_t dtype) { return uint64_t{1} << (dtype - 1); }

// ---- error reporting (same convention as vecops' generated adapters,
// src/compiler/KernelCompiler.cpp:272-278) ---------------------------------------
int32_t report(VecopsError* error, int32_t code, const std::string& message) {
  if (error != nullptr && error->struct_size >= sizeof(VecopsError)) {
    error->code = code;
    error->message_required = message.size() + 1;
    if (error->message != nullptr && error->message_capacity > 0) {
      const size_t n = message.size() < error->message_capacity - 1 ? message.size() : error->message_capacity - 1;
      memcpy(error->message, message.data(), n);
      error->message[n] = '\0';
    }
  }
  return code;
}

int32_t report_hip(VecopsError* error, const char* what, hipError_t e) {
  return report(error, VECOPS_STATUS_EXECUTION_ERROR, std::string(what) + ": " + hipGetErrorString(e));
}

int32_t report_kernel(VecopsError* error, int32_t rc) { return report(error, rc, vecops_hip_last_error()); }

size_t dtype_bytes(uint32_t dt) {
  switch (dt) {
    case VECOPS_DTYPE_I8: case VECOPS_DTYPE_U8: case VECOPS_DTYPE_BOOL: return 1;
    case VECOPS_DTYPE_I16: case VECOPS_DTYPE_U16: case VECOPS_DTYPE_F16: case VECOPS_DTYPE_BF16: return 2;
    case VECOPS_DTYPE_I32: case VECOPS_DTYPE_U32: case VECOPS_DTYPE_F32: return 4;
    default: return 8;
  }
}

const VecopsTensorView* tensor_arg(const VecopsCall* call, uint32_t index) {
  if (index >= call->num_values) return nullptr;
  const VecopsValue& v = call->values[index];
  return v.kind == VECOPS_VALUE_TENSOR ? &v.value.tensor : nullptr;
}

hipStream_t stream_of(const VecopsCall* call) {
  const VecopsExecutionContext* ctx = call->context;
  if (ctx == nullptr || ctx->struct_size < offsetof(VecopsExecutionContext, stream) + sizeof(void*)) return nullptr;
  return static_cast<hipStream_t>(ctx->stream);
}

// Logical element zero of a view.
char* origin(const VecopsTensorView* t) { return static_cast<char*>(t->data) + t->byte_offset; }

bool fill_operand(const VecopsTensorView* t, void* data, VecopsHipOperand* o) {
  if (t->rank != 2 && t->rank != 3) return false;
  memset(o, 0, sizeof(*o));
  o->data = data;
  o->dtype = t->dtype;
  o->rank = t->rank;
  for (uint32_t i = 0; i < t->rank; ++i) {
    o->sizes[i] = t->sizes[i];
    o->strides[i] = t->strides[i];
  }
  return true;
}

// ---- host staging --------------------------------------------------------------------------
// A host view is mirrored as the smallest byte range that holds all of its
// elements; strides carry over unchanged.  Views with the same origin share one
// device buffer, so a C input that aliases the output stays aliased.
struct Staged {
  const VecopsTensorView* view = nullptr;
  void* device = nullptr;
  size_t bytes = 0;
  bool write_back = false;
  bool owner = true;
};

class Staging {
public:
  explicit Staging(hipStream_t stream) : stream_(stream) {}
  ~Staging() {
    for (auto& s : items_)
      if (s.owner && s.device != nullptr) (void)hipFree(s.device);
    if (workspace_ != nullptr) (void)hipFree(workspace_);
  }

  // Returns the device address of the view's logical element zero (null for an empty view).
  hipError_t add(const VecopsTensorView* t, bool write_back, void** device_origin, std::string* why) {
    *device_origin = nullptr;
    size_t span = 1;
    for (uint32_t i = 0; i < t->rank; ++i) {
      if (t->sizes[i] == 0) return hipSuccess;
      if (t->strides[i] < 0) {
        *why = "negative strides are not supported by the HIP artifacts";
        return hipErrorInvalidValue;
      }
      span += static_cast<size_t>(t->sizes[i] - 1) * static_cast<size_t>(t->strides[i]);
    }
    const size_t bytes = span * dtype_bytes(t->dtype);
    for (auto& s : items_) {
      if (origin(s.view) == origin(t) && s.bytes >= bytes) {
        s.write_back = s.write_back || write_back;
        *device_origin = s.device;
        return hipSuccess;
      }
    }
    Staged s;
    s.view = t;
    s.bytes = bytes;
    s.write_back = write_back;
    hipError_t e = hipMalloc(&s.device, bytes);
    if (e != hipSuccess) return e;
    items_.push_back(s);
    // outputs are uploaded too: a strided output must keep the bytes between its elements
    e = hipMemcpyAsync(s.device, origin(t), bytes, hipMemcpyHostToDevice, stream_);
    *device_origin = s.device;
    return e;
  }

  hipError_t workspace(uint64_t bytes, void** out) {
    *out = nullptr;
    if (bytes == 0) return hipSuccess;
    hipError_t e = hipMalloc(&workspace_, bytes);
    *out = workspace_;
    return e;
  }

  hipError_t finish() {
    for (auto& s : items_) {
      if (!s.write_back) continue;
      hipError_t e = hipMemcpyAsync(origin(s.view), s.device, s.bytes, hipMemcpyDeviceToHost, stream_);
      if (e != hipSuccess) return e;
    }
    return hipStreamSynchronize(stream_);
  }

private:
  hipStream_t stream_;
  std::vector<Staged> items_;
  void* workspace_ = nullptr;
};

// Resolves the device address of each tensor argument: in place for device
// artifacts, through `staging` for host artifacts.
int32_t device_address(const VecopsTensorView* t, bool is_output, Staging* staging, void** out, VecopsError* error) {
#if VECOPS_ARTIFACT_DEVICE
  (void)is_output;
  (void)staging;
  (void)error;
  *out = origin(t);
  return VECOPS_STATUS_OK;
#else
  std::string why;
  hipError_t e = staging->add(t, is_output, out, &why);
  if (e != hipSuccess) {
    if (!why.empty()) return report(error, VECOPS_STATUS_INVALID_ARGUMENT, why);
    return report_hip(error, "staging a host tensor in device memory", e);
  }
  return VECOPS_STATUS_OK;
#endif
}

// Embedding flag of the execution context (vecops: "embedding-defined flags", runtime/CallAbi.h:369-370): the caller
// orders its own work on context->stream, so a device-memory artifact returns once its kernels are enqueued
// instead of waiting for them (the default: ABI functions are synchronous, runtime/CallAbi.h:15-16).
bool stream_ordered(const VecopsCall* call) {
  const VecopsExecutionContext* ctx = call->context;
  return ctx != nullptr && ctx->struct_size >= offsetof(VecopsExecutionContext, flags) + sizeof(uint64_t) &&
         (ctx->flags & VECOPS_HIP_CONTEXT_STREAM_ORDERED) != 0;
}

int32_t finish(const VecopsCall* call, Staging* staging, hipStream_t stream, VecopsError* error) {
#if VECOPS_ARTIFACT_DEVICE
  (void)staging;
  hipError_t e = stream_ordered(call) ? hipSuccess : hipStreamSynchronize(stream);
#else
  (void)call;
  (void)stream;
  hipError_t e = staging->finish();
#endif
  if (e != hipSuccess) return report_hip(error, "waiting for the kernels", e);
  return VECOPS_STATUS_OK;
}

int32_t check_call(const VecopsCall* call, uint32_t expected, VecopsError* error) {
  if (call == nullptr || call->struct_size < offsetof(VecopsCall, context) + sizeof(void*))
    return report(error, VECOPS_STATUS_ABI_MISMATCH, "call record is smaller than ABI v1");
  if (call->num_values != expected || (expected != 0 && call->values == nullptr))
    return report(error, VECOPS_STATUS_INVALID_ARGUMENT, "wrong number of arguments for this artifact");
  return VECOPS_STATUS_OK;
}

// =================================================================================================
#if VECOPS_ARTIFACT_KIND <= 2 || VECOPS_ARTIFACT_KIND == 5 || VECOPS_ARTIFACT_KIND == 9  // vecops::matmul (a, b, c_in?, c)
// =================================================================================================

#if VECOPS_ARTIFACT_KIND == 0
#define OPERANDS "bf16"
#define COMPUTE "bf16"
constexpr uint64_t kInMask = bit(VECOPS_DTYPE_BF16);
constexpr uint64_t kOutMask = bit(VECOPS_DTYPE_F32) | bit(VECOPS_DTYPE_BF16);
#elif VECOPS_ARTIFACT_KIND == 9
#define OPERANDS "f16"
#define COMPUTE "f16"
constexpr uint64_t kInMask = bit(VECOPS_DTYPE_F16);
constexpr uint64_t kOutMask = bit(VECOPS_DTYPE_F32) | bit(VECOPS_DTYPE_F16);
#elif VECOPS_ARTIFACT_KIND == 1
#define OPERANDS "f32"
#define COMPUTE "bf16"
constexpr uint64_t kInMask = bit(VECOPS_DTYPE_F32);
constexpr uint64_t kOutMask = bit(VECOPS_DTYPE_F32) | bit(VECOPS_DTYPE_BF16);
#elif VECOPS_ARTIFACT_KIND == 5
#define OPERANDS "f32"
#define COMPUTE "f32"
#define COMPUTE_CODE VECOPS_HIP_COMPUTE_F32
constexpr uint64_t kInMask = bit(VECOPS_DTYPE_F32);
constexpr uint64_t kOutMask = bit(VECOPS_DTYPE_F32) | bit(VECOPS_DTYPE_BF16);
#else
#define OPERANDS "i8"
#define COMPUTE "i32"
constexpr uint64_t kInMask = bit(VECOPS_DTYPE_I8) | bit(VECOPS_DTYPE_U8);  // either side may be unsigned
constexpr uint64_t kOutMask = bit(VECOPS_DTYPE_I32);
#endif

#ifndef COMPUTE_CODE
#define COMPUTE_CODE VECOPS_HIP_COMPUTE_BF16
#endif
constexpr const char* kOperatorName = "vecops::matmul";
// An artifact built with -DVECOPS_ARTIFACT_FAMILY=<VecopsHipKernelFamily> serves calls that REQUIRE that kernel
// family (the `Family` specialization value; vecops' family_selection::Require<F>, matmul/Family.h:234-239): the
// family is part of its key, and a call the family cannot serve fails with "not applicable".
#ifndef VECOPS_ARTIFACT_FAMILY
#define VECOPS_ARTIFACT_FAMILY 0
#endif
#if VECOPS_ARTIFACT_FAMILY == 0
#define FAMILY_KEY ""
#elif VECOPS_ARTIFACT_FAMILY == 1
#define FAMILY_KEY ";family=tile_256"
#elif VECOPS_ARTIFACT_FAMILY == 2
#define FAMILY_KEY ";family=tile_128"
#elif VECOPS_ARTIFACT_FAMILY == 3
#define FAMILY_KEY ";family=tile_64"
#elif VECOPS_ARTIFACT_FAMILY == 4
#define FAMILY_KEY ";family=skinny"
#elif VECOPS_ARTIFACT_FAMILY == 6
#define FAMILY_KEY ";family=tile_256x128"
#elif VECOPS_ARTIFACT_FAMILY == 7
#define FAMILY_KEY ";family=tile_128x256"
#elif VECOPS_ARTIFACT_FAMILY == 8
#define FAMILY_KEY ";family=tile_256x352"
#elif VECOPS_ARTIFACT_FAMILY == 9
#define FAMILY_KEY ";family=tile_192"
#else
#error "VECOPS_ARTIFACT_FAMILY names no kernel family a caller can require"
#endif
constexpr const char* kKey =
  "vecops::matmul;operands=" OPERANDS ";compute=" COMPUTE FAMILY_KEY ";memory=" MEMORY_NAME ";backend=hip-gfx950";
constexpr VecopsHipFamilyRequest kFamilyRequest = {sizeof(VecopsHipFamilyRequest),
                                                   VECOPS_ARTIFACT_FAMILY ? VECOPS_HIP_SELECT_REQUIRE : VECOPS_HIP_SELECT_AUTOMATIC,
                                                   VECOPS_ARTIFACT_FAMILY, 0};

#define TENSOR_PARAM(NAME, MASK, RANK, OPTIONAL, FLAGS)                                                       \
  {sizeof(VecopsParameterDescriptor), VECOPS_VALUE_TENSOR, NAME,                                              \
   {.tensor = {sizeof(VecopsTensorParameter), MASK, kDeviceType, -1, RANK, OPTIONAL,                          \
               sizeof(VecopsDimensionConstraint), nullptr, nullptr, FLAGS}}}

const VecopsParameterDescriptor kParameters[] = {
  TENSOR_PARAM("a", kInMask, -1, 0, VECOPS_TENSOR_READ),
  TENSOR_PARAM("b", kInMask, -1, 0, VECOPS_TENSOR_READ),
  TENSOR_PARAM("c_in", kOutMask, -1, 1, VECOPS_TENSOR_READ),
  TENSOR_PARAM("c", kOutMask, -1, 0, VECOPS_TENSOR_WRITE),
};

int32_t plan(const VecopsCall* call, VecopsHipOperand ops[4], bool* has_cin, VecopsHipPlan* out, VecopsError* error) {
  if (int32_t rc = check_call(call, 4, error); rc != VECOPS_STATUS_OK) return rc;
  const VecopsTensorView* a = tensor_arg(call, 0);
  const VecopsTensorView* b = tensor_arg(call, 1);
  const VecopsTensorView* cin = tensor_arg(call, 2);
  const VecopsTensorView* c = tensor_arg(call, 3);
  if (a == nullptr || b == nullptr || c == nullptr)
    return report(error, VECOPS_STATUS_INVALID_ARGUMENT, "a, b and c must be tensors");
  *has_cin = cin != nullptr;
  // 16 is a stand-in address with the alignment real allocations have; plan() only reads metadata
  if (!fill_operand(a, reinterpret_cast<void*>(16), &ops[0]) || !fill_operand(b, reinterpret_cast<void*>(16), &ops[1]) ||
      !fill_operand(c, reinterpret_cast<void*>(16), &ops[3]) ||
      (cin != nullptr && !fill_operand(cin, reinterpret_cast<void*>(16), &ops[2])))
    return report(error, VECOPS_STATUS_INVALID_ARGUMENT, "tensors must have rank 2 or 3");
#if VECOPS_ARTIFACT_DEVICE
  ops[0].data = origin(a);
  ops[1].data = origin(b);
  ops[3].data = origin(c);
  if (cin != nullptr) ops[2].data = origin(cin);
#endif
  int32_t rc = vecops_hip_plan_matmul_family(&ops[0], &ops[1], *has_cin ? &ops[2] : nullptr, &ops[3], COMPUTE_CODE,
                                             &kFamilyRequest, out);
  if (rc != VECOPS_STATUS_OK) return report_kernel(error, rc);
  return VECOPS_STATUS_OK;
}

int32_t workspace_impl(const VecopsCall* call, uint64_t* bytes, VecopsError* error) {
  VecopsHipOperand ops[4];
  bool has_cin = false;
  VecopsHipPlan p;
  if (int32_t rc = plan(call, ops, &has_cin, &p, error); rc != VECOPS_STATUS_OK) return rc;
#if VECOPS_ARTIFACT_DEVICE
  *bytes = p.workspace_bytes;  // device scratch the caller must hand in
#else
  *bytes = 0;  // host callers cannot supply device scratch; run() allocates it
#endif
  return VECOPS_STATUS_OK;
}

int32_t run_impl(const VecopsCall* call, VecopsError* error) {
  VecopsHipOperand ops[4];
  bool has_cin = false;
  VecopsHipPlan p;
  if (int32_t rc = plan(call, ops, &has_cin, &p, error); rc != VECOPS_STATUS_OK) return rc;
  if (p.family == VECOPS_HIP_FAMILY_NONE) return VECOPS_STATUS_OK;
  hipStream_t stream = stream_of(call);
  Staging staging(stream);
  void* ws = call->workspace;
  uint64_t ws_size = call->workspace_size;
#if !VECOPS_ARTIFACT_DEVICE
  // c first: if c_in aliases c they share the staged buffer and the write-back flag
  const uint32_t order[4] = {3, 2, 0, 1};
  for (uint32_t idx : order) {
    const VecopsTensorView* t = tensor_arg(call, idx);
    if (t == nullptr) continue;
    void* dev = nullptr;
    if (int32_t rc = device_address(t, idx == 3, &staging, &dev, error); rc != VECOPS_STATUS_OK) return rc;
    ops[idx].data = dev;
  }
  if (hipError_t e = staging.workspace(p.workspace_bytes, &ws); e != hipSuccess)
    return report_hip(error, "allocating split-K scratch", e);
  ws_size = p.workspace_bytes;
#endif
  int32_t rc = vecops_hip_matmul_family(&ops[0], &ops[1], has_cin ? &ops[2] : nullptr, &ops[3], COMPUTE_CODE,
                                        &kFamilyRequest, ws, ws_size, stream);
  if (rc != VECOPS_STATUS_OK) return report_kernel(error, rc);
  return finish(call, &staging, stream, error);
}

// =================================================================================================
#elif VECOPS_ARTIFACT_KIND == 3  // vecops::matmul_i8_dequant (a, b, row_scales, column_scales, correction?, c)
// =================================================================================================

constexpr const char* kOperatorName = "vecops::matmul_i8_dequant";
constexpr const char* kKey =
  "vecops::matmul_i8_dequant;operands=i8;epilogue=row_col_dequant;memory=" MEMORY_NAME ";backend=hip-gfx950";

#define TENSOR_PARAM(NAME, MASK, RANK, OPTIONAL, FLAGS)                                                       \
  {sizeof(VecopsParameterDescriptor), VECOPS_VALUE_TENSOR, NAME,                                              \
   {.tensor = {sizeof(VecopsTensorParameter), MASK, kDeviceType, -1, RANK, OPTIONAL,                          \
               sizeof(VecopsDimensionConstraint), nullptr, nullptr, FLAGS}}}

const VecopsParameterDescriptor kParameters[] = {
  TENSOR_PARAM("a", bit(VECOPS_DTYPE_I8), -1, 0, VECOPS_TENSOR_READ),
  TENSOR_PARAM("b", bit(VECOPS_DTYPE_I8), -1, 0, VECOPS_TENSOR_READ),
  TENSOR_PARAM("row_scales", bit(VECOPS_DTYPE_F32), -1, 0, VECOPS_TENSOR_READ),
  TENSOR_PARAM("column_scales", bit(VECOPS_DTYPE_F32), -1, 0, VECOPS_TENSOR_READ),
  TENSOR_PARAM("correction", bit(VECOPS_DTYPE_I32), -1, 1, VECOPS_TENSOR_READ),
  TENSOR_PARAM("c", bit(VECOPS_DTYPE_F32), -1, 0, VECOPS_TENSOR_WRITE),
};

struct DequantArgs {
  const VecopsTensorView *a, *b, *rs, *cs, *corr, *c;
  int64_t m, n, k;
};

int32_t decode(const VecopsCall* call, DequantArgs* d, VecopsError* error) {
  if (int32_t rc = check_call(call, 6, error); rc != VECOPS_STATUS_OK) return rc;
  d->a = tensor_arg(call, 0);
  d->b = tensor_arg(call, 1);
  d->rs = tensor_arg(call, 2);
  d->cs = tensor_arg(call, 3);
  d->corr = tensor_arg(call, 4);
  d->c = tensor_arg(call, 5);
  if (!d->a || !d->b || !d->rs || !d->cs || !d->c)
    return report(error, VECOPS_STATUS_INVALID_ARGUMENT, "a, b, row_scales, column_scales and c must be tensors");
  if (d->a->rank != 2 || d->b->rank != 2 || d->c->rank != 2 || d->rs->rank != 1 || d->cs->rank != 1 ||
      (d->corr && d->corr->rank != 1))
    return report(error, VECOPS_STATUS_INVALID_ARGUMENT, "matmul_i8_dequant takes rank-2 matrices and rank-1 vectors");
  d->m = d->a->sizes[0];
  d->k = d->a->sizes[1];
  d->n = d->b->sizes[0];
  if (d->b->sizes[1] != d->k || d->c->sizes[0] != d->m || d->c->sizes[1] != d->n || d->rs->sizes[0] != d->m ||
      d->cs->sizes[0] != d->n || (d->corr && d->corr->sizes[0] != d->n))
    return report(error, VECOPS_STATUS_INVALID_ARGUMENT, "matmul_i8_dequant: extents disagree");
  auto unit = [](const VecopsTensorView* t, uint32_t axis) { return t->sizes[axis] <= 1 || t->strides[axis] == 1; };
  if (!unit(d->a, 1) || !unit(d->b, 1) || !unit(d->c, 1) || !unit(d->rs, 0) || !unit(d->cs, 0) ||
      (d->corr && !unit(d->corr, 0)))
    return report(error, VECOPS_STATUS_NOT_APPLICABLE, "matmul_i8_dequant: last axes must be contiguous");
  return VECOPS_STATUS_OK;
}

int32_t workspace_impl(const VecopsCall* call, uint64_t* bytes, VecopsError* error) {
  DequantArgs d;
  if (int32_t rc = decode(call, &d, error); rc != VECOPS_STATUS_OK) return rc;
#if VECOPS_ARTIFACT_DEVICE
  *bytes = vecops_hip_matmul_i8_dequant_workspace(d.m, d.n, d.k);
#else
  *bytes = 0;
#endif
  return VECOPS_STATUS_OK;
}

int32_t run_impl(const VecopsCall* call, VecopsError* error) {
  DequantArgs d;
  if (int32_t rc = decode(call, &d, error); rc != VECOPS_STATUS_OK) return rc;
  if (d.m == 0 || d.n == 0) return VECOPS_STATUS_OK;
  hipStream_t stream = stream_of(call);
  Staging staging(stream);
  void *a = nullptr, *b = nullptr, *rs = nullptr, *cs = nullptr, *corr = nullptr, *c = nullptr;
  int32_t rc;
  if ((rc = device_address(d.c, true, &staging, &c, error)) != VECOPS_STATUS_OK) return rc;
  if ((rc = device_address(d.a, false, &staging, &a, error)) != VECOPS_STATUS_OK) return rc;
  if ((rc = device_address(d.b, false, &staging, &b, error)) != VECOPS_STATUS_OK) return rc;
  if ((rc = device_address(d.rs, false, &staging, &rs, error)) != VECOPS_STATUS_OK) return rc;
  if ((rc = device_address(d.cs, false, &staging, &cs, error)) != VECOPS_STATUS_OK) return rc;
  if (d.corr && (rc = device_address(d.corr, false, &staging, &corr, error)) != VECOPS_STATUS_OK) return rc;
  void* ws = call->workspace;
  uint64_t ws_size = call->workspace_size;
#if !VECOPS_ARTIFACT_DEVICE
  ws_size = vecops_hip_matmul_i8_dequant_workspace(d.m, d.n, d.k);
  if (hipError_t e = staging.workspace(ws_size, &ws); e != hipSuccess)
    return report_hip(error, "allocating split-K scratch", e);
#endif
  rc = vecops_hip_matmul_i8_dequant(static_cast<const int8_t*>(a), d.a->strides[0], static_cast<const int8_t*>(b),
                                    d.b->strides[0], static_cast<const float*>(rs), static_cast<const float*>(cs),
                                    static_cast<const int32_t*>(corr), static_cast<float*>(c), d.c->strides[0], d.m,
                                    d.n, d.k, ws, ws_size, stream);
  if (rc != VECOPS_STATUS_OK) return report_kernel(error, rc);
  return finish(call, &staging, stream, error);
}

// =================================================================================================
#elif VECOPS_ARTIFACT_KIND >= 6 && VECOPS_ARTIFACT_KIND != 9 && VECOPS_ARTIFACT_KIND < 11  // vecops::matmul_fused (a, b, c_in?, row_scales?, column_scales?, 5 scalars, c)
// =================================================================================================

#if VECOPS_ARTIFACT_KIND == 6
#define OPERANDS "bf16"
constexpr uint64_t kInMask = bit(VECOPS_DTYPE_BF16);
#elif VECOPS_ARTIFACT_KIND == 7
#define OPERANDS "f32"
constexpr uint64_t kInMask = bit(VECOPS_DTYPE_F32);
#elif VECOPS_ARTIFACT_KIND == 10
#define OPERANDS "f16"
constexpr uint64_t kInMask = bit(VECOPS_DTYPE_F16);
#else
#define OPERANDS "i8"
constexpr uint64_t kInMask = bit(VECOPS_DTYPE_I8) | bit(VECOPS_DTYPE_U8);
#endif
#if VECOPS_ARTIFACT_KIND == 8
constexpr uint64_t kCinMask = bit(VECOPS_DTYPE_I32);
constexpr uint64_t kOutMask = bit(VECOPS_DTYPE_F32) | bit(VECOPS_DTYPE_U8) | bit(VECOPS_DTYPE_I8);
#elif VECOPS_ARTIFACT_KIND == 10
constexpr uint64_t kCinMask = bit(VECOPS_DTYPE_F32) | bit(VECOPS_DTYPE_F16);
constexpr uint64_t kOutMask = bit(VECOPS_DTYPE_F32) | bit(VECOPS_DTYPE_F16);
#else
constexpr uint64_t kCinMask = bit(VECOPS_DTYPE_F32) | bit(VECOPS_DTYPE_BF16);
constexpr uint64_t kOutMask = bit(VECOPS_DTYPE_F32) | bit(VECOPS_DTYPE_BF16);
#endif

constexpr const char* kOperatorName = "vecops::matmul_fused";
constexpr const char* kKey = "vecops::matmul_fused;operands=" OPERANDS ";memory=" MEMORY_NAME ";backend=hip-gfx950";

#define TENSOR_PARAM(NAME, MASK, RANK, OPTIONAL, FLAGS)                                                       \
  {sizeof(VecopsParameterDescriptor), VECOPS_VALUE_TENSOR, NAME,                                              \
   {.tensor = {sizeof(VecopsTensorParameter), MASK, kDeviceType, -1, RANK, OPTIONAL,                          \
               sizeof(VecopsDimensionConstraint), nullptr, nullptr, FLAGS}}}
#define SCALAR_PARAM(NAME, MASK) \
  {sizeof(VecopsParameterDescriptor), VECOPS_VALUE_SCALAR, NAME, {.scalar = {sizeof(VecopsScalarParameter), MASK}}}

constexpr uint64_t kRealMask = bit(VECOPS_DTYPE_F32) | bit(VECOPS_DTYPE_F64);

const VecopsParameterDescriptor kParameters[] = {
  TENSOR_PARAM("a", kInMask, -1, 0, VECOPS_TENSOR_READ),
  TENSOR_PARAM("b", kInMask, -1, 0, VECOPS_TENSOR_READ),
  TENSOR_PARAM("c_in", kCinMask, -1, 1, VECOPS_TENSOR_READ),
  TENSOR_PARAM("row_scales", bit(VECOPS_DTYPE_F32), -1, 1, VECOPS_TENSOR_READ),
  TENSOR_PARAM("column_scales", bit(VECOPS_DTYPE_F32), -1, 1, VECOPS_TENSOR_READ),
  SCALAR_PARAM("activation", bit(VECOPS_DTYPE_I64) | bit(VECOPS_DTYPE_I32)),
  SCALAR_PARAM("scale", kRealMask),
  SCALAR_PARAM("shift", kRealMask),
  SCALAR_PARAM("clamp_lo", kRealMask),
  SCALAR_PARAM("clamp_hi", kRealMask),
  TENSOR_PARAM("c", kOutMask, -1, 0, VECOPS_TENSOR_WRITE),
};

// Scalars travel as 64-bit storage whatever their dtype says (runtime/CallAbi.h: i64 / u64 / f64).
bool scalar_arg(const VecopsCall* call, uint32_t index, const VecopsScalar** out) {
  if (index >= call->num_values || call->values[index].kind != VECOPS_VALUE_SCALAR) return false;
  *out = &call->values[index].value.scalar;
  return true;
}

struct FusedArgs {
  const VecopsTensorView *a, *b, *cin, *rs, *cs, *c;
  VecopsHipOperand ops[4];  // a, b, c_in, c
  VecopsHipEpilogue ep;
};

int32_t decode(const VecopsCall* call, FusedArgs* f, VecopsError* error) {
  if (int32_t rc = check_call(call, 11, error); rc != VECOPS_STATUS_OK) return rc;
  f->a = tensor_arg(call, 0);
  f->b = tensor_arg(call, 1);
  f->cin = tensor_arg(call, 2);
  f->rs = tensor_arg(call, 3);
  f->cs = tensor_arg(call, 4);
  f->c = tensor_arg(call, 10);
  if (f->a == nullptr || f->b == nullptr || f->c == nullptr)
    return report(error, VECOPS_STATUS_INVALID_ARGUMENT, "a, b and c must be tensors");
  const VecopsScalar* s[5];
  for (uint32_t i = 0; i < 5; ++i)
    if (!scalar_arg(call, 5 + i, &s[i]))
      return report(error, VECOPS_STATUS_INVALID_ARGUMENT, "activation, scale, shift, clamp_lo and clamp_hi must be scalars");
  if (s[0]->value.i64 < 0 || s[0]->value.i64 > VECOPS_HIP_ACT_SILU)
    return report(error, VECOPS_STATUS_INVALID_ARGUMENT, "activation must be 0 (none), 1 relu, 2 clamp, 3 sigmoid or 4 silu");
  auto unit = [](const VecopsTensorView* t) { return t->rank == 1 && (t->sizes[0] <= 1 || t->strides[0] == 1); };
  if ((f->rs && !unit(f->rs)) || (f->cs && !unit(f->cs)))
    return report(error, VECOPS_STATUS_INVALID_ARGUMENT, "row_scales and column_scales must be dense rank-1 tensors");
  memset(&f->ep, 0, sizeof(f->ep));
  f->ep.struct_size = sizeof(f->ep);
  f->ep.activation = static_cast<uint32_t>(s[0]->value.i64);
  const float scale = static_cast<float>(s[1]->value.f64), shift = static_cast<float>(s[2]->value.f64);
  // a scale of exactly 1 and a shift of exactly 0 stand for "no such step" (the call ABI has no optional scalars)
  if (scale != 1.0f) f->ep.flags |= VECOPS_HIP_EPILOGUE_SCALE;
  if (shift != 0.0f) f->ep.flags |= VECOPS_HIP_EPILOGUE_SHIFT;
  f->ep.scale = scale;
  f->ep.shift = shift;
  f->ep.clamp_lo = static_cast<float>(s[3]->value.f64);
  f->ep.clamp_hi = static_cast<float>(s[4]->value.f64);
  // 16 is a stand-in address with the alignment real allocations have; planning only reads metadata
  if (!fill_operand(f->a, reinterpret_cast<void*>(16), &f->ops[0]) || !fill_operand(f->b, reinterpret_cast<void*>(16), &f->ops[1]) ||
      !fill_operand(f->c, reinterpret_cast<void*>(16), &f->ops[3]) ||
      (f->cin != nullptr && !fill_operand(f->cin, reinterpret_cast<void*>(16), &f->ops[2])))
    return report(error, VECOPS_STATUS_INVALID_ARGUMENT, "tensors must have rank 2 or 3");
  const int64_t batch = f->a->rank == 3 ? f->a->sizes[0] : 1;
  if ((f->rs && f->rs->sizes[0] != batch * f->a->sizes[f->a->rank - 2]) || (f->cs && f->cs->sizes[0] != f->b->sizes[f->b->rank - 2]))
    return report(error, VECOPS_STATUS_INVALID_ARGUMENT, "scale vectors must have one entry per row of a / per row of b");
#if VECOPS_ARTIFACT_DEVICE
  f->ops[0].data = origin(f->a);
  f->ops[1].data = origin(f->b);
  f->ops[3].data = origin(f->c);
  if (f->cin != nullptr) f->ops[2].data = origin(f->cin);
  f->ep.row_scales = f->rs ? reinterpret_cast<const float*>(origin(f->rs)) : nullptr;
  f->ep.column_scales = f->cs ? reinterpret_cast<const float*>(origin(f->cs)) : nullptr;
#else
  // stand-ins so that planning sees which scale vectors exist
  f->ep.row_scales = f->rs ? reinterpret_cast<const float*>(16) : nullptr;
  f->ep.column_scales = f->cs ? reinterpret_cast<const float*>(16) : nullptr;
#endif
  return VECOPS_STATUS_OK;
}

int32_t plan(FusedArgs* f, VecopsHipPlan* out, VecopsError* error) {
  int32_t rc = vecops_hip_plan_matmul_fused(&f->ops[0], &f->ops[1], f->cin ? &f->ops[2] : nullptr, &f->ops[3],
                                            VECOPS_HIP_COMPUTE_BF16, &f->ep, out);
  return rc == VECOPS_STATUS_OK ? rc : report_kernel(error, rc);
}

int32_t workspace_impl(const VecopsCall* call, uint64_t* bytes, VecopsError* error) {
  FusedArgs f;
  VecopsHipPlan p;
  if (int32_t rc = decode(call, &f, error); rc != VECOPS_STATUS_OK) return rc;
  if (int32_t rc = plan(&f, &p, error); rc != VECOPS_STATUS_OK) return rc;
#if VECOPS_ARTIFACT_DEVICE
  *bytes = p.workspace_bytes;
#else
  *bytes = 0;
#endif
  return VECOPS_STATUS_OK;
}

int32_t run_impl(const VecopsCall* call, VecopsError* error) {
  FusedArgs f;
  VecopsHipPlan p;
  if (int32_t rc = decode(call, &f, error); rc != VECOPS_STATUS_OK) return rc;
  if (int32_t rc = plan(&f, &p, error); rc != VECOPS_STATUS_OK) return rc;
  if (p.family == VECOPS_HIP_FAMILY_NONE) return VECOPS_STATUS_OK;
  hipStream_t stream = stream_of(call);
  Staging staging(stream);
  void* ws = call->workspace;
  uint64_t ws_size = call->workspace_size;
#if !VECOPS_ARTIFACT_DEVICE
  // c first: if c_in aliases c they share the staged buffer and the write-back flag
  const VecopsTensorView* views[4] = {f.a, f.b, f.cin, f.c};
  const uint32_t order[4] = {3, 2, 0, 1};
  for (uint32_t idx : order) {
    if (views[idx] == nullptr) continue;
    void* dev = nullptr;
    if (int32_t rc = device_address(views[idx], idx == 3, &staging, &dev, error); rc != VECOPS_STATUS_OK) return rc;
    f.ops[idx].data = dev;
  }
  void* dev = nullptr;
  if (f.rs) {
    if (int32_t rc = device_address(f.rs, false, &staging, &dev, error); rc != VECOPS_STATUS_OK) return rc;
    f.ep.row_scales = static_cast<const float*>(dev);
  }
  if (f.cs) {
    if (int32_t rc = device_address(f.cs, false, &staging, &dev, error); rc != VECOPS_STATUS_OK) return rc;
    f.ep.column_scales = static_cast<const float*>(dev);
  }
  if (hipError_t e = staging.workspace(p.workspace_bytes, &ws); e != hipSuccess)
    return report_hip(error, "allocating split-K scratch", e);
  ws_size = p.workspace_bytes;
#endif
  int32_t rc = vecops_hip_matmul_fused(&f.ops[0], &f.ops[1], f.cin ? &f.ops[2] : nullptr, &f.ops[3],
                                       VECOPS_HIP_COMPUTE_BF16, &f.ep, ws, ws_size, stream);
  if (rc != VECOPS_STATUS_OK) return report_kernel(error, rc);
  return finish(call, &staging, stream, error);
}

// =================================================================================================
#elif VECOPS_ARTIFACT_KIND == 11 || VECOPS_ARTIFACT_KIND == 12 || VECOPS_ARTIFACT_KIND == 17 || VECOPS_ARTIFACT_KIND == 19 || \
  (VECOPS_ARTIFACT_KIND >= 21 && VECOPS_ARTIFACT_KIND <= 24) || VECOPS_ARTIFACT_KIND == 30 || VECOPS_ARTIFACT_KIND == 31
// vecops::matmul_pack_b (b, a_zero_point, packed, compensation?)  /  vecops::matmul_pack_a (a, packed)
// =================================================================================================

#if (VECOPS_ARTIFACT_KIND >= 21 && VECOPS_ARTIFACT_KIND <= 24) || VECOPS_ARTIFACT_KIND == 31
#define VECOPS_PACK_SIDE_A 1
#else
#define VECOPS_PACK_SIDE_A 0
#endif
#if VECOPS_ARTIFACT_KIND == 30 || VECOPS_ARTIFACT_KIND == 31
#define OPERANDS "f32"
constexpr uint64_t kInMask = bit(VECOPS_DTYPE_F32);  // elements stay fp32: the pack of the fp32-compute atom
constexpr uint32_t kPackedDtype = VECOPS_DTYPE_F32;
#elif VECOPS_ARTIFACT_KIND == 11 || VECOPS_ARTIFACT_KIND == 21
#define OPERANDS "bf16"
constexpr uint64_t kInMask = bit(VECOPS_DTYPE_BF16) | bit(VECOPS_DTYPE_F32);  // fp32 sources are rounded to bf16
constexpr uint32_t kPackedDtype = VECOPS_DTYPE_BF16;
#elif VECOPS_ARTIFACT_KIND == 17 || VECOPS_ARTIFACT_KIND == 22
#define OPERANDS "f16"
constexpr uint64_t kInMask = bit(VECOPS_DTYPE_F16);
constexpr uint32_t kPackedDtype = VECOPS_DTYPE_F16;
#elif VECOPS_ARTIFACT_KIND == 19 || VECOPS_ARTIFACT_KIND == 24
#define OPERANDS "u8"
constexpr uint64_t kInMask = bit(VECOPS_DTYPE_U8);
constexpr uint32_t kPackedDtype = VECOPS_DTYPE_U8;
#else
#define OPERANDS "i8"
constexpr uint64_t kInMask = bit(VECOPS_DTYPE_I8);
constexpr uint32_t kPackedDtype = VECOPS_DTYPE_I8;
#endif
#if VECOPS_PACK_SIDE_A
#define PACK_OPERATOR "vecops::matmul_pack_a"
#else
#define PACK_OPERATOR "vecops::matmul_pack_b"
#endif
constexpr const char* kOperatorName = PACK_OPERATOR;
constexpr const char* kKey = PACK_OPERATOR ";operands=" OPERANDS ";memory=" MEMORY_NAME ";backend=hip-gfx950";

#define TENSOR_PARAM(NAME, MASK, RANK, OPTIONAL, FLAGS)                                                       \
  {sizeof(VecopsParameterDescriptor), VECOPS_VALUE_TENSOR, NAME,                                              \
   {.tensor = {sizeof(VecopsTensorParameter), MASK, kDeviceType, -1, RANK, OPTIONAL,                          \
               sizeof(VecopsDimensionConstraint), nullptr, nullptr, FLAGS}}}

#if VECOPS_PACK_SIDE_A
const VecopsParameterDescriptor kParameters[] = {
  TENSOR_PARAM("a", kInMask, -1, 0, VECOPS_TENSOR_READ),
  TENSOR_PARAM("packed", bit(VECOPS_DTYPE_U8), -1, 0, VECOPS_TENSOR_WRITE),
};
constexpr uint32_t kArguments = 2, kPackedAt = 1;
#else
const VecopsParameterDescriptor kParameters[] = {
  TENSOR_PARAM("b", kInMask, -1, 0, VECOPS_TENSOR_READ),
  {sizeof(VecopsParameterDescriptor), VECOPS_VALUE_SCALAR, "a_zero_point",
   {.scalar = {sizeof(VecopsScalarParameter), bit(VECOPS_DTYPE_I64) | bit(VECOPS_DTYPE_I32)}}},
  TENSOR_PARAM("packed", bit(VECOPS_DTYPE_U8), -1, 0, VECOPS_TENSOR_WRITE),
  TENSOR_PARAM("compensation", bit(VECOPS_DTYPE_I32), -1, 1, VECOPS_TENSOR_WRITE),
};
constexpr uint32_t kArguments = 4, kPackedAt = 2;
#endif

int32_t workspace_impl(const VecopsCall* call, uint64_t* bytes, VecopsError* error) {
  if (int32_t rc = check_call(call, kArguments, error); rc != VECOPS_STATUS_OK) return rc;
  *bytes = 0;
  return VECOPS_STATUS_OK;
}

int32_t run_impl(const VecopsCall* call, VecopsError* error) {
  if (int32_t rc = check_call(call, kArguments, error); rc != VECOPS_STATUS_OK) return rc;
  const VecopsTensorView* b = tensor_arg(call, 0);
  const VecopsTensorView* packed = tensor_arg(call, kPackedAt);
#if VECOPS_PACK_SIDE_A
  const VecopsTensorView* comp = nullptr;
  if (b == nullptr || packed == nullptr) return report(error, VECOPS_STATUS_INVALID_ARGUMENT, "a and packed must be tensors");
#else
  const VecopsTensorView* comp = tensor_arg(call, 3);
  if (b == nullptr || packed == nullptr || call->values[1].kind != VECOPS_VALUE_SCALAR)
    return report(error, VECOPS_STATUS_INVALID_ARGUMENT, "b and packed must be tensors, a_zero_point a scalar");
#endif
  if (b->rank != 2 || packed->rank != 1 || (packed->sizes[0] > 1 && packed->strides[0] != 1) ||
      (comp && (comp->rank != 1 || (comp->sizes[0] > 1 && comp->strides[0] != 1))))
    return report(error, VECOPS_STATUS_INVALID_ARGUMENT, PACK_OPERATOR " takes a rank-2 source and dense rank-1 outputs");
  const int64_t n = b->sizes[0], k = b->sizes[1];
  const uint64_t need = vecops_hip_packed_b_bytes(kPackedDtype, n, k);   // (one format serves both sides)
  if (static_cast<uint64_t>(packed->sizes[0]) < need)
    return report(error, VECOPS_STATUS_INVALID_ARGUMENT,
                  "packed holds " + std::to_string(packed->sizes[0]) + " bytes, " + std::to_string(need) + " are needed");
  if (comp && (kPackedDtype != VECOPS_DTYPE_I8 || comp->sizes[0] != n))
    return report(error, VECOPS_STATUS_INVALID_ARGUMENT, "compensation goes with an int8 b and has N entries");
  if (need == 0) return VECOPS_STATUS_OK;
  hipStream_t stream = stream_of(call);
  Staging staging(stream);
  void *b_dev = nullptr, *p_dev = nullptr, *c_dev = nullptr;
  int32_t rc;
  if ((rc = device_address(packed, true, &staging, &p_dev, error)) != VECOPS_STATUS_OK) return rc;
  if ((rc = device_address(b, false, &staging, &b_dev, error)) != VECOPS_STATUS_OK) return rc;
  if (comp && (rc = device_address(comp, true, &staging, &c_dev, error)) != VECOPS_STATUS_OK) return rc;
  VecopsHipOperand ob;
  if (!fill_operand(b, b_dev, &ob)) return report(error, VECOPS_STATUS_INVALID_ARGUMENT, "the source must have rank 2");
#if VECOPS_PACK_SIDE_A || VECOPS_ARTIFACT_KIND == 30
  rc = vecops_hip_pack_as(&ob, kPackedDtype, p_dev, static_cast<uint64_t>(packed->sizes[0]), stream);
#else
  if (comp)
    rc = vecops_hip_pack_b_compensated(&ob, static_cast<int32_t>(call->values[1].value.scalar.value.i64), p_dev,
                                       static_cast<uint64_t>(packed->sizes[0]), static_cast<int32_t*>(c_dev), stream);
  else
    rc = vecops_hip_pack_b(&ob, p_dev, static_cast<uint64_t>(packed->sizes[0]), stream);
#endif
  if (rc != VECOPS_STATUS_OK) return report_kernel(error, rc);
  return finish(call, &staging, stream, error);
}

// =================================================================================================
#elif (VECOPS_ARTIFACT_KIND >= 13 && VECOPS_ARTIFACT_KIND <= 15) || VECOPS_ARTIFACT_KIND == 18 || VECOPS_ARTIFACT_KIND == 20 || \
  (VECOPS_ARTIFACT_KIND >= 25 && VECOPS_ARTIFACT_KIND <= 29) || VECOPS_ARTIFACT_KIND == 32 || VECOPS_ARTIFACT_KIND == 33
// vecops::matmul_packed_b (a, packed_b, c_in?, c)  /  vecops::matmul_packed_a (packed_a, b, c_in?, c)
// =================================================================================================

#if (VECOPS_ARTIFACT_KIND >= 25 && VECOPS_ARTIFACT_KIND <= 29) || VECOPS_ARTIFACT_KIND == 33
#define VECOPS_PACK_SIDE_A 1
#else
#define VECOPS_PACK_SIDE_A 0
#endif
#if VECOPS_ARTIFACT_KIND == 32 || VECOPS_ARTIFACT_KIND == 33
#define OPERANDS "f32;compute=f32"
constexpr uint64_t kInMask = bit(VECOPS_DTYPE_F32);
#elif VECOPS_ARTIFACT_KIND == 13 || VECOPS_ARTIFACT_KIND == 25
#define OPERANDS "bf16"
constexpr uint64_t kInMask = bit(VECOPS_DTYPE_BF16);
#elif VECOPS_ARTIFACT_KIND == 14 || VECOPS_ARTIFACT_KIND == 26
#define OPERANDS "f32"
constexpr uint64_t kInMask = bit(VECOPS_DTYPE_F32);
#elif VECOPS_ARTIFACT_KIND == 18 || VECOPS_ARTIFACT_KIND == 27
#define OPERANDS "f16"
constexpr uint64_t kInMask = bit(VECOPS_DTYPE_F16);
#elif VECOPS_ARTIFACT_KIND == 20 || VECOPS_ARTIFACT_KIND == 29
#define OPERANDS "i8;packed=u8"
constexpr uint64_t kInMask = bit(VECOPS_DTYPE_I8) | bit(VECOPS_DTYPE_U8);
#else
#define OPERANDS "i8"
constexpr uint64_t kInMask = bit(VECOPS_DTYPE_I8) | bit(VECOPS_DTYPE_U8);
#endif
#if VECOPS_ARTIFACT_KIND == 32 || VECOPS_ARTIFACT_KIND == 33
constexpr uint64_t kOutMask = bit(VECOPS_DTYPE_F32);
constexpr uint32_t kPackedDtype = VECOPS_DTYPE_F32;
#elif VECOPS_ARTIFACT_KIND == 15 || VECOPS_ARTIFACT_KIND == 28
constexpr uint64_t kOutMask = bit(VECOPS_DTYPE_I32);
constexpr uint32_t kPackedDtype = VECOPS_DTYPE_I8;
#elif VECOPS_ARTIFACT_KIND == 20 || VECOPS_ARTIFACT_KIND == 29
constexpr uint64_t kOutMask = bit(VECOPS_DTYPE_I32);
constexpr uint32_t kPackedDtype = VECOPS_DTYPE_U8;
#elif VECOPS_ARTIFACT_KIND == 18 || VECOPS_ARTIFACT_KIND == 27
constexpr uint64_t kOutMask = bit(VECOPS_DTYPE_F32) | bit(VECOPS_DTYPE_F16);
constexpr uint32_t kPackedDtype = VECOPS_DTYPE_F16;
#else
constexpr uint64_t kOutMask = bit(VECOPS_DTYPE_F32) | bit(VECOPS_DTYPE_BF16);
constexpr uint32_t kPackedDtype = VECOPS_DTYPE_BF16;
#endif
#if VECOPS_PACK_SIDE_A
#define PACKED_OPERATOR "vecops::matmul_packed_a"
constexpr uint32_t kDenseAt = 1, kPackedAt = 0;
#else
#define PACKED_OPERATOR "vecops::matmul_packed_b"
constexpr uint32_t kDenseAt = 0, kPackedAt = 1;
#endif
constexpr const char* kOperatorName = PACKED_OPERATOR;
constexpr const char* kKey = PACKED_OPERATOR ";operands=" OPERANDS ";memory=" MEMORY_NAME ";backend=hip-gfx950";

#define TENSOR_PARAM(NAME, MASK, RANK, OPTIONAL, FLAGS)                                                       \
  {sizeof(VecopsParameterDescriptor), VECOPS_VALUE_TENSOR, NAME,                                              \
   {.tensor = {sizeof(VecopsTensorParameter), MASK, kDeviceType, -1, RANK, OPTIONAL,                          \
               sizeof(VecopsDimensionConstraint), nullptr, nullptr, FLAGS}}}

const VecopsParameterDescriptor kParameters[] = {
#if VECOPS_PACK_SIDE_A
  TENSOR_PARAM("packed_a", bit(VECOPS_DTYPE_U8), -1, 0, VECOPS_TENSOR_READ),
  TENSOR_PARAM("b", kInMask, -1, 0, VECOPS_TENSOR_READ),
#else
  TENSOR_PARAM("a", kInMask, -1, 0, VECOPS_TENSOR_READ),
  TENSOR_PARAM("packed_b", bit(VECOPS_DTYPE_U8), -1, 0, VECOPS_TENSOR_READ),
#endif
  TENSOR_PARAM("c_in", kOutMask, -1, 1, VECOPS_TENSOR_READ),
  TENSOR_PARAM("c", kOutMask, -1, 0, VECOPS_TENSOR_WRITE),
};

// `a` is the dense operand ([..,M,K] of matmul_packed_b, [..,N,K] of matmul_packed_a), `n` the rows of the packed one
// (N resp. M), taken from c.
struct PackedArgs {
  const VecopsTensorView *a, *packed, *cin, *c;
  VecopsHipOperand oa, ocin, oc;
  int64_t n;
};

int32_t plan_packed(const PackedArgs& d, VecopsHipPlan* plan) {
#if VECOPS_PACK_SIDE_A
  return vecops_hip_plan_matmul_packed_a(kPackedDtype, d.n, &d.oa, d.cin ? &d.ocin : nullptr, &d.oc, plan);
#else
  return vecops_hip_plan_matmul_packed_b(&d.oa, kPackedDtype, d.n, d.cin ? &d.ocin : nullptr, &d.oc, plan);
#endif
}

int32_t decode(const VecopsCall* call, PackedArgs* d, VecopsHipPlan* plan, VecopsError* error) {
  if (int32_t rc = check_call(call, 4, error); rc != VECOPS_STATUS_OK) return rc;
  d->a = tensor_arg(call, kDenseAt);
  d->packed = tensor_arg(call, kPackedAt);
  d->cin = tensor_arg(call, 2);
  d->c = tensor_arg(call, 3);
  if (d->a == nullptr || d->packed == nullptr || d->c == nullptr)
    return report(error, VECOPS_STATUS_INVALID_ARGUMENT, "the dense operand, the packed operand and c must be tensors");
  if (d->packed->rank != 1 || (d->packed->sizes[0] > 1 && d->packed->strides[0] != 1))
    return report(error, VECOPS_STATUS_INVALID_ARGUMENT, "the packed operand must be a dense rank-1 byte tensor");
  if (!fill_operand(d->a, reinterpret_cast<void*>(16), &d->oa) || !fill_operand(d->c, reinterpret_cast<void*>(16), &d->oc) ||
      (d->cin != nullptr && !fill_operand(d->cin, reinterpret_cast<void*>(16), &d->ocin)))
    return report(error, VECOPS_STATUS_INVALID_ARGUMENT, "tensors must have rank 2 or 3");
  d->n = d->c->sizes[d->c->rank - (VECOPS_PACK_SIDE_A ? 2 : 1)];
  const int64_t k = d->a->sizes[d->a->rank - 1];
  const uint64_t need = vecops_hip_packed_b_bytes(kPackedDtype, d->n, k);
  if (static_cast<uint64_t>(d->packed->sizes[0]) < need)
    return report(error, VECOPS_STATUS_INVALID_ARGUMENT,
                  "the packed operand holds " + std::to_string(d->packed->sizes[0]) + " bytes, " + std::to_string(need) +
                    " are needed for " + std::to_string(d->n) + " rows, K = " + std::to_string(k));
#if VECOPS_ARTIFACT_DEVICE
  d->oa.data = origin(d->a);
  d->oc.data = origin(d->c);
  if (d->cin != nullptr) d->ocin.data = origin(d->cin);
#endif
  int32_t rc = plan_packed(*d, plan);
  return rc == VECOPS_STATUS_OK ? rc : report_kernel(error, rc);
}

int32_t workspace_impl(const VecopsCall* call, uint64_t* bytes, VecopsError* error) {
  PackedArgs d;
  VecopsHipPlan p;
  if (int32_t rc = decode(call, &d, &p, error); rc != VECOPS_STATUS_OK) return rc;
#if VECOPS_ARTIFACT_DEVICE
  *bytes = p.workspace_bytes;
#else
  *bytes = 0;
#endif
  return VECOPS_STATUS_OK;
}

int32_t run_impl(const VecopsCall* call, VecopsError* error) {
  PackedArgs d;
  VecopsHipPlan p;
  if (int32_t rc = decode(call, &d, &p, error); rc != VECOPS_STATUS_OK) return rc;
  if (p.family == VECOPS_HIP_FAMILY_NONE) return VECOPS_STATUS_OK;
  hipStream_t stream = stream_of(call);
  Staging staging(stream);
  void* ws = call->workspace;
  uint64_t ws_size = call->workspace_size;
  void* packed_dev = nullptr;
  int32_t rc;
#if VECOPS_ARTIFACT_DEVICE
  packed_dev = origin(d.packed);
#else
  void* dev = nullptr;
  if ((rc = device_address(d.c, true, &staging, &dev, error)) != VECOPS_STATUS_OK) return rc;
  d.oc.data = dev;
  if (d.cin && (rc = device_address(d.cin, false, &staging, &dev, error)) != VECOPS_STATUS_OK) return rc;
  if (d.cin) d.ocin.data = dev;
  if ((rc = device_address(d.a, false, &staging, &dev, error)) != VECOPS_STATUS_OK) return rc;
  d.oa.data = dev;
  if ((rc = device_address(d.packed, false, &staging, &packed_dev, error)) != VECOPS_STATUS_OK) return rc;
  if (hipError_t e = staging.workspace(p.workspace_bytes, &ws); e != hipSuccess)
    return report_hip(error, "allocating split-K scratch", e);
  ws_size = p.workspace_bytes;
#endif
#if VECOPS_PACK_SIDE_A
  rc = vecops_hip_matmul_packed_a(packed_dev, kPackedDtype, d.n, &d.oa, d.cin ? &d.ocin : nullptr, &d.oc, ws, ws_size, stream);
#else
  rc = vecops_hip_matmul_packed_b(&d.oa, packed_dev, kPackedDtype, d.n, d.cin ? &d.ocin : nullptr, &d.oc, ws, ws_size,
                                  stream);
#endif
  if (rc != VECOPS_STATUS_OK) return report_kernel(error, rc);
  return finish(call, &staging, stream, error);
}

// =================================================================================================
#elif VECOPS_ARTIFACT_KIND == 16  // vecops::matmul_runtime_quant (a, b, multipliers, zero_point, row_scales, column_scales, correction?, c)
// =================================================================================================

constexpr const char* kOperatorName = "vecops::matmul_runtime_quant";
constexpr const char* kKey =
  "vecops::matmul_runtime_quant;operands=f32_i8;epilogue=row_col_dequant;memory=" MEMORY_NAME ";backend=hip-gfx950";

#define TENSOR_PARAM(NAME, MASK, RANK, OPTIONAL, FLAGS)                                                       \
  {sizeof(VecopsParameterDescriptor), VECOPS_VALUE_TENSOR, NAME,                                              \
   {.tensor = {sizeof(VecopsTensorParameter), MASK, kDeviceType, -1, RANK, OPTIONAL,                          \
               sizeof(VecopsDimensionConstraint), nullptr, nullptr, FLAGS}}}

const VecopsParameterDescriptor kParameters[] = {
  TENSOR_PARAM("a", bit(VECOPS_DTYPE_F32), -1, 0, VECOPS_TENSOR_READ),
  TENSOR_PARAM("b", bit(VECOPS_DTYPE_I8), -1, 0, VECOPS_TENSOR_READ),
  TENSOR_PARAM("multipliers", bit(VECOPS_DTYPE_F32), -1, 0, VECOPS_TENSOR_READ),
  {sizeof(VecopsParameterDescriptor), VECOPS_VALUE_SCALAR, "zero_point",
   {.scalar = {sizeof(VecopsScalarParameter), bit(VECOPS_DTYPE_I64) | bit(VECOPS_DTYPE_I32)}}},
  TENSOR_PARAM("row_scales", bit(VECOPS_DTYPE_F32), -1, 0, VECOPS_TENSOR_READ),
  TENSOR_PARAM("column_scales", bit(VECOPS_DTYPE_F32), -1, 0, VECOPS_TENSOR_READ),
  TENSOR_PARAM("correction", bit(VECOPS_DTYPE_I32), -1, 1, VECOPS_TENSOR_READ),
  TENSOR_PARAM("c", bit(VECOPS_DTYPE_F32), -1, 0, VECOPS_TENSOR_WRITE),
};

struct QuantArgs {
  const VecopsTensorView *a, *b, *mult, *rs, *cs, *corr, *c;
  VecopsHipOperand oa, ob, oc;
  int32_t zero_point;
};

int32_t decode(const VecopsCall* call, QuantArgs* d, VecopsError* error) {
  if (int32_t rc = check_call(call, 8, error); rc != VECOPS_STATUS_OK) return rc;
  d->a = tensor_arg(call, 0);
  d->b = tensor_arg(call, 1);
  d->mult = tensor_arg(call, 2);
  d->rs = tensor_arg(call, 4);
  d->cs = tensor_arg(call, 5);
  d->corr = tensor_arg(call, 6);
  d->c = tensor_arg(call, 7);
  if (!d->a || !d->b || !d->mult || !d->rs || !d->cs || !d->c || call->values[3].kind != VECOPS_VALUE_SCALAR)
    return report(error, VECOPS_STATUS_INVALID_ARGUMENT,
                  "a, b, multipliers, row_scales, column_scales and c must be tensors, zero_point a scalar");
  if (d->a->rank != 2 || d->b->rank != 2 || d->c->rank != 2 || d->mult->rank != 1 || d->rs->rank != 1 ||
      d->cs->rank != 1 || (d->corr && d->corr->rank != 1))
    return report(error, VECOPS_STATUS_INVALID_ARGUMENT, "matmul_runtime_quant takes rank-2 matrices and rank-1 vectors");
  const int64_t m = d->a->sizes[0], k = d->a->sizes[1], n = d->b->sizes[0];
  if (d->b->sizes[1] != k || d->c->sizes[0] != m || d->c->sizes[1] != n || d->mult->sizes[0] != m ||
      d->rs->sizes[0] != m || d->cs->sizes[0] != n || (d->corr && d->corr->sizes[0] != n))
    return report(error, VECOPS_STATUS_INVALID_ARGUMENT, "matmul_runtime_quant: extents disagree");
  auto unit = [](const VecopsTensorView* t) { return t->sizes[0] <= 1 || t->strides[0] == 1; };
  if (!unit(d->mult) || !unit(d->rs) || !unit(d->cs) || (d->corr && !unit(d->corr)))
    return report(error, VECOPS_STATUS_NOT_APPLICABLE, "matmul_runtime_quant: the vectors must be contiguous");
  d->zero_point = static_cast<int32_t>(call->values[3].value.scalar.value.i64);
  void* const probe = reinterpret_cast<void*>(16);
  if (!fill_operand(d->a, probe, &d->oa) || !fill_operand(d->b, probe, &d->ob) || !fill_operand(d->c, probe, &d->oc))
    return report(error, VECOPS_STATUS_INVALID_ARGUMENT, "tensors must have rank 2");
  return VECOPS_STATUS_OK;
}

int32_t workspace_impl(const VecopsCall* call, uint64_t* bytes, VecopsError* error) {
  QuantArgs d;
  if (int32_t rc = decode(call, &d, error); rc != VECOPS_STATUS_OK) return rc;
#if VECOPS_ARTIFACT_DEVICE
  *bytes = vecops_hip_matmul_runtime_quant_workspace(&d.oa, &d.ob, &d.oc);
#else
  *bytes = 0;
#endif
  return VECOPS_STATUS_OK;
}

int32_t run_impl(const VecopsCall* call, VecopsError* error) {
  QuantArgs d;
  if (int32_t rc = decode(call, &d, error); rc != VECOPS_STATUS_OK) return rc;
  if (d.a->sizes[0] == 0 || d.b->sizes[0] == 0) return VECOPS_STATUS_OK;
  hipStream_t stream = stream_of(call);
  Staging staging(stream);
  void *mult = nullptr, *rs = nullptr, *cs = nullptr, *corr = nullptr, *dev = nullptr;
  int32_t rc;
  if ((rc = device_address(d.c, true, &staging, &dev, error)) != VECOPS_STATUS_OK) return rc;
  d.oc.data = dev;
  if ((rc = device_address(d.a, false, &staging, &dev, error)) != VECOPS_STATUS_OK) return rc;
  d.oa.data = dev;
  if ((rc = device_address(d.b, false, &staging, &dev, error)) != VECOPS_STATUS_OK) return rc;
  d.ob.data = dev;
  if ((rc = device_address(d.mult, false, &staging, &mult, error)) != VECOPS_STATUS_OK) return rc;
  if ((rc = device_address(d.rs, false, &staging, &rs, error)) != VECOPS_STATUS_OK) return rc;
  if ((rc = device_address(d.cs, false, &staging, &cs, error)) != VECOPS_STATUS_OK) return rc;
  if (d.corr && (rc = device_address(d.corr, false, &staging, &corr, error)) != VECOPS_STATUS_OK) return rc;
  void* ws = call->workspace;
  uint64_t ws_size = call->workspace_size;
#if !VECOPS_ARTIFACT_DEVICE
  ws_size = vecops_hip_matmul_runtime_quant_workspace(&d.oa, &d.ob, &d.oc);
  if (hipError_t e = staging.workspace(ws_size, &ws); e != hipSuccess)
    return report_hip(error, "allocating the quantised activations", e);
#endif
  rc = vecops_hip_matmul_runtime_quant(&d.oa, static_cast<const float*>(mult), d.zero_point, &d.ob,
                                       static_cast<const int32_t*>(corr), static_cast<const float*>(rs),
                                       static_cast<const float*>(cs), &d.oc, ws, ws_size, stream);
  if (rc != VECOPS_STATUS_OK) return report_kernel(error, rc);
  return finish(call, &staging, stream, error);
}

// =================================================================================================
#else  // vecops::matmul_w8a16_group (x, w, scales, y)
// =================================================================================================

constexpr const char* kOperatorName = "vecops::matmul_w8a16_group";
constexpr const char* kKey = "vecops::matmul_w8a16_group;G=" VSTR(VECOPS_ARTIFACT_GROUP) ";memory=" MEMORY_NAME
                             ";backend=hip-gfx950";

#define TENSOR_PARAM(NAME, MASK, RANK, OPTIONAL, FLAGS)                                                       \
  {sizeof(VecopsParameterDescriptor), VECOPS_VALUE_TENSOR, NAME,                                              \
   {.tensor = {sizeof(VecopsTensorParameter), MASK, kDeviceType, -1, RANK, OPTIONAL,                          \
               sizeof(VecopsDimensionConstraint), nullptr, nullptr, FLAGS}}}

const VecopsParameterDescriptor kParameters[] = {
  TENSOR_PARAM("x", bit(VECOPS_DTYPE_BF16), -1, 0, VECOPS_TENSOR_READ),
  TENSOR_PARAM("w", bit(VECOPS_DTYPE_I8), -1, 0, VECOPS_TENSOR_READ),
  TENSOR_PARAM("scales", bit(VECOPS_DTYPE_F32), -1, 0, VECOPS_TENSOR_READ),
  TENSOR_PARAM("y", bit(VECOPS_DTYPE_BF16), -1, 0, VECOPS_TENSOR_WRITE),
};

int32_t workspace_impl(const VecopsCall* call, uint64_t* bytes, VecopsError* error) {
  if (int32_t rc = check_call(call, 4, error); rc != VECOPS_STATUS_OK) return rc;
  *bytes = 0;
  return VECOPS_STATUS_OK;
}

int32_t run_impl(const VecopsCall* call, VecopsError* error) {
  if (int32_t rc = check_call(call, 4, error); rc != VECOPS_STATUS_OK) return rc;
  const VecopsTensorView* x = tensor_arg(call, 0);
  const VecopsTensorView* w = tensor_arg(call, 1);
  const VecopsTensorView* s = tensor_arg(call, 2);
  const VecopsTensorView* y = tensor_arg(call, 3);
  if (!x || !w || !s || !y || x->rank != 2 || w->rank != 2 || s->rank != 2 || y->rank != 2)
    return report(error, VECOPS_STATUS_INVALID_ARGUMENT, "x, w, scales and y must be rank-2 tensors");
  const int64_t m = x->sizes[0], k = x->sizes[1], n = w->sizes[0], g = VECOPS_ARTIFACT_GROUP;
  if (w->sizes[1] != k || y->sizes[0] != m || y->sizes[1] != n || k % g != 0 || s->sizes[0] != n ||
      s->sizes[1] != k / g)
    return report(error, VECOPS_STATUS_INVALID_ARGUMENT, "matmul_w8a16_group: extents disagree");
  auto unit = [](const VecopsTensorView* t) { return t->sizes[1] <= 1 || t->strides[1] == 1; };
  if (!unit(x) || !unit(w) || !unit(y) || !unit(s) || (s->sizes[0] > 1 && s->strides[0] != s->sizes[1]))
    return report(error, VECOPS_STATUS_NOT_APPLICABLE, "matmul_w8a16_group: rows must be contiguous, scales dense");
  if (m == 0 || n == 0) return VECOPS_STATUS_OK;
  hipStream_t stream = stream_of(call);
  Staging staging(stream);
  void *dx = nullptr, *dw = nullptr, *ds = nullptr, *dy = nullptr;
  int32_t rc;
  if ((rc = device_address(y, true, &staging, &dy, error)) != VECOPS_STATUS_OK) return rc;
  if ((rc = device_address(x, false, &staging, &dx, error)) != VECOPS_STATUS_OK) return rc;
  if ((rc = device_address(w, false, &staging, &dw, error)) != VECOPS_STATUS_OK) return rc;
  if ((rc = device_address(s, false, &staging, &ds, error)) != VECOPS_STATUS_OK) return rc;
  rc = vecops_hip_matmul_w8a16_group(dx, x->strides[0], static_cast<const int8_t*>(dw), w->strides[0],
                                     static_cast<const float*>(ds), dy, y->strides[0], m, n, k, g, stream);
  if (rc != VECOPS_STATUS_OK) return report_kernel(error, rc);
  return finish(call, &staging, stream, error);
}

#endif

// ---- callbacks: nothing may escape as an exception --------------------------------------------------
int32_t workspace_entry(const VecopsCall* call, uint64_t* bytes, VecopsError* error) {
  try {
    if (bytes == nullptr) return report(error, VECOPS_STATUS_INVALID_ARGUMENT, "null workspace size pointer");
    return workspace_impl(call, bytes, error);
  } catch (const std::exception& e) {
    return report(error, VECOPS_STATUS_EXECUTION_ERROR, e.what());
  } catch (...) {
    return report(error, VECOPS_STATUS_EXECUTION_ERROR, "unknown exception in the workspace query");
  }
}

int32_t run_entry(const VecopsCall* call, VecopsError* error) {
  try {
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0)
      return report(error, VECOPS_STATUS_EXECUTION_ERROR,
                    std::string("no HIP device available: ") + (e != hipSuccess ? hipGetErrorString(e) : "0 devices"));
    return run_impl(call, error);
  } catch (const std::exception& e) {
    return report(error, VECOPS_STATUS_EXECUTION_ERROR, e.what());
  } catch (...) {
    return report(error, VECOPS_STATUS_EXECUTION_ERROR, "unknown exception in the kernel artifact");
  }
}

const VecopsKernelDescriptorV1 kDescriptor = {
  sizeof(VecopsKernelDescriptorV1),
  VECOPS_KERNEL_ABI_VERSION_MAJOR,
  VECOPS_KERNEL_ABI_VERSION_MINOR,
  kOperatorName,
  kKey,
  static_cast<uint32_t>(sizeof(kParameters) / sizeof(kParameters[0])),
  sizeof(VecopsParameterDescriptor),
  kParameters,
  workspace_entry,
  run_entry,
  0,
};

}  // namespace

extern "C" VECOPS_RUNTIME_EXPORT const VecopsKernelDescriptorV1* vecops_kernel_query_v1(void) { return &kDescriptor; }
