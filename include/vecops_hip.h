/*
 * vecops_hip.h - C ABI of libvecops_hip.so, the gfx950 (MI355X) kernels behind
 * the vecops matmul path.
 *
 * Every entry point takes plain device pointers, element extents and element
 * strides; none allocates, none synchronises: work is enqueued on `stream`
 * (a hipStream_t passed as void*, null = the default stream) and the call
 * returns.  The artifact DSOs that plug into vecops::runtime::Executable call
 * these functions from their `run` callback and then wait for the stream,
 * because the vecops kernel ABI is synchronous (runtime/CallAbi.h:7-16).
 *
 * Return values are VecopsStatusCode numbers (runtime/CallAbi.h:34-51):
 * 0 ok, 1 invalid argument, 2 not applicable, 6 execution error.  A failing
 * call leaves a message readable with vecops_hip_last_error() on the same
 * host thread.
 *
 * dtype codes are VecopsDType numbers (runtime/CallAbi.h:62-91):
 * 2 i8, 3 u8, 6 i32, 11 bf16, 12 f32.
 */
#ifndef VECOPS_HIP_H
#define VECOPS_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define VECOPS_HIP_EXPORT __attribute__((visibility("default")))

#define VECOPS_HIP_ABI_VERSION 1u

/*
 * Flag for VecopsExecutionContext::flags of a call that reaches the kernels through vecops' artifact ABI (the field
 * is "embedding-defined", runtime/CallAbi.h:369-370): the caller orders its own work on context->stream, so an artifact
 * whose tensors live in device memory returns once its kernels are enqueued.  Without it such an artifact waits for
 * them (vecops' ABI functions are synchronous, runtime/CallAbi.h:15-16).  Artifacts that stage host tensors always
 * wait: their results have to be back in host memory on return.
 */
#define VECOPS_HIP_CONTEXT_STREAM_ORDERED 1ull

/* One operand of a matmul: `data` addresses logical element zero in device
 * memory.  rank 2 = [rows, cols]; rank 3 = [batch, rows, cols].  Strides are in
 * elements; a zero batch stride broadcasts the operand over the batch
 * (planning/families/ArchitectureFamily.h:393-421). */
typedef struct VecopsHipOperand {
  void* data;
  uint32_t dtype;
  uint32_t rank;
  int64_t sizes[3];
  int64_t strides[3];
} VecopsHipOperand;

/* How fp32 operands are multiplied (bf16 and int8 operands ignore it).
 *   BF16: round each fp32 operand element to bf16 (nearest even) on load and use
 *         the bf16 matrix cores - what vecops' x86 path does, which has no fp32
 *         atom (matmul/details/kernel/amx/Atoms.h:51-60).
 *   F32 : multiply in fp32 on the fp32 matrix cores - vecops' SME_F32F32 atom
 *         (matmul/details/kernel/sme/Atoms.h:65-76). */
typedef enum VecopsHipCompute { VECOPS_HIP_COMPUTE_BF16 = 0, VECOPS_HIP_COMPUTE_F32 = 1 } VecopsHipCompute;

/* Kernel families of the GPU rule table (vecops_hip_select_kernel). */
typedef enum VecopsHipKernelFamily {
  VECOPS_HIP_FAMILY_NONE = 0,          /* empty problem: nothing to launch */
  VECOPS_HIP_FAMILY_TILE_256 = 1,      /* 256x256 workgroup tile, MFMA */
  VECOPS_HIP_FAMILY_TILE_128 = 2,      /* 128x128 workgroup tile, MFMA (16-bit compute with 8 <= K <= 32, K-contiguous
                                          operands and plain fp32 / bf16 / f16 results: a kernel of 32x256 tiles whose
                                          life is the write of C) */
  VECOPS_HIP_FAMILY_TILE_64 = 3,       /* 64x64 workgroup tile, MFMA */
  VECOPS_HIP_FAMILY_SKINNY = 4,        /* one side <= 16 rows: wavefronts split K, the wide operand is read once */
  VECOPS_HIP_FAMILY_ZERO_K = 5,        /* K == 0: C = Cin or zeros */
  VECOPS_HIP_FAMILY_TILE_256X128 = 6,  /* 256 (M) x 128 (N) workgroup tile, MFMA */
  VECOPS_HIP_FAMILY_TILE_128X256 = 7,  /* 128 (M) x 256 (N) workgroup tile, MFMA */
  VECOPS_HIP_FAMILY_TILE_256X352 = 8,  /* 256 (M) x 352 (N) workgroup tile of signed 8-bit, bf16 or f16 operands (aligned,
                                          K-contiguous, K in whole K tiles of 128 bytes): the tile
                                          that covers 2048 x 11008 in one round */
  VECOPS_HIP_FAMILY_TILE_192 = 9       /* 192x192 workgroup tile of bf16, f16 or signed 8-bit operands (16-byte aligned
                                          bases, rows and batches; both K-contiguous, or 16-bit ones with B as [K,N];
                                          B not prepacked): the tile that covers 3072 x 3072 in one round */
} VecopsHipKernelFamily;

typedef struct VecopsHipPlan {
  uint32_t family;     /* VecopsHipKernelFamily */
  uint32_t split_k;    /* >= 1; > 1 needs workspace */
  uint32_t vector_a;   /* 1 = 16-byte loads along K usable for A */
  uint32_t vector_b;   /* 1 = 16-byte loads usable for B */
  uint32_t b_layout;   /* 0 = K contiguous, 1 = N contiguous, 2 = generic */
  uint32_t peeled_columns; /* > 0: the last so many columns of c are a second product with a plan of its own (few
                              tiles, K split), cut off so that the rest fills whole rounds of workgroups */
  uint64_t workspace_bytes;
} VecopsHipPlan;

/* ABI version of the loaded library. */
VECOPS_HIP_EXPORT uint32_t vecops_hip_abi_version(void);

/* Message of the last failing call on this host thread ("" if none). */
VECOPS_HIP_EXPORT const char* vecops_hip_last_error(void);

/* Number of HIP devices visible, or a negative number when the HIP runtime
 * cannot be initialised. */
VECOPS_HIP_EXPORT int32_t vecops_hip_device_count(void);

/*
 * GPU counterpart of vecops' runtime shape selector
 * (matmul/details/kernel/RuntimeDispatch.h:24-83,
 * src/MatmulRuntimeDispatch.cpp:12-32 and its call sites
 * matmul/details/kernel/amx/Backend.h:2724-2757): a pure function of the
 * operand metadata that chooses the kernel family, the split-K factor and the
 * external workspace a call needs.  No device access.
 */
VECOPS_HIP_EXPORT int32_t vecops_hip_plan_matmul(const VecopsHipOperand* a, const VecopsHipOperand* b,
                                                 const VecopsHipOperand* c_in, const VecopsHipOperand* c,
                                                 uint32_t compute, VecopsHipPlan* plan);

/*
 * C[..,M,N] = C_in + A[..,M,K] . B[..,N,K]^T  - replaces
 * ops::Matmul<Config>::operator() (ops/Matmul.h:530-570) for
 *   a,b bf16 -> c f32|bf16      (AMX_BF16F32)
 *   a,b f16  -> c f32|f16       (AMX_F16F32 / SME_F16F32; IEEE half, round to nearest even)
 *   a,b f32  -> c f32|bf16      (bf16 or fp32 compute, see VecopsHipCompute)
 *   a,b i8|u8 -> c i32          (AMX_I8I32<A,B>, either side signed or unsigned;
 *                                accumulators wrap mod 2^32)
 *   a,b f64  -> c f64           (SME_F64F64, matmul/details/kernel/sme/Atoms.h:108-112; dtype 13; a kernel of its own
 *                                on v_mfma_f64_16x16x4_f64: family tile_128, K never split, no fused transform)
 * c_in may be null (zero accumulator); otherwise it has c's dtype class (f32,
 * bf16, i32 or f64) and may alias c element for element.  K == 0 writes zeros or
 * C_in; zero M, N or batch writes nothing (ops/Matmul.h:41-43).  Operand
 * metadata is validated as planning/families/ArchitectureFamily.h:1590-1652
 * does.  `workspace` must hold vecops_hip_plan_matmul(...).workspace_bytes.
 */
VECOPS_HIP_EXPORT int32_t vecops_hip_matmul(const VecopsHipOperand* a, const VecopsHipOperand* b,
                                            const VecopsHipOperand* c_in, const VecopsHipOperand* c, uint32_t compute,
                                            void* workspace, uint64_t workspace_size, void* stream);

/*
 * vecops_hip_matmul with the plan made beforehand - the prepared invocation of vecops (ops::Matmul<Config>::prepare /
 * Prepared / PatternPrepared, ops/Matmul.h:183-500; the prepared-call cache of docs/Runtime.md:196-206): `plan` is what
 * vecops_hip_plan_matmul or vecops_hip_plan_matmul_family returned for operands of the same metadata (extents, strides,
 * dtypes, alignment); the rule table is not consulted again.  The plan is checked against the operands - a family
 * that cannot serve them, a K split beyond the K tiles or columns peeled where the table peels none is status 1
 * (invalid argument), nothing is launched - and its workspace need is recomputed, never trusted.
 */
VECOPS_HIP_EXPORT int32_t vecops_hip_matmul_planned(const VecopsHipOperand* a, const VecopsHipOperand* b,
                                                    const VecopsHipOperand* c_in, const VecopsHipOperand* c,
                                                    uint32_t compute, const VecopsHipPlan* plan, void* workspace,
                                                    uint64_t workspace_size, void* stream);

/*
 * The first tier of vecops' owner selection: an explicit family request (matmul::family_selection::Automatic /
 * Prefer<F> / Require<F>, matmul/Family.h:216-239; consulted first by Backend<AMX>::run,
 * matmul/details/kernel/amx/Backend.h:2724-2757).  PREFER takes the family when it can serve the call and the rule
 * table's choice otherwise; REQUIRE returns 2 (not applicable) and launches nothing when it cannot - the C-ABI form
 * of the exception of tests/ops/MatmulTest.cpp:514-536.  The tile families serve every non-empty product, the skinny
 * family only its own shapes.  split_k = 0 leaves the K split to the rule table; another value (tile families only)
 * fixes it, clamped to the K tiles there are.
 */
typedef enum VecopsHipFamilySelection {
  VECOPS_HIP_SELECT_AUTOMATIC = 0,
  VECOPS_HIP_SELECT_PREFER = 1,
  VECOPS_HIP_SELECT_REQUIRE = 2
} VecopsHipFamilySelection;

typedef struct VecopsHipFamilyRequest {
  uint32_t struct_size;  /* sizeof(VecopsHipFamilyRequest) */
  uint32_t selection;    /* VecopsHipFamilySelection */
  uint32_t family;       /* VecopsHipKernelFamily */
  uint32_t split_k;      /* 0 = the rule table's */
} VecopsHipFamilyRequest;

/* vecops_hip_plan_matmul / vecops_hip_matmul under a family request (null = automatic). */
VECOPS_HIP_EXPORT int32_t vecops_hip_plan_matmul_family(const VecopsHipOperand* a, const VecopsHipOperand* b,
                                                        const VecopsHipOperand* c_in, const VecopsHipOperand* c,
                                                        uint32_t compute, const VecopsHipFamilyRequest* request,
                                                        VecopsHipPlan* plan);
VECOPS_HIP_EXPORT int32_t vecops_hip_matmul_family(const VecopsHipOperand* a, const VecopsHipOperand* b,
                                                   const VecopsHipOperand* c_in, const VecopsHipOperand* c,
                                                   uint32_t compute, const VecopsHipFamilyRequest* request,
                                                   void* workspace, uint64_t workspace_size, void* stream);

/*
 * vecops_hip_matmul without a workspace argument, for callers that cannot allocate device memory at all:
 * code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in
 * vecops (its callers size and own every workspace, ops/Matmul.h:504-526).  The split-K partial sums and the
 * unsigned-operand terms live in a buffer of VECOPS_HIP_STATIC_WORKSPACE_BYTES that belongs to the library's
 * code object on each GPU (8 MiB, held until the process ends; the K splits of problems with few output tiles of
 * 64 x 64 need at most 4 MiB, the row sums of unsigned operands 4 bytes per row of a and b); the call allocates and
 * frees nothing.  A plan of vecops_hip_matmul whose partial sums would not fit - K of a problem with 128 to 200 tiles
 * of 128 x 128 split two to four ways (24-32 MB), or of few 128 x 128 tiles of fp32 operands - is not taken here: the
 * split is halved until the sums fit, down to an unsplit product (the sums then differ from vecops_hip_matmul's in
 * their order).  A call that still needs more than the buffer - the row sums of an unsigned operand with more than two
 * million rows - returns 2 (not applicable) and launches nothing.  Otherwise the same kernels and therefore the same
 * results, bit for bit, as vecops_hip_matmul.  `stream` must belong to the current device (each GPU has its own copy
 * of the buffer; a stream of another device is status 1).  Every call on one GPU shares that GPU's buffer: calls that
 * overlap on one GPU (different streams or host threads) race; calls on one stream, or otherwise ordered, do not.
 */
#define VECOPS_HIP_STATIC_WORKSPACE_BYTES (8u << 20)
VECOPS_HIP_EXPORT uint64_t vecops_hip_static_workspace_bytes(void);
VECOPS_HIP_EXPORT int32_t vecops_hip_matmul_static_workspace(const VecopsHipOperand* a, const VecopsHipOperand* b,
                                                             const VecopsHipOperand* c_in, const VecopsHipOperand* c,
                                                             uint32_t compute, void* stream);

/*
 * Several independent products in one call: c[i] = c_in[i] + a[i] . b[i]^T for i < count, every group with its own
 * extents, strides and pointers (irregular batches).  vecops' batch planner serves batches that share an operand by
 * flattening them into one product (planning/families/ArchitectureBatchPlanner.h:30-160; vecops_hip_matmul does the
 * same) and everything else batch by batch; this entry point is the form for batches that share nothing, not even
 * their shapes.  a, b, c (and c_in, which may be null; an entry of rank 0 means "no C input for this group") are
 * arrays of count descriptors obeying the rules of vecops_hip_matmul group by group.  Groups of one operand
 * class - bf16, f16, int8 x int8, 8-bit integers with an unsigned side, or fp32 in either compute type - run as ONE
 * launch over a table of problem records (written into the workspace by small kernels fed through their arguments: no
 * host buffer has to outlive the call, nothing is allocated; the row-sum terms of unsigned sides are computed group by
 * group into the workspace first); fp64 operands, a mix of classes (signed x signed bytes beside groups with an
 * unsigned side count as a mix), groups with K = 0 and groups whose K vecops_hip_matmul would split (few output tiles,
 * long K: they run that call's plan, partial sums behind the table) run as launches of their own on the same stream.
 * Results
 * are those of vecops_hip_matmul on each group (bit-equal when that call runs the same tile shape without splitting K -
 * except 16-bit products with K <= 256 on 128 x 128 tiles, where the single call takes the other MFMA shape; otherwise equal up to the order of the fp32 sums - integer results are always the same bits).  workspace: vecops_hip_matmul_grouped_workspace bytes, 16-byte aligned.
 */
VECOPS_HIP_EXPORT uint64_t vecops_hip_matmul_grouped_workspace(uint32_t count, const VecopsHipOperand* a,
                                                               const VecopsHipOperand* b, const VecopsHipOperand* c_in,
                                                               const VecopsHipOperand* c, uint32_t compute);
VECOPS_HIP_EXPORT int32_t vecops_hip_matmul_grouped(uint32_t count, const VecopsHipOperand* a, const VecopsHipOperand* b,
                                                    const VecopsHipOperand* c_in, const VecopsHipOperand* c,
                                                    uint32_t compute, void* workspace, uint64_t workspace_size,
                                                    void* stream);

/*
 * Fused output transforms - the catalogue that vecops' tests build from
 * elementwise and lane-local output transforms on tensor::output
 * (tests/ops/MatmulFusionTest.cpp:29-112; tests/ops/MatmulConversionTestCommon.h:
 * bias + relu :439-497, runtime and per-column scale :621-702, bias + clamp
 * :705-760, relu / sigmoid :1028-1092, silu :1095-1168, integer bias with
 * per-column (re)quantisation :1171-1290).  With acc = C_in + A.B^T (a bias is a
 * C_in row with row stride 0):
 *   v = float(acc)                      (int32 accumulators; fp32 ones are v already)
 *   v = v * row_scales[row]             (row_scales != null)
 *   v = v * column_scales[col]          (column_scales != null)
 *   v = v * scale                       (flags & VECOPS_HIP_EPILOGUE_SCALE)
 *   v = v + shift                       (flags & VECOPS_HIP_EPILOGUE_SHIFT)
 *   v = activation(v)                   relu max(v,0); clamp min(max(v,lo),hi);
 *                                       sigmoid 1/(1+exp(-v)); silu v*sigmoid(v)
 *   c = convert(v)                      fp32; bf16 round-to-nearest-even; u8 / i8:
 *                                       truncate toward zero, saturate (NaN and
 *                                       values outside int32 become INT32_MIN before
 *                                       the saturation, as vecops' x86 vector store
 *                                       does, vec/details/x86/Conversion.h:522-528)
 * Every step is one fp32 operation, never contracted.  Scales, shift, relu and
 * clamp are bit-exact against the reference on int32 accumulators; sigmoid and
 * silu use the hardware exponential (within 1e-6 relative of the exact value).
 */
enum VecopsHipActivation {
  VECOPS_HIP_ACT_NONE = 0,
  VECOPS_HIP_ACT_RELU = 1,
  VECOPS_HIP_ACT_CLAMP = 2,
  VECOPS_HIP_ACT_SIGMOID = 3,
  VECOPS_HIP_ACT_SILU = 4
};
enum { VECOPS_HIP_EPILOGUE_SCALE = 1u, VECOPS_HIP_EPILOGUE_SHIFT = 2u };

typedef struct VecopsHipEpilogue {
  uint32_t struct_size;        /* sizeof(VecopsHipEpilogue) */
  uint32_t activation;         /* VecopsHipActivation */
  uint32_t flags;              /* VECOPS_HIP_EPILOGUE_* */
  float scale;
  float shift;
  float clamp_lo, clamp_hi;
  const float* row_scales;     /* device, [M] (rank 3: [batch][M] dense), or null */
  const float* column_scales;  /* device, [N], or null */
} VecopsHipEpilogue;

/* vecops_hip_plan_matmul for a call of vecops_hip_matmul_fused. */
VECOPS_HIP_EXPORT int32_t vecops_hip_plan_matmul_fused(const VecopsHipOperand* a, const VecopsHipOperand* b,
                                                       const VecopsHipOperand* c_in, const VecopsHipOperand* c,
                                                       uint32_t compute, const VecopsHipEpilogue* epilogue,
                                                       VecopsHipPlan* plan);

/*
 * vecops_hip_matmul with the transform above between the accumulator and c.
 *   a,b bf16 | f32 -> c f32 | bf16      (c_in f32 | bf16)
 *   a,b f16        -> c f32 | f16       (c_in f32 | f16)
 *   a,b i8 | u8    -> c f32 | u8 | i8   (c_in i32)
 * Operands, strides, batches, zero extents and the workspace rule are those of
 * vecops_hip_matmul (K == 0 writes transform(C_in or 0)).
 */
VECOPS_HIP_EXPORT int32_t vecops_hip_matmul_fused(const VecopsHipOperand* a, const VecopsHipOperand* b,
                                                  const VecopsHipOperand* c_in, const VecopsHipOperand* c,
                                                  uint32_t compute, const VecopsHipEpilogue* epilogue,
                                                  void* workspace, uint64_t workspace_size, void* stream);

/*
 * c[i,j] = (float(acc[i,j]) * row_scales[i]) * column_scales[j],
 * acc = sum_k a[i,k]*b[j,k] (+ correction[j]) in wrapping int32 - replaces
 * ops::matmul with AMX_I8I32<int8,int8> and an output carrying
 * RuntimePerRowColumnDequantizeTransform (matmul/Quantization.h:195-250); the
 * optional correction row is the stride-0 int32 C-input of
 * tests/ops/MatmulConversionTestCommon.h:1467-1472.  a is [M,K] with row
 * stride lda, b is [N,K] with row stride ldb (both K contiguous), c is fp32
 * [M,N] with row stride ldc.  Bit-exact.
 */
VECOPS_HIP_EXPORT int32_t vecops_hip_matmul_i8_dequant(const int8_t* a, int64_t lda, const int8_t* b, int64_t ldb,
                                                       const float* row_scales, const float* column_scales,
                                                       const int32_t* correction, float* c, int64_t ldc, int64_t m,
                                                       int64_t n, int64_t k, void* workspace, uint64_t workspace_size,
                                                       void* stream);

/*
 * q[..,r,k] = u8( x[..,r,k] * multipliers[row] + (float)zero_point ), row = batch * M + r:
 * vecops' RuntimePerRowAsymmetricQuantizeTransform on an fp32 input read as the atom's uint8
 * (matmul/Quantization.h:91-146, formula :123-128; tensor::input<uint8_t>(a, quantize) in
 * tests/ops/MatmulConversionTestCommon.h:1503-1506).  The multiply and the add are rounded
 * separately; the conversion truncates toward zero, sends NaN and values outside int32 to 0 and
 * saturates at 0 and 255 (the x86 vector conversion, vec/details/x86/Conversion.h:522-528).  x is f32,
 * q is u8 with the same extents (rank 2 or 3, any strides).  Bit-exact.
 */
VECOPS_HIP_EXPORT int32_t vecops_hip_quantize_rows(const VecopsHipOperand* x, const float* multipliers,
                                                   int32_t zero_point, const VecopsHipOperand* q, void* stream);

/*
 * The runtime-quantised product of tests/ops/MatmulConversionTestCommon.h:1437-1540 in one call:
 *   q = quantize_rows(a);  acc = sum_k q[i,k] * b[j,k] + correction[j]  (AMX_I8I32<uint8_t, int8_t>, wrapping);
 *   c[i,j] = (float(acc) * row_scales[i]) * column_scales[j].
 * a f32 [M,K], b i8 [N,K], c f32 [M,N] (rank 2, any strides), or the batched forms of
 * tests/ops/MatmulConversionTestCommon.h:1277-1434: a [batch,M,K] and c [batch,M,N] with b either rank 2 (one set of
 * weights for every batch; when the rows of a and c run on from batch to batch the batches fold into one
 * [batch * M, K] product) or [batch,N,K]; a batch stride of 0 on a or b shares that operand.  Batch strides of the
 * vectors follow the reference's tests: multipliers and row_scales have batch * M entries (batch_stride = M) unless a
 * is shared (then M entries), correction has batch * N entries when b is per batch, else N
 * (vecops_hip_matmul_runtime_quant_batched takes the strides explicitly).  correction (usually
 * -zero_point * sum_k b[j,k], see vecops_hip_pack_b_compensated) may be null.  The workspace holds the
 * quantised activations (kept as q - 128 for the signed kernels), the correction rows with 128 * sum_k b[j,k]
 * added, and the product's own scratch: vecops_hip_matmul_runtime_quant_workspace bytes, 16-byte aligned.
 * Bit-exact (the sums are integers mod 2^32 either way).
 */
VECOPS_HIP_EXPORT uint64_t vecops_hip_matmul_runtime_quant_workspace(const VecopsHipOperand* a,
                                                                     const VecopsHipOperand* b,
                                                                     const VecopsHipOperand* c);
VECOPS_HIP_EXPORT int32_t vecops_hip_matmul_runtime_quant(const VecopsHipOperand* a, const float* multipliers,
                                                          int32_t zero_point, const VecopsHipOperand* b,
                                                          const int32_t* correction, const float* row_scales,
                                                          const float* column_scales, const VecopsHipOperand* c,
                                                          void* workspace, uint64_t workspace_size, void* stream);

/*
 * The same with the batch strides given: batch i quantises with multipliers[i * scale_batch_stride + row], dequantises
 * with row_scales[i * scale_batch_stride + row] (vecops' `batch_stride` of the two runtime transforms,
 * matmul/Quantization.h:91-146,195-250) and adds correction[i * correction_batch_stride + col] (the strides {n or 0, 0, 1}
 * of the reference's correction tensor).  a and c rank 3, b rank 2 or 3.
 */
VECOPS_HIP_EXPORT uint64_t vecops_hip_matmul_runtime_quant_batched_workspace(const VecopsHipOperand* a,
                                                                             int64_t scale_batch_stride,
                                                                             const VecopsHipOperand* b,
                                                                             int64_t correction_batch_stride,
                                                                             const VecopsHipOperand* c);
VECOPS_HIP_EXPORT int32_t vecops_hip_matmul_runtime_quant_batched(const VecopsHipOperand* a, const float* multipliers,
                                                                  int32_t zero_point, int64_t scale_batch_stride,
                                                                  const VecopsHipOperand* b, const int32_t* correction,
                                                                  int64_t correction_batch_stride, const float* row_scales,
                                                                  const float* column_scales, const VecopsHipOperand* c,
                                                                  void* workspace, uint64_t workspace_size, void* stream);

/* The same with b packed by vecops_hip_pack_b (int8; n rows) - exactly the operands of
 * tests/ops/MatmulConversionTestCommon.h:1484-1510, where B is packed first. */
VECOPS_HIP_EXPORT uint64_t vecops_hip_matmul_runtime_quant_packed_b_workspace(const VecopsHipOperand* a, int64_t n,
                                                                              const VecopsHipOperand* c);
VECOPS_HIP_EXPORT int32_t vecops_hip_matmul_runtime_quant_packed_b(const VecopsHipOperand* a, const float* multipliers,
                                                                   int32_t zero_point, const void* packed_b, int64_t n,
                                                                   const int32_t* correction, const float* row_scales,
                                                                   const float* column_scales, const VecopsHipOperand* c,
                                                                   void* workspace, uint64_t workspace_size,
                                                                   void* stream);

/* Workspace bytes vecops_hip_matmul_i8_dequant needs for these extents. */
VECOPS_HIP_EXPORT uint64_t vecops_hip_matmul_i8_dequant_workspace(int64_t m, int64_t n, int64_t k);

/*
 * y[m,n] = bf16( sum_g scales[n,g] * sum_{k in group g} float(x[m,k]) * float(w[n,k]) )
 * x bf16 [M,K] (row stride ldx), w int8 [N,K] (row stride ldw), scales fp32
 * [N, K/group] dense, y bf16 [M,N] (row stride ldy); fp32 accumulation.
 * No counterpart in vecops (it has no weight-only group-scaled matmul); this
 * is the decode-shaped GEMV / skinny GEMM.  m <= 16,
 * k a multiple of `group`, group a multiple of 16.
 */
VECOPS_HIP_EXPORT int32_t vecops_hip_matmul_w8a16_group(const void* x, int64_t ldx, const int8_t* w, int64_t ldw,
                                                        const float* scales, void* y, int64_t ldy, int64_t m,
                                                        int64_t n, int64_t k, int64_t group, void* stream);

/*
 * Prepacked B operand - the GPU counterpart of ops::matmul_pack with side B and
 * matmul::packed_layout (ops/MatmulPack.h:9-117; x86 block format
 * matmul/details/packing/amx/Format.h:27-58).  Packing is a permutation plus
 * zero padding, so a matmul on the packed operand returns exactly what the
 * plain one returns; weights that are multiplied many times are packed once and
 * the multiplication then fetches them straight into matrix-core registers.
 *
 * Layout (EPC = elements per 16 bytes: 8 for bf16, 16 for i8; KS = k-steps of
 * 2*EPC elements, K rounded up to a multiple of 8*EPC):
 *   dim order [ panel (N/32) ][ k-step (KS) ][ k-half (2) ][ row (32) ][ k (EPC) ]
 * i.e. element B[n,k] sits at byte
 *   ((n/32 * KS + k/(2*EPC)) * 64 + (k/EPC % 2) * 32 + n % 32) * 16 + (k % EPC) * sizeof(element);
 * rows past N and k past K are zero.
 *
 * packed dtypes: 11 bf16 (from a bf16 or f32 source; f32 is rounded to nearest
 * even, as the matmul itself rounds it), 10 f16, 2 i8 and 3 u8.  An unsigned operand is stored as the signed
 * b - 128 (its bytes xor 0x80, padding still zero), so that the product runs on the signed matrix-core instruction and
 * adds 128 * sum_k a[m,k] back in its epilogue: AMX_I8I32<int8_t, uint8_t> and <uint8_t, uint8_t> with a packed B
 * (tests/ops/MatmulMixedPackingTest.cpp:137-153).
 *
 * The [M,K] operand packs into the same 32-row panels (vecops_hip_pack_a; vecops keeps a format per side,
 * ops/MatmulPack.h:63-65 - here one format serves both, but a packed operand still has to be passed as the side it was
 * packed for).
 */

/* Bytes of the packed form of a [N,K] operand; 0 for an unsupported dtype. */
VECOPS_HIP_EXPORT uint64_t vecops_hip_packed_b_bytes(uint32_t packed_dtype, int64_t n, int64_t k);

/* Packs b (rank 2, [N,K], any strides; bf16, f16, f32, i8 or u8) into `packed`
 * (16-byte aligned, at least vecops_hip_packed_b_bytes).  Replaces
 * ops::MatmulPack<MatmulPackConfig<Atom, Operand::B>>::operator()
 * (ops/MatmulPack.h:132-190). */
VECOPS_HIP_EXPORT int32_t vecops_hip_pack_b(const VecopsHipOperand* b, void* packed, uint64_t packed_size,
                                            void* stream);
/* The same with the packed dtype named by the caller: what vecops_hip_pack_b chooses (bf16 for a bf16 or f32 source,
 * the source's own dtype otherwise), or 12 (f32) for an f32 source whose elements stay fp32 - the pack of the
 * fp32-compute atom (ops::MatmulPack is generic over atoms, ops/MatmulPack.h:9-117; SME_F32F32,
 * matmul/details/kernel/sme/Atoms.h): 4 elements per 16-byte chunk, the same 32-row panels; products against it
 * (vecops_hip_matmul_packed_b / _packed_a / _packed_ab with packed dtype 12, an f32 dense operand, f32 c) multiply in
 * fp32.  Serves either side. */
VECOPS_HIP_EXPORT int32_t vecops_hip_pack_as(const VecopsHipOperand* b, uint32_t packed_dtype, void* packed,
                                             uint64_t packed_size, void* stream);

/* Packs an int8 b and also writes compensation[n] = -a_zero_point * sum_k b[n,k]
 * (wrapping int32), the C-input row that corrects an asymmetrically quantised
 * A - replaces ops::MatmulPackBCompensated (ops/MatmulPack.h:25-33,100-117). */
VECOPS_HIP_EXPORT int32_t vecops_hip_pack_b_compensated(const VecopsHipOperand* b, int32_t a_zero_point, void* packed,
                                                        uint64_t packed_size, int32_t* compensation, void* stream);

/* vecops_hip_plan_matmul for a packed b of `n` rows (family, split-K, workspace). */
VECOPS_HIP_EXPORT int32_t vecops_hip_plan_matmul_packed_b(const VecopsHipOperand* a, uint32_t packed_dtype, int64_t n,
                                                          const VecopsHipOperand* c_in, const VecopsHipOperand* c,
                                                          VecopsHipPlan* plan);

/*
 * C[..,M,N] = C_in + A[..,M,K] . B[N,K]^T with B prepacked; the one packed
 * operand serves every batch of a rank-3 A (vecops: a packed tensor passed as B
 * lets the planner skip the packing stage, ops/MatmulPack.h:22-24).
 *   packed bf16: a bf16 or f32 (rounded to bf16), c f32|bf16
 *   packed f16 : a f16, c f32|f16
 *   packed i8  : a i8 or u8 (AMX_I8I32<uint8_t, int8_t>, the atom the compensated pack serves,
 *                ops/MatmulPack.h:52-58; the workspace then also holds 4 * batch * (M + N) bytes), c i32
 *   packed u8  : a i8 or u8, c i32 (the same workspace term)
 *   packed f32 : a f32, c f32, products in fp32 (vecops_hip_pack_as)
 * Integer results are those of vecops_hip_matmul on the unpacked operand, bit for bit; floating-point results too
 * when that call runs its 256-row or 256-column tiles with the same split of K (the packed kernels multiply on the
 * 32x32 matrix instructions, the small plain tiles on the 16x16 ones: the fp32 sums are then taken in another order).
 */
VECOPS_HIP_EXPORT int32_t vecops_hip_matmul_packed_b(const VecopsHipOperand* a, const void* packed_b,
                                                     uint32_t packed_dtype, int64_t n, const VecopsHipOperand* c_in,
                                                     const VecopsHipOperand* c, void* workspace,
                                                     uint64_t workspace_size, void* stream);

/*
 * Side A: ops::MatmulPack<MatmulPackConfig<Atom, Operand::A>> (ops/MatmulPack.h:81-96,132-190) and the product with a
 * packed A (tests/ops/MatmulMixedPackingTest.cpp:24-28).  C = C_in + A . B^T with A[M,K] prepacked runs as
 * C^T = C_in^T + B . A^T on the packed-operand kernels: b is then the operand that travels through LDS and the
 * packed a the one fetched straight into registers; c and c_in are written and read through their transposed views
 * (any strides are legal, the stores of a row-major c are element-wise).  Same sums in the same order as the plain
 * product.  b rank 2 or 3 (the one packed a serves every batch), dtypes as for vecops_hip_matmul_packed_b with the
 * sides exchanged.
 */
VECOPS_HIP_EXPORT int32_t vecops_hip_pack_a(const VecopsHipOperand* a, void* packed, uint64_t packed_size, void* stream);
VECOPS_HIP_EXPORT int32_t vecops_hip_plan_matmul_packed_a(uint32_t packed_dtype, int64_t m, const VecopsHipOperand* b,
                                                          const VecopsHipOperand* c_in, const VecopsHipOperand* c,
                                                          VecopsHipPlan* plan);
VECOPS_HIP_EXPORT int32_t vecops_hip_matmul_packed_a(const void* packed_a, uint32_t packed_dtype, int64_t m,
                                                     const VecopsHipOperand* b, const VecopsHipOperand* c_in,
                                                     const VecopsHipOperand* c, void* workspace, uint64_t workspace_size,
                                                     void* stream);

/*
 * Both operands packed (tests/ops/MatmulMixedPackingTest.cpp:31-108, check_both_packed): c[M,N] = c_in + A . B^T with
 * A packed by vecops_hip_pack_a ([M,K], a_dtype) and B by vecops_hip_pack_b ([N,K], b_dtype).  The matrix cores take one
 * operand from registers and one through LDS, so A is first written back to a dense [M,K] matrix at the front of the
 * workspace (a permutation) and then multiplied with the packed B.  c rank 2.  workspace:
 * vecops_hip_matmul_packed_ab_workspace bytes, 16-byte aligned.
 */
VECOPS_HIP_EXPORT uint64_t vecops_hip_matmul_packed_ab_workspace(uint32_t a_dtype, int64_t m, uint32_t b_dtype, int64_t n,
                                                                 int64_t k, const VecopsHipOperand* c_in,
                                                                 const VecopsHipOperand* c);
VECOPS_HIP_EXPORT int32_t vecops_hip_matmul_packed_ab(const void* packed_a, uint32_t a_dtype, int64_t m, const void* packed_b,
                                                      uint32_t b_dtype, int64_t n, int64_t k, const VecopsHipOperand* c_in,
                                                      const VecopsHipOperand* c, void* workspace, uint64_t workspace_size,
                                                      void* stream);

/* vecops_hip_matmul_i8_dequant with b prepacked (i8); workspace as for the
 * plain call with the same extents. */
VECOPS_HIP_EXPORT int32_t vecops_hip_matmul_i8_dequant_packed_b(const int8_t* a, int64_t lda, const void* packed_b,
                                                                const float* row_scales, const float* column_scales,
                                                                const int32_t* correction, float* c, int64_t ldc,
                                                                int64_t m, int64_t n, int64_t k, void* workspace,
                                                                uint64_t workspace_size, void* stream);

/*
 * Measurement yardstick, no counterpart in vecops: `workgroups` workgroups of four wavefronts (one per SIMD) each
 * issue iters x 32 independent matrix-core instructions of the tile kernels' shape (dtype 11: v_mfma_f32_32x32x16_bf16,
 * dtype 2: v_mfma_i32_32x32x32_i8, sixteen 32x32 accumulator tiles per wavefront) on operand registers filled from
 * `operands` (device memory, 16-byte aligned, operand_bytes of it) - no memory traffic inside the loop.  The rate it
 * sustains is what a GEMM on those operand values can reach at most on this machine: the clocks follow the power the
 * multipliers draw.  `out` receives workgroups x 256 words.  vecops_hip_mfma_stream_ops gives the operations one
 * launch performs (2 per multiply-add).
 */
VECOPS_HIP_EXPORT uint64_t vecops_hip_mfma_stream_ops(uint32_t dtype, int32_t workgroups, int32_t iters);
VECOPS_HIP_EXPORT int32_t vecops_hip_mfma_stream(uint32_t dtype, const void* operands, uint64_t operand_bytes,
                                                 int32_t workgroups, int32_t iters, void* out, void* stream);
/*
 * The same yardstick on either matrix-instruction shape the tile kernels use.  shape 0: the 32x32 instructions above;
 * shape 1: v_mfma_f32_16x16x32_bf16 (dtype 11) / v_mfma_i32_16x16x64_i8 (dtype 2), sixteen 16x16 accumulator quads per
 * wavefront - the shape of the 256x256 tile's written-out K loop and of the small tiles, which draws less power per
 * multiply-add.  Operations per launch: vecops_hip_mfma_stream_shape_ops.
 */
VECOPS_HIP_EXPORT uint64_t vecops_hip_mfma_stream_shape_ops(uint32_t dtype, uint32_t shape, int32_t workgroups, int32_t iters);
VECOPS_HIP_EXPORT int32_t vecops_hip_mfma_stream_shape(uint32_t dtype, uint32_t shape, const void* operands,
                                                       uint64_t operand_bytes, int32_t workgroups, int32_t iters, void* out,
                                                       void* stream);

/*
 * Read-only yardstick of the skinny (HBM-bound) kernels, no counterpart in vecops: `workgroups` workgroups of 256 lanes
 * stream the first bytes / 16 16-byte pieces of `src` (16-byte aligned) with eight loads in flight per lane and write
 * one word per lane to `out` (workgroups x 256 words).  Launched back to back on a buffer of a GEMV's size it shows the
 * rate at which this machine delivers that many bytes to any kernel, launch and ramp included.
 */
VECOPS_HIP_EXPORT int32_t vecops_hip_read_stream(const void* src, uint64_t bytes, int32_t workgroups, void* out, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* VECOPS_HIP_H */
