/*
 * TEST INFRASTRUCTURE ONLY.  CPU restatement of the vecops matmul semantics,
 * used as the checker for the gfx950 kernels.  Nothing in the product path
 * (the HIP library, the runtime host code, the artifact DSOs) links, loads or
 * calls this file; only tests, the smoke check and the CPU-baseline leg of the
 * benchmark do.
 *
 * Each function names the reference file:line whose behaviour it restates
 * (paths relative to the vecops tree).
 *
 * Pinning status (what fixes each function besides its own formula):
 *   vo_bf16_from_f32 / vo_f32_from_bf16   - exhaustive agreement with the
 *       "add 0x7fff + lsb, shift" closed form and with IEEE nearest-even
 *       computed in fp64 (tests/test_oracle.py), NaN -> 0x7fc0.
 *   vo_f16_from_f32                       - numpy's float16 conversion on random and
 *       structured inputs, the exhaustive half -> float -> half round trip.
 *   vo_f32_to_i32_sat                     - known answers at the saturation
 *       edges and NaN (tests/test_oracle.py).
 *   vo_matmul (int paths)                 - exact integer arithmetic mod 2^32:
 *       int64 numpy product reduced mod 2^32, the K=262145 wrap case of
 *       tests/ops/MatmulTest.cpp:1025-1055, and the real reference through
 *       oracle/_ref where that library is built.
 *   vo_matmul (floating paths)            - fp64 numpy product on the rounded
 *       inputs, the modular-sequence cases of tests/ops/MatmulTest.cpp:36-97
 *       whose products are exact, and oracle/_ref.
 *   vo_matmul_i8_dequant                  - numpy float32 two-step multiply and
 *       oracle/_ref (bit-exact).
 *   vo_fused_outputs                      - golden vectors of the real reference
 *       (tests/golden: every step, activation and output dtype, byte outputs with
 *       out-of-range and NaN values) and oracle/_ref; sigmoid / silu within the
 *       reference tests' own 8e-4 tolerance, everything else bit for bit.
 *   vo_amx_small_vector_profitable & co   - the static_assert table of
 *       tests/matmul/TilerTest.cpp:86-98.
 *   vo_matmul_w8a16_group                 - the reference has no weight-only
 *       group-scaled matmul; the contract is stated at the function and pinned by
 *       the mathematics (tests/test_oracle.py, test_w8a16_group_*): an independent
 *       float64 einsum, unit scales reducing it to vo_matmul, one group's scale
 *       moving exactly that group's dot, a hand-worked table.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define VO_EXPORT __attribute__((visibility("default")))

/* dtype codes = VecopsDType numeric values (runtime/CallAbi.h:62-91). */
enum { VO_I8 = 2, VO_U8 = 3, VO_I32 = 6, VO_F16 = 10, VO_BF16 = 11, VO_F32 = 12, VO_F64 = 13 };

/* Compute (atom) selection for vo_matmul.
 *   VO_ATOM_BF16F32 : operands rounded to bf16, fp32 accumulate (AMX_BF16F32,
 *                     matmul/details/kernel/amx/Atoms.h:51-60)
 *   VO_ATOM_F32F32  : operands kept in fp32 (SME_F32F32, kernel/sme/Atoms.h:65-76)
 *   VO_ATOM_F16F32  : operands rounded to IEEE half, fp32 accumulate (AMX_F16F32,
 *                     matmul/details/kernel/amx/Atoms.h:62-71; the reference build needs AMX-FP16,
 *                     which the build host lacks: pinned by closed forms only)
 *   VO_ATOM_F64F64  : fp64 operands, fp64 accumulate, one fused multiply-add per k in k order (SME_F64F64,
 *                     kernel/sme/Atoms.h:108-112: FMOPA .d, one fp64 per K step); a, b, cin and c are VO_F64
 *   VO_ATOM_I8I32   : 8-bit integers, int32 accumulate wrapping mod 2^32
 *                     (AMX_I8I32<A,B>, amx/Atoms.h:73-86; wrap pinned by
 *                     tests/ops/MatmulTest.cpp:1025-1055) */
enum { VO_ATOM_BF16F32 = 0, VO_ATOM_F32F32 = 1, VO_ATOM_I8I32 = 2, VO_ATOM_F16F32 = 3, VO_ATOM_F64F64 = 4 };

typedef struct vo_tensor {
  void* data;
  int32_t dtype;
  int32_t rank;        /* 2 or 3 */
  int64_t sizes[3];    /* [batch,] rows, cols */
  int64_t strides[3];  /* elements; 0 = broadcast */
} vo_tensor;

/* ---- scalar conversions -------------------------------------------------- */

static inline uint32_t f32_bits(float x) { uint32_t u; memcpy(&u, &x, 4); return u; }
static inline float bits_f32(uint32_t u) { float x; memcpy(&x, &u, 4); return x; }

/* util/BFloat16.h:25-37: round to nearest even, every NaN becomes 0x7fc0. */
VO_EXPORT uint16_t vo_bf16_from_f32(float x) {
  if (x != x) return 0x7fc0;
  uint32_t bits = f32_bits(x);
  uint32_t bias = ((bits >> 16) & 1u) + 0x7fffu;
  return (uint16_t)((bits + bias) >> 16);
}

/* util/BFloat16.h:57-63: widening is a 16-bit left shift. */
VO_EXPORT float vo_f32_from_bf16(uint16_t h) { return bits_f32((uint32_t)h << 16); }

/* IEEE binary16 -> binary32 (exact). */
static float f32_from_f16(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu, man = h & 0x3ffu;
  if (exp == 0) {
    if (man == 0) return bits_f32(sign);
    float v = ldexpf((float)man, -24);
    return sign ? -v : v;
  }
  if (exp == 31) return bits_f32(sign | 0x7f800000u | (man << 13));
  return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

/* binary32 -> IEEE binary16, round to nearest even, overflow to infinity, NaN kept quiet: what vecops'
 * Float16(float) does through F16C (util/Float16.h, _cvtss_sh with nearest rounding).  Pinned against
 * numpy's float16 conversion on random and structured inputs and by the exhaustive half -> float -> half
 * round trip (tests/test_oracle.py). */
VO_EXPORT uint16_t vo_f16_from_f32(float x) {
  const uint32_t bits = f32_bits(x);
  const uint32_t sign = (bits >> 16) & 0x8000u;
  const uint32_t mag = bits & 0x7fffffffu;
  if (mag > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((mag >> 13) & 0x3ffu));  /* NaN */
  if (mag >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);  /* >= 65520 rounds to infinity (and infinity) */
  if (mag < 0x38800000u) {                                     /* below 2^-14: subnormal half or zero */
    if (mag < 0x33000000u) return (uint16_t)sign;              /* below 2^-25: rounds to zero */
    const uint32_t man = (mag & 0x7fffffu) | 0x800000u;
    const uint32_t shift = 126u - (mag >> 23);                 /* 14 .. 24 */
    const uint32_t kept = man >> shift, rest = man & ((1u << shift) - 1u), half = 1u << (shift - 1u);
    return (uint16_t)(sign | (kept + ((rest > half || (rest == half && (kept & 1u))) ? 1u : 0u)));
  }
  const uint32_t base = ((mag >> 23) - 112u) << 10 | ((mag >> 13) & 0x3ffu);
  const uint32_t rest = mag & 0x1fffu;
  return (uint16_t)(sign | (base + ((rest > 0x1000u || (rest == 0x1000u && (base & 1u))) ? 1u : 0u)));
}

VO_EXPORT float vo_f32_from_f16(uint16_t h);

VO_EXPORT void vo_f16_from_f32_array(const float* in, uint16_t* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = vo_f16_from_f32(in[i]);
}

/* util/ScalarConvert.h:60-86: float -> signed int truncates toward zero after a
 * clamp in the floating domain; NaN -> 0. */
VO_EXPORT int32_t vo_f32_to_i32_sat(float f) {
  if (f != f) return 0;
  const float hi = (float)INT32_MAX; /* rounds to 2^31 */
  const float lo = (float)INT32_MIN;
  if (f >= hi) return INT32_MAX;
  if (f <= lo) return INT32_MIN;
  return (int32_t)f;
}

VO_EXPORT void vo_bf16_from_f32_array(const float* in, uint16_t* out, int64_t n) {
  for (int64_t i = 0; i < n; ++i) out[i] = vo_bf16_from_f32(in[i]);
}

/* ---- element access ------------------------------------------------------- */

static inline int64_t elem_size(int dtype) {
  switch (dtype) {
    case VO_I8: case VO_U8: return 1;
    case VO_F16: case VO_BF16: return 2;
    case VO_F64: return 8;
    default: return 4;
  }
}

static inline float load_as_f32(const void* p, int dtype, int64_t off) {
  switch (dtype) {
    case VO_F32: return ((const float*)p)[off];
    case VO_BF16: return vo_f32_from_bf16(((const uint16_t*)p)[off]);
    case VO_F16: return f32_from_f16(((const uint16_t*)p)[off]);
    case VO_I8: return (float)((const int8_t*)p)[off];
    case VO_U8: return (float)((const uint8_t*)p)[off];
    case VO_I32: return (float)((const int32_t*)p)[off];
    default: return NAN;
  }
}

static inline int32_t load_as_i32(const void* p, int dtype, int64_t off) {
  switch (dtype) {
    case VO_I8: return ((const int8_t*)p)[off];
    case VO_U8: return ((const uint8_t*)p)[off];
    case VO_I32: return ((const int32_t*)p)[off];
    case VO_F32: return vo_f32_to_i32_sat(((const float*)p)[off]);
    default: return 0;
  }
}

/* Output conversion from the accumulator domain to the memory dtype
 * (docs/Tensor.md:253-299; fp32 -> bf16 is RNE, fp32 -> int saturates). */
static inline void store_from_f32(void* p, int dtype, int64_t off, float v) {
  switch (dtype) {
    case VO_F32: ((float*)p)[off] = v; break;
    case VO_BF16: ((uint16_t*)p)[off] = vo_bf16_from_f32(v); break;
    case VO_F16: ((uint16_t*)p)[off] = vo_f16_from_f32(v); break;
    case VO_I32: ((int32_t*)p)[off] = vo_f32_to_i32_sat(v); break;
    default: break;
  }
}

static inline void store_from_i32(void* p, int dtype, int64_t off, int32_t v) {
  switch (dtype) {
    case VO_I32: ((int32_t*)p)[off] = v; break;
    case VO_F32: ((float*)p)[off] = (float)v; break;
    default: break;
  }
}

VO_EXPORT float vo_f32_from_f16(uint16_t h) { return f32_from_f16(h); }

static inline float to_compute(float v, int atom) {
  if (atom == VO_ATOM_F16F32) return f32_from_f16(vo_f16_from_f32(v));
  return atom == VO_ATOM_BF16F32 ? vo_f32_from_bf16(vo_bf16_from_f32(v)) : v;
}

static inline int64_t boff(const vo_tensor* t, int64_t batch) {
  return t->rank == 3 ? batch * t->strides[0] : 0;
}
static inline int64_t rs(const vo_tensor* t) { return t->strides[t->rank - 2]; }
static inline int64_t cs(const vo_tensor* t) { return t->strides[t->rank - 1]; }
static inline int64_t rows(const vo_tensor* t) { return t->sizes[t->rank - 2]; }
static inline int64_t cols(const vo_tensor* t) { return t->sizes[t->rank - 1]; }

/* planning/families/ArchitectureFamily.h:1590-1652 and GenericTiled.h:100-154:
 * equal ranks, non-negative extents, A=[..,M,K], B=[..,N,K], C=[..,M,N], batch
 * extents equal across operands.  Returns 0 when well formed. */
static int validate(const vo_tensor* a, const vo_tensor* b, const vo_tensor* cin, const vo_tensor* c) {
  if (a->rank != b->rank || a->rank != c->rank || (a->rank != 2 && a->rank != 3)) return 1;
  if (cin && cin->rank != a->rank) return 1;
  for (int i = 0; i < a->rank; ++i)
    if (a->sizes[i] < 0 || b->sizes[i] < 0 || c->sizes[i] < 0) return 1;
  if (cols(a) != cols(b) || rows(c) != rows(a) || cols(c) != rows(b)) return 1;
  if (cin && (rows(cin) != rows(c) || cols(cin) != cols(c))) return 1;
  if (a->rank == 3) {
    if (a->sizes[0] != b->sizes[0] || a->sizes[0] != c->sizes[0]) return 1;
    if (cin && cin->sizes[0] != c->sizes[0]) return 1;
  }
  return 0;
}

/*
 * C[..,M,N] = Cin + A[..,M,K] . B[..,N,K]^T      (ops/Matmul.h:13-17,530-570)
 *
 * Pipeline per output element (planning/families/ArchitectureFamily.h:
 * 2025-2030): load -> convert to the atom's compute type -> multiply-accumulate
 * in TAcc -> add Cin converted to TAcc -> convert to the memory dtype of C.
 * Zero K writes zeros (single-C form) or Cin (explicit-C form); zero M, N or
 * batch writes nothing (ops/Matmul.h:41-43).
 *
 * acc_f64 != 0 accumulates floating paths in double, in k order, and rounds to
 * float once at the end: the tolerance anchor for kernels whose fp32 summation
 * order differs (vec/WideningDot.h:100-103 leaves that order unspecified).
 * acc_f64 == 0 is the sequential fp32 loop of tests/ops/MatmulTest.cpp:82-90.
 */
VO_EXPORT int vo_matmul(const vo_tensor* a, const vo_tensor* b, const vo_tensor* cin, const vo_tensor* c,
                        int atom, int acc_f64) {
  if (validate(a, b, cin, c)) return 1;
  if ((atom == VO_ATOM_F64F64) != (a->dtype == VO_F64) || (a->dtype == VO_F64) != (b->dtype == VO_F64) ||
      (a->dtype == VO_F64) != (c->dtype == VO_F64) || (cin && (cin->dtype == VO_F64) != (c->dtype == VO_F64)))
    return 1;  /* fp64 operands go with the fp64 atom and nothing else */
  const int64_t batch = a->rank == 3 ? a->sizes[0] : 1;
  const int64_t M = rows(a), N = rows(b), K = cols(a);
  if (batch == 0 || M == 0 || N == 0) return 0;
  for (int64_t bi = 0; bi < batch; ++bi) {
    const int64_t ao = boff(a, bi), bo = boff(b, bi), co = boff(c, bi), cio = cin ? boff(cin, bi) : 0;
#pragma omp parallel for schedule(dynamic, 4)
    for (int64_t i = 0; i < M; ++i) {
      for (int64_t j = 0; j < N; ++j) {
        const int64_t ci = co + i * rs(c) + j * cs(c);
        if (atom == VO_ATOM_F64F64) {
          double acc = 0.0;
          for (int64_t k = 0; k < K; ++k)
            acc = fma(((const double*)a->data)[ao + i * rs(a) + k * cs(a)], ((const double*)b->data)[bo + j * rs(b) + k * cs(b)], acc);
          if (cin) acc += ((const double*)cin->data)[cio + i * rs(cin) + j * cs(cin)];
          ((double*)c->data)[ci] = acc;
        } else if (atom == VO_ATOM_I8I32) {
          uint32_t acc = 0;
          for (int64_t k = 0; k < K; ++k) {
            int32_t x = load_as_i32(a->data, a->dtype, ao + i * rs(a) + k * cs(a));
            int32_t y = load_as_i32(b->data, b->dtype, bo + j * rs(b) + k * cs(b));
            acc += (uint32_t)(x * y);
          }
          if (cin) acc += (uint32_t)load_as_i32(cin->data, cin->dtype, cio + i * rs(cin) + j * cs(cin));
          store_from_i32(c->data, c->dtype, ci, (int32_t)acc);
        } else {
          float result;
          if (acc_f64) {
            double acc = 0.0;
            for (int64_t k = 0; k < K; ++k) {
              float x = to_compute(load_as_f32(a->data, a->dtype, ao + i * rs(a) + k * cs(a)), atom);
              float y = to_compute(load_as_f32(b->data, b->dtype, bo + j * rs(b) + k * cs(b)), atom);
              acc += (double)x * (double)y;
            }
            if (cin) acc += (double)load_as_f32(cin->data, cin->dtype, cio + i * rs(cin) + j * cs(cin));
            result = (float)acc;
          } else {
            float acc = 0.0f;
            for (int64_t k = 0; k < K; ++k) {
              float x = to_compute(load_as_f32(a->data, a->dtype, ao + i * rs(a) + k * cs(a)), atom);
              float y = to_compute(load_as_f32(b->data, b->dtype, bo + j * rs(b) + k * cs(b)), atom);
              acc += x * y;
            }
            if (cin) acc += load_as_f32(cin->data, cin->dtype, cio + i * rs(cin) + j * cs(cin));
            result = acc;
          }
          store_from_f32(c->data, c->dtype, ci, result);
        }
      }
    }
  }
  return 0;
}

/*
 * Fused output transform on finished accumulators (the accumulator already holds
 * C_in / the bias row): the restatement of what vecops' tests attach to
 * tensor::output as elementwise and lane-local transforms
 * (tests/ops/MatmulConversionTestCommon.h: per-column scale :652-660, runtime scale
 * :647-651, clamp :735-740, relu :1047-1050, sigmoid :1051-1057, silu :1121-1128,
 * requantisation :1222-1234), in this order, each step one fp32 operation:
 *   v = float(acc);  v *= row_scales[row];  v *= column_scales[col];  v *= scale (flags & 1);
 *   v += shift (flags & 2);  v = activation(v);  c = convert(v)
 * acc_is_int selects int32 accumulators (converted with a plain int -> float cast).
 * sigmoid and silu are evaluated in double and rounded once (the tests' own
 * expectation, :1086-1087, :1157-1160); the reference's vector exp differs from that by
 * a few ulp, so they are compared with a tolerance, the others bit for bit.
 * out_dtype: VO_F32, VO_BF16 (round to nearest even), VO_U8 / VO_I8: the x86 vector
 * store (vec/details/x86/Conversion.h:522-528) = truncating convert to int32, where NaN
 * and values outside int32 give INT32_MIN, then a saturating narrow.
 * Pinned by golden vectors of the real reference (tests/golden) for every step and
 * output dtype, including the out-of-range and NaN cases of the byte outputs.
 */
static int32_t cvtt_i32(float v) {
  if (!(v >= -2147483648.0f && v < 2147483648.0f)) return INT32_MIN;
  return (int32_t)v;
}

VO_EXPORT int vo_fused_outputs(const void* acc, int acc_is_int, int64_t M, int64_t N, const float* row_scales,
                               const float* column_scales, uint32_t flags, float scale, float shift, int activation,
                               float lo, float hi, int out_dtype, void* out) {
  if (activation < 0 || activation > 4) return 1;
  for (int64_t i = 0; i < M; ++i) {
    for (int64_t j = 0; j < N; ++j) {
      const int64_t at = i * N + j;
      float v = acc_is_int ? (float)((const int32_t*)acc)[at] : ((const float*)acc)[at];
      if (row_scales) v = v * row_scales[i];
      if (column_scales) v = v * column_scales[j];
      if (flags & 1u) v = v * scale;
      if (flags & 2u) v = v + shift;
      switch (activation) {
        case 1: v = (v > 0.0f) ? v : 0.0f; break;                        /* max_ps(v, 0): NaN -> 0 */
        case 2: v = (v > lo) ? v : lo; v = (v < hi) ? v : hi; break;     /* min_ps(max_ps(v, lo), hi) */
        case 3: v = (float)(1.0 / (1.0 + exp(-(double)v))); break;
        case 4: v = (float)((double)v / (1.0 + exp(-(double)v))); break;
        default: break;
      }
      switch (out_dtype) {
        case VO_F32: ((float*)out)[at] = v; break;
        case VO_BF16: ((uint16_t*)out)[at] = vo_bf16_from_f32(v); break;
        case VO_U8: { int32_t t = cvtt_i32(v); ((uint8_t*)out)[at] = (uint8_t)(t < 0 ? 0 : t > 255 ? 255 : t); break; }
        case VO_I8: { int32_t t = cvtt_i32(v); ((int8_t*)out)[at] = (int8_t)(t < -128 ? -128 : t > 127 ? 127 : t); break; }
        default: return 1;
      }
    }
  }
  return 0;
}

/* RuntimePerRowAsymmetricQuantizeTransform (matmul/Quantization.h:91-146, formula :123-128) followed
 * by the conversion of the transformed fp32 value to the atom's uint8 compute type:
 *   q[r][k] = u8( a[r][k] * multipliers[r] + (float)zero_point )
 * - a multiply and an add, each rounded to fp32 (two vector instructions, never fused), then the x86
 * vector conversion cvtt_i32 above (truncation toward zero; NaN and values outside int32 give
 * INT32_MIN) and a saturating narrow to 0..255.  Pinned by golden vectors of the real vecops build
 * (tests/golden/vecops_quant_golden.npz): an edge-value table read back through an identity B, and
 * elements built so that a fused multiply-add would give a different byte. */
VO_EXPORT void vo_quantize_rows_u8(const float* a, int64_t M, int64_t K, int64_t lda, const float* multipliers,
                                   int32_t zero_point, uint8_t* q, int64_t ldq) {
  const float zp = (float)zero_point;
  for (int64_t r = 0; r < M; ++r)
    for (int64_t k = 0; k < K; ++k) {
      volatile float prod = a[r * lda + k] * multipliers[r];
      const float t = prod + zp;
      const int32_t v = cvtt_i32(t);
      q[r * ldq + k] = (uint8_t)(v < 0 ? 0 : v > 255 ? 255 : v);
    }
}

/* Selected outputs of the rank-2 product only: out[s] = acc(rows_idx[s], cols_idx[s])
 * as double (floating atoms) - lets a test check a 4096^3 product in seconds.  Pinned against
 * vo_matmul's float64 accumulators at the same indices (tests/test_oracle.py). */
VO_EXPORT int vo_matmul_sampled(const vo_tensor* a, const vo_tensor* b, int atom, const int64_t* rows_idx,
                                const int64_t* cols_idx, int64_t count, double* out) {
  if (a->rank != 2 || b->rank != 2 || cols(a) != cols(b)) return 1;
  const int64_t K = cols(a);
#pragma omp parallel for schedule(static)
  for (int64_t s = 0; s < count; ++s) {
    const int64_t i = rows_idx[s], j = cols_idx[s];
    double acc = 0.0;
    for (int64_t k = 0; k < K; ++k) {
      float x = to_compute(load_as_f32(a->data, a->dtype, i * rs(a) + k * cs(a)), atom);
      float y = to_compute(load_as_f32(b->data, b->dtype, j * rs(b) + k * cs(b)), atom);
      acc += (double)x * (double)y;
    }
    out[s] = acc;
  }
  return 0;
}

/* Dense K-contiguous int8 x int8 -> int32 (wrapping), written so the compiler
 * can vectorise it: integer addition is associative, so any order is exact.
 * Same semantics as vo_matmul with VO_ATOM_I8I32 on dense operands. */
VO_EXPORT void vo_matmul_i8_dense(const int8_t* a, const int8_t* b, int32_t* c, int64_t M, int64_t N, int64_t K) {
#pragma omp parallel for schedule(dynamic, 8)
  for (int64_t i = 0; i < M; ++i) {
    const int8_t* ar = a + i * K;
    for (int64_t j = 0; j < N; ++j) {
      const int8_t* br = b + j * K;
      int32_t acc = 0;
      for (int64_t k = 0; k < K; ++k) acc += (int32_t)ar[k] * (int32_t)br[k];
      c[i * N + j] = acc;
    }
  }
}

/*
 * c[i,j] = (float(acc[i,j]) * row_scales[i]) * column_scales[j]
 * matmul/Quantization.h:195-250 (vector form :224-231, scalar form :240-243;
 * restated without vectors in src/arch/sme/RuntimeQuantInt8.cpp:80-92): two
 * separate fp32 multiplies, row scale first, no fused multiply-add.
 * acc = sum_k a[i,k]*b[j,k] (+ correction[j], the stride-0 int32 C-input row of
 * tests/ops/MatmulConversionTestCommon.h:1467-1472,1503-1510), wrapping int32.
 */
VO_EXPORT void vo_matmul_i8_dequant(const int8_t* a, const int8_t* b, const float* row_scales,
                                    const float* column_scales, const int32_t* correction, float* c, int64_t M,
                                    int64_t N, int64_t K) {
#pragma omp parallel for schedule(dynamic, 8)
  for (int64_t i = 0; i < M; ++i) {
    const int8_t* ar = a + i * K;
    for (int64_t j = 0; j < N; ++j) {
      const int8_t* br = b + j * K;
      int32_t acc = 0;
      for (int64_t k = 0; k < K; ++k) acc += (int32_t)ar[k] * (int32_t)br[k];
      if (correction) acc = (int32_t)((uint32_t)acc + (uint32_t)correction[j]);
      volatile float t = (float)acc * row_scales[i]; /* volatile: forbid contraction */
      c[i * N + j] = t * column_scales[j];
    }
  }
}

/*
 * Weight-only int8 with per-group scales (no reference counterpart; contract
 * stated by this build):
 *   y[m,n] = bf16_rne( sum_g S[n,g] * sum_{k in group g} float(x[m,k]) * float(W[n,k]) )
 * x bf16 [M,K], W int8 [N,K], S fp32 [N,K/G], y bf16 [M,N].  Accumulated here
 * in double; kernels accumulate in fp32 and are compared with a tolerance.
 * Pinned (tests/test_oracle.py, test_w8a16_group_*) by a numpy float64 einsum that shares
 * no loop with this one, by unit scales reducing it to vo_matmul, by one group's scale
 * moving exactly that group's dot, and by a hand-worked table.
 */
VO_EXPORT int vo_matmul_w8a16_group(const uint16_t* x, const int8_t* w, const float* scales, uint16_t* y,
                                    double* y_f64, int64_t M, int64_t N, int64_t K, int64_t G) {
  if (G <= 0 || K % G != 0) return 1;
  const int64_t groups = K / G;
#pragma omp parallel for schedule(dynamic, 16)
  for (int64_t n = 0; n < N; ++n) {
    for (int64_t m = 0; m < M; ++m) {
      double total = 0.0;
      for (int64_t g = 0; g < groups; ++g) {
        double part = 0.0;
        for (int64_t k = g * G; k < (g + 1) * G; ++k)
          part += (double)vo_f32_from_bf16(x[m * K + k]) * (double)w[n * K + k];
        total += (double)scales[n * groups + g] * part;
      }
      if (y) y[m * N + n] = vo_bf16_from_f32((float)total);
      if (y_f64) y_f64[m * N + n] = total;
    }
  }
  return 0;
}

/* ---- runtime dispatch predicates -------------------------------------------
 * matmul/details/kernel/RuntimeDispatch.h:14-83 and the non-inline wrappers of
 * src/MatmulRuntimeDispatch.cpp:12-32. */
enum { VO_SHAPE_AMX_BF16 = 0, VO_SHAPE_AMX_I8_SAME = 1, VO_SHAPE_AMX_I8_MIXED = 2, VO_SHAPE_SME_F16 = 3,
       VO_SHAPE_SME_OTHER = 4 };

static int area_at_most(int64_t m, int64_t n, int64_t limit) { return m > 0 && n > 0 && n <= limit / m; }
static int skinny_at_most(int64_t m, int64_t n, int64_t limit) {
  return (m == 1 && 1 <= n && n <= limit) || (n == 1 && 1 <= m && m <= limit);
}
static int large_m1(int64_t m, int64_t n) { return m == 1 && 128 <= n && n <= 4096; }
static int large_n1(int64_t m, int64_t n) { return n == 1 && 128 <= m && m <= 4096; }

VO_EXPORT int vo_amx_small_vector_profitable(int shape, int64_t m, int64_t n, int64_t k) {
  if (m < 1 || n < 1 || k < 1) return 0;
  if (skinny_at_most(m, n, 64)) return 1;
  if (shape == VO_SHAPE_AMX_BF16)
    return area_at_most(m, n, 16) || (area_at_most(m, n, 32) && k <= 256) || (area_at_most(m, n, 64) && k <= 64) ||
           (k >= 32 && k % 32 <= 1 && (large_m1(m, n) || (large_n1(m, n) && k != 256)));
  if (shape == VO_SHAPE_AMX_I8_SAME)
    return area_at_most(m, n, 32) || (k >= 64 && k % 64 <= 1 && (large_m1(m, n) || large_n1(m, n)));
  if (shape == VO_SHAPE_AMX_I8_MIXED)
    return area_at_most(m, n, 32) || (area_at_most(m, n, 64) && k <= 128) ||
           (k >= 64 && k % 64 <= 1 && (large_m1(m, n) || (large_n1(m, n) && k != 64)));
  return 0;
}

VO_EXPORT int vo_sme_small_vector_profitable(int shape, int64_t m, int64_t n, int64_t k) {
  if (m < 0 || n < 0 || k < 0) return 0;
  const int64_t limit = shape == VO_SHAPE_SME_F16 ? 16 : 64;
  return (m == 1 && n <= limit) || (n == 1 && m <= limit);
}

VO_EXPORT int vo_small_area_profitable(int64_t m, int64_t n, int64_t k, int64_t limit) {
  return k > 0 && area_at_most(m, n, limit);
}

VO_EXPORT int vo_amx_residual_split_profitable(int64_t m, int64_t n, int64_t k) {
  const int sm = m == 17 || m == 18 || m == 20, sn = n == 33 || n == 47 || n == 48;
  const int tm = n == 17 || n == 18 || n == 20, tn = m == 33 || m == 47 || m == 48;
  return ((sm && sn) || (tm && tn)) && k == 1024;
}

/* ---- CPU-baseline kernels (timed by the benchmark, never used as a checker of
 * themselves): the same semantics as vo_matmul on dense K-contiguous operands,
 * written so the compiler vectorises them across all host cores. -------------- */
#include <omp.h>

VO_EXPORT int vo_threads(void) { return omp_get_max_threads(); }

/* bf16 x bf16 -> fp32 accumulate -> fp32 or bf16 out (AMX_BF16F32 semantics,
 * vectorised summation order). */
VO_EXPORT void vo_matmul_bf16_dense(const uint16_t* a, const uint16_t* b, float* c_f32, uint16_t* c_bf16, int64_t M,
                                    int64_t N, int64_t K) {
  float* bf = (float*)malloc((size_t)N * K * sizeof(float));
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < N * K; ++i) bf[i] = vo_f32_from_bf16(b[i]);
#pragma omp parallel
  {
    float* ar = (float*)malloc((size_t)K * sizeof(float));
#pragma omp for schedule(dynamic, 1)
    for (int64_t i = 0; i < M; ++i) {
      for (int64_t k = 0; k < K; ++k) ar[k] = vo_f32_from_bf16(a[i * K + k]);
      for (int64_t j = 0; j < N; ++j) {
        const float* br = bf + j * K;
        float acc = 0.0f;
#pragma omp simd reduction(+ : acc)
        for (int64_t k = 0; k < K; ++k) acc += ar[k] * br[k];
        if (c_f32) c_f32[i * N + j] = acc;
        if (c_bf16) c_bf16[i * N + j] = vo_bf16_from_f32(acc);
      }
    }
    free(ar);
  }
  free(bf);
}
