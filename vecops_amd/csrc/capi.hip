// C ABI of libvecops_hip.so (declared in include/vecops_hip.h): operand
// validation, the GPU kernel-selection rule table and the kernel launches.
#include <hip/hip_runtime.h>

#include <atomic>
#include <vector>
#include <cstdarg>
#include <cstdio>
#include <cstring>

#include "gemm_f64.h"
#include "skinny_dense.h"
#include "skinny_w8a16.h"
#include "tile_gemm_launch.h"
#include "tile_gemm_packed.h"
#include "vecops_hip.h"

namespace {

using namespace vecops_hip;

enum : int32_t { ST_OK = 0, ST_INVALID = 1, ST_NOT_APPLICABLE = 2, ST_EXEC = 6 };
enum : uint32_t { DT_I8 = 2, DT_U8 = 3, DT_I32 = 6, DT_F16 = 10, DT_BF16 = 11, DT_F32 = 12, DT_F64 = 13 };
// fp64 operands run on a kernel of their own (gemm_f64.hip), outside the tile kernels' operand classes and outputs
constexpr int kSrcF64 = 100, kOutF64 = 100;

thread_local char g_error[512] = "";

int32_t fail(int32_t code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

int64_t dtype_bytes(uint32_t dt) {
  switch (dt) {
    case DT_I8: case DT_U8: return 1;
    case DT_F16: case DT_BF16: return 2;
    case DT_I32: case DT_F32: return 4;
    case DT_F64: return 8;
    default: return 0;
  }
}

struct View {  // rank-3 normalised operand
  void* data;
  uint32_t dtype;
  int64_t batch, rows, cols;
  int64_t bs, rs, cs;
};

bool normalise(const VecopsHipOperand* o, View* v) {
  if (o == nullptr || (o->rank != 2 && o->rank != 3)) return false;
  const int base = o->rank == 3 ? 1 : 0;
  v->data = o->data;
  v->dtype = o->dtype;
  v->batch = o->rank == 3 ? o->sizes[0] : 1;
  v->bs = o->rank == 3 ? o->strides[0] : 0;
  v->rows = o->sizes[base];
  v->cols = o->sizes[base + 1];
  v->rs = o->strides[base];
  v->cs = o->strides[base + 1];
  return v->batch >= 0 && v->rows >= 0 && v->cols >= 0;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
uint64_t round_up_256(uint64_t v) { return (v + 255u) & ~uint64_t{255}; }

// 16-byte loads along K: unit K stride.  Rows need not be 16-byte aligned: global and buffer loads
// take any byte address on this target (the compiler itself emits dwordx4 loads for under-aligned
// vectors); a misaligned chunk merely touches one more cache line.  The kernels address a tile
// through a buffer descriptor based at its first row, with a 32-bit byte offset per lane (up to
// 256 rows) plus the K offset: together they must stay below 2 GiB.
bool k_vector_ok(const View& v) {
  const int64_t eb = dtype_bytes(v.dtype);
  return v.cs == 1 && v.rs >= 0 && (v.rs * 256 + v.cols + 256) * eb < (int64_t{1} << 31);
}

// B stored [K,N] row-major: unit stride along N and N a multiple of 8 elements (the loader has no
// N tail), 16-bit or 32-bit source elements.
bool n_vector_ok(const View& v) {
  const int64_t eb = dtype_bytes(v.dtype);
  return v.rs == 1 && v.rows % 8 == 0 && v.rows >= 8 && v.cs > 0 &&
         (v.cs * 64 + 512) * eb < (int64_t{1} << 31);  // 32-bit offsets inside a K tile
}

struct Problem {
  View a, b, c, cin;
  bool has_cin;
  int src;       // SrcKind
  bool a_unsigned, b_unsigned;  // 8-bit integer operands only
  int out_kind;  // OutKind
  int cin_kind;
  int64_t batch, m, n, k;
  bool packed_b;  // b.data addresses a prepacked operand (vecops_hip_pack_b), shared by every batch
  bool dequant;   // the int32 accumulators leave through the per-row x per-column dequantisation
  int64_t row_scales_bs, correction_bs;  // batch b reads row_scales[b * row_scales_bs + row], correction[b * correction_bs + col]
  const VecopsHipEpilogue* fused;  // non-null: c is written through the fused output transform
};

// Same rules as vecops' validate() (planning/families/ArchitectureFamily.h:1590-1652,
// planning/families/GenericTiled.h:100-154) plus the dtype combinations this library implements.
int32_t describe(const VecopsHipOperand* a, const VecopsHipOperand* b, const VecopsHipOperand* cin,
                 const VecopsHipOperand* c, uint32_t compute, Problem* pr, const VecopsHipEpilogue* fused = nullptr,
                 bool may_fold = true) {
  pr->fused = fused;
  pr->row_scales_bs = pr->correction_bs = 0;
  if (!normalise(a, &pr->a) || !normalise(b, &pr->b) || !normalise(c, &pr->c))
    return fail(ST_INVALID, "matmul: operands must be rank 2 or 3 with non-negative extents");
  pr->packed_b = false;
  pr->dequant = false;
  pr->has_cin = cin != nullptr;
  if (pr->has_cin && !normalise(cin, &pr->cin)) return fail(ST_INVALID, "matmul: malformed c_in");
  if (a->rank != b->rank || a->rank != c->rank || (pr->has_cin && cin->rank != c->rank))
    return fail(ST_INVALID, "matmul: operand ranks differ");
  if (pr->a.cols != pr->b.cols)
    return fail(ST_INVALID, "matmul: K of a (%lld) and b (%lld) differ", (long long)pr->a.cols, (long long)pr->b.cols);
  if (pr->c.rows != pr->a.rows || pr->c.cols != pr->b.rows)
    return fail(ST_INVALID, "matmul: c must be [M=%lld, N=%lld]", (long long)pr->a.rows, (long long)pr->b.rows);
  if (pr->a.batch != pr->b.batch || pr->a.batch != pr->c.batch)
    return fail(ST_INVALID, "matmul: batch extents differ");
  if (pr->has_cin && (pr->cin.rows != pr->c.rows || pr->cin.cols != pr->c.cols || pr->cin.batch != pr->c.batch))
    return fail(ST_INVALID, "matmul: c_in extents differ from c");
  pr->batch = pr->a.batch;
  pr->m = pr->a.rows;
  pr->n = pr->b.rows;
  pr->k = pr->a.cols;
  if (pr->m > INT32_MAX || pr->n > INT32_MAX || pr->k > INT32_MAX - 256 || pr->batch > 65535 * 16)
    return fail(ST_INVALID, "matmul: extent too large");

  const uint32_t da = pr->a.dtype, db = pr->b.dtype, dc = pr->c.dtype;
  const bool bytes_a = da == DT_I8 || da == DT_U8, bytes_b = db == DT_I8 || db == DT_U8;
  pr->a_unsigned = da == DT_U8;
  pr->b_unsigned = db == DT_U8;
  if (da != db && !(bytes_a && bytes_b))
    return fail(ST_NOT_APPLICABLE, "matmul: a and b dtypes differ (%u, %u)", da, db);
  if (bytes_a) {
    // AMX_I8I32<A, B> with A, B in {int8, uint8} (matmul/details/kernel/amx/Atoms.h:73-86)
    pr->src = (pr->a_unsigned || pr->b_unsigned) ? SRC_I8_FLIP : SRC_I8;
  } else if (da == DT_BF16) {
    pr->src = SRC_BF16;
  } else if (da == DT_F16) {
    pr->src = SRC_F16;  // AMX_F16F32 / SME_F16F32 (matmul/details/kernel/amx/Atoms.h:62-71)
  } else if (da == DT_F64) {
    pr->src = kSrcF64;  // SME_F64F64 (matmul/details/kernel/sme/Atoms.h:108-112)
    if (fused) return fail(ST_NOT_APPLICABLE, "matmul_fused: fp64 operands have no fused output transform");
  } else if (da == DT_F32) {
    if (compute != VECOPS_HIP_COMPUTE_BF16 && compute != VECOPS_HIP_COMPUTE_F32)
      return fail(ST_INVALID, "matmul: unknown compute type %u", compute);
    pr->src = compute == VECOPS_HIP_COMPUTE_F32 ? SRC_F32 : SRC_F32_AS_BF16;
  } else {
    return fail(ST_NOT_APPLICABLE, "matmul: operand dtype %u not supported", da);
  }
  const bool is_int = pr->src == SRC_I8 || pr->src == SRC_I8_FLIP;
  if (is_int && fused) {
    // the transform works on float(accumulator); the result is stored as fp32 or as a requantised byte
    if (dc == DT_F32) pr->out_kind = OUT_F32;
    else if (dc == DT_U8) pr->out_kind = OUT_U8;
    else if (dc == DT_I8) pr->out_kind = OUT_I8;
    else return fail(ST_NOT_APPLICABLE, "matmul_fused: int8 operands need an f32, u8 or i8 c");
  } else if (is_int) {
    if (dc != DT_I32) return fail(ST_NOT_APPLICABLE, "matmul: int8 operands need an int32 c");
    pr->out_kind = OUT_I32;
  } else if (pr->src == kSrcF64) {
    if (dc != DT_F64) return fail(ST_NOT_APPLICABLE, "matmul: fp64 operands need an fp64 c");
    pr->out_kind = kOutF64;
  } else {
    if (dc == DT_F32) pr->out_kind = OUT_F32;
    else if (dc == DT_BF16 && pr->src != SRC_F16) pr->out_kind = OUT_BF16;
    else if (dc == DT_F16 && pr->src == SRC_F16) pr->out_kind = OUT_F16;
    else return fail(ST_NOT_APPLICABLE, "matmul: floating operands need an f32 c or one of their own 16-bit type");
  }
  // Rank 3 with one B for every batch and the rows of A and C (and C_in) running on from batch to batch:
  // the same product as [batch * M, K] x B - folded into one rank-2 problem, which fills bigger tiles
  // (vecops' shared-operand flattening, planning/families/ArchitectureFamily.h:430-463).
  auto rows_run_on = [](const View& v) { return v.bs == v.rows * v.rs; };
  if (may_fold && pr->batch > 1 && pr->b.bs == 0 && pr->m > 0 && rows_run_on(pr->a) && rows_run_on(pr->c) &&
      (!pr->has_cin || rows_run_on(pr->cin) || (pr->cin.bs == 0 && pr->cin.rs == 0)) &&
      pr->batch * pr->m <= INT32_MAX) {
    for (View* v : {&pr->a, &pr->c, &pr->cin}) {
      v->rows *= pr->batch;
      v->batch = 1;
      v->bs = 0;
    }
    pr->b.batch = 1;
    pr->m *= pr->batch;
    pr->batch = 1;
  }
  // The mirror case: one row of A for every batch (M = 1, batch stride 0) against weights whose rows run on from
  // batch to batch, the outputs laid end to end: the [1, batch * N] product of A with [batch * N, K]
  // (vecops' batch-columns flattening, planning/families/ArchitectureBatchPlanner.h:82-160).  A per-column C input
  // shared by every batch has no such view and keeps the batched form.
  auto cols_run_on = [](const View& v) { return v.bs == v.cols * v.cs; };
  if (may_fold && pr->batch > 1 && pr->m == 1 && pr->a.bs == 0 && pr->n > 0 && rows_run_on(pr->b) && cols_run_on(pr->c) &&
      (!pr->has_cin || cols_run_on(pr->cin)) && pr->batch * pr->n <= INT32_MAX) {
    pr->b.rows *= pr->batch;
    for (View* v : {&pr->c, &pr->cin}) v->cols *= pr->batch;
    for (View* v : {&pr->a, &pr->b, &pr->c, &pr->cin}) {
      v->batch = 1;
      v->bs = 0;
    }
    pr->n *= pr->batch;
    pr->batch = 1;
  }
  pr->cin_kind = is_int ? OUT_I32 : pr->out_kind;
  if (pr->has_cin) {
    const uint32_t di = pr->cin.dtype;
    if (is_int) {
      if (di != DT_I32) return fail(ST_NOT_APPLICABLE, "matmul: c_in must be int32");
      pr->cin_kind = OUT_I32;
    } else if (pr->src == kSrcF64) {
      if (di != DT_F64) return fail(ST_NOT_APPLICABLE, "matmul: c_in must be fp64");
      pr->cin_kind = kOutF64;
    } else if (di == DT_F32) {
      pr->cin_kind = OUT_F32;
    } else if (di == DT_BF16 && pr->src != SRC_F16) {
      pr->cin_kind = OUT_BF16;
    } else if (di == DT_F16 && pr->src == SRC_F16) {
      pr->cin_kind = OUT_F16;
    } else {
      return fail(ST_NOT_APPLICABLE, "matmul: c_in must be f32 or the operands' 16-bit type");
    }
  }
  return ST_OK;
}

constexpr int kComputeUnits = 256;
constexpr int kStreamGroupsPerUnit = 2;  // workgroups of 4 wavefronts per compute unit of the streaming GEMV
// Work per compute unit and second of the smaller tiles relative to 256x256, per mille (see choose()): bf16 4096^3
// required of each tile family (`bench.py --only families`) takes 105 / 133 / 130 / 112 us (256x256, 256x128, 128x256,
// 128x128; two 128x128 workgroups share a compute unit), 5120^3 221 / 309 / 307 / 255, 2048 x 14336 x 4096
// 185 / 247 / 246 / 204; int8 4096^3 70 / 83 / 84 / 71.5, 5120^3 142 / 184 / 192 / 150, 2048 x 14336 x 4096
// 123 / 153 / 159 / 127.
// Operands that go through registers into LDS (rows that are not 16-byte aligned, fp32 memory, unsigned bytes) keep
// the pricing their kernels were calibrated with: 0.85, rounds of 256, and the margin of the rectangles (8 x 777 x
// 1000 x 3001 64 us on 128x256 tiles against 73.5 on 128x128; fp32 memory 2048^3 32 us on 128x128 against 43).
// Where the loads write LDS themselves the 256x256 tile runs its written-out K loop on the 16x16 matrix instructions,
// a tenth faster than before, and the smaller tiles are priced against that: bf16 4096^3 93 / 122 / 118 / 114 us (the
// rectangles on the 16x16 shapes; 133 / 130 before), int8 4096^3 58 / 75 / 77 / 70 (`bench.py --only families`,
// `--only rule_check`).
constexpr int64_t kQuality256x128 = 800, kQuality128 = 900, kQuality128Int8 = 970, kQuality128Staged = 850;
constexpr int64_t kQuality256x128Direct = 780, kQuality128Direct = 830, kQuality128Int8Direct = 850, kQuality192 = 850;

// Every other number the rule table and the split rule compare against, in one place, each with the mechanism it
// stands for and the command that measures it.  `bench.py --only rule_check` runs nineteen shapes on every tile family
// and K split against the table's own plan and reports the regret: the regression test of these constants.
struct RuleConstants {
  // -- occupancy: a candidate tile must give at least this share of the compute units a workgroup (a tile shape that
  //    leaves more than half the chip idle loses to the next smaller one; rule_check, 384 x 384 x 1024 .. 1024 x 4096^2)
  int64_t min_busy_num = 1, min_busy_den = 2;
  // -- two 128x128 workgroups share a compute unit where the loads write LDS themselves (64 KiB of LDS, 256 registers)
  int64_t small_tile_workgroups_per_unit = 2;
  // -- a rectangle must undercut the bigger tile's cost by this margin: its round count flatters it (more L2 traffic
  //    per flop); rule_check, 1536 / 2048 x 4096 x 4096
  int64_t rectangle_margin_num = 11, rectangle_margin_den = 10;
  // -- more 64x64 tiles than this many rounds of the chip: 128x128 tiles after all
  int64_t many_small_tiles_rounds = 4;
  // -- fp32 compute (64-cycle matrix instructions, no power limit in sight): time follows the tiles the fullest compute
  //    unit gets times their area, so up to this many 128x128 tiles (one each on three quarters of the units) lose to
  //    four times as many 64x64 ones (three each); fp32 1536^3 103 -> 75-78 us
  int64_t f32_small_tiles_up_to_tiles128 = 192;
  // -- a tile's life is its start-up and its stores when K is this short (K tiles of 16-bit / 8-bit operands): small
  //    tiles, of which two or three overlap on a unit; `bench.py --only batched --batched-shape 3000,3000,17`
  int64_t short_k_tiles_16bit = 4, short_k_tiles_8bit = 8;
  // -- at most this share of the units holding one 128x128 workgroup each: 64x64 tiles instead (512 x 4096 x 4096)
  int64_t lonely_tiles_num = 3, lonely_tiles_den = 4;
  // -- the mid band (CU / 8 .. CU tiles of 128x128) splits K so that two workgroups sit on every unit: K tiles a part
  //    must keep (one workgroup's per-tile latency, 0.3 us, against a second kernel and the partial sums' round trip),
  //    from 200 tiles on twice as many; never fewer than min_parts where the tiles are few (rule_check, 768 x 3072 x
  //    12288, 512 x 2048 x 16384, 1024 x 4096 x 11008)
  int64_t band_k_tiles_per_part = 20, band_k_tiles_per_part_full = 40, band_full_from_tiles = 200, band_min_parts = 6;
  // -- the big tile in four parts where 64 of them would fill a quarter of the chip: K tiles a part must keep
  int64_t big_tile_parts = 4, big_tile_k_tiles_per_part = 40;
  // -- fp32 operands multiplied as bf16: 128x128 tiles in two K parts from this many tiles (up to half the units) and K tiles
  int64_t staged_halves_from_tiles = 96, staged_halves_min_k_tiles = 32;
  // -- one round of 256x256 or 192x192 tiles by a K split of two to four parts against 128x128 pairs (`bench.py --only
  //    rule_check`: 2304 x 2304 x 8192, 768 x 3072 x 12288, 2048 x 4096 x 11008)
  int64_t one_round_max_parts = 4, one_round_k_tiles_per_part = 40, one_round_ps_per_unit = 21600, one_round_split_ns = 3000;
  int64_t one_round_ns_per_kb_num = 28, one_round_ns_per_kb_den = 100, one_round_margin_num = 104, one_round_margin_den = 100;
  // -- peeling the last columns of tiles: only with this many K tiles (the peeled product splits them), an overhang of
  //    at most 1 / peel_overhang_den of a round, and at most 1 / peel_columns_den of the tile columns cut off
  //    (1536 x 11008 x 4096: 141 -> 125 us)
  int64_t peel_min_k_tiles = 32, peel_overhang_den = 8, peel_columns_den = 4;
  // -- few workgroups (at most half the units): split K, as long as what a part no longer walks (per K tile: one
  //    workgroup on a unit waits out every tile's loads; fp32 compute: sixteen 64-cycle instructions per block) outweighs
  //    a second kernel plus the partial sums' way to memory and back (384 x 384 x 1024, 640 x 640 x 2048, 512 x 512 x
  //    4096, 512^3 in fp32: `bench.py --only rule_check`)
  int64_t split_min_k_tiles = 8, split_k_tiles_per_part = 4, split_max = 64;
  int64_t k_tile_ns = 300, k_tile_ns_f32 = 1000, split_fixed_ns = 5000, split_ns_per_kb_num = 3, split_ns_per_kb_den = 4;
  // -- 128x128 tiles that leave a compute unit at most one workgroup run the four-stage kernel (tile_gemm_deep128.hip),
  //    from this many K tiles per workgroup on (rule_check, 1024 x 4096 x 4096)
  int64_t deep_max_workgroups = 256, deep_min_k_tiles = 8;
  // -- planning for that kernel (operands it serves): from deep_alone_from_tiles tiles of 128x128 on (three eighths of the
  //    units) the tiles stay whole or split in two, whichever the split rule's costs favour, with deep_k_tile_ns per K
  //    tile (a lone workgroup of this kernel walks a K tile in 0.3 us) and deep_fixed_ns per launch; between
  //    deep_fill_from_tiles and that, K is split so that the parts fill the units once, if a part keeps
  //    deep_fill_k_tiles_per_part K tiles.  Where more than half but at most deep_idle_tiles of the units would hold a
  //    tile and a part of the two-stage kernel's split keeps deep_idle_k_tiles_per_part K tiles, that split stays (two
  //    co-resident workgroups on every unit beat one on 56 % of them: bf16 768 x 3072 x 12288 63 against 71 us).
  //    `bench.py --only rule_check`: 512 / 768 / 1024 x 4096 x 4096, 1024 x 4096 x 11008, 512 x 2048 x 16384.
  int64_t deep_alone_from_tiles = 96, deep_fill_from_tiles = 32, deep_fill_k_tiles_per_part = 12;
  int64_t deep_idle_tiles = 160, deep_idle_k_tiles_per_part = 60, deep_k_tile_ns = 300, deep_fixed_ns = 8000;
  int64_t deep_halves_ns_per_kb_num = 3, deep_halves_ns_per_kb_den = 10;
  // -- a 128x128 plan of 16-bit compute with K up to this (one matrix instruction deep) runs the kernel that loads its
  //    fragments straight from memory and overlaps a tile's stores with the next tile's loads (tile_gemm_short_k.hip:
  //    batch 8 of 3000 x 3000 x 17 to fp32 54 us against 69, to bf16 42 against 53; 8192 x 8192 x 32 43 against 57; with
  //    a second step along K - its loads are not overlapped - the two-stage kernel is ahead, 65 against 71 us at K = 64)
  int64_t short_k_direct_max_k = 32;
};
constexpr RuleConstants kRules{};

// Every operand class but the unsigned bytes, with K contiguous on both sides, no C input, one side <= 16 rows, the
// other >= 512 (vecops' small-vector leaves serve every atom, matmul/details/kernel/amx/Backend.h:767-992)
bool skinny_applies(const Problem& pr) {
  if (pr.fused) return false;  // the skinny kernels have no output transform
  if (pr.src == SRC_I8_FLIP || pr.src == kSrcF64 || pr.has_cin || pr.packed_b) return false;
  const int64_t per = pr.src == SRC_I8 ? 16 : pr.src == SRC_F32 ? 4 : 8;  // elements a lane takes per step
  if (!k_vector_ok(pr.a) || !k_vector_ok(pr.b) || pr.k % per != 0 || pr.k < 8 * per) return false;
  const int64_t narrow = pr.m < pr.n ? pr.m : pr.n, wide = pr.m < pr.n ? pr.n : pr.m;
  // (the skinny kernels read one set of scales and one correction row for every batch)
  if (pr.batch > 1 && (pr.row_scales_bs != 0 || pr.correction_bs != 0)) return false;
  return narrow <= 16 && wide >= 512 && pr.batch <= 65535;
}

// elements of K in one 128-byte K tile of the compute type
int k_tile_elements(int src) { return src == SRC_I8 || src == SRC_I8_FLIP ? 128 : src == SRC_F32 ? 32 : 64; }

// Workgroup tile of a tile family (0 x 0 for the others).
void tile_of_family(uint32_t family, int* tile_m, int* tile_n) {
  switch (family) {
    case VECOPS_HIP_FAMILY_TILE_256: *tile_m = *tile_n = 256; break;
    case VECOPS_HIP_FAMILY_TILE_256X128: *tile_m = 256; *tile_n = 128; break;
    case VECOPS_HIP_FAMILY_TILE_128X256: *tile_m = 128; *tile_n = 256; break;
    case VECOPS_HIP_FAMILY_TILE_256X352: *tile_m = 256; *tile_n = 352; break;
    case VECOPS_HIP_FAMILY_TILE_192: *tile_m = *tile_n = 192; break;
    case VECOPS_HIP_FAMILY_TILE_128: *tile_m = *tile_n = 128; break;
    case VECOPS_HIP_FAMILY_TILE_64: *tile_m = *tile_n = 64; break;
    default: *tile_m = *tile_n = 0; break;
  }
}

// Split-K factor and workspace of a plan whose family is a tile family: K is split when the tiles leave most
// compute units idle (forced_split > 0: the caller's factor, clamped to the K tiles there are).
void finish_tile_plan(const Problem& pr, VecopsHipPlan* plan, uint32_t forced_split) {
  int tile_m = 0, tile_n = 0;
  tile_of_family(plan->family, &tile_m, &tile_n);
  const int64_t ktile = k_tile_elements(pr.src);
  const int64_t k_tiles = (pr.k + ktile - 1) / ktile;
  const int64_t wgs = ((pr.m + tile_m - 1) / tile_m) * ((pr.n + tile_n - 1) / tile_n) * pr.batch;
  int64_t split = 1;
  if (plan->family == VECOPS_HIP_FAMILY_TILE_256X352) forced_split = 1;  // its kernel walks the whole K
  if (forced_split > 0) {
    split = forced_split < k_tiles ? forced_split : k_tiles;
  } else if (wgs <= kComputeUnits / 2 && k_tiles >= kRules.split_min_k_tiles) {
    split = kComputeUnits / wgs;
    if (split > k_tiles / kRules.split_k_tiles_per_part) split = k_tiles / kRules.split_k_tiles_per_part;
    if (split > kRules.split_max) split = kRules.split_max;
    // A split buys K tiles a workgroup no longer walks (0.2-0.4 us each, 0.3 in the rule: one workgroup on a compute unit waits out
    // every tile's loads) and costs a second kernel plus the partial sums' way to memory and back: about 5 us and
    // 0.75 us per MB (384 x 384 x 1024: 7.3 us unsplit against 10.4 in four parts; 640 x 640 x 2048: 10.4 against
    // 12.7 in two; 512 x 512 x 4096: 24.2 against 13.2 in four).  Halve the factor until it pays.
    // (a K tile of fp32 compute is sixteen 64-cycle MFMAs per 32 x 32 block: about 1 us - 512^3 in fp32 21.2 us
    // unsplit, 13.9 in four parts)
    const int64_t per_split_kb = pr.batch * pr.m * pr.n * 4 / 1024;
    const int64_t tile_ns = pr.src == SRC_F32 ? kRules.k_tile_ns_f32 : kRules.k_tile_ns;
    while (split > 1) {
      const int64_t saved_ns = (k_tiles - (k_tiles + split - 1) / split) * tile_ns;
      const int64_t cost_ns = kRules.split_fixed_ns + split * per_split_kb * kRules.split_ns_per_kb_num / kRules.split_ns_per_kb_den;
      if (saved_ns > cost_ns) break;
      split /= 2;
    }
  }
  if (split < 1) split = 1;
  plan->split_k = static_cast<uint32_t>(split);
  plan->workspace_bytes = 0;
  if (split > 1) plan->workspace_bytes = static_cast<uint64_t>(split) * pr.batch * pr.m * pr.n * 4u;
  // an unsigned 8-bit operand needs the sums of the other operand's rows: after the partials
  if (pr.src == SRC_I8_FLIP) plan->workspace_bytes += static_cast<uint64_t>(pr.batch) * (pr.m + pr.n) * 4u;
}

int fetch_mode(const Problem& pr, const VecopsHipPlan& plan);
bool lines_up(const Problem& pr, const View& v, int64_t line_stride);

// The two halves of a problem cut between columns n_main - 1 and n_main of C: rows of B, columns of C and C_in.
void cut_columns(const Problem& pr, int64_t n_main, Problem* main, Problem* rest) {
  *main = pr;
  *rest = pr;
  main->n = main->b.rows = main->c.cols = n_main;
  rest->n = rest->b.rows = rest->c.cols = pr.n - n_main;
  rest->b.data = static_cast<char*>(pr.b.data) + n_main * pr.b.rs * dtype_bytes(pr.b.dtype);
  rest->c.data = static_cast<char*>(pr.c.data) + n_main * pr.c.cs * dtype_bytes(pr.c.dtype);
  if (pr.has_cin) {
    main->cin.cols = n_main;
    rest->cin.cols = pr.n - n_main;
    rest->cin.data = static_cast<char*>(pr.cin.data) + n_main * pr.cin.cs * dtype_bytes(pr.cin.dtype);
  }
}

// Whether the 256 x 352 tile (tile_gemm_wide_i8.hip) can run a problem: signed 8-bit, bf16 or f16 operands, both
// K-contiguous with 16-byte aligned bases and rows, K a whole number of K tiles of 128 bytes (two or more), any M, N a
// multiple of 4, one batch, a row-major C with 16-byte aligned rows; a C input with contiguous rows (not under the
// dequantisation), any fused transform and output type of the class.
bool wide_tile_serves(const Problem& pr) {
  const bool bytes = pr.src == SRC_I8;
  if ((!bytes && pr.src != SRC_BF16 && pr.src != SRC_F16) || pr.batch != 1) return false;
  // (a C input: contiguous rows, and not under the kernels' dequantisation stage - which a fused transform's two scale
  // vectors on int32 sums are too: the C input joins the sums before them)
  const bool dequant_stage = pr.dequant || (bytes && pr.fused != nullptr && pr.fused->row_scales != nullptr && pr.fused->column_scales != nullptr);
  if (pr.has_cin && (pr.cin.cs != 1 || dequant_stage)) return false;
  const int64_t elem = bytes ? 1 : 2, ktile = 128 / elem;
  if (pr.k % ktile != 0 || pr.k < 2 * ktile || pr.n % 4 != 0 || pr.m == 0 || pr.n == 0) return false;
  if (pr.a.cs != 1 || (pr.a.rs * elem) % 16 != 0 || !aligned16(pr.a.data) || !aligned16(pr.b.data)) return false;
  if (pr.packed_b) {  // (a prepacked B: its 32-row panels are the tile's parts; 32-bit offsets into it)
    if ((pr.n + 31) / 32 * (pr.k * elem / 32) * 1024 >= (int64_t{1} << 31)) return false;
  } else if (pr.b.cs != 1 || (pr.b.rs * elem) % 16 != 0 || 352 * pr.b.rs * elem >= (int64_t{1} << 31)) {
    return false;
  }
  if (pr.c.cs != 1 || pr.c.rs % 4 != 0 || !aligned16(pr.c.data)) return false;
  if (256 * pr.a.rs * elem >= (int64_t{1} << 31)) return false;
  // (every output type of the class: straight from the registers or through the epilogue's finishing step)
  return bytes || !pr.dequant;
}

// How the operands of a (non-empty) problem can be fetched: the plan's vector flags and B's layout.
void plan_fetch_flags(const Problem& pr, VecopsHipPlan* plan) {
  plan->vector_a = k_vector_ok(pr.a) ? 1 : 0;
  plan->vector_b = pr.packed_b || (k_vector_ok(pr.b) || (pr.b.rs == 1 && pr.b.cs != 1 && n_vector_ok(pr.b) && dtype_bytes(pr.b.dtype) != 1)) ? 1 : 0;
  plan->b_layout = pr.b.cs == 1 ? 0 : (pr.b.rs == 1 ? 1 : 2);
}

// Whether the 192 x 192 tile can run a problem: bf16, f16 or signed 8-bit operands with 16-byte aligned bases, rows
// and batches (its only instances are fed by loads that write LDS themselves) - both K-contiguous, or 16-bit ones
// with B handed over as [K,N] -, B not prepacked.
bool tile_192_serves(const Problem& pr, const VecopsHipPlan& plan) {
  if (pr.src != SRC_BF16 && pr.src != SRC_F16 && pr.src != SRC_I8) return false;
  if (pr.packed_b) return false;
  const int mode = fetch_mode(pr, plan);
  return mode == MODE_KVEC_DMA || (mode == MODE_NVEC_B_DMA && pr.src != SRC_I8);
}

// The GPU rule table.  Like vecops' runtime_*_profitable predicates it is a pure
// integer function of (operand class, m, n, k); it picks the workgroup tile by
// how many tiles the problem yields against the 256 compute units and splits K
// when even the smallest tile leaves most of them idle.  A part-filled last round
// of big tiles is not worth avoiding: the chip runs against its power limit on real
// data, a lightly loaded round clocks higher, and narrower tiles (256x192 was
// measured) cost more LDS and L2 traffic per flop than the better balance saves.
// (scratch_limit: partial sums the caller can hold - the mid-band K split below is skipped where it needs more)
// (peel_allowed: false for the product of a peel itself)
void choose(const Problem& pr, VecopsHipPlan* plan, uint64_t scratch_limit = UINT64_MAX, bool peel_allowed = true) {
  memset(plan, 0, sizeof(*plan));
  plan->split_k = 1;
  if (pr.batch == 0 || pr.m == 0 || pr.n == 0) {
    plan->family = VECOPS_HIP_FAMILY_NONE;
    return;
  }
  if (pr.k == 0) {
    plan->family = VECOPS_HIP_FAMILY_ZERO_K;
    return;
  }
  plan_fetch_flags(pr, plan);

  if (pr.src == kSrcF64) {  // one kernel: 128 x 128 tiles, K never split
    plan->family = VECOPS_HIP_FAMILY_TILE_128;
    return;
  }
  // Skinny family: one operand has at most 16 rows and the other is long - the GPU reading of
  // vecops' small-vector shapes (runtime_dispatch_rules::skinny_at_most / large_m1 / large_n1,
  // matmul/details/kernel/RuntimeDispatch.h:24-83): HBM-bound, the wide operand is read once.
  // (the dequantising epilogue multiplies by A's row scale first: the skinny kernel applies the narrow side's
  // scale first, so it serves a dequantised product only when A is the narrow side)
  if (skinny_applies(pr) && !(pr.dequant && pr.m >= pr.n)) {
    plan->family = VECOPS_HIP_FAMILY_SKINNY;
    return;
  }

  auto tiles2 = [&](int64_t tm, int64_t tn) { return ((pr.m + tm - 1) / tm) * ((pr.n + tn - 1) / tn) * pr.batch; };
  auto tiles = [&](int64_t t) { return tiles2(t, t); };
  // Candidate workgroup tiles with the work each does per compute unit and second relative to 256x256
  // (per mille; measured on bf16 problems that fill exactly one round).  A candidate must keep at least
  // half the compute units busy; among those the cheapest wins, cost = rounds x tile area / quality -
  // so a part-filled last round, rows or columns of padding and a less efficient small tile are all
  // priced in one number (4096^3: 256 tiles of 256x256, one round; 2048x11008: 344 of them in two rounds, which
  // 1376 tiles of 128x128 in three undercut - int8 measured 117-123 us against 92-97, 115-123 for the 688
  // rectangles; 4096x4224: 1056 tiles of 128x128, 151 us against 176 for 272 big ones whose second round is 6 % full;
  // 8 x 777x1000: 224 tiles of 128x256 in one round; 3072x4096x4096, 5120^3, 2048x14336x4096, 8192^3: big tiles,
  // 7-15 % ahead for bf16 and 3-6 % for int8).
  struct Candidate { uint32_t family; int64_t tm, tn, quality; };
  const bool bytes = pr.src == SRC_I8 || pr.src == SRC_I8_FLIP;
  const int mode = fetch_mode(pr, *plan);
  const bool direct = mode == MODE_KVEC_DMA || mode == MODE_NVEC_B_DMA;  // loads that write LDS themselves
  const Candidate candidates[] = {{VECOPS_HIP_FAMILY_TILE_256, 256, 256, 1000},
                                  {VECOPS_HIP_FAMILY_TILE_256X128, 256, 128, direct ? kQuality256x128Direct : kQuality256x128},
                                  {VECOPS_HIP_FAMILY_TILE_128X256, 128, 256, direct ? kQuality256x128Direct : kQuality256x128},
                                  // (256 tiles of 192 x 192 cover 3072 x 3072: one round where 144 big tiles leave 112
                                  //  units idle - bf16 3000^3 71 us against 81, 768 x 11008 x 4096 64 against 80)
                                  {VECOPS_HIP_FAMILY_TILE_192, 192, 192, kQuality192},
                                  {VECOPS_HIP_FAMILY_TILE_128, 128, 128,
                                   !direct ? kQuality128Staged : bytes ? kQuality128Int8Direct : kQuality128Direct}};
  uint32_t family = VECOPS_HIP_FAMILY_TILE_64;
  int64_t tile_m = 64, tile_n = 64, best_cost = INT64_MAX;
  const bool serves_192 = tile_192_serves(pr, *plan);
  for (const Candidate& c : candidates) {
    // (the 192 x 192 tile: for counts that fit one round - over several rounds the big tiles' loops are ahead)
    if (c.family == VECOPS_HIP_FAMILY_TILE_192 && (!serves_192 || tiles2(c.tm, c.tn) > kComputeUnits)) continue;
    if (pr.m <= c.tm / 2 || pr.n <= c.tn / 2) continue;  // a tile more than half empty in one direction
    const int64_t count = tiles2(c.tm, c.tn);
    if (count * kRules.min_busy_den < kComputeUnits * kRules.min_busy_num) continue;
    // two 128x128 workgroups live on a compute unit at a time (64 KiB of LDS and at most 256 registers each): a
    // round of them is 512 tiles
    const int64_t per_unit = c.family == VECOPS_HIP_FAMILY_TILE_128 && direct ? kRules.small_tile_workgroups_per_unit : 1;
    const int64_t slots = per_unit * kComputeUnits;
    const int64_t rounds = (count + slots - 1) / slots;
    int64_t cost = rounds * per_unit * c.tm * c.tn * 1000 / c.quality;
    // a single part-filled round runs faster than a full one (the chip is power-limited: fewer busy compute units
    // clock higher): half full costs three quarters (3000^3 as 144 big tiles 87 us against 105 for 576 small ones;
    // 8 x 777 x 1000 x 3001 as 224 tiles of 128x256 65 us, as 256 of 256x128 73, as 128 of 256x256 86)
    if (rounds == 1) cost = cost * (slots + count) / (2 * slots);
    // a rectangle has to be 10 % cheaper than the big tile: the round count flatters it (more L2 traffic per flop,
    // and its quality falls with the problem size).  The 128x128 tile competes on its cost alone (1536 x 4096 x 4096:
    // 49 us against 60 for the rectangles, 2048 x 4096 x 4096 58 against 67; int8 31 against 38 and 36 against 42).
    const bool smaller = best_cost != INT64_MAX && c.tm * c.tn < tile_m * tile_n &&
                         !(c.family == VECOPS_HIP_FAMILY_TILE_128 && direct);
    if (best_cost == INT64_MAX ||
        (smaller ? cost * kRules.rectangle_margin_num < best_cost * kRules.rectangle_margin_den : cost < best_cost)) {
      best_cost = cost;
      family = c.family;
      tile_m = c.tm;
      tile_n = c.tn;
    }
  }
  // The 256 x 352 tile of 8-bit operands: priced like the big tile (its loop is the same, with a tenth less operand
  // traffic per multiply-add), it wins where its count fits rounds that the square tiles' counts do not - 2048 x 11008:
  // 256 tiles in one round against 344 of 256 x 256 (two rounds) and 1376 of 128 x 128 (three).
  if (wide_tile_serves(pr) && pr.n > 176 && pr.m > 128) {   // (a tile at most half empty in either direction)
    const int64_t count = tiles2(256, 352), rounds = (count + kComputeUnits - 1) / kComputeUnits;
    if (count * kRules.min_busy_den >= kComputeUnits * kRules.min_busy_num) {
      int64_t cost = rounds * 256 * 352;
      if (rounds == 1) cost = cost * (kComputeUnits + count) / (2 * kComputeUnits);
      if (cost < best_cost) {
        best_cost = cost;
        family = VECOPS_HIP_FAMILY_TILE_256X352;
        tile_m = 256;
        tile_n = 352;
      }
    }
  }
  if (pr.src == SRC_F32 && family == VECOPS_HIP_FAMILY_TILE_128 && tiles(128) <= kRules.f32_small_tiles_up_to_tiles128 &&
      (tiles(64) + kComputeUnits - 1) / kComputeUnits <= 3) {
    family = VECOPS_HIP_FAMILY_TILE_64;
    tile_m = tile_n = 64;
  }
  if (family == VECOPS_HIP_FAMILY_TILE_64 && pr.m > 64 && pr.n > 64 && tiles(64) > kRules.many_small_tiles_rounds * kComputeUnits) {
    family = VECOPS_HIP_FAMILY_TILE_128;
    tile_m = tile_n = 128;
  }
  const int64_t ktile = k_tile_elements(pr.src);
  const int64_t k_tiles = (pr.k + ktile - 1) / ktile;
  // operands the four-stage 128x128 kernel (tile_gemm_deep128.hip) serves: fetched by loads that write LDS (both
  // K-contiguous, or 16-bit operands with B as [K,N]), K in whole K tiles
  const bool deep_tr = mode == MODE_NVEC_B_DMA && (pr.src == SRC_BF16 || pr.src == SRC_F16) && pr.n % 8 == 0 &&
                       pr.k * pr.b.cs * 2 + 256 < (int64_t{1} << 31);   // B as [K,N]: 16-bit operands, 32-bit K offsets
  // (a prepacked B keeps its pack order in LDS there: A's alignment decides)
  const bool deep_pk = pr.packed_b && (pr.src == SRC_BF16 || pr.src == SRC_F16 || pr.src == SRC_I8) && plan->vector_a != 0 &&
                       lines_up(pr, pr.a, pr.a.rs);
  const bool deep_ok = (pr.packed_b ? deep_pk
                                    : (mode == MODE_KVEC_DMA && (pr.src == SRC_BF16 || pr.src == SRC_F16 || pr.src == SRC_I8)) || deep_tr) &&
                       pr.k % ktile == 0 && k_tiles >= kRules.deep_min_k_tiles;
  // At most four K tiles of 16-bit or 8-bit operands: the tile's life is its start-up and its stores, and
  // two or three 128x128 workgroups on a compute unit overlap one's stores with another's loads, which a
  // single big tile cannot (batch 8 of 3000x3000x17 to fp32: 93 us against 111; 8 x 1000x1000x100: 17.7
  // against 21.7; 4096x4096x256 to bf16: 17.9 against 20.2; level at 8192x8192x256, behind from K = 512).
  // (int8, whose big tile gains least from its size: up to eight, 4096 x 4096 x 1024 29.6 us against 32.9)
  const int64_t short_k = bytes ? kRules.short_k_tiles_8bit : kRules.short_k_tiles_16bit;
  if (k_tiles <= short_k && pr.src != SRC_F32 && family != VECOPS_HIP_FAMILY_TILE_64 && family != VECOPS_HIP_FAMILY_TILE_128 &&
      pr.m > 64 && pr.n > 64 && tiles(128) * kRules.min_busy_den >= kComputeUnits * kRules.min_busy_num) {
    family = VECOPS_HIP_FAMILY_TILE_128;
    tile_m = tile_n = 128;
  }
  // Fewer 128x128 tiles than compute units (and more than four K tiles): a unit holds one workgroup and has
  // nothing to overlap its start-up, barriers and stores with, while four times as many 64x64 tiles put two or
  // more on every unit (512 x 4096 x 4096: 28.7 us against 45.9; 1536^3: 18.0 against 20.7; 768 x 4096 x 4096:
  // 42.7 against 46.7; from 256 tiles on - 1024 x 4096 x 4096, 2048^3 - the bigger tile is ahead again).
  // (not where the four-stage 128x128 kernel serves: a lone workgroup of it does not wait out its loads)
  // (fp32 operands multiplied as bf16 - twice the bytes through the staging registers, which the small tile fetches twice
  // as often: only up to half the units - 1536^3, 144 tiles: 23 us on 128x128 against 29; 1408^3, 121 tiles: 20 on 64x64
  // against 23)
  else if (k_tiles > kRules.short_k_tiles_16bit && family == VECOPS_HIP_FAMILY_TILE_128 && pr.src != SRC_F32 && !deep_ok &&
           tiles(128) <= (pr.src == SRC_F32_AS_BF16 ? kComputeUnits / 2 : kRules.lonely_tiles_num * kComputeUnits / kRules.lonely_tiles_den)) {
    family = VECOPS_HIP_FAMILY_TILE_64;
    tile_m = tile_n = 64;
  }
  // 128 to 200 tiles of 128x128 and a long K: half to three quarters of the compute units hold one workgroup each,
  // and 64x64 tiles fill them with work that is a third less efficient.  K split two to four ways puts two
  // 128x128 workgroups on (nearly) every unit; it pays from twenty K tiles per part (bf16: 768 x 3072 x 12288 108 us
  // -> 64, 768 x 4096 x 8192 78 -> 60, 1024 x 2048 x 8192 52 -> 43, 640 x 4096 x 4096 41 -> 34, 768 x 4096 x 4096
  // 41 -> 39; int8: 768 x 3072 x 12288 58 -> 42; with sixteen per part - 512 x 4096 x 4096, int8 1024 x 2048 x 8192 -
  // the unsplit small tiles stay ahead, 28.0 against 30.8 and 28.8 against 33.0).  Measured with loads that write
  // LDS themselves, so only there (a prepacked B: only the four-stage kernel's branches below).
  // The same from 32 tiles of 128x128 on, five to sixteen ways (bf16 512 x 2048 x 16384 73 us -> 43, 384 x 3072 x 8192
  // 46 -> 33, 512 x 3072 x 8192 48 -> 40; the 64x64 tiles the table took there are 128 workgroups or more, which the
  // rule for few workgroups leaves whole): fewer parts, down to six, where that reaches the twenty K tiles (int8
  // 512 x 2048 x 16384 40 -> 31 in six parts; bf16 128 x 8192 x 8192 44 -> 36).  (Not for a
  // prepacked B: its kernels were not measured this way.)
  // And up to 256 tiles (one workgroup on every unit) in two parts, from forty K tiles per part (bf16 1024 x 4096 x
  // 11008 116 us -> 90, 896 x 4096 x 11008 114 -> 81, 1024 x 4096 x 6144 66 -> 58; int8 896 x 4096 x 11008 61 -> 52;
  // with thirty-two per part - bf16 1024 x 4096 x 4096, int8 ... x 8192 - the unsplit tiles are level or ahead).
  uint32_t band_split = 0;
  bool deep_planned = false;
  if (((direct && !pr.packed_b) || (deep_pk && deep_ok)) && (family == VECOPS_HIP_FAMILY_TILE_64 || family == VECOPS_HIP_FAMILY_TILE_128) &&
      tiles(128) >= kComputeUnits / 8 && tiles(128) <= kComputeUnits) {
    const int64_t count = tiles(128);
    int64_t parts = kRules.small_tile_workgroups_per_unit * kComputeUnits / count;
    while (parts > kRules.band_min_parts && k_tiles / parts < kRules.band_k_tiles_per_part) --parts;
    const int64_t least = count > kRules.band_full_from_tiles ? kRules.band_k_tiles_per_part_full
                                                              : kRules.band_k_tiles_per_part;  // K tiles per part
    const bool fits = static_cast<uint64_t>(parts) * pr.batch * pr.m * pr.n * 4u <= scratch_limit;
    // Where the four-stage kernel serves, a workgroup alone on its unit is no longer the slow case (1024 x 4096 x 4096
    // unsplit 31-34 us against 43 on the two-stage kernel, 768 x 4096 x 4096 27 against 38 in two parts, 512 x 4096 x
    // 4096 25 against 28 on 64x64 tiles, 1024 x 4096 x 11008 79 against 84 on the big tile in four parts; int8
    // 1024 x 4096 x 4096 21 against 28): at most one workgroup per unit, K split only to fill the units.
    const bool idle_units_long_k = count > kComputeUnits / 2 && count <= kRules.deep_idle_tiles &&
                                   k_tiles / parts >= kRules.deep_idle_k_tiles_per_part && fits;
    if (deep_ok && count >= kRules.deep_alone_from_tiles && !idle_units_long_k) {
      // whole, or in two parts where the units allow and the split rule's costs favour it
      int64_t best_parts = 1;
      if (2 * count <= kRules.deep_max_workgroups && k_tiles / 2 >= kRules.deep_min_k_tiles &&
          2ull * pr.batch * pr.m * pr.n * 4u <= scratch_limit) {
        const int64_t kb = pr.batch * pr.m * pr.n * 4 / 1024;
        const int64_t whole_ns = k_tiles * kRules.deep_k_tile_ns + kRules.deep_fixed_ns;
        // (the partial sums of two full-chip parts move at 0.3 ns a KiB - int8 512 x 4096 x 11008 33 us in halves against
        //  37.5 whole, bf16 512 x 4096 x 4096 25.0 whole against 26.2 - where the few-workgroup rule's small launches pay 0.75)
        const int64_t halves_ns = (k_tiles + 1) / 2 * kRules.deep_k_tile_ns + kRules.deep_fixed_ns + kRules.split_fixed_ns +
                                  2 * kb * kRules.deep_halves_ns_per_kb_num / kRules.deep_halves_ns_per_kb_den;
        if (halves_ns < whole_ns) best_parts = 2;
      }
      family = VECOPS_HIP_FAMILY_TILE_128;
      band_split = static_cast<uint32_t>(best_parts);
      deep_planned = true;
    } else if (deep_ok && count >= kRules.deep_fill_from_tiles && count < kRules.deep_alone_from_tiles &&
               k_tiles / (kRules.deep_max_workgroups / count) >= kRules.deep_fill_k_tiles_per_part &&
               static_cast<uint64_t>(kRules.deep_max_workgroups / count) * pr.batch * pr.m * pr.n * 4u <= scratch_limit) {
      // few tiles and a long K: as many parts as fill the units once (512 x 2048 x 16384: 37 us in four parts against 46
      // in eight parts of the two-stage kernel)
      family = VECOPS_HIP_FAMILY_TILE_128;
      band_split = static_cast<uint32_t>(kRules.deep_max_workgroups / count);
      deep_planned = true;
    } else if (!pr.packed_b && k_tiles / parts >= least && fits) {
      family = VECOPS_HIP_FAMILY_TILE_128;
      band_split = static_cast<uint32_t>(parts);
    }
  }
  // fp32 operands multiplied as bf16 (register-staged: none of the rules above), 96 to 128 tiles of 128x128 and 64 K
  // tiles or more: two K parts of the 128x128 tile fill the units (1024 x 2048 x 4096 37 us against 47 on 64x64 tiles,
  // 1280 x 1280 x 4096 37 against 49; at K = 2048 - 768 x 2048 x 2048 - 24.6 against 25.7; at K = 1024 the small tiles
  // stay ahead, 15.7 against 22.6).
  if (pr.src == SRC_F32_AS_BF16 && !pr.packed_b && band_split == 0 && tiles(128) >= kRules.staged_halves_from_tiles &&
      tiles(128) <= kComputeUnits / 2 && k_tiles >= kRules.staged_halves_min_k_tiles &&
      2ull * pr.batch * pr.m * pr.n * 4u <= scratch_limit) {
    family = VECOPS_HIP_FAMILY_TILE_128;
    tile_m = tile_n = 128;
    band_split = 2;
  }
  // 256 tiles of 128x128 that are 64 of 256x256, and a K of 160 tiles or more: the big tile in four parts puts one
  // workgroup of its (faster) loop on every unit (bf16 1024 x 4096 x 11008: 84 us against 89-92 for the two parts of
  // 128x128 tiles above and 116 unsplit; with a shorter K - 1024 x 4096 x 4096, 16 K tiles per part - it loses, 48 against 44).
  if (direct && !pr.packed_b && !deep_planned && band_split == 2 && tiles(256) * kRules.big_tile_parts == kComputeUnits &&
      k_tiles / kRules.big_tile_parts >= kRules.big_tile_k_tiles_per_part &&
      static_cast<uint64_t>(kRules.big_tile_parts) * pr.batch * pr.m * pr.n * 4u <= scratch_limit) {
    family = VECOPS_HIP_FAMILY_TILE_256;
    band_split = static_cast<uint32_t>(kRules.big_tile_parts);
  }
  // One round of bigger tiles by a K split, against 128x128 pairs that fill their round badly or are split already
  // (16-bit operands, a long K).  Both sides are priced in ns: a workgroup's area / quality per K tile at one_round_ps_per
  // _unit (a 256x256 workgroup walks a K tile in 1.4 us), the single part-filled round's discount as above, and for a
  // split one_round_split_ns plus one_round_ns_per_kb for every KiB of partial sums (2304 x 2304 x 8192: 81 tiles of
  // 256x256 in three parts 80 us against 88-93 for 324 unsplit pairs; 768 x 3072 x 12288: 64 tiles of 192x192 in four
  // parts 60 against 63-67 for 144 tiles in three).  The parts must fill nine tenths of the units and keep
  // one_round_k_tiles_per_part K tiles, and the estimate has to be 4 % ahead (2048 x 4096 x 11008, where 128 big tiles in
  // two parts measure 4 % ahead of 512 pairs, stays as it is: the estimate sees 2 %, and sees the same for 1024 x 8192 x 11008,
  // where the big tiles in two parts are 7 % behind).
  if (direct && !pr.packed_b && !deep_planned && pr.batch == 1 && (pr.src == SRC_BF16 || pr.src == SRC_F16) &&
      family == VECOPS_HIP_FAMILY_TILE_128) {
    const int64_t c_kb = pr.m * pr.n * 4 / 1024;
    auto split_ns = [&](int64_t parts) { return parts > 1 ? kRules.one_round_split_ns + parts * c_kb * kRules.one_round_ns_per_kb_num / kRules.one_round_ns_per_kb_den : 0; };
    auto walk_ns = [&](int64_t units) { return units * k_tiles * kRules.one_round_ps_per_unit / 1000000; };
    const int64_t own_parts = band_split > 0 ? band_split : 1;
    const int64_t own_slots = kRules.small_tile_workgroups_per_unit * kComputeUnits, own_wgs = tiles(128) * own_parts;
    const int64_t own_rounds = (own_wgs + own_slots - 1) / own_slots;
    int64_t own_units = own_rounds * kRules.small_tile_workgroups_per_unit * 128 * 128 * 1000 / kQuality128Direct / own_parts;
    if (own_rounds == 1) own_units = own_units * (own_slots + own_wgs) / (2 * own_slots);
    int64_t best_ns = (walk_ns(own_units) + split_ns(own_parts)) * kRules.one_round_margin_den / kRules.one_round_margin_num;
    const struct { uint32_t family; int64_t tile, quality; bool serves; } bigger[] = {
        {VECOPS_HIP_FAMILY_TILE_256, 256, 1000, true}, {VECOPS_HIP_FAMILY_TILE_192, 192, kQuality192, serves_192}};
    for (const auto& c : bigger) {
      if (!c.serves) continue;
      const int64_t count = tiles(c.tile), parts = count > 0 ? kComputeUnits / count : 0;
      if (parts < 2 || parts > kRules.one_round_max_parts || count * parts * 10 < kComputeUnits * 9 ||
          k_tiles / parts < kRules.one_round_k_tiles_per_part || static_cast<uint64_t>(parts) * pr.m * pr.n * 4u > scratch_limit)
        continue;
      const int64_t units = c.tile * c.tile * 1000 / c.quality / parts * (kComputeUnits + count * parts) / (2 * kComputeUnits);
      const int64_t ns = walk_ns(units) + split_ns(parts);
      if (ns < best_ns) {
        best_ns = ns;
        family = c.family;
        tile_m = tile_n = c.tile;
        band_split = static_cast<uint32_t>(parts);
      }
    }
  }
  plan->family = family;
  finish_tile_plan(pr, plan, band_split);
  // Two or more rounds of workgroups and a last one that is nearly empty (1536 x 11008: 1032 tiles of 128x128 are two
  // rounds of 512 and eight tiles, which cost a third round: 141 us where two would take 95): the last columns of
  // tiles are cut off, so that the rest fills whole rounds, and run as a product of their own - few tiles and the
  // whole K, which the rules above split.  peeled_columns = the columns of C that second product computes.
  if (direct && !pr.packed_b && !pr.dequant && pr.fused == nullptr && pr.src != SRC_I8_FLIP && pr.batch == 1 && plan->split_k == 1 &&
      (family == VECOPS_HIP_FAMILY_TILE_128 || family == VECOPS_HIP_FAMILY_TILE_256) && k_tiles >= kRules.peel_min_k_tiles &&
      peel_allowed) {
    const int64_t slots = family == VECOPS_HIP_FAMILY_TILE_128 ? kRules.small_tile_workgroups_per_unit * kComputeUnits : kComputeUnits;
    const int64_t tiles_m = (pr.m + tile_m - 1) / tile_m, tiles_n = (pr.n + tile_n - 1) / tile_n;
    const int64_t count = tiles_m * tiles_n, over = count % slots;
    if (count > slots && over > 0 && over * kRules.peel_overhang_den <= slots) {
      const int64_t cut = (over + tiles_m - 1) / tiles_m;  // columns of tiles
      if (cut * kRules.peel_columns_den <= tiles_n) {
        const int64_t n_main = (tiles_n - cut) * tile_n;
        Problem main, rest;
        cut_columns(pr, n_main, &main, &rest);
        VecopsHipPlan rest_plan;
        choose(rest, &rest_plan, scratch_limit, false);
        if (rest_plan.workspace_bytes <= scratch_limit) {
          plan->peeled_columns = static_cast<uint32_t>(pr.n - n_main);
          plan->workspace_bytes = rest_plan.workspace_bytes;
        }
      }
    }
  }
}

const char* family_name(uint32_t family) {
  static const char* const names[] = {"none", "tile_256", "tile_128", "tile_64", "skinny", "zero_k", "tile_256x128", "tile_128x256",
                                      "tile_256x352", "tile_192"};
  return family < 10 ? names[family] : "unknown";
}

// The first tier of vecops' owner selection (matmul/details/kernel/amx/Backend.h:2724-2757; matmul/Family.h:216-239):
// a caller may prefer or require a kernel family.  A family that cannot serve the call is skipped when preferred
// and is an error when required (family_selection::Require turns an inapplicable family into a hard error,
// tests/ops/MatmulTest.cpp:514-536).  The tile families serve every non-empty product; the skinny family only its
// own shapes; none / zero_k only the degenerate problems they name.
int32_t apply_request(const Problem& pr, const VecopsHipFamilyRequest* request, VecopsHipPlan* plan) {
  if (request == nullptr || request->selection == VECOPS_HIP_SELECT_AUTOMATIC) return ST_OK;
  if (request->struct_size < sizeof(VecopsHipFamilyRequest)) return fail(ST_INVALID, "matmul: family request record too short");
  if (request->selection != VECOPS_HIP_SELECT_PREFER && request->selection != VECOPS_HIP_SELECT_REQUIRE)
    return fail(ST_INVALID, "matmul: unknown family selection %u", request->selection);
  if (request->family > VECOPS_HIP_FAMILY_TILE_192) return fail(ST_INVALID, "matmul: unknown family %u", request->family);
  const bool degenerate = plan->family == VECOPS_HIP_FAMILY_NONE || plan->family == VECOPS_HIP_FAMILY_ZERO_K;
  int tile_m = 0, tile_n = 0;
  tile_of_family(request->family, &tile_m, &tile_n);
  bool serves;
  if (pr.src == kSrcF64 && !degenerate) {
    serves = request->family == VECOPS_HIP_FAMILY_TILE_128;  // the fp64 kernel's only tile
    if (serves) return ST_OK;
  } else if (degenerate || tile_m == 0) {
    // nothing to multiply: only the family that names the case; the skinny family: its own shapes
    serves = request->family == plan->family ||
             (request->family == VECOPS_HIP_FAMILY_SKINNY && !degenerate && skinny_applies(pr) && !(pr.dequant && pr.m >= pr.n));
  } else {
    // every tile family serves every product, but the 256 x 352 tile its own class of them, K unsplit,
    // and the 192 x 192 tile operands whose loads write LDS themselves
    serves = request->family == VECOPS_HIP_FAMILY_TILE_256X352 ? wide_tile_serves(pr) && request->split_k <= 1
             : request->family == VECOPS_HIP_FAMILY_TILE_192   ? tile_192_serves(pr, *plan)
                                                               : true;
  }
  if (!serves) {
    if (request->selection == VECOPS_HIP_SELECT_PREFER) return ST_OK;  // the rule table's choice stands
    return fail(ST_NOT_APPLICABLE, "matmul: the required family %s cannot serve this call (the rule table chooses %s)",
                family_name(request->family), family_name(plan->family));
  }
  if (request->family == plan->family && request->split_k == 0) {
    if (plan->peeled_columns > 0) {  // a requested family runs the whole product (a peel's second product is the table's choice)
      plan->peeled_columns = 0;
      finish_tile_plan(pr, plan, 1);
    }
    return ST_OK;
  }
  plan->family = request->family;
  plan->peeled_columns = 0;  // (the rule table's peel belongs to its own choice of family)
  if (tile_m != 0) {
    finish_tile_plan(pr, plan, request->split_k);
  } else {
    plan->split_k = 1;
    plan->workspace_bytes = 0;
  }
  return ST_OK;
}

// A launch needs a current device.  (The rule table and the streaming kernels' grids are calibrated for the 256
// compute units of an MI355X - kComputeUnits; a device with another count - a partitioned one, another gfx950 part -
// runs the same kernels, correct and tuned for the other machine.)
int32_t check_device() {
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return fail(ST_EXEC, "hipGetDevice: %s", hipGetErrorString(e));
  return ST_OK;
}

bool lines_up(const Problem& pr, const View& v, int64_t line_stride) {
  const int64_t elem_bytes = (pr.src == SRC_BF16 || pr.src == SRC_F16) ? 2 : 1;
  return aligned16(v.data) && (line_stride * elem_bytes) % 16 == 0 && (v.bs * elem_bytes) % 16 == 0;
}

// The kernels' parameter record of a problem, before any tiling is chosen.
TileGemmParams base_params(const Problem& pr, const float* row_scales, const float* column_scales, const int32_t* correction,
                           void* workspace) {
  TileGemmParams p;
  memset(&p, 0, sizeof(p));
  p.a = pr.a.data;
  p.b = pr.b.data;
  p.c = pr.c.data;
  p.cin = pr.has_cin ? pr.cin.data : nullptr;
  p.partial = workspace;
  p.row_scales = row_scales;
  p.column_scales = column_scales;
  p.correction = correction;
  p.row_scales_bs = pr.batch > 1 ? pr.row_scales_bs : 0;
  p.correction_bs = pr.batch > 1 ? pr.correction_bs : 0;
  p.m = static_cast<int32_t>(pr.m);
  p.n = static_cast<int32_t>(pr.n);
  p.k = static_cast<int32_t>(pr.k);
  p.batch = static_cast<int32_t>(pr.batch);
  p.out_kind = pr.out_kind;
  p.cin_kind = pr.cin_kind;
  p.a_rs = pr.a.rs; p.a_ks = pr.a.cs; p.a_bs = pr.a.bs;
  p.b_rs = pr.b.rs; p.b_ks = pr.b.cs; p.b_bs = pr.b.bs;
  p.c_rs = pr.c.rs; p.c_cs = pr.c.cs; p.c_bs = pr.c.bs;
  if (pr.has_cin) { p.cin_rs = pr.cin.rs; p.cin_cs = pr.cin.cs; p.cin_bs = pr.cin.bs; }
  const bool is_int = pr.src == SRC_I8 || pr.src == SRC_I8_FLIP;
  if (pr.fused) {
    const VecopsHipEpilogue& ep = *pr.fused;
    p.fused = 1;
    p.ep_act = static_cast<int32_t>(ep.activation);
    p.ep_flags = ep.flags & (VECOPS_HIP_EPILOGUE_SCALE | VECOPS_HIP_EPILOGUE_SHIFT);
    p.ep_scale = ep.scale;
    p.ep_shift = ep.shift;
    p.ep_lo = ep.clamp_lo;
    p.ep_hi = ep.clamp_hi;
    if (is_int && ep.row_scales && ep.column_scales && pr.batch == 1) {
      // both scales on int32 sums: the dequantisation stage of the kernels, the same two multiplies
      p.row_scales = ep.row_scales;
      p.column_scales = ep.column_scales;
    } else {
      p.ep_row_scales = ep.row_scales;
      p.ep_column_scales = ep.column_scales;
    }
  }

  return p;
}

// How a problem's operands can be fetched (LoadMode), from the plan's vector flags and the operands' alignment.
int fetch_mode(const Problem& pr, const VecopsHipPlan& plan) {
  int mode = MODE_GENERIC;
  if (plan.vector_a && k_vector_ok(pr.b)) mode = MODE_KVEC;
  else if (plan.vector_a && plan.vector_b && plan.b_layout == 1) mode = MODE_NVEC_B;
  // 16-byte aligned bases, rows and batches: the loads may write LDS themselves
  if ((pr.src == SRC_BF16 || pr.src == SRC_F16 || pr.src == SRC_I8) && lines_up(pr, pr.a, pr.a.rs)) {
    if (mode == MODE_KVEC && lines_up(pr, pr.b, pr.b.rs)) mode = MODE_KVEC_DMA;
    else if (mode == MODE_NVEC_B && lines_up(pr, pr.b, pr.b.cs)) mode = MODE_NVEC_B_DMA;
  }
  return mode;
}

// Unsigned 8-bit sides (SRC_I8_FLIP): the kernels multiply the signed images x - 128 (bytes xor 0x80) and the epilogue
// restores the sum with 128 * (row sums of the other operand's image) per row / column (+ 16384 K when both sides are
// unsigned).  Launches the row-sum kernels into `terms` (batch * (m + n) int32) and fills the flips and term pointers
// of `p`.
int32_t unsigned_side_terms(const Problem& pr, TileGemmParams* params, int32_t* terms, hipStream_t stream) {
  TileGemmParams& p = *params;
  hipError_t e;
  int32_t* row_term = terms;
  int32_t* col_term = row_term + pr.batch * pr.m;
  p.a_flip = pr.a_unsigned ? 0x80808080u : 0u;
  p.b_flip = pr.b_unsigned ? 0x80808080u : 0u;
  if (pr.b_unsigned) {  // + 128 * sum_k a'[m,k] per row
    e = launch_byte_row_sums(pr.a.data, p.batch, p.m, p.k, pr.a.bs, pr.a.rs, pr.a.cs, p.a_flip, 128u, nullptr, 0, row_term, stream);
    if (e != hipSuccess) return fail(ST_EXEC, "row-sum kernel launch: %s", hipGetErrorString(e));
    p.row_term = row_term;
  }
  if (pr.a_unsigned && pr.packed_b) {  // the same term from the packed rows, one copy per batch
    e = launch_packed_row_sums(pr.b.data, p.n, p.k, p.batch, 128u, nullptr, col_term, stream);
    if (e != hipSuccess) return fail(ST_EXEC, "row-sum kernel launch: %s", hipGetErrorString(e));
    p.col_term = col_term;
  } else if (pr.a_unsigned) {  // + 128 * sum_k b'[n,k] per column
    e = launch_byte_row_sums(pr.b.data, p.batch, p.n, p.k, pr.b.bs, pr.b.rs, pr.b.cs, p.b_flip, 128u, nullptr, 0, col_term, stream);
    if (e != hipSuccess) return fail(ST_EXEC, "row-sum kernel launch: %s", hipGetErrorString(e));
    p.col_term = col_term;
  }
  if (pr.a_unsigned && pr.b_unsigned) p.const_term = 16384u * static_cast<uint32_t>(pr.k);
  // u8 x s8 (AMX_I8I32<uint8_t, int8_t>), one batch, no correction row of the caller's: the column term is
  // a correction row, which every fast epilogue adds (the general path took 450 us at 2048 x 4096 x 11008)
  if (pr.a_unsigned && !pr.b_unsigned && p.batch == 1 && p.correction == nullptr) {
    p.correction = p.col_term;
    p.col_term = nullptr;
  }
  return ST_OK;
}

int32_t run_problem(const Problem& pr, const VecopsHipPlan& plan, const float* row_scales, const float* column_scales,
                    const int32_t* correction, void* workspace, uint64_t workspace_size, hipStream_t stream) {
  if (plan.family == VECOPS_HIP_FAMILY_NONE) return ST_OK;
  if (int32_t rc = check_device(); rc != ST_OK) return rc;
  if (pr.a.data == nullptr && pr.k > 0) return fail(ST_INVALID, "matmul: a has no storage");
  if (pr.b.data == nullptr && pr.k > 0) return fail(ST_INVALID, "matmul: b has no storage");
  if (pr.packed_b && plan.family == VECOPS_HIP_FAMILY_SKINNY) return fail(ST_INVALID, "matmul: plan does not fit a packed b");
  if (pr.c.data == nullptr) return fail(ST_INVALID, "matmul: c has no storage");
  if (plan.workspace_bytes > workspace_size || (plan.workspace_bytes > 0 && workspace == nullptr))
    return fail(ST_INVALID, "matmul: workspace of %llu bytes required, %llu supplied",
                (unsigned long long)plan.workspace_bytes, (unsigned long long)workspace_size);

  if (plan.peeled_columns > 0) {
    // the last columns of C as a product of their own (choose() planned it with the same limit and found that it fits)
    Problem main, rest;
    cut_columns(pr, pr.n - plan.peeled_columns, &main, &rest);
    VecopsHipPlan main_plan = plan, rest_plan;
    main_plan.peeled_columns = 0;
    main_plan.workspace_bytes = 0;
    choose(rest, &rest_plan, workspace_size, false);
    // (checked before anything is launched: the main product must not have written C when the call fails)
    if (rest_plan.workspace_bytes > workspace_size || (rest_plan.workspace_bytes > 0 && workspace == nullptr))
      return fail(ST_INVALID, "matmul: the peeled columns need a workspace of %llu bytes, %llu supplied",
                  (unsigned long long)rest_plan.workspace_bytes, (unsigned long long)workspace_size);
    int32_t rc = run_problem(main, main_plan, row_scales, column_scales, correction, nullptr, 0, stream);
    if (rc != ST_OK) return rc;
    return run_problem(rest, rest_plan, row_scales, column_scales, correction, workspace, workspace_size, stream);
  }

  TileGemmParams p = base_params(pr, row_scales, column_scales, correction, workspace);
  const bool is_int = pr.src == SRC_I8 || pr.src == SRC_I8_FLIP;

  if (pr.src == kSrcF64) {  // (K = 0 included: the kernel then writes C_in or zeros)
    GemmF64Params q;
    memset(&q, 0, sizeof(q));
    q.a = static_cast<const double*>(pr.a.data);
    q.b = static_cast<const double*>(pr.b.data);
    q.c = static_cast<double*>(pr.c.data);
    q.cin = pr.has_cin ? static_cast<const double*>(pr.cin.data) : nullptr;
    q.m = p.m; q.n = p.n; q.k = p.k; q.batch = p.batch;
    q.a_rs = pr.a.rs; q.a_ks = pr.a.cs; q.a_bs = pr.a.bs;
    q.b_rs = pr.b.rs; q.b_ks = pr.b.cs; q.b_bs = pr.b.bs;
    q.c_rs = pr.c.rs; q.c_cs = pr.c.cs; q.c_bs = pr.c.bs;
    if (pr.has_cin) { q.cin_rs = pr.cin.rs; q.cin_cs = pr.cin.cs; q.cin_bs = pr.cin.bs; }
    if (pr.batch > 65535) return fail(ST_INVALID, "matmul: more than 65535 fp64 batches");
    hipError_t e64 = launch_gemm_f64(q, stream);
    if (e64 != hipSuccess) return fail(ST_EXEC, "fp64 kernel launch: %s", hipGetErrorString(e64));
    return ST_OK;
  }
  if (plan.family == VECOPS_HIP_FAMILY_ZERO_K) {
    p.split_k = 0;  // empty sum: the reduce kernel emits epilogue(0)
    hipError_t e = launch_splitk_reduce(p, is_int, stream);
    if (e != hipSuccess) return fail(ST_EXEC, "zero-K kernel launch: %s", hipGetErrorString(e));
    return ST_OK;
  }

  if (plan.family == VECOPS_HIP_FAMILY_SKINNY) {
    const bool a_narrow = pr.m < pr.n;  // else b is the narrow side
    const View& wide = a_narrow ? pr.b : pr.a;
    const View& narrow = a_narrow ? pr.a : pr.b;
    SkinnyDenseParams q;
    memset(&q, 0, sizeof(q));
    q.w = wide.data;
    q.x = narrow.data;
    q.y = pr.c.data;
    q.ldw = wide.rs;
    q.ldx = narrow.rs;
    q.w_bs = wide.bs;
    q.x_bs = narrow.bs;
    q.y_bs = pr.c.bs;
    q.y_stride_r = a_narrow ? pr.c.cs : pr.c.rs;
    q.y_stride_s = a_narrow ? pr.c.rs : pr.c.cs;
    q.rows = static_cast<int32_t>(wide.rows);
    q.s = static_cast<int32_t>(narrow.rows);
    q.k = static_cast<int32_t>(pr.k);
    if (is_int) {
      q.out_kind = row_scales != nullptr ? SKINNY_OUT_DEQUANT_F32 : SKINNY_OUT_I32;
      q.narrow_scales = row_scales;  // dequantisation comes here only with A as the narrow side
      q.wide_scales = column_scales;
      q.wide_term = correction;
    } else {
      q.out_kind = pr.out_kind == OUT_BF16 ? SKINNY_OUT_BF16 : pr.out_kind == OUT_F16 ? SKINNY_OUT_F16 : SKINNY_OUT_F32;
    }
    // 64 wide rows per workgroup when that still leaves most compute units a workgroup, else 32 or 16
    const int64_t wgs64 = (wide.rows + 63) / 64 * pr.batch;
    const dim3 block(512);
    auto launch = [&](auto src_tag) {
      constexpr int SRC = decltype(src_tag)::value;
      if (wgs64 >= 200) {
        hipLaunchKernelGGL((skinny_dense_kernel<SRC, 2, 2>), dim3(static_cast<unsigned>((wide.rows + 63) / 64), p.batch),
                           block, 0, stream, q);
      } else if (wgs64 * 2 >= 200) {
        hipLaunchKernelGGL((skinny_dense_kernel<SRC, 1, 2>), dim3(static_cast<unsigned>((wide.rows + 31) / 32), p.batch),
                           block, 0, stream, q);
      } else {
        hipLaunchKernelGGL((skinny_dense_kernel<SRC, 1, 1>), dim3(static_cast<unsigned>((wide.rows + 15) / 16), p.batch),
                           block, 0, stream, q);
      }
    };
    if (is_int) launch(std::integral_constant<int, SRC_I8>{});
    else if (pr.src == SRC_F16) launch(std::integral_constant<int, SRC_F16>{});
    else if (pr.src == SRC_F32_AS_BF16) launch(std::integral_constant<int, SRC_F32_AS_BF16>{});
    else if (pr.src == SRC_F32) launch(std::integral_constant<int, SRC_F32>{});
    else launch(std::integral_constant<int, SRC_BF16>{});
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(ST_EXEC, "skinny kernel launch: %s", hipGetErrorString(e));
    return ST_OK;
  }

  int tile_m = 0, tile_n = 0;
  tile_of_family(plan.family, &tile_m, &tile_n);
  if (tile_m == 0) return fail(ST_INVALID, "matmul: plan names no kernel family (%u)", plan.family);
  const int ktile = k_tile_elements(pr.src);
  p.tiles_m = static_cast<int32_t>((pr.m + tile_m - 1) / tile_m);
  p.tiles_n = static_cast<int32_t>((pr.n + tile_n - 1) / tile_n);
  const int k_tiles = static_cast<int>((pr.k + ktile - 1) / ktile);
  p.split_k = static_cast<int32_t>(plan.split_k);
  p.k_tiles_per_split = (k_tiles + p.split_k - 1) / p.split_k;
  const int mode = fetch_mode(pr, plan);

  hipError_t e;
  if (pr.src == SRC_I8_FLIP) {
    // terms of the unsigned side(s), kept behind the split-K partials in the workspace
    const uint64_t partial_bytes = plan.split_k > 1 ? static_cast<uint64_t>(plan.split_k) * pr.batch * pr.m * pr.n * 4u : 0;
    int32_t rc = unsigned_side_terms(pr, &p, reinterpret_cast<int32_t*>(static_cast<char*>(workspace) + partial_bytes), stream);
    if (rc != ST_OK) return rc;
  }
  if (plan.family == VECOPS_HIP_FAMILY_TILE_192 && !tile_192_serves(pr, plan))
    return fail(ST_INVALID, "matmul: the plan's family tile_192 cannot serve this call");
  if (plan.family == VECOPS_HIP_FAMILY_TILE_256X352) {
    if (!wide_tile_serves(pr) || !launch_tile_gemm_wide_serves(pr.src, p, mode, pr.packed_b))
      return fail(ST_INVALID, "matmul: the plan's family tile_256x352 cannot serve this call");
    e = launch_tile_gemm_wide(pr.src, p, pr.packed_b, stream);
  } else if (!pr.packed_b && tile_m == 128 && tile_n == 128 && pr.k <= kRules.short_k_direct_max_k &&
             launch_tile_gemm_short_k_serves(pr.src, p)) {
    // a K tile or two: the kernel that is all stores
    e = launch_tile_gemm_short_k(pr.src, p, stream);
  } else if (pr.packed_b && launch_tile_gemm_packed16_serves(pr.src, p, tile_m, tile_n)) {
    e = launch_tile_gemm_packed16(pr.src, p, stream);
  } else if (pr.packed_b && tile_m == 128 && tile_n == 128 && p.k_tiles_per_split >= kRules.deep_min_k_tiles &&
             static_cast<int64_t>(p.tiles_m) * p.tiles_n * p.batch * p.split_k <= kRules.deep_max_workgroups &&
             launch_tile_gemm_deep128_serves(pr.src, p, mode, true)) {
    // at most one workgroup per compute unit: the four-stage kernel with the pack kept in its order in LDS
    e = launch_tile_gemm_deep128(pr.src, p, mode, true, stream);
  } else if (pr.packed_b) {
    const int a_mode = plan.vector_a == 0 ? 0 : ((pr.src == SRC_BF16 || pr.src == SRC_F16 || pr.src == SRC_I8) && lines_up(pr, pr.a, pr.a.rs)) ? 2 : 1;
    e = launch_tile_gemm_packed_b(pr.src, p, tile_m, tile_n, a_mode, stream);
  } else if (tile_m == 128 && tile_n == 128 && p.k_tiles_per_split >= kRules.deep_min_k_tiles &&
             static_cast<int64_t>(p.tiles_m) * p.tiles_n * p.batch * p.split_k <= kRules.deep_max_workgroups &&
             launch_tile_gemm_deep128_serves(pr.src, p, mode, false)) {
    // at most one workgroup per compute unit: the four-stage kernel, whose loads run three K tiles ahead
    e = launch_tile_gemm_deep128(pr.src, p, mode, false, stream);
  } else if (pr.src == SRC_F32 && tile_m == tile_n && (tile_m == 64 || tile_m == 128) && (mode == MODE_KVEC || mode == MODE_NVEC_B) &&
             p.k_tiles_per_split >= kRules.deep_min_k_tiles &&
             static_cast<int64_t>(p.tiles_m) * p.tiles_n * p.batch * p.split_k <= kRules.deep_max_workgroups &&
             launch_tile_gemm_deep_f32_serves(p, tile_m, mode == MODE_NVEC_B)) {
    // fp32 compute, at most one workgroup per compute unit: the ring of LDS stages (tile_gemm_deep_f32.hip)
    e = launch_tile_gemm_deep_f32(p, tile_m, mode == MODE_NVEC_B, stream);
  } else switch (pr.src) {
    case SRC_I8_FLIP: e = launch_tile_gemm_i8_flip(p, tile_m, tile_n, mode, stream); break;
    case SRC_BF16: e = launch_tile_gemm_bf16(p, tile_m, tile_n, mode, stream); break;
    case SRC_F16: e = launch_tile_gemm_f16(p, tile_m, tile_n, mode, stream); break;
    case SRC_F32_AS_BF16: e = launch_tile_gemm_f32_as_bf16(p, tile_m, tile_n, mode, stream); break;
    case SRC_F32: e = launch_tile_gemm_f32(p, tile_m, tile_n, mode, stream); break;
    default: e = launch_tile_gemm_i8(p, tile_m, tile_n, mode, stream); break;
  }
  if (e != hipSuccess) return fail(ST_EXEC, "tile kernel launch: %s", hipGetErrorString(e));
  if (p.split_k > 1) {
    e = launch_splitk_reduce(p, is_int, stream);
    if (e != hipSuccess) return fail(ST_EXEC, "split-K reduce launch: %s", hipGetErrorString(e));
  }
  return ST_OK;
}

void make_operand(VecopsHipOperand* o, const void* data, uint32_t dtype, int64_t rows, int64_t cols, int64_t rs) {
  memset(o, 0, sizeof(*o));
  o->data = const_cast<void*>(data);
  o->dtype = dtype;
  o->rank = 2;
  o->sizes[0] = rows;
  o->sizes[1] = cols;
  o->strides[0] = rs;
  o->strides[1] = 1;
}

template <int MB, int ROWS, int UNROLL>
void launch_skinny(const SkinnyW8A16Params& p, hipStream_t stream) {
  const int64_t waves = (p.n + ROWS - 1) / ROWS;
  const int64_t blocks = (waves + 3) / 4;
  hipLaunchKernelGGL((skinny_w8a16_kernel<MB, ROWS, UNROLL>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream,
                     p);
}

template <int SPG, int TILES>
void launch_skinny_mfma(const SkinnyW8A16Params& p, hipStream_t stream) {
  constexpr int kWaves = 8;
  const int64_t blocks = (p.n + 16 * TILES - 1) / (16 * TILES);
  hipLaunchKernelGGL((skinny_w8a16_mfma_kernel<kWaves, SPG, TILES>), dim3(static_cast<unsigned>(blocks)),
                     dim3(64 * kWaves), 0, stream, p);
}

// The register-resident variant: K must be exactly 8 wavefronts x 8 steps x 64.
template <int SPG, int TILES, int PASSES>
void launch_skinny_mfma_resident(const SkinnyW8A16Params& p, hipStream_t stream) {
  const int64_t rows_per_wg = static_cast<int64_t>(16) * TILES * PASSES;
  const int64_t blocks = (p.n + rows_per_wg - 1) / rows_per_wg;
  hipLaunchKernelGGL((skinny_w8a16_mfma_resident_kernel<SPG, TILES, PASSES>), dim3(static_cast<unsigned>(blocks)), dim3(512),
                     0, stream, p);
}

// Elements per 16-byte chunk of a packed operand of this dtype (0: no such pack).
int packed_elems_per_chunk(uint32_t packed_dtype) {
  return (packed_dtype == DT_I8 || packed_dtype == DT_U8) ? 16 : (packed_dtype == DT_BF16 || packed_dtype == DT_F16) ? 8
         : packed_dtype == DT_F32 ? 4 : 0;
}

// Problem description of a matmul whose B operand is prepacked: b is described as the dense
// [N,K] operand it was packed from (its strides are never used), with `packed` as its storage.
int32_t describe_packed(const VecopsHipOperand* a, const void* packed, uint32_t packed_dtype, int64_t n,
                        const VecopsHipOperand* cin, const VecopsHipOperand* c, Problem* pr, bool may_fold = true) {
  if (a == nullptr || (a->rank != 2 && a->rank != 3)) return fail(ST_INVALID, "matmul_packed_b: malformed a");
  if (n < 0) return fail(ST_INVALID, "matmul_packed_b: negative n");
  const uint32_t da = a->dtype;
  if (packed_dtype == DT_BF16) {
    if (da != DT_BF16 && da != DT_F32) return fail(ST_NOT_APPLICABLE, "matmul_packed_b: a bf16-packed b needs a bf16 or f32 a");
  } else if (packed_dtype == DT_F16) {
    if (da != DT_F16) return fail(ST_NOT_APPLICABLE, "matmul_packed_b: an f16-packed b needs an f16 a");
  } else if (packed_dtype == DT_I8 || packed_dtype == DT_U8) {
    if (da != DT_I8 && da != DT_U8) return fail(ST_NOT_APPLICABLE, "matmul_packed_b: an 8-bit packed b needs an i8 or u8 a");
  } else if (packed_dtype == DT_F32) {  // the fp32-compute atom: operands stay fp32
    if (da != DT_F32) return fail(ST_NOT_APPLICABLE, "matmul_packed_b: an f32-packed b needs an f32 a");
  } else {
    return fail(ST_NOT_APPLICABLE, "matmul_packed_b: packed dtype %u not supported", packed_dtype);
  }
  VecopsHipOperand b;
  memset(&b, 0, sizeof(b));
  b.data = const_cast<void*>(packed);
  // (an unsigned operand is packed as b - 128, signed: the product's epilogue adds 128 * sum_k a[m,k] back)
  b.dtype = (packed_dtype == DT_I8 || packed_dtype == DT_U8) ? packed_dtype : da;
  b.rank = a->rank;
  const int base = a->rank == 3 ? 1 : 0;
  const int64_t k = a->sizes[base + 1];
  if (a->rank == 3) b.sizes[0] = a->sizes[0];  // batch stride 0: one packed operand for every batch
  b.sizes[base] = n;
  b.sizes[base + 1] = k;
  b.strides[base] = k;
  b.strides[base + 1] = 1;
  int32_t rc = describe(a, &b, cin, c, packed_dtype == DT_F32 ? VECOPS_HIP_COMPUTE_F32 : VECOPS_HIP_COMPUTE_BF16, pr, nullptr,
                        may_fold);
  if (rc != ST_OK) return rc;
  pr->packed_b = true;
  // 32-bit offsets inside one workgroup's eight 32-row panels of the packed operand
  const int64_t ks_total = packed_k_steps(pr->k, packed_elems_per_chunk(packed_dtype));
  if (ks_total * 1024 * 8 >= (int64_t{1} << 31)) return fail(ST_NOT_APPLICABLE, "matmul_packed_b: k too large");
  return ST_OK;
}

// The pack kernel for a source dtype and the dtype it is packed as (half operands are packed by the bf16 kernel: a
// permutation of 16-bit elements either way); -1: no such pack.
int src_of_pack(uint32_t source, uint32_t packed_dtype) {
  if (source == DT_BF16 && packed_dtype == DT_BF16) return SRC_BF16;
  if (source == DT_F16 && packed_dtype == DT_F16) return SRC_BF16;
  if (source == DT_F32 && packed_dtype == DT_BF16) return SRC_F32_AS_BF16;
  if (source == DT_F32 && packed_dtype == DT_F32) return SRC_F32;
  if ((source == DT_I8 || source == DT_U8) && packed_dtype == source) return SRC_I8;
  return -1;
}

}  // namespace

extern "C" {

uint64_t vecops_hip_packed_b_bytes(uint32_t packed_dtype, int64_t n, int64_t k) {
  const int epc = packed_elems_per_chunk(packed_dtype);
  if (n < 0 || k < 0 || epc == 0) return 0;
  return static_cast<uint64_t>(packed_b_bytes(n, k, epc));
}

int32_t vecops_hip_pack_as(const VecopsHipOperand* b, uint32_t packed_dtype, void* packed, uint64_t packed_size, void* stream) {
  View v;
  if (!normalise(b, &v) || b->rank != 2) return fail(ST_INVALID, "pack: the source must be a rank-2 [rows, K] operand");
  const int src = src_of_pack(v.dtype, packed_dtype);
  if (src < 0) return fail(ST_NOT_APPLICABLE, "pack: dtype %u cannot be packed as dtype %u", v.dtype, packed_dtype);
  if (v.rows > INT32_MAX || v.cols > INT32_MAX - 256) return fail(ST_INVALID, "pack_b: extent too large");
  const uint64_t need = static_cast<uint64_t>(packed_b_bytes(v.rows, v.cols, packed_elems_per_chunk(packed_dtype)));
  if (packed_size < need)
    return fail(ST_INVALID, "pack_b: %llu bytes required, %llu supplied", (unsigned long long)need,
                (unsigned long long)packed_size);
  if (need == 0) return ST_OK;
  if (packed == nullptr || !aligned16(packed)) return fail(ST_INVALID, "pack_b: packed storage must be 16-byte aligned");
  if (v.data == nullptr) return fail(ST_INVALID, "pack_b: b has no storage");
  PackBParams q;
  q.b = v.data;
  q.packed = packed;
  q.rs = v.rs;
  q.ks = v.cs;
  q.n = static_cast<int32_t>(v.rows);
  q.k = static_cast<int32_t>(v.cols);
  q.flip = v.dtype == DT_U8 ? 0x80u : 0u;
  hipError_t e = launch_pack_b(src, q, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return fail(ST_EXEC, "pack kernel launch: %s", hipGetErrorString(e));
  return ST_OK;
}

int32_t vecops_hip_pack_b(const VecopsHipOperand* b, void* packed, uint64_t packed_size, void* stream) {
  if (b == nullptr) return fail(ST_INVALID, "pack_b: b must be a rank-2 [N,K] operand");
  // the default pack of a dtype: fp32 sources are rounded to bf16 (the x86 reference's behaviour), the others keep theirs
  return vecops_hip_pack_as(b, b->dtype == DT_F32 ? DT_BF16 : b->dtype, packed, packed_size, stream);
}

int32_t vecops_hip_pack_b_compensated(const VecopsHipOperand* b, int32_t a_zero_point, void* packed,
                                      uint64_t packed_size, int32_t* compensation, void* stream) {
  if (b == nullptr || b->dtype != DT_I8) return fail(ST_NOT_APPLICABLE, "pack_b_compensated: b must be int8");
  int32_t rc = vecops_hip_pack_b(b, packed, packed_size, stream);
  if (rc != ST_OK) return rc;
  View v;
  normalise(b, &v);
  if (v.rows == 0) return ST_OK;
  if (compensation == nullptr) return fail(ST_INVALID, "pack_b_compensated: null compensation");
  // -a_zero_point * sum_k b[n,k], wrapping like every int32 accumulator of the path
  hipError_t e = launch_byte_row_sums(v.data, 1, static_cast<int32_t>(v.rows), static_cast<int32_t>(v.cols), 0, v.rs, v.cs,
                                      0u, 0u - static_cast<uint32_t>(a_zero_point), nullptr, 0, compensation,
                                      static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return fail(ST_EXEC, "row-sum kernel launch: %s", hipGetErrorString(e));
  return ST_OK;
}

int32_t vecops_hip_plan_matmul_packed_b(const VecopsHipOperand* a, uint32_t packed_dtype, int64_t n,
                                        const VecopsHipOperand* c_in, const VecopsHipOperand* c, VecopsHipPlan* plan) {
  if (plan == nullptr) return fail(ST_INVALID, "plan_matmul_packed_b: null plan");
  Problem pr{};
  int32_t rc = describe_packed(a, reinterpret_cast<void*>(16), packed_dtype, n, c_in, c, &pr);
  if (rc != ST_OK) return rc;
  choose(pr, plan);
  return ST_OK;
}

int32_t vecops_hip_matmul_packed_b(const VecopsHipOperand* a, const void* packed_b, uint32_t packed_dtype, int64_t n,
                                   const VecopsHipOperand* c_in, const VecopsHipOperand* c, void* workspace,
                                   uint64_t workspace_size, void* stream) {
  Problem pr{};
  int32_t rc = describe_packed(a, packed_b, packed_dtype, n, c_in, c, &pr);
  if (rc != ST_OK) return rc;
  if (pr.k > 0 && pr.n > 0 && !aligned16(packed_b)) return fail(ST_INVALID, "matmul_packed_b: packed b must be 16-byte aligned");
  VecopsHipPlan plan;
  choose(pr, &plan);
  return run_problem(pr, plan, nullptr, nullptr, nullptr, workspace, workspace_size, static_cast<hipStream_t>(stream));
}

int32_t vecops_hip_pack_a(const VecopsHipOperand* a, void* packed, uint64_t packed_size, void* stream) {
  // the [M,K] operand in the same 32-row panels: the two sides share one format here
  return vecops_hip_pack_b(a, packed, packed_size, stream);
}

namespace {
// The descriptor of the transposed matrix (the last two dimensions swapped).
VecopsHipOperand transposed(const VecopsHipOperand& o) {
  VecopsHipOperand t = o;
  if (o.rank == 2 || o.rank == 3) {
    const int i = static_cast<int>(o.rank) - 2;
    t.sizes[i] = o.sizes[i + 1]; t.sizes[i + 1] = o.sizes[i];
    t.strides[i] = o.strides[i + 1]; t.strides[i + 1] = o.strides[i];
  }
  return t;
}

// A packed: C^T = B . A^T is the product of the plain operand b with the packed operand a.
int32_t describe_packed_a(const void* packed_a, uint32_t packed_dtype, int64_t m, const VecopsHipOperand* b,
                          const VecopsHipOperand* c_in, const VecopsHipOperand* c, VecopsHipOperand* ct,
                          VecopsHipOperand* cint, Problem* pr) {
  if (b == nullptr || c == nullptr) return fail(ST_INVALID, "matmul_packed_a: null operand");
  *ct = transposed(*c);
  if (c_in != nullptr) *cint = transposed(*c_in);
  return describe_packed(b, packed_a, packed_dtype, m, c_in ? cint : nullptr, ct, pr);
}
}  // namespace

int32_t vecops_hip_plan_matmul_packed_a(uint32_t packed_dtype, int64_t m, const VecopsHipOperand* b,
                                        const VecopsHipOperand* c_in, const VecopsHipOperand* c, VecopsHipPlan* plan) {
  if (plan == nullptr) return fail(ST_INVALID, "plan_matmul_packed_a: null plan");
  Problem pr{};
  VecopsHipOperand ct, cint;
  int32_t rc = describe_packed_a(reinterpret_cast<void*>(16), packed_dtype, m, b, c_in, c, &ct, &cint, &pr);
  if (rc != ST_OK) return rc;
  choose(pr, plan);
  return ST_OK;
}

int32_t vecops_hip_matmul_packed_a(const void* packed_a, uint32_t packed_dtype, int64_t m, const VecopsHipOperand* b,
                                   const VecopsHipOperand* c_in, const VecopsHipOperand* c, void* workspace,
                                   uint64_t workspace_size, void* stream) {
  Problem pr{};
  VecopsHipOperand ct, cint;
  int32_t rc = describe_packed_a(packed_a, packed_dtype, m, b, c_in, c, &ct, &cint, &pr);
  if (rc != ST_OK) return rc;
  if (pr.k > 0 && pr.n > 0 && !aligned16(packed_a)) return fail(ST_INVALID, "matmul_packed_a: packed a must be 16-byte aligned");
  VecopsHipPlan plan;
  choose(pr, &plan);
  return run_problem(pr, plan, nullptr, nullptr, nullptr, workspace, workspace_size, static_cast<hipStream_t>(stream));
}

namespace {
// Both operands packed: A is unpacked into the front of the workspace (a dense [M,K] matrix of its own dtype) and
// multiplied with the packed B.
struct BothPacked {
  VecopsHipOperand a;
  Problem pr{};
  VecopsHipPlan plan;
  uint64_t a_bytes;
};
int32_t describe_packed_ab(uint32_t a_dtype, int64_t m, uint32_t b_dtype, int64_t n, int64_t k, const VecopsHipOperand* c_in,
                           const VecopsHipOperand* c, void* workspace, BothPacked* d) {
  if (m < 0 || n < 0 || k < 0) return fail(ST_INVALID, "matmul_packed_ab: negative extent");
  if (packed_elems_per_chunk(a_dtype) == 0)
    return fail(ST_NOT_APPLICABLE, "matmul_packed_ab: packed dtype %u not supported", a_dtype);
  if (c == nullptr || c->rank != 2) return fail(ST_NOT_APPLICABLE, "matmul_packed_ab: c must be rank 2 (a packed operand has no batches)");
  make_operand(&d->a, workspace, a_dtype, m, k, k);
  d->a_bytes = round_up_256(static_cast<uint64_t>(m) * k * dtype_bytes(a_dtype));
  int32_t rc = describe_packed(&d->a, reinterpret_cast<void*>(16), b_dtype, n, c_in, c, &d->pr);
  if (rc != ST_OK) return rc;
  choose(d->pr, &d->plan);
  return ST_OK;
}
}  // namespace

uint64_t vecops_hip_matmul_packed_ab_workspace(uint32_t a_dtype, int64_t m, uint32_t b_dtype, int64_t n, int64_t k,
                                               const VecopsHipOperand* c_in, const VecopsHipOperand* c) {
  BothPacked d;
  if (describe_packed_ab(a_dtype, m, b_dtype, n, k, c_in, c, reinterpret_cast<void*>(256), &d) != ST_OK) return 0;
  return d.a_bytes + d.plan.workspace_bytes;
}

int32_t vecops_hip_matmul_packed_ab(const void* packed_a, uint32_t a_dtype, int64_t m, const void* packed_b, uint32_t b_dtype,
                                    int64_t n, int64_t k, const VecopsHipOperand* c_in, const VecopsHipOperand* c,
                                    void* workspace, uint64_t workspace_size, void* stream) {
  BothPacked d;
  int32_t rc = describe_packed_ab(a_dtype, m, b_dtype, n, k, c_in, c, workspace ? workspace : reinterpret_cast<void*>(256), &d);
  if (rc != ST_OK) return rc;
  if (d.plan.family == VECOPS_HIP_FAMILY_NONE) return ST_OK;
  const uint64_t need = d.a_bytes + d.plan.workspace_bytes;
  if (need > workspace_size || (need > 0 && (workspace == nullptr || !aligned16(workspace))))
    return fail(ST_INVALID, "matmul_packed_ab: %llu bytes of 16-byte aligned workspace required, %llu supplied",
                (unsigned long long)need, (unsigned long long)workspace_size);
  if (k > 0 && (packed_a == nullptr || packed_b == nullptr || !aligned16(packed_a) || !aligned16(packed_b)))
    return fail(ST_INVALID, "matmul_packed_ab: packed operands must be 16-byte aligned");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (k > 0 && m > 0) {
    PackBParams q;
    q.b = workspace;
    q.packed = const_cast<void*>(packed_a);
    q.rs = k;
    q.ks = 1;
    q.n = static_cast<int32_t>(m);
    q.k = static_cast<int32_t>(k);
    q.flip = a_dtype == DT_U8 ? 0x80u : 0u;
    hipError_t e = launch_unpack_b((a_dtype == DT_I8 || a_dtype == DT_U8) ? SRC_I8 : a_dtype == DT_F32 ? SRC_F32 : SRC_BF16, q, s);
    if (e != hipSuccess) return fail(ST_EXEC, "unpack kernel launch: %s", hipGetErrorString(e));
  }
  d.pr.b.data = const_cast<void*>(packed_b);
  return run_problem(d.pr, d.plan, nullptr, nullptr, nullptr, static_cast<char*>(workspace) + d.a_bytes,
                     workspace_size - d.a_bytes, s);
}

int32_t vecops_hip_matmul_i8_dequant_packed_b(const int8_t* a, int64_t lda, const void* packed_b,
                                              const float* row_scales, const float* column_scales,
                                              const int32_t* correction, float* c, int64_t ldc, int64_t m, int64_t n,
                                              int64_t k, void* workspace, uint64_t workspace_size, void* stream) {
  if (m < 0 || n < 0 || k < 0) return fail(ST_INVALID, "matmul_i8_dequant_packed_b: negative extent");
  if (m > 0 && n > 0 && (row_scales == nullptr || column_scales == nullptr))
    return fail(ST_INVALID, "matmul_i8_dequant_packed_b: scales are required");
  VecopsHipOperand oa, oc;
  make_operand(&oa, a, DT_I8, m, k, lda);
  make_operand(&oc, c, DT_I32, m, n, ldc);  // accumulator class; the epilogue writes fp32
  Problem pr{};
  int32_t rc = describe_packed(&oa, packed_b, DT_I8, n, nullptr, &oc, &pr);
  if (rc != ST_OK) return rc;
  if (pr.k > 0 && pr.n > 0 && !aligned16(packed_b)) return fail(ST_INVALID, "matmul_i8_dequant_packed_b: packed b must be 16-byte aligned");
  VecopsHipPlan plan;
  choose(pr, &plan);
  return run_problem(pr, plan, row_scales, column_scales, correction, workspace, workspace_size,
                     static_cast<hipStream_t>(stream));
}

int32_t vecops_hip_quantize_rows(const VecopsHipOperand* x, const float* multipliers, int32_t zero_point,
                                 const VecopsHipOperand* q, void* stream) {
  View vx, vq;
  if (!normalise(x, &vx) || !normalise(q, &vq)) return fail(ST_INVALID, "quantize_rows: operands must be rank 2 or 3");
  if (vx.dtype != DT_F32 || vq.dtype != DT_U8) return fail(ST_NOT_APPLICABLE, "quantize_rows: x must be f32 and q u8");
  if (x->rank != q->rank || vx.batch != vq.batch || vx.rows != vq.rows || vx.cols != vq.cols)
    return fail(ST_INVALID, "quantize_rows: x and q differ in shape");
  if (vx.batch == 0 || vx.rows == 0 || vx.cols == 0) return ST_OK;
  if (vx.data == nullptr || vq.data == nullptr || multipliers == nullptr) return fail(ST_INVALID, "quantize_rows: null operand");
  if (vx.batch * vx.rows > INT32_MAX || vx.rows > INT32_MAX || vx.cols > INT32_MAX)
    return fail(ST_INVALID, "quantize_rows: extent too large");
  hipError_t e = launch_quantize_rows(static_cast<const float*>(vx.data), static_cast<int32_t>(vx.batch),
                                      static_cast<int32_t>(vx.rows), static_cast<int32_t>(vx.cols), vx.bs, vx.rs, vx.cs,
                                      multipliers, vx.rows, zero_point, 0u, static_cast<uint8_t*>(vq.data), vq.bs, vq.rs, vq.cs,
                                      static_cast<hipStream_t>(stream));
  if (e != hipSuccess) return fail(ST_EXEC, "quantize kernel launch: %s", hipGetErrorString(e));
  return ST_OK;
}

namespace {
// The pieces of vecops_hip_matmul_runtime_quant.  The activations are quantised to q - 128 as int8 (the byte
// xor 0x80), so that the product runs on the signed kernels with their fast dequantising epilogue, and
//   sum_k q * b = sum_k (q - 128) * b + 128 * sum_k b[n,k]
// goes into the correction rows.  Workspace: the quantised activations (one [M,K] matrix per batch, or a single
// one when every batch shares activations and multipliers), the correction rows (N int32 per batch, or a single
// row when every batch shares weights and correction) - both rounded up to 256 bytes - then the product's own
// scratch.
struct RuntimeQuant {
  VecopsHipOperand a3, b3, c3, q, c_acc;
  Problem pr{};
  VecopsHipPlan plan;
  int64_t batch, m, n, k;
  int64_t q_batches, row_batches;  // distinct quantised matrices / correction rows
  int64_t scale_bs, correction_bs;
  uint64_t q_bytes, row_bytes;
};

// Rank 2 as the rank 3 of one batch.
bool as_rank3(const VecopsHipOperand* o, VecopsHipOperand* out) {
  if (o == nullptr || (o->rank != 2 && o->rank != 3)) return false;
  *out = *o;
  if (o->rank == 3) return true;
  memset(out->sizes, 0, sizeof(out->sizes));
  memset(out->strides, 0, sizeof(out->strides));
  out->rank = 3;
  out->sizes[0] = 1;
  for (int i = 0; i < 2; ++i) { out->sizes[i + 1] = o->sizes[i]; out->strides[i + 1] = o->strides[i]; }
  return true;
}

// b is the int8 operand (rank 2: one set of weights for every batch; rank 3: its batch stride may be 0), or null with
// `packed` / `packed_n` describing weights packed by vecops_hip_pack_b.  scale_bs / correction_bs: batch strides of
// multipliers and row_scales / of the correction row (vecops' batch_stride of the two transforms,
// matmul/Quantization.h:91-146,195-250; tests/ops/MatmulConversionTestCommon.h:1277-1434 runs M and 0, N and 0).
int32_t describe_runtime_quant(const VecopsHipOperand* a_given, const VecopsHipOperand* b_given, const void* packed,
                               int64_t packed_n, const VecopsHipOperand* c_given, int64_t scale_bs, int64_t correction_bs,
                               void* workspace, RuntimeQuant* d) {
  if (!as_rank3(a_given, &d->a3) || !as_rank3(c_given, &d->c3) || a_given->rank != c_given->rank)
    return fail(ST_INVALID, "matmul_runtime_quant: a and c must be rank 2 or both rank 3");
  if (d->a3.dtype != DT_F32) return fail(ST_NOT_APPLICABLE, "matmul_runtime_quant: a must be an f32 operand");
  if (d->c3.dtype != DT_F32) return fail(ST_NOT_APPLICABLE, "matmul_runtime_quant: c must be an f32 operand");
  d->batch = d->c3.sizes[0];
  d->m = d->a3.sizes[1];
  d->k = d->a3.sizes[2];
  if (d->a3.sizes[0] != d->batch) return fail(ST_INVALID, "matmul_runtime_quant: a and c differ in batch extent");
  if (packed == nullptr) {
    if (b_given == nullptr || b_given->dtype != DT_I8 || !as_rank3(b_given, &d->b3))
      return fail(ST_NOT_APPLICABLE, "matmul_runtime_quant: b must be a rank-2 or rank-3 i8 operand");
    if (b_given->rank == 2) {  // one set of weights for every batch
      d->b3.sizes[0] = d->batch;
      d->b3.strides[0] = 0;
    } else if (a_given->rank != 3 || d->b3.sizes[0] != d->batch) {
      return fail(ST_INVALID, "matmul_runtime_quant: a rank-3 b needs rank-3 a and c of the same batch extent");
    }
    d->n = d->b3.sizes[1];
  } else {
    d->n = packed_n;
  }
  if (d->batch < 0 || d->m < 0 || d->k < 0 || d->n < 0) return fail(ST_INVALID, "matmul_runtime_quant: negative extent");
  if (scale_bs < 0 || correction_bs < 0) return fail(ST_INVALID, "matmul_runtime_quant: negative batch stride");
  if (d->batch <= 1) scale_bs = correction_bs = 0;
  d->scale_bs = scale_bs;
  d->correction_bs = correction_bs;
  const bool shared_b = packed != nullptr || d->b3.strides[0] == 0 || d->batch <= 1;
  d->q_batches = (d->batch > 1 && (d->a3.strides[0] != 0 || scale_bs != 0)) ? d->batch : 1;
  d->row_batches = (d->batch > 1 && (!shared_b || correction_bs != 0)) ? d->batch : 1;
  d->q_bytes = (static_cast<uint64_t>(d->q_batches) * d->m * d->k + 255u) & ~uint64_t{255};
  d->row_bytes = (static_cast<uint64_t>(d->row_batches) * d->n * 4u + 255u) & ~uint64_t{255};
  // the quantised activations: dense [batch, M, K], every batch the same matrix when there is only one
  memset(&d->q, 0, sizeof(d->q));
  d->q.data = workspace;
  d->q.dtype = DT_I8;
  d->q.rank = a_given->rank;
  const int base = a_given->rank == 3 ? 1 : 0;
  if (base) { d->q.sizes[0] = d->batch; d->q.strides[0] = d->q_batches > 1 ? d->m * d->k : 0; }
  d->q.sizes[base] = d->m; d->q.strides[base] = d->k;
  d->q.sizes[base + 1] = d->k; d->q.strides[base + 1] = 1;
  d->c_acc = *c_given;
  d->c_acc.dtype = DT_I32;  // accumulator class; the epilogue writes fp32
  // Batches fold into rows ([batch * M, K] x the one B) only when the scales run on with the rows and one
  // correction row serves every batch.
  const bool may_fold = d->q_batches > 1 && scale_bs == d->m && d->row_batches == 1;
  int32_t rc;
  if (packed != nullptr) {
    rc = describe_packed(&d->q, packed, DT_I8, d->n, nullptr, &d->c_acc, &d->pr, may_fold);
  } else {
    const VecopsHipOperand* b = a_given->rank == 3 ? &d->b3 : b_given;
    rc = describe(&d->q, b, nullptr, &d->c_acc, 0, &d->pr, nullptr, may_fold);
  }
  if (rc != ST_OK) return rc;
  d->pr.dequant = true;
  if (d->pr.batch > 1) {
    d->pr.row_scales_bs = scale_bs;
    d->pr.correction_bs = d->row_batches > 1 ? d->n : 0;
  }
  choose(d->pr, &d->plan);
  return ST_OK;
}

int32_t run_runtime_quant(const VecopsHipOperand* a, const float* multipliers, int32_t zero_point, int64_t scale_bs,
                          const VecopsHipOperand* b, const void* packed, int64_t packed_n, const int32_t* correction,
                          int64_t correction_bs, const float* row_scales, const float* column_scales,
                          const VecopsHipOperand* c, void* workspace, uint64_t workspace_size, void* stream) {
  RuntimeQuant d{};
  int32_t rc = describe_runtime_quant(a, b, packed, packed_n, c, scale_bs, correction_bs,
                                      workspace ? workspace : reinterpret_cast<void*>(256), &d);
  if (rc != ST_OK) return rc;
  if (d.plan.family == VECOPS_HIP_FAMILY_NONE) return ST_OK;
  if (row_scales == nullptr || column_scales == nullptr || multipliers == nullptr)
    return fail(ST_INVALID, "matmul_runtime_quant: multipliers and both scale vectors are required");
  if (packed != nullptr && d.pr.k > 0 && !aligned16(packed)) return fail(ST_INVALID, "matmul_runtime_quant: packed b must be 16-byte aligned");
  if (d.batch * d.m > INT32_MAX || d.batch * d.n > INT32_MAX) return fail(ST_INVALID, "matmul_runtime_quant: extent too large");
  const uint64_t need = d.q_bytes + d.row_bytes + d.plan.workspace_bytes;
  if (need > workspace_size || workspace == nullptr || !aligned16(workspace))
    return fail(ST_INVALID, "matmul_runtime_quant: %llu bytes of 16-byte aligned workspace required, %llu supplied",
                (unsigned long long)need, (unsigned long long)workspace_size);
  hipStream_t s = static_cast<hipStream_t>(stream);
  View vx;
  normalise(&d.a3, &vx);
  // correction[batch][n] + 128 * sum_k b[batch][n,k]
  int32_t* rows = reinterpret_cast<int32_t*>(static_cast<char*>(workspace) + d.q_bytes);
  if (packed == nullptr && d.q_batches * d.m * d.k > 0 && d.row_batches * d.n > 0) {
    // the activations' quantisation and the weight rows' sums in one launch: neither needs the other
    View vb;
    normalise(&d.b3, &vb);
    hipError_t both = launch_quantize_and_row_sums(
        static_cast<const float*>(vx.data), static_cast<int32_t>(d.q_batches), static_cast<int32_t>(d.m), static_cast<int32_t>(d.k),
        vx.bs, vx.rs, vx.cs, multipliers, d.scale_bs, zero_point, 0x80u, static_cast<uint8_t*>(workspace), d.m * d.k, d.k, 1,
        vb.data, static_cast<int32_t>(d.row_batches), static_cast<int32_t>(d.n), vb.bs, vb.rs, vb.cs, 0u, 128u, correction,
        d.correction_bs, rows, s);
    if (both != hipSuccess) return fail(ST_EXEC, "quantize and row-sum kernel launch: %s", hipGetErrorString(both));
    return run_problem(d.pr, d.plan, row_scales, column_scales, rows, static_cast<char*>(workspace) + d.q_bytes + d.row_bytes,
                       workspace_size - d.q_bytes - d.row_bytes, s);
  }
  hipError_t e = launch_quantize_rows(static_cast<const float*>(vx.data), static_cast<int32_t>(d.q_batches),
                                      static_cast<int32_t>(d.m), static_cast<int32_t>(d.k), vx.bs, vx.rs, vx.cs,
                                      multipliers, d.scale_bs, zero_point, 0x80u, static_cast<uint8_t*>(workspace),
                                      d.m * d.k, d.k, 1, s);
  if (e != hipSuccess) return fail(ST_EXEC, "quantize kernel launch: %s", hipGetErrorString(e));
  if (packed != nullptr) {
    // one packed operand: the same sums for every batch, the caller's correction per batch
    for (int64_t bi = 0; bi < d.row_batches && e == hipSuccess; ++bi)
      e = launch_packed_row_sums(packed, static_cast<int32_t>(d.n), static_cast<int32_t>(d.k), 1, 128u,
                                 correction ? correction + bi * d.correction_bs : nullptr, rows + bi * d.n, s);
  } else {
    View vb;
    normalise(&d.b3, &vb);
    e = launch_byte_row_sums(vb.data, static_cast<int32_t>(d.row_batches), static_cast<int32_t>(d.n),
                             static_cast<int32_t>(d.k), vb.bs, vb.rs, vb.cs, 0u, 128u, correction, d.correction_bs, rows, s);
  }
  if (e != hipSuccess) return fail(ST_EXEC, "row-sum kernel launch: %s", hipGetErrorString(e));
  return run_problem(d.pr, d.plan, row_scales, column_scales, rows, static_cast<char*>(workspace) + d.q_bytes + d.row_bytes,
                     workspace_size - d.q_bytes - d.row_bytes, s);
}

// The batch strides of the reference's tests: scales run on with the rows of a ([batch * M]) unless every batch
// shares a, the correction rows run on ([batch * N]) when the weights are per batch.
void conventional_strides(const VecopsHipOperand* a, const VecopsHipOperand* b, int64_t* scale_bs, int64_t* correction_bs) {
  *scale_bs = (a != nullptr && a->rank == 3 && a->strides[0] != 0) ? a->sizes[1] : 0;
  *correction_bs = (b != nullptr && b->rank == 3 && b->strides[0] != 0) ? b->sizes[1] : 0;
}
}  // namespace

uint64_t vecops_hip_matmul_runtime_quant_workspace(const VecopsHipOperand* a, const VecopsHipOperand* b,
                                                   const VecopsHipOperand* c) {
  RuntimeQuant d{};
  int64_t scale_bs = 0, correction_bs = 0;
  conventional_strides(a, b, &scale_bs, &correction_bs);
  if (describe_runtime_quant(a, b, nullptr, 0, c, scale_bs, correction_bs, reinterpret_cast<void*>(256), &d) != ST_OK) return 0;
  return d.q_bytes + d.row_bytes + d.plan.workspace_bytes;
}

int32_t vecops_hip_matmul_runtime_quant(const VecopsHipOperand* a, const float* multipliers, int32_t zero_point,
                                        const VecopsHipOperand* b, const int32_t* correction, const float* row_scales,
                                        const float* column_scales, const VecopsHipOperand* c, void* workspace,
                                        uint64_t workspace_size, void* stream) {
  if (b == nullptr) return fail(ST_INVALID, "matmul_runtime_quant: null b");
  int64_t scale_bs = 0, correction_bs = 0;
  conventional_strides(a, b, &scale_bs, &correction_bs);
  return run_runtime_quant(a, multipliers, zero_point, scale_bs, b, nullptr, 0, correction, correction_bs, row_scales,
                           column_scales, c, workspace, workspace_size, stream);
}

uint64_t vecops_hip_matmul_runtime_quant_batched_workspace(const VecopsHipOperand* a, int64_t scale_batch_stride,
                                                           const VecopsHipOperand* b, int64_t correction_batch_stride,
                                                           const VecopsHipOperand* c) {
  RuntimeQuant d{};
  if (describe_runtime_quant(a, b, nullptr, 0, c, scale_batch_stride, correction_batch_stride, reinterpret_cast<void*>(256),
                             &d) != ST_OK)
    return 0;
  return d.q_bytes + d.row_bytes + d.plan.workspace_bytes;
}

int32_t vecops_hip_matmul_runtime_quant_batched(const VecopsHipOperand* a, const float* multipliers, int32_t zero_point,
                                                int64_t scale_batch_stride, const VecopsHipOperand* b,
                                                const int32_t* correction, int64_t correction_batch_stride,
                                                const float* row_scales, const float* column_scales,
                                                const VecopsHipOperand* c, void* workspace, uint64_t workspace_size,
                                                void* stream) {
  if (b == nullptr) return fail(ST_INVALID, "matmul_runtime_quant_batched: null b");
  return run_runtime_quant(a, multipliers, zero_point, scale_batch_stride, b, nullptr, 0, correction, correction_batch_stride,
                           row_scales, column_scales, c, workspace, workspace_size, stream);
}

uint64_t vecops_hip_matmul_runtime_quant_packed_b_workspace(const VecopsHipOperand* a, int64_t n, const VecopsHipOperand* c) {
  RuntimeQuant d{};
  int64_t scale_bs = 0, correction_bs = 0;
  conventional_strides(a, nullptr, &scale_bs, &correction_bs);
  if (describe_runtime_quant(a, nullptr, reinterpret_cast<const void*>(256), n, c, scale_bs, 0, reinterpret_cast<void*>(256), &d) != ST_OK)
    return 0;
  return d.q_bytes + d.row_bytes + d.plan.workspace_bytes;
}

int32_t vecops_hip_matmul_runtime_quant_packed_b(const VecopsHipOperand* a, const float* multipliers, int32_t zero_point,
                                                 const void* packed_b, int64_t n, const int32_t* correction,
                                                 const float* row_scales, const float* column_scales,
                                                 const VecopsHipOperand* c, void* workspace, uint64_t workspace_size,
                                                 void* stream) {
  if (packed_b == nullptr && n > 0 && a != nullptr && a->sizes[a->rank - 1] > 0)
    return fail(ST_INVALID, "matmul_runtime_quant_packed_b: null packed b");
  int64_t scale_bs = 0, correction_bs = 0;
  conventional_strides(a, nullptr, &scale_bs, &correction_bs);
  return run_runtime_quant(a, multipliers, zero_point, scale_bs, nullptr, packed_b ? packed_b : reinterpret_cast<const void*>(256),
                           n, correction, 0, row_scales, column_scales, c, workspace, workspace_size, stream);
}

}  // extern "C"

namespace vecops_hip {
// Table set-up of a grouped launch.  The records travel as kernel arguments, so no host buffer has to outlive the call.
__global__ __launch_bounds__(64) void write_groups_kernel(const GroupChunk chunk, int32_t* __restrict__ first,
                                                          TileGemmParams* __restrict__ groups) {
  const int lane = threadIdx.x;
  constexpr int kWords = sizeof(TileGemmParams) / 4;
  for (int g = 0; g < chunk.count; ++g) {
    const uint32_t* src = reinterpret_cast<const uint32_t*>(&chunk.params[g]);
    uint32_t* dst = reinterpret_cast<uint32_t*>(&groups[chunk.offset + g]);
    for (int w = lane; w < kWords; w += 64) dst[w] = src[w];
  }
  if (lane <= chunk.count) first[chunk.offset + lane] = chunk.first[lane];
}

// group_of[w] = the group whose run of workgroups holds w (binary search over first[0 .. groups])
__global__ __launch_bounds__(256) void expand_groups_kernel(const int32_t* __restrict__ first, int32_t groups,
                                                            int32_t* __restrict__ group_of) {
  const int total = first[groups];
  for (int w = blockIdx.x * 256 + threadIdx.x; w < total; w += gridDim.x * 256) {
    int lo = 0, hi = groups - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (first[mid] <= w) lo = mid;
      else hi = mid - 1;
    }
    group_of[w] = lo;
  }
}
}  // namespace vecops_hip

namespace {
// A grouped call: several independent products (irregular batches - every group with its own extents, strides and
// pointers).  bf16 and int8 groups that all multiply run as ONE launch of tile_gemm_grouped_kernel over a table of
// problem records in the workspace (so do f16 groups and fp32 groups, in either compute type, and groups with an
// unsigned 8-bit side, whose row-sum terms are computed group by group into the workspace first); fp64 operands,
// groups of mixed classes, and groups with K = 0, run as launches of their own on the same stream.  So do groups whose K the rule table splits (few output tiles, long K):
// the grouped kernel walks a group's whole K in every workgroup, and two workgroups with 128 K tiles each would
// be what the whole launch waits for (eight products, 255 x 63 x 8191 among them: 99 us in one launch).
struct Grouped {
  std::vector<Problem> problems;
  std::vector<VecopsHipPlan> plans;
  std::vector<int> table_groups;  // indices of the groups served by the one grouped launch
  std::vector<int> split_groups;  // ... and of those that split K: launches of their own
  bool one_launch = false;
  int src = -1, tile = 0, mode = 0;
  std::vector<int32_t> first;     // first workgroup of each table group, and the end
  uint64_t first_bytes = 0, record_bytes = 0, map_bytes = 0, term_bytes = 0, loop_workspace = 0;
  std::vector<uint64_t> term_offset;  // unsigned 8-bit sides: where a table group's row and column terms lie
};

int32_t describe_grouped(uint32_t count, const VecopsHipOperand* a, const VecopsHipOperand* b, const VecopsHipOperand* c_in,
                         const VecopsHipOperand* c, uint32_t compute, Grouped* g) {
  if (count > 0 && (a == nullptr || b == nullptr || c == nullptr)) return fail(ST_INVALID, "matmul_grouped: null operand array");
  if (count > 65536) return fail(ST_INVALID, "matmul_grouped: more than 65536 groups");
  g->problems.resize(count);
  g->plans.resize(count);
  bool same_class = true;
  for (uint32_t i = 0; i < count; ++i) {
    const VecopsHipOperand* cin = (c_in != nullptr && c_in[i].rank != 0) ? &c_in[i] : nullptr;
    // the groups are independent problems: nothing folds across them, each may fold its own batches
    int32_t rc = describe(&a[i], &b[i], cin, &c[i], compute, &g->problems[i]);
    if (rc != ST_OK) return rc;
    choose(g->problems[i], &g->plans[i]);
    const VecopsHipPlan& plan = g->plans[i];
    if (plan.family == VECOPS_HIP_FAMILY_NONE) continue;
    if (plan.workspace_bytes > g->loop_workspace) g->loop_workspace = plan.workspace_bytes;
    if (plan.family == VECOPS_HIP_FAMILY_ZERO_K) continue;
    if (g->src < 0) g->src = g->problems[i].src;
    else if (g->src != g->problems[i].src) same_class = false;
    if (plan.split_k > 1) g->split_groups.push_back(static_cast<int>(i));
    else g->table_groups.push_back(static_cast<int>(i));
  }
  g->one_launch = same_class && g->src != kSrcF64 && g->table_groups.size() > 1;
  if (!g->one_launch) return ST_OK;
  // One workgroup tile for every group: the biggest square tile that still yields two rounds' worth of
  // workgroups over all groups together (priced like the rule table's candidates), else 64 x 64.
  auto tiles = [&](int64_t t) {
    int64_t total = 0;
    for (int i : g->table_groups) {
      const Problem& pr = g->problems[i];
      total += ((pr.m + t - 1) / t) * ((pr.n + t - 1) / t) * pr.batch;
    }
    return total;
  };
  g->tile = 64;
  int64_t best = INT64_MAX;
  const struct { int tile; int64_t quality; } candidates[] = {{256, 1000}, {128, kQuality128}};
  for (const auto& cand : candidates) {
    const int64_t n_tiles = tiles(cand.tile);
    if (n_tiles < kComputeUnits / 2) continue;
    const int64_t rounds = (n_tiles + kComputeUnits - 1) / kComputeUnits;
    int64_t cost = rounds * cand.tile * cand.tile * 1000 / cand.quality;
    if (rounds == 1) cost = cost * (kComputeUnits + n_tiles) / (2 * kComputeUnits);
    if (best == INT64_MAX || cost * 11 < best * 10) {
      best = cost;
      g->tile = cand.tile;
    }
  }
  // the weakest fetch mode any group needs serves them all
  bool all_k = true, all_n = true, all_dma = true;
  for (int i : g->table_groups) {
    const int mode = fetch_mode(g->problems[i], g->plans[i]);
    all_k = all_k && (mode == MODE_KVEC || mode == MODE_KVEC_DMA);
    all_n = all_n && (mode == MODE_NVEC_B || mode == MODE_NVEC_B_DMA);
    all_dma = all_dma && (mode == MODE_KVEC_DMA || mode == MODE_NVEC_B_DMA);
    // (the 256 x 256 tile's written-out K loop walks a [K,N] operand with 32-bit byte offsets)
    if (mode == MODE_NVEC_B_DMA && g->problems[i].k * g->problems[i].b.cs * 2 >= (int64_t{1} << 31)) all_dma = false;
  }
  g->mode = all_k ? (all_dma ? MODE_KVEC_DMA : MODE_KVEC) : all_n ? (all_dma ? MODE_NVEC_B_DMA : MODE_NVEC_B) : MODE_GENERIC;
  int64_t next = 0;
  for (int i : g->table_groups) {
    const Problem& pr = g->problems[i];
    g->first.push_back(static_cast<int32_t>(next));
    const int64_t wgs = ((pr.m + g->tile - 1) / g->tile) * ((pr.n + g->tile - 1) / g->tile) * pr.batch;
    next += (wgs + 7) & ~int64_t{7};  // a multiple of eight: the XCD renumbering then works per group
    if (next > INT32_MAX) return fail(ST_INVALID, "matmul_grouped: too many workgroups");
  }
  g->first.push_back(static_cast<int32_t>(next));
  g->first_bytes = round_up_256(g->first.size() * 4u);
  g->record_bytes = round_up_256(g->table_groups.size() * sizeof(TileGemmParams));
  g->map_bytes = round_up_256(static_cast<uint64_t>(next) * 4u);
  if (g->src == SRC_I8_FLIP) {
    for (int i : g->table_groups) {
      const Problem& pr = g->problems[i];
      g->term_offset.push_back(g->term_bytes);
      g->term_bytes += round_up_256(static_cast<uint64_t>(pr.batch) * (pr.m + pr.n) * 4u);
    }
  }
  return ST_OK;
}

uint64_t grouped_table_bytes(const Grouped& g) {
  return g.one_launch ? g.first_bytes + g.record_bytes + g.map_bytes + g.term_bytes : 0;
}

uint64_t grouped_workspace(const Grouped& g) {
  // the table, and behind it the scratch of the groups that run as launches of their own (one launch at a time, so
  // the largest need serves them all: with a table these are the groups that split K - K = 0 groups need none)
  if (!g.one_launch) return g.loop_workspace;
  uint64_t most = 0;
  for (int i : g.split_groups) most = g.plans[i].workspace_bytes > most ? g.plans[i].workspace_bytes : most;
  return grouped_table_bytes(g) + most;
}
}  // namespace

extern "C" {

uint64_t vecops_hip_matmul_grouped_workspace(uint32_t count, const VecopsHipOperand* a, const VecopsHipOperand* b,
                                             const VecopsHipOperand* c_in, const VecopsHipOperand* c, uint32_t compute) {
  Grouped g;
  if (describe_grouped(count, a, b, c_in, c, compute, &g) != ST_OK) return 0;
  return grouped_workspace(g);
}

int32_t vecops_hip_matmul_grouped(uint32_t count, const VecopsHipOperand* a, const VecopsHipOperand* b,
                                  const VecopsHipOperand* c_in, const VecopsHipOperand* c, uint32_t compute, void* workspace,
                                  uint64_t workspace_size, void* stream) {
  Grouped g;
  int32_t rc = describe_grouped(count, a, b, c_in, c, compute, &g);
  if (rc != ST_OK) return rc;
  const uint64_t need = grouped_workspace(g);
  if (need > workspace_size || (need > 0 && (workspace == nullptr || !aligned16(workspace))))
    return fail(ST_INVALID, "matmul_grouped: %llu bytes of 16-byte aligned workspace required, %llu supplied",
                (unsigned long long)need, (unsigned long long)workspace_size);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (!g.one_launch) {
    for (uint32_t i = 0; i < count; ++i) {
      rc = run_problem(g.problems[i], g.plans[i], nullptr, nullptr, nullptr, workspace, workspace_size, s);
      if (rc != ST_OK) return rc;
    }
    return ST_OK;
  }
  if (int32_t device_rc = check_device(); device_rc != ST_OK) return device_rc;
  // K = 0 groups: c = c_in (or zero), a launch each
  for (uint32_t i = 0; i < count; ++i) {
    if (g.plans[i].family != VECOPS_HIP_FAMILY_ZERO_K) continue;
    rc = run_problem(g.problems[i], g.plans[i], nullptr, nullptr, nullptr, nullptr, 0, s);
    if (rc != ST_OK) return rc;
  }
  char* base = static_cast<char*>(workspace);
  // groups that split K: their own plan, partial sums behind the table
  for (int i : g.split_groups) {
    const uint64_t table = grouped_table_bytes(g);
    rc = run_problem(g.problems[i], g.plans[i], nullptr, nullptr, nullptr, base + table, workspace_size - table, s);
    if (rc != ST_OK) return rc;
  }
  int32_t* first = reinterpret_cast<int32_t*>(base);
  TileGemmParams* records = reinterpret_cast<TileGemmParams*>(base + g.first_bytes);
  int32_t* group_of = reinterpret_cast<int32_t*>(base + g.first_bytes + g.record_bytes);
  const int groups = static_cast<int>(g.table_groups.size());
  const int ktile = k_tile_elements(g.src);
  for (int offset = 0; offset < groups; offset += kGroupChunk) {
    GroupChunk chunk;
    memset(&chunk, 0, sizeof(chunk));
    chunk.offset = offset;
    chunk.count = groups - offset < kGroupChunk ? groups - offset : kGroupChunk;
    for (int j = 0; j < chunk.count; ++j) {
      const Problem& pr = g.problems[g.table_groups[offset + j]];
      if (pr.a.data == nullptr || pr.b.data == nullptr || pr.c.data == nullptr)
        return fail(ST_INVALID, "matmul_grouped: group %d has an operand without storage", g.table_groups[offset + j]);
      TileGemmParams& p = chunk.params[j];
      p = base_params(pr, nullptr, nullptr, nullptr, nullptr);
      if (g.src == SRC_I8_FLIP) {
        char* terms = base + g.first_bytes + g.record_bytes + g.map_bytes + g.term_offset[offset + j];
        rc = unsigned_side_terms(pr, &p, reinterpret_cast<int32_t*>(terms), s);
        if (rc != ST_OK) return rc;
      }
      p.tiles_m = static_cast<int32_t>((pr.m + g.tile - 1) / g.tile);
      p.tiles_n = static_cast<int32_t>((pr.n + g.tile - 1) / g.tile);
      p.split_k = 1;
      p.k_tiles_per_split = static_cast<int32_t>((pr.k + ktile - 1) / ktile);
    }
    for (int j = 0; j <= chunk.count; ++j) chunk.first[j] = g.first[offset + j];
    hipLaunchKernelGGL(write_groups_kernel, dim3(1), dim3(64), 0, s, chunk, first, records);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(ST_EXEC, "group table launch: %s", hipGetErrorString(e));
  }
  const int32_t workgroups = g.first.back();
  int blocks = (workgroups + 255) / 256;
  if (blocks > 1024) blocks = 1024;
  hipLaunchKernelGGL(expand_groups_kernel, dim3(blocks), dim3(256), 0, s, first, groups, group_of);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(ST_EXEC, "group map launch: %s", hipGetErrorString(e));
  GroupedTables t{group_of, first, records, workgroups};
  switch (g.src) {
    case SRC_BF16: e = launch_tile_gemm_grouped_bf16(t, g.tile, g.mode, s); break;
    case SRC_F16: e = launch_tile_gemm_grouped_f16(t, g.tile, g.mode, s); break;
    case SRC_F32_AS_BF16: e = launch_tile_gemm_grouped_f32_as_bf16(t, g.tile, g.mode, s); break;
    case SRC_F32: e = launch_tile_gemm_grouped_f32(t, g.tile, g.mode, s); break;
    case SRC_I8_FLIP: e = launch_tile_gemm_grouped_i8_flip(t, g.tile, g.mode, s); break;
    default: e = launch_tile_gemm_grouped_i8(t, g.tile, g.mode, s); break;
  }
  if (e != hipSuccess) return fail(ST_EXEC, "grouped tile kernel launch: %s", hipGetErrorString(e));
  return ST_OK;
}

uint32_t vecops_hip_abi_version(void) { return VECOPS_HIP_ABI_VERSION; }

const char* vecops_hip_last_error(void) { return g_error; }

int32_t vecops_hip_device_count(void) {
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess) {
    fail(ST_EXEC, "hipGetDeviceCount: %s", hipGetErrorString(e));
    return -1;
  }
  return n;
}

int32_t vecops_hip_plan_matmul(const VecopsHipOperand* a, const VecopsHipOperand* b, const VecopsHipOperand* c_in,
                               const VecopsHipOperand* c, uint32_t compute, VecopsHipPlan* plan) {
  if (plan == nullptr) return fail(ST_INVALID, "plan_matmul: null plan");
  Problem pr{};
  int32_t rc = describe(a, b, c_in, c, compute, &pr);
  if (rc != ST_OK) return rc;
  choose(pr, plan);
  return ST_OK;
}

namespace {
int32_t check_epilogue(const VecopsHipEpilogue* ep) {
  if (ep == nullptr) return fail(ST_INVALID, "matmul_fused: null epilogue");
  if (ep->struct_size < sizeof(VecopsHipEpilogue)) return fail(ST_INVALID, "matmul_fused: epilogue record too short");
  if (ep->activation > VECOPS_HIP_ACT_SILU) return fail(ST_INVALID, "matmul_fused: unknown activation %u", ep->activation);
  return ST_OK;
}
}  // namespace

int32_t vecops_hip_plan_matmul_fused(const VecopsHipOperand* a, const VecopsHipOperand* b, const VecopsHipOperand* c_in,
                                     const VecopsHipOperand* c, uint32_t compute, const VecopsHipEpilogue* epilogue,
                                     VecopsHipPlan* plan) {
  if (plan == nullptr) return fail(ST_INVALID, "plan_matmul_fused: null plan");
  int32_t rc = check_epilogue(epilogue);
  if (rc != ST_OK) return rc;
  Problem pr{};
  rc = describe(a, b, c_in, c, compute, &pr, epilogue);
  if (rc != ST_OK) return rc;
  choose(pr, plan);
  return ST_OK;
}

int32_t vecops_hip_matmul_fused(const VecopsHipOperand* a, const VecopsHipOperand* b, const VecopsHipOperand* c_in,
                                const VecopsHipOperand* c, uint32_t compute, const VecopsHipEpilogue* epilogue,
                                void* workspace, uint64_t workspace_size, void* stream) {
  int32_t rc = check_epilogue(epilogue);
  if (rc != ST_OK) return rc;
  Problem pr{};
  rc = describe(a, b, c_in, c, compute, &pr, epilogue);
  if (rc != ST_OK) return rc;
  VecopsHipPlan plan;
  choose(pr, &plan);
  return run_problem(pr, plan, nullptr, nullptr, nullptr, workspace, workspace_size, static_cast<hipStream_t>(stream));
}

}  // extern "C"

// Scratch of the entry point that takes no workspace (vecops_hip_matmul_static_workspace): device memory owned
// by the library's code object - one copy per GPU, at its own address on each, held until the process ends.
// In host code the array's name is only a handle for hipGetSymbolAddress; kernels and copies get the address
// that call returns.
static __device__ __align__(256) unsigned char scratch[VECOPS_HIP_STATIC_WORKSPACE_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_address[kMaxDevices];

// Address of `scratch` on the current device, looked up once per device.  The kernels of a call go to the caller's
// stream: that stream must belong to the current device (its copy of the array is the one whose address is used).
int32_t static_workspace(hipStream_t stream, void** address) {
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return fail(ST_EXEC, "hipGetDevice: %s", hipGetErrorString(e));
  if (stream != nullptr) {
    int stream_device = -1;
    if (hipStreamGetDevice(stream, &stream_device) == hipSuccess && stream_device != device)
      return fail(ST_INVALID, "matmul_static_workspace: the stream belongs to device %d, the current device is %d",
                  stream_device, device);
  }
  if (device < 0 || device >= kMaxDevices) return fail(ST_EXEC, "device ordinal %d out of range", device);
  void* known = g_scratch_address[device].load(std::memory_order_acquire);
  if (known == nullptr) {
    void* found = nullptr;
    e = hipGetSymbolAddress(&found, HIP_SYMBOL(scratch));
    if (e != hipSuccess || found == nullptr)
      return fail(ST_EXEC, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
    // two host threads may both look it up: they get the same address
    g_scratch_address[device].store(found, std::memory_order_release);
    known = found;
  }
  *address = known;
  return ST_OK;
}
}  // namespace

extern "C" {

uint64_t vecops_hip_static_workspace_bytes(void) { return VECOPS_HIP_STATIC_WORKSPACE_BYTES; }

int32_t vecops_hip_matmul_static_workspace(const VecopsHipOperand* a, const VecopsHipOperand* b,
                                           const VecopsHipOperand* c_in, const VecopsHipOperand* c, uint32_t compute,
                                           void* stream) {
  Problem pr{};
  int32_t rc = describe(a, b, c_in, c, compute, &pr);
  if (rc != ST_OK) return rc;
  VecopsHipPlan plan;
  choose(pr, &plan, VECOPS_HIP_STATIC_WORKSPACE_BYTES);
  // A K split whose partial sums do not fit the buffer is halved until they do (unsplit, a product needs no scratch
  // beyond the row sums of an unsigned operand): the call is then slower than with a caller's workspace, not refused.
  int tile_m = 0, tile_n = 0;
  tile_of_family(plan.family, &tile_m, &tile_n);
  while (tile_m != 0 && plan.peeled_columns == 0 && plan.split_k > 1 && plan.workspace_bytes > VECOPS_HIP_STATIC_WORKSPACE_BYTES)
    finish_tile_plan(pr, &plan, plan.split_k / 2);
  if (plan.workspace_bytes > VECOPS_HIP_STATIC_WORKSPACE_BYTES)
    return fail(ST_NOT_APPLICABLE, "matmul_static_workspace: the call needs %llu bytes of scratch, the library holds %llu",
                (unsigned long long)plan.workspace_bytes, (unsigned long long)VECOPS_HIP_STATIC_WORKSPACE_BYTES);
  void* address = nullptr;
  if (plan.workspace_bytes > 0) {
    rc = static_workspace(static_cast<hipStream_t>(stream), &address);
    if (rc != ST_OK) return rc;
  }
  // Nothing in the scratch has to start at zero: every split writes each of its partial sums before the
  // reduction reads them, and the unsigned-operand terms are written by their own kernels first.
  return run_problem(pr, plan, nullptr, nullptr, nullptr, address, plan.workspace_bytes, static_cast<hipStream_t>(stream));
}

int32_t vecops_hip_plan_matmul_family(const VecopsHipOperand* a, const VecopsHipOperand* b, const VecopsHipOperand* c_in,
                                      const VecopsHipOperand* c, uint32_t compute, const VecopsHipFamilyRequest* request,
                                      VecopsHipPlan* plan) {
  if (plan == nullptr) return fail(ST_INVALID, "plan_matmul_family: null plan");
  Problem pr{};
  int32_t rc = describe(a, b, c_in, c, compute, &pr);
  if (rc != ST_OK) return rc;
  choose(pr, plan);
  return apply_request(pr, request, plan);
}

int32_t vecops_hip_matmul_family(const VecopsHipOperand* a, const VecopsHipOperand* b, const VecopsHipOperand* c_in,
                                 const VecopsHipOperand* c, uint32_t compute, const VecopsHipFamilyRequest* request,
                                 void* workspace, uint64_t workspace_size, void* stream) {
  Problem pr{};
  int32_t rc = describe(a, b, c_in, c, compute, &pr);
  if (rc != ST_OK) return rc;
  VecopsHipPlan plan;
  choose(pr, &plan);
  rc = apply_request(pr, request, &plan);
  if (rc != ST_OK) return rc;
  return run_problem(pr, plan, nullptr, nullptr, nullptr, workspace, workspace_size, static_cast<hipStream_t>(stream));
}

int32_t vecops_hip_matmul(const VecopsHipOperand* a, const VecopsHipOperand* b, const VecopsHipOperand* c_in,
                          const VecopsHipOperand* c, uint32_t compute, void* workspace, uint64_t workspace_size,
                          void* stream) {
  Problem pr{};
  int32_t rc = describe(a, b, c_in, c, compute, &pr);
  if (rc != ST_OK) return rc;
  VecopsHipPlan plan;
  choose(pr, &plan);
  return run_problem(pr, plan, nullptr, nullptr, nullptr, workspace, workspace_size, static_cast<hipStream_t>(stream));
}

int32_t vecops_hip_matmul_planned(const VecopsHipOperand* a, const VecopsHipOperand* b, const VecopsHipOperand* c_in,
                                  const VecopsHipOperand* c, uint32_t compute, const VecopsHipPlan* plan, void* workspace,
                                  uint64_t workspace_size, void* stream) {
  if (plan == nullptr) return fail(ST_INVALID, "matmul_planned: null plan");
  Problem pr{};
  int32_t rc = describe(a, b, c_in, c, compute, &pr);
  if (rc != ST_OK) return rc;
  // What the plan may say is what the planning entries can return for these operands.  Its family and K split go
  // through the same check as a required family (which also recomputes the workspace need); columns are peeled only in
  // the rule table's own plan, so a plan that peels is compared with that - the one case that consults the table.
  VecopsHipPlan checked;
  if (plan->peeled_columns != 0) {
    choose(pr, &checked);
    if (plan->family != checked.family || plan->split_k != checked.split_k || plan->peeled_columns != checked.peeled_columns)
      return fail(ST_INVALID, "matmul_planned: the plan peels %u columns, the rule table's own plan for these operands %u",
                  plan->peeled_columns, checked.peeled_columns);
  } else {
    memset(&checked, 0, sizeof(checked));
    checked.split_k = 1;
    if (pr.batch == 0 || pr.m == 0 || pr.n == 0) {
      checked.family = VECOPS_HIP_FAMILY_NONE;
    } else if (pr.k == 0) {
      checked.family = VECOPS_HIP_FAMILY_ZERO_K;
    } else {
      checked.family = VECOPS_HIP_FAMILY_TILE_64;  // (a stand-in for "some product": the request below decides)
      plan_fetch_flags(pr, &checked);
    }
    if (plan->split_k == 0) return fail(ST_INVALID, "matmul_planned: a finished plan splits K at least one way");
    VecopsHipFamilyRequest request;
    request.struct_size = sizeof(request);
    request.selection = VECOPS_HIP_SELECT_REQUIRE;
    request.family = plan->family;
    request.split_k = plan->split_k;
    if (apply_request(pr, &request, &checked) != ST_OK)
      return fail(ST_INVALID, "matmul_planned: the plan's family %s cannot serve these operands", family_name(plan->family));
    checked.family = plan->family;
    if (checked.split_k != plan->split_k)
      return fail(ST_INVALID, "matmul_planned: the plan splits K %u ways, these operands allow %u", plan->split_k, checked.split_k);
  }
  return run_problem(pr, checked, nullptr, nullptr, nullptr, workspace, workspace_size, static_cast<hipStream_t>(stream));
}

uint64_t vecops_hip_matmul_i8_dequant_workspace(int64_t m, int64_t n, int64_t k) {
  // The plan depends on how the rows lie (16-byte aligned rows take other kernels, and with them other K splits),
  // which this query is not told: the largest need of dense rows, of rows padded to 16 bytes and of rows that are not
  // 16-byte aligned.
  uint64_t most = 0;
  for (const int64_t ld : {k, (k + 15) & ~int64_t{15}, k | 1}) {
    VecopsHipOperand a, b, c;
    make_operand(&a, reinterpret_cast<void*>(16), DT_I8, m, k, ld);
    make_operand(&b, reinterpret_cast<void*>(16), DT_I8, n, k, ld);
    make_operand(&c, reinterpret_cast<void*>(16), DT_I32, m, n, n);
    Problem pr{};
    if (describe(&a, &b, nullptr, &c, 0, &pr) != ST_OK) return 0;
    pr.dequant = true;
    VecopsHipPlan plan;
    choose(pr, &plan);
    most = plan.workspace_bytes > most ? plan.workspace_bytes : most;
  }
  return most;
}

int32_t vecops_hip_matmul_i8_dequant(const int8_t* a, int64_t lda, const int8_t* b, int64_t ldb,
                                     const float* row_scales, const float* column_scales, const int32_t* correction,
                                     float* c, int64_t ldc, int64_t m, int64_t n, int64_t k, void* workspace,
                                     uint64_t workspace_size, void* stream) {
  if (m < 0 || n < 0 || k < 0) return fail(ST_INVALID, "matmul_i8_dequant: negative extent");
  if (m > 0 && n > 0 && (row_scales == nullptr || column_scales == nullptr))
    return fail(ST_INVALID, "matmul_i8_dequant: scales are required");
  VecopsHipOperand oa, ob, oc;
  make_operand(&oa, a, DT_I8, m, k, lda);
  make_operand(&ob, b, DT_I8, n, k, ldb);
  make_operand(&oc, c, DT_I32, m, n, ldc);  // accumulator class; the epilogue writes fp32
  Problem pr{};
  int32_t rc = describe(&oa, &ob, nullptr, &oc, 0, &pr);
  if (rc != ST_OK) return rc;
  pr.dequant = true;
  VecopsHipPlan plan;
  choose(pr, &plan);
  return run_problem(pr, plan, row_scales, column_scales, correction, workspace, workspace_size,
                     static_cast<hipStream_t>(stream));
}

int32_t vecops_hip_matmul_w8a16_group(const void* x, int64_t ldx, const int8_t* w, int64_t ldw, const float* scales,
                                      void* y, int64_t ldy, int64_t m, int64_t n, int64_t k, int64_t group,
                                      void* stream) {
  if (m < 0 || n < 0 || k < 0) return fail(ST_INVALID, "matmul_w8a16_group: negative extent");
  if (m > 16) return fail(ST_NOT_APPLICABLE, "matmul_w8a16_group: m = %lld exceeds 16", (long long)m);
  if (group <= 0 || group % 16 != 0 || k % group != 0)
    return fail(ST_INVALID, "matmul_w8a16_group: group must be a multiple of 16 that divides k");
  if (m == 0 || n == 0) return ST_OK;
  if (x == nullptr || w == nullptr || scales == nullptr || y == nullptr)
    return fail(ST_INVALID, "matmul_w8a16_group: null operand");
  if (!aligned16(x) || !aligned16(w) || ldx % 8 != 0 || ldw % 16 != 0)
    return fail(ST_INVALID, "matmul_w8a16_group: x and w rows must be 16-byte aligned");
  if (n > INT32_MAX || k > INT32_MAX) return fail(ST_INVALID, "matmul_w8a16_group: extent too large");
  SkinnyW8A16Params p;
  p.x = static_cast<const uint16_t*>(x);
  p.w = w;
  p.scales = scales;
  p.y = static_cast<uint16_t*>(y);
  p.ldx = ldx;
  p.ldw = ldw;
  p.ldy = ldy;
  p.m = static_cast<int32_t>(m);
  p.n = static_cast<int32_t>(n);
  p.k = static_cast<int32_t>(k);
  p.group = static_cast<int32_t>(group);
  p.groups = static_cast<int32_t>(k / group);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (int32_t rc = check_device(); rc != ST_OK) return rc;
  // GPU rule table of the skinny family: matrix cores once the widening of a weight
  // byte can be shared by three or more activation rows
  const bool mfma_ok = group % 64 == 0 && (group == 64 || group == 128 || group == 256);
  if (m == 2 && k == 4096 && n >= 4096) {
    // two rows of activations: the streaming walk of M = 1 with both rows resident (13.9 us at N = 14336 where
    // the matrix-core kernel takes 17.0)
    hipLaunchKernelGGL((skinny_w8a16_stream_rows_kernel<2, 4>), dim3(kComputeUnits * kStreamGroupsPerUnit), dim3(256), 0, s, p);
  } else if (m >= 2 && k == 4096 && (group == 128 || group == 256) && n >= 2048 && ldx < (int64_t{1} << 26)) {
    // (the activation rows are fetched through 32-bit byte offsets)
    // activations resident in registers; a workgroup walks two blocks of 32 rows (224 workgroups at
    // N = 14336).  More passes reuse the activations further but leave too few workgroups to pull
    // the bandwidth: 4 passes measured 50 % slower.
    if (group == 128) launch_skinny_mfma_resident<2, 2, 2>(p, s);
    else launch_skinny_mfma_resident<4, 2, 2>(p, s);
  } else if (m >= 3 && mfma_ok) {
    const int tiles = m > 4 ? 2 : 1;  // more weight rows per workgroup = fewer activation reloads
    if (group == 64) { if (tiles == 2) launch_skinny_mfma<1, 2>(p, s); else launch_skinny_mfma<1, 1>(p, s); }
    else if (group == 128) { if (tiles == 2) launch_skinny_mfma<2, 2>(p, s); else launch_skinny_mfma<2, 1>(p, s); }
    else { if (tiles == 2) launch_skinny_mfma<4, 2>(p, s); else launch_skinny_mfma<4, 1>(p, s); }
  } else if (m == 1 && k == 4096 && n >= 4096) {
    // one row of activations against a long matrix: 8 wavefronts per compute unit stream the rows
    // (1, 3, 4 and 6 workgroups per unit measured 14.6, 12.5, 14.2 and 13.4 us against 12.3 for 2 at N = 14336;
    // the one-shot kernel below 13.8)
    hipLaunchKernelGGL((skinny_w8a16_stream_kernel<4>), dim3(kComputeUnits * kStreamGroupsPerUnit), dim3(256), 0, s, p);
  } else if (m == 1) launch_skinny<1, 2, 2>(p, s);
  else if (m == 2) launch_skinny<2, 2, 2>(p, s);
  else if (m <= 4) launch_skinny<4, 2, 1>(p, s);
  else if (m <= 8) launch_skinny<8, 2, 1>(p, s);
  else launch_skinny<16, 1, 1>(p, s);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(ST_EXEC, "skinny kernel launch: %s", hipGetErrorString(e));
  return ST_OK;
}

}  // extern "C"
