"""Pins the CPU restatement (oracle/vecops_oracle.c) against things it did not
compute itself: closed forms, exact integer arithmetic, the reference's own
known-answer tests, the committed golden vectors and - where it was built - the
real vecops CPU matmul."""
import numpy as np
import pytest

from oracle import oracle as O
from vecops_amd import synth
from conftest import rel_err


# --- scalar conversions ---------------------------------------------------------

def _bf16_nearest_even_via_f64(x: np.ndarray) -> np.ndarray:
    """Independent derivation: pick the nearer of the two neighbouring bf16 values
    in fp64, ties to the even mantissa."""
    bits = x.view(np.uint32).astype(np.uint64)
    lo_bits = (bits & np.uint64(0xFFFF0000)).astype(np.uint32)
    hi_bits = (lo_bits.astype(np.uint64) + np.uint64(0x10000)).astype(np.uint32)  # next magnitude
    lo = lo_bits.view(np.float32).astype(np.float64)
    hi = hi_bits.view(np.float32).astype(np.float64)
    xd = x.astype(np.float64)
    dlo, dhi = np.abs(xd - lo), np.abs(hi - xd)
    lo_even = ((lo_bits >> np.uint32(16)) & np.uint32(1)) == 0
    take_hi = (dhi < dlo) | ((dhi == dlo) & ~lo_even)
    return np.where(take_hi, hi_bits >> np.uint32(16), lo_bits >> np.uint32(16)).astype(np.uint16)


def test_bf16_rounding_matches_nearest_even(oracle):
    rng = np.random.default_rng(0)
    raw = rng.integers(0, 2 ** 32, size=1 << 20, dtype=np.uint64).astype(np.uint32)
    # every exponent with tie / just-below / just-above tie low halves
    exps = np.arange(1, 254, dtype=np.uint32)[:, None] << np.uint32(23)
    lows = np.array([0x0000, 0x7FFF, 0x8000, 0x8001, 0xFFFF, 0x18000, 0x17FFF, 0x28000], dtype=np.uint32)[None, :]
    structured = (exps | lows | np.uint32(0x00010000)).ravel()
    bits = np.concatenate([raw, structured, structured | np.uint32(0x80000000)])
    x = bits.view(np.float32)
    finite = np.isfinite(x) & (np.abs(x) < 3.0e38)  # the rounding may legitimately reach inf above this
    x = np.ascontiguousarray(x[finite])
    assert np.array_equal(oracle.bf16_from_f32(x), _bf16_nearest_even_via_f64(x))
    assert np.array_equal(oracle.bf16_from_f32(x), synth.bf16_round(x))


def test_bf16_special_values(oracle):
    lib = oracle.lib
    assert lib.vo_bf16_from_f32(float("nan")) == 0x7FC0  # util/BFloat16.h:28-29
    assert lib.vo_bf16_from_f32(float("inf")) == 0x7F80
    assert lib.vo_bf16_from_f32(-0.0) == 0x8000
    assert lib.vo_bf16_from_f32(1.0) == 0x3F80
    assert lib.vo_bf16_from_f32(1.00390625) == 0x3F80   # tie to even (down)
    assert lib.vo_bf16_from_f32(1.01171875) == 0x3F82   # tie to even (up)
    assert lib.vo_f32_from_bf16(0x3F80) == 1.0
    assert lib.vo_f32_from_bf16(0xC000) == -2.0


def test_float_to_int_saturates(oracle):
    f = oracle.lib.vo_f32_to_i32_sat  # util/ScalarConvert.h:60-86
    assert f(float("nan")) == 0
    assert f(3.99) == 3 and f(-3.99) == -3
    assert f(3.0e9) == 2 ** 31 - 1 and f(-3.0e9) == -2 ** 31
    assert f(2147483648.0) == 2 ** 31 - 1
    assert f(float("inf")) == 2 ** 31 - 1 and f(float("-inf")) == -2 ** 31


# --- integer matmul ---------------------------------------------------------------

@pytest.mark.parametrize("m,n,k", [(19, 21, 69), (1, 128, 65), (128, 1, 65), (1, 16, 129), (35, 53, 257)])
def test_int8_matches_exact_integer_product(oracle, m, n, k):
    a, b = synth.int8_sym(1, (m, k)), synth.int8_sym(2, (n, k))
    want = (a.astype(np.int64) @ b.astype(np.int64).T).astype(np.int32)
    got = np.zeros((m, n), np.int32)
    oracle.matmul(a, b, got, atom=O.ATOM_I8I32)
    assert np.array_equal(got, want)
    assert np.array_equal(oracle.matmul_i8_dense(a, b), want)


def test_int8_u8_operands(oracle):
    a = (synth.draws(3, 19 * 69) % np.uint64(256)).astype(np.uint8).reshape(19, 69)
    b = synth.int8_sym(4, (21, 69))
    want = (a.astype(np.int64) @ b.astype(np.int64).T).astype(np.int32)
    got = np.zeros((19, 21), np.int32)
    oracle.matmul(a, b, got, atom=O.ATOM_I8I32)
    assert np.array_equal(got, want)


def test_int32_accumulator_wraps(oracle):
    # tests/ops/MatmulTest.cpp:1025-1055: K = 262145 copies of 127*127 wrap mod 2^32
    K = 262145
    a = np.full((1, K), 127, np.int8)
    got = np.zeros((1, 1), np.int32)
    oracle.matmul(a, a, got, atom=O.ATOM_I8I32)
    expected = np.uint32((127 * 127 * K) % 2 ** 32).astype(np.int32)
    assert got[0, 0] == expected and expected < 0
    u = np.full((1, K), 255, np.uint8)
    oracle.matmul(u, u, got, atom=O.ATOM_I8I32)
    assert got[0, 0] == np.uint32((255 * 255 * K) % 2 ** 32).astype(np.int32)
    assert oracle.matmul_i8_dense(a, a)[0, 0] == expected


def test_int32_c_input_accumulates(oracle):
    a, b = synth.int8_sym(1, (7, 33)), synth.int8_sym(2, (9, 33))
    cin = (synth.draws(5, 63) % np.uint64(100000)).astype(np.int32).reshape(7, 9)
    got = np.zeros((7, 9), np.int32)
    oracle.matmul(a, b, got, cin=cin, atom=O.ATOM_I8I32)
    assert np.array_equal(got, (a.astype(np.int64) @ b.astype(np.int64).T + cin).astype(np.int32))


# --- floating matmul ---------------------------------------------------------------

def _modular(count, modulus, as_bf16):
    # tests/ops/MatmulTest.cpp:36-41: (i % modulus - modulus/2) / modulus
    x = ((np.arange(count) % modulus) - modulus // 2).astype(np.float32) / np.float32(modulus)
    return synth.bf16_round(x) if as_bf16 else x


SHAPES = [(16, 16, 35), (16, 32, 67), (16, 48, 79), (1, 48, 79), (32, 16, 33), (48, 16, 65), (32, 32, 97),
          (16, 64, 67), (16, 80, 67), (16, 96, 67), (64, 16, 67), (80, 16, 67), (96, 16, 67), (37, 51, 79),
          (1, 128, 65), (512, 1, 256)]  # tests/ops/MatmulTest.cpp:434-452


@pytest.mark.parametrize("m,n,k", SHAPES)
def test_bf16_matches_fp64_product(oracle, m, n, k):
    a = _modular(m * k, 13, True).reshape(m, k)
    b = _modular(n * k, 11, True).reshape(n, k)
    want = synth.bf16_to_f32(a).astype(np.float64) @ synth.bf16_to_f32(b).astype(np.float64).T
    for acc_f64 in (False, True):
        got = np.zeros((m, n), np.float32)
        oracle.matmul(a, b, got, acc_f64=acc_f64)
        # the reference's own tolerance for this check (MatmulTest.cpp:92) is 2e-4 absolute
        assert np.abs(got - want).max() <= 2.0e-4


def test_fp32_memory_is_rounded_to_bf16_for_the_bf16_atom(oracle):
    m, n, k = 33, 65, 257
    a, b = synth.uniform_pm1(1, (m, k)), synth.uniform_pm1(2, (n, k))
    ar, br = synth.bf16_to_f32(synth.bf16_round(a)), synth.bf16_to_f32(synth.bf16_round(b))
    want = ar.astype(np.float64) @ br.astype(np.float64).T
    got = np.zeros((m, n), np.float32)
    oracle.matmul(a, b, got, atom=O.ATOM_BF16F32, acc_f64=True)
    assert np.array_equal(got, want.astype(np.float32))
    # the fp32 atom must NOT round
    oracle.matmul(a, b, got, atom=O.ATOM_F32F32, acc_f64=True)
    assert np.array_equal(got, (a.astype(np.float64) @ b.astype(np.float64).T).astype(np.float32))
    # bf16 output = RNE of the accumulator
    out = np.zeros((m, n), np.uint16)
    oracle.matmul(a, b, out, atom=O.ATOM_BF16F32, acc_f64=True)
    assert np.array_equal(out, synth.bf16_round(want.astype(np.float32)))


def test_strided_broadcast_and_accumulate_forms(oracle):
    m, n, k, batch = 9, 14, 40, 3
    a = synth.bf16_round(synth.uniform_pm1(1, (batch, m, k)))
    b = synth.bf16_round(synth.uniform_pm1(2, (n, k)))
    bb = np.broadcast_to(b, (batch, n, k))  # stride-0 batch
    cin = synth.uniform_pm1(3, (batch, m, n))
    got = np.zeros((batch, m, n), np.float32)
    oracle.matmul(a, bb, got, cin=cin, acc_f64=True)
    af, bf = synth.bf16_to_f32(a).astype(np.float64), synth.bf16_to_f32(b).astype(np.float64)
    want = np.einsum("bmk,nk->bmn", af, bf) + cin
    assert np.array_equal(got, want.astype(np.float32))
    # B handed over as [K,N] row-major = strided [N,K] view
    b_kn = np.ascontiguousarray(b.T)
    got2 = np.zeros((m, n), np.float32)
    oracle.matmul(a[0], b_kn.T, got2, acc_f64=True)
    assert np.array_equal(got2, (af[0] @ bf.T).astype(np.float32))


def test_zero_extents(oracle):
    a = np.zeros((4, 0), np.uint16)
    b = np.zeros((5, 0), np.uint16)
    c = np.full((4, 5), 3.0, np.float32)
    oracle.matmul(a, b, c)                      # K == 0, single-C form: zeros (ops/Matmul.h:41-43)
    assert np.array_equal(c, np.zeros((4, 5), np.float32))
    cin = np.full((4, 5), 2.5, np.float32)
    oracle.matmul(a, b, c, cin=cin)             # K == 0, explicit C: copy of Cin
    assert np.array_equal(c, cin)
    c0 = np.zeros((0, 5), np.float32)
    oracle.matmul(np.zeros((0, 8), np.uint16), np.zeros((5, 8), np.uint16), c0)  # M == 0: nothing


def test_shape_validation(oracle):
    with pytest.raises(ValueError):
        oracle.matmul(np.zeros((4, 8), np.uint16), np.zeros((5, 9), np.uint16), np.zeros((4, 5), np.float32))
    with pytest.raises(ValueError):
        oracle.matmul(np.zeros((4, 8), np.uint16), np.zeros((5, 8), np.uint16), np.zeros((4, 6), np.float32))


# --- dequantisation epilogue ------------------------------------------------------

def test_dequant_is_two_separate_fp32_multiplies(oracle):
    m, n, k = 67, 129, 515
    a, b = synth.int8_sym(1, (m, k)), synth.int8_sym(2, (n, k))
    rs, cs = synth.scales(3, m), synth.scales(4, n)
    corr = ((synth.draws(5, n) % np.uint64(2001)).astype(np.int64) - 1000).astype(np.int32)
    acc = (a.astype(np.int64) @ b.astype(np.int64).T + corr[None, :]).astype(np.int32)
    want = (acc.astype(np.float32) * rs[:, None]) * cs[None, :]      # matmul/Quantization.h:224-231
    got = oracle.matmul_i8_dequant(a, b, rs, cs, corr)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    fused_wrong_order = acc.astype(np.float32) * (rs[:, None] * cs[None, :])
    assert not np.array_equal(fused_wrong_order.view(np.uint32), want.view(np.uint32))  # the order matters


# --- dispatch predicates ------------------------------------------------------------

def test_dispatch_predicates_known_answers(oracle):
    # tests/matmul/TilerTest.cpp:86-98
    assert oracle.amx_small_vector_profitable(O.SHAPE_AMX_BF16, 1, 16, 65)
    assert not oracle.amx_small_vector_profitable(O.SHAPE_AMX_BF16, 19, 21, 65)
    assert oracle.amx_small_vector_profitable(O.SHAPE_AMX_I8_MIXED, 8, 8, 128)
    assert oracle.sme_small_vector_profitable(O.SHAPE_SME_F16, 1, 16, 17)
    assert not oracle.sme_small_vector_profitable(O.SHAPE_SME_F16, 1, 17, 17)
    assert oracle.amx_residual_split_profitable(17, 33, 1024)
    assert oracle.amx_residual_split_profitable(33, 17, 1024)
    assert not oracle.amx_residual_split_profitable(19, 33, 1024)
    # properties of the rule text (RuntimeDispatch.h:24-83)
    assert not oracle.amx_small_vector_profitable(O.SHAPE_AMX_BF16, 0, 4, 4)
    assert oracle.amx_small_vector_profitable(O.SHAPE_AMX_BF16, 1, 4096, 64)       # large_m1, k % 32 == 0
    assert not oracle.amx_small_vector_profitable(O.SHAPE_AMX_BF16, 1, 4097, 64)   # beyond large_m1
    assert not oracle.amx_small_vector_profitable(O.SHAPE_AMX_BF16, 1, 14336, 4096)  # decode shape -> tiles
    assert not oracle.amx_small_vector_profitable(O.SHAPE_AMX_BF16, 4096, 1, 256)  # large_n1 excludes k == 256
    assert oracle.small_area_profitable(4, 4, 1, 16) and not oracle.small_area_profitable(4, 4, 0, 16)


def test_dispatch_predicates_match_reference(oracle, reference):
    # sweep domain of tests/matmul/TilerTest.cpp:115-134, widened
    for shape in (O.SHAPE_AMX_BF16, O.SHAPE_AMX_I8_SAME, O.SHAPE_AMX_I8_MIXED):
        for m in (0, 1, 2, 8, 16, 19, 64, 65, 128, 4096, 4097):
            for n in (0, 1, 4, 16, 64, 65, 129, 4096, 4097):
                for k in (0, 1, 31, 32, 33, 64, 65, 128, 129, 256, 257, 1024):
                    assert oracle.amx_small_vector_profitable(shape, m, n, k) == \
                        reference.predicate("amx_small_vector_profitable", shape, m, n, k), (shape, m, n, k)
    for m in (17, 18, 19, 20, 33, 47, 48):
        for n in (17, 20, 33, 47, 48, 49):
            for k in (1023, 1024):
                assert oracle.amx_residual_split_profitable(m, n, k) == \
                    reference.predicate("amx_residual_split_profitable", m, n, k)


# --- against the real reference (build container only) ----------------------------------

@pytest.mark.parametrize("m,n,k", SHAPES + [(255, 63, 1023), (130, 70, 513)])
def test_oracle_matches_reference_bf16(oracle, reference, m, n, k):
    a = synth.bf16_round(synth.uniform_pm1(1, (m, k)))
    b = synth.bf16_round(synth.uniform_pm1(2, (n, k)))
    want = np.zeros((m, n), np.float32)
    reference.matmul_bf16_f32(a, b, want)
    got = np.zeros((m, n), np.float32)
    oracle.matmul(a, b, got, acc_f64=True)
    assert rel_err(got, want) <= 2e-6 * max(1, k / 64)  # fp32 accumulation-order noise only
    wb = np.zeros((m, n), np.uint16)
    reference.matmul_bf16_bf16(a, b, wb)
    gb = np.zeros((m, n), np.uint16)
    oracle.matmul(a, b, gb, acc_f64=True)
    assert rel_err(synth.bf16_to_f32(gb), synth.bf16_to_f32(wb)) <= 2 ** -7  # at most one bf16 ulp


def test_oracle_matches_reference_fp32_memory(oracle, reference):
    m, n, k = 33, 65, 257
    a, b = synth.uniform_pm1(1, (m, k)), synth.uniform_pm1(2, (n, k))
    want = np.zeros((m, n), np.float32)
    reference.matmul_f32_f32(a, b, want)
    got = np.zeros((m, n), np.float32)
    oracle.matmul(a, b, got, atom=O.ATOM_BF16F32, acc_f64=True)
    assert rel_err(got, want) <= 1e-5
    true_f32 = np.zeros((m, n), np.float32)
    oracle.matmul(a, b, true_f32, atom=O.ATOM_F32F32, acc_f64=True)
    assert rel_err(true_f32, want) > 1e-4  # the reference really rounded its operands to bf16


def test_oracle_matches_reference_int8_and_dequant(oracle, reference):
    m, n, k = 67, 129, 515
    a, b = synth.int8_sym(1, (m, k)), synth.int8_sym(2, (n, k))
    want = np.zeros((m, n), np.int32)
    reference.matmul_i8_i32(a, b, want)
    assert np.array_equal(oracle.matmul_i8_dense(a, b), want)
    rs, cs = synth.scales(3, m), synth.scales(4, n)
    corr = ((synth.draws(5, n) % np.uint64(2001)).astype(np.int64) - 1000).astype(np.int32)
    for c in (None, corr):
        d_ref = reference.matmul_i8_dequant(a, b, rs, cs, c)
        d_got = oracle.matmul_i8_dequant(a, b, rs, cs, c)
        assert np.array_equal(d_got.view(np.uint32), d_ref.view(np.uint32))
    u = (synth.draws(6, m * k) % np.uint64(256)).astype(np.uint8).reshape(m, k)
    want_u = np.zeros((m, n), np.int32)
    reference.matmul_u8i8_i32(u, b, want_u)
    got_u = np.zeros((m, n), np.int32)
    oracle.matmul(u, b, got_u, atom=O.ATOM_I8I32)
    assert np.array_equal(got_u, want_u)


def test_oracle_matches_reference_views(oracle, reference):
    m, n, k, batch = 19, 21, 35, 3
    # inner stride 2 and padded rows (tests/ops/MatmulTest.cpp:220-279)
    a_store = synth.bf16_round(synth.uniform_pm1(1, (m, 2 * k + 3)))
    b_store = synth.bf16_round(synth.uniform_pm1(2, (n, 2 * k + 5)))
    a, b = a_store[:, 0:2 * k:2], b_store[:, 0:2 * k:2]
    want = np.zeros((m, n), np.float32)
    reference.matmul_bf16_f32(a, b, want)
    got = np.zeros((m, n), np.float32)
    oracle.matmul(a, b, got, acc_f64=True)
    assert rel_err(got, want) <= 2e-6
    # rank 3 with a broadcast B (tests/ops/MatmulBatchTest.cpp:176-335)
    a3 = synth.bf16_round(synth.uniform_pm1(3, (batch, m, k)))
    b3 = np.broadcast_to(synth.bf16_round(synth.uniform_pm1(4, (n, k))), (batch, n, k))
    want3 = np.zeros((batch, m, n), np.float32)
    reference.matmul_bf16_f32_batched(a3, b3, want3)
    got3 = np.zeros((batch, m, n), np.float32)
    oracle.matmul(a3, b3, got3, acc_f64=True)
    assert rel_err(got3, want3) <= 2e-6
    # explicit C input, aliased with the output
    c = synth.uniform_pm1(5, (m, n))
    want_c = c.copy()
    reference.matmul_bf16_f32(a, b, want_c, cin=want_c)
    got_c = c.copy()
    oracle.matmul(a, b, got_c, cin=got_c, acc_f64=True)
    assert rel_err(got_c, want_c) <= 2e-6


# --- IEEE half -------------------------------------------------------------------

def test_f16_rounding_matches_numpy_and_round_trips(oracle):
    """vo_f16_from_f32 against numpy's float32 -> float16 (IEEE round to nearest even), which shares no
    code with it: random bit patterns, every half value's neighbourhood (ties included), the subnormal
    range, the overflow edge; and half -> float -> half is the identity for every non-NaN half."""
    rng = np.random.default_rng(3)
    raw = rng.integers(0, 2 ** 32, size=1 << 20, dtype=np.uint64).astype(np.uint32).view(np.float32)
    halves = np.arange(0, 0x7C00, dtype=np.uint16).view(np.float16).astype(np.float32)
    ulp = np.spacing(halves.view(np.uint32).view(np.float32))
    ties = halves + np.float32(0.5) * np.diff(np.append(halves, np.float32(65536.0)))    # exact midpoints
    near = np.concatenate([halves, ties, np.nextafter(ties, np.float32(0)), np.nextafter(ties, np.float32(1e9))])
    edge = np.array([65503.9, 65504.0, 65519.9, 65520.0, 65536.0, 1e9, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001,
                     2.0 ** -26, 0.0, -0.0], np.float32)
    x = np.concatenate([raw[np.isfinite(raw)], near, -near, edge, -edge]).astype(np.float32)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(oracle.f16_from_f32(x), want)
    every = np.arange(0, 1 << 16, dtype=np.uint16)
    not_nan = ~np.isnan(every.view(np.float16))
    back = oracle.f16_from_f32(every.view(np.float16).astype(np.float32))
    assert np.array_equal(back[not_nan], every[not_nan])
    assert oracle.lib.vo_f32_from_f16(0x3C00) == 1.0 and oracle.lib.vo_f32_from_f16(0x0001) == 2.0 ** -24
    del ulp


def test_f16_atom_matches_fp64_product(oracle):
    """AMX_F16F32 semantics: half operands multiply exactly in fp32; the oracle's fp64-accumulated sums equal a
    numpy float64 product, the output conversion is the half rounding pinned above."""
    rng = np.random.default_rng(4)
    a = rng.uniform(-1, 1, (19, 65)).astype(np.float16)
    b = rng.uniform(-1, 1, (23, 65)).astype(np.float16)
    want = a.astype(np.float64) @ b.astype(np.float64).T
    c = np.zeros((19, 23), np.float32)
    oracle.matmul(a, b, c, atom=O.ATOM_F16F32, acc_f64=True)
    assert np.array_equal(c, want.astype(np.float32))
    ch = np.zeros((19, 23), np.float16)
    oracle.matmul(a, b, ch, atom=O.ATOM_F16F32, acc_f64=True)
    assert np.array_equal(ch.view(np.uint16), want.astype(np.float32).astype(np.float16).view(np.uint16))
    # fp32 memory is rounded to half on the way in
    a32 = rng.uniform(-1, 1, (5, 33)).astype(np.float32)
    b32 = rng.uniform(-1, 1, (7, 33)).astype(np.float32)
    c32 = np.zeros((5, 7), np.float32)
    oracle.matmul(a32, b32, c32, atom=O.ATOM_F16F32, acc_f64=True)
    want32 = a32.astype(np.float16).astype(np.float64) @ b32.astype(np.float16).astype(np.float64).T
    assert np.array_equal(c32, want32.astype(np.float32))


# --- weight-only int8 with per-group scales (no reference counterpart) -----------------

def _w8a16_inputs(seed, m, n, k, group):
    rng = np.random.default_rng(seed)
    x = synth.bf16_to_f32(synth.bf16_round(rng.standard_normal((m, k)).astype(np.float32)))   # bf16-exact fp32
    w = rng.integers(-127, 128, (n, k), dtype=np.int8)
    s = (2.0 ** -7 * (1.0 + rng.random((n, k // group)))).astype(np.float32)
    return x, w, s


@pytest.mark.parametrize("m,n,k,group", [(1, 5, 32, 16), (3, 7, 128, 128), (4, 9, 256, 64), (16, 33, 384, 128),
                                         (2, 1, 512, 256), (5, 6, 48, 16)])
def test_w8a16_group_matches_an_independent_fp64_evaluation(oracle, m, n, k, group):
    """y = sum_g S[n,g] * sum_{k in g} x[m,k] * W[n,k], evaluated by numpy in float64 through an einsum over the
    [groups, group] reshaping - shares no code and no loop structure with the oracle; G = 16, one group and
    N = 1 included.  The bf16 result is the pinned rounding of that float64 sum rounded to fp32."""
    x, w, s = _w8a16_inputs(10 + m, m, n, k, group)
    groups = k // group
    xg = x.astype(np.float64).reshape(m, groups, group)
    wg = w.astype(np.float64).reshape(n, groups, group)
    want = np.einsum("mgk,ngk,ng->mn", xg, wg, s.astype(np.float64))
    y_bits, y64 = oracle.matmul_w8a16_group(synth.bf16_round(x), w, s, group)
    assert np.allclose(y64, want, rtol=1e-13, atol=1e-13)
    assert np.array_equal(y_bits, oracle.bf16_from_f32(y64.astype(np.float32)))


def test_w8a16_group_with_unit_scales_is_the_pinned_plain_product(oracle):
    """All scales 1: the contract reduces to x . W^T, which vo_matmul (pinned by the real reference and by fp64
    products) computes on the weights widened to bf16 (every int8 is a bf16 value)."""
    m, n, k, group = 4, 21, 256, 128
    x, w, _ = _w8a16_inputs(3, m, n, k, group)
    ones = np.ones((n, k // group), np.float32)
    _, y64 = oracle.matmul_w8a16_group(synth.bf16_round(x), w, ones, group)
    want = np.zeros((m, n), np.float32)
    oracle.matmul(x, w.astype(np.float32), want, acc_f64=True)   # fp32 memory -> bf16 compute: exact for int8 values
    assert np.array_equal(y64.astype(np.float32), want)


def test_w8a16_group_scale_of_one_group_moves_exactly_that_groups_dot(oracle):
    """Doubling S[n0, g0] adds S[n0, g0] * (x[:, g0] . W[n0, g0]) to column n0 and nothing anywhere else - fails
    when the scale index (n * groups + g) or a group boundary is off by one."""
    m, n, k, group = 3, 8, 512, 128
    x, w, s = _w8a16_inputs(5, m, n, k, group)
    _, base = oracle.matmul_w8a16_group(synth.bf16_round(x), w, s, group)
    for n0, g0 in [(0, 0), (5, 3), (7, 1)]:
        s2 = s.copy()
        s2[n0, g0] *= 2.0
        _, moved = oracle.matmul_w8a16_group(synth.bf16_round(x), w, s2, group)
        part = np.zeros((m, 1), np.float32)
        oracle.matmul(np.ascontiguousarray(x[:, g0 * group:(g0 + 1) * group]),
                      np.ascontiguousarray(w[n0:n0 + 1, g0 * group:(g0 + 1) * group]).astype(np.float32), part, acc_f64=True)
        want = np.zeros_like(base)
        want[:, n0] = float(s[n0, g0]) * part[:, 0].astype(np.float64)
        # the pinned routine hands the group's dot back rounded to fp32: 2^-24 relative
        assert np.allclose(moved - base, want, rtol=2e-7, atol=1e-9)
        other = np.ones(n, bool)
        other[n0] = False
        assert np.array_equal(moved[:, other], base[:, other])


def test_w8a16_group_known_answer(oracle):
    """Worked by hand.  x[0] = 1 everywhere, x[1] = k % 4 - 1.5 (bf16-exact); W[0] = 1, W[1, k] = k - 16 for K = 32,
    two groups of 16; S = [[0.5, 2], [0.25, -1]].
      row 0 of x: W[0] -> 0.5*16 + 2*16 = 40;  W[1]: group sums -136 and 120 -> 0.25*-136 + -1*120 = -154
      row 1 of x: per 4 elements the pattern sums to 0 against W[0] -> 0; against W[1]: sum over a group of
      (k%4 - 1.5)(k - 16) = sum (k%4 - 1.5) k = 4 blocks * 5 = 20 per group -> 0.25*20 - 20 = -15."""
    k = np.arange(32)
    x = np.stack([np.ones(32), k % 4 - 1.5]).astype(np.float32)
    w = np.stack([np.ones(32), k - 16]).astype(np.int8)
    s = np.array([[0.5, 2.0], [0.25, -1.0]], np.float32)
    y_bits, y64 = oracle.matmul_w8a16_group(synth.bf16_round(x), w, s, 16)
    assert np.array_equal(y64, np.array([[40.0, -154.0], [0.0, -15.0]]))
    assert np.array_equal(y_bits, np.array([[0x4220, 0xC31A], [0x0000, 0xC170]], np.uint16))


def test_w8a16_group_rejects_a_ragged_group(oracle):
    x, w, s = _w8a16_inputs(1, 1, 2, 48, 16)
    with pytest.raises(ValueError):
        oracle.matmul_w8a16_group(synth.bf16_round(x), w, s, 32)


# --- sampled products (the checker of the full-size tests) -----------------------------

@pytest.mark.parametrize("kind", ["bf16_ragged", "f32_memory", "kn_view"])
def test_sampled_product_equals_the_full_product_at_the_sampled_indices(oracle, kind):
    """vo_matmul_sampled(i, j) == vo_matmul(acc_f64)[i, j] (the latter pinned above) on a ragged bf16 case, on
    fp32 memory rounded to bf16 on the way in, and with B handed over as a [K,N] view (strides (1, N))."""
    m, n, k = 37, 45, 131
    a = synth.uniform_pm1(21, (m, k))
    b = synth.uniform_pm1(22, (n, k))
    if kind != "f32_memory":
        a, b = synth.bf16_round(a), synth.bf16_round(b)   # bf16 bits
    if kind == "kn_view":
        b = np.ascontiguousarray(b.T).T   # [N,K] view of a [K,N] array
        assert b.strides == (b.itemsize, b.itemsize * n)
    rng = np.random.default_rng(9)
    rows = np.concatenate([rng.integers(0, m, 200), [0, m - 1, 0, m - 1]])
    cols = np.concatenate([rng.integers(0, n, 200), [0, n - 1, n - 1, 0]])
    got = oracle.matmul_sampled(a, b, rows, cols)
    full = np.zeros((m, n), np.float32)
    oracle.matmul(a, b, full, acc_f64=True)
    assert np.array_equal(got.astype(np.float32), full[rows, cols])
    as_f64 = lambda v: synth.bf16_to_f32(v if v.dtype == np.uint16 else synth.bf16_round(np.ascontiguousarray(v))).astype(np.float64)
    want64 = as_f64(np.ascontiguousarray(a)) @ as_f64(np.ascontiguousarray(b)).T
    assert np.allclose(got, want64[rows, cols], rtol=1e-13, atol=1e-13)


def test_f64_atom_is_the_sequential_fused_sum(oracle):
    """VO_ATOM_F64F64 (vecops' SME_F64F64: fp64 operands and accumulate, one fused multiply-add per k, in k order) pinned
    by the mathematics: an independent Python loop of math.fma-free exact arithmetic on small cases (fractions), the
    reordering bound against numpy's product, exactness on integers, C input, strided views, and the rejection of
    fp64 operands under any other atom."""
    from fractions import Fraction
    from oracle import oracle as O
    m, n, k = 7, 5, 23
    a = (synth.uniform_pm1(1, (m, k)).astype(np.float64) + synth.uniform_pm1(2, (m, k)).astype(np.float64) * 2.0 ** -30)
    b = (synth.uniform_pm1(3, (n, k)).astype(np.float64) + synth.uniform_pm1(4, (n, k)).astype(np.float64) * 2.0 ** -30)
    cin = synth.uniform_pm1(5, (m, n)).astype(np.float64)
    got = np.zeros((m, n), np.float64)
    oracle.matmul(a, b, got, atom=O.ATOM_F64F64)
    # the fused sequential sum, step by step in exact rational arithmetic rounded once per step
    def fused(x, y, acc):
        return float(Fraction(x) * Fraction(y) + Fraction(acc))      # float(Fraction) rounds to nearest even
    for i in range(m):
        for j in range(n):
            acc = 0.0
            for kk in range(k):
                acc = fused(a[i, kk], b[j, kk], acc)
            assert got[i, j] == acc, (i, j)
    # an unfused product-then-add differs on these operands somewhere: the test would notice a dropped fusion
    unfused = np.zeros((m, n))
    for kk in range(k):
        unfused = unfused + a[:, kk:kk + 1] * b[:, kk][None, :]
    assert (unfused != got).any()
    with_c = np.zeros((m, n), np.float64)
    oracle.matmul(a, b, with_c, cin=cin, atom=O.ATOM_F64F64)
    assert np.array_equal(with_c, got + cin)
    # numpy's product: another order of the same sum
    assert (np.abs(got - a @ b.T) <= k * 2.0 ** -52 * (np.abs(a) @ np.abs(b).T)).all()
    # integers: exact whatever the order; views with strides
    ai = (synth.draws(6, 40 * 64) % np.uint64(2 ** 20)).astype(np.float64).reshape(40, 64)
    bi = (synth.draws(7, 30 * 64) % np.uint64(2 ** 20)).astype(np.float64).reshape(30, 64)
    exact = (ai.astype(object) @ bi.astype(object).T).astype(np.float64)
    out = np.zeros((40, 30), np.float64)
    oracle.matmul(ai, bi, out, atom=O.ATOM_F64F64)
    assert np.array_equal(out, exact)
    out_t = np.zeros((30, 40), np.float64)
    oracle.matmul(np.ascontiguousarray(ai.T).T, np.ascontiguousarray(bi.T).T, out_t.T, atom=O.ATOM_F64F64)
    assert np.array_equal(out_t.T, exact)
    with pytest.raises(ValueError):
        oracle.matmul(ai, bi, out)                                      # fp64 operands under the bf16 atom
    with pytest.raises(ValueError):
        oracle.matmul(ai.astype(np.float32), bi.astype(np.float32), out, atom=O.ATOM_F64F64)
