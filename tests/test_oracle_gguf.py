"""The oracle's GGUF functions against the reference's golden vectors and invariants (CPU)."""
import hashlib
import json
import os

import numpy as np
import pytest

from tests import oracle as orc

HERE = os.path.dirname(os.path.abspath(__file__))
GOLDENS = json.load(open(os.path.join(HERE, "golden", "gguf_dequantization.json")))
# gguf_reference_test.mm:23-30: fixture(f, 256, 1024, 7 + f)
ROWS, COLUMNS, SEED = 256, 1024, 7


@pytest.mark.parametrize("name,fmt", orc.ALL_FORMATS)
def test_dequant_matches_ggml_golden_hash(name, fmt):
    native = orc.fixture(fmt, ROWS, COLUMNS, SEED + fmt)
    values = orc.dequant_rows(fmt, native, ROWS, COLUMNS)
    assert hashlib.sha256(values.tobytes()).hexdigest() == GOLDENS[name]


@pytest.mark.parametrize("name,fmt", [("q3k", orc.FMT_Q3K), ("q40", orc.FMT_Q40), ("q50", orc.FMT_Q50)])
def test_dequant_of_the_rewritten_formats_matches_ggml_golden_hash(name, fmt):
    """goldens.json:8,18,22 (dequantize_row_q3_K, _q4_0, _q5_0): the oracle's Q3_K, Q4_0 and Q5_0, which the kernels read
    rewritten as Q6_K and Q8_0 blocks."""
    native = orc.fixture(fmt, ROWS, COLUMNS, SEED + fmt)
    values = orc.dequant_rows(fmt, native, ROWS, COLUMNS)
    assert hashlib.sha256(values.tobytes()).hexdigest() == GOLDENS[name]


@pytest.mark.skipif(orc.ref is None, reason="oracle/_ref was not built (no reference tree)")
@pytest.mark.parametrize("fmt", [f for _, f in orc.ALL_FORMATS] + [orc.FMT_Q3K, orc.FMT_Q40, orc.FMT_Q50])
def test_restatement_equals_compiled_reference(fmt):
    native = orc.fixture(fmt, 64, 1024, 99)
    assert np.array_equal(native, orc.fixture(fmt, 64, 1024, 99, library=orc.ref))
    a = orc.dequant_rows(fmt, native, 64, 1024)
    b = orc.dequant_rows(fmt, native, 64, 1024, library=orc.ref)
    assert a.tobytes() == b.tobytes()
    realistic = orc.make_native(fmt, 32, 512, 5)
    assert np.array_equal(realistic, orc.make_native(fmt, 32, 512, 5, library=orc.ref))


@pytest.mark.skipif(orc.ref is None, reason="oracle/_ref was not built (no reference tree)")
def test_half_conversions_equal_reference():
    rng = np.random.default_rng(1)
    bits = np.concatenate([np.arange(0, 65536, 7, dtype=np.uint32), [0, 1, 0x3FF, 0x400, 0x7BFF, 0x7C00, 0x8000, 0xFC00]])
    orc.ref.ref_h2f.restype = orc.c_f
    orc.ref.ref_f2h.restype = orc.ctypes.c_uint16
    orc.ref.ref_f2h.argtypes = [orc.c_f]
    orc.ref.ref_h2f.argtypes = [orc.ctypes.c_uint16]
    for h in bits:
        a, b = orc.lib.orc_h2f(int(h)), orc.ref.ref_h2f(int(h))
        assert (a == b) or (a != a and b != b)
    floats = np.concatenate([rng.standard_normal(2000).astype(np.float32) * 10.0 ** rng.integers(-9, 6, 2000),
                             np.float32([0, 65504, 65519.99, 65520, 1e-8, 5.96e-8, 2.98e-8, 2.9802322e-8, 6.1e-5, 6.0975e-5])])
    for f in floats:
        assert orc.lib.orc_f2h(float(f)) == orc.ref.ref_f2h(float(f)), f


@pytest.mark.parametrize("fmt,tol", [(orc.FMT_Q4K, 0.08), (orc.FMT_Q6K, 0.02)])
def test_quantizer_round_trip_error(fmt, tol):
    """The K-quantizer is parity-unpinned (llama.cpp's); its round trip must still be a quantizer's."""
    rng = np.random.default_rng(3)
    w = (rng.standard_normal((16, 1024)) * 0.02).astype(np.float32)
    native = orc.quantize_rows(fmt, w)
    back = orc.dequant_rows(fmt, native, 16, 1024)
    rel = np.sqrt(np.mean((back - w) ** 2)) / np.sqrt(np.mean(w ** 2))
    assert rel < tol, rel
    assert np.all(np.isfinite(back))


@pytest.mark.parametrize("fmt", [orc.FMT_Q4K, orc.FMT_Q6K])
def test_register_chain_lies_inside_projection_bound(fmt):
    """The fp32 register rule against the fp64 dot and the reference's projectionBound
    (GgufFormatReference.hpp:739-742); a dropped correction term or a wrong group scale fails it."""
    rng = np.random.default_rng(11)
    N, K, M = 64, 1024, 5
    native = orc.make_native(fmt, N, K, 21)
    x = orc.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    r = orc.gemm(fmt, native, x, N)
    assert np.all(np.abs(r["chain"] - r["exact"]) <= r["bound"])
    # the exact dot equals a numpy fp64 matmul over the dequantized weights
    w = orc.dequant_rows(fmt, native, N, K).astype(np.float64)
    ref = orc.bf16_to_f32(x).astype(np.float64) @ w.T
    assert np.allclose(r["exact"], ref, rtol=1e-12, atol=1e-12)


ALL_FORMATS = [orc.FMT_Q4K, orc.FMT_Q6K, orc.FMT_Q5K, orc.FMT_Q80, orc.FMT_IQ4XS, orc.FMT_IQ4NL]


@pytest.mark.parametrize("fmt", ALL_FORMATS)
def test_staged_projection_is_the_half_rounded_weights_and_the_reference_bound(fmt):
    """orc_gemm_staged against statements of its own parts: its exact dot and its staged value are numpy fp64 products
    over the dequantized weights and over numpy's float16 rounding of them (gguf_staged.h:12-19: each value rounded
    once to half); its bounds are the reference's own dot + projectionBound(staged) and (register tile) on sample
    pairs (a dropped 2^-11 or 2^-25 term, or the accumulation term over sum|x w| instead of sum|x| max|w|, fails)."""
    rng = np.random.default_rng(17 + fmt)
    N, K, M = 48, 1024, 6
    native = orc.make_native(fmt, N, K, 31 + fmt)
    x = orc.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    r = orc.gemm_staged(fmt, native, x, N)
    w = orc.dequant_rows(fmt, native, N, K)
    xf = orc.bf16_to_f32(x).astype(np.float64)
    assert np.allclose(r["exact"], xf @ w.astype(np.float64).T, rtol=1e-12, atol=1e-12)
    w16 = w.astype(np.float16).astype(np.float64)
    assert np.any(w16 != w)     # the rounding is one: these weights are not halves already
    assert np.array_equal(r["staged"], (xf @ w16.T).astype(np.float32))
    # the staged value lies inside the reference's interval, and its distance is of the rounding's size
    assert np.all(np.abs(r["staged"] - r["exact"]) <= r["bound"])
    assert np.all(r["accumulation"] < r["bound"])
    if orc.ref is None:
        pytest.skip("oracle/_ref is not built here")
    f64p = orc.ctypes.POINTER(orc.ctypes.c_double)
    for fn in (orc.ref.ref_dot_bound, orc.ref.ref_dot_bound_staged):
        fn.argtypes = [orc.f32p, orc.f32p, orc.c_u32, f64p, f64p]
        fn.restype = None
    xf32 = orc.bf16_to_f32(x)
    for m, n in [(0, 0), (3, 17), (5, 47), (2, 31)]:
        value, staged_bound, plain_bound = (orc.ctypes.c_double() for _ in range(3))
        xr, wr = np.ascontiguousarray(xf32[m]), np.ascontiguousarray(w[n])
        orc.ref.ref_dot_bound_staged(orc._p(xr, orc.f32p), orc._p(wr, orc.f32p), K, orc.ctypes.byref(value), orc.ctypes.byref(staged_bound))
        orc.ref.ref_dot_bound(orc._p(xr, orc.f32p), orc._p(wr, orc.f32p), K, orc.ctypes.byref(value), orc.ctypes.byref(plain_bound))
        assert value.value == r["exact"][m, n]
        assert staged_bound.value == r["bound"][m, n] and plain_bound.value == r["accumulation"][m, n]


# ---- the column tile's order (orc_gemv_column; kernels/common/gguf_column_tile.h:25-68) ----
def q80_rows(codes, d=1.0):
    """Q8_0 native rows of int8 codes [N][K] under one scale d: a block is the fp16 scale, then 32 codes."""
    codes = np.asarray(codes, dtype=np.int8)
    N, K = codes.shape
    blocks = np.zeros((N, K // 32, 34), dtype=np.uint8)
    blocks[:, :, :2] = np.frombuffer(np.float16(d).tobytes(), dtype=np.uint8)
    blocks[:, :, 2:] = codes.reshape(N, K // 32, 32).view(np.uint8)
    return np.ascontiguousarray(blocks.reshape(N, -1))


def column_total(codes, x, d=1.0):
    x_bits = orc.f32_to_bf16(np.asarray(x, dtype=np.float32)[None, :])
    assert np.array_equal(orc.bf16_to_f32(x_bits)[0], np.asarray(x, dtype=np.float32))   # the inputs are bf16 numbers
    return float(orc.gemv_column(orc.FMT_Q80, q80_rows(np.asarray(codes)[None, :], d), x_bits, 1)[0, 0])


def test_the_column_rule_adds_a_group_in_element_order():
    """Weights 1, one input 2^24 and 31 inputs 1 in a group: added in element order after 2^24 every 1 is lost (a tie
    rounds to the even 2^24); with 2^24 last the ones make 31 first and 2^24 + 31 rounds to 2^24 + 32. A pairwise or
    reversed order gives the other number in each case."""
    K = 256
    ones = np.zeros(K, dtype=np.int8)
    ones[:32] = 1
    x = np.zeros(K, dtype=np.float32)
    x[:32] = 1.0
    x[0] = 2.0 ** 24
    assert column_total(ones, x) == 2.0 ** 24
    x[0], x[31] = 1.0, 2.0 ** 24
    assert column_total(ones, x) == 2.0 ** 24 + 32


def test_the_column_rule_restarts_its_chain_every_group_and_sums_parts_apart():
    """K = 1280: eight parts of five groups, so parts end inside super-blocks. Group 0 sums to 2^24 and each later group of
    its part holds 32 ones: a chain that ran on through the groups would lose every one, a chain a group adds 32 a
    group. Then a one in each group of part 1: added to a sum that ran over all groups each would be lost after 2^24;
    added to their own part's sum they make 5, and (2^24 + 128) + 5 rounds once, to the even 2^24 + 132. Last, 2^24 in
    part 7 after 35 ones in parts 0 to 6: the parts are added from the first, so 35 + 2^24 rounds to 2^24 + 36; with
    2^24 first every part would be lost."""
    K = 1280
    codes = np.ones(K, dtype=np.int8)
    x = np.zeros(K, dtype=np.float32)
    x[0] = 2.0 ** 24          # group 0: the chain holds 2^24 (its other inputs are 0)
    x[32:160] = 1.0           # groups 1..4, the rest of part 0: 32 each
    assert column_total(codes, x) == 2.0 ** 24 + 128
    for g in range(5, 10):    # part 1: a one a group, 5 in all
        x[32 * g] = 1.0
    want = np.float32(np.float32(2.0 ** 24 + 128) + np.float32(5.0))   # one rounding of the parts' sum: ties to even
    assert column_total(codes, x) == float(want) and float(want) == 2.0 ** 24 + 132
    # the eight parts are added in order from the first: a 2^24 in part 7 arrives after everything else
    x = np.zeros(K, dtype=np.float32)
    x[32 * 35] = 2.0 ** 24    # part 7 = groups 35..39
    for g in range(0, 35):
        x[32 * g] = 1.0       # parts 0..6: 5 each, 35 in all, exact
    assert column_total(codes, x) == 2.0 ** 24 + 36   # 35 + 2^24 rounds to even: + 36; 2^24 first would lose every part


def test_the_column_rule_rounds_each_weight_to_half_first():
    """A scale of 1 + 2^-10 and code 3: the fp32 value 3 + 3 * 2^-10 is not a half (their spacing at 3 is 2^-9), and the
    total is the half it rounds to times the input, not the fp32 value times the input."""
    K = 256
    codes = np.zeros(K, dtype=np.int8)
    codes[0] = 3
    x = np.zeros(K, dtype=np.float32)
    x[0] = 1.0
    d = np.float16(1.0 + 2.0 ** -10)                  # a half: the block's scale field is one
    value = np.float32(d) * np.float32(3)              # 3 + 3 * 2^-10: fp32 holds it, a half (spacing 2^-9 at 3) does not
    assert float(np.float16(value)) != float(value)
    assert column_total(codes, x, d=float(d)) == float(np.float16(value))


@pytest.mark.parametrize("name,fmt", orc.ALL_FORMATS)
def test_the_column_rule_lies_in_the_staged_interval(name, fmt):
    """On random weights and rows the totals lie within the reference's bound for a staged projection of the exact dot
    (projectionBound(staged)) and within the accumulation term of the dot over the half-rounded weights."""
    rng = np.random.default_rng(5)
    N, K, M = 48, 1280, 2
    native = orc.make_native(fmt, N, K, 9)
    x = orc.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    got = orc.gemv_column(fmt, native, x, N).astype(np.float64)
    want = orc.gemm_staged(fmt, native, x, N)
    assert np.all(np.abs(got - want["exact"]) <= want["bound"])
    assert np.all(np.abs(got - want["staged"].astype(np.float64)) <= want["accumulation"] + np.abs(want["staged"]) * 2.0 ** -23)
