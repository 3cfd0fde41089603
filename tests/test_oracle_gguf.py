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


@pytest.mark.skipif(orc.ref is None, reason="oracle/_ref was not built (no reference tree)")
@pytest.mark.parametrize("fmt", [f for _, f in orc.ALL_FORMATS])
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
