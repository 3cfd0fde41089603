"""GPU tests of the prefill projection (ops::Linear::addPrefill, kernels gguf_prefill_*): a chunk of many rows under
the staged rule, against the oracle's staged projection and the 64-row staged tile."""
import numpy as np
import pytest

import splash_amd
from splash_amd import ops
from tests import oracle as orc

pytestmark = pytest.mark.gpu

ALL_FORMATS = [ops.FMT_Q4K, ops.FMT_Q6K, ops.FMT_Q5K, ops.FMT_Q80, ops.FMT_IQ4XS, ops.FMT_IQ4NL]


def run_prefill(backend, parts, K, x_bits, float32=False, residual_bits=None):
    M = x_bits.shape[0]
    proj = ops.Projection.from_native(backend, parts, K, float32=float32)
    N = proj.output_size
    out = backend.allocate_buffer(M * N * (4 if float32 else 2))
    out.fill(0xEE)
    table = backend.allocate_buffer(ops.Linear.prefill_table_bytes(K, M))
    residual = backend.from_array(residual_bits) if residual_bits is not None else None
    graph = splash_amd.CommandGraph()
    ops.Linear.add_prefill(graph, proj, backend.from_array(x_bits), out, table, M, residual=residual)
    backend.run(graph)
    return out.download(np.float32 if float32 else np.uint16).reshape(M, N), len(graph)


def inside(got_f32, want):
    lo, hi = orc.projection_interval(want["exact"], want["bound"])
    return (got_f32 >= lo) & (got_f32 <= hi)


@pytest.mark.parametrize("fmt", ALL_FORMATS)
@pytest.mark.parametrize("M", [1, 100, 128, 300, 1000])
def test_a_chunk_lies_in_the_staged_interval(backend, fmt, M):
    """gguf_projection_test.mm:217-237 with staged = true, at row counts that fill no, one and several 128-row
    workgroups and end inside a 16-row tile, a 64-row piece and a 256-row table pass. The fp32 results lie within the
    accumulation term of the dot over the half-rounded weights, as the staged tile's do."""
    print(f"case prefill fmt={fmt} M={M}", flush=True)
    rng = np.random.default_rng(900 + M)
    N, K = 256, 1024
    native = orc.make_native(fmt, N, K, 80 + M)
    x = orc.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    want = orc.gemm_staged(fmt, native, x, N)
    got, dispatches = run_prefill(backend, [(fmt, N, native)], K, x)
    assert dispatches == (M + 255) // 256 + 1
    ok = inside(orc.bf16_to_f32(got), want)
    assert ok.all(), (int((~ok).sum()), np.argwhere(~ok)[:4])
    got32, _ = run_prefill(backend, [(fmt, N, native)], K, x, float32=True)
    distance = np.abs(got32.astype(np.float64) - want["staged"].astype(np.float64))
    assert np.all(distance <= want["accumulation"] + np.abs(want["staged"]) * 2.0 ** -23), float((distance / want["accumulation"]).max())


def test_a_chunk_of_three_tensors_with_a_residual(backend):
    """A fused projection's tensors, each of its own format, land at their columns; the residual rows are added in fp32."""
    print("case prefill segments", flush=True)
    rng = np.random.default_rng(5)
    K, M = 2048, 200
    parts = [(ops.FMT_Q4K, 256, orc.make_native(ops.FMT_Q4K, 256, K, 1)), (ops.FMT_Q6K, 128, orc.make_native(ops.FMT_Q6K, 128, K, 2)),
             (ops.FMT_Q80, 128, orc.make_native(ops.FMT_Q80, 128, K, 3))]
    x = orc.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    residual = orc.f32_to_bf16(rng.standard_normal((M, 512)).astype(np.float32))
    plain, dispatches = run_prefill(backend, parts, K, x)
    assert dispatches == 1 + 3
    with_residual, _ = run_prefill(backend, parts, K, x, residual_bits=residual)
    at = 0
    for fmt, n, native in parts:
        want = orc.gemm_staged(fmt, native, x, n)
        assert inside(orc.bf16_to_f32(plain[:, at:at + n]), want).all(), fmt
        r = orc.bf16_to_f32(residual[:, at:at + n])
        lo = np.nextafter((want["exact"] - want["bound"]).astype(np.float32), -np.inf) + r
        hi = np.nextafter((want["exact"] + want["bound"]).astype(np.float32), np.inf) + r
        value = orc.bf16_to_f32(with_residual[:, at:at + n])
        assert np.all((value >= orc.bf16_to_f32(orc.f32_to_bf16(lo))) & (value <= orc.bf16_to_f32(orc.f32_to_bf16(hi)))), fmt
        at += n


def test_a_row_does_not_depend_on_its_chunk(backend):
    """Rows are independent: a row carries the same bits alone, in a chunk of 100 and in a chunk of 700, and a re-run
    repeats them."""
    print("case prefill rows", flush=True)
    rng = np.random.default_rng(6)
    N, K = 384, 2048
    native = orc.make_native(ops.FMT_Q4K, N, K, 9)
    x = orc.f32_to_bf16(rng.standard_normal((700, K)).astype(np.float32))
    whole, _ = run_prefill(backend, [(ops.FMT_Q4K, N, native)], K, x, float32=True)
    again, _ = run_prefill(backend, [(ops.FMT_Q4K, N, native)], K, x, float32=True)
    assert whole.tobytes() == again.tobytes()
    for rows in (1, 100, 129):
        part, _ = run_prefill(backend, [(ops.FMT_Q4K, N, native)], K, x[:rows], float32=True)
        assert part.tobytes() == whole[:rows].tobytes()
    # ... and in the 64-row staged tile walking K whole: the same products in the same order
    linear = ops.Linear(backend)
    proj = ops.Projection.from_native(backend, [(ops.FMT_Q4K, N, native)], K, float32=True)
    plan = linear.plan(proj, 64, splits=1, whole_groups=0, staged=True)
    out = backend.allocate_buffer(64 * N * 4)
    graph = splash_amd.CommandGraph()
    linear.add(graph, proj, plan, backend.from_array(x[:64]), out, linear.scratch_for(backend, [plan]))
    backend.run(graph)
    assert out.download(np.float32).reshape(64, N).tobytes() == whole[:64].tobytes()


def test_prefill_rejects_what_it_does_not_take(backend):
    K = 1024
    x = backend.allocate_buffer(64 * K * 2)
    out = backend.allocate_buffer(64 * 192 * 2)
    narrow = ops.Projection.from_native(backend, [(ops.FMT_Q4K, 192, orc.make_native(ops.FMT_Q4K, 192, K, 1))], K)
    graph = splash_amd.CommandGraph()
    with pytest.raises(splash_amd.SplashError):      # 192 columns are not whole 128-column workgroups
        ops.Linear.add_prefill(graph, narrow, x, out, backend.allocate_buffer(ops.Linear.prefill_table_bytes(K, 64)), 64)
    wide = ops.Projection.from_native(backend, [(ops.FMT_Q4K, 256, orc.make_native(ops.FMT_Q4K, 256, K, 1))], K)
    with pytest.raises(splash_amd.SplashError):      # a table of fewer rows
        ops.Linear.add_prefill(graph, wide, x, backend.allocate_buffer(64 * 256 * 2), backend.allocate_buffer(ops.Linear.prefill_table_bytes(K, 16)), 64)
    with pytest.raises(splash_amd.SplashError):      # no rows
        ops.Linear.add_prefill(graph, wide, x, backend.allocate_buffer(64 * 256 * 2), backend.allocate_buffer(ops.Linear.prefill_table_bytes(K, 64)), 0)
    assert len(graph) == 0
