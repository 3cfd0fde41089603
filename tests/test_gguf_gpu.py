"""GPU parity of the GGUF weight image and the dequant-GEMM against the oracle, through the C ABI."""
import hashlib
import json
import os

import numpy as np
import pytest

import splash_amd
from splash_amd import ops
from tests import oracle as orc

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
GOLDENS = json.load(open(os.path.join(HERE, "golden", "gguf_dequantization.json")))


def dequant_on_gpu(backend, fmt, native, rows, K):
    image = backend.from_array(ops.pack_gguf_image(fmt, native, rows, K), label="image")
    out = backend.allocate_buffer(rows * K * 4, label="values")
    graph = splash_amd.CommandGraph()
    ops.add_dequant(graph, fmt, image, out, rows, K)
    backend.run(graph)
    return out.download(np.float32).reshape(rows, K)


ALL_FORMATS = list(ops.FORMATS)


@pytest.mark.parametrize("name,fmt", orc.ALL_FORMATS)
def test_image_dequantization_matches_ggml_golden_hash(backend, name, fmt):
    """gguf_reference_test.mm:23-30 + gguf_dequant_test.mm:44-58: the kernels' unpacking of the
    re-tiled image gives GGML's fp32 values bit for bit."""
    print(f"case dequant golden {name}", flush=True)
    native = orc.fixture(fmt, 256, 1024, 7 + fmt)
    values = dequant_on_gpu(backend, fmt, native, 256, 1024)
    assert hashlib.sha256(values.tobytes()).hexdigest() == GOLDENS[name]


@pytest.mark.parametrize("fmt", [ops.FMT_Q4K, ops.FMT_Q6K])
def test_image_dequantization_of_quantized_weights(backend, fmt):
    print(f"case dequant quantized fmt={fmt}", flush=True)
    rng = np.random.default_rng(5)
    w = (rng.standard_normal((64, 2048)) * 0.02).astype(np.float32)
    native = orc.quantize_rows(fmt, w)
    values = dequant_on_gpu(backend, fmt, native, 64, 2048)
    assert values.tobytes() == orc.dequant_rows(fmt, native, 64, 2048).tobytes()


def ulp_key(bits):
    """bf16 bit patterns as integers that order like their values."""
    x = np.asarray(bits).astype(np.int32)
    return np.where(x & 0x8000, 0x8000 - x, x)


def run_projection(backend, linear, fmt, native_segments, K, x_bits, epilogue=ops.EPILOGUE_NONE, float32=False,
                   residual_bits=None, gate_native=None, splits=None, whole_groups=None, staged=False):
    M = x_bits.shape[0]
    proj = ops.Projection.from_native(backend, [(fmt, n, nat) for n, nat in native_segments], K, float32=float32)
    gate = ops.Projection.from_native(backend, [(fmt, native_segments[0][0], gate_native)], K) if gate_native is not None else None
    N = proj.output_size
    plan = linear.plan(proj, M, epilogue, splits=splits, whole_groups=whole_groups, staged=staged)
    scratch = linear.scratch_for(backend, [plan])
    x = backend.from_array(x_bits, label="x")
    out = backend.allocate_buffer(M * N * (4 if float32 else 2), label="out")
    res = backend.from_array(residual_bits, label="residual") if residual_bits is not None else None
    graph = splash_amd.CommandGraph()
    linear.add(graph, proj, plan, x, out, scratch, residual=res, gate=gate)
    backend.run(graph)
    got = out.download(np.float32 if float32 else np.uint16).reshape(M, N)
    return got, plan, scratch


def check_interval(got_f32, oracle_result):
    lo, hi = orc.projection_interval(oracle_result["exact"], oracle_result["bound"])
    bad = ~((got_f32 >= lo) & (got_f32 <= hi))
    assert not bad.any(), (int(bad.sum()), got_f32[bad][:4], lo[bad][:4], hi[bad][:4])


@pytest.mark.parametrize("fmt", ALL_FORMATS)
@pytest.mark.parametrize("M", [1, 4, 8, 16, 32, 64])
def test_projection_lies_in_the_reference_interval(backend, fmt, M):
    """gguf_projection_test.mm:217-237: the bf16 result lies in [bf16(lo), bf16(hi)] of the fp64 dot
    +- projectionBound; fp32 logits lie within the bound itself."""
    print(f"case projection fmt={fmt} M={M}", flush=True)
    rng = np.random.default_rng(100 + M)
    N, K = 192, 2048
    native = orc.make_native(fmt, N, K, 40 + M)
    x = orc.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    linear = ops.Linear(backend)
    want = orc.gemm(fmt, native, x, N)
    got, plan, _ = run_projection(backend, linear, fmt, [(N, native)], K, x)
    check_interval(orc.bf16_to_f32(got), want)
    got32, _, _ = run_projection(backend, linear, fmt, [(N, native)], K, x, float32=True)
    assert np.all(np.abs(got32.astype(np.float64) - want["exact"]) <= want["bound"])


@pytest.mark.parametrize("fmt", ALL_FORMATS)
def test_rows_do_not_depend_on_the_block_or_the_partition(backend, fmt):
    """Tested invariants of the reference (gguf_projection_test.mm): a row's result is bitwise the same
    alone or in a taller block, and splits sum in split order so a re-run is bit-identical."""
    print(f"case projection invariants fmt={fmt}", flush=True)
    rng = np.random.default_rng(7)
    N, K = 256, 4096
    native = orc.make_native(fmt, N, K, 3)
    x = orc.f32_to_bf16(rng.standard_normal((32, K)).astype(np.float32))
    linear = ops.Linear(backend)
    full, _, _ = run_projection(backend, linear, fmt, [(N, native)], K, x, float32=True, splits=1, whole_groups=0)
    for rows in (1, 5, 16):
        part, _, _ = run_projection(backend, linear, fmt, [(N, native)], K, x[:rows], float32=True, splits=1, whole_groups=0)
        assert part.tobytes() == full[:rows].tobytes()
    want = orc.gemm(fmt, native, x, N)
    for splits, whole_groups in ((1, 0), (2, 0), (4, 0), (16, 0), (4, 1), (3, 2), (2, 3), (2, 4)):
        a, _, _ = run_projection(backend, linear, fmt, [(N, native)], K, x, float32=True, splits=splits, whole_groups=whole_groups)
        b, _, _ = run_projection(backend, linear, fmt, [(N, native)], K, x, float32=True, splits=splits, whole_groups=whole_groups)
        assert a.tobytes() == b.tobytes()
        assert np.all(np.abs(a.astype(np.float64) - want["exact"]) <= want["bound"])


@pytest.mark.parametrize("fmt", [ops.FMT_Q4K, ops.FMT_Q6K])
@pytest.mark.parametrize("M", [65, 80, 128, 200])
def test_more_rows_than_a_workgroup_takes_run_as_pieces(backend, fmt, M):
    """A dispatch of more than 64 rows (eight lanes of a hybrid step) runs 64-row pieces side by side: every row
    carries the bits it has in a dispatch of its own piece alone, plain, split, with a residual and as a gate/up pair."""
    print(f"case projection pieces fmt={fmt} M={M}", flush=True)
    rng = np.random.default_rng(300 + M)
    N, K = 320, 2048
    native, gate_native = orc.make_native(fmt, N, K, 70), orc.make_native(fmt, N, K, 71)
    x = orc.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    residual = orc.f32_to_bf16(rng.standard_normal((M, N)).astype(np.float32))
    linear = ops.Linear(backend)
    cases = [dict(float32=True, splits=1, whole_groups=0), dict(float32=True, splits=4, whole_groups=0), dict(splits=2, whole_groups=3),
             dict(epilogue=ops.EPILOGUE_RESIDUAL, splits=4, whole_groups=1), dict(epilogue=ops.EPILOGUE_GATE_UP, splits=2, whole_groups=0)]
    for case in cases:
        extra = dict(case)
        if extra.get("epilogue") == ops.EPILOGUE_RESIDUAL:
            extra["residual_bits"] = residual
        if extra.get("epilogue") == ops.EPILOGUE_GATE_UP:
            extra["gate_native"] = gate_native
        whole, _, _ = run_projection(backend, linear, fmt, [(N, native)], K, x, **extra)
        for first in range(0, M, 64):
            rows = slice(first, min(M, first + 64))
            if "residual_bits" in extra:
                extra["residual_bits"] = residual[rows]
            piece, _, _ = run_projection(backend, linear, fmt, [(N, native)], K, x[rows], **extra)
            assert piece.tobytes() == whole[rows].tobytes(), (case, first)
            extra.pop("residual_bits", None)
            if case.get("epilogue") == ops.EPILOGUE_RESIDUAL:
                extra["residual_bits"] = residual
    want = orc.gemm(fmt, native, x, N)
    got, _, _ = run_projection(backend, linear, fmt, [(N, native)], K, x, float32=True)
    assert np.all(np.abs(got.astype(np.float64) - want["exact"]) <= want["bound"])


def test_fused_segments_equal_each_alone(backend):
    """A fused q|k|v dispatch gives each segment the bits it gets alone (LinearGguf.cpp:78-96)."""
    print("case fused segments", flush=True)
    rng = np.random.default_rng(9)
    K, sizes = 1024, (160, 32, 48)
    natives = [orc.make_native(ops.FMT_Q4K, n, K, 60 + i) for i, n in enumerate(sizes)]
    x = orc.f32_to_bf16(rng.standard_normal((16, K)).astype(np.float32))
    linear = ops.Linear(backend)
    fused, _, _ = run_projection(backend, linear, ops.FMT_Q4K, list(zip(sizes, natives)), K, x, splits=1, whole_groups=0)
    at = 0
    for n, native in zip(sizes, natives):
        alone, _, _ = run_projection(backend, linear, ops.FMT_Q4K, [(n, native)], K, x, splits=1, whole_groups=0)
        assert np.array_equal(fused[:, at:at + n], alone)
        at += n


@pytest.mark.parametrize("formats", [(ops.FMT_Q4K, ops.FMT_Q4K, ops.FMT_Q6K), (ops.FMT_Q80, ops.FMT_Q5K, ops.FMT_Q6K), (ops.FMT_IQ4XS, ops.FMT_Q4K, ops.FMT_IQ4NL),
                                     (ops.FMT_Q6K, ops.FMT_Q4K)])
@pytest.mark.parametrize("M", [16, 40, 80])
def test_segments_of_several_formats_equal_each_alone(backend, formats, M):
    """The reference's fused projection takes a format per segment (gguf_linear.metal:237-261): one dispatch gives
    each segment the bits it gets alone under the same partition of K, and the device's own plan stays in the
    reference interval."""
    print(f"case mixed segments formats={formats} M={M}", flush=True)
    rng = np.random.default_rng(19)
    K, sizes = 2048, (256, 64, 128)[:len(formats)]
    natives = [orc.make_native(f, n, K, 70 + i) for i, (f, n) in enumerate(zip(formats, sizes))]
    x = orc.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    linear = ops.Linear(backend)

    def run(segments, **config):
        proj = ops.Projection.from_native(backend, segments, K)
        plan = linear.plan(proj, M, ops.EPILOGUE_NONE, **config)
        out = backend.allocate_buffer(M * proj.output_size * 2)
        graph = splash_amd.CommandGraph()
        linear.add(graph, proj, plan, backend.from_array(x), out, linear.scratch_for(backend, [plan]))
        assert ("mixed" in graph.kernels()[-1]) == (len({f for f, _, _ in segments}) > 1)
        backend.run(graph)
        return out.download(np.uint16).reshape(M, proj.output_size)

    everything = list(zip(formats, sizes, natives))
    for splits in (1, 2, 8):
        fused, at = run(everything, splits=splits, whole_groups=0), 0
        for segment in everything:
            alone = run([segment], splits=splits, whole_groups=0)
            assert np.array_equal(fused[:, at:at + segment[1]], alone), (splits, segment[0])
            at += segment[1]
    fused, at = run(everything), 0
    for f, n, native in everything:
        check_interval(orc.bf16_to_f32(fused[:, at:at + n]), orc.gemm(f, native, x, n))
        at += n
    # whole workgroups a segment, and no epilogue
    with pytest.raises(splash_amd.SplashError):
        run([(formats[0], 32, natives[0][:natives[0].size // sizes[0] * 32]), everything[-1]])


@pytest.mark.parametrize("fmt", ALL_FORMATS)
def test_residual_and_gate_up_epilogues(backend, fmt):
    """gguf_tile.h:10-16, gguf_linear.metal:34-71: bf16(v + res) and bf16(bf16(up) silu(bf16(gate)));
    the one-pass pair equals the two projections' fp32 sums put through the oracle's epilogue."""
    print(f"case epilogues fmt={fmt}", flush=True)
    rng = np.random.default_rng(13)
    N, K, M = 96, 1024, 16
    up_native = orc.make_native(fmt, N, K, 70)
    gate_native = orc.make_native(fmt, N, K, 71)
    x = orc.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    res = orc.f32_to_bf16(rng.standard_normal((M, N)).astype(np.float32))
    linear = ops.Linear(backend)
    kw = dict(splits=2, whole_groups=1)
    up32, _, _ = run_projection(backend, linear, fmt, [(N, up_native)], K, x, float32=True, **kw)
    gate32, _, _ = run_projection(backend, linear, fmt, [(N, gate_native)], K, x, float32=True, **kw)
    got, _, _ = run_projection(backend, linear, fmt, [(N, up_native)], K, x, epilogue=ops.EPILOGUE_RESIDUAL,
                               residual_bits=res, **kw)
    want = orc.f32_to_bf16(up32 + orc.bf16_to_f32(res))
    assert np.array_equal(got, want)
    pair, _, _ = run_projection(backend, linear, fmt, [(N, up_native)], K, x, epilogue=ops.EPILOGUE_GATE_UP,
                                gate_native=gate_native, **kw)
    want = orc.swiglu(gate32, up32)
    # exp2 differs in its last bits between the CPU and the GPU: allow one bf16 step on a few values
    diff = np.abs(pair.astype(np.int32) - want.astype(np.int32))
    assert diff.max() <= 1 and (diff > 0).mean() < 0.02, (diff.max(), (diff > 0).mean())


@pytest.mark.parametrize("M", [16, 5, 40])
def test_gate_up_table_epilogue_equals_the_table_pass(backend, M):
    """The one-pass gate/up may write the down projection's activation table from its epilogue: table,
    intermediate rows and the block's output are bit-identical to the path with a separate table pass,
    and the table is the one the rows define."""
    print(f"case swiglu table epilogue M={M}", flush=True)
    rng = np.random.default_rng(31 + M)
    hidden, ffn = 1024, 768
    linear = ops.Linear(backend)
    gate = ops.Projection.from_native(backend, [(ops.FMT_Q4K, ffn, orc.make_native(ops.FMT_Q4K, ffn, hidden, 5))], hidden)
    up = ops.Projection.from_native(backend, [(ops.FMT_Q4K, ffn, orc.make_native(ops.FMT_Q4K, ffn, hidden, 6))], hidden)
    down = ops.Projection.from_native(backend, [(ops.FMT_Q6K, hidden, orc.make_native(ops.FMT_Q6K, hidden, ffn, 7))], ffn)
    x = backend.from_array(orc.f32_to_bf16(rng.standard_normal((M, hidden)).astype(np.float32)))
    res = backend.from_array(orc.f32_to_bf16(rng.standard_normal((M, hidden)).astype(np.float32)))
    tiles = (M + 15) // 16
    results = []
    for fused in (False, True):
        sizes = [linear.scratch_size(ffn, hidden, M), linear.scratch_size(hidden, ffn, M)]
        scratch = ops.LinearScratch(backend, *[max(s[i] for s in sizes) for i in range(3)])
        table2 = backend.allocate_buffer(ops.gguf_table_bytes(ffn, M)) if fused else None
        mid = backend.allocate_buffer(M * ffn * 2)
        out = backend.allocate_buffer(M * hidden * 2)
        graph = splash_amd.CommandGraph()
        linear.add_swiglu(graph, gate, up, down, x, mid, res, out, M, scratch, next_table=table2)
        assert len(graph) == (3 if fused else 4)
        backend.run(graph)
        table = (table2 if fused else scratch.table).download(np.uint8)[:ops.gguf_table_bytes(ffn, M)]
        results.append((mid.download(np.uint16).reshape(M, ffn), out.download(np.uint16), table))
    assert np.array_equal(results[0][0], results[1][0])
    assert np.array_equal(results[0][1], results[1][1])
    for mid, _, table in results:
        values, s32, s16 = orc.split_activation_table(table, ffn, tiles)
        wv, w32, w16 = orc.activation_table(mid)
        assert np.array_equal(values, wv)
        assert s32.tobytes() == w32.tobytes() and s16.tobytes() == w16.tobytes()


@pytest.mark.parametrize("fmt,N,K,M,config", [(ops.FMT_Q4K, 5120, 8192, 16, None), (ops.FMT_Q6K, 5120, 5120, 16, None),
                                              (ops.FMT_Q4K, 1024, 2048, 5, (1, 0)), (ops.FMT_Q4K, 1024, 2048, 40, (4, 3)),
                                              (ops.FMT_Q6K, 768, 1024, 64, (2, 0)), (ops.FMT_Q4K, 512, 1024, 100, None)])
def test_residual_norm_epilogue(backend, fmt, N, K, M, config):
    """A residual projection may also leave its rows as the activation table of the projection after their RMS
    norm. Its output rows are bit-identical to the plain residual projection's; the table is bit for bit the
    table of bf16(output * weight) (an exact fp32 product, rounded once) and ends with every 64-column group's
    sums of squares of the output rows. The projection that reads the table as one that lacks its scale gives the
    oracle's projection of those table rows times each row's inverse RMS, to the oracle's own error bound; against
    the norm pass's rounding (bf16(output * inverse RMS * weight)) it differs by that one operand rounding."""
    print(f"case residual norm epilogue fmt={fmt} N={N} K={K} M={M} config={config}", flush=True)
    rng = np.random.default_rng(N + M)
    linear = ops.Linear(backend)
    native = orc.make_native(fmt, N, K, 9)
    proj = ops.Projection.from_native(backend, [(fmt, N, native)], K)
    x = backend.from_array(orc.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32)))
    residual_bits = orc.f32_to_bf16(rng.standard_normal((M, N)).astype(np.float32))
    weight_bits = orc.f32_to_bf16((1 + 0.1 * rng.standard_normal(N)).astype(np.float32))
    residual, weight = backend.from_array(residual_bits), backend.from_array(weight_bits)
    kwargs = dict(splits=config[0], whole_groups=config[1]) if config else {}
    plain_plan = linear.plan(proj, M, ops.EPILOGUE_RESIDUAL, **kwargs)
    plan = linear.plan(proj, M, ops.EPILOGUE_RESIDUAL_NORM, **kwargs)
    assert (plan.splits, plan.whole_groups) == (plain_plan.splits, plain_plan.whole_groups)
    # the projection after the norm: N inputs, 256 fp32 outputs
    N2 = 256
    native2 = orc.make_native(ops.FMT_Q4K, N2, N, 5)
    proj2 = ops.Projection.from_native(backend, [(ops.FMT_Q4K, N2, native2)], N, float32=True)
    plan2 = linear.plan(proj2, M)
    scratch = linear.scratch_for(backend, [plan, plain_plan, plan2])
    out_plain, out = backend.allocate_buffer(M * N * 2), backend.allocate_buffer(M * N * 2)
    table_bytes = ops.gguf_table_bytes(N, M)
    next_scratch = ops.LinearScratch(backend, table_bytes)
    next_scratch.partials, next_scratch.counters = scratch.partials, scratch.counters
    after = backend.allocate_buffer(M * N2 * 4)
    normalized = backend.allocate_buffer(M * N * 2)   # stands for the rows the table holds; never read
    graph = splash_amd.CommandGraph()
    linear.add(graph, proj, plain_plan, x, out_plain, scratch, residual=residual)
    backend.run(graph)
    graph = splash_amd.CommandGraph()
    linear.add(graph, proj, plan, x, out, scratch, residual=residual, norm_weight=weight, next_table=next_scratch.table)
    assert len(graph) == 2          # the table pass of its own input, then the projection
    linear.add(graph, proj2, plan2, normalized, after, next_scratch, prepared=ops.PREPARED_UNSCALED)
    assert len(graph) == 3          # no table pass: the table is there
    backend.run(graph)
    hidden = out.download(np.uint16).reshape(M, N)
    assert np.array_equal(hidden, out_plain.download(np.uint16).reshape(M, N))
    raw = next_scratch.table.download(np.uint8)[:table_bytes].copy()
    # pieces of 64 rows, each with a table of its own
    scaled = orc.f32_to_bf16(orc.bf16_to_f32(hidden) * orc.bf16_to_f32(weight_bits)[None, :])
    inverse = np.empty(M)
    at = 0
    for first in range(0, M, 64):
        rows = min(64, M - first)
        tiles = (rows + 15) // 16
        size = ops.gguf_table_bytes(N, rows)
        piece = raw[at:at + size]
        at += size
        values, s32, s16 = orc.split_activation_table(piece, N, tiles)
        wv, w32, w16 = orc.activation_table(scaled[first:first + rows])
        assert np.array_equal(values, wv)
        assert s32.tobytes() == w32.tobytes() and s16.tobytes() == w16.tobytes()
        stride = max(16 * tiles, 32)     # floats an entry: whole 128-byte lines
        squares = piece[size - (N // 64) * stride * 4:].view(np.float32).reshape(N // 64, stride)[:, :16 * tiles]
        h = orc.bf16_to_f32(hidden[first:first + rows]).astype(np.float64)
        want = (h.reshape(rows, N // 64, 64) ** 2).sum(axis=2).T
        assert np.allclose(squares[:, :rows], want, rtol=1e-5, atol=0)
        assert not squares[:, rows:].any()
        inverse[first:first + rows] = 1.0 / np.sqrt(want.sum(axis=0) / N + 1e-6)
    assert at == table_bytes
    got = after.download(np.float32).reshape(M, N2)
    res = orc.gemm(ops.FMT_Q4K, native2, scaled, N2, want=("exact", "bound"))
    error = np.abs(got - res["exact"] * inverse[:, None])
    assert (error <= res["bound"] * inverse[:, None] * 1.01 + 1e-5 * np.abs(got)).all(), error.max()
    # against the rounding points of a norm pass before the projection
    normed = orc.rms_norm(hidden, weight_bits)
    reference = orc.gemm(ops.FMT_Q4K, native2, normed, N2, want=("exact",))["exact"]
    assert np.abs(got - reference).max() <= 2e-2 * np.sqrt((reference ** 2).mean())
    cosine = (got * reference).sum() / np.sqrt((got ** 2).sum() * (reference ** 2).sum())
    assert cosine >= 0.99999
    # a second run repeats the table bit for bit
    backend.run(graph)
    assert np.array_equal(next_scratch.table.download(np.uint8)[:table_bytes], raw)
    assert np.array_equal(after.download(np.float32).reshape(M, N2), got)
    with pytest.raises(ValueError, match="next projection table"):
        linear.add(splash_amd.CommandGraph(), proj, plan, x, out, scratch, residual=residual, norm_weight=weight)


def test_linear_rejects_bad_buffers_before_adding_anything(backend):
    """Operators throw std::invalid_argument before any dispatch is added (LinearGguf.cpp:126-163)."""
    native = orc.make_native(ops.FMT_Q4K, 32, 512, 1)
    proj = ops.Projection.from_native(backend, [(ops.FMT_Q4K, 32, native)], 512)
    linear = ops.Linear(backend)
    plan = linear.plan(proj, 16)
    scratch = linear.scratch_for(backend, [plan])
    x = backend.allocate_buffer(16 * 512 * 2)
    small = backend.allocate_buffer(16)
    graph = splash_amd.CommandGraph()
    with pytest.raises(ValueError, match="too small"):
        linear.add(graph, proj, plan, x, small, scratch)
    with pytest.raises(ValueError, match="too small"):
        linear.add(graph, proj, plan, small, x, scratch)
    with pytest.raises(ValueError):
        linear.plan(proj, 257)
    with pytest.raises(ValueError):
        linear.plan(proj, 16, splits=3)
    assert len(graph) == 0


def test_backend_one_command_in_flight_and_unknown_kernel(backend):
    """MetalBackend.hpp:474-476: a second command is refused until the first ticket is consumed."""
    import ctypes
    a = backend.allocate_buffer(4096)
    graph = splash_amd.CommandGraph()

    class P(ctypes.Structure):
        _fields_ = [("x", ctypes.c_uint32)]
    graph.add("no_such_kernel", [a], P(1), (1, 1, 1))
    with pytest.raises(ValueError, match="no kernel"):
        backend.submit_command_async(graph)
    native = orc.make_native(ops.FMT_Q4K, 16, 256, 1)
    image = backend.from_array(ops.pack_gguf_image(ops.FMT_Q4K, native, 16, 256))
    out = backend.allocate_buffer(16 * 256 * 4)
    g2 = splash_amd.CommandGraph()
    ops.add_dequant(g2, ops.FMT_Q4K, image, out, 16, 256)
    t1 = backend.submit_command_async(g2)
    with pytest.raises(splash_amd.SplashError) as e:
        backend.submit_command_async(g2)
    assert e.value.status == 4  # SP_BUSY
    gpu, wall = t1.wait()
    assert gpu >= 0 and wall > 0 and backend.healthy() and not backend.command_in_flight()
    # a recorded command replays to the same bytes
    first = out.download(np.float32).copy()
    out.fill(0)
    rec = backend.record(g2)
    rec.submit().wait()
    assert np.array_equal(out.download(np.float32), first)


@pytest.mark.parametrize("name,fmt,widths,K", [("gate_up", ops.FMT_Q4K, (25600,), 5120), ("fused_qkv", ops.FMT_Q4K, (5120, 1024, 1024), 5120),
                                               ("down", ops.FMT_Q6K, (5120,), 25600)])
def test_config2_projections_at_full_size(backend, name, fmt, widths, K):
    """BASELINE.json config 2's shapes (K 5120 with N 25600 and the fused 5120 + 2 x 1024; the down projection K 25600,
    N 5120 in Q6_K) at M = 1, 4, 8, 16, 32 rows, through properties that do not need the oracle over the whole matrix:
    a sample of columns lies in the reference interval of the fp64 dot (gguf_projection_test.mm:217-237); doubling the
    input doubles every fp32 output bit for bit; and a row's result is the same in a block of any height."""
    print(f"case config 2 full size {name}", flush=True)
    rng = np.random.default_rng(len(name))
    natives = [orc.make_native(fmt, n, K, 900 + i) for i, n in enumerate(widths)]
    N = sum(widths)
    proj = ops.Projection.from_native(backend, [(fmt, n, native) for n, native in zip(widths, natives)], K, float32=True)
    linear = ops.Linear(backend)
    x = orc.f32_to_bf16(rng.standard_normal((32, K)).astype(np.float32))
    row_bytes = natives[0].size // widths[0]
    sample = np.sort(rng.choice(widths[0], 48, replace=False))
    sampled_native = np.concatenate([natives[0][c * row_bytes:(c + 1) * row_bytes] for c in sample])
    want = orc.gemm(fmt, sampled_native, x, len(sample), want=("exact", "bound"))

    def run(rows_bits, plan):
        out = backend.allocate_buffer(rows_bits.shape[0] * N * 4)
        graph = splash_amd.CommandGraph()
        linear.add(graph, proj, plan, backend.from_array(rows_bits), out, linear.scratch_for(backend, [plan]))
        backend.run(graph)
        return out.download(np.float32).reshape(rows_bits.shape[0], N)
    tallest = linear.plan(proj, 32, ops.EPILOGUE_NONE)
    full = run(x, tallest)
    for M in (1, 4, 8, 16, 32):
        got = run(x[:M], linear.plan(proj, M, ops.EPILOGUE_NONE))
        assert np.all(np.abs(got[:, sample].astype(np.float64) - want["exact"][:M]) <= want["bound"][:M]), M
        assert np.isfinite(got).all()
        # the same partition of K as the tallest block's: the rows are its rows, bit for bit
        same = linear.plan(proj, M, ops.EPILOGUE_NONE, splits=tallest.splits, whole_groups=tallest.whole_groups)
        if same.storage_rows == tallest.storage_rows:
            assert run(x[:M], same).tobytes() == full[:M].tobytes(), M
    doubled = orc.f32_to_bf16(2 * orc.bf16_to_f32(x[:16]))
    plan = linear.plan(proj, 16, ops.EPILOGUE_NONE)
    assert (2 * run(x[:16], plan)).tobytes() == run(doubled, plan).tobytes()


@pytest.mark.parametrize("fmt", ALL_FORMATS)
@pytest.mark.parametrize("M", [1, 16, 40, 64, 100])
def test_the_staged_rule_rounds_each_weight_once_to_half(backend, fmt, M):
    """The staged tile (kernels/common/gguf_staged.h:12-66; gguf_projection_test.mm:217-237 with staged = true): the
    bf16 result lies in [bf16(lo), bf16(hi)] of the fp64 dot +- projectionBound(staged). The fp32 result, beyond that,
    lies within the accumulation term alone (2^-16 sum|x| max|w|) of the fp64 dot over the HALF-ROUNDED weights, which
    the same products over unrounded weights miss (the two dots differ by up to 2^-11 sum|x w|): the weights are halves.
    With a residual; bit-identical re-runs over K partitions."""
    print(f"case staged projection fmt={fmt} M={M}", flush=True)
    rng = np.random.default_rng(500 + M)
    N, K = 192, 2048
    native = orc.make_native(fmt, N, K, 60 + M)
    x = orc.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    linear = ops.Linear(backend)
    want = orc.gemm_staged(fmt, native, x, N)
    got, plan, _ = run_projection(backend, linear, fmt, [(N, native)], K, x, staged=True)
    assert plan.tile == 1
    check_interval(orc.bf16_to_f32(got), want)
    got32, _, _ = run_projection(backend, linear, fmt, [(N, native)], K, x, float32=True, staged=True)
    distance = np.abs(got32.astype(np.float64) - want["staged"].astype(np.float64))
    assert np.all(distance <= want["accumulation"] + np.abs(want["staged"]) * 2.0 ** -23), float((distance / want["accumulation"]).max())
    # ... and the unrounded weights' dot is further away than that for most outputs: the test tells the two apart
    assert np.mean(np.abs(want["exact"] - want["staged"]) > 2 * distance) > 0.5
    residual = orc.f32_to_bf16(rng.standard_normal((M, N)).astype(np.float32))
    with_residual, _, _ = run_projection(backend, linear, fmt, [(N, native)], K, x, epilogue=ops.EPILOGUE_RESIDUAL, residual_bits=residual,
                                         staged=True)
    # gguf_projection_test.mm:242-245: fl(p + r) is monotonic, so the sum's interval is the rounded sums of the ends
    r = orc.bf16_to_f32(residual)
    lo = np.nextafter((want["exact"] - want["bound"]).astype(np.float32), -np.inf) + r
    hi = np.nextafter((want["exact"] + want["bound"]).astype(np.float32), np.inf) + r
    value = orc.bf16_to_f32(with_residual)
    assert np.all((value >= orc.bf16_to_f32(orc.f32_to_bf16(lo))) & (value <= orc.bf16_to_f32(orc.f32_to_bf16(hi))))
    for splits in (1, 2, 8):
        a, _, _ = run_projection(backend, linear, fmt, [(N, native)], K, x, float32=True, splits=splits, whole_groups=0, staged=True)
        b, _, _ = run_projection(backend, linear, fmt, [(N, native)], K, x, float32=True, splits=splits, whole_groups=0, staged=True)
        assert a.tobytes() == b.tobytes()
        assert np.all(np.abs(a.astype(np.float64) - want["exact"]) <= want["bound"])


def test_the_staged_rule_takes_plain_and_residual_plans_of_one_format(backend):
    linear = ops.Linear(backend)
    K = 1024
    one = ops.Projection.from_native(backend, [(ops.FMT_Q4K, 128, orc.make_native(ops.FMT_Q4K, 128, K, 1))], K)
    with pytest.raises(splash_amd.SplashError):
        linear.plan(one, 16, ops.EPILOGUE_GATE_UP, staged=True)
    with pytest.raises(splash_amd.SplashError):
        linear.plan(one, 16, ops.EPILOGUE_RESIDUAL_NORM, staged=True)
    mixed = ops.Projection.from_native(backend, [(ops.FMT_Q4K, 64, orc.make_native(ops.FMT_Q4K, 64, K, 2)),
                                                 (ops.FMT_Q6K, 64, orc.make_native(ops.FMT_Q6K, 64, K, 3))], K)
    with pytest.raises(splash_amd.SplashError):
        linear.plan(mixed, 16, staged=True)


def run_column(backend, linear, segments, K, x_bits, epilogue=ops.EPILOGUE_NONE, float32=False, residual_bits=None, gate=None):
    """segments: (format, columns, native rows) of the projection's tensors. The column tile reads the rows as they are."""
    M = x_bits.shape[0]
    proj = ops.Projection.from_native(backend, segments, K, float32=float32)
    gate_proj = ops.Projection.from_native(backend, [gate], K) if gate is not None else None
    N = proj.output_size
    plan = linear.plan(proj, M, epilogue, column=True)
    assert plan.tile == 2 and plan.splits == 1
    scratch = linear.scratch_for(backend, [plan])
    out = backend.allocate_buffer(M * N * (4 if float32 else 2), label="out")
    out.fill(0xEE)
    res = backend.from_array(residual_bits, label="residual") if residual_bits is not None else None
    graph = splash_amd.CommandGraph()
    linear.add(graph, proj, plan, backend.from_array(x_bits, label="x"), out, scratch, residual=res, gate=gate_proj)
    assert len(graph) == len(segments)      # a dispatch a tensor and no table pass
    backend.run(graph)
    return out.download(np.float32 if float32 else np.uint16).reshape(M, N)


@pytest.mark.parametrize("fmt", ALL_FORMATS)
@pytest.mark.parametrize("M,K", [(1, 1280), (2, 2048), (2, 5120), (1, 256)])
def test_the_column_tile_adds_in_the_reference_order(backend, fmt, M, K):
    """linear_gguf_column.metal:33-66 and gguf_column_tile.h:25-68 fix every addition of a column's sum, so the fp32
    totals are the oracle's bit for bit (K = 1280 and 256: parts that end inside a super-block, parts of less than a
    group's worth), and the epilogues those of the tiles on them."""
    print(f"case column tile fmt={fmt} M={M} K={K}", flush=True)
    rng = np.random.default_rng(K + M)
    N = 80
    native = orc.make_native(fmt, N, K, 17 + M)
    x = orc.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    linear = ops.Linear(backend)
    want = orc.gemv_column(fmt, native, x, N)
    got32 = run_column(backend, linear, [(fmt, N, native)], K, x, float32=True)
    assert got32.tobytes() == want.tobytes(), int((got32 != want).sum())
    got = run_column(backend, linear, [(fmt, N, native)], K, x)
    assert np.array_equal(got, orc.f32_to_bf16(want))
    res = orc.f32_to_bf16(rng.standard_normal((M, N)).astype(np.float32))
    got = run_column(backend, linear, [(fmt, N, native)], K, x, epilogue=ops.EPILOGUE_RESIDUAL, residual_bits=res)
    assert np.array_equal(got, orc.f32_to_bf16(want + orc.bf16_to_f32(res)))
    gate_native = orc.make_native(fmt, N, K, 18 + M)
    pair = run_column(backend, linear, [(fmt, N, native)], K, x, epilogue=ops.EPILOGUE_GATE_UP, gate=(fmt, N, gate_native))
    swiglu = orc.swiglu(orc.gemv_column(fmt, gate_native, x, N), want)
    diff = np.abs(pair.astype(np.int32) - swiglu.astype(np.int32))   # exp2's last bits differ between the CPU and the GPU
    assert diff.max() <= 1 and (diff > 0).mean() < 0.02, (diff.max(), (diff > 0).mean())


def test_the_column_tile_takes_a_format_a_tensor_and_closed_forms(backend):
    """A fused projection's tensors, each of its own format, are a dispatch each at their columns; and the closed forms
    that pin the oracle's order hold on the GPU: 2^24 then ones in a group, ones then 2^24."""
    print("case column tile segments", flush=True)
    rng = np.random.default_rng(3)
    K, M = 2304, 2
    parts = [(ops.FMT_Q4K, 64, orc.make_native(ops.FMT_Q4K, 64, K, 1)), (ops.FMT_Q6K, 16, orc.make_native(ops.FMT_Q6K, 16, K, 2)),
             (ops.FMT_IQ4XS, 32, orc.make_native(ops.FMT_IQ4XS, 32, K, 3))]
    x = orc.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    linear = ops.Linear(backend)
    got = run_column(backend, linear, parts, K, x, float32=True)
    want = np.concatenate([orc.gemv_column(f, nat, x, n) for f, n, nat in parts], axis=1)
    assert got.tobytes() == want.tobytes()
    # Q8_0 rows of ones under a scale of one: a block is the fp16 scale and 32 codes
    K = 256
    blocks = np.zeros((16, K // 32, 34), dtype=np.uint8)
    blocks[:, :, :2] = np.frombuffer(np.float16(1.0).tobytes(), dtype=np.uint8)
    blocks[:, :, 2:] = 1
    native = np.ascontiguousarray(blocks.reshape(16, -1))
    values = np.zeros((2, K), dtype=np.float32)
    values[:, :32] = 1.0
    values[0, 0] = 2.0 ** 24      # row 0: the ones after it are lost
    values[1, 31] = 2.0 ** 24     # row 1: 31 first, then 2^24 + 31 rounds to 2^24 + 32
    got = run_column(backend, linear, [(ops.FMT_Q80, 16, native)], K, orc.f32_to_bf16(values), float32=True)
    assert np.all(got[0] == 2.0 ** 24) and np.all(got[1] == 2.0 ** 24 + 32)


def test_the_column_tile_rejects_what_it_does_not_run(backend):
    linear = ops.Linear(backend)
    K, N = 512, 32
    proj = ops.Projection.from_native(backend, [(ops.FMT_Q4K, N, orc.make_native(ops.FMT_Q4K, N, K, 1))], K)
    with pytest.raises(splash_amd.SplashError):
        linear.plan(proj, 3, column=True)                      # more than two rows
    plan = linear.plan(proj, 2, column=True)
    plan.splits = 2
    with pytest.raises(splash_amd.SplashError):
        ops.check(ops.lib.spo_linear_plan_with(proj.handle, ops.ctypes.byref(plan)))     # a partition of K
