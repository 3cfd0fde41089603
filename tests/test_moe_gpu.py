"""Mixture-of-experts routing, grouped expert projections and combine on the GPU against the oracle."""
import numpy as np
import pytest

import splash_amd
from splash_amd import ops
from tests import oracle as orc

pytestmark = pytest.mark.gpu


def run_layer(backend, rng, hidden, ffn, experts, top_k, rows, down_fmt=ops.FMT_Q4K, following=None, shared=0, gated=False, sigmoid=False,
              fmt=ops.FMT_Q4K):
    """shared: slices of a shared expert, whose images follow the routed experts'; gated: they weigh sigmoid(x . gate)."""
    gate = [orc.make_native(fmt, ffn, hidden, 100 + e) for e in range(experts + shared)]
    up = [orc.make_native(fmt, ffn, hidden, 300 + e) for e in range(experts + shared)]
    down = [orc.make_native(down_fmt, hidden, ffn, 500 + e) for e in range(experts + shared)]
    images = [backend.from_array(np.concatenate([ops.pack_gguf_image(f, n, r, k) for n in natives]))
              for natives, f, r, k in ((gate, fmt, ffn, hidden), (up, fmt, ffn, hidden), (down, down_fmt, hidden, ffn))]
    x = orc.f32_to_bf16(rng.standard_normal((rows, hidden)).astype(np.float32))
    res = orc.f32_to_bf16(rng.standard_normal((rows, hidden)).astype(np.float32))
    scores = rng.standard_normal((rows, experts)).astype(np.float32)
    scores[0, :] = 0.5                                 # a row of ties: experts 0..top_k-1 in id order
    moe = ops.MoE(backend, hidden, ffn, experts, top_k, rows, shared_slices=shared, shared_gate=gated, sigmoid_router=sigmoid)
    out = backend.allocate_buffer(rows * hidden * 2)
    graph = splash_amd.CommandGraph()
    scalar_gate = (rng.standard_normal(hidden) * 0.05).astype(np.float32) if gated else None
    moe.add_routing(graph, backend.from_array(scores), input=backend.from_array(x) if gated else None,
                    shared_scalar_gate=backend.from_array(scalar_gate) if gated else None)
    extra = dict(norm_weight=following[0], next_table=following[1]) if following else {}
    moe.add_routed(graph, backend.from_array(x), backend.from_array(res), out, *images, fmt=fmt, down_fmt=down_fmt, **extra)
    assert len(graph) == 6
    backend.run(graph)
    got = out.download(np.uint16).reshape(rows, hidden)
    want = orc.moe_layer(x, res, scores, top_k, gate, up, down, ffn, fmt=fmt, down_fmt=down_fmt, shared=shared, shared_gate=scalar_gate,
                         sigmoid_router=sigmoid)
    return moe, got, want


def check_layer(moe, got, want, rows, experts, top_k, shared=0):
    selected, weights, y, out = want
    b = moe.buffers
    routed = top_k
    top_k, experts = top_k + shared, experts + shared      # the shared slices are further routes of a row, and experts
    assert np.array_equal(selected[:, routed:], np.tile(experts - shared + np.arange(shared), (rows, 1)))
    got_selected = b["selected"].download(np.uint32)[:rows * top_k].reshape(rows, top_k)
    assert np.array_equal(got_selected, selected)                        # routing is exact, ties by id
    got_weights = b["weights"].download(np.float32)[:rows * top_k].reshape(rows, top_k)
    assert np.abs(got_weights - weights).max() <= 1e-6
    # grouping: every route has its own slot, in a tile of its expert, routes of an expert in route order
    tiles = int(b["tile_total"].download(np.uint32)[0])
    tile_expert = b["tile_expert"].download(np.uint32)[:tiles]
    tile_rows = b["tile_rows"].download(np.uint32)[:tiles]
    slot = b["route_slot"].download(np.uint32)[:rows * top_k]
    slot_row = b["slot_row"].download(np.uint32)
    assert len(set(slot.tolist())) == rows * top_k
    flat = selected.ravel()
    assert np.array_equal(tile_expert[slot // 16], flat)
    assert np.array_equal(slot_row[slot], np.arange(rows * top_k) // top_k)
    assert int(tile_rows.sum()) == rows * top_k and np.all(np.diff(tile_expert.astype(np.int64)) >= 0)
    assert tiles == sum((np.count_nonzero(flat == e) + 15) // 16 for e in range(experts))
    for e in np.unique(flat):
        assert np.all(np.diff(slot[flat == e].astype(np.int64)) > 0)
    # expert outputs of the routes, then the combined rows: exp2 and the SwiGLU's exp2 differ in their
    # last bits between host and GPU, which moves a few values by one bf16 step
    # (a step of an intermediate value moves a down-projection sum by its weight, however small the sum: the
    # error is bounded against the row's size, not the element's)
    def close(got_bits, want_bits):
        g, w = orc.bf16_to_f32(got_bits).astype(np.float64), orc.bf16_to_f32(want_bits).astype(np.float64)
        scale = np.abs(w).max(axis=-1, keepdims=True)
        assert np.all(np.abs(g - w) <= 2.0 ** -7 * np.abs(w) + 2.0 ** -8 * scale), np.abs(g - w).max()
        assert (got_bits != want_bits).mean() < 0.03
    got_y = b["expert_output"].download(np.uint16).reshape(-1, y.shape[2])[slot].reshape(y.shape)
    close(got_y, y)
    close(got, out)


@pytest.mark.parametrize("config", [(512, 256, 8, 2, 20), (256, 256, 5, 5, 3), (1024, 512, 64, 4, 48)])
def test_moe_layer_matches_the_oracle(backend, config):
    print(f"case moe {config}", flush=True)
    hidden, ffn, experts, top_k, rows = config
    rng = np.random.default_rng(experts)
    moe, got, want = run_layer(backend, rng, hidden, ffn, experts, top_k, rows)
    check_layer(moe, got, want, rows, experts, top_k)


@pytest.mark.parametrize("config", [(512, 256, 8, 2, 20, 1, True), (256, 256, 6, 3, 40, 2, False), (1024, 512, 64, 4, 48, 1, False),
                                    (2048, 768, 128, 8, 128, 1, True)])
def test_shared_expert_slices_ride_every_row(backend, config):
    """The shared expert as further routes of every row (moe.metal:5-8, :42-65; MoE.hpp:50-63): ids `experts` on, gated
    by the sigmoid of the row's product with the block's scalar gate or weighing 1, through the same grouping, expert
    projections and combine; the last case is a 35B-A3B layer with its shared expert."""
    print(f"case moe shared {config}", flush=True)
    hidden, ffn, experts, top_k, rows, shared, gated = config
    rng = np.random.default_rng(experts + shared)
    moe, got, want = run_layer(backend, rng, hidden, ffn, experts, top_k, rows, shared=shared, gated=gated)
    check_layer(moe, got, want, rows, experts, top_k, shared)
    if not gated:
        assert np.all(want[1][:, top_k:] == 1.0)


@pytest.mark.parametrize("fmt,down_fmt", [(ops.FMT_IQ4XS, ops.FMT_Q5K), (ops.FMT_Q5K, ops.FMT_Q6K), (ops.FMT_Q80, ops.FMT_IQ4NL), (ops.FMT_Q6K, ops.FMT_Q80)])
def test_expert_tensors_of_every_image_format(backend, fmt, down_fmt):
    """The experts of a real file are not all Q4_K: every weight-image format serves the one-pass gate/up and the down
    projection of the routed experts."""
    print(f"case moe formats {fmt} {down_fmt}", flush=True)
    rng = np.random.default_rng(fmt * 7 + down_fmt)
    moe, got, want = run_layer(backend, rng, 512, 256, 8, 2, 24, fmt=fmt, down_fmt=down_fmt)
    check_layer(moe, got, want, 24, 8, 2)


def test_sigmoid_router_weighs_by_normalized_sigmoids(backend):
    """MoeRouter::SigmoidNormalized (moe.metal:21, :104-110): the same selection, each weight its score's sigmoid over the
    sum of the selected ones'; with an ungated shared expert twice the routed width (two slices), as the reference's
    Flint blocks have it."""
    print("case moe sigmoid router", flush=True)
    rng = np.random.default_rng(31)
    moe, got, want = run_layer(backend, rng, 512, 256, 16, 4, 40, shared=2, sigmoid=True)
    check_layer(moe, got, want, 40, 16, 4, 2)
    weights = want[1][:, :4]
    assert np.all(np.abs(weights.sum(axis=1) - 1) < 1e-5) and np.all(np.diff(weights, axis=1) <= 1e-7)


def test_moe_layer_at_the_35b_shape(backend):
    """Hidden 2048, 128 experts of FFN 768, top-8, eight lanes of sixteen rows (BASELINE.json config 5's MoE layer)."""
    print("case moe 35B shape", flush=True)
    rng = np.random.default_rng(9)
    moe, got, want = run_layer(backend, rng, 2048, 768, 128, 8, 128)
    check_layer(moe, got, want, 128, 128, 8)


@pytest.mark.parametrize("rows", [20, 100])
def test_combine_writes_the_next_norms_table(backend, rows):
    """The combine may also leave its rows as the activation table of the projection after their RMS norm, as a
    residual projection's norm epilogue does: the rows are unchanged, the table is bit for bit that of
    bf16(row * weight) in pieces of 64 rows, with each 64-column group's sums of squares of the rows."""
    print(f"case moe combine table rows={rows}", flush=True)
    hidden, ffn, experts, top_k = 512, 256, 8, 2
    rng = np.random.default_rng(rows)
    _, plain, _ = run_layer(backend, np.random.default_rng(rows), hidden, ffn, experts, top_k, rows)
    weight_bits = orc.f32_to_bf16((1 + 0.1 * rng.standard_normal(hidden)).astype(np.float32))
    table_bytes = ops.gguf_table_bytes(hidden, rows)
    table = backend.allocate_buffer(table_bytes)
    _, got, _ = run_layer(backend, np.random.default_rng(rows), hidden, ffn, experts, top_k, rows,
                          following=(backend.from_array(weight_bits), table))
    assert np.array_equal(got, plain)
    raw = table.download(np.uint8)[:table_bytes]
    scaled = orc.f32_to_bf16(orc.bf16_to_f32(got) * orc.bf16_to_f32(weight_bits)[None, :])
    at = 0
    for first in range(0, rows, 64):
        count = min(64, rows - first)
        tiles = (count + 15) // 16
        size = ops.gguf_table_bytes(hidden, count)
        piece = raw[at:at + size]
        at += size
        values, s32, s16 = orc.split_activation_table(piece, hidden, tiles)
        wv, w32, w16 = orc.activation_table(scaled[first:first + count])
        live = orc.table_rows(values, hidden, tiles)[:count]
        assert np.array_equal(live, orc.table_rows(wv, hidden, tiles)[:count])
        rows_of = lambda sums: sums.transpose(0, 2, 1).reshape(tiles * 16, -1)[:count]     # [tile][entry][16 rows] -> [row][entry]
        assert np.array_equal(rows_of(s32), rows_of(w32)) and np.array_equal(rows_of(s16), rows_of(w16))
        stride = max(16 * tiles, 32)     # floats an entry: whole 128-byte lines
        squares = piece[size - (hidden // 64) * stride * 4:].view(np.float32).reshape(hidden // 64, stride)[:, :16 * tiles]
        h = orc.bf16_to_f32(got[first:first + count]).astype(np.float64)
        assert np.allclose(squares[:, :count], (h.reshape(count, hidden // 64, 64) ** 2).sum(axis=2).T, rtol=1e-5, atol=0)
    assert at == table_bytes


def test_moe_rejects_bad_arguments(backend):
    with pytest.raises(ValueError):
        ops.MoE(backend, 2048, 768, 128, 8, 300)
    with pytest.raises(ValueError):
        ops.MoE(backend, 2048, 700, 128, 8, 16)
    moe = ops.MoE(backend, 512, 256, 8, 2, 4)
    graph = splash_amd.CommandGraph()
    with pytest.raises(ValueError):
        moe.add_routing(graph, backend.allocate_buffer(16))
    assert len(graph) == 0
