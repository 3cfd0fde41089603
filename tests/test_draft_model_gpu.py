"""model::DFlashDraft on the GPU against the oracle's composition of its operators (tests/draft_reference.py): the
context side (prompt rows into a lane's window and rings, a verify step's retained rows through the masks and lane rows
on the device, the rings rebuilt from the window) and the forward pass of a step's lanes from the rings those left, to
the vocabulary head and the selector's rows, which the candidate selection then reads without a copy."""
import numpy as np
import pytest

import splash_amd
from splash_amd import ops, verify
from tests import oracle as orc
from tests.draft_reference import DraftModel, bits, rope_tables, ROWS, KVH, D, WINDOW, RING

pytestmark = pytest.mark.gpu


def ulps(a, b):
    """Distance in bf16 steps between two arrays of bf16 bits (as ordered integers)."""
    key = lambda x: np.where(x & 0x8000, 0x8000 - (x & 0x7FFF).astype(np.int32), 0x8000 + (x & 0x7FFF).astype(np.int32))
    return np.abs(key(np.asarray(a, np.uint16)) - key(np.asarray(b, np.uint16)))


def close_rows(got_bits, want_bits, label, ulp=2, fraction=0.02, floor=2.0 ** -9):
    """bf16 rows that differ by roundings of fp32 sums: within `ulp` steps (or `floor` of the rows' scale near zero), and
    all but `fraction` of them equal to a step."""
    got, want = orc.bf16_to_f32(got_bits).astype(np.float64), orc.bf16_to_f32(want_bits).astype(np.float64)
    scale = np.abs(want).max()
    distance = ulps(got_bits, want_bits)
    near = np.abs(got - want) <= floor * scale
    assert np.all((distance <= ulp) | near), (label, int(distance[~near].max()), float(np.abs(got - want).max()), float(scale))
    assert (distance > 1).mean() <= fraction, (label, float((distance > 1).mean()))


def cosine(a, b):
    a, b = np.asarray(a, np.float64).ravel(), np.asarray(b, np.float64).ravel()
    return float(a @ b / np.sqrt((a @ a) * (b @ b)))


def ring_view(raw, model, lane, layer):
    """(keys [8][2048][128], values [8][128][2048]) of a lane's layer in the downloaded rings."""
    at = (lane * model.layer_count + layer) * 2 * RING
    return raw[at:at + RING].reshape(KVH, WINDOW, D), raw[at + RING:at + 2 * RING].reshape(KVH, D, WINDOW)


@pytest.fixture(scope="module")
def draft(backend):
    model = DraftModel(seed=31, hidden=1024, vocabulary=4096, intermediate=2048, layers=2, target_layers=2)
    gpu = model.build_gpu(backend, max_lanes=3, context_rows=64)
    yield model, gpu
    gpu.close()


def prefill(backend, model, gpu, lane, rows, start, rng):
    captured = bits(rng.standard_normal((rows, model.target_layers * model.hidden)))
    cosines, sines = rope_tables(start + np.arange(rows))
    gpu.buffer(verify.DFLASH_CAPTURED_TARGET_HIDDEN).upload(captured)
    gpu.buffer(verify.DFLASH_CONTEXT_ROPE_COS).upload(cosines)
    gpu.buffer(verify.DFLASH_CONTEXT_ROPE_SIN).upload(sines)
    backend.run(gpu.encode_context_prefill(lane, rows, start))
    return captured, cosines, sines


def test_prompt_rows_fill_a_lanes_window_and_rings(backend, draft):
    print("case draft model context prefill", flush=True)
    model, gpu = draft
    rng = np.random.default_rng(1)
    rows, start, lane = 50, 2030, 1          # the last 32 rows wrap the ring
    before = gpu.buffer(verify.DFLASH_RINGS).download(np.uint16)
    captured, cosines, sines = prefill(backend, model, gpu, lane, rows, start, rng)
    hidden = gpu.buffer(verify.DFLASH_CONTEXT_HIDDEN).download(np.uint16)[:rows * model.hidden].reshape(rows, model.hidden)
    close_rows(hidden, model.oracle_context_hidden(captured), "context rows")
    # from the GPU's own context rows on: the window byte for byte, the rings to the projection's rounding
    windows = gpu.buffer(verify.DFLASH_WINDOWS).download(np.uint8)
    size = ops.DraftAttention.window_bytes(model.hidden)
    want = np.zeros(size, np.uint8)
    orc.draft_window_store(hidden, np.arange(rows), start, want)
    assert np.array_equal(windows[lane * size:(lane + 1) * size], want)
    assert not windows[:lane * size].any() and not windows[(lane + 1) * size:].any()
    after = gpu.buffer(verify.DFLASH_RINGS).download(np.uint16)
    slots = (start + np.arange(rows)) % WINDOW
    for layer in range(model.layer_count):
        keys, values = (a.copy() for a in ring_view(before, model, lane, layer))
        orc.draft_context_write(model.oracle_context_kv(hidden, layer), model.layers[layer]["key_norm"], cosines, sines, np.arange(rows),
                                start + np.arange(rows), np.arange(rows), keys, values)
        got_keys, got_values = ring_view(after, model, lane, layer)
        close_rows(got_keys[:, slots], keys[:, slots], f"ring keys of layer {layer}", ulp=3, fraction=0.03)
        close_rows(got_values[:, :, slots], values[:, :, slots], f"ring values of layer {layer}")
        others = np.setdiff1d(np.arange(WINDOW), slots)
        assert np.array_equal(got_keys[:, others], keys[:, others]) and np.array_equal(got_values[:, :, others], values[:, :, others])
    other_lanes = np.ones(after.size, bool)
    other_lanes[lane * model.layer_count * 2 * RING:(lane + 1) * model.layer_count * 2 * RING] = False
    assert np.array_equal(after[other_lanes], before[other_lanes])


def test_a_steps_rows_through_the_draft(backend, draft):
    """Three lanes: one with no context, one with a short one, one past the window (lane 1, whose ring the test above and
    this one fill). The oracle runs from the rings the GPU holds, so only the step's own arithmetic is compared."""
    print("case draft model decode", flush=True)
    model, gpu = draft
    rng = np.random.default_rng(2)
    prefill(backend, model, gpu, 2, 40, 0, rng)
    prefill(backend, model, gpu, 1, 64, 2080, rng)
    cache_lengths = [0, 2144, 40]
    lanes = len(cache_lengths)
    raw = gpu.buffer(verify.DFLASH_RINGS).download(np.uint16)
    rings = [[[a.ravel() for a in ring_view(raw, model, lane, layer)] for layer in range(model.layer_count)] for lane in range(lanes)]
    hidden = bits(rng.standard_normal((lanes * ROWS, model.hidden)))     # row 0 of a lane: its anchor's embedding; the rest are overwritten
    gpu.buffer(verify.DFLASH_HIDDEN, 0).upload(hidden)
    tables = [rope_tables(c + np.arange(16)) for c in cache_lengths]
    cosines, sines = np.stack([t[0] for t in tables]), np.stack([t[1] for t in tables])
    gpu.buffer(verify.DFLASH_ROPE_COS).upload(cosines)
    gpu.buffer(verify.DFLASH_ROPE_SIN).upload(sines)
    graph = gpu.encode_decode(cache_lengths)
    print(f"  {len(graph.kernels())} dispatches", flush=True)
    backend.run(graph)
    masked = hidden.reshape(lanes, ROWS, -1).copy()
    masked[:, 1:] = model.mask_embedding
    masked = masked.reshape(lanes * ROWS, -1)
    after, final, logits, selector = model.oracle_decode(masked, rings, cache_lengths, cosines, sines)
    got_hidden = gpu.buffer(verify.DFLASH_HIDDEN, model.layer_count & 1).download(np.uint16)[:masked.size].reshape(masked.shape)
    got_final = gpu.buffer(verify.DFLASH_FINAL_HIDDEN).download(np.uint16)[:masked.size].reshape(masked.shape)
    got_logits = gpu.buffer(verify.DFLASH_LOGITS).download(np.float32)[:lanes * ROWS * model.vocabulary].reshape(lanes * ROWS, -1)
    got_selector = gpu.buffer(verify.DFLASH_SELECTOR_HIDDEN).download(np.uint16)[:lanes * ROWS * 256].reshape(lanes * ROWS, 256)
    f = lambda b: orc.bf16_to_f32(b).astype(np.float64)
    report = dict(hidden=cosine(f(got_hidden), f(after[-1])), final=cosine(f(got_final), f(final)), logits=cosine(got_logits, logits),
                  selector=cosine(f(got_selector), f(selector)))
    worst = float(np.abs(got_logits - logits).max() / np.abs(logits).max())
    print(f"  cosines {report}; logits' largest difference over their largest magnitude {worst:.5f}", flush=True)
    assert min(report.values()) >= 0.9999 and worst <= 2e-2
    # the final stage from the GPU's own rows: the norm to a step, the head inside its rounding, greedy ids equal where the
    # oracle's margin exceeds it
    close_rows(got_final, orc.rms_norm(got_hidden, model.final_norm), "final norm", ulp=1, fraction=0.0)
    exact = orc.gemm(orc.FMT_Q6K, model.head, got_final, model.vocabulary, want=("exact", "bound"))
    assert np.all(np.abs(got_logits - exact["exact"]) <= exact["bound"] + 1e-6)
    top = np.sort(exact["exact"], axis=1)
    clear = top[:, -1] - top[:, -2] > 2 * exact["bound"].max()
    assert np.array_equal(got_logits.argmax(axis=1)[clear], exact["exact"].argmax(axis=1)[clear]) and clear.sum() >= lanes * ROWS // 2


def test_the_selector_reads_the_drafts_rows_in_place(backend, draft):
    """The candidates of every proposal position from the logits and selector rows the draft left, against the oracle's
    selection over the same downloaded logits."""
    print("case draft model candidates", flush=True)
    model, gpu = draft
    lanes, V = 3, model.vocabulary
    rng = np.random.default_rng(5)
    codebooks = [backend.from_array(bits(rng.standard_normal((V, 256)) * 0.1)) for _ in range(2)]
    candidates = backend.allocate_buffer(lanes * 7 * 16 * 4)
    unary = backend.allocate_buffer(lanes * 7 * 16 * 4)
    edges = backend.allocate_buffer(lanes * 7 * 16 * 16 * 4)
    scratch = backend.allocate_buffer(max(ops.DraftSelector.candidate_scratch_bytes(lanes, V), 16))
    graph = splash_amd.CommandGraph()
    ops.DraftSelector.add_candidates(graph, gpu.buffer(verify.DFLASH_LOGITS), gpu.buffer(verify.DFLASH_SELECTOR_HIDDEN), scratch, candidates,
                                     unary, edges, codebooks[0], codebooks[1], V, V, V, [1, 2, 3])
    backend.run(graph)
    logits = gpu.buffer(verify.DFLASH_LOGITS).download(np.float32)[:lanes * ROWS * V].reshape(lanes * ROWS, V)
    want_ids, want_logits = orc.draft_candidates(logits, lanes)
    assert np.array_equal(candidates.download(np.uint32).reshape(want_ids.shape), want_ids)
    assert np.array_equal(unary.download(np.float32).reshape(want_logits.shape), want_logits)


def test_retained_rows_of_a_step_enter_the_context(backend, draft):
    print("case draft model context commit", flush=True)
    model, gpu = draft
    rng = np.random.default_rng(3)
    lane_rows = np.array([(0, 9), (9, 16), (25, 4)], np.uint32)
    retained = np.array([0b100010011, 0xFFFF, 0b0001], np.uint32)
    starts = [0, 2144, 40]
    rows = 29
    captured = bits(rng.standard_normal((rows, model.target_layers * model.hidden)))
    tables = [rope_tables(s + np.arange(16)) for s in starts]
    cosines, sines = np.concatenate([t[0] for t in tables]), np.concatenate([t[1] for t in tables])
    gpu.buffer(verify.DFLASH_CAPTURED_TARGET_HIDDEN).upload(captured)
    gpu.buffer(verify.DFLASH_CONTEXT_ROPE_COS).upload(cosines)
    gpu.buffer(verify.DFLASH_CONTEXT_ROPE_SIN).upload(sines)
    before_rings = gpu.buffer(verify.DFLASH_RINGS).download(np.uint16)
    before_windows = gpu.buffer(verify.DFLASH_WINDOWS).download(np.uint8)
    backend.run(gpu.encode_context_commit(backend.from_array(retained), backend.from_array(lane_rows), starts, rows, 16))
    hidden = gpu.buffer(verify.DFLASH_CONTEXT_HIDDEN).download(np.uint16)[:rows * model.hidden].reshape(rows, model.hidden)
    close_rows(hidden, model.oracle_context_hidden(captured), "context rows")
    after_rings = gpu.buffer(verify.DFLASH_RINGS).download(np.uint16)
    windows = gpu.buffer(verify.DFLASH_WINDOWS).download(np.uint8)
    size = ops.DraftAttention.window_bytes(model.hidden)
    for lane in range(3):
        path = np.array([b for b in range(16) if retained[lane] >> b & 1])
        want = before_windows[lane * size:(lane + 1) * size].copy()
        orc.draft_window_store(hidden, lane_rows[lane, 0] + path, starts[lane], want)
        assert np.array_equal(windows[lane * size:(lane + 1) * size], want), lane
        slots = (starts[lane] + np.arange(len(path))) % WINDOW
        for layer in range(model.layer_count):
            keys, values = (a.copy() for a in ring_view(before_rings, model, lane, layer))
            orc.draft_context_write(model.oracle_context_kv(hidden, layer), model.layers[layer]["key_norm"], cosines, sines,
                                    lane_rows[lane, 0] + path, starts[lane] + np.arange(len(path)), 16 * lane + np.arange(len(path)), keys, values)
            got_keys, got_values = ring_view(after_rings, model, lane, layer)
            close_rows(got_keys[:, slots], keys[:, slots], f"lane {lane} keys of layer {layer}", ulp=3, fraction=0.03)
            close_rows(got_values[:, :, slots], values[:, :, slots], f"lane {lane} values of layer {layer}")
            others = np.setdiff1d(np.arange(WINDOW), slots)
            assert np.array_equal(got_keys[:, others], keys[:, others]) and np.array_equal(got_values[:, :, others], values[:, :, others])


def test_rings_rebuilt_from_the_window(backend, draft):
    """A lane restored from its cached form holds its window alone: its rings come back from the window's rows, every
    layer's keys and values of the 4-bit rows the window restores."""
    print("case draft model context rebuild", flush=True)
    model, gpu = draft
    lane, rows, start = 2, 41, 0      # the 40 prompt rows and the one row the commit above added
    size = ops.DraftAttention.window_bytes(model.hidden)
    window = gpu.buffer(verify.DFLASH_WINDOWS).download(np.uint8)[lane * size:(lane + 1) * size]
    cosines, sines = rope_tables(start + np.arange(rows))
    gpu.buffer(verify.DFLASH_CONTEXT_ROPE_COS).upload(cosines)
    gpu.buffer(verify.DFLASH_CONTEXT_ROPE_SIN).upload(sines)
    before = gpu.buffer(verify.DFLASH_RINGS).download(np.uint16)
    backend.run(gpu.encode_context_prefill(lane, rows, start, rebuild=True))
    restored = orc.draft_window_load(window, rows, start, model.hidden)
    assert np.array_equal(gpu.buffer(verify.DFLASH_CONTEXT_HIDDEN).download(np.uint16)[:restored.size].reshape(restored.shape), restored)
    after = gpu.buffer(verify.DFLASH_RINGS).download(np.uint16)
    slots = (start + np.arange(rows)) % WINDOW
    for layer in range(model.layer_count):
        keys, values = (a.copy() for a in ring_view(before, model, lane, layer))
        orc.draft_context_write(model.oracle_context_kv(restored, layer), model.layers[layer]["key_norm"], cosines, sines, np.arange(rows),
                                start + np.arange(rows), np.arange(rows), keys, values)
        got_keys, got_values = ring_view(after, model, lane, layer)
        close_rows(got_keys[:, slots], keys[:, slots], f"rebuilt keys of layer {layer}", ulp=3, fraction=0.03)
        close_rows(got_values[:, :, slots], values[:, :, slots], f"rebuilt values of layer {layer}")
        # and they are the rows the prompt left, to the 4-bit window's step
        old_keys, _ = ring_view(before, model, lane, layer)
        assert cosine(orc.bf16_to_f32(got_keys[:, slots]), orc.bf16_to_f32(old_keys[:, slots])) > 0.98


def test_a_head_over_a_subset_of_the_vocabulary(backend):
    """The draft's logits over the target's first 1024 tokens and those from 3072 on (the reference's DraftVocabulary): the
    head is a view of the same image's rows, its logits those columns of the whole head's (inside the projection's fp64
    interval, both), and the candidates name the tokens, not the columns."""
    print("case draft model vocabulary subset", flush=True)
    model = DraftModel(seed=33, hidden=1024, vocabulary=4096, intermediate=1024, layers=1, target_layers=1)
    rng = np.random.default_rng(9)
    hidden = bits(rng.standard_normal((ROWS, model.hidden)))
    cosines, sines = rope_tables(np.arange(16))
    logits = {}
    for name, ranges in (("whole", None), ("subset", [(0, 1024), (3072, 1024)])):
        gpu = model.build_gpu(backend, max_lanes=1, head_ranges=ranges)
        gpu.buffer(verify.DFLASH_HIDDEN, 0).upload(hidden)
        gpu.buffer(verify.DFLASH_ROPE_COS).upload(cosines)
        gpu.buffer(verify.DFLASH_ROPE_SIN).upload(sines)
        backend.run(gpu.encode_decode([0]))
        columns = 2048 if ranges else 4096
        logits[name] = gpu.buffer(verify.DFLASH_LOGITS).download(np.float32)[:ROWS * columns].reshape(ROWS, columns).copy()
        final = gpu.buffer(verify.DFLASH_FINAL_HIDDEN).download(np.uint16)[:ROWS * model.hidden].reshape(ROWS, model.hidden).copy()
        if ranges:
            candidates, unary = backend.allocate_buffer(7 * 16 * 4), backend.allocate_buffer(7 * 16 * 4)
            graph = splash_amd.CommandGraph()
            ops.DraftSelector.add_candidates(graph, gpu.buffer(verify.DFLASH_LOGITS), gpu.buffer(verify.DFLASH_SELECTOR_HIDDEN),
                                             backend.allocate_buffer(max(ops.DraftSelector.candidate_scratch_bytes(1, columns), 16)), candidates, unary,
                                             backend.allocate_buffer(7 * 256 * 4), backend.from_array(bits(rng.standard_normal((4096, 256)) * 0.1)),
                                             backend.from_array(bits(rng.standard_normal((4096, 256)) * 0.1)), 1024, 3072, 4096, [5])
            backend.run(graph)
            want_ids, want_logits = orc.draft_candidates(logits[name], 1, leading=1024, trailing=3072)
            ids = candidates.download(np.uint32).reshape(7, 16)
            assert np.array_equal(ids, want_ids) and np.all((ids < 1024) | (ids >= 3072)) and (ids >= 3072).any()
        gpu.close()
    exact = orc.gemm(orc.FMT_Q6K, model.head, final, model.vocabulary, want=("exact", "bound"))
    keep = np.r_[0:1024, 3072:4096]
    assert np.all(np.abs(logits["whole"] - exact["exact"]) <= exact["bound"] + 1e-6)
    assert np.all(np.abs(logits["subset"] - exact["exact"][:, keep]) <= exact["bound"][:, keep] + 1e-6)


def test_the_draft_refuses_what_it_cannot_run(backend, draft):
    print("case draft model refusals", flush=True)
    model, gpu = draft
    with pytest.raises(splash_amd.SplashError):
        gpu.encode_decode([0, 0, 0, 0])             # more lanes than it was created for
    with pytest.raises(splash_amd.SplashError):
        gpu.encode_context_prefill(0, 65, 0)        # more rows than a context call takes
    with pytest.raises(splash_amd.SplashError):
        gpu.encode_context_prefill(3, 8, 0)         # no such lane
    with pytest.raises(splash_amd.SplashError):
        verify.DFlashDraft(backend, 2, 1000, 4096, 2048, 2, 1)     # a hidden size of a partial group
