"""Parity of the dense verify step at BASELINE.json's headline shape (config 4: 64 layers, hidden 5120, 64 q / 8 kv
heads x 128, SwiGLU 25600, vocabulary 151936, Q4_K with Q6_K down-projection and LM head, 32K INT8 context, 16-row
draft block), through the C ABI. The 64 layers cycle through four drawn weight sets and four drawn contexts (each
layer's weights and context are its own copy in HBM), so that a layer's roundings meet other weights in the next.

Tolerances: hidden rows and logits, teacher-forced (each GPU layer against the oracle run on the GPU's own layer input):
cosine >= 0.9999 and |delta| <= max(2e-2, two bf16 steps); greedy ids, accepted counts and retained masks bit-exact
against the oracle's acceptance of the GPU's logits, and equal to the oracle's own ids wherever the oracle's top-2 gap
exceeds the logits' tolerance; lanes of a batch bit for bit what each lane gives alone."""
import numpy as np
import pytest

import splash_amd
from splash_amd import ops, verify
from tests import oracle as orc
from tests.dense_reference import DenseModel

pytestmark = pytest.mark.gpu

C4 = dict(hidden=5120, q_heads=64, kv_heads=8, head_dim=128, ffn=25600, vocabulary=151936, layers=64)
V = C4["vocabulary"]
# lane 0 is the headline lane: a 16-row block ending a 32768-token context; the others are ragged
LANE_ROWS = [16, 16, 7, 16]
LANE_COMMITTED = [32768 - 16, 8000, 300, 20001]


def cosine(a, b):
    a, b = np.asarray(a, np.float64).ravel(), np.asarray(b, np.float64).ravel()
    return float((a * b).sum() / np.sqrt((a * a).sum() * (b * b).sum()))


def bf16_steps(got_bits, want_bits):
    """|got - want| in bf16 steps of want's binade (a step is 2^(exponent - 7)), per element."""
    g, w = orc.bf16_to_f32(got_bits).astype(np.float64), orc.bf16_to_f32(want_bits).astype(np.float64)
    step = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(w), 2.0 ** -100))) - 7)
    return np.abs(g - w) / step, g, w


def stage_close(name, got_bits, want_bits, steps_allowed=2, cos_floor=0.99999):
    """A stage fed the GPU's own input rows: cosine >= 0.99999 and every element within max(2e-2, `steps_allowed` bf16
    steps of the oracle's value) -- the oracle sums its projections exactly, the GPU in fp32 chains inside the
    reference's projection bound, so results straddle a bf16 rounding boundary now and then."""
    steps, g, w = bf16_steps(got_bits, want_bits)
    c = cosine(g, w)
    worst = float(np.where(np.abs(g - w) <= 2e-2, 0, steps).max())
    print(f"  {name}: cosine {c:.7f} max-abs {np.abs(g - w).max():.4f} worst {steps.max():.1f} bf16 steps, "
          f"{(steps > 1).mean() * 100:.3f}% of elements past one step", flush=True)
    assert c >= cos_floor and worst <= steps_allowed, (name, c, worst)


@pytest.fixture(scope="module")
def c4(backend):
    print("case config 4: building the 27B-shaped model", flush=True)
    model = DenseModel(seed=41, down_format=orc.FMT_Q6K, distinct_layers=4, **C4)
    gpu = model.build_gpu(backend, max_lanes=4, context_tokens=[c + 16 for c in LANE_COMMITTED])
    model.seed_context(gpu, None, np.random.default_rng(42), distinct=4)
    print("case config 4: model resident", flush=True)
    yield model, gpu
    del gpu


def lanes_of(model, which, temperature=0.0):
    return [verify.Lane(LANE_ROWS[i], LANE_COMMITTED[i], table_first=model.table_first[i], temperature=temperature) for i in which]


def logits_of(gpu, rows):
    return gpu.buffer(verify.LOGITS).download(np.float32, rows * V).reshape(rows, V)


def test_config4_layers_and_head_teacher_forced_and_greedy_acceptance(backend, c4):
    """Layers 0, 31 and 63 and the head at the headline shape against the oracle, each from the GPU's own input rows;
    greedy acceptance of the step bit-exact against the oracle's walk over the step's logits; and the oracle's own
    chain of all 64 layers run free beside them, against which the step (its norms left to the projections that read
    them) drifts no further than its parts run one by one (each after a norm pass)."""
    model, gpu = c4
    print("case config 4 teacher-forced layers, batch 1, 32K context", flush=True)
    rows, committed = LANE_ROWS[0], LANE_COMMITTED[0]
    lane = lanes_of(model, [0])
    tokens = np.random.default_rng(5).integers(0, V, rows).astype(np.uint32)
    gpu.set_block(lane, tokens)
    backend.run(gpu.encode(lane, commit=False))                     # the whole step: rope tables, 64 layers, head, acceptance
    step_logits = logits_of(gpu, rows)
    selected, retained, accepted, mask = gpu.results(lane)
    assert np.isfinite(step_logits).all()
    picks = np.array([orc.argmax(step_logits[r]) for r in range(rows)], dtype=np.uint32)
    kept, acc, m = orc.accept_tree(ops.chain_tree_rows([rows]), tokens, picks)
    assert retained[0] == len(kept) and accepted[0] == acc and mask[0] == m and np.array_equal(selected[:len(kept)], kept)
    # Part by part. After a layer has run alone its stages' rows are still in the driver's buffers: the fused q|k|v rows,
    # the attention rows, the rows after the output projection (hidden stream 1), the SwiGLU rows, the layer's output
    # (stream 0). Each stage of the oracle is fed the GPU's rows of the stage before it.
    H, W = C4["hidden"], (C4["q_heads"] + 2 * C4["kv_heads"]) * C4["head_dim"]
    rows_of = lambda which, width, index=0: gpu.buffer(which, index).download(np.uint16, rows * width).reshape(rows, width)
    hidden_of = lambda: rows_of(verify.HIDDEN, H)
    backend.run(gpu.encode_part(0, 0, lane))
    assert np.array_equal(hidden_of(), model.oracle_embedding(tokens))
    free = model.oracle_embedding(tokens)       # the oracle's own chain, fed nothing of the GPU's
    for layer in range(64):
        before = hidden_of() if layer in (0, 31, 63) else None
        backend.run(gpu.encode_part(1, layer, lane))
        free = model.oracle_layer(free, layer, committed, model.table_first[0])
        if layer % 16 == 15:
            g, w = orc.bf16_to_f32(hidden_of()).astype(np.float64), orc.bf16_to_f32(free).astype(np.float64)
            print(f" after layer {layer}, parts against the oracle's chain: cosine {cosine(g, w):.6f} relative rms "
                  f"{np.sqrt(((g - w) ** 2).mean() / (w ** 2).mean()):.4f}", flush=True)
        if before is None:
            continue
        print(f" layer {layer}", flush=True)
        first = model.table_first[0]
        qkv = rows_of(verify.QKV_ROWS, W)
        stage_close("q|k|v projection", qkv, model.oracle_qkv(before, layer))
        attention = rows_of(verify.ATTENTION_ROWS, C4["q_heads"] * C4["head_dim"])
        want, want64 = model.oracle_attention(qkv, layer, committed, first, want64=True)
        got = orc.bf16_to_f32(attention).astype(np.float64)
        # the attention's own gate: against the fp64 softmax over the dequantized pages (north_star: max-abs 2e-2, cosine
        # >= 0.9999), and within a bf16 step or two of the oracle's page loop
        print(f"  attention vs fp64: cosine {cosine(got, want64):.7f} max-abs {np.abs(got - want64).max():.5f}", flush=True)
        assert cosine(got, want64) >= 0.9999 and np.abs(got - want64).max() <= 2e-2
        stage_close("attention vs page loop", attention, want, steps_allowed=2, cos_floor=0.9999)
        hidden1 = rows_of(verify.HIDDEN, H, 1)
        stage_close("output projection + residual", hidden1, model.oracle_output(attention, before, layer))
        ffn = rows_of(verify.FFN_ROWS, C4["ffn"])
        # the output projection left the post-attention norm to the gate/up pass (its table holds bf16(h w), the inverse
        # RMS scales the sums): the oracle with the operand rounded there is what the kernel computes; the norm pass's
        # rounding, bf16((h inv) w), gives rows one operand rounding away, bounded here by their cosine
        stage_close("gate/up SwiGLU", ffn, model.oracle_ffn_rows(hidden1, layer, deferred=True))
        passed = orc.bf16_to_f32(model.oracle_ffn_rows(hidden1, layer))
        assert cosine(orc.bf16_to_f32(ffn), passed) >= 0.9999
        after = hidden_of()
        stage_close("down projection + residual", after, model.oracle_down(ffn, hidden1, layer))
        # the layer as a whole from its input rows: the stages' roundings compound (the attention rows' relative error,
        # bounded by its own gate above, passes through the post-attention norm at full size)
        whole = model.oracle_layer(before, layer, committed, first)
        steps, g, w = bf16_steps(after, whole)
        print(f"  whole layer: cosine {cosine(g, w):.7f} max-abs {np.abs(g - w).max():.4f} worst {steps.max():.1f} bf16 steps", flush=True)
        assert cosine(g, w) >= 0.9999
    final = hidden_of()
    backend.run(gpu.encode_part(2, 0, lane))
    got = logits_of(gpu, rows)
    want = model.oracle_head(final)
    err = float(np.abs(got - want).max())
    print(f"  head: cosine {cosine(got, want):.7f} max-abs {err:.4f}", flush=True)
    assert cosine(got, want) >= 0.9999 and err <= 2e-2
    # the ids the GPU takes from these logits are the oracle's wherever the oracle's own top two are further apart than
    # twice the tolerance, and one of its near-ties elsewhere
    want_ids = np.array([orc.argmax(want[r].astype(np.float32)) for r in range(rows)], dtype=np.uint32)
    part = np.partition(want, -2, axis=1)
    sure = part[:, -1] - part[:, -2] > 2 * 2e-2
    got_ids = np.array([orc.argmax(got[r]) for r in range(rows)], dtype=np.uint32)
    assert sure.sum() >= rows // 2 and np.array_equal(got_ids[sure], want_ids[sure])
    assert (want[np.arange(rows), got_ids] >= want.max(axis=1) - 2 * 2e-2).all()
    # The whole step against its parts run one after the other: a part starts with a norm pass, the step leaves every
    # norm but the first to the projection after it, so the two differ by one operand rounding a norm, and 64 layers of a
    # bf16 residual stream carry that on: free-running logits agree to cosine >= 0.999, not to the teacher-forced 2e-2.
    drift = float(np.abs(step_logits - got).max())
    print(f"  whole step vs parts, free-running over 64 layers: cosine {cosine(step_logits, got):.6f} max-abs {drift:.4f}", flush=True)
    assert cosine(step_logits, got) >= 0.999
    # Both against the oracle's own chain: six bf16 roundings a layer, each now and then a step apart between a sum
    # taken in fp32 and one taken exactly, over 64 layers of distinct weights (the differences add in quadrature:
    # about 0.7 % of the rows' size after a layer, 5 % after 64). The step's deferred norms must not add to that:
    # its logits lie as near the chain's as the parts' do, and where the chain's top two are well apart the ids agree.
    chain = model.oracle_head(free)
    rms = lambda a: float(np.sqrt(((a - chain) ** 2).mean()))
    chain_ids = chain.argmax(axis=1)
    part2 = np.partition(chain, -2, axis=1)
    apart = part2[:, -1] - part2[:, -2] > 0.25
    print(f"  against the oracle's chain: step cosine {cosine(step_logits, chain):.6f} rms {rms(step_logits):.4f} max-abs "
          f"{np.abs(step_logits - chain).max():.4f}; parts cosine {cosine(got, chain):.6f} rms {rms(got):.4f} max-abs "
          f"{np.abs(got - chain).max():.4f}; logits rms {float(np.sqrt((chain ** 2).mean())):.3f}; ids equal "
          f"{int((step_logits.argmax(axis=1) == chain_ids).sum())}/16 (step) {int((got.argmax(axis=1) == chain_ids).sum())}/16 (parts)", flush=True)
    assert cosine(step_logits, chain) >= 0.998 and cosine(got, chain) >= 0.998
    assert rms(step_logits) <= 1.15 * rms(got)
    assert np.array_equal(step_logits.argmax(axis=1)[apart], chain_ids[apart])


def test_config4_batch_of_four_lanes_equals_each_lane_alone(backend, c4):
    """Batch 4 (config 4's second batch size), ragged: 16 + 16 + 7 + 16 rows over contexts of 32752, 8000, 300 and 20001
    tokens. Every lane's logits, selections and acceptance are bit for bit what the lane gives alone."""
    model, gpu = c4
    print("case config 4 batch 4 against each lane alone", flush=True)
    rng = np.random.default_rng(6)
    lanes = lanes_of(model, range(4))
    rows = sum(LANE_ROWS)
    tokens = rng.integers(0, V, rows).astype(np.uint32)
    gpu.set_block(lanes, tokens)
    backend.run(gpu.encode(lanes, commit=False))
    together = logits_of(gpu, rows)
    selected, retained, accepted, mask = gpu.results(lanes)
    first = 0
    for i in range(4):
        n = LANE_ROWS[i]
        alone = lanes_of(model, [i])
        gpu.set_block(alone, tokens[first:first + n])
        backend.run(gpu.encode(alone, commit=False))
        got = logits_of(gpu, n)
        s1, r1, a1, m1 = gpu.results(alone)
        same = np.array_equal(got.view(np.uint32), together[first:first + n].view(np.uint32))
        print(f"  lane {i}: {n} rows, committed {LANE_COMMITTED[i]}: bitwise {same}, max-abs {np.abs(got - together[first:first + n]).max():.3g}",
              flush=True)
        assert same, i
        assert (r1[0], a1[0], m1[0]) == (retained[i], accepted[i], mask[i])
        assert np.array_equal(s1[:r1[0]], selected[first:first + r1[0]])
        picks = np.array([orc.argmax(got[r]) for r in range(n)], dtype=np.uint32)
        kept, acc, m = orc.accept_tree(ops.chain_tree_rows([n]), tokens[first:first + n], picks)
        assert r1[0] == len(kept) and a1[0] == acc and m1[0] == m and np.array_equal(s1[:len(kept)], kept)
        first += n


def test_config4_rejection_sampling_at_temperature_through_the_driver(backend, c4):
    """Config 4's sampled acceptance: T = 0.7 against a full-vocabulary draft distribution softmax(N(0, 2)), through
    DenseVerify (mass, residual ranges, draw) at 151936 columns: every row's token is the oracle's rejection_row over the
    step's own logits, except where a comparison lies within 1e-5 of its threshold, and the acceptance walk follows."""
    model, gpu = c4
    print("case config 4 rejection sampling T=0.7", flush=True)
    rng = np.random.default_rng(7)
    T = 0.7
    which = [0, 2]
    lanes = lanes_of(model, which, temperature=T)
    counts = [LANE_ROWS[i] for i in which]
    rows = sum(counts)
    tokens = rng.integers(0, V, rows).astype(np.uint32)
    uniforms = rng.random((rows, 2), dtype=np.float32)
    dl = rng.normal(0.0, 2.0, (rows, V))
    draft = np.exp(dl - dl.max(axis=1, keepdims=True))
    draft = (draft / draft.sum(axis=1, keepdims=True)).astype(np.float32)
    # first a greedy pass for the target's logits, so that the block can carry likely and unlikely children
    greedy = lanes_of(model, which)
    gpu.set_block(greedy, tokens)
    backend.run(gpu.encode(greedy, commit=False))
    logits = logits_of(gpu, rows)
    first = 0
    for n in counts:
        for r in range(first + 1, first + n):     # row r's token is the child drawn at row r - 1
            d64 = draft[r - 1].astype(np.float64)
            tokens[r] = int(np.argmax(logits[r - 1])) if r % 2 else int(rng.choice(V, p=d64 / d64.sum()))
        first += n
    # the block's rows changed, so did the logits after the first row: run the sampled step and read its own logits
    gpu.set_block(lanes, tokens, uniforms=uniforms)
    gpu.buffer(verify.DRAFT_PROBABILITIES).upload(draft)
    backend.run(gpu.encode(lanes, commit=False))
    logits = logits_of(gpu, rows)
    selected, retained, accepted, mask = gpu.results(lanes)

    def plausible(row, token, child):
        """The law in float64 with a tolerance where the oracle's comparison is within rounding of its threshold: a row
        whose child passes u q < p selects it; otherwise it draws, in id order, from max(p - q, 0) (from p without a child)
        at the point u_row of that mass."""
        x = logits[row].astype(np.float64)
        w = np.exp((x - x.max()) / T)
        p = w / w.sum()
        weights = p
        if child != orc.NO_TOKEN:
            q = draft[row].astype(np.float64)
            lhs, rhs = float(uniforms[row, 1]) * q[child], p[child]
            if token == child:
                return lhs < rhs * (1 + 1e-4)
            if lhs < rhs * (1 - 1e-4):
                return False
            weights = np.maximum(p - q, 0)
        cdf = np.cumsum(weights)
        point, slack = float(uniforms[row, 0]) * cdf[-1], 1e-4 * cdf[-1]
        return (cdf[token - 1] if token else 0.0) - slack <= point <= cdf[token] + slack and weights[token] > 0

    first, exact_rows, total_rows = 0, 0, 0
    for li, n in enumerate(counts):
        kept = selected[first:first + retained[li]]
        assert 1 <= retained[li] <= n and accepted[li] == retained[li] - 1 and mask[li] == (1 << retained[li]) - 1
        for r, token in enumerate(kept):
            row = first + r
            child = int(tokens[row + 1]) if r + 1 < n else orc.NO_TOKEN
            want, took, close = orc.rejection_row(logits[row], T, draft[row] if child != orc.NO_TOKEN else None, child,
                                                  float(uniforms[row, 1]), float(uniforms[row, 0]))
            if close > 1e-5:
                assert token == want, (li, r, token, want, took)
                exact_rows += 1
            assert plausible(row, int(token), child), (li, r, token, want, close)
            # the walk goes on exactly while a row selects its child
            assert (token == child) == (r + 1 < len(kept)), (li, r)
            total_rows += 1
        first += n
    print(f"  {total_rows} rows on the lanes' paths, {exact_rows} of them away from every threshold", flush=True)
    assert total_rows >= 2
