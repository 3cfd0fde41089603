"""Parity of the hybrid mixture-of-experts verify step at BASELINE.json config 5's full shape (48 layers, three Gated
DeltaNet layers to one attention layer, hidden 2048, 128 experts top-8 of FFN 768 in Q4_K, GDN 16 key / 32 value heads
with 128 x 128 fp32 states, attention 32 q / 4 kv heads x 128 over INT8 KV, vocabulary 151936; batch 8 of 16-row blocks,
contexts up to 16K), through the C ABI. The 48 layers share four drawn weight sets (one period of the layer pattern), the
twelve attention layers one drawn context; a sample of layers -- GDN and attention, first, middle and last -- is checked
against the oracle from the GPU's own layer inputs, cells and tapes, then the head and the acceptance. A second
step of the same eight lanes then folds the path each lane retained of the first (some lanes' drafts follow the target
for a few rows, so the paths differ in length): the cells it leaves equal the oracle's fold of the first step's tape bit
for bit, and nothing of a rejected row reaches them."""
import numpy as np
import pytest

from splash_amd import verify
from tests import oracle as orc
from tests.hybrid_reference import HybridModel
from tests.test_hybrid_step_gpu import check_step

pytestmark = pytest.mark.gpu

C5 = dict(hidden=2048, vocabulary=151936, layers=48, q_heads=32, kv_heads=4, head_dim=128, gdn_key_heads=16, gdn_value_heads=32,
          experts=128, top_k=8, expert_ffn=768)
COMMITTED = [16384 - 16, 9000, 300, 4096, 16000, 1, 12345, 2047]      # ragged contexts, the first the configuration's 16K
ROWS = [16, 16, 16, 16, 16, 16, 16, 16]


def test_config5_full_shape_step_of_eight_lanes(backend):
    print("case config 5 full shape: building the 35B-A3B-shaped model", flush=True)
    model = HybridModel(seed=51, distinct_layers=4, **C5)
    pages = (16384 + 255) // 256
    gpu = model.build_gpu(backend, max_lanes=8, pages_per_lane=pages)
    rng = np.random.default_rng(52)
    model.seed_context(rng, distinct=1)
    model.seed_states(rng, lanes=8)
    print("case config 5 full shape: model resident", flush=True)
    lanes = [verify.HybridLane(ROWS[i], COMMITTED[i], table_first=i * pages) for i in range(8)]
    tokens = rng.integers(0, C5["vocabulary"], sum(ROWS)).astype(np.uint32)
    # lanes 0, 3 and 6: the draft continues the target's own choices for two, four and six rows, then departs
    V = C5["vocabulary"]
    for r in range(1, 7):
        gpu.set_block(lanes, tokens)
        backend.run(gpu.encode(lanes, commit=False))
        picks = gpu.buffer(verify.LOGITS).download(np.float32, sum(ROWS) * V).reshape(-1, V).argmax(axis=1)
        for lane, follows in ((0, 2), (3, 4), (6, 6)):
            if r <= follows:
                tokens[16 * lane + r] = picks[16 * lane + r - 1]
    # layers 0-2 GDN, 3 attention (first period); 22 GDN, 23 attention (middle); 46 GDN, 47 attention (last)
    logits, (selected, retained, accepted, masks) = check_step(backend, model, gpu, lanes, tokens, checked_layers={0, 3, 22, 23, 46, 47}, deep=True)
    assert np.isfinite(logits).all() and all(1 <= r <= 16 for r in retained)
    assert accepted[0] >= 2 and accepted[3] >= 4 and accepted[6] >= 6, accepted
    # The second step: every lane folds the rows it retained, from the tape of parity 0 into the cell of parity 0,
    # reading the cell of parity 1 (the state before the first block). A sample of the 36 GDN layers is read back.
    sample = [0, 1, 17, 34, 35]
    before = {(i, g): model.read_cell(i, 1, g) for i in range(8) for g in sample}
    tapes = {(i, g): model.read_tape(i, 0, g) for i in range(8) for g in sample}
    print("case config 5 full shape: the second step folds each lane's retained path", [int(r) for r in retained], flush=True)
    lanes2 = [verify.HybridLane(ROWS[i], COMMITTED[i] + int(retained[i]), table_first=i * pages, pending_path=int(masks[i]), parity=1)
              for i in range(8)]
    tokens2 = rng.integers(0, V, sum(ROWS)).astype(np.uint32)
    gpu.set_block(lanes2, tokens2)
    backend.run(gpu.encode(lanes2, commit=True))
    selected2, retained2, accepted2, masks2 = gpu.results(lanes2)
    assert all(1 <= r <= 16 for r in retained2) and np.isfinite(gpu.buffer(verify.LOGITS).download(np.float32, sum(ROWS) * V)).all()
    for (i, g), (conv0, state0) in before.items():
        count = bin(int(masks[i])).count("1")
        rc, conv, state = orc.gdn_fold(model.gdn_shape, conv0, state0, tapes[(i, g)], int(masks[i]), count)
        got_conv, got_state = model.read_cell(i, 0, g)
        assert rc == 0 and np.array_equal(conv, got_conv) and state.tobytes() == got_state.tobytes(), (i, g)
        # a lane that kept only its first row: the cell is one step of the recurrence away from the one before, not the block's sixteen
        assert not np.array_equal(got_state, state0)
