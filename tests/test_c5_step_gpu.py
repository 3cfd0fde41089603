"""Parity of the hybrid mixture-of-experts verify step at BASELINE.json config 5's full shape (48 layers, three Gated
DeltaNet layers to one attention layer, hidden 2048, 128 experts top-8 of FFN 768 in Q4_K, GDN 16 key / 32 value heads
with 128 x 128 fp32 states, attention 32 q / 4 kv heads x 128 over INT8 KV, vocabulary 151936; batch 8 of 16-row blocks,
contexts up to 16K), through the C ABI. The 48 layers share four drawn weight sets (one period of the layer pattern), the
twelve attention layers one drawn context; a sample of layers -- GDN and attention, first, middle and last -- is checked
against the oracle from the GPU's own layer inputs, cells and tapes, then the head and the acceptance."""
import numpy as np
import pytest

from splash_amd import verify
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
    # layers 0-2 GDN, 3 attention (first period); 22 GDN, 23 attention (middle); 46 GDN, 47 attention (last)
    logits, (selected, retained, accepted, masks) = check_step(backend, model, gpu, lanes, tokens, checked_layers={0, 3, 22, 23, 46, 47}, deep=True)
    assert np.isfinite(logits).all() and all(1 <= r <= 16 for r in retained)
