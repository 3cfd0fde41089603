"""Two decode cycles of two lanes with every hand-off on the device: the draft model proposes (its rows from the anchors'
embeddings, the rings its context writers filled), the selector grows each lane's tree, the rows go in slots into the
target's step, the target verifies and commits its cache, and the rows each lane kept -- the masks the acceptance wrote,
the lane rows the proposer wrote, the hidden rows the target's layers captured -- enter the draft's context for the next
cycle. The host reads only what the reference's host reads between cycles: how many tokens each lane kept."""
import numpy as np
import pytest

import splash_amd
from splash_amd import ops, verify
from tests import oracle as orc
from tests.dense_reference import DenseModel
from tests.draft_reference import DraftModel, bits, rope_tables, KVH, D, WINDOW
from tests.test_draft_model_gpu import close_rows, cosine, ring_view

pytestmark = pytest.mark.gpu


def test_a_decode_cycle_stays_on_the_device(backend):
    print("case draft and target cycles", flush=True)
    V, H, cap, lanes_n = 4096, 1024, 16, 2
    prompts = (37, 20)
    target_model = DenseModel(seed=5, hidden=H, q_heads=8, kv_heads=2, head_dim=128, ffn=2048, vocabulary=V, layers=4)
    draft_model = DraftModel(seed=6, hidden=H, vocabulary=V, intermediate=2048, layers=2, target_layers=2)
    draft_model.head = target_model.head            # the draft shares the target's head
    rng = np.random.default_rng(7)
    target = target_model.build_gpu(backend, max_lanes=lanes_n, context_tokens=[p + 64 for p in prompts], prefill_rows=64)
    draft = draft_model.build_gpu(backend, max_lanes=lanes_n, context_rows=64)
    captured = draft.buffer(verify.DFLASH_CAPTURED_TARGET_HIDDEN)
    target.set_capture([1, 3], captured)
    up = backend.from_array

    # ---- the prompts: the target's chunk, whose captured rows are the draft's context rows
    committed = [0, 0]
    for lane, count in enumerate(prompts):
        tokens = rng.integers(0, V, count).astype(np.uint32)
        target.set_prefill_block(tokens)
        backend.run(target.encode_prefill(target_model.table_first[lane], 0, count))
        cosines, sines = rope_tables(np.arange(count))
        draft.buffer(verify.DFLASH_CONTEXT_ROPE_COS).upload(cosines)
        draft.buffer(verify.DFLASH_CONTEXT_ROPE_SIN).upload(sines)
        backend.run(draft.encode_context_prefill(lane, count, 0))
        # the last captured layer is the target's last: its slot holds the hidden rows the chunk left
        rows = captured.download(np.uint16)[:count * 2 * H].reshape(count, 2 * H)
        assert np.array_equal(rows[:, H:], target.buffer(verify.HIDDEN, 0).download(np.uint16)[:count * H].reshape(count, H))
        committed[lane] = count

    codebooks = [up(bits(rng.standard_normal((V, 256)) * 0.08)) for _ in range(2)]
    b = dict(candidates=backend.allocate_buffer(lanes_n * 7 * 16 * 4), unary=backend.allocate_buffer(lanes_n * 7 * 16 * 4),
             edges=backend.allocate_buffer(lanes_n * 7 * 256 * 4), scratch=backend.allocate_buffer(ops.DraftSelector.candidate_scratch_bytes(lanes_n, V)),
             tokens=backend.allocate_buffer(128), trees=backend.allocate_buffer(256), scores=backend.allocate_buffer(256), sizes=backend.allocate_buffer(16),
             draws=backend.allocate_buffer(128), next=backend.allocate_buffer(2048), caps=backend.allocate_buffer(128), lane_rows=backend.allocate_buffer(16),
             sources=backend.allocate_buffer(128), ids=backend.allocate_buffer(32 * 16 * 4), q=backend.allocate_buffer(32 * 16 * 4),
             drawn=backend.allocate_buffer(32 * 4))
    anchors = [int(t) for t in rng.integers(0, V, lanes_n)]
    embedding = up(target_model.embedding)
    hidden0 = draft.buffer(verify.DFLASH_HIDDEN, 0)
    total_kept = 0
    for cycle in range(2):
        print(f"  cycle {cycle}: committed {committed}, anchors {anchors}", flush=True)
        # what the host knows before a cycle: each lane's committed tokens and its anchor
        tables = [rope_tables(c + np.arange(16)) for c in committed]
        for which, index in ((verify.DFLASH_ROPE_COS, 0), (verify.DFLASH_ROPE_SIN, 1), (verify.DFLASH_CONTEXT_ROPE_COS, 0), (verify.DFLASH_CONTEXT_ROPE_SIN, 1)):
            draft.buffer(which).upload(np.concatenate([t[index] for t in tables]))
        lanes = [verify.Lane(cap, c, table_first=f) for c, f in zip(committed, target_model.table_first)]
        # Random weights never agree, so lane 0 also carries a host chain (the reference's lookup branch) that the target
        # will accept: its own greedy continuation of the anchor, found by three chain steps that commit nothing.
        chain = [anchors[0]]
        for _ in range(3):
            alone = [verify.Lane(len(chain), committed[0], table_first=target_model.table_first[0])]
            target.set_block(alone, np.array(chain, np.uint32))
            backend.run(target.encode(alone, commit=False))
            chain.append(int(target.results(alone)[0][len(chain) - 1]))
        chain_tokens = np.zeros((lanes_n, 15), np.uint32)
        chain_tokens[0, :3] = chain[1:]
        chain_rates = np.zeros((lanes_n, 15, 4), np.float32)
        chain_rates[0, :3] = 0.97
        graph = splash_amd.CommandGraph()
        for lane, anchor in enumerate(anchors):
            ops.Embedding.add(graph, orc.FMT_Q4K, embedding, V, H, up(np.array([anchor], np.uint32)), hidden0.view(lane * 8 * H * 2, H * 2), 1)
        draft.encode_decode(committed, graph=graph)
        ops.DraftSelector.add_candidates(graph, draft.buffer(verify.DFLASH_LOGITS), draft.buffer(verify.DFLASH_SELECTOR_HIDDEN), b["scratch"],
                                         b["candidates"], b["unary"], b["edges"], codebooks[0], codebooks[1], V, V, V, anchors)
        tree_lanes = [dict(anchor=anchors[0], depth=15, children=3, intercept=[0.3] * 7, chain=3),
                      dict(anchor=anchors[1], depth=6, children=2, intercept=[0.3] * 7)]
        ops.DraftSelector.add_tree(graph, b["candidates"], b["unary"], b["edges"], up(chain_tokens), up(chain_rates),
                                   b["tokens"], b["trees"], b["scores"], b["sizes"], b["draws"], b["next"], b["caps"], tree_lanes)
        ops.DraftSelector.add_verify_row_slots(graph, b["tokens"], b["trees"], b["scores"], b["sizes"], target.buffer(verify.INPUT_TOKENS),
                                               target.buffer(verify.TREE_ROWS), b["lane_rows"], b["sources"], lanes_n, cap)
        ops.DraftSelector.add_verify_children(graph, b["sources"], b["lane_rows"], target.buffer(verify.TREE_ROWS), b["candidates"], b["next"],
                                              b["draws"], b["ids"], b["q"], b["drawn"], target.buffer(verify.DEPTHS), lanes_n, lanes_n * cap)
        target.encode(lanes, commit=True, graph=graph)
        draft.encode_context_commit(target.buffer(verify.RETAINED_ROWS), b["lane_rows"], committed, lanes_n * cap, cap, graph=graph)
        before = draft.buffer(verify.DFLASH_RINGS).download(np.uint16)
        backend.run(graph)        # one command: nothing crosses the host inside a cycle

        selected, retained, accepted, masks = (np.array(a).copy() for a in target.results(lanes))
        lane_rows = b["lane_rows"].download(np.uint32)[:2 * lanes_n].reshape(lanes_n, 2)
        print(f"    trees of {lane_rows[:, 1].tolist()} rows; kept {retained.tolist()} (masks {[bin(m) for m in masks]})", flush=True)
        assert lane_rows[:, 0].tolist() == [0, cap] and all(1 <= r <= n for r, n in zip(retained, lane_rows[:, 1]))
        assert retained[0] == 4 and selected[:3].tolist() == chain[1:]      # the chain's three tokens and the token after them
        assert all(int(m) >> int(n) == 0 for m, n in zip(masks, lane_rows[:, 1]))       # nothing past a lane's own rows
        # the context rows the commit computed, and where the kept ones went
        context = draft.buffer(verify.DFLASH_CONTEXT_HIDDEN).download(np.uint16)[:lanes_n * cap * H].reshape(lanes_n * cap, H)
        rows = captured.download(np.uint16)[:lanes_n * cap * 2 * H].reshape(lanes_n * cap, 2 * H)
        assert np.array_equal(rows[:, H:], target.buffer(verify.HIDDEN, 0).download(np.uint16)[:lanes_n * cap * H].reshape(lanes_n * cap, H))
        close_rows(context, draft_model.oracle_context_hidden(rows), "context rows")
        after = draft.buffer(verify.DFLASH_RINGS).download(np.uint16)
        cosines, sines = (np.concatenate([t[i] for t in tables]) for i in (0, 1))
        for lane in range(lanes_n):
            path = np.array([bit for bit in range(cap) if masks[lane] >> bit & 1])
            assert len(path) == retained[lane]
            slots = (committed[lane] + np.arange(len(path))) % WINDOW
            for layer in range(draft_model.layer_count):
                keys, values = (a.copy() for a in ring_view(before, draft_model, lane, layer))
                orc.draft_context_write(draft_model.oracle_context_kv(context, layer), draft_model.layers[layer]["key_norm"], cosines, sines,
                                        lane * cap + path, committed[lane] + np.arange(len(path)), 16 * lane + np.arange(len(path)), keys, values)
                got_keys, got_values = ring_view(after, draft_model, lane, layer)
                close_rows(got_keys[:, slots], keys[:, slots], f"cycle {cycle} lane {lane} keys of layer {layer}", ulp=3, fraction=0.03)
                close_rows(got_values[:, :, slots], values[:, :, slots], f"cycle {cycle} lane {lane} values of layer {layer}")
                others = np.setdiff1d(np.arange(WINDOW), slots)
                assert np.array_equal(got_keys[:, others], keys[:, others]) and np.array_equal(got_values[:, :, others], values[:, :, others])
        # the host's part of a cycle: each lane moves on by what it kept, from the last token it kept
        for lane in range(lanes_n):
            committed[lane] += int(retained[lane])
            anchors[lane] = int(selected[lane * cap + int(retained[lane]) - 1])
            total_kept += int(retained[lane])
    assert sum(committed) == sum(prompts) + total_kept and total_kept >= 2 * lanes_n
    draft.close()


def test_a_hybrid_targets_cycles_fold_what_each_lane_kept(backend):
    """The same cycles over the hybrid target (Gated DeltaNet and attention layers, a mixture of experts): a lane's next
    step folds, from the tape of the step before, the path whose mask that step's acceptance left, at the other parity;
    the draft's context takes the same mask's rows of the hidden rows the hybrid's layers captured. Three cycles of two
    lanes, lane 0 with a host chain the target accepts."""
    from tests.hybrid_reference import HybridModel
    print("case draft and hybrid target cycles", flush=True)
    shape = dict(hidden=256, vocabulary=1024, layers=4, q_heads=8, kv_heads=2, head_dim=128, gdn_key_heads=2, gdn_value_heads=4,
                 experts=16, top_k=2, expert_ffn=256)
    V, H, cap, lanes_n = shape["vocabulary"], shape["hidden"], 16, 2
    prompts = (50, 23)
    target_model = HybridModel(seed=45, **shape)
    draft_model = DraftModel(seed=46, hidden=H, vocabulary=V, intermediate=512, layers=2, target_layers=2)
    draft_model.head = target_model.head
    rng = np.random.default_rng(47)
    target = target_model.build_gpu(backend, max_lanes=lanes_n, pages_per_lane=2, prefill_rows=64)
    draft = draft_model.build_gpu(backend, max_lanes=lanes_n, context_rows=64)
    captured = draft.buffer(verify.DFLASH_CAPTURED_TARGET_HIDDEN)
    target.set_capture([1, 3], captured)
    up = backend.from_array
    table_first = [lane * target_model.pages_per_lane for lane in range(lanes_n)]

    # ---- the prompts: every layer of the hybrid (its GDN layers from the lane's cell 0 to its cell 1), captured rows into the draft
    committed, parity = [0, 0], [1, 1]           # after the prompt a lane's state lies in its cell 1
    for lane, count in enumerate(prompts):
        target.set_prefill_block(rng.integers(0, V, count).astype(np.uint32))
        backend.run(target.encode_prefill(lane, table_first[lane], 0, count, parity=0))
        cosines, sines = rope_tables(np.arange(count))
        draft.buffer(verify.DFLASH_CONTEXT_ROPE_COS).upload(cosines)
        draft.buffer(verify.DFLASH_CONTEXT_ROPE_SIN).upload(sines)
        backend.run(draft.encode_context_prefill(lane, count, 0))
        committed[lane] = count

    codebooks = [up(bits(rng.standard_normal((V, 256)) * 0.08)) for _ in range(2)]
    b = dict(candidates=backend.allocate_buffer(lanes_n * 7 * 16 * 4), unary=backend.allocate_buffer(lanes_n * 7 * 16 * 4),
             edges=backend.allocate_buffer(lanes_n * 7 * 256 * 4), scratch=backend.allocate_buffer(max(ops.DraftSelector.candidate_scratch_bytes(lanes_n, V), 16)),
             tokens=backend.allocate_buffer(128), trees=backend.allocate_buffer(256), scores=backend.allocate_buffer(256), sizes=backend.allocate_buffer(16),
             draws=backend.allocate_buffer(128), next=backend.allocate_buffer(2048), caps=backend.allocate_buffer(128), lane_rows=backend.allocate_buffer(16),
             sources=backend.allocate_buffer(128), ids=backend.allocate_buffer(32 * 16 * 4), q=backend.allocate_buffer(32 * 16 * 4),
             drawn=backend.allocate_buffer(32 * 4))
    anchors = [int(t) for t in rng.integers(0, V, lanes_n)]
    pending = [0, 0]
    embedding = up(target_model.embedding)
    hidden0 = draft.buffer(verify.DFLASH_HIDDEN, 0)
    kept_history = []
    for cycle in range(3):
        print(f"  cycle {cycle}: committed {committed}, parity {parity}, pending {[bin(m) for m in pending]}", flush=True)
        tables = [rope_tables(c + np.arange(16)) for c in committed]
        for which, index in ((verify.DFLASH_ROPE_COS, 0), (verify.DFLASH_ROPE_SIN, 1), (verify.DFLASH_CONTEXT_ROPE_COS, 0), (verify.DFLASH_CONTEXT_ROPE_SIN, 1)):
            draft.buffer(which).upload(np.concatenate([t[index] for t in tables]))
        lane_of = lambda i, rows: verify.HybridLane(rows, committed[i], table_first=table_first[i], pending_path=pending[i], parity=parity[i])
        # lane 0's host chain: the target's own continuation of its anchor, by chain steps that commit nothing and write
        # only what the real step writes again (the folded cell and the step's tape)
        chain = [anchors[0]]
        for _ in range(3):
            alone = [lane_of(0, len(chain))]
            target.set_block(alone, np.array(chain, np.uint32))
            backend.run(target.encode(alone, commit=False))
            chain.append(int(target.results(alone)[0][len(chain) - 1]))
        chain_tokens = np.zeros((lanes_n, 15), np.uint32)
        chain_tokens[0, :3] = chain[1:]
        chain_rates = np.zeros((lanes_n, 15, 4), np.float32)
        chain_rates[0, :3] = 0.97
        lanes = [lane_of(i, cap) for i in range(lanes_n)]
        graph = splash_amd.CommandGraph()
        for lane, anchor in enumerate(anchors):
            ops.Embedding.add(graph, orc.FMT_Q4K, embedding, V, H, up(np.array([anchor], np.uint32)), hidden0.view(lane * 8 * H * 2, H * 2), 1)
        draft.encode_decode(committed, graph=graph)
        ops.DraftSelector.add_candidates(graph, draft.buffer(verify.DFLASH_LOGITS), draft.buffer(verify.DFLASH_SELECTOR_HIDDEN), b["scratch"],
                                         b["candidates"], b["unary"], b["edges"], codebooks[0], codebooks[1], V, V, V, anchors)
        tree_lanes = [dict(anchor=anchors[0], depth=15, children=3, intercept=[0.3] * 7, chain=3),
                      dict(anchor=anchors[1], depth=6, children=2, intercept=[0.3] * 7)]
        ops.DraftSelector.add_tree(graph, b["candidates"], b["unary"], b["edges"], up(chain_tokens), up(chain_rates),
                                   b["tokens"], b["trees"], b["scores"], b["sizes"], b["draws"], b["next"], b["caps"], tree_lanes)
        ops.DraftSelector.add_verify_row_slots(graph, b["tokens"], b["trees"], b["scores"], b["sizes"], target.buffer(verify.INPUT_TOKENS),
                                               target.buffer(verify.TREE_ROWS), b["lane_rows"], b["sources"], lanes_n, cap)
        ops.DraftSelector.add_verify_children(graph, b["sources"], b["lane_rows"], target.buffer(verify.TREE_ROWS), b["candidates"], b["next"],
                                              b["draws"], b["ids"], b["q"], b["drawn"], target.buffer(verify.DEPTHS), lanes_n, lanes_n * cap)
        target.encode(lanes, commit=True, graph=graph)
        draft.encode_context_commit(target.buffer(verify.RETAINED_ROWS), b["lane_rows"], committed, lanes_n * cap, cap, graph=graph)
        before = draft.buffer(verify.DFLASH_RINGS).download(np.uint16)
        # what the fold of this step must leave: the state before the pending path, and the tape that path's rows lie on
        gdn = range(target.gdn_layers)
        old_cells = [[target_model.read_cell(i, parity[i], g) for g in gdn] for i in range(lanes_n)]
        old_tapes = [[target_model.read_tape(i, parity[i] ^ 1, g) for g in gdn] for i in range(lanes_n)]
        backend.run(graph)

        selected, retained, accepted, masks = (np.array(a).copy() for a in target.results(lanes))
        lane_rows = b["lane_rows"].download(np.uint32)[:2 * lanes_n].reshape(lanes_n, 2)
        print(f"    trees of {lane_rows[:, 1].tolist()} rows; kept {retained.tolist()} (masks {[bin(m) for m in masks]})", flush=True)
        assert retained[0] == 4 and selected[:3].tolist() == chain[1:] and retained[1] >= 1
        # the recurrent state the step started from: the cell before, advanced along the path the step before kept, bit for bit
        for i in range(lanes_n):
            count = bin(pending[i]).count("1")
            for g in gdn:
                got_conv, got_state = target_model.read_cell(i, parity[i] ^ 1, g)
                if count:
                    rc, conv, state = orc.gdn_fold(target_model.gdn_shape, old_cells[i][g][0], old_cells[i][g][1], old_tapes[i][g], pending[i], count)
                    assert rc == 0
                else:
                    conv, state = old_cells[i][g]
                assert np.array_equal(conv, got_conv) and state.tobytes() == got_state.tobytes(), (cycle, i, g)
        # the draft's context: the kept rows of the captured rows, in the slots of their positions
        context = draft.buffer(verify.DFLASH_CONTEXT_HIDDEN).download(np.uint16)[:lanes_n * cap * H].reshape(lanes_n * cap, H)
        rows = captured.download(np.uint16)[:lanes_n * cap * 2 * H].reshape(lanes_n * cap, 2 * H)
        assert np.array_equal(rows[:, H:], target.buffer(verify.HIDDEN, 0).download(np.uint16, lanes_n * cap * H).reshape(lanes_n * cap, H))
        close_rows(context, draft_model.oracle_context_hidden(rows), "context rows")
        after = draft.buffer(verify.DFLASH_RINGS).download(np.uint16)
        cosines, sines = (np.concatenate([t[i] for t in tables]) for i in (0, 1))
        for lane in range(lanes_n):
            path = np.array([bit for bit in range(cap) if masks[lane] >> bit & 1])
            slots = (committed[lane] + np.arange(len(path))) % WINDOW
            for layer in range(draft_model.layer_count):
                keys, values = (a.copy() for a in ring_view(before, draft_model, lane, layer))
                orc.draft_context_write(draft_model.oracle_context_kv(context, layer), draft_model.layers[layer]["key_norm"], cosines, sines,
                                        lane * cap + path, committed[lane] + np.arange(len(path)), 16 * lane + np.arange(len(path)), keys, values)
                got_keys, got_values = ring_view(after, draft_model, lane, layer)
                close_rows(got_keys[:, slots], keys[:, slots], f"cycle {cycle} lane {lane} keys of layer {layer}", ulp=3, fraction=0.03)
                close_rows(got_values[:, :, slots], values[:, :, slots], f"cycle {cycle} lane {lane} values of layer {layer}")
        for lane in range(lanes_n):
            committed[lane] += int(retained[lane])
            anchors[lane] = int(selected[lane * cap + int(retained[lane]) - 1])
            pending[lane] = int(masks[lane])
            parity[lane] ^= 1
        kept_history.append(retained.tolist())
    assert committed == [prompts[0] + 12, prompts[1] + sum(k[1] for k in kept_history)]
    draft.close()
