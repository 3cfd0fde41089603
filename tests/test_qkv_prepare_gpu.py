"""GPU tests of the q|k|v projection that prepares its attention block from its epilogue
(ops::PagedAttention::addFusedProjection) against the projection and the prepare kernel dispatched one after the other:
the packed rows, the staged queries, their sums and every byte of the pool are the same."""
import numpy as np
import pytest

import splash_amd
from splash_amd import ops
from tests import oracle as orc

pytestmark = pytest.mark.gpu

Q4, Q6 = ops.FMT_Q4K, ops.FMT_Q6K


class Block:
    """An attention block's projection at a geometry: `tensors` lists (format, heads) of the projection's segments."""

    def __init__(self, backend, linear, geometry, hidden, sequences, tensors, seed, pairs=None, normalize=True, splits=None):
        rng = np.random.default_rng(seed)
        self.backend, self.linear = backend, linear
        self.q_heads, self.kv_heads, self.D = q_heads, kv_heads, D = geometry
        self.rows = rows = sum(r for r, _ in sequences)
        self.width = width = (q_heads + 2 * kv_heads) * D
        parts = [(fmt, heads * D, orc.make_native(fmt, heads * D, hidden, seed + 1 + i)) for i, (fmt, heads) in enumerate(tensors)]
        assert sum(n for _, n, _ in parts) == width
        self.projection = ops.Projection.from_native(backend, parts, hidden)
        self.plan = linear.plan(self.projection, rows, splits=splits)
        self.pairs = pairs = D // 4 if pairs is None else pairs
        self.normalize = normalize
        # the sequences' pages, one table: sequence s's logical pages start at table_first[s]
        PT = ops.PAGE_TOKENS
        self.attention_rows, first_row, table_first = [], 0, 0
        for r, committed in sequences:
            self.attention_rows.append((first_row, r, committed, table_first))
            first_row += r
            table_first += (committed + r + PT - 1) // PT
        self.physical = table_first + 2
        self.table = rng.permutation(self.physical)[:table_first]
        self.attention = ops.AttentionPlan(q_heads, kv_heads, D, self.attention_rows, rotary_pairs=pairs, normalize=normalize)
        bits = lambda shape: orc.f32_to_bf16(rng.standard_normal(shape).astype(np.float32))
        self.input = backend.from_array(bits((rows, hidden)))
        self.query_norm = backend.from_array(orc.f32_to_bf16((1 + 0.1 * rng.standard_normal(D)).astype(np.float32)))
        self.key_norm = backend.from_array(orc.f32_to_bf16((1 + 0.1 * rng.standard_normal(D)).astype(np.float32)))
        angles = rng.uniform(0, 6.28, (rows, max(pairs, 1))).astype(np.float32)
        self.cos, self.sin = backend.from_array(np.cos(angles).astype(np.float32)), backend.from_array(np.sin(angles).astype(np.float32))
        self.pool_bytes = rng.integers(0, 256, (self.physical, ops.kv_page_bytes(kv_heads, D)), dtype=np.uint8)
        # partials whatever the plan's parts: parts x 64-column workgroups x storage rows x 256 bytes; a counter a workgroup
        groups = width // 64
        self.scratch = ops.LinearScratch(backend, ops.gguf_table_bytes(hidden, rows),
                                         max(self.plan.scratch_partials, self.plan.splits * groups * self.plan.storage_rows * 256), groups * 4)
        self.scratch.counters.fill(0)

    def fuses(self):
        return ops.PagedAttention.fuses_projection(self.attention, self.projection, self.plan)

    def run(self, fused, runs=1):
        b = self.backend
        kv = ops.KvPages(b, self.kv_heads, self.D, self.physical, self.table)
        ws = ops.AttentionWorkspace(b, self.attention)
        packed = b.allocate_buffer(self.rows * self.width * 2)
        extras = dict(query_norm=self.query_norm if self.normalize else None, key_norm=self.key_norm if self.normalize else None,
                      rope_cos=self.cos if self.pairs else None, rope_sin=self.sin if self.pairs else None)
        link = dict(projection=self.projection, plan=self.plan, input=self.input, output=packed, scratch=self.scratch)
        graph = splash_amd.CommandGraph()
        if fused:
            ops.PagedAttention.add_fused_projection(graph, self.linear, self.attention, ws, kv, **extras, **link)
            assert len(graph) == 2      # the table pass and the projection
        else:
            self.linear.add_link(graph, **link)
            ops.PagedAttention.add_projection(graph, self.attention, packed, ws, kv, **extras)
            assert len(graph) == 3
        results = []
        for _ in range(runs):
            kv.upload(self.pool_bytes)
            for buffer in (packed, ws.queries, ws.query_sums):
                buffer.fill(0xEE)
            b.run(graph)
            results.append(dict(packed=packed.download(np.uint16).copy(), queries=ws.queries.download(np.uint16).copy(),
                                sums=ws.query_sums.download(np.uint32).copy(), pool=kv.download().copy()))
        assert not self.scratch.counters.download(np.uint32).any()    # every count returned to zero
        return results


@pytest.mark.parametrize("geometry,hidden,sequences,tensors", [
    ((16, 4, 128), 1024, [(16, 250)], [(Q4, 24)]),                                   # one tensor; the block crosses a page
    ((16, 8, 64), 1024, [(7, 1000)], [(Q6, 16), (Q6, 8), (Q6, 8)]),                   # heads of 64, three tensors of a format
    ((32, 4, 128), 1024, [(16, 0), (8, 300), (16, 4090)], [(Q4, 32), (Q4, 4), (Q6, 4)]),  # several formats, three sequences, 40 rows
    ((16, 4, 128), 2048, [(16, 77), (16, 5), (16, 600), (16, 255)], [(ops.FMT_Q5K, 16), (ops.FMT_Q80, 4), (ops.FMT_IQ4XS, 4)]),  # 64 rows
    ((64, 8, 128), 5120, [(16, 32752)], [(Q4, 64), (Q4, 8), (Q6, 8)]),                # the 27B target's block
    ((64, 8, 128), 5120, [(1, 100)], [(Q4, 80)]),                                     # one row
])
def test_the_fused_projection_equals_the_two_dispatches(backend, geometry, hidden, sequences, tensors):
    print(f"case qkv prepare geometry={geometry} hidden={hidden} sequences={sequences} tensors={tensors}", flush=True)
    linear = ops.Linear(backend)
    block = Block(backend, linear, geometry, hidden, sequences, tensors, seed=hidden + geometry[0] + len(sequences))
    assert block.fuses()
    want = block.run(fused=False)[0]
    for run, got in enumerate(block.run(fused=True, runs=3)):
        for name in want:
            assert np.array_equal(got[name], want[name]), (run, name, int((got[name] != want[name]).sum()))
    # the block's slots changed and nothing else of the pool did
    changed = (want["pool"] != block.pool_bytes).any(axis=1)
    slots = {int(block.table[t + (c + r) // ops.PAGE_TOKENS]) for (_, rows, c, t) in block.attention_rows for r in range(rows)}
    assert set(np.flatnonzero(changed)) <= slots and changed.any()


@pytest.mark.parametrize("pairs,normalize,splits", [(0, False, None), (32, False, 1), (0, True, 2), (64, True, 1)])
def test_without_norms_or_rope_and_unsplit(backend, pairs, normalize, splits):
    """The block's options one by one, and a plan of one part of K (the workgroups still meet at the head's counter)."""
    print(f"case qkv prepare options pairs={pairs} normalize={normalize} splits={splits}", flush=True)
    linear = ops.Linear(backend)
    block = Block(backend, linear, (16, 4, 128), 1024, [(5, 300), (16, 10)], [(Q4, 16), (Q6, 8)], seed=pairs + 3, pairs=pairs,
                  normalize=normalize, splits=splits)
    assert block.fuses() and (splits is None or block.plan.splits == splits)
    want = block.run(fused=False)[0]
    for got in block.run(fused=True, runs=2):
        for name in want:
            assert np.array_equal(got[name], want[name]), name


def test_pairs_the_kernels_do_not_take(backend):
    linear = ops.Linear(backend)
    # more rows than one piece
    tall = Block(backend, linear, (16, 4, 128), 1024, [(16, 0)] * 5, [(Q4, 24)], seed=1)
    assert not tall.fuses()
    # a tensor that ends inside a head
    split_head = Block(backend, linear, (16, 4, 128), 1024, [(16, 0)], [(Q4, 24)], seed=2)
    parts = [(Q4, 64, orc.make_native(Q4, 64, 1024, 5)), (Q4, 24 * 128 - 64, orc.make_native(Q4, 24 * 128 - 64, 1024, 6))]
    split_head.projection = ops.Projection.from_native(backend, parts, 1024)
    split_head.plan = linear.plan(split_head.projection, 16)
    assert not split_head.fuses()
    # INT8 query codes
    coded = Block(backend, linear, (16, 4, 128), 1024, [(16, 0)], [(Q4, 24)], seed=3)
    coded.attention = ops.AttentionPlan(16, 4, 128, coded.attention_rows, rotary_pairs=32, normalize=True, int8_queries=True)
    assert not coded.fuses()
    with pytest.raises(splash_amd.SplashError):
        coded.run(fused=True)
    # another block's geometry
    other = Block(backend, linear, (16, 4, 128), 1024, [(16, 0)], [(Q4, 24)], seed=4)
    other.attention = ops.AttentionPlan(64, 8, 128, other.attention_rows, rotary_pairs=32, normalize=True)
    assert not other.fuses()
    # partials of the plan's own size do not hold an unsplit plan's sums
    small = Block(backend, linear, (16, 4, 128), 1024, [(16, 0)], [(Q4, 24)], seed=5, splits=1)
    small.scratch = ops.LinearScratch(backend, ops.gguf_table_bytes(1024, 16), 4096, 24 * 2 * 4)
    with pytest.raises(splash_amd.SplashError):
        small.run(fused=True)
