"""GPU tests of chained projections (ops::Linear::addChain): a layer's output projection, gate/up pair, down projection
and the projection after it as one dispatch, against the same four dispatched one by one."""
from types import SimpleNamespace

import numpy as np
import pytest

import splash_amd
from splash_amd import ops
from tests import oracle as orc

pytestmark = pytest.mark.gpu


class Tail:
    """A layer's projections after its attention at a given shape, with buffers of their own for every link."""

    def __init__(self, backend, linear, hidden, attention, ffn, following, rows, formats, seed, float32_following=False):
        rng = np.random.default_rng(seed)
        self.backend, self.linear, self.rows = backend, linear, rows
        self.widths = dict(hidden=hidden, attention=attention, ffn=ffn, following=following)
        f_o, f_gu, f_down, f_next = formats
        make = lambda fmt, n, k, s, **kw: ops.Projection.from_native(backend, [(fmt, n, orc.make_native(fmt, n, k, s))], k, **kw)
        self.output = make(f_o, hidden, attention, seed + 1)
        self.gate, self.up = make(f_gu, ffn, hidden, seed + 2), make(f_gu, ffn, hidden, seed + 3)
        self.down = make(f_down, hidden, ffn, seed + 4)
        if isinstance(f_next, (list, tuple)):   # segments of several formats
            parts = [(fmt, n, orc.make_native(fmt, n, hidden, seed + 5 + i)) for i, (fmt, n) in enumerate(f_next)]
            assert sum(n for _, n, _ in parts) == following
            self.following = ops.Projection.from_native(backend, parts, hidden)
        else:
            self.following = make(f_next, following, hidden, seed + 5, float32=float32_following)
        self.float32_following = float32_following
        bits = lambda shape, scale=1.0: orc.f32_to_bf16((scale * rng.standard_normal(shape)).astype(np.float32))
        self.attention_rows = backend.from_array(bits((rows, attention)))
        self.residual = backend.from_array(bits((rows, hidden)))
        self.next_norm = backend.from_array(orc.f32_to_bf16((1 + 0.1 * rng.standard_normal(hidden)).astype(np.float32)))
        self.post_norm = backend.from_array(orc.f32_to_bf16((1 + 0.1 * rng.standard_normal(hidden)).astype(np.float32)))
        self.plans = [linear.plan(self.output, rows, ops.EPILOGUE_RESIDUAL_NORM), linear.plan(self.up, rows, ops.EPILOGUE_GATE_UP),
                      linear.plan(self.down, rows, ops.EPILOGUE_RESIDUAL_NORM), linear.plan(self.following, rows)]
        table = lambda k: ops.gguf_table_bytes(k, rows)
        self.scratch = [ops.LinearScratch(backend, table(k), p.scratch_partials, p.scratch_counters)
                        for k, p in zip((attention, hidden, ffn, hidden), self.plans)]
        self.normalized = backend.allocate_buffer(rows * hidden * 2)   # names the rows a table stands for; never read

    def outputs(self):
        w, rows, b = self.widths, self.rows, self.backend
        return dict(hidden1=b.allocate_buffer(rows * w["hidden"] * 2), intermediate=b.allocate_buffer(rows * w["ffn"] * 2),
                    hidden2=b.allocate_buffer(rows * w["hidden"] * 2),
                    following=b.allocate_buffer(rows * w["following"] * (4 if self.float32_following else 2)))

    def links(self, out):
        s = self.scratch
        return [dict(projection=self.output, plan=self.plans[0], input=self.attention_rows, output=out["hidden1"], scratch=s[0],
                     residual=self.residual, prepared=ops.PREPARED_TABLE, norm_weight=self.post_norm, next_table=s[1].table),
                dict(projection=self.up, gate=self.gate, plan=self.plans[1], input=self.normalized, output=out["intermediate"],
                     scratch=s[1], prepared=ops.PREPARED_UNSCALED, next_table=s[2].table),
                dict(projection=self.down, plan=self.plans[2], input=out["intermediate"], output=out["hidden2"], scratch=s[2],
                     residual=out["hidden1"], prepared=ops.PREPARED_TABLE, norm_weight=self.next_norm, next_table=s[3].table),
                dict(projection=self.following, plan=self.plans[3], input=self.normalized, output=out["following"], scratch=s[3],
                     prepared=ops.PREPARED_UNSCALED)]

    def one_by_one(self):
        """Also leaves the first link's table, of the attention rows, where the chain finds it (an attention merge
        would have written it)."""
        out = self.outputs()
        graph = splash_amd.CommandGraph()
        links = self.links(out)
        self.linear.add_link(graph, **dict(links[0], prepared=0))
        for link in links[1:]:
            self.linear.add_link(graph, **link)
        assert len(graph) == 5      # the first link's table pass and the four projections
        self.backend.run(graph)
        return {k: v.download(np.uint8).copy() for k, v in out.items()}

    def chained(self, progress, count=4, runs=1):
        out = self.outputs()
        graph = splash_amd.CommandGraph()
        self.linear.add_chain(graph, self.links(out)[:count], progress)
        assert len(graph) == 1
        results = []
        for _ in range(runs):
            for buffer in out.values():
                buffer.fill(0xEE)
            self.backend.run(graph)
            results.append({k: v.download(np.uint8).copy() for k, v in out.items()})
        return results


def progress_words(backend):
    progress = backend.allocate_buffer(ops.Linear.CHAIN_PROGRESS_BYTES)
    progress.fill(0)
    return progress


Q4, Q6 = ops.FMT_Q4K, ops.FMT_Q6K


@pytest.mark.parametrize("shape,rows,formats", [
    ((1024, 1024, 2048, 1536), 16, (Q4, Q4, Q6, Q4)),
    ((1024, 1024, 2048, 1536), 5, (Q6, Q4, Q4, Q6)),
    ((1024, 2048, 3072, 1024), 40, (Q4, Q4, Q6, Q4)),
    ((1024, 1024, 2048, 1536), 64, (ops.FMT_Q5K, ops.FMT_IQ4XS, ops.FMT_Q80, ops.FMT_IQ4NL)),
    ((1024, 1024, 2048, 1536), 16, (Q4, Q4, Q6, [(Q4, 1024), (Q6, 512)])),
    ((5120, 8192, 17408, 10240), 16, (Q4, Q4, Q6, Q4)),
])
def test_a_chain_equals_its_links_one_by_one(backend, shape, rows, formats):
    """Bit for bit, on every output of every link and on five runs in a row (the counts return to zero by themselves)."""
    print(f"case chain shape={shape} rows={rows} formats={formats}", flush=True)
    linear = ops.Linear(backend)
    tail = Tail(backend, linear, *shape, rows, formats, seed=rows + shape[0])
    want = tail.one_by_one()
    progress = progress_words(backend)
    for run, got in enumerate(tail.chained(progress, runs=5)):
        for name in want:
            assert np.array_equal(got[name], want[name]), (run, name)
        assert not progress.download(np.uint32).any(), run


def test_a_chain_ends_with_the_head(backend):
    """The last layer's chain: output, gate/up, down, then a wide fp32 projection of the final norm's rows."""
    print("case chain with an fp32 head", flush=True)
    linear = ops.Linear(backend)
    tail = Tail(backend, linear, 1024, 1024, 2048, 32000, 16, (Q4, Q4, Q4, Q6), seed=3, float32_following=True)
    want = tail.one_by_one()
    progress = progress_words(backend)
    for got in tail.chained(progress, runs=3):
        for name in want:
            assert np.array_equal(got[name], want[name]), name


@pytest.mark.parametrize("count", [1, 2, 3])
def test_shorter_chains(backend, count):
    print(f"case chain of {count} links", flush=True)
    linear = ops.Linear(backend)
    tail = Tail(backend, linear, 1024, 1024, 2048, 1536, 16, (Q4, Q4, Q6, Q4), seed=count)
    want = tail.one_by_one()
    progress = progress_words(backend)
    names = ["hidden1", "intermediate", "hidden2", "following"][:count]
    for got in tail.chained(progress, count=count, runs=3):
        for name in names:
            assert np.array_equal(got[name], want[name]), name
    assert not progress.download(np.uint32).any()


def test_a_wait_that_gives_up_says_so_and_ends(backend):
    """With no polls allowed, a workgroup that finds the link before it unfinished gives up at once: the dispatch ends
    like any other, the status word reads nonzero, and after the host has cleared the progress words the chain runs
    again with its results intact."""
    print("case chain whose waits give up", flush=True)
    linear = ops.Linear(backend)
    tail = Tail(backend, linear, 5120, 8192, 17408, 10240, 16, (Q4, Q4, Q6, Q4), seed=11)
    want = tail.one_by_one()
    progress = progress_words(backend)
    linear.set_chain_spin_limit(0)
    tail.chained(progress)
    words = progress.download(np.uint32)
    assert words[ops.Linear.CHAIN_STATUS_OFFSET // 4] == 1, words
    progress.fill(0)
    for scratch in tail.scratch:      # a link cut short may have left its split counters mid-count
        scratch.counters.fill(0)
    linear.set_chain_spin_limit(1 << 16)
    got, = tail.chained(progress)
    for name in want:
        assert np.array_equal(got[name], want[name]), name
    assert not progress.download(np.uint32).any()


def test_chains_reject_what_would_race(backend):
    linear = ops.Linear(backend)
    tail = Tail(backend, linear, 1024, 1024, 2048, 1536, 16, (Q4, Q4, Q6, Q4), seed=5)
    out, progress = tail.outputs(), progress_words(backend)
    graph = splash_amd.CommandGraph()
    links = tail.links(out)
    with pytest.raises(splash_amd.SplashError, match="one to four"):
        linear.add_chain(graph, links + links[:1], progress)
    shared = [dict(l) for l in links]
    both = SimpleNamespace(table=links[1]["scratch"].table, partials=links[3]["scratch"].partials, counters=links[3]["scratch"].counters)
    shared[3]["scratch"] = both                           # the fourth link reads the second's table
    with pytest.raises(splash_amd.SplashError, match="tables of their own"):
        linear.add_chain(graph, shared, progress)
    unprepared = [dict(l) for l in links]
    unprepared[1]["prepared"] = 0
    with pytest.raises(splash_amd.SplashError, match="already there"):
        linear.add_chain(graph, unprepared, progress)
    plain_residual = [dict(l) for l in links]
    plain_residual[2] = dict(links[2], plan=linear.plan(tail.down, tail.rows, ops.EPILOGUE_RESIDUAL), norm_weight=None, next_table=None)
    with pytest.raises(splash_amd.SplashError, match="norms its rows"):
        linear.add_chain(graph, plain_residual[:3], progress)
    taller = [dict(l) for l in links]
    taller[3] = dict(links[3], plan=linear.plan(tail.following, 40))
    with pytest.raises(splash_amd.SplashError, match="one tile height"):
        linear.add_chain(graph, taller, progress)
    with pytest.raises(splash_amd.SplashError, match="chain progress"):
        linear.add_chain(graph, links, backend.allocate_buffer(8))
    assert len(graph) == 0
