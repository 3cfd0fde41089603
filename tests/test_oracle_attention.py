"""The oracle's KV store and attention against the reference's closed forms and invariants (CPU)."""
import numpy as np
import pytest

from tests import oracle as orc


@pytest.mark.skipif(orc.ref is None, reason="oracle/_ref was not built (no reference tree)")
def test_kv_store_rule_equals_compiled_reference():
    """Q8PageFormatReference.hpp:107-122 storedScale / quantize, value by value."""
    orc.ref.ref_kv_scale.restype = orc.c_f
    orc.ref.ref_kv_scale.argtypes = [orc.c_f]
    orc.ref.ref_kv_code.restype = orc.c_int
    orc.ref.ref_kv_code.argtypes = [orc.c_f, orc.c_f]
    rng = np.random.default_rng(2)
    for D in (64, 128):
        v = rng.standard_normal((40, D)).astype(np.float32)
        v[3] = 0
        v[4, 7] = 100.0
        codes, scales = orc.kv_quantize(v, half_scale=False)
        for r in range(v.shape[0]):
            mx = float(np.max(np.abs(v[r])))
            assert scales[r] == orc.ref.ref_kv_scale(mx)
            for d in range(D):
                assert codes[r, d] == orc.ref.ref_kv_code(float(v[r, d]), mx)
        # the fp16 scale is the rounded fp32 scale
        _, half = orc.kv_quantize(v, half_scale=True)
        assert np.array_equal(half, scales.astype(np.float16).astype(np.float32))


def make_case(rng, q_heads, kv_heads, D, rows, committed, pages_extra=1):
    PT = 256
    total = committed + rows
    pages = (total + PT - 1) // PT
    phys = pages + pages_extra
    table = rng.permutation(phys)[:pages].astype(np.uint32)
    k = rng.standard_normal((phys, kv_heads, PT, D)).astype(np.float32)
    v = rng.standard_normal((phys, kv_heads, PT, D)).astype(np.float32)
    kc, ks = orc.kv_quantize(k)
    vc, vs = orc.kv_quantize(v)
    q = orc.f32_to_bf16(rng.standard_normal((rows, q_heads, D)).astype(np.float32))
    anc = np.array([(2 << r) - 1 for r in range(rows)], dtype=np.uint32)
    return q, kc, ks, vc, vs, table, anc


def dense_reference(q, kc, ks, vc, vs, table, anc, committed):
    """Textbook softmax attention in numpy fp64 over the dequantized cache: what the page loop must equal."""
    rows, q_heads, D = q.shape
    kv_heads, PT = kc.shape[1], kc.shape[2]
    total = committed + rows
    K = np.concatenate([kc[p].astype(np.float64) * ks[p][..., None] for p in table], axis=1)[:, :total]
    V = np.concatenate([vc[p].astype(np.float64) * vs[p][..., None] for p in table], axis=1)[:, :total]
    out = np.zeros((rows, q_heads, D))
    group = q_heads // kv_heads
    qf = orc.bf16_to_f32(q).astype(np.float64)
    for r in range(rows):
        vis = np.array([t < committed or ((int(anc[r]) >> (t - committed)) & 1) for t in range(total)], dtype=bool)
        for h in range(q_heads):
            s = (K[h // group] @ qf[r, h]) / np.sqrt(D)
            s[~vis] = -np.inf
            p = np.exp(s - s.max())
            out[r, h] = (p / p.sum()) @ V[h // group]
    return out


@pytest.mark.parametrize("committed,splits,pps", [(0, 1, 99), (200, 1, 99), (700, 1, 99), (700, 3, 1), (1500, 4, 2)])
def test_page_loop_equals_dense_softmax(committed, splits, pps):
    """ctx = 0 and single-page cases reduce to dense softmax; splits merge to the same result."""
    rng = np.random.default_rng(committed + splits)
    q, kc, ks, vc, vs, table, anc = make_case(rng, 4, 2, 64, 5, committed)
    got, got64 = orc.attention(q, kc, ks, vc, vs, table, anc, committed, splits=splits, pages_per_split=pps)
    ref = dense_reference(q, kc, ks, vc, vs, table, anc, committed)
    assert np.allclose(got64, ref, rtol=1e-9, atol=1e-12)
    g = orc.bf16_to_f32(got).astype(np.float64)
    cos = (g * ref).sum() / np.sqrt((g * g).sum() * (ref * ref).sum())
    # the reference's gate against the fp64 reference on stored pages (q8_flash_attention_metal_test.mm:788-799)
    assert cos > 0.9995 and np.abs(g - ref).max() < 0.02


def test_page_table_permutation_and_tree_rows():
    """Permuting the page table with its pages changes nothing; a tree row equals the chain of its path."""
    rng = np.random.default_rng(8)
    q, kc, ks, vc, vs, table, anc = make_case(rng, 4, 2, 64, 6, 300, pages_extra=3)
    base, _ = orc.attention(q, kc, ks, vc, vs, table, anc, 300, splits=2, pages_per_split=1)
    perm = rng.permutation(kc.shape[0])
    inv = np.argsort(perm)
    moved, _ = orc.attention(q, kc[perm], ks[perm], vc[perm], vs[perm], inv[table].astype(np.uint32), anc, 300, splits=2,
                             pages_per_split=1)
    assert np.array_equal(base, moved)
    # tree: row 3 branches from row 1 (path 0, 1, 3): it must equal a chain block whose third row is row 3's K/V/q
    tree_anc = anc.copy()
    tree_anc[3] = 0b1011
    tree, _ = orc.attention(q, kc, ks, vc, vs, table, tree_anc, 300)
    kc2, ks2, vc2, vs2 = kc.copy(), ks.copy(), vc.copy(), vs.copy()
    PT = 256
    def slot(t):
        return table[t // PT], t % PT
    p3, t3 = slot(303)
    p2, t2 = slot(302)
    for arr in (kc2, vc2):
        arr[p2, :, t2] = arr[p3, :, t3]
    for arr in (ks2, vs2):
        arr[p2, :, t2] = arr[p3, :, t3]
    q2 = q.copy()
    q2[2] = q[3]
    chain, _ = orc.attention(q2, kc2, ks2, vc2, vs2, table, anc, 300)
    assert np.array_equal(tree[3], chain[2])


def test_int8_activation_block_follows_its_closed_form():
    """common/int8_activations.h:22-28: code = clamp(rint(x * (127 / m))) with the quotient rounded first, scale = m / 127;
    a block at or below 2^-100 codes as zeros with scale 0; a block holding an infinity or a NaN takes a NaN scale. Against
    numpy float32 arithmetic written from that rule (not from the oracle's code), and its invariants."""
    import numpy as np
    from tests import oracle as orc
    rng = np.random.default_rng(3)
    for _ in range(50):
        x = (rng.standard_normal(128) * rng.uniform(1e-3, 30)).astype(np.float32)
        codes, scale = orc.int8_activation_block(x)
        m = np.abs(x).max()
        inverse = np.float32(127.0) / m                                        # correctly rounded float32 quotient
        want = np.clip(np.rint(x * inverse), -127, 127).astype(np.int8)        # float32 product, ties to even
        assert np.array_equal(codes, want) and scale == np.float32(m) / np.float32(127.0)
        assert np.abs(codes).max() == 127                                      # the largest magnitude codes as +-127
        assert np.abs(codes.astype(np.float64) * scale - x).max() <= 0.5001 * scale   # a value restores within half a step
    # the quotient 127 / m is rounded before the product: for this pair x * (127 / m) rounds to 112, where x * 127 / m
    # (the KV store's order of operations) would give 113
    m, x = np.float32(0.5596824884414673), np.float32(0.4957817494869232)
    assert np.rint(x * (np.float32(127) / m)) == 112 and np.rint(x * np.float32(127) / m) == 113
    codes, scale = orc.int8_activation_block(np.array([m, x, -x], np.float32))
    assert list(codes) == [127, 112, -112] and scale == m / np.float32(127.0)
    # ties go to even: with m = 127 the codes are rint(x)
    codes, _ = orc.int8_activation_block(np.array([127.0, 0.5, 1.5, 2.5, -0.5, -1.5], np.float32))
    assert list(codes) == [127, 0, 2, 2, 0, -2]
    codes, scale = orc.int8_activation_block(np.full(8, 2.0 ** -101, np.float32))
    assert not codes.any() and scale == 0.0
    codes, scale = orc.int8_activation_block(np.zeros(8, np.float32))
    assert not codes.any() and scale == 0.0
    for bad in (np.inf, -np.inf, np.nan):
        _, scale = orc.int8_activation_block(np.array([1.0, bad, 2.0], np.float32))
        assert np.isnan(scale)


def test_int8_query_attention_scores_the_codes_exactly():
    """paged_attention_tile.h:294-322: with INT8 queries the score product runs on the queries' codes and the row's scale
    multiplies it. On one page with unit key scales and a one-hot value per token the page loop's output is the softmax
    itself: it equals the fp64 softmax of (codes . keys) * qscale / sqrt(D); and against bf16 queries it stays inside the
    reference's attention gate."""
    import numpy as np
    from tests import oracle as orc
    rng = np.random.default_rng(4)
    q_heads, kv_heads, D, rows, committed = 4, 2, 64, 3, 40
    q = orc.f32_to_bf16(rng.standard_normal((rows, q_heads, D)).astype(np.float32))
    kc = rng.integers(-127, 128, (1, kv_heads, 256, D)).astype(np.int8)
    ks = np.full((1, kv_heads, 256), 0.02, np.float32)
    vc = np.zeros((1, kv_heads, 256, D), np.int8)
    for t in range(D):
        vc[0, :, t, t] = 100                                                   # token t's value is 100 e_t
    vs = np.full((1, kv_heads, 256), 0.01, np.float32)
    anc = np.array([(2 << r) - 1 for r in range(rows)], np.uint32)
    table = np.zeros(1, np.uint32)
    got, _ = orc.attention(q, kc, ks, vc, vs, table, anc, committed, int8_queries=True)
    exact, exact64 = orc.attention(q, kc, ks, vc, vs, table, anc, committed)
    got = orc.bf16_to_f32(got).astype(np.float64)
    for r in range(rows):
        for h in range(q_heads):
            codes, scale = orc.int8_activation_block(orc.bf16_to_f32(q[r, h]))
            visible = committed + r + 1
            s = (kc[0, h // 2, :visible].astype(np.int64) @ codes.astype(np.int64)).astype(np.float64) * scale * 0.02 / np.sqrt(D)
            p = np.exp(s - s.max()); p /= p.sum()
            want = np.zeros(D); want[:min(D, visible)] = p[:D]                 # P . V with V = e_t: the probabilities themselves
            assert np.abs(got[r, h] - want).max() <= 2.0 ** -8 * max(want.max(), 1e-3) + 1e-6
    cos = (got * exact64).sum() / np.sqrt((got ** 2).sum() * (exact64 ** 2).sum())
    assert cos >= 0.9995 and np.abs(got - exact64).max() < 0.02
