"""ctypes bindings of the CPU oracle (oracle/liboracle.so) and, where it was built, of the
reference's own header-only CPU references (oracle/_ref/libref.so). Test infrastructure only."""
import ctypes
import os

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FMT_Q4K, FMT_IQ4XS, FMT_IQ4NL, FMT_Q5K, FMT_Q6K, FMT_Q80 = 0, 1, 2, 3, 4, 6
FMT_Q3K, FMT_Q40, FMT_Q50 = 5, 15, 39   # the oracle dequantizes them; the kernels read them rewritten as Q6_K / Q8_0 blocks
ALL_FORMATS = [("q4k", FMT_Q4K), ("q6k", FMT_Q6K), ("q5k", FMT_Q5K), ("q80", FMT_Q80), ("iq4xs", FMT_IQ4XS), ("iq4nl", FMT_IQ4NL)]
NO_TOKEN = 0xFFFFFFFF

_path = os.path.join(ROOT, "oracle", "liboracle.so")
if not os.path.exists(_path):
    raise ImportError(f"{_path} is missing: run `make -C oracle` (or __graft_entry__.build())")
lib = ctypes.CDLL(_path)
_ref_path = os.path.join(ROOT, "oracle", "_ref", "libref.so")
ref = ctypes.CDLL(_ref_path) if os.path.exists(_ref_path) else None

u8p, u16p, u32p, f32p, f64p, i8p = (ctypes.POINTER(t) for t in (ctypes.c_uint8, ctypes.c_uint16, ctypes.c_uint32,
                                                             ctypes.c_float, ctypes.c_double, ctypes.c_int8))
c_u32, c_int, c_f = ctypes.c_uint32, ctypes.c_int, ctypes.c_float


def _p(a, t):
    return a.ctypes.data_as(t) if a is not None else None


lib.orc_f2h.restype = ctypes.c_uint16
lib.orc_f2h.argtypes = [c_f]
lib.orc_h2f.restype = c_f
lib.orc_h2f.argtypes = [ctypes.c_uint16]
lib.orc_f2bf.restype = ctypes.c_uint16
lib.orc_f2bf.argtypes = [c_f]
lib.orc_bf2f.restype = c_f
lib.orc_bf2f.argtypes = [ctypes.c_uint16]
lib.orc_row_bytes.restype = ctypes.c_uint64
lib.orc_row_bytes.argtypes = [c_u32, c_u32]
lib.orc_silu.restype = c_f
lib.orc_silu.argtypes = [c_f]
lib.orc_epilogue_swiglu.restype = ctypes.c_uint16
lib.orc_epilogue_swiglu.argtypes = [c_f, c_f]
lib.orc_epilogue_residual.restype = ctypes.c_uint16
lib.orc_epilogue_residual.argtypes = [c_f, ctypes.c_uint16]


def bf16_to_f32(bits):
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16(values):
    """Round to nearest even, as the kernels and the oracle do."""
    u = np.ascontiguousarray(values, dtype=np.float32).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r[nan] = ((u[nan] >> 16) | 0x40).astype(np.uint16)
    return r


def row_bytes(fmt, K):
    return lib.orc_row_bytes(fmt, K)


def fixture(fmt, rows, K, seed, library=None):
    out = np.empty(rows * row_bytes(fmt, K), dtype=np.uint8)
    fn = (library or lib).orc_fixture if library is None else library.ref_fixture
    assert fn(c_u32(fmt), c_u32(rows), c_u32(K), c_u32(seed), _p(out, u8p)) == 0
    return out


def make_native(fmt, rows, K, seed, library=None):
    out = np.empty(rows * row_bytes(fmt, K), dtype=np.uint8)
    fn = lib.orc_make_native if library is None else library.ref_make_native
    assert fn(c_u32(fmt), c_u32(rows), c_u32(K), c_u32(seed), _p(out, u8p)) == 0
    return out


def dequant_rows(fmt, native, rows, K, library=None):
    out = np.empty((rows, K), dtype=np.float32)
    fn = lib.orc_dequant_rows if library is None else library.ref_dequant_rows
    assert fn(c_u32(fmt), _p(native, u8p), c_u32(rows), c_u32(K), _p(out, f32p)) == 0
    return out


def quantize_rows(fmt, values):
    values = np.ascontiguousarray(values, dtype=np.float32)
    rows, K = values.shape
    out = np.empty(rows * row_bytes(fmt, K), dtype=np.uint8)
    assert lib.orc_quantize_rows(c_u32(fmt), _p(values, f32p), c_u32(rows), c_u32(K), _p(out, u8p)) == 0
    return out


def gemm(fmt, native, x_bf16, N, want=("exact", "bound", "chain"), threads=0):
    """x_bf16: uint16 [M][K]. Returns dict of exact (f64), bound (f64), chain (f32), each [M][N]."""
    x = np.ascontiguousarray(x_bf16, dtype=np.uint16)
    M, K = x.shape
    out = {}
    exact = np.empty((M, N), dtype=np.float64) if "exact" in want else None
    bound = np.empty((M, N), dtype=np.float64) if "bound" in want else None
    chain = np.empty((M, N), dtype=np.float32) if "chain" in want else None
    assert lib.orc_gemm(c_u32(fmt), _p(native, u8p), _p(x, u16p), c_u32(M), c_u32(K), c_u32(N), _p(exact, f64p),
                        _p(bound, f64p), _p(chain, f32p), c_int(threads)) == 0
    if exact is not None:
        out["exact"] = exact
    if bound is not None:
        out["bound"] = bound
    if chain is not None:
        out["chain"] = chain
    return out


def gemm_staged(fmt, native, x_bf16, N, threads=0):
    """The staged tile's projection. Returns dict of exact (f64), bound (f64: the reference's staged projectionBound),
    staged (f32: the fp64 dot with half-rounded weights) and accumulation (f64: the bound of the fp32 accumulation alone),
    each [M][N]."""
    x = np.ascontiguousarray(x_bf16, dtype=np.uint16)
    M, K = x.shape
    exact, bound = np.empty((M, N), dtype=np.float64), np.empty((M, N), dtype=np.float64)
    staged, accumulation = np.empty((M, N), dtype=np.float32), np.empty((M, N), dtype=np.float64)
    assert lib.orc_gemm_staged(c_u32(fmt), _p(native, u8p), _p(x, u16p), c_u32(M), c_u32(K), c_u32(N), _p(exact, f64p),
                               _p(bound, f64p), _p(staged, f32p), _p(accumulation, f64p), c_int(threads)) == 0
    return dict(exact=exact, bound=bound, staged=staged, accumulation=accumulation)


def gemv_column(fmt, native, x_bf16, N, threads=0):
    """The column tile's fp32 totals [M][N]: every addition in the reference's order."""
    x = np.ascontiguousarray(x_bf16, dtype=np.uint16)
    M, K = x.shape
    out = np.empty((M, N), dtype=np.float32)
    assert lib.orc_gemv_column(c_u32(fmt), _p(native, u8p), _p(x, u16p), c_u32(M), c_u32(K), c_u32(N), _p(out, f32p), c_int(threads)) == 0
    return out


lib.orc_float_projection.restype = None
lib.orc_float_projection.argtypes = [u16p, ctypes.c_void_p, c_u32, c_u32, c_u32, c_u32, f32p]


def float_projection(x_bits, weights):
    """fp32 [rows][n] = x (bf16 bits [rows][k]) times weights^T; weights float32 [n][k], or uint16 bf16 bits."""
    x = np.ascontiguousarray(x_bits, np.uint16)
    w = np.ascontiguousarray(weights)
    assert w.dtype in (np.float32, np.uint16) and w.shape[1] == x.shape[1]
    out = np.zeros((x.shape[0], w.shape[0]), np.float32)
    lib.orc_float_projection(_p(x, u16p), w.ctypes.data_as(ctypes.c_void_p), int(w.dtype == np.uint16), x.shape[0], w.shape[0], w.shape[1],
                             _p(out, f32p))
    return out


def rms_norm(x_bf16, w_bf16):
    x = np.ascontiguousarray(x_bf16, dtype=np.uint16)
    w = np.ascontiguousarray(w_bf16, dtype=np.uint16)
    out = np.empty_like(x)
    lib.orc_rms_norm(_p(x, u16p), _p(w, u16p), c_u32(x.shape[0]), c_u32(x.shape[1]), _p(out, u16p))
    return out


def embed(fmt, table, vocab, hidden, tokens):
    tokens = np.ascontiguousarray(tokens, dtype=np.uint32)
    out = np.empty((len(tokens), hidden), dtype=np.uint16)
    assert lib.orc_embed(c_u32(fmt), _p(table, u8p), c_u32(vocab), c_u32(hidden), _p(tokens, u32p), c_u32(len(tokens)),
                         _p(out, u16p)) == 0
    return out


def swiglu(gate_f32, up_f32):
    g = np.ascontiguousarray(gate_f32, dtype=np.float32).ravel()
    u = np.ascontiguousarray(up_f32, dtype=np.float32).ravel()
    out = np.empty(g.size, dtype=np.uint16)
    for i in range(g.size):
        out[i] = lib.orc_epilogue_swiglu(float(g[i]), float(u[i]))
    return out.reshape(np.shape(gate_f32))


def projection_interval(exact, bound):
    """[bf16(lo), bf16(hi)] of the reference's projection check (gguf_projection_test.mm:217-237)."""
    lo = bf16_to_f32(f32_to_bf16((exact - bound).astype(np.float32)))
    hi = bf16_to_f32(f32_to_bf16((exact + bound).astype(np.float32)))
    # float32 rounding of lo/hi before bf16 can move them inward by an fp32 ulp: widen by it.
    return np.nextafter(lo, -np.inf), np.nextafter(hi, np.inf)


class OrcAttention(ctypes.Structure):
    _fields_ = [("q_heads", c_u32), ("kv_heads", c_u32), ("head_dim", c_u32), ("rows", c_u32), ("committed", c_u32),
                ("page_tokens", c_u32), ("splits", c_u32), ("pages_per_split", c_u32), ("half_scale", c_u32), ("int8_queries", c_u32)]


def kv_quantize(values, half_scale=True):
    """values float32 [..., D] -> (codes int8 [..., D], scales float32 [...]) by the reference's store rule."""
    v = np.ascontiguousarray(values, dtype=np.float32)
    flat = v.reshape(-1, v.shape[-1])
    codes = np.empty(flat.shape, dtype=np.int8)
    scales = np.empty(flat.shape[0], dtype=np.float32)
    s = c_f()
    for i in range(flat.shape[0]):
        lib.orc_kv_quantize(_p(flat[i], f32p), c_u32(flat.shape[1]), c_int(int(half_scale)), _p(codes[i], i8p), ctypes.byref(s))
        scales[i] = s.value
    return codes.reshape(v.shape), scales.reshape(v.shape[:-1])


def attention_prepare(q_heads, kv_heads, head_dim, qkv_bits, qw, kw, cosv, sinv, pairs):
    rows = qkv_bits.shape[0]
    a = OrcAttention(q_heads, kv_heads, head_dim, rows, 0, 256, 1, 1, 1)
    q = np.empty((rows, q_heads, head_dim), dtype=np.uint16)
    k = np.empty((rows, kv_heads, head_dim), dtype=np.float32)
    v = np.empty((rows, kv_heads, head_dim), dtype=np.float32)
    qkv_bits = np.ascontiguousarray(qkv_bits, dtype=np.uint16)
    lib.orc_attention_prepare(ctypes.byref(a), _p(qkv_bits, u16p), _p(qw, u16p), _p(kw, u16p), _p(cosv, f32p), _p(sinv, f32p),
                              c_u32(pairs), _p(q, u16p), _p(k, f32p), _p(v, f32p))
    return q, k, v


def int8_activation_block(values):
    """common/int8_activations.h: (codes int8, scale) of one block of float32 values."""
    x = np.ascontiguousarray(values, np.float32).ravel()
    codes = np.empty(x.size, np.int8)
    scale = c_f()
    lib.orc_int8_activation_block(_p(x, f32p), c_u32(x.size), _p(codes, i8p), ctypes.byref(scale))
    return codes, scale.value


def attention(q_bits, kcodes, kscales, vcodes, vscales, page_table, ancestors, committed, splits=1, pages_per_split=1 << 20,
              want64=True, threads=0, int8_queries=False):
    """q_bits uint16 [rows][q_heads][D]; K/V logical pages [phys][kv_heads][256][D] int8, scales [phys][kv_heads][256]."""
    rows, q_heads, D = q_bits.shape
    kv_heads, PT = kcodes.shape[1], kcodes.shape[2]
    a = OrcAttention(q_heads, kv_heads, D, rows, committed, PT, splits, pages_per_split, 1, int(int8_queries))
    out = np.empty((rows, q_heads, D), dtype=np.uint16)
    out64 = np.empty((rows, q_heads, D), dtype=np.float64) if want64 else None
    q_bits = np.ascontiguousarray(q_bits, dtype=np.uint16)
    kcodes, vcodes = np.ascontiguousarray(kcodes, dtype=np.int8), np.ascontiguousarray(vcodes, dtype=np.int8)
    kscales, vscales = np.ascontiguousarray(kscales, dtype=np.float32), np.ascontiguousarray(vscales, dtype=np.float32)
    pt = np.ascontiguousarray(page_table, dtype=np.uint32)
    anc = np.ascontiguousarray(ancestors, dtype=np.uint32)
    lib.orc_attention(ctypes.byref(a), _p(q_bits, u16p), _p(kcodes, i8p), _p(kscales, f32p), _p(vcodes, i8p), _p(vscales, f32p),
                      _p(pt, u32p), _p(anc, u32p), _p(out, u16p), _p(out64, f64p), c_int(threads))
    return out, out64


class OrcTreeRow(ctypes.Structure):
    _fields_ = [("ancestors", c_u32), ("parent", ctypes.c_uint16), ("depth", ctypes.c_uint16)]


lib.orc_argmax.restype = c_u32


def argmax(logits):
    x = np.ascontiguousarray(logits, dtype=np.float32)
    return lib.orc_argmax(_p(x, f32p), c_u32(x.size))


def penalize(logits, words, input_tokens, ancestors, repetition=1.0, presence=0.0, frequency=0.0):
    """One lane's verify rows [rows][vocabulary] under the sampling penalties; returns the rewritten copy."""
    x = np.array(logits, dtype=np.float32, order="C")
    rows, vocabulary = x.shape
    w = np.ascontiguousarray(words, dtype=np.uint32)
    tokens = np.ascontiguousarray(input_tokens, dtype=np.uint32)
    paths = np.ascontiguousarray(ancestors, dtype=np.uint32)
    assert w.size == vocabulary and tokens.size == rows and paths.size == rows
    lib.orc_penalize.restype = None
    lib.orc_penalize(_p(x, f32p), c_u32(rows), c_u32(vocabulary), c_u32(vocabulary), _p(w, u32p), _p(tokens, u32p), _p(paths, u32p),
                     c_f(repetition), c_f(presence), c_f(frequency))
    return x


def thinking_cutoff(selected, input_tokens, tree, vocabulary, row, end, also_ends=NO_TOKEN, admits=None):
    """One lane's selections under its thinking cutoff; returns the rewritten copy. admits: per row, whether its
    constraint mask admits end[0] (an end that waits for its mask), or None."""
    rows = len(tree)
    nodes = (OrcTreeRow * rows)(*[OrcTreeRow(int(t["ancestors"]), int(t["parent"]), int(t["depth"])) for t in tree])
    out = np.array(selected, dtype=np.uint32)
    if row >= rows:
        return out
    tok = np.ascontiguousarray(input_tokens, dtype=np.uint32)
    ends = np.ascontiguousarray(end, dtype=np.uint32)
    count = min(len(ends), 16 - row)
    flags = None if admits is None else np.ascontiguousarray(admits, dtype=np.uint8)
    lib.orc_thinking_cutoff.restype = None
    lib.orc_thinking_cutoff(_p(out, u32p), _p(tok, u32p), nodes, c_u32(rows), c_u32(vocabulary), c_u32(row), _p(ends, u32p), c_u32(count),
                            c_u32(int(ends[-1])), c_u32(also_ends), None if flags is None else flags.ctypes.data_as(ctypes.c_void_p))
    return out


def accept_tree(tree, tokens, selected, remaining=0xFFFFFFFF, stop_tokens=()):
    """tree: structured array (ancestors, parent, depth). Returns (kept tokens, accepted, retained_rows)."""
    rows = len(tree)
    nodes = (OrcTreeRow * rows)(*[OrcTreeRow(int(t["ancestors"]), int(t["parent"]), int(t["depth"])) for t in tree])
    tok = np.ascontiguousarray(tokens, dtype=np.uint32)
    sel = np.ascontiguousarray(selected, dtype=np.uint32)
    stops = np.ascontiguousarray(list(stop_tokens) or [NO_TOKEN], dtype=np.uint32)
    out = np.zeros(rows, dtype=np.uint32)
    acc, ret = c_u32(), c_u32()
    lib.orc_accept_tree.restype = c_u32
    kept = lib.orc_accept_tree(nodes, _p(tok, u32p), _p(sel, u32p), c_u32(rows), c_u32(remaining), _p(stops, u32p), c_u32(len(stops)),
                               _p(out, u32p), ctypes.byref(acc), ctypes.byref(ret))
    return out[:kept].copy(), acc.value, ret.value


def rejection_row(logits, temperature, q, draft_token, u_child, u_row):
    """Returns (token, accepted_draft, closeness)."""
    x = np.ascontiguousarray(logits, dtype=np.float32)
    qq = np.ascontiguousarray(q, dtype=np.float32) if q is not None else None
    acc, close = c_int(), ctypes.c_double()
    lib.orc_rejection_row.restype = c_u32
    tok = lib.orc_rejection_row(_p(x, f32p), c_u32(x.size), c_f(temperature), _p(qq, f32p), c_u32(draft_token), c_f(u_child),
                                c_f(u_row), ctypes.byref(acc), ctypes.byref(close))
    return tok, bool(acc.value), close.value


class SamplingPolicy(ctypes.Structure):
    _fields_ = [("temperature", c_f), ("min_p", c_f), ("top_k", c_u32), ("top_p", c_f)]


def distribution_end(logits, temperature, min_p=0.0, top_k=0, top_p=1.0):
    """Returns (key, last id, kept mass, kept count, closeness)."""
    x = np.ascontiguousarray(logits, dtype=np.float32)
    policy = SamplingPolicy(temperature, min_p, top_k, top_p)
    key, last, mass, close = c_u32(), c_u32(), c_f(), ctypes.c_double()
    lib.orc_distribution_end.restype = c_u32
    count = lib.orc_distribution_end(_p(x, f32p), c_u32(x.size), ctypes.byref(policy), ctypes.byref(key), ctypes.byref(last),
                                     ctypes.byref(mass), ctypes.byref(close))
    return key.value, last.value, mass.value, count, close.value


def rejection_row_policy(logits, policy, q, draft_token, u_child, u_row):
    """policy: (temperature, min_p, top_k, top_p). Returns (token, accepted_draft, closeness)."""
    x = np.ascontiguousarray(logits, dtype=np.float32)
    qq = np.ascontiguousarray(q, dtype=np.float32) if q is not None else None
    acc, close = c_int(), ctypes.c_double()
    lib.orc_rejection_row_policy.restype = c_u32
    tok = lib.orc_rejection_row_policy(_p(x, f32p), c_u32(x.size), ctypes.byref(SamplingPolicy(*policy)), _p(qq, f32p), c_u32(draft_token),
                                       c_f(u_child), c_f(u_row), ctypes.byref(acc), ctypes.byref(close))
    return tok, bool(acc.value), close.value


def rejection_law_policy(logits, policy, q):
    x = np.ascontiguousarray(logits, dtype=np.float32)
    qq = np.ascontiguousarray(q, dtype=np.float32)
    out = np.empty(x.size, dtype=np.float64)
    lib.orc_rejection_law_policy.restype = None
    lib.orc_rejection_law_policy(_p(x, f32p), c_u32(x.size), ctypes.byref(SamplingPolicy(*policy)), _p(qq, f32p), _p(out, f64p))
    return out


def logit_key(values):
    """The order-preserving unsigned key of fp32 logits (sampling.metal:197-207), vectorised."""
    bits = np.ascontiguousarray(values, dtype=np.float32).view(np.uint32).copy()
    bits[(bits << np.uint32(1)) == 0] = 0
    return np.where(bits & 0x80000000, ~bits, bits | np.uint32(0x80000000)).astype(np.uint32)


def rejection_law(logits, temperature, q):
    x = np.ascontiguousarray(logits, dtype=np.float32)
    qq = np.ascontiguousarray(q, dtype=np.float32)
    out = np.empty(x.size, dtype=np.float64)
    lib.orc_rejection_law(_p(x, f32p), c_u32(x.size), c_f(temperature), _p(qq, f32p), _p(out, f64p))
    return out


def activation_table(x_bits, tiles=None):
    """The activation table of bf16 rows [M][K] (K a multiple of 32) as the projection kernels read it:
    values uint16 [tiles][K/32][64][8] (lane kq*16 + r holds inputs 16 (e//4) + 4 kq + (0,2,1,3)[e%4] of
    the group for row 16 t + r), fp32 sums of each row's 32 inputs [tiles][K/32][16] and 16 inputs
    [tiles][K/16][16], added in input order: runs of four as (x0 + x1) + (x2 + x3), the four runs of a
    half in order, then the two halves. Rows past M are zero. Returns (values, sums32, sums16)."""
    M, K = x_bits.shape
    tiles = tiles or (M + 15) // 16
    G = K // 32
    x = np.zeros((tiles * 16, K), dtype=np.uint16)
    x[:M] = x_bits
    order = np.array([0, 2, 1, 3])
    e = np.arange(8)
    kq = np.arange(4)
    inputs = 16 * (e[None, :] // 4) + 4 * kq[:, None] + order[e[None, :] % 4]      # [kq][e]
    grouped = x.reshape(tiles, 16, G, 32)                                          # [t][r][g][i]
    values = grouped[:, :, :, inputs]                                              # [t][r][g][kq][e]
    values = np.ascontiguousarray(values.transpose(0, 2, 3, 1, 4)).reshape(tiles, G, 64, 8)
    f = bf16_to_f32(x).reshape(tiles, 16, 2 * G, 4, 4)                             # [t][r][half block][run][i]
    runs = (f[..., 0] + f[..., 1]) + (f[..., 2] + f[..., 3])
    s16 = ((runs[..., 0] + runs[..., 1]) + runs[..., 2]) + runs[..., 3]            # [t][r][2G]
    s32 = s16[..., 0::2] + s16[..., 1::2]
    return values, np.ascontiguousarray(s32.transpose(0, 2, 1)), np.ascontiguousarray(s16.transpose(0, 2, 1))


def table_rows(values, K, tiles):
    """The bf16 rows [tiles * 16][K] an activation table's values hold (the inverse of activation_table's layout)."""
    G = K // 32
    order = np.array([0, 2, 1, 3])
    e = np.arange(8)
    kq = np.arange(4)
    inputs = 16 * (e[None, :] // 4) + 4 * kq[:, None] + order[e[None, :] % 4]      # [kq][e]
    v = np.asarray(values).reshape(tiles, G, 4, 16, 8).transpose(0, 3, 1, 2, 4)   # [t][r][g][kq][e]
    rows = np.zeros((tiles, 16, G, 32), dtype=np.uint16)
    rows[:, :, :, inputs] = v
    return rows.reshape(tiles * 16, K)


def split_activation_table(raw_bytes, K, tiles):
    """(values, sums32, sums16) views of a table downloaded as bytes."""
    G = K // 32
    nv = tiles * K * 16 * 2
    n32 = tiles * G * 16 * 4
    values = raw_bytes[:nv].view(np.uint16).reshape(tiles, G, 64, 8)
    s32 = raw_bytes[nv:nv + n32].view(np.float32).reshape(tiles, G, 16)
    s16 = raw_bytes[nv + n32:nv + 3 * n32].view(np.float32).reshape(tiles, 2 * G, 16)
    return values, s32, s16


def assert_table_holds(raw_bytes, x_bits, piece_bytes):
    """A downloaded activation table equals the one the bf16 rows x_bits [M][K] define, piece by piece of 64 rows;
    piece_bytes(rows) is a piece's size. Rows of a tile past M are not compared: a writer of live rows leaves them."""
    M, K = x_bits.shape
    at = 0
    for first in range(0, M, 64):
        count = min(64, M - first)
        tiles = (count + 15) // 16
        size = piece_bytes(count)
        values, s32, s16 = split_activation_table(raw_bytes[at:at + size], K, tiles)
        wv, w32, w16 = activation_table(x_bits[first:first + count])
        assert np.array_equal(table_rows(values, K, tiles)[:count], table_rows(wv, K, tiles)[:count])
        live = lambda sums: sums.transpose(0, 2, 1).reshape(tiles * 16, -1)[:count]
        assert live(s32).tobytes() == live(w32).tobytes() and live(s16).tobytes() == live(w16).tobytes()
        at += size


# ---- Gated DeltaNet ----
class GdnShape(ctypes.Structure):
    _fields_ = [("key_heads", c_u32), ("value_heads", c_u32), ("conv_dim", c_u32), ("packed_width", c_u32), ("flags", c_u32)]


lib.orc_gdn_tape_bytes.restype = ctypes.c_uint64
lib.orc_gdn_tape_bytes.argtypes = [ctypes.POINTER(GdnShape)]
lib.orc_gdn_step.restype = None
lib.orc_gdn_step.argtypes = [f32p, c_u32, f32p, f32p, c_f, c_f, f32p, f32p]


def gdn_shape(key_heads, value_heads, flags=0, packed_width=None):
    conv = (2 * key_heads + value_heads) * 128
    return GdnShape(key_heads, value_heads, conv, packed_width or conv + value_heads * 128 + 2 * value_heads, flags)


def gdn_tape_bytes(shape):
    return int(lib.orc_gdn_tape_bytes(ctypes.byref(shape)))


def gdn_split_tape(shape, tape):
    """(inputs [16][conv], kv [16][kv width], decay [16][vh] f32, beta [16][vh]) views of one layer's tape bytes."""
    kvw = (shape.key_heads + shape.value_heads) * 128
    a = 16 * shape.conv_dim * 2
    b = a + 16 * kvw * 2
    c = b + 16 * shape.value_heads * 4
    d = c + 16 * shape.value_heads * 2
    return (tape[:a].view(np.uint16).reshape(16, shape.conv_dim), tape[a:b].view(np.uint16).reshape(16, kvw),
            tape[b:c].view(np.float32).reshape(16, shape.value_heads), tape[c:d].view(np.uint16).reshape(16, shape.value_heads))


def gdn_decode(shape, packed, conv_weights, a_scale, dt_bias, norm_weight, conv_in, state_in, pending_tape=None, pending_path=0,
               ancestors=None):
    """One lane, one layer, a block of packed.shape[0] rows (a chain without `ancestors`, the rows' path masks).
    Returns (conv_out, state_out, step_tape bytes, hidden)."""
    rows = packed.shape[0]
    vh = shape.value_heads
    conv_out = np.zeros((3, shape.conv_dim), np.uint16)
    state_out = np.zeros((vh, 128, 128), np.float32)
    tape = np.zeros(gdn_tape_bytes(shape), np.uint8)
    hidden = np.zeros((rows, vh * 128), np.uint16)
    packed, conv_weights, a_scale, dt_bias, norm_weight, conv_in, state_in = (np.ascontiguousarray(x) for x in (
        packed, conv_weights, a_scale, dt_bias, norm_weight, conv_in, state_in))
    masks = None if ancestors is None else np.ascontiguousarray(ancestors, np.uint32)
    rc = lib.orc_gdn_decode(ctypes.byref(shape), _p(packed, u16p), rows, _p(masks, u32p), _p(conv_weights, u16p), _p(a_scale, f32p), _p(dt_bias, u16p),
                            norm_weight.ctypes.data_as(ctypes.c_void_p), _p(conv_in, u16p), _p(state_in, f32p),
                            _p(pending_tape, u8p), pending_path, _p(conv_out, u16p), _p(state_out, f32p), _p(tape, u8p), _p(hidden, u16p))
    assert rc == 0
    return conv_out, state_out, tape, hidden


lib.orc_gdn_decode.restype = c_int
lib.orc_gdn_decode.argtypes = [ctypes.POINTER(GdnShape), u16p, c_u32, u32p, u16p, f32p, u16p, ctypes.c_void_p, u16p, f32p, u8p, c_u32, u16p,
                               f32p, u8p, u16p]
lib.orc_gdn_fold.restype = c_int
lib.orc_gdn_fold.argtypes = [ctypes.POINTER(GdnShape), u16p, f32p, u8p, c_u32, c_u32, u16p, f32p]
lib.orc_gdn_reference.restype = c_int
lib.orc_gdn_reference.argtypes = [ctypes.POINTER(GdnShape), u16p, c_u32, u16p, f32p, u16p, u16p, f32p, f64p, f64p, f64p, f64p, f64p]


lib.orc_gdn_prefill.restype = c_int
lib.orc_gdn_prefill.argtypes = [ctypes.POINTER(GdnShape), u16p, c_u32, u16p, f32p, u16p, ctypes.c_void_p, u16p, f32p, u16p, u16p, u16p, f32p,
                                u16p, u16p, f32p, u16p, u16p]


def gdn_prefill(shape, packed, conv_weights, a_scale, dt_bias, norm_weight, conv_in, state_in):
    """A prompt chunk of one lane and layer. Returns dict(queries, keys, values, decay, beta, conv_out, state_out,
    recurrent, hidden)."""
    tokens, vh, kh = packed.shape[0], shape.value_heads, shape.key_heads
    out = dict(queries=np.zeros((tokens, kh * 128), np.uint16), keys=np.zeros((tokens, kh * 128), np.uint16),
               values=np.zeros((tokens, vh * 128), np.uint16), decay=np.zeros((tokens, vh), np.float32),
               beta=np.zeros((tokens, vh), np.uint16), conv_out=np.zeros((3, shape.conv_dim), np.uint16),
               state_out=np.zeros((vh, 128, 128), np.float32), recurrent=np.zeros((tokens, vh * 128), np.uint16),
               hidden=np.zeros((tokens, vh * 128), np.uint16))
    packed, conv_weights, a_scale, dt_bias, norm_weight, conv_in, state_in = (np.ascontiguousarray(x) for x in (
        packed, conv_weights, a_scale, dt_bias, norm_weight, conv_in, state_in))
    rc = lib.orc_gdn_prefill(ctypes.byref(shape), _p(packed, u16p), tokens, _p(conv_weights, u16p), _p(a_scale, f32p), _p(dt_bias, u16p),
                             norm_weight.ctypes.data_as(ctypes.c_void_p), _p(conv_in, u16p), _p(state_in, f32p),
                             _p(out["queries"], u16p), _p(out["keys"], u16p), _p(out["values"], u16p), _p(out["decay"], f32p),
                             _p(out["beta"], u16p), _p(out["conv_out"], u16p), _p(out["state_out"], f32p), _p(out["recurrent"], u16p),
                             _p(out["hidden"], u16p))
    assert rc == 0
    return out


def gdn_fold(shape, conv_in, state_in, step_tape, path, rows):
    conv_out = np.zeros((3, shape.conv_dim), np.uint16)
    state_out = np.zeros_like(state_in)
    conv_in, state_in = np.ascontiguousarray(conv_in), np.ascontiguousarray(state_in)
    rc = lib.orc_gdn_fold(ctypes.byref(shape), _p(conv_in, u16p), _p(state_in, f32p), _p(step_tape, u8p), path, rows,
                          _p(conv_out, u16p), _p(state_out, f32p))
    return rc, conv_out, state_out


def gdn_reference(shape, packed, conv_weights, a_scale, dt_bias, conv_in, state_in):
    """fp64: (kv rows [rows][kv width], beta, decay [rows][vh], state after the rows, outputs [rows][vh][128])."""
    rows, vh = packed.shape[0], shape.value_heads
    kvw = (shape.key_heads + vh) * 128
    kv = np.zeros((rows, kvw)); beta = np.zeros((rows, vh)); decay = np.zeros((rows, vh))
    state = np.zeros((vh, 128, 128)); out = np.zeros((rows, vh, 128))
    packed, conv_weights, a_scale, dt_bias, conv_in, state_in = (np.ascontiguousarray(x) for x in (
        packed, conv_weights, a_scale, dt_bias, conv_in, state_in))
    rc = lib.orc_gdn_reference(ctypes.byref(shape), _p(packed, u16p), rows, _p(conv_weights, u16p), _p(a_scale, f32p), _p(dt_bias, u16p),
                               _p(conv_in, u16p), _p(state_in, f32p), _p(kv, f64p), _p(beta, f64p), _p(decay, f64p), _p(state, f64p),
                               _p(out, f64p))
    assert rc == 0
    return kv, beta, decay, state, out


def gdn_step(S, k, v, decay, beta, q=None):
    S = np.ascontiguousarray(S, np.float32).copy()
    o = np.zeros(S.shape[0], np.float32)
    k, v = np.ascontiguousarray(k, np.float32), np.ascontiguousarray(v, np.float32)
    qq = np.ascontiguousarray(q, np.float32) if q is not None else None
    lib.orc_gdn_step(_p(S, f32p), S.shape[0], _p(k, f32p), _p(v, f32p), decay, beta, _p(qq, f32p), _p(o, f32p) if q is not None else None)
    return S, o


# ---- mixture of experts ----
lib.orc_moe_route.restype = None
lib.orc_moe_route.argtypes = [f32p, c_u32, c_u32, c_u32, c_u32, u32p, f32p]
lib.orc_moe_combine.restype = None
lib.orc_moe_combine.argtypes = [u16p, f32p, u16p, c_u32, c_u32, c_u32, u16p]


def moe_route(scores, top_k, shared=0, x_bits=None, shared_gate=None, sigmoid_router=False):
    """Each row's routes: its top_k routed experts, then `shared` slices of the shared expert (ids experts on), each
    weighing sigmoid(x . shared_gate) or, without a gate, 1."""
    scores = np.ascontiguousarray(scores, np.float32)
    rows, experts = scores.shape
    selected = np.zeros((rows, top_k), np.uint32)
    weights = np.zeros((rows, top_k), np.float32)
    route = lib.orc_moe_route_sigmoid if sigmoid_router else lib.orc_moe_route
    route(_p(scores, f32p), rows, experts, experts, top_k, _p(selected, u32p), _p(weights, f32p))
    if shared:
        gate = np.ones(rows, np.float32)
        if shared_gate is not None:
            x = np.ascontiguousarray(x_bits, np.uint16)
            g = np.ascontiguousarray(shared_gate, np.float32)
            lib.orc_moe_shared_weights(_p(x, u16p), _p(g, f32p), rows, x.shape[1], _p(gate, f32p))
        selected = np.concatenate([selected, np.tile(experts + np.arange(shared, dtype=np.uint32), (rows, 1))], axis=1)
        weights = np.concatenate([weights, np.tile(gate[:, None], (1, shared))], axis=1)
    return selected, weights


def moe_combine(y_bits, weights, residual_bits):
    rows, top_k, hidden = y_bits.shape
    out = np.zeros((rows, hidden), np.uint16)
    y_bits, weights, residual_bits = (np.ascontiguousarray(a) for a in (y_bits, weights, residual_bits))
    lib.orc_moe_combine(_p(y_bits, u16p), _p(weights, f32p), _p(residual_bits, u16p), rows, top_k, hidden, _p(out, u16p))
    return out


def moe_layer(x_bits, residual_bits, scores, top_k, gate_native, up_native, down_native, ffn, fmt=FMT_Q4K, down_fmt=FMT_Q4K,
              shared=0, shared_gate=None, sigmoid_router=False):
    """The routed experts of a layer: x bf16 [rows][hidden] (normalized), natives per expert (the shared slices' after
    the routed experts'). Each expert's rows go through the oracle's projections together; a row's result does not
    depend on the rows beside it."""
    rows, hidden = x_bits.shape
    selected, weights = moe_route(scores, top_k, shared, x_bits, shared_gate, sigmoid_router)
    y = np.zeros((rows, top_k + shared, hidden), np.uint16)
    for e in np.unique(selected):
        r, k = np.nonzero(selected == e)
        xe = np.ascontiguousarray(x_bits[r])
        gate = gemm(fmt, gate_native[e], xe, ffn, want=("chain",))["chain"]
        up = gemm(fmt, up_native[e], xe, ffn, want=("chain",))["chain"]
        mid = swiglu(gate, up).reshape(len(r), ffn)
        down = gemm(down_fmt, down_native[e], mid, hidden, want=("chain",))["chain"]
        y[r, k] = f32_to_bf16(down)
    return selected, weights, y, moe_combine(y, weights, residual_bits)


# ---- the cached form of recurrent layers ----
def state_codec_bytes(rows, columns):
    lib.orc_state_codec_bytes.restype = ctypes.c_uint64
    return lib.orc_state_codec_bytes(c_u32(rows), c_u32(columns))


def state_codes(values, library=None):
    """fp32 [rows][columns] -> the layer's codes and scales (uint8)."""
    values = np.ascontiguousarray(values, dtype=np.float32)
    rows, columns = values.shape
    image = np.zeros(state_codec_bytes(rows, columns), dtype=np.uint8)
    fn = (library or lib).ref_state_codes if library is not None else lib.orc_state_codes
    assert fn(_p(values, f32p), c_u32(rows), c_u32(columns), _p(image, u8p)) == 0
    return image


def state_values(image, rows, columns):
    image = np.ascontiguousarray(image, dtype=np.uint8)
    values = np.empty((rows, columns), dtype=np.float32)
    assert lib.orc_state_values(_p(image, u8p), c_u32(rows), c_u32(columns), _p(values, f32p)) == 0
    return values


TREE_DTYPE = np.dtype([("ancestors", "<u4"), ("parent", "<u2"), ("depth", "<u2")])


def draft_candidates(logits, lanes, leading=None, trailing=None):
    """(candidates uint32 [lanes * 7][16], unary fp32 [lanes * 7][16]) of logits fp32 [lanes * 8][columns]."""
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    columns = logits.shape[1]
    leading = columns if leading is None else leading
    trailing = leading if trailing is None else trailing
    candidates, unary = np.zeros((lanes * 7, 16), np.uint32), np.zeros((lanes * 7, 16), np.float32)
    lib.orc_draft_candidates.restype = None
    lib.orc_draft_candidates(_p(logits, f32p), c_u32(lanes), c_u32(columns), c_u32(leading), c_u32(trailing), _p(candidates, u32p),
                             _p(unary, f32p))
    return candidates, unary


def draft_edges(candidates, anchors, vocabulary, hidden, predecessor_codebook, successor_codebook):
    """edges fp32 [lanes * 7][16][16]; hidden and the codebooks as bf16 bit patterns (uint16)."""
    candidates = np.ascontiguousarray(candidates, dtype=np.uint32)
    anchors = np.ascontiguousarray(anchors, dtype=np.uint32)
    hidden, before, after = (np.ascontiguousarray(a, dtype=np.uint16) for a in (hidden, predecessor_codebook, successor_codebook))
    edges = np.zeros((candidates.shape[0], 16, 16), np.float32)
    u16p = ctypes.POINTER(ctypes.c_uint16)
    lib.orc_draft_edges.restype = None
    lib.orc_draft_edges(_p(candidates, u32p), _p(anchors, u32p), c_u32(len(anchors)), c_u32(vocabulary), _p(hidden, u16p), _p(before, u16p),
                        _p(after, u16p), _p(edges, f32p))
    return edges


def draft_verify_rows(tree_tokens, trees, scores, sizes, rows, lane_cap, floor=0.0):
    """draft_verify_rows: (tokens [rows], tree rows [rows], lane rows [lanes][2], sources [rows]) of a step laid out from
    each lane's tree: tree_tokens uint32 [lanes][16], trees TREE_DTYPE [lanes][16], scores fp32 [lanes][16][2]."""
    lanes = len(sizes)
    tree_tokens = np.ascontiguousarray(tree_tokens, dtype=np.uint32)
    trees = np.ascontiguousarray(trees, dtype=TREE_DTYPE)
    scores = np.ascontiguousarray(scores, dtype=np.float32)
    sizes = np.ascontiguousarray(sizes, dtype=np.uint32)
    tokens, tree = np.zeros(rows, np.uint32), np.zeros(rows, TREE_DTYPE)
    lane_rows, sources = np.zeros((lanes, 2), np.uint32), np.zeros(rows, np.uint32)
    lib.orc_draft_verify_rows.restype = None
    lib.orc_draft_verify_rows(_p(tree_tokens, u32p), trees.ctypes.data_as(ctypes.c_void_p), _p(scores, f32p), _p(sizes, u32p), c_u32(lanes),
                              c_u32(rows), c_u32(lane_cap), c_f(floor), _p(tokens, u32p), tree.ctypes.data_as(ctypes.c_void_p),
                              _p(lane_rows, u32p), _p(sources, u32p))
    return tokens, tree, lane_rows, sources


def draft_verify_row_slots(tree_tokens, trees, scores, sizes, lane_cap, floor=0.0):
    """The verify rows in slots: lane l's rows from row l * lane_cap on, the rest of its slot inert."""
    lanes = len(sizes)
    rows = lanes * lane_cap
    tree_tokens = np.ascontiguousarray(tree_tokens, dtype=np.uint32)
    trees = np.ascontiguousarray(trees, dtype=TREE_DTYPE)
    scores = np.ascontiguousarray(scores, dtype=np.float32)
    sizes = np.ascontiguousarray(sizes, dtype=np.uint32)
    tokens, tree = np.zeros(rows, np.uint32), np.zeros(rows, TREE_DTYPE)
    lane_rows, sources = np.zeros((lanes, 2), np.uint32), np.zeros(rows, np.uint32)
    lib.orc_draft_verify_row_slots.restype = None
    lib.orc_draft_verify_row_slots(_p(tree_tokens, u32p), trees.ctypes.data_as(ctypes.c_void_p), _p(scores, f32p), _p(sizes, u32p), c_u32(lanes),
                                   c_u32(lane_cap), c_f(floor), _p(tokens, u32p), tree.ctypes.data_as(ctypes.c_void_p),
                                   _p(lane_rows, u32p), _p(sources, u32p))
    return tokens, tree, lane_rows, sources


class DraftTreeLane(ctypes.Structure):
    """One lane's DraftTreeParams (Sampling.h:242-252)."""
    _fields_ = [("anchor", c_u32), ("depth", c_u32), ("chain", c_u32), ("children", c_u32), ("slope", c_f), ("intercept", c_f * 7),
                ("temperature", c_f), ("noise", c_u32 * 2)]


def draft_tree_lane(anchor, depth, children, slope=1.0, intercept=None, temperature=0.0, noise=0, chain=0):
    lane = DraftTreeLane(anchor, depth, chain, children, slope, (c_f * 7)(*(intercept if intercept is not None else [0.0] * 7)), temperature,
                         (c_u32 * 2)(noise & 0xFFFFFFFF, noise >> 32))
    return lane


def draft_tree(candidates, unary, edges, lane, chain_tokens=None, chain_rates=None):
    """draft_select_tree of one lane: candidates uint32 [7][16], unary fp32 [7][16], edges fp32 [7][16][16]. Returns a dict:
    tokens [n], tree TREE_DTYPE [n], q [n], estimate [n], draws uint8 [n][4], next fp32 [n][16], caps [n]."""
    candidates = np.ascontiguousarray(candidates, np.uint32)
    unary, edges = np.ascontiguousarray(unary, np.float32), np.ascontiguousarray(edges, np.float32)
    chain_tokens = np.ascontiguousarray(chain_tokens if chain_tokens is not None else np.zeros(15), np.uint32)
    chain_rates = np.ascontiguousarray(chain_rates if chain_rates is not None else np.zeros((15, 4)), np.float32)
    tokens, tree, scores = np.zeros(16, np.uint32), np.zeros(16, TREE_DTYPE), np.zeros((16, 2), np.float32)
    size = c_u32(0)
    draws, nxt, caps = np.zeros((16, 4), np.uint8), np.zeros((16, 16), np.float32), np.zeros(16, np.float32)
    lib.orc_draft_tree.restype = None
    lib.orc_draft_tree(_p(candidates, u32p), _p(unary, f32p), _p(edges, f32p), _p(chain_tokens, u32p), _p(chain_rates, f32p), ctypes.byref(lane),
                       _p(tokens, u32p), tree.ctypes.data_as(ctypes.c_void_p), _p(scores, f32p), ctypes.byref(size), _p(draws, u8p),
                       _p(nxt, f32p), _p(caps, f32p))
    n = size.value
    return dict(tokens=tokens[:n], tree=tree[:n], q=scores[:n, 0], estimate=scores[:n, 1], draws=draws[:n], next=nxt[:n], caps=caps[:n])


# ---- glue: rope tables, the sigmoid router, the shared expert's gate ----
lib.orc_rope_tables.restype = None
lib.orc_rope_tables.argtypes = [c_u32, u32p, c_u32, f32p, c_u32, f32p, f32p]
lib.orc_moe_shared_weights.restype = None
lib.orc_moe_shared_weights.argtypes = [u16p, f32p, c_u32, c_u32, f32p]


def rope_tables(anchor, depth, invfreq):
    depth = np.ascontiguousarray(depth, np.uint32)
    invfreq = np.ascontiguousarray(invfreq, np.float32)
    cosv = np.empty((len(depth), len(invfreq)), np.float32)
    sinv = np.empty_like(cosv)
    lib.orc_rope_tables(c_u32(anchor), _p(depth, u32p), c_u32(len(depth)), _p(invfreq, f32p), c_u32(len(invfreq)), _p(cosv, f32p),
                        _p(sinv, f32p))
    return cosv, sinv


def silu(x):
    return np.array([lib.orc_silu(float(v)) for v in np.ravel(x)], np.float32).reshape(np.shape(x))


def moe_shared_weights(x_bits, gate):
    x = np.ascontiguousarray(x_bits, np.uint16)
    g = np.ascontiguousarray(gate, np.float32)
    out = np.empty(x.shape[0], np.float32)
    lib.orc_moe_shared_weights(_p(x, u16p), _p(g, f32p), x.shape[0], x.shape[1], _p(out, f32p))
    return out


# ---- a tree block's sampled rows: up to four drawn children among sixteen candidates ----
def children_row(logits, policy, ids, q, draws, u_children, u_row):
    """orc_children_row: (token, closeness). policy: (temperature, min_p, top_k, top_p); draws: candidate indices in the
    order drawn (at most four)."""
    x = np.ascontiguousarray(logits, np.float32)
    ids = np.ascontiguousarray(ids, np.uint32)
    q = np.ascontiguousarray(q, np.float32)
    d = np.full(4, 0xFF, np.uint8)
    d[:len(draws)] = draws
    u = np.zeros(4, np.float32)
    u[:len(u_children)] = u_children
    pol = SamplingPolicy(*policy)
    close = ctypes.c_double()
    lib.orc_children_row.restype = c_u32
    token = lib.orc_children_row(_p(x, f32p), c_u32(x.size), ctypes.byref(pol), _p(ids, u32p), _p(q, f32p), _p(d, u8p), c_u32(len(draws)),
                                 _p(u, f32p), c_f(u_row), ctypes.byref(close))
    return token, close.value


def children_law(p_target, ids, q, n_draws):
    p = np.ascontiguousarray(p_target, np.float64)
    ids = np.ascontiguousarray(ids, np.uint32)
    q = np.ascontiguousarray(q, np.float64)
    out = np.zeros(p.size, np.float64)
    lib.orc_children_law.restype = None
    lib.orc_children_law(_p(p, f64p), c_u32(p.size), _p(ids, u32p), _p(q, f64p), c_u32(n_draws), _p(out, f64p))
    return out


# ---- the draft model's attention block (oracle/draft_attention.cpp) ----
DRAFT_ROWS, DRAFT_QUERY_HEADS, DRAFT_KV_HEADS, DRAFT_D, DRAFT_WINDOW = 8, 32, 8, 128, 2048


def draft_conv(x, dynamic, base, residual, finish):
    """bf16 bits [lanes * 8][hidden] through one stage of the dynamic convolution."""
    x = np.ascontiguousarray(x, np.uint16)
    lanes, hidden = x.shape[0] // DRAFT_ROWS, x.shape[1]
    residual = np.ascontiguousarray(residual if residual is not None else x, np.uint16)
    dynamic, base = np.ascontiguousarray(dynamic, np.uint16), np.ascontiguousarray(base, np.uint16)
    out = np.empty_like(x)
    lib.orc_draft_conv(_p(x, u16p), _p(dynamic, u16p), _p(base, u16p), _p(residual, u16p), _p(out, u16p), c_u32(hidden), c_u32(lanes),
                       ctypes.c_int(int(finish)))
    return out


def draft_prepare(qkv, query_norm, key_norm, cosines, sines):
    """qkv bf16 bits [lanes * 8][6144]; cosines / sines fp32 [lanes][16][64]. Returns the grouped queries
    [lanes][32][8][128], the rows' keys [lanes][8][8][128] and their values [lanes][8][128][8]."""
    qkv = np.ascontiguousarray(qkv, np.uint16)
    lanes = qkv.shape[0] // DRAFT_ROWS
    cosines, sines = np.ascontiguousarray(cosines, np.float32), np.ascontiguousarray(sines, np.float32)
    q = np.empty((lanes, DRAFT_QUERY_HEADS, DRAFT_ROWS, DRAFT_D), np.uint16)
    k = np.empty((lanes, DRAFT_KV_HEADS, DRAFT_ROWS, DRAFT_D), np.uint16)
    v = np.empty((lanes, DRAFT_KV_HEADS, DRAFT_D, DRAFT_ROWS), np.uint16)
    lib.orc_draft_prepare(_p(qkv, u16p), _p(np.ascontiguousarray(query_norm, np.uint16), u16p), _p(np.ascontiguousarray(key_norm, np.uint16), u16p),
                          _p(cosines, f32p), _p(sines, f32p), c_u32(lanes), _p(q, u16p), _p(k, u16p), _p(v, u16p))
    return q, k, v


def draft_context_write(context_kv, key_norm, cosines, sines, source_rows, positions, rope_rows, ring_keys, ring_values):
    """Writes context rows into one lane's rings in place: ring_keys [8][2048][128], ring_values [8][128][2048] (bf16 bits)."""
    context_kv = np.ascontiguousarray(context_kv, np.uint16)
    cosines, sines = np.ascontiguousarray(cosines, np.float32), np.ascontiguousarray(sines, np.float32)
    src, pos, rope = (np.ascontiguousarray(a, np.uint32) for a in (source_rows, positions, rope_rows))
    assert ring_keys.flags.c_contiguous and ring_values.flags.c_contiguous and ring_keys.dtype == np.uint16
    lib.orc_draft_context_write(_p(context_kv, u16p), _p(np.ascontiguousarray(key_norm, np.uint16), u16p), _p(cosines, f32p), _p(sines, f32p),
                                _p(src, u32p), _p(pos, u32p), _p(rope, u32p), c_u32(len(src)), _p(ring_keys, u16p), _p(ring_values, u16p))


def draft_attention(queries, ring_keys, ring_values, query_keys, query_values, cache_length):
    """One lane and KV head in fp64: queries [32][128], ring_keys [2048][128], ring_values [128][2048], query_keys
    [8][128], query_values [128][8] (bf16 bits). Returns float64 [32][128]."""
    args = [np.ascontiguousarray(a, np.uint16) for a in (queries, ring_keys, ring_values, query_keys, query_values)]
    out = np.empty((4 * DRAFT_ROWS, DRAFT_D), np.float64)
    lib.orc_draft_attention(*[_p(a, u16p) for a in args], c_u32(cache_length), _p(out, ctypes.POINTER(ctypes.c_double)))
    return out


def draft_window_bytes(width):
    lib.orc_draft_window_bytes.restype = ctypes.c_uint64
    return int(lib.orc_draft_window_bytes(c_u32(width)))


def draft_window_store(context, source_rows, start, window):
    """Stores rows source_rows of context (bf16 bits [.][width]) into the slots of positions start on, in place."""
    context = np.ascontiguousarray(context, np.uint16)
    src = np.ascontiguousarray(source_rows, np.uint32)
    assert window.dtype == np.uint8 and window.flags.c_contiguous and window.size == draft_window_bytes(context.shape[1])
    lib.orc_draft_window_store(_p(context, u16p), _p(src, u32p), c_u32(len(src)), c_u32(start), c_u32(context.shape[1]), _p(window, u8p))


def draft_window_load(window, rows, start, width):
    out = np.empty((rows, width), np.uint16)
    lib.orc_draft_window_load(_p(np.ascontiguousarray(window, np.uint8), u8p), c_u32(rows), c_u32(start), c_u32(width), _p(out, u16p))
    return out
