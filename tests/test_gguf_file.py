"""The GGUF header parser (CPU) and the loading of a file's tensors as the operators' inputs (GPU)."""
import hashlib
import json
import os

import numpy as np
import pytest

import splash_amd
from splash_amd import gguf, ops
from tests import gguf_writer as gw
from tests import oracle as orc


def model_file(path, alignment=32):
    rng = np.random.default_rng(4)
    tensors = [
        ("blk.0.attn_q.weight", gw.GGML_Q4_K, [512, 96], orc.make_native(orc.FMT_Q4K, 96, 512, 1)),
        ("blk.0.attn_v.weight", gw.GGML_Q6_K, [512, 32], orc.make_native(orc.FMT_Q6K, 32, 512, 2)),
        ("blk.0.ffn_down.weight", gw.GGML_Q5_K, [768, 64], orc.make_native(orc.FMT_Q5K, 64, 768, 3)),
        ("output.weight", gw.GGML_Q8_0, [512, 48], orc.make_native(orc.FMT_Q80, 48, 512, 4)),
        ("blk.0.ffn_gate.weight", gw.GGML_IQ4_XS, [512, 64], orc.make_native(orc.FMT_IQ4XS, 64, 512, 5)),
        ("blk.0.ffn_up.weight", gw.GGML_IQ4_NL, [512, 64], orc.make_native(orc.FMT_IQ4NL, 64, 512, 6)),
        ("blk.0.attn_norm.weight", gw.GGML_F32, [512], (1 + 0.1 * rng.standard_normal(512)).astype(np.float32)),
        ("output_norm.weight", gw.GGML_BF16, [512], orc.f32_to_bf16((1 + 0.1 * rng.standard_normal(512)).astype(np.float32))),
        ("blk.0.post_norm.weight", gw.GGML_F16, [512], (1 + 0.1 * rng.standard_normal(512)).astype(np.float16)),
    ]
    metadata = [("general.architecture", gw.STRING, "qwen3"), ("general.alignment", gw.U32, alignment),
                ("qwen3.block_count", gw.U32, 1), ("qwen3.rope.freq_base", gw.F32, 1e6), ("qwen3.attention.layer_norm_rms_epsilon", gw.F64, 1e-6),
                ("general.quantized", gw.BOOL, 1), ("general.negative", gw.I32, -2),
                ("tokenizer.ggml.tokens", gw.ARRAY, (gw.STRING, ["a", "bc", "def"])), ("tokenizer.ggml.scores", gw.ARRAY, (gw.F32, [0.5, 1.5]))]
    gw.write_gguf(path, metadata, tensors, alignment=alignment)
    return tensors


@pytest.mark.parametrize("alignment", [32, 64])
def test_header_metadata_and_tensor_table(tmp_path, alignment):
    path = tmp_path / "model.gguf"
    tensors = model_file(path, alignment)
    f = gguf.GgufFile(path)
    assert f.string("general.architecture") == "qwen3" and f.unsigned("qwen3.block_count") == 1
    assert f.float("qwen3.rope.freq_base") == 1e6 and f.float("qwen3.attention.layer_norm_rms_epsilon") == 1e-6
    assert f.unsigned("general.quantized") == 1 and f.unsigned("general.negative") == 2 ** 64 - 2
    assert f.string("missing") is None and f.unsigned("general.architecture") is None and f.string("tokenizer.ggml.tokens") is None
    assert [t.name for t in f.tensors] == [t[0] for t in tensors]
    for got, (name, kind, dims, data) in zip(f.tensors, tensors):
        assert (got.ggml_type, got.dims, got.bytes) == (kind, dims, np.asarray(data).nbytes)
        assert np.array_equal(f.data(got), np.frombuffer(np.ascontiguousarray(data).tobytes(), np.uint8))
    assert [f.find(n).format for n in ("blk.0.attn_q.weight", "blk.0.attn_v.weight", "blk.0.ffn_down.weight", "output.weight",
                                       "blk.0.ffn_gate.weight", "blk.0.ffn_up.weight")] == \
        [ops.FMT_Q4K, ops.FMT_Q6K, ops.FMT_Q5K, ops.FMT_Q80, ops.FMT_IQ4XS, ops.FMT_IQ4NL]
    assert f.find("output_norm.weight").format is None and f.find("nothing") is None


def test_malformed_files_are_refused(tmp_path):
    good = tmp_path / "good.gguf"
    model_file(good)
    raw = open(good, "rb").read()
    cases = {"magic": b"GGML" + raw[4:], "version": raw[:4] + (2).to_bytes(4, "little") + raw[8:], "truncated header": raw[:200],
             "truncated data": raw[:-4096], "empty": b""}
    for name, content in cases.items():
        path = tmp_path / f"{name}.gguf"
        open(path, "wb").write(content)
        with pytest.raises(splash_amd.SplashError):
            gguf.GgufFile(path)
    with pytest.raises(splash_amd.SplashError):
        gguf.GgufFile(tmp_path / "absent.gguf")
    # an unknown tensor type, rows that do not hold whole blocks, a misaligned offset, an alignment that is no power of two
    x = np.zeros(144, np.uint8)
    for name, tensors, alignment in (("type", [("t", 99, [256], x)], 32), ("blocks", [("t", gw.GGML_Q4_K, [100], x)], 32),
                                      ("alignment", [("t", gw.GGML_Q4_K, [256], x)], 48)):
        path = tmp_path / f"bad_{name}.gguf"
        gw.write_gguf(path, [("general.alignment", gw.U32, alignment)], tensors, alignment=alignment)
        with pytest.raises(splash_amd.SplashError):
            gguf.GgufFile(path)
    # a key holds one value (the reference's GgufFile.cpp:191-194, as llama.cpp's reader): a repeated key is refused,
    # whatever its second value
    twice = tmp_path / "twice.gguf"
    gw.write_gguf(twice, [("general.architecture", gw.STRING, "qwen3"), ("qwen3.block_count", gw.U32, 1), ("qwen3.block_count", gw.U32, 2)],
                  [("t", gw.GGML_Q4_K, [256], x)])
    with pytest.raises(splash_amd.SplashError, match="duplicate GGUF metadata key"):
        gguf.GgufFile(twice)


GOLDENS = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "gguf_dequantization.json")))
# ggml types with no kernels of their own: (golden's name, the oracle's format, ggml type, the format they are read as)
REWRITTEN = [("q3k", orc.FMT_Q3K, gw.GGML_Q3_K, orc.FMT_Q6K), ("q40", orc.FMT_Q40, gw.GGML_Q4_0, orc.FMT_Q80),
             ("q50", orc.FMT_Q50, gw.GGML_Q5_0, orc.FMT_Q80)]


@pytest.mark.parametrize("name,source,kind,read_as", REWRITTEN)
def test_rewritten_blocks_keep_every_value(name, source, kind, read_as):
    """The loader's rewrite of Q3_K blocks as Q6_K and of Q4_0 and Q5_0 blocks as Q8_0 (spo_gguf_rewrite): the written
    blocks' values are GGML's dequantize_row_* of the source bit for bit (the reference's golden hashes,
    goldens.json:8,18,22), over every scale and code the random fixture holds, and so are the oracle's projections."""
    native = orc.fixture(source, 256, 1024, 7 + source)
    fmt, rewritten = ops.rewrite_native(kind, native)
    assert fmt == read_as and rewritten.size == orc.row_bytes(read_as, 1024) * 256
    assert hashlib.sha256(orc.dequant_rows(read_as, rewritten, 256, 1024).tobytes()).hexdigest() == GOLDENS[name]
    if source == orc.FMT_Q3K:
        blocks = native.reshape(-1, 110)
        scales = np.concatenate([blocks[:, 96:104] & 15, blocks[:, 96:104] >> 4], axis=1) | \
            (((blocks[:, 104:108][:, np.arange(16) % 4] >> (2 * (np.arange(16) // 4))) & 3) << 4)
        assert set(np.unique(scales)) == set(range(64))   # every scale value occurs
        assert np.array_equal(rewritten.reshape(-1, 210)[:, 192:208].view(np.int8), scales.astype(np.int16) - 32)
    else:
        codes = rewritten.reshape(-1, 34)[:, 2:].view(np.int8)
        assert (codes.min(), codes.max()) == ((-8, 7) if source == orc.FMT_Q40 else (-16, 15))
    realistic = orc.make_native(source, 64, 512, 3)
    x_bits = orc.f32_to_bf16(np.random.default_rng(1).standard_normal((5, 512)).astype(np.float32))
    a = orc.gemm(source, realistic, x_bits, 64, want=("exact", "bound"))
    b = orc.gemm(read_as, ops.rewrite_native(kind, realistic)[1], x_bits, 64, want=("exact", "bound"))
    assert np.array_equal(a["exact"], b["exact"]) and np.array_equal(a["bound"], b["bound"])
    with pytest.raises(splash_amd.SplashError):
        ops.rewrite_native(kind, native[:109])
    with pytest.raises(splash_amd.SplashError):
        ops.rewrite_native(gw.GGML_Q4_K, native)


@pytest.mark.gpu
@pytest.mark.parametrize("name,source,kind,read_as", REWRITTEN)
def test_a_rewritten_tensor_loads_as_the_image_of_its_values(backend, tmp_path, name, source, kind, read_as):
    """A Q3_K, Q4_0 or Q5_0 tensor of a file: its image is the Q6_K or Q8_0 image of the rewritten blocks, whole or a
    slice of rows; the kernels' unpacking of it gives GGML's dequantize_row_* values (the golden hash); and its projection
    is the oracle's of the source rows."""
    fixture = orc.fixture(source, 256, 1024, 7 + source)
    realistic = orc.make_native(source, 64, 512, 3)
    path = tmp_path / "rewritten.gguf"
    gw.write_gguf(path, [("general.architecture", gw.STRING, "qwen3")],
                  [("fixture.weight", kind, [1024, 256], fixture), ("blk.0.attn_v.weight", kind, [512, 64], realistic)])
    f = gguf.GgufFile(path)
    print(f"case {name} golden through the file", flush=True)
    fmt, rows, input_size, image = f.load_image(backend, f.find("fixture.weight"))
    assert (fmt, rows, input_size) == (read_as, 256, 1024)
    assert np.array_equal(image.download(np.uint8)[:ops.gguf_image_bytes(fmt, 256, 1024)],
                          ops.pack_gguf_image(fmt, ops.rewrite_native(kind, fixture)[1], 256, 1024))
    out = backend.allocate_buffer(256 * 1024 * 4)
    graph = splash_amd.CommandGraph()
    ops.add_dequant(graph, fmt, image, out, 256, 1024)
    backend.run(graph)
    assert hashlib.sha256(out.download(np.float32, 256 * 1024).tobytes()).hexdigest() == GOLDENS[name]
    print(f"case {name} rows 32..63", flush=True)
    fmt, rows, _, image = f.load_image(backend, f.find("fixture.weight"), first_row=32, rows=32)
    row_bytes = orc.row_bytes(source, 1024)
    assert rows == 32 and np.array_equal(image.download(np.uint8)[:ops.gguf_image_bytes(fmt, 32, 1024)],
                                         ops.pack_gguf_image(fmt, ops.rewrite_native(kind, fixture[32 * row_bytes:64 * row_bytes])[1], 32, 1024))
    print(f"case {name} projection", flush=True)
    fmt, rows, input_size, image = f.load_image(backend, f.find("blk.0.attn_v.weight"))
    linear = ops.Linear(backend)
    x_bits = orc.f32_to_bf16(np.random.default_rng(8).standard_normal((5, 512)).astype(np.float32))
    projection = ops.Projection([(fmt, 64, image)], 512, float32=True)
    plan = linear.plan(projection, 5)
    out = backend.allocate_buffer(5 * 64 * 4)
    graph = splash_amd.CommandGraph()
    linear.add(graph, projection, plan, backend.from_array(x_bits), out, linear.scratch_for(backend, [plan]))
    backend.run(graph)
    want = orc.gemm(source, realistic, x_bits, 64, want=("exact", "bound"))
    assert np.all(np.abs(out.download(np.float32).reshape(5, 64) - want["exact"]) <= want["bound"])


@pytest.mark.gpu
def test_projections_and_norms_load_from_a_file(backend, tmp_path):
    """A file's tensors become the operators' inputs: each projection format's rows give the result of the same
    native rows packed by hand, a slice of rows is that slice, and 16- and 32-bit vectors arrive as bf16."""
    path = tmp_path / "model.gguf"
    tensors = {t[0]: t for t in model_file(path)}
    f = gguf.GgufFile(path)
    linear = ops.Linear(backend)
    rng = np.random.default_rng(8)
    for name in ("blk.0.attn_q.weight", "blk.0.attn_v.weight", "blk.0.ffn_down.weight", "output.weight", "blk.0.ffn_gate.weight",
                 "blk.0.ffn_up.weight"):
        print(f"case gguf file tensor {name}", flush=True)
        _, _, (K, N), native = tensors[name]
        fmt, rows, input_size, image = f.load_image(backend, f.find(name))
        assert (rows, input_size) == (N, K) and fmt == f.find(name).format
        assert np.array_equal(image.download(np.uint8)[:ops.gguf_image_bytes(fmt, N, K)], ops.pack_gguf_image(fmt, native, N, K))
        x_bits = orc.f32_to_bf16(rng.standard_normal((5, K)).astype(np.float32))
        results = []
        for projection in (ops.Projection([(fmt, N, image)], K, float32=True), ops.Projection.from_native(backend, [(fmt, N, native)], K, float32=True)):
            plan = linear.plan(projection, 5)
            out = backend.allocate_buffer(5 * N * 4)
            graph = splash_amd.CommandGraph()
            linear.add(graph, projection, plan, backend.from_array(x_bits), out, linear.scratch_for(backend, [plan]))
            backend.run(graph)
            results.append(out.download(np.float32).reshape(5, N))
        assert np.array_equal(results[0], results[1])
        want = orc.gemm(fmt, native, x_bits, N, want=("exact", "bound"))
        assert np.all(np.abs(results[0] - want["exact"]) <= want["bound"])
    # rows 32..63 of a tensor alone
    _, _, (K, N), native = tensors["blk.0.attn_q.weight"]
    fmt, rows, _, image = f.load_image(backend, f.find("blk.0.attn_q.weight"), first_row=32, rows=32)
    row_bytes = len(native) // N
    assert rows == 32 and np.array_equal(image.download(np.uint8)[:ops.gguf_image_bytes(fmt, 32, K)],
                                         ops.pack_gguf_image(fmt, native[32 * row_bytes:64 * row_bytes], 32, K))
    with pytest.raises(ValueError):
        f.load_image(backend, f.find("blk.0.attn_q.weight"), first_row=8, rows=16)
    with pytest.raises(ValueError):
        f.load_image(backend, f.find("output_norm.weight"))
    for name in ("blk.0.attn_norm.weight", "output_norm.weight", "blk.0.post_norm.weight"):
        data = tensors[name][3]
        want = data if data.dtype == np.uint16 else orc.f32_to_bf16(np.asarray(data, np.float32))
        assert np.array_equal(f.load_bf16(backend, f.find(name)).download(np.uint16)[:512], want)
    with pytest.raises(ValueError):
        f.load_bf16(backend, f.find("output.weight"))


def dense_model_file(path, model, value_format, tied, extra=(), skip=(), more_metadata=(), parts=1):
    """A dense decoder's GGUF as llama.cpp names its tensors: blk.N.attn_q / attn_k / attn_v (the values requantized to
    `value_format`, as a Q4_K_M file keeps them) ..., norms as F32, the token table, and the head unless tied."""
    d = model.dims
    H, D, F, V = d["hidden"], d["head_dim"], d["ffn"], d["vocabulary"]
    kinds = {orc.FMT_Q4K: gw.GGML_Q4_K, orc.FMT_Q6K: gw.GGML_Q6_K, orc.FMT_Q5K: gw.GGML_Q5_K, orc.FMT_Q80: gw.GGML_Q8_0,
             orc.FMT_Q3K: gw.GGML_Q3_K, orc.FMT_Q40: gw.GGML_Q4_0, orc.FMT_Q50: gw.GGML_Q5_0}
    f32 = lambda bits: orc.bf16_to_f32(bits).astype(np.float32)
    tensors = [("token_embd.weight", kinds[getattr(model, "table_format", orc.FMT_Q4K)], [H, V], model.embedding)]
    for i, w in enumerate(model.layers):
        p = f"blk.{i}."
        tensors += [(p + "attn_norm.weight", gw.GGML_F32, [H], f32(w["input_norm"])),
                    (p + "attn_q.weight", gw.GGML_Q4_K, [H, d["q_heads"] * D], w["q"]),
                    (p + "attn_k.weight", gw.GGML_Q4_K, [H, d["kv_heads"] * D], w["k"]),
                    (p + "attn_v.weight", kinds[value_format], [H, d["kv_heads"] * D], w["v"]),
                    (p + "attn_q_norm.weight", gw.GGML_F32, [D], f32(w["q_norm"])),
                    (p + "attn_k_norm.weight", gw.GGML_BF16, [D], w["k_norm"]),
                    (p + "attn_output.weight", gw.GGML_Q4_K, [d["q_heads"] * D, H], w["o"]),
                    (p + "ffn_norm.weight", gw.GGML_F32, [H], f32(w["post_norm"])),
                    (p + "ffn_gate.weight", gw.GGML_Q4_K, [H, F], w["gate"]), (p + "ffn_up.weight", gw.GGML_Q4_K, [H, F], w["up"]),
                    (p + "ffn_down.weight", kinds[model.down_format], [F, H], w["down"])]
    tensors.append(("output_norm.weight", gw.GGML_F32, [H], f32(model.final_norm)))
    if not tied:
        tensors.append(("output.weight", gw.GGML_Q6_K, [H, V], model.head))
    tensors = [t for t in tensors if t[0] not in skip] + list(extra)
    metadata = [("general.architecture", gw.STRING, "qwen3"), ("qwen3.block_count", gw.U32, d["layers"]),
                ("qwen3.embedding_length", gw.U32, H), ("qwen3.feed_forward_length", gw.U32, F),
                ("qwen3.attention.head_count", gw.U32, d["q_heads"]), ("qwen3.attention.head_count_kv", gw.U32, d["kv_heads"]),
                ("qwen3.attention.key_length", gw.U32, D), ("qwen3.attention.value_length", gw.U32, D),
                ("qwen3.attention.layer_norm_rms_epsilon", gw.F32, 1e-6), ("qwen3.rope.freq_base", gw.F32, model.rope_theta)]
    if parts == 1:
        gw.write_gguf(path, metadata + list(more_metadata), tensors)
        return path
    return write_split(path, metadata + list(more_metadata), tensors, parts)


def write_split(path, metadata, tensors, parts):
    """The file as a split GGUF of `parts` parts, NAME-0000K-of-0000N.gguf: the first holds the metadata and no tensor
    (as llama.cpp's splitter may leave it), the others the tensors in order and split.* alone."""
    stem = str(path)[:-len(".gguf")]
    names = [f"{stem}-{k + 1:05d}-of-{parts:05d}.gguf" for k in range(parts)]
    split = lambda k: [("split.no", gw.U16, k), ("split.count", gw.U16, parts), ("split.tensors.count", gw.I32, len(tensors))]
    gw.write_gguf(names[0], list(metadata) + split(0), [])
    share = (len(tensors) + parts - 2) // (parts - 1)
    for k in range(1, parts):
        gw.write_gguf(names[k], split(k), tensors[(k - 1) * share:k * share])
    return names


def test_a_split_file_reads_as_one(tmp_path):
    """GgufFile.cpp:167-201: the parts in split order are one file, with the first part's metadata and one tensor
    numbering; a part alone, parts out of order, a part missing or twice, and a wrong tensor count are refused."""
    whole = tmp_path / "whole.gguf"
    tensors = model_file(whole)
    raw = open(whole, "rb").read()
    assert raw[:4] == b"GGUF"
    metadata = [("general.architecture", gw.STRING, "qwen3"), ("qwen3.block_count", gw.U32, 1)]
    names = write_split(tmp_path / "model.gguf", metadata, tensors, 3)
    f, one = gguf.GgufFile(names), gguf.GgufFile(whole)
    assert f.string("general.architecture") == "qwen3" and f.unsigned("split.count") == 3 and f.unsigned("split.no") == 0
    assert [t.name for t in f.tensors] == [t.name for t in one.tensors]
    for a, b in zip(f.tensors, one.tensors):
        assert (a.ggml_type, a.dims, a.bytes, a.format) == (b.ggml_type, b.dims, b.bytes, b.format)
        assert np.array_equal(f.data(a), one.data(b))
    assert f.find("output.weight").name == "output.weight"
    for bad in ([names[1]], names[:2], [names[0], names[2], names[1]], names + [names[2]], [names[1], names[0], names[2]]):
        with pytest.raises(splash_amd.SplashError):
            gguf.GgufFile(bad)
    # another number of tensors than the first part states
    short = write_split(tmp_path / "short.gguf", metadata, tensors, 3)
    gw.write_gguf(short[2], [("split.no", gw.U16, 2), ("split.count", gw.U16, 3)], [])
    with pytest.raises(splash_amd.SplashError, match="split.tensors.count"):
        gguf.GgufFile(short)
    # a later part's general.alignment is not read: its tensors lie at the first part's alignment (here 32, which the
    # part's own claim of 4096 would refuse for offsets that are multiples of 32 only)
    claims = write_split(tmp_path / "claims.gguf", metadata, tensors, 3)
    share = (len(tensors) + 1) // 2
    gw.write_gguf(claims[2], [("split.no", gw.U16, 2), ("split.count", gw.U16, 3), ("general.alignment", gw.U32, 4096)], tensors[share:], alignment=32)
    claimed = gguf.GgufFile(claims)
    offsets = np.cumsum([0] + [(np.asarray(d).nbytes + 31) // 32 * 32 for _, _, _, d in tensors[share:]])[:-1]
    assert any(int(o) % 4096 for o in offsets)                                 # the layout really is the first part's
    for a, b in zip(claimed.tensors, one.tensors):
        assert a.name == b.name and np.array_equal(claimed.data(a), one.data(b))
    # a single file that says it is a part of several
    alone = tmp_path / "alone.gguf"
    gw.write_gguf(alone, metadata + [("split.count", gw.U16, 2)], tensors)
    with pytest.raises(splash_amd.SplashError, match="split.count"):
        gguf.GgufFile(alone)


@pytest.mark.gpu
@pytest.mark.parametrize("value_format,tied,parts", [(orc.FMT_Q6K, False, 1), (orc.FMT_Q4K, True, 1), (orc.FMT_Q6K, False, 3),
                                                     (orc.FMT_Q3K, True, 1), (orc.FMT_Q40, True, 1), (orc.FMT_Q50, False, 1)])
def test_a_dense_decoder_loads_from_a_file(tmp_path, value_format, tied, parts):
    """spg_dense_dimensions and spo_dense_verify_load_gguf: the driver built from a file gives, bit for bit, the logits
    and the acceptance of the driver built by hand from the same tensors: q | k | v fused with the values in another
    format than the queries and keys, a tied head, and the refusal of tensors the loader would ignore. The Q3_K, Q4_0 and
    Q5_0 cases keep the values and the token table in that format, which the hand-built driver takes as the rewritten
    Q6_K or Q8_0 blocks."""
    from splash_amd import verify
    from tests.dense_reference import DenseModel
    backend = splash_amd.Backend(0)
    model = DenseModel(seed=5, hidden=512, q_heads=16, kv_heads=8, head_dim=64, ffn=768, vocabulary=2048, layers=2, down_format=orc.FMT_Q6K)
    rewritten = {orc.FMT_Q3K: gw.GGML_Q3_K, orc.FMT_Q40: gw.GGML_Q4_0, orc.FMT_Q50: gw.GGML_Q5_0}
    if value_format in rewritten:
        for i, w in enumerate(model.layers):
            w["v"] = orc.make_native(value_format, 512, 512, 40 + i)
        model.embedding = orc.make_native(value_format, 2048, 512, 50)
        model.table_format = value_format
    elif value_format != orc.FMT_Q4K:   # the values in the format a Q4_K_M file keeps them in
        for w in model.layers:
            w["v"] = orc.quantize_rows(value_format, orc.dequant_rows(orc.FMT_Q4K, w["v"], 512, 512))
    if tied:
        model.head = model.embedding
    # what the kernels read: a Q3_K tensor as the Q6_K blocks of its values
    seen = lambda fmt, native: ops.rewrite_native(rewritten[fmt], native) if fmt in rewritten else (fmt, native)
    table_format = value_format if value_format in rewritten else orc.FMT_Q4K
    path = dense_model_file(tmp_path / "dense.gguf", model, value_format, tied, parts=parts)   # a path, or a split file's parts
    rows, context = 16, 200
    rng = np.random.default_rng(1)
    tokens = rng.integers(0, 2048, rows).astype(np.uint32)
    pages = (context + 16 + ops.PAGE_TOKENS - 1) // ops.PAGE_TOKENS
    loaded = verify.DenseVerify.from_gguf(backend, gguf.GgufFile(path), max_lanes=1, physical_pages=pages + 1, page_table_entries=pages)
    d = loaded.dims
    assert (d.hidden, d.q_heads, d.kv_heads, d.head_dim, d.ffn, d.vocabulary, d.layers, d.rotary_pairs, d.normalize_heads) == \
        (512, 16, 8, 64, 768, 2048, 2, 32, 1) and d.rope_theta == model.rope_theta

    def hand_built():
        from splash_amd import ops as o
        P = lambda segs, k, f32=False: o.Projection.from_native(backend, segs, k, float32=f32)
        gpu = verify.DenseVerify(backend, 512, 16, 8, 64, 768, 2048, 2, rope_theta=model.rope_theta, max_lanes=1, physical_pages=pages + 1,
                                 page_table_entries=pages)
        for i, w in enumerate(model.layers):
            value_seen, values = seen(value_format, w["v"])
            gpu.set_layer(i, P([(orc.FMT_Q4K, 1024, w["q"]), (orc.FMT_Q4K, 512, w["k"]), (value_seen, 512, values)], 512),
                          P([(orc.FMT_Q4K, 512, w["o"])], 1024), P([(orc.FMT_Q4K, 768, w["gate"])], 512), P([(orc.FMT_Q4K, 768, w["up"])], 512),
                          P([(orc.FMT_Q6K, 512, w["down"])], 768), backend.from_array(w["input_norm"]), backend.from_array(w["post_norm"]),
                          backend.from_array(w["q_norm"]), backend.from_array(w["k_norm"]))
        table_seen, table = seen(table_format, model.embedding)
        head_seen, head = seen(table_format if tied else orc.FMT_Q6K, model.head)
        gpu.set_head(table_seen, backend.from_array(table), backend.from_array(model.final_norm), P([(head_seen, 2048, head)], 512, True))
        return gpu
    outputs = []
    for gpu in (loaded, hand_built()):
        model.physical_pages = pages + 1
        model.table = np.random.default_rng(99).permutation(pages + 1)[:pages].astype(np.uint64)
        gpu.buffer(verify.PAGE_TABLE).upload(model.table)
        model.seed_context(gpu, context, np.random.default_rng(3))
        lane = verify.Lane(rows, context)
        gpu.set_block([lane], tokens)
        backend.run(gpu.encode([lane], commit=True))
        outputs.append((gpu.buffer(verify.LOGITS).download(np.float32, rows * 2048), gpu.results([lane])))
    assert outputs[0][0].tobytes() == outputs[1][0].tobytes()
    for a, b in zip(outputs[0][1], outputs[1][1]):
        assert np.array_equal(a, b)
    assert np.isfinite(outputs[0][0]).all() and np.abs(outputs[0][0]).max() > 0
    # a tensor the loader would ignore, a missing one and a wrong shape are refused, all named in one message
    bad = tmp_path / "bad.gguf"
    dense_model_file(bad, model, value_format, tied, extra=[("blk.0.attn_q.bias", gw.GGML_F32, [512], np.zeros(512, np.float32))])
    with pytest.raises(splash_amd.SplashError, match="attn_q.bias"):
        verify.DenseVerify.from_gguf(backend, gguf.GgufFile(bad), physical_pages=pages + 1)
    dense_model_file(bad, model, value_format, tied, skip=("blk.1.ffn_up.weight", "output_norm.weight"))
    with pytest.raises(splash_amd.SplashError, match="blk.1.ffn_up.weight is missing; output_norm.weight is missing"):
        verify.DenseVerify.from_gguf(backend, gguf.GgufFile(bad), physical_pages=pages + 1)
    backend.close()


def test_dense_geometry_from_metadata(tmp_path):
    """spg_dense_dimensions (no device): the geometry a file's metadata and token table name; a missing key, another
    epsilon and a partial rotary embedding are refused."""
    from splash_amd import _native as nat
    import ctypes
    from tests.dense_reference import DenseModel
    model = DenseModel(seed=6, hidden=256, q_heads=4, kv_heads=2, head_dim=64, ffn=256, vocabulary=256, layers=1, rope_theta=5e5)
    path = tmp_path / "tiny.gguf"
    dense_model_file(path, model, orc.FMT_Q4K, tied=True)
    d = nat.DenseDimensions()
    f = gguf.GgufFile(path)
    splash_amd.check(splash_amd.lib.spg_dense_dimensions(f.handle, ctypes.byref(d)))
    assert (d.hidden, d.q_heads, d.kv_heads, d.head_dim, d.ffn, d.vocabulary, d.layers, d.rotary_pairs, d.normalize_heads, d.rope_theta) == \
        (256, 4, 2, 64, 256, 256, 1, 32, 1, 5e5)
    raw = open(path, "rb").read()
    # Same-length byte edits of the file: a key that is no longer there, an architecture whose rows are laid out for
    # another rotation (llama: interleaved pairs), a missing RoPE base; each is refused with a message that names it.
    for name, edit, message in (("key", lambda b: b.replace(b"qwen3.block_count", b"qwen3.block_coumt"), "block_count"),
                                ("architecture", lambda b: b.replace(b"general.architecture", b"general.architectura"), "architecture"),
                                ("llama", lambda b: b.replace(b"qwen3", b"llama"), "llama is not one the dense driver computes"),
                                ("base", lambda b: b.replace(b"qwen3.rope.freq_base", b"qwen3.rope.freq_bass"), "rope.freq_base")):
        bad = tmp_path / f"{name}.gguf"
        open(bad, "wb").write(edit(raw))
        broken = gguf.GgufFile(bad)
        with pytest.raises(splash_amd.SplashError, match=message):
            splash_amd.check(splash_amd.lib.spg_dense_dimensions(broken.handle, ctypes.byref(d)))
    # a long-context file (YaRN or linear RoPE scaling) has no tensor the loader would miss: its metadata refuses it,
    # and one error names everything the metadata asks for that the kernels do not do
    for scaling, refused in (("none", False), ("yarn", True), ("linear", True)):
        scaled = tmp_path / f"{scaling}.gguf"
        dense_model_file(scaled, model, orc.FMT_Q4K, tied=True, more_metadata=[("qwen3.rope.scaling.type", gw.STRING, scaling)])
        g = gguf.GgufFile(scaled)
        if refused:
            with pytest.raises(splash_amd.SplashError, match=f"rope.scaling.type {scaling}"):
                splash_amd.check(splash_amd.lib.spg_dense_dimensions(g.handle, ctypes.byref(d)))
        else:
            splash_amd.check(splash_amd.lib.spg_dense_dimensions(g.handle, ctypes.byref(d)))
    both = tmp_path / "both.gguf"
    dense_model_file(both, model, orc.FMT_Q4K, tied=True, more_metadata=[("qwen3.rope.scaling.type", gw.STRING, "yarn"),
                                                                         ("qwen3.rope.dimension_count", gw.U32, 32)])
    g = gguf.GgufFile(both)
    with pytest.raises(splash_amd.SplashError, match="partial rotary.*rope.scaling.type yarn"):
        splash_amd.check(splash_amd.lib.spg_dense_dimensions(g.handle, ctypes.byref(d)))


# ------------------------------------------------------------------ the hybrid targets' files (qwen35, qwen35moe)
HYBRID = dict(hidden=256, vocabulary=1024, layers=4, q_heads=8, kv_heads=2, head_dim=128, gdn_key_heads=2, gdn_value_heads=4,
              experts=16, top_k=2, expert_ffn=256)


def test_hybrid_dimensions_come_from_the_metadata(tmp_path):
    """GgufImage.cpp:874-936: the geometry of a qwen35moe file, the prediction blocks after the target's layers left out,
    and the refusals: an architecture the hybrid driver does not compute, a state size the kernels do not hold."""
    from splash_amd import _native as nat
    from tests.dense_reference import DenseModel
    from tests.hybrid_reference import HybridModel, hybrid_model_file
    import ctypes
    model = HybridModel(seed=3, **HYBRID, shared_slices=1, shared_gate=True, gated_attention=True, file_form=True)
    path = hybrid_model_file(tmp_path / "hybrid.gguf", model, more_metadata=[("qwen35moe.nextn_predict_layers", gw.U32, 0)])
    d = nat.HybridDimensions()
    f = gguf.GgufFile(str(path))
    nat.check(nat.lib.spg_hybrid_dimensions(f.handle, ctypes.byref(d)))
    assert (d.hidden, d.vocabulary, d.layers, d.attention_interval, d.q_heads, d.kv_heads, d.head_dim, d.rotary_pairs) == (256, 1024, 4, 4, 8, 2, 128, 64)
    assert (d.gdn_key_heads, d.gdn_value_heads, d.experts, d.top_k, d.expert_ffn, d.shared_slices, d.shared_gate, d.dense_ffn) == (2, 4, 16, 2, 256, 1, 1, 0)
    assert d.gdn_packed_width == model.packed_width == 1600 and d.gated_attention == 1 and d.normalize_heads == 1
    # a dense file is not a hybrid one
    dense = DenseModel(seed=5, hidden=512, q_heads=8, kv_heads=2, head_dim=64, ffn=768, vocabulary=256, layers=1)
    other = gguf.GgufFile(str(dense_model_file(tmp_path / "dense.gguf", dense, orc.FMT_Q6K, tied=True)))
    with pytest.raises(splash_amd.SplashError, match="qwen35"):
        nat.check(nat.lib.spg_hybrid_dimensions(other.handle, ctypes.byref(d)))
    # the last block is a prediction block: one layer fewer
    path = hybrid_model_file(tmp_path / "nextn.gguf", model, more_metadata=[("qwen35moe.nextn_predict_layers", gw.U32, 1)])
    later = gguf.GgufFile(str(path))
    nat.check(nat.lib.spg_hybrid_dimensions(later.handle, ctypes.byref(d)))
    assert d.layers == 3
    # a state size the kernels do not hold: the same file with the value patched
    path = hybrid_model_file(tmp_path / "state.gguf", model)
    raw = bytearray(open(path, "rb").read())
    at = raw.index(b"qwen35moe.ssm.state_size") + len(b"qwen35moe.ssm.state_size") + 4
    raw[at:at + 4] = (64).to_bytes(4, "little")
    open(tmp_path / "state64.gguf", "wb").write(raw)
    patched = gguf.GgufFile(str(tmp_path / "state64.gguf"))
    with pytest.raises(splash_amd.SplashError, match="ssm.state_size"):
        nat.check(nat.lib.spg_hybrid_dimensions(patched.handle, ctypes.byref(d)))


@pytest.mark.gpu
def test_a_hybrid_decoder_from_a_file_computes_the_oracles_step(backend, tmp_path):
    """A qwen35moe file as llama.cpp lays it out (value heads tiled, F32 gates, router and norms, experts of three
    dimensions, a gated shared expert, gated attention) through spg_hybrid_dimensions and spo_hybrid_verify_load_gguf:
    the step, layer by layer, against the oracle over the model's own (grouped) tensors. The file with the fused
    ffn_gate_up_exps gives the same logits bit for bit; refusals name what the loader cannot read."""
    from splash_amd import verify
    from tests.hybrid_reference import HybridModel, hybrid_model_file
    from tests.test_hybrid_step_gpu import check_step
    print("case hybrid gguf", flush=True)
    model = HybridModel(seed=43, **HYBRID, shared_slices=1, shared_gate=True, gated_attention=True, file_form=True)
    path = hybrid_model_file(tmp_path / "hybrid.gguf", model)
    rng = np.random.default_rng(9)
    lanes = [verify.HybridLane(6, 70, table_first=0), verify.HybridLane(16, 300, table_first=2)]
    tokens = rng.integers(0, 1024, 22).astype(np.uint32)

    def run(file_path):
        gpu = model.build_gpu_from_file(backend, file_path, max_lanes=2, pages_per_lane=2)
        seed = np.random.default_rng(10)
        model.seed_context(seed)
        model.seed_states(seed, lanes=2)
        return gpu
    check_step(backend, model, run(path), lanes, tokens)

    def whole_step(gpu):
        gpu.set_block(lanes, tokens)
        backend.run(gpu.encode(lanes, commit=False))
        return gpu.buffer(verify.LOGITS).download(np.float32, 22 * 1024).copy()
    assert np.array_equal(whole_step(run(hybrid_model_file(tmp_path / "fused.gguf", model, fused_gate_up=True))), whole_step(run(path)))
    # what the loader refuses: a quantized gate tensor, a tensor nobody reads, a missing one
    w0 = model.layers[0]
    quantized_beta = ("blk.0.ssm_beta.weight", gw.GGML_Q4_K, [256, 4], orc.quantize_rows(orc.FMT_Q4K, w0["gate_rows"][:4]))
    for name, kwargs, needle in (("quantized", dict(skip=("blk.0.ssm_beta.weight",), extra=(quantized_beta,)), "ssm_beta.weight is not of 16- or 32-bit floats"),
                                 ("bias", dict(extra=(("blk.1.ffn_gate_inp.bias", gw.GGML_F32, [16], np.zeros(16, np.float32)),)), "ffn_gate_inp.bias is not read"),
                                 ("missing", dict(skip=("blk.2.ssm_out.weight",)), "blk.2.ssm_out.weight is missing")):
        with pytest.raises(splash_amd.SplashError, match=needle):
            model.build_gpu_from_file(backend, hybrid_model_file(tmp_path / f"{name}.gguf", model, **kwargs), max_lanes=1, pages_per_lane=2)
