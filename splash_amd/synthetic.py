"""Synthetic weights and contexts of the named shapes, generated directly in GGUF's native block
formats (no quantizer pass): codes are uniform, scale fields are drawn so that the dequantized
weights are zero-mean with a standard deviation near 0.02, the magnitudes a model's have (the
reference's GEMM fixtures draw their scales the same way: dev/tests/engine/GgufFormatReference.hpp:295-323)."""
import numpy as np

from . import ops


def q4k_native(rng, rows, k):
    """Native Q4_K rows [rows][k / 256][144]: value = d sc code - dmin mn with mn = round(7.5 sc), dmin = d."""
    blocks = k // 256
    out = np.empty((rows, blocks, 144), dtype=np.uint8)
    d = rng.uniform(0.0005, 0.0009, (rows, blocks)).astype(np.float16)
    out[..., 0:2] = d.view(np.uint8).reshape(rows, blocks, 2)
    out[..., 2:4] = out[..., 0:2]
    sc = rng.integers(4, 9, (rows, blocks, 8), dtype=np.uint8)
    mn = np.rint(7.5 * sc).astype(np.uint8)
    s = np.empty((rows, blocks, 12), dtype=np.uint8)
    s[..., 0:4] = sc[..., 0:4] | ((sc[..., 4:8] >> 4) << 6)
    s[..., 4:8] = mn[..., 0:4] | ((mn[..., 4:8] >> 4) << 6)
    s[..., 8:12] = (sc[..., 4:8] & 0xF) | ((mn[..., 4:8] & 0xF) << 4)
    out[..., 4:16] = s
    out[..., 16:] = rng.integers(0, 256, (rows, blocks, 128), dtype=np.uint8)
    return out.reshape(-1)


def q6k_native(rng, rows, k):
    """Native Q6_K rows [rows][k / 256][210]: value = d sc (q - 32)."""
    blocks = k // 256
    out = np.empty((rows, blocks, 210), dtype=np.uint8)
    out[..., :192] = rng.integers(0, 256, (rows, blocks, 192), dtype=np.uint8)
    sc = rng.integers(12, 29, (rows, blocks, 16)).astype(np.int8) * rng.choice(np.array([-1, 1], dtype=np.int8), (rows, blocks, 16))
    out[..., 192:208] = sc.view(np.uint8)
    d = rng.uniform(0.00004, 0.00007, (rows, blocks)).astype(np.float16)
    out[..., 208:210] = d.view(np.uint8).reshape(rows, blocks, 2)
    return out.reshape(-1)


def native(rng, fmt, rows, k):
    return q4k_native(rng, rows, k) if fmt == ops.FMT_Q4K else q6k_native(rng, rows, k)


def kv_pages(rng, kv_heads, head_dim, pages):
    """Raw page bytes [pages][page_bytes] of an INT8 context: codes uniform in [-127, 127], fp16 scales
    of values whose largest magnitude is a few units (K/V ~ N(0, 1))."""
    helper = ops.KvPages.__new__(ops.KvPages)
    helper.kv_heads, helper.head_dim, helper.page_bytes = kv_heads, head_dim, ops.kv_page_bytes(kv_heads, head_dim)
    shape = (pages, kv_heads, ops.PAGE_TOKENS, head_dim)
    kc = np.clip(np.rint(rng.standard_normal(shape, dtype=np.float32) * 36), -127, 127).astype(np.int8)
    vc = np.clip(np.rint(rng.standard_normal(shape, dtype=np.float32) * 36), -127, 127).astype(np.int8)
    ks = rng.uniform(2.5, 4.5, shape[:3]).astype(np.float32) / 127
    vs = rng.uniform(2.5, 4.5, shape[:3]).astype(np.float32) / 127
    return helper.pack_pages(kc, ks, vc, vs)
