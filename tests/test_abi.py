"""The C-ABI library loads without a GPU and exports every symbol include/*.h declares (CPU)."""
import ctypes
import os
import re

import numpy as np
import pytest

import splash_amd
from splash_amd import ops
from tests import oracle as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    names = set()
    for header in ("splash_hip.h", "splash_ops.h", "splash_gguf.h"):
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names.update(re.findall(r"\b(sp[og]?_[a-z0-9_]+)\s*\(", text))
    names.discard("sp_completion")
    return sorted(names)


def test_library_exports_every_declared_symbol():
    symbols = declared_symbols()
    assert len(symbols) > 50
    missing = [s for s in symbols if not hasattr(splash_amd.lib, s)]
    assert not missing, missing


def test_kernels_are_registered_by_name():
    for name in ("gguf_prepare_table", "gguf_dequant_q4k", "gguf_dequant_q6k", "gguf_dequant_q5k", "gguf_dequant_q80",
                 "gguf_decode_q4k_m16_a", "gguf_decode_q6k_m16_a_f32", "gguf_decode_q4k_m32_g", "gguf_decode_q6k_m64_r",
                 "gguf_decode_q5k_m16_gt", "gguf_decode_q80_m64_rn", "gguf_decode_mixed_m16_a", "gguf_decode_mixed_m64_a",
                 "gguf_dequant_iq4xs", "gguf_decode_iq4xs_m16_rn", "gguf_decode_iq4nl_m32_gt", "gguf_embed_iq4xs", "gguf_embed_iq4nl", "state_quantize", "state_dequantize_bf16_state", "state_copy",
                 "draft_verify_rows"):
        assert splash_amd.lib.sp_kernel_exists(name.encode()), name
    assert not splash_amd.lib.sp_kernel_exists(b"no_such_kernel")


@pytest.mark.parametrize("fmt", ops.FORMATS)
def test_image_is_a_permutation_of_the_native_rows(fmt):
    """decode(retile(native)) == decode(native) follows from unpack(pack(native)) == native."""
    native = orc.fixture(fmt, 48, 768, 5)
    image = ops.pack_gguf_image(fmt, native, 48, 768)
    assert image.size == native.size == ops.gguf_image_bytes(fmt, 48, 768)
    assert np.array_equal(ops.unpack_gguf_image(fmt, image, 48, 768), native)
    if fmt in (ops.FMT_Q4K, ops.FMT_IQ4XS, ops.FMT_IQ4NL, ops.FMT_Q80):  # byte-for-byte re-ordering
        assert np.array_equal(np.sort(image), np.sort(native))


def test_pack_rejects_partial_tiles():
    native = np.zeros(144 * 3 * 10, dtype=np.uint8)
    with pytest.raises(ValueError):
        ops.pack_gguf_image(ops.FMT_Q4K, native, 10, 768)
    with pytest.raises(ValueError):
        ops.pack_gguf_image(7, native, 16, 768)


def test_linear_plans_without_a_device():
    """Linear::plan partitions K to fill the device; LinearPlan rejects what no tile runs."""
    linear = ops.Linear(calibration=(256, 8, 2))

    class FakeProjection:
        pass
    # plans need only shapes: build a projection handle over no memory is not possible, so check
    # the scratch sizing entry point, which plans every epilogue
    table, partials, counters = linear.scratch_size(5120, 25600, 16)
    assert table == ops.gguf_table_bytes(25600, 16)
    assert partials > 0 and counters > 0   # a 5120-column projection of K 25600 splits across workgroups
    table, partials, counters = linear.scratch_size(151936, 5120, 16)
    # the LM head fills the device in whole rounds; only the workgroups of the last, partial round split
    assert partials <= 16 * 255 * 4 * 256 * 4
    with pytest.raises(ValueError):
        linear.scratch_size(5120, 25600, 257)
    with pytest.raises(ValueError):
        linear.scratch_size(5121, 25600, 16)


def test_headers_are_plain_c_and_a_c_caller_links(tmp_path):
    """The boundary is a C ABI: every header compiles as C11 on its own, and a C program that calls host-side entry
    points (a weight image's size, the rewrite of a Q4_0 block, a lookup index) links against the library and runs."""
    import shutil
    import subprocess
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no C compiler here")
    include = os.path.join(ROOT, "include")
    for header in sorted(os.listdir(include)):
        done = subprocess.run([gcc, "-x", "c", "-std=c11", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", "-I", include, "-"],
                              input=f'#include "{header}"\n', text=True, capture_output=True)
        assert done.returncode == 0, (header, done.stderr[-800:])
    source = tmp_path / "caller.c"
    source.write_text(r'''
#include "splash_ops.h"
#include <stdio.h>
#include <string.h>
int main(void) {
  if (spo_gguf_image_bytes(0, 16, 256) != 16u * 144u) return 1;
  unsigned char q40[8 * 18], q80[8 * 34];
  memset(q40, 0x21, sizeof q40);                       /* nibbles 1 and 2: codes - 8 = -7 and -6 */
  if (spo_gguf_rewrite_format(2) != 6 || spo_gguf_rewrite(2, q40, 1, q80) != SP_OK) return 2;
  if ((signed char)q80[2] != -7 || (signed char)q80[2 + 16] != -6 || q80[0] != 0x21) return 3;
  spo_lookup_index *index = NULL;
  const uint32_t tokens[] = {1, 2, 3, 4, 9, 1, 2, 3};
  uint32_t length = 0, end = 0, next[2] = {0, 0};
  if (spo_lookup_index_create(&index) != SP_OK || spo_lookup_index_append(index, tokens, 8) != SP_OK) return 4;
  if (spo_lookup_index_match(index, &length, &end) != SP_OK || length != 3 || end != 2) return 5;
  if (spo_lookup_index_proposals(index, 2, next) != 2 || next[0] != 4 || next[1] != 9) return 6;
  spo_lookup_index_destroy(index);
  puts("ok");
  return 0;
}
''')
    from splash_amd import _native as nat
    library = nat.library_path()
    binary = tmp_path / "caller"
    done = subprocess.run([gcc, "-std=c11", "-Wall", "-Werror", "-I", include, str(source), "-o", str(binary), library,
                           f"-Wl,-rpath,{os.path.dirname(library)}"], capture_output=True, text=True)
    assert done.returncode == 0, done.stderr[-1500:]
    ran = subprocess.run([str(binary)], capture_output=True, text=True, timeout=120)
    assert ran.returncode == 0 and ran.stdout.strip() == "ok", (ran.returncode, ran.stdout, ran.stderr[-800:])
