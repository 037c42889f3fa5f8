"""CPU-only checks of the C ABI: the library loads, exports every symbol the header declares,
and rejects bad arguments before touching a GPU (return code -1 + message)."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "kascade_hip.h")


@pytest.fixture(scope="module")
def lib():
    from kascade_amd import _lib
    if not _lib.LIB_PATH.exists():
        from kascade_amd import build
        build.build()
    return _lib.load()


def _declared_functions():
    import glob
    names = set()
    for path in glob.glob(os.path.join(ROOT, "include", "*.h")):
        text = re.sub(r"/\*.*?\*/", "", open(path).read(), flags=re.S)
        names |= set(re.findall(r"\b(kascade_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


def test_header_symbols_are_exported_and_bound(lib):
    from kascade_amd import _lib
    names = _declared_functions()
    assert len(names) >= 14
    for n in names:
        assert hasattr(lib, n), f"{n} declared under include/ but not exported"
        assert n in _lib.SIGNATURES, f"{n} has no ctypes signature"
    assert sorted(_lib.SIGNATURES) == names


def test_abi_version_and_error_buffer(lib):
    assert lib.kascade_abi_version() >= 1
    assert isinstance(lib.kascade_get_last_error(), bytes)


def test_topk_workspace_sizing(lib):
    assert lib.kascade_topk_workspace_bytes(128, 1000) == 0          # short rows: one workgroup per row
    assert lib.kascade_topk_workspace_bytes(8192, 32768) == 0        # too many rows for the workspace
    n = lib.kascade_topk_workspace_bytes(32, 524288)
    assert n == 4 * 32 * (2048 + 2 + 8 + 16 * 36)   # 16 chunks of 32768 entries


def _err(lib):
    return lib.kascade_get_last_error().decode()


def test_sorted_topk_workspace_and_argument_checks(lib):
    import ctypes
    assert lib.kascade_topk_sorted_workspace_bytes(8192, 32768, 3328) == 0     # lists of up to 4096 entries: LDS
    assert (lib.kascade_topk_sorted_workspace_bytes(32, 524288, 52480)
            == (8 * 32 * 52480 + 255) // 256 * 256 + lib.kascade_topk_workspace_bytes(32, 524288))
    p = ctypes.c_void_p(256)
    assert lib.kascade_topk_sorted_call(p, p, 4, 10000, 10000, None, 1, 5000, None, None) == -1
    assert "workspace" in _err(lib)
    assert lib.kascade_topk_sorted_call(p, p, 4, 100, 100, None, 1, 101, p, None) == -1
    assert "k <= uniform_len" in _err(lib)


def test_null_pointers_are_rejected(lib):
    from kascade_amd._lib import Strides
    s = Strides(8, 8, 8)
    assert lib.kascade_decode_reuse_call(None, None, None, None, None, None, None, None, 1, 128, 128, 8, None, None) == -1
    assert "null pointer" in _err(lib)
    assert lib.kascade_decode_dense_paged_call(None, None, None, None, None, None, None, 1, 128, 8, None, 0, 16, None, None, None, None, None) == -1
    assert "null pointer" in _err(lib)
    assert lib.kascade_decode_recompute_paged_call(None, None, None, None, None, None, None, None, None, None,
                                                   1, 128, 128, 8, 1, None, 0, 16, None, None, None, None, None) == -1
    assert lib.kascade_topk_call(None, None, 1, 10, 10, None, None, 1, 4, 0, None, None) == -1
    assert lib.kascade_prefill_dense_call(None, None, None, None, None, 1, 64, s, s, 1, None) == -1
    assert lib.kascade_prefill_aggregate_call(None, None, None, None, 1, 64, s, s, 0, None) == -1
    assert lib.kascade_prefill_reuse_call(None, None, None, None, None, 10.0, None, 1, 64, 128, 1, s, s, None, None) == -1
    assert lib.kascade_paged_kv_append_call(None, None, None, None, None, None, 1, 1, 1, 16, s, None, None) == -1
    assert lib.kascade_rope_append_paged_call(None, None, None, None, None, None, 64, None, None, 1e-6, None, 0,
                                              None, None, None, None, 4, 16, 1, 1, None) == -1
    assert "null pointer" in _err(lib)


def test_bad_sizes_are_rejected(lib):
    from kascade_amd._lib import Strides
    buf = (C.c_char * 4096)()
    p = C.addressof(buf) & ~15          # fake, 16-byte aligned, never dereferenced: validation fails first
    p += 16
    assert lib.kascade_decode_reuse_paged_call(p, p, p, None, p, p, 0.0, p, p, p, 0, 128, 128, 8, None, 0, 16, None, None, None, None, None, None) == -1
    assert "batch" in _err(lib)
    assert lib.kascade_decode_reuse_paged_call(p, p, p, None, p, p, 10.0, p, p, p, 1, 128, 128, 8, None, 0, 16, None, None, None, None, None, None) == -1
    assert "cache_seqlens" in _err(lib)
    assert lib.kascade_decode_dense_paged_call(p, p, p, None, p, p, p, 1, 128, 8, p, 4, 12, None, None, None, None, None) == -1
    assert "power of two" in _err(lib)
    assert lib.kascade_decode_dense_paged_call(p + 2, p, p, None, p, p, p, 1, 128, 8, None, 0, 16, None, None, None, None, None) == -1
    assert "aligned" in _err(lib)
    hf = Strides(8 * 128 * 128, 128, 128 * 128)      # a head-major [B,G,L,D] cache seen as [B,L,G,D]
    assert lib.kascade_decode_dense_paged_call(p, p, p, None, p, p, p, 1, 128, 8, p, 4, 16, C.byref(hf), None, None, None, None) == -1
    assert "exclude each other" in _err(lib)
    assert lib.kascade_decode_dense_paged_call(p, p, p, None, p, p, p, 1, 128, 8, None, 0, 16,
                                               C.byref(Strides(1024, 4, 128)), None, None, None, None) == -1
    assert "strides" in _err(lib)
    assert lib.kascade_decode_dense_paged_call(p, p, p, None, p, p, p, 1, 128, 8, None, 0, 16, None, p, None, None, None) == -1
    assert "come together" in _err(lib)
    assert lib.kascade_decode_budgets_call(None, 1, 10.0, 1, None, None, None) == -1
    assert lib.kascade_decode_budgets_call(p, 1, 101.0, 1, None, None, None) == -1
    assert "topk_percent" in _err(lib)
    assert lib.kascade_topk_call(p, p, 4, 100, 200, None, None, 1, 8, 0, None, None) == -1
    assert "uniform_len" in _err(lib)
    assert lib.kascade_rope_append_paged_call(p, None, p, p, None, p, 64, None, None, 1e-6, p, 0, p, p, p, p,
                                              4, 12, 1, 1, None) == -1
    assert "power of two" in _err(lib)
    assert lib.kascade_rope_append_paged_call(p, C.byref(Strides(6144, 6140, 128)), p, p, None, p, 64, None, None,
                                              1e-6, p, 0, p, p, p, p, 4, 16, 1, 1, None) == -1
    assert "strides" in _err(lib)
    assert lib.kascade_rope_append_paged_call(p, None, p, p, None, p, 0, None, None, 1e-6, p, 0, p, p, p, p,
                                              4, 16, 1, 1, None) == -1
    assert "max_pos" in _err(lib)
    bad = Strides(100, 4, 128)          # not multiples of 8 elements
    ok = Strides(4096 * 128, 4096, 128)
    assert lib.kascade_prefill_dense_call(p, p, p, p, p, 1, 64, bad, ok, 1, None) == -1
    assert "strides" in _err(lib)
    assert lib.kascade_prefill_reuse_call(p, p, p, p, p, 0.0, p, 1, 64, 128, 1, ok, ok, None, None) == -1
    assert "rolling" in _err(lib)
    assert lib.kascade_prefill_reuse_call(p, p, p, p, p, 10.0, p, 1, 64, 0, 0, ok, ok, None, None) == -1
    assert "max_topk_num" in _err(lib)


def test_shape_descriptors_are_validated(lib):
    """Every *_shaped_call checks its kascade_shape before anything else."""
    from kascade_amd._lib import Shape, Strides
    buf = (C.c_char * 4096)()
    p = (C.addressof(buf) & ~15) + 16
    ok = Strides(4096 * 128, 4096, 128)
    rope = (p, None, p, p, None, p, 64, None, None, 1e-6, p, 0, p, p, p, p, 4, 16, 1, 1, None)
    chunk_dense = (p, p, p, p, p, 1, 0, 64, ok, p, 4, 16, 8, 1, None, None, None)
    budgets = (p, 1, 10.0, 1, None, None, None)
    for fn, args in ((lib.kascade_rope_append_paged_shaped_call, rope),
                     (lib.kascade_prefill_chunk_dense_shaped_call, chunk_dense),
                     (lib.kascade_decode_budgets_shaped_call, budgets)):
        assert fn(None, *args) == -1
        assert "shape" in _err(lib)
        assert fn(C.byref(Shape(8, 96, 0)), *args) == -1
        assert "head_dim" in _err(lib)
        assert fn(C.byref(Shape(0, 128, 0)), *args) == -1
        assert "kv_heads" in _err(lib)
        assert fn(C.byref(Shape(8, 128, 2)), *args) == -1
        assert "dtype" in _err(lib)
    # a valid shape reaches the argument checks of the call itself
    sh = C.byref(Shape(2, 64, 1))
    assert lib.kascade_prefill_chunk_dense_shaped_call(sh, p, p, p, p, p, 1, 16, 64, ok, p, 4, 16, 8, 1, None, None, None) == -1
    assert "multiple of 32" in _err(lib)
    assert lib.kascade_prefill_chunk_dense_shaped_call(sh, p, p, p, p, p, 1, 32, 64, ok, p, 8, 16, 8, 1, None, p, None) == -1
    assert "q_len_rows comes with q_start_rows" in _err(lib)
    assert lib.kascade_rope_append_paged_shaped_call(sh, p, None, p, p, None, p, 0, None, None, 1e-6, p, 0, p, p, p, p,
                                                     4, 16, 1, 1, None) == -1
    assert "max_pos" in _err(lib)
    assert lib.kascade_decode_budgets_shaped_call(sh, p, 1, 101.0, 1, None, None, None) == -1
    assert "topk_percent" in _err(lib)


def test_python_wrappers_fail_loudly_without_gpu():
    import torch
    from kascade_amd import kernels
    from kascade_amd._lib import KascadeError
    if torch.cuda.is_available():
        pytest.skip("GPU present")
    q = torch.zeros(1, 32, 128, dtype=torch.float16)
    with pytest.raises((KascadeError, RuntimeError)):
        kernels.decode_reuse(q, q, q, q, q, q, q)


def test_header_is_plain_c_and_links_from_c(lib, tmp_path):
    """The boundary is a C ABI: the header compiles as C99 (no C++ needed) and a C program
    linked against the library reads the ABI version and gets the error convention
    (-1 + message) without a GPU."""
    import shutil
    import subprocess
    from kascade_amd import _lib
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    src = tmp_path / "abi.c"
    src.write_text(
        '#include <stdio.h>\n#include <string.h>\n#include "kascade_hip.h"\n'
        "int main(void) {\n"
        "    if (kascade_abi_version() < 1) return 2;\n"
        "    if (kascade_topk_call(0, 0, 1, 10, 10, 0, 0, 1, 4, 0, 0, 0) != -1) return 3;\n"
        "    if (strlen(kascade_get_last_error()) == 0) return 4;\n"
        '    printf("%d\\n", kascade_abi_version());\n'
        "    return 0;\n}\n")
    exe = tmp_path / "abi"
    libdir = str(_lib.LIB_PATH.parent)
    subprocess.run([gcc, "-std=c99", "-Wall", "-Werror", "-pedantic", "-I", os.path.join(ROOT, "include"),
                    str(src), "-o", str(exe), "-L", libdir, "-l:" + _lib.LIB_PATH.name,
                    "-Wl,-rpath," + libdir], check=True, capture_output=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True)
    assert int(out.stdout.strip()) == lib.kascade_abi_version()
