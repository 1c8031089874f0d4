"""The C-ABI library: builds in-tree, exports every symbol include/iris_dev.h
declares, and behaves sanely without a GPU (no compute is attempted here)."""
import os
import re

import pytest

import iris_c_amd

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(iris_c_amd.LIB_PATH):
        iris_c_amd.build()
    return iris_c_amd.load()


def declared_functions():
    names = []
    for header in ("iris_dev.h", "iris_rope.h"):
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names += re.findall(r"\b(iris_(?:dev|rope)_\w+)\s*\(", text)
    return names


def test_every_declared_symbol_is_exported_and_bound(lib):
    names = declared_functions()
    assert len(names) >= 14
    assert set(names) == set(iris_c_amd.ABI), set(names) ^ set(iris_c_amd.ABI)
    for n in names:
        assert getattr(lib, n) is not None


def test_reference_signatures_are_kept():
    """Argument lists of the two hot-path entries, as the reference header declares them."""
    text = re.sub(r"\s+", " ", open(os.path.join(ROOT, "include", "iris_dev.h")).read())
    assert ("void iris_dev_head_norm_rope(uint16_t *x, int ld, const float *w, const float *rope_cos, "
            "const float *rope_sin, int seq, int heads, int head_dim, float eps, int split_half);") in text
    assert ("void iris_dev_attention(uint16_t *out, int ldo, const uint16_t *q, const uint16_t *k, "
            "const uint16_t *v, int ldi, int seq_q, int seq_k, int heads, int kv_heads, int head_dim, "
            "float scale, int causal, const int *key_mask);") in text


def test_no_gpu_means_no_silent_fallback(lib):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    assert lib.iris_dev_init() == 0
    assert lib.iris_dev_available() == 0
    assert lib.iris_dev_alloc(16) is None
    lib.iris_dev_last_error()
    # compute entries refuse to run (and say so) instead of computing on the CPU
    lib.iris_dev_attention(None, 0, None, None, None, 0, 4, 4, 1, 1, 128, 1.0, 0, None)
    assert lib.iris_dev_last_error() != 0
    lib.iris_dev_head_norm_rope(None, 0, None, None, None, 4, 1, 128, 1e-6, 0)
    assert lib.iris_dev_last_error() != 0
    lib.iris_dev_attention_qnorm(None, 0, None, None, None, 0, 4, 4, 1, 1, 128, 1.0, 0, None, None, None, None, 1e-6, 0)
    assert lib.iris_dev_last_error() != 0
    lib.iris_dev_linear_bf16(None, None, None, 4, 8, 4)
    lib.iris_dev_linear_bf16_qknorm(None, None, None, 4, 8, 4, 1, 1, 2, None, None, None, None, 1e-6, 0)
    assert lib.iris_dev_last_error() != 0
    lib.iris_dev_conv2d(None, None, None, None, 4, 4, 64, 128, 3, 1, 1, 1)
    assert lib.iris_dev_last_error() != 0
    lib.iris_dev_group_norm_noalloc(None, None, None, None, 4, 8, 2, 1e-6, 0)
    assert lib.iris_dev_last_error() != 0
    # device-side table generation likewise; the host builders of the same header need no device
    lib.iris_dev_rope_qwen3_tables(None, None, None, 4, 128, 1e6, 0)
    assert lib.iris_dev_last_error() != 0


def test_product_does_not_link_the_oracle(lib):
    import subprocess
    out = subprocess.run(["ldd", iris_c_amd.LIB_PATH], capture_output=True, text=True).stdout
    assert "oracle" not in out and "iris_ref" not in out
    for root, _, files in os.walk(os.path.join(ROOT, "iris_c_amd")):
        for f in files:
            if f.endswith((".c", ".h", ".hip", ".py")):
                src = open(os.path.join(root, f)).read()
                assert "import oracle" not in src and "iris_oracle.h" not in src and "orc_" not in src, f


def test_unmodified_reference_links_against_this_backend(lib):
    """The reference's own host program (models, sampler, CLI, main), compiled with its device path
    enabled, links against this library in place of the reference's GPU backend: every iris_dev_*
    symbol it uses is exported here. Link check only (built where the reference tree exists)."""
    import subprocess
    if not os.path.isdir("/root/reference"):
        pytest.skip("reference tree not present on this machine")
    subprocess.check_call(["make", "-s", "-C", os.path.join(ROOT, "oracle"), "linkcheck"])
    exe = os.path.join(ROOT, "oracle", "_ref", "iris_linked_to_this_backend")
    undefined = subprocess.run(["nm", "-D", "--undefined-only", exe], capture_output=True, text=True, check=True).stdout
    used = sorted({line.split()[-1] for line in undefined.splitlines() if " iris_dev_" in line})
    assert len(used) >= 28
    import iris_c_amd
    assert set(used) <= set(iris_c_amd.ABI), sorted(set(used) - set(iris_c_amd.ABI))
    ldd = subprocess.run(["ldd", exe], capture_output=True, text=True, check=True).stdout
    assert "libiris_dev.so" in ldd and "not found" not in ldd


def test_path_only_archive_links_next_to_a_host_backend():
    """libiris_dev_path.a (the hot path for a host that keeps its own backend): defines the two operators, their
    additions and attach / detach, none of the setup / memory / other-operator symbols, and links into a program
    that defines those itself (tests/path_only_link.c)."""
    import subprocess
    subprocess.check_call(["make", "-s", "-C", ROOT, "path", "pathcheck"], stderr=subprocess.DEVNULL)
    out = subprocess.run(["nm", "--defined-only", os.path.join(ROOT, "iris_c_amd", "libiris_dev_path.a")],
                         capture_output=True, text=True, check=True).stdout
    defined = {line.split()[-1] for line in out.splitlines() if " T iris_dev_" in line}
    assert defined == {"iris_dev_head_norm_rope", "iris_dev_head_norm_rope_qk", "iris_dev_head_norm_rope_qk_streams", "iris_dev_attention",
                       "iris_dev_attention_qnorm",
                       "iris_dev_last_error", "iris_dev_last_kernel", "iris_dev_path_attach", "iris_dev_path_detach"}
    text = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "iris_dev_path.h")).read(), flags=re.S)
    assert set(re.findall(r"\b(iris_dev_\w+)\s*\(", text)) == {"iris_dev_path_attach", "iris_dev_path_detach"}
    assert os.path.exists(os.path.join(ROOT, "tests", "path_only_link.bin"))


def test_division_constant_of_the_norm_rope_kernel(lib):
    """The fast norm+rope kernel turns a unit index into (token, head) with one multiply-high by
    the constant its launcher computes (0 = "one head, no division"). Checked the way the kernel
    uses it, over the whole range the dispatcher admits: unit < 2^24, 1 <= heads < 256."""
    import ctypes as C
    import numpy as np
    magic = lib.iris_norm_rope_magic
    magic.restype, magic.argtypes = C.c_uint32, [C.c_int]
    assert magic(1) == 0                               # 2^32 does not fit: the kernel takes unit / 1 = unit
    top = 1 << 24
    edge = np.array([0, 1, 2, top - 2, top - 1], dtype=np.uint64)
    for d in range(2, 256):
        m = np.uint64(magic(d))
        assert 0 < m < (1 << 32)
        if d in (2, 3, 24, 30, 32, 40, 48, 60, 64, 96, 255):
            units = np.arange(top, dtype=np.uint64)    # every admitted unit
        else:                                          # multiples of d and their neighbours, a stride, the ends
            mult = np.arange(0, top, d, dtype=np.uint64)[-4096:]
            units = np.unique(np.concatenate([edge, mult, mult - np.uint64(1), mult[:-1] + np.uint64(d - 1),
                                              np.arange(0, top, 4099, dtype=np.uint64), np.arange(70000, dtype=np.uint64)]))
            units = units[units < top]
        assert np.array_equal((units * m) >> np.uint64(32), units // np.uint64(d)), d
