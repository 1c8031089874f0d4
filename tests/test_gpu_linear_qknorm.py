"""iris_dev_linear_bf16_qknorm: the projection that normalises its own Q and K columns.

Two yardsticks. The CPU oracle's chain (its linear layer rounded to bf16, then its norm+rope on the Q and on
the K columns: the three calls of iris_transformer_flux.c:3833-3837), to the relative bar of the other
kernels. And the library's own two-call form on its own GEMM, bit for bit: the one-launch kernel rounds the
projection to bf16 and then runs the same function as the stand-alone norm+rope kernel.
"""
import numpy as np
import pytest

import oracle as O
from gpu_harness import Dev, ptr_add, assert_parity

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    d = Dev()
    yield d
    d.lib.iris_dev_linear_backend(0)


def bf16_to_f32(u):
    return (u.astype(np.uint32) << 16).view(np.float32)


def make(seed, rows, k, q_heads, k_heads, extra_cols, hd=128):
    g = np.random.default_rng(seed)
    out = (q_heads + k_heads) * hd + extra_cols
    x = O.f32_to_bf16((g.standard_normal((rows, k)) * 1.3 + 0.1).astype(np.float32))
    w = O.f32_to_bf16((g.standard_normal((out, k)) / np.sqrt(k)).astype(np.float32))
    ang = g.uniform(-3.0, 3.0, (rows, hd // 2)).astype(np.float32)
    return dict(rows=rows, k=k, out=out, q_heads=q_heads, k_heads=k_heads, hd=hd, x=x, w=w,
                wq=(1 + 0.05 * g.standard_normal(hd)).astype(np.float32), wk=(1 + 0.05 * g.standard_normal(hd)).astype(np.float32),
                cos=np.cos(ang), sin=np.sin(ang))


def run(dev, c, one_launch, split, backend):
    lib = dev.lib
    lib.iris_dev_linear_backend(backend)
    x, w, wq, wk, cos, sin = (dev.put(c[n]) for n in ("x", "w", "wq", "wk", "cos", "sin"))
    y = dev.alloc(c["rows"] * c["out"] * 2)
    if one_launch:
        lib.iris_dev_linear_bf16_qknorm(y, x, w, c["rows"], c["k"], c["out"], c["q_heads"], c["k_heads"], c["hd"], wq, wk, cos, sin,
                                        1e-6, split)
    else:
        lib.iris_dev_linear_bf16(y, x, w, c["rows"], c["k"], c["out"])
        if c["q_heads"]:
            lib.iris_dev_head_norm_rope(y, c["out"], wq, cos, sin, c["rows"], c["q_heads"], c["hd"], 1e-6, split)
        if c["k_heads"]:
            lib.iris_dev_head_norm_rope(ptr_add(y, 2 * c["q_heads"] * c["hd"]), c["out"], wk, cos, sin, c["rows"], c["k_heads"], c["hd"],
                                        1e-6, split)
    kernel = dev.dev.last_kernel()
    dev.check()
    got = dev.get(y, (c["rows"], c["out"]), np.uint16)
    dev.free_all()
    return got, kernel


def oracle_chain(orc, c, split):
    y = O.f32_to_bf16(orc.dev_linear(c["x"], c["w"]))
    if c["q_heads"]:
        orc.head_norm_rope_bf16(y, c["out"], c["wq"], c["cos"], c["sin"], c["rows"], c["q_heads"], c["hd"], 1e-6, split, col0=0)
    if c["k_heads"]:
        orc.head_norm_rope_bf16(y, c["out"], c["wk"], c["cos"], c["sin"], c["rows"], c["k_heads"], c["hd"], 1e-6, split,
                                col0=c["q_heads"] * c["hd"])
    return y


# rows, in, q heads, k heads, columns after K, pairing
ONE_LAUNCH = [
    (256, 64, 2, 2, 256, 0),        # whole tiles, the smallest the kernel takes
    (333, 384, 3, 3, 384 + 1536, 0),  # ragged rows; a tile that holds a Q head and a K head; FLUX single-block layout
    (600, 256, 2, 2, 256 + 1024, 1),  # split halves
    (700, 640, 8, 2, 256, 1),       # text encoder: 8 query heads on 2 kv heads, split halves
    (512, 128, 3, 0, 128, 0),       # Q only, and a last tile of 128 columns
    (300, 192, 0, 1, 128, 1),       # K only
    (1000, 512, 5, 5, 0, 0),        # nothing after K; 1280 columns = five tiles
    (512, 256, 2, 2, 256, 0),       # whole tiles and in % 128 == 0: the four-wave kernel's epilogue
    (768, 384, 3, 1, 0, 1),         # the same, split halves, three query heads on one kv head
    (256, 128, 1, 1, 256, 1),       # its smallest case: two k tiles, one tile with a Q and a K head, one without
]


@pytest.mark.parametrize("rows,k,q_heads,k_heads,extra,split", ONE_LAUNCH)
def test_one_launch_matches_oracle_chain_and_own_two_calls(dev, orc, rows, k, q_heads, k_heads, extra, split):
    c = make(rows + k, rows, k, q_heads, k_heads, extra)
    got, kernel = run(dev, c, True, split, 1)
    assert kernel == "linear_mfma_qknorm"
    want = oracle_chain(orc, c, split)
    assert_parity(bf16_to_f32(got), bf16_to_f32(want), f"rows {rows} in {k} heads {q_heads}+{k_heads}")
    two, _ = run(dev, c, False, split, 1)
    assert np.array_equal(got, two), "one launch and the library's own linear + norm+rope calls differ"
    # the columns after K are the plain projection
    qk = (q_heads + k_heads) * 128
    plain, _ = run(dev, dict(c, q_heads=0, k_heads=0), False, split, 1)
    assert np.array_equal(got[:, qk:], plain[:, qk:])
    assert not np.array_equal(got[:, :qk], plain[:, :qk])


def test_vendor_backend_against_oracle(dev, orc):
    """With the vendor GEMM selected (2) and present the entry issues that GEMM and the norm kernel; without it the
    one-launch kernel. Either way the oracle's chain is the yardstick."""
    c = make(5, 512, 256, 4, 4, 512)
    got, kernel = run(dev, c, True, 0, 2)
    assert kernel in ("norm_rope_hd128", "linear_mfma_qknorm")
    assert_parity(bf16_to_f32(got), bf16_to_f32(oracle_chain(orc, c, 0)), "vendor backend")
    two, _ = run(dev, c, False, 0, 2)
    assert np.array_equal(got, two)


# shapes the tiled kernel does not take: the entry runs the two steps
TWO_STEP = [
    (80, 256, 2, 2, 256, 128, 0),     # fewer than 256 rows
    (300, 256, 2, 2, 192, 128, 0),    # width not a multiple of 128
    (300, 200, 2, 2, 256, 128, 1),    # in not a multiple of 64
    (300, 256, 4, 4, 256, 64, 0),     # head_dim 64
    (300, 256, 1, 1, 64, 96, 1),      # head_dim 96, width 256
]


@pytest.mark.parametrize("rows,k,q_heads,k_heads,extra,hd,split", TWO_STEP)
def test_other_shapes_run_the_two_steps(dev, orc, rows, k, q_heads, k_heads, extra, hd, split):
    c = make(rows + hd, rows, k, q_heads, k_heads, extra, hd)
    for backend in (2, 0):
        got, kernel = run(dev, c, True, split, backend)
        assert kernel.startswith("norm_rope")
        two, _ = run(dev, c, False, split, backend)
        assert np.array_equal(got, two)
    assert_parity(bf16_to_f32(got), bf16_to_f32(oracle_chain(orc, c, split)), f"two-step rows {rows} hd {hd}")


def test_bad_arguments(dev):
    lib = dev.lib
    y = dev.alloc(256 * 256 * 2)
    lib.iris_dev_linear_bf16_qknorm(y, y, y, 256, 64, 256, 2, 1, 128, y, y, y, y, 1e-6, 0)   # 3 heads of 128 > 256 columns
    assert lib.iris_dev_last_error() != 0
    lib.iris_dev_linear_bf16_qknorm(y, y, y, 256, 0, 256, 1, 1, 128, y, y, y, y, 1e-6, 0)
    assert lib.iris_dev_last_error() != 0
    dev.free_all()
