"""Seeded random sweeps of the linear layers (own kernels), convolution and group norm on the GPU
against the CPU oracle: sizes that are ragged against every tile edge, inner dimensions on both sides of
the 64-multiple that selects the direct-to-LDS kernels, channel counts on both sides of the
implicit-GEMM condition, strides, paddings, optional bias.
"""
import numpy as np
import pytest

import oracle as O
from gpu_harness import Dev

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    return Dev()


def test_random_linear_shapes_on_the_own_kernels(dev, orc):
    rng, lib = np.random.default_rng(3), dev.lib
    lib.iris_dev_linear_backend(1)
    try:
        for case in range(40):
            M, N = int(rng.integers(1, 800)), int(rng.integers(1, 800))
            K = 64 * int(rng.integers(1, 9)) if rng.random() < 0.8 else 8 * int(rng.integers(1, 40))
            out_bf16 = bool(rng.integers(0, 2))
            x = O.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
            W = O.f32_to_bf16((rng.standard_normal((N, K)) / np.sqrt(K)).astype(np.float32))
            dx, dW, dy = dev.put(x), dev.put(W), dev.alloc(M * N * 4 + 64)
            want = orc.dev_linear(x, W)
            if out_bf16:
                lib.iris_dev_linear_bf16(dy, dx, dW, M, K, N)
                got, tol = O.bf16_to_f32(dev.get(dy, (M, N), np.uint16)), 2e-2
            else:
                lib.iris_dev_linear_f32(dy, dx, dW, M, K, N)
                got, tol = dev.get(dy, (M, N), np.float32), 2e-4
            dev.check()
            dev.free_all()
            err = float(np.abs(got - want).max())
            assert err <= tol, f"case {case}: M {M} K {K} N {N} bf16 {out_bf16}: max-abs {err}"
    finally:
        lib.iris_dev_linear_backend(0)


def test_random_convolutions(dev, orc):
    rng, lib = np.random.default_rng(4), dev.lib
    for case in range(40):
        h, w = int(rng.integers(1, 40)), int(rng.integers(1, 40))
        cin, cout = int(rng.choice([64, 128, 192, 32, 8])), int(rng.choice([128, 130, 200, 256, 320, 64, 400]))
        k, stride = int(rng.choice([1, 3])), int(rng.choice([1, 2]))
        pb, pa = int(rng.integers(0, 2)), int(rng.integers(0, 2))
        if h + pb + pa < k or w + pb + pa < k:
            continue
        use_bias = bool(rng.integers(0, 2))
        img = rng.standard_normal((h * w, cin)).astype(np.float32)
        wt = O.f32_to_bf16((rng.standard_normal((cout, k * k * cin)) / np.sqrt(k * k * cin)).astype(np.float32))
        bias = rng.standard_normal(cout).astype(np.float32)
        want = orc.dev_conv2d(img, wt, bias, h, w, k, stride, pb, pa)
        if not use_bias:
            want = want - bias[None, :]
        dimg, dw, db, dout = dev.put(img), dev.put(wt), dev.put(bias), dev.alloc(want.size * 4 + 64)
        lib.iris_dev_conv2d(dout, dimg, dw, db if use_bias else None, h, w, cin, cout, k, stride, pb, pa)
        dev.check()
        got = dev.get(dout, want.shape, np.float32)
        dev.free_all()
        err = float(np.abs(got - want).max())
        assert err <= 1e-3, f"case {case}: {h}x{w} cin {cin} cout {cout} k {k} stride {stride} pad {pb},{pa} bias {use_bias}: max-abs {err}"


def test_random_group_norms(dev, orc):
    rng, lib = np.random.default_rng(5), dev.lib
    for case in range(30):
        hw, groups, cg = int(rng.integers(1, 5000)), int(rng.choice([1, 2, 4, 8, 32])), int(rng.choice([1, 2, 4, 8, 16, 3]))
        c, silu = groups * cg, int(rng.integers(0, 2))
        img = (rng.standard_normal((hw, c)) * rng.choice([0.5, 2.0]) + rng.choice([0.0, 10.0])).astype(np.float32)
        gamma, beta = (1 + 0.1 * rng.standard_normal(c)).astype(np.float32), (0.1 * rng.standard_normal(c)).astype(np.float32)
        dimg, dg, db, dout = dev.put(img), dev.put(gamma), dev.put(beta), dev.alloc(hw * c * 4)
        lib.iris_dev_group_norm(dout, dimg, dg, db, hw, c, groups, 1e-6, silu)
        dev.check()
        got = dev.get(dout, (hw, c), np.float32)
        dev.free_all()
        err = float(np.abs(got - orc.dev_group_norm(img, gamma, beta, groups, 1e-6, silu)).max())
        assert err <= 2e-4, f"case {case}: hw {hw} c {c} groups {groups} silu {silu}: max-abs {err}"
