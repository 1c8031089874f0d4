"""Pins of the oracle's restatement of the remaining device operators
(oracle/iris_oracle_ops.c): against the compiled reference where its CPU code has the
same operator (NCHW there, channels-last here: the test transposes), against torch
library routines, and against numpy closed forms."""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle as O

_p = C.c_void_p


def ptr(a):
    return a.ctypes.data_as(_p)


def rnd(shape, seed, sigma=1.0):
    return (np.random.default_rng(seed).standard_normal(shape) * sigma).astype(np.float32)


def bf(a):
    return O.bf16_to_f32(O.f32_to_bf16(a))


# ------------------------------------------------------------------ linear
def test_linear_vs_numpy_and_reference(orc, ref_ieee):
    rows, k, out = 7, 96, 33
    x, W = O.f32_to_bf16(rnd((rows, k), 1)), O.f32_to_bf16(rnd((out, k), 2, 0.1))
    y = orc.dev_linear(x, W)
    want = O.bf16_to_f32(x).astype(np.float64) @ O.bf16_to_f32(W).astype(np.float64).T
    np.testing.assert_allclose(y, want, rtol=0, atol=1e-6)
    # compiled reference: f32 activations (here bf16-representable) x bf16 weights
    yr = np.empty((rows, out), np.float32)
    xf = np.ascontiguousarray(O.bf16_to_f32(x))
    ref_ieee.lib.iris_linear_nobias_bf16(ptr(yr), ptr(xf), ptr(W), C.c_int(rows), C.c_int(k), C.c_int(out))
    np.testing.assert_allclose(y, yr, rtol=0, atol=2e-5)


def test_linear_transposed_operand_would_fail(orc):
    """W is [out, in]: a square W and its transpose give different answers."""
    x, W = O.f32_to_bf16(rnd((3, 16), 3)), O.f32_to_bf16(rnd((16, 16), 4))
    assert np.abs(orc.dev_linear(x, W) - orc.dev_linear(x, np.ascontiguousarray(W.T))).max() > 0.1


# ------------------------------------------------------------------ norms
def test_layer_norm_mod(orc):
    x, shift, scale = rnd((5, 64), 5, 3.0) + 1.5, rnd(64, 6), rnd(64, 7, 0.3)
    got = O.bf16_to_f32(orc.dev_layer_norm_mod(x, shift, scale, 1e-6))
    t = torch.nn.functional.layer_norm(torch.from_numpy(x), (64,), eps=1e-6).numpy()
    want = t * (1 + scale) + shift
    assert np.abs(got - bf(want)).max() <= 2 ** -6           # one bf16 ulp of values up to ~4
    plain = O.bf16_to_f32(orc.dev_layer_norm_mod(x, None, None, 1e-6))
    assert np.abs(plain - bf(t)).max() <= 2 ** -6
    assert abs(plain.mean()) < 1e-2 and abs(plain.std() - 1) < 1e-2


def test_rms_norm_vs_reference_and_numpy(orc, ref_ieee):
    x, w, scale = rnd((6, 80), 8, 2.0), 1 + rnd(80, 9, 0.1), rnd(80, 10, 0.2)
    got = O.bf16_to_f32(orc.dev_rms_norm_mod(x, w, None, 1e-5))
    yr = np.empty_like(x)
    ref_ieee.lib.iris_rms_norm(ptr(yr), ptr(x), ptr(w), C.c_int(6), C.c_int(80), C.c_float(1e-5))
    assert np.abs(got - bf(yr)).max() <= 2 ** -6
    want = x / np.sqrt((x.astype(np.float64) ** 2).mean(-1, keepdims=True) + 1e-5) * w * (1 + scale)
    got2 = O.bf16_to_f32(orc.dev_rms_norm_mod(x, w, scale, 1e-5))
    assert np.abs(got2 - bf(want.astype(np.float32))).max() <= 2 ** -6


def test_rms_norm_residual(orc):
    x, a, w, gate = rnd((4, 48), 11), rnd((4, 48), 12, 2.0), 1 + rnd(48, 13, 0.1), rnd(48, 14)
    n = a / np.sqrt((a.astype(np.float64) ** 2).mean(-1, keepdims=True) + 1e-6) * w
    np.testing.assert_allclose(orc.dev_rms_norm_residual(x, a, w, gate, 1e-6), x + np.tanh(gate.astype(np.float64)) * n, atol=2e-6)
    np.testing.assert_allclose(orc.dev_rms_norm_residual(x, a, w, None, 1e-6), x + n, atol=2e-6)


# ------------------------------------------------------------------ activations / elementwise
def test_silu_and_swiglu(orc, ref_ieee):
    x = rnd(1000, 15, 3.0)
    got = orc.dev_silu(x)
    np.testing.assert_allclose(got, torch.nn.functional.silu(torch.from_numpy(x)).numpy(), atol=1e-6)
    xr = x.copy()
    ref_ieee.lib.iris_silu(ptr(xr), C.c_int(x.size))
    np.testing.assert_allclose(got, xr, atol=1e-6)
    # swiglu on a strided [gate | up | pad] buffer
    rows, cols, ldi = 5, 24, 56
    gu = O.f32_to_bf16(rnd((rows, ldi), 16, 2.0))
    out = orc.dev_swiglu(gu, cols, ldo=32)
    g, u = O.bf16_to_f32(gu[:, :cols]), O.bf16_to_f32(gu[:, cols:2 * cols])
    gm = np.ascontiguousarray(g.copy())
    ref_ieee.lib.iris_silu_mul(ptr(gm), ptr(np.ascontiguousarray(u)), C.c_int(g.size))
    assert np.abs(O.bf16_to_f32(out[:, :cols]) - bf(gm)).max() <= 2 ** -5
    assert np.all(out[:, cols:] == 0)                      # nothing written past the columns


def test_residual_add_bias_fill(orc):
    x, a, gate = rnd((3, 10), 17), rnd((3, 10), 18), rnd(10, 19)
    np.testing.assert_allclose(orc.dev_residual(x, a, gate), x + gate * a, atol=1e-6)      # the C compiler may fuse the multiply-add
    np.testing.assert_array_equal(orc.dev_residual(x, a, None), x + a)
    np.testing.assert_array_equal(orc.dev_add(x, a), x + a)
    np.testing.assert_array_equal(orc.dev_add_bias(x, gate), x + gate[None, :])
    np.testing.assert_array_equal(orc.dev_fill_rows(gate, 4), np.tile(gate, (4, 1)))


# ------------------------------------------------------------------ VAE layers (channels-last here, NCHW in the reference)
@pytest.mark.parametrize("h,w,cin,cout,k,stride,pb,pa", [(6, 5, 8, 4, 3, 1, 1, 1), (7, 7, 3, 5, 1, 1, 0, 0), (8, 8, 4, 6, 3, 2, 0, 1)])
def test_conv2d_vs_torch_and_reference(orc, ref_ieee, h, w, cin, cout, k, stride, pb, pa):
    img = bf(rnd((h * w, cin), 20))                        # bf16-representable, so the input rounding is a no-op
    wt = O.f32_to_bf16(rnd((cout, k * k * cin), 21, 0.2))
    bias = rnd(cout, 22)
    got = orc.dev_conv2d(img, wt, bias, h, w, k, stride, pb, pa)
    # torch: NCHW input, weight [cout, cin, ky, kx]; asymmetric padding through F.pad
    x = torch.from_numpy(img.reshape(h, w, cin).transpose(2, 0, 1).copy())[None]
    wk = torch.from_numpy(O.bf16_to_f32(wt).reshape(cout, k, k, cin).transpose(0, 3, 1, 2).copy())
    xp = torch.nn.functional.pad(x, (pb, pa, pb, pa))
    t = torch.nn.functional.conv2d(xp.double(), wk.double(), torch.from_numpy(bias).double(), stride=stride)[0]
    oh, ow = t.shape[1], t.shape[2]
    np.testing.assert_allclose(got, t.numpy().transpose(1, 2, 0).reshape(oh * ow, cout), atol=1e-5)
    if pb == pa:                                           # the reference CPU conv pads symmetrically
        yr = np.empty((cout, oh, ow), np.float32)
        ref_ieee.lib.iris_conv2d(ptr(yr), ptr(np.ascontiguousarray(x[0].numpy())), ptr(np.ascontiguousarray(wk.numpy())), ptr(bias),
                                 C.c_int(1), C.c_int(cin), C.c_int(cout), C.c_int(h), C.c_int(w), C.c_int(k), C.c_int(k),
                                 C.c_int(stride), C.c_int(pb))
        np.testing.assert_allclose(got, yr.transpose(1, 2, 0).reshape(oh * ow, cout), atol=2e-5)


def test_conv2d_rounds_its_input_to_bf16(orc):
    img = rnd((16, 4), 23)
    wt = O.f32_to_bf16(rnd((2, 4), 24))
    np.testing.assert_array_equal(orc.dev_conv2d(img, wt, None, 4, 4, 1, 1, 0, 0), orc.dev_conv2d(bf(img), wt, None, 4, 4, 1, 1, 0, 0))


@pytest.mark.parametrize("silu", [0, 1])
def test_group_norm_vs_torch_and_reference(orc, ref_ieee, silu):
    hw, c, groups = 30, 16, 4
    img, gamma, beta = rnd((hw, c), 25, 2.0) + 0.5, 1 + rnd(c, 26, 0.1), rnd(c, 27, 0.1)
    got = orc.dev_group_norm(img, gamma, beta, groups, 1e-6, silu)
    x = torch.from_numpy(img.T.copy())[None]               # [1, c, hw]
    t = torch.nn.functional.group_norm(x.double(), groups, torch.from_numpy(gamma).double(), torch.from_numpy(beta).double(), 1e-6)
    if silu:
        t = torch.nn.functional.silu(t)
    np.testing.assert_allclose(got, t[0].numpy().T, atol=2e-6)
    if not silu:
        yr = np.empty((c, hw), np.float32)
        ref_ieee.lib.iris_group_norm(ptr(yr), ptr(np.ascontiguousarray(img.T)), ptr(gamma), ptr(beta), C.c_int(1), C.c_int(c),
                                     C.c_int(5), C.c_int(6), C.c_int(groups), C.c_float(1e-6))
        np.testing.assert_allclose(got, yr.T, atol=1e-5)


def test_upsample2x_vs_reference(orc, ref_ieee):
    h, w, c = 3, 4, 5
    img = rnd((h * w, c), 28)
    got = orc.dev_upsample2x(img, h, w)
    yr = np.empty((c, 2 * h, 2 * w), np.float32)
    ref_ieee.lib.iris_upsample_nearest(ptr(yr), ptr(np.ascontiguousarray(img.T)), C.c_int(1), C.c_int(c), C.c_int(h), C.c_int(w),
                                       C.c_int(2), C.c_int(2))
    np.testing.assert_array_equal(got, yr.reshape(c, 4 * h * w).T)
    np.testing.assert_array_equal(got.reshape(2 * h, 2 * w, c)[::2, ::2], img.reshape(h, w, c))
