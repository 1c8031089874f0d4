"""GPU parity of the other device operators (linear, norms, gated activations, residuals,
convolution, group norm, upsampling) through the C ABI against the oracle.

Tolerances: outputs stored as bf16 within one bf16 ulp of the oracle's value (the oracle
accumulates in double, the device in f32); f32 outputs within 1e-5 relative to the row's scale,
GEMM-like sums within 2e-3 relative to sqrt(K) * |x||w| scale."""
import numpy as np
import pytest

import oracle as O
from gpu_harness import Dev, ptr_add

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    d = Dev()
    yield d
    d.free_all()


def rnd(shape, seed, sigma=1.0):
    return (np.random.default_rng(seed).standard_normal(shape) * sigma).astype(np.float32)


def bf16_close(got_u16, want_u16, what):
    """Both bf16: equal, or one ulp apart (the f32 value sat next to a rounding boundary), or within 1e-4."""
    g, w = O.bf16_to_f32(got_u16), O.bf16_to_f32(want_u16)
    ulp = np.maximum(np.abs(w), 2.0 ** -126) * 2.0 ** -7
    bad = (np.abs(g - w) > ulp * 1.01) & (np.abs(g - w) > 1e-4)   # next to zero (cancellation) the f32 noise of O(1) terms decides
    assert not bad.any(), f"{what}: {bad.sum()} of {bad.size} differ by more than one bf16 ulp, worst {np.abs(g - w).max()}"
    assert (g != w).mean() < 0.05, f"{what}: {100 * (g != w).mean():.1f}% of the values differ"


def run(dev, fn, outs):
    fn()
    dev.check()
    res = [dev.get(p, shape, dt) for p, shape, dt in outs]
    dev.free_all()
    return res if len(res) > 1 else res[0]


# ------------------------------------------------------------------ linear
@pytest.mark.parametrize("rows,k,out", [(1, 8, 1), (5, 64, 7), (128, 128, 128), (130, 200, 260), (333, 3072, 520), (64, 96, 64),
                                        # the 256 x 256 kernel (rows, out >= 256, k % 64 == 0): ragged edges, and an `out` that
                                        # rules out 16-byte stores (its epilogue then stores straight from the accumulators)
                                        (300, 128, 258), (257, 64, 257), (512, 192, 256), (700, 256, 1000),
                                        # whole 256 x 256 tiles and k % 128 == 0: the four-wave kernel (two k tiles at least)
                                        (256, 128, 256), (512, 256, 512), (768, 640, 1024)])
@pytest.mark.parametrize("out_bf16", [False, True])
@pytest.mark.parametrize("backend", ["library", "own"])
def test_linear(dev, orc, rows, k, out, out_bf16, backend):
    """Both GEMM paths: the vendor library (taken when present) and this library's own MFMA kernel."""
    x, W = O.f32_to_bf16(rnd((rows, k), rows + k)), O.f32_to_bf16(rnd((out, k), out, 0.05))
    want = orc.dev_linear(x, W)
    dx, dW = dev.put(x), dev.put(W)
    dy = dev.alloc(rows * out * (2 if out_bf16 else 4))
    fn = dev.lib.iris_dev_linear_bf16 if out_bf16 else dev.lib.iris_dev_linear_f32
    dev.lib.iris_dev_linear_backend(0 if backend == "own" else 2)
    try:
        got = run(dev, lambda: fn(dy, dx, dW, rows, k, out), [(dy, (rows, out), np.uint16 if out_bf16 else np.float32)])
        kernel = dev.dev.last_kernel()
    finally:
        dev.lib.iris_dev_linear_backend(0)
    assert kernel == "linear_mfma" if backend == "own" else kernel in ("linear_hipblaslt", "linear_mfma")
    scale = np.sqrt(k) * 0.05
    if out_bf16:
        # round to nearest: half a bf16 ulp of the value, plus the f32 accumulation noise
        assert np.all(np.abs(O.bf16_to_f32(got) - want) <= np.abs(want) * 2.0 ** -8 * 1.01 + scale * 2e-5)
    else:
        assert np.abs(got - want).max() <= scale * 2e-5


@pytest.mark.parametrize("rows,k,out,width", [(4608, 128, 9216, 224), (4608, 256, 3072, 224), (4608, 128, 27648, 256), (2048, 128, 2048, 192)])
@pytest.mark.parametrize("out_bf16", [False, True])
def test_four_wave_gemm_every_tile_width(dev, orc, rows, k, out, width, out_bf16):
    """The four-wave kernel at each of its tile widths (192, 224, 256 columns), f32 and bf16 output, WHOLE output:
    the widths the model projections take (4608 rows -> 9216 / 3072 columns: 224, with a last tile moved back because
    9216 % 224 != 0; -> 27648: 256) with a short reduction so that the comparison stays cheap. Against a float64
    product of the same bf16 operands (numpy's BLAS, an independent routine; the f32 accumulation error over 128-256
    terms is far below the bar), and the oracle on sampled rows."""
    import ctypes as C
    plan = (C.c_int * 2)()
    dev.lib.iris_hip_linear_plan(rows, k, out, 2 if out_bf16 else 4, plan)
    assert (plan[0], plan[1]) == (3, width), list(plan)
    x, W = O.f32_to_bf16(rnd((rows, k), rows + k)), O.f32_to_bf16(rnd((out, k), out, 0.05))
    want = O.bf16_to_f32(x).astype(np.float64) @ O.bf16_to_f32(W).astype(np.float64).T
    pick = np.random.default_rng(out).integers(0, rows, 16)
    np.testing.assert_allclose(orc.dev_linear(np.ascontiguousarray(x[pick]), W), want[pick], atol=np.sqrt(k) * 0.05 * 2e-5)
    dx, dW = dev.put(x), dev.put(W)
    dy = dev.alloc(rows * out * (2 if out_bf16 else 4))
    fn = dev.lib.iris_dev_linear_bf16 if out_bf16 else dev.lib.iris_dev_linear_f32
    dev.lib.iris_dev_linear_backend(1)
    try:
        got = run(dev, lambda: fn(dy, dx, dW, rows, k, out), [(dy, (rows, out), np.uint16 if out_bf16 else np.float32)])
        kernel = dev.dev.last_kernel()
    finally:
        dev.lib.iris_dev_linear_backend(0)
    assert kernel == "linear_mfma"
    scale = np.sqrt(k) * 0.05
    if out_bf16:
        assert np.all(np.abs(O.bf16_to_f32(got) - want) <= np.abs(want) * 2.0 ** -8 * 1.01 + scale * 2e-5)
    else:
        assert np.abs(got - want).max() <= scale * 2e-5


def test_linear_unaligned_k_uses_the_scalar_kernel(dev, orc):
    rows, k, out = 37, 27, 19                              # k*k*cin of the 3-channel input convolution
    x, W = O.f32_to_bf16(rnd((rows, k), 1)), O.f32_to_bf16(rnd((out, k), 2))
    dx, dW, dy = dev.put(x), dev.put(W), dev.alloc(rows * out * 4)
    got = run(dev, lambda: dev.lib.iris_dev_linear_f32(dy, dx, dW, rows, k, out), [(dy, (rows, out), np.float32)])
    np.testing.assert_allclose(got, orc.dev_linear(x, W), atol=1e-4)


def test_own_gemm_is_the_default_and_the_vendor_library_is_opt_in(dev):
    """A linear layer runs on the library's own kernel unless the vendor GEMM is asked for (the yardstick of the
    benchmark); on a ROCm machine hipBLASLt is there, so asking for it must be honoured."""
    rows, k, out = 64, 128, 64
    dx, dW, dy = dev.put(np.zeros((rows, k), np.uint16)), dev.put(np.zeros((out, k), np.uint16)), dev.alloc(rows * out * 4)
    dev.lib.iris_dev_linear_f32(dy, dx, dW, rows, k, out)
    dev.check()
    assert dev.dev.last_kernel() == "linear_mfma"
    dev.lib.iris_dev_linear_backend(2)
    dev.lib.iris_dev_linear_f32(dy, dx, dW, rows, k, out)
    dev.lib.iris_dev_linear_backend(0)
    dev.check()
    assert dev.dev.last_kernel() == "linear_hipblaslt"
    dev.free_all()


@pytest.mark.parametrize("backend", ["library", "own"])
def test_linear_full_size_properties(dev, orc, backend):
    """The QKV projection of the bench configuration (4608 x 3072 -> 9216): sampled entries against
    the oracle, and linearity in x: (x1 + x2) W == x1 W + x2 W for bf16-exact sums."""
    rows, k, out = 4608, 3072, 9216
    dev.lib.iris_dev_linear_backend(0 if backend == "own" else 2)
    rng = np.random.default_rng(5)
    x = O.f32_to_bf16(rng.integers(-4, 5, (rows, k)).astype(np.float32) / 8)     # small dyadic values: exact in bf16
    W = O.f32_to_bf16(rng.integers(-4, 5, (out, k)).astype(np.float32) / 8)
    dx, dW, dy = dev.put(x), dev.put(W), dev.alloc(rows * out * 4)
    got = run(dev, lambda: dev.lib.iris_dev_linear_f32(dy, dx, dW, rows, k, out), [(dy, (rows, out), np.float32)])
    r = rng.integers(0, rows, 24); c = rng.integers(0, out, 24)
    xs, Ws = O.bf16_to_f32(x[r]).astype(np.float64), O.bf16_to_f32(W[c]).astype(np.float64)
    want = np.einsum("ik,ik->i", xs, Ws)
    dev.lib.iris_dev_linear_backend(0)
    np.testing.assert_allclose(got[r, c], want, atol=1e-3)           # dyadic products: sums are exact in f32
    assert np.all(got == np.round(got * 64) / 64)                     # every entry is a multiple of 1/64


# ------------------------------------------------------------------ norms
@pytest.mark.parametrize("rows,dim", [(3, 3072), (5, 3840), (2, 100), (1, 4100), (4, 6144)])
def test_layer_norm_mod_and_rms_norms(dev, orc, rows, dim):
    x = rnd((rows, dim), dim, 2.0) + 0.7
    shift, scale, w = rnd(dim, 1, 0.5), rnd(dim, 2, 0.3), 1 + rnd(dim, 3, 0.1)
    dx, dsh, dsc, dw = dev.put(x), dev.put(shift), dev.put(scale), dev.put(w)
    d1, d2, d3, d4 = (dev.alloc(rows * dim * 2) for _ in range(4))
    def fn():
        dev.lib.iris_dev_layer_norm_mod(d1, dx, dsh, dsc, rows, dim, 1e-6)
        dev.lib.iris_dev_layer_norm_mod(d2, dx, None, None, rows, dim, 1e-6)
        dev.lib.iris_dev_rms_norm(d3, dx, dw, rows, dim, 1e-5)
        dev.lib.iris_dev_rms_norm_mod(d4, dx, dw, dsc, rows, dim, 1e-5)
    g1, g2, g3, g4 = run(dev, fn, [(d, (rows, dim), np.uint16) for d in (d1, d2, d3, d4)])
    bf16_close(g1, orc.dev_layer_norm_mod(x, shift, scale, 1e-6), "layer_norm_mod")
    bf16_close(g2, orc.dev_layer_norm_mod(x, None, None, 1e-6), "layer_norm")
    bf16_close(g3, orc.dev_rms_norm_mod(x, w, None, 1e-5), "rms_norm")
    bf16_close(g4, orc.dev_rms_norm_mod(x, w, scale, 1e-5), "rms_norm_mod")


@pytest.mark.parametrize("gated", [False, True])
def test_rms_norm_residual(dev, orc, gated):
    rows, dim = 6, 2560
    x, a, w, gate = rnd((rows, dim), 1), rnd((rows, dim), 2, 3.0), 1 + rnd(dim, 3, 0.1), rnd(dim, 4)
    dx, da, dw, dg = dev.put(x), dev.put(a), dev.put(w), dev.put(gate)
    got = run(dev, lambda: dev.lib.iris_dev_rms_norm_residual(dx, da, dw, dg if gated else None, rows, dim, 1e-6), [(dx, (rows, dim), np.float32)])
    np.testing.assert_allclose(got, orc.dev_rms_norm_residual(x, a, w, gate if gated else None, 1e-6), atol=2e-5)


# ------------------------------------------------------------------ elementwise
@pytest.mark.parametrize("n", [1, 7, 8, 1000, 4096, 1 << 20])
def test_f32_to_bf16_bit_exact(dev, n):
    x = rnd(n, n, 10.0)
    dx, dy = dev.put(x), dev.alloc(n * 2)
    got = run(dev, lambda: dev.lib.iris_dev_f32_to_bf16(dy, dx, n), [(dy, (n,), np.uint16)])
    np.testing.assert_array_equal(got, O.f32_to_bf16(x))


@pytest.mark.parametrize("rows,dim", [(4, 3072), (3, 10), (1, 1)])
def test_elementwise(dev, orc, rows, dim):
    x, a, g = rnd((rows, dim), 1, 3.0), rnd((rows, dim), 2), rnd(dim, 3)
    n = rows * dim
    d = [dev.put(x) for _ in range(5)]
    da, dg, dfill = dev.put(a), dev.put(g), dev.alloc(n * 4)
    def fn():
        dev.lib.iris_dev_silu(d[0], n)
        dev.lib.iris_dev_add(d[1], da, n)
        dev.lib.iris_dev_add_bias(d[2], dg, rows, dim)
        dev.lib.iris_dev_residual(d[3], da, dg, rows, dim)
        dev.lib.iris_dev_residual(d[4], da, None, rows, dim)
        dev.lib.iris_dev_fill_rows(dfill, dg, rows, dim)
    r = run(dev, fn, [(p, (rows, dim), np.float32) for p in d] + [(dfill, (rows, dim), np.float32)])
    np.testing.assert_allclose(r[0], orc.dev_silu(x).reshape(rows, dim), rtol=2e-6, atol=1e-6)
    np.testing.assert_array_equal(r[1], orc.dev_add(x, a))
    np.testing.assert_array_equal(r[2], orc.dev_add_bias(x, g))
    np.testing.assert_allclose(r[3], orc.dev_residual(x, a, g), atol=1e-6)
    np.testing.assert_array_equal(r[4], orc.dev_residual(x, a, None))
    np.testing.assert_array_equal(r[5], orc.dev_fill_rows(g, rows))


@pytest.mark.parametrize("rows,cols,ldi,ldo", [(5, 24, 56, 32), (7, 9216, 18432, 9216), (3, 5, 11, 7)])
def test_swiglu(dev, orc, rows, cols, ldi, ldo):
    gu = O.f32_to_bf16(rnd((rows, ldi), cols, 2.0))
    dgu = dev.put(gu)
    dout = dev.put(np.zeros((rows, ldo), np.uint16))
    got = run(dev, lambda: dev.lib.iris_dev_swiglu(dout, ldo, dgu, ptr_add(dgu, 2 * cols), ldi, rows, cols), [(dout, (rows, ldo), np.uint16)])
    want = orc.dev_swiglu(gu, cols, ldo=ldo)
    bf16_close(got[:, :cols], want[:, :cols], "swiglu")
    assert np.all(got[:, cols:] == 0)


# ------------------------------------------------------------------ VAE layers
@pytest.mark.parametrize("h,w,cin,cout,k,stride,pb,pa", [(6, 5, 8, 4, 3, 1, 1, 1), (7, 7, 3, 5, 3, 1, 1, 1), (8, 8, 16, 6, 3, 2, 0, 1),
                                                         (16, 16, 128, 128, 3, 1, 1, 1), (9, 9, 32, 64, 1, 1, 0, 0),
                                                         # cin % 64 == 0 and cout >= 128: the implicit-GEMM path
                                                         (20, 17, 64, 128, 3, 1, 1, 1), (16, 16, 128, 256, 3, 1, 1, 1),
                                                         (33, 20, 64, 320, 3, 2, 0, 1), (12, 12, 128, 130, 1, 1, 0, 0),
                                                         (24, 40, 192, 128, 3, 1, 1, 1), (5, 4, 64, 512, 3, 1, 1, 1),
                                                         (40, 36, 128, 128, 3, 2, 1, 1)])
def test_conv2d(dev, orc, h, w, cin, cout, k, stride, pb, pa):
    img = rnd((h * w, cin), h + cin)
    wt = O.f32_to_bf16(rnd((cout, k * k * cin), cout, 0.1))
    bias = rnd(cout, 3)
    want = orc.dev_conv2d(img, wt, bias, h, w, k, stride, pb, pa)
    dimg, dw, db = dev.put(img), dev.put(wt), dev.put(bias)
    dout = dev.alloc(want.size * 4)
    got = run(dev, lambda: dev.lib.iris_dev_conv2d(dout, dimg, dw, db, h, w, cin, cout, k, stride, pb, pa), [(dout, want.shape, np.float32)])
    np.testing.assert_allclose(got, want, atol=2e-5 * np.sqrt(k * k * cin))
    # no bias
    dimg, dw = dev.put(img), dev.put(wt)
    dout = dev.alloc(want.size * 4)
    got = run(dev, lambda: dev.lib.iris_dev_conv2d(dout, dimg, dw, None, h, w, cin, cout, k, stride, pb, pa), [(dout, want.shape, np.float32)])
    np.testing.assert_allclose(got, want - bias[None, :], atol=2e-5 * np.sqrt(k * k * cin))


def test_conv2d_large_image_in_chunks_sampled_pixels(dev):
    """An image whose bf16 copy does not fit the library's 256 MB of convolution scratch is processed in
    chunks of output rows with their halo rows. 1040 x 1024 x 128 -> 128, 3 x 3: sampled output pixels
    (corners, edges, the rows around every possible chunk boundary, random ones) against the definition
    in float64 on bf16-rounded inputs."""
    h, w, cin, cout, k = 1040, 1024, 128, 128, 3
    rng = np.random.default_rng(11)
    img = rng.standard_normal((h * w, cin), dtype=np.float32)
    wt = O.f32_to_bf16((rng.standard_normal((cout, k * k * cin)) * 0.05).astype(np.float32))
    bias = rng.standard_normal(cout).astype(np.float32)
    dimg, dw, db = dev.put(img), dev.put(wt), dev.put(bias)
    dout = dev.alloc(h * w * cout * 4)
    got = run(dev, lambda: dev.lib.iris_dev_conv2d(dout, dimg, dw, db, h, w, cin, cout, k, 1, 1, 1), [(dout, (h * w, cout), np.float32)])
    wf = O.bf16_to_f32(wt).astype(np.float64).reshape(cout, k, k, cin)
    ys = np.r_[0, 1, h - 2, h - 1, rng.integers(0, h, 40), np.arange(1016, 1030)]
    xs = np.r_[0, 1, w - 2, w - 1, rng.integers(0, w, 12)]
    image = img.reshape(h, w, cin)
    worst = 0.0
    for yy in ys:
        for xx in xs:
            acc = bias.astype(np.float64).copy()
            for ky in range(k):
                for kx in range(k):
                    iy, ix = yy + ky - 1, xx + kx - 1
                    if 0 <= iy < h and 0 <= ix < w:
                        acc += wf[:, ky, kx, :] @ O.bf16_to_f32(O.f32_to_bf16(image[iy, ix])).astype(np.float64)
            worst = max(worst, float(np.abs(got[yy * w + xx] - acc).max()))
    assert worst <= 2e-5 * np.sqrt(k * k * cin) * 4, worst


@pytest.mark.parametrize("hw,c,groups,silu", [(30, 16, 4, 0), (4096, 128, 32, 1), (100, 6, 3, 1)])
def test_group_norm(dev, orc, hw, c, groups, silu):
    img, gamma, beta = rnd((hw, c), hw, 2.0) + 0.5, 1 + rnd(c, 1, 0.1), rnd(c, 2, 0.1)
    dimg, dg, db = dev.put(img), dev.put(gamma), dev.put(beta)
    dout = dev.alloc(hw * c * 4)
    got = run(dev, lambda: dev.lib.iris_dev_group_norm(dout, dimg, dg, db, hw, c, groups, 1e-6, silu), [(dout, (hw, c), np.float32)])
    np.testing.assert_allclose(got, orc.dev_group_norm(img, gamma, beta, groups, 1e-6, silu), atol=2e-5)


@pytest.mark.parametrize("hw,c,groups", [(70000, 128, 32), (5000, 512, 32), (3001, 6, 3), (1, 8, 2)])
def test_group_norm_single_pass_statistics_far_from_zero(dev, orc, hw, c, groups):
    """The statistics are taken in one pass with shifted sums and merged moments; data with a mean of 100
    standard deviations is where a careless one-pass formula loses everything. More workgroups than
    the partial-moment table has rows (70000 pixels), many channels per group, the scalar path, one pixel."""
    img = rnd((hw, c), hw + c, 0.5) + 50.0 + np.arange(c, dtype=np.float32)[None, :] * 0.01
    gamma, beta = 1 + rnd(c, 1, 0.1), rnd(c, 2, 0.1)
    dimg, dg, db = dev.put(img), dev.put(gamma), dev.put(beta)
    dout = dev.alloc(hw * c * 4)
    got = run(dev, lambda: dev.lib.iris_dev_group_norm(dout, dimg, dg, db, hw, c, groups, 1e-6, 0), [(dout, (hw, c), np.float32)])
    want = orc.dev_group_norm(img, gamma, beta, groups, 1e-6, 0)
    np.testing.assert_allclose(got, want, atol=2e-4)


@pytest.mark.parametrize("h,w,c", [(3, 4, 5), (16, 16, 128)])
def test_upsample2x(dev, orc, h, w, c):
    img = rnd((h * w, c), c)
    dimg, dout = dev.put(img), dev.alloc(4 * h * w * c * 4)
    got = run(dev, lambda: dev.lib.iris_dev_upsample2x(dout, dimg, h, w, c), [(dout, (4 * h * w, c), np.float32)])
    np.testing.assert_array_equal(got, orc.dev_upsample2x(img, h, w))


def test_cleanup_and_second_init(dev, orc):
    """iris_dev_cleanup releases the stream and every private scratch (convolution patches, group-norm
    partials, table staging, the GEMM library's handle and workspace); a later iris_dev_init must bring
    all of it back: the reference's program initialises once per process, a test harness may not."""
    lib = dev.lib
    rows, k, out = 64, 128, 64
    x, W = O.f32_to_bf16(rnd((rows, k), 1)), O.f32_to_bf16(rnd((out, k), 2, 0.05))
    want = orc.dev_linear(x, W)

    def linear_once():
        dx, dW, dy = dev.put(x), dev.put(W), dev.alloc(rows * out * 4)
        return run(dev, lambda: lib.iris_dev_linear_f32(dy, dx, dW, rows, k, out), [(dy, (rows, out), np.float32)])

    lib.iris_dev_linear_backend(2)                           # the vendor GEMM, so that its handle and workspace exist
    try:
        np.testing.assert_allclose(linear_once(), want, atol=1e-4)
        lib.iris_dev_cleanup()
        assert lib.iris_dev_available() == 0
        assert lib.iris_dev_alloc(16) is None                    # refused, not crashed
        lib.iris_dev_last_error()
        assert lib.iris_dev_init() == 1 and lib.iris_dev_available() == 1
        np.testing.assert_allclose(linear_once(), want, atol=1e-4)
        assert dev.dev.last_kernel() == "linear_hipblaslt"       # the library was opened again
    finally:
        lib.iris_dev_linear_backend(0)
    np.testing.assert_allclose(linear_once(), want, atol=1e-4)
    assert dev.dev.last_kernel() == "linear_mfma"
    # an operator with private scratch after the re-init
    img, gamma, beta = rnd((100, 8), 5), 1 + rnd(8, 1, 0.1), rnd(8, 2, 0.1)
    dimg, dg, db, dout = dev.put(img), dev.put(gamma), dev.put(beta), dev.alloc(100 * 8 * 4)
    got = run(dev, lambda: lib.iris_dev_group_norm(dout, dimg, dg, db, 100, 8, 2, 1e-6, 0), [(dout, (100, 8), np.float32)])
    np.testing.assert_allclose(got, orc.dev_group_norm(img, gamma, beta, 2, 1e-6, 0), atol=2e-5)
