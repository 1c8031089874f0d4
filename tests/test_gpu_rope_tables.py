"""Rotary tables generated on the device (iris_dev_rope_*) against the host
builders of the same library, which the CPU tests pin bit for bit to the
reference's tables.

Bar: the device forms the same float (or double) angle and rounds a double
cosine / sine once, the host calls libm's cosf / sinf, which are faithful
(< 1 ulp) but not always correctly rounded. So every entry must be within
1 float ulp, nearly all identical, and unrotated entries exactly (1, 0).
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def drt():
    import iris_c_amd
    from iris_c_amd.rope import DevRopeTables
    return DevRopeTables(iris_c_amd.IrisDev())


def ulp_diff(a, b):
    """distance in float32 representable steps (sign-magnitude bits mapped to a line)"""
    def line(x):
        u = np.ascontiguousarray(x, np.float32).view(np.int32).astype(np.int64)
        return np.where(u < 0, -(u & 0x7FFFFFFF), u)
    return np.abs(line(a) - line(b))


def close_tables(dev, host, what):
    for d, h, name in zip(dev, host, ("cos", "sin")):
        assert d.shape == h.shape, what
        u = ulp_diff(d, h)
        # near a zero of the function one ulp is tiny: fall back to an absolute 2^-24 there
        bad = (u > 1) & (np.abs(d.astype(np.float64) - h.astype(np.float64)) > 2.0 ** -24)
        assert not bad.any(), f"{what} {name}: {bad.sum()} entries beyond 1 ulp, worst {u.max()}"
        same = (u == 0).mean()
        print(f"{what} {name}: {100 * same:.3f}% identical, max {u.max()} ulp", flush=True)
        assert same > 0.95, f"{what} {name}: only {same:.4f} identical"


def test_flux2_joint(drt):
    refs = [(32, 32), (16, 24)]
    host = drt.flux2_tables(512, 64, 64, refs)
    dev = drt.dev_flux2_tables(512, 64, 64, refs)
    close_tables(dev, host, "flux2 512+64x64+refs")
    # text rows leave the T, H, W axes unrotated, image rows the L axis: exact (1, 0)
    assert (dev[0][:512, :48] == 1.0).all() and (dev[1][:512, :48] == 0.0).all()
    assert (dev[0][512:, 48:] == 1.0).all() and (dev[1][512:, 48:] == 0.0).all()


def test_flux2_custom_t_offsets_and_small(drt):
    host = drt.flux2_tables(3, 2, 2, [(3, 4)], ref_t=[7])
    dev = drt.dev_flux2_tables(3, 2, 2, [(3, 4)], ref_t=[7])
    close_tables(dev, host, "flux2 tiny")


def test_flux3_joint_double_math(drt):
    refs = [(20, 12), (8, 8)]
    host = drt.flux3_tables(80, 48, 40, refs, theta=2000.0)
    dev = drt.dev_flux3_tables(80, 48, 40, refs, theta=2000.0)
    close_tables(dev, host, "flux3 80+48x40+refs")


def test_zimage_bounded_axes(drt):
    pos, mask, ip, cp = drt.zimage_positions(img_seq=1000, wt=40, cap_seq=77)
    lens = (64, 20, 512)
    host = drt.zimage_tables(pos, (32, 48, 48), lens)
    dev = drt.dev_zimage_tables(pos, (32, 48, 48), lens)
    close_tables(dev, host, "zimage")
    oob = pos[:, 1] >= 20
    assert (dev[0][oob, 16:40] == 1.0).all() and (dev[1][oob, 16:40] == 0.0).all()


def test_qwen3_large_angles(drt):
    # positions up to 3000 at frequency 1: the angle is reduced from thousands of radians
    mask = (np.arange(3000) < 2100).astype(np.int32)
    for pad in (False, True):
        host = drt.qwen3_tables(3000, 128, 1e6, mask=mask, pad_at_one=pad)
        dev = drt.dev_qwen3_tables(3000, 128, 1e6, mask=mask, pad_at_one=pad)
        close_tables(dev, host, f"qwen3 pad_at_one={pad}")


def test_generic_expand_both_modes(drt):
    g = np.random.default_rng(11)
    pos = g.integers(0, 5000, size=(777, 3)).astype(np.int32)
    rc, hc, hs = drt.expand_i32(pos, (16, 40, 72), 500.0)
    assert rc == 0
    close_tables(drt.dev_expand_i32(pos, (16, 40, 72), 500.0), (hc, hs), "expand_i32")
    fpos = (g.integers(-40, 400, size=(333, 4)) * 0.5).astype(np.float32)
    rc, hc, hs = drt.expand_f64(fpos, (8, 28, 28, 64), 10000.0)
    assert rc == 0
    close_tables(drt.dev_expand_f64(fpos, (8, 28, 28, 64), 10000.0), (hc, hs), "expand_f64")


def test_staging_buffer_reuse_smaller_then_larger(drt):
    """The private staging buffer grows on demand and is reused: a small table after a large one,
    then a larger one again, must all be right."""
    for seq in (4000, 7, 9000, 64):
        host = drt.qwen3_tables(seq, 128, 1e6)
        close_tables(drt.dev_qwen3_tables(seq, 128, 1e6), host, f"qwen3 seq {seq}")


def test_bad_arguments_report_an_error_and_write_nothing(drt):
    import ctypes as C
    dev, lib = drt.dev, drt.lib
    buf = np.full((4, 32), 7.0, np.float32)
    dc, ds = dev.to_device(buf), dev.to_device(buf)
    pos = np.zeros((4, 2), np.int32)
    dims = np.array([31, 33], np.int32)                     # odd axis sizes
    lib.iris_dev_rope_expand_i32(dc, ds, pos.ctypes.data_as(C.c_void_p), 4, 2, dims.ctypes.data_as(C.c_void_p), None, 100.0)
    assert lib.iris_dev_last_error() != 0                   # reading clears it
    assert (dev.to_host(dc, (4, 32), np.float32) == 7.0).all()
    lib.iris_dev_free(dc); lib.iris_dev_free(ds)


def test_device_tables_drive_norm_rope(drt):
    """End to end: head_norm_rope with device-made tables against host-made tables on the same rows.
    A table entry one float ulp apart can move a bf16 result by at most one bf16 step, rarely."""
    from gpu_harness import Dev
    seq_parts = (40, 12, 12)
    seq = seq_parts[0] + seq_parts[1] * seq_parts[2]
    heads, hd = 6, 128
    g = np.random.default_rng(3)
    rows = (g.standard_normal((seq, heads * hd)).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    w = (1 + 0.02 * g.standard_normal(hd)).astype(np.float32)
    hc, hs = drt.flux2_tables(*seq_parts)
    dc, ds = drt.dev_flux2_tables(*seq_parts)
    d = Dev()
    a = d.norm_rope(rows.copy(), heads * hd, 0, w, hc, hs, seq, heads, hd, 1e-6, 0)
    b = d.norm_rope(rows.copy(), heads * hd, 0, w, dc, ds, seq, heads, hd, 1e-6, 0)
    diff = np.abs(a.astype(np.int32) - b.astype(np.int32))
    assert diff.max() <= 1 and (diff != 0).mean() < 1e-3
