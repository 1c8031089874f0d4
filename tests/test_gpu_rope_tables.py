"""Rotary tables expanded on the device (iris_dev_rope_*): bit for bit against the reference's
golden tables (tests/golden/ref_vectors.npz, written from the reference's compiled routines) and
against the oracle's restatement of those routines on the real layouts. The host builders of the
library are not the yardstick here; the CPU tests hold them to the same references.
"""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ref_vectors.npz")
REFS = [(2, 3), (3, 2)]


@pytest.fixture(scope="module")
def gold():
    return np.load(GOLD, allow_pickle=False)


@pytest.fixture(scope="module")
def drt():
    import iris_c_amd
    from iris_c_amd.rope import DevRopeTables
    return DevRopeTables(iris_c_amd.IrisDev())


def same_bits(dev, want, what):
    for d, w, name in zip(dev, want, ("cos", "sin")):
        d = np.ascontiguousarray(d, np.float32); w = np.ascontiguousarray(w, np.float32)
        assert d.shape == w.shape, f"{what} {name}: shape {d.shape} vs {w.shape}"
        differ = d.view(np.uint32) != w.view(np.uint32)
        assert not differ.any(), f"{what} {name}: {differ.sum()} of {differ.size} entries differ"


# ---- against the reference's own output (golden fixtures) ----

def test_golden_flux2_flux3_qwen3(drt, gold):
    same_bits(drt.dev_flux2_tables(8, 4, 5, REFS), (gold["flux2_cos"], gold["flux2_sin"]), "flux2 golden")
    same_bits(drt.dev_flux2_tables(8, 4, 5, REFS, ref_t=[10, 20]), (gold["flux2_cos"], gold["flux2_sin"]), "flux2 golden t")
    same_bits(drt.dev_flux3_tables(8, 4, 5, REFS, theta=10000.0), (gold["flux3_cos"], gold["flux3_sin"]), "flux3 golden")
    same_bits(drt.dev_qwen3_tables(24, 128, 1e6), (gold["qwen3_cos"], gold["qwen3_sin"]), "qwen3 golden")
    mask = np.r_[np.ones(15), np.zeros(9)].astype(np.int32)
    same_bits(drt.dev_qwen3_tables(24, 128, 1e6, mask=mask, pad_at_one=True), (gold["qwen3_f3_cos"], gold["qwen3_f3_sin"]),
              "qwen3 golden, padding at position one")


def test_golden_zimage_axis_tables(drt, gold):
    dims, off = (32, 48, 48), 0
    for ax, d in enumerate(dims):
        pos = np.zeros((40, 3), np.int32)
        pos[:, ax] = np.arange(40)
        c, s = drt.dev_zimage_tables(pos, dims, (40, 40, 40))
        same_bits((c[:, off:off + d // 2], s[:, off:off + d // 2]), (gold[f"zimage_cos_{ax}"], gold[f"zimage_sin_{ax}"]),
                  f"zimage axis {ax}")
        off += d // 2


# ---- against the oracle on the real layouts ----

def test_flux2_joint_full_size(drt, orc):
    refs = [(32, 32), (16, 24)]
    dev = drt.dev_flux2_tables(512, 64, 64, refs)
    same_bits(dev, orc.flux2_joint_tables(512, 64, 64, refs), "flux2 512+64x64+refs")
    # text rows leave the T, H, W axes unrotated, image rows the L axis: exact (1, 0)
    assert (dev[0][:512, :48] == 1.0).all() and (dev[1][:512, :48] == 0.0).all()
    assert (dev[0][512:, 48:] == 1.0).all() and (dev[1][512:, 48:] == 0.0).all()


def test_flux2_stress_layout_12800_rows(drt, orc):
    refs = [(64, 64), (64, 64)]
    same_bits(drt.dev_flux2_tables(512, 64, 64, refs), orc.flux2_joint_tables(512, 64, 64, refs), "flux2 12800 rows")


def test_flux2_custom_t_offsets_and_small(drt, orc):
    c, s = drt.dev_flux2_tables(3, 2, 2, [(3, 4)], ref_t=[7])
    oc, os_ = orc.flux2_rope_image(3, 4, t_offset=7)
    same_bits((c[7:], s[7:]), (oc[:, ::2], os_[:, ::2]), "flux2 tiny")


def test_flux3_joint_double_math(drt, orc):
    refs = [(20, 12), (8, 8)]
    dims = (32, 32, 32, 32)
    pos = orc.flux3_joint_positions(80, 48, 40, refs)
    same_bits(drt.dev_flux3_tables(80, 48, 40, refs, theta=2000.0), orc.flux3_rope_rows(pos, dims, 2000.0), "flux3 80+48x40+refs")


def test_zimage_bounded_axes(drt, orc):
    pos, mask, ip, cp = orc.zimage_positions(1000, 40, 77)
    lens = (64, 20, 512)
    dev = drt.dev_zimage_tables(pos, (32, 48, 48), lens)
    same_bits(dev, orc.zimage_gather(pos, (32, 48, 48), lens), "zimage")
    oob = pos[:, 1] >= 20
    assert oob.any() and (dev[0][oob, 16:40] == 1.0).all() and (dev[1][oob, 16:40] == 0.0).all()


def test_zimage_bench_layout(drt, orc):
    pos, mask, ip, cp = orc.zimage_positions(img_seq=4096, wt=64, cap_seq=256)
    same_bits(drt.dev_zimage_tables(pos, (32, 48, 48), (1024, 1024, 1024)), orc.zimage_gather(pos), "zimage 4096+256")


def test_qwen3_large_angles(drt, orc):
    # positions up to 3000 at frequency 1: the angle is reduced from thousands of radians
    mask = (np.arange(3000) < 2100).astype(np.int32)
    for pad in (False, True):
        same_bits(drt.dev_qwen3_tables(3000, 128, 1e6, mask=mask, pad_at_one=pad),
                  orc.qwen3_rope_table(3000, 128, 1e6, mask=mask, pad_at_one=pad), f"qwen3 pad_at_one={pad}")


def test_generic_expand_both_modes(drt, orc):
    g = np.random.default_rng(11)
    fpos = (g.integers(-40, 400, size=(333, 4)) * 0.5).astype(np.float32)
    same_bits(drt.dev_expand_f64(fpos, (8, 28, 28, 64), 10000.0), orc.flux3_rope_rows(fpos, (8, 28, 28, 64), 10000.0), "expand_f64")
    # integer positions on uneven axes: the oracle's Z-Image gather is the same rule with other sizes
    pos = g.integers(0, 5000, size=(777, 3)).astype(np.int32)
    same_bits(drt.dev_expand_i32(pos, (32, 48, 48), 256.0, axis_lens=(4000, 5000, 100)),
              orc.zimage_gather(pos, (32, 48, 48), (4000, 5000, 100)), "expand_i32")


def test_staging_buffer_reuse_smaller_then_larger(drt, orc):
    """The private staging buffer grows on demand and is reused: a small table after a large one,
    then a larger one again, must all be right."""
    for seq in (4000, 7, 9000, 64):
        same_bits(drt.dev_qwen3_tables(seq, 128, 1e6), orc.qwen3_rope_table(seq, 128, 1e6), f"qwen3 seq {seq}")


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


def test_device_tables_drive_norm_rope(drt, orc):
    """End to end: head_norm_rope with device-made tables gives the bits it gives with the oracle's tables."""
    from gpu_harness import Dev
    seq_parts = (40, 12, 12)
    seq = seq_parts[0] + seq_parts[1] * seq_parts[2]
    heads, hd = 6, 128
    g = np.random.default_rng(3)
    rows = (g.standard_normal((seq, heads * hd)).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    w = (1 + 0.02 * g.standard_normal(hd)).astype(np.float32)
    oc, os_ = orc.flux2_joint_tables(*seq_parts)
    dc, ds = drt.dev_flux2_tables(*seq_parts)
    d = Dev()
    a = d.norm_rope(rows.copy(), heads * hd, 0, w, oc, os_, seq, heads, hd, 1e-6, 0)
    b = d.norm_rope(rows.copy(), heads * hd, 0, w, dc, ds, seq, heads, hd, 1e-6, 0)
    assert np.array_equal(a, b)
