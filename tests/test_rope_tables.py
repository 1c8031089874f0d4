"""Host builders of the rotary tables (include/iris_rope.h, inside libiris_dev.so)
against the golden tables written from the reference's compiled routines, and
against the oracle on larger layouts. Bit-exact. No GPU needed: these entry
points are plain C + libm.
"""
import os

import numpy as np
import pytest

from iris_c_amd.rope import RopeTables

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ref_vectors.npz")
REFS = [(2, 3), (3, 2)]


@pytest.fixture(scope="module")
def gold():
    return np.load(GOLD, allow_pickle=False)


@pytest.fixture(scope="module")
def rt():
    return RopeTables()


def same_bits(a, b):
    a = np.ascontiguousarray(a, dtype=np.float32); b = np.ascontiguousarray(b, dtype=np.float32)
    return a.shape == b.shape and np.array_equal(a.view(np.uint32), b.view(np.uint32))


# ---- against the reference's own output (golden fixtures) ----

def test_flux2_joint_matches_reference_tables(rt, gold):
    c, s = rt.flux2_tables(8, 4, 5, REFS)                      # ref_t NULL -> 10, 20
    assert same_bits(c, gold["flux2_cos"]) and same_bits(s, gold["flux2_sin"])
    c, s = rt.flux2_tables(8, 4, 5, REFS, ref_t=[10, 20])
    assert same_bits(c, gold["flux2_cos"]) and same_bits(s, gold["flux2_sin"])


def test_flux3_joint_matches_reference_tables(rt, gold):
    c, s = rt.flux3_tables(8, 4, 5, REFS, theta=10000.0)
    assert same_bits(c, gold["flux3_cos"]) and same_bits(s, gold["flux3_sin"])


def test_qwen3_matches_reference_tables(rt, gold):
    c, s = rt.qwen3_tables(24, 128, 1e6)
    assert same_bits(c, gold["qwen3_cos"]) and same_bits(s, gold["qwen3_sin"])
    mask = np.r_[np.ones(15), np.zeros(9)].astype(np.int32)
    c, s = rt.qwen3_tables(24, 128, 1e6, mask=mask, pad_at_one=True)
    assert same_bits(c, gold["qwen3_f3_cos"]) and same_bits(s, gold["qwen3_f3_sin"])
    # without pad_at_one the mask does not move any row
    c2, s2 = rt.qwen3_tables(24, 128, 1e6, mask=mask, pad_at_one=False)
    assert same_bits(c2, gold["qwen3_cos"]) and same_bits(s2, gold["qwen3_sin"])


def test_zimage_axis_tables_match_reference(rt, gold):
    # position p on one axis, 0 on the others: the axis block must be row p of the reference's axis table
    dims, off = (32, 48, 48), 0
    for ax, d in enumerate(dims):
        pos = np.zeros((40, 3), np.int32)
        pos[:, ax] = np.arange(40)
        c, s = rt.zimage_tables(pos, dims, (40, 40, 40))
        assert same_bits(c[:, off:off + d // 2], gold[f"zimage_cos_{ax}"])
        assert same_bits(s[:, off:off + d // 2], gold[f"zimage_sin_{ax}"])
        off += d // 2


def test_zimage_positions_match_reference(rt, gold):
    pos, mask, ip, cp = rt.zimage_positions(img_seq=27, wt=9, cap_seq=5)
    assert (ip, cp) == (32, 32)
    assert np.array_equal(pos, gold["zi_pos"]) and np.array_equal(mask, gold["zi_mask"])


# ---- against the oracle on the real layouts ----

def test_flux2_full_size_equals_oracle(rt, orc):
    refs = [(32, 32), (16, 24)]
    c, s = rt.flux2_tables(512, 64, 64, refs)
    oc, os_ = orc.flux2_joint_tables(512, 64, 64, refs)
    assert same_bits(c, oc) and same_bits(s, os_)


def test_flux2_custom_t_offsets(rt, orc):
    # a reference image's T coordinate is the caller's: compare with the oracle's image builder
    c, s = rt.flux2_tables(3, 2, 2, [(3, 4)], ref_t=[7])
    oc, os_ = orc.flux2_rope_image(3, 4, t_offset=7)
    assert same_bits(c[7:], oc[:, ::2]) and same_bits(s[7:], os_[:, ::2])


def test_flux3_full_size_equals_oracle(rt, orc):
    refs = [(20, 12)]
    dims = (32, 32, 32, 32)
    c, s = rt.flux3_tables(80, 48, 40, refs, axes_dim=dims, theta=2000.0)
    pos = orc.flux3_joint_positions(80, 48, 40, refs)
    assert np.array_equal(pos, rt.flux3_positions(80, 48, 40, refs))
    oc, os_ = orc.flux3_rope_rows(pos, dims, 2000.0)
    assert same_bits(c, oc) and same_bits(s, os_)


def test_flux3_uneven_axes(rt, orc):
    dims = (8, 28, 28, 64)
    pos = orc.flux3_joint_positions(5, 7, 3, [(2, 2)])
    rc, c, s = rt.expand_f64(pos, dims, 10000.0)
    oc, os_ = orc.flux3_rope_rows(pos, dims, 10000.0)
    assert rc == 0 and same_bits(c, oc) and same_bits(s, os_)


def test_zimage_full_layout_equals_oracle(rt, orc):
    pos, mask, ip, cp = rt.zimage_positions(img_seq=1000, wt=40, cap_seq=77)
    opos, omask, oip, ocp = orc.zimage_positions(1000, 40, 77)
    assert (ip, cp) == (oip, ocp) and np.array_equal(pos, opos) and np.array_equal(mask, omask)
    lens = (64, 20, 512)               # small bounds: caption slots beyond 63 and image rows beyond 19 stay unrotated
    c, s = rt.zimage_tables(pos, (32, 48, 48), lens)
    oc, os_ = orc.zimage_gather(pos, (32, 48, 48), lens)
    assert same_bits(c, oc) and same_bits(s, os_)
    out_of_range = pos[:, 1] >= 20
    assert out_of_range.any()
    assert (c[out_of_range, 16:40] == 1.0).all() and (s[out_of_range, 16:40] == 0.0).all()


def test_qwen3_long_sequence_equals_oracle(rt, orc):
    mask = (np.arange(3000) < 2100).astype(np.int32)
    for pad in (False, True):
        c, s = rt.qwen3_tables(3000, 128, 1e6, mask=mask, pad_at_one=pad)
        oc, os_ = orc.qwen3_rope_table(3000, 128, 1e6, mask=mask, pad_at_one=pad)
        assert same_bits(c, oc) and same_bits(s, os_)


# ---- the engine itself ----

def test_reuse_of_positions_never_changes_a_value(rt):
    """More distinct positions than reuse slots, in an order that makes slots evict each other:
    every row must still equal the row computed alone."""
    g = np.random.default_rng(5)
    pos = g.integers(0, 100000, size=(6000, 2)).astype(np.int32)
    pos[::3] = pos[0]                                       # repeats between evictions
    rc, c, s = rt.expand_i32(pos, (32, 64), 10000.0)
    assert rc == 0
    for i in g.integers(0, 6000, size=200):
        rc1, c1, s1 = rt.expand_i32(pos[i:i + 1], (32, 64), 10000.0)
        assert same_bits(c[i], c1[0]) and same_bits(s[i], s1[0])


def test_dictionary_form_expands_to_the_same_bits(rt, gold):
    """The device entries upload a dictionary of the distinct (axis, position) rows plus one offset per
    (token, axis), and a kernel expands it. Expanded here in numpy: it must give the bits of the direct
    builders, hold each distinct position once, and match the reference's golden tables."""
    # FLUX.2 joint layout: text + image + two reference images
    pos = rt.flux2_positions(8, 4, 5, REFS)
    rc, values, index = rt.dictionary(pos, (32, 32, 32, 32), 2000.0)
    assert rc == 0
    c, s = rt.expand_dictionary(values, index, (32, 32, 32, 32))
    assert same_bits(c, gold["flux2_cos"]) and same_bits(s, gold["flux2_sin"])
    distinct = sum(len(np.unique(pos[:, a])) for a in range(4))
    assert values.size == distinct * 32                      # 16 cos + 16 sin per distinct (axis, position)
    # FLUX.3: float positions, double arithmetic
    fpos = rt.flux3_positions(8, 4, 5, REFS)
    rc, values, index = rt.dictionary(fpos, (32, 32, 32, 32), 10000.0, use_double=True)
    c, s = rt.expand_dictionary(values, index, (32, 32, 32, 32))
    assert rc == 0 and same_bits(c, gold["flux3_cos"]) and same_bits(s, gold["flux3_sin"])
    # Z-Image: bounded axes, uneven axis sizes; many rows, few positions
    zpos, _, _, _ = rt.zimage_positions(img_seq=1000, wt=40, cap_seq=77)
    lens = (64, 20, 512)
    rc, values, index = rt.dictionary(zpos, (32, 48, 48), 256.0, axis_lens=lens)
    c, s = rt.expand_dictionary(values, index, (32, 48, 48))
    hc, hs = rt.zimage_tables(zpos, (32, 48, 48), lens)
    assert rc == 0 and same_bits(c, hc) and same_bits(s, hs)
    assert values.size * 4 < c.nbytes // 10                 # the point of the form: far smaller than the tables
    # every position distinct (text encoder): the dictionary is the table
    rc, values, index = rt.dictionary(np.arange(3000, dtype=np.int32), (128,), 1e6)
    c, s = rt.expand_dictionary(values, index, (128,))
    hc, hs = rt.qwen3_tables(3000, 128, 1e6)
    assert rc == 0 and same_bits(c, hc) and same_bits(s, hs) and values.size == 3000 * 128
    # random positions incl. collisions in the position map
    g = np.random.default_rng(8)
    rpos = g.integers(0, 50000, size=(5000, 3)).astype(np.int32)
    rpos[::5] = rpos[3]
    rc, values, index = rt.dictionary(rpos, (16, 40, 72), 500.0)
    c, s = rt.expand_dictionary(values, index, (16, 40, 72))
    rc2, hc, hs = rt.expand_i32(rpos, (16, 40, 72), 500.0)
    assert rc == 0 and rc2 == 0 and same_bits(c, hc) and same_bits(s, hs)
    # refused arguments
    assert rt.dictionary(rpos, (15, 40, 72), 500.0)[0] == -1
    rc, values, index = rt.dictionary(np.zeros((0, 2), np.int32), (32, 32), 100.0)
    assert rc == 0 and values.size == 0


def test_closed_form(rt):
    """cos / sin of p * theta^(-2j/d), evaluated in double, within float rounding of the angle."""
    pos = np.array([[0, 1], [3, 250], [4095, 17]], np.int32)
    rc, c, s = rt.expand_i32(pos, (32, 96), 2000.0)
    assert rc == 0 and c.shape == (3, 64)
    assert (c[0, :16] == 1.0).all() and (s[0, :16] == 0.0).all()          # position 0: exactly unrotated
    for ax, (d, off) in enumerate(((32, 0), (96, 16))):
        j = np.arange(d // 2)
        freq = (1.0 / np.power(np.float32(2000.0), (2 * j).astype(np.float32) / np.float32(d))).astype(np.float32)
        ang = (pos[:, ax:ax + 1].astype(np.float32) * freq[None, :]).astype(np.float32).astype(np.float64)
        # the float angle may sit one ulp from this numpy restatement (powf rounding): allow |angle| * 2^-22
        tol = np.abs(ang) * 2.0 ** -22 + 1e-7
        assert (np.abs(c[:, off:off + d // 2] - np.cos(ang)) <= tol).all()
        assert (np.abs(s[:, off:off + d // 2] - np.sin(ang)) <= tol).all()
    # cos^2 + sin^2 = 1
    np.testing.assert_allclose(c.astype(np.float64) ** 2 + s.astype(np.float64) ** 2, 1.0, atol=3e-7)


def test_bad_arguments_are_refused(rt):
    pos = np.zeros((4, 2), np.int32)
    c = np.full((4, 32), 7.0, np.float32); s = c.copy()
    P = lambda a: a.ctypes.data
    dims_odd = np.array([31, 33], np.int32)
    assert rt.lib.iris_rope_expand_i32(P(c), P(s), P(pos), 4, 2, P(dims_odd), None, 100.0) == -1
    dims = np.array([32, 32], np.int32)
    assert rt.lib.iris_rope_expand_i32(P(c), P(s), P(pos), 4, 0, P(dims), None, 100.0) == -1
    assert rt.lib.iris_rope_expand_i32(P(c), P(s), P(pos), -1, 2, P(dims), None, 100.0) == -1
    assert rt.lib.iris_rope_expand_i32(None, P(s), P(pos), 4, 2, P(dims), None, 100.0) == -1
    assert (c == 7.0).all() and (s == 7.0).all()            # outputs untouched
    assert rt.lib.iris_rope_expand_i32(P(c), P(s), P(pos), 0, 2, P(dims), None, 100.0) == 0      # empty: fine


def test_empty_parts(rt, orc):
    c, s = rt.flux2_tables(0, 3, 3)
    oc, os_ = orc.flux2_joint_tables(0, 3, 3)
    assert same_bits(c, oc) and same_bits(s, os_)
    c, s = rt.flux2_tables(5, 0, 0)
    oc, os_ = orc.flux2_joint_tables(5, 0, 0)
    assert same_bits(c, oc) and same_bits(s, os_)
    assert rt.joint_rows(0, 0, 0) == 0
