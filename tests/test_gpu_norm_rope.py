"""Fused per-head RMSNorm + RoPE on the GPU (through the C ABI) against the
CPU oracle's restatement of the device semantics on identical bf16 inputs.

Bar: max-abs <= 2e-2, mean-abs <= 2e-3 (bf16 vs fp32 oracle). In practice the
kernel rounds the same f32 value once, so results are also required to be
within one bf16 ulp everywhere and bit-identical almost everywhere.
"""
import numpy as np
import pytest

import oracle as O
import workloads as W
from gpu_harness import Dev, assert_parity

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    return Dev()


def ulp_diff(a, b):
    """Distance in bf16 code points (sign-magnitude order)."""
    def key(u):
        u = u.astype(np.int32)
        return np.where(u & 0x8000, 0x8000 - (u & 0x7fff), 0x8000 + u)
    return np.abs(key(a) - key(b))


def compare(got_buf, want_buf, cols):
    g, w = got_buf[:, cols], want_buf[:, cols]
    assert_parity(O.bf16_to_f32(g), O.bf16_to_f32(w), "norm+rope")
    # One rounding of (nearly) the same f32 value: at most one bf16 code point
    # apart, except where a*c - b*s cancels to ~0 and the f32 operation order
    # (fma vs mul+add) decides the low bits: there the absolute gap is tiny.
    d = ulp_diff(g, w)
    gap = np.abs(O.bf16_to_f32(g) - O.bf16_to_f32(w))
    assert np.all((d <= 1) | (gap <= 1e-5)), f"max bf16 ulp distance {d.max()}, max gap {gap[d > 1].max()}"
    assert (d != 0).mean() < 0.02, f"{(d != 0).mean():.4f} of the values differ"


def run_both(dev, orc, case, which, seq=None):
    seq = seq or case["seq"]
    col0 = 0 if which == "q" else case["q_dim"]
    heads = case["heads"] if which == "q" else case["kv_heads"]
    w = case["wq"] if which == "q" else case["wk"]
    buf = case["buf"][:seq].copy()
    want = buf.copy()
    orc.head_norm_rope_bf16(want, case["ldi"], w, case["cos"], case["sin"], seq, heads, 128, case["eps"],
                            case["split_half"], col0=col0)
    got = dev.norm_rope(buf, case["ldi"], col0, w, case["cos"], case["sin"], seq, heads, 128, case["eps"],
                        case["split_half"])
    return got, want, slice(col0, col0 + heads * 128)


@pytest.mark.parametrize("maker,shrink", [(W.c1, 1), (W.c2, 16), (W.c4, 1), (W.c5, 64)])
def test_norm_rope_matches_oracle(dev, orc, maker, shrink):
    case = maker(shrink)
    for which in ("q", "k"):
        got, want, cols = run_both(dev, orc, case, which)
        compare(got, want, cols)
        # everything outside the normalised columns is untouched
        rest = np.ones(case["ldi"], bool); rest[cols] = False
        assert np.array_equal(got[:, rest], case["buf"][:, rest])
        assert dev.dev.last_kernel() == "norm_rope_hd128"


def test_norm_rope_zimage_eps_and_tables(dev, orc):
    cond, _ = W.c3(shrink=16)
    got, want, cols = run_both(dev, orc, cond, "q")
    compare(got, want, cols)


def test_fused_qk_equals_two_calls(dev, orc):
    for case in (W.c2(shrink=32), W.c4(shrink=2)):
        buf = case["buf"].copy()
        fused = dev.norm_rope_qk(buf, case["ldi"], 0, case["q_dim"], case["wq"], case["wk"], case["cos"],
                                 case["sin"], case["seq"], case["heads"], case["kv_heads"], 128, case["eps"],
                                 case["split_half"])
        two = dev.norm_rope(buf, case["ldi"], 0, case["wq"], case["cos"], case["sin"], case["seq"],
                            case["heads"], 128, case["eps"], case["split_half"])
        two = dev.norm_rope(two, case["ldi"], case["q_dim"], case["wk"], case["cos"], case["sin"], case["seq"],
                            case["kv_heads"], 128, case["eps"], case["split_half"])
        assert np.array_equal(fused, two)
        vcols = slice(case["q_dim"] + case["kv_dim"], None)
        assert np.array_equal(fused[:, vcols], case["buf"][:, vcols])


@pytest.mark.parametrize("seq,heads", [(1, 1), (5, 1), (700, 1), (3, 5), (17, 30), (2, 255)])
def test_ragged_sizes(dev, orc, seq, heads):
    """Includes one head over several tokens: the (token, head) split of the fast kernel has no
    32-bit division constant for a divisor of one and must take the unit index as the token."""
    rng = np.random.default_rng(seq * 100 + heads)
    ld = heads * 128 + 8
    buf = O.f32_to_bf16(rng.standard_normal((seq, ld)).astype(np.float32) * 3)
    w = (1 + 0.02 * rng.standard_normal(128)).astype(np.float32)
    ang = rng.uniform(-3, 3, (seq, 64))
    c, s = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    for split in (0, 1):
        want = buf.copy()
        orc.head_norm_rope_bf16(want, ld, w, c, s, seq, heads, 128, 1e-6, split)
        got = dev.norm_rope(buf, ld, 0, w, c, s, seq, heads, 128, 1e-6, split)
        assert dev.dev.last_kernel() == "norm_rope_hd128"
        compare(got, want, slice(0, heads * 128))
        assert np.array_equal(got[:, heads * 128:], buf[:, heads * 128:])


def test_empty_input_is_a_no_op(dev):
    buf = np.arange(256, dtype=np.uint16).reshape(1, 256)
    w = np.ones(128, np.float32); t = np.ones((1, 64), np.float32)
    assert np.array_equal(dev.norm_rope(buf, 256, 0, w, t, t, 0, 2, 128, 1e-6, 0), buf)


@pytest.mark.parametrize("hd,split", [(64, 0), (64, 1), (256, 0), (96, 1), (2048, 0), (2050, 1)])
def test_other_head_dims_take_the_generic_kernel(dev, orc, hd, split):
    rng = np.random.default_rng(hd)
    seq, heads = 9, 3
    ld = heads * hd
    buf = O.f32_to_bf16(rng.standard_normal((seq, ld)).astype(np.float32))
    w = (1 + 0.02 * rng.standard_normal(hd)).astype(np.float32)
    ang = rng.uniform(-3, 3, (seq, hd // 2))
    c, s = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    want = buf.copy()
    orc.head_norm_rope_bf16(want, ld, w, c, s, seq, heads, hd, 1e-6, split)
    got = dev.norm_rope(buf, ld, 0, w, c, s, seq, heads, hd, 1e-6, split)
    assert dev.dev.last_kernel() == "norm_rope_generic"
    compare(got, want, slice(0, ld))


def test_misaligned_rows_take_the_generic_kernel(dev, orc):
    rng = np.random.default_rng(77)
    seq, heads, ld = 5, 2, 2 * 128 + 3          # ld not a multiple of 8 elements
    buf = O.f32_to_bf16(rng.standard_normal((seq, ld)).astype(np.float32))
    w = np.ones(128, np.float32)
    ang = rng.uniform(-3, 3, (seq, 64))
    c, s = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    want = buf.copy()
    orc.head_norm_rope_bf16(want, ld, w, c, s, seq, heads, 128, 1e-6, 0)
    got = dev.norm_rope(buf, ld, 0, w, c, s, seq, heads, 128, 1e-6, 0)
    assert dev.dev.last_kernel() == "norm_rope_generic"
    compare(got, want, slice(0, 256))


def test_full_size_c2_properties(dev, orc):
    """4608 x 24 x 128 (the benchmark shape): every row against the
    oracle, and two size-independent properties: unit RMS per head when w = 1
    and table = identity; rotation by the tables then by their conjugate
    restores the normalised input to within two roundings."""
    case = W.c2()
    seq, ldi = case["seq"], case["ldi"]
    got = dev.norm_rope(case["buf"], ldi, 0, case["wq"], case["cos"], case["sin"], seq, 24, 128, 1e-6, 0)
    want = case["buf"].copy()                                  # every one of the 4608 rows
    orc.head_norm_rope_bf16(want, ldi, case["wq"], case["cos"], case["sin"], seq, 24, 128, 1e-6, 0)
    compare(got, want, slice(0, 3072))
    assert np.array_equal(got[:, 3072:], case["buf"][:, 3072:])

    ones, eye_c, eye_s = np.ones(128, np.float32), np.ones((seq, 64), np.float32), np.zeros((seq, 64), np.float32)
    normed = dev.norm_rope(case["buf"], ldi, 0, ones, eye_c, eye_s, seq, 24, 128, 1e-6, 0)
    x = O.bf16_to_f32(normed[:, :3072]).reshape(seq, 24, 128)
    rms = np.sqrt((x.astype(np.float64) ** 2).mean(-1))
    assert np.abs(rms - 1).max() < 4e-3
    rot = dev.norm_rope(normed, ldi, 0, ones, case["cos"], case["sin"], seq, 24, 128, 0.0, 0)
    back = dev.norm_rope(rot, ldi, 0, ones, case["cos"], -case["sin"], seq, 24, 128, 0.0, 0)
    y = O.bf16_to_f32(back[:, :3072]).reshape(seq, 24, 128)
    assert np.abs(y - x).max() < 0.08 and np.abs(y - x).mean() < 6e-3


@pytest.mark.parametrize("name", ["C3-cond", "C3-uncond", "C5"])
def test_full_size_c3_c5_every_row(dev, orc, name):
    """The Z-Image pair (4352 rows x 30 heads, eps 1e-5, its own tables) and the multi-reference configuration
    (12800 rows x 24 heads) at full size: the Q call, the K call and the one-launch Q+K form, every row against the
    oracle."""
    case = {"C3-cond": lambda: W.c3()[0], "C3-uncond": lambda: W.c3()[1], "C5": W.c5}[name]()
    seq, ldi, heads, qd = case["seq"], case["ldi"], case["heads"], case["q_dim"]
    want = case["buf"].copy()
    orc.head_norm_rope_bf16(want, ldi, case["wq"], case["cos"], case["sin"], seq, heads, 128, case["eps"], 0)
    orc.head_norm_rope_bf16(want, ldi, case["wk"], case["cos"], case["sin"], seq, heads, 128, case["eps"], 0, col0=qd)
    got = dev.norm_rope(case["buf"], ldi, 0, case["wq"], case["cos"], case["sin"], seq, heads, 128, case["eps"], 0)
    assert dev.dev.last_kernel() == "norm_rope_hd128"
    compare(got, want, slice(0, qd))
    assert np.array_equal(got[:, qd:], case["buf"][:, qd:])
    got = dev.norm_rope(got, ldi, qd, case["wk"], case["cos"], case["sin"], seq, heads, 128, case["eps"], 0)
    compare(got, want, slice(qd, 2 * qd))
    assert np.array_equal(got[:, 2 * qd:], case["buf"][:, 2 * qd:])
    fused = dev.norm_rope_qk(case["buf"], ldi, 0, qd, case["wq"], case["wk"], case["cos"], case["sin"], seq, heads, heads, 128,
                             case["eps"], 0)
    assert np.array_equal(fused, got), "one Q+K launch differs from the two calls"


def test_c1_against_the_vector_the_compiled_reference_wrote(dev):
    """C1 at full shape: the device's Q and K rows after norm + rope against the f32 rows that the reference's
    apply_qk_norm -> apply_rope_2d produced from the same seeded inputs (tests/golden/c1_chain.npz, written by
    tests/golden/make_golden.py where the reference tree is present): one bf16 rounding apart."""
    import os
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "c1_chain.npz"), allow_pickle=False)
    case = W.c1()
    got = dev.norm_rope_qk(case["buf"], case["ldi"], 0, 3072, case["wq"], case["wk"], case["cos"], case["sin"], case["seq"], 24, 24,
                           128, case["eps"], 0)
    rows = g["rows"]
    for col0, key in ((0, "q_rows"), (3072, "k_rows")):
        have, want = O.bf16_to_f32(got[rows, col0:col0 + 3072]), g[key]
        assert_parity(have, want, f"C1 {key} vs reference")
        # the reference keeps f32; the device rounds once to bf16: half a bf16 step of the value, plus the
        # f32 operation-order noise of the two implementations
        assert np.all(np.abs(have - want) <= np.abs(want) * 2.0 ** -8 + 2e-6), np.abs(have - want).max()


@pytest.mark.parametrize("seq,rows_a,q_heads,k_heads,hd,split", [(320, 64, 24, 24, 128, 0), (77, 0, 3, 3, 128, 0), (77, 77, 3, 1, 128, 1),
                                                               (130, 129, 8, 2, 128, 1), (50, 20, 2, 2, 64, 0), (33, 1, 5, 0, 128, 0)])
def test_two_weight_pairs_in_one_launch(dev, orc, seq, rows_a, q_heads, k_heads, hd, split):
    """iris_dev_head_norm_rope_qk_streams: rows [0, rows_a) with one weight pair, the rest with another, one launch,
    against the oracle applied range by range (the reference's four calls, iris_transformer_flux.c:3796-3803), and
    bit for bit against the library's own four calls."""
    rng = np.random.default_rng(seq + rows_a)
    qd, kd = q_heads * hd, k_heads * hd
    ld = qd + 2 * max(kd, hd) + 8
    buf = O.f32_to_bf16(rng.standard_normal((seq, ld)).astype(np.float32))
    w = [(1 + 0.1 * rng.standard_normal(hd)).astype(np.float32) for _ in range(4)]      # wq_a, wk_a, wq_b, wk_b
    ang = rng.uniform(-3, 3, (seq, hd // 2)).astype(np.float32)
    cos, sin = np.cos(ang), np.sin(ang)
    want = buf.copy()
    for first, n, wq, wk in ((0, rows_a, w[0], w[1]), (rows_a, seq - rows_a, w[2], w[3])):
        if n == 0:
            continue
        orc.head_norm_rope_bf16(want, ld, wq, cos[first:], sin[first:], n, q_heads, hd, 1e-6, split, col0=first * ld)
        if k_heads:
            orc.head_norm_rope_bf16(want, ld, wk, cos[first:], sin[first:], n, k_heads, hd, 1e-6, split, col0=first * ld + qd)
    from gpu_harness import ptr_add
    d = dev.put(buf)
    dw = [dev.put(x) for x in w]
    dc, ds = dev.put(cos), dev.put(sin)
    dev.lib.iris_dev_head_norm_rope_qk_streams(d, ptr_add(d, 2 * qd) if k_heads else None, ld, dw[0], dw[1], dw[2], dw[3], rows_a,
                                               dc, ds, seq, q_heads, k_heads, hd, 1e-6, split)
    dev.check()
    assert dev.dev.last_kernel() == ("norm_rope_hd128" if hd == 128 else "norm_rope_generic")
    got = dev.get(d, buf.shape, np.uint16)
    d2 = dev.put(buf)
    for first, n, wq, wk in ((0, rows_a, dw[0], dw[1]), (rows_a, seq - rows_a, dw[2], dw[3])):
        x = ptr_add(d2, 2 * first * ld)
        c, s_ = ptr_add(dc, 4 * first * (hd // 2)), ptr_add(ds, 4 * first * (hd // 2))
        dev.lib.iris_dev_head_norm_rope(x, ld, wq, c, s_, n, q_heads, hd, 1e-6, split)
        if k_heads:
            dev.lib.iris_dev_head_norm_rope(ptr_add(x, 2 * qd), ld, wk, c, s_, n, k_heads, hd, 1e-6, split)
    dev.check()
    four = dev.get(d2, buf.shape, np.uint16)
    dev.free_all()
    compare(got, want, slice(0, qd + kd))
    assert np.array_equal(got[:, qd + kd:], buf[:, qd + kd:])
    assert np.array_equal(got, four), "one launch differs from the four calls"
