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


@pytest.mark.parametrize("hd,split", [(64, 0), (64, 1), (256, 0), (96, 1)])
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
    """4608 x 24 x 128 (the benchmark shape): a sample of rows against the
    oracle, and two size-independent properties: unit RMS per head when w = 1
    and table = identity; rotation by the tables then by their conjugate
    restores the normalised input to within two roundings."""
    case = W.c2()
    seq, ldi = case["seq"], case["ldi"]
    got = dev.norm_rope(case["buf"], ldi, 0, case["wq"], case["cos"], case["sin"], seq, 24, 128, 1e-6, 0)
    rows = np.r_[0:4, 510:514, 2300:2304, seq - 4:seq]
    want = case["buf"][rows].copy()
    orc.head_norm_rope_bf16(want, ldi, case["wq"], case["cos"][rows], case["sin"][rows], rows.size, 24, 128, 1e-6, 0)
    compare(got[rows], want, slice(0, 3072))
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
