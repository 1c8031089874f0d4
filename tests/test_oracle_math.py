"""Pins of the oracle that need no reference build: published generator
vectors, closed forms in float64, invariants, brute force, and independent
library routines (torch.bfloat16 casting, torch SDPA). Each is chosen so a
plausible mistake (dropped term, wrong sign or index, transposed operand)
fails it.
"""
import numpy as np
import pytest
import torch

import oracle as O


# ---------------------------------------------------------------- generators
def test_splitmix64_published_vector(orc):
    st = orc.rng(0)
    # SplitMix64 from seed 0 (widely published first outputs)
    assert [int(x) for x in st.s][:3] == [0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4, 0x06C45D188009454F]


def test_xoshiro256ss_published_vector(orc):
    st = orc.rng(0)
    for i, v in enumerate((1, 2, 3, 4)):
        st.s[i] = v
    got = [orc.rng_next(st) for _ in range(4)]
    assert got == [11520, 0, 1509978240, 1215971899390074240]


def test_uniform_is_53bit_fraction(orc):
    st, st2 = orc.rng(99), orc.rng(99)
    for _ in range(100):
        u = orc.rng_uniform(st)
        raw = orc.rng_next(st2)
        assert u == np.float32((raw >> 11) * (1.0 / 9007199254740992.0))
        assert 0.0 <= u <= 1.0


def test_normal_moments(orc):
    x = orc.randn(orc.rng(3), 200000)
    assert abs(x.mean()) < 0.01 and abs(x.std() - 1) < 0.01


# ---------------------------------------------------------------- bf16
def test_bf16_rne_exhaustive_upper_halves(orc):
    """All 2^16 upper halves x lower halves around the tie, vs the closed form."""
    hi = np.arange(1 << 16, dtype=np.uint32)
    finite = ((hi >> 7) & 0xFF) != 0xFF
    for lo in (0x0000, 0x0001, 0x7FFF, 0x8000, 0x8001, 0xFFFF):
        u = (hi << 16) | lo
        got = O.f32_to_bf16(u.view(np.float32))
        if lo < 0x8000:
            want = hi
        elif lo > 0x8000:
            want = hi + 1
        else:
            want = hi + (hi & 1)        # tie -> even
        assert np.array_equal(got[finite], (want & 0xFFFF).astype(np.uint16)[finite]), hex(lo)


def test_bf16_matches_torch_cast(orc):
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(100000).astype(np.float32) * 10.0 ** rng.integers(-20, 20, 100000),
                        np.array([0.0, -0.0, 1.0, 3.3895314e38, 1e-40, np.inf, -np.inf], dtype=np.float32)])
    got = O.f32_to_bf16(x)
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got, want)
    assert np.array_equal(O.bf16_to_f32(got), torch.from_numpy(x).to(torch.bfloat16).float().numpy())


# ---------------------------------------------------------------- exp / softmax
def test_fast_expf_accuracy_and_cutoffs(orc):
    xs = np.linspace(-87.0, 80.0, 20001)
    got = np.array([orc.fast_expf(float(x)) for x in xs])
    rel = np.abs(got - np.exp(xs)) / np.exp(xs)
    # degree-5 Taylor on |r| <= ln2/2 (2.4e-6) plus the single-constant range reduction
    assert rel.max() < 1e-5
    assert orc.fast_expf(-87.31) == 0.0 and orc.fast_expf(-1e9) == 0.0
    assert orc.fast_expf(0.0) == 1.0


def test_softmax_rows_vs_float64(orc):
    rng = np.random.default_rng(1)
    x = (rng.standard_normal((9, 77)) * 5).astype(np.float32)
    got = orc.softmax_rows(x)
    e = np.exp(x.astype(np.float64) - x.max(1, keepdims=True))
    np.testing.assert_allclose(got, e / e.sum(1, keepdims=True), rtol=1e-5)
    np.testing.assert_allclose(got.sum(1), 1.0, rtol=1e-6)


# ---------------------------------------------------------------- norm + rope
def test_rms_norm_closed_form_and_unit_rms(orc):
    rng = np.random.default_rng(2)
    x = rng.standard_normal((64, 128)).astype(np.float32) * 3
    w = (1 + 0.02 * rng.standard_normal(128)).astype(np.float32)
    eps = 1e-6
    x64 = x.astype(np.float64)
    want = x64 / np.sqrt((x64 ** 2).mean(1, keepdims=True) + eps) * w
    np.testing.assert_allclose(orc.rms_norm_rows(x, w, eps), want, rtol=2e-6)
    y = orc.rms_norm_rows(x, np.ones(128, np.float32), eps).astype(np.float64)
    ms = (x64 ** 2).mean(1)
    np.testing.assert_allclose(np.sqrt((y ** 2).mean(1)), 1 / np.sqrt(1 + eps / ms), rtol=1e-6)


def test_rope_pairs_is_complex_multiply(orc):
    rng = np.random.default_rng(3)
    x = rng.standard_normal((7, 2, 128)).astype(np.float32)
    ang = rng.uniform(-3, 3, (7, 64))
    c, s = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    z = (x[..., 0::2] + 1j * x[..., 1::2]) * (c + 1j * s)[:, None, :]
    got = orc.rope_pairs(x, c, s)
    np.testing.assert_allclose(got[..., 0::2], z.real, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(got[..., 1::2], z.imag, rtol=1e-5, atol=1e-6)
    # split-half: same rotation on pairs (i, i+64)
    z2 = (x[..., :64] + 1j * x[..., 64:]) * (c + 1j * s)[:, None, :]
    got2 = orc.rope_split(x, c, s)
    np.testing.assert_allclose(got2[..., :64], z2.real, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(got2[..., 64:], z2.imag, rtol=1e-5, atol=1e-6)


def test_rope_invariants(orc):
    rng = np.random.default_rng(4)
    x = rng.standard_normal((5, 3, 128)).astype(np.float32)
    ang = rng.uniform(-3, 3, (5, 64))
    c, s = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    for fn in (orc.rope_pairs, orc.rope_split):
        y = fn(x, c, s)
        np.testing.assert_allclose((y ** 2).sum(-1), (x ** 2).sum(-1), rtol=1e-5)   # norm preserved
        np.testing.assert_allclose(fn(y, c, -s), x, rtol=1e-4, atol=1e-5)           # rotate back
        ident = fn(x, np.ones_like(c), np.zeros_like(s))
        assert np.array_equal(ident, x)                                             # position 0


def test_head_norm_rope_f32_is_norm_then_rope(orc):
    rng = np.random.default_rng(5)
    x = rng.standard_normal((6, 4, 128)).astype(np.float32)
    w = (1 + 0.02 * rng.standard_normal(128)).astype(np.float32)
    ang = rng.uniform(-3, 3, (6, 64))
    c, s = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    for split, rope in ((0, orc.rope_pairs), (1, orc.rope_split)):
        normed = orc.rms_norm_rows(x.reshape(24, 128), w, 1e-6).reshape(6, 4, 128)
        np.testing.assert_allclose(orc.head_norm_rope_f32(x, w, c, s, 1e-6, split), rope(normed, c, s),
                                   rtol=1e-5, atol=1e-6)


def test_head_norm_rope_bf16_strided_and_rounding(orc):
    """Device semantics on bf16 storage: interior column offset, row stride
    larger than the payload, untouched neighbours, one rounding at the end."""
    rng = np.random.default_rng(6)
    seq, heads, hd, ld, col0 = 9, 3, 128, 3 * 3 * 128 + 64, 3 * 128
    buf = O.f32_to_bf16(rng.standard_normal((seq, ld)).astype(np.float32))
    before = buf.copy()
    w = (1 + 0.02 * rng.standard_normal(hd)).astype(np.float32)
    ang = rng.uniform(-3, 3, (seq, 64))
    c, s = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    orc.head_norm_rope_bf16(buf, ld, w, c, s, seq, heads, hd, 1e-6, 0, col0=col0)
    cols = slice(col0, col0 + heads * hd)
    assert np.array_equal(buf[:, :col0], before[:, :col0])
    assert np.array_equal(buf[:, col0 + heads * hd:], before[:, col0 + heads * hd:])
    xin = O.bf16_to_f32(before[:, cols]).reshape(seq, heads, hd)
    want = orc.head_norm_rope_f32(xin, w, c, s, 1e-6, 0)
    got = O.bf16_to_f32(buf[:, cols]).reshape(seq, heads, hd)
    # one RNE rounding of an f32 value: within half a bf16 ulp (2^-9 relative)
    assert np.all(np.abs(got - want) <= np.abs(want) * 2.0 ** -8 + 1e-30)
    assert np.array_equal(buf[:, cols], O.f32_to_bf16(want).reshape(seq, -1))


# ---------------------------------------------------------------- tables: closed forms
def _closed(pos, dim, theta):
    d = np.arange(dim // 2, dtype=np.float64)
    ang = np.asarray(pos, dtype=np.float64)[:, None] * theta ** (-2 * d / dim)
    return np.cos(ang), np.sin(ang)


def test_flux2_tables_closed_form_and_layout(orc):
    txt, h, w = 12, 5, 7
    c, s = orc.flux2_joint_tables(txt, h, w, [(3, 4)])
    assert c.shape == (txt + h * w + 12, 64)
    # text rows: axes T,H,W identity exactly, L = token index
    assert np.all(c[:txt, :48] == 1.0) and np.all(s[:txt, :48] == 0.0)
    cc, ss = _closed(np.arange(txt), 32, 2000.0)
    np.testing.assert_allclose(c[:txt, 48:], cc, atol=2e-6); np.testing.assert_allclose(s[:txt, 48:], ss, atol=2e-6)
    # image rows: T identity, H = row, W = column, L identity
    img = slice(txt, txt + h * w)
    ys, xs = np.divmod(np.arange(h * w), w)
    assert np.all(c[img, :16] == 1.0) and np.all(s[img, :16] == 0.0)
    assert np.all(c[img, 48:] == 1.0) and np.all(s[img, 48:] == 0.0)
    np.testing.assert_allclose(c[img, 16:32], _closed(ys, 32, 2000.0)[0], atol=2e-6)
    np.testing.assert_allclose(s[img, 32:48], _closed(xs, 32, 2000.0)[1], atol=2e-6)
    # reference image 0: T = 10
    r0 = slice(txt + h * w, txt + h * w + 12)
    np.testing.assert_allclose(c[r0, :16], np.repeat(_closed([10], 32, 2000.0)[0], 12, 0), atol=2e-6)
    np.testing.assert_allclose(s[r0, :16], np.repeat(_closed([10], 32, 2000.0)[1], 12, 0), atol=2e-6)


def test_zimage_positions_and_mask_exact(orc):
    pos, mask, ip, cp = orc.zimage_positions(img_seq=50, wt=10, cap_seq=21)
    assert (ip, cp) == (64, 32)
    want = np.zeros((96, 3), np.int32)
    want[:50, 0] = cp + 1
    want[:50, 1] = np.arange(50) // 10
    want[:50, 2] = np.arange(50) % 10
    want[64:, 0] = 1 + np.arange(32)
    assert np.array_equal(pos, want)
    assert np.array_equal(mask, np.r_[np.ones(50), np.zeros(14), np.ones(21), np.zeros(11)].astype(np.int32))


def test_zimage_gather_closed_form(orc):
    pos = np.array([[33, 4, 9], [0, 0, 0], [5, 1023, 1024], [-1, 3, 2]], np.int32)
    c, s = orc.zimage_gather(pos)
    assert c.shape == (4, 64)
    for ax, (lo, hi, dim) in enumerate(((0, 16, 32), (16, 40, 48), (40, 64, 48))):
        cc, ss = _closed(pos[:, ax], dim, 256.0)
        valid = (pos[:, ax] >= 0) & (pos[:, ax] < 1024)
        np.testing.assert_allclose(c[valid, lo:hi], cc[valid], atol=3e-5)
        np.testing.assert_allclose(s[valid, lo:hi], ss[valid], atol=3e-5)
        assert np.all(c[~valid, lo:hi] == 1.0) and np.all(s[~valid, lo:hi] == 0.0)


def test_flux3_positions_and_tables(orc):
    pos = orc.flux3_joint_positions(3, 2, 3, [(1, 2), (2, 1)])
    want = np.array([[0, 0, 0, 0], [0, 0, 0, 1], [0, 0, 0, 2],
                     [0, 0, 0, 0], [0, 0, .5, 0], [0, 0, 1, 0], [0, .5, 0, 0], [0, .5, .5, 0], [0, .5, 1, 0],
                     [0, 0, 0, -1], [0, 0, .5, -1],
                     [0, 0, 0, -2], [0, .5, 0, -2]], np.float32)
    assert np.array_equal(pos, want)
    c, s = orc.flux3_rope_rows(pos)
    for ax in range(4):
        cc, ss = _closed(pos[:, ax], 32, 10000.0)
        assert np.array_equal(c[:, 16 * ax:16 * ax + 16], cc.astype(np.float32))   # double math, then one cast
        assert np.array_equal(s[:, 16 * ax:16 * ax + 16], ss.astype(np.float32))


def test_qwen3_table_closed_form_and_pad_relocation(orc):
    c, s = orc.qwen3_rope_table(512, 128, 1e6)
    cc, ss = _closed(np.arange(512), 128, 1e6)
    np.testing.assert_allclose(c, cc, atol=4e-5); np.testing.assert_allclose(s, ss, atol=4e-5)
    mask = [1] * 5 + [0] * 3
    c1, s1 = orc.qwen3_rope_table(8, 128, 1e6, mask=mask, pad_at_one=True)
    assert np.array_equal(c1[:5], c[:5]) and np.array_equal(c1[5:], np.repeat(c[1:2], 3, 0))
    c0, _ = orc.qwen3_rope_table(8, 128, 1e6, mask=mask, pad_at_one=False)
    assert np.array_equal(c0, c[:8])


# ---------------------------------------------------------------- attention
def _brute(q, k, v, heads, kv_heads, scale, causal=False, mask=None):
    """float64 attention over [seq, heads*hd] rows; masked keys dropped."""
    sq, sk = q.shape[0], k.shape[0]
    hd = q.shape[1] // heads
    out = np.zeros((sq, heads * hd))
    for h in range(heads):
        g = h // (heads // kv_heads)
        qh, kh, vh = (a.astype(np.float64) for a in (q[:, h * hd:(h + 1) * hd], k[:, g * hd:(g + 1) * hd], v[:, g * hd:(g + 1) * hd]))
        sc = qh @ kh.T * scale
        ok = np.ones((sq, sk), bool)
        if causal:
            ok &= np.arange(sk)[None, :] <= np.arange(sq)[:, None]
        if mask is not None:
            ok &= np.asarray(mask, bool)[None, :]
        sc = np.where(ok, sc, -np.inf)
        p = np.exp(sc - sc.max(1, keepdims=True))
        out[:, h * hd:(h + 1) * hd] = (p / p.sum(1, keepdims=True)) @ vh
    return out


@pytest.mark.parametrize("sq,sk,heads,kv,causal,masked", [
    (7, 11, 2, 2, False, False), (70, 140, 3, 3, False, False), (16, 16, 4, 1, True, False),
    (40, 40, 8, 2, True, True), (33, 65, 2, 2, False, True)])
def test_attention_vs_float64_brute_force(orc, sq, sk, heads, kv, causal, masked):
    rng = np.random.default_rng(sq + sk)
    hd = 32
    q = rng.standard_normal((sq, heads * hd)).astype(np.float32)
    k = rng.standard_normal((sk, kv * hd)).astype(np.float32)
    v = rng.standard_normal((sk, kv * hd)).astype(np.float32)
    mask = None
    if masked:
        mask = (rng.random(sk) < 0.6).astype(np.int32)
        mask[0] = 1
    want = _brute(q, k, v, heads, kv, 1 / np.sqrt(hd), causal, mask)
    got = orc.attention_strided(q, k, v, heads, kv, 1 / np.sqrt(hd), causal, mask)
    np.testing.assert_allclose(got, want, rtol=2e-4, atol=2e-5)
    if not causal and not masked and heads == kv:
        np.testing.assert_allclose(orc.attention_flash(q, k, v, heads, 1 / np.sqrt(hd)), want, rtol=2e-4, atol=2e-5)
        Q = q.reshape(sq, heads, hd).transpose(1, 0, 2)[None]
        K = k.reshape(sk, heads, hd).transpose(1, 0, 2)[None]
        V = v.reshape(sk, heads, hd).transpose(1, 0, 2)[None]
        naive = orc.attention_naive(Q, K, V, 1 / np.sqrt(hd))[0].transpose(1, 0, 2).reshape(sq, -1)
        np.testing.assert_allclose(naive, want, rtol=2e-4, atol=2e-5)


@pytest.mark.parametrize("causal,gqa,masked", [(False, False, False), (False, False, True), (True, True, True), (True, True, False)])
def test_attention_vs_torch_sdpa(orc, causal, gqa, masked):
    torch.manual_seed(0)
    sq = sk = 48
    heads, kv, hd = (8, 2, 64) if gqa else (4, 4, 64)
    q, k, v = torch.randn(sq, heads * hd), torch.randn(sk, kv * hd), torch.randn(sk, kv * hd)
    valid = 29
    mask = np.r_[np.ones(valid), np.zeros(sk - valid)].astype(np.int32) if masked else None
    Q = q.view(sq, heads, hd).transpose(0, 1)[None]
    K = k.view(sk, kv, hd).transpose(0, 1)[None].repeat_interleave(heads // kv, 1)
    V = v.view(sk, kv, hd).transpose(0, 1)[None].repeat_interleave(heads // kv, 1)
    bias = torch.zeros(sq, sk)
    if causal:
        bias = bias.masked_fill(torch.ones(sq, sk).triu(1).bool(), float("-inf"))
    if masked:
        bias = bias.masked_fill(torch.from_numpy(mask == 0)[None, :], float("-inf"))
    want = torch.nn.functional.scaled_dot_product_attention(Q, K, V, attn_mask=bias)[0].transpose(0, 1).reshape(sq, -1)
    got = orc.attention_strided(q.numpy(), k.numpy(), v.numpy(), heads, kv, 1 / np.sqrt(hd), causal, mask)
    np.testing.assert_allclose(got, want.numpy(), rtol=2e-4, atol=2e-5)


def test_attention_invariants(orc):
    rng = np.random.default_rng(8)
    heads, hd, sq, sk = 2, 32, 9, 21
    q = rng.standard_normal((sq, heads * hd)).astype(np.float32)
    k = rng.standard_normal((sk, heads * hd)).astype(np.float32)
    v = rng.standard_normal((sk, heads * hd)).astype(np.float32)
    sc = 1 / np.sqrt(hd)
    base = orc.attention_strided(q, k, v, heads, heads, sc)
    # constant V -> constant output
    vc = np.tile(v[:1], (sk, 1))
    np.testing.assert_allclose(orc.attention_strided(q, k, vc, heads, heads, sc), np.tile(v[:1], (sq, 1)), rtol=1e-5, atol=1e-6)
    # key permutation invariance (non causal)
    perm = rng.permutation(sk)
    np.testing.assert_allclose(orc.attention_strided(q, k[perm], v[perm], heads, heads, sc), base, rtol=1e-4, atol=1e-5)
    # masked == compacted
    mask = (rng.random(sk) < 0.5).astype(np.int32); mask[3] = 1
    np.testing.assert_allclose(orc.attention_strided(q, k, v, heads, heads, sc, key_mask=mask),
                               orc.attention_strided(q, k[mask == 1], v[mask == 1], heads, heads, sc), rtol=1e-4, atol=1e-5)
    # single valid key -> that V row; causal row 0 -> V[0]
    one = np.zeros(sk, np.int32); one[5] = 1
    np.testing.assert_allclose(orc.attention_strided(q, k, v, heads, heads, sc, key_mask=one), np.tile(v[5:6], (sq, 1)), rtol=1e-6)
    cz = orc.attention_strided(q, k[:sq], v[:sq], heads, heads, sc, causal=True)
    np.testing.assert_allclose(cz[0], v[0], rtol=1e-6)
    # GQA head h == MHA with kv head h // group
    kv = 1
    g = orc.attention_strided(q, k[:, :hd], v[:, :hd], heads, kv, sc)
    m = orc.attention_strided(q, np.tile(k[:, :hd], (1, heads)), np.tile(v[:, :hd], (1, heads)), heads, heads, sc)
    np.testing.assert_allclose(g, m, rtol=1e-6)


def test_attention_bf16_entry_points(orc):
    """bf16-storage wrappers: fused [q|k|v] rows, interior columns, row subset."""
    rng = np.random.default_rng(9)
    heads, kv, hd, seq = 4, 2, 32, 19
    qd, kd = heads * hd, kv * hd
    ldi = qd + 2 * kd + 8
    buf = O.f32_to_bf16(rng.standard_normal((seq, ldi)).astype(np.float32))
    f = O.bf16_to_f32(buf)
    mask = np.r_[np.ones(13), np.zeros(6)].astype(np.int32)
    want = orc.attention_strided(f[:, :qd], f[:, qd:qd + kd], f[:, qd + kd:qd + 2 * kd], heads, kv, 0.2, True, mask)
    got = orc.attention_bf16(buf, ldi, 0, qd, qd + kd, seq, seq, heads, kv, hd, 0.2, True, mask)
    assert np.array_equal(got, want)
    rows = [0, 7, 18]
    sub = orc.attention_bf16(buf, ldi, 0, qd, qd + kd, seq, seq, heads, kv, hd, 0.2, True, mask, rows=rows)
    assert np.array_equal(sub, want[rows])
