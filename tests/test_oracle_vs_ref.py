"""Pin the oracle against the reference's own C code compiled in place
(oracle/_ref). Skipped where that library was not built (no reference tree).

Two builds of the same sources exist. `ref` uses the reference Makefile's
-O3 -ffast-math: there gcc vectorises the RoPE base-frequency loops with
libmvec's powf (accurate to a few ulp, not correctly rounded), so its
tables are a compiler artefact. `ref_ieee` is built with IEEE semantics and
scalar libm: tables, ids and the RNG are compared with it bit for bit, and
with `ref` to within the libmvec error. f32 arithmetic that a compiler may
reassociate is compared within a few ulp.
"""
import numpy as np
import pytest

import refcalls as R

RTOL = 2e-6


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def assert_bit_equal(a, b):
    assert a.shape == b.shape
    bad = np.nonzero(bits(a) != bits(b))
    assert bad[0].size == 0, f"{bad[0].size} of {a.size} entries differ, first at {[x[0] for x in bad]}"


# ---------------------------------------------------------------- RNG
@pytest.mark.parametrize("seed", [0, 1, 42, 20250102])
def test_rng_uniform_and_normal_bit_exact(orc, ref, seed):
    st = orc.rng(seed)
    mine = np.array([orc.rng_uniform(st) for _ in range(64)], dtype=np.float32)
    assert_bit_equal(mine, R.rng_u64(ref, seed, 64))
    st = orc.rng(seed)
    assert_bit_equal(orc.randn(st, 4096), R.randn(ref, seed, 4096))


# ---------------------------------------------------------------- softmax / norm
def test_softmax_rows_vs_ref(orc, ref):
    rng = np.random.default_rng(0)
    x = (rng.standard_normal((17, 133)) * 6).astype(np.float32)
    x[3, 5:40] = -1e9          # masked entries -> exactly zero
    a, b = orc.softmax_rows(x), R.softmax_rows(ref, x)
    np.testing.assert_allclose(a, b, rtol=RTOL, atol=1e-9)
    assert np.all(a[3, 5:40] == 0.0) and np.all(b[3, 5:40] == 0.0)


@pytest.mark.parametrize("eps", [1e-6, 1e-5])
def test_rms_norm_vs_ref(orc, ref, eps):
    rng = np.random.default_rng(1)
    x = rng.standard_normal((48, 128)).astype(np.float32)
    w = (1 + 0.02 * rng.standard_normal(128)).astype(np.float32)
    np.testing.assert_allclose(orc.rms_norm_rows(x, w, eps), R.rms_norm(ref, x, w, eps), rtol=1e-5)
    x3 = x.reshape(6, 8, 128)
    for fn in (R.flux3_head_rms_norm, R.zi_qk_norm):
        np.testing.assert_allclose(orc.rms_norm_rows(x, w, eps).reshape(6, 8, 128), fn(ref, x3, w, eps), rtol=1e-5)
    q, k = R.flux2_qk_norm(ref, x3, x3[::-1], w, w[::-1].copy(), eps)
    np.testing.assert_allclose(orc.rms_norm_rows(x, w, eps).reshape(6, 8, 128), q, rtol=1e-5)


# ---------------------------------------------------------------- RoPE tables
@pytest.mark.parametrize("theta", [2000.0, 10000.0])
def test_flux2_tables_bit_exact(orc, ref_ieee, theta):
    c, s = orc.flux2_rope_text(77, 32, theta)
    rc, rs = R.flux2_rope_text(ref_ieee, 77, 32, theta)
    assert_bit_equal(c, rc); assert_bit_equal(s, rs)
    c, s = orc.flux2_rope_image(9, 13, 32, theta)
    rc, rs = R.flux2_rope_2d(ref_ieee, 9, 13, 32, theta)
    assert_bit_equal(c, rc); assert_bit_equal(s, rs)
    for t in (10, 20, 30):
        c, s = orc.flux2_rope_image(7, 5, 32, theta, t_offset=t)
        rc, rs = R.flux2_rope_2d(ref_ieee, 7, 5, 32, theta, t_offset=t)
        assert_bit_equal(c, rc); assert_bit_equal(s, rs)


def test_flux2_joint_compacted_bit_exact(orc, ref_ieee):
    refs = [(6, 4), (3, 8)]
    c, s = orc.flux2_joint_tables(19, 8, 8, refs)
    rc, rs = R.flux2_joint_compact(ref_ieee, 19, 8, 8, refs)
    assert c.shape == (19 + 64 + 24 + 24, 64)
    assert_bit_equal(c, rc); assert_bit_equal(s, rs)


def test_flux2_full_size_tables_bit_exact(orc, ref_ieee):
    # 512 text + 64x64 image + two 64x64 references (the 12800-token case)
    c, s = orc.flux2_joint_tables(512, 64, 64, [(64, 64), (64, 64)])
    rc, rs = R.flux2_joint_compact(ref_ieee, 512, 64, 64, [(64, 64), (64, 64)])
    assert_bit_equal(c, rc); assert_bit_equal(s, rs)


def test_zimage_tables_bit_exact(orc, ref_ieee):
    dims, lens = (32, 48, 48), (1024, 1024, 1024)
    for ax in range(3):
        c, s = orc.zimage_axis_table(dims[ax], lens[ax])
        rc, rs = R.zi_axis_table(ref_ieee, ax, dims, lens)
        assert_bit_equal(c, rc); assert_bit_equal(s, rs)


def test_zimage_gather_matches_ref_rotation(orc, ref_ieee):
    """The gathered [seq,64] table applied with consecutive pairs must equal
    the reference's per-axis rotation from position ids, including positions
    outside the table (left unrotated)."""
    rng = np.random.default_rng(5)
    pos, mask, ip, cp = orc.zimage_positions(img_seq=50, wt=10, cap_seq=21)
    pos = pos.copy()
    pos[3] = (-1, 2000, 1024)          # invalid on every axis
    pos[4] = (1023, 0, -5)
    c, s = orc.zimage_gather(pos)
    x = rng.standard_normal((ip + cp, 3, 128)).astype(np.float32)
    mine = orc.rope_pairs(x, c, s)
    theirs = R.zi_apply_rope(ref_ieee, x, pos)
    np.testing.assert_allclose(mine, theirs, rtol=RTOL, atol=1e-7)
    assert np.array_equal(mine[3], x[3])


@pytest.mark.parametrize("refs", [(), [(5, 3)], [(4, 4), (2, 6), (3, 3)]])
def test_flux3_tables_bit_exact(orc, ref_ieee, refs):
    pos = orc.flux3_joint_positions(23, 6, 7, refs)
    c, s = orc.flux3_rope_rows(pos)
    rc, rs = R.flux3_joint_rope(ref_ieee, 23, 6, 7, refs)
    assert_bit_equal(c, rc); assert_bit_equal(s, rs)


@pytest.mark.parametrize("theta", [1e6, 5e6])
def test_qwen3_tables_bit_exact(orc, ref_ieee, theta):
    mask = [1] * 37 + [0] * 27
    for flux3_mode in (False, True):
        c, s = orc.qwen3_rope_table(64, 128, theta, mask=mask, pad_at_one=flux3_mode)
        rc, rs = R.qwen3_rope_table(ref_ieee, 64, 128, theta, mask=mask, flux3_mode=flux3_mode)
        assert_bit_equal(c, rc); assert_bit_equal(s, rs)
    c, s = orc.qwen3_rope_table(512, 128, theta)
    rc, rs = R.qwen3_rope_table(ref_ieee, 512, 128, theta)
    assert_bit_equal(c, rc); assert_bit_equal(s, rs)


def test_public_rope_freqs_bit_exact(orc, ref_ieee):
    pos = [0, 1, 2, 3, 50, 511, 4095]
    assert_bit_equal(orc.rope_freqs_interleaved(pos, 128, 10000.0), R.rope_freqs(ref_ieee, pos, 128, 10000.0))


# ---------------------------------------------------------------- RoPE application
def test_rope_application_vs_ref(orc, ref):
    rng = np.random.default_rng(2)
    x = rng.standard_normal((11, 3, 128)).astype(np.float32)
    c, s = orc.flux2_joint_tables(3, 2, 4)
    np.testing.assert_allclose(orc.rope_pairs(x, c, s), R.flux3_apply_rope(ref, x, c, s), rtol=RTOL, atol=1e-7)
    cd, sd = np.repeat(c, 2, axis=1), np.repeat(s, 2, axis=1)
    np.testing.assert_allclose(orc.rope_pairs_dup(x, cd, sd), R.flux2_apply_rope_2d(ref, x, cd, sd), rtol=RTOL, atol=1e-7)
    np.testing.assert_allclose(orc.rope_pairs(x, c, s), R.flux2_apply_rope_2d(ref, x, cd, sd), rtol=RTOL, atol=1e-7)
    fr = orc.rope_freqs_interleaved(np.arange(11), 128, 1e6)
    x4 = x[None]
    np.testing.assert_allclose(orc.rope_split_interleaved(x4, fr), R.apply_rope_interleaved(ref, x4, fr), rtol=RTOL, atol=1e-7)
    np.testing.assert_allclose(orc.rope_split(x, fr[..., 0], fr[..., 1]), R.apply_rope_interleaved(ref, x4, fr)[0], rtol=RTOL, atol=1e-7)


# ---------------------------------------------------------------- attention
@pytest.mark.parametrize("sq,sk", [(5, 9), (64, 128), (65, 129), (33, 200), (130, 64)])
def test_flash_attention_vs_ref_both_branches(orc, ref, sq, sk):
    rng = np.random.default_rng(sq * 1000 + sk)
    heads, hd = 3, 32
    Q = rng.standard_normal((sq, heads * hd)).astype(np.float32)
    K = rng.standard_normal((sk, heads * hd)).astype(np.float32)
    V = rng.standard_normal((sk, heads * hd)).astype(np.float32)
    scale = 1 / np.sqrt(hd)
    a, b = orc.attention_flash(Q, K, V, heads, scale), R.attention_flash(ref, Q, K, V, heads, scale)
    np.testing.assert_allclose(a, b, rtol=2e-5, atol=2e-6)
    # and the strided oracle (materialised softmax) agrees with both
    c = orc.attention_strided(Q, K, V, heads, heads, scale)
    np.testing.assert_allclose(c, b, rtol=1e-4, atol=1e-5)


def test_naive_attention_vs_ref(orc, ref):
    rng = np.random.default_rng(9)
    Q = rng.standard_normal((2, 3, 17, 16)).astype(np.float32)
    K = rng.standard_normal((2, 3, 29, 16)).astype(np.float32)
    V = rng.standard_normal((2, 3, 29, 16)).astype(np.float32)
    np.testing.assert_allclose(orc.attention_naive(Q, K, V, 0.25), R.attention_naive(ref, Q, K, V, 0.25), rtol=2e-5, atol=2e-6)


def test_flux3_chunked_attention_vs_strided(orc, ref):
    rng = np.random.default_rng(10)
    heads, hd, seq = 2, 128, 300          # > one 256-query chunk
    q, k, v = (rng.standard_normal((seq, heads * hd)).astype(np.float32) for _ in range(3))
    np.testing.assert_allclose(orc.attention_strided(q, k, v, heads, heads, 1 / np.sqrt(hd)),
                               R.flux3_attention(ref, q, k, v, heads), rtol=1e-4, atol=1e-5)


def test_zimage_masked_attention_chain_vs_ref(orc, ref):
    """Whole Z-Image CPU attention (projection, QK norm, RoPE from ids, key
    mask, softmax, PV) against norm+rope+strided attention of the oracle."""
    rng = np.random.default_rng(11)
    dims = (8, 12, 12)
    hd, heads = 32, 2
    dim = hd * heads
    pos, mask, ip, cp = orc.zimage_positions(img_seq=27, wt=9, cap_seq=5)
    seq = ip + cp
    x = rng.standard_normal((seq, dim)).astype(np.float32)
    wq, wk, wv = (rng.standard_normal((dim, dim)).astype(np.float32) / np.sqrt(dim) for _ in range(3))
    wo = np.eye(dim, dtype=np.float32)
    nq = (1 + 0.02 * rng.standard_normal(hd)).astype(np.float32)
    nk = (1 + 0.02 * rng.standard_normal(hd)).astype(np.float32)
    theirs = R.zi_attention(ref, x, wq, wk, wv, wo, nq, nk, pos, mask, heads, dims)

    q = (x.astype(np.float64) @ wq.T.astype(np.float64)).astype(np.float32).reshape(seq, heads, hd)
    k = (x.astype(np.float64) @ wk.T.astype(np.float64)).astype(np.float32).reshape(seq, heads, hd)
    v = (x.astype(np.float64) @ wv.T.astype(np.float64)).astype(np.float32)
    c, s = orc.zimage_gather(pos, axes_dims=dims)
    q = orc.head_norm_rope_f32(q, nq, c, s, 1e-5, 0).reshape(seq, dim)
    k = orc.head_norm_rope_f32(k, nk, c, s, 1e-5, 0).reshape(seq, dim)
    mine = orc.attention_strided(q, k, v, heads, heads, 1 / np.sqrt(hd), key_mask=mask)
    np.testing.assert_allclose(mine, theirs, rtol=2e-4, atol=2e-5)


@pytest.mark.parametrize("valid", [40, 7, 1])
def test_qwen3_causal_gqa_chain_vs_ref(orc, ref, valid):
    rng = np.random.default_rng(12 + valid)
    heads, kv, hd, hidden, seq = 8, 2, 32, 24, 40
    mask = [1] * valid + [0] * (seq - valid)
    x = rng.standard_normal((seq, hidden)).astype(np.float32)
    wq = rng.standard_normal((heads * hd, hidden)).astype(np.float32) / np.sqrt(hidden)
    wk = rng.standard_normal((kv * hd, hidden)).astype(np.float32) / np.sqrt(hidden)
    wv = rng.standard_normal((kv * hd, hidden)).astype(np.float32) / np.sqrt(hidden)
    nq = (1 + 0.02 * rng.standard_normal(hd)).astype(np.float32)
    nk = (1 + 0.02 * rng.standard_normal(hd)).astype(np.float32)
    attn, rq, rk, rv = R.qwen3_attention(ref, x, wq, wk, wv, nq, nk, mask, heads, kv, hd)

    q = (x.astype(np.float64) @ wq.T).astype(np.float32).reshape(seq, heads, hd)
    k = (x.astype(np.float64) @ wk.T).astype(np.float32).reshape(seq, kv, hd)
    v = (x.astype(np.float64) @ wv.T).astype(np.float32)
    c, s = orc.qwen3_rope_table(seq, hd, 1e6)
    q = orc.head_norm_rope_f32(q, nq, c, s, 1e-6, 1).reshape(seq, -1)
    k = orc.head_norm_rope_f32(k, nk, c, s, 1e-6, 1).reshape(seq, -1)
    np.testing.assert_allclose(q, rq, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(k, rk, rtol=1e-4, atol=1e-5)
    mine = orc.attention_strided(q, k, v, heads, kv, 1 / np.sqrt(hd), causal=True, key_mask=mask)
    # rows whose causal window holds a valid key (all of them: key 0 is valid)
    np.testing.assert_allclose(mine, attn, rtol=2e-4, atol=2e-5)


# ---------------------------------------------------------------- fast-math build
def test_tables_close_to_fast_math_build(orc, ref):
    """Against the -ffast-math build the base frequency differs by the
    libmvec powf error (a few ulp), i.e. angle error <= pos * 4e-7 * freq."""
    c, s = orc.flux2_joint_tables(512, 64, 64, [(64, 64)])
    rc, rs = R.flux2_joint_compact(ref, 512, 64, 64, [(64, 64)])
    assert np.abs(c - rc).max() < 3e-4 and np.abs(s - rs).max() < 3e-4
    assert (bits(c) != bits(rc)).mean() < 0.6
    c, s = orc.qwen3_rope_table(512)
    rc, rs = R.qwen3_rope_table(ref, 512)
    assert np.abs(c - rc).max() < 3e-4 and np.abs(s - rs).max() < 3e-4
    pos = orc.flux3_joint_positions(64, 16, 16, [(8, 8)])
    c, s = orc.flux3_rope_rows(pos)
    rc, rs = R.flux3_joint_rope(ref, 64, 16, 16, [(8, 8)])
    assert np.abs(c - rc).max() < 1e-6 and np.abs(s - rs).max() < 1e-6


def test_rng_bit_exact_vs_ieee_build(orc, ref_ieee):
    st = orc.rng(7)
    assert_bit_equal(orc.randn(st, 2048), R.randn(ref_ieee, 7, 2048))
