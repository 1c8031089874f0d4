"""Oracle against the committed golden vectors (tests/golden/ref_vectors.npz,
written by tests/golden/make_golden.py from the reference's own compiled
code). Runs anywhere: needs neither the reference tree nor a GPU.
"""
import os

import numpy as np
import pytest

import oracle as O

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ref_vectors.npz")


@pytest.fixture(scope="module")
def gold():
    return np.load(GOLD, allow_pickle=False)


def inputs(seed, *shape):
    return np.random.default_rng(seed).standard_normal(shape).astype(np.float32)


def same_bits(a, b):
    a = np.ascontiguousarray(a, dtype=np.float32); b = np.ascontiguousarray(b, dtype=np.float32)
    return a.shape == b.shape and np.array_equal(a.view(np.uint32), b.view(np.uint32))


@pytest.mark.parametrize("seed", [0, 1, 42])
def test_rng_bit_exact(orc, gold, seed):
    st = orc.rng(seed)
    assert same_bits(np.array([orc.rng_uniform(st) for _ in range(32)], np.float32), gold[f"rng_uniform_{seed}"])
    assert same_bits(orc.randn(orc.rng(seed), 256), gold[f"rng_normal_{seed}"])


def test_tables_bit_exact(orc, gold):
    c, s = orc.flux2_joint_tables(8, 4, 5, [(2, 3), (3, 2)])
    assert same_bits(c, gold["flux2_cos"]) and same_bits(s, gold["flux2_sin"])
    c, s = orc.flux3_rope_rows(orc.flux3_joint_positions(8, 4, 5, [(2, 3), (3, 2)]))
    assert same_bits(c, gold["flux3_cos"]) and same_bits(s, gold["flux3_sin"])
    c, s = orc.qwen3_rope_table(24, 128, 1e6)
    assert same_bits(c, gold["qwen3_cos"]) and same_bits(s, gold["qwen3_sin"])
    mask = np.r_[np.ones(15), np.zeros(9)].astype(np.int32)
    c, s = orc.qwen3_rope_table(24, 128, 1e6, mask=mask, pad_at_one=True)
    assert same_bits(c, gold["qwen3_f3_cos"]) and same_bits(s, gold["qwen3_f3_sin"])
    for ax, d in enumerate((32, 48, 48)):
        c, s = orc.zimage_axis_table(d, 40)
        assert same_bits(c, gold[f"zimage_cos_{ax}"]) and same_bits(s, gold[f"zimage_sin_{ax}"])
    assert same_bits(orc.rope_freqs_interleaved([0, 1, 7, 300], 128, 10000.0), gold["rope_freqs"])


def test_zimage_ids_bit_exact(orc, gold):
    pos, mask, ip, cp = orc.zimage_positions(img_seq=27, wt=9, cap_seq=5)
    assert np.array_equal(pos, gold["zi_pos"]) and np.array_equal(mask, gold["zi_mask"])


def test_elementwise_ops(orc, gold):
    x = inputs(100, 6, 3, 128)
    w = (1 + 0.02 * inputs(101, 128)).astype(np.float32)
    np.testing.assert_allclose(orc.rms_norm_rows(x.reshape(18, 128), w, 1e-6).reshape(6, 3, 128), gold["head_rms_norm"], rtol=1e-5)
    np.testing.assert_allclose(orc.rope_pairs(x, gold["flux2_cos"][8:14], gold["flux2_sin"][8:14]), gold["rope_pairs"], rtol=2e-6, atol=1e-7)
    c, s = orc.qwen3_rope_table(6, 128, 1e6)
    np.testing.assert_allclose(orc.rope_split(x, c, s), gold["rope_split"], rtol=2e-6, atol=1e-7)
    np.testing.assert_allclose(orc.softmax_rows(inputs(102, 5, 37) * 4), gold["softmax"], rtol=2e-6, atol=1e-9)


@pytest.mark.parametrize("name,sq,sk", [("small", 5, 9), ("edge", 64, 128), ("tiled", 65, 129)])
def test_flash_attention(orc, gold, name, sq, sk):
    Q, K, V = inputs(110, sq, 64), inputs(111, sk, 64), inputs(112, sk, 64)
    np.testing.assert_allclose(orc.attention_flash(Q, K, V, 2, 1 / np.sqrt(32)), gold[f"flash_{name}"], rtol=2e-5, atol=2e-6)
    np.testing.assert_allclose(orc.attention_strided(Q, K, V, 2, 2, 1 / np.sqrt(32)), gold[f"flash_{name}"], rtol=1e-4, atol=1e-5)


def test_zimage_masked_chain(orc, gold):
    dims, heads, hd, dim = (8, 12, 12), 2, 32, 64
    pos, mask = gold["zi_pos"], gold["zi_mask"]
    seq = pos.shape[0]
    x = inputs(120, seq, dim).astype(np.float64)
    wq, wk, wv = (inputs(s, dim, dim) / 8 for s in (121, 122, 123))
    nq, nk = 1 + 0.02 * inputs(124, 32), 1 + 0.02 * inputs(125, 32)
    q = (x @ wq.T.astype(np.float64)).astype(np.float32).reshape(seq, heads, hd)
    k = (x @ wk.T.astype(np.float64)).astype(np.float32).reshape(seq, heads, hd)
    v = (x @ wv.T.astype(np.float64)).astype(np.float32)
    c, s = orc.zimage_gather(pos, axes_dims=dims)
    q = orc.head_norm_rope_f32(q, nq, c, s, 1e-5, 0).reshape(seq, dim)
    k = orc.head_norm_rope_f32(k, nk, c, s, 1e-5, 0).reshape(seq, dim)
    got = orc.attention_strided(q, k, v, heads, heads, 1 / np.sqrt(hd), key_mask=mask)
    np.testing.assert_allclose(got, gold["zi_attention"], rtol=2e-4, atol=2e-5)


def test_qwen3_causal_gqa_chain(orc, gold):
    heads, kv, hd, hidden, seq = 8, 2, 32, 24, 40
    mask = np.r_[np.ones(23), np.zeros(17)].astype(np.int32)
    x = inputs(130, seq, hidden).astype(np.float64)
    wq, wk, wv = inputs(131, heads * hd, hidden) / 5, inputs(132, kv * hd, hidden) / 5, inputs(133, kv * hd, hidden) / 5
    nq, nk = 1 + 0.02 * inputs(134, hd), 1 + 0.02 * inputs(135, hd)
    q = (x @ wq.T.astype(np.float64)).astype(np.float32).reshape(seq, heads, hd)
    k = (x @ wk.T.astype(np.float64)).astype(np.float32).reshape(seq, kv, hd)
    v = (x @ wv.T.astype(np.float64)).astype(np.float32)
    c, s = orc.qwen3_rope_table(seq, hd, 1e6)
    q = orc.head_norm_rope_f32(q, nq, c, s, 1e-6, 1).reshape(seq, -1)
    k = orc.head_norm_rope_f32(k, nk, c, s, 1e-6, 1).reshape(seq, -1)
    np.testing.assert_allclose(q, gold["qwen3_q"], rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(k, gold["qwen3_k"], rtol=1e-4, atol=1e-5)
    got = orc.attention_strided(q, k, v, heads, kv, 1 / np.sqrt(hd), causal=True, key_mask=mask)
    np.testing.assert_allclose(got, gold["qwen3_attention"], rtol=2e-4, atol=2e-5)


def test_other_device_operators(orc, gold):
    """The oracle's device-operator restatements against outputs of the reference's CPU twins
    (written by make_golden.py; the reference works in NCHW, the fixtures are stored channels-last)."""
    xl, Wl = O.f32_to_bf16(inputs(140, 7, 96)), O.f32_to_bf16(inputs(141, 33, 96) * 0.1)
    np.testing.assert_allclose(orc.dev_linear(xl, Wl), gold["ops_linear"], atol=2e-5)
    np.testing.assert_allclose(orc.dev_silu(inputs(142, 500) * 3), gold["ops_silu"], atol=1e-6)
    h, w, cin, cout, k = 6, 5, 8, 4, 3
    img = O.bf16_to_f32(O.f32_to_bf16(inputs(143, h * w, cin)))
    wt = O.f32_to_bf16(inputs(144, cout, k * k * cin) * 0.2)
    np.testing.assert_allclose(orc.dev_conv2d(img, wt, inputs(145, cout), h, w, k, 1, 1, 1), gold["ops_conv2d"], atol=2e-5)
    gimg = inputs(146, 30, 16) * 2 + 0.5
    gamma, beta = (1 + 0.1 * inputs(147, 16)).astype(np.float32), (0.1 * inputs(148, 16)).astype(np.float32)
    np.testing.assert_allclose(orc.dev_group_norm(gimg, gamma, beta, 4, 1e-6, 0), gold["ops_group_norm"], atol=1e-5)
    np.testing.assert_array_equal(orc.dev_upsample2x(inputs(149, 12, 5), 3, 4), gold["ops_upsample2x"])


# ---- the metric's own chain at head_dim 128 (configuration C1, full shape), held by the compiled reference
C1_GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "c1_chain.npz")


def test_c1_chain_f32_plumbing(orc):
    """apply_qk_norm -> apply_rope_2d -> iris_flash_attention of the reference on C1 at full shape (24 x 128, 320
    tokens; vector written by tests/golden/make_golden.py:c1_chain) against the oracle's f32 chain on the same seeded
    inputs: <= 1e-4 absolute, the tolerance of the fp32 plumbing configuration."""
    import workloads as W
    g = np.load(C1_GOLD, allow_pickle=False)
    case = W.c1()
    seq, heads, hd, dim = case["seq"], 24, 128, 3072
    f = O.bf16_to_f32(case["buf"])
    q, k, v = (np.ascontiguousarray(f[:, i * dim:(i + 1) * dim]) for i in range(3))
    qn = orc.head_norm_rope_f32(q.reshape(seq, heads, hd), case["wq"], case["cos"], case["sin"], case["eps"], 0).reshape(seq, dim)
    kn = orc.head_norm_rope_f32(k.reshape(seq, heads, hd), case["wk"], case["cos"], case["sin"], case["eps"], 0).reshape(seq, dim)
    rows = g["rows"]
    assert np.abs(qn[rows] - g["q_rows"]).max() <= 1e-5 and np.abs(kn[rows] - g["k_rows"]).max() <= 1e-5
    out = orc.attention_flash(qn, kn, v, heads, case["scale"])
    assert np.abs(out[rows] - g["out_rows"]).max() <= 1e-4
    np.testing.assert_allclose([out.astype(np.float64).sum(), np.abs(out).astype(np.float64).sum()], g["out_checksum"], rtol=1e-5)
    # the strided routine the GPU tests compare with, on the same rows
    strided = orc.attention_strided(qn, kn, v, heads, heads, case["scale"])
    assert np.abs(strided[rows] - g["out_rows"]).max() <= 1e-4
