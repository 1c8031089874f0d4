"""Writes tests/golden/ref_vectors.npz from the reference's own C code
compiled in place (oracle/_ref, built by `make -C oracle ref`). Run in the
container that holds the reference tree:

    python tests/golden/make_golden.py

The file holds inputs' seeds/shapes and the reference's outputs only (data,
no reference text). Tables, ids and RNG draws come from the IEEE build of the
reference sources (bit-exact targets); attention / norm / rope outputs come
from the build with the reference Makefile's flags (tolerance targets).
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import oracle  # noqa: E402
import refcalls as R  # noqa: E402


def inputs(seed, *shape):
    """Deterministic inputs shared with the test: numpy PCG64 normal draws."""
    return np.random.default_rng(seed).standard_normal(shape).astype(np.float32)


def main():
    ref, refi = oracle.reference(), oracle.reference(ieee=True)
    assert ref is not None and refi is not None, "build oracle/_ref first"
    g = {}
    # --- seeded inputs
    for seed in (0, 1, 42):
        g[f"rng_uniform_{seed}"] = R.rng_u64(refi, seed, 32)
        g[f"rng_normal_{seed}"] = R.randn(refi, seed, 256)
    # --- tables (bit-exact targets)
    g["flux2_cos"], g["flux2_sin"] = R.flux2_joint_compact(refi, 8, 4, 5, [(2, 3), (3, 2)])
    g["flux3_cos"], g["flux3_sin"] = R.flux3_joint_rope(refi, 8, 4, 5, [(2, 3), (3, 2)])
    g["qwen3_cos"], g["qwen3_sin"] = R.qwen3_rope_table(refi, 24, 128, 1e6)
    mask = np.r_[np.ones(15), np.zeros(9)].astype(np.int32)
    g["qwen3_f3_cos"], g["qwen3_f3_sin"] = R.qwen3_rope_table(refi, 24, 128, 1e6, mask=mask, flux3_mode=True)
    for ax, (d, n) in enumerate(((32, 40), (48, 40), (48, 40))):
        g[f"zimage_cos_{ax}"], g[f"zimage_sin_{ax}"] = R.zi_axis_table(refi, ax, (32, 48, 48), (n, n, n))
    g["rope_freqs"] = R.rope_freqs(refi, [0, 1, 7, 300], 128, 10000.0)
    # --- f32 operators (tolerance targets)
    x = inputs(100, 6, 3, 128)
    w = (1 + 0.02 * inputs(101, 128)).astype(np.float32)
    g["head_rms_norm"] = R.flux3_head_rms_norm(ref, x, w, 1e-6)
    g["rope_pairs"] = R.flux3_apply_rope(ref, x[:6], g["flux2_cos"][8:14], g["flux2_sin"][8:14])
    q4 = x[None]
    fr = R.rope_freqs(refi, np.arange(6), 128, 1e6)
    g["rope_split"] = R.apply_rope_interleaved(ref, q4, fr)[0]
    g["softmax"] = R.softmax_rows(ref, inputs(102, 5, 37) * 4)
    for name, (sq, sk) in {"small": (5, 9), "edge": (64, 128), "tiled": (65, 129)}.items():
        Q, K, V = inputs(110, sq, 64), inputs(111, sk, 64), inputs(112, sk, 64)
        g[f"flash_{name}"] = R.attention_flash(ref, Q, K, V, 2, 1 / np.sqrt(32))
    # Z-Image masked chain and Qwen3 causal GQA chain (see test for the inputs)
    orc = oracle.oracle()
    dims = (8, 12, 12)
    pos, zmask, ip, cp = orc.zimage_positions(img_seq=27, wt=9, cap_seq=5)
    seq, dim = ip + cp, 64
    g["zi_attention"] = R.zi_attention(ref, inputs(120, seq, dim), inputs(121, dim, dim) / 8, inputs(122, dim, dim) / 8,
                                       inputs(123, dim, dim) / 8, np.eye(dim, dtype=np.float32),
                                       1 + 0.02 * inputs(124, 32), 1 + 0.02 * inputs(125, 32), pos, zmask, 2, dims)
    g["zi_pos"], g["zi_mask"] = pos, zmask
    heads, kv, hd, hidden, seq = 8, 2, 32, 24, 40
    qmask = np.r_[np.ones(23), np.zeros(17)].astype(np.int32)
    attn, rq, rk, rv = R.qwen3_attention(ref, inputs(130, seq, hidden), inputs(131, heads * hd, hidden) / 5,
                                         inputs(132, kv * hd, hidden) / 5, inputs(133, kv * hd, hidden) / 5,
                                         1 + 0.02 * inputs(134, hd), 1 + 0.02 * inputs(135, hd), qmask, heads, kv, hd)
    g["qwen3_attention"], g["qwen3_q"], g["qwen3_k"] = attn, rq, rk
    # --- the other device operators: outputs of the reference's CPU twins (NCHW there; the test transposes)
    import ctypes as C
    P = lambda a: a.ctypes.data_as(C.c_void_p)
    xl = oracle.bf16_to_f32(oracle.f32_to_bf16(inputs(140, 7, 96)))
    Wl = oracle.f32_to_bf16(inputs(141, 33, 96) * 0.1)
    yl = np.empty((7, 33), np.float32)
    refi.lib.iris_linear_nobias_bf16(P(yl), P(np.ascontiguousarray(xl)), P(Wl), C.c_int(7), C.c_int(96), C.c_int(33))
    g["ops_linear"] = yl
    xs = inputs(142, 500) * 3
    ys = xs.copy()
    refi.lib.iris_silu(P(ys), C.c_int(ys.size))
    g["ops_silu"] = ys
    h, w, cin, cout, k = 6, 5, 8, 4, 3
    img = oracle.bf16_to_f32(oracle.f32_to_bf16(inputs(143, h * w, cin)))
    wt = oracle.bf16_to_f32(oracle.f32_to_bf16(inputs(144, cout, k * k * cin) * 0.2))
    bias = inputs(145, cout)
    x_nchw = np.ascontiguousarray(img.reshape(h, w, cin).transpose(2, 0, 1))
    w_nchw = np.ascontiguousarray(wt.reshape(cout, k, k, cin).transpose(0, 3, 1, 2))
    yc = np.empty((cout, h, w), np.float32)
    refi.lib.iris_conv2d(P(yc), P(x_nchw), P(w_nchw), P(bias), C.c_int(1), C.c_int(cin), C.c_int(cout), C.c_int(h), C.c_int(w),
                         C.c_int(k), C.c_int(k), C.c_int(1), C.c_int(1))
    g["ops_conv2d"] = np.ascontiguousarray(yc.transpose(1, 2, 0).reshape(h * w, cout))
    gimg, gamma, beta = inputs(146, 30, 16) * 2 + 0.5, 1 + 0.1 * inputs(147, 16), 0.1 * inputs(148, 16)
    yg = np.empty((16, 30), np.float32)
    refi.lib.iris_group_norm(P(yg), P(np.ascontiguousarray(gimg.T)), P(gamma.astype(np.float32)), P(beta.astype(np.float32)),
                             C.c_int(1), C.c_int(16), C.c_int(5), C.c_int(6), C.c_int(4), C.c_float(1e-6))
    g["ops_group_norm"] = np.ascontiguousarray(yg.T)
    uimg = inputs(149, 12, 5)
    yu = np.empty((5, 6, 8), np.float32)
    refi.lib.iris_upsample_nearest(P(yu), P(np.ascontiguousarray(uimg.T)), C.c_int(1), C.c_int(5), C.c_int(3), C.c_int(4), C.c_int(2), C.c_int(2))
    g["ops_upsample2x"] = np.ascontiguousarray(yu.reshape(5, 48).T)
    out = os.path.join(HERE, "ref_vectors.npz")
    np.savez_compressed(out, **g)
    print("wrote", out, os.path.getsize(out), "bytes,", len(g), "arrays")
    c1_chain(ref, refi)


C1_ROWS = [0, 1, 17, 31, 32, 63, 64, 65, 79, 80, 127, 128, 159, 191, 192, 200, 255, 256, 257, 300, 318, 319]


def c1_chain(ref, refi):
    """The metric's own chain at head_dim 128, configuration C1 at full shape (24 heads x 128, 64 text + 16 x 16
    image tokens), through the reference's compiled code: apply_qk_norm -> apply_rope_2d on Q and on K ->
    iris_flash_attention (iris_transformer_flux.c:1289-1343, 952-974, iris_kernels.c:899-991). The inputs are the
    seeded draws of tests/workloads.py:c1 (generator bit-exact with the reference's, checked here), rounded to bf16 and
    taken as f32; the tables are the reference's own full [seq, 128] tables. Stored: the reference's Q and K after
    norm + rope and its attention output, on C1_ROWS (both streams, both sides of the text / image boundary)."""
    import workloads as W
    case = W.c1()
    seq, heads, hd, dim = case["seq"], 24, 128, 3072
    st_check = R.randn(refi, W.SEED0 + 1, 512)
    orc = oracle.oracle()
    assert np.array_equal(st_check.view(np.uint32), orc.randn(orc.rng(W.SEED0 + 1), 512).view(np.uint32))
    f = oracle.bf16_to_f32(case["buf"])
    q, k, v = (np.ascontiguousarray(f[:, i * dim:(i + 1) * dim]) for i in range(3))
    ct, st = R.flux2_rope_text(refi, 64)
    ci, si = R.flux2_rope_2d(refi, 16, 16)
    cos_full, sin_full = np.concatenate([ct, ci]), np.concatenate([st, si])
    assert np.array_equal(np.ascontiguousarray(cos_full[:, 0::2]).view(np.uint32), case["cos"].view(np.uint32))
    qn, kn = R.flux2_qk_norm(ref, q.reshape(seq, heads, hd), k.reshape(seq, heads, hd), case["wq"], case["wk"], case["eps"])
    qr = R.flux2_apply_rope_2d(ref, qn, cos_full, sin_full).reshape(seq, dim)
    kr = R.flux2_apply_rope_2d(ref, kn, cos_full, sin_full).reshape(seq, dim)
    o = R.attention_flash(ref, qr, kr, v, heads, case["scale"])
    rows = np.array(C1_ROWS)
    out = os.path.join(HERE, "c1_chain.npz")
    np.savez_compressed(out, rows=rows, q_rows=qr[rows], k_rows=kr[rows], out_rows=o[rows],
                        out_checksum=np.array([np.float64(o.astype(np.float64).sum()), np.float64(np.abs(o).astype(np.float64).sum())]))
    print("wrote", out, os.path.getsize(out), "bytes")


if __name__ == "__main__":
    main()
