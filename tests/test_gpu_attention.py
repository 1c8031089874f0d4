"""iris_dev_attention on the GPU (through the C ABI) against the fp32 CPU
oracle on identical bf16 inputs. Bar: max-abs <= 2e-2, mean-abs <= 2e-3, and
relative to the expected values max-abs <= 4e-2 max|want|, mean-abs <= 1e-2
mean|want| (gpu_harness.assert_parity), so that small outputs are held as
tightly as large ones.
"""
import numpy as np
import pytest

import oracle as O
import workloads as W
from gpu_harness import Dev, error_stats, assert_parity, MAX_ABS, MEAN_ABS

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    return Dev()


@pytest.fixture
def fa():
    """Name of the matrix-core kernel every head_dim-128, aligned call must take."""
    return "fa_hd128"


def gpu_attention(dev, case, **over):
    a = dict(case); a.update(over)
    out, kernel = dev.attention(a["buf"], a["ldi"], 0, a["q_dim"], a["q_dim"] + a["kv_dim"], a["seq"], a["seq"],
                                a["heads"], a["kv_heads"], 128, a["scale"], a["causal"], a["key_mask"], ldo=a["ldo"])
    return O.bf16_to_f32(out[:, :a["q_dim"]]), kernel


def cpu_attention(orc, case, rows=None):
    return orc.attention_bf16(case["buf"], case["ldi"], 0, case["q_dim"], case["q_dim"] + case["kv_dim"], case["seq"],
                              case["seq"], case["heads"], case["kv_heads"], 128, case["scale"], case["causal"],
                              case["key_mask"], rows=rows)


def assert_close(got, want, what="", **kw):
    """max-abs <= 2e-2 and mean-abs <= 2e-3, and both small against the expected values themselves."""
    return assert_parity(got, want, what, **kw)


def after_norm_rope(dev, case):
    """The caller's sequence: norm+rope on Q, on K, then attention."""
    buf = dev.norm_rope_qk(case["buf"], case["ldi"], 0, case["q_dim"], case["wq"], case["wk"], case["cos"], case["sin"],
                           case["seq"], case["heads"], case["kv_heads"], 128, case["eps"], case["split_half"])
    out = dict(case); out["buf"] = buf
    return out


# ------------------------------------------------------------------ the five configurations, shrunk
def test_c1_plumbing_full_size(dev, orc, fa):
    case = after_norm_rope(dev, W.c1())           # 64 text + 16x16 image, 24 heads
    got, kernel = gpu_attention(dev, case)
    assert kernel == fa
    assert_close(got, cpu_attention(orc, case), "C1")
    # and against the reference-shaped f32 flash attention on the same inputs
    f = O.bf16_to_f32(case["buf"])
    flash = orc.attention_flash(f[:, :3072], f[:, 3072:6144], f[:, 6144:], 24, case["scale"])
    assert_close(got, flash, "C1 vs flash")


def test_c1_against_the_vector_the_compiled_reference_wrote(dev, fa):
    """C1 at full shape (24 x 128, 64 text + 256 image tokens): norm + rope on Q and K, then attention, on the GPU,
    against the output rows that the reference's own compiled apply_qk_norm -> apply_rope_2d ->
    iris_flash_attention produced from the same seeded inputs (tests/golden/c1_chain.npz, written by
    tests/golden/make_golden.py where the reference tree is present). The stated bar of the bf16 path."""
    import os
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "c1_chain.npz"), allow_pickle=False)
    case = after_norm_rope(dev, W.c1())
    got, kernel = gpu_attention(dev, case)
    assert kernel == fa
    assert_close(got[g["rows"]], g["out_rows"], "C1 vs the reference's vector")
    # the same with Q normalised inside the attention kernel
    raw = W.c1()
    buf = dev.norm_rope(raw["buf"], raw["ldi"], 3072, raw["wk"], raw["cos"], raw["sin"], raw["seq"], 24, 128, raw["eps"], 0)
    out, kernel, _ = dev.attention_qnorm(buf, raw["ldi"], 0, 3072, 6144, raw["seq"], raw["seq"], 24, 24, 128, raw["scale"],
                                         raw["wq"], raw["cos"], raw["sin"], raw["eps"], 0)
    assert kernel == "fa_hd128_qnorm"
    assert_close(O.bf16_to_f32(out)[g["rows"]], g["out_rows"], "C1 (Q norm inside attention) vs the reference's vector")


@pytest.mark.parametrize("maker,shrink", [(W.c2, 8), (W.c5, 32)])
def test_joint_attention_shrunk(dev, orc, fa, maker, shrink):
    case = after_norm_rope(dev, maker(shrink))
    got, kernel = gpu_attention(dev, case)
    assert kernel == fa
    assert_close(got, cpu_attention(orc, case), case["name"])


def test_c3_cfg_pair_with_key_mask(dev, orc, fa):
    for case in W.c3(shrink=8):
        case = after_norm_rope(dev, case)
        got, kernel = gpu_attention(dev, case)
        assert kernel == fa
        assert_close(got, cpu_attention(orc, case), case["name"])


@pytest.mark.parametrize("shrink", [1, 4])
def test_c4_causal_gqa_padding(dev, orc, fa, shrink):
    case = after_norm_rope(dev, W.c4(shrink))
    got, kernel = gpu_attention(dev, case)
    assert kernel == fa
    assert_close(got, cpu_attention(orc, case), "C4")


# ------------------------------------------------------------------ full sizes: sampled rows + properties
def sample_rows(seq, n=40, seed=0):
    rng = np.random.default_rng(seed)
    fixed = [0, 1, 127, 128, 511, 512, seq // 2, seq - 129, seq - 128, seq - 1]
    return np.unique(np.r_[fixed, rng.integers(0, seq, n)]).astype(np.int32)


def test_c2_full_size_sampled_rows_and_properties(dev, orc):
    case = after_norm_rope(dev, W.c2())
    got, kernel = gpu_attention(dev, case)
    assert kernel == "fa_hd128"
    rows = sample_rows(case["seq"])
    assert_close(got[rows], cpu_attention(orc, case, rows=rows), "C2 sampled")
    # key-permutation invariance (non-causal): shuffle K/V rows together
    perm = np.random.default_rng(1).permutation(case["seq"])
    shuf = case["buf"].copy()
    shuf[:, 3072:] = case["buf"][perm][:, 3072:]
    got2, _ = gpu_attention(dev, case, buf=shuf)
    assert_close(got2, got, "C2 permuted keys")
    # constant V -> every output row equals that V row
    const = case["buf"].copy()
    const[:, 6144:] = case["buf"][7, 6144:]
    got3, _ = gpu_attention(dev, case, buf=const)
    want = np.tile(O.bf16_to_f32(case["buf"][7, 6144:]), (case["seq"], 1))
    assert_close(got3, want, "C2 constant V")


@pytest.mark.parametrize("seq,heads,kv,causal,masked", [
    (200, 6, 6, False, False), (200, 6, 2, True, True),              # 78 waves of 16 queries: one-wave workgroups
    (40, 40, 10, False, False), (60, 48, 12, True, True),            # one key tile
    (330, 24, 24, False, False), (300, 24, 8, True, True),           # two waves of 16 queries per workgroup
    (600, 16, 4, False, True), (600, 16, 16, True, False),           # four
    (1300, 16, 16, False, False), (1300, 16, 8, True, True),         # eight
    (2100, 24, 8, False, True), (2100, 24, 24, True, False),         # 32 queries per wave: 128- or 256-query workgroups
    (4200, 8, 8, False, False), (1500, 24, 24, False, True),
    (4608, 24, 24, False, True), (8704, 24, 8, False, False),        # workgroups of two sizes: 256 queries, then 192
])
def test_every_workgroup_width(dev, orc, seq, heads, kv, causal, masked):
    """The launcher picks the workgroup from the problem size: 1, 2, 4 or 8 waves of 16 queries for up to 2048 such
    waves, 4 or 8 waves of 32 queries beyond, the last ones of a head with 32 and 16 queries per wave when that evens
    out the last round (or, for few workgroups and many key tiles, the kernel that splits the keys over the waves);
    each shape is its own instantiation of the kernel (pieces of a key tile per wave, LDS stages).
    Sampled rows against the oracle, including the rows around every workgroup boundary."""
    rng = np.random.default_rng(seq + heads)
    ldi = (heads + 2 * kv) * 128
    buf = O.f32_to_bf16(rng.standard_normal((seq, ldi)).astype(np.float32))
    mask = None
    if masked:
        mask = (rng.random(seq) < 0.7).astype(np.int32)
        mask[0] = 1                                                     # every causal row keeps a valid key
    case = W._case(buf=buf, heads=heads, kv_heads=kv, causal=causal, key_mask=mask)
    case["ldo"] = heads * 128
    got, kernel = gpu_attention(dev, case)
    assert kernel == "fa_hd128"
    rows = np.unique(np.r_[sample_rows(seq, n=24, seed=seq), [31, 32, 63, 64, 255, 256 % seq, seq - 33, seq - 32]]).astype(np.int32)
    rows = rows[(rows >= 0) & (rows < seq)]
    assert_close(got[rows], cpu_attention(orc, case, rows=rows), f"seq {seq} heads {heads}/{kv}")


@pytest.mark.parametrize("seq,heads,kv,causal,valid", [
    (512, 32, 8, True, 40), (512, 32, 8, True, 1), (512, 32, 8, False, 65),        # a short prompt padded to 512
    (2100, 24, 8, False, 130), (2100, 24, 24, True, 700), (4608, 24, 24, False, 4113),
])
def test_padding_behind_the_last_valid_key_is_not_walked(dev, orc, seq, heads, kv, causal, valid):
    """A key mask that is a prefix (a prompt padded to a fixed length): the kernel stops at the last key tile that
    holds a valid key. Same results as the oracle, which walks every key; padded query rows included."""
    rng = np.random.default_rng(seq + valid)
    ldi = (heads + 2 * kv) * 128
    buf = O.f32_to_bf16(rng.standard_normal((seq, ldi)).astype(np.float32))
    mask = (np.arange(seq) < valid).astype(np.int32)
    case = W._case(buf=buf, heads=heads, kv_heads=kv, causal=causal, key_mask=mask)
    case["ldo"] = heads * 128
    got, kernel = gpu_attention(dev, case)
    assert kernel == "fa_hd128"
    rows = np.unique(np.r_[sample_rows(seq, n=24, seed=valid), [valid - 1, valid % seq, 63, 64]]).astype(np.int32)
    rows = rows[(rows >= 0) & (rows < seq)]
    assert_close(got[rows], cpu_attention(orc, case, rows=rows), f"seq {seq}, {valid} valid keys")


def test_very_long_masked_key_sequence_takes_the_generic_kernel(dev, orc):
    """The matrix-core kernel keeps the key mask in LDS, one bit per key, which bounds a masked
    seq_k at 250000; beyond that the call must still be answered (by the generic kernel)."""
    seq_k, seq_q, ldi = 250_001, 2, 256                    # q in columns 0..127 of the first rows, k = v in 128..255
    rng = np.random.default_rng(77)
    buf = O.f32_to_bf16((rng.integers(-8, 9, (seq_k, ldi)) / 8).astype(np.float32))
    mask = (rng.random(seq_k) < 0.5).astype(np.int32)
    out, kernel = dev.attention(buf, ldi, 0, 128, 128, seq_q, seq_k, 1, 1, 128, 0.09, False, mask, ldo=128)
    assert kernel == "attention_generic"
    want = orc.attention_bf16(buf, ldi, 0, 128, 128, seq_q, seq_k, 1, 1, 128, 0.09, False, mask)
    assert_close(O.bf16_to_f32(out), want, "250001 masked keys")
    # one key fewer than the limit still runs on the matrix cores
    out, kernel = dev.attention(buf, ldi, 0, 128, 128, seq_q, 249_984, 1, 1, 128, 0.09, False, mask[:249_984], ldo=128)
    assert kernel == "fa_hd128"
    want = orc.attention_bf16(buf, ldi, 0, 128, 128, seq_q, 249_984, 1, 1, 128, 0.09, False, mask[:249_984])
    assert_close(O.bf16_to_f32(out), want, "249984 masked keys")


def test_long_sequence_offsets(dev, orc):
    """40000 tokens: row offsets beyond 2^31 bytes into the fused buffer must not wrap."""
    seq, heads = 40_000, 2
    ldi = 3 * heads * 128 + 26_000                           # wide rows: 40000 x 26768 x 2 B = 2.1 GB
    ldi -= ldi % 8
    rng = np.random.default_rng(9)
    buf = np.zeros((seq, ldi), np.uint16)
    buf[:, :3 * heads * 128] = O.f32_to_bf16(rng.standard_normal((seq, 3 * heads * 128)).astype(np.float32))
    case = W._case(buf=buf, heads=heads, kv_heads=heads)
    case["ldo"] = heads * 128
    got, kernel = gpu_attention(dev, case)
    assert kernel == "fa_hd128"
    rows = np.array([0, 1, 255, 19_999, 39_000, 39_999], np.int32)
    assert_close(got[rows], cpu_attention(orc, case, rows=rows), "40000 tokens, 2.1 GB of rows")


def test_c5_full_size_sampled_rows(dev, orc):
    case = after_norm_rope(dev, W.c5())           # 12800 tokens
    got, kernel = gpu_attention(dev, case)
    assert kernel == "fa_hd128"
    rows = sample_rows(case["seq"], n=20)
    assert_close(got[rows], cpu_attention(orc, case, rows=rows), "C5 sampled")


def test_c3_cond_full_size_sampled_rows(dev, orc, fa):
    """The conditional half of the Z-Image pair at full size: 30 heads, 4096 image + 256 caption tokens, no mask."""
    cond, _ = W.c3()
    cond = after_norm_rope(dev, cond)
    got, kernel = gpu_attention(dev, cond)
    assert kernel == fa
    rows = sample_rows(cond["seq"], n=20)
    assert_close(got[rows], cpu_attention(orc, cond, rows=rows), "C3 cond sampled")


def test_c3_full_size_masked_equals_compacted(dev, orc, fa):
    cond, unc = W.c3()
    unc = after_norm_rope(dev, unc)
    got, kernel = gpu_attention(dev, unc)
    assert kernel == fa
    rows = sample_rows(unc["seq"], n=20)
    assert_close(got[rows], cpu_attention(orc, unc, rows=rows), "C3 uncond sampled")
    # masked keys == the same problem with those K/V rows removed
    keep = np.nonzero(unc["key_mask"])[0]
    small = dict(unc); small["buf"] = np.ascontiguousarray(unc["buf"][keep]); small["seq"] = keep.size; small["key_mask"] = None
    got_small, _ = gpu_attention(dev, small)
    assert_close(got[keep], got_small, "C3 masked vs compacted")


# ------------------------------------------------------------------ edge cases
@pytest.mark.parametrize("seq_q,seq_k,heads,kv,causal,masked", [
    (77, 400, 8, 2, False, True),          # seven key tiles over four waves: three waves take two tiles
    (40, 130, 3, 3, False, False),         # three tiles: below the length where the split pays, one wave walks them
    (500, 500, 4, 2, True, True),          # causal: the waves of the first query blocks have no tile at all
    (1000, 1000, 2, 2, True, True),        # four tiles per wave: the masks of the later ones are read in the loop
    (33, 3000, 1, 1, False, True),         # twelve turns per wave, ragged last tile
    (512, 512, 8, 8, False, False),        # 128 workgroups x 4 waves
])
def test_keys_split_over_the_waves_of_a_workgroup(dev, orc, seq_q, seq_k, heads, kv, causal, masked):
    """Few (head, 32-query block) pairs and more than one key tile: every wave of a workgroup takes every S-th
    key tile of the same queries and the partial results are merged at the end. All rows against the oracle."""
    rng = np.random.default_rng(seq_q + seq_k)
    buf, ldi = random_case(seq_q * 3 + seq_k, seq_q, seq_k, heads, kv)
    qd, kd = heads * 128, kv * 128
    mask = None
    if masked:
        mask = (rng.random(seq_k) < 0.7).astype(np.int32)
        mask[0] = 1
        mask[64:128] = 0                       # a whole tile without a valid key: that wave's partial result is empty
    out, kernel = dev.attention(buf, ldi, 0, qd, qd + kd, seq_q, seq_k, heads, kv, 128, 0.0884, causal, mask)
    assert kernel == "fa_hd128"
    want = orc.attention_bf16(buf, ldi, 0, qd, qd + kd, seq_q, seq_k, heads, kv, 128, 0.0884, causal, mask)
    assert_close(O.bf16_to_f32(out[:seq_q]), want, f"{seq_q}x{seq_k} heads {heads}/{kv} causal={causal} masked={masked}")


def test_split_keys_with_rows_that_have_no_valid_key(dev, orc):
    """Rows whose every key is masked give zeros from the merge as well (all partial maxima are -inf)."""
    seq, heads = 300, 2
    buf, ldi = random_case(9, seq, seq, heads, heads)
    mask = np.zeros(seq, np.int32)
    mask[200:] = 1                               # causal rows 0 .. 199 see no valid key
    out, kernel = dev.attention(buf, ldi, 0, heads * 128, 2 * heads * 128, seq, seq, heads, heads, 128, 0.0884, True, mask)
    got = O.bf16_to_f32(out)
    assert np.all(got[:200] == 0.0) and np.isfinite(got).all()
    want = orc.attention_bf16(buf, ldi, 0, heads * 128, 2 * heads * 128, seq, seq, heads, heads, 128, 0.0884, True, mask)
    assert_close(got[200:], want[200:], "rows behind the empty ones")     # (the fp32 CPU attention has no zero-row rule)


def random_case(seed, seq_q, seq_k, heads, kv_heads, hd=128, pad=0, sigma=1.0):
    rng = np.random.default_rng(seed)
    seq = max(seq_q, seq_k)
    ldi = (heads + 2 * kv_heads) * hd + pad
    buf = O.f32_to_bf16(rng.standard_normal((seq, ldi)).astype(np.float32) * sigma)
    return buf, ldi


@pytest.mark.parametrize("seq_q,seq_k", [(1, 1), (1, 64), (5, 63), (33, 65), (128, 128), (129, 191), (200, 31), (257, 1000)])
@pytest.mark.parametrize("causal", [False, True])
def test_ragged_shapes(dev, orc, fa, seq_q, seq_k, causal):
    heads, kv = 4, 2
    buf, ldi = random_case(seq_q * 7 + seq_k, seq_q, seq_k, heads, kv)
    qd, kd = heads * 128, kv * 128
    out, kernel = dev.attention(buf, ldi, 0, qd, qd + kd, seq_q, seq_k, heads, kv, 128, 0.0884, causal)
    assert kernel == fa
    want = orc.attention_bf16(buf, ldi, 0, qd, qd + kd, seq_q, seq_k, heads, kv, 128, 0.0884, causal)
    assert_close(O.bf16_to_f32(out[:seq_q]), want, f"{seq_q}x{seq_k} causal={causal}")


@pytest.mark.parametrize("seq_q,seq_k,heads,kv", [(3000, 5000, 24, 24), (5000, 3000, 16, 4), (2817, 70, 24, 8)])
def test_large_calls_with_different_query_and_key_counts(dev, orc, fa, seq_q, seq_k, heads, kv):
    """The workgroups are cut by the number of queries alone (one size, or 256 queries then 192); the keys only set the
    length of the walk. Sampled query rows against the oracle, with the last rows of both workgroup sizes among them."""
    buf, ldi = random_case(seq_q + seq_k, seq_q, seq_k, heads, kv)
    qd, kd = heads * 128, kv * 128
    out, kernel = dev.attention(buf, ldi, 0, qd, qd + kd, seq_q, seq_k, heads, kv, 128, 0.0884, False)
    assert kernel == fa
    rows = np.unique(np.r_[sample_rows(seq_q, n=30, seed=seq_k), [255, 256, 447, 448, seq_q - 193, seq_q - 192, seq_q - 65, seq_q - 64]])
    rows = rows[(rows >= 0) & (rows < seq_q)].astype(np.int32)
    want = orc.attention_bf16(buf, ldi, 0, qd, qd + kd, seq_q, seq_k, heads, kv, 128, 0.0884, False, None, rows=rows)
    assert_close(O.bf16_to_f32(out[:seq_q])[rows], want, f"{seq_q} queries x {seq_k} keys")


def test_random_key_masks_and_empty_rows(dev, orc, fa):
    heads, seq = 3, 300
    buf, ldi = random_case(5, seq, seq, heads, heads)
    rng = np.random.default_rng(6)
    mask = (rng.random(seq) < 0.5).astype(np.int32)
    out, _ = dev.attention(buf, ldi, 0, 384, 768, seq, seq, heads, heads, 128, 0.0884, False, mask)
    want = orc.attention_bf16(buf, ldi, 0, 384, 768, seq, seq, heads, heads, 128, 0.0884, False, mask)
    assert_close(O.bf16_to_f32(out), want, "random mask")
    # causal + mask whose first valid key is 10: queries 0..9 have no valid key -> zero rows
    mask2 = np.ones(seq, np.int32); mask2[:10] = 0
    out, _ = dev.attention(buf, ldi, 0, 384, 768, seq, seq, heads, heads, 128, 0.0884, True, mask2)
    got = O.bf16_to_f32(out)
    assert np.all(got[:10] == 0.0)
    want = orc.attention_bf16(buf, ldi, 0, 384, 768, seq, seq, heads, heads, 128, 0.0884, True, mask2)
    assert_close(got[10:], want[10:], "causal + mask")
    # all keys masked -> all-zero output
    out, _ = dev.attention(buf, ldi, 0, 384, 768, seq, seq, heads, heads, 128, 0.0884, False, np.zeros(seq, np.int32))
    assert np.all(O.bf16_to_f32(out) == 0.0)


def test_large_scores_stay_finite(dev, orc, fa):
    heads, seq = 2, 130
    buf, ldi = random_case(9, seq, seq, heads, heads, sigma=6.0)     # |score| up to ~100
    out, _ = dev.attention(buf, ldi, 0, 256, 512, seq, seq, heads, heads, 128, 0.0884)
    got = O.bf16_to_f32(out)
    assert np.all(np.isfinite(got))
    want = orc.attention_bf16(buf, ldi, 0, 256, 512, seq, seq, heads, heads, 128, 0.0884)
    mx, mean = error_stats(got, want)
    assert mx <= 0.13 and mean <= 4e-3      # outputs are O(6): same relative bar as 2e-2 on O(1) values


def test_output_stride_and_interior_pointers(dev, orc, fa):
    heads, seq = 2, 70
    buf, ldi = random_case(11, seq, seq, heads, heads, pad=64)
    ldo, out_col = 2 * 256 + 8, 256
    out, kernel = dev.attention(buf, ldi, 0, 256, 512, seq, seq, heads, heads, 128, 0.0884, ldo=ldo, out_col=out_col)
    assert kernel == fa
    want = orc.attention_bf16(buf, ldi, 0, 256, 512, seq, seq, heads, heads, 128, 0.0884)
    assert_close(O.bf16_to_f32(out[:, out_col:out_col + 256]), want, "strided out")
    assert np.all(out[:, :out_col] == 0x7fc0) and np.all(out[:, out_col + 256:] == 0x7fc0)


@pytest.mark.parametrize("hd,heads,kv", [(512, 1, 1), (512, 2, 1), (256, 3, 3), (256, 4, 2)])
@pytest.mark.parametrize("seq_q,seq_k,causal,masked", [(150, 150, False, False), (1, 1, False, False), (33, 95, False, True),
                                                         (64, 64, True, False), (257, 257, True, True), (130, 1000, False, False)])
def test_wide_heads_256_512(dev, orc, hd, heads, kv, seq_q, seq_k, causal, masked):
    """head_dim 256 / 512 run on the matrix cores too (the VAE's single 512-wide head; with key mask and causal limit
    too), in the kernel whose waves own whole queries."""
    buf, ldi = random_case(hd + heads + seq_q, seq_q, seq_k, heads, kv, hd=hd)
    qd, kd = heads * hd, kv * hd
    mask = None
    if masked:
        mask = (np.random.default_rng(seq_k).random(seq_k) < 0.6).astype(np.int32)
        mask[0] = 1                                        # every causal row keeps a valid key
    scale = float(1 / np.sqrt(hd))
    out, kernel = dev.attention(buf, ldi, 0, qd, qd + kd, seq_q, seq_k, heads, kv, hd, scale, causal, mask)
    assert kernel == f"fa_hd{hd}"
    want = orc.attention_bf16(buf, ldi, 0, qd, qd + kd, seq_q, seq_k, heads, kv, hd, scale, causal, mask)
    assert_close(O.bf16_to_f32(out[:seq_q]), want, f"wide hd={hd} {seq_q}x{seq_k}")


def test_vae_shape_full_size_sampled_rows(dev, orc):
    """One head of 512 over 4096 tokens (a 512x512 image's mid-block attention, reference
    iris_vae.c:1112-1124): sampled rows against the oracle, and constant V => constant output."""
    seq, hd = 4096, 512
    buf, ldi = random_case(77, seq, seq, 1, 1, hd=hd)
    scale = float(1 / np.sqrt(hd))
    out, kernel = dev.attention(buf, ldi, 0, hd, 2 * hd, seq, seq, 1, 1, hd, scale)
    assert kernel == "fa_hd512"
    rows = sample_rows(seq, n=20)
    want = orc.attention_bf16(buf, ldi, 0, hd, 2 * hd, seq, seq, 1, 1, hd, scale, rows=rows)
    assert_close(O.bf16_to_f32(out)[rows], want, "VAE shape sampled")
    const = buf.copy()
    const[:, 2 * hd:] = buf[5, 2 * hd:]
    out2, _ = dev.attention(const, ldi, 0, hd, 2 * hd, seq, seq, 1, 1, hd, scale)
    assert_close(O.bf16_to_f32(out2), np.tile(O.bf16_to_f32(buf[5, 2 * hd:]), (seq, 1)), "VAE shape constant V")


def test_vae_shape_at_its_largest_50176_tokens(dev, orc):
    """The largest image the reference decodes in one piece is 1792 x 1792: (1792 / 8)^2 = 50176 tokens through the
    mid-block attention (iris_vae.c:1112-1124), one head of 512. Sampled rows against the oracle (first and last
    workgroups, workgroup boundaries) and constant V over all rows."""
    seq, hd = 50176, 512
    buf, ldi = random_case(78, seq, seq, 1, 1, hd=hd)
    scale = float(1 / np.sqrt(hd))
    out, kernel = dev.attention(buf, ldi, 0, hd, 2 * hd, seq, seq, 1, 1, hd, scale)
    assert kernel == "fa_hd512"
    rows = np.unique(np.r_[sample_rows(seq, n=10), [127, 128, 25087, 25088, seq - 129, seq - 128]]).astype(np.int32)
    want = orc.attention_bf16(buf, ldi, 0, hd, 2 * hd, seq, seq, 1, 1, hd, scale, rows=rows)
    assert_close(O.bf16_to_f32(out[rows]), want, "VAE 50176 tokens sampled")
    buf[:, 2 * hd:] = buf[5, 2 * hd:]
    out2, _ = dev.attention(buf, ldi, 0, hd, 2 * hd, seq, seq, 1, 1, hd, scale)
    got2 = O.bf16_to_f32(out2)
    assert np.array_equal(got2, np.tile(got2[0], (seq, 1)))
    assert_close(got2[:4], np.tile(O.bf16_to_f32(buf[5, 2 * hd:]), (4, 1)), "VAE 50176 tokens constant V")


@pytest.mark.parametrize("hd", [128, 256, 512, 64])
@pytest.mark.parametrize("seq_q,seq_k", [(1, 1), (40, 5), (31, 31), (20, 33), (77, 77), (100, 1000), (700, 1027)])
@pytest.mark.parametrize("causal,masked", [(False, False), (True, True)])
def test_rows_behind_the_last_key_never_reach_the_output(dev, orc, hd, seq_q, seq_k, causal, masked):
    """The kernels load K and V in tiles of 32 or 64 whole rows; what a tile holds behind the last key must not count,
    and not by being multiplied with a zero probability either: the 48 rows that follow the last key in the buffer
    are NaN here (q, k and v columns alike), and every output stays finite and within the bar."""
    heads, kv = 2, 1
    buf, ldi = random_case(hd + 3 * seq_q + seq_k, seq_q, seq_k, heads, kv, hd=hd)
    padded = np.full((max(seq_q, seq_k) + 48, ldi), 0x7fc0, np.uint16)
    padded[:seq_q, :heads * hd] = buf[:seq_q, :heads * hd]
    padded[:seq_k, heads * hd:] = buf[:seq_k, heads * hd:]
    mask = None
    if masked:
        mask = (np.random.default_rng(seq_k).random(seq_k) < 0.7).astype(np.int32)
        mask[0] = 1
    scale = float(1 / np.sqrt(hd))
    qd, kd = heads * hd, kv * hd
    out, _ = dev.attention(padded, ldi, 0, qd, qd + kd, seq_q, seq_k, heads, kv, hd, scale, causal, mask)
    got = O.bf16_to_f32(out[:seq_q])
    assert np.all(np.isfinite(got)), f"NaN rows {np.unique(np.argwhere(~np.isfinite(got))[:, 0])[:8]}"
    want = orc.attention_bf16(np.ascontiguousarray(padded), ldi, 0, qd, qd + kd, seq_q, seq_k, heads, kv, hd, scale, causal, mask)
    assert_close(got, want, f"NaN behind the keys, hd {hd} {seq_q}x{seq_k}")


@pytest.mark.parametrize("seq,hd", [(30, 512), (100, 256), (19, 256)])
def test_wide_heads_empty_rows_and_large_scores(dev, orc, seq, hd):
    buf, ldi = random_case(21, seq, seq, 1, 1, hd=hd, sigma=3.0)          # |score| up to ~100
    scale = float(1 / np.sqrt(hd))
    mask = np.ones(seq, np.int32); mask[:10] = 0
    out, kernel = dev.attention(buf, ldi, 0, hd, 2 * hd, seq, seq, 1, 1, hd, scale, True, mask)
    assert kernel == f"fa_hd{hd}"
    got = O.bf16_to_f32(out)
    assert np.all(np.isfinite(got)) and np.all(got[:10] == 0.0)
    want = orc.attention_bf16(buf, ldi, 0, hd, 2 * hd, seq, seq, 1, 1, hd, scale, True, mask)
    mx, mean = error_stats(got[10:], want[10:])
    assert mx <= 0.07 and mean <= 4e-3      # outputs are O(3): same relative bar as 2e-2 on O(1) values


@pytest.mark.parametrize("hd,heads,kv,causal,masked", [(64, 4, 4, False, False), (64, 4, 2, True, True),
                                                       (384, 1, 1, False, False), (96, 2, 1, True, False),
                                                       (40, 3, 3, False, True), (2, 2, 1, False, False),
                                                       (130, 2, 2, True, True), (200, 4, 2, False, False)])
def test_other_head_dims_run_on_the_matrix_cores_through_a_padded_copy(dev, orc, hd, heads, kv, causal, masked):
    """Head sizes other than 128 / 256 / 512 (odd ones included): q, k and v are copied into a fused row
    buffer with every head padded with zeros to the next of those sizes, the matrix-core kernel of that
    size runs on the copy, and the first head_dim output columns of every head are copied back."""
    seq = 150
    buf, ldi = random_case(hd + heads, seq, seq, heads, kv, hd=hd)
    qd, kd = heads * hd, kv * hd
    mask = None
    if masked:
        mask = (np.arange(seq) < 101).astype(np.int32)
    scale = 1 / np.sqrt(hd)
    ldo = heads * hd + 3
    out, kernel = dev.attention(buf, ldi, 0, qd, qd + kd, seq, seq, heads, kv, hd, scale, causal, mask, ldo=ldo)
    wide = "fa_hd512_packed" if hd > 256 else "fa_hd256_packed"
    assert kernel == ("fa_hd128_packed" if hd <= 128 else wide)
    want = orc.attention_bf16(buf, ldi, 0, qd, qd + kd, seq, seq, heads, kv, hd, scale, causal, mask)
    assert_close(O.bf16_to_f32(out[:, :heads * hd]), want, f"padded copy hd={hd}")
    assert np.all(out[:, heads * hd:] == 0x7fc0)              # nothing written past the head columns


@pytest.mark.parametrize("hd,pad,qoff", [(128, 3, 0), (128, 0, 1), (512, 5, 0), (256, 8, 3)])
def test_misaligned_rows_run_on_the_matrix_cores_through_an_aligned_copy(dev, orc, hd, pad, qoff):
    """A row stride that is not a multiple of 8 elements, or q / k / v that do not start on 16 bytes."""
    heads, seq = 2, 70
    buf, ldi = random_case(13 + hd + pad, seq, seq, heads, heads, hd=hd, pad=pad + qoff)
    qd = heads * hd
    scale = float(1 / np.sqrt(hd))
    out, kernel = dev.attention(buf, ldi, qoff, qoff + qd, qoff + 2 * qd, seq, seq, heads, heads, hd, scale)
    assert kernel == {128: "fa_hd128_packed", 256: "fa_hd256_packed", 512: "fa_hd512_packed"}[hd]
    want = orc.attention_bf16(buf, ldi, qoff, qoff + qd, qoff + 2 * qd, seq, seq, heads, heads, hd, scale)
    assert_close(O.bf16_to_f32(out), want, f"misaligned hd={hd} pad={pad} offset={qoff}")


def test_padded_copy_with_fewer_queries_than_keys_and_large_sizes(dev, orc):
    """seq_q != seq_k (the fused copy has max(seq_q, seq_k) rows) and a size where the copy is grown."""
    for seq_q, seq_k, hd, heads, kv in ((45, 333, 64, 4, 2), (700, 90, 96, 2, 2), (2000, 2000, 64, 8, 8)):
        buf, ldi = random_case(seq_q + seq_k, seq_q, seq_k, heads, kv, hd=hd)
        qd, kd = heads * hd, kv * hd
        scale = float(1 / np.sqrt(hd))
        out, kernel = dev.attention(buf, ldi, 0, qd, qd + kd, seq_q, seq_k, heads, kv, hd, scale)
        assert kernel == "fa_hd128_packed"
        rows = sample_rows(seq_q, n=12) if seq_q > 300 else np.arange(seq_q, dtype=np.int32)
        rows = rows[(rows >= 0) & (rows < seq_q)]
        want = orc.attention_bf16(buf, ldi, 0, qd, qd + kd, seq_q, seq_k, heads, kv, hd, scale, rows=rows)
        assert_close(O.bf16_to_f32(out[:seq_q])[rows], want, f"padded copy {seq_q}x{seq_k}")


@pytest.mark.parametrize("hd,heads,kv,causal", [(640, 2, 1, True), (1024, 1, 1, False), (2048, 1, 1, False), (1100, 2, 2, False),
                                                (2050, 1, 1, True), (2304, 2, 1, False), (5000, 1, 1, False)])
def test_head_dims_beyond_512_on_the_scalar_kernel(dev, orc, hd, heads, kv, causal):
    """The reference answers any head_dim (its fallback is two GEMMs, iris_cuda.cu:897-936); here sizes beyond the
    matrix-core kernels' 512 go to the scalar kernel, which walks the dims in chunks of 512: up to 2048 with the
    workgroup's queries in the LDS, beyond that reading them from global memory. No limit on head_dim."""
    seq = 70
    buf, ldi = random_case(hd, seq, seq, heads, kv, hd=hd)
    qd, kd = heads * hd, kv * hd
    scale = float(1 / np.sqrt(hd))
    mask = (np.arange(seq) != 7).astype(np.int32)
    out, kernel = dev.attention(buf, ldi, 0, qd, qd + kd, seq, seq, heads, kv, hd, scale, causal, mask)
    assert kernel == "attention_generic"
    want = orc.attention_bf16(buf, ldi, 0, qd, qd + kd, seq, seq, heads, kv, hd, scale, causal, mask)
    assert_close(O.bf16_to_f32(out), want, f"scalar hd={hd}")


def test_scalar_kernel_still_answers_what_the_matrix_cores_cannot(dev, orc):
    """A non-positive scale (the matrix-core kernels fold the scale into the exponent base) goes to the scalar kernel."""
    heads, seq = 2, 40
    buf, ldi = random_case(13, seq, seq, heads, heads)
    out, kernel = dev.attention(buf, ldi, 0, 256, 512, seq, seq, heads, heads, 128, -0.0884)
    assert kernel == "attention_generic"
    want = orc.attention_bf16(buf, ldi, 0, 256, 512, seq, seq, heads, heads, 128, -0.0884)
    assert_close(O.bf16_to_f32(out), want, "negative scale")


def test_bad_arguments_are_reported_not_fatal(dev):
    buf, ldi = random_case(1, 8, 8, 3, 2)
    d = dev.put(buf)
    dev.lib.iris_dev_last_error()
    dev.lib.iris_dev_attention(d, 384, d, d, d, ldi, 8, 8, 3, 2, 128, 0.1, 0, None)    # 3 % 2 != 0
    assert dev.lib.iris_dev_last_error() != 0
    dev.lib.iris_dev_attention(d, 4096, d, d, d, ldi, 8, 8, 1, 1, 0, 0.1, 0, None)      # head_dim must be positive
    assert dev.lib.iris_dev_last_error() != 0
    dev.free_all()
