"""The attention kernel for wide heads (one wave per SIMD owns 32 whole queries): head_dim 512 — the VAE mid-block call
of the reference, iris_vae.c:1112-1124, and the same head size with a key mask or a causal limit, which the device
interface allows — and head_dim 256, the same kernel with half the products per tile. Through the C ABI and, for the
number of key ranges, through the kernel's own launcher, against the fp32 CPU oracle on identical bf16 inputs. Bars
as in test_gpu_attention.py. The planner tests at the end need no GPU.
"""
import ctypes as C
import os

import numpy as np
import pytest

import oracle as O
from gpu_harness import Dev, assert_parity, ptr_add

HD = 512
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def dev():
    return Dev()


def random_case(seed, seq_q, seq_k, heads, kv, sigma=1.0, pad=0, hd=HD):
    rng = np.random.default_rng(seed)
    ldi = (heads + 2 * kv) * hd + pad
    buf = O.f32_to_bf16(rng.standard_normal((max(seq_q, seq_k), ldi)).astype(np.float32) * sigma)
    return buf, ldi


def sample_rows(seq, n, seed=0):
    fixed = [0, 1, 31, 32, 127, 128, seq // 2, seq - 129, seq - 128, seq - 1]
    rng = np.random.default_rng(seed)
    return np.unique(np.clip(np.r_[fixed, rng.integers(0, seq, n)], 0, seq - 1)).astype(np.int32)


def plan(lib, seq_q, seq_k, heads, causal=False, masked=False, hd=HD):
    fn = getattr(lib, f"iris_hip_fa_hd{hd}_plan")
    fn.restype = C.c_size_t
    fn.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_int)]
    splits = C.c_int(0)
    need = fn(seq_q, seq_k, heads, int(causal), int(masked), C.byref(splits))
    return splits.value, need


# ------------------------------------------------------------------ through the ABI
@pytest.mark.gpu
@pytest.mark.parametrize("seq_q,seq_k,heads,kv", [(1, 1, 1, 1), (7, 33, 1, 1), (128, 32, 1, 1), (129, 31, 2, 1), (64, 45, 1, 1),
                                                  (40, 63, 2, 2), (300, 1000, 2, 2), (1000, 300, 3, 1), (1024, 1024, 1, 1),
                                                  (2500, 2500, 1, 1), (640, 4100, 4, 2), (200, 1027, 1, 1)])
@pytest.mark.parametrize("hd", [512, 256])
def test_shapes_against_the_oracle(dev, orc, hd, seq_q, seq_k, heads, kv):
    """Ragged query and key counts (tiles of 32 keys, workgroups of 128 queries), grouped kv heads, and sizes whose
    keys the launcher cuts into one to eight ranges. A key count that is not a multiple of 32 moves the last tile back
    to end with the sequence and masks the keys it then shares with the tile before (33: all but one of them); fewer
    than 32 keys are one tile padded with its last key (the 1 x 1 call reads nothing but its one row: any row beyond
    it would be outside the buffer)."""
    buf, ldi = random_case(seq_q + 3 * seq_k + heads, seq_q, seq_k, heads, kv, pad=8, hd=hd)
    qd, kd = heads * hd, kv * hd
    scale = float(1 / np.sqrt(hd))
    out, kernel = dev.attention(buf, ldi, 0, qd, qd + kd, seq_q, seq_k, heads, kv, hd, scale, ldo=qd + 4, out_col=4)
    assert kernel == f"fa_hd{hd}"
    want = orc.attention_bf16(buf, ldi, 0, qd, qd + kd, seq_q, seq_k, heads, kv, hd, scale)
    assert_parity(O.bf16_to_f32(out[:, 4:]), want, f"hd{hd} {seq_q}x{seq_k} heads {heads}/{kv}")
    assert np.all(out[:, :4] == 0x7fc0)                      # nothing written in front of the output columns


@pytest.mark.gpu
def test_peaked_rows_rescale_and_stay_finite(dev, orc):
    """Scores up to ~ +-100 after scaling: the running max is raised several times along a row and the accumulators
    are rescaled; rows stay finite and within the relative bar."""
    seq_q, seq_k = 200, 3000
    buf, ldi = random_case(5, seq_q, seq_k, 1, 1, sigma=4.0)
    scale = float(1 / np.sqrt(HD))
    out, kernel = dev.attention(buf, ldi, 0, HD, 2 * HD, seq_q, seq_k, 1, 1, HD, scale)
    assert kernel == "fa_hd512"
    got = O.bf16_to_f32(out)
    assert np.all(np.isfinite(got))
    want = orc.attention_bf16(buf, ldi, 0, HD, 2 * HD, seq_q, seq_k, 1, 1, HD, scale)
    assert np.abs(got - want).max() <= 2e-2 * 4.0 and np.abs(got - want).mean() <= 2e-3 * 4.0   # outputs are O(4)


@pytest.mark.gpu
def test_vae_16384_tokens_sampled_rows_and_constant_values(dev, orc):
    """One head of 512 over the 16384 latent positions of a 1024 x 1024 image (two key ranges and a merge): sampled
    rows against the oracle, and with every value row the same the output is that row in every query."""
    seq = 16384
    buf, ldi = random_case(79, seq, seq, 1, 1)
    scale = float(1 / np.sqrt(HD))
    out, kernel = dev.attention(buf, ldi, 0, HD, 2 * HD, seq, seq, 1, 1, HD, scale)
    assert kernel == "fa_hd512" and plan(dev.lib, seq, seq, 1)[0] >= 2
    rows = np.unique(np.r_[sample_rows(seq, 12), [8191, 8192]]).astype(np.int32)
    want = orc.attention_bf16(buf, ldi, 0, HD, 2 * HD, seq, seq, 1, 1, HD, scale, rows=rows)
    assert_parity(O.bf16_to_f32(out[rows]), want, "VAE 16384 tokens sampled")
    buf[:, 2 * HD:] = buf[9, 2 * HD:]
    out2, _ = dev.attention(buf, ldi, 0, HD, 2 * HD, seq, seq, 1, 1, HD, scale)
    assert np.array_equal(out2, np.tile(buf[9, 2 * HD:], (seq, 1)))


def key_mask_of(kind, seq_k, seed=0):
    """'random': 60 % of the keys; 'sparse': 3 %; 'prefix': the padding mask of a text encoder, first 2/3 valid;
    'holes': whole tiles of 32 keys missing, others whole."""
    rng = np.random.default_rng(seed + seq_k)
    if kind == "random":
        m = rng.random(seq_k) < 0.6
    elif kind == "sparse":
        m = rng.random(seq_k) < 0.03
    elif kind == "prefix":
        m = np.arange(seq_k) < max(1, 2 * seq_k // 3)
    else:
        m = np.repeat(rng.random((seq_k + 31) // 32) < 0.5, 32)[:seq_k]
    if not m.any():
        m[seq_k // 2] = True          # a row without any valid key is zero on the device and an average in the oracle: its own test
    return m.astype(np.int32)


def assert_parity_where_keys_are_visible(out, want, causal, mask, what):
    """Causal rows in front of the first valid key see no key: zero on the device (the oracle's masked-score convention
    averages the values there instead); all other rows to the parity bar."""
    first = int(np.argmax(mask)) if (causal and mask is not None) else 0
    first = min(first, out.shape[0])
    assert not out[:first].any(), what
    if first < out.shape[0]:
        assert_parity(O.bf16_to_f32(out[first:]), want[first:], what)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["random", "sparse", "prefix", "holes"])
@pytest.mark.parametrize("seq_q,seq_k,heads,kv", [(128, 32, 1, 1), (100, 77, 1, 1), (40, 63, 2, 2), (300, 1000, 2, 1), (1000, 300, 3, 1),
                                                  (1024, 1024, 1, 1), (640, 4100, 2, 2)])
@pytest.mark.parametrize("hd", [512, 256])
def test_key_masks_against_the_oracle(dev, orc, hd, kind, seq_q, seq_k, heads, kv):
    """The key mask reaches the kernel as one word per tile of 32 keys (a pack kernel in front of it); a tile moved back
    to end with the sequence has the keys it shares with its neighbour cleared there. Masks that leave tiles whole,
    empty or ragged; a mask that leaves no key at all gives zero rows."""
    buf, ldi = random_case(7 * seq_q + seq_k, seq_q, seq_k, heads, kv, hd=hd)
    qd, kd = heads * hd, kv * hd
    scale = float(1 / np.sqrt(hd))
    mask = key_mask_of(kind, seq_k)
    out, kernel = dev.attention(buf, ldi, 0, qd, qd + kd, seq_q, seq_k, heads, kv, hd, scale, False, mask)
    assert kernel == f"fa_hd{hd}"
    want = orc.attention_bf16(buf, ldi, 0, qd, qd + kd, seq_q, seq_k, heads, kv, hd, scale, False, mask)
    assert_parity(O.bf16_to_f32(out), want, f"hd{hd} {kind} mask {seq_q}x{seq_k} heads {heads}/{kv}")


@pytest.mark.gpu
def test_a_mask_without_any_key_gives_zero_rows(dev):
    buf, ldi = random_case(3, 300, 1000, 1, 1)
    out, kernel = dev.attention(buf, ldi, 0, HD, 2 * HD, 300, 1000, 1, 1, HD, 0.05, False, np.zeros(1000, np.int32))
    assert kernel == "fa_hd512" and not out.any()


@pytest.mark.gpu
@pytest.mark.parametrize("masked", [False, True])
@pytest.mark.parametrize("seq_q,seq_k,heads,kv", [(128, 32, 1, 1), (128, 128, 1, 1), (100, 77, 1, 1), (77, 100, 1, 1), (1027, 1027, 1, 1),
                                                  (300, 1000, 2, 1), (1000, 300, 2, 1), (2500, 2500, 1, 1), (513, 999, 3, 3),
                                                  (4100, 4100, 2, 1)])
@pytest.mark.parametrize("hd", [512, 256])
def test_causal_calls_against_the_oracle(dev, orc, hd, masked, seq_q, seq_k, heads, kv):
    """Query i sees keys 0 .. i: a workgroup walks the key tiles in front of its last query only, the launcher cuts
    the keys into ranges as for the full call (a range behind a workgroup's queries does not exist for it), and
    the workgroups are numbered by falling length. More queries than keys, more keys than queries, and a key mask on
    top (rows whose visible keys are all masked are zero, as in the oracle)."""
    buf, ldi = random_case(5 * seq_q + seq_k, seq_q, seq_k, heads, kv, hd=hd)
    qd, kd = heads * hd, kv * hd
    scale = float(1 / np.sqrt(hd))
    mask = key_mask_of("random", seq_k, seed=1) if masked else None
    out, kernel = dev.attention(buf, ldi, 0, qd, qd + kd, seq_q, seq_k, heads, kv, hd, scale, True, mask)
    assert kernel == f"fa_hd{hd}"
    want = orc.attention_bf16(buf, ldi, 0, qd, qd + kd, seq_q, seq_k, heads, kv, hd, scale, True, mask)
    assert_parity_where_keys_are_visible(out, want, True, mask, f"hd{hd} causal {seq_q}x{seq_k} heads {heads}/{kv} masked {masked}")


@pytest.mark.gpu
def test_masked_causal_rows_with_large_scores_stay_finite(dev, orc):
    seq = 100
    buf, ldi = random_case(21, seq, seq, 1, 1, sigma=3.0)          # |score| up to ~100
    scale = float(1 / np.sqrt(HD))
    mask = np.ones(seq, np.int32)
    mask[:10] = 0
    out, kernel = dev.attention(buf, ldi, 0, HD, 2 * HD, seq, seq, 1, 1, HD, scale, True, mask)
    assert kernel == "fa_hd512"
    got = O.bf16_to_f32(out)
    assert np.all(np.isfinite(got)) and np.all(got[:10] == 0.0)
    want = orc.attention_bf16(buf, ldi, 0, HD, 2 * HD, seq, seq, 1, 1, HD, scale, True, mask)
    gap = np.abs(got[10:] - want[10:])
    assert gap.max() <= 0.07 and gap.mean() <= 4e-3      # outputs are O(3): same relative bar as 2e-2 on O(1) values


@pytest.mark.gpu
def test_causal_16384_tokens_sampled_rows(dev, orc):
    """16384 tokens, causal, with and without a padding mask: several key ranges, workgroups of 4 to 128 turns. Sampled
    rows against the oracle, among them the first and last rows of workgroups and of key ranges."""
    seq = 16384
    buf, ldi = random_case(80, seq, seq, 1, 1)
    scale = float(1 / np.sqrt(HD))
    splits = plan(dev.lib, seq, seq, 1, causal=True)[0]
    assert splits >= 2
    per = 32 * (-(-(seq // 32) // splits))
    edges = [r * per + d for r in range(1, splits) for d in (-1, 0, 1)]
    rows = np.unique(np.r_[sample_rows(seq, 12), edges]).astype(np.int32)
    for mask in (None, key_mask_of("prefix", seq)):
        out, kernel = dev.attention(buf, ldi, 0, HD, 2 * HD, seq, seq, 1, 1, HD, scale, True, mask)
        assert kernel == "fa_hd512"
        want = orc.attention_bf16(buf, ldi, 0, HD, 2 * HD, seq, seq, 1, 1, HD, scale, True, mask, rows=rows)
        assert_parity(O.bf16_to_f32(out[rows]), want, f"causal 16384 tokens sampled, mask {mask is not None}")


@pytest.mark.gpu
@pytest.mark.parametrize("seed", [1, 2])
def test_random_shapes(dev, orc, seed):
    """Seeded random sweep at head_dim 512 and 256: 32 .. 1500 keys (ragged against the tiles of 32 keys and, through the
    launcher's choice, against every number of key ranges), 1 .. 700 queries, one to three kv heads with one or two
    query heads each, padded row strides, two scales and two input spreads; a third of the cases causal, a third
    with a key mask."""
    rng = np.random.default_rng(seed)
    for case in range(25):
        hd = int(rng.choice([512, 256]))
        kv = int(rng.choice([1, 1, 2, 3]))
        heads = kv * int(rng.choice([1, 1, 2]))
        seq_k = int(rng.integers(32, 1500))
        seq_q = seq_k if rng.random() < 0.5 else int(rng.integers(1, 700))
        qd, kd = heads * hd, kv * hd
        ldi = qd + 2 * kd + int(rng.choice([0, 0, 8, 64]))
        buf = O.f32_to_bf16((rng.standard_normal((max(seq_q, seq_k), ldi)) * rng.choice([0.3, 1.0])).astype(np.float32))
        scale = float(rng.choice([1 / np.sqrt(hd), 0.02]))
        causal = bool(rng.random() < 1 / 3)
        mask = key_mask_of(str(rng.choice(["random", "prefix", "holes"])), seq_k, seed=case) if rng.random() < 1 / 3 else None
        what = (f"seed {seed} case {case}: hd {hd} q {seq_q} k {seq_k} heads {heads}/{kv} ldi {ldi} scale {scale:.4f} causal {causal} "
                f"masked {mask is not None} ranges {plan(dev.lib, seq_q, seq_k, heads, causal, mask is not None, hd)[0]}")
        out, kernel = dev.attention(buf, ldi, 0, qd, qd + kd, seq_q, seq_k, heads, kv, hd, scale, causal, mask)
        assert kernel == f"fa_hd{hd}", what
        want = orc.attention_bf16(buf, ldi, 0, qd, qd + kd, seq_q, seq_k, heads, kv, hd, scale, causal, mask)
        assert_parity_where_keys_are_visible(out, want, causal, mask, what)


# ------------------------------------------------------------------ every number of key ranges
def launch_with_ranges(dev, buf, ldi, seq_q, seq_k, heads, kv, scale, splits, causal=False, mask=None, hd=HD):
    lib = dev.lib
    run = getattr(lib, f"iris_hip_fa_hd{hd}")
    run.restype = C.c_int
    run.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int,
                                      C.c_int, C.c_int, C.c_int, C.c_float, C.c_int, C.c_void_p, C.c_int, C.c_void_p]
    lib.iris_dev_stream.restype = C.c_void_p
    qd, kd = heads * hd, kv * hd
    d = dev.put(buf)
    out0 = np.full((seq_q, qd), 0x7fc0, dtype=np.uint16)
    do = dev.put(out0)
    scratch = dev.alloc(max(16, seq_q * heads * splits * (hd + 2) * 4) + 4 * ((seq_k + 31) // 32 + 8))
    dm = dev.put(np.ascontiguousarray(mask, np.int32)) if mask is not None else None
    err = run(lib.iris_dev_stream(), do, qd, d, ptr_add(d, 2 * qd), ptr_add(d, 2 * (qd + kd)), ldi, seq_q, seq_k,
                                heads, kv, scale, int(causal), dm, splits, scratch)
    dev.check()
    out = dev.get(do, out0.shape, np.uint16)
    dev.free_all()
    return err, out


@pytest.mark.gpu
@pytest.mark.parametrize("hd", [512, 256])
def test_every_number_of_key_ranges_gives_the_same_rows(dev, orc, hd):
    """1 to 8 ranges on 2 heads x 260 queries x 1500 keys (47 tiles, the last one partly filled, ranges of unequal
    length): each against the oracle, and against the one-range result: the probabilities of a range are rounded to
    bf16 relative to that range's own running max, so the rows differ by rounding noise only, a small fraction of
    a bf16 step of the outputs' spread on average."""
    seq_q, seq_k, heads, kv = 260, 1500, 2, 1
    buf, ldi = random_case(11, seq_q, seq_k, heads, kv, hd=hd)
    scale = float(1 / np.sqrt(hd))
    want = orc.attention_bf16(buf, ldi, 0, heads * hd, (heads + kv) * hd, seq_q, seq_k, heads, kv, hd, scale)
    tiles = (seq_k + 31) // 32
    one = None
    for splits in range(1, 9):
        per = (tiles + splits - 1) // splits
        err, out = launch_with_ranges(dev, buf, ldi, seq_q, seq_k, heads, kv, scale, splits, hd=hd)
        if (tiles + per - 1) // per != splits:              # this count would leave a range empty: refused, nothing written
            assert err != 0 and np.all(out == 0x7fc0)
            continue
        assert err == 0
        got = O.bf16_to_f32(out)
        assert_parity(got, want, f"{splits} key ranges")
        if one is None:
            one = got
        else:
            gap = np.abs(got - one)
            assert gap.max() <= 2.0 ** -6 * one.std() * 4 and gap.mean() <= 2.0 ** -8 * one.std()


@pytest.mark.gpu
@pytest.mark.parametrize("valid", [1000, 70, 1])
def test_every_number_of_key_ranges_with_a_padding_mask(dev, orc, valid):
    """With a key mask the kernel ends its walk at the last tile that has a valid key and cuts the tiles up to there
    into the call's ranges: 1000 of 1500 keys valid (32 tiles over 1 .. 8 ranges), 70 (3 tiles: more ranges than
    tiles, the spare ones record that they are empty), 1."""
    seq_q, seq_k, heads, kv = 260, 1500, 2, 1
    buf, ldi = random_case(13, seq_q, seq_k, heads, kv)
    scale = float(1 / np.sqrt(HD))
    mask = (np.arange(seq_k) < valid).astype(np.int32)
    want = orc.attention_bf16(buf, ldi, 0, heads * HD, (heads + kv) * HD, seq_q, seq_k, heads, kv, HD, scale, False, mask)
    tiles = (seq_k + 31) // 32
    for splits in range(1, 9):
        per = (tiles + splits - 1) // splits
        if (tiles + per - 1) // per != splits:
            continue
        err, out = launch_with_ranges(dev, buf, ldi, seq_q, seq_k, heads, kv, scale, splits, False, mask)
        assert err == 0
        assert_parity(O.bf16_to_f32(out), want, f"{valid} valid keys, {splits} key ranges")


@pytest.mark.gpu
@pytest.mark.parametrize("masked", [False, True])
@pytest.mark.parametrize("hd", [512, 256])
def test_every_number_of_key_ranges_of_a_causal_call(dev, orc, hd, masked):
    """1 to 8 ranges on 2 heads x 1500 queries x 1500 keys, causal: the pairs (query tile, range) that exist are
    numbered by falling length, the others are neither launched nor merged. Each count against the oracle."""
    seq, heads, kv = 1500, 2, 1
    buf, ldi = random_case(12, seq, seq, heads, kv, hd=hd)
    scale = float(1 / np.sqrt(hd))
    mask = key_mask_of("random", seq, seed=2) if masked else None
    want = orc.attention_bf16(buf, ldi, 0, heads * hd, (heads + kv) * hd, seq, seq, heads, kv, hd, scale, True, mask)
    tiles = (seq + 31) // 32
    ran = 0
    for splits in range(1, 9):
        per = (tiles + splits - 1) // splits
        err, out = launch_with_ranges(dev, buf, ldi, seq, seq, heads, kv, scale, splits, True, mask, hd=hd)
        if (tiles + per - 1) // per != splits:
            assert err != 0 and np.all(out == 0x7fc0)
            continue
        assert err == 0
        assert_parity_where_keys_are_visible(out, want, True, mask, f"causal, {splits} key ranges, masked {masked}")
        ran += 1
    assert ran >= 6


# ------------------------------------------------------------------ no GPU needed
def test_planner_never_leaves_a_range_empty():
    import iris_c_amd
    lib = C.CDLL(iris_c_amd.LIB_PATH)
    rng = np.random.default_rng(0)
    sizes = [(1, 1, 1), (16384, 16384, 1), (4096, 4096, 1), (50176, 50176, 1), (1024, 1024, 1), (128, 33, 1), (300, 255, 5)]
    sizes += [tuple(int(x) for x in (rng.integers(1, 60000), rng.integers(1, 60000), rng.integers(1, 5))) for _ in range(300)]
    for n, (seq_q, seq_k, heads) in enumerate(sizes):
        for causal in (False, True):
            for masked in (False, True):
                HD = (512, 256)[n % 2]
                splits, need = plan(lib, seq_q, seq_k, heads, causal, masked, HD)
                tiles = (seq_k + 31) // 32
                per = (tiles + splits - 1) // splits
                assert 1 <= splits <= min(8, tiles) and (tiles + per - 1) // per == splits, (seq_q, seq_k, heads, splits)
                words = (tiles + 7) // 8 * 8 if masked else 0       # one word per tile, a multiple of eight
                assert need == (0 if splits == 1 else seq_q * heads * splits * (HD + 2) * 4) + 4 * words
    assert plan(lib, 16384, 16384, 1)[0] == 2                 # 128 workgroups of 128 queries on 256 CUs
    assert plan(lib, 128, 64, 1)[0] == 1
    assert plan(lib, 16384, 16384, 1, causal=True)[0] in (3, 4)        # workgroups of up to 512 turns otherwise
    assert plan(lib, 128, 128, 1, causal=True)[0] == 1


def test_causal_workgroups_are_numbered_by_falling_length_and_none_is_missing():
    """Every (query tile, key range) pair of a causal call that has a key tile gets exactly one number, no other pair
    gets one that would do work twice, and the lengths never rise along the numbers (up to the rounding of a range's
    length to whole query tiles)."""
    import iris_c_amd
    lib = C.CDLL(iris_c_amd.LIB_PATH)
    qt, rg = C.c_int(0), C.c_int(0)
    rng = np.random.default_rng(1)
    cases = [(16384, 16384, s) for s in range(1, 9)] + [(1500, 1500, 5), (100, 3000, 3), (3000, 100, 2), (130, 130, 4)]
    cases += [(int(rng.integers(1, 20000)), int(rng.integers(32, 20000)), int(rng.integers(1, 9))) for _ in range(60)]
    for seq_q, seq_k, splits in cases:
        tiles, q_tiles = (seq_k + 31) // 32, (seq_q + 127) // 128
        splits = min(splits, tiles)
        per = (tiles + splits - 1) // splits
        if (tiles + per - 1) // per != splits:
            continue
        def length(q, r):
            keys = min(seq_k, 128 * q + 128)
            return max(0, min((keys + 31) // 32 - r * per, per))
        pairs = lib.iris_hip_fa_hd512_causal_order(-1, q_tiles, per, splits, C.byref(qt), C.byref(rg))
        seen, lengths = set(), []
        for j in range(pairs):
            lib.iris_hip_fa_hd512_causal_order(j, q_tiles, per, splits, C.byref(qt), C.byref(rg))
            assert 0 <= qt.value < q_tiles and 0 <= rg.value < splits and (qt.value, rg.value) not in seen
            seen.add((qt.value, rg.value))
            lengths.append(length(qt.value, rg.value))
        missing = [(q, r) for q in range(q_tiles) for r in range(splits) if length(q, r) > 0 and (q, r) not in seen]
        assert not missing, (seq_q, seq_k, splits, missing[:4])
        if seq_q <= seq_k:                           # with more queries than keys the last query tiles are all equally long
            slack = 4 + (per % 4) * (splits - 1)     # a range's length is rounded down to whole query tiles in the order
            assert all(b <= a + slack for a, b in zip(lengths, lengths[1:])), (seq_q, seq_k, splits)
