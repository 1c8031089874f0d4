"""The head_dim-512 attention kernel (one wave per SIMD owns 32 whole queries; the VAE mid-block call of the
reference, iris_vae.c:1112-1124) through the C ABI and, for the number of key ranges, through the kernel's own
launcher, against the fp32 CPU oracle on identical bf16 inputs. Bars as in test_gpu_attention.py.
The planner test at the end needs no GPU.
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


def random_case(seed, seq_q, seq_k, heads, kv, sigma=1.0, pad=0):
    rng = np.random.default_rng(seed)
    ldi = (heads + 2 * kv) * HD + pad
    buf = O.f32_to_bf16(rng.standard_normal((max(seq_q, seq_k), ldi)).astype(np.float32) * sigma)
    return buf, ldi


def sample_rows(seq, n, seed=0):
    fixed = [0, 1, 31, 32, 127, 128, seq // 2, seq - 129, seq - 128, seq - 1]
    rng = np.random.default_rng(seed)
    return np.unique(np.clip(np.r_[fixed, rng.integers(0, seq, n)], 0, seq - 1)).astype(np.int32)


def plan(lib, seq_q, seq_k, heads):
    lib.iris_hip_fa_hd512_plan.restype = C.c_size_t
    lib.iris_hip_fa_hd512_plan.argtypes = [C.c_int, C.c_int, C.c_int, C.POINTER(C.c_int)]
    splits = C.c_int(0)
    need = lib.iris_hip_fa_hd512_plan(seq_q, seq_k, heads, C.byref(splits))
    return splits.value, need


# ------------------------------------------------------------------ through the ABI
@pytest.mark.gpu
@pytest.mark.parametrize("seq_q,seq_k,heads,kv", [(1, 1, 1, 1), (7, 33, 1, 1), (128, 32, 1, 1), (129, 31, 2, 1), (64, 45, 1, 1),
                                                  (40, 63, 2, 2), (300, 1000, 2, 2), (1000, 300, 3, 1), (1024, 1024, 1, 1),
                                                  (2500, 2500, 1, 1), (640, 4100, 4, 2), (200, 1027, 1, 1)])
def test_shapes_against_the_oracle(dev, orc, seq_q, seq_k, heads, kv):
    """Ragged query and key counts (tiles of 32 keys, workgroups of 128 queries), grouped kv heads, and sizes whose
    keys the launcher cuts into one to eight ranges. A key count that is not a multiple of 32 moves the last tile back
    to end with the sequence and masks the keys it then shares with the tile before (33: all but one of them)."""
    buf, ldi = random_case(seq_q + 3 * seq_k + heads, seq_q, seq_k, heads, kv, pad=8)
    qd, kd = heads * HD, kv * HD
    scale = float(1 / np.sqrt(HD))
    out, kernel = dev.attention(buf, ldi, 0, qd, qd + kd, seq_q, seq_k, heads, kv, HD, scale, ldo=qd + 4, out_col=4)
    assert kernel == ("fa_hd512" if seq_k >= 32 else "fa_sliced")       # its key tiles are 32 whole rows
    want = orc.attention_bf16(buf, ldi, 0, qd, qd + kd, seq_q, seq_k, heads, kv, HD, scale)
    assert_parity(O.bf16_to_f32(out[:, 4:]), want, f"hd512 {seq_q}x{seq_k} heads {heads}/{kv}")
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


@pytest.mark.gpu
@pytest.mark.parametrize("seed", [1, 2])
def test_random_shapes(dev, orc, seed):
    """Seeded random sweep at head_dim 512: 32 .. 1500 keys (ragged against the tiles of 32 keys and, through the
    launcher's choice, against every number of key ranges), 1 .. 700 queries, one to three kv heads with one or two
    query heads each, padded row strides, two scales and two input spreads."""
    rng = np.random.default_rng(seed)
    for case in range(25):
        kv = int(rng.choice([1, 1, 2, 3]))
        heads = kv * int(rng.choice([1, 1, 2]))
        seq_k = int(rng.integers(32, 1500))
        seq_q = seq_k if rng.random() < 0.5 else int(rng.integers(1, 700))
        qd, kd = heads * HD, kv * HD
        ldi = qd + 2 * kd + int(rng.choice([0, 0, 8, 64]))
        buf = O.f32_to_bf16((rng.standard_normal((max(seq_q, seq_k), ldi)) * rng.choice([0.3, 1.0])).astype(np.float32))
        scale = float(rng.choice([1 / np.sqrt(HD), 0.02]))
        what = f"seed {seed} case {case}: q {seq_q} k {seq_k} heads {heads}/{kv} ldi {ldi} scale {scale:.4f} ranges {plan(dev.lib, seq_q, seq_k, heads)[0]}"
        out, kernel = dev.attention(buf, ldi, 0, qd, qd + kd, seq_q, seq_k, heads, kv, HD, scale)
        assert kernel == "fa_hd512", what
        want = orc.attention_bf16(buf, ldi, 0, qd, qd + kd, seq_q, seq_k, heads, kv, HD, scale)
        assert_parity(O.bf16_to_f32(out), want, what)


# ------------------------------------------------------------------ every number of key ranges
def launch_with_ranges(dev, buf, ldi, seq_q, seq_k, heads, kv, scale, splits):
    lib = dev.lib
    lib.iris_hip_fa_hd512.restype = C.c_int
    lib.iris_hip_fa_hd512.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int,
                                      C.c_int, C.c_int, C.c_int, C.c_float, C.c_int, C.c_void_p]
    lib.iris_dev_stream.restype = C.c_void_p
    qd, kd = heads * HD, kv * HD
    d = dev.put(buf)
    out0 = np.full((seq_q, qd), 0x7fc0, dtype=np.uint16)
    do = dev.put(out0)
    scratch = dev.alloc(max(16, seq_q * heads * splits * (HD + 2) * 4))
    err = lib.iris_hip_fa_hd512(lib.iris_dev_stream(), do, qd, d, ptr_add(d, 2 * qd), ptr_add(d, 2 * (qd + kd)), ldi, seq_q, seq_k,
                                heads, kv, scale, splits, scratch)
    dev.check()
    out = dev.get(do, out0.shape, np.uint16)
    dev.free_all()
    return err, out


@pytest.mark.gpu
def test_every_number_of_key_ranges_gives_the_same_rows(dev, orc):
    """1 to 8 ranges on 2 heads x 260 queries x 1500 keys (47 tiles, the last one partly filled, ranges of unequal
    length): each against the oracle, and against the one-range result: the probabilities of a range are rounded to
    bf16 relative to that range's own running max, so the rows differ by rounding noise only, a small fraction of
    a bf16 step of the outputs' spread on average."""
    seq_q, seq_k, heads, kv = 260, 1500, 2, 1
    buf, ldi = random_case(11, seq_q, seq_k, heads, kv)
    scale = float(1 / np.sqrt(HD))
    want = orc.attention_bf16(buf, ldi, 0, heads * HD, (heads + kv) * HD, seq_q, seq_k, heads, kv, HD, scale)
    tiles = (seq_k + 31) // 32
    one = None
    for splits in range(1, 9):
        per = (tiles + splits - 1) // splits
        err, out = launch_with_ranges(dev, buf, ldi, seq_q, seq_k, heads, kv, scale, splits)
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


# ------------------------------------------------------------------ no GPU needed
def test_planner_never_leaves_a_range_empty():
    import iris_c_amd
    lib = C.CDLL(iris_c_amd.LIB_PATH)
    rng = np.random.default_rng(0)
    sizes = [(1, 1, 1), (16384, 16384, 1), (4096, 4096, 1), (50176, 50176, 1), (1024, 1024, 1), (128, 33, 1), (300, 255, 5)]
    sizes += [tuple(int(x) for x in (rng.integers(1, 60000), rng.integers(1, 60000), rng.integers(1, 5))) for _ in range(300)]
    for seq_q, seq_k, heads in sizes:
        splits, need = plan(lib, seq_q, seq_k, heads)
        tiles = (seq_k + 31) // 32
        per = (tiles + splits - 1) // splits
        assert 1 <= splits <= min(8, tiles) and (tiles + per - 1) // per == splits, (seq_q, seq_k, heads, splits)
        assert need == (0 if splits == 1 else seq_q * heads * splits * (HD + 2) * 4)
    assert plan(lib, 16384, 16384, 1)[0] == 2                 # 128 workgroups of 128 queries on 256 CUs
    assert plan(lib, 128, 64, 1)[0] == 1
