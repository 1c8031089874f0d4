"""iris_dev_attention_qnorm on the GPU (through the C ABI): attention with the
RMSNorm + rotary embedding of Q applied while Q is loaded.

The bar is the strictest one available: bit-for-bit equality with the two
calls it replaces (iris_dev_head_norm_rope on Q, then iris_dev_attention),
which are themselves held to the oracle by the other GPU tests; plus the
oracle directly (max-abs <= 2e-2, mean-abs <= 2e-3) where the fused path
takes other kernels than the two calls do. Q in memory must not change.
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


def k_normalised(dev, case):
    """The state the fused call expects: K normalised and rotated in place, Q still raw."""
    buf = dev.norm_rope(case["buf"], case["ldi"], case["q_dim"], case["wk"], case["cos"], case["sin"], case["seq"],
                        case["kv_heads"], 128, case["eps"], case["split_half"])
    out = dict(case); out["buf"] = buf
    return out


def two_calls(dev, case):
    buf = dev.norm_rope(case["buf"], case["ldi"], 0, case["wq"], case["cos"], case["sin"], case["seq"], case["heads"], 128,
                        case["eps"], case["split_half"])
    out, kernel = dev.attention(buf, case["ldi"], 0, case["q_dim"], case["q_dim"] + case["kv_dim"], case["seq"],
                                case["seq"], case["heads"], case["kv_heads"], 128, case["scale"], case["causal"],
                                case["key_mask"], ldo=case["ldo"])
    return out, kernel, buf


def fused(dev, case):
    return dev.attention_qnorm(case["buf"], case["ldi"], 0, case["q_dim"], case["q_dim"] + case["kv_dim"], case["seq"],
                               case["seq"], case["heads"], case["kv_heads"], 128, case["scale"], case["wq"], case["cos"],
                               case["sin"], case["eps"], case["split_half"], case["causal"], case["key_mask"],
                               ldo=case["ldo"])


def check_case(dev, case, what):
    case = k_normalised(dev, case)
    want, k2, _ = two_calls(dev, case)
    got, k1, after = fused(dev, case)
    assert (k1, k2) == ("fa_hd128_qnorm", "fa_hd128")
    assert np.array_equal(after, case["buf"]), f"{what}: the fused call changed its inputs"
    assert np.array_equal(got, want), f"{what}: {np.count_nonzero(got != want)} of {got.size} outputs differ from the two calls"


@pytest.mark.parametrize("name,make", [
    ("C1", lambda: W.c1()), ("C2/8", lambda: W.c2(8)), ("C3/8 cond", lambda: W.c3(8)[0]), ("C3/8 uncond", lambda: W.c3(8)[1]),
    ("C4", lambda: W.c4(1)), ("C4/4", lambda: W.c4(4)), ("C5/32", lambda: W.c5(32)),
])
def test_equals_the_two_calls_bit_for_bit(dev, name, make):
    """Consecutive pairs (FLUX, Z-Image eps and tables) and split-half pairs with causal GQA + padding mask (Qwen3)."""
    check_case(dev, make(), name)


@pytest.mark.parametrize("seq,heads,kv,causal,split", [
    (200, 6, 2, True, 1),            # 32-query workgroups
    (600, 16, 4, False, 0),          # 64
    (1300, 16, 16, False, 1),        # 128
    (2100, 24, 8, True, 0),          # 256
])
def test_every_workgroup_width(dev, orc, seq, heads, kv, causal, split):
    rng = np.random.default_rng(seq)
    ldi = (heads + 2 * kv) * 128
    buf = O.f32_to_bf16((rng.standard_normal((seq, ldi)) * 1.7).astype(np.float32))
    ang = rng.uniform(-3.0, 3.0, (seq, 64)).astype(np.float32)
    case = W._case(buf=buf, heads=heads, kv_heads=kv, causal=causal, split_half=split)
    case.update(ldo=heads * 128, cos=np.cos(ang), sin=np.sin(ang), wq=(1 + 0.1 * rng.standard_normal(128)).astype(np.float32),
                wk=(1 + 0.1 * rng.standard_normal(128)).astype(np.float32))
    check_case(dev, case, f"seq {seq}")
    # and one of them against the oracle end to end: oracle norm+rope on Q and K, oracle attention
    if seq == 600:
        ref = case["buf"].copy()
        orc.head_norm_rope_bf16(ref, ldi, case["wq"], case["cos"], case["sin"], seq, heads, 128, case["eps"], split, col0=0)
        orc.head_norm_rope_bf16(ref, ldi, case["wk"], case["cos"], case["sin"], seq, kv, 128, case["eps"], split,
                                col0=case["q_dim"])
        want = orc.attention_bf16(ref, ldi, 0, case["q_dim"], case["q_dim"] + case["kv_dim"], seq, seq, heads, kv, 128,
                                  case["scale"], causal, None)
        got, _, _ = fused(dev, k_normalised(dev, case))
        assert_parity(O.bf16_to_f32(got), want, f"qnorm seq {seq} vs oracle chain")


def test_fewer_queries_than_keys(dev):
    """seq_q != seq_k: the tables have one row per QUERY row; query rows past the last full block of 32."""
    rng = np.random.default_rng(5)
    seq_k, seq_q, heads = 333, 45, 3
    ldi = 3 * heads * 128
    buf = O.f32_to_bf16(rng.standard_normal((seq_k, ldi)).astype(np.float32))
    ang = rng.uniform(-3.0, 3.0, (seq_q, 64)).astype(np.float32)
    w = (1 + 0.1 * rng.standard_normal(128)).astype(np.float32)
    scale = 0.0884
    q_only = dev.norm_rope(buf[:seq_q].copy(), ldi, 0, w, np.cos(ang), np.sin(ang), seq_q, heads, 128, 1e-6, 0)
    ref = buf.copy(); ref[:seq_q] = q_only
    want, _ = dev.attention(ref, ldi, 0, heads * 128, 2 * heads * 128, seq_q, seq_k, heads, heads, 128, scale)
    got, kernel, after = dev.attention_qnorm(buf, ldi, 0, heads * 128, 2 * heads * 128, seq_q, seq_k, heads, heads, 128,
                                             scale, w, np.cos(ang), np.sin(ang), 1e-6, 0)
    assert kernel == "fa_hd128_qnorm"
    assert np.array_equal(after, buf) and np.array_equal(got, want)


@pytest.mark.parametrize("hd,ldi_extra,split", [(64, 0, 0), (64, 0, 1), (128, 2, 0), (256, 0, 1)])
def test_other_shapes_go_through_the_normalised_copy(dev, orc, hd, ldi_extra, split):
    """head_dim != 128 or rows that are not 16-byte aligned: a normalised copy of Q in private scratch, then the
    padded copy and the matrix-core kernel; checked against the oracle, q untouched."""
    rng = np.random.default_rng(hd + ldi_extra)
    seq, heads, kv = 70, 4, 2
    q_dim, kv_dim = heads * hd, kv * hd
    ldi = q_dim + 2 * kv_dim + ldi_extra
    buf = O.f32_to_bf16(rng.standard_normal((seq, ldi)).astype(np.float32))
    ang = rng.uniform(-3.0, 3.0, (seq, hd // 2)).astype(np.float32)
    w = (1 + 0.1 * rng.standard_normal(hd)).astype(np.float32)
    scale = float(1.0 / np.sqrt(hd))
    mask = (rng.random(seq) < 0.8).astype(np.int32); mask[0] = 1
    got, kernel, after = dev.attention_qnorm(buf, ldi, 0, q_dim, q_dim + kv_dim, seq, seq, heads, kv, hd, scale, w,
                                             np.cos(ang), np.sin(ang), 1e-5, split, causal=True, key_mask=mask)
    assert kernel == ("fa_hd128_packed_qnorm" if hd <= 128 else "fa_hd256_packed_qnorm")
    assert np.array_equal(after, buf)
    ref = buf.copy()
    orc.head_norm_rope_bf16(ref, ldi, w, np.cos(ang), np.sin(ang), seq, heads, hd, 1e-5, split, col0=0)
    want = orc.attention_bf16(ref, ldi, 0, q_dim, q_dim + kv_dim, seq, seq, heads, kv, hd, scale, True, mask)
    assert_parity(O.bf16_to_f32(got), want, f"qnorm fallback hd {hd}")


def test_scratch_copy_grows_and_is_reused(dev, orc):
    """Two fallback calls in a row, the second larger (the private copy is reallocated), then a smaller one."""
    for seq in (20, 90, 33):
        rng = np.random.default_rng(seq)
        heads, hd = 2, 64
        ldi = 3 * heads * hd
        buf = O.f32_to_bf16(rng.standard_normal((seq, ldi)).astype(np.float32))
        ang = rng.uniform(-3.0, 3.0, (seq, hd // 2)).astype(np.float32)
        w = np.ones(hd, np.float32)
        got, kernel, _ = dev.attention_qnorm(buf, ldi, 0, heads * hd, 2 * heads * hd, seq, seq, heads, heads, hd, 0.125, w,
                                             np.cos(ang), np.sin(ang), 1e-6, 0)
        assert kernel == "fa_hd128_packed_qnorm"
        ref = buf.copy()
        orc.head_norm_rope_bf16(ref, ldi, w, np.cos(ang), np.sin(ang), seq, heads, hd, 1e-6, 0, col0=0)
        want = orc.attention_bf16(ref, ldi, 0, heads * hd, 2 * heads * hd, seq, seq, heads, heads, hd, 0.125)
        assert_parity(O.bf16_to_f32(got), want, f"qnorm fallback seq {seq}")


def test_missing_weights_or_tables_are_reported_not_fatal(dev):
    lib = dev.lib
    buf = dev.put(np.zeros((4, 384), np.uint16)); out = dev.alloc(4 * 128 * 2)
    w = dev.put(np.ones(128, np.float32)); t = dev.put(np.zeros((4, 64), np.float32))
    lib.iris_dev_last_error()
    lib.iris_dev_attention_qnorm(out, 128, buf, buf, buf, 384, 4, 4, 1, 1, 128, 0.09, 0, None, None, t, t, 1e-6, 0)
    assert lib.iris_dev_last_error() != 0
    lib.iris_dev_attention_qnorm(out, 128, buf, buf, buf, 384, 4, 4, 1, 1, 128, 0.09, 0, None, w, None, t, 1e-6, 0)
    assert lib.iris_dev_last_error() != 0
    lib.iris_dev_attention_qnorm(out, 128, buf, buf, buf, 384, 4, 4, 1, 1, 128, 0.09, 0, None, w, t, t, 1e-6, 0)
    assert lib.iris_dev_last_error() == 0
    dev.free_all()
