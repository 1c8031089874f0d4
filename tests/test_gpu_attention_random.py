"""Seeded random sweep of iris_dev_attention / iris_dev_attention_qnorm shapes on the GPU against the
CPU oracle: sequence lengths 1 .. 900 (ragged against every tile and workgroup size), seq_q != seq_k,
grouped kv heads, causal, key masks of varying density, padded row strides, both pairings of the rotary
embedding. Rows without a valid key follow the device convention (zeros; reference iris_cuda.cu:531,
650, 676) where the CPU oracle averages uniformly. Bar: max-abs <= 2e-2, mean-abs <= 2e-3.
"""
import numpy as np
import pytest

import oracle as O
from gpu_harness import Dev, assert_parity

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    return Dev()


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_random_shapes(dev, orc, seed):
    rng = np.random.default_rng(seed)
    for case in range(40):
        kv = int(rng.choice([1, 2, 3, 4, 8]))
        heads = kv * int(rng.choice([1, 1, 2, 4]))
        seq_k = int(rng.integers(1, 900))
        causal = bool(rng.integers(0, 2))
        seq_q = seq_k if causal or rng.random() < 0.6 else int(rng.integers(1, seq_k + 1))
        qnorm, split = bool(rng.integers(0, 2)), int(rng.integers(0, 2))
        q_dim, kv_dim = heads * 128, kv * 128
        ldi = q_dim + 2 * kv_dim + int(rng.choice([0, 0, 8, 64]))
        buf = O.f32_to_bf16((rng.standard_normal((max(seq_q, seq_k), ldi)) * rng.choice([0.3, 1.0])).astype(np.float32))
        mask = None
        if rng.integers(0, 2):
            mask = (rng.random(seq_k) < rng.choice([0.1, 0.5, 0.9])).astype(np.int32)
            if rng.random() < 0.7:
                mask[0] = 1
        scale = float(rng.choice([0.0884, 0.05]))
        what = (f"seed {seed} case {case}: q {seq_q} k {seq_k} heads {heads}/{kv} causal {causal} "
                f"mask {None if mask is None else round(float(mask.mean()), 2)} qnorm {qnorm} split {split} ldi {ldi}")
        if qnorm:
            ang = rng.uniform(-3, 3, (seq_q, 64)).astype(np.float32)
            w = (1 + 0.1 * rng.standard_normal(128)).astype(np.float32)
            got, kernel, after = dev.attention_qnorm(buf, ldi, 0, q_dim, q_dim + kv_dim, seq_q, seq_k, heads, kv, 128, scale, w,
                                                     np.cos(ang), np.sin(ang), 1e-6, split, causal=causal, key_mask=mask)
            assert np.array_equal(after, buf), what
            ref = buf.copy()
            orc.head_norm_rope_bf16(ref, ldi, w, np.cos(ang), np.sin(ang), seq_q, heads, 128, 1e-6, split, col0=0)
        else:
            got, kernel = dev.attention(buf, ldi, 0, q_dim, q_dim + kv_dim, seq_q, seq_k, heads, kv, 128, scale, causal, mask)
            ref = buf
        assert kernel in ("fa_hd128", "fa_hd128_qnorm"), what
        want = orc.attention_bf16(ref, ldi, 0, q_dim, q_dim + kv_dim, seq_q, seq_k, heads, kv, 128, scale, causal, mask)
        if mask is not None:
            valid_so_far = np.cumsum(mask)
            for r in range(seq_q):
                if (valid_so_far[min(r, seq_k - 1)] if causal else valid_so_far[-1]) == 0:
                    want[r] = 0.0
        # a mask without a valid key (or none up to the causal row) makes zero rows, possibly all of them
        assert_parity(O.bf16_to_f32(got[:, :q_dim]), want, what, zero_reference_ok=mask is not None)
