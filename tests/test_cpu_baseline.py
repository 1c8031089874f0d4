"""The CPU timing baseline (reference BLAS-build structure) computes the same
attention as the oracle, with whichever sgemm provider was found."""
import numpy as np
import pytest

import oracle as O


@pytest.fixture(scope="module")
def base():
    return O.cpu_baseline()


def test_thread_rule(base):
    # largest divisor of heads <= cpu limit (reference iris_transformer_flux.c:1569-1579)
    assert base.threads_for(24, 8) == 8 and base.threads_for(24, 7) == 6 and base.threads_for(30, 16) == 15
    assert base.threads_for(24, 1) == 1 and base.threads_for(5, 64) == 5


@pytest.mark.parametrize("heads,kv,causal,masked,chunk", [(4, 4, False, False, 0), (4, 4, False, False, 16),
                                                          (8, 2, True, True, 0), (6, 6, False, True, 7)])
def test_matches_oracle(base, orc, heads, kv, causal, masked, chunk):
    rng = np.random.default_rng(heads + chunk)
    seq, hd = 50, 32
    q = rng.standard_normal((seq, heads * hd)).astype(np.float32)
    k = rng.standard_normal((seq, kv * hd)).astype(np.float32)
    v = rng.standard_normal((seq, kv * hd)).astype(np.float32)
    mask = (np.arange(seq) < 31).astype(np.int32) if masked else None
    got, nt = base.attention(q, k, v, heads, kv, 0.17, causal, mask, q_chunk=chunk, threads=3)
    assert heads % nt == 0 and nt <= 3
    want = orc.attention_strided(q, k, v, heads, kv, 0.17, causal, mask)
    np.testing.assert_allclose(got, want, rtol=2e-4, atol=2e-5)


def test_norm_rope_matches_oracle(base, orc):
    rng = np.random.default_rng(3)
    x = rng.standard_normal((10, 3, 128)).astype(np.float32)
    w = (1 + 0.02 * rng.standard_normal(128)).astype(np.float32)
    ang = rng.uniform(-3, 3, (10, 64))
    c, s = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    for split in (0, 1):
        np.testing.assert_allclose(base.norm_rope(x, w, c, s, 1e-6, split), orc.head_norm_rope_f32(x, w, c, s, 1e-6, split),
                                   rtol=1e-5, atol=1e-6)
