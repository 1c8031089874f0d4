"""One single-stream transformer block issued the way the reference issues it
(iris_transformer_flux.c:3826-3839): layer norm + modulation, the fused
input projection into [q | k | v | gate | up] rows, norm+rope on the Q and K
columns of those rows, joint attention writing into the first columns of the
[attention | swiglu] rows, SwiGLU into the rest, output projection, gated
residual. Every pointer but the first is interior, every stride differs from
the row width: this is the layout contract of the device API, exercised as a
chain and compared with the same chain composed from the CPU oracle's
operators.
"""
import numpy as np
import pytest

import oracle as O
from gpu_harness import Dev, ptr_add, error_stats

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    return Dev()


def make_block(seed, seq, heads, mlp):
    rng = np.random.default_rng(seed)
    dim = heads * 128
    ldh, ldc = 3 * dim + 2 * mlp, dim + mlp
    f = lambda *shape, s=1.0: (rng.standard_normal(shape) * s).astype(np.float32)
    ang = rng.uniform(-3.0, 3.0, (seq, 64)).astype(np.float32)
    return dict(seq=seq, heads=heads, dim=dim, mlp=mlp, ldh=ldh, ldc=ldc,
                x=f(seq, dim, s=1.5) + 0.2, mod=f(3 * dim, s=0.3),
                w_in=O.f32_to_bf16(f(ldh, dim, s=1.0 / np.sqrt(dim))), w_out=O.f32_to_bf16(f(dim, ldc, s=1.0 / np.sqrt(ldc))),
                norm_q=1 + f(128, s=0.05), norm_k=1 + f(128, s=0.05), cos=np.cos(ang), sin=np.sin(ang),
                scale=float(1.0 / np.sqrt(128.0)))


def oracle_block(orc, b):
    seq, dim, mlp, ldh, ldc, heads = b["seq"], b["dim"], b["mlp"], b["ldh"], b["ldc"], b["heads"]
    norm = orc.dev_layer_norm_mod(b["x"], b["mod"][:dim], b["mod"][dim:2 * dim], 1e-6)
    h = O.f32_to_bf16(orc.dev_linear(norm, b["w_in"]))
    orc.head_norm_rope_bf16(h, ldh, b["norm_q"], b["cos"], b["sin"], seq, heads, 128, 1e-6, 0, col0=0)
    orc.head_norm_rope_bf16(h, ldh, b["norm_k"], b["cos"], b["sin"], seq, heads, 128, 1e-6, 0, col0=dim)
    att = orc.attention_bf16(h, ldh, 0, dim, 2 * dim, seq, seq, heads, heads, 128, b["scale"])
    cat = np.zeros((seq, ldc), np.uint16)
    cat[:, :dim] = O.f32_to_bf16(att)
    cat[:, dim:] = orc.dev_swiglu(np.ascontiguousarray(h[:, 3 * dim:]), mlp)
    out = orc.dev_linear(cat, b["w_out"])
    return orc.dev_residual(b["x"], out, b["mod"][2 * dim:])


def device_block(dev, b, q_norm_inside_attention):
    lib = dev.lib
    seq, dim, mlp, ldh, ldc, heads = b["seq"], b["dim"], b["mlp"], b["ldh"], b["ldc"], b["heads"]
    x, mod = dev.put(b["x"]), dev.put(b["mod"])
    w_in, w_out = dev.put(b["w_in"]), dev.put(b["w_out"])
    nq, nk, cos, sin = dev.put(b["norm_q"]), dev.put(b["norm_k"]), dev.put(b["cos"]), dev.put(b["sin"])
    norm, h, cat, out = dev.alloc(seq * dim * 2), dev.alloc(seq * ldh * 2), dev.alloc(seq * ldc * 2), dev.alloc(seq * dim * 4)
    col = lambda p, elems: ptr_add(p, 2 * elems)
    lib.iris_dev_layer_norm_mod(norm, x, mod, ptr_add(mod, 4 * dim), seq, dim, 1e-6)
    lib.iris_dev_linear_bf16(h, norm, w_in, seq, dim, ldh)
    if q_norm_inside_attention:
        lib.iris_dev_head_norm_rope(col(h, dim), ldh, nk, cos, sin, seq, heads, 128, 1e-6, 0)
        lib.iris_dev_attention_qnorm(cat, ldc, h, col(h, dim), col(h, 2 * dim), ldh, seq, seq, heads, heads, 128, b["scale"], 0,
                                     None, nq, cos, sin, 1e-6, 0)
    else:
        lib.iris_dev_head_norm_rope(h, ldh, nq, cos, sin, seq, heads, 128, 1e-6, 0)
        lib.iris_dev_head_norm_rope(col(h, dim), ldh, nk, cos, sin, seq, heads, 128, 1e-6, 0)
        lib.iris_dev_attention(cat, ldc, h, col(h, dim), col(h, 2 * dim), ldh, seq, seq, heads, heads, 128, b["scale"], 0, None)
    kernel = dev.dev.last_kernel()
    lib.iris_dev_swiglu(col(cat, dim), ldc, col(h, 3 * dim), col(h, 3 * dim + mlp), ldh, seq, mlp)
    lib.iris_dev_linear_f32(out, cat, w_out, seq, ldc, dim)
    lib.iris_dev_residual(x, out, ptr_add(mod, 8 * dim), seq, dim)
    dev.check()
    got = dev.get(x, (seq, dim), np.float32)
    dev.free_all()
    return got, kernel


@pytest.mark.parametrize("seq,heads,mlp,backend", [(80, 4, 1024, 0), (333, 3, 768, 1), (600, 2, 512, 1)])
def test_single_stream_block_chain(dev, orc, seq, heads, mlp, backend):
    """backend 0: linear layers on the vendor GEMM when present; 1: on the library's own kernels (333 and 600 rows
    reach the 256 x 256 kernel with ragged edges)."""
    b = make_block(seq + heads, seq, heads, mlp)
    dev.lib.iris_dev_linear_backend(backend)
    try:
        got, kernel = device_block(dev, b, False)
        fused, kernel_fused = device_block(dev, b, True)
    finally:
        dev.lib.iris_dev_linear_backend(0)
    assert (kernel, kernel_fused) == ("fa_hd128", "fa_hd128_qnorm")
    want = oracle_block(orc, b)
    # judged on the block's update of the residual stream, whose entries are O(1)
    mx, mean = error_stats(got - b["x"], want - b["x"])
    assert mx <= 3e-2 and mean <= 3e-3, f"max-abs {mx:.4g}, mean-abs {mean:.4g}"
    assert np.array_equal(got, fused), "the block with Q normalised inside attention differs from the three-call block"
