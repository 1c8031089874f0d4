"""Synthetic workloads of the five benchmark configurations (test side).

Inputs come from the oracle's restatement of the reference generator
(SplitMix64 -> xoshiro256** -> Box-Muller), seed 20250101 + config number,
drawn in the order Q, K, V, wq, wk, then mask lengths. Tables come from the
oracle's table builders. Every case is a dict with the fused bf16 row buffer
`buf` [seq, ldi] (q at column 0, k at q_dim, v at q_dim + kv_dim), the norm
weights, the RoPE tables and the attention arguments.

`shrink` divides the token counts so the CPU oracle finishes in seconds; the
layout, strides, head counts and masks keep their shape.
"""
import numpy as np

import oracle as O

SEED0 = 20250101


def _fused(orc, st, seq, q_dim, kv_dim, ldi, sigma):
    buf = np.zeros((seq, ldi), dtype=np.uint16)
    off = 0
    for width in (q_dim, kv_dim, kv_dim):
        x = orc.randn(st, seq * width).reshape(seq, width) * np.float32(sigma)
        buf[:, off:off + width] = O.f32_to_bf16(x)
        off += width
    return buf


def _weights(orc, st, hd=128):
    wq = (1.0 + 0.02 * orc.randn(st, hd)).astype(np.float32)
    wk = (1.0 + 0.02 * orc.randn(st, hd)).astype(np.float32)
    return wq, wk


def _case(**kw):
    kw.setdefault("kv_heads", kw["heads"])
    kw.setdefault("causal", False)
    kw.setdefault("key_mask", None)
    kw.setdefault("split_half", 0)
    kw.setdefault("eps", 1e-6)
    kw["hd"] = 128
    kw["scale"] = float(np.float32(1.0) / np.sqrt(np.float32(128.0)))
    kw["q_dim"] = kw["heads"] * 128
    kw["kv_dim"] = kw["kv_heads"] * 128
    kw["seq"] = kw["buf"].shape[0]
    kw["ldi"] = kw["buf"].shape[1]
    return kw


def flux2_case(cfg, txt, grid, refs=0, shrink=1, sigma=None):
    """C1 (cfg 1: 64 + 16x16), C2 (cfg 2: 512 + 64x64), C5 (cfg 5: + 2 reference images)."""
    orc = O.oracle()
    txt = max(txt // shrink, 1)
    g = max(int(round(grid / np.sqrt(shrink))), 1)
    ref_list = [(g, g)] * refs
    seq = txt + g * g * (1 + refs)
    heads, dim = 24, 3072
    st = orc.rng(SEED0 + cfg)
    sig = sigma if sigma is not None else 1.0
    buf = _fused(orc, st, seq, dim, dim, 3 * dim, sig)
    wq, wk = _weights(orc, st)
    cos, sin = orc.flux2_joint_tables(txt, g, g, ref_list)
    return _case(name=f"C{cfg}", buf=buf, heads=heads, ldo=dim, wq=wq, wk=wk, cos=cos, sin=sin)


def c1(shrink=1):
    return flux2_case(1, 64, 16, shrink=shrink)


def c2(shrink=1):
    return flux2_case(2, 512, 64, shrink=shrink, sigma=1.0 / np.sqrt(128.0))


def c5(shrink=1):
    return flux2_case(5, 512, 64, refs=2, shrink=shrink)


def c3(shrink=1):
    """Z-Image shaped CFG pair: 30 heads, [IMAGE 64x64 | CAPTION 256]; returns (cond, uncond)."""
    orc = O.oracle()
    g = max(int(round(64 / np.sqrt(shrink))), 1)
    cap = max(256 // shrink, 32)
    heads, dim = 30, 3840
    pos, mask_pad, ip, cp = orc.zimage_positions(img_seq=g * g, wt=g, cap_seq=cap)
    seq = ip + cp
    cos, sin = orc.zimage_gather(pos)
    st = orc.rng(SEED0 + 3)
    cond_buf = _fused(orc, st, seq, dim, dim, 3 * dim, 1.0 / np.sqrt(128.0))
    unc_buf = _fused(orc, st, seq, dim, dim, 3 * dim, 0.1)
    wq, wk = _weights(orc, st)
    lo = min(16, cap)
    length = lo + int(orc.rng_next(st) % (cap - lo + 1))
    key_mask = mask_pad.copy()
    key_mask[ip:] = (np.arange(cp) < length).astype(np.int32)
    common = dict(heads=heads, ldo=dim, wq=wq, wk=wk, cos=cos, sin=sin, eps=1e-5)
    cond = _case(name="C3-cond", buf=cond_buf, key_mask=None if ip == g * g else mask_pad, **common)
    unc = _case(name="C3-uncond", buf=unc_buf, key_mask=key_mask, **common)
    unc["valid_text"] = length
    return cond, unc


def c4(shrink=1):
    """Qwen3-4B shaped: causal GQA 32/8, split-half RoPE theta 1e6, right padding."""
    orc = O.oracle()
    seq = max(512 // shrink, 8)
    heads, kv = 32, 8
    st = orc.rng(SEED0 + 4)
    buf = _fused(orc, st, seq, heads * 128, kv * 128, (heads + 2 * kv) * 128, 1.0)
    wq, wk = _weights(orc, st)
    lo = min(8, seq)
    length = lo + int(orc.rng_next(st) % (seq - lo + 1))
    cos, sin = orc.qwen3_rope_table(seq, 128, 1e6)
    mask = (np.arange(seq) < length).astype(np.int32)
    case = _case(name="C4", buf=buf, heads=heads, kv_heads=kv, ldo=heads * 128, wq=wq, wk=wk, cos=cos,
                 sin=sin, causal=True, key_mask=mask, split_half=1)
    case["valid_len"] = length
    return case


def attention_flops(case):
    """4 * head_dim * sum over (head, query) of the number of valid keys."""
    seq = case["seq"]
    valid = np.ones(seq, dtype=np.int64) if case["key_mask"] is None else (np.asarray(case["key_mask"]) != 0).astype(np.int64)
    if case["causal"]:
        per_query = np.cumsum(valid)
    else:
        per_query = np.full(seq, valid.sum())
    return 4 * case["hd"] * case["heads"] * int(per_query.sum())


def norm_rope_bytes(seq, heads, hd=128):
    """Algorithmic bytes of one head_norm_rope call: x read + x written + both tables + w."""
    return 4 * seq * heads * hd + 2 * seq * (hd // 2) * 4 + hd * 4
