"""Thin numpy wrappers over the compiled reference (oracle/_ref/libiris_ref.so).

Used by the live oracle-vs-reference tests and by golden/make_golden.py.
Everything here calls the reference's own code, compiled where it lies.
"""
import ctypes as C

import numpy as np

_f, _i, _p = C.c_float, C.c_int, C.c_void_p


def _ptr(a):
    return None if a is None else a.ctypes.data_as(_p)


def _ints(v):
    return np.ascontiguousarray(np.asarray(v, dtype=np.int32))


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def rng_u64(ref, seed, n):
    """Raw generator outputs recovered from iris_random_uniform (53-bit mantissa
    is lost in the float return), so compare uniforms and normals instead."""
    ref.lib.iris_rng_seed(C.c_uint64(seed))
    return np.array([ref.lib.iris_random_uniform() for _ in range(n)], dtype=np.float32)


def randn(ref, seed, n):
    ref.lib.iris_rng_seed(C.c_uint64(seed))
    out = np.empty(n, dtype=np.float32)
    ref.lib.iris_randn(_ptr(out), _i(n))
    return out


def softmax_rows(ref, x):
    x = np.array(x, dtype=np.float32, order="C")
    ref.lib.iris_softmax_cpu(_ptr(x), _i(x.shape[0]), _i(x.shape[1]))
    return x


def rms_norm(ref, x, w, eps):
    x, w = _f32(x), _f32(w)
    out = np.empty_like(x)
    ref.lib.iris_rms_norm(_ptr(out), _ptr(x), _ptr(w), _i(x.shape[0]), _i(x.shape[1]), _f(eps))
    return out


def attention_naive(ref, Q, K, V, scale):
    Q, K, V = _f32(Q), _f32(K), _f32(V)
    b, h, sq, d = Q.shape
    out = np.empty_like(Q)
    ref.lib.iris_attention(_ptr(out), _ptr(Q), _ptr(K), _ptr(V), _i(b), _i(h), _i(sq), _i(K.shape[2]),
                           _i(d), _f(scale))
    return out


def attention_flash(ref, Q, K, V, heads, scale):
    Q, K, V = _f32(Q), _f32(K), _f32(V)
    out = np.empty_like(Q)
    ref.lib.iris_flash_attention(_ptr(out), _ptr(Q), _ptr(K), _ptr(V), _i(Q.shape[0]), _i(K.shape[0]),
                                 _i(heads), _i(Q.shape[1] // heads), _f(scale))
    return out


def apply_rope_interleaved(ref, x, freqs):
    x = np.array(x, dtype=np.float32, order="C")
    b, seq, heads, hd = x.shape
    freqs = _f32(freqs)
    ref.lib.iris_apply_rope(_ptr(x), _ptr(freqs), _i(b), _i(seq), _i(heads), _i(hd))
    return x


def rope_freqs(ref, pos, dim, theta):
    pos = _ints(pos)
    out = np.empty((pos.size, dim // 2, 2), dtype=np.float32)
    ref.lib.iris_compute_rope_freqs(_ptr(out), _ptr(pos), _i(pos.size), _i(dim), _f(theta))
    return out


# ---- FLUX.2 statics ----
def flux2_rope_text(ref, txt_seq, axis_dim=32, theta=2000.0):
    c = np.empty((txt_seq, 4 * axis_dim), dtype=np.float32)
    s = np.empty_like(c)
    ref.lib.ref_flux2_rope_text(_ptr(c), _ptr(s), _i(txt_seq), _i(axis_dim), _f(theta))
    return c, s


def flux2_rope_2d(ref, ph, pw, axis_dim=32, theta=2000.0, t_offset=None):
    c = np.empty((ph * pw, 4 * axis_dim), dtype=np.float32)
    s = np.empty_like(c)
    if t_offset is None:
        ref.lib.ref_flux2_rope_2d(_ptr(c), _ptr(s), _i(ph), _i(pw), _i(axis_dim), _f(theta))
    else:
        ref.lib.ref_flux2_rope_2d_t(_ptr(c), _ptr(s), _i(ph), _i(pw), _i(axis_dim), _f(theta), _i(t_offset))
    return c, s


def flux2_joint_compact(ref, txt_seq, img_h, img_w, refs=(), axis_dim=32, theta=2000.0):
    """What forward_dev_flux uploads: [TEXT | IMAGE | REFS] tables, even entries kept."""
    cs, ss = [], []
    c, s = flux2_rope_text(ref, txt_seq, axis_dim, theta); cs.append(c); ss.append(s)
    c, s = flux2_rope_2d(ref, img_h, img_w, axis_dim, theta); cs.append(c); ss.append(s)
    for i, (h, w) in enumerate(refs):
        c, s = flux2_rope_2d(ref, h, w, axis_dim, theta, t_offset=10 * (i + 1)); cs.append(c); ss.append(s)
    c, s = np.concatenate(cs), np.concatenate(ss)
    return np.ascontiguousarray(c[:, 0::2]), np.ascontiguousarray(s[:, 0::2])


def flux2_apply_rope_2d(ref, x, c, s):
    x = np.array(x, dtype=np.float32, order="C")
    seq, heads, hd = x.shape
    ref.lib.ref_flux2_apply_rope_2d(_ptr(x), _ptr(_f32(c)), _ptr(_f32(s)), _i(seq), _i(heads), _i(hd), _i(hd // 4))
    return x


def flux2_qk_norm(ref, q, k, qw, kw, eps):
    q = np.array(q, dtype=np.float32, order="C")
    k = np.array(k, dtype=np.float32, order="C")
    seq, heads, hd = q.shape
    ref.lib.ref_flux2_apply_qk_norm(_ptr(q), _ptr(k), _ptr(_f32(qw)), _ptr(_f32(kw)), _i(seq), _i(heads), _i(hd), _f(eps))
    return q, k


# ---- FLUX.3 statics ----
def flux3_joint_rope(ref, txt_seq, img_h, img_w, refs=(), head_dim=128, theta=10000.0):
    rh, rw = _ints([r[0] for r in refs]), _ints([r[1] for r in refs])
    seq = txt_seq + img_h * img_w + sum(h * w for h, w in refs)
    c = np.empty((seq, head_dim // 2), dtype=np.float32)
    s = np.empty_like(c)
    n = ref.lib.ref_flux3_joint_rope(_ptr(c), _ptr(s), _i(head_dim), _f(theta), _i(txt_seq), _i(img_h), _i(img_w),
                                     _ptr(rh), _ptr(rw), _i(len(refs)))
    assert n == seq
    return c, s


def flux3_head_rms_norm(ref, x, w, eps):
    x = np.array(x, dtype=np.float32, order="C")
    seq, heads, hd = x.shape
    ref.lib.ref_flux3_head_rms_norm(_ptr(x), _ptr(_f32(w)), _i(seq), _i(heads), _i(hd), _f(eps))
    return x


def flux3_apply_rope(ref, x, c, s):
    x = np.array(x, dtype=np.float32, order="C")
    seq, heads, hd = x.shape
    ref.lib.ref_flux3_apply_rope(_ptr(x), _ptr(_f32(c)), _ptr(_f32(s)), _i(seq), _i(heads), _i(hd))
    return x


def flux3_attention(ref, q, k, v, heads):
    q, k, v = _f32(q), _f32(k), _f32(v)
    out = np.empty_like(q)
    ref.lib.ref_flux3_attention(_ptr(out), _ptr(q), _ptr(k), _ptr(v), _i(q.shape[0]), _i(heads), _i(q.shape[1] // heads))
    return out


# ---- Z-Image statics ----
def zi_axis_table(ref, ax, axes_dims=(32, 48, 48), axes_lens=(1024, 1024, 1024), theta=256.0):
    c = np.empty((axes_lens[ax], axes_dims[ax] // 2), dtype=np.float32)
    s = np.empty_like(c)
    ref.lib.ref_zi_axis_table(_ptr(c), _ptr(s), _i(ax), _ptr(_ints(axes_dims)), _ptr(_ints(axes_lens)), _f(theta))
    return c, s


def zi_apply_rope(ref, x, pos, axes_dims=(32, 48, 48), axes_lens=(1024, 1024, 1024), theta=256.0):
    x = np.array(x, dtype=np.float32, order="C")
    seq, heads, hd = x.shape
    pos = np.ascontiguousarray(pos, dtype=np.int32)
    ref.lib.ref_zi_apply_rope(_ptr(x), _ptr(pos), _i(seq), _i(heads), _ptr(_ints(axes_dims)), _ptr(_ints(axes_lens)), _f(theta))
    return x


def zi_qk_norm(ref, x, w, eps):
    x = np.array(x, dtype=np.float32, order="C")
    seq, heads, hd = x.shape
    ref.lib.ref_zi_qk_norm(_ptr(x), _ptr(_f32(w)), _i(seq), _i(heads), _i(hd), _f(eps))
    return x


def zi_attention(ref, x, wq, wk, wv, wo, nq, nk, pos, mask, n_heads, axes_dims, axes_lens=(1024, 1024, 1024), theta=256.0):
    x = _f32(x)
    seq, dim = x.shape
    out = np.empty_like(x)
    wq, wk, wv, wo, nq, nk = (np.array(a, dtype=np.float32, order="C") for a in (wq, wk, wv, wo, nq, nk))
    pos = np.ascontiguousarray(pos, dtype=np.int32)
    m = _ints(mask) if mask is not None else None
    ref.lib.ref_zi_attention(_ptr(out), _ptr(x), _ptr(wq), _ptr(wk), _ptr(wv), _ptr(wo), _ptr(nq), _ptr(nk),
                             _ptr(pos), _ptr(m), _i(seq), _i(n_heads), _ptr(_ints(axes_dims)),
                             _ptr(_ints(axes_lens)), _f(theta))
    return out


# ---- Qwen3 statics ----
def qwen3_rope_table(ref, seq, head_dim=128, theta=1e6, mask=None, flux3_mode=False):
    c = np.empty((seq, head_dim // 2), dtype=np.float32)
    s = np.empty_like(c)
    m = _ints(mask) if mask is not None else None
    ref.lib.ref_qwen3_rope_table(_ptr(c), _ptr(s), _ptr(m), _i(seq), _i(head_dim), _f(theta), _i(int(flux3_mode)))
    return c, s


def qwen3_attention(ref, x, wq, wk, wv, nq, nk, mask, heads, kv_heads, hd, theta=1e6):
    x = _f32(x)
    seq, hidden = x.shape
    wq, wk, wv, nq, nk = (np.array(a, dtype=np.float32, order="C") for a in (wq, wk, wv, nq, nk))
    attn = np.empty((seq, heads * hd), dtype=np.float32)
    q = np.empty((seq, heads * hd), dtype=np.float32)
    k = np.empty((seq, kv_heads * hd), dtype=np.float32)
    v = np.empty((seq, kv_heads * hd), dtype=np.float32)
    m = _ints(mask) if mask is not None else None
    ref.lib.ref_qwen3_attention(_ptr(attn), _ptr(q), _ptr(k), _ptr(v), _ptr(x), _ptr(wq), _ptr(wk), _ptr(wv),
                                _ptr(nq), _ptr(nk), _ptr(m), _i(seq), _i(hidden), _i(heads), _i(kv_heads), _i(hd),
                                _f(theta))
    return attn, q, k, v
