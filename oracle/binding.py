"""ctypes bindings of the CPU oracle libraries (test infrastructure only)."""
import ctypes as C
import glob
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
REF_TREE = "/root/reference"

_f = C.c_float
_i = C.c_int
_p = C.c_void_p


def build(with_ref=True):
    """Compile the oracle (and the reference library when its tree is present)."""
    subprocess.check_call(["make", "-s", "-C", HERE, "oracle"])
    if with_ref and os.path.isdir(REF_TREE):
        subprocess.check_call(["make", "-s", "-C", HERE, "ref"])


def _ptr(a):
    if a is None:
        return None
    assert isinstance(a, np.ndarray) and a.flags["C_CONTIGUOUS"], "need a C-contiguous ndarray"
    return a.ctypes.data_as(_p)


def _ints(v):
    return np.ascontiguousarray(np.asarray(v, dtype=np.int32))


def f32_to_bf16(a):
    """numpy float32 -> uint16 bf16 bit patterns, round to nearest even."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    out = np.empty(a.shape, dtype=np.uint16)
    oracle().lib.orc_f2bf_n(_ptr(out), _ptr(a), C.c_size_t(a.size))
    return out


def bf16_to_f32(a):
    a = np.ascontiguousarray(a, dtype=np.uint16)
    return (a.astype(np.uint32) << 16).view(np.float32)


class _RngState(C.Structure):
    _fields_ = [("s", C.c_uint64 * 4)]


class Oracle:
    """libiris_oracle.so: our fp32 restatement of the reference CPU path."""

    def __init__(self):
        path = os.path.join(HERE, "libiris_oracle.so")
        if not os.path.exists(path):
            build(with_ref=False)
        self.lib = C.CDLL(path)
        L = self.lib
        L.orc_rng_next.restype = C.c_uint64
        L.orc_rng_uniform.restype = _f
        L.orc_rng_normal.restype = _f
        L.orc_f2bf.restype = C.c_uint16
        L.orc_f2bf.argtypes = [_f]
        L.orc_bf2f.restype = _f
        L.orc_bf2f.argtypes = [C.c_uint16]
        L.orc_fast_expf.restype = _f
        L.orc_fast_expf.argtypes = [_f]

    # ---- seeded inputs ----
    def rng(self, seed):
        st = _RngState()
        self.lib.orc_rng_seed(C.byref(st), C.c_uint64(seed))
        return st

    def rng_next(self, st):
        return self.lib.orc_rng_next(C.byref(st))

    def rng_uniform(self, st):
        return self.lib.orc_rng_uniform(C.byref(st))

    def randn(self, st, n):
        out = np.empty(int(n), dtype=np.float32)
        self.lib.orc_randn(C.byref(st), _ptr(out), C.c_size_t(out.size))
        return out

    # ---- elementwise ----
    def fast_expf(self, x):
        return float(self.lib.orc_fast_expf(_f(x)))

    def softmax_rows(self, x):
        x = np.array(x, dtype=np.float32, order="C")
        self.lib.orc_softmax_rows(_ptr(x), _i(x.shape[0]), _i(x.shape[1]))
        return x

    def rms_norm_rows(self, x, w, eps):
        x = np.ascontiguousarray(x, dtype=np.float32)
        w = np.ascontiguousarray(w, dtype=np.float32)
        out = np.empty_like(x)
        self.lib.orc_rms_norm_rows(_ptr(out), _ptr(x), _ptr(w), _i(x.shape[0]), _i(x.shape[1]), _f(eps))
        return out

    # ---- rope application: x is [seq, heads, hd] f32, returned rotated ----
    def _rope(self, fn, x, cos_t, sin_t):
        x = np.array(x, dtype=np.float32, order="C")
        seq, heads, hd = x.shape
        cos_t = np.ascontiguousarray(cos_t, dtype=np.float32)
        sin_t = np.ascontiguousarray(sin_t, dtype=np.float32)
        fn(_ptr(x), _ptr(cos_t), _ptr(sin_t), _i(seq), _i(heads), _i(hd))
        return x

    def rope_pairs(self, x, c, s):
        return self._rope(self.lib.orc_rope_pairs, x, c, s)

    def rope_pairs_dup(self, x, c, s):
        return self._rope(self.lib.orc_rope_pairs_dup, x, c, s)

    def rope_split(self, x, c, s):
        return self._rope(self.lib.orc_rope_split, x, c, s)

    def rope_split_interleaved(self, x, freqs):
        x = np.array(x, dtype=np.float32, order="C")   # [batch, seq, heads, hd]
        b, seq, heads, hd = x.shape
        freqs = np.ascontiguousarray(freqs, dtype=np.float32)
        self.lib.orc_rope_split_interleaved(_ptr(x), _ptr(freqs), _i(b), _i(seq), _i(heads), _i(hd))
        return x

    def rope_freqs_interleaved(self, pos, dim, theta):
        pos = _ints(pos)
        out = np.empty((pos.size, dim // 2, 2), dtype=np.float32)
        self.lib.orc_rope_freqs_interleaved(_ptr(out), _ptr(pos), _i(pos.size), _i(dim), _f(theta))
        return out

    def head_norm_rope_bf16(self, x, ld, w, cos_t, sin_t, seq, heads, hd, eps, split_half, col0=0):
        """In-place device semantics on a uint16 buffer `x` viewed as rows of ld."""
        assert x.dtype == np.uint16 and x.flags["C_CONTIGUOUS"]
        base = x.reshape(-1)[col0:]
        w = np.ascontiguousarray(w, dtype=np.float32)
        cos_t = np.ascontiguousarray(cos_t, dtype=np.float32)
        sin_t = np.ascontiguousarray(sin_t, dtype=np.float32)
        self.lib.orc_head_norm_rope_bf16(C.c_void_p(base.ctypes.data), _i(ld), _ptr(w), _ptr(cos_t),
                                         _ptr(sin_t), _i(seq), _i(heads), _i(hd), _f(eps),
                                         _i(split_half))

    def head_norm_rope_f32(self, x, w, cos_t, sin_t, eps, split_half):
        x = np.array(x, dtype=np.float32, order="C")   # [seq, heads, hd]
        seq, heads, hd = x.shape
        w = np.ascontiguousarray(w, dtype=np.float32)
        cos_t = np.ascontiguousarray(cos_t, dtype=np.float32)
        sin_t = np.ascontiguousarray(sin_t, dtype=np.float32)
        self.lib.orc_head_norm_rope_f32(_ptr(x), _i(heads * hd), _ptr(w), _ptr(cos_t), _ptr(sin_t),
                                        _i(seq), _i(heads), _i(hd), _f(eps), _i(split_half))
        return x

    # ---- tables ----
    def flux2_rope_text(self, txt_seq, axis_dim=32, theta=2000.0):
        c = np.empty((txt_seq, 4 * axis_dim), dtype=np.float32)
        s = np.empty_like(c)
        self.lib.orc_flux2_rope_text(_ptr(c), _ptr(s), _i(txt_seq), _i(axis_dim), _f(theta))
        return c, s

    def flux2_rope_image(self, ph, pw, axis_dim=32, theta=2000.0, t_offset=-1):
        c = np.empty((ph * pw, 4 * axis_dim), dtype=np.float32)
        s = np.empty_like(c)
        self.lib.orc_flux2_rope_image(_ptr(c), _ptr(s), _i(ph), _i(pw), _i(axis_dim), _f(theta),
                                      _i(t_offset))
        return c, s

    def flux2_joint_tables(self, txt_seq, img_h, img_w, refs=(), axis_dim=32, theta=2000.0):
        rh, rw = _ints([r[0] for r in refs]), _ints([r[1] for r in refs])
        seq = txt_seq + img_h * img_w + sum(h * w for h, w in refs)
        c = np.empty((seq, 2 * axis_dim), dtype=np.float32)
        s = np.empty_like(c)
        self.lib.orc_flux2_joint_tables(_ptr(c), _ptr(s), _i(txt_seq), _i(img_h), _i(img_w),
                                        _ptr(rh), _ptr(rw), _i(len(refs)), _i(axis_dim), _f(theta))
        return c, s

    def zimage_axis_table(self, axis_dim, max_pos, theta=256.0):
        c = np.empty((max_pos, axis_dim // 2), dtype=np.float32)
        s = np.empty_like(c)
        self.lib.orc_zimage_axis_table(_ptr(c), _ptr(s), _i(axis_dim), _i(max_pos), _f(theta))
        return c, s

    def zimage_positions(self, img_seq, wt, cap_seq):
        ip = (img_seq + 31) // 32 * 32
        cp = (cap_seq + 31) // 32 * 32
        pos = np.empty((ip + cp, 3), dtype=np.int32)
        mask = np.empty(ip + cp, dtype=np.int32)
        self.lib.orc_zimage_positions(_ptr(pos), _ptr(mask), _i(img_seq), _i(wt), _i(cap_seq), None, None)
        return pos, mask, ip, cp

    def zimage_gather(self, pos, axes_dims=(32, 48, 48), axes_lens=(1024, 1024, 1024), theta=256.0):
        pos = np.ascontiguousarray(pos, dtype=np.int32)
        seq = pos.shape[0]
        half = sum(axes_dims) // 2
        c = np.empty((seq, half), dtype=np.float32)
        s = np.empty_like(c)
        self.lib.orc_zimage_gather(_ptr(c), _ptr(s), _ptr(pos), _i(seq), _ptr(_ints(axes_dims)),
                                   _ptr(_ints(axes_lens)), _f(theta))
        return c, s

    def flux3_joint_positions(self, txt_seq, img_h, img_w, refs=()):
        rh, rw = _ints([r[0] for r in refs]), _ints([r[1] for r in refs])
        seq = txt_seq + img_h * img_w + sum(h * w for h, w in refs)
        pos = np.empty((seq, 4), dtype=np.float32)
        self.lib.orc_flux3_joint_positions(_ptr(pos), _i(txt_seq), _i(img_h), _i(img_w), _ptr(rh),
                                           _ptr(rw), _i(len(refs)))
        return pos

    def flux3_rope_rows(self, pos4, axes_dim=(32, 32, 32, 32), theta=10000.0):
        pos4 = np.ascontiguousarray(pos4, dtype=np.float32)
        seq = pos4.shape[0]
        half = sum(axes_dim) // 2
        c = np.empty((seq, half), dtype=np.float32)
        s = np.empty_like(c)
        self.lib.orc_flux3_rope_rows(_ptr(c), _ptr(s), _ptr(pos4), _i(seq), _ptr(_ints(axes_dim)), _f(theta))
        return c, s

    def qwen3_rope_table(self, seq, head_dim=128, theta=1e6, mask=None, pad_at_one=False):
        c = np.empty((seq, head_dim // 2), dtype=np.float32)
        s = np.empty_like(c)
        m = _ints(mask) if mask is not None else None
        self.lib.orc_qwen3_rope_table(_ptr(c), _ptr(s), _ptr(m), _i(seq), _i(head_dim), _f(theta),
                                      _i(1 if pad_at_one else 0))
        return c, s

    # ---- attention ----
    def attention_naive(self, Q, K, V, scale):
        Q, K, V = (np.ascontiguousarray(a, dtype=np.float32) for a in (Q, K, V))
        b, h, sq, d = Q.shape
        sk = K.shape[2]
        out = np.empty_like(Q)
        self.lib.orc_attention_naive(_ptr(out), _ptr(Q), _ptr(K), _ptr(V), _i(b), _i(h), _i(sq),
                                     _i(sk), _i(d), _f(scale))
        return out

    def attention_flash(self, Q, K, V, heads, scale):
        Q, K, V = (np.ascontiguousarray(a, dtype=np.float32) for a in (Q, K, V))
        sq, sk = Q.shape[0], K.shape[0]
        hd = Q.shape[1] // heads
        out = np.empty_like(Q)
        self.lib.orc_attention_flash(_ptr(out), _ptr(Q), _ptr(K), _ptr(V), _i(sq), _i(sk), _i(heads),
                                     _i(hd), _f(scale))
        return out

    def attention_strided(self, q, k, v, heads, kv_heads, scale, causal=False, key_mask=None):
        """q [seq_q, heads*hd], k/v [seq_k, kv_heads*hd] f32 -> [seq_q, heads*hd]."""
        q, k, v = (np.ascontiguousarray(a, dtype=np.float32) for a in (q, k, v))
        sq, sk = q.shape[0], k.shape[0]
        hd = q.shape[1] // heads
        out = np.empty_like(q)
        m = _ints(key_mask) if key_mask is not None else None
        self.lib.orc_attention_strided(_ptr(out), _i(q.shape[1]), _ptr(q), _ptr(k), _ptr(v),
                                       _i(q.shape[1]), _i(k.shape[1]), _i(sq), _i(sk), _i(heads),
                                       _i(kv_heads), _i(hd), _f(scale), _i(int(causal)), _ptr(m))
        return out

    def attention_bf16(self, buf, ldi, q_col, k_col, v_col, seq_q, seq_k, heads, kv_heads, hd, scale,
                       causal=False, key_mask=None, rows=None):
        """bf16 (uint16) buffer of rows `ldi`; q/k/v start at the given columns.
        Returns f32 [seq_q or len(rows), heads*hd]."""
        assert buf.dtype == np.uint16 and buf.flags["C_CONTIGUOUS"]
        flat = buf.reshape(-1)
        addr = lambda col: C.c_void_p(flat.ctypes.data + 2 * col)
        m = _ints(key_mask) if key_mask is not None else None
        if rows is None:
            out = np.empty((seq_q, heads * hd), dtype=np.float32)
            self.lib.orc_attention_bf16(_ptr(out), _i(heads * hd), addr(q_col), addr(k_col), addr(v_col),
                                        _i(ldi), _i(seq_q), _i(seq_k), _i(heads), _i(kv_heads), _i(hd),
                                        _f(scale), _i(int(causal)), _ptr(m))
        else:
            rows = _ints(rows)
            out = np.empty((rows.size, heads * hd), dtype=np.float32)
            self.lib.orc_attention_bf16_rows(_ptr(out), addr(q_col), addr(k_col), addr(v_col), _i(ldi),
                                             _ptr(rows), _i(rows.size), _i(seq_k), _i(heads),
                                             _i(kv_heads), _i(hd), _f(scale), _i(int(causal)), _ptr(m))
        return out


    # ---- the other device operators (iris_oracle_ops.c) ----
    def dev_linear(self, x, W):
        """x bf16 [rows, in], W bf16 [out, in] -> f32 [rows, out]."""
        rows, k = x.shape
        out = np.empty((rows, W.shape[0]), np.float32)
        self.lib.orc_dev_linear(_ptr(out), _ptr(x), _ptr(W), _i(rows), _i(k), _i(W.shape[0]))
        return out

    def dev_layer_norm_mod(self, x, shift, scale, eps):
        out = np.empty(x.shape, np.uint16)
        self.lib.orc_dev_layer_norm_mod(_ptr(out), _ptr(x), _ptr(shift), _ptr(scale), _i(x.shape[0]), _i(x.shape[1]), _f(eps))
        return out

    def dev_rms_norm_mod(self, x, w, scale, eps):
        out = np.empty(x.shape, np.uint16)
        self.lib.orc_dev_rms_norm_mod(_ptr(out), _ptr(x), _ptr(w), _ptr(scale), _i(x.shape[0]), _i(x.shape[1]), _f(eps))
        return out

    def dev_rms_norm_residual(self, x, a, w, gate, eps):
        x = x.copy()
        self.lib.orc_dev_rms_norm_residual(_ptr(x), _ptr(a), _ptr(w), _ptr(gate), _i(x.shape[0]), _i(x.shape[1]), _f(eps))
        return x

    def dev_swiglu(self, gate_up, cols, ldo=None):
        """gate_up bf16 [rows, ldi] with gate at column 0 and up at column `cols`."""
        rows, ldi = gate_up.shape
        ldo = ldo or cols
        out = np.zeros((rows, ldo), np.uint16)
        flat = gate_up.reshape(-1)
        self.lib.orc_dev_swiglu(_ptr(out), _i(ldo), _ptr(flat), C.c_void_p(flat.ctypes.data + 2 * cols), _i(ldi), _i(rows), _i(cols))
        return out

    def dev_residual(self, x, a, gate):
        x = x.copy()
        self.lib.orc_dev_residual(_ptr(x), _ptr(a), _ptr(gate), _i(x.shape[0]), _i(x.shape[1]))
        return x

    def dev_silu(self, x):
        x = np.ascontiguousarray(x, np.float32).copy()
        self.lib.orc_dev_silu(_ptr(x), C.c_size_t(x.size))
        return x

    def dev_add(self, x, a):
        x = x.copy()
        self.lib.orc_dev_add(_ptr(x), _ptr(a), C.c_size_t(x.size))
        return x

    def dev_add_bias(self, y, bias):
        y = y.copy()
        self.lib.orc_dev_add_bias(_ptr(y), _ptr(bias), _i(y.shape[0]), _i(y.shape[1]))
        return y

    def dev_fill_rows(self, row, rows):
        out = np.empty((rows, row.size), np.float32)
        self.lib.orc_dev_fill_rows(_ptr(out), _ptr(row), _i(rows), _i(row.size))
        return out

    def dev_conv2d(self, img, w, bias, h, width, k, stride, pad_before, pad_after):
        """img f32 [h*width, cin], w bf16 [cout, k*k*cin] -> f32 [oh*ow, cout]."""
        cin, cout = img.shape[1], w.shape[0]
        oh = (h + pad_before + pad_after - k) // stride + 1
        ow = (width + pad_before + pad_after - k) // stride + 1
        out = np.empty((oh * ow, cout), np.float32)
        self.lib.orc_dev_conv2d(_ptr(out), _ptr(img), _ptr(w), _ptr(bias), _i(h), _i(width), _i(cin), _i(cout), _i(k),
                                _i(stride), _i(pad_before), _i(pad_after))
        return out

    def dev_group_norm(self, img, gamma, beta, groups, eps, silu):
        out = np.empty(img.shape, np.float32)
        self.lib.orc_dev_group_norm(_ptr(out), _ptr(img), _ptr(gamma), _ptr(beta), _i(img.shape[0]), _i(img.shape[1]),
                                    _i(groups), _f(eps), _i(int(silu)))
        return out

    def dev_upsample2x(self, img, h, width):
        out = np.empty((4 * h * width, img.shape[1]), np.float32)
        self.lib.orc_dev_upsample2x(_ptr(out), _ptr(img), _i(h), _i(width), _i(img.shape[1]))
        return out


class CpuBaseline:
    """libiris_cpu_baseline.so: the reference's BLAS-build CPU structure, for timing."""

    def __init__(self):
        path = os.path.join(HERE, "libiris_cpu_baseline.so")
        if not os.path.exists(path):
            build(with_ref=False)
        self.lib = C.CDLL(path)
        self.lib.cpu_baseline_provider.restype = C.c_char_p
        self.bound = bool(self.lib.cpu_baseline_bind_blas(None, b""))
        if not self.bound:
            import importlib.util
            for pkg, prefix in (("scipy", b"scipy_"), ("numpy", b"scipy_")):
                spec = importlib.util.find_spec(pkg)
                if not spec or not spec.submodule_search_locations:
                    continue
                root = os.path.dirname(list(spec.submodule_search_locations)[0])
                # the LP64 build only: the 64-bit-index build has other symbol names
                cands = [p for p in sorted(glob.glob(os.path.join(root, pkg + ".libs", "libscipy_openblas*.so")))
                         if "openblas64" not in os.path.basename(p)]
                for cand in cands:
                    if self.lib.cpu_baseline_bind_blas(cand.encode(), prefix):
                        self.bound = True
                        break
                if self.bound:
                    break

    @property
    def provider(self):
        return self.lib.cpu_baseline_provider().decode()

    def online_cpus(self):
        return int(self.lib.cpu_baseline_online_cpus())

    def threads_for(self, heads, limit=0):
        return int(self.lib.cpu_baseline_threads(_i(heads), _i(limit)))

    def attention(self, q, k, v, heads, kv_heads, scale, causal=False, key_mask=None, q_chunk=0,
                  threads=0):
        q, k, v = (np.ascontiguousarray(a, dtype=np.float32) for a in (q, k, v))
        sq, sk = q.shape[0], k.shape[0]
        hd = q.shape[1] // heads
        out = np.empty_like(q)
        m = _ints(key_mask) if key_mask is not None else None
        nt = self.lib.cpu_baseline_attention(_ptr(out), _i(q.shape[1]), _ptr(q), _ptr(k), _ptr(v),
                                             _i(q.shape[1]), _i(k.shape[1]), _i(sq), _i(sk), _i(heads),
                                             _i(kv_heads), _i(hd), _f(scale), _i(int(causal)), _ptr(m),
                                             _i(q_chunk), _i(threads))
        if nt < 0:
            raise MemoryError("cpu baseline: score buffer allocation failed")
        return out, nt

    def norm_rope(self, x, w, cos_t, sin_t, eps, split_half):
        x = np.array(x, dtype=np.float32, order="C")   # [seq, heads, hd]
        seq, heads, hd = x.shape
        self.lib.cpu_baseline_norm_rope(_ptr(x), _ptr(np.ascontiguousarray(w, dtype=np.float32)),
                                        _ptr(np.ascontiguousarray(cos_t, dtype=np.float32)),
                                        _ptr(np.ascontiguousarray(sin_t, dtype=np.float32)),
                                        _i(seq), _i(heads), _i(hd), _f(eps), _i(split_half))
        return x


class Reference:
    """_ref/libiris_ref.so: the reference's own C sources compiled in place
    (generic build) plus include-harness wrappers around its static functions.
    Exists only where the reference tree was present at build time."""

    def __init__(self, variant=""):
        path = os.path.join(HERE, "_ref", "libiris_ref%s.so" % variant)
        if not os.path.exists(path):
            raise FileNotFoundError(path)
        self.lib = C.CDLL(path)
        L = self.lib
        L.iris_random_uniform.restype = _f
        L.iris_random_normal.restype = _f


_singletons = {}


def _get(cls):
    if cls not in _singletons:
        _singletons[cls] = cls()
    return _singletons[cls]


def oracle():
    return _get(Oracle)


def cpu_baseline():
    return _get(CpuBaseline)


def reference(ieee=False):
    """The compiled reference, or None when it was not built. ieee=True picks
    the build of the same sources without -ffast-math (scalar libm calls)."""
    key = ("ref", ieee)
    try:
        if key not in _singletons:
            _singletons[key] = Reference("_ieee" if ieee else "")
        return _singletons[key]
    except (FileNotFoundError, OSError):
        return None
