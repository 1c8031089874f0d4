"""numpy mirror of include/iris_rope.h: the rotary-table builders of libiris_dev.so.

Host builders need no GPU (the functions are plain C + libm inside the same
library); the `dev_*` forms take an `IrisDev` and return the table expanded on
the device, downloaded. Used by tests and the benchmark only.
"""
import ctypes as C

import numpy as np

from . import IrisDev, load

_vp = C.c_void_p


def _p(a):
    return None if a is None else a.ctypes.data_as(_vp)


def _ints(v):
    return None if v is None else np.ascontiguousarray(v, dtype=np.int32)


def _refs(refs):
    h = _ints([r[0] for r in refs])
    w = _ints([r[1] for r in refs])
    return h, w, len(refs)


class RopeTables:
    def __init__(self, lib=None):
        self.lib = lib if lib is not None else load()

    # ---- positions
    def joint_rows(self, txt_seq, img_h, img_w, refs=()):
        h, w, n = _refs(refs)
        return self.lib.iris_rope_joint_rows(txt_seq, img_h, img_w, _p(h), _p(w), n)

    def flux2_positions(self, txt_seq, img_h, img_w, refs=(), ref_t=None):
        h, w, n = _refs(refs)
        pos = np.empty((self.joint_rows(txt_seq, img_h, img_w, refs), 4), np.int32)
        self.lib.iris_rope_flux2_positions(_p(pos), txt_seq, img_h, img_w, _p(h), _p(w), _p(_ints(ref_t)), n)
        return pos

    def flux3_positions(self, txt_seq, img_h, img_w, refs=()):
        h, w, n = _refs(refs)
        pos = np.empty((self.joint_rows(txt_seq, img_h, img_w, refs), 4), np.float32)
        self.lib.iris_rope_flux3_positions(_p(pos), txt_seq, img_h, img_w, _p(h), _p(w), n)
        return pos

    def zimage_positions(self, img_seq, wt, cap_seq):
        ip, cp = (img_seq + 31) // 32 * 32, (cap_seq + 31) // 32 * 32
        pos, mask = np.empty((ip + cp, 3), np.int32), np.empty(ip + cp, np.int32)
        a, b = C.c_int(), C.c_int()
        self.lib.iris_rope_zimage_positions(_p(pos), _p(mask), img_seq, wt, cap_seq, C.byref(a), C.byref(b))
        assert (a.value, b.value) == (ip, cp)
        return pos, mask, ip, cp

    # ---- host tables
    @staticmethod
    def _out(rows, half):
        return np.empty((rows, half), np.float32), np.empty((rows, half), np.float32)

    def expand_i32(self, pos, axis_dims, theta, axis_lens=None):
        pos, dims = _ints(pos), _ints(axis_dims)
        pos = pos.reshape(-1, len(dims))
        c, s = self._out(len(pos), int(dims.sum()) // 2 if (dims % 2 == 0).all() else 0)
        rc = self.lib.iris_rope_expand_i32(_p(c), _p(s), _p(pos), len(pos), len(dims), _p(dims), _p(_ints(axis_lens)),
                                           theta)
        return rc, c, s

    def expand_f64(self, pos, axis_dims, theta):
        pos, dims = np.ascontiguousarray(pos, np.float32), _ints(axis_dims)
        pos = pos.reshape(-1, len(dims))
        c, s = self._out(len(pos), int(dims.sum()) // 2)
        rc = self.lib.iris_rope_expand_f64(_p(c), _p(s), _p(pos), len(pos), len(dims), _p(dims), theta)
        return rc, c, s

    def flux2_tables(self, txt_seq, img_h, img_w, refs=(), ref_t=None, axis_dim=32, theta=2000.0):
        h, w, n = _refs(refs)
        c, s = self._out(self.joint_rows(txt_seq, img_h, img_w, refs), 2 * axis_dim)
        rc = self.lib.iris_rope_flux2_tables(_p(c), _p(s), txt_seq, img_h, img_w, _p(h), _p(w), _p(_ints(ref_t)), n,
                                             axis_dim, theta)
        assert rc == 0
        return c, s

    def flux3_tables(self, txt_seq, img_h, img_w, refs=(), axes_dim=(32, 32, 32, 32), theta=2000.0):
        h, w, n = _refs(refs)
        dims = _ints(axes_dim)
        c, s = self._out(self.joint_rows(txt_seq, img_h, img_w, refs), int(dims.sum()) // 2)
        rc = self.lib.iris_rope_flux3_tables(_p(c), _p(s), txt_seq, img_h, img_w, _p(h), _p(w), n, _p(dims), theta)
        assert rc == 0
        return c, s

    def zimage_tables(self, pos3, axes_dims=(32, 48, 48), axes_lens=(1536, 512, 512), theta=256.0):
        pos3, dims, lens = _ints(pos3), _ints(axes_dims), _ints(axes_lens)
        c, s = self._out(len(pos3), int(dims.sum()) // 2)
        rc = self.lib.iris_rope_zimage_tables(_p(c), _p(s), _p(pos3), len(pos3), _p(dims), _p(lens), theta)
        assert rc == 0
        return c, s

    def qwen3_tables(self, seq, head_dim=128, theta=1e6, mask=None, pad_at_one=False):
        c, s = self._out(seq, head_dim // 2)
        rc = self.lib.iris_rope_qwen3_tables(_p(c), _p(s), _p(_ints(mask)), seq, head_dim, theta, int(pad_at_one))
        assert rc == 0
        return c, s


    # ---- the dictionary the device entries upload (internal symbol; for the tests of that path)
    def dictionary(self, pos, axis_dims, theta, axis_lens=None, use_double=False):
        """(values, index): distinct (axis, position) rows and one offset per (row, axis)."""
        dims, lens = _ints(axis_dims), _ints(axis_lens)
        pos = (np.ascontiguousarray(pos, np.float32) if use_double else _ints(pos)).reshape(-1, len(dims))
        fn = self.lib.iris_rope_dictionary_
        fn.restype = C.c_int
        fn.argtypes = [_vp, C.c_int, C.c_int, C.c_int, _vp, _vp, C.c_float, C.POINTER(_vp), C.POINTER(C.c_size_t),
                       C.POINTER(_vp)]
        values, index, n = _vp(), _vp(), C.c_size_t()
        rc = fn(_p(pos), int(use_double), len(pos), len(dims), _p(dims), _p(lens), theta, C.byref(values), C.byref(n),
                C.byref(index))
        if rc != 0:
            return rc, None, None
        libc = C.CDLL(None)
        libc.free.argtypes = [_vp]
        v = np.ctypeslib.as_array(C.cast(values, C.POINTER(C.c_float)), shape=(max(n.value, 1),))[:n.value].copy()
        i = np.ctypeslib.as_array(C.cast(index, C.POINTER(C.c_uint32)), shape=(max(pos.size, 1),))[:pos.size].copy()
        libc.free(values); libc.free(index)
        return 0, v, i.reshape(pos.shape)

    @staticmethod
    def expand_dictionary(values, index, axis_dims):
        """What the device kernel does, in numpy."""
        cos_t, sin_t = [], []
        for a, d in enumerate(axis_dims):
            n = d // 2
            at = index[:, a].astype(np.int64)[:, None] + np.arange(n)[None, :]
            cos_t.append(values[at]); sin_t.append(values[at + n])
        return np.concatenate(cos_t, axis=1), np.concatenate(sin_t, axis=1)


class DevRopeTables(RopeTables):
    """The same tables written by the device kernel; each call returns them downloaded."""

    def __init__(self, dev: IrisDev):
        super().__init__(dev.lib)
        self.dev = dev

    def _run(self, rows, half, call):
        n = rows * half * 4
        dc, ds = self.lib.iris_dev_alloc(n), self.lib.iris_dev_alloc(n)
        try:
            call(dc, ds)
            self.dev.check()
            return self.dev.to_host(dc, (rows, half), np.float32), self.dev.to_host(ds, (rows, half), np.float32)
        finally:
            self.lib.iris_dev_free(dc)
            self.lib.iris_dev_free(ds)

    def dev_expand_i32(self, pos, axis_dims, theta, axis_lens=None):
        pos, dims, lens = _ints(pos), _ints(axis_dims), _ints(axis_lens)
        pos = pos.reshape(-1, len(dims))
        return self._run(len(pos), int(dims.sum()) // 2, lambda c, s: self.lib.iris_dev_rope_expand_i32(
            c, s, _p(pos), len(pos), len(dims), _p(dims), _p(lens), theta))

    def dev_expand_f64(self, pos, axis_dims, theta):
        pos, dims = np.ascontiguousarray(pos, np.float32), _ints(axis_dims)
        pos = pos.reshape(-1, len(dims))
        return self._run(len(pos), int(dims.sum()) // 2, lambda c, s: self.lib.iris_dev_rope_expand_f64(
            c, s, _p(pos), len(pos), len(dims), _p(dims), theta))

    def dev_flux2_tables(self, txt_seq, img_h, img_w, refs=(), ref_t=None, axis_dim=32, theta=2000.0):
        h, w, n = _refs(refs)
        t = _ints(ref_t)
        return self._run(self.joint_rows(txt_seq, img_h, img_w, refs), 2 * axis_dim,
                         lambda c, s: self.lib.iris_dev_rope_flux2_tables(c, s, txt_seq, img_h, img_w, _p(h), _p(w),
                                                                          _p(t), n, axis_dim, theta))

    def dev_flux3_tables(self, txt_seq, img_h, img_w, refs=(), axes_dim=(32, 32, 32, 32), theta=2000.0):
        h, w, n = _refs(refs)
        dims = _ints(axes_dim)
        return self._run(self.joint_rows(txt_seq, img_h, img_w, refs), int(dims.sum()) // 2,
                         lambda c, s: self.lib.iris_dev_rope_flux3_tables(c, s, txt_seq, img_h, img_w, _p(h), _p(w),
                                                                          n, _p(dims), theta))

    def dev_zimage_tables(self, pos3, axes_dims=(32, 48, 48), axes_lens=(1536, 512, 512), theta=256.0):
        pos3, dims, lens = _ints(pos3), _ints(axes_dims), _ints(axes_lens)
        return self._run(len(pos3), int(dims.sum()) // 2, lambda c, s: self.lib.iris_dev_rope_zimage_tables(
            c, s, _p(pos3), len(pos3), _p(dims), _p(lens), theta))

    def dev_qwen3_tables(self, seq, head_dim=128, theta=1e6, mask=None, pad_at_one=False):
        m = _ints(mask)
        return self._run(seq, head_dim // 2, lambda c, s: self.lib.iris_dev_rope_qwen3_tables(
            c, s, _p(m), seq, head_dim, theta, int(pad_at_one)))
