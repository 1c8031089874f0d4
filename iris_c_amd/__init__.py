"""MI355X-native attention hot path of iris.c behind the reference's C device API.

The product is `libiris_dev.so` (C ABI declared in include/iris_dev.h, built by
`make rocm`). This module is only a ctypes mirror of that ABI for tests and
benchmarks: same names, same argument order. It has no CPU fallback: loading
fails loudly when the library has not been built.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
LIB_PATH = os.path.join(HERE, "libiris_dev.so")

_vp, _i, _f, _sz = C.c_void_p, C.c_int, C.c_float, C.c_size_t

# name -> (restype, argtypes); the exported C ABI, one entry per declaration of include/iris_dev.h
# and include/iris_rope.h
ABI = {
    "iris_dev_init": (_i, []),
    "iris_dev_available": (_i, []),
    "iris_dev_name": (C.c_char_p, []),
    "iris_dev_cleanup": (None, []),
    "iris_dev_alloc": (_vp, [_sz]),
    "iris_dev_free": (None, [_vp]),
    "iris_dev_upload": (None, [_vp, _vp, _sz]),
    "iris_dev_download": (None, [_vp, _vp, _sz]),
    "iris_dev_upload_2d": (None, [_vp, _sz, _vp, _sz, _sz, _sz]),
    "iris_dev_sync": (None, []),
    "iris_dev_head_norm_rope": (None, [_vp, _i, _vp, _vp, _vp, _i, _i, _i, _f, _i]),
    "iris_dev_attention": (None, [_vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _f, _i, _vp]),
    "iris_dev_attention_qnorm": (None, [_vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _f, _i, _vp,
                                        _vp, _vp, _vp, _f, _i]),
    "iris_dev_f32_to_bf16": (None, [_vp, _vp, _sz]),
    "iris_dev_linear_f32": (None, [_vp, _vp, _vp, _i, _i, _i]),
    "iris_dev_linear_bf16": (None, [_vp, _vp, _vp, _i, _i, _i]),
    "iris_dev_linear_bf16_qknorm": (None, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _f, _i]),
    "iris_dev_layer_norm_mod": (None, [_vp, _vp, _vp, _vp, _i, _i, _f]),
    "iris_dev_rms_norm": (None, [_vp, _vp, _vp, _i, _i, _f]),
    "iris_dev_rms_norm_mod": (None, [_vp, _vp, _vp, _vp, _i, _i, _f]),
    "iris_dev_rms_norm_residual": (None, [_vp, _vp, _vp, _vp, _i, _i, _f]),
    "iris_dev_swiglu": (None, [_vp, _i, _vp, _vp, _i, _i, _i]),
    "iris_dev_residual": (None, [_vp, _vp, _vp, _i, _i]),
    "iris_dev_silu": (None, [_vp, _sz]),
    "iris_dev_add": (None, [_vp, _vp, _sz]),
    "iris_dev_add_bias": (None, [_vp, _vp, _i, _i]),
    "iris_dev_fill_rows": (None, [_vp, _vp, _i, _i]),
    "iris_dev_conv2d": (None, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i]),
    "iris_dev_group_norm": (None, [_vp, _vp, _vp, _vp, _i, _i, _i, _f, _i]),
    "iris_dev_group_norm_noalloc": (None, [_vp, _vp, _vp, _vp, _i, _i, _i, _f, _i]),
    "iris_dev_upsample2x": (None, [_vp, _vp, _i, _i, _i]),
    "iris_dev_head_norm_rope_qk": (None, [_vp, _vp, _i, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _f, _i]),
    "iris_dev_head_norm_rope_qk_streams": (None, [_vp, _vp, _i, _vp, _vp, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _i, _f, _i]),
    "iris_dev_stream": (_vp, []),
    "iris_dev_last_error": (_i, []),
    "iris_dev_last_kernel": (C.c_char_p, []),
    "iris_dev_linear_backend": (None, [_i]),
    # include/iris_rope.h: host builders (run without a GPU) ...
    "iris_rope_expand_i32": (_i, [_vp, _vp, _vp, _i, _i, _vp, _vp, _f]),
    "iris_rope_expand_f64": (_i, [_vp, _vp, _vp, _i, _i, _vp, _f]),
    "iris_rope_joint_rows": (_i, [_i, _i, _i, _vp, _vp, _i]),
    "iris_rope_flux2_positions": (None, [_vp, _i, _i, _i, _vp, _vp, _vp, _i]),
    "iris_rope_flux2_tables": (_i, [_vp, _vp, _i, _i, _i, _vp, _vp, _vp, _i, _i, _f]),
    "iris_rope_flux3_positions": (None, [_vp, _i, _i, _i, _vp, _vp, _i]),
    "iris_rope_flux3_tables": (_i, [_vp, _vp, _i, _i, _i, _vp, _vp, _i, _vp, _f]),
    "iris_rope_zimage_positions": (None, [_vp, _vp, _i, _i, _i, _vp, _vp]),
    "iris_rope_zimage_tables": (_i, [_vp, _vp, _vp, _i, _vp, _vp, _f]),
    "iris_rope_qwen3_tables": (_i, [_vp, _vp, _vp, _i, _i, _f, _i]),
    # ... and the same tables generated on the device
    "iris_dev_rope_expand_i32": (None, [_vp, _vp, _vp, _i, _i, _vp, _vp, _f]),
    "iris_dev_rope_expand_f64": (None, [_vp, _vp, _vp, _i, _i, _vp, _f]),
    "iris_dev_rope_flux2_tables": (None, [_vp, _vp, _i, _i, _i, _vp, _vp, _vp, _i, _i, _f]),
    "iris_dev_rope_flux3_tables": (None, [_vp, _vp, _i, _i, _i, _vp, _vp, _i, _vp, _f]),
    "iris_dev_rope_zimage_tables": (None, [_vp, _vp, _vp, _i, _vp, _vp, _f]),
    "iris_dev_rope_qwen3_tables": (None, [_vp, _vp, _vp, _i, _i, _f, _i]),
}


def build():
    """Compile the library in-tree with the repo Makefile (hipcc, gfx950)."""
    import subprocess
    subprocess.check_call(["make", "-s", "-C", ROOT, "rocm"])


def load(path=LIB_PATH):
    """dlopen the C-ABI library and attach prototypes. Raises if it is missing."""
    if not os.path.exists(path):
        raise FileNotFoundError(
            f"{path} not found: build it with `make rocm` (there is no fallback implementation)")
    lib = C.CDLL(path)
    for name, (res, args) in ABI.items():
        fn = getattr(lib, name)      # AttributeError if a declared symbol is not exported
        fn.restype, fn.argtypes = res, args
    return lib


class IrisDev:
    """Thin object wrapper over the C ABI; method names drop the iris_dev_ prefix."""

    def __init__(self, path=LIB_PATH):
        self.lib = load(path)
        if not self.lib.iris_dev_init():
            raise RuntimeError("iris_dev_init() found no usable gfx950 GPU")

    def __getattr__(self, name):
        return getattr(self.lib, "iris_dev_" + name)

    def name(self):
        return self.lib.iris_dev_name().decode()

    def last_kernel(self):
        return self.lib.iris_dev_last_kernel().decode()

    # ---- numpy conveniences (host <-> device through the ABI's own copies) ----
    def to_device(self, arr):
        import numpy as np
        arr = np.ascontiguousarray(arr)
        p = self.lib.iris_dev_alloc(arr.nbytes)
        if not p:
            raise MemoryError(f"iris_dev_alloc({arr.nbytes}) failed")
        self.lib.iris_dev_upload(p, arr.ctypes.data_as(_vp), arr.nbytes)
        return p

    def to_host(self, p, shape, dtype):
        import numpy as np
        out = np.empty(shape, dtype=dtype)
        self.lib.iris_dev_download(out.ctypes.data_as(_vp), p, out.nbytes)
        return out

    def check(self):
        e = self.lib.iris_dev_last_error()
        if e:
            raise RuntimeError(f"iris_dev reported error {e} (see stderr)")
