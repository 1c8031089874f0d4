"""The hot path under HIP graph capture. The library enqueues on one stream that it hands out
(iris_dev_stream), and the two hot-path operators allocate nothing on the layouts the matrix-core
kernels take directly (head_dim 128 / 256 / 512, 16-byte aligned rows), so a caller can capture a
step -- norm+rope on Q, on K, attention -- into a graph once and replay it (what a launch-bound loop
such as the 36 layers of the text encoder wants). Every replay is checked against the eager result,
with eager work and synchronisations of the program between the replays.
"""
import ctypes as C

import numpy as np
import pytest

import workloads as W
from gpu_harness import Dev, ptr_add

pytestmark = pytest.mark.gpu
_vp = C.c_void_p


class Graphs:
    def __init__(self):
        self.rt = C.CDLL("libamdhip64.so")
        self.rt.hipStreamBeginCapture.argtypes = [_vp, C.c_int]
        self.rt.hipStreamEndCapture.argtypes = [_vp, C.POINTER(_vp)]
        self.rt.hipGraphInstantiate.argtypes = [C.POINTER(_vp), _vp, _vp, _vp, C.c_size_t]
        self.rt.hipGraphLaunch.argtypes = [_vp, _vp]
        self.rt.hipGraphExecDestroy.argtypes = [_vp]
        self.rt.hipGraphDestroy.argtypes = [_vp]

    def capture(self, stream, fn):
        assert self.rt.hipStreamBeginCapture(stream, 0) == 0          # hipStreamCaptureModeGlobal
        fn()
        graph, run = _vp(), _vp()
        assert self.rt.hipStreamEndCapture(stream, C.byref(graph)) == 0 and graph
        assert self.rt.hipGraphInstantiate(C.byref(run), graph, None, None, 0) == 0
        self.rt.hipGraphDestroy(graph)
        return run


@pytest.mark.parametrize("maker", [W.c1, W.c4, lambda: W.c2(shrink=4), W.c2], ids=["c1", "c4", "c2-shrunk", "c2-two-size-grid"])
def test_step_replayed_from_a_graph_equals_the_eager_step(maker):
    case = maker()
    dev, g = Dev(), Graphs()
    lib, stream = dev.lib, _vp(dev.lib.iris_dev_stream())
    seq, ldi, qd, kd = case["seq"], case["ldi"], case["q_dim"], case["kv_dim"]
    rows, out = dev.put(case["buf"]), dev.alloc(seq * case["ldo"] * 2)
    wq, wk, cos, sin = dev.put(case["wq"]), dev.put(case["wk"]), dev.put(case["cos"]), dev.put(case["sin"])
    mask = dev.put(np.ascontiguousarray(case["key_mask"], np.int32)) if case["key_mask"] is not None else None

    def step():
        lib.iris_dev_head_norm_rope(rows, ldi, wq, cos, sin, seq, case["heads"], 128, case["eps"], case["split_half"])
        lib.iris_dev_head_norm_rope(ptr_add(rows, 2 * qd), ldi, wk, cos, sin, seq, case["kv_heads"], 128, case["eps"], case["split_half"])
        lib.iris_dev_attention(out, case["ldo"], rows, ptr_add(rows, 2 * qd), ptr_add(rows, 2 * (qd + kd)), ldi, seq, seq,
                               case["heads"], case["kv_heads"], 128, case["scale"], int(case["causal"]), mask)

    step()                                              # eager (also the first launch of each kernel: attributes are set here)
    dev.check()
    want = dev.get(out, (seq, case["ldo"]), np.uint16)
    assert want.any()
    run = g.capture(stream, step)
    dev.check()
    host = np.ascontiguousarray(case["buf"])
    for replay in range(4):
        # eager work of the program between the replays: the rows are normalised in place, so they are uploaded again,
        # and the output is overwritten with a pattern
        lib.iris_dev_upload(rows, host.ctypes.data_as(_vp), host.nbytes)
        junk = np.full((seq, case["ldo"]), 0x7fc0 + replay, np.uint16)
        lib.iris_dev_upload(out, junk.ctypes.data_as(_vp), junk.nbytes)
        assert g.rt.hipGraphLaunch(run, stream) == 0
        lib.iris_dev_sync()
        dev.check()
        got = dev.get(out, (seq, case["ldo"]), np.uint16)
        assert np.array_equal(got, want), f"replay {replay} differs from the eager step"
    g.rt.hipGraphExecDestroy(run)
    dev.free_all()


def test_a_layout_that_needs_scratch_is_refused_during_capture_until_the_scratch_exists():
    """head_dim 64 runs on the matrix cores through a padded private copy of q | k | v. Growing that copy means
    synchronise + free + allocate, which would invalidate a capture: inside a capture the call is refused (error
    reported, nothing enqueued, the capture stays valid); after one call outside, the same call is captured and
    replays to the eager result."""
    import oracle as O
    dev, g = Dev(), Graphs()
    lib, stream = dev.lib, _vp(dev.lib.iris_dev_stream())
    rng = np.random.default_rng(3)
    seq, heads, hd = 30000, 2, 64          # a 46 MB copy: larger than anything another test has left in the scratch
    buf = O.f32_to_bf16(rng.standard_normal((seq, 3 * heads * hd)).astype(np.float32))
    rows, out = dev.put(buf), dev.alloc(seq * heads * hd * 2)
    args = (out, heads * hd, rows, ptr_add(rows, 2 * heads * hd), ptr_add(rows, 4 * heads * hd), 3 * heads * hd, seq, seq, heads, heads, hd,
            0.125, 0, None)
    assert g.rt.hipStreamBeginCapture(stream, 0) == 0
    lib.iris_dev_attention(*args)
    refused = lib.iris_dev_last_error()
    graph = _vp()
    assert g.rt.hipStreamEndCapture(stream, C.byref(graph)) == 0, "the refused call must leave the capture valid"
    if graph:
        g.rt.hipGraphDestroy(graph)
    assert refused == -1
    lib.iris_dev_attention(*args)                                   # outside: allocates the scratch
    dev.check()
    assert dev.dev.last_kernel() == "fa_hd128_packed"
    want = dev.get(out, (seq, heads * hd), np.uint16)
    assert want.any()
    run = g.capture(stream, lambda: lib.iris_dev_attention(*args))
    dev.check()
    for replay in range(2):
        junk = np.full((seq, heads * hd), 0x7fc0 + replay, np.uint16)
        lib.iris_dev_upload(out, junk.ctypes.data_as(_vp), junk.nbytes)
        assert g.rt.hipGraphLaunch(run, stream) == 0
        lib.iris_dev_sync()
        assert np.array_equal(dev.get(out, (seq, heads * hd), np.uint16), want)
    g.rt.hipGraphExecDestroy(run)
    dev.free_all()


def test_double_stream_step_replayed_from_a_graph():
    """The joint block's step with the one-launch norm of both streams (iris_dev_head_norm_rope_qk_streams: text rows
    and image rows with their own weight pairs) and attention, captured once and replayed: every replay equals the
    eager step bit for bit."""
    case = W.c2(shrink=4)
    dev, g = Dev(), Graphs()
    lib, stream = dev.lib, _vp(dev.lib.iris_dev_stream())
    seq, ldi, qd, kd = case["seq"], case["ldi"], case["q_dim"], case["kv_dim"]
    txt = 512 // 4
    rows, out = dev.put(case["buf"]), dev.alloc(seq * case["ldo"] * 2)
    wq, wk, cos, sin = dev.put(case["wq"]), dev.put(case["wk"]), dev.put(case["cos"]), dev.put(case["sin"])
    wq2, wk2 = dev.put(case["wq"][::-1].copy()), dev.put(case["wk"][::-1].copy())

    def step():
        lib.iris_dev_head_norm_rope_qk_streams(rows, ptr_add(rows, 2 * qd), ldi, wq, wk, wq2, wk2, txt, cos, sin, seq, case["heads"],
                                               case["kv_heads"], 128, case["eps"], 0)
        lib.iris_dev_attention(out, case["ldo"], rows, ptr_add(rows, 2 * qd), ptr_add(rows, 2 * (qd + kd)), ldi, seq, seq,
                               case["heads"], case["kv_heads"], 128, case["scale"], 0, None)

    step()
    dev.check()
    want = dev.get(out, (seq, case["ldo"]), np.uint16)
    assert want.any()
    run = g.capture(stream, step)
    dev.check()
    host = np.ascontiguousarray(case["buf"])
    for replay in range(3):
        lib.iris_dev_upload(rows, host.ctypes.data_as(_vp), host.nbytes)
        junk = np.full((seq, case["ldo"]), 0x7fc0 + replay, np.uint16)
        lib.iris_dev_upload(out, junk.ctypes.data_as(_vp), junk.nbytes)
        assert g.rt.hipGraphLaunch(run, stream) == 0
        lib.iris_dev_sync()
        dev.check()
        assert np.array_equal(dev.get(out, (seq, case["ldo"]), np.uint16), want), f"replay {replay} differs from the eager step"
    g.rt.hipGraphExecDestroy(run)
    dev.free_all()


@pytest.mark.parametrize("causal_and_masked", [False, True], ids=["plain", "causal-masked"])
def test_head_dim_512_attention_with_key_ranges_replayed_from_a_graph(causal_and_masked):
    """The VAE's attention call at 4096 tokens: two launches (key ranges, then their merge through private scratch), and
    with a key mask a third in front that packs the mask into the same scratch. Once the scratch exists the call is
    captured; every replay, with eager calls of another size between them that overwrite the same scratch, equals
    the eager result."""
    import oracle as O
    dev, g = Dev(), Graphs()
    lib, stream = dev.lib, _vp(dev.lib.iris_dev_stream())
    rng = np.random.default_rng(5)
    seq, hd = 4096, 512
    buf = O.f32_to_bf16(rng.standard_normal((seq, 3 * hd)).astype(np.float32))
    rows, out, other = dev.put(buf), dev.alloc(seq * hd * 2), dev.alloc(seq * hd * 2)
    scale = float(1 / np.sqrt(hd))
    causal = int(causal_and_masked)
    mask = dev.put((rng.random(seq) < 0.7).astype(np.int32)) if causal_and_masked else None
    args = (out, hd, rows, ptr_add(rows, 2 * hd), ptr_add(rows, 4 * hd), 3 * hd, seq, seq, 1, 1, hd, scale, causal, mask)
    small = (other, hd, rows, ptr_add(rows, 2 * hd), ptr_add(rows, 4 * hd), 3 * hd, 1000, 1000, 1, 1, hd, scale, causal, mask)
    lib.iris_dev_attention(*args)                                   # outside: the scratch is sized
    dev.check()
    assert dev.dev.last_kernel() == "fa_hd512"
    want = dev.get(out, (seq, hd), np.uint16)
    run = g.capture(stream, lambda: lib.iris_dev_attention(*args))
    dev.check()
    for replay in range(3):
        junk = np.full((seq, hd), 0x7fc0 + replay, np.uint16)
        lib.iris_dev_upload(out, junk.ctypes.data_as(_vp), junk.nbytes)
        lib.iris_dev_attention(*small)                              # eager work on the same scratch between the replays
        assert g.rt.hipGraphLaunch(run, stream) == 0
        lib.iris_dev_sync()
        assert np.array_equal(dev.get(out, (seq, hd), np.uint16), want), f"replay {replay}"
    g.rt.hipGraphExecDestroy(run)
    dev.free_all()
