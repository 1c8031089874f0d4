#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

A step is what every transformer block of the reference issues for one
sequence: fused per-head RMSNorm + RoPE on Q, on K, then joint attention
(reference iris_transformer_flux.c:3834-3839), on the 24 heads x 128,
512 text + 4096 image token configuration, bf16, inputs resident in HBM.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--settle-ms T] [--no-cpu] [--no-shapes] [--no-machine]
    python bench.py --only WIDE [--steps K]       one head of 512 / 256 dims with key masks and causal limit, 4096 - 50176 tokens
    python bench.py --only CONFIG [--steps K]     launches of one configuration only (C1 .. C5, C3-cond, C3-uncond,
                                                  VAE), for profiler runs
    python bench.py --copy-only MiB               the plain copy kernel that calibrates the byte counters

Prints ONE JSON line. `value` is attention TFLOP/s over the whole step
(algorithmic attention FLOPs / wall time of the triple) with settled clocks,
`value_from_idle` the same over the first 50 steps after the GPU sat idle.
`roofline` is the attention kernel alone, timed with HIP events on the
library's stream around the attention launch of every step (mean, median,
min, and the latency of a single launch between two synchronisations); its
`traffic` is read from the committed counter summary it names. `norm_rope`
reports the bandwidth-bound kernel over back-to-back launches (cold rows,
fused Q+K, rows in the Infinity Cache) and the kernel-only durations on file.
`shapes` lists, for every benchmark configuration, the attention latency
(mean / median / min / single launch) with its fraction of the matrix peak,
the norm+rope calls with their fraction of the HBM peak, the whole step
(two norm+rope calls and attention) issued call by call and replayed from a
HIP graph of 16 steps, for a configuration with a key mask the number of valid
keys drawn from the seed and the same launch with every key valid (the kernel
stops at the last key tile that holds a valid key), and the seconds of the CPU
port on this host's cores; `other_ops` the other device operators
at this configuration's shapes, among them the q | k | v projection with
and without the normalisation in its epilogue; `rope_tables` the time to
build one forward pass's rotary tables (host builder + upload, and straight
into device memory); `machine` the measured ceilings of the GPU and the
attention kernel by number of busy CUs. `cpu_baseline` times the
reference's BLAS-build CPU structure on this host's cores.

Clock settling: after idle the GPU's power management takes tens of
milliseconds of sustained load to reach its steady clocks; the same
attention launch measures 0.27 ms right after idle, 0.30 ms a few
milliseconds later and 0.24-0.25 ms from about 30 ms on. A model runs for
seconds, so the steady state is the figure of interest: before the W warmup
steps the bench runs the same step, untimed, until --settle-ms of wall time
have passed (`settle_steps` in the output), and every other timed loop is
preceded by the same kind of load. --settle-ms 0 switches it off.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2516.6      # MI355X dense bf16 matrix peak (vendor figure)
PEAK_HBM_GBPS = 8000.0         # MI355X HBM3E peak
# HBM bytes one C2 attention launch moves come from hardware counters (FETCH_SIZE, WRITE_SIZE scaled by a 1 GiB
# copy kernel), which a separate profiler run collects: the summary of that run is read here, so the figure in the
# output line is the one on file and says so.
TRAFFIC_PROFILE = os.path.join("profiles", "k_fa_fwd_hd128__c2__hbm_traffic.txt")


ATTENTION_SOURCE = os.path.join("iris_c_amd", "csrc", "fa_fwd_gfx950.hip")


def source_sha256(rel=ATTENTION_SOURCE):
    import hashlib
    try:
        return hashlib.sha256(open(os.path.join(ROOT, rel), "rb").read()).hexdigest()[:16]
    except OSError:
        return None


def traffic_on_file():
    """(bytes per launch, source file, stale) from the committed counter summary: the line
    'total_bytes_per_launch: N', and 'kernel_source_sha256: H', the hash of the kernel source the counters were taken
    on; stale = that hash is not the hash of the kernel source in this tree."""
    nbytes, sha = None, None
    try:
        for line in open(os.path.join(ROOT, TRAFFIC_PROFILE)):
            if line.startswith("total_bytes_per_launch:"):
                nbytes = int(line.split(":")[1].strip().replace(",", ""))
            if line.startswith("kernel_source_sha256:"):
                sha = line.split(":")[1].split()[0]
    except OSError:
        return None, None, None
    return nbytes, TRAFFIC_PROFILE, sha != source_sha256()


def attention_kernel_name(lib, c):
    """The __global__ function an iris_dev_attention call of configuration c launches, from the launcher's own
    planner (host arithmetic, nothing launched)."""
    plan = (C.c_int * 5)()
    lib.iris_hip_fa_hd128_plan.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_int)]
    lib.iris_hip_fa_hd128_plan.restype = None
    lib.iris_hip_fa_hd128_plan(c["seq"], c["seq"], c["heads"], int(c["causal"]), plan)
    flags = f"{'true' if c['causal'] else 'false'}, {'true' if c['key_mask'] is not None else 'false'}"
    kind, waves, nb = plan[0], plan[1], plan[2]
    if kind == 1:
        return f"k_fa_fwd_hd128_two_sizes<{flags}>", {"workgroups_of_256_queries_per_head": plan[3], "workgroups_of_192_queries_per_head": plan[4]}
    if kind == 2:
        return f"k_fa_short_hd128<4, {flags}>", {}
    return f"k_fa_fwd_hd128<{waves}, {nb}, {flags}>", {"queries_per_workgroup": 16 * nb * waves}

NORM_ROPE_PROFILE = os.path.join("profiles", "k_norm_rope_hd128__c2__kernel_trace.txt")


def kernel_only_on_file():
    """Kernel-only durations (us) of the norm+rope series from the committed kernel trace: lines 'name: value'."""
    found = {}
    try:
        for line in open(os.path.join(ROOT, NORM_ROPE_PROFILE)):
            for name in ("q_call_kernel_us_cold", "qk_fused_kernel_us_cold", "q_call_kernel_us_warm"):
                if line.startswith(name + ":"):
                    found[name] = float(line.split(":")[1])
    except (OSError, ValueError):
        pass
    return found

_vp = C.c_void_p


# ----------------------------------------------------------------------------- inputs
def to_bf16(x):
    """float32 ndarray -> uint16 bf16 patterns, round to nearest even."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def make_config(name, rng):
    """Synthetic data of one benchmark configuration (numpy PCG64 normals); rotary tables from the
    library's own host builders (include/iris_rope.h)."""
    from iris_c_amd.rope import RopeTables
    rt = RopeTables()
    hd = 128
    c = dict(name=name, hd=hd, causal=False, key_mask=None, split_half=0, eps=1e-6)
    if name in ("C1", "C2", "C5"):
        txt, grid, refs, sigma = {"C1": (64, 16, 0, 1.0), "C2": (512, 64, 0, 1 / np.sqrt(128)), "C5": (512, 64, 2, 1.0)}[name]
        c.update(heads=24, kv_heads=24, seq=txt + grid * grid * (1 + refs), sigma=[sigma])
        c["layout"] = (txt, grid, grid, [(grid, grid)] * refs)
        c["cos"], c["sin"] = rt.flux2_tables(*c["layout"])
    elif name in ("C3-cond", "C3-uncond"):
        seq = 4096 + 256
        c.update(heads=30, kv_heads=30, seq=seq, eps=1e-5, sigma=[1 / np.sqrt(128)] if name == "C3-cond" else [0.1])
        pos, _, ip, cp = rt.zimage_positions(img_seq=4096, wt=64, cap_seq=256)      # [image | caption]
        assert ip + cp == seq
        c["cos"], c["sin"] = rt.zimage_tables(pos, (32, 48, 48), (1536, 512, 512), 256.0)
        if name == "C3-uncond":
            length = int(rng.integers(16, 257))
            c["key_mask"] = np.r_[np.ones(4096), np.arange(256) < length].astype(np.int32)
    elif name == "C4":
        seq = 512
        c.update(heads=32, kv_heads=8, seq=seq, causal=True, split_half=1, sigma=[1.0])
        c["cos"], c["sin"] = rt.qwen3_tables(seq, 128, 1e6)
        c["key_mask"] = (np.arange(seq) < int(rng.integers(8, 513))).astype(np.int32)
    else:
        raise ValueError(name)
    c["q_dim"], c["kv_dim"] = c["heads"] * hd, c["kv_heads"] * hd
    c["ldi"] = c["q_dim"] + 2 * c["kv_dim"]
    c["ldo"] = c["q_dim"]
    c["scale"] = float(1.0 / np.sqrt(np.float32(hd)))
    buf = rng.standard_normal((c["seq"], c["ldi"]), dtype=np.float32) * np.float32(c["sigma"][0])
    c["buf"] = to_bf16(buf)
    c["wq"] = (1 + 0.02 * rng.standard_normal(hd)).astype(np.float32)
    c["wk"] = (1 + 0.02 * rng.standard_normal(hd)).astype(np.float32)
    return c


def attention_flops(c):
    valid = np.ones(c["seq"], np.int64) if c["key_mask"] is None else (c["key_mask"] != 0).astype(np.int64)
    per_query = np.cumsum(valid) if c["causal"] else np.full(c["seq"], valid.sum())
    return 4 * c["hd"] * c["heads"] * int(per_query.sum())


def norm_rope_bytes(seq, heads, hd=128):
    return 4 * seq * heads * hd + 2 * seq * (hd // 2) * 4 + hd * 4


# ----------------------------------------------------------------------------- device plumbing
class Hip:
    """The few HIP runtime calls the timing needs (events on the library's stream)."""

    def __init__(self):
        self.rt = C.CDLL("libamdhip64.so")
        self.rt.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), _vp, _vp]
        self.rt.hipEventRecord.argtypes = [_vp, _vp]
        self.rt.hipEventSynchronize.argtypes = [_vp]

    def event(self):
        ev = _vp()
        assert self.rt.hipEventCreate(C.byref(ev)) == 0
        return ev

    def record(self, ev, stream):
        assert self.rt.hipEventRecord(ev, stream) == 0

    def elapsed_ms(self, a, b):
        assert self.rt.hipEventSynchronize(b) == 0
        ms = C.c_float()
        assert self.rt.hipEventElapsedTime(C.byref(ms), a, b) == 0
        return float(ms.value)

    def capture(self, stream, fn):
        """Records what fn enqueues on the library's stream into a graph; returns the executable graph."""
        rt = self.rt
        rt.hipStreamBeginCapture.argtypes = [_vp, C.c_int]
        rt.hipStreamEndCapture.argtypes = [_vp, C.POINTER(_vp)]
        rt.hipGraphInstantiate.argtypes = [C.POINTER(_vp), _vp, _vp, _vp, C.c_size_t]
        rt.hipGraphLaunch.argtypes = [_vp, _vp]
        rt.hipGraphExecDestroy.argtypes = [_vp]
        rt.hipGraphDestroy.argtypes = [_vp]
        assert rt.hipStreamBeginCapture(stream, 0) == 0
        fn()
        graph, run = _vp(), _vp()
        assert rt.hipStreamEndCapture(stream, C.byref(graph)) == 0 and graph
        assert rt.hipGraphInstantiate(C.byref(run), graph, None, None, 0) == 0
        rt.hipGraphDestroy(graph)
        return run


class Resident:
    """One configuration's tensors in HBM, `copies` rotating row buffers."""

    def __init__(self, dev, c, copies):
        self.c, self.dev, self.lib = c, dev, dev.lib
        self.bufs = [dev.to_device(c["buf"]) for _ in range(copies)]
        self.out = self.lib.iris_dev_alloc(c["seq"] * c["ldo"] * 2)
        self.wq, self.wk = dev.to_device(c["wq"]), dev.to_device(c["wk"])
        self.wq2, self.wk2 = dev.to_device(c["wq"][::-1].copy()), dev.to_device(c["wk"][::-1].copy())   # the image stream's pair
        self.cos, self.sin = dev.to_device(c["cos"]), dev.to_device(c["sin"])
        self.mask = dev.to_device(c["key_mask"]) if c["key_mask"] is not None else None
        assert self.out and all(self.bufs)

    def col(self, i, elems):
        return _vp(self.bufs[i % len(self.bufs)] + 2 * elems)

    def norm_q(self, i):
        c = self.c
        self.lib.iris_dev_head_norm_rope(self.col(i, 0), c["ldi"], self.wq, self.cos, self.sin, c["seq"], c["heads"],
                                         c["hd"], c["eps"], c["split_half"])

    def norm_k(self, i):
        c = self.c
        self.lib.iris_dev_head_norm_rope(self.col(i, c["q_dim"]), c["ldi"], self.wk, self.cos, self.sin, c["seq"],
                                         c["kv_heads"], c["hd"], c["eps"], c["split_half"])

    def norm_qk(self, i):
        c = self.c
        self.lib.iris_dev_head_norm_rope_qk(self.col(i, 0), self.col(i, c["q_dim"]), c["ldi"], self.wq, self.wk, self.cos,
                                            self.sin, c["seq"], c["heads"], c["kv_heads"], c["hd"], c["eps"], c["split_half"])

    def attention(self, i):
        c = self.c
        self.lib.iris_dev_attention(self.out, c["ldo"], self.col(i, 0), self.col(i, c["q_dim"]),
                                    self.col(i, c["q_dim"] + c["kv_dim"]), c["ldi"], c["seq"], c["seq"], c["heads"],
                                    c["kv_heads"], c["hd"], c["scale"], int(c["causal"]), self.mask)

    def step(self, i):
        """The caller's triple, as the reference models issue it (two norm calls, one attention)."""
        self.norm_q(i); self.norm_k(i); self.attention(i)

    def step_fused_qk(self, i):
        """The same work with the library's one-launch Q+K normalisation (an addition to the reference API)."""
        self.norm_qk(i); self.attention(i)

    # The double-stream block (reference iris_transformer_flux.c:3786-3804): text rows [0, txt) and image rows
    # [txt, seq) of the joint q | k | v rows are normalised separately, each stream with its own weight pair and the
    # tables offset to its first row; then one attention over all rows.
    def _streams(self, txt):
        return ((0, txt, self.wq, self.wk), (txt, self.c["seq"] - txt, self.wq2, self.wk2))

    def norm_double_stream(self, i, txt):
        """four launches, as the reference issues them"""
        c = self.c
        for first, n, wq, wk in self._streams(txt):
            qkv = self.bufs[i % len(self.bufs)] + 2 * first * c["ldi"]
            rc, rs = _vp(self.cos + 4 * first * 64), _vp(self.sin + 4 * first * 64)
            self.lib.iris_dev_head_norm_rope(_vp(qkv), c["ldi"], wq, rc, rs, n, c["heads"], c["hd"], c["eps"], 0)
            self.lib.iris_dev_head_norm_rope(_vp(qkv + 2 * c["q_dim"]), c["ldi"], wk, rc, rs, n, c["kv_heads"], c["hd"], c["eps"], 0)

    def norm_double_stream_qk(self, i, txt):
        """one Q+K launch per stream"""
        c = self.c
        for first, n, wq, wk in self._streams(txt):
            qkv = self.bufs[i % len(self.bufs)] + 2 * first * c["ldi"]
            rc, rs = _vp(self.cos + 4 * first * 64), _vp(self.sin + 4 * first * 64)
            self.lib.iris_dev_head_norm_rope_qk(_vp(qkv), _vp(qkv + 2 * c["q_dim"]), c["ldi"], wq, wk, rc, rs, n, c["heads"],
                                                c["kv_heads"], c["hd"], c["eps"], 0)

    def norm_double_stream_one(self, i, txt):
        """one launch for both streams and both tensors"""
        c = self.c
        self.lib.iris_dev_head_norm_rope_qk_streams(self.col(i, 0), self.col(i, c["q_dim"]), c["ldi"], self.wq, self.wk, self.wq2,
                                                    self.wk2, txt, self.cos, self.sin, c["seq"], c["heads"], c["kv_heads"],
                                                    c["hd"], c["eps"], 0)

    def attention_qnorm(self, i):
        c = self.c
        self.lib.iris_dev_attention_qnorm(self.out, c["ldo"], self.col(i, 0), self.col(i, c["q_dim"]),
                                          self.col(i, c["q_dim"] + c["kv_dim"]), c["ldi"], c["seq"], c["seq"], c["heads"],
                                          c["kv_heads"], c["hd"], c["scale"], int(c["causal"]), self.mask, self.wq,
                                          self.cos, self.sin, c["eps"], c["split_half"])

    def step_q_norm_in_attention(self, i):
        """The same work with Q normalised while the attention kernel loads it (an addition to the reference API):
        one norm launch on K, one attention launch."""
        self.norm_k(i); self.attention_qnorm(i)

    def free(self):
        for p in self.bufs + [self.out, self.wq, self.wk, self.wq2, self.wk2, self.cos, self.sin] + ([self.mask] if self.mask else []):
            self.lib.iris_dev_free(p)


def settle(lib, fn, ms):
    """Runs fn(i) back to back, untimed, until `ms` of wall time have passed; returns the number of calls."""
    n, t0 = 0, time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < ms:
        for _ in range(10):
            fn(n)
            n += 1
        lib.iris_dev_sync()
    return n


def event_time(hip, stream, fn, reps, start=0):
    """Average ms of `fn(i)` over `reps` back-to-back launches between two events."""
    a, b = hip.event(), hip.event()
    hip.record(a, stream)
    for i in range(reps):
        fn(start + i)
    hip.record(b, stream)
    return hip.elapsed_ms(a, b) / reps


def single_launch_ms(hip, stream, lib, fn, reps=5):
    """One launch on an idle stream, events around it: what a caller that waits for the result sees
    beyond the kernel itself (median of `reps`)."""
    ts = []
    for i in range(reps):
        lib.iris_dev_sync()
        a, b = hip.event(), hip.event()
        hip.record(a, stream); fn(i); hip.record(b, stream)
        ts.append(hip.elapsed_ms(a, b))
    return float(np.median(ts))


def step_times(hip, stream, lib, step, steps_per_graph=16, launches=8):
    """(eager, graph) microseconds per step: the caller's triple issued call by call, and the same steps captured
    once into a HIP graph of `steps_per_graph` steps and replayed (what a launch-bound loop such as the layers of the
    text encoder would do; the library's operators allocate nothing, so its stream can be captured)."""
    n = steps_per_graph * launches
    for i in range(steps_per_graph):
        step(i)
    lib.iris_dev_sync()
    t0 = time.perf_counter()
    for i in range(n):
        step(i)
    lib.iris_dev_sync()
    eager = (time.perf_counter() - t0) / n * 1e6
    run = hip.capture(stream, lambda: [step(i) for i in range(steps_per_graph)])
    assert hip.rt.hipGraphLaunch(run, stream) == 0
    lib.iris_dev_sync()
    t0 = time.perf_counter()
    for _ in range(launches):
        assert hip.rt.hipGraphLaunch(run, stream) == 0
    lib.iris_dev_sync()
    graph = (time.perf_counter() - t0) / n * 1e6
    hip.rt.hipGraphExecDestroy(run)
    return eager, graph


def per_launch_times(hip, stream, fn, reps, before=None):
    """Per-launch ms with an event pair around every launch (for kernels >> event cost); `before(i)`, if given,
    is enqueued ahead of each timed launch, outside its event pair."""
    evs = [(hip.event(), hip.event()) for _ in range(reps)]
    for i, (a, b) in enumerate(evs):
        if before:
            before(i)
        hip.record(a, stream); fn(i); hip.record(b, stream)
    return [hip.elapsed_ms(a, b) for a, b in evs]


# ----------------------------------------------------------------------------- the other operators
def other_ops(dev, hip, stream, rng, settle_ms=0.0):
    """Latency of the other device operators at the shapes a transformer block of the bench configuration
    uses (4608 tokens, width 3072): linear layers in TFLOP/s, one-pass kernels in GB/s (bytes read + written)."""
    lib = dev.lib
    rows, dim = 4608, 3072
    res = []

    def timed(fn, reps=10):
        fn(0); lib.iris_dev_sync(); dev.check()
        settle(lib, fn, settle_ms)
        return min(event_time(hip, stream, fn, reps) for _ in range(3))

    x = dev.to_device(to_bf16(rng.standard_normal((rows, 12288), dtype=np.float32)))
    W = dev.to_device(to_bf16(rng.standard_normal((27648 * 3072,), dtype=np.float32) * 0.02))
    y = lib.iris_dev_alloc(rows * 27648 * 4)
    for k, n in ((3072, 9216), (3072, 3072), (3072, 18432), (9216, 3072), (3072, 27648), (12288, 3072)):
        for name, fn in (("linear_f32", lib.iris_dev_linear_f32), ("linear_bf16", lib.iris_dev_linear_bf16)):
            for backend in (2, 0):            # 2: the vendor GEMM library when present (the yardstick), 0: own MFMA kernel (the default)
                lib.iris_dev_linear_backend(backend)
                ms = timed(lambda i: fn(y, x, W, rows, k, n), 5)
                res.append({"op": name, "kernel": dev.last_kernel(), "shape": f"{rows}x{k}->{n}", "us": round(ms * 1e3, 1),
                            "tflops": round(2 * rows * k * n / ms / 1e9, 1)})
    # the fused q | k | v (| gate | up) projection with the norm+rope of its Q and K columns: the reference's three calls
    # (iris_transformer_flux.c:3833-3837) and the entry that takes them as one
    w1 = dev.to_device(np.ones(dim, np.float32))
    ang = rng.uniform(-3.0, 3.0, (rows, 64)).astype(np.float32)
    cos, sin = dev.to_device(np.cos(ang)), dev.to_device(np.sin(ang))
    heads = dim // 128
    for n in (9216, 27648):
        def three_calls(i):
            lib.iris_dev_linear_bf16(y, x, W, rows, dim, n)
            lib.iris_dev_head_norm_rope(y, n, w1, cos, sin, rows, heads, 128, 1e-6, 0)
            lib.iris_dev_head_norm_rope(_vp(y + 2 * dim), n, w1, cos, sin, rows, heads, 128, 1e-6, 0)

        def one_call(i):
            lib.iris_dev_linear_bf16_qknorm(y, x, W, rows, dim, n, heads, heads, 128, w1, w1, cos, sin, 1e-6, 0)
        for backend in (2, 0):
            lib.iris_dev_linear_backend(backend)
            for name, fn in (("linear_bf16 + 2 x head_norm_rope", three_calls), ("linear_bf16_qknorm", one_call)):
                ms = timed(fn, 5)
                res.append({"op": name, "linear_backend": backend, "kernel": dev.last_kernel(), "shape": f"{rows}x{dim}->{n}",
                            "us": round(ms * 1e3, 1)})
    lib.iris_dev_linear_backend(0)
    for p in (cos, sin):
        lib.iris_dev_free(p)
    xf, af = _vp(y), _vp(y + rows * dim * 4)
    ob = _vp(x)
    n = rows * dim
    one_pass = [("layer_norm_mod", lambda i: lib.iris_dev_layer_norm_mod(ob, xf, w1, w1, rows, dim, 1e-6), 6 * n),
                ("rms_norm", lambda i: lib.iris_dev_rms_norm(ob, xf, w1, rows, dim, 1e-6), 6 * n),
                ("rms_norm_residual", lambda i: lib.iris_dev_rms_norm_residual(xf, af, w1, w1, rows, dim, 1e-6), 12 * n),
                ("residual", lambda i: lib.iris_dev_residual(xf, af, w1, rows, dim), 12 * n),
                ("f32_to_bf16", lambda i: lib.iris_dev_f32_to_bf16(ob, xf, n), 6 * n),
                ("swiglu 4608x9216", lambda i: lib.iris_dev_swiglu(ob, 9216, _vp(y), _vp(y + 2 * 9216), 18432, rows, 9216), 6 * rows * 9216)]
    for name, fn, nbytes in one_pass:
        ms = timed(fn, 20)
        res.append({"op": name, "shape": f"{rows}x{dim}" if "swiglu" not in name else "", "us": round(ms * 1e3, 1),
                    "gbps": round(nbytes / ms / 1e6, 0)})
    for p in (x, W, y, w1):
        lib.iris_dev_free(p)
    # the VAE's operators at two of its shapes: 3 x 3 convolution and group norm + SiLU, channels last, f32 in and out
    for side, ch in ((512, 128), (256, 512)):
        hw = side * side
        img = dev.to_device(rng.standard_normal((hw, ch), dtype=np.float32))
        out = lib.iris_dev_alloc(hw * ch * 4)
        wt = dev.to_device(to_bf16(rng.standard_normal((ch, 9 * ch), dtype=np.float32) * 0.02))
        g1 = dev.to_device(np.ones(ch, np.float32))
        ms = timed(lambda i: lib.iris_dev_conv2d(out, img, wt, g1, side, side, ch, ch, 3, 1, 1, 1), 5)
        res.append({"op": "conv2d 3x3", "shape": f"{side}x{side}x{ch}->{ch}", "us": round(ms * 1e3, 1),
                    "tflops": round(2 * hw * 9 * ch * ch / ms / 1e9, 1)})
        ms = timed(lambda i: lib.iris_dev_group_norm(out, img, g1, g1, hw, ch, 32, 1e-6, 1), 5)
        res.append({"op": "group_norm+silu", "shape": f"{side}x{side}x{ch}", "us": round(ms * 1e3, 1),
                    "gbps": round(8 * hw * ch / ms / 1e6, 0)})
        for p in (img, out, wt, g1):
            lib.iris_dev_free(p)
    return res


def rope_table_times(dev, c):
    """Building the rotary tables of one forward pass of the bench configuration (wall clock, host side
    included): the library's host builder + upload, and its device generator (positions staged, kernel run)."""
    from iris_c_amd.rope import RopeTables
    lib, rt = dev.lib, RopeTables(dev.lib)
    txt, gh, gw, refs = c["layout"]
    rows, nbytes = c["seq"], c["cos"].nbytes
    dc, ds = lib.iris_dev_alloc(nbytes), lib.iris_dev_alloc(nbytes)

    def best(fn, n=5):
        ts = []
        for _ in range(n):
            t0 = time.perf_counter(); fn(); lib.iris_dev_sync(); ts.append(time.perf_counter() - t0)
        return min(ts) * 1e3

    def host():
        cos, sin = rt.flux2_tables(txt, gh, gw, refs)
        lib.iris_dev_upload(dc, cos.ctypes.data_as(_vp), nbytes)
        lib.iris_dev_upload(ds, sin.ctypes.data_as(_vp), nbytes)

    host_ms = best(host)
    dev_ms = best(lambda: lib.iris_dev_rope_flux2_tables(dc, ds, txt, gh, gw, None, None, None, len(refs), 32, 2000.0))
    dev.check()
    lib.iris_dev_free(dc); lib.iris_dev_free(ds)
    return {"rows": rows, "table_bytes": 2 * nbytes, "host_build_and_upload_ms": round(host_ms, 3),
            "device_generate_ms": round(dev_ms, 3)}


# ----------------------------------------------------------------------------- machine ceilings
def microbench_lib():
    mb = C.CDLL(os.path.join(ROOT, "iris_c_amd", "libiris_microbench.so"))
    mb.iris_mb_mfma.argtypes = [_vp, _vp, C.c_int, C.c_int]
    mb.iris_mb_mfma_data.argtypes = [_vp, _vp, _vp, C.c_int, C.c_int]
    mb.iris_mb_mfma_data16.argtypes = [_vp, _vp, _vp, C.c_int, C.c_int]
    mb.iris_mb_copy.argtypes = [_vp, _vp, _vp, C.c_size_t]
    mb.iris_mb_rmw.argtypes = [_vp, _vp, C.c_size_t]
    mb.iris_mb_read.argtypes = [_vp, _vp, C.c_size_t, _vp]
    mb.iris_mb_write.argtypes = [_vp, _vp, C.c_size_t]
    return mb


def vae_case(rng, seq=16384):
    """The VAE mid-block attention of a 1024 x 1024 image: one head of 512 over (1024 / 8)^2 tokens, rows q | k | v."""
    hd = 512
    c = dict(name="VAE", hd=hd, causal=False, key_mask=None, heads=1, kv_heads=1, seq=seq, q_dim=hd, kv_dim=hd,
             ldi=3 * hd, ldo=hd, scale=float(1.0 / np.sqrt(np.float32(hd))))
    c["buf"] = to_bf16(rng.standard_normal((seq, 3 * hd), dtype=np.float32))
    return c


def only_one(dev, hip, stream, rng, name, steps, settle_ms):
    """Launches of one configuration only (for profiler runs)."""
    lib = dev.lib
    if name == "VAE":
        c = vae_case(rng)
        d, o = dev.to_device(c["buf"]), lib.iris_dev_alloc(c["seq"] * c["ldo"] * 2)
        fn = lambda i: lib.iris_dev_attention(o, c["ldo"], d, _vp(d + 2 * c["q_dim"]), _vp(d + 2 * (c["q_dim"] + c["kv_dim"])),
                                              c["ldi"], c["seq"], c["seq"], 1, 1, c["hd"], c["scale"], 0, None)
        settle(lib, fn, settle_ms)
        ts = per_launch_times(hip, stream, fn, steps)
        dev.check()
        kernel = dev.last_kernel()
        lib.iris_dev_free(d); lib.iris_dev_free(o)
    else:
        c = make_config(name, rng)
        r = Resident(dev, c, 2)
        settle(lib, r.step, settle_ms)
        ts = per_launch_times(hip, stream, r.attention, steps, before=lambda i: (r.norm_q(i), r.norm_k(i)))
        dev.check()
        kernel = dev.last_kernel()
        r.free()
    fl = attention_flops(c)
    return {"config": name, "kernel": kernel, "launches": steps, "attention_ms_mean": round(float(np.mean(ts)), 4),
            "attention_ms_median": round(float(np.median(ts)), 4), "attention_ms_min": round(float(np.min(ts)), 4),
            "flops_per_launch": fl, "tflops": round(fl / float(np.mean(ts)) / 1e9, 1)}


def wide_heads(dev, hip, stream, rng, steps, settle_ms):
    """One head of 512 (the VAE's call) and of 256 dims with what the device interface allows on top: a key mask that
    leaves 60 % of the keys at random (every tile ragged), a padding mask over the last third, a causal limit, and
    causal + mask. Average us over `steps` back-to-back calls between two events, after a settling load of the same
    call; TFLOP/s count the (query, key) pairs the call may look at."""
    lib, rows = dev.lib, []
    for hd in (512, 256):
        for seq in (4096, 16384, 50176):
            buf = to_bf16(rng.standard_normal((seq, 3 * hd), dtype=np.float32))
            d, o = dev.to_device(buf), lib.iris_dev_alloc(seq * hd * 2)
            masks = {"none": None, "60 % at random": (rng.random(seq) < 0.6).astype(np.int32),
                     "padding, last third": (np.arange(seq) < 2 * seq // 3).astype(np.int32)}
            dm = {k: (dev.to_device(v) if v is not None else None) for k, v in masks.items()}
            for causal, mask in ((0, "none"), (0, "60 % at random"), (0, "padding, last third"), (1, "none"), (1, "60 % at random")):
                fn = lambda i: lib.iris_dev_attention(o, hd, d, _vp(d + 2 * hd), _vp(d + 4 * hd), 3 * hd, seq, seq, 1, 1, hd,
                                                      float(1.0 / np.sqrt(np.float32(hd))), causal, dm[mask])
                settle(lib, fn, settle_ms)
                ms = event_time(hip, stream, fn, steps if seq < 50000 else max(steps // 4, 3))
                lib.iris_dev_sync()
                dev.check()
                seen = (0.5 if causal else 1.0) * (2 / 3 if mask.startswith("padding") else 1.0)
                fl = 4.0 * seq * seq * hd * seen
                rows.append({"head_dim": hd, "tokens": seq, "causal": bool(causal), "key_mask": mask, "kernel": dev.last_kernel(),
                             "us": round(ms * 1e3, 1), "tflops_of_visible_pairs": round(fl / ms / 1e9, 1),
                             "frac_of_peak": round(fl / ms / 1e9 / PEAK_BF16_TFLOPS, 4)})
            for v in dm.values():
                if v is not None:
                    lib.iris_dev_free(v)
            lib.iris_dev_free(d); lib.iris_dev_free(o)
    return rows


def occupancy_probe(dev, hip, stream, rng, settle_ms):
    """The attention kernel on one round of workgroups that fills all 256 CUs, 176 of them and 128 of them
    (4096 tokens x 16 / 11 / 8 heads: 256 / 176 / 128 workgroups of 256 queries, each walking the same 64 key
    tiles). The schedule of a workgroup is the same in all three; what changes is how many CUs draw power."""
    lib, res = dev.lib, []
    for heads in (16, 11, 8):
        c = dict(name=f"{heads}h", hd=128, causal=False, key_mask=None, heads=heads, kv_heads=heads, seq=4096,
                 q_dim=heads * 128, kv_dim=heads * 128, ldi=3 * heads * 128, ldo=heads * 128,
                 scale=float(1.0 / np.sqrt(np.float32(128))))
        c["buf"] = to_bf16(rng.standard_normal((4096, c["ldi"]), dtype=np.float32))
        d, o = dev.to_device(c["buf"]), lib.iris_dev_alloc(4096 * c["ldo"] * 2)
        fn = lambda i: lib.iris_dev_attention(o, c["ldo"], d, _vp(d + 2 * c["q_dim"]), _vp(d + 2 * (c["q_dim"] + c["kv_dim"])),
                                              c["ldi"], 4096, 4096, heads, heads, 128, c["scale"], 0, None)
        settle(lib, fn, settle_ms)
        ms = float(np.median(per_launch_times(hip, stream, fn, 30)))
        dev.check()
        fl = attention_flops(c)
        res.append({"workgroups": heads * 16, "launch_us": round(ms * 1e3, 1), "tflops": round(fl / ms / 1e9, 1),
                    "tflops_per_busy_cu": round(fl / ms / 1e9 / min(heads * 16, 256), 3)})
        lib.iris_dev_free(d); lib.iris_dev_free(o)
    return res


def copy_only(dev, hip, stream, nbytes, reps):
    """`reps` launches of the plain copy kernel (reads nbytes, writes nbytes)."""
    lib, mb = dev.lib, microbench_lib()
    src, dst = lib.iris_dev_alloc(nbytes), lib.iris_dev_alloc(nbytes)
    assert src and dst
    mb.iris_mb_copy(stream, dst, src, nbytes)
    ms = event_time(hip, stream, lambda i: mb.iris_mb_copy(stream, dst, src, nbytes), reps)
    dev.check()
    lib.iris_dev_free(src); lib.iris_dev_free(dst)
    return {"kernel": "k_copy", "bytes_read": nbytes, "bytes_written": nbytes, "launches": reps + 1,
            "us_per_launch": round(ms * 1e3, 2), "gbps_read_plus_write": round(2 * nbytes / ms / 1e6, 1)}


def machine_ceilings(dev, hip, stream):
    """What this GPU sustains on the two limits the kernels are priced against: a loop of nothing but
    v_mfma_f32_32x32x16_bf16 (4 waves x 1024 blocks), and a 16 B/lane copy / in-place update of 1 GiB."""
    lib, mb = dev.lib, microbench_lib()
    sink = lib.iris_dev_alloc(64)
    blocks, iters = 1024, 4000
    mb.iris_mb_mfma(stream, sink, blocks, 16)
    ms = min(event_time(hip, stream, lambda i: mb.iris_mb_mfma(stream, sink, blocks, iters), 1) for _ in range(3))
    mfma = blocks * 4 * iters * 4 * 32768 / ms / 1e9
    # the same MFMA loop on N(0,1) bf16 operands, long enough (tens of ms) for the clock to settle
    ops = dev.to_device(to_bf16(np.random.default_rng(7).standard_normal(8 * 256 * 8).astype(np.float32)))
    it2 = 5000
    mb.iris_mb_mfma_data(stream, ops, sink, blocks, 16)
    ms2 = min(event_time(hip, stream, lambda i: mb.iris_mb_mfma_data(stream, ops, sink, blocks, it2), 1) for _ in range(3))
    mfma_data = blocks * 4 * it2 * 16 * 32768 / ms2 / 1e9
    mb.iris_mb_mfma_data16(stream, ops, sink, blocks, 16)
    ms3 = min(event_time(hip, stream, lambda i: mb.iris_mb_mfma_data16(stream, ops, sink, blocks, it2), 1) for _ in range(3))
    mfma_data16 = blocks * 4 * it2 * 32 * 16384 / ms3 / 1e9
    n = 1 << 30
    a, b = lib.iris_dev_alloc(n), lib.iris_dev_alloc(n)
    assert a and b
    mb.iris_mb_copy(stream, b, a, n)
    cp = min(event_time(hip, stream, lambda i: mb.iris_mb_copy(stream, b, a, n), 2) for _ in range(3))
    rw = min(event_time(hip, stream, lambda i: mb.iris_mb_rmw(stream, a, n), 2) for _ in range(3))
    # the same in-place update at the size of ONE norm+rope call of the bench workload (27 MiB of rows), on 24
    # rotating buffers so that the rows come from HBM: what a launch of that size can reach at all
    small = 27 << 20
    ring = [lib.iris_dev_alloc(small) for _ in range(24)]
    assert all(ring)
    settle(lib, lambda i: mb.iris_mb_rmw(stream, _vp(ring[i % 24]), small), 20)
    rw_small = min(event_time(hip, stream, lambda i: mb.iris_mb_rmw(stream, _vp(ring[i % 24]), small), 48) for _ in range(3))
    # Yardsticks that are not this library's kernels or shapes: the runtime's own device-to-device copy
    # (hipMemcpyDtoDAsync on the library's stream), a read-only and a write-only stream; at 1 GiB and at the volume of
    # one fused Q+K norm+rope call of the bench workload (54 MiB of rows) on the rotating buffers.
    hip.rt.hipMemcpyDtoDAsync.argtypes = [_vp, _vp, C.c_size_t, _vp]
    dtod = lambda dst, src, nbytes: hip.rt.hipMemcpyDtoDAsync(dst, src, nbytes, stream)
    assert dtod(b, a, n) == 0
    lib.iris_dev_sync()
    dd = min(event_time(hip, stream, lambda i: dtod(b, a, n), 2) for _ in range(3))
    rd = min(event_time(hip, stream, lambda i: mb.iris_mb_read(stream, a, n, sink), 2) for _ in range(3))
    wr = min(event_time(hip, stream, lambda i: mb.iris_mb_write(stream, b, n), 2) for _ in range(3))
    pair = lambda i: (_vp(ring[(2 * i) % 24]), _vp(ring[(2 * i + 1) % 24]))
    dd_small = min(event_time(hip, stream, lambda i: dtod(*pair(i), small), 48) for _ in range(3))
    cp_small = min(event_time(hip, stream, lambda i: mb.iris_mb_copy(stream, *pair(i), small), 48) for _ in range(3))
    rd_small = min(event_time(hip, stream, lambda i: mb.iris_mb_read(stream, _vp(ring[i % 24]), small, sink), 48) for _ in range(3))
    wr_small = min(event_time(hip, stream, lambda i: mb.iris_mb_write(stream, _vp(ring[i % 24]), small), 48) for _ in range(3))
    # a SIMD's matrix core and its vector ALU, fed by two different waves: each stream alone, then both together
    mb.iris_mb_mfma_with_valu.argtypes = [_vp, _vp, C.c_int, C.c_int, C.c_int, C.c_int]
    two = {}
    for kind, name, per in ((1, "v_fma_f32", 12), (2, "v_exp_f32", 10), (3, "one_exp_per_two_fma", 11)):
        mi = 6000
        vi = mi * 8 * 16 // (16 * per)
        run = lambda m, v: min(event_time(hip, stream, lambda i: mb.iris_mb_mfma_with_valu(stream, sink, 256, m, v, kind), 2) for _ in range(2))
        run(16, 16)
        a_ms, v_ms, both_ms = run(mi, 0), run(0, vi), run(mi, vi)
        two[name] = {"products_alone_us": round(a_ms * 1e3, 1), "vector_alone_us": round(v_ms * 1e3, 1),
                     "together_us": round(both_ms * 1e3, 1), "together_over_longer": round(both_ms / max(a_ms, v_ms), 3),
                     "vector_cycles_per_instruction_alone": round(v_ms * 1e-3 * 2.4e9 / (vi * 16), 1)}
    two["note"] = ("256 blocks of eight waves, two per SIMD: waves 0-3 issue 16x16x32 products on constant operands, waves 4-7 "
                   "independent vector instructions of one kind. together_over_longer near 1: the two streams run at the same "
                   "time when they come from different waves; a wave that is alone issues one vector instruction per ~10 "
                   "cycles (cycles at the nominal 2.4 GHz)")
    dev.check()
    for p in [sink, a, b, ops] + ring:
        lib.iris_dev_free(p)
    yard = {"hip_memcpy_dtod_1gib_gbps": round(2 * n / dd / 1e6, 1), "read_only_1gib_gbps": round(n / rd / 1e6, 1),
            "write_only_1gib_gbps": round(n / wr / 1e6, 1),
            "hip_memcpy_dtod_27mib_cold_gbps": round(2 * small / dd_small / 1e6, 1),
            "hip_memcpy_dtod_27mib_cold_us": round(dd_small * 1e3, 2),
            "copy_27mib_cold_gbps": round(2 * small / cp_small / 1e6, 1), "copy_27mib_cold_us": round(cp_small * 1e3, 2),
            "read_only_27mib_cold_gbps": round(small / rd_small / 1e6, 1), "read_only_27mib_cold_us": round(rd_small * 1e3, 2),
            "write_only_27mib_cold_gbps": round(small / wr_small / 1e6, 1), "write_only_27mib_cold_us": round(wr_small * 1e3, 2),
            "note": "bytes counted read + written for the copies, one direction for the one-way streams; 27 MiB series "
                    "over 24 rotating buffers (648 MiB > the Infinity Cache), back-to-back launches between two events"}
    return {"streaming_yardsticks": yard, "matrix_and_vector_from_two_waves": two,
            "inplace_update_27mib_cold_us": round(rw_small * 1e3, 2),
            "inplace_update_27mib_cold_gbps": round(2 * small / rw_small / 1e6, 1),
            "mfma_only_tflops": round(mfma, 1), "mfma_only_frac_of_peak": round(mfma / PEAK_BF16_TFLOPS, 4),
            "mfma_only_normal_data_tflops": round(mfma_data, 1),
            "mfma_only_normal_data_frac_of_peak": round(mfma_data / PEAK_BF16_TFLOPS, 4),
            "mfma16x16x32_only_normal_data_tflops": round(mfma_data16, 1),
            "mfma16x16x32_only_normal_data_frac_of_peak": round(mfma_data16 / PEAK_BF16_TFLOPS, 4),
            "copy_1gib_gbps": round(2 * n / cp / 1e6, 1), "inplace_update_1gib_gbps": round(2 * n / rw / 1e6, 1),
            "note": "measured ceilings of this GPU: a pure 32x32x16 MFMA loop on constant operands (short burst), "
                    "the same and the 16x16x32 shape (the one the attention kernel uses) on N(0,1) operands "
                    "(sustained; the clock drops with the data-dependent power draw), and "
                    "streaming 16 B per lane, bytes counted read + written; inplace_update_27mib_cold is the "
                    "plain update at the data volume of one norm+rope call (launch gaps included, like norm_rope.*)"}


# ----------------------------------------------------------------------------- CPU baseline
def cpu_baseline(c):
    """The reference's BLAS-build CPU attention (heads over pthreads, per head
    sgemm -> softmax -> sgemm) on the same configuration, f32, on this host."""
    import oracle
    base = oracle.cpu_baseline()
    f = (c["buf"].astype(np.uint32) << 16).view(np.float32)
    q = np.ascontiguousarray(f[:, :c["q_dim"]])
    k = np.ascontiguousarray(f[:, c["q_dim"]:c["q_dim"] + c["kv_dim"]])
    v = np.ascontiguousarray(f[:, c["q_dim"] + c["kv_dim"]:])
    cores = base.online_cpus()
    box_share = int(os.environ.get("OMP_NUM_THREADS", "0") or 0)
    limit = min(cores, box_share) if box_share > 0 else cores
    calls, times = 8, []                  # 8 full calls: a few seconds of wall clock, ~30 core-seconds
    for _ in range(calls):
        t0 = time.perf_counter()
        _, threads = base.attention(q, k, v, c["heads"], c["kv_heads"], c["scale"], c["causal"], c["key_mask"],
                                    q_chunk=0, threads=limit)
        times.append(time.perf_counter() - t0)
    dt = float(np.mean(times[1:]))        # first call pays page faults and thread start
    flops = attention_flops(c)
    x = np.ascontiguousarray(q.reshape(c["seq"], c["heads"], c["hd"]))
    t1 = time.perf_counter()
    base.norm_rope(x, c["wq"], c["cos"], c["sin"], c["eps"], c["split_half"])
    dn = time.perf_counter() - t1
    t2 = time.perf_counter()
    oracle.oracle().flux2_joint_tables(*c["layout"])     # the reference's routine restated: libm on every entry
    dtab = time.perf_counter() - t2
    # the reference's own CPU attention (its generic, BLAS-free build, compiled from its sources where they were
    # present), when that library travelled with the tree: 6 of the heads, one thread
    ref_leg = None
    ref = oracle.reference()
    if ref is not None and not c["causal"] and c["key_mask"] is None and c["heads"] == c["kv_heads"]:
        nh = min(6, c["heads"])
        qs, ks, vs = (np.ascontiguousarray(a[:, :nh * c["hd"]]) for a in (q, k, v))
        o = np.empty_like(qs)
        ptr = lambda a: a.ctypes.data_as(_vp)
        t3 = time.perf_counter()
        ref.lib.iris_flash_attention(ptr(o), ptr(qs), ptr(ks), ptr(vs), C.c_int(c["seq"]), C.c_int(c["seq"]), C.c_int(nh),
                                     C.c_int(c["hd"]), C.c_float(c["scale"]))
        dr = time.perf_counter() - t3
        ref_leg = {"value": round(flops * nh / c["heads"] / dr / 1e12, 5), "unit": "TFLOP/s", "cores": 1, "kind": "reference",
                   "sample": f"iris_flash_attention of the compiled reference (its generic BLAS-free build, -O3 -ffast-math -mavx2 -mfma) on "
                             f"{nh} of the {c['heads']} heads, all {c['seq']} tokens: {dr:.2f} s"}
    return {"value": round(flops / dt / 1e12, 4), "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "reference_generic_build": ref_leg,
            "sample": f"{calls} full {c['name']} attention calls ({c['heads']}h x {c['seq']} tok, f32), mean of the last "
                      f"{calls - 1}: {dt:.2f} s each; "
                      f"sgemm from {os.path.basename(base.provider)}; host has {cores} CPUs online",
            "attention_seconds": round(dt, 3),
            "norm_rope_gbps": round(2 * x.nbytes / dn / 1e9, 3), "norm_rope_cores": 1,
            "rope_tables_ms": round(dtab * 1e3, 2)}


def cpu_seconds(c, calls=1):
    """Seconds per attention call of the reference's BLAS-build CPU structure on this host for configuration c
    (f32; 256-query chunks where the full score matrix would not fit, as the reference's FLUX.3 path does)."""
    import oracle
    base = oracle.cpu_baseline()
    f = (c["buf"].astype(np.uint32) << 16).view(np.float32)
    q = np.ascontiguousarray(f[:, :c["q_dim"]])
    k = np.ascontiguousarray(f[:, c["q_dim"]:c["q_dim"] + c["kv_dim"]])
    v = np.ascontiguousarray(f[:, c["q_dim"] + c["kv_dim"]:])
    cores = base.online_cpus()
    box_share = int(os.environ.get("OMP_NUM_THREADS", "0") or 0)
    limit = min(cores, box_share) if box_share > 0 else cores
    chunk = 256 if c["seq"] > 6000 else 0
    times, threads = [], 0
    for _ in range(calls + 1):
        t0 = time.perf_counter()
        _, threads = base.attention(q, k, v, c["heads"], c["kv_heads"], c["scale"], c["causal"], c["key_mask"],
                                    q_chunk=chunk, threads=limit)
        times.append(time.perf_counter() - t0)
    return float(np.mean(times[1:])), threads, chunk


# ----------------------------------------------------------------------------- main
def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--settle-ms", type=float, default=150.0,
                    help="untimed steps before the warmup until this much wall time has passed "
                         "(the clocks need tens of ms of load to settle); 0 = none")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-shapes", action="store_true", help="skip the per-configuration table")
    ap.add_argument("--no-machine", action="store_true", help="skip the MFMA-only / stream-copy ceilings")
    ap.add_argument("--no-variants", action="store_true",
                    help="skip the two alternative forms of the step (fused Q+K norm, Q norm inside attention), so that "
                         "a profile of the run holds the launches of the reference's call pattern only")
    ap.add_argument("--only", default="", metavar="CONFIG",
                    help="only launch one configuration's kernels, --steps times each, after the settling load: "
                         "C1, C2, C3-cond, C3-uncond, C4, C5 (norm+rope on Q, on K, attention) or VAE (the 512-wide "
                         "single head over 16384 tokens). For profiler runs of the other configurations.")
    ap.add_argument("--copy-only", type=int, default=0, metavar="MiB",
                    help="only launch the plain copy kernel on MiB of data, --steps times (the known-size "
                         "launch that hardware byte counters are scaled by)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (heads are independent, so the path would shard by "
                 "head with no exchange); run with --gpus 1")

    import iris_c_amd
    dev = iris_c_amd.IrisDev()            # raises if the HIP library is missing or no gfx950 GPU
    lib, hip = dev.lib, Hip()
    stream = lib.iris_dev_stream()
    rng = np.random.default_rng(20250101)
    if args.copy_only:
        print(json.dumps(copy_only(dev, hip, stream, args.copy_only << 20, args.steps)))
        return

    if args.only == "WIDE":
        print(json.dumps({"wide_heads": wide_heads(dev, hip, stream, rng, args.steps, min(args.settle_ms, 60))}))
        return
    if args.only:
        print(json.dumps(only_one(dev, hip, stream, rng, args.only, args.steps, args.settle_ms)))
        return

    c2 = make_config("C2", rng)
    copies = 8                             # 8 x 85 MB rows > 256 MB Infinity Cache: norm+rope reads come from HBM
    res = Resident(dev, c2, copies)
    flops = attention_flops(c2)

    # for the record: the same step timed right after the GPU sat idle during the uploads, clocks not yet settled
    lib.iris_dev_sync()
    t0 = time.perf_counter()
    for i in range(50):
        res.step(i)
    lib.iris_dev_sync()
    idle_ms = (time.perf_counter() - t0) / 50 * 1e3
    settle_steps = settle(lib, res.step, args.settle_ms)
    for i in range(args.warmup):
        res.step(i)
    lib.iris_dev_sync()
    t0 = time.perf_counter()
    for i in range(args.steps):
        res.step(i)
    lib.iris_dev_sync()
    wall = time.perf_counter() - t0
    ms_per_step = wall / args.steps * 1e3
    dev.check()

    # the same step with Q and K normalised by one launch, and with Q normalised inside the attention kernel
    # (reported beside `value`, never as `value`)
    fused_ms = qnorm_ms = None
    if not args.no_variants:
        t0 = time.perf_counter()
        for i in range(args.steps):
            res.step_fused_qk(i)
        lib.iris_dev_sync()
        fused_ms = (time.perf_counter() - t0) / args.steps * 1e3
        t0 = time.perf_counter()
        for i in range(args.steps):
            res.step_q_norm_in_attention(i)
        lib.iris_dev_sync()
        qnorm_ms = (time.perf_counter() - t0) / args.steps * 1e3

    # the double-stream block's call pattern: four norm launches on row sub-ranges (512 text rows, 4096 image rows; Q
    # and K each; two weight pairs) + attention; the same with one Q+K launch per stream, and with one launch in all
    double = None
    if not args.no_variants:
        txt = c2["layout"][0]
        double = {}
        for key, norm in (("four_norm_launches", res.norm_double_stream), ("one_qk_launch_per_stream", res.norm_double_stream_qk),
                          ("one_norm_launch", res.norm_double_stream_one)):
            def step(i, norm=norm):
                norm(i, txt); res.attention(i)
            for i in range(args.warmup):
                step(i)
            lib.iris_dev_sync()
            t0 = time.perf_counter()
            for i in range(args.steps):
                step(i)
            lib.iris_dev_sync()
            ms = (time.perf_counter() - t0) / args.steps * 1e3
            n_ms = event_time(hip, stream, lambda i, norm=norm: norm(i, txt), max(args.steps, 2 * copies))
            double[key] = {"ms_per_step": round(ms, 4), "tflops": round(flops / (ms * 1e-3) / 1e12, 2),
                           "norm_launches_us": round(n_ms * 1e3, 2)}
        dev.check()
        double["note"] = ("reference iris_transformer_flux.c:3786-3804: per stream (512 text rows, 4096 image rows) norm+rope on Q "
                          "and on K of the joint rows with the stream's own weights, then one attention over all 4608 rows; "
                          "norm_launches_us = the norm launches alone, back to back over rotating (cold) rows")

    # dominant kernel in its place in the step: events around the attention launch of every step (Q and K rows
    # just rewritten by the two norm calls, V rows not touched since the buffer's last turn)
    att = per_launch_times(hip, stream, res.attention, max(args.steps, 10),
                           before=lambda i: (res.norm_q(i), res.norm_k(i)))
    att_ms = float(np.mean(att))
    att_single = single_launch_ms(hip, stream, lib, res.attention)
    traffic, traffic_source, traffic_stale = traffic_on_file()
    kernel_name, kernel_grid = attention_kernel_name(lib, c2)
    # bandwidth-bound kernel: back-to-back launches over rotating buffers (cold) and one buffer (warm)
    reps = max(args.steps, 2 * copies)
    nr_q_ms = event_time(hip, stream, res.norm_q, reps)
    nr_qk_ms = event_time(hip, stream, res.norm_qk, reps)
    nr_warm_ms = event_time(hip, stream, lambda i: res.norm_q(0), reps)
    q_bytes = norm_rope_bytes(c2["seq"], c2["heads"])
    qk_bytes = q_bytes + norm_rope_bytes(c2["seq"], c2["kv_heads"])
    dev.check()

    out = {
        "metric": "joint_attention_tflops", "value": round(flops / (ms_per_step * 1e-3) / 1e12, 2), "unit": "TFLOP/s",
        "value_from_idle": round(flops / (idle_ms * 1e-3) / 1e12, 2),
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "settle_steps": settle_steps,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "C2: norm+rope(Q), norm+rope(K), joint attention; 24 heads x 128, 512 text + 4096 image "
                               "tokens, fused qkv rows (ldi 9216), one sequence",
                   "device": dev.name()},
        "first_50_steps_after_idle": {"ms_per_step": round(idle_ms, 4), "tflops": round(flops / (idle_ms * 1e-3) / 1e12, 2),
                                      "note": "before the settling load: the clocks take tens of ms of load to reach their "
                                              "steady state (includes first-launch costs)"},
        "step_with_fused_qk_norm": None if fused_ms is None else {
            "ms_per_step": round(fused_ms, 4), "tflops": round(flops / (fused_ms * 1e-3) / 1e12, 2),
            "note": "two launches: iris_dev_head_norm_rope_qk + iris_dev_attention"},
        "step_with_q_norm_in_attention": None if qnorm_ms is None else {
            "ms_per_step": round(qnorm_ms, 4), "tflops": round(flops / (qnorm_ms * 1e-3) / 1e12, 2),
            "note": "two launches: iris_dev_head_norm_rope on K + iris_dev_attention_qnorm"},
        "step_double_stream": double,
        "roofline": {"kernel": kernel_name, "kernel_grid": kernel_grid, "kernel_source_sha256": source_sha256(),
                     "bound": "mfma", "achieved": round(flops / (att_ms * 1e-3) / 1e12, 2),
                     "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": round(flops / (att_ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 4),
                     "traffic": traffic, "traffic_unit": "bytes per launch, hardware counters of a separate profiler run",
                     "traffic_source": traffic_source, "traffic_source_stale": traffic_stale,
                     "algorithmic_bytes": 4 * c2["seq"] * c2["q_dim"] * 2, "launch_ms": round(att_ms, 4),
                     "launch_ms_median": round(float(np.median(att)), 4), "launch_ms_min": round(float(np.min(att)), 4),
                     "single_launch_ms": round(att_single, 4),
                     "flops_per_launch": flops},
        "norm_rope": {"kernel": "k_norm_rope_hd128<false, false, false>", "bound": "hbm", "unit": "GB/s", "peak": PEAK_HBM_GBPS,
                      "bytes_per_call": q_bytes,
                      "q_call_us": round(nr_q_ms * 1e3, 2), "q_call_gbps": round(q_bytes / (nr_q_ms * 1e-3) / 1e9, 1),
                      "q_call_frac": round(q_bytes / (nr_q_ms * 1e-3) / 1e9 / PEAK_HBM_GBPS, 4),
                      "qk_fused_us": round(nr_qk_ms * 1e3, 2), "qk_fused_gbps": round(qk_bytes / (nr_qk_ms * 1e-3) / 1e9, 1),
                      "qk_fused_frac": round(qk_bytes / (nr_qk_ms * 1e-3) / 1e9 / PEAK_HBM_GBPS, 4),
                      "warm_cache_q_call_us": round(nr_warm_ms * 1e3, 2),
                      "warm_cache_q_call_frac": round(q_bytes / (nr_warm_ms * 1e-3) / 1e9 / PEAK_HBM_GBPS, 4),
                      "q_call_single_launch_us": round(single_launch_ms(hip, stream, lib, res.norm_q) * 1e3, 2),
                      "kernel_only_us_on_file": kernel_only_on_file(), "kernel_only_source": NORM_ROPE_PROFILE,
                      "note": "cold = 8 rotating 85 MB row buffers (> 256 MB Infinity Cache); warm = same buffer every call; "
                              "averages over back-to-back launches between two events. kernel_only_us_on_file: the kernel-only "
                              "durations of the same three series in the committed kernel trace (a separate profiler run)"},
    }
    res.free()

    if not args.no_shapes:
        shapes = []
        for name in ("C1", "C2", "C3-cond", "C3-uncond", "C4", "C5"):
            c = c2 if name == "C2" else make_config(name, rng)
            # enough rotating row buffers that the norm+rope reads come from HBM (> 2 x the 256 MB Infinity Cache)
            r = Resident(dev, c, int(min(64, max(2, np.ceil(600e6 / c["buf"].nbytes)))))
            for i in range(3):
                r.step(i)
            settle(lib, r.attention, args.settle_ms / 2)
            n = 20
            a = per_launch_times(hip, stream, r.attention, n)
            a_ms = float(np.mean(a))
            q_ms = event_time(hip, stream, r.norm_q, 2 * n)
            qk_ms = event_time(hip, stream, r.norm_qk, 2 * n)
            fl = attention_flops(c)
            qb = norm_rope_bytes(c["seq"], c["heads"])
            nb = qb + norm_rope_bytes(c["seq"], c["kv_heads"])
            entry = {"config": name, "seq": c["seq"], "heads": c["heads"], "kv_heads": c["kv_heads"],
                     "attention_ms": round(a_ms, 4), "attention_ms_median": round(float(np.median(a)), 4),
                     "attention_ms_min": round(float(np.min(a)), 4),
                     "attention_single_launch_ms": round(single_launch_ms(hip, stream, lib, r.attention), 4),
                     "attention_tflops": round(fl / a_ms / 1e9, 2),
                     "attention_frac_of_mfma_peak": round(fl / a_ms / 1e9 / PEAK_BF16_TFLOPS, 4),
                     "norm_rope_q_us": round(q_ms * 1e3, 2), "norm_rope_q_gbps": round(qb / q_ms / 1e6, 1),
                     "norm_rope_q_frac_of_hbm_peak": round(qb / q_ms / 1e6 / PEAK_HBM_GBPS, 4),
                     "norm_rope_qk_us": round(qk_ms * 1e3, 2), "norm_rope_qk_gbps": round(nb / qk_ms / 1e6, 1),
                     "norm_rope_qk_frac_of_hbm_peak": round(nb / qk_ms / 1e6 / PEAK_HBM_GBPS, 4)}
            eager_us, graph_us = step_times(hip, stream, lib, r.step)
            entry.update(step_us=round(eager_us, 2), step_us_in_hip_graph=round(graph_us, 2))
            if c["key_mask"] is not None:
                # the kernel stops at the last key tile that holds a valid key, so the time depends on the mask drawn
                # from the seed: the same launch with every key valid is timed beside it
                drawn, every = r.mask, dev.to_device(np.ones(c["seq"], np.int32))
                r.mask = every
                settle(lib, r.attention, args.settle_ms / 10)
                entry.update(valid_keys=int((c["key_mask"] != 0).sum()), attention_ms_with_every_key_valid=round(
                    float(np.mean(per_launch_times(hip, stream, r.attention, n))), 4))
                r.mask = drawn
                lib.iris_dev_sync()
                lib.iris_dev_free(every)
            dev.check()
            r.free()
            if not args.no_cpu:
                secs, threads, chunk = cpu_seconds(c)
                entry.update(cpu_seconds=round(secs, 4), cpu_tflops=round(fl / secs / 1e12, 4), cpu_threads=threads,
                             cpu_query_chunk=chunk)
            shapes.append(entry)
        # the VAE's mid-block attention of a 1024 x 1024 image: one head of 512 over 16384 tokens (no norm+rope in front)
        v = only_one(dev, hip, stream, rng, "VAE", 20, args.settle_ms / 2)
        shapes.append({"config": "VAE", "seq": 16384, "heads": 1, "kv_heads": 1, "head_dim": 512, "kernel": v["kernel"],
                       "attention_ms": v["attention_ms_mean"], "attention_ms_median": v["attention_ms_median"],
                       "attention_ms_min": v["attention_ms_min"], "attention_tflops": v["tflops"],
                       "attention_frac_of_mfma_peak": round(v["tflops"] / PEAK_BF16_TFLOPS, 4)})
        out["shapes"] = shapes

    if not args.no_shapes:
        out["other_ops"] = other_ops(dev, hip, stream, rng, args.settle_ms / 5)
        out["rope_tables"] = rope_table_times(dev, c2)
    if not args.no_machine:
        out["machine"] = machine_ceilings(dev, hip, stream)
        out["machine"]["attention_by_busy_cus"] = occupancy_probe(dev, hip, stream, rng, args.settle_ms / 3)
        # The ABI takes device pointers, so `value` has no host transfer in it. For a caller that had the
        # fused qkv rows in host memory, this is the rate with the upload of those rows counted.
        row_bytes = c2["buf"].nbytes
        d = lib.iris_dev_alloc(row_bytes)
        lib.iris_dev_upload(d, c2["buf"].ctypes.data_as(_vp), row_bytes)
        t0 = time.perf_counter()
        lib.iris_dev_upload(d, c2["buf"].ctypes.data_as(_vp), row_bytes)
        up = time.perf_counter() - t0
        lib.iris_dev_free(d)
        out["machine"]["host_upload_gbps"] = round(row_bytes / up / 1e9, 2)
        out["machine"]["pcie_inclusive_tflops"] = round(flops / (up + ms_per_step * 1e-3) / 1e12, 2)
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(c2)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
