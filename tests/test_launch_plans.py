"""The launchers' choices are host arithmetic: which workgroup shape an attention problem gets, and for the two-size
grid how many workgroups of 256 and of 192 queries per head (iris_hip_fa_hd128_plan); which GEMM kernel and tile width
a linear layer gets (iris_hip_linear_plan). Runs without a GPU: the library loads, nothing is launched."""
import ctypes as C

import pytest

import iris_c_amd


@pytest.fixture(scope="module")
def plan():
    lib = C.CDLL(iris_c_amd.LIB_PATH)
    lib.iris_hip_fa_hd128_plan.argtypes = [C.c_int] * 4 + [C.POINTER(C.c_int)]
    lib.iris_hip_fa_hd128_plan.restype = None

    def call(seq_q, seq_k, heads, causal=0):
        out = (C.c_int * 5)()
        lib.iris_hip_fa_hd128_plan(seq_q, seq_k, heads, causal, out)
        return dict(kind=out[0], waves=out[1], nb=out[2], full=out[3], tails=out[4])
    return call


def test_benchmark_configurations(plan):
    assert plan(320, 320, 24) == dict(kind=0, waves=2, nb=1, full=0, tails=0)            # C1: 480 waves of 16 queries
    assert plan(512, 512, 32, 1) == dict(kind=0, waves=4, nb=1, full=0, tails=0)         # C4: 1024 such waves
    assert plan(4608, 4608, 24) == dict(kind=1, waves=8, nb=2, full=10, tails=11)        # C2: 432 x 256 queries = 1.69 rounds
    assert plan(4352, 4352, 30) == dict(kind=0, waves=8, nb=2, full=0, tails=0)          # C3: 510 workgroups, two full rounds
    p = plan(12800, 12800, 24)                                                            # C5: 4.69 rounds
    assert p["kind"] == 1 and 256 * p["full"] + 192 * p["tails"] >= 12800 and 24 * p["full"] <= 4 * 256


def test_short_sequences_split_the_keys_when_workgroups_are_few(plan):
    assert plan(512, 512, 1)["kind"] == 2 and plan(512, 512, 1)["waves"] == 4             # 8 key tiles: four waves
    assert plan(32, 448, 8)["kind"] == 2                                                  # 7 tiles: two turns of four waves + merge
    assert plan(128, 200, 4)["kind"] == 0                                                 # 4 tiles: the chain is shorter than a merge
    assert plan(64, 64, 8)["kind"] == 0                                                   # one key tile: nothing to split
    assert plan(512, 512, 32)["kind"] == 0                                                # 512 (head, 32-query block) pairs > 256 CUs


@pytest.mark.parametrize("heads", [8, 16, 20, 24, 30, 32, 40, 48])
def test_two_size_grids_cover_every_query_and_never_lose_to_one_size(plan, heads):
    for seq in range(2048 * 16 // heads + 64, 9000, 331):
        p = plan(seq, seq, heads)
        assert p["waves"] in (4, 8) and p["nb"] == 2, (seq, p)
        if p["kind"] == 1:
            assert p["full"] >= 0 and p["tails"] >= 0 and 256 * p["full"] + 192 * p["tails"] >= seq, (seq, p)
            assert 256 * p["full"] <= seq and 192 * (p["tails"] - 1) < seq - 256 * p["full"], (seq, p)     # no empty workgroup
            # priced per shader engine (8 CUs, a 192-query workgroup at 0.78): never above the rounds of the 8-wave kernel
            full_x, tail_x = -(-p["full"] * heads // 8), -(-p["tails"] * heads // 8)
            rounds_one_size = -(-(-(-seq // 256) * heads) // 256)
            per_engine = -(-(full_x + tail_x) // 4)
            assert per_engine <= 8 * (rounds_one_size + 1), (seq, p)
        assert plan(seq, seq, heads, 1)["kind"] == 0                                      # causal calls keep one size


def test_exact_rounds_keep_one_size(plan):
    for heads, seq in ((16, 4096), (32, 2048), (8, 8192), (32, 4096), (30, 4352)):
        assert plan(seq, seq, heads)["kind"] == 0, (heads, seq)


# ------------------------------------------------------------------ the linear layers' kernel choice
@pytest.fixture(scope="module")
def linear_plan():
    lib = C.CDLL(iris_c_amd.LIB_PATH)
    lib.iris_hip_linear_plan.argtypes = [C.c_int] * 4 + [C.POINTER(C.c_int)]
    lib.iris_hip_linear_plan.restype = None

    def call(rows, k, out, out_bytes=2):
        p = (C.c_int * 2)()
        lib.iris_hip_linear_plan(rows, k, out, out_bytes, p)
        return p[0], p[1]
    return call


def test_linear_layers_of_the_models_take_the_four_wave_kernel_in_the_width_that_fills_the_rounds(linear_plan):
    assert linear_plan(4608, 3072, 9216) == (3, 224)        # 756 tiles = 2.95 rounds of 256 CUs (648 of 256 columns: 2.53)
    assert linear_plan(4608, 3072, 3072) == (3, 224)        # 252 tiles: one round (216 of 256 columns: also one, but wider)
    assert linear_plan(4608, 3072, 27648) == (3, 256)       # 1944 tiles = 7.6 rounds; narrower tiles need 9 or 11
    assert linear_plan(4608, 3072, 18432)[1] in (224, 192)  # 1296 tiles of 256 columns are 5.06 rounds
    for rows, k, out in ((300, 128, 258), (257, 64, 257), (512, 192, 256)):
        assert linear_plan(rows, k, out)[0] == 2             # k not a multiple of 128, or rows of 2 bytes not 16-byte aligned
    assert linear_plan(700, 256, 1000) == (3, 256) or linear_plan(700, 256, 1000)[0] == 3
    assert linear_plan(64, 128, 64)[0] == 1 and linear_plan(37, 27, 19)[0] == 0
    assert linear_plan(512, 256, 258, 4)[0] == 2             # f32 rows of 258 columns cannot take 16-byte stores


def test_profile_summaries_say_which_source_they_were_taken_on():
    """Every summary under profiles/ names the commit and the hash of the kernel source it was measured on, and
    bench.py can tell from the C2 counter file whether its traffic figure belongs to the kernel source in the tree."""
    import glob
    import os
    import re
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    files = sorted(glob.glob(os.path.join(root, "profiles", "*.txt")))
    assert len(files) >= 10
    for path in files:
        text = open(path).read()
        assert re.search(r"^taken_on_commit: [0-9a-f]{40}$", text, re.M), path
        assert re.search(r"^kernel_source_sha256: [0-9a-f]{16}\s+\(iris_c_amd/csrc/\w+\.hip\)$", text, re.M), path
    sys.path.insert(0, root)
    import bench
    nbytes, source, stale = bench.traffic_on_file()
    assert nbytes and nbytes > 113_246_208 and source.endswith("hbm_traffic.txt") and stale in (True, False)
