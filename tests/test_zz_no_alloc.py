"""iris_dev_group_norm_noalloc: the group norm whose scratch is an array inside the library (for
callers that cannot allocate device memory), through the C ABI against iris_dev_group_norm, which
allocates its scratch: same kernels, so the same bits; and both against the oracle. Two calls in a
row, the second on a smaller input (the shared array keeps the first call's contents)."""
import numpy as np
import pytest

from gpu_harness import Dev

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    return Dev()


def both(dev, orc, hw, c, groups, silu, seed):
    rng = np.random.default_rng(seed)
    img = (rng.standard_normal((hw, c)) * 2 + 0.5).astype(np.float32)
    gamma = (1 + 0.1 * rng.standard_normal(c)).astype(np.float32)
    beta = (0.1 * rng.standard_normal(c)).astype(np.float32)
    d_in, d_g, d_b = dev.put(img), dev.put(gamma), dev.put(beta)
    outs = []
    for entry in (dev.lib.iris_dev_group_norm, dev.lib.iris_dev_group_norm_noalloc):
        d_out = dev.put(np.full((hw, c), np.nan, np.float32))
        entry(d_out, d_in, d_g, d_b, hw, c, groups, 1e-6, int(silu))
        dev.check()
        outs.append(dev.get(d_out, (hw, c), np.float32))
    dev.free_all()
    want = orc.dev_group_norm(img, gamma, beta, groups, 1e-6, silu)
    return outs[0], outs[1], want


def test_two_calls_in_a_row_the_second_smaller(dev, orc):
    # a VAE-sized image (coalesced statistics kernel, many partial moments per group), then a much smaller one
    for hw, c, groups, silu, seed in ((128 * 128, 128, 32, True, 1), (9 * 7, 64, 32, False, 2)):
        alloc, noalloc, want = both(dev, orc, hw, c, groups, silu, seed)
        assert np.array_equal(alloc.view(np.uint32), noalloc.view(np.uint32)), (hw, c)
        np.testing.assert_allclose(noalloc, want, atol=2e-5)       # the bar of the allocating entry's own test


def test_shapes_of_the_scalar_statistics_kernel_and_the_group_limit(dev, orc):
    # channel counts that the coalesced kernel does not take; 64 groups is the most the built-in scratch holds
    for hw, c, groups, silu, seed in ((300, 6, 3, True, 3), (50, 128, 64, False, 4), (1, 8, 2, False, 5)):
        alloc, noalloc, want = both(dev, orc, hw, c, groups, silu, seed)
        assert np.array_equal(alloc.view(np.uint32), noalloc.view(np.uint32)), (hw, c)
        np.testing.assert_allclose(noalloc, want, atol=2e-5)


def test_more_groups_than_the_scratch_holds_is_refused(dev):
    hw, c, groups = 10, 130, 65
    img = np.ones((hw, c), np.float32)
    d_in, d_g, d_b = dev.put(img), dev.put(np.ones(c, np.float32)), dev.put(np.zeros(c, np.float32))
    d_out = dev.put(np.full((hw, c), 7.0, np.float32))
    dev.lib.iris_dev_last_error()
    dev.lib.iris_dev_group_norm_noalloc(d_out, d_in, d_g, d_b, hw, c, groups, 1e-6, 0)
    assert dev.lib.iris_dev_last_error() != 0
    assert (dev.get(d_out, (hw, c), np.float32) == 7.0).all()          # nothing was launched
    dev.lib.iris_dev_group_norm(d_out, d_in, d_g, d_b, hw, c, groups, 1e-6, 0)   # the allocating entry takes it
    dev.check()
    assert np.abs(dev.get(d_out, (hw, c), np.float32)).max() < 1e-2     # a constant image normalises to ~0
    dev.free_all()
