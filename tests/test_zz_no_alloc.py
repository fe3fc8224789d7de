"""The entry point that allocates nothing: cct_hip_backward_bias_noalloc against
cct_hip_backward_bias, through the C ABI, on two calls in a row (the second with a smaller input,
so the built-in scratch still holds the first call's partial sums and counters)."""
import numpy as np
import pytest

from gpu_util import dev, driver, empty, host

pytestmark = pytest.mark.gpu


def test_backward_bias_noalloc_matches_backward_bias_twice_in_a_row(oracle):
    drv = driver()
    rng = np.random.default_rng(5)
    # (batch, depth, fmap): both split the batch over several workgroups per channel (scratch in use)
    for batch, depth, fmap in ((64, 96, 27 * 27), (16, 20, 24 * 24)):
        og = rng.standard_normal((batch, depth, fmap)).astype(np.float32)
        d_og = dev(og)
        want, got = empty((depth,)), empty((depth,))
        drv.backward_bias(want, d_og, fmap, depth, batch)
        drv.backward_bias_noalloc(got, d_og, fmap, depth, batch)
        np.testing.assert_array_equal(host(got), host(want))       # same kernel, same summation order
        ref = oracle.bias_backward(og.reshape(-1), fmap, depth, batch)
        assert np.abs(host(got) - ref).max() <= 1e-4 * np.abs(ref).max()
    # a third call on the first shape again: counters left by the smaller call do not disturb it
    batch, depth, fmap = 64, 96, 27 * 27
    og = rng.standard_normal((batch, depth, fmap)).astype(np.float32)
    want, got = empty((depth,)), empty((depth,))
    drv.backward_bias(want, dev(og), fmap, depth, batch)
    drv.backward_bias_noalloc(got, dev(og), fmap, depth, batch)
    np.testing.assert_array_equal(host(got), host(want))


def test_backward_bias_noalloc_rejects_sizes_beyond_its_scratch():
    from caffecontroll_amd import CctHipError
    drv = driver()
    og, out = empty((4, 5000, 4), fill=1.0), empty((5000,))
    with pytest.raises(CctHipError, match="exceeds the built-in scratch"):
        drv.backward_bias_noalloc(out, og, 4, 5000, 4)
