"""The entry point that allocates nothing (l2j_running_sums_noalloc: the terms and sums pass through a fixed device
array of the library) against the entry point it is a variant of (l2j_running_sums, which allocates a device buffer
per call): bit-identical sums on two calls in a row, the second with a smaller input, so that what the first call
left in the array cannot leak into the second."""
import numpy as np
import pytest

import llama2j_amd as l2j

pytestmark = pytest.mark.gpu


def test_no_alloc_running_sums_equal_the_allocating_entry_point():
    g = l2j.Transformer(l2j.Config(64, 128, 1, 4, 4, 64, 8, 1))
    rng = np.random.default_rng(77)
    first = rng.random(36864).astype(np.float32)          # the largest input the array takes
    second = (rng.random(5000) * 1e-3).astype(np.float32)  # smaller, other magnitudes
    for terms in (first, second, second[:1], first[:1025]):
        want = g.running_sums(terms)
        got = g.running_sums_noalloc(terms)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), terms.size
        # and both are the sequential float32 sums (numpy's cumsum adds one element after the other)
        assert np.array_equal(got.view(np.uint32), np.cumsum(terms, dtype=np.float32).view(np.uint32)), terms.size
    with pytest.raises(l2j.L2JError) as e:
        g.running_sums_noalloc(np.ones(36865, np.float32))
    assert e.value.code == -2 and "36864" in str(e.value)
    g.close()
