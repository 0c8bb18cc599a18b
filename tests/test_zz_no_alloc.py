"""The entry point that allocates nothing (TSHip_TopPSampleNoAlloc: the top-p pipeline on a fixed scratch array inside
the library) against the entry point it is a variant of (TSHip_TopPSample), through the C ABI: bit-equal choices on two
calls in a row, the second with a smaller input, so that what the first call left in the shared scratch cannot leak into
the second; then the size limit."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_no_alloc_top_p_matches_the_allocating_entry_point(oracle):
    from seq2seqsharp_amd import ops
    from seq2seqsharp_amd._lib import TSHipError
    from seq2seqsharp_amd.tensor import HipTensor as HT
    rng = np.random.default_rng(5)
    for rows, K in ((8, 32000), (3, 1500)):                  # the second call is smaller than the first
        p = oracle.softmax((2.0 * rng.standard_normal((rows, K))).astype(np.float32))
        p[1, 10:20] = p[1, 5]                                # exact ties
        p[2, ::3] = 0.0                                      # entries the reference drops
        u = rng.random(rows).astype(np.float32)
        dp, du = HT.from_numpy(p), HT.from_numpy(u)
        for top_p in (0.3, 0.9, 1.0):
            want = ops.toppsample(None, dp, du, top_p).numpy().reshape(-1)
            out = HT([rows, 1])
            got = ops.toppsample_noalloc(out, dp, du, top_p).numpy().reshape(-1)
            assert np.array_equal(got, want), (rows, K, top_p)
            assert np.array_equal(got, oracle.toppsample(p, top_p, 0.0, None, u))
    # beyond the fixed scratch: a clear error, nothing launched
    big = HT([16, 32000])
    with pytest.raises(TSHipError, match="scratch"):
        ops.toppsample_noalloc(HT([16, 1]), big, HT([16]), 0.9)
