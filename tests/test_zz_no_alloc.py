"""The entry point that allocates nothing (bam_scan_noalloc) against the one it is a variant of (bam_scan), through the C-ABI."""
import numpy as np
import pytest

import oracle
from test_gpu_parity import Rig, SEED, bam, _u64  # noqa: F401  (bam is the module fixture)

pytestmark = pytest.mark.gpu


def test_scan_without_allocation_matches_scan_twice_in_a_row(bam):
    """two calls in a row on one device, the second with a smaller input (the scratch array keeps what the first call
    left in it), each bit-exact against bam_scan and against the running sums of the store's words; then the limit"""
    import torch
    n_elems = 1 << 20
    with Rig(bam, n_elems * 8, n_queues=8, depth=256) as r:
        a = r.array(n_elems, 4096, 512)
        words = oracle.store(SEED, 0, n_elems)
        for n, block in ((n_elems - 3, 256), (70_001, 64), (1, 64), (0, 64)):
            out = torch.full((n + 1,), -1, dtype=torch.int64, device="cuda")
            a.scan_noalloc(n, out, block_size=block)
            torch.cuda.synchronize()
            want = _u64(a.scan(n, block_size=block))
            got = _u64(out)
            assert np.array_equal(got, want), "n = %d" % n
            assert got[0] == 0 and np.array_equal(got[1:], np.cumsum(words[:n], dtype=np.uint64))
        assert not r.c.aborted()
    # beyond what the fixed scratch array holds (65536 blocks of 2 * 64 elements): refused with a message, nothing launched
    n_big = (1 << 23) + 1
    with Rig(bam, (n_big * 8 + 4095) // 4096 * 4096, n_queues=4, depth=64) as r:
        a = r.array(n_big, 4096, 64)
        out = torch.full((8,), 7, dtype=torch.int64, device="cuda")
        with pytest.raises(Exception) as e:
            a.scan_noalloc(n_big, out, block_size=64)
        assert "block totals" in str(e.value)
        torch.cuda.synchronize()
        assert bool((out == 7).all())
        a.scan_noalloc(1000, torch.empty(1001, dtype=torch.int64, device="cuda"), block_size=64)      # within the limit on the same array: fine
        torch.cuda.synchronize()
        assert not r.c.aborted()
