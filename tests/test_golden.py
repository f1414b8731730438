"""The committed fixture of benchmark configuration 1 pins the workload generator and the checker (CPU) and
the HIP path (GPU) to the same numbers."""
import os
import sys

import numpy as np
import pytest

import oracle

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden"))
from make_golden import c1_problem, digest  # noqa: E402

GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "c1_decode.npz"))


def test_generator_and_checker_reproduce_the_fixture():
    p = c1_problem()
    assert digest(p.pool) == str(GOLD["pool_sha256"]) and digest(p.q) == str(GOLD["q_sha256"])
    assert np.array_equal(p.indices, GOLD["indices"]) and np.array_equal(p.indptr, GOLD["indptr"])
    assert list(p.last_page_len) == [1, 16, 2, 15] and int(p.indptr[-1]) == 31  # 2+4+9+16 pages of the 64
    out, lse = oracle.batch_decode(p.q, p.dtype, p.oracle_kv(), p.Hq, want_lse=True)
    assert np.array_equal(out, GOLD["out"]) and np.array_equal(lse, GOLD["lse"])


@pytest.mark.gpu
def test_hip_path_matches_the_fixture():
    from _gpu import DeviceDecode
    from blitz_scale_amd._lib import BZ_F32
    p = c1_problem()
    dev = DeviceDecode(p)
    dev.plan()
    got32 = dev.decode(BZ_F32)
    assert np.abs(got32 - GOLD["out"]).max() <= 2e-5
    assert np.abs(dev.decode() - GOLD["out"]).max() <= 2e-3  # f16 result
