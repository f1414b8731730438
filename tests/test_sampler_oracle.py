"""CPU tests pinning the checker's row gathers and argmax (src/kernel/embedding.cu, sampler.cu) against
numpy: plain fancy indexing for the gathers, numpy.argmax on the decoded values for the argmax
(numpy.argmax returns the first maximum, which is the tie rule the checker states), plus the special
cases: ties, -inf rows, NaN entries, rows below the reference's -65400 starting value."""
import numpy as np
import pytest

import oracle
from blitz_scale_amd import workloads as wl
from blitz_scale_amd._lib import BZ_BF16, BZ_F16


def test_embedding_is_a_row_gather():
    rng = np.random.default_rng(1)
    w = rng.integers(0, 1 << 16, size=(1000, 64), dtype=np.uint16)
    ids = rng.integers(0, 1000, size=37).astype(np.uint32)
    assert np.array_equal(oracle.embedding(ids, w), w[ids])
    loc = rng.permutation(50)[:37].astype(np.int32)  # scatter into a zeroed buffer (the TP variant)
    out = oracle.embedding(ids, w, out_rows=50, out_loc=loc)
    want = np.zeros((50, 64), np.uint16)
    want[loc] = w[ids]
    assert np.array_equal(out, want)


def test_gather_last_token_takes_whole_rows_and_zeroes_empty_requests():
    rng = np.random.default_rng(2)
    tok = rng.integers(1, 1 << 16, size=(20, 48), dtype=np.uint16)
    ip = np.array([0, 3, 3, 11, 20], np.int32)  # second request is empty
    out = oracle.gather_last_token(tok, ip)
    assert np.array_equal(out[0], tok[2]) and np.array_equal(out[2], tok[10]) and np.array_equal(out[3], tok[19])
    assert not out[1].any()


@pytest.mark.parametrize("dtype", [BZ_F16, BZ_BF16])
def test_batch_find_max_matches_numpy_argmax(dtype):
    rng = np.random.default_rng(3)
    x = wl.randn_bits(rng, (9, 1000), dtype)
    assert np.array_equal(oracle.batch_find_max(x, dtype), np.argmax(wl.to_f32(x, dtype), axis=1))
    # 16-bit values collide often in 50k draws: the first maximum must win
    y = wl.randn_bits(rng, (4, 50000), dtype)
    f = wl.to_f32(y, dtype)
    assert (np.sum(f == f.max(axis=1, keepdims=True), axis=1) >= 1).all()
    assert np.array_equal(oracle.batch_find_max(y, dtype), np.argmax(f, axis=1))


@pytest.mark.parametrize("dtype", [BZ_F16, BZ_BF16])
def test_batch_find_max_special_cases(dtype):
    enc = (lambda v: wl.to_bits(np.asarray(v, np.float32), dtype))
    ninf, nan = np.float32(-np.inf), np.float32(np.nan)
    rows = np.stack([
        enc([1, 5, 5, 2, 5, 0, 0, 0]),                 # tie: smallest index
        enc([ninf] * 8),                                # all -inf: index 0
        enc([ninf, ninf, -70000 if dtype == BZ_BF16 else -65504, ninf, ninf, ninf, ninf, ninf]),  # below -65400
        enc([nan, 3, nan, 7, nan, 7, 1, 0]),            # NaN never wins
        enc([nan] * 8),                                 # no non-NaN element: 0
        enc([-0.0, 0.0, -1, -2, -3, -4, -5, -6]),       # -0 == +0: first one
    ])
    assert oracle.batch_find_max(rows, dtype).tolist() == [1, 0, 2, 3, 0, 0]
