"""GPU parity (bit-exact): embedding gather, last-token gather and argmax through the C ABI against the
CPU checker, at the reference's shapes (hidden 4096/5120/8192, vocab 32000/128256) and at ragged and
unaligned ones."""
import numpy as np
import pytest
import torch

import oracle
from blitz_scale_amd import kernel as K
from blitz_scale_amd import workloads as wl
from blitz_scale_amd._lib import BZ_BF16, BZ_F16

from _gpu import to_dev, to_host_bits

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [BZ_F16, BZ_BF16])
@pytest.mark.parametrize("vocab,hidden,n", [(32000, 4096, 257), (128256, 4096, 64), (1000, 5120, 1), (50, 8, 33)])
def test_embedding(dtype, vocab, hidden, n):
    rng = np.random.default_rng(vocab + n)
    w = rng.integers(0, 1 << 16, size=(vocab, hidden), dtype=np.uint16)
    ids = rng.integers(0, vocab, size=n).astype(np.uint32)
    ids[0], ids[-1] = vocab - 1, 0
    wd = to_dev(w, dtype)
    idd = torch.from_numpy(ids.view(np.int32)).cuda()
    out = torch.zeros((n, hidden), dtype=wd.dtype, device="cuda")
    K.embedding(out, idd, wd, n, hidden)
    torch.cuda.synchronize()
    assert np.array_equal(to_host_bits(out), oracle.embedding(ids, w))
    # scatter variant into a larger zeroed buffer
    rows = n + 5
    loc = rng.permutation(rows)[:n].astype(np.int32)
    out2 = torch.zeros((rows, hidden), dtype=wd.dtype, device="cuda")
    K.embedding(out2, idd, wd, n, hidden, out_loc=torch.from_numpy(loc).cuda())
    torch.cuda.synchronize()
    assert np.array_equal(to_host_bits(out2), oracle.embedding(ids, w, out_rows=rows, out_loc=loc))


@pytest.mark.parametrize("dtype", [BZ_F16, BZ_BF16])
@pytest.mark.parametrize("hidden", [4096, 8192, 264])
def test_gather_last_token(dtype, hidden):
    rng = np.random.default_rng(hidden)
    lens = np.array([5, 1, 0, 300, 17, 0, 64], np.int64)  # two empty requests
    ip = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    tok = rng.integers(1, 1 << 16, size=(int(ip[-1]), hidden), dtype=np.uint16)
    out = torch.full((len(lens), hidden), 7.0, dtype=to_dev(tok[:1], dtype).dtype, device="cuda")
    K.gather_last_token(out, to_dev(tok, dtype), torch.from_numpy(ip).cuda(), int(ip[-1]), len(lens), hidden)
    torch.cuda.synchronize()
    assert np.array_equal(to_host_bits(out), oracle.gather_last_token(tok, ip))


@pytest.mark.parametrize("dtype", [BZ_F16, BZ_BF16])
@pytest.mark.parametrize("batch,length", [(64, 32000), (128, 128256), (3, 1), (5, 7), (4, 1031), (2, 8200)])
def test_batch_find_max(dtype, batch, length):
    rng = np.random.default_rng(batch * 7 + length)
    x = wl.randn_bits(rng, (batch, length), dtype)
    if length > 16:  # plant ties, NaN and -inf
        f = wl.to_f32(x, dtype)
        x[0, length - 1] = x[0, int(np.argmax(f[0]))]            # tie at the far end: the first one wins
        x[1 % batch, 3] = wl.to_bits(np.float32([np.nan]), dtype)[0]
        x[2 % batch, :] = wl.to_bits(np.float32([-np.inf]), dtype)[0]
    xd = to_dev(x, dtype)
    out = torch.full((batch,), -1, dtype=torch.int32, device="cuda")
    K.batch_find_max(out, xd, batch, length)
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy().view(np.uint32), oracle.batch_find_max(x, dtype))
    # an odd row length makes every second row start off a 16-byte boundary: covered by 1031 and 7 above


def test_argmax_of_all_nan_row_is_zero():
    x = np.full((2, 100), 0x7E00, np.uint16)  # f16 quiet NaN
    out = torch.full((2,), -1, dtype=torch.int32, device="cuda")
    K.batch_find_max(out, to_dev(x, BZ_F16), 2, 100)
    torch.cuda.synchronize()
    assert out.cpu().tolist() == [0, 0]


@pytest.mark.parametrize("dtype", [BZ_F16, BZ_BF16])
@pytest.mark.parametrize("length", [8, 40, 9000, 128256])
def test_argmax_special_values_anywhere_in_the_row(dtype, length):
    """Ties (also between -0 and +0, and between values met by different lanes, loads and waves), -inf, NaN of both
    signs, subnormals and rows without a finite value: the smallest index of the largest non-NaN value."""
    rng = np.random.default_rng(length)
    enc = (lambda v: wl.to_bits(np.asarray(v, np.float32), dtype))
    ninf, nan = np.float32(-np.inf), np.float32(np.nan)
    neg_nan = np.uint16(0xFE00 if dtype == BZ_F16 else 0xFFC0)
    sub = np.uint16(0x0001)  # smallest positive subnormal of either format

    def fill(v):
        return np.full(length, enc([v])[0], np.uint16)

    def at(n):
        return np.sort(rng.choice(length, size=min(n, length), replace=False))

    rows = []
    r = fill(1.0); r[at(5)] = enc([5.0])[0]; rows.append(r)                     # ties of the maximum
    rows.append(fill(ninf))                                                       # all -inf: index 0
    r = fill(ninf); r[at(1)] = enc([-65504.0])[0]; rows.append(r)                 # one finite value, very negative
    r = fill(nan); p = at(3); r[p] = enc([7.0])[0]; r[p[0]] = enc([3.0])[0]; rows.append(r)  # NaN never wins
    rows.append(fill(nan))                                                        # no non-NaN element: 0
    r = fill(-1.0); p = at(4); r[p] = enc([0.0])[0]; r[p[::2]] = enc([-0.0])[0]; rows.append(r)  # -0 == +0: the first
    r = fill(ninf); r[:] = neg_nan; r[at(2)] = enc([ninf])[0]; rows.append(r)     # negative NaN against -inf
    r = fill(0.0); r[at(2)] = sub; rows.append(r)                                 # a subnormal above zero
    r = fill(-0.0); r[0] = enc([nan])[0]; rows.append(r)                          # NaN first, then zeros
    x = np.stack(rows)
    out = torch.full((len(rows),), -1, dtype=torch.int32, device="cuda")
    K.batch_find_max(out, to_dev(x, dtype), len(rows), length)
    torch.cuda.synchronize()
    want = oracle.batch_find_max(x, dtype)
    f = wl.to_f32(x, dtype)
    assert want[4] == 0 and (length < 2 or want[8] == 1) and f[0, want[0]] == 5.0  # (the checker itself, on these rows)
    assert np.array_equal(out.cpu().numpy().view(np.uint32), want)
