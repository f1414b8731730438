"""Pool planes larger than 4 GiB: page ids whose element offset exceeds 2^31 and whose byte offset
exceeds 2^32 (a 288 GB card holds millions of 64 KiB pages).  The same problem is laid out twice: on the
host with small page ids for the CPU checker, and on the device with most pages moved 70 000 pages up
(page placement does not change the result: the checker's page-permutation invariance).  Decode (MFMA
and general kernel), append, prefill store and the migration pack are run on the high pages and compared
with the checker's results on the low ones; copies bit-exact, attention max-abs <= 2e-3 (+ bf16 step)."""
import os

import numpy as np
import pytest
import torch

import oracle
from blitz_scale_amd import kernel as K
from blitz_scale_amd import workloads as wl
from blitz_scale_amd._lib import BZ_BF16, BZ_LAYOUT_HND, BZ_ROPE_NONE

from _gpu import TORCH_OF, to_dev, to_host_bits
from _util import DecodeProblem, ulp_tol

pytestmark = pytest.mark.gpu

HIGH = 70000  # pages; x 32768 elements x 2 bytes = 4.59 GB


class HighPool:
    def __init__(self, p):
        self.p = p
        sp = p.stride_page
        assert HIGH * sp > 2 ** 31 and HIGH * sp * 2 > 2 ** 32
        self.total_pages = HIGH + p.pool_pages
        self.pool = torch.empty(self.total_pages * sp, dtype=TORCH_OF[p.dtype], device="cuda")
        # sequence 0 keeps its low pages, the others move up
        self.indices = p.indices.copy()
        self.indices[p.indptr[1]:] += HIGH
        host = torch.from_numpy(p.pool.view(np.int16))
        view = self.pool.view(torch.int16)
        for old, new in zip(p.indices, self.indices):  # plain tensor copies, none of the library's code
            view[int(new) * sp:(int(new) + 1) * sp] = host[int(old) * sp:(int(old) + 1) * sp].cuda()
        self.pt = K.PageTable(p.B, p.P, p.Hkv, p.D, self.pool, layout=p.layout)
        self.pt.indices, self.pt.indptr, self.pt.last_page_len = self.indices, p.indptr, p.last_page_len
        self.pt.upload()
        self.float_ws = torch.empty(32 << 20, dtype=torch.uint8, device="cuda")
        self.int_ws = torch.empty(8 << 20, dtype=torch.uint8, device="cuda")
        self.handler = K.BlitzBatchDecodeHandler()

    def page_bits(self, new_id):
        sp = self.p.stride_page
        return to_host_bits(self.pool[int(new_id) * sp:(int(new_id) + 1) * sp])

    def assert_pages_equal(self, pool_low):
        sp = self.p.stride_page
        for old, new in zip(self.p.indices, self.indices):
            assert np.array_equal(self.page_bits(new), pool_low[int(old) * sp:(int(old) + 1) * sp]), (old, new)


def test_pool_offsets_beyond_four_gib():
    dtype, Hq, Hkv, D, P = BZ_BF16, 32, 8, 128, 16
    p = DecodeProblem(0x4616, [100, 2100, 33, 700], Hq, Hkv, D, P, dtype, layout=BZ_LAYOUT_HND)
    hp = HighPool(p)
    ref = oracle.batch_decode(p.q, dtype, p.oracle_kv(), Hq, rope_mode=BZ_ROPE_NONE)
    q = to_dev(p.q, dtype)
    for path in ("mfma", "general"):
        if path == "general":
            os.environ["BZ_DECODE_PATH"] = "general"
        try:
            hp.handler.plan(hp.float_ws, hp.float_ws.numel(), hp.int_ws, hp.int_ws.numel(), p.indptr, p.last_page_len,
                            p.B, Hq, Hkv, D, P, split_tokens=512)
        finally:
            os.environ.pop("BZ_DECODE_PATH", None)
        out = torch.full((p.B, Hq, D), float("nan"), dtype=TORCH_OF[dtype], device="cuda")
        K.batch_decode_attention(hp.handler, q, hp.pt, out, Hq, rope_mode=BZ_ROPE_NONE)
        torch.cuda.synchronize()
        got = out.float().cpu().numpy()
        assert (np.abs(got - ref) <= ulp_tol(ref, dtype)).all(), (path, float(np.abs(got - ref).max()))

    # append (raw copy): the new rows land in the high pages, bit for bit where the checker puts them
    rng = np.random.default_rng(3)
    kn, vn = wl.randn_bits(rng, (p.B, Hkv, D), dtype), wl.randn_bits(rng, (p.B, Hkv, D), dtype)
    low = p.pool.copy()
    oracle.append_decode_kv(p.oracle_kv(low), kn, vn, dtype)
    K.append_decode_kv_cache(hp.pt, to_dev(kn, dtype), to_dev(vn, dtype))
    torch.cuda.synchronize()
    assert (low != p.pool).any()
    hp.assert_pages_equal(low)

    # prefill store of whole sequences over the same table
    lens = [int(c) - 1 for c in p.ctx]
    indptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    N = int(indptr[-1])
    k, v = wl.randn_bits(rng, (N, Hkv, D), dtype), wl.randn_bits(rng, (N, Hkv, D), dtype)
    oracle.store_prefill_kv(p.oracle_kv(low), k, v, dtype, indptr)
    K.store_prefill_kv_cache(hp.pt, to_dev(k, dtype), to_dev(v, dtype), torch.from_numpy(indptr).cuda(), num_tokens=N)
    torch.cuda.synchronize()
    hp.assert_pages_equal(low)

    # migration payload gathered from the high pages == the checker's gathered from the low ones
    ids_low = p.indices[p.indptr[1]:p.indptr[2]].astype(np.int32)
    ids_high = hp.indices[p.indptr[1]:p.indptr[2]].astype(np.int32)
    want = oracle.kv_pages_pack(low, dtype, p.pool_pages, p.stride_page, ids_low, 0, 1)
    wire = torch.zeros(want.nbytes, dtype=torch.uint8, device="cuda")
    K.pack_kv_pages(hp.pt, hp.total_pages, torch.from_numpy(ids_high).cuda(), 0, 1, wire)
    torch.cuda.synchronize()
    assert np.array_equal(wire.cpu().numpy(), want.view(np.uint8))
    # ... and scattered back into other high pages
    hp.pool.view(torch.int16)[(HIGH - 500) * p.stride_page:HIGH * p.stride_page] = 0
    dst = (np.arange(len(ids_high)) + HIGH - 400).astype(np.int32)
    K.unpack_kv_pages(hp.pt, hp.total_pages, torch.from_numpy(dst).cuda(), 0, 1, wire)
    torch.cuda.synchronize()
    for s_id, d_id in zip(ids_high, dst):
        assert np.array_equal(hp.page_bits(d_id), hp.page_bits(s_id))
