"""CPU tests of the host page-table logic (bz_cm_* in libbz_hip.so, no GPU needed) against the
checker's restatement of src/blitz/cache_manager.h and src/blitz/batch.h: bit-exact integer results
over random sequences of prefill / grow / filter / extend / release, plus the invariants the
reference asserts (cache_manager.h:214-215,301,320-323; batch.h:399,540-542)."""
import ctypes as C

import numpy as np
import pytest

import oracle
from blitz_scale_amd import _lib
from blitz_scale_amd._lib import BZ_ERR_BAD_ARG, BZ_ERR_NO_PAGES, BZ_F16, BZ_LAYOUT_HND


class Product:
    def __init__(self, P, max_pages):
        self.lib = _lib.load()
        self.cm = C.c_void_p()
        assert self.lib.bz_cm_create(C.byref(self.cm), 8, 2, 128, P, max_pages, BZ_F16, BZ_LAYOUT_HND, 0) == 0

    def close(self):
        self.lib.bz_cm_destroy(self.cm)

    def prefill(self, lens):
        a = np.asarray(lens, np.int32)
        bid = C.c_int(-1)
        rc = self.lib.bz_cm_batch_prefill(self.cm, a.ctypes.data_as(C.c_void_p), len(a), C.byref(bid))
        return rc, bid.value

    def grow(self, bid):
        return self.lib.bz_cm_batch_grow(self.cm, bid)

    def filter(self, bid, keep):
        k = np.asarray(keep, np.uint32)
        return self.lib.bz_cm_batch_filter(self.cm, bid, k.ctypes.data_as(C.c_void_p), len(k))

    def extend(self, dst, src):
        return self.lib.bz_cm_batch_extend(self.cm, dst, src)

    def release(self, bid):
        return self.lib.bz_cm_batch_release(self.cm, bid)

    def table(self, bid):
        ind, ip, lpl = C.c_void_p(), C.c_void_p(), C.c_void_p()
        nnz, B = C.c_uint32(), C.c_uint32()
        assert self.lib.bz_cm_batch_table(self.cm, bid, C.byref(ind), C.byref(nnz), C.byref(ip), C.byref(lpl), C.byref(B)) == 0
        rd = lambda p, n: np.ctypeslib.as_array(C.cast(p, C.POINTER(C.c_int32)), shape=(max(n, 1),))[:n].copy()
        indices, indptr, last = rd(ind, nnz.value), rd(ip, B.value + 1), rd(lpl, B.value)
        # the blob order Stub::forward uploads in one copy: indices | indptr | last_page_len
        assert ip.value == ind.value + 4 * nnz.value and lpl.value == ip.value + 4 * (B.value + 1)
        return indices, indptr, last

    def stats(self):
        f, a, t = C.c_uint64(), C.c_uint64(), C.c_uint64()
        assert self.lib.bz_cm_stats(self.cm, C.byref(f), C.byref(a), C.byref(t)) == 0
        return f.value, a.value, t.value


class Model:
    """The same operations from the checker's primitives and plain list handling."""

    def __init__(self, P, max_pages):
        self.P, self.mask, self.batches = P, np.ones(max_pages, np.uint8), {}

    def prefill(self, lens):
        indptr, lpl = oracle.prefill_reservation(lens, self.P)
        pages = oracle.first_fit(self.mask, int(indptr[-1]))
        if pages is None:
            return None
        return [pages, indptr, lpl]

    def grow(self, t):
        r = oracle.table_grow(t[0], t[1], t[2], self.P, self.mask)
        if r is None:
            return False
        t[0], t[1], t[2] = r
        return True

    def split(self, t):
        return [list(t[0][t[1][i]:t[1][i + 1]]) for i in range(len(t[2]))]

    def join(self, lists, lpl):
        ind = np.array([p for l in lists for p in l], np.int32)
        ip = np.concatenate([[0], np.cumsum([len(l) for l in lists])]).astype(np.int32)
        return [ind, ip, np.asarray(lpl, np.int32)]

    def filter(self, t, keep):
        lists = self.split(t)
        for i, l in enumerate(lists):
            if i not in keep:
                self.mask[l] = 1
        return self.join([lists[i] for i in keep], [t[2][i] for i in keep])

    def extend(self, a, b):
        return self.join(self.split(a) + self.split(b), list(a[2]) + list(b[2]))

    def release(self, t):
        self.mask[t[0]] = 1


def same(prod_table, model_table):
    return all(np.array_equal(a, b) for a, b in zip(prod_table, model_table))


def check_invariants(table, P, max_pages):
    ind, ip, lpl = table
    assert len(ip) == len(lpl) + 1 and ip[0] == 0 and ip[-1] == len(ind)  # cache_manager.h:214-215
    assert (np.diff(ip) >= 1).all() and ((lpl >= 1) & (lpl <= P)).all()
    assert len(set(ind.tolist())) == len(ind) and (ind >= 0).all() and (ind < max_pages).all()


@pytest.mark.parametrize("P", [16, 64])
def test_random_operation_sequences_match_bit_for_bit(P):
    rng = np.random.default_rng(300 + P)
    max_pages = 400
    prod, model = Product(P, max_pages), Model(P, max_pages)
    live = {}  # product batch id -> model table
    for step in range(400):
        op = rng.choice(["prefill", "grow", "grow", "grow", "filter", "extend", "release"])
        if op == "prefill" or not live:
            lens = rng.integers(1, 6 * P, size=rng.integers(1, 6))
            rc, bid = prod.prefill(lens)
            t = model.prefill(lens)
            assert (rc == 0) == (t is not None)
            if rc:
                assert rc == BZ_ERR_NO_PAGES  # exhaustion surfaces as an error (cache_manager.h:174-182)
                continue
            live[bid] = t
        else:
            bid = int(rng.choice(list(live)))
            t = live[bid]
            if op == "grow":
                rc, ok = prod.grow(bid), model.grow(t)
                assert (rc == 0) == ok
            elif op == "filter" and len(t[2]) > 1:
                keep = sorted(rng.choice(len(t[2]), size=rng.integers(1, len(t[2])), replace=False).tolist())
                assert prod.filter(bid, keep) == 0
                live[bid] = model.filter(t, keep)
            elif op == "extend" and len(live) > 1:
                other = int(rng.choice([b for b in live if b != bid]))
                assert prod.extend(bid, other) == 0
                live[bid] = model.extend(t, live.pop(other))
            elif op == "release":
                assert prod.release(bid) == 0
                model.release(live.pop(bid))
        for b, t in live.items():
            got = prod.table(b)
            assert same(got, t), (step, op)
            check_invariants(got, P, max_pages)
        free, alloc, total = prod.stats()
        assert total == max_pages and free + alloc == total and free == int(model.mask.sum())
    prod.close()


def test_len_plus_one_reservation_and_lowest_ids():
    prod = Product(16, 64)
    rc, bid = prod.prefill([15, 16, 31])
    ind, ip, lpl = prod.table(bid)
    assert list(ip) == [0, 1, 3, 5] and list(lpl) == [16, 1, 16]  # len+1 slots (batch.h:246-250)
    assert list(ind) == [0, 1, 2, 3, 4]  # lowest free ids, request order (cache_manager.h:161-184)
    assert prod.grow(bid) == 0  # sequences 0 and 2 had full last pages
    ind, ip, lpl = prod.table(bid)
    assert list(ip) == [0, 2, 4, 7] and list(lpl) == [1, 2, 1] and list(ind) == [0, 5, 1, 2, 3, 4, 6]
    assert prod.filter(bid, [1]) == 0
    ind, ip, lpl = prod.table(bid)
    assert list(ind) == [1, 2] and list(ip) == [0, 2] and list(lpl) == [2]
    rc, b2 = prod.prefill([1])
    assert list(prod.table(b2)[0]) == [0]  # freed ids are reused lowest first
    prod.close()


def test_error_paths():
    prod = Product(16, 4)
    rc, bid = prod.prefill([100])  # needs 7 pages of 16
    assert rc == BZ_ERR_NO_PAGES and prod.stats()[0] == 4
    rc, bid = prod.prefill([47])  # 3 pages, last one full
    assert rc == 0
    assert prod.grow(bid) == 0 and prod.grow(999) == BZ_ERR_BAD_ARG
    assert prod.filter(bid, [3]) == BZ_ERR_BAD_ARG
    for _ in range(15):
        assert prod.grow(bid) == 0
    assert prod.grow(bid) == BZ_ERR_NO_PAGES  # pool exhausted: table unchanged
    assert list(prod.table(bid)[2]) == [16]
    prod.close()
