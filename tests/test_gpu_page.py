"""GPU parity: KV page writes (prefill store, decode append, fused RoPE, e4m3 quantisation).
Placement and raw copies are bit-exact; rotated / quantised rows are compared value-wise because the
device's sincosf may differ from the host's in the last place (one storage step on rare elements; the rotation
itself rounds every product and sum on its own on both sides)."""
import numpy as np
import pytest
import torch

import oracle
from blitz_scale_amd import kernel as K
from blitz_scale_amd import workloads as wl
from blitz_scale_amd._lib import BZ_BF16, BZ_E4M3, BZ_F16, BZ_LAYOUT_HND, BZ_LAYOUT_NHD

from _gpu import DeviceDecode, to_dev, to_host_bits
from _util import DecodeProblem

pytestmark = pytest.mark.gpu
SENT = 0x7BFF


def _setup(seed, lens, Hq, Hkv, D, P, dtype, layout, kv_dtype=None, reserve_extra=1):
    p = DecodeProblem(seed, [l + reserve_extra for l in lens], Hq, Hkv, D, P, dtype, kv_dtype=kv_dtype, layout=layout)
    fill = SENT if p.kv_dtype != BZ_E4M3 else 0x55
    p.pool = np.full_like(p.pool, fill)
    return p, fill


@pytest.mark.parametrize("layout", [BZ_LAYOUT_NHD, BZ_LAYOUT_HND])
@pytest.mark.parametrize("dtype,D,P", [(BZ_F16, 128, 16), (BZ_BF16, 128, 64), (BZ_F16, 64, 8)])
def test_store_prefill_bit_exact(layout, dtype, D, P):
    rng = np.random.default_rng(50)
    lens, Hkv = [1, 15, 16, 17, 100, 333], 4
    p, fill = _setup(51, lens, 8, Hkv, D, P, dtype, layout)
    ri = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    k, v = wl.randn_bits(rng, (ri[-1], Hkv, D), dtype), wl.randn_bits(rng, (ri[-1], Hkv, D), dtype)
    want = p.pool.copy()
    oracle.store_prefill_kv(p.oracle_kv(want), k, v, dtype, ri)
    dev = DeviceDecode(p)
    K.store_prefill_kv_cache(dev.pt, to_dev(k, dtype), to_dev(v, dtype), to_dev(ri.view(np.float32), 3).view(torch.int32))
    torch.cuda.synchronize()
    got = to_host_bits(dev.pool)
    assert np.array_equal(got, want)
    assert (got != fill).sum() >= 2 * ri[-1] * Hkv * D - 64  # only the stored rows changed


@pytest.mark.parametrize("layout", [BZ_LAYOUT_NHD, BZ_LAYOUT_HND])
@pytest.mark.parametrize("dtype", [BZ_F16, BZ_BF16])
def test_append_decode_bit_exact(layout, dtype):
    rng = np.random.default_rng(52)
    ctx, Hkv, D, P = [1, 16, 17, 32, 33, 500, 0], 8, 128, 16
    p = DecodeProblem(53, ctx, 32, Hkv, D, P, dtype, layout=layout)
    p.pool = np.full_like(p.pool, SENT)
    k, v = wl.randn_bits(rng, (len(ctx), Hkv, D), dtype), wl.randn_bits(rng, (len(ctx), Hkv, D), dtype)
    want = p.pool.copy()
    oracle.append_decode_kv(p.oracle_kv(want), k, v, dtype)
    dev = DeviceDecode(p)
    K.append_decode_kv_cache(dev.pt, to_dev(k, dtype), to_dev(v, dtype))
    torch.cuda.synchronize()
    assert np.array_equal(to_host_bits(dev.pool), want)
    # position rule: page indices[indptr[b+1]-1], slot last_page_len[b]-1
    b = 4
    page, slot = int(p.indices[p.indptr[b + 1] - 1]), int(p.last_page_len[b]) - 1
    off = page * p.stride_page + slot * p.stride_n + 3 * p.stride_h
    assert np.array_equal(want[off:off + D], k[b, 3])


@pytest.mark.parametrize("theta", [1e4, 5e5])
def test_fused_rope_append(theta):
    """Decode path: q rotated in place and the new K rotated into the cache at position seq_len-1."""
    rng = np.random.default_rng(54)
    ctx, Hq, Hkv, D, P, dtype = [1, 40, 2048, 8191], 32, 8, 128, 16, BZ_BF16
    p = DecodeProblem(55, ctx, Hq, Hkv, D, P, dtype)
    k, v = wl.randn_bits(rng, (4, Hkv, D), dtype), wl.randn_bits(rng, (4, Hkv, D), dtype)
    want = p.pool.copy()
    kv = p.oracle_kv(want)
    oracle.append_decode_kv(kv, k, v, dtype, rope=True, rope_theta=theta)
    want_q = oracle.rope_decode_q(p.q, dtype, kv, Hq, theta)
    dev = DeviceDecode(p)
    K.append_decode_kv_cache(dev.pt, to_dev(k, dtype), to_dev(v, dtype), q=dev.q, num_qo_heads=Hq, rope=True,
                             rope_theta=theta)
    torch.cuda.synchronize()
    got, got_q = to_host_bits(dev.pool), to_host_bits(dev.q)
    for g, w in ((got, want), (got_q, want_q)):
        gf, wf = wl.to_f32(g, dtype), wl.to_f32(w, dtype)
        assert np.abs(gf - wf).max() <= 2.0 ** -6  # at most one bf16 step at |x| < 4
        assert (g != w).mean() < 2e-3
    # and the decode over the appended cache agrees with the checker
    dev.plan()
    out = dev.decode(3)
    ref = oracle.batch_decode(want_q, dtype, kv, Hq)
    assert np.abs(out - ref).max() < 2e-3


def test_fused_rope_store_prefill():
    rng = np.random.default_rng(56)
    lens, Hq, Hkv, D, P, dtype, theta = [3, 64, 130], 8, 4, 128, 16, BZ_F16, 1e4
    p, fill = _setup(57, lens, Hq, Hkv, D, P, dtype, BZ_LAYOUT_HND)
    ri = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    q = wl.randn_bits(rng, (ri[-1], Hq, D), dtype)
    k, v = wl.randn_bits(rng, (ri[-1], Hkv, D), dtype), wl.randn_bits(rng, (ri[-1], Hkv, D), dtype)
    want = p.pool.copy()
    oracle.store_prefill_kv(p.oracle_kv(want), k, v, dtype, ri, rope=True, rope_theta=theta)
    want_q = oracle.rope_ragged(q, dtype, ri, Hq, D, theta)
    want_k = oracle.rope_ragged(k, dtype, ri, Hkv, D, theta)
    dev = DeviceDecode(p)
    qd, kd = to_dev(q, dtype), to_dev(k, dtype)
    K.store_prefill_kv_cache(dev.pt, kd, to_dev(v, dtype), to_dev(ri.view(np.float32), 3).view(torch.int32),
                             q=qd, num_qo_heads=Hq, rope=True, rope_theta=theta)
    torch.cuda.synchronize()
    # pool, q rows and the caller's k rows all carry the rotation
    for g, w in ((to_host_bits(dev.pool), want), (to_host_bits(qd), want_q), (to_host_bits(kd), want_k)):
        assert np.abs(wl.to_f32(g, dtype) - wl.to_f32(w, dtype)).max() <= 2.0 ** -8
        assert (g != w).mean() < 2e-3


def test_append_quantises_to_e4m3():
    rng = np.random.default_rng(58)
    ctx, Hkv, D, P = [5, 16, 100], 8, 128, 16
    p = DecodeProblem(59, ctx, 64, Hkv, D, P, BZ_BF16, kv_dtype=BZ_E4M3)
    k, v = wl.randn_bits(rng, (3, Hkv, D), BZ_BF16), wl.randn_bits(rng, (3, Hkv, D), BZ_BF16)
    want = p.pool.copy()
    oracle.append_decode_kv(p.oracle_kv(want), k, v, BZ_BF16, k_scale=p.k_scale, v_scale=p.v_scale)
    dev = DeviceDecode(p)
    K.append_decode_kv_cache(dev.pt, to_dev(k, BZ_BF16), to_dev(v, BZ_BF16), k_scale=dev.k_scale, v_scale=dev.v_scale)
    torch.cuda.synchronize()
    assert np.array_equal(to_host_bits(dev.pool), want)  # x / scale and RNE-saturating e4m3: bit exact


@pytest.mark.parametrize("rope", [False, True])
def test_store_prefill_token_count_from_the_ragged_index(rope):
    """The reference's four-argument call does not pass a token count (src/kernel/page.h:66-67): the kernel
    reads ragged_indptr[batch] on the device and a fixed launch strides over the tokens.  Same pool bits as
    the launch with the count given, and as the checker; long enough that workgroups take several tokens."""
    from blitz_scale_amd._lib import BZ_NUM_TOKENS_FROM_INDPTR
    rng = np.random.default_rng(60)
    lens, Hkv, D, P, dtype = [1, 4000, 16, 5000, 333, 3000], 4, 128, 16, BZ_F16
    p, fill = _setup(61, lens, 8, Hkv, D, P, dtype, BZ_LAYOUT_HND)
    ri = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    assert ri[-1] > 8192
    k, v = wl.randn_bits(rng, (ri[-1], Hkv, D), dtype), wl.randn_bits(rng, (ri[-1], Hkv, D), dtype)
    want = p.pool.copy()
    oracle.store_prefill_kv(p.oracle_kv(want), k, v, dtype, ri, rope=rope, rope_theta=1e4)
    ri_d = to_dev(ri.view(np.float32), 3).view(torch.int32)
    pools = []
    for n in (int(ri[-1]), BZ_NUM_TOKENS_FROM_INDPTR):
        dev = DeviceDecode(p)
        kd = to_dev(k, dtype)
        K.store_prefill_kv_cache(dev.pt, kd, to_dev(v, dtype), ri_d, num_tokens=n, rope=rope, rope_theta=1e4)
        torch.cuda.synchronize()
        pools.append(to_host_bits(dev.pool))
        assert np.array_equal(to_host_bits(kd), k)  # without q the caller's k rows are left alone
    assert np.array_equal(pools[0], pools[1])
    if rope:  # rotated rows: the device's sincosf may differ from the host's in the last place
        assert np.abs(wl.to_f32(pools[1], dtype) - wl.to_f32(want, dtype)).max() <= 2.0 ** -8
        assert (pools[1] != want).mean() < 2e-3
    else:
        assert np.array_equal(pools[1], want)


def test_store_prefill_drops_tokens_beyond_the_listed_pages():
    """A ragged length longer than the pages of its table row (the reference asserts against it,
    src/kernel/page.cu:43): the tokens without a page are dropped and no other page is touched."""
    rng = np.random.default_rng(62)
    Hkv, D, P, dtype = 2, 128, 16, BZ_F16
    p, fill = _setup(63, [20, 40], 4, Hkv, D, P, dtype, BZ_LAYOUT_HND, reserve_extra=0)  # 2 and 3 pages
    lens_claimed = [20, 100]                                                              # request 1 claims 7 pages' worth
    ri = np.concatenate([[0], np.cumsum(lens_claimed)]).astype(np.int32)
    k, v = wl.randn_bits(rng, (ri[-1], Hkv, D), dtype), wl.randn_bits(rng, (ri[-1], Hkv, D), dtype)
    want = p.pool.copy()
    ri_fit = np.array([0, 20, 20 + 48], np.int32)  # what fits: 3 pages x 16 slots of request 1
    k_fit = np.concatenate([k[:20], k[20:68]])
    v_fit = np.concatenate([v[:20], v[20:68]])
    oracle.store_prefill_kv(p.oracle_kv(want), k_fit, v_fit, dtype, ri_fit)
    dev = DeviceDecode(p)
    K.store_prefill_kv_cache(dev.pt, to_dev(k, dtype), to_dev(v, dtype), to_dev(ri.view(np.float32), 3).view(torch.int32))
    torch.cuda.synchronize()
    assert np.array_equal(to_host_bits(dev.pool), want)


@pytest.mark.parametrize("with_q", [False, True])
def test_store_prefill_rotates_in_place_also_what_it_cannot_cache(with_q):
    """Tokens beyond the listed pages are not cached, but a store that rotates in place (rope = 2, or the fused
    form with q) still rotates their rows: the attention call that follows must see the whole request rotated."""
    rng = np.random.default_rng(66)
    Hq, Hkv, D, P, dtype, theta = 4, 2, 128, 16, BZ_F16, 1e4
    p, fill = _setup(67, [20, 40], Hq, Hkv, D, P, dtype, BZ_LAYOUT_HND, reserve_extra=0)  # 2 and 3 pages
    ri = np.array([0, 20, 120], np.int32)                                                 # request 1 claims 100 tokens
    q = wl.randn_bits(rng, (120, Hq, D), dtype)
    k, v = wl.randn_bits(rng, (120, Hkv, D), dtype), wl.randn_bits(rng, (120, Hkv, D), dtype)
    want = p.pool.copy()
    ri_fit = np.array([0, 20, 68], np.int32)  # what fits: 3 pages x 16 slots of request 1
    oracle.store_prefill_kv(p.oracle_kv(want), k[:68], v[:68], dtype, ri_fit, rope=True, rope_theta=theta)
    want_k = oracle.rope_ragged(k, dtype, ri, Hkv, D, theta)
    want_q = oracle.rope_ragged(q, dtype, ri, Hq, D, theta)
    dev = DeviceDecode(p)
    qd, kd, vd = to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype)
    rid = to_dev(ri.view(np.float32), 3).view(torch.int32)
    if with_q:
        K.store_prefill_kv_cache(dev.pt, kd, vd, rid, q=qd, num_qo_heads=Hq, rope=True, rope_theta=theta)
    else:
        K.store_prefill_kv_cache(dev.pt, kd, vd, rid, rope=2, rope_theta=theta)
    torch.cuda.synchronize()
    pairs = [(to_host_bits(dev.pool), want), (to_host_bits(kd), want_k)] + ([(to_host_bits(qd), want_q)] if with_q else [])
    for g, w in pairs:
        assert np.abs(wl.to_f32(g, dtype) - wl.to_f32(w, dtype)).max() <= 2.0 ** -8
        assert (g != w).mean() < 2e-3
    if not with_q:
        assert np.array_equal(to_host_bits(qd), q)
    assert np.array_equal(to_host_bits(vd), v)


def test_store_prefill_rotates_k_in_place_without_q():
    """rope = 2: K is rotated into the pages AND in the caller's rows (q is left to the attention call, which
    rotates it in registers); same bits in both places."""
    rng = np.random.default_rng(64)
    lens, Hkv, D, P, dtype, theta = [3, 64, 130], 4, 128, 16, BZ_F16, 1e4
    p, fill = _setup(65, lens, 8, Hkv, D, P, dtype, BZ_LAYOUT_HND)
    ri = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    k, v = wl.randn_bits(rng, (ri[-1], Hkv, D), dtype), wl.randn_bits(rng, (ri[-1], Hkv, D), dtype)
    want = p.pool.copy()
    oracle.store_prefill_kv(p.oracle_kv(want), k, v, dtype, ri, rope=True, rope_theta=theta)
    want_k = oracle.rope_ragged(k, dtype, ri, Hkv, D, theta)
    dev = DeviceDecode(p)
    kd, vd = to_dev(k, dtype), to_dev(v, dtype)
    K.store_prefill_kv_cache(dev.pt, kd, vd, to_dev(ri.view(np.float32), 3).view(torch.int32), rope=2, rope_theta=theta)
    torch.cuda.synchronize()
    got_pool, got_k = to_host_bits(dev.pool), to_host_bits(kd)
    for g, w in ((got_pool, want), (got_k, want_k)):
        assert np.abs(wl.to_f32(g, dtype) - wl.to_f32(w, dtype)).max() <= 2.0 ** -8
        assert (g != w).mean() < 2e-3
    assert np.array_equal(to_host_bits(vd), v)
    # the caller's rows and the cached rows are the same bits
    kv = p.oracle_kv(got_pool)
    K0, _ = DecodeProblem.gather_kv.__get__(type("X", (), dict(ctx=np.array(lens), pool=got_pool, kv_dtype=dtype, P=P, Hkv=Hkv, D=D,
                                                               indices=p.indices, indptr=p.indptr, stride_page=p.stride_page,
                                                               stride_n=p.stride_n, stride_h=p.stride_h))())(2)
    assert np.array_equal(K0, wl.to_f32(got_k, dtype).reshape(-1, Hkv, D)[ri[2]:ri[3]])


@pytest.mark.parametrize("dtype,D,P,layout", [(BZ_F16, 128, 16, BZ_LAYOUT_HND), (BZ_BF16, 128, 64, BZ_LAYOUT_NHD),
                                              (BZ_F16, 64, 8, BZ_LAYOUT_HND)])
def test_raw_k_cache_converted_once_then_served_by_the_fast_decode_path(dtype, D, P, layout):
    """A cache that holds K as the projection left it (the reference's convention: kRoPELlama inside every decode
    call, src/kernel/attention_decode.cu:35) is rotated in place once; decode with BZ_ROPE_Q_ONLY over it then gives
    the checker's kRoPELlama result on the raw cache.  V, the unused slots and the pages of no sequence are not
    touched; the inverse pass restores the raw rows to within one rounding."""
    from blitz_scale_amd._lib import BZ_F32, BZ_ROPE_FULL, BZ_ROPE_Q_ONLY
    theta = 5e5
    p = DecodeProblem(70, [1, 17, 300, 0, 2049, 64, 1000], 8, 2, D, P, dtype, layout=layout)
    ref = oracle.batch_decode(p.q, p.dtype, p.oracle_kv(), p.Hq, rope_mode=oracle.ROPE_FULL, rope_theta=theta, parallel=True)
    dev = DeviceDecode(p)
    dev.plan(1024)
    K.rope_cached_k(dev.pt, rope_theta=theta)
    torch.cuda.synchronize()
    pool_rot = to_host_bits(dev.pool)
    # the checker's rotation of the same rows: gather every sequence's K, rotate, compare where the pool changed
    want = p.pool.copy()
    k_rows = np.zeros(p.pool.size, bool)  # the elements of cached K rows: everything else must stay as it is
    for b in range(p.B):
        n = int(p.ctx[b])
        if n == 0:
            continue
        Kb, _ = p.gather_kv(b)  # fp32 [n, Hkv, D]
        rot = oracle.rope_ragged(wl.to_bits(Kb, dtype), dtype, np.array([0, n], np.int32), p.Hkv, D, theta)
        for t in range(n):
            page = int(p.indices[p.indptr[b] + t // P])
            for h in range(p.Hkv):
                off = page * p.stride_page + (t % P) * p.stride_n + h * p.stride_h
                want[off:off + D] = rot[t, h]
                k_rows[off:off + D] = True
    assert np.abs(wl.to_f32(pool_rot, dtype) - wl.to_f32(want, dtype)).max() <= (2.0 ** -8 if dtype == BZ_F16 else 2.0 ** -5)
    assert (pool_rot != want).mean() < 2e-3
    assert np.array_equal(pool_rot[~k_rows], p.pool[~k_rows])  # V halves, unused slots, pages of no sequence
    got = dev.decode(BZ_F32, BZ_ROPE_Q_ONLY, theta)
    assert np.abs(got - ref).max() <= 2e-3, float(np.abs(got - ref).max())
    K.rope_cached_k(dev.pt, rope_theta=theta, inverse=True)
    torch.cuda.synchronize()
    back = to_host_bits(dev.pool)
    step = np.maximum(np.abs(wl.to_f32(p.pool, dtype)), 1.0) * (2.0 ** -9 if dtype == BZ_F16 else 2.0 ** -6)
    assert (np.abs(wl.to_f32(back, dtype) - wl.to_f32(p.pool, dtype)) <= step).all()
    assert np.array_equal(back[~k_rows], p.pool[~k_rows])
