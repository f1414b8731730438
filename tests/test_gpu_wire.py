"""GPU parity of the KV migration wire format (bz_kv_pages_pack / bz_kv_pages_unpack through the C ABI)
against the CPU checker: byte-exact in every case, the e4m3 wire included (same fp32 divide, same
round-to-nearest-even)."""
import numpy as np
import pytest
import torch

import oracle
from blitz_scale_amd import kernel as K
from blitz_scale_amd import workloads as wl
from blitz_scale_amd._lib import BZ_BF16, BZ_E4M3, BZ_F16, BZ_LAYOUT_HND, BZ_LAYOUT_NHD, BzError

from _gpu import TORCH_OF, to_dev, to_host_bits

pytestmark = pytest.mark.gpu


def make(rng, layers, max_pages, Hkv, P, D, dtype, layout=BZ_LAYOUT_HND):
    sp = 2 * Hkv * P * D
    if dtype == BZ_E4M3:
        bits = rng.integers(0, 256, size=layers * max_pages * sp, dtype=np.uint8)
        bits[(bits & 0x7f) == 0x7f] = 0x3c
    else:
        bits = wl.randn_bits(rng, (layers * max_pages * sp,), dtype)
    pool = to_dev(bits, dtype)
    pt = K.PageTable(1, P, Hkv, D, pool, layout=layout)
    return bits, pool, pt, sp


def wire_tensor(nbytes, fill=0xA5):
    return torch.full((nbytes,), fill, dtype=torch.uint8, device="cuda")


@pytest.mark.parametrize("dtype,layout,Hkv,P,D", [
    (BZ_BF16, BZ_LAYOUT_HND, 8, 16, 128),  # Llama-3-8B page: 64 KiB per (page, layer)
    (BZ_F16, BZ_LAYOUT_NHD, 4, 16, 64),
    (BZ_E4M3, BZ_LAYOUT_HND, 8, 16, 128),
    (BZ_F16, BZ_LAYOUT_HND, 3, 4, 8),      # 192 elements per chunk: chunks smaller than a workgroup's share
])
def test_pack_and_unpack_are_byte_exact(dtype, layout, Hkv, P, D):
    rng = np.random.default_rng(21)
    layers, max_pages = 4, 37
    bits, pool, pt, sp = make(rng, layers, max_pages, Hkv, P, D, dtype, layout)
    ids = rng.permutation(max_pages)[:13].astype(np.int32)
    ids_d = torch.from_numpy(ids).cuda()
    for start, cnt in ((0, layers), (1, 2), (3, 1)):
        nbytes = K.kv_wire_bytes(pt, len(ids), cnt)
        want = oracle.kv_pages_pack(bits, dtype, max_pages, sp, ids, start, cnt)
        assert nbytes == want.nbytes
        wire = wire_tensor(nbytes + 64)
        K.pack_kv_pages(pt, max_pages, ids_d, start, cnt, wire)
        torch.cuda.synchronize()
        got = wire.cpu().numpy()
        assert np.array_equal(got[:nbytes], want.view(np.uint8)), (start, cnt)
        assert (got[nbytes:] == 0xA5).all()  # nothing past the payload
        # the receiving side: other page ids, a pool full of a sentinel
        dst_pages = 29
        dst_ids = rng.permutation(dst_pages)[:13].astype(np.int32)
        sent = 0x5a if dtype == BZ_E4M3 else 0x7bcd
        dst_bits = np.full(layers * dst_pages * sp, sent, bits.dtype)
        dst = to_dev(dst_bits, dtype)
        dpt = K.PageTable(1, P, Hkv, D, dst, layout=layout)
        K.unpack_kv_pages(dpt, dst_pages, torch.from_numpy(dst_ids).cuda(), start, cnt, wire)
        torch.cuda.synchronize()
        oracle.kv_pages_unpack(dst_bits, dtype, dst_pages, sp, dst_ids, start, cnt, want)
        assert np.array_equal(to_host_bits(dst), dst_bits), (start, cnt)


@pytest.mark.parametrize("dtype,layout", [(BZ_BF16, BZ_LAYOUT_HND), (BZ_F16, BZ_LAYOUT_NHD)])
def test_e4m3_wire(dtype, layout):
    rng = np.random.default_rng(22)
    layers, max_pages, Hkv, P, D = 3, 19, 8, 16, 128
    bits, pool, pt, sp = make(rng, layers, max_pages, Hkv, P, D, dtype, layout)
    _, _, stride_h = wl.strides(layout, Hkv, P, D)
    # per-(layer, head) scale amax/448 as the e4m3 pools use, plus one head scaled to saturate
    ks = rng.uniform(4.0, 5.0, (2, Hkv)).astype(np.float32) / np.float32(448)
    vs = rng.uniform(4.0, 5.0, (2, Hkv)).astype(np.float32) / np.float32(448)
    ks[1, 3] = np.float32(1.0 / 448)
    ids = rng.permutation(max_pages)[:7].astype(np.int32)
    kw = dict(wire_dtype=BZ_E4M3, num_kv_heads=Hkv, stride_h=stride_h, k_scale=ks, v_scale=vs)
    want = oracle.kv_pages_pack(bits, dtype, max_pages, sp, ids, 1, 2, **kw)
    nbytes = K.kv_wire_bytes(pt, len(ids), 2, BZ_E4M3)
    assert nbytes == want.nbytes == len(ids) * 2 * sp
    wire = wire_tensor(nbytes)
    ids_d, ks_d, vs_d = torch.from_numpy(ids).cuda(), torch.from_numpy(ks).cuda(), torch.from_numpy(vs).cuda()
    K.pack_kv_pages(pt, max_pages, ids_d, 1, 2, wire, wire_dtype=BZ_E4M3, k_scale=ks_d, v_scale=vs_d)
    torch.cuda.synchronize()
    assert np.array_equal(wire.cpu().numpy(), want)
    assert (want == 0x7e).any() or (want == 0xfe).any()  # the saturating head reached +-448
    dst_bits = np.zeros_like(bits)
    dst = to_dev(dst_bits, dtype)
    dpt = K.PageTable(1, P, Hkv, D, dst, layout=layout)
    K.unpack_kv_pages(dpt, max_pages, ids_d, 1, 2, wire, wire_dtype=BZ_E4M3, k_scale=ks_d, v_scale=vs_d)
    torch.cuda.synchronize()
    oracle.kv_pages_unpack(dst_bits, dtype, max_pages, sp, ids, 1, 2, want, **kw)
    assert np.array_equal(to_host_bits(dst), dst_bits)
    # without scales the wire is the plain conversion
    want1 = oracle.kv_pages_pack(bits, dtype, max_pages, sp, ids, 0, 1, wire_dtype=BZ_E4M3)
    K.pack_kv_pages(pt, max_pages, ids_d, 0, 1, wire, wire_dtype=BZ_E4M3)
    torch.cuda.synchronize()
    assert np.array_equal(wire.cpu().numpy()[:want1.size], want1)


def test_a_whole_prompt_batch_round_trips():
    """Llama-3-8B geometry, 8 layers of a 12-request batch: sender pool -> wire -> receiver pool at other
    page ids; the receiver's pages then pack to the identical stream (size-independent check: no host
    copy of the pools is compared)."""
    g = torch.Generator(device="cuda")
    g.manual_seed(5)
    layers, max_pages, Hkv, P, D = 8, 1024, 8, 16, 128
    sp = 2 * Hkv * P * D
    src = torch.randn(layers * max_pages * sp, dtype=torch.bfloat16, device="cuda", generator=g)
    dst = torch.zeros_like(src)
    rng = np.random.default_rng(23)
    lens = rng.integers(100, 2000, 12)
    n = int(((lens + P - 1) // P).sum())
    src_ids = torch.from_numpy(rng.permutation(max_pages)[:n].astype(np.int32)).cuda()
    dst_ids = torch.from_numpy(rng.permutation(max_pages)[:n].astype(np.int32)).cuda()
    spt = K.PageTable(12, P, Hkv, D, src)
    dpt = K.PageTable(12, P, Hkv, D, dst)
    nbytes = K.kv_wire_bytes(spt, n, layers)
    assert nbytes == n * layers * sp * 2
    wire = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    wire2 = torch.empty_like(wire)
    K.pack_kv_pages(spt, max_pages, src_ids, 0, layers, wire)
    K.unpack_kv_pages(dpt, max_pages, dst_ids, 0, layers, wire)
    K.pack_kv_pages(dpt, max_pages, dst_ids, 0, layers, wire2)
    torch.cuda.synchronize()
    assert torch.equal(wire, wire2)
    s3 = src.view(torch.int16).view(layers, max_pages, sp)
    d3 = dst.view(torch.int16).view(layers, max_pages, sp)
    assert torch.equal(s3[:, src_ids.long()], d3[:, dst_ids.long()])
    rest = torch.ones(max_pages, dtype=torch.bool, device="cuda")
    rest[dst_ids.long()] = False
    assert not d3[:, rest].any()


def test_empty_and_rejected_arguments():
    rng = np.random.default_rng(24)
    bits, pool, pt, sp = make(rng, 2, 4, 2, 4, 16, BZ_F16)
    wire = wire_tensor(256)
    ids_d = torch.zeros(0, dtype=torch.int32, device="cuda")
    K.pack_kv_pages(pt, 4, ids_d, 0, 2, wire)  # no pages: nothing launched
    K.pack_kv_pages(pt, 4, torch.zeros(1, dtype=torch.int32, device="cuda"), 0, 0, wire)  # no layers
    torch.cuda.synchronize()
    assert (wire.cpu().numpy() == 0xA5).all()
    # a page id that is not in the pool is not dereferenced; its chunk of the stream carries zeros
    bad = torch.tensor([1, 4, -1, 1 << 30, 2], dtype=torch.int32, device="cuda")
    sp = 2 * 2 * 4 * 16
    big = wire_tensor(5 * 2 * sp * 2)
    K.pack_kv_pages(pt, 4, bad, 0, 2, big)
    torch.cuda.synchronize()
    got = big.cpu().numpy().view(np.uint16).reshape(5, 2 * sp)
    pool3 = bits.reshape(2, 4, sp)
    for i, pg in enumerate([1, None, None, None, 2]):
        if pg is None:
            assert not got[i].any()
        else:
            assert np.array_equal(got[i], np.concatenate([pool3[0, pg], pool3[1, pg]]))
    with pytest.raises(BzError):  # a 16-bit wire for the other 16-bit type is not a format of this library
        K.pack_kv_pages(pt, 4, torch.zeros(1, dtype=torch.int32, device="cuda"), 0, 1, wire, wire_dtype=BZ_BF16)
    bits8, pool8, pt8, _ = make(rng, 2, 4, 2, 4, 16, BZ_E4M3)
    with pytest.raises(BzError):  # an e4m3 pool does not widen on the wire
        K.pack_kv_pages(pt8, 4, torch.zeros(1, dtype=torch.int32, device="cuda"), 0, 1, wire, wire_dtype=BZ_F16)
