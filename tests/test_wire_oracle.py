"""The CPU checker's KV migration wire format against independent statements of the same thing.

What fixes the format (src/blitz/migration_manager.h:86-92, 455-467): the pool is
[layer][page][stride_page elements]; the sender walks requests, their prompt blocks and the layers,
and sends the stride_page elements at get_page_ptr(block, layer) as one message each; the receiver
walks its own block ids in the same order.  The checks below state that with array indexing instead
of the checker's address arithmetic, with a literal message loop over a batch's 2-D block lists, and
through round trips; the e4m3 wire is held to the numpy encoder of the workloads module, which shares
no code with the checker's C converter.
"""
import numpy as np
import pytest

import oracle
from blitz_scale_amd import workloads as wl
from blitz_scale_amd._lib import BZ_BF16, BZ_E4M3, BZ_F16, BZ_LAYOUT_HND, BZ_LAYOUT_NHD


def make_pool(rng, layers, max_pages, Hkv, P, D, dtype):
    stride_page = 2 * Hkv * P * D
    if dtype == BZ_E4M3:
        bits = rng.integers(0, 256, size=layers * max_pages * stride_page, dtype=np.uint8)
        bits[(bits & 0x7f) == 0x7f] = 0x3c  # no NaN codes
        return bits, stride_page
    return wl.randn_bits(rng, (layers * max_pages * stride_page,), dtype), stride_page


@pytest.mark.parametrize("dtype", [BZ_F16, BZ_BF16, BZ_E4M3])
def test_pack_is_the_indexed_gather(dtype):
    rng = np.random.default_rng(7)
    layers, max_pages, Hkv, P, D = 5, 23, 2, 4, 16
    pool, sp = make_pool(rng, layers, max_pages, Hkv, P, D, dtype)
    ids = rng.permutation(max_pages)[:9]
    wire = oracle.kv_pages_pack(pool, dtype, max_pages, sp, ids, 1, 3)
    want = pool.reshape(layers, max_pages, sp)[1:4][:, ids].transpose(1, 0, 2).reshape(-1)
    assert np.array_equal(wire, want)
    assert wire.dtype == pool.dtype and wire.size == 9 * 3 * sp


def test_pack_is_the_reference_message_stream():
    """A literal walk of the sender: requests, prompt blocks (a request may own one block more than its
    prompt needs: the slot reserved for the first generated token), layers."""
    rng = np.random.default_rng(8)
    layers, max_pages, Hkv, P, D = 4, 40, 2, 8, 8
    pool, sp = make_pool(rng, layers, max_pages, Hkv, P, D, BZ_F16)
    perm = [int(x) for x in rng.permutation(max_pages)]
    indices_2d = [perm[0:3], perm[3:4], perm[4:9]]
    num_prompt_blocks = [3, 1, 4]  # the last request's fifth block is not a prompt block
    messages = []
    for blocks, need in zip(indices_2d, num_prompt_blocks):
        assert len(blocks) in (need, need + 1)
        for i in range(need):
            for layer in range(0, layers):
                base = layer * max_pages * sp + blocks[i] * sp
                messages.append(pool[base:base + sp])
    ids = [b for blocks, need in zip(indices_2d, num_prompt_blocks) for b in blocks[:need]]
    wire = oracle.kv_pages_pack(pool, BZ_F16, max_pages, sp, ids, 0, layers)
    assert np.array_equal(wire, np.concatenate(messages))


@pytest.mark.parametrize("dtype", [BZ_F16, BZ_E4M3])
def test_round_trip_into_other_pages(dtype):
    rng = np.random.default_rng(9)
    layers, max_pages, Hkv, P, D = 3, 17, 2, 4, 16
    src, sp = make_pool(rng, layers, max_pages, Hkv, P, D, dtype)
    src_ids = rng.permutation(max_pages)[:6]
    wire = oracle.kv_pages_pack(src, dtype, max_pages, sp, src_ids, 0, layers)
    dst_pages = 11
    sentinel = 0x5a if dtype == BZ_E4M3 else 0x7bcd
    dst = np.full(layers * dst_pages * sp, sentinel, src.dtype)
    dst_ids = rng.permutation(dst_pages)[:6]
    oracle.kv_pages_unpack(dst, dtype, dst_pages, sp, dst_ids, 0, layers, wire)
    s3, d3 = src.reshape(layers, max_pages, sp), dst.reshape(layers, dst_pages, sp)
    for a, b in zip(src_ids, dst_ids):
        assert np.array_equal(s3[:, a], d3[:, b])
    untouched = np.setdiff1d(np.arange(dst_pages), dst_ids)
    assert (d3[:, untouched] == sentinel).all()
    # and the receiver's pages pack to the same stream
    assert np.array_equal(oracle.kv_pages_pack(dst, dtype, dst_pages, sp, dst_ids, 0, layers), wire)


@pytest.mark.parametrize("layout", [BZ_LAYOUT_HND, BZ_LAYOUT_NHD])
@pytest.mark.parametrize("dtype", [BZ_F16, BZ_BF16])
def test_e4m3_wire_scales_by_layer_and_head(dtype, layout):
    rng = np.random.default_rng(10)
    layers, max_pages, Hkv, P, D = 3, 9, 4, 4, 8
    pool, sp = make_pool(rng, layers, max_pages, Hkv, P, D, dtype)
    _, _, stride_h = wl.strides(layout, Hkv, P, D)
    ks = rng.uniform(0.004, 0.02, (2, Hkv)).astype(np.float32)
    vs = rng.uniform(0.004, 0.02, (2, Hkv)).astype(np.float32)
    ids = [5, 0, 7]
    wire = oracle.kv_pages_pack(pool, dtype, max_pages, sp, ids, 1, 2, wire_dtype=BZ_E4M3, num_kv_heads=Hkv,
                                stride_h=stride_h, k_scale=ks, v_scale=vs)
    assert wire.dtype == np.uint8 and wire.size == 3 * 2 * sp
    # independent statement: view a page as [K|V][...] in its layout and divide by the head's scale
    x = wl.to_f32(pool, dtype).reshape(layers, max_pages, 2, *((Hkv, P, D) if layout == BZ_LAYOUT_HND else (P, Hkv, D)))
    sc = np.stack([ks, vs], axis=1)  # [layer][K|V][head]
    sc = sc[:, :, :, None, None] if layout == BZ_LAYOUT_HND else sc[:, :, None, :, None]
    want = []
    for page in ids:
        for l in range(2):
            want.append(wl.f32_to_e4m3_bits((x[1 + l, page] / sc[l]).astype(np.float32)).reshape(-1))
    assert np.array_equal(wire, np.concatenate(want))
    # the way back multiplies by the same scale and rounds to the pool's type
    dst = np.zeros_like(pool)
    oracle.kv_pages_unpack(dst, dtype, max_pages, sp, ids, 1, 2, wire, wire_dtype=BZ_E4M3, num_kv_heads=Hkv,
                           stride_h=stride_h, k_scale=ks, v_scale=vs)
    back = wl.to_f32(dst, dtype).reshape(x.shape)
    for i, page in enumerate(ids):
        for l in range(2):
            w = wl.to_f32(want[2 * i + l], BZ_E4M3).reshape(x.shape[2:])
            assert np.array_equal(back[1 + l, page], wl.to_f32(wl.to_bits((w * sc[l]).astype(np.float32), dtype), dtype))
            # quantisation error of e4m3 at these scales: 2^-4 relative, plus the saturation bound
            ref = np.clip(x[1 + l, page], -448 * sc[l], 448 * sc[l])
            assert np.abs(back[1 + l, page] - ref).max() <= np.abs(ref).max() * 2.0 ** -4 + 1e-3
    assert not dst.reshape(layers, max_pages, sp)[0].any()


def test_empty_inputs():
    pool = np.zeros(64, np.uint16)
    assert oracle.kv_pages_pack(pool, BZ_F16, 2, 32, [], 0, 1).size == 0
    assert oracle.kv_pages_pack(pool, BZ_F16, 2, 32, [1], 0, 0).size == 0
