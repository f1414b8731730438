"""Many decode steps from ONE page-table upload and ONE plan: the table is grown H steps ahead on the
host, a device counter says how many steps the present lags behind it, and append + decode work at the
present length.  Every step is compared with the CPU checker run on a table truncated to that step's
lengths (the checker knows nothing of the counter), the pool is checked after every append (the new rows
where they belong, every other element untouched, the random contents of the slots still to come
included), and the same sequence of steps is also replayed from one HIP graph.

Tolerances as in the per-kernel tests: attention max-abs <= 2e-3 (+ bf16 storage step), rotated rows
within one storage step of the checker's, placement bit-exact."""
import numpy as np
import pytest
import torch

import oracle
from blitz_scale_amd import kernel as K
from blitz_scale_amd import workloads as wl
from blitz_scale_amd._lib import BZ_BF16, BZ_E4M3, BZ_F16, BZ_LAYOUT_HND, BZ_LAYOUT_NHD, BZ_ROPE_NONE

from _gpu import TORCH_OF, DeviceDecode, to_dev, to_host_bits
from _util import DecodeProblem, ulp_tol

pytestmark = pytest.mark.gpu

THETA = 5e5


def truncated_kv(p, pool, lens):
    """The checker's view of the pool with every sequence cut to lens[b] tokens (first pages of its list)."""
    ind, ptr, last = [], [0], []
    for b in range(p.B):
        n = (int(lens[b]) + p.P - 1) // p.P
        ind.extend(p.indices[p.indptr[b]:p.indptr[b] + n])
        ptr.append(len(ind))
        last.append(int(lens[b]) - (n - 1) * p.P if n else 0)
    half = p.stride_page // 2
    return oracle.PagedKV(pool, pool[half:], np.asarray(ind, np.int32), np.asarray(ptr, np.int32),
                          np.asarray(last, np.int32), p.P, p.Hkv, p.D, p.stride_page, p.stride_n, p.stride_h,
                          p.kv_dtype)


def row_elements(p, b, pos):
    """Pool element indices of token `pos` of sequence b, K and V, all heads."""
    page = int(p.indices[p.indptr[b] + pos // p.P])
    base = page * p.stride_page + (pos % p.P) * p.stride_n
    idx = (base + np.arange(p.Hkv)[:, None] * p.stride_h + np.arange(p.D)[None, :]).reshape(-1)
    return np.concatenate([idx, idx + p.stride_page // 2])


@pytest.mark.parametrize("use_graph", [False, True])
@pytest.mark.parametrize("dtype,kv_dtype,Hq,Hkv,D,P,layout,ctx0,split", [
    # MFMA kernel: a sequence split over K, lengths that cross 32-token tiles and pages during the run
    (BZ_BF16, None, 32, 8, 128, 16, BZ_LAYOUT_HND, [5, 31, 0, 100, 2040, 17, 63, 1000], 2048),
    # MFMA kernel over an e4m3 pool in the reference's in-page order
    (BZ_F16, BZ_E4M3, 16, 4, 128, 32, BZ_LAYOUT_NHD, [1, 40, 90, 700], 256),
    # general kernel (head_dim 64), split
    (BZ_F16, None, 4, 4, 64, 8, BZ_LAYOUT_HND, [0, 7, 64, 130, 255], 64),
])
def test_decode_steps_from_one_plan(dtype, kv_dtype, Hq, Hkv, D, P, layout, ctx0, split, use_graph):
    H = 37
    ctx0 = np.asarray(ctx0)
    p = DecodeProblem(0xA4EAD, ctx0 + H, Hq, Hkv, D, P, dtype, kv_dtype=kv_dtype, layout=layout)
    kvd = p.kv_dtype
    dev = DeviceDecode(p)
    dev.plan(split_tokens=split)  # one plan, from the table as it will be after H steps
    ahead = torch.tensor([H - 1], dtype=torch.int32, device="cuda")
    dev.pt.steps_ahead_d = ahead
    tdt = TORCH_OF[dtype]
    qs = torch.empty((p.B, Hq, D), dtype=tdt, device="cuda")
    ks = torch.empty((p.B, Hkv, D), dtype=tdt, device="cuda")
    vs = torch.empty((p.B, Hkv, D), dtype=tdt, device="cuda")
    outs = torch.empty((p.B, Hq, D), dtype=tdt, device="cuda")

    def step(stream):
        K.append_decode_kv_cache(dev.pt, ks, vs, q=qs, num_qo_heads=Hq, rope=True, rope_theta=THETA,
                                 k_scale=dev.k_scale, v_scale=dev.v_scale, stream=stream)
        K.batch_decode_attention(dev.handler, qs, dev.pt, outs, Hq, rope_mode=BZ_ROPE_NONE, k_scale=dev.k_scale,
                                 v_scale=dev.v_scale, stream=stream)
        K.steps_ahead_advance(ahead, stream=stream)

    graph = None
    if use_graph:
        side = torch.cuda.Stream()
        pool0, a0 = dev.pool.clone(), ahead.clone()
        for t in (qs, ks, vs):
            t.zero_()
        torch.cuda.synchronize()
        with torch.cuda.stream(side):
            step(side.cuda_stream)  # warm-up: one-time attribute calls stay outside the capture
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            step(torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        dev.pool.copy_(pool0)
        ahead.copy_(a0)

    rng = np.random.default_rng(77)
    pool_ref = p.pool.copy()
    step_tol = 2.0 ** -6 if kvd != BZ_E4M3 else None
    for i in range(H):
        lens = ctx0 + 1 + i
        q_bits = wl.randn_bits(rng, (p.B, Hq, D), dtype)
        k_bits = wl.randn_bits(rng, (p.B, Hkv, D), dtype)
        v_bits = wl.randn_bits(rng, (p.B, Hkv, D), dtype)
        qs.copy_(to_dev(q_bits, dtype)); ks.copy_(to_dev(k_bits, dtype)); vs.copy_(to_dev(v_bits, dtype))
        outs.fill_(float("nan"))
        torch.cuda.synchronize()
        if graph is not None:
            graph.replay()
        else:
            step(None)
        torch.cuda.synchronize()
        assert int(ahead.item()) == max(H - 2 - i, 0)

        # the pool: this step's rows changed, nothing else did
        pool_before = pool_ref.copy()
        oracle.append_decode_kv(truncated_kv(p, pool_ref, lens), k_bits, v_bits, dtype, rope=True, rope_theta=THETA,
                                k_scale=p.k_scale, v_scale=p.v_scale)
        pool_got = to_host_bits(dev.pool)
        touched = np.concatenate([row_elements(p, b, int(lens[b]) - 1) for b in range(p.B)])
        mask = np.ones(pool_got.size, bool)
        mask[touched] = False
        assert np.array_equal(pool_got[mask], pool_before[mask]), f"step {i}: elements outside the new rows changed"
        assert (pool_ref[touched] != pool_before[touched]).any()
        if kvd == BZ_E4M3:
            assert (pool_got[touched] != pool_ref[touched]).mean() < 5e-3, f"step {i}"
        else:
            diff = np.abs(wl.to_f32(pool_got[touched], kvd) - wl.to_f32(pool_ref[touched], kvd))
            assert diff.max() <= step_tol and (pool_got[touched] != pool_ref[touched]).mean() < 2e-3, f"step {i}"
        pool_ref = pool_got.copy()  # later steps are judged on what the device actually holds

        # attention over the present lengths, with the q the device rotated
        ref = oracle.batch_decode(to_host_bits(qs), dtype, truncated_kv(p, pool_ref, lens), Hq, rope_mode=BZ_ROPE_NONE,
                                  k_scale=p.k_scale, v_scale=p.v_scale)
        got = outs.float().cpu().numpy()
        base = 3e-2 if kvd == BZ_E4M3 else 2e-3
        assert not np.isnan(got).any(), f"step {i}"
        err = np.abs(got - ref)
        assert (err <= ulp_tol(ref, dtype, base)).all(), f"step {i}: max abs err {err.max()}"

    # past the horizon the counter stays at zero and the table is the present
    assert int(ahead.item()) == 0


@pytest.mark.parametrize("Hq,Hkv,D", [(32, 8, 128), (4, 4, 64)])
def test_counter_larger_than_a_sequence(Hq, Hkv, D):
    """A counter that leaves a sequence without tokens: the append skips it, its output row is zero, the
    other sequences are unaffected (MFMA kernel and general kernel)."""
    dtype, P = BZ_F16, 16
    ctx = np.asarray([3, 40, 5, 200])
    ahead_n = 5
    p = DecodeProblem(0xB0B, ctx, Hq, Hkv, D, P, dtype)
    dev = DeviceDecode(p)
    dev.plan(split_tokens=64)
    dev.pt.steps_ahead_d = torch.tensor([ahead_n], dtype=torch.int32, device="cuda")
    lens = np.maximum(ctx - ahead_n, 0)  # [0, 35, 0, 195]
    rng = np.random.default_rng(5)
    k_bits, v_bits = wl.randn_bits(rng, (p.B, Hkv, D), dtype), wl.randn_bits(rng, (p.B, Hkv, D), dtype)
    K.append_decode_kv_cache(dev.pt, to_dev(k_bits, dtype), to_dev(v_bits, dtype))
    torch.cuda.synchronize()
    want = p.pool.copy()
    live = [b for b in range(p.B) if lens[b] > 0]
    for b in live:  # raw copy: bit-exact
        idx = row_elements(p, b, int(lens[b]) - 1)
        half = idx.size // 2
        want[idx[:half]] = k_bits[b].reshape(-1)
        want[idx[half:]] = v_bits[b].reshape(-1)
    pool_got = to_host_bits(dev.pool)
    assert np.array_equal(pool_got, want)
    got = dev.decode(None, BZ_ROPE_NONE)
    ref = oracle.batch_decode(p.q, dtype, truncated_kv(p, pool_got, lens), Hq, rope_mode=BZ_ROPE_NONE)
    assert not got[lens == 0].any()
    assert (np.abs(got[lens > 0] - ref[lens > 0]) <= 2e-3).all()
