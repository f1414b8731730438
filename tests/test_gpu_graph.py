"""A decode step (fused RoPE + KV append, paged attention with split-K, combine) recorded into a HIP
graph and replayed: the launch path makes no allocation, copy, memset or synchronisation of its own,
so a caller can capture it once per batch shape and replay it per layer and per step.

The replays run with new q / k / v contents each time, with eager work and synchronisations between
them, and every replay is compared bit for bit with the same step launched eagerly (same kernels, same
plan, deterministic reduction order).  The step is also checked once against the CPU checker.
"""
import numpy as np
import pytest
import torch

import oracle
from blitz_scale_amd import kernel as K
from blitz_scale_amd import workloads as wl
from blitz_scale_amd._lib import BZ_BF16, BZ_F16, BZ_ROPE_NONE

from _gpu import TORCH_OF, DeviceDecode, to_dev, to_host_bits
from _util import DecodeProblem, ulp_tol

pytestmark = pytest.mark.gpu


def _step(dev, q, k, v, out, stream):
    """One layer's attention step the way src/layer/attn.h:188-204 sequences it: append, then decode."""
    p = dev.p
    K.append_decode_kv_cache(dev.pt, k, v, q=q, num_qo_heads=p.Hq, rope=True, rope_theta=5e5, stream=stream)
    K.batch_decode_attention(dev.handler, q, dev.pt, out, p.Hq, rope_mode=BZ_ROPE_NONE, stream=stream)


@pytest.mark.parametrize("dtype,Hq,Hkv,ctx", [
    (BZ_BF16, 32, 8, [70, 4100, 16, 1500, 2049, 333, 9, 2600]),  # MFMA kernel, two sequences split over K
    (BZ_F16, 4, 4, [17, 64, 130, 255]),                           # general kernel (D = 64 below)
])
def test_decode_step_replays_from_a_hip_graph(dtype, Hq, Hkv, ctx):
    D = 128 if Hq == 32 else 64
    p = DecodeProblem(0xC0FFEE, ctx, Hq, Hkv, D, 16, dtype)
    dev = DeviceDecode(p)
    info = dev.plan(split_tokens=2048 if Hq == 32 else 0)
    tdt = TORCH_OF[dtype]
    pool0 = dev.pool.clone()
    side = torch.cuda.Stream()
    qs = torch.empty((p.B, Hq, D), dtype=tdt, device="cuda")
    ks = torch.empty((p.B, Hkv, D), dtype=tdt, device="cuda")
    vs = torch.empty((p.B, Hkv, D), dtype=tdt, device="cuda")
    outs = torch.empty((p.B, Hq, D), dtype=tdt, device="cuda")

    def fresh(seed):
        rng = np.random.default_rng(seed)
        return [wl.randn_bits(rng, shape, dtype) for shape in ((p.B, Hq, D), (p.B, Hkv, D), (p.B, Hkv, D))]

    def load(bits):
        for dst, b in zip((qs, ks, vs), bits):
            dst.copy_(to_dev(b, dtype))

    # warm-up on the capture stream (one-time kernel attribute calls happen here, outside the capture)
    load(fresh(1))
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        _step(dev, qs, ks, vs, outs, side.cuda_stream)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    load(fresh(1))
    torch.cuda.synchronize()
    with torch.cuda.graph(graph, stream=side):
        _step(dev, qs, ks, vs, outs, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()

    for r in range(4):
        bits = fresh(100 + r)
        # eager run of the same step on a copy of the pool
        dev.pool.copy_(pool0)
        load(bits)
        out_e = torch.full_like(outs, float("nan"))
        torch.cuda.synchronize()
        _step(dev, qs, ks, vs, out_e, None)
        torch.cuda.synchronize()
        pool_e = dev.pool.clone()
        q_e = qs.clone()
        # replay on the same inputs
        dev.pool.copy_(pool0)
        load(bits)
        outs.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(outs.view(torch.int16), out_e.view(torch.int16)), f"replay {r}: output differs"
        assert torch.equal(dev.pool.view(torch.int16), pool_e.view(torch.int16)), f"replay {r}: pool differs"
        assert torch.equal(qs.view(torch.int16), q_e.view(torch.int16)), f"replay {r}: rotated q differs"
        # some unrelated eager work between the replays
        (torch.randn(1 << 16, device="cuda") * 2).sum().item()

    # the last replay against the CPU checker: the appended rows (rotations may differ by one storage step
    # in rare places, as in the eager append test), then attention over the replay's own pool and q
    q_bits, k_bits, v_bits = bits
    pool_ref = to_host_bits(pool0).copy()
    oracle.append_decode_kv(p.oracle_kv(pool_ref), k_bits, v_bits, dtype, rope=True, rope_theta=5e5)
    pool_got = to_host_bits(dev.pool)
    assert np.abs(wl.to_f32(pool_got, dtype) - wl.to_f32(pool_ref, dtype)).max() <= 2.0 ** -6
    assert (pool_got != pool_ref).mean() < 2e-3
    assert (pool_got != to_host_bits(pool0)).sum() > 0
    ref = oracle.batch_decode(to_host_bits(qs), dtype, p.oracle_kv(pool_got), Hq, rope_mode=BZ_ROPE_NONE)
    got = outs.float().cpu().numpy()
    assert (np.abs(got - ref) <= ulp_tol(ref, dtype, 2e-3)).all(), f"max abs err {np.abs(got - ref).max()}"
    if Hq == 32:
        assert info["split_seqs"] >= 2
