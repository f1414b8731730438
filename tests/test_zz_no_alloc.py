"""GPU: the decode entry point that allocates nothing (bz_batch_decode_noalloc) against bz_batch_decode.

Both run the same kernels on the same plan; the only difference is where the split-K partial results
live (the library's fixed device array instead of the plan's float workspace), so the outputs must be
bit-identical, and both are held to the checker's bar.  Two calls in a row share the array: the second
works on a smaller batch and must not be disturbed by what the first left behind.
"""
import os

import numpy as np
import pytest
import torch

import oracle
from blitz_scale_amd import kernel as K
from blitz_scale_amd import _lib
from blitz_scale_amd._lib import BZ_BF16, BZ_E4M3, BZ_F16, BZ_F32, BZ_ROPE_NONE, BZ_ROPE_Q_ONLY

from _gpu import TORCH_OF, DeviceDecode, to_host_f32
from _util import DecodeProblem, ulp_tol

pytestmark = pytest.mark.gpu


def _both(dev, out_dtype, rope_mode, theta, poison_ws):
    p = dev.p
    outs = []
    for fn in (K.batch_decode_attention, K.batch_decode_attention_noalloc):
        out = torch.full((p.B, p.Hq, p.D), float("nan"), dtype=TORCH_OF[out_dtype], device="cuda")
        lse = torch.full((p.B, p.Hq), float("nan"), dtype=torch.float32, device="cuda")
        if fn is K.batch_decode_attention_noalloc and poison_ws:
            dev.float_ws.fill_(0xFF)  # NaN patterns: the new entry point must not read the plan's float workspace
        fn(dev.handler, dev.q, dev.pt, out, p.Hq, rope_mode=rope_mode, rope_theta=theta, k_scale=dev.k_scale,
           v_scale=dev.v_scale, lse=lse)
        torch.cuda.synchronize()
        outs.append((out, lse))
    return outs


def _run(p, split_tokens, rope_mode=BZ_ROPE_NONE, theta=1e4, expect_splits=True):
    ref, ref_lse = oracle.batch_decode(p.q, p.dtype, p.oracle_kv(), p.Hq, rope_mode=rope_mode, rope_theta=theta,
                                       k_scale=p.k_scale, v_scale=p.v_scale, want_lse=True, parallel=True)
    dev = DeviceDecode(p)
    info = dev.plan(split_tokens)
    if expect_splits:
        assert info["split_seqs"] >= 1, info  # otherwise the scratch array is not exercised
    base = 3e-2 if p.kv_dtype == BZ_E4M3 else 2e-3
    for out_dtype in (BZ_F32, p.dtype):
        (o_ws, l_ws), (o_na, l_na) = _both(dev, out_dtype, rope_mode, theta, poison_ws=True)
        assert torch.equal(o_ws.view(torch.uint8), o_na.view(torch.uint8)), "outputs differ bitwise"
        live = torch.from_numpy(p.ctx > 0).cuda()
        assert torch.equal(l_ws[live], l_na[live])
        got = to_host_f32(o_na)
        if out_dtype == BZ_F32 and p.kv_dtype != BZ_E4M3:
            assert np.abs(got - ref).max() <= (1e-4 if rope_mode != BZ_ROPE_NONE else 2e-5)
        else:
            assert (np.abs(got - ref) <= ulp_tol(ref, p.dtype, base)).all(), float(np.abs(got - ref).max())
    return info


def test_two_calls_in_a_row_second_smaller():
    """Matrix-core kernel, bf16, split sequences; then a smaller batch through the same array."""
    big = DecodeProblem(901, [5000, 17, 2049, 640, 8192, 1, 0, 300], 32, 8, 128, 16, BZ_BF16)
    _run(big, 1024, rope_mode=BZ_ROPE_Q_ONLY, theta=5e5)
    small = DecodeProblem(902, [2500, 33], 32, 8, 128, 16, BZ_BF16)
    _run(small, 1024, rope_mode=BZ_ROPE_Q_ONLY, theta=5e5)


def test_general_kernel_and_e4m3():
    """The general kernel (head_dim 64) and the e4m3 pool take their partials from the same array."""
    _run(DecodeProblem(903, [700, 64, 3000], 8, 2, 64, 16, BZ_F16), 256)
    _run(DecodeProblem(904, [4096, 100, 1024], 64, 8, 128, 16, BZ_BF16, kv_dtype=BZ_E4M3), 1024)
    os.environ["BZ_DECODE_PATH"] = "general"
    try:
        _run(DecodeProblem(905, [3000, 5], 32, 8, 128, 16, BZ_BF16), 512)
    finally:
        del os.environ["BZ_DECODE_PATH"]


def test_rejects_plans_beyond_the_fixed_array():
    """More partials than the array holds: BZ_ERR_WORKSPACE before anything is launched (host check only)."""
    cap = _lib.load().bz_batch_decode_noalloc_scratch_bytes()
    assert cap == 32 << 20
    # 4 sequences x 8 kv heads, 8192 tokens cut every 32 tokens: 256 partials per (sequence, kv head)
    p = DecodeProblem(906, [8192] * 4, 32, 8, 128, 16, BZ_BF16, oversub=1.0)
    dev = DeviceDecode(p, float_ws_bytes=128 << 20, int_ws_bytes=16 << 20)
    dev.plan(32)
    n_partials = int(dev.handler.host_schedule(6)[:, 3].sum())
    assert n_partials * 8256 > cap
    out = torch.zeros((p.B, p.Hq, p.D), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(K.BzError, match="workspace too small"):
        K.batch_decode_attention_noalloc(dev.handler, dev.q, dev.pt, out, p.Hq, rope_mode=BZ_ROPE_NONE)
    torch.cuda.synchronize()
    assert not out.any()  # nothing ran
    K.batch_decode_attention(dev.handler, dev.q, dev.pt, out, p.Hq, rope_mode=BZ_ROPE_NONE)  # the workspace form still works
    torch.cuda.synchronize()
    assert out.any()


def test_recorded_into_a_hip_graph_and_replayed():
    """The call only launches kernels, so it can be captured: three replays with new q contents, eager work and
    synchronisations between them, each compared bit for bit with the same call launched eagerly."""
    p = DecodeProblem(907, [5000, 17, 2049, 640, 1, 300], 32, 8, 128, 16, BZ_BF16)
    dev = DeviceDecode(p)
    info = dev.plan(1024)  # (bz_decode_plan looks the array up: nothing but launches is left to the call)
    assert info["split_seqs"] >= 1
    side = torch.cuda.Stream()
    q = dev.q.clone()
    out_g = torch.empty((p.B, p.Hq, p.D), dtype=torch.bfloat16, device="cuda")
    out_e = torch.empty_like(out_g)

    def call(out, stream):
        K.batch_decode_attention_noalloc(dev.handler, q, dev.pt, out, p.Hq, rope_mode=BZ_ROPE_Q_ONLY, rope_theta=5e5,
                                         stream=stream)

    with torch.cuda.stream(side):
        call(out_g, side.cuda_stream)  # warm-up on the capture stream, outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        call(out_g, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    g = torch.Generator(device="cuda")
    g.manual_seed(907)
    for _ in range(3):
        q.copy_(torch.randn(q.shape, dtype=torch.float32, device="cuda", generator=g).to(q.dtype))
        out_g.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        call(out_e, None)
        torch.cuda.synchronize()
        assert not torch.isnan(out_g.float()).any()
        assert torch.equal(out_g.view(torch.int16), out_e.view(torch.int16))
