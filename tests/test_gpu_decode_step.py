"""GPU parity: the one-call decode step (bz_decode_step) against the CPU checker and against the two calls
it stands for (append_decode_kv_cache, then batch_decode_attention; src/layer/attn.h:196-203).

The pool must receive exactly the bits the append kernel writes (bit-exact against the two-call path; against
the checker up to the device's sincosf, as in the append tests).  The attention result is compared with the
checker run on the very bits the device cached: max-abs <= 2e-3 for 16-bit results (widened to half a bf16
step where the storage grid is coarser), <= 3e-2 with an e4m3 pool, and <= 1e-4 for the fp32-output
instantiation (q is rotated inside the kernels).  The caller's q, k and v rows must stay untouched.
"""
import os

import numpy as np
import pytest
import torch

import oracle
from blitz_scale_amd import kernel as K
from blitz_scale_amd import workloads as wl
from blitz_scale_amd._lib import BZ_BF16, BZ_E4M3, BZ_F16, BZ_F32, BZ_LAYOUT_HND, BZ_LAYOUT_NHD, BZ_ROPE_NONE, BZ_ROPE_Q_ONLY

from _gpu import TORCH_OF, DeviceDecode, to_dev, to_host_bits, to_host_f32
from _util import DecodeProblem, ulp_tol

pytestmark = pytest.mark.gpu


def run_step(p, split_tokens=0, rope=True, theta=5e5, expect_units=True, form="one_call", float_ws_bytes=128 << 20):
    """form "one_call": the two-launch form wherever it applies, also on batches where the library would choose
    the two calls (BZ_DECODE_PATH=one_call at plan time); "library": the library's own choice.  Returns the form
    that ran beside the results."""
    rng = np.random.default_rng(999)
    k = wl.randn_bits(rng, (p.B, p.Hkv, p.D), p.dtype)
    v = wl.randn_bits(rng, (p.B, p.Hkv, p.D), p.dtype)
    base = 3e-2 if p.kv_dtype == BZ_E4M3 else 2e-3

    # ---- the two calls, on their own copy of the pool
    two = DeviceDecode(p)
    two.plan(split_tokens)
    K.append_decode_kv_cache(two.pt, to_dev(k, p.dtype), to_dev(v, p.dtype), rope=rope, rope_theta=theta,
                             k_scale=two.k_scale, v_scale=two.v_scale)
    out_two = two.decode(BZ_F32, BZ_ROPE_Q_ONLY if rope else BZ_ROPE_NONE, theta)
    pool_two = to_host_bits(two.pool)

    # ---- the one call
    dev = DeviceDecode(p, float_ws_bytes=float_ws_bytes)  # default: the reference's size (src/model/llama.h:111), one partial per piece fits
    if form == "one_call":
        os.environ["BZ_DECODE_PATH"] = "one_call"
    try:
        dev.plan(split_tokens)
    finally:
        if form == "one_call":
            del os.environ["BZ_DECODE_PATH"]
    dev.form = dev.handler.step_form()
    if form == "one_call" and expect_units:
        assert dev.form == "one_call"
    if expect_units:
        assert len(dev.handler.host_schedule(7)) == int((p.ctx > 0).sum()) * p.Hkv * max(1, (p.Hq // p.Hkv + 15) // 16)
    kd, vd = to_dev(k, p.dtype), to_dev(v, p.dtype)
    results = {}
    for out_dtype in (BZ_F32, p.dtype):
        dev.pool.copy_(to_dev(p.pool, p.kv_dtype))
        out = torch.full((p.B, p.Hq, p.D), float("nan"), dtype=TORCH_OF[out_dtype], device="cuda")
        lse = torch.full((p.B, p.Hq), float("nan"), dtype=torch.float32, device="cuda")
        K.decode_step(dev.handler, dev.q, kd, vd, dev.pt, out, p.Hq, rope=rope, rope_theta=theta, k_scale=dev.k_scale,
                      v_scale=dev.v_scale, lse=lse)
        torch.cuda.synchronize()
        results[out_dtype] = (to_host_f32(out), lse.cpu().numpy())
    pool_one = to_host_bits(dev.pool)
    assert np.array_equal(to_host_bits(dev.q), p.q), "q was modified"
    assert np.array_equal(to_host_bits(kd), k) and np.array_equal(to_host_bits(vd), v), "k / v rows were modified"
    assert np.array_equal(pool_one, pool_two), "the appended rows differ from the append kernel's"

    # ---- the checker: the appended rows, then attention over the bits the device cached
    want_pool = p.pool.copy()
    oracle.append_decode_kv(p.oracle_kv(want_pool), k, v, p.dtype, rope=rope, rope_theta=theta, k_scale=p.k_scale,
                            v_scale=p.v_scale)
    if p.kv_dtype == BZ_E4M3:
        assert (pool_one != want_pool).mean() < 2e-3
    else:
        assert np.abs(wl.to_f32(pool_one, p.kv_dtype) - wl.to_f32(want_pool, p.kv_dtype)).max() <= 2.0 ** -6
        assert (pool_one != want_pool).mean() < 2e-3
    ref, ref_lse = oracle.batch_decode(p.q, p.dtype, p.oracle_kv(pool_one), p.Hq,
                                       rope_mode=oracle.ROPE_Q_ONLY if rope else oracle.ROPE_NONE, rope_theta=theta,
                                       k_scale=p.k_scale, v_scale=p.v_scale, want_lse=True, parallel=True)
    got32, lse32 = results[BZ_F32]
    live = p.ctx > 0
    if p.kv_dtype != BZ_E4M3:
        assert np.abs(got32 - ref).max() <= 1e-4, float(np.abs(got32 - ref).max())
        assert np.abs(got32 - out_two).max() <= 1e-4
    else:
        assert np.abs(got32 - ref).max() <= 3e-2
    assert np.abs(lse32[live] - ref_lse[live]).max() < 1e-3
    got, _ = results[p.dtype]
    assert (np.abs(got - ref) <= ulp_tol(ref, p.dtype, base)).all(), float(np.abs(got - ref).max())
    assert not got32[~live].any()  # sequences without pages: zero rows
    return dev, got32, ref


@pytest.mark.parametrize("dtype", [BZ_BF16, BZ_F16])
@pytest.mark.parametrize("layout", [BZ_LAYOUT_HND, BZ_LAYOUT_NHD])
def test_step_with_split_and_whole_sequences(dtype, layout):
    """Sequences from one token (the new one only) to several split pieces; one without pages."""
    ctx = [1, 2, 5000, 17, 2049, 640, 32, 33, 0, 8192, 300, 31]
    run_step(DecodeProblem(300, ctx, 32, 8, 128, 16, dtype, layout=layout), split_tokens=1024)


def test_step_one_token_only_gives_v():
    """A sequence whose only token is the new one: the output is that token's V row (as cached), exactly."""
    p = DecodeProblem(301, [1, 1, 1], 8, 2, 128, 16, BZ_F16)
    dev, got32, ref = run_step(p, rope=True, theta=1e4)
    pool = wl.to_f32(to_host_bits(dev.pool), p.kv_dtype)
    for b in range(3):
        page = int(p.indices[p.indptr[b]])
        for h in range(8):
            off = page * p.stride_page + p.stride_page // 2 + (h // 4) * p.stride_h
            assert np.array_equal(got32[b, h], pool[off:off + 128])


def test_step_e4m3_pool():
    p = DecodeProblem(302, [100, 1024, 4096, 31, 1], 64, 8, 128, 16, BZ_BF16, kv_dtype=BZ_E4M3)
    run_step(p, split_tokens=1024)


def test_step_e4m3_pool_with_several_tiles_per_wave_slot():
    """700 short sequences on 4 kv heads: four or five tiles per wave slot, pieces of one to seven tiles, so the
    two-tiles-in-flight pipeline of the one-byte-pool kernel runs with odd and even counts and opens pieces on
    consecutive tiles, in step mode (every piece leaves a partial, the newest token is left to the second kernel)."""
    ctx = np.random.default_rng(79).integers(1, 201, size=700).tolist()
    run_step(DecodeProblem(305, ctx, 16, 4, 128, 16, BZ_BF16, kv_dtype=BZ_E4M3), split_tokens=2048)


def test_step_takes_the_faster_form():
    """Left to itself the call takes its two-launch form where most (sequence, kv head)s are split over wave slots
    (few long sequences) and the two calls where most are whole (many short ones); same results either way."""
    dev, _, _ = run_step(DecodeProblem(308, [3000, 4100, 2500, 3300], 32, 8, 128, 16, BZ_BF16), form="library")
    assert dev.form == "one_call"
    ctx = np.random.default_rng(80).integers(1, 120, size=1100).tolist()
    dev, _, _ = run_step(DecodeProblem(309, ctx, 16, 4, 128, 16, BZ_BF16), form="library")
    assert dev.form == "two_calls"


def test_step_with_many_finished_pieces_per_wave_slot():
    """2 600 sequences of one or two tiles on 8 kv heads, one q head each: a wave slot finishes ten and more pieces,
    more than the space for their parked rows holds, in the two-launch form (every piece a partial row)."""
    ctx = np.random.default_rng(82).integers(1, 41, size=2600).tolist()
    dev, _, _ = run_step(DecodeProblem(310, ctx, 8, 8, 128, 16, BZ_BF16), form="one_call", float_ws_bytes=256 << 20)  # 8 KB per piece
    info = dev.handler.info()
    assert info["segments"] >= 9 * info["workgroups"]


def test_step_without_rope_and_with_many_partials():
    run_step(DecodeProblem(303, [20000, 77], 32, 8, 128, 16, BZ_BF16), split_tokens=2048, rope=False)


def test_step_groups_of_more_than_sixteen_heads():
    run_step(DecodeProblem(304, [70, 1500, 16, 2600], 32, 1, 128, 64, BZ_BF16), split_tokens=1024)


def test_step_headline_shape_full_size():
    """Llama-3-8B GQA decode at full size (batch 128, log-normal contexts): the one call against the checker."""
    cfg = wl.CONFIGS["C3"]
    ctx = wl.ctx_lens_for(cfg, np.random.default_rng(wl.DEFAULT_SEED))
    p = DecodeProblem(wl.DEFAULT_SEED, ctx, cfg["Hq"], cfg["Hkv"], cfg["D"], cfg["P"], cfg["dtype"], oversub=2.0)
    run_step(p, split_tokens=2048, theta=5e5)


def test_step_falls_back_where_the_matrix_core_kernel_does_not_apply():
    """head_dim 64 (general kernel) and a float workspace without room for one partial per piece: the call
    runs the two-call sequence itself, same results."""
    run_step(DecodeProblem(305, [17, 64, 130, 255, 1], 4, 4, 64, 16, BZ_F16), expect_units=False, theta=1e4)
    os.environ["BZ_DECODE_PATH"] = "general"
    try:
        run_step(DecodeProblem(306, [700, 3000], 32, 8, 128, 16, BZ_BF16), split_tokens=512, form="library")
    finally:
        del os.environ["BZ_DECODE_PATH"]


def test_step_replays_from_a_hip_graph_and_runs_steps_ahead():
    """Three steps from one plan and one table that runs ahead (device counter), replayed from one graph: every
    step equals the eager two-call sequence on the table truncated to the present."""
    H = 3
    ctx0 = np.array([40, 2100, 15, 700])
    p = DecodeProblem(307, ctx0 + H, 32, 8, 128, 16, BZ_BF16)  # the table as it will be after H steps
    rng = np.random.default_rng(5)
    dev = DeviceDecode(p)
    dev.plan(1024)
    counter = torch.tensor([H - 1], dtype=torch.int32, device="cuda")
    dev.pt.steps_ahead_d = counter
    tdt = TORCH_OF[p.dtype]
    qs = torch.empty((p.B, p.Hq, p.D), dtype=tdt, device="cuda")
    ks = torch.empty((p.B, p.Hkv, p.D), dtype=tdt, device="cuda")
    vs = torch.empty_like(ks)
    outs = torch.empty_like(qs)
    side = torch.cuda.Stream()

    def step(stream):
        K.decode_step(dev.handler, qs, ks, vs, dev.pt, outs, p.Hq, rope=True, rope_theta=5e5, stream=stream)
        K.steps_ahead_advance(counter, stream=stream)

    for t in (qs, ks, vs):
        t.normal_()
    pool0 = dev.pool.clone()
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        step(side.cuda_stream)  # warm-up outside the capture
    torch.cuda.synchronize()
    dev.pool.copy_(pool0)
    counter.fill_(H - 1)
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.graph(graph, stream=side):
        step(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    dev.pool.copy_(pool0)
    counter.fill_(H - 1)
    pool_ref = to_host_bits(pool0).copy()
    for i in range(H):
        bits = [wl.randn_bits(rng, s, p.dtype) for s in ((p.B, p.Hq, p.D), (p.B, p.Hkv, p.D), (p.B, p.Hkv, p.D))]
        for dst, b in zip((qs, ks, vs), bits):
            dst.copy_(to_dev(b, p.dtype))
        outs.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        (torch.randn(1 << 14, device="cuda") * 2).sum().item()  # unrelated eager work between replays
        # the checker on the table as it is at this step
        now = DecodeProblem(307, ctx0 + i + 1, 32, 8, 128, 16, BZ_BF16)
        now.indices, now.indptr = p.indices, p.indptr  # same pages; shorter last pages
        lens = ctx0 + i + 1
        now.indptr = np.concatenate([[0], np.cumsum((lens + 15) // 16)]).astype(np.int32)
        now.indices = np.concatenate([p.indices[p.indptr[b]:p.indptr[b] + (lens[b] + 15) // 16] for b in range(p.B)]).astype(np.int32)
        now.last_page_len = ((lens - 1) % 16 + 1).astype(np.int32)
        oracle.append_decode_kv(now.oracle_kv(pool_ref), bits[1], bits[2], p.dtype, rope=True, rope_theta=5e5)
        pool_got = to_host_bits(dev.pool)
        assert np.abs(wl.to_f32(pool_got, p.dtype) - wl.to_f32(pool_ref, p.dtype)).max() <= 2.0 ** -6
        pool_ref = pool_got.copy()  # continue from the device's bits
        ref = oracle.batch_decode(bits[0], p.dtype, now.oracle_kv(pool_got), p.Hq, rope_mode=oracle.ROPE_Q_ONLY,
                                  rope_theta=5e5, parallel=True)
        got = outs.float().cpu().numpy()
        assert (np.abs(got - ref) <= ulp_tol(ref, p.dtype, 2e-3)).all(), (i, float(np.abs(got - ref).max()))
    assert int(counter.item()) == 0
