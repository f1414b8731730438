"""GPU parity: paged batch decode through the C ABI against the CPU checker on identical bits.

Tolerances (stated by the task): max-abs <= 2e-3 for f16/bf16 results, <= 3e-2 with an e4m3 KV pool.
The fp32-output instantiation is held to 2e-5 to show the arithmetic itself agrees; where the result
is stored in bf16 the bound is widened to half a bf16 step for |o| >= 0.5 (the storage grid is then
coarser than 2e-3).
"""
import os

import numpy as np
import pytest
import torch

import oracle
from blitz_scale_amd import kernel as K
from blitz_scale_amd import workloads as wl
from blitz_scale_amd._lib import (BZ_BF16, BZ_E4M3, BZ_F16, BZ_F32, BZ_LAYOUT_HND, BZ_LAYOUT_NHD, BZ_ROPE_FULL,
                                  BZ_ROPE_NONE, BZ_ROPE_Q_ONLY)

from _gpu import DeviceDecode, to_dev, to_host_bits
from _util import DecodeProblem, ulp_tol

pytestmark = pytest.mark.gpu


def check(p, split_tokens=0, rope_mode=BZ_ROPE_NONE, theta=1e4, f32_tol=2e-5, parallel=False):
    """Both kernels are held to the same bar: the MFMA kernel where it applies (library default) and
    the general kernel (BZ_DECODE_PATH=general at plan time)."""
    ref, ref_lse = oracle.batch_decode(p.q, p.dtype, p.oracle_kv(), p.Hq, rope_mode=rope_mode, rope_theta=theta,
                                       k_scale=p.k_scale, v_scale=p.v_scale, want_lse=True, parallel=parallel)
    os.environ["BZ_DECODE_PATH"] = "general"
    try:
        _check_one(p, split_tokens, rope_mode, theta, f32_tol, ref, ref_lse)
    finally:
        del os.environ["BZ_DECODE_PATH"]
    return _check_one(p, split_tokens, rope_mode, theta, f32_tol, ref, ref_lse)


def _check_one(p, split_tokens, rope_mode, theta, f32_tol, ref, ref_lse):
    dev = DeviceDecode(p)
    info = dev.plan(split_tokens)
    got32, lse = dev.decode(BZ_F32, rope_mode, theta, want_lse=True)
    err32 = np.abs(got32 - ref).max()
    assert err32 <= f32_tol, f"fp32-out max abs err {err32}"
    live = p.ctx > 0
    assert np.abs(lse[live] - ref_lse[live]).max() < 1e-3
    got = dev.decode(None, rope_mode, theta)
    base = 3e-2 if p.kv_dtype == BZ_E4M3 else 2e-3
    assert (np.abs(got - ref) <= ulp_tol(ref, p.dtype, base)).all(), f"max abs err {np.abs(got - ref).max()}"
    return info, got32, ref


def test_c1_plumbing_config():
    """benchmark configuration 1: fp16, batch 4, 4/4 heads, D 64, P 16, ctx {17,64,130,255}, 64-page pool, no RoPE."""
    cfg = wl.CONFIGS["C1"]
    p = DecodeProblem(wl.DEFAULT_SEED, cfg["ctx"], cfg["Hq"], cfg["Hkv"], cfg["D"], cfg["P"], cfg["dtype"],
                      pool_pages=cfg["pool_pages"])
    assert int(p.indptr[-1]) == 31
    info, got, ref = check(p)
    assert np.abs(got - ref).max() < 2e-5


@pytest.mark.parametrize("layout", [BZ_LAYOUT_NHD, BZ_LAYOUT_HND])
@pytest.mark.parametrize("dtype", [BZ_F16, BZ_BF16])
@pytest.mark.parametrize("Hq,Hkv,D,P", [(4, 4, 64, 16), (8, 4, 128, 16), (32, 8, 128, 16), (16, 2, 128, 64),
                                         (8, 8, 128, 1), (8, 1, 64, 8)])
def test_shapes_layouts_dtypes(layout, dtype, Hq, Hkv, D, P):
    ctx = [1, 2, 15, 16, 17, 63, 64, 65, 255, 300, 1000]
    check(DecodeProblem(100 + Hq + D + P, ctx, Hq, Hkv, D, P, dtype, layout=layout))


def test_empty_and_single_token_sequences():
    p = DecodeProblem(7, [0, 1, 0, 33, 1], 8, 2, 128, 16, BZ_F16)
    info, got, ref = check(p)
    assert np.array_equal(got[0], np.zeros_like(got[0])) and np.array_equal(got[2], np.zeros_like(got[2]))
    K, V = p.gather_kv(1)
    assert np.array_equal(got[1], np.repeat(V[0], 4, axis=0))  # ctx = 1: o == v0 exactly


@pytest.mark.parametrize("split_tokens", [16, 64, 256, 2048])
def test_split_k_equals_unsplit(split_tokens):
    p = DecodeProblem(8, [5000, 17, 2049, 640, 8192], 32, 8, 128, 16, BZ_BF16)
    dev = DeviceDecode(p)
    dev.plan(0xFFFFFFFF)
    whole = dev.decode(BZ_F32)
    info = dev.plan(split_tokens)
    assert info["split_seqs"] >= 3
    split = dev.decode(BZ_F32)
    assert np.abs(split - whole).max() < 2e-6
    ref = oracle.batch_decode(p.q, p.dtype, p.oracle_kv(), p.Hq, parallel=True)
    assert np.abs(split - ref).max() < 2e-5


def test_contexts_above_2048_are_split_by_default():
    p = DecodeProblem(9, [2048, 2049, 100], 8, 2, 128, 16, BZ_F16)
    dev = DeviceDecode(p)
    info = dev.plan(0)
    assert info["split_seqs"] >= 1


@pytest.mark.parametrize("rope_mode", [BZ_ROPE_Q_ONLY, BZ_ROPE_FULL])
@pytest.mark.parametrize("theta", [1e4, 5e5])
def test_rope_modes(rope_mode, theta):
    p = DecodeProblem(10, [3, 77, 500, 2100], 8, 2, 128, 16, BZ_F16)
    check(p, rope_mode=rope_mode, theta=theta, f32_tol=1e-4)


def test_page_permutation_is_bit_invariant():
    p = DecodeProblem(11, [700, 64, 3000], 32, 8, 128, 16, BZ_BF16)
    dev = DeviceDecode(p)
    dev.plan()
    a = dev.decode(BZ_F32)
    perm = np.random.default_rng(1).permutation(p.pool_pages)
    pool2 = np.empty_like(p.pool).reshape(p.pool_pages, -1)
    pool2[perm] = p.pool.reshape(p.pool_pages, -1)
    p.pool, p.indices = pool2.reshape(-1), perm[p.indices].astype(np.int32)
    dev2 = DeviceDecode(p)
    dev2.plan()
    assert np.array_equal(dev2.decode(BZ_F32), a)


def test_e4m3_kv_pool():
    """Q bf16, K/V e4m3 with per-kv-head fp32 scales amax/448, dequantised inside the kernel."""
    p = DecodeProblem(12, [100, 1024, 4096, 31], 64, 8, 128, 16, BZ_BF16, kv_dtype=BZ_E4M3)
    check(p, f32_tol=2e-5, parallel=True)


@pytest.mark.parametrize("batch", [12, 24])
@pytest.mark.parametrize("dtype,kv_dtype,rope_mode", [(BZ_F16, None, BZ_ROPE_NONE), (BZ_BF16, None, BZ_ROPE_Q_ONLY),
                                                       (BZ_F16, BZ_E4M3, BZ_ROPE_NONE), (BZ_BF16, BZ_E4M3, BZ_ROPE_Q_ONLY)])
def test_both_sides_of_the_streaming_threshold(batch, dtype, kv_dtype, rope_mode):
    """The planner picks the kernel instantiation whose K/V loads carry the non-temporal hint once every
    wave slot has two tiles or more.  12 and 24 sequences of 512 tokens on 8 kv heads are 1 536 and 3 072
    tiles, i.e. one tile per slot (plain loads) and two (hinted loads) on 256 compute units."""
    ctx = [512] * (batch - 1) + [497]
    p = DecodeProblem(40 + batch, ctx, 16, 8, 128, 16, dtype, kv_dtype=kv_dtype)
    check(p, rope_mode=rope_mode, theta=5e5, f32_tol=1e-4, parallel=True)


def test_c2_shape_reduced_batch():
    """Llama-2-7B MHA decode shape (32/32 heads, D 128, fp16, ctx U[512,2048]) at batch 8, q rotated in-kernel."""
    rng = np.random.default_rng(wl.DEFAULT_SEED)
    ctx = rng.integers(512, 2049, size=8)
    check(DecodeProblem(13, ctx, 32, 32, 128, 16, BZ_F16), rope_mode=BZ_ROPE_Q_ONLY, theta=1e4, f32_tol=1e-4,
          parallel=True)


def test_c3_headline_config_full_size():
    """Llama-3-8B GQA decode at full size: bf16, batch 128, 32/8 heads, log-normal contexts, 2x pool."""
    cfg = wl.CONFIGS["C3"]
    rng = np.random.default_rng(wl.DEFAULT_SEED)
    ctx = wl.ctx_lens_for(cfg, rng)
    p = DecodeProblem(wl.DEFAULT_SEED, ctx, cfg["Hq"], cfg["Hkv"], cfg["D"], cfg["P"], cfg["dtype"], oversub=2.0)
    info, got, ref = check(p, split_tokens=2048, rope_mode=BZ_ROPE_Q_ONLY, theta=5e5, f32_tol=1e-4, parallel=True)
    assert info["split_seqs"] == int((ctx > 2048).sum()) or info["split_seqs"] >= int((ctx > 2048).sum())


def test_c5_shape_reduced_batch():
    """Llama-3-70B GQA decode, e4m3 KV, uniform context 4096, at batch 8."""
    p = DecodeProblem(14, [4096] * 8, 64, 8, 128, 16, BZ_BF16, kv_dtype=BZ_E4M3)
    check(p, parallel=True)


def test_error_codes():
    from blitz_scale_amd import kernel as K
    p = DecodeProblem(15, [5], 4, 2, 64, 16, BZ_F16)
    dev = DeviceDecode(p)
    out = torch.empty((1, 4, 64), dtype=torch.float16, device="cuda")
    with pytest.raises(K.BzError, match="batchDecodeAttention error"):
        K.batch_decode_attention(dev.handler, dev.q, dev.pt, out, 4)  # plan() not called
    dev.plan()
    with pytest.raises(K.BzError):
        K.batch_decode_attention(dev.handler, dev.q, dev.pt, out, 8)  # head count differs from the plan
    with pytest.raises(K.BzError, match="Handler plan"):
        dev.handler.plan(dev.float_ws, dev.float_ws.numel(), dev.int_ws, 16, p.indptr, p.last_page_len, p.B, p.Hq,
                         p.Hkv, p.D, p.P)  # int workspace too small


def test_plan_fits_the_workspace_it_reports():
    """bz_decode_plan_workspace names the bytes plan() needs for the matrix-core kernel and the one-call step:
    buffers of exactly that size are enough; without room for the last section (the unit list of the one-call
    step) the matrix-core schedule is still taken; one more section less and the plan falls back to the general
    kernel (same results every time)."""
    from blitz_scale_amd import kernel as K
    p = DecodeProblem(77, [3000, 40, 900, 2100, 64, 1], 32, 8, 128, 16, BZ_BF16)
    ref = oracle.batch_decode(p.q, p.dtype, p.oracle_kv(), p.Hq)
    h = K.BlitzBatchDecodeHandler()
    fb, ib = h.workspace(p.indptr, p.last_page_len, p.B, p.Hq, p.Hkv, p.D, p.P, split_tokens=1024)
    slots = len(h.host_schedule(4)) - 1
    unit_bytes = (len(h.host_schedule(7)) * 32 + 255) // 256 * 256
    assert fb > 0 and ib > 0 and slots > 0 and unit_bytes > 0
    infos = []
    for int_bytes in (ib, ib - 256, ib - unit_bytes - 256):
        dev = DeviceDecode(p, float_ws_bytes=fb, int_ws_bytes=int_bytes)
        info = dev.plan(1024)
        got = dev.decode(None, BZ_ROPE_NONE)
        assert (np.abs(got - ref) <= ulp_tol(ref, p.dtype)).all()
        infos.append(info)
    assert infos[0]["workgroups"] == slots          # the matrix-core schedule was taken
    assert infos[1]["workgroups"] == slots          # still: only the one-call step's unit list is missing
    assert infos[2]["workgroups"] != slots          # no room for it: page-aligned segments x kv heads


@pytest.mark.parametrize("ctx,expect_min_partials", [
    ([20000], 65),            # one long sequence over the whole chip: hundreds of partials per kv head
    ([1024] * 8, 17),         # small batch: every (sequence, kv head) cut into ~32 one-tile pieces
    ([3000, 5], 17),
])
def test_splits_with_many_partials(ctx, expect_min_partials):
    """The split-K combine takes its sliced form (4 or 8 slices merged through LDS) when a (sequence, kv
    head) has more than 16 partials; results as for any other decode."""
    from blitz_scale_amd import kernel as K
    p = DecodeProblem(4242, ctx, 32, 8, 128, 16, BZ_BF16)
    ref, ref_lse = oracle.batch_decode(p.q, p.dtype, p.oracle_kv(), p.Hq, want_lse=True, parallel=True)
    dev = DeviceDecode(p)
    dev.plan(2048)
    counts = dev.handler.host_schedule(6)[:, 3]
    assert counts.max() >= expect_min_partials
    got32, lse = dev.decode(BZ_F32, BZ_ROPE_NONE, want_lse=True)
    assert np.abs(got32 - ref).max() <= 2e-5
    assert np.abs(lse - ref_lse).max() < 1e-3
    got = dev.decode(None, BZ_ROPE_NONE)
    assert (np.abs(got - ref) <= ulp_tol(ref, p.dtype)).all()


@pytest.mark.parametrize("Hq,Hkv,kv_dtype", [(32, 1, None), (48, 2, None), (128, 2, None), (64, 2, BZ_E4M3)])
def test_more_than_sixteen_q_heads_per_kv_head(Hq, Hkv, kv_dtype):
    """Groups of 24, 32 and 64 q heads run on the matrix-core kernel as equal parts of at most 16 (each part
    reads its kv head's K/V; with an e4m3 pool the scales are those of the kv head, not of the part)."""
    p = DecodeProblem(515, [70, 1500, 16, 333, 2600], Hq, Hkv, 128, 16, BZ_BF16, kv_dtype=kv_dtype)
    ref = oracle.batch_decode(p.q, p.dtype, p.oracle_kv(), Hq, k_scale=p.k_scale, v_scale=p.v_scale, parallel=True)
    dev = DeviceDecode(p)
    info = dev.plan(1024)
    G = Hq // Hkv
    parts = next(q for q in range((G + 15) // 16, G + 1) if G % q == 0)
    pieces = dev.handler.host_schedule(5)
    assert len(pieces) > 0 and pieces[:, 1].max() == Hkv * parts - 1   # the matrix-core schedule was built
    got = dev.decode(None, BZ_ROPE_NONE)
    base = 3e-2 if kv_dtype == BZ_E4M3 else 2e-3
    assert (np.abs(got - ref) <= ulp_tol(ref, p.dtype, base)).all(), float(np.abs(got - ref).max())
    if kv_dtype is None:
        got32 = dev.decode(BZ_F32, BZ_ROPE_NONE)
        assert np.abs(got32 - ref).max() <= 2e-5


@pytest.mark.parametrize("case", ["short_pieces", "chunk_crossing"])
@pytest.mark.parametrize("rope_mode", [BZ_ROPE_NONE, BZ_ROPE_Q_ONLY])
def test_e4m3_pool_with_several_tiles_per_wave_slot(case, rope_mode):
    """The one-byte-pool kernel keeps two tiles in flight per wave (two register sets taking turns).  Regimes of
    that pipeline on 256 compute units (2 048 wave slots):
      short_pieces    700 sequences of 1..200 tokens on 4 kv heads: ~4 or 5 tiles per slot (odd and even counts),
                      pieces of one to seven tiles, so consecutive tiles open new pieces and the q rows of a
                      piece are fetched one tile ahead several times in a row;
      chunk_crossing  150 sequences of 100..3 000 tokens on 8 kv heads: ~29 tiles per slot, i.e. the tile
                      descriptions come in more than one batch of 16 and ragged last tiles sit anywhere."""
    rng = np.random.default_rng(77 if case == "short_pieces" else 78)
    if case == "short_pieces":
        ctx, Hq, Hkv = rng.integers(1, 201, size=700).tolist(), 16, 4
    else:
        ctx, Hq, Hkv = rng.integers(100, 3001, size=150).tolist(), 32, 8
    p = DecodeProblem(500 + len(ctx), ctx, Hq, Hkv, 128, 16, BZ_BF16, kv_dtype=BZ_E4M3)
    ref = oracle.batch_decode(p.q, p.dtype, p.oracle_kv(), p.Hq, rope_mode=rope_mode, rope_theta=5e5, k_scale=p.k_scale,
                              v_scale=p.v_scale, parallel=True)
    dev = DeviceDecode(p)
    info = dev.plan(0)
    tiles = sum((c + 31) // 32 for c in ctx) * Hkv
    assert info["workgroups"] >= 2000 and tiles / info["workgroups"] > (3 if case == "short_pieces" else 20)
    got32 = dev.decode(BZ_F32, rope_mode, 5e5)
    assert np.abs(got32 - ref).max() <= (2e-5 if rope_mode == BZ_ROPE_NONE else 1e-4)
    got = dev.decode(None, rope_mode, 5e5)
    assert (np.abs(got - ref) <= ulp_tol(ref, p.dtype, 3e-2)).all()


@pytest.mark.parametrize("Hq,Hkv,kv_dtype", [(8, 8, None), (16, 8, None), (64, 4, None), (8, 8, BZ_E4M3)])
def test_many_finished_pieces_per_wave_slot(Hq, Hkv, kv_dtype):
    """Thousands of sequences of one or two tiles: a wave slot finishes ten and more (sequence, kv head)s, whose
    normalised rows wait in LDS until the slot is done.  The space holds 8 pieces or 16 rows, so it is emptied in
    the middle of a slot: by the piece count with one or two q heads per kv head, by the row count with sixteen.
    Final rows (16-bit and fp32) and log-sum-exps are checked for every sequence."""
    rng = np.random.default_rng(81)
    B = 2600 if Hkv == 8 else 5200
    ctx = rng.integers(1, 41, size=B).tolist()
    p = DecodeProblem(700 + Hq, ctx, Hq, Hkv, 128, 16, BZ_BF16, kv_dtype=kv_dtype)
    ref, ref_lse = oracle.batch_decode(p.q, p.dtype, p.oracle_kv(), p.Hq, k_scale=p.k_scale, v_scale=p.v_scale, want_lse=True,
                                       parallel=True)
    dev = DeviceDecode(p, float_ws_bytes=128 << 20)
    info = dev.plan(0)
    assert info["segments"] >= 9 * info["workgroups"]  # pieces per wave slot
    got32, lse = dev.decode(BZ_F32, BZ_ROPE_NONE, 1e4, want_lse=True)
    assert np.abs(got32 - ref).max() <= (3e-2 if kv_dtype == BZ_E4M3 else 2e-5)
    assert np.abs(lse - ref_lse).max() < 1e-3
    got = dev.decode(None, BZ_ROPE_NONE, 1e4)
    assert (np.abs(got - ref) <= ulp_tol(ref, p.dtype, 3e-2 if kv_dtype == BZ_E4M3 else 2e-3)).all()


@pytest.mark.parametrize("dtype,kv_dtype", [(BZ_F16, None), (BZ_BF16, None), (BZ_BF16, BZ_E4M3)])
def test_logits_with_a_large_dynamic_range(dtype, kv_dtype):
    """q rows eight times the usual size: logits of +-40 base-2 units, rows that attend to one or two tokens, and
    split-K partials whose log-sum-exps differ by tens of units (two-call path with the combine kernel, and the
    one-call step with its finishing kernel)."""
    from test_gpu_decode_step import run_step
    p = DecodeProblem(60, [3000, 40, 700, 1, 5000, 129], 32, 8, 128, 16, dtype, kv_dtype=kv_dtype)
    p.q = wl.to_bits(wl.to_f32(p.q, dtype) * np.float32(8.0), dtype)
    check(p, split_tokens=512, f32_tol=2e-5, parallel=True)  # matrix-core kernel and general kernel
    run_step(p, split_tokens=512, rope=False)


@pytest.mark.parametrize("Hq,Hkv,D", [(8, 2, 128), (4, 4, 64), (16, 2, 128)])
def test_rope_full_with_and_without_the_angle_table(Hq, Hkv, D):
    """kRoPELlama on a raw-K cache takes the angles of the cached rows from a table in the plan's float workspace
    when there is room behind the partials (groups of one, two and four q heads per workgroup), and evaluates
    them on the fly otherwise (no room; groups of eight).  Same results either way, also after a call in another
    mode has used the workspace in between."""
    p = DecodeProblem(70 + Hq, [3, 77, 500, 2100, 64], Hq, Hkv, D, 16, BZ_F16)
    ref = oracle.batch_decode(p.q, p.dtype, p.oracle_kv(), p.Hq, rope_mode=BZ_ROPE_FULL, rope_theta=5e5, parallel=True)
    roomy = DeviceDecode(p)                       # 32 MiB: partials + 2100 positions x D/2 x 8 bytes fit
    roomy.plan(256)
    a = roomy.decode(BZ_F32, BZ_ROPE_FULL, 5e5)
    assert np.abs(a - ref).max() <= 1e-4
    roomy.decode(BZ_F32, BZ_ROPE_Q_ONLY, 5e5)     # matrix-core path where it applies: its partials overwrite the table
    b = roomy.decode(BZ_F32, BZ_ROPE_FULL, 5e5)   # rebuilt
    assert np.array_equal(a, b)
    c = roomy.decode(BZ_F32, BZ_ROPE_FULL, 1e4)   # another base: rebuilt as well
    ref2 = oracle.batch_decode(p.q, p.dtype, p.oracle_kv(), p.Hq, rope_mode=BZ_ROPE_FULL, rope_theta=1e4, parallel=True)
    assert np.abs(c - ref2).max() <= 1e-4
    need = K.BlitzBatchDecodeHandler().workspace(p.indptr, p.last_page_len, p.B, Hq, Hkv, D, 16, split_tokens=256)[0]
    tight = DeviceDecode(p, float_ws_bytes=max(int(need), 4096))  # room for the partials only
    tight.plan(256)
    d = tight.decode(BZ_F32, BZ_ROPE_FULL, 5e5)
    assert np.abs(d - ref).max() <= 1e-4 and np.abs(d - a).max() <= 2e-6
