"""Seeded random shapes through the C ABI against the CPU checker: batch sizes, ragged context lengths
(zero and one included), head groupings, page sizes, layouts, types, split thresholds and RoPE modes
drawn at random, so that combinations nobody thought of writing down get exercised too.  The draws are
fixed by the seed; tolerances as in the per-kernel tests (max-abs <= 2e-3 for f16/bf16 with the bf16
storage-step widening, <= 3e-2 with an e4m3 pool, page placement bit-exact)."""
import numpy as np
import pytest
import torch

import oracle
from blitz_scale_amd import kernel as K
from blitz_scale_amd import workloads as wl
from blitz_scale_amd._lib import (BZ_BF16, BZ_E4M3, BZ_F16, BZ_LAYOUT_HND, BZ_LAYOUT_NHD, BZ_ROPE_FULL, BZ_ROPE_NONE,
                                  BZ_ROPE_Q_ONLY)

from _gpu import DeviceDecode, to_dev, to_host_bits
from _util import LN2, PREFILL_BF16_WIDEN_V_ERR, DecodeProblem, ulp_tol
from test_gpu_prefill import Prefill


def prefill_tol(ref, dtype):
    """bf16 prefill runs in its default mode here (V widened to f16 on chip): see _util.PREFILL_BF16_WIDEN_V_ERR."""
    return ulp_tol(ref, dtype, before_rounding=PREFILL_BF16_WIDEN_V_ERR if dtype == BZ_BF16 else 0.0)

pytestmark = pytest.mark.gpu


def draw_lens(rng, B, longest):
    kind = rng.integers(0, 3)
    if kind == 0:
        lens = rng.integers(0, longest + 1, B)
    elif kind == 1:  # mostly short with a few long ones
        lens = np.where(rng.random(B) < 0.2, rng.integers(longest // 2, longest + 1, B), rng.integers(0, 70, B))
    else:            # around tile and page boundaries
        lens = rng.choice([0, 1, 15, 16, 17, 31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 256, 257], B)
    return [int(x) for x in lens]


@pytest.mark.parametrize("case", range(24))
def test_decode_random_shapes(case):
    rng = np.random.default_rng(9000 + case)
    B = int(rng.integers(1, 33))
    Hkv = int(rng.choice([1, 2, 4, 8]))
    G = int(rng.choice([1, 2, 3, 4, 6, 7, 8, 12, 16, 32]))
    D = int(rng.choice([64, 128, 128, 128]))
    P = int(rng.choice([8, 16, 16, 32, 64]))
    dtype = int(rng.choice([BZ_F16, BZ_BF16]))
    kv_dtype = BZ_E4M3 if rng.random() < 0.25 else dtype
    layout = int(rng.choice([BZ_LAYOUT_HND, BZ_LAYOUT_NHD]))
    rope_mode = int(rng.choice([BZ_ROPE_NONE, BZ_ROPE_NONE, BZ_ROPE_Q_ONLY, BZ_ROPE_FULL]))
    if kv_dtype == BZ_E4M3 and rope_mode == BZ_ROPE_FULL:
        rope_mode = BZ_ROPE_Q_ONLY  # rotating quantised K on the fly is not a mode of the library
    split_tokens = int(rng.choice([0, 64, 256, 2048, 0xFFFFFFFF]))
    ctx = draw_lens(rng, B, 2500)
    if not any(ctx):
        ctx[0] = 40
    p = DecodeProblem(9100 + case, ctx, Hkv * G, Hkv, D, P, dtype, kv_dtype=kv_dtype, layout=layout)
    theta = float(rng.choice([1e4, 5e5]))
    ref = oracle.batch_decode(p.q, dtype, p.oracle_kv(), p.Hq, rope_mode=rope_mode, rope_theta=theta,
                              k_scale=p.k_scale, v_scale=p.v_scale, parallel=True)
    dev = DeviceDecode(p)
    dev.plan(split_tokens)
    got = dev.decode(None, rope_mode, theta)
    base = 3e-2 if kv_dtype == BZ_E4M3 else 2e-3
    live = p.ctx > 0
    err = np.abs(got - ref)
    assert (err[live] <= ulp_tol(ref, dtype, base)[live]).all(), (case, float(err[live].max()))
    assert not got[~live].any()


@pytest.mark.parametrize("case", range(12))
def test_prefill_random_shapes(case):
    rng = np.random.default_rng(9500 + case)
    B = int(rng.integers(1, 7))
    Hkv = int(rng.choice([1, 2, 4]))
    G = int(rng.choice([1, 2, 3, 4, 7, 8]))
    dtype = int(rng.choice([BZ_F16, BZ_BF16]))
    causal = bool(rng.random() < 0.75)
    lens = [max(1, x) for x in draw_lens(rng, B, 700)]
    pf = Prefill(9600 + case, lens, Hkv * G, Hkv, 128, dtype)
    rope_mode = BZ_ROPE_FULL if case % 2 else BZ_ROPE_NONE
    got = pf.run(causal=causal, rope_mode=rope_mode, theta=1e4)
    assert not np.isnan(got).any()
    if rope_mode == BZ_ROPE_NONE:
        ref = oracle.batch_prefill_ragged(pf.q, pf.k, pf.v, dtype, pf.indptr, Hkv * G, Hkv, 128, causal=causal,
                                          parallel=True)
        tol = prefill_tol(ref, dtype)
    else:
        # kRoPELlama inside the call: the k rows are rotated in place (one rounding to the storage type, at most
        # one step away from the checker's rotated rows), q in registers; the attention itself is then checked
        # on the k bits the device left behind.
        k_rot = oracle.rope_ragged(pf.k, dtype, pf.indptr, Hkv, 128, 1e4)
        step = 2.0 ** -8 if dtype == BZ_F16 else 2.0 ** -5
        assert np.abs(wl.to_f32(pf.k_after, dtype) - wl.to_f32(k_rot, dtype)).max() <= step
        assert (pf.k_after != k_rot).mean() < 3e-3
        assert np.array_equal(pf.q_after, pf.q)
        # q as it enters the matrix cores (rotated in fp32, scaled, rounded once): the stated bar for both types
        q_fed = pf.q_as_fed(1e4)
        ref = oracle.batch_prefill_ragged(q_fed, pf.k_after, pf.v, dtype, pf.indptr, Hkv * G, Hkv, 128, causal=causal,
                                          sm_scale=LN2, parallel=True)
        tol = prefill_tol(ref, dtype)
    assert (np.abs(got - ref) <= tol).all(), (case, float(np.abs(got - ref).max()))


@pytest.mark.parametrize("case", range(12))
def test_prefill_random_shapes_q_rotated_in_registers(case):
    """BZ_ROPE_Q_ONLY of the prefill call: q is rotated on its way into the operand registers (angle table in the
    float workspace), k is taken as it is; the checker does the same in fp32.  Float workspaces with and without
    room for the table (without: q is rotated in place by a separate kernel first)."""
    rng = np.random.default_rng(9700 + case)
    B = int(rng.integers(1, 7))
    Hkv = int(rng.choice([1, 2, 4]))
    G = int(rng.choice([1, 2, 3, 4, 7, 8]))
    dtype = int(rng.choice([BZ_F16, BZ_F16, BZ_BF16]))
    causal = bool(rng.random() < 0.75)
    theta = float(rng.choice([1e4, 5e5]))
    lens = [max(1, x) for x in draw_lens(rng, B, 900)]
    pf = Prefill(9750 + case, lens, Hkv * G, Hkv, 128, dtype)
    roomy = bool(rng.random() < 0.75)
    pf.float_ws = torch.empty((1 << 20) if roomy else 256, dtype=torch.uint8, device="cuda")
    got = pf.run(causal=causal, rope_mode=BZ_ROPE_Q_ONLY, theta=theta)
    assert np.array_equal(pf.k_after, pf.k)
    assert not np.isnan(got).any()
    if roomy:
        assert np.array_equal(pf.q_after, pf.q)
        # q as it enters the matrix cores (rotated in fp32, scaled, rounded once): the stated bar for both types
        q_fed = pf.q_as_fed(theta)
        ref = oracle.batch_prefill_ragged(q_fed, pf.k, pf.v, dtype, pf.indptr, Hkv * G, Hkv, 128, causal=causal,
                                          sm_scale=LN2, parallel=True)
    else:
        ref = oracle.batch_prefill_ragged(pf.q_after, pf.k, pf.v, dtype, pf.indptr, Hkv * G, Hkv, 128, causal=causal,
                                          parallel=True)
    tol = prefill_tol(ref, dtype)
    assert (np.abs(got - ref) <= tol).all(), (case, float(np.abs(got - ref).max()))


@pytest.mark.parametrize("case", range(16))
def test_decode_step_random_shapes(case):
    """The one-call decode step (append + attention) on random shapes: matrix-core path and the fallback, e4m3
    pools, both layouts, with and without RoPE; checked against the two-call sequence and the checker.  Even
    cases force the two-launch form wherever it applies, odd ones leave the choice of form to the library."""
    from test_gpu_decode_step import run_step
    rng = np.random.default_rng(9300 + case)
    B = int(rng.integers(1, 41))
    Hkv = int(rng.choice([1, 2, 4, 8]))
    G = int(rng.choice([1, 2, 3, 4, 6, 8, 12, 16, 32]))
    D = int(rng.choice([64, 128, 128, 128, 128]))
    P = int(rng.choice([8, 16, 16, 32, 64]))
    dtype = int(rng.choice([BZ_F16, BZ_BF16]))
    kv_dtype = BZ_E4M3 if rng.random() < 0.3 else dtype
    layout = int(rng.choice([BZ_LAYOUT_HND, BZ_LAYOUT_NHD]))
    split_tokens = int(rng.choice([0, 64, 256, 2048]))
    ctx = [max(1, x) for x in draw_lens(rng, B, 2500)]  # the newest token included
    if rng.random() < 0.3:
        ctx[int(rng.integers(0, B))] = 0               # a sequence without pages
    if not any(ctx):
        ctx[0] = 40
    p = DecodeProblem(9400 + case, ctx, Hkv * G, Hkv, D, P, dtype, kv_dtype=kv_dtype, layout=layout)
    parts = (G + 15) // 16
    while parts < G and G % parts:
        parts += 1
    mfma = D == 128 and P % 16 == 0 and parts <= 8
    if mfma:
        dev = DeviceDecode(p)
        dev.plan(split_tokens)
        assert len(dev.handler.host_schedule(7)) == int((p.ctx > 0).sum()) * Hkv * parts
    run_step(p, split_tokens=split_tokens, rope=bool(rng.random() < 0.7), theta=float(rng.choice([1e4, 5e5])),
             expect_units=False, form="one_call" if case % 2 == 0 else "library")


@pytest.mark.parametrize("case", range(6))
def test_store_and_append_random_shapes(case):
    """Prefill store followed by a decode append into the same table: page placement bit-exact."""
    rng = np.random.default_rng(9800 + case)
    B = int(rng.integers(1, 9))
    Hkv = int(rng.choice([1, 2, 8]))
    D = int(rng.choice([64, 128]))
    P = int(rng.choice([8, 16, 64]))
    dtype = int(rng.choice([BZ_F16, BZ_BF16]))
    layout = int(rng.choice([BZ_LAYOUT_HND, BZ_LAYOUT_NHD]))
    lens = [max(1, x) for x in draw_lens(rng, B, 300)]
    p = DecodeProblem(9900 + case, [l + 1 for l in lens], Hkv, Hkv, D, P, dtype, layout=layout)  # len+1 slots reserved
    indptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    N = int(indptr[-1])
    k, v = wl.randn_bits(rng, (N, Hkv, D), dtype), wl.randn_bits(rng, (N, Hkv, D), dtype)
    kn, vn = wl.randn_bits(rng, (B, Hkv, D), dtype), wl.randn_bits(rng, (B, Hkv, D), dtype)
    want = p.pool.copy()
    oracle.store_prefill_kv(p.oracle_kv(want), k, v, dtype, indptr)
    oracle.append_decode_kv(p.oracle_kv(want), kn, vn, dtype)
    dev = DeviceDecode(p)
    K.store_prefill_kv_cache(dev.pt, to_dev(k, dtype), to_dev(v, dtype), torch.from_numpy(indptr).cuda(), num_tokens=N)
    K.append_decode_kv_cache(dev.pt, to_dev(kn, dtype), to_dev(vn, dtype))
    torch.cuda.synchronize()
    assert np.array_equal(to_host_bits(dev.pool), want), case


@pytest.mark.parametrize("case", range(8))
def test_elementwise_random_shapes(case):
    """RMSNorm, add+RMSNorm, SiLU-gate and residual add at odd row counts and widths (multiples of 8)."""
    rng = np.random.default_rng(9950 + case)
    N = int(rng.integers(1, 90))
    h = 8 * int(rng.integers(1, 1400))
    I = 8 * int(rng.integers(1, 2000))
    dtype = int(rng.choice([BZ_F16, BZ_BF16]))
    x, r = wl.randn_bits(rng, (N, h), dtype), wl.randn_bits(rng, (N, h), dtype)
    w = wl.randn_bits(rng, (h,), dtype, mean=1.0, std=0.02)
    gu = wl.randn_bits(rng, (N, 2 * I), dtype)

    def close(got_bits, ref):
        got = wl.to_f32(got_bits, dtype)
        assert (np.abs(got - ref) <= ulp_tol(ref, dtype)).all(), (case, float(np.abs(got - ref).max()))

    xd, rd, wd = to_dev(x, dtype), to_dev(r, dtype), to_dev(w, dtype)
    out = torch.empty_like(xd)
    K.rms_norm(xd, wd, out, N, h)
    torch.cuda.synchronize()
    close(to_host_bits(out), oracle.rms_norm(x, w, dtype, 1e-5))
    ref, ref_res = oracle.add_rms_norm(x, r, w, dtype)
    K.add_rms_norm(xd, rd, wd, N, h)
    torch.cuda.synchronize()
    assert np.array_equal(to_host_bits(rd), ref_res)
    close(to_host_bits(xd), ref)
    act = torch.empty((N, I), dtype=xd.dtype, device="cuda")
    K.silu_and_mul(to_dev(gu, dtype), act, N, I)
    torch.cuda.synchronize()
    close(to_host_bits(act), oracle.silu_and_mul(gu, dtype))
    a2, b2 = to_dev(x, dtype), to_dev(r, dtype)
    K.add_residual(a2, b2, N, h)
    torch.cuda.synchronize()
    assert np.array_equal(to_host_bits(b2), oracle.add_residual(x, r, dtype))


@pytest.mark.parametrize("case", range(6))
def test_wire_random_shapes(case):
    """Migration payload at random geometry: byte-exact pack, and unpack into other pages."""
    rng = np.random.default_rng(9980 + case)
    layers, max_pages = int(rng.integers(1, 6)), int(rng.integers(3, 40))
    Hkv, P, D = int(rng.choice([1, 2, 5, 8])), int(rng.choice([4, 16, 64])), int(rng.choice([64, 128]))
    dtype = int(rng.choice([BZ_F16, BZ_BF16, BZ_E4M3]))
    layout = int(rng.choice([BZ_LAYOUT_HND, BZ_LAYOUT_NHD]))
    sp = 2 * Hkv * P * D
    if dtype == BZ_E4M3:
        bits = rng.integers(0, 256, size=layers * max_pages * sp, dtype=np.uint8)
    else:
        bits = wl.randn_bits(rng, (layers * max_pages * sp,), dtype)
    n = int(rng.integers(1, max_pages + 1))
    ids = rng.permutation(max_pages)[:n].astype(np.int32)
    start = int(rng.integers(0, layers))
    cnt = int(rng.integers(1, layers - start + 1))
    pool = to_dev(bits, dtype)
    pt = K.PageTable(1, P, Hkv, D, pool, layout=layout)
    want = oracle.kv_pages_pack(bits, dtype, max_pages, sp, ids, start, cnt)
    wire = torch.zeros(want.nbytes, dtype=torch.uint8, device="cuda")
    ids_d = torch.from_numpy(ids).cuda()
    K.pack_kv_pages(pt, max_pages, ids_d, start, cnt, wire)
    torch.cuda.synchronize()
    assert np.array_equal(wire.cpu().numpy(), want.view(np.uint8)), case
    dst_bits = np.zeros_like(bits)
    dst = to_dev(dst_bits, dtype)
    dpt = K.PageTable(1, P, Hkv, D, dst, layout=layout)
    dst_ids = rng.permutation(max_pages)[:n].astype(np.int32)
    K.unpack_kv_pages(dpt, max_pages, torch.from_numpy(dst_ids).cuda(), start, cnt, wire)
    torch.cuda.synchronize()
    oracle.kv_pages_unpack(dst_bits, dtype, max_pages, sp, dst_ids, start, cnt, want)
    assert np.array_equal(to_host_bits(dst), dst_bits), case


@pytest.mark.parametrize("case", range(18))
def test_prefill_random_shapes_with_q_rows_for_the_last_tokens(case):
    """Distinct ragged indices (src/kernel/attention.h:9-22 carries both): every request has K/V rows for all its tokens
    and q rows for a random number of its last ones (none to all), in every RoPE mode and storage type, causal or not.
    The result must be those rows of self-attention over the whole request, which is what the checker computes."""
    from blitz_scale_amd._lib import BZ_PREFILL_BF16_HEAD_TAIL, BZ_PREFILL_BF16_WIDEN_V
    from _gpu import to_dev, to_host_bits
    from _util import prefill_angle_table, prefill_q_as_fed
    rng = np.random.default_rng(9900 + case)
    B = int(rng.integers(1, 6))
    dtype, mode = [(BZ_F16, None), (BZ_BF16, BZ_PREFILL_BF16_WIDEN_V), (BZ_BF16, BZ_PREFILL_BF16_HEAD_TAIL)][case % 3]
    Hkv = int(rng.choice([1, 2, 4]))
    Hq = Hkv * int(rng.choice([1, 2, 4, 8]))
    D = 128
    kv_lens = rng.integers(1, int(rng.choice([40, 130, 300, 700])) + 1, B)
    q_lens = np.array([int(rng.integers(0, l + 1)) for l in kv_lens])
    q_lens[int(rng.integers(0, B))] = max(1, int(q_lens.max()))  # at least one q row in the batch
    q_lens = np.minimum(q_lens, kv_lens)
    causal = bool(rng.random() < 0.7)
    rope_mode = [BZ_ROPE_NONE, BZ_ROPE_Q_ONLY, BZ_ROPE_FULL][(case // 3) % 3]
    theta = float(rng.choice([1e4, 5e5]))
    kvp = np.concatenate([[0], np.cumsum(kv_lens)]).astype(np.int32)
    qop = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32)
    Nkv = int(kvp[-1])
    q_full = wl.randn_bits(rng, (Nkv, Hq, D), dtype)
    k = wl.randn_bits(rng, (Nkv, Hkv, D), dtype)
    v = wl.randn_bits(rng, (Nkv, Hkv, D), dtype)
    rows = np.concatenate([np.arange(kvp[b + 1] - q_lens[b], kvp[b + 1]) for b in range(B)]).astype(np.int32)
    k_in = oracle.rope_ragged(k, dtype, kvp, Hkv, D, theta) if rope_mode == BZ_ROPE_Q_ONLY else k
    fws = torch.empty(1 << 20, dtype=torch.uint8, device="cuda")
    iws = torch.empty(1 << 20, dtype=torch.uint8, device="cuda")
    h = K.BatchPrefillRaggedHandler()
    if mode is not None:
        h.set_bf16_mode(mode)
    h.plan(fws, fws.numel(), iws, iws.numel(), qop, kvp, B, Hq, Hkv, D, 16)
    qd, kd, vd = to_dev(q_full[rows], dtype), to_dev(k_in, dtype), to_dev(v, dtype)
    out = torch.full_like(qd, float("nan"))
    K.batch_prefill_attention(h, qd, torch.from_numpy(qop).cuda(), kd, vd, torch.from_numpy(kvp).cuda(), out, B, Hq, Hkv, D,
                              causal=causal, rope_mode=rope_mode, rope_theta=theta)
    torch.cuda.synchronize()
    got = wl.to_f32(to_host_bits(out), dtype)
    assert not np.isnan(got).any()
    k_after = to_host_bits(kd)
    if rope_mode == BZ_ROPE_NONE:
        ref = oracle.batch_prefill_ragged(q_full, k, v, dtype, kvp, Hq, Hkv, D, causal=causal, rows=rows, parallel=True)
    else:
        q_fed = prefill_q_as_fed(q_full, dtype, kvp, Hq, D, theta, prefill_angle_table(fws, int(kv_lens.max()), D))
        ref = oracle.batch_prefill_ragged(q_fed, k_after, v, dtype, kvp, Hq, Hkv, D, causal=causal, sm_scale=LN2, rows=rows,
                                          parallel=True)
    tol = ulp_tol(ref, dtype, before_rounding=PREFILL_BF16_WIDEN_V_ERR if mode == BZ_PREFILL_BF16_WIDEN_V else 0.0)
    assert (np.abs(got - ref) <= tol).all(), (case, float(np.abs(got - ref).max()))
