"""GPU parity: ragged (causal) prefill attention through the C ABI against the CPU checker.
Tolerance: max-abs <= 2e-3, widened to half a storage step where the storage grid is coarser than that (bf16
results >= 0.5).  bf16 runs in both of its modes: head + tail probabilities at that bar, V widened to f16 (the
default) with 5e-4 allowed before the final rounding (see _util.PREFILL_BF16_WIDEN_V_ERR).  Where the kernel
rotates q itself, the checker is given the q rows as the kernel feeds them to the matrix cores (rotated, scaled,
rounded once: _util.prefill_q_as_fed), so that no allowance for that rounding is needed."""
import numpy as np
import pytest
import torch

import oracle
from blitz_scale_amd import kernel as K
from blitz_scale_amd import workloads as wl
from blitz_scale_amd._lib import (BZ_BF16, BZ_F16, BZ_LAYOUT_HND, BZ_PREFILL_BF16_HEAD_TAIL, BZ_PREFILL_BF16_WIDEN_V,
                                  BZ_ROPE_FULL, BZ_ROPE_NONE, BZ_ROPE_Q_ONLY)

from _gpu import DeviceDecode, to_dev, to_host_bits
from _util import LN2, PREFILL_BF16_WIDEN_V_ERR, DecodeProblem, prefill_angle_table, prefill_q_as_fed, ulp_tol

# (storage type, bf16 mode) as the tests are parametrised
F16 = (BZ_F16, None)
BF16_WIDEN_V = (BZ_BF16, BZ_PREFILL_BF16_WIDEN_V)
BF16_HEAD_TAIL = (BZ_BF16, BZ_PREFILL_BF16_HEAD_TAIL)
KINDS = [F16, BF16_WIDEN_V, BF16_HEAD_TAIL]
KIND_IDS = ["f16", "bf16-widen-v", "bf16-head-tail"]


def kind_tol(ref, kind):
    dtype, mode = kind
    return ulp_tol(ref, dtype, before_rounding=PREFILL_BF16_WIDEN_V_ERR if mode == BZ_PREFILL_BF16_WIDEN_V else 0.0)

pytestmark = pytest.mark.gpu


class Prefill:
    def __init__(self, seed, lens, Hq, Hkv, D, dtype, bf16_mode=None):
        rng = np.random.default_rng(seed)
        self.lens, self.Hq, self.Hkv, self.D, self.dtype = lens, Hq, Hkv, D, dtype
        self.indptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        N = int(self.indptr[-1])
        self.q = wl.randn_bits(rng, (N, Hq, D), dtype)
        self.k = wl.randn_bits(rng, (N, Hkv, D), dtype)
        self.v = wl.randn_bits(rng, (N, Hkv, D), dtype)
        self.float_ws = torch.empty(1 << 20, dtype=torch.uint8, device="cuda")
        self.int_ws = torch.empty(8 << 20, dtype=torch.uint8, device="cuda")
        self.handler = K.BatchPrefillRaggedHandler()
        if bf16_mode is not None:
            self.handler.set_bf16_mode(bf16_mode)

    def run(self, causal=True, rope_mode=BZ_ROPE_NONE, theta=1e4):
        B = len(self.lens)
        self.handler.plan(self.float_ws, self.float_ws.numel(), self.int_ws, self.int_ws.numel(), self.indptr,
                          self.indptr, B, self.Hq, self.Hkv, self.D, 16)
        qd, kd, vd = to_dev(self.q, self.dtype), to_dev(self.k, self.dtype), to_dev(self.v, self.dtype)
        ip = torch.from_numpy(self.indptr).cuda()
        out = torch.full_like(qd, float("nan"))
        K.batch_prefill_attention(self.handler, qd, ip, kd, vd, ip, out, B, self.Hq, self.Hkv, self.D, causal=causal,
                                  rope_mode=rope_mode, rope_theta=theta)
        torch.cuda.synchronize()
        self.q_after, self.k_after = to_host_bits(qd), to_host_bits(kd)
        return wl.to_f32(to_host_bits(out), self.dtype)

    def q_as_fed(self, theta):
        """The q rows as the last run fed them to the matrix cores (it rotated them in registers)."""
        table = prefill_angle_table(self.float_ws, int(max(self.lens)), self.D)
        return prefill_q_as_fed(self.q, self.dtype, self.indptr, self.Hq, self.D, theta, table)


@pytest.mark.parametrize("kind", KINDS, ids=KIND_IDS)
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("Hq,Hkv", [(4, 4), (8, 2)])
def test_small_ragged_full_check(kind, causal, Hq, Hkv):
    dtype = kind[0]
    pf = Prefill(200 + Hq, [1, 7, 64, 65, 127, 128, 129, 300, 2, 31, 32, 33, 96], Hq, Hkv, 128, dtype, kind[1])
    got = pf.run(causal=causal)
    ref = oracle.batch_prefill_ragged(pf.q, pf.k, pf.v, dtype, pf.indptr, Hq, Hkv, 128, causal=causal, parallel=True)
    assert not np.isnan(got).any()
    assert (np.abs(got - ref) <= kind_tol(ref, kind)).all(), np.abs(got - ref).max()
    if dtype == BZ_F16:
        assert np.abs(got - ref).max() <= 2e-3


@pytest.mark.parametrize("kind", KINDS, ids=KIND_IDS)
@pytest.mark.parametrize("float_ws_bytes", [1 << 20, 1 << 10])
def test_rope_inside_the_call(kind, float_ws_bytes):
    """BZ_ROPE_FULL, the reference's kRoPELlama: k rows are rotated in place (the page store that follows
    copies them), q is rotated in registers from the angle table in the float workspace and stays untouched in
    memory -- unless the workspace has no room for the table (second case), then q is rotated in place too.
    BZ_ROPE_Q_ONLY on the rotated k gives the same output and touches nothing."""
    dtype = kind[0]
    theta = 1e4
    lens = [5, 200, 131, 1, 64]
    pf = Prefill(210, lens, 8, 4, 128, dtype, kind[1])
    pf.float_ws = torch.empty(float_ws_bytes, dtype=torch.uint8, device="cuda")
    got = pf.run(causal=True, rope_mode=BZ_ROPE_FULL, theta=theta)
    q_rot = oracle.rope_ragged(pf.q, dtype, pf.indptr, 8, 128, theta)
    k_rot = oracle.rope_ragged(pf.k, dtype, pf.indptr, 4, 128, theta)
    step = 2.0 ** -8 if dtype == BZ_F16 else 2.0 ** -5
    assert np.abs(wl.to_f32(pf.k_after, dtype) - wl.to_f32(k_rot, dtype)).max() <= step
    assert (pf.k_after != k_rot).mean() < 2e-3
    if float_ws_bytes >= 200 * 512:
        assert np.array_equal(pf.q_after, pf.q)  # q is read only
        # q rotated in registers: the checker gets the rows as they enter the matrix cores (rotated in fp32, scaled,
        # rounded once) and the k bits the device left behind -- the stated bar, for both storage types
        q_fed = pf.q_as_fed(theta)
        ref = oracle.batch_prefill_ragged(q_fed, pf.k_after, pf.v, dtype, pf.indptr, 8, 4, 128, causal=True,
                                          sm_scale=LN2, parallel=True)
    else:
        assert np.abs(wl.to_f32(pf.q_after, dtype) - wl.to_f32(q_rot, dtype)).max() <= step
        assert (pf.q_after != q_rot).mean() < 2e-3
        # attention over the rotated rows as the device left them in memory
        ref = oracle.batch_prefill_ragged(pf.q_after, pf.k_after, pf.v, dtype, pf.indptr, 8, 4, 128, causal=True, parallel=True)
    assert (np.abs(got - ref) <= kind_tol(ref, kind)).all(), np.abs(got - ref).max()
    # Sanity bound only (it catches a wrong angle or pairing, not a rounding): kRoPELlama on the raw rows with the
    # rotation in fp32 and NO rounding of q and k.  The rounding of the rotated rows to the storage type alone
    # moves the logits by ~1e-3 (f16) / ~1e-2 (bf16), which is what these bounds allow for.
    ref_raw = oracle.batch_prefill_ragged(pf.q, pf.k, pf.v, dtype, pf.indptr, 8, 4, 128, causal=True, rope=True,
                                          rope_theta=theta, parallel=True)
    assert np.abs(got - ref_raw).max() <= (2e-3 if dtype == BZ_F16 else 3e-2), np.abs(got - ref_raw).max()
    if float_ws_bytes >= 200 * 512:
        # q only: k as the first call left it
        pf2 = Prefill(210, lens, 8, 4, 128, dtype, kind[1])
        pf2.k = pf.k_after
        got2 = pf2.run(causal=True, rope_mode=BZ_ROPE_Q_ONLY, theta=theta)
        assert np.array_equal(got2, got)
        assert np.array_equal(pf2.q_after, pf2.q) and np.array_equal(pf2.k_after, pf2.k)


@pytest.mark.parametrize("kind", KINDS, ids=KIND_IDS)
@pytest.mark.parametrize("pattern", ["rising", "falling", "spikes"])
@pytest.mark.parametrize("rope_mode", [BZ_ROPE_NONE, BZ_ROPE_Q_ONLY])
def test_logits_with_a_large_dynamic_range(kind, pattern, rope_mode):
    """The kernel keeps one reference maximum per row and moves it only when a score exceeds it by 2^15 or more
    (probabilities are computed on that assumption first and again if it did not hold).  Here the K rows are
    scaled along the sequence so that the row maxima climb by far more than that from tile to tile (rising), sit
    in the first tile with everything after it far below (falling), or jump at a few isolated tokens (spikes);
    the logits span about +-40 in base-2 units."""
    dtype = kind[0]
    lens = [700, 130, 64, 1000]
    pf = Prefill(220, lens, 8, 2, 128, dtype, kind[1])
    rng = np.random.default_rng(221)
    k = wl.to_f32(pf.k, dtype)
    for b in range(len(lens)):
        lo, hi = int(pf.indptr[b]), int(pf.indptr[b + 1])
        pos = np.arange(hi - lo, dtype=np.float32) / max(1, hi - lo - 1)
        if pattern == "rising":
            scale = 0.5 + 7.5 * pos
        elif pattern == "falling":
            scale = 8.0 - 7.5 * pos
        else:
            scale = np.where(rng.random(hi - lo) < 0.02, 9.0, 0.7).astype(np.float32)
        k[lo:hi] *= scale[:, None, None]
    pf.k = wl.to_bits(k, dtype)
    got = pf.run(causal=True, rope_mode=rope_mode, theta=1e4)
    if rope_mode == BZ_ROPE_Q_ONLY:
        # the q rows as they enter the matrix cores (rotated, scaled, rounded once)
        q_fed = pf.q_as_fed(1e4)
        ref = oracle.batch_prefill_ragged(q_fed, pf.k, pf.v, dtype, pf.indptr, 8, 2, 128, causal=True, sm_scale=LN2,
                                          parallel=True)
    else:
        ref = oracle.batch_prefill_ragged(pf.q, pf.k, pf.v, dtype, pf.indptr, 8, 2, 128, causal=True, parallel=True)
    assert not np.isnan(got).any()
    err = np.abs(got - ref)
    # q and k enter the matrix cores with the bits the checker reads: the stated bar.  Rows that attend to a
    # single token reach |o| > 4 here, where half an f16 step is 1.95e-3 by itself; the probabilities enter
    # the second contraction rounded to 11 (bf16 head + tail: 16) significant bits, relative 2^-12, which is allowed
    # for on top.
    assert (err <= kind_tol(ref, kind) + 2.0 ** -12 * np.abs(ref)).all(), float(err.max())


def test_prefill_then_store_then_decode_is_consistent():
    """Row i of the prefill output equals a decode over the first i+1 cached tokens (GPU against GPU and
    against the checker): ties the three kernels of the path together."""
    dtype, Hq, Hkv, D, P = BZ_F16, 8, 2, 128, 16
    pf = Prefill(220, [77, 300], Hq, Hkv, D, dtype)
    got = pf.run(causal=True)
    for r, L in enumerate(pf.lens):
        p = DecodeProblem(221 + r, [L], Hq, Hkv, D, P, dtype)
        dev = DeviceDecode(p)
        s, e = pf.indptr[r], pf.indptr[r + 1]
        ri = torch.tensor([0, L], dtype=torch.int32, device="cuda")
        K.store_prefill_kv_cache(dev.pt, to_dev(pf.k[s:e], dtype), to_dev(pf.v[s:e], dtype), ri)
        dev.plan()
        dec = dev.decode(3, q=to_dev(pf.q[e - 1:e], dtype))
        assert np.abs(dec[0] - got[e - 1]).max() <= 2e-3


@pytest.mark.parametrize("batch", [4, 16])
def test_c4_shape_sampled_rows(batch):
    """Llama-2-13B-shaped prefill (40/40 heads, D 128, f16, lengths U[128,4096], causal); batch 16 is the
    full benchmark configuration 4.  The checker evaluates a seeded sample of rows (all heads) plus the first and
    last row of every request."""
    cfg = wl.CONFIGS["C4"]
    rng = np.random.default_rng(wl.DEFAULT_SEED)
    lens = [int(x) for x in rng.integers(128, 4097, size=batch)]
    pf = Prefill(wl.DEFAULT_SEED, lens, cfg["Hq"], cfg["Hkv"], cfg["D"], cfg["dtype"])
    got = pf.run(causal=True)
    N = int(pf.indptr[-1])
    rows = np.unique(np.concatenate([rng.integers(0, N, size=48), pf.indptr[:-1], pf.indptr[1:] - 1])).astype(np.int32)
    ref = oracle.batch_prefill_ragged(pf.q, pf.k, pf.v, cfg["dtype"], pf.indptr, cfg["Hq"], cfg["Hkv"], cfg["D"],
                                      causal=True, rows=rows, parallel=True)
    assert not np.isnan(got).any()
    assert np.abs(got[rows] - ref).max() <= 2e-3


def test_c4_one_whole_request_of_full_length():
    """benchmark configuration 4 at full size (16 prompts, 40/40 heads): EVERY row of the longest request (all heads)
    against the checker, i.e. every causal length from 1 to the request's end through every q tile and wave."""
    cfg = wl.CONFIGS["C4"]
    rng = np.random.default_rng(wl.DEFAULT_SEED)
    lens = [int(x) for x in rng.integers(128, 4097, size=16)]
    lens[5] = 4096  # one request at the maximum length
    pf = Prefill(wl.DEFAULT_SEED + 1, lens, cfg["Hq"], cfg["Hkv"], cfg["D"], cfg["dtype"])
    got = pf.run(causal=True)
    rows = np.arange(pf.indptr[5], pf.indptr[6], dtype=np.int32)
    assert len(rows) == 4096
    ref = oracle.batch_prefill_ragged(pf.q, pf.k, pf.v, cfg["dtype"], pf.indptr, cfg["Hq"], cfg["Hkv"], cfg["D"],
                                      causal=True, rows=rows, parallel=True)
    assert not np.isnan(got).any()
    assert np.abs(got[rows] - ref).max() <= 2e-3


def test_c4_rope_store_then_attention_at_full_size():
    """benchmark configuration 4 as the layer runs it (src/layer/attn.h:173-193 with this library's order of calls), at full
    size: 16 prompts U[128,4096], 40/40 heads, f16, RoPE theta 1e4, page size 16, seeded page placement with the
    reference's len+1 reservation.  store_prefill_kv_cache(rope = 2) rotates K into the pages and in the caller's
    rows, batch_prefill_attention(BZ_ROPE_Q_ONLY) rotates q in registers.  Checked: the pool against the checker's
    store with rotation; the k rows against the checker's rotation; the attention output, on a seeded sample of
    rows plus the first and last row of every request and EVERY row of one whole request, against the checker on
    the q rows as fed to the matrix cores (the stated bar) and, as a labelled sanity bound, against the checker's
    own kRoPELlama on the raw rows."""
    cfg = wl.CONFIGS["C4"]
    dtype, Hq, Hkv, D, P, theta = cfg["dtype"], cfg["Hq"], cfg["Hkv"], cfg["D"], cfg["P"], cfg["rope_theta"]
    rng = np.random.default_rng(wl.DEFAULT_SEED)
    lens = wl.ctx_lens_for(cfg, rng)
    assert len(lens) == 16 and lens.min() >= 128 and lens.max() <= 4096
    pf = Prefill(wl.DEFAULT_SEED + 2, [int(x) for x in lens], Hq, Hkv, D, dtype)
    N = int(pf.indptr[-1])
    need = int(((lens + 1 + P - 1) // P).sum())
    pool_pages = int(np.ceil(need * cfg["oversub"]))
    indices, pindptr, lpl = wl.page_table_for(lens + 1, P, pool_pages, rng)
    stride_page, stride_n, stride_h = wl.strides(BZ_LAYOUT_HND, Hkv, P, D)
    pool = torch.zeros(pool_pages * stride_page, dtype=torch.float16, device="cuda")
    pt = K.PageTable(len(lens), P, Hkv, D, pool, layout=BZ_LAYOUT_HND)
    pt.indices, pt.indptr, pt.last_page_len = indices, pindptr, lpl
    pt.upload()
    qd, kd, vd = to_dev(pf.q, dtype), to_dev(pf.k, dtype), to_dev(pf.v, dtype)
    ip = torch.from_numpy(pf.indptr).cuda()
    out = torch.full_like(qd, float("nan"))
    K.store_prefill_kv_cache(pt, kd, vd, ip, num_tokens=N, rope=2, rope_theta=theta)
    fw = torch.empty(4 << 20, dtype=torch.uint8, device="cuda")
    pf.handler.plan(fw, fw.numel(), pf.int_ws, pf.int_ws.numel(), pf.indptr, pf.indptr, len(lens), Hq, Hkv, D, P)
    K.batch_prefill_attention(pf.handler, qd, ip, kd, vd, ip, out, len(lens), Hq, Hkv, D, causal=True,
                              rope_mode=BZ_ROPE_Q_ONLY, rope_theta=theta)
    torch.cuda.synchronize()
    got = wl.to_f32(to_host_bits(out), dtype)
    k_after, pool_after = to_host_bits(kd), to_host_bits(pool)
    assert np.array_equal(to_host_bits(qd), pf.q)  # q is read only
    # -- the pool and the caller's k rows (the device's sincosf may differ from the host's in the last place)
    want_pool = np.zeros(pool_pages * stride_page, np.uint16)
    half = stride_page // 2
    kv = oracle.PagedKV(want_pool, want_pool[half:], indices, pindptr, lpl, P, Hkv, D, stride_page, stride_n, stride_h, dtype)
    oracle.store_prefill_kv(kv, pf.k, pf.v, dtype, pf.indptr, rope=True, rope_theta=theta)
    k_rot = oracle.rope_ragged(pf.k, dtype, pf.indptr, Hkv, D, theta)
    for g, w in ((pool_after, want_pool), (k_after, k_rot)):
        assert np.abs(wl.to_f32(g, dtype) - wl.to_f32(w, dtype)).max() <= 2.0 ** -8
        assert (g != w).mean() < 2e-3
    # -- attention: sampled rows, the ends of every request, one whole request
    b_whole = int(np.argmin(np.abs(lens - 1000)))  # a request of about a thousand tokens: every row, every head
    rows = np.unique(np.concatenate([rng.integers(0, N, size=48), pf.indptr[:-1], pf.indptr[1:] - 1,
                                     np.arange(pf.indptr[b_whole], pf.indptr[b_whole + 1])])).astype(np.int32)
    assert not np.isnan(got).any()
    q_fed = prefill_q_as_fed(pf.q, dtype, pf.indptr, Hq, D, theta, prefill_angle_table(fw, int(lens.max()), D))
    ref = oracle.batch_prefill_ragged(q_fed, k_after, pf.v, dtype, pf.indptr, Hq, Hkv, D, causal=True, sm_scale=LN2,
                                      rows=rows, parallel=True)
    assert np.abs(got[rows] - ref).max() <= 2e-3, float(np.abs(got[rows] - ref).max())
    # sanity bound only: rotation in fp32 without any rounding of q and k (the rounding of the rotated f16 rows
    # moves the result by about 1e-3)
    ref_raw = oracle.batch_prefill_ragged(pf.q, pf.k, pf.v, dtype, pf.indptr, Hq, Hkv, D, causal=True, rope=True,
                                          rope_theta=theta, rows=rows, parallel=True)
    assert np.abs(got[rows] - ref_raw).max() <= 3e-3, float(np.abs(got[rows] - ref_raw).max())


@pytest.mark.parametrize("kind", KINDS, ids=KIND_IDS)
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("rope_mode,float_ws_bytes", [(BZ_ROPE_NONE, 1 << 20), (BZ_ROPE_Q_ONLY, 1 << 20), (BZ_ROPE_FULL, 1 << 20),
                                                      (BZ_ROPE_FULL, 1 << 10)])
def test_q_rows_for_the_last_tokens_of_a_request_only(kind, causal, rope_mode, float_ws_bytes):
    """qo_indptr != kv_indptr (src/kernel/attention.h:9-22 carries both): every request brings K/V rows for all its
    tokens and q rows for the last ones only -- a chunk of a prompt attending to the whole prefix.  q row i sits at
    position kv_len - qo_len + i.  The result must be the rows of plain self-attention over the whole request that
    belong to those tokens, which is what the checker computes (the other q rows of its input are never looked at)."""
    dtype, theta, Hq, Hkv, D = kind[0], 1e4, 8, 2, 128
    kv_lens = np.array([300, 64, 129, 1000, 33, 5, 200, 257])
    q_lens = np.array([100, 64, 1, 37, 32, 5, 0, 130])  # offsets 200, 0, 128, 963 (not a multiple of a tile), 1, 0, -, 127
    kv_indptr = np.concatenate([[0], np.cumsum(kv_lens)]).astype(np.int32)
    qo_indptr = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32)
    rng = np.random.default_rng(260)
    Nkv, Nq, B = int(kv_indptr[-1]), int(qo_indptr[-1]), len(kv_lens)
    q_full = wl.randn_bits(rng, (Nkv, Hq, D), dtype)
    k = wl.randn_bits(rng, (Nkv, Hkv, D), dtype)
    v = wl.randn_bits(rng, (Nkv, Hkv, D), dtype)
    rows = np.concatenate([np.arange(kv_indptr[b + 1] - q_lens[b], kv_indptr[b + 1]) for b in range(B)]).astype(np.int32)
    q = q_full[rows]
    k_rot = oracle.rope_ragged(k, dtype, kv_indptr, Hkv, D, theta)
    k_in = k_rot if rope_mode == BZ_ROPE_Q_ONLY else k
    float_ws = torch.empty(float_ws_bytes, dtype=torch.uint8, device="cuda")
    int_ws = torch.empty(1 << 20, dtype=torch.uint8, device="cuda")
    handler = K.BatchPrefillRaggedHandler()
    if kind[1] is not None:
        handler.set_bf16_mode(kind[1])
    fb, ib = handler.workspace(qo_indptr, kv_indptr, B, Hq, Hkv, D)
    assert fb == 512 * 1000 and ib <= int_ws.numel()
    handler.plan(float_ws, float_ws.numel(), int_ws, int_ws.numel(), qo_indptr, kv_indptr, B, Hq, Hkv, D, 16)
    qd, kd, vd = to_dev(q, dtype), to_dev(k_in, dtype), to_dev(v, dtype)
    out = torch.full_like(qd, float("nan"))
    K.batch_prefill_attention(handler, qd, torch.from_numpy(qo_indptr).cuda(), kd, vd, torch.from_numpy(kv_indptr).cuda(), out,
                              B, Hq, Hkv, D, causal=causal, rope_mode=rope_mode, rope_theta=theta)
    torch.cuda.synchronize()
    got = wl.to_f32(to_host_bits(out), dtype)
    assert not np.isnan(got).any()
    assert np.array_equal(to_host_bits(vd), v)
    k_after = to_host_bits(kd)
    step = 2.0 ** -8 if dtype == BZ_F16 else 2.0 ** -5
    if rope_mode == BZ_ROPE_FULL:  # K rotated in place, every row at its own index
        assert np.abs(wl.to_f32(k_after, dtype) - wl.to_f32(k_rot, dtype)).max() <= step and (k_after != k_rot).mean() < 2e-3
    else:
        assert np.array_equal(k_after, k_in)
    table_fits = float_ws_bytes >= 512 * 1000
    if rope_mode == BZ_ROPE_NONE:
        assert np.array_equal(to_host_bits(qd), q)
        ref = oracle.batch_prefill_ragged(q_full, k, v, dtype, kv_indptr, Hq, Hkv, D, causal=causal, rows=rows, parallel=True)
    elif table_fits:
        assert np.array_equal(to_host_bits(qd), q)  # rotated in registers
        q_fed = prefill_q_as_fed(q_full, dtype, kv_indptr, Hq, D, theta, prefill_angle_table(float_ws, 1000, D))
        ref = oracle.batch_prefill_ragged(q_fed, k_after, v, dtype, kv_indptr, Hq, Hkv, D, causal=causal, sm_scale=LN2,
                                          rows=rows, parallel=True)
    else:  # no room for the table: q rotated in place, at the positions of its tokens
        q_rot = oracle.rope_ragged(q_full, dtype, kv_indptr, Hq, D, theta)[rows]
        q_after = to_host_bits(qd)
        assert np.abs(wl.to_f32(q_after, dtype) - wl.to_f32(q_rot, dtype)).max() <= step and (q_after != q_rot).mean() < 2e-3
        q_full_after = q_full.copy()
        q_full_after[rows] = q_after
        ref = oracle.batch_prefill_ragged(q_full_after, k_after, v, dtype, kv_indptr, Hq, Hkv, D, causal=causal, rows=rows,
                                          parallel=True)
    assert (np.abs(got - ref) <= kind_tol(ref, kind)).all(), np.abs(got - ref).max()


def test_a_batch_without_q_rows_still_rotates_k():
    """BZ_ROPE_FULL promises rotated k rows in the caller's buffer (the page store that follows copies them), also
    when no request of the batch has a q row."""
    rng = np.random.default_rng(270)
    kv_lens, Hq, Hkv, D, dtype, theta = [5, 70], 4, 2, 128, BZ_F16, 1e4
    kvp = np.concatenate([[0], np.cumsum(kv_lens)]).astype(np.int32)
    qop = np.zeros(3, np.int32)
    k, v = wl.randn_bits(rng, (75, Hkv, D), dtype), wl.randn_bits(rng, (75, Hkv, D), dtype)
    fws = torch.empty(1 << 20, dtype=torch.uint8, device="cuda")
    iws = torch.empty(1 << 20, dtype=torch.uint8, device="cuda")
    h = K.BatchPrefillRaggedHandler()
    h.plan(fws, fws.numel(), iws, iws.numel(), qop, kvp, 2, Hq, Hkv, D, 16)
    qd = torch.zeros((1, Hq, D), dtype=torch.float16, device="cuda")  # (a valid pointer; no row is read)
    kd, vd = to_dev(k, dtype), to_dev(v, dtype)
    K.batch_prefill_attention(h, qd, torch.from_numpy(qop).cuda(), kd, vd, torch.from_numpy(kvp).cuda(), qd.clone(), 2, Hq, Hkv,
                              D, causal=True, rope_mode=BZ_ROPE_FULL, rope_theta=theta)
    torch.cuda.synchronize()
    k_rot = oracle.rope_ragged(k, dtype, kvp, Hkv, D, theta)
    got = to_host_bits(kd)
    assert np.abs(wl.to_f32(got, dtype) - wl.to_f32(k_rot, dtype)).max() <= 2.0 ** -8 and (got != k_rot).mean() < 2e-3


def test_fewer_kv_rows_than_q_rows_is_refused():
    h = K.BatchPrefillRaggedHandler()
    with pytest.raises(K.BzError, match="Handler workspace"):
        h.workspace(np.array([0, 10], np.int32), np.array([0, 9], np.int32), 1, 4, 4, 128)


def test_prefill_error_codes():
    pf = Prefill(230, [5], 4, 4, 128, BZ_F16)
    qd = to_dev(pf.q, BZ_F16)
    ip = torch.from_numpy(pf.indptr).cuda()
    with pytest.raises(K.BzError, match="BatchPrefillWithRaggedKVCache error"):
        K.batch_prefill_attention(pf.handler, qd, ip, qd, qd, ip, qd, 1, 4, 4, 128)  # not planned
    with pytest.raises(K.BzError, match="Handler plan"):
        pf.handler.plan(pf.float_ws, 1, pf.int_ws, 1, pf.indptr, pf.indptr, 1, 4, 4, 64, 16)  # head_dim 64
