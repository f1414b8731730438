"""GPU parity: ragged (causal) prefill attention through the C ABI against the CPU checker.
Tolerance: max-abs <= 2e-3 for f16 (widened to half a storage step for bf16 results >= 0.5)."""
import numpy as np
import pytest
import torch

import oracle
from blitz_scale_amd import kernel as K
from blitz_scale_amd import workloads as wl
from blitz_scale_amd._lib import BZ_BF16, BZ_F16, BZ_LAYOUT_HND, BZ_ROPE_FULL, BZ_ROPE_NONE, BZ_ROPE_Q_ONLY

from _gpu import DeviceDecode, to_dev, to_host_bits
from _util import DecodeProblem, ulp_tol

pytestmark = pytest.mark.gpu


class Prefill:
    def __init__(self, seed, lens, Hq, Hkv, D, dtype):
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


@pytest.mark.parametrize("dtype", [BZ_F16, BZ_BF16])
@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("Hq,Hkv", [(4, 4), (8, 2)])
def test_small_ragged_full_check(dtype, causal, Hq, Hkv):
    pf = Prefill(200 + Hq, [1, 7, 64, 65, 127, 128, 129, 300, 2], Hq, Hkv, 128, dtype)
    got = pf.run(causal=causal)
    ref = oracle.batch_prefill_ragged(pf.q, pf.k, pf.v, dtype, pf.indptr, Hq, Hkv, 128, causal=causal, parallel=True)
    assert not np.isnan(got).any()
    assert (np.abs(got - ref) <= ulp_tol(ref, dtype)).all(), np.abs(got - ref).max()
    if dtype == BZ_F16:
        assert np.abs(got - ref).max() <= 2e-3


@pytest.mark.parametrize("dtype", [BZ_F16, BZ_BF16])
@pytest.mark.parametrize("float_ws_bytes", [1 << 20, 1 << 10])
def test_rope_inside_the_call(dtype, float_ws_bytes):
    """BZ_ROPE_FULL, the reference's kRoPELlama: k rows are rotated in place (the page store that follows
    copies them), q is rotated in registers from the angle table in the float workspace and stays untouched in
    memory -- unless the workspace has no room for the table (second case), then q is rotated in place too.
    BZ_ROPE_Q_ONLY on the rotated k gives the same output and touches nothing."""
    theta = 1e4
    pf = Prefill(210, [5, 200, 131, 1, 64], 8, 4, 128, dtype)
    pf.float_ws = torch.empty(float_ws_bytes, dtype=torch.uint8, device="cuda")
    got = pf.run(causal=True, rope_mode=BZ_ROPE_FULL, theta=theta)
    q_rot = oracle.rope_ragged(pf.q, dtype, pf.indptr, 8, 128, theta)
    k_rot = oracle.rope_ragged(pf.k, dtype, pf.indptr, 4, 128, theta)
    step = 2.0 ** -8 if dtype == BZ_F16 else 2.0 ** -5
    assert np.abs(wl.to_f32(pf.k_after, dtype) - wl.to_f32(k_rot, dtype)).max() <= step
    assert (pf.k_after != k_rot).mean() < 2e-3
    if float_ws_bytes >= 200 * 512:
        assert np.array_equal(pf.q_after, pf.q)  # q is read only
    else:
        assert np.abs(wl.to_f32(pf.q_after, dtype) - wl.to_f32(q_rot, dtype)).max() <= step
        assert (pf.q_after != q_rot).mean() < 2e-3
    if float_ws_bytes >= 200 * 512:
        # q rotated in registers (fp32, rounded once together with the softmax scale): the checker rotates q in
        # fp32 as well and reads the k bits the device left behind
        ref = oracle.batch_prefill_ragged(pf.q, pf.k_after, pf.v, dtype, pf.indptr, 8, 4, 128, causal=True, rope="q",
                                          rope_theta=theta, parallel=True)
        # (for bf16 the one rounding of the rotated, scaled q row to 8 significant bits moves the logits by up
        # to ~1e-2; the same holds for any kernel that feeds bf16 operands to the matrix cores)
        assert np.abs(got - ref).max() <= (2e-3 if dtype == BZ_F16 else 2e-2), np.abs(got - ref).max()
    else:
        # attention over the rotated rows as the device left them in memory
        ref = oracle.batch_prefill_ragged(pf.q_after, pf.k_after, pf.v, dtype, pf.indptr, 8, 4, 128, causal=True, parallel=True)
        assert (np.abs(got - ref) <= ulp_tol(ref, dtype)).all(), np.abs(got - ref).max()
    # and against kRoPELlama on the raw rows (rotation in fp32, no rounding of q and k).  For f16 the same bar;
    # for bf16 the rounding of the rotated rows to 8 significant bits alone moves the logits by ~1e-2, which is
    # why K is compared on the bits as cached above (the bound here only catches a wrong angle or pairing)
    ref_raw = oracle.batch_prefill_ragged(pf.q, pf.k, pf.v, dtype, pf.indptr, 8, 4, 128, causal=True, rope=True,
                                          rope_theta=theta, parallel=True)
    assert np.abs(got - ref_raw).max() <= (2e-3 if dtype == BZ_F16 else 3e-2), np.abs(got - ref_raw).max()
    if float_ws_bytes >= 200 * 512:
        # q only: k as the first call left it
        pf2 = Prefill(210, [5, 200, 131, 1, 64], 8, 4, 128, dtype)
        pf2.k = pf.k_after
        got2 = pf2.run(causal=True, rope_mode=BZ_ROPE_Q_ONLY, theta=theta)
        assert np.array_equal(got2, got)
        assert np.array_equal(pf2.q_after, pf2.q) and np.array_equal(pf2.k_after, pf2.k)


@pytest.mark.parametrize("dtype", [BZ_F16, BZ_BF16])
@pytest.mark.parametrize("pattern", ["rising", "falling", "spikes"])
@pytest.mark.parametrize("rope_mode", [BZ_ROPE_NONE, BZ_ROPE_Q_ONLY])
def test_logits_with_a_large_dynamic_range(dtype, pattern, rope_mode):
    """The kernel keeps one reference maximum per row and moves it only when a score exceeds it by 2^15 or more
    (probabilities are computed on that assumption first and again if it did not hold).  Here the K rows are
    scaled along the sequence so that the row maxima climb by far more than that from tile to tile (rising), sit
    in the first tile with everything after it far below (falling), or jump at a few isolated tokens (spikes);
    the logits span about +-40 in base-2 units."""
    lens = [700, 130, 64, 1000]
    pf = Prefill(220, lens, 8, 2, 128, dtype)
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
    ref = oracle.batch_prefill_ragged(pf.q, pf.k, pf.v, dtype, pf.indptr, 8, 2, 128, causal=True,
                                      rope="q" if rope_mode == BZ_ROPE_Q_ONLY else False, rope_theta=1e4, parallel=True)
    assert not np.isnan(got).any()
    err = np.abs(got - ref)
    if rope_mode == BZ_ROPE_NONE:
        # q and k enter the matrix cores with the bits the checker reads: the stated bar.  Rows that attend to a
        # single token reach |o| > 4 here, where half an f16 step is 1.95e-3 by itself; the probabilities enter
        # the second contraction rounded to f16 (relative 2^-12), which is allowed for on top.
        assert (err <= ulp_tol(ref, dtype) + 2.0 ** -12 * np.abs(ref)).all(), float(err.max())
    else:
        # the rotated q row is rounded to the storage type on its way into the matrix cores (the checker keeps it
        # in fp32): a logit of magnitude 30 moves by 30 * 2^-12 (f16) or 30 * 2^-9 (bf16), and the output with
        # it; the bounds catch a wrong maximum or a lost tile, which show up as errors of order one or NaN
        big, med = (2e-2, 2e-3) if dtype == BZ_F16 else (0.35, 2e-2)
        assert err.max() <= big and np.median(err) <= med, (float(err.max()), float(np.median(err)))


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
    full BASELINE config 4.  The checker evaluates a seeded sample of rows (all heads) plus the first and
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
    """BASELINE config 4 at full size (16 prompts, 40/40 heads): EVERY row of the longest request (all heads)
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


def test_prefill_error_codes():
    pf = Prefill(230, [5], 4, 4, 128, BZ_F16)
    qd = to_dev(pf.q, BZ_F16)
    ip = torch.from_numpy(pf.indptr).cuda()
    with pytest.raises(K.BzError, match="BatchPrefillWithRaggedKVCache error"):
        K.batch_prefill_attention(pf.handler, qd, ip, qd, qd, ip, qd, 1, 4, 4, 128)  # not planned
    with pytest.raises(K.BzError, match="Handler plan"):
        pf.handler.plan(pf.float_ws, 1, pf.int_ws, 1, pf.indptr, pf.indptr, 1, 4, 4, 64, 16)  # head_dim 64
