"""GPU parity of the one-call decode step (bz_append_and_decode): same pool contents and same attention
output as the checker's append followed by its decode, and as the library's own two-call sequence.

Tolerances: attention output max-abs <= 2e-3 (f16/bf16, widened to half a storage step where the
result is stored in bf16 and |o| >= 0.5); appended rows equal to the checker's except for rotated
elements that land within half a unit of a rounding boundary (at most one storage step, rare), as in
the append tests; untouched pool elements and q bit-exact.
"""
import numpy as np
import pytest
import torch

import oracle
from blitz_scale_amd import kernel as K
from blitz_scale_amd import workloads as wl
from blitz_scale_amd._lib import BZ_BF16, BZ_F16, BZ_LAYOUT_HND, BZ_LAYOUT_NHD, BZ_ROPE_NONE

from _gpu import TORCH_OF, DeviceDecode, to_dev, to_host_bits
from _util import DecodeProblem, ulp_tol

pytestmark = pytest.mark.gpu


def run_case(ctx, Hq, Hkv, D, P, dtype, layout=BZ_LAYOUT_HND, rope=True, theta=5e5, split_tokens=0, seed=77):
    rng = np.random.default_rng(seed)
    p = DecodeProblem(seed + 1, ctx, Hq, Hkv, D, P, dtype, layout=layout)
    B = p.B
    k_new, v_new = wl.randn_bits(rng, (B, Hkv, D), dtype), wl.randn_bits(rng, (B, Hkv, D), dtype)
    # the checker: append (K rotated), q rotated, attention without further rotation
    want_pool = p.pool.copy()
    kv = p.oracle_kv(want_pool)
    oracle.append_decode_kv(kv, k_new, v_new, dtype, rope=rope, rope_theta=theta)
    want_q = oracle.rope_decode_q(p.q, dtype, kv, Hq, theta) if rope else p.q
    ref = oracle.batch_decode(want_q, dtype, kv, Hq, rope_mode=BZ_ROPE_NONE)
    # the library, one call
    dev = DeviceDecode(p)
    info = dev.plan(split_tokens)
    out = torch.full((B, Hq, D), float("nan"), dtype=TORCH_OF[dtype], device="cuda")
    kd, vd = to_dev(k_new, dtype), to_dev(v_new, dtype)
    K.append_and_decode_attention(dev.handler, dev.q, dev.pt, kd, vd, out, Hq, rope=rope, rope_theta=theta)
    torch.cuda.synchronize()
    got, got_pool = out.float().cpu().numpy(), to_host_bits(dev.pool)
    assert np.array_equal(to_host_bits(dev.q), p.q), "q must not be modified"
    live = p.ctx > 0
    err = np.abs(got - ref)
    assert (err[live] <= ulp_tol(ref, dtype, 2e-3)[live]).all(), f"max abs err {err[live].max()}"
    assert not got[~live].any()
    gf, wf = wl.to_f32(got_pool, dtype), wl.to_f32(want_pool, dtype)
    assert np.abs(gf - wf).max() <= 2.0 ** -6
    assert (got_pool != want_pool).mean() < 2e-3
    changed = got_pool != p.pool
    assert 0 < changed.sum() <= 2 * live.sum() * Hkv * D
    # the library, two calls, on a fresh copy of the same pool
    dev2 = DeviceDecode(p)
    dev2.plan(split_tokens)
    q2 = dev2.q.clone()
    out2 = torch.empty_like(out)
    K.append_decode_kv_cache(dev2.pt, kd, vd, q=q2, num_qo_heads=Hq, rope=rope, rope_theta=theta)
    K.batch_decode_attention(dev2.handler, q2, dev2.pt, out2, Hq, rope_mode=BZ_ROPE_NONE)
    torch.cuda.synchronize()
    assert np.array_equal(to_host_bits(dev2.pool), got_pool), "one call and two calls leave different pools"
    d = np.abs(out2.float().cpu().numpy() - got)[live]
    assert d.max() <= 2e-3
    return info


@pytest.mark.parametrize("dtype", [BZ_BF16, BZ_F16])
def test_fused_step_matches_append_then_decode(dtype):
    """MFMA kernel: contexts whose last token sits at every interesting place of a 32-token tile and of a
    16-token page (first slot of a fresh page, last slot, tile boundary), GQA 4:1."""
    ctx = [1, 2, 16, 17, 31, 32, 33, 48, 49, 64, 65, 300, 1000, 1023, 1024, 1025]
    run_case(ctx, 32, 8, 128, 16, dtype)


def test_fused_step_with_split_sequences_and_empty_ones():
    info = run_case([5000, 0, 17, 2049, 640, 0, 8192, 4097], 32, 8, 128, 16, BZ_BF16, split_tokens=2048)
    assert info["split_seqs"] >= 3


@pytest.mark.parametrize("layout", [BZ_LAYOUT_HND, BZ_LAYOUT_NHD])
def test_fused_step_mha_page_64_both_layouts(layout):
    run_case([63, 64, 65, 129, 700], 8, 8, 128, 64, BZ_F16, layout=layout, theta=1e4)


def test_fused_step_without_rope():
    run_case([40, 333, 2100], 16, 4, 128, 16, BZ_BF16, rope=False)


def test_fused_step_falls_back_where_the_mfma_kernel_does_not_apply():
    """head_dim 64 and page size 8: the call makes the two launches itself, same results."""
    run_case([17, 64, 130, 255], 4, 4, 64, 16, BZ_F16, theta=1e4)
    run_case([9, 100], 8, 2, 128, 8, BZ_F16, theta=1e4)
