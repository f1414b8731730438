"""GPU parity: RMSNorm, add+RMSNorm, SiLU-gate and residual add against the CPU checker.
f16 results are held to 2e-3 max-abs; bf16 results to 2e-3 or half a bf16 step where that is
larger; the residual add is bit-exact (one rounding)."""
import numpy as np
import pytest
import torch

import oracle
from blitz_scale_amd import kernel as K
from blitz_scale_amd import workloads as wl
from blitz_scale_amd._lib import BZ_BF16, BZ_F16

from _gpu import to_dev, to_host_bits
from _util import ulp_tol

pytestmark = pytest.mark.gpu


def _close(got_bits, ref_f32, dtype):
    got = wl.to_f32(got_bits, dtype)
    assert (np.abs(got - ref_f32) <= ulp_tol(ref_f32, dtype)).all(), np.abs(got - ref_f32).max()


@pytest.mark.parametrize("dtype", [BZ_F16, BZ_BF16])
@pytest.mark.parametrize("N,h", [(64, 4096), (1, 4096), (7, 5120), (3, 8192), (5, 256), (2, 11008)])
def test_rms_norm(dtype, N, h):
    rng = np.random.default_rng(60 + N)
    x, w = wl.randn_bits(rng, (N, h), dtype), wl.randn_bits(rng, (h,), dtype, mean=1.0, std=0.02)
    ref = oracle.rms_norm(x, w, dtype, 1e-5)
    xd, wd = to_dev(x, dtype), to_dev(w, dtype)
    out = torch.empty_like(xd)
    K.rms_norm(xd, wd, out, N, h)
    torch.cuda.synchronize()
    _close(to_host_bits(out), ref, dtype)
    if dtype == BZ_F16:
        assert np.abs(wl.to_f32(to_host_bits(out), dtype) - ref).max() <= 2e-3
    K.rms_norm(xd, wd, xd, N, h)  # in place, as the final norm is called (src/model/llama.h:389-391)
    torch.cuda.synchronize()
    assert np.array_equal(to_host_bits(xd), to_host_bits(out))


@pytest.mark.parametrize("dtype", [BZ_F16, BZ_BF16])
@pytest.mark.parametrize("N,h", [(64, 4096), (3, 5120)])
def test_add_rms_norm(dtype, N, h):
    rng = np.random.default_rng(70)
    x, r = wl.randn_bits(rng, (N, h), dtype), wl.randn_bits(rng, (N, h), dtype)
    w = wl.randn_bits(rng, (h,), dtype, mean=1.0, std=0.02)
    ref, ref_res = oracle.add_rms_norm(x, r, w, dtype)
    xd, rd, wd = to_dev(x, dtype), to_dev(r, dtype), to_dev(w, dtype)
    K.add_rms_norm(xd, rd, wd, N, h)
    torch.cuda.synchronize()
    assert np.array_equal(to_host_bits(rd), ref_res)  # residual += input: same single fp32 add, same rounding
    _close(to_host_bits(xd), ref, dtype)


@pytest.mark.parametrize("dtype", [BZ_F16, BZ_BF16])
@pytest.mark.parametrize("N,I", [(64, 11008), (1, 14336), (5, 8)])
def test_silu_and_mul(dtype, N, I):
    rng = np.random.default_rng(80)
    x = wl.randn_bits(rng, (N, 2 * I), dtype)
    ref = oracle.silu_and_mul(x, dtype)
    # output sits right before the input in one workspace, as in src/layer/glu.h:92-96
    ws = torch.empty(N * I + N * 2 * I, dtype=to_dev(x[:1, :8], dtype).dtype, device="cuda")
    out, inp = ws[:N * I], ws[N * I:]
    inp.copy_(to_dev(x, dtype).reshape(-1))
    K.silu_and_mul(inp, out, N, I)
    torch.cuda.synchronize()
    _close(to_host_bits(out).reshape(N, I), ref, dtype)
    assert np.array_equal(to_host_bits(inp).reshape(N, 2 * I), x)


@pytest.mark.parametrize("dtype", [BZ_F16, BZ_BF16])
def test_add_residual_bit_exact(dtype):
    rng = np.random.default_rng(90)
    N, h = 64, 4096
    a = wl.to_bits((rng.standard_normal((N, h)) * np.exp(rng.uniform(-10, 6, (N, h)))).astype(np.float32), dtype)
    b = wl.to_bits((rng.standard_normal((N, h)) * np.exp(rng.uniform(-10, 6, (N, h)))).astype(np.float32), dtype)
    want = oracle.add_residual(a, b, dtype)
    ad, bd = to_dev(a, dtype), to_dev(b, dtype)
    K.add_residual(ad, bd, N, h)
    torch.cuda.synchronize()
    assert np.array_equal(to_host_bits(bd), want)
    assert np.array_equal(to_host_bits(ad), a)
