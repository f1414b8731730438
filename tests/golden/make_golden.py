"""Writes tests/golden/c1_decode.npz: benchmark configuration 1 (fp16, batch 4, 4/4 heads, D 64, P 16,
ctx {17,64,130,255}, 64-page pool, scale 1/8, no RoPE) generated from the seeded workload generator,
with the CPU checker's fp32 output and digests of the input bits.  The reference holds no numeric
vectors for this path, so this fixture pins the generator and the checker against drift; the GPU
result is compared with it as well.  Run from the repo root: python tests/golden/make_golden.py"""
import hashlib
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import oracle  # noqa: E402
from blitz_scale_amd import workloads as wl  # noqa: E402
from _util import DecodeProblem  # noqa: E402


def c1_problem():
    cfg = wl.CONFIGS["C1"]
    return DecodeProblem(wl.DEFAULT_SEED, cfg["ctx"], cfg["Hq"], cfg["Hkv"], cfg["D"], cfg["P"], cfg["dtype"],
                         pool_pages=cfg["pool_pages"])


def digest(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


if __name__ == "__main__":
    p = c1_problem()
    out, lse = oracle.batch_decode(p.q, p.dtype, p.oracle_kv(), p.Hq, want_lse=True)
    np.savez(os.path.join(ROOT, "tests", "golden", "c1_decode.npz"), out=out, lse=lse, indices=p.indices,
             indptr=p.indptr, last_page_len=p.last_page_len, q=p.q, pool_sha256=digest(p.pool), q_sha256=digest(p.q))
    print("wrote c1_decode.npz", out.shape, digest(p.pool)[:16])
