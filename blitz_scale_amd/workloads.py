"""Seeded synthetic workloads of the benchmark configurations (numpy on the host).

Everything is generated as storage bits (uint16 for f16/bf16, uint8 for e4m3) so that the HIP
path and any checker read bit-identical inputs.  Values are i.i.d. N(0,1) drawn in fp32 and
rounded to nearest-even; page placement is a seeded permutation of the pool.
"""
import numpy as np

from ._lib import BZ_BF16, BZ_E4M3, BZ_F16, BZ_F32, BZ_LAYOUT_HND, BZ_LAYOUT_NHD

DEFAULT_SEED = 0x5EED


# ---- storage conversions (numpy) -----------------------------------------------------------
def f32_to_bf16_bits(x):
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    r = 0x7FFF + ((u >> 16) & 1)
    return ((u + r) >> 16).astype(np.uint16)


def bf16_bits_to_f32(b):
    return (np.ascontiguousarray(b, np.uint16).astype(np.uint32) << 16).view(np.float32)


def f32_to_f16_bits(x):
    return np.ascontiguousarray(x, np.float32).astype(np.float16).view(np.uint16)


def f16_bits_to_f32(b):
    return np.ascontiguousarray(b, np.uint16).view(np.float16).astype(np.float32)


def _e4m3_table():
    codes = np.arange(127)
    e, m = codes >> 3, codes & 7
    return np.where(e == 0, m / 8.0 * 2.0 ** -6, (1 + m / 8.0) * 2.0 ** (e.astype(np.float64) - 7)).astype(np.float32)


_E4M3_POS = _e4m3_table()  # value of codes 0x00..0x7e (0x7f is NaN)


def e4m3_bits_to_f32(b):
    b = np.ascontiguousarray(b, np.uint8)
    mag = b & 0x7F
    v = np.where(mag == 0x7F, np.float32(np.nan), _E4M3_POS[np.minimum(mag, 126)])
    return np.where(b & 0x80, -v, v).astype(np.float32)


def f32_to_e4m3_bits(x):
    """OCP e4m3fn, round-to-nearest-even, saturating at +-448."""
    x = np.ascontiguousarray(x, np.float32)
    a = np.minimum(np.abs(x), np.float32(448.0))
    lo = np.searchsorted(_E4M3_POS, a, side="right") - 1
    hi = np.minimum(lo + 1, 126)
    dlo, dhi = a - _E4M3_POS[lo], _E4M3_POS[hi] - a
    pick = np.where(dlo < dhi, lo, np.where(dhi < dlo, hi, np.where(lo & 1, hi, lo)))
    return (pick | np.where(np.signbit(x), 0x80, 0)).astype(np.uint8)


def to_bits(x, dtype):
    return {BZ_F16: f32_to_f16_bits, BZ_BF16: f32_to_bf16_bits, BZ_E4M3: f32_to_e4m3_bits}[dtype](x)


def to_f32(bits, dtype):
    if dtype == BZ_F32:
        return np.asarray(bits, np.float32)
    return {BZ_F16: f16_bits_to_f32, BZ_BF16: bf16_bits_to_f32, BZ_E4M3: e4m3_bits_to_f32}[dtype](bits)


def randn_bits(rng, shape, dtype, mean=0.0, std=1.0):
    return to_bits((rng.standard_normal(shape, dtype=np.float32) * np.float32(std) + np.float32(mean)), dtype)


# ---- page tables -----------------------------------------------------------------------------
def strides(layout, num_kv_heads, page_size, head_dim):
    """(stride_page, stride_n, stride_h) in elements; stride_page = 2*H*P*D for both layouts."""
    sp = 2 * num_kv_heads * page_size * head_dim
    if layout == BZ_LAYOUT_HND:
        return sp, head_dim, page_size * head_dim
    return sp, num_kv_heads * head_dim, head_dim


def page_table_for(ctx_lens, page_size, pool_pages, rng):
    """CSR page table with pages placed at a seeded random permutation of the pool."""
    ctx_lens = np.asarray(ctx_lens, np.int64)
    npages = (ctx_lens + page_size - 1) // page_size
    indptr = np.zeros(len(ctx_lens) + 1, np.int32)
    indptr[1:] = np.cumsum(npages)
    total = int(indptr[-1])
    if total > pool_pages:
        raise ValueError(f"{total} pages needed, pool has {pool_pages}")
    indices = rng.permutation(pool_pages)[:total].astype(np.int32)
    last_page_len = np.where(ctx_lens > 0, ctx_lens - (npages - 1) * page_size, 0).astype(np.int32)
    return indices, indptr, last_page_len


def lognormal_ctx(rng, batch, mean=1024.0, sigma=1.0, lo=64, hi=8192):
    """Context lengths exp(mu + sigma z), mu = ln(mean) - sigma^2/2, rounded and clipped to [lo, hi]."""
    mu = np.log(mean) - sigma * sigma / 2
    z = rng.standard_normal(batch)
    return np.clip(np.rint(np.exp(mu + sigma * z)), lo, hi).astype(np.int64)


# ---- the benchmark configurations (the target file's `configs`, in order) -----------------------
CONFIGS = {
    "C1": dict(kind="decode", dtype=BZ_F16, kv_dtype=BZ_F16, batch=4, Hq=4, Hkv=4, D=64, P=16, pool_pages=64,
               ctx=[17, 64, 130, 255], rope_theta=None),
    "C2": dict(kind="decode", dtype=BZ_F16, kv_dtype=BZ_F16, batch=64, Hq=32, Hkv=32, D=128, P=16, oversub=1.25,
               ctx=("uniform", 512, 2048), rope_theta=1e4, hidden=4096, inter=11008),
    "C3": dict(kind="decode", dtype=BZ_BF16, kv_dtype=BZ_BF16, batch=128, Hq=32, Hkv=8, D=128, P=16, oversub=2.0,
               ctx=("lognormal", 1024.0, 1.0, 64, 8192), rope_theta=5e5, split_tokens=2048),
    "C4": dict(kind="prefill", dtype=BZ_F16, kv_dtype=BZ_F16, batch=16, Hq=40, Hkv=40, D=128, P=16, oversub=1.25,
               ctx=("uniform", 128, 4096), rope_theta=1e4),
    "C5": dict(kind="decode", dtype=BZ_BF16, kv_dtype=BZ_E4M3, batch=256, Hq=64, Hkv=8, D=128, P=16, oversub=1.0,
               ctx=("const", 4096), rope_theta=None),
}


def ctx_lens_for(cfg, rng):
    c = cfg["ctx"]
    if isinstance(c, list):
        return np.asarray(c, np.int64)
    if c[0] == "uniform":
        return rng.integers(c[1], c[2] + 1, size=cfg["batch"]).astype(np.int64)
    if c[0] == "lognormal":
        return lognormal_ctx(rng, cfg["batch"], c[1], c[2], c[3], c[4])
    if c[0] == "const":
        return np.full(cfg["batch"], c[1], np.int64)
    raise ValueError(c)


def pool_pages_for(cfg, ctx_lens):
    if "pool_pages" in cfg:
        return cfg["pool_pages"]
    need = int(((np.asarray(ctx_lens) + cfg["P"] - 1) // cfg["P"]).sum())
    return int(np.ceil(need * cfg.get("oversub", 1.0)))


def decode_algorithmic_bytes(ctx_lens, Hq, Hkv, D, kv_bytes, q_bytes, page_size):
    """Bytes one decode step has to move: every K and V row once per kv head, q in, o out, the page
    table, and the new token's K,V row written by the append."""
    ctx = np.asarray(ctx_lens, np.int64)
    B = len(ctx)
    nnz = int(((ctx + page_size - 1) // page_size).sum())
    kv = int(ctx.sum()) * 2 * Hkv * D * kv_bytes
    qo = 2 * B * Hq * D * q_bytes
    table = 4 * (nnz + 2 * B + 1)
    new = 2 * B * Hkv * D * kv_bytes
    return kv + qo + table + new
