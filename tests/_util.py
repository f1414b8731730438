"""Shared helpers for the tests: small problem builders on top of blitz_scale_amd.workloads and an
independent float64 dense attention used to pin the checker."""
import numpy as np

import oracle
from blitz_scale_amd import workloads as wl
from blitz_scale_amd._lib import BZ_BF16, BZ_E4M3, BZ_F16, BZ_LAYOUT_HND, BZ_LAYOUT_NHD


class DecodeProblem:
    """Host image of one decode step: q bits, one pool plane (bits), page table."""

    def __init__(self, seed, ctx, Hq, Hkv, D, P, dtype, kv_dtype=None, layout=BZ_LAYOUT_HND, pool_pages=None,
                 oversub=1.5, kv_std=1.0):
        kv_dtype = dtype if kv_dtype is None else kv_dtype
        rng = np.random.default_rng(seed)
        self.ctx = np.asarray(ctx, np.int64)
        self.B, self.Hq, self.Hkv, self.D, self.P = len(self.ctx), Hq, Hkv, D, P
        self.dtype, self.kv_dtype, self.layout = dtype, kv_dtype, layout
        need = int(((self.ctx + P - 1) // P).sum())
        self.pool_pages = pool_pages or max(1, int(np.ceil(need * oversub)))
        self.indices, self.indptr, self.last_page_len = wl.page_table_for(self.ctx, P, self.pool_pages, rng)
        self.stride_page, self.stride_n, self.stride_h = wl.strides(layout, Hkv, P, D)
        self.q = wl.randn_bits(rng, (self.B, Hq, D), dtype)
        self.k_scale = self.v_scale = None
        if kv_dtype == BZ_E4M3:
            # N(0,1) values, per-kv-head scale amax/448 (taken over the whole plane), then e4m3
            raw = rng.standard_normal((self.pool_pages, 2, Hkv, P, D), dtype=np.float32) * np.float32(kv_std)
            amax = np.abs(raw).max(axis=(0, 3, 4))  # [2, Hkv]
            self.k_scale = (amax[0] / 448.0).astype(np.float32)
            self.v_scale = (amax[1] / 448.0).astype(np.float32)
            sc = np.stack([self.k_scale, self.v_scale])[None, :, :, None, None]
            bits = wl.f32_to_e4m3_bits(raw / sc)  # canonical HND order [page][K|V][head][slot][dim]
            if layout == BZ_LAYOUT_NHD:
                bits = bits.transpose(0, 1, 3, 2, 4)
            self.pool = np.ascontiguousarray(bits).reshape(-1)
        else:
            self.pool = wl.randn_bits(rng, (self.pool_pages * self.stride_page,), kv_dtype, std=kv_std)

    def oracle_kv(self, pool=None):
        pool = self.pool if pool is None else pool
        half = self.stride_page // 2
        return oracle.PagedKV(pool, pool[half:], self.indices, self.indptr, self.last_page_len, self.P, self.Hkv,
                              self.D, self.stride_page, self.stride_n, self.stride_h, self.kv_dtype)

    def gather_kv(self, b):
        """Dense fp32 K, V of sequence b: [L, Hkv, D] each (independent of the checker's addressing code)."""
        L = int(self.ctx[b])
        f = wl.to_f32(self.pool, self.kv_dtype)
        K = np.empty((L, self.Hkv, self.D), np.float32)
        V = np.empty_like(K)
        for j in range(L):
            page = int(self.indices[self.indptr[b] + j // self.P])
            for h in range(self.Hkv):
                off = page * self.stride_page + (j % self.P) * self.stride_n + h * self.stride_h
                K[j, h] = f[off:off + self.D]
                V[j, h] = f[off + self.stride_page // 2: off + self.stride_page // 2 + self.D]
        return K, V


def rope_f64(x, pos, theta):
    """Textbook Llama rotate-half in float64: pairs (i, i+D/2), angle pos * theta^(-2i/D)."""
    x = np.asarray(x, np.float64)
    D = x.shape[-1]
    i = np.arange(D // 2)
    ang = pos * theta ** (-2.0 * i / D)
    c, s = np.cos(ang), np.sin(ang)
    a, b = x[..., :D // 2], x[..., D // 2:]
    return np.concatenate([a * c - b * s, b * c + a * s], axis=-1)


def dense_attention_f64(q, K, V, scale):
    """q [Hq, D], K,V [L, Hkv, D] -> o [Hq, D] in float64 (plain softmax, no tricks)."""
    q, K, V = (np.asarray(a, np.float64) for a in (q, K, V))
    Hq, Hkv = q.shape[0], K.shape[1]
    G = Hq // Hkv
    out = np.empty_like(q)
    for h in range(Hq):
        s = K[:, h // G, :] @ q[h] * scale
        p = np.exp(s - s.max())
        out[h] = (p / p.sum()) @ V[:, h // G, :]
    return out


def ulp_tol(ref, dtype, base=2e-3):
    """Per-element tolerance for a result stored in `dtype`: `base`, widened to just over half a
    unit in the last place where the storage grid itself is coarser than that."""
    mant = 10 if dtype == BZ_F16 else 7
    a = np.maximum(np.abs(ref), 1e-30)
    half_ulp = 2.0 ** (np.floor(np.log2(a)) - mant - 1)
    return np.maximum(base, 1.02 * half_ulp + 1e-6)
