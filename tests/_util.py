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


def ulp_tol(ref, dtype, base=2e-3, before_rounding=0.0):
    """Per-element tolerance for a result stored in `dtype`: `base`, widened to just over half a
    unit in the last place where the storage grid itself is coarser than that.  `before_rounding`: the error
    allowed for the value before it is rounded to the storage grid (a value that close to the middle between two
    grid points may round either way, which puts the stored result half a unit plus that much from the reference)."""
    mant = 10 if dtype == BZ_F16 else 7
    a = np.maximum(np.abs(ref), 1e-30)
    half_ulp = 2.0 ** (np.floor(np.log2(a)) - mant - 1)
    return np.maximum(base, 1.02 * half_ulp + 1e-6 + before_rounding)


# bf16 prefill with V widened to f16 on chip (the default, BZ_PREFILL_BF16_WIDEN_V): the probabilities enter the
# second contraction as f16 (relative 2^-12), which leaves the result within this of the reference before it is
# rounded to bf16 (measured 1.5e-4 .. 3e-4); the head + tail mode keeps ~1e-6 and is held to the plain bar
PREFILL_BF16_WIDEN_V_ERR = 5e-4


def prefill_angle_table(float_ws, max_len, D=128):
    """The (cos, sin) table the prefill call keeps in its float workspace for the q rotation, as the device computed
    it (sincosf(pos * f_i)), returned as fp32 [D/2 pairs][max_len positions][2]; max_len is the longest request of the
    plan.  (The device keeps it as [pairs / 2][max_len][cos i, sin i, cos i+1, sin i+1].)"""
    raw = float_ws[: (D // 2) * max_len * 8].cpu().numpy().view(np.float32)
    return raw.reshape(D // 4, max_len, 2, 2).transpose(0, 2, 1, 3).reshape(D // 2, max_len, 2)


def prefill_q_as_fed(q_bits, dtype, indptr, Hq, D, theta, table, sm_scale=None):
    """The q rows as the prefill kernel feeds them to the matrix cores when it rotates them itself
    (BZ_ROPE_Q_ONLY / BZ_ROPE_FULL): rotated at their offset inside the request with the entries of the device's own
    table (`table`, from prefill_angle_table: cos and sin times sm_scale * log2(e); the device's sincosf may differ from
    the host's in the last place, and one such difference, rounded the other way and multiplied by logits of +-40, is
    visible in the output) and rounded ONCE to the storage type -- every step an IEEE fp32 operation in the kernel's
    order, so the bits are the kernel's.  Attention over these rows with sm_scale = ln 2 (exp(s ln 2) = 2^s) and no
    further rotation of q is what the kernel computes, so the comparison needs no allowance for that rounding.  The
    table itself is held against the host's sincos (two units in the last place)."""
    q = wl.to_f32(q_bits, dtype)
    N = q.shape[0]
    indptr = np.asarray(indptr)
    pos = np.arange(N) - np.repeat(indptr[:-1], np.diff(indptr))
    f = oracle.rope_freqs(D, theta)
    ang = pos[None, :].astype(np.float32) * f[:, None]  # [pairs][tokens], one fp32 multiply as on the device
    if sm_scale is None:
        sm_scale = np.float32(1.0) / np.sqrt(np.float32(D))
    scale = np.float32(np.float32(sm_scale) * np.float32(1.4426950408889634))
    c, s_ = table[:, pos, 0], table[:, pos, 1]
    tol = 2.0 ** -22 * float(scale)
    assert np.abs(c - np.cos(ang.astype(np.float64)) * float(scale)).max() <= tol
    assert np.abs(s_ - np.sin(ang.astype(np.float64)) * float(scale)).max() <= tol
    c, s_ = c.T[:, None, :], s_.T[:, None, :]            # [tokens][1][pairs]
    x, y = q[:, :, : D // 2], q[:, :, D // 2:]
    xr = (x * c).astype(np.float32) - (y * s_).astype(np.float32)
    yr = (y * c).astype(np.float32) + (x * s_).astype(np.float32)
    return wl.to_bits(np.concatenate([xr, yr], axis=2).astype(np.float32), dtype)


LN2 = float(np.float32(0.6931471805599453))
