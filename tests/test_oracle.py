"""CPU tests that pin the checker (oracle/bz_oracle.c) before anything is compared with it.

The reference holds no numeric fixtures for this path (no tests, FlashInfer fork absent), so each
function is pinned by an independent implementation (numpy / torch CPU library routines, a float64
dense restatement written differently), by closed forms and by invariants chosen so that a dropped
term, a wrong sign or a wrong index fails at least one of them.  Structural fixtures the reference
does hold (Warmup page table, prefill len+1 reservation, seq_len formula) are checked literally.
"""
import numpy as np
import pytest
import torch

import oracle
from blitz_scale_amd import workloads as wl
from blitz_scale_amd._lib import BZ_BF16, BZ_E4M3, BZ_F16, BZ_LAYOUT_HND, BZ_LAYOUT_NHD

from _util import DecodeProblem, dense_attention_f64, rope_f64


# ---------------------------------------------------------------- conversions
def test_f16_decode_exhaustive_vs_numpy():
    codes = np.arange(65536, dtype=np.uint16)
    got = oracle.to_f32(codes, oracle.F16)
    want = codes.view(np.float16).astype(np.float32)
    assert np.array_equal(got.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
    assert np.isnan(got[np.isnan(want)]).all()


def test_f16_encode_vs_numpy():
    rng = np.random.default_rng(1)
    # every f16 value, every midpoint between neighbours (ties), and random fp32 over all binades
    codes = np.arange(0x7C00, dtype=np.uint16)
    vals = codes.view(np.float16).astype(np.float64)
    mids = ((vals[:-1] + vals[1:]) / 2).astype(np.float32)
    rnd = (rng.standard_normal(200000) * np.exp(rng.uniform(-20, 12, 200000))).astype(np.float32)
    edge = np.array([65504, 65519.99, 65520, 1e9, 2 ** -25, np.nextafter(np.float32(2 ** -25), 1), 2 ** -24,
                     0.0, -0.0], np.float32)
    x = np.concatenate([vals.astype(np.float32), mids, rnd, edge, -mids, -rnd])
    assert np.array_equal(oracle.from_f32(x, oracle.F16), x.astype(np.float16).view(np.uint16))


def test_bf16_exhaustive_and_rne():
    codes = np.arange(65536, dtype=np.uint16)
    got = oracle.to_f32(codes, oracle.BF16)
    assert np.array_equal(got.view(np.uint32), codes.astype(np.uint32) << 16)
    finite = np.isfinite(got)
    assert np.array_equal(oracle.from_f32(got[finite], oracle.BF16), codes[finite])  # round trip
    # RNE against torch's independent conversion, including exact ties
    rng = np.random.default_rng(2)
    x = (rng.standard_normal(300000) * np.exp(rng.uniform(-30, 30, 300000))).astype(np.float32)
    ties = ((codes[:0x7F7F].astype(np.uint32) << 16) | 0x8000).view(np.float32)
    x = np.concatenate([x, ties, -ties])
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(oracle.from_f32(x, oracle.BF16), want)
    assert np.array_equal(wl.f32_to_bf16_bits(x), want)  # the generator's numpy conversion too


def test_e4m3_table_and_encode():
    codes = np.arange(256, dtype=np.uint8)
    got = oracle.to_f32(codes, oracle.E4M3)
    want = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
    nan = np.isnan(want)
    assert nan.sum() == 2 and np.isnan(got[nan]).all()
    assert np.array_equal(got[~nan], want[~nan])
    assert got[0x7E] == 448.0 and got[0x08] == 2.0 ** -6 and got[0x01] == 2.0 ** -9  # OCP e4m3fn landmarks
    assert np.array_equal(wl.e4m3_bits_to_f32(codes)[~nan], want[~nan])
    # encode: round trip, ties to even between neighbours, saturation at +-448
    fin = codes[~nan]
    assert np.array_equal(oracle.from_f32(got[~nan], oracle.E4M3) & 0x7F, fin & 0x7F)
    pos = got[:0x7F].astype(np.float64)
    mids = ((pos[:-1] + pos[1:]) / 2).astype(np.float32)
    enc = oracle.from_f32(mids, oracle.E4M3)
    lo = np.arange(0x7E)
    assert np.array_equal(enc, np.where(lo & 1, lo + 1, lo).astype(np.uint8))
    assert list(oracle.from_f32(np.array([1e6, -1e6, 448, 464.1, 0.0], np.float32), oracle.E4M3)) == [0x7E, 0xFE, 0x7E, 0x7E, 0]
    rng = np.random.default_rng(3)
    x = (rng.standard_normal(100000) * np.exp(rng.uniform(-8, 6, 100000))).astype(np.float32)
    x = x[np.abs(x) <= 448]
    want_enc = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got_enc = oracle.from_f32(x, oracle.E4M3)
    assert np.array_equal(got_enc & 0x7F, want_enc & 0x7F)
    assert np.array_equal(wl.f32_to_e4m3_bits(x), got_enc)


# ---------------------------------------------------------------- RoPE
@pytest.mark.parametrize("D,theta", [(64, 1e4), (128, 1e4), (128, 5e5)])
def test_rope_properties(D, theta):
    rng = np.random.default_rng(4)
    x, y = rng.standard_normal(D).astype(np.float32), rng.standard_normal(D).astype(np.float32)
    assert np.array_equal(oracle.rope_llama(x, 0, theta), x)  # position 0 is the identity
    for pos in (1, 7, 100, 4095):
        r = oracle.rope_llama(x, pos, theta)
        assert abs(np.linalg.norm(r) - np.linalg.norm(x)) < 1e-4  # rotation
        # textbook formula in float64; the fp32 angle pos*f costs up to pos*2^-24 rad
        assert np.abs(r - rope_f64(x, pos, theta)).max() < 5e-6 + pos * 3e-7
    # <rope(x,m), rope(y,n)> depends on m-n only
    d1 = oracle.rope_llama(x, 17, theta) @ oracle.rope_llama(y, 5, theta)
    d2 = oracle.rope_llama(x, 112, theta) @ oracle.rope_llama(y, 100, theta)
    assert abs(d1 - d2) < 1e-3
    # pairing is (i, i+D/2), not (2i, 2i+1): rotating e_0 moves weight to element D/2 only
    e0 = np.zeros(D, np.float32)
    e0[0] = 1
    r = oracle.rope_llama(e0, 1, theta)
    assert abs(r[0] - np.cos(1.0)) < 1e-6 and abs(r[D // 2] - np.sin(1.0)) < 1e-6
    assert np.abs(np.delete(r, [0, D // 2])).max() == 0
    f = oracle.rope_freqs(D, theta)
    assert f[0] == 1.0 and np.allclose(f, theta ** (-2.0 * np.arange(D // 2) / D), rtol=1e-6)


# ---------------------------------------------------------------- paged decode
@pytest.mark.parametrize("layout", [BZ_LAYOUT_NHD, BZ_LAYOUT_HND])
@pytest.mark.parametrize("dtype", [BZ_F16, BZ_BF16])
def test_decode_vs_dense_f64(layout, dtype):
    p = DecodeProblem(11, [1, 5, 16, 17, 40], Hq=4, Hkv=2, D=64, P=8, dtype=dtype, layout=layout)
    out, lse = oracle.batch_decode(p.q, dtype, p.oracle_kv(), p.Hq, want_lse=True)
    qf = wl.to_f32(p.q, dtype)
    for b in range(p.B):
        K, V = p.gather_kv(b)
        ref = dense_attention_f64(qf[b], K, V, 1 / np.sqrt(p.D))
        assert np.abs(out[b] - ref).max() < 2e-6
        s = np.einsum("hd,lhd->hl", qf[b].astype(np.float64), np.repeat(K, 2, axis=1)) / np.sqrt(p.D)
        assert np.abs(lse[b] - np.log(np.exp(s).sum(-1))).max() < 1e-5


def test_decode_rope_modes_vs_dense_f64():
    theta, dtype = 1e4, BZ_F16
    p = DecodeProblem(12, [3, 33, 70], Hq=2, Hkv=2, D=64, P=16, dtype=dtype)
    qf = wl.to_f32(p.q, dtype)
    full = oracle.batch_decode(p.q, dtype, p.oracle_kv(), p.Hq, rope_mode=oracle.ROPE_FULL, rope_theta=theta)
    qonly = oracle.batch_decode(p.q, dtype, p.oracle_kv(), p.Hq, rope_mode=oracle.ROPE_Q_ONLY, rope_theta=theta)
    for b in range(p.B):
        K, V = p.gather_kv(b)
        L = len(K)
        qr = rope_f64(qf[b], L - 1, theta)
        Kr = np.stack([rope_f64(K[j], j, theta) for j in range(L)])
        assert np.abs(full[b] - dense_attention_f64(qr, Kr, V, 1 / 8)).max() < 1e-5
        assert np.abs(qonly[b] - dense_attention_f64(qr, K, V, 1 / 8)).max() < 1e-5


def test_decode_invariants():
    dtype = BZ_F16
    p = DecodeProblem(13, [1, 31, 64, 100], Hq=8, Hkv=2, D=64, P=16, dtype=dtype)
    out = oracle.batch_decode(p.q, dtype, p.oracle_kv(), p.Hq)
    # ctx = 1: o == v0 exactly
    K, V = p.gather_kv(0)
    assert np.array_equal(out[0], np.repeat(V[0], 4, axis=0))
    # convex combination of V rows
    for b in range(p.B):
        K, V = p.gather_kv(b)
        Vq = np.repeat(V, 4, axis=1)
        assert (out[b] <= Vq.max(0) + 1e-6).all() and (out[b] >= Vq.min(0) - 1e-6).all()
    # moving the pages to other physical ids (indices updated) changes nothing, bit for bit
    rng = np.random.default_rng(5)
    perm = rng.permutation(p.pool_pages)
    pool2 = np.empty_like(p.pool).reshape(p.pool_pages, -1)
    pool2[perm] = p.pool.reshape(p.pool_pages, -1)
    kv2 = oracle.PagedKV(pool2.reshape(-1), pool2.reshape(-1)[p.stride_page // 2:], perm[p.indices].astype(np.int32),
                         p.indptr, p.last_page_len, p.P, p.Hkv, p.D, p.stride_page, p.stride_n, p.stride_h, dtype)
    assert np.array_equal(oracle.batch_decode(p.q, dtype, kv2, p.Hq), out)
    # GQA == MHA with K/V heads repeated (NHD pool rebuilt with 8 kv heads)
    B, Hq, D, P = p.B, p.Hq, p.D, p.P
    sp, sn, sh = wl.strides(BZ_LAYOUT_NHD, Hq, P, D)
    pool8 = np.zeros(p.pool_pages * sp, np.uint16)
    for b in range(B):
        for j in range(int(p.ctx[b])):
            page = int(p.indices[p.indptr[b] + j // P])
            for h in range(Hq):
                src = page * p.stride_page + (j % P) * p.stride_n + (h // 4) * p.stride_h
                dst = page * sp + (j % P) * sn + h * sh
                pool8[dst:dst + D] = p.pool[src:src + D]
                pool8[dst + sp // 2:dst + sp // 2 + D] = p.pool[src + p.stride_page // 2:src + p.stride_page // 2 + D]
    kv8 = oracle.PagedKV(pool8, pool8[sp // 2:], p.indices, p.indptr, p.last_page_len, P, Hq, D, sp, sn, sh, dtype)
    assert np.array_equal(oracle.batch_decode(p.q, dtype, kv8, Hq), out)


def test_decode_closed_forms():
    D, P, dtype = 64, 16, BZ_F16
    p = DecodeProblem(14, [50], Hq=2, Hkv=2, D=D, P=P, dtype=dtype)
    pool = p.pool.copy()
    # all K rows equal -> uniform softmax -> o = mean of V
    krow = wl.to_bits(np.random.default_rng(6).standard_normal(D).astype(np.float32), dtype)
    for j in range(50):
        page = int(p.indices[j // P])
        for h in range(2):
            off = page * p.stride_page + (j % P) * p.stride_n + h * p.stride_h
            pool[off:off + D] = krow
    p2 = DecodeProblem(14, [50], Hq=2, Hkv=2, D=D, P=P, dtype=dtype)
    p2.pool = pool
    out = oracle.batch_decode(p.q, dtype, p2.oracle_kv(), 2)
    _, V = p2.gather_kv(0)
    assert np.abs(out[0] - V.mean(0)).max() < 1e-5
    # one key aligned with a large q: softmax is one-hot on it -> o = that v
    q = np.zeros((1, 2, D), np.float32)
    q[..., 3] = 200.0
    pool = p.pool.copy()
    for j in range(50):
        page = int(p.indices[j // P])
        for h in range(2):
            off = page * p.stride_page + (j % P) * p.stride_n + h * p.stride_h
            pool[off + 3] = wl.to_bits(np.float32([10.0 if j == 37 else -10.0]), dtype)[0]
    p2.pool = pool
    out = oracle.batch_decode(wl.to_bits(q, dtype), dtype, p2.oracle_kv(), 2)
    _, V = p2.gather_kv(0)
    assert np.abs(out[0] - V[37]).max() < 1e-6


def test_decode_e4m3_scales_vs_dense():
    p = DecodeProblem(15, [20, 45], Hq=8, Hkv=2, D=64, P=16, dtype=BZ_BF16, kv_dtype=BZ_E4M3)
    assert p.pool.dtype == np.uint8 and np.abs(wl.to_f32(p.pool, BZ_E4M3)).max() == 448.0  # amax/448 scaling
    out = oracle.batch_decode(p.q, BZ_BF16, p.oracle_kv(), 8, k_scale=p.k_scale, v_scale=p.v_scale)
    qf = wl.to_f32(p.q, BZ_BF16)
    for b in range(2):
        K, V = p.gather_kv(b)
        ref = dense_attention_f64(qf[b], K * p.k_scale[None, :, None], V * p.v_scale[None, :, None], 1 / 8)
        assert np.abs(out[b] - ref).max() < 1e-5


def test_seq_len_formula_and_warmup_fixture():
    # the Warmup page table of src/service/service.cc:224-257: 256 pages of 16, last_page_len 16 -> 4096 tokens
    kv = oracle.PagedKV(np.zeros(8, np.uint16), np.zeros(8, np.uint16), np.arange(256), [0, 256], [16], 16, 1, 8, 256,
                        8, 8, BZ_F16)
    assert list(kv.seq_lens()) == [4096]
    kv = oracle.PagedKV(np.zeros(8, np.uint16), np.zeros(8, np.uint16), np.arange(6), [0, 1, 1, 6], [3, 0, 16], 16, 1,
                        8, 256, 8, 8, BZ_F16)
    assert list(kv.seq_lens()) == [3, 0, 80]  # (n-1)*P + last_page_len; no pages -> empty


# ---------------------------------------------------------------- ragged prefill
@pytest.mark.parametrize("causal", [True, False])
def test_prefill_vs_torch_sdpa(causal):
    rng = np.random.default_rng(21)
    lens, Hq, Hkv, D, dtype = [1, 7, 33], 4, 2, 64, BZ_F16
    indptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    N = int(indptr[-1])
    q, k, v = (wl.randn_bits(rng, (N, H, D), dtype) for H in (Hq, Hkv, Hkv))
    out = oracle.batch_prefill_ragged(q, k, v, dtype, indptr, Hq, Hkv, D, causal=causal)
    qf, kf, vf = (torch.from_numpy(wl.to_f32(a, dtype)).double() for a in (q, k, v))
    for r in range(len(lens)):
        s, e = indptr[r], indptr[r + 1]
        ref = torch.nn.functional.scaled_dot_product_attention(
            qf[s:e].transpose(0, 1), kf[s:e].transpose(0, 1).repeat_interleave(2, 0),
            vf[s:e].transpose(0, 1).repeat_interleave(2, 0), is_causal=causal).transpose(0, 1).numpy()
        assert np.abs(out[s:e] - ref).max() < 3e-6


def test_prefill_row_equals_decode_of_prefix_and_rope():
    rng = np.random.default_rng(22)
    L, Hq, Hkv, D, P, dtype, theta = 37, 4, 2, 64, 8, BZ_F16, 1e4
    indptr = np.array([0, L], np.int32)
    q, k, v = (wl.randn_bits(rng, (L, H, D), dtype) for H in (Hq, Hkv, Hkv))
    pre = oracle.batch_prefill_ragged(q, k, v, dtype, indptr, Hq, Hkv, D, rope=True, rope_theta=theta)
    sub = oracle.batch_prefill_ragged(q, k, v, dtype, indptr, Hq, Hkv, D, rope=True, rope_theta=theta, rows=[5, 36])
    assert np.array_equal(sub, pre[[5, 36]])
    # store the raw K,V into pages, then decode row i over the first i+1 tokens with on-the-fly RoPE
    for i in (0, 8, 36):
        p = DecodeProblem(23, [i + 1], Hq, Hkv, D, P, dtype, layout=BZ_LAYOUT_NHD)
        kv = p.oracle_kv()
        oracle.store_prefill_kv(kv, k[:i + 1], v[:i + 1], dtype, [0, i + 1])
        dec = oracle.batch_decode(q[i:i + 1], dtype, kv, Hq, rope_mode=oracle.ROPE_FULL, rope_theta=theta)
        assert np.abs(dec[0] - pre[i]).max() < 2e-6


# ---------------------------------------------------------------- page writes
@pytest.mark.parametrize("layout", [BZ_LAYOUT_NHD, BZ_LAYOUT_HND])
def test_store_and_append_placement(layout):
    rng = np.random.default_rng(31)
    lens, Hkv, D, P, dtype = [5, 16, 21], 2, 64, 8, BZ_F16
    p = DecodeProblem(32, [l + 1 for l in lens], 2, Hkv, D, P, dtype, layout=layout)  # len+1 slots reserved
    SENT = 0x7BFF
    pool = np.full_like(p.pool, SENT)
    kv = p.oracle_kv(pool)
    ri = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    k = wl.randn_bits(rng, (ri[-1], Hkv, D), dtype)
    v = wl.randn_bits(rng, (ri[-1], Hkv, D), dtype)
    k[k == SENT] = 0
    v[v == SENT] = 0
    oracle.store_prefill_kv(kv, k, v, dtype, ri)
    assert (pool != SENT).sum() == 2 * ri[-1] * Hkv * D  # exactly the stored rows changed
    for b, l in enumerate(lens):
        for t in (0, l - 1):
            page = int(p.indices[p.indptr[b] + t // P])  # page.cu:49-52
            for h in range(Hkv):
                off = page * p.stride_page + (t % P) * p.stride_n + h * p.stride_h
                assert np.array_equal(pool[off:off + D], k[ri[b] + t, h])
                assert np.array_equal(pool[off + p.stride_page // 2:off + p.stride_page // 2 + D], v[ri[b] + t, h])
    # append goes to position seq_len-1 = len: last page, slot last_page_len-1
    before = pool.copy()
    nk, nv = wl.randn_bits(rng, (3, Hkv, D), dtype), wl.randn_bits(rng, (3, Hkv, D), dtype)
    oracle.append_decode_kv(kv, nk, nv, dtype)
    assert (pool != before).sum() <= 2 * 3 * Hkv * D and (pool != before).sum() > 2 * 3 * Hkv * D - 8
    for b, l in enumerate(lens):
        page = int(p.indices[p.indptr[b + 1] - 1])
        slot = int(p.last_page_len[b]) - 1
        assert slot == l % P
        off = page * p.stride_page + slot * p.stride_n + 1 * p.stride_h
        assert np.array_equal(pool[off:off + D], nk[b, 1])


def test_store_with_rope_and_e4m3_quant():
    rng = np.random.default_rng(33)
    L, Hkv, D, P, theta = 9, 2, 64, 4, 1e4
    p = DecodeProblem(34, [L], 2, Hkv, D, P, BZ_BF16, kv_dtype=BZ_E4M3)
    pool = np.zeros_like(p.pool)
    kv = p.oracle_kv(pool)
    k, v = wl.randn_bits(rng, (L, Hkv, D), BZ_BF16), wl.randn_bits(rng, (L, Hkv, D), BZ_BF16)
    ks, vs = np.float32([0.01, 0.02]), np.float32([0.015, 0.03])
    oracle.store_prefill_kv(kv, k, v, BZ_BF16, [0, L], rope=True, rope_theta=theta, k_scale=ks, v_scale=vs)
    K, V = DecodeProblem.gather_kv(type("P", (), dict(ctx=[L], pool=pool, kv_dtype=BZ_E4M3, Hkv=Hkv, D=D, P=P,
                                                     indices=p.indices, indptr=p.indptr, stride_page=p.stride_page,
                                                     stride_n=p.stride_n, stride_h=p.stride_h))(), 0)
    kf, vf = wl.to_f32(k, BZ_BF16), wl.to_f32(v, BZ_BF16)
    for t in range(L):
        for h in range(Hkv):
            want_k = wl.e4m3_bits_to_f32(wl.f32_to_e4m3_bits((rope_f64(kf[t, h], t, theta) / ks[h]).astype(np.float32)))
            # rotation in fp32 vs float64 may flip a rounding on rare elements: allow one e4m3 step there
            assert (np.abs(K[t, h] - want_k) <= np.maximum(np.abs(want_k) * 0.13, 2.0 ** -9)).all()
            assert (K[t, h] == want_k).mean() > 0.9
            assert np.array_equal(V[t, h], wl.e4m3_bits_to_f32(wl.f32_to_e4m3_bits(vf[t, h] / vs[h])))


# ---------------------------------------------------------------- element-wise
def test_rms_norm_closed_form_and_torch():
    h, dtype = 256, BZ_F16
    c = 0.75
    x = wl.to_bits(np.full((2, h), c, np.float32), dtype)
    w = wl.to_bits(np.linspace(0.5, 1.5, h).astype(np.float32), dtype)
    out = oracle.rms_norm(x, w, dtype, eps=1e-5)
    assert np.abs(out[0] - wl.to_f32(w, dtype) * c / np.sqrt(c * c + 1e-5)).max() < 1e-6
    rng = np.random.default_rng(41)
    x, w = wl.randn_bits(rng, (5, h), dtype), wl.randn_bits(rng, (h,), dtype, mean=1.0, std=0.02)
    ref = torch.nn.functional.rms_norm(torch.from_numpy(wl.to_f32(x, dtype)).double(), (h,),
                                       torch.from_numpy(wl.to_f32(w, dtype)).double(), eps=1e-5).numpy()
    assert np.abs(oracle.rms_norm(x, w, dtype) - ref).max() < 5e-6
    # fused add: residual' = round(in + res), out = rms_norm(residual')
    r = wl.randn_bits(rng, (5, h), dtype)
    out, res2 = oracle.add_rms_norm(x, r, w, dtype)
    want_res = (wl.to_f32(x, dtype) + wl.to_f32(r, dtype)).astype(np.float16).view(np.uint16)
    assert np.array_equal(res2, want_res)
    assert np.abs(out - oracle.rms_norm(want_res, w, dtype)).max() == 0


def test_silu_and_mul_vs_torch():
    rng = np.random.default_rng(42)
    I, dtype = 96, BZ_F16
    x = wl.randn_bits(rng, (3, 2 * I), dtype, std=3.0)
    xf = torch.from_numpy(wl.to_f32(x, dtype)).double()
    ref = (torch.nn.functional.silu(xf[:, :I]) * xf[:, I:]).numpy()  # gate is the first half
    assert np.abs(oracle.silu_and_mul(x, dtype) - ref).max() < 1e-5
    z = wl.to_bits(np.float32([[0.0, 30.0, 5.0, 7.0]]), dtype)  # silu(0)=0, silu(30)~30
    assert np.allclose(oracle.silu_and_mul(z, dtype), [[0.0, 210.0]], atol=1e-3)


@pytest.mark.parametrize("dtype", [BZ_F16, BZ_BF16])
def test_add_residual_single_rounding(dtype):
    rng = np.random.default_rng(43)
    n = 200000
    a = wl.to_bits((rng.standard_normal(n) * np.exp(rng.uniform(-12, 8, n))).astype(np.float32), dtype)
    b = wl.to_bits((rng.standard_normal(n) * np.exp(rng.uniform(-12, 8, n))).astype(np.float32), dtype)
    exact = wl.to_f32(a, dtype).astype(np.float64) + wl.to_f32(b, dtype).astype(np.float64)
    if dtype == BZ_F16:
        want = exact.astype(np.float16).view(np.uint16)  # numpy rounds double -> half once
    else:
        want = torch.from_numpy(exact).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = oracle.add_residual(a, b, dtype)
    assert np.array_equal(got, want)


# ---------------------------------------------------------------- host page-table logic
def test_prefill_reservation_matches_reference_rule():
    # src/blitz/batch.h:246-250: need_slots = len+1, blocks = ceil(need_slots/P), last = need_slots-(blocks-1)*P
    lens, P = [1, 15, 16, 17, 31, 32, 4096], 16
    indptr, lpl = oracle.prefill_reservation(lens, P)
    assert list(np.diff(indptr)) == [1, 1, 2, 2, 2, 3, 257]
    assert list(lpl) == [2, 16, 1, 2, 16, 1, 1]
    assert all(1 <= x <= P for x in lpl)
    # the table describes len+1 slots through the kernel's seq_len formula (page.cu:38-40)
    assert list((np.diff(indptr) - 1) * P + lpl) == [l + 1 for l in lens]


# ---- row-major (batched) GEMM of the layers' GEMM boundary ------------------------------------------
@pytest.mark.parametrize("transa", [False, True])
@pytest.mark.parametrize("transb", [False, True])
def test_gemm_against_numpy_matmul(transa, transb):
    """Pinned by numpy.matmul on the logical operands: small integers make every product and sum exact, so
    any index, transpose or stride mistake changes bits; m, n, k and the batch strides are all different."""
    rng = np.random.default_rng(5)
    m, n, k, batch = 5, 7, 11, 3
    sa, sb, sc = m * k + 3, k * n + 5, m * n + 2          # padded strides between the matrices of a batch
    A = rng.integers(-4, 5, size=(batch, m, k)).astype(np.float32)
    B = rng.integers(-4, 5, size=(batch, k, n)).astype(np.float32)
    C0 = rng.integers(-8, 9, size=(batch, m, n)).astype(np.float32)
    a_store = np.zeros(batch * sa, np.float32)
    b_store = np.zeros(batch * sb, np.float32)
    c_store = np.full(batch * sc, 77.0, np.float32)       # the gaps between matrices must stay untouched
    for b in range(batch):
        a_store[b * sa:b * sa + m * k] = (A[b].T if transa else A[b]).reshape(-1)
        b_store[b * sb:b * sb + k * n] = (B[b].T if transb else B[b]).reshape(-1)
        c_store[b * sc:b * sc + m * n] = C0[b].reshape(-1)
    for dt in (oracle.F16, oracle.BF16):
        got = oracle.gemm_strided_batched(oracle.from_f32(a_store, dt), oracle.from_f32(b_store, dt), dt, m, n, k,
                                          transa=transa, transb=transb, alpha=2.0, beta=-1.0,
                                          c_bits=oracle.from_f32(c_store, dt), stride_a=sa, stride_b=sb, stride_c=sc,
                                          batch=batch)
        got = oracle.to_f32(got, dt)
        for b in range(batch):
            want = 2.0 * np.matmul(A[b].astype(np.float64), B[b].astype(np.float64)) - C0[b]
            assert np.array_equal(got[b * sc:b * sc + m * n].reshape(m, n), want.astype(np.float32))
            assert np.all(got[b * sc + m * n:(b + 1) * sc] == 77.0)


def test_gemm_rounding_and_defaults():
    """alpha = 1, beta = 0, contiguous batch (what gemm / gemmBatched of the reference reduce to): one
    rounding of an fp32 sum; C's previous contents (NaN here) are not read when beta is 0."""
    rng = np.random.default_rng(6)
    m, n, k = 9, 33, 257
    A = wl.randn_bits(rng, (2, m, k), BZ_F16)
    B = wl.randn_bits(rng, (2, k, n), BZ_F16, std=1.0 / np.sqrt(k))
    c0 = np.full(2 * m * n, 0x7E00, np.uint16)
    got = oracle.to_f32(oracle.gemm_strided_batched(A, B, oracle.F16, m, n, k, c_bits=c0, batch=2), oracle.F16)
    want = np.matmul(wl.to_f32(A, BZ_F16).astype(np.float64), wl.to_f32(B, BZ_F16).astype(np.float64))
    want16 = want.astype(np.float16).astype(np.float64)
    # fp32 accumulation error (~1e-6) can only move a result across a rounding boundary: at most one f16 step
    step = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(want), 2.0 ** -14))) - 10)
    assert (np.abs(got.reshape(2, m, n) - want16) <= step).all()
    assert (got.reshape(2, m, n) == want16).mean() > 0.99


def test_prefill_rope_q_only_mode():
    """rope="q" (q rotated, k rows hold rotated K already) is pinned by the full mode: with fp32 storage nothing
    is rounded in between, so rotating k beforehand with rope_llama and asking for q only must give the very
    same numbers as rotating both inside the call."""
    rng = np.random.default_rng(3)
    lens = [5, 17, 1]
    ip = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    N = int(ip[-1])
    q = rng.standard_normal((N, 4, 128)).astype(np.float32)
    k = rng.standard_normal((N, 2, 128)).astype(np.float32)
    v = rng.standard_normal((N, 2, 128)).astype(np.float32)
    both = oracle.batch_prefill_ragged(q, k, v, oracle.F32, ip, 4, 2, 128, rope=True, rope_theta=5e5)
    kr = k.copy()
    for r, L in enumerate(lens):
        for t in range(L):
            for h in range(2):
                kr[ip[r] + t, h] = oracle.rope_llama(k[ip[r] + t, h], t, 5e5)
    assert np.array_equal(oracle.batch_prefill_ragged(q, kr, v, oracle.F32, ip, 4, 2, 128, rope="q", rope_theta=5e5), both)
    assert not np.array_equal(oracle.batch_prefill_ragged(q, kr, v, oracle.F32, ip, 4, 2, 128, rope=False), both)
