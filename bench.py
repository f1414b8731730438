"""Headline benchmark: Llama-3-8B-shaped GQA paged decode (BASELINE config 3) on one MI355X.

A step is one layer's decode-time attention block over the whole batch: the fused RoPE + KV append
of the new token followed by batch decode over the paged KV cache (src/layer/attn.h:196-203 of the
reference).  Steps cycle over several layer planes of the pool, as a model's layer loop does, so the
KV a step reads has not just been read by the previous step.  plan() runs once per model step in the
reference (src/model/llama.h:363-375), outside the layer loop, and is timed separately here.

Prints ONE JSON line.  One GPU only.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--layers", type=int, default=8, help="layer planes of the KV pool the steps cycle over")
    ap.add_argument("--seed", type=lambda s: int(s, 0), default=0x5EED)
    ap.add_argument("--sigma", type=float, default=1.0, help="sigma of the log-normal context lengths")
    ap.add_argument("--split-tokens", type=int, default=2048)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (--gpus 1); the path shards by kv head / by sequence "
                 "without any exchange inside attention, and nothing here launches a second rank.")

    import numpy as np
    import torch

    from blitz_scale_amd import _lib, kernel as K, workloads as wl
    from blitz_scale_amd._lib import BZ_BF16, BZ_LAYOUT_HND, BZ_ROPE_NONE

    _lib.load()  # fails loudly if the HIP library is not built
    torch.cuda.set_device(0)
    dev = "cuda"
    cfg = dict(wl.CONFIGS["C3"])
    B, Hq, Hkv, D, P = cfg["batch"], cfg["Hq"], cfg["Hkv"], cfg["D"], cfg["P"]
    theta = cfg["rope_theta"]
    rng = np.random.default_rng(args.seed)
    ctx = wl.lognormal_ctx(rng, B, 1024.0, args.sigma, 64, 8192)
    need = int(((ctx + P - 1) // P).sum())
    pool_pages = int(np.ceil(need * cfg["oversub"]))
    indices, indptr, lpl = wl.page_table_for(ctx, P, pool_pages, rng)
    stride_page, _, _ = wl.strides(BZ_LAYOUT_HND, Hkv, P, D)
    L = args.layers

    g = torch.Generator(device=dev)
    g.manual_seed(args.seed)
    pool = torch.empty(L * pool_pages * stride_page, dtype=torch.bfloat16, device=dev)
    plane = pool_pages * stride_page
    for l in range(L):
        pool[l * plane:(l + 1) * plane].normal_(generator=g)
    q = torch.randn((B, Hq, D), dtype=torch.bfloat16, device=dev, generator=g)
    k_new = torch.randn((B, Hkv, D), dtype=torch.bfloat16, device=dev, generator=g)
    v_new = torch.randn((B, Hkv, D), dtype=torch.bfloat16, device=dev, generator=g)
    out = torch.empty((B, Hq, D), dtype=torch.bfloat16, device=dev)

    pt = K.PageTable(B, P, Hkv, D, pool, layout=BZ_LAYOUT_HND)
    pt.indices, pt.indptr, pt.last_page_len = indices, indptr, lpl
    pt.upload()
    float_ws = torch.empty(128 << 20, dtype=torch.uint8, device=dev)  # sizes of src/model/llama.h:111-112
    int_ws = torch.empty(8 << 20, dtype=torch.uint8, device=dev)
    handler = K.BlitzBatchDecodeHandler()

    def plan():
        handler.plan(float_ws, float_ws.numel(), int_ws, int_ws.numel(), indptr, lpl, B, Hq, Hkv, D, P,
                     split_tokens=args.split_tokens)

    t0 = time.perf_counter()
    for _ in range(10):
        plan()
    torch.cuda.synchronize()
    plan_ms = (time.perf_counter() - t0) / 10 * 1e3
    info = handler.info()

    def step(i, ev=None):
        pt.set_layer(i % L, pool_pages)
        K.append_decode_kv_cache(pt, k_new, v_new, q=q, num_qo_heads=Hq, rope=True, rope_theta=theta)
        if ev is not None:
            ev[0].record()
        K.batch_decode_attention(handler, q, pt, out, Hq, rope_mode=BZ_ROPE_NONE)
        if ev is not None:
            ev[1].record()

    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i, events[i])
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3
    dec_ms = np.array([a.elapsed_time(b) for a, b in events])

    alg_bytes = wl.decode_algorithmic_bytes(ctx, Hq, Hkv, D, 2, 2, P)
    dec_avg_s = float(dec_ms.mean()) * 1e-3
    achieved = alg_bytes / dec_avg_s / 1e9

    res = {
        "metric": "paged_decode_us_per_step",
        "value": round(ms_per_step * 1e3, 3),
        "unit": "us/step",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 6),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": "C3: Llama-3-8B-shaped GQA paged decode, one layer per step (fused RoPE+append, batch decode)",
            "batch": B, "num_qo_heads": Hq, "num_kv_heads": Hkv, "head_dim": D, "page_size": P,
            "ctx": f"lognormal(mean 1024, sigma {args.sigma}) clipped [64,8192]", "sum_ctx": int(ctx.sum()),
            "max_ctx": int(ctx.max()), "pool_pages_per_layer": pool_pages, "layer_planes_cycled": L,
            "kv_layout": "HND", "rope_theta": theta, "split_tokens": args.split_tokens, "seed": hex(args.seed),
            "plan": info,
        },
        "tokens_per_s": round(B / (ms_per_step * 1e-3), 1),
        "plan_ms_per_model_step": round(plan_ms, 4),
        "decode_kernel_us": {"mean": round(float(dec_ms.mean()) * 1e3, 3),
                             "p10": round(float(np.percentile(dec_ms, 10)) * 1e3, 3),
                             "p50": round(float(np.percentile(dec_ms, 50)) * 1e3, 3),
                             "p90": round(float(np.percentile(dec_ms, 90)) * 1e3, 3)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": None,
                     "algorithmic_bytes_per_launch": int(alg_bytes),
                     "kernel": "batch decode (main kernel + split-K combine), HIP events on the launch stream"},
    }

    if not args.no_cpu_baseline:
        import oracle  # the checker, used here only as the timed CPU baseline
        plane0 = pool[:plane].view(torch.int16).cpu().numpy().view(np.uint16)
        qh = q.view(torch.int16).cpu().numpy().view(np.uint16)
        sp, sn, sh = wl.strides(BZ_LAYOUT_HND, Hkv, P, D)
        kv = oracle.PagedKV(plane0, plane0[sp // 2:], indices, indptr, lpl, P, Hkv, D, sp, sn, sh, oracle.BF16)
        t0 = time.perf_counter()
        ref = oracle.batch_decode(qh, oracle.BF16, kv, Hq, parallel=True)
        cpu_s = time.perf_counter() - t0
        # the same call on the GPU for the same plane, as a last sanity check of what was timed
        pt.set_layer(0, pool_pages)
        out32 = torch.empty((B, Hq, D), dtype=torch.float32, device=dev)
        K.batch_decode_attention(handler, q, pt, out32, Hq, rope_mode=BZ_ROPE_NONE)
        torch.cuda.synchronize()
        res["max_abs_err_vs_cpu"] = float(np.abs(out32.cpu().numpy() - ref).max())
        res["cpu_baseline"] = {"value": round(cpu_s * 1e6, 1), "unit": "us/step", "cores": oracle.num_threads(True),
                               "kind": "port",
                               "sample": "full C3 batch, decode only (no append), 1 repetition, OpenMP over sequences",
                               "host_cpus": os.cpu_count()}
    print(json.dumps(res))


if __name__ == "__main__":
    main()
