"""Benchmark of the paged-attention compute path on one MI355X.  Prints ONE JSON line.

Default workload (the headline, benchmark configuration 3): Llama-3-8B-shaped GQA paged decode, bf16, batch
128, 32/8 heads, head_dim 128, page_size 16, log-normal contexts.  A step is one layer's decode-time
attention block over the whole batch: the KV append of the new token (K rotated) and the batch decode
over the paged KV cache (src/layer/attn.h:196-203 of the reference), issued as the library's one-call
decode step (bz_decode_step: two launches).  Steps cycle over several layer planes of the pool, as a
model's layer loop does, so the KV a step reads has not just been read by the previous step; the value
reported is the step replayed from one HIP graph of that layer loop (the eagerly launched step is
reported beside it).  plan() runs once per model step in the reference (src/model/llama.h:363-375),
outside the layer loop, and is timed separately.

--workload C2 | C4 | C5 run the other configurations (C2 adds the RMSNorm and SiLU-gate kernels of the
layer, C4 is the ragged causal prefill + page store, C5 the e4m3-KV decode); ENDS and MIGRATE time the
row gathers / argmax either side of the layer loop and the KV migration pack / unpack, LAYERS a
small-batch 32-layer decode step launched eagerly and replayed from a HIP graph.  One GPU only.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0     # MI355X HBM3E
MFMA_PEAK_TFLOPS = 2500.0  # dense f16 / bf16


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None)
    ap.add_argument("--warmup", type=int, default=None)
    ap.add_argument("--workload", default="C3", choices=["C2", "C3", "C4", "C5", "ENDS", "MIGRATE", "LAYERS", "RAWK", "MFMA_CEILING"])
    ap.add_argument("--layers", type=int, default=None, help="layer planes of the KV pool the steps cycle over")
    ap.add_argument("--seed", type=lambda s: int(s, 0), default=0x5EED)
    ap.add_argument("--sigma", type=float, default=1.0, help="sigma of the log-normal context lengths (C3)")
    ap.add_argument("--split-tokens", type=int, default=2048)
    ap.add_argument("--page-size", type=int, default=None,
                    help="tokens per KV page for the decode workloads (default: the configuration's 16; the "
                         "reference's production value is 64, src/server/disaggregate.cc:310)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--two-call", action="store_true",
                    help="decode workloads: issue the step as append_decode_kv_cache + batch_decode_attention "
                         "(three launches) instead of the one-call decode step")
    ap.add_argument("--no-graph", action="store_true", help="decode workloads: skip the HIP-graph replay pass")
    ap.add_argument("--no-rope", action="store_true", help="decode workloads: leave RoPE out of the step (diagnostic)")
    ap.add_argument("--q-rope", default="attention", choices=["attention", "store"],
                    help="C4: where q is rotated. attention: in registers inside the attention kernel (q read once, "
                         "never written; the page store rotates k only); store: in place by the page-store kernel "
                         "(the attention kernel then takes q and k as they are)")
    ap.add_argument("--prefill-dtype", default="f16", choices=["f16", "bf16", "bf16-head-tail"],
                    help="C4: storage type of q, k, v and the output; bf16 runs the second product in f16 with V widened in "
                         "LDS, bf16-head-tail with the probabilities as two bf16 operands (any range of V)")
    ap.add_argument("--prefill-lens", default=None,
                    help="C4: comma-separated prompt lengths instead of the configuration's 16 x U[128, 4096], `8x1024` for "
                         "eight of 1024 (diagnostic; the workload name says so)")
    ap.add_argument("--prefill-heads", default=None,
                    help="C4: q heads/kv heads instead of the configuration's 40/40, e.g. 32/8 (diagnostic, as above)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch a few plain device copies of 1 GiB (reference point for rocprofv3 --pmc byte counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (--gpus 1); the path shards by kv head / by sequence "
                 "without any exchange inside attention, and nothing here launches a second rank.")
    return args


class HipEvents:
    """Plain HIP events (ctypes on the HIP runtime torch already loaded), for timing a launch on the
    stream it is issued to from inside the library."""

    def __init__(self, n):
        import ctypes as C
        self.C = C
        self.hip = C.CDLL("libamdhip64.so")
        self.ev = []
        for _ in range(2 * n):
            e = C.c_void_p()
            assert self.hip.hipEventCreate(C.byref(e)) == 0
            self.ev.append(e)

    def pair(self, i):
        return self.ev[2 * i], self.ev[2 * i + 1]

    def elapsed_ms(self, i):
        ms = self.C.c_float()
        assert self.hip.hipEventElapsedTime(self.C.byref(ms), self.ev[2 * i], self.ev[2 * i + 1]) == 0
        return ms.value


def pct(a):
    import numpy as np
    return {"mean": round(float(a.mean()) * 1e3, 3), "p10": round(float(np.percentile(a, 10)) * 1e3, 3),
            "p50": round(float(np.percentile(a, 50)) * 1e3, 3), "p90": round(float(np.percentile(a, 90)) * 1e3, 3)}


def timed(step, steps, warmup, torch_events=True):
    """W untimed steps, then exactly K steps between two device synchronisations.  step(i, ev) gets a pair
    of torch events (recorded on torch's current stream, the stream every launch goes to) to bracket the
    dominant kernel, or True when the step brings its own events."""
    import numpy as np
    import torch
    for i in range(warmup):
        step(i, None)
    torch.cuda.synchronize()
    events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        step(i, events[i] if torch_events else True)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    return elapsed / steps * 1e3, (np.array([a.elapsed_time(b) for a, b in events]) if torch_events else None)


def measured_traffic(name, args):
    """HBM bytes per launch of the dominant kernel, measured offline with rocprofv3 --pmc (profiles/*.md);
    only reported for the exact workload it was measured on."""
    if args.seed != 0x5EED or args.sigma != 1.0 or args.split_tokens != 2048 or args.page_size:
        return None
    if name == "C4" and (args.prefill_lens or args.prefill_heads or args.prefill_dtype != "f16"):
        return None
    try:
        with open(os.path.join(ROOT, "blitz_scale_amd", "measured_traffic.json")) as f:
            return json.load(f)["bytes_per_launch"].get(name)
    except OSError:
        return None


def bench_decode(args, name):
    import numpy as np
    import torch

    from blitz_scale_amd import kernel as K, workloads as wl
    from blitz_scale_amd._lib import BZ_BF16, BZ_E4M3, BZ_F16, BZ_LAYOUT_HND, BZ_ROPE_NONE, BZ_ROPE_Q_ONLY

    dev = "cuda"
    cfg = dict(wl.CONFIGS[name])
    B, Hq, Hkv, D, P = cfg["batch"], cfg["Hq"], cfg["Hkv"], cfg["D"], args.page_size or cfg["P"]
    theta = cfg["rope_theta"]
    tdt = torch.float16 if cfg["dtype"] == BZ_F16 else torch.bfloat16
    fp8 = cfg["kv_dtype"] == BZ_E4M3
    rng = np.random.default_rng(args.seed)
    if name == "C3":
        ctx = wl.lognormal_ctx(rng, B, 1024.0, args.sigma, 64, 8192)
        ctx_desc = f"lognormal(mean 1024, sigma {args.sigma}) clipped [64,8192]"
    else:
        ctx = wl.ctx_lens_for(cfg, rng)
        ctx_desc = str(cfg["ctx"])
    need = int(((ctx + P - 1) // P).sum())
    pool_pages = int(np.ceil(need * cfg.get("oversub", 1.0)))
    indices, indptr, lpl = wl.page_table_for(ctx, P, pool_pages, rng)
    stride_page, _, _ = wl.strides(BZ_LAYOUT_HND, Hkv, P, D)
    kv_bytes = 1 if fp8 else 2
    plane = pool_pages * stride_page
    L = args.layers or max(2, min(8, int(12e9 // (plane * kv_bytes))))
    steps = args.steps or (400 if name == "C3" else 200)
    warmup = args.warmup if args.warmup is not None else 40

    g = torch.Generator(device=dev)
    g.manual_seed(args.seed)
    k_scale = v_scale = None
    if fp8:
        # N(0,1) values, per-kv-head scale amax/448 with amax taken as 5.5 sigma, stored as e4m3 bytes
        scale = torch.full((Hkv,), 5.5 / 448.0, dtype=torch.float32, device=dev)
        k_scale, v_scale = scale, scale.clone()
        pool = torch.empty(L * plane, dtype=torch.uint8, device=dev)
        chunk = 1 << 26
        for off in range(0, L * plane, chunk):
            n = min(chunk, L * plane - off)
            x = torch.randn(n, dtype=torch.float32, device=dev, generator=g) / (5.5 / 448.0)
            pool[off:off + n] = x.clamp_(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8)
    else:
        pool = torch.empty(L * plane, dtype=tdt, device=dev)
        for l in range(L):
            pool[l * plane:(l + 1) * plane].normal_(generator=g)
    q = torch.randn((B, Hq, D), dtype=tdt, device=dev, generator=g)
    k_new = torch.randn((B, Hkv, D), dtype=tdt, device=dev, generator=g)
    v_new = torch.randn((B, Hkv, D), dtype=tdt, device=dev, generator=g)
    out = torch.empty((B, Hq, D), dtype=tdt, device=dev)

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

    extra = {}
    if name == "C2":  # the layer's RMSNorm and SiLU-gate kernels ride along (hidden 4096, inter 11008)
        h, I = cfg["hidden"], cfg["inter"]
        x = torch.randn((B, h), dtype=tdt, device=dev, generator=g)
        res = torch.randn((B, h), dtype=tdt, device=dev, generator=g)
        w = (1 + 0.02 * torch.randn((h,), device=dev, generator=g)).to(tdt)
        gate_up = torch.randn((B, 2 * I), dtype=tdt, device=dev, generator=g)
        act = torch.empty((B, I), dtype=tdt, device=dev)
        extra = {"hidden": h, "inter": I}

    kev = HipEvents(steps)  # recorded by the library around the decode kernel launch itself

    rope = theta is not None and not args.no_rope

    def attention(stream=None):
        """One layer's append + decode.  One call (two launches: decode kernel over the cached tokens, then the
        kernel that appends the new token, adds its term and folds the split-K partials), or with --two-call
        the reference's two calls (three launches); either way q, k and v stay as the projection left them."""
        if args.two_call:
            K.append_decode_kv_cache(pt, k_new, v_new, rope=rope, rope_theta=theta or 1e4, k_scale=k_scale,
                                     v_scale=v_scale, stream=stream)
            K.batch_decode_attention(handler, q, pt, out, Hq, rope_mode=BZ_ROPE_Q_ONLY if rope else BZ_ROPE_NONE,
                                     rope_theta=theta or 1e4, k_scale=k_scale, v_scale=v_scale, stream=stream)
        else:
            K.decode_step(handler, q, k_new, v_new, pt, out, Hq, rope=rope, rope_theta=theta or 1e4, k_scale=k_scale,
                          v_scale=v_scale, stream=stream)

    def step(i, ev, stream=None):
        pt.set_layer(i % L, pool_pages)
        if ev == "call":      # informational pass: torch events around the attention call(s)
            call_ev[i][0].record()
        elif ev is not None:  # timed pass: the library records a HIP event pair around the decode kernel launch
            handler.set_timing_events(*kev.pair(i))
        attention(stream)
        if ev == "call":
            call_ev[i][1].record()
        if name == "C2":
            K.add_rms_norm(x, res, w, B, h, stream=stream)
            K.silu_and_mul(gate_up, act, B, I, stream=stream)

    eager_ms, _ = timed(step, steps, warmup, torch_events=False)
    handler.set_timing_events(None, None)
    kern_ms = np.array([kev.elapsed_ms(i) for i in range(steps)])
    ncall = min(steps, 100)
    call_ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(ncall)]
    for i in range(ncall):
        step(i, "call")
    torch.cuda.synchronize()
    dec_ms = np.array([a.elapsed_time(b) for a, b in call_ev])

    # ---- the same steps as a layer loop would issue them in production: L consecutive layers' steps recorded
    # into one HIP graph and replayed (no host work between the launches); outputs compared with the eager step
    ms_per_step, graph_note, region_us, device_us = eager_ms, "eager launches (no graph pass)", None, None
    if not args.no_graph:
        step(L - 1, None)
        torch.cuda.synchronize()
        want = out.clone()
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):
            step(0, None, side.cuda_stream)  # warm-up on the capture stream, outside the capture
        torch.cuda.synchronize()
        graphs = {}

        def graph_of(n):
            """n consecutive steps (layer planes 0 .. L-1, cyclically) as one HIP graph"""
            if n not in graphs:
                gr = torch.cuda.CUDAGraph()
                with torch.cuda.graph(gr, stream=side):
                    for l in range(n):
                        step(l % L, None, torch.cuda.current_stream().cuda_stream)
                torch.cuda.synchronize()
                graphs[n] = gr
            return graphs[n]

        # A timed region of exactly `steps` steps: one graph of that many steps while that is a graph of modest
        # size (every graph launch at the start of a region is host time inside the bracket), else whole replays
        # of a 64-step graph and one shorter graph for the rest.
        GN = 64

        def run_steps(n):
            for _ in range(n // GN):
                graph_of(GN).replay()
            if n % GN:
                graph_of(n % GN).replay()

        out.zero_()
        graph_of(L).replay()
        torch.cuda.synchronize()
        same = bool(torch.equal(out.view(torch.int16), want.view(torch.int16)))
        for n in {GN if max(steps, warmup) >= GN else 0, steps % GN, warmup % GN} - {0}:
            graph_of(n)
        replays = steps // GN + (1 if steps % GN else 0)
        # >= 25 graph replays in all, >= 5 timed regions, >= 2000 timed steps: the first hundred steps or so after the
        # idle gap in front of the regions (graph construction) run 1-4 % slower while the memory clocks come up, and
        # that start-up transient should weigh in proportion to a serving loop's steady state, not as a fifth of 25
        # short regions
        regions = max(5, -(-25 // replays), -(-2000 // steps))
        done = torch.cuda.Event()
        dev_ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(regions)]
        run_steps(warmup)
        torch.cuda.synchronize()
        region_ms = []
        for r in range(regions):
            # one timed region: exactly `steps` steps between two device synchronisations.  The host polls an
            # event for the end of the last step before it synchronises, so that the wake-up of a blocked
            # host thread (tens of microseconds) is not counted into a region of a few milliseconds.
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            run_steps(steps)
            done.record()
            while not done.query():
                pass
            torch.cuda.synchronize()
            region_ms.append((time.perf_counter() - t0) * 1e3)
        for r in range(regions):  # the same regions once more between two events on the stream (not part of `value`)
            torch.cuda.synchronize()
            dev_ev[r][0].record()
            run_steps(steps)
            dev_ev[r][1].record()
        torch.cuda.synchronize()
        region_us = np.array(region_ms) / steps  # ms per step of each region; pct() scales to us
        device_us = np.array([a.elapsed_time(b) for a, b in dev_ev]) / steps
        ms_per_step = float(region_us.mean())
        graph_note = (f"HIP graphs of up to {GN} consecutive layers' steps (layer planes cycled); a timed region is exactly "
                      f"{steps} steps ({replays} graph launches) between two device synchronisations by the host's "
                      f"clock (graph launch latency included), value = mean of {regions} regions "
                      f"after {warmup} warm-up steps; last layer's output bit-identical to the eager step: {same}")
    alg_bytes = wl.decode_algorithmic_bytes(ctx, Hq, Hkv, D, kv_bytes, 2, P)
    achieved = alg_bytes / (float(kern_ms.mean()) * 1e-3) / 1e9
    traffic = measured_traffic(name, args)
    frac_call = alg_bytes / (float(dec_ms.mean()) * 1e-3) / 1e9 / HBM_PEAK_GBPS
    frac_step = alg_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBPS
    res_json = {
        "metric": "paged_decode_us_per_step", "value": round(ms_per_step * 1e3, 3), "unit": "us/step",
        "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": round(ms_per_step, 6),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": ("bf16" if tdt == torch.bfloat16 else "f16") + (" q, e4m3 kv" if fp8 else ""), "data": "synthetic",
        "config": dict({
            "workload": {"C2": "C2: Llama-2-7B-shaped MHA decode step of one layer (fused RoPE+append, batch decode, "
                               "add+RMSNorm, SiLU-gate)",
                         "C3": "C3: Llama-3-8B-shaped GQA paged decode, one layer per step (KV append with RoPE + batch decode)",
                         "C5": "C5: Llama-3-70B-shaped GQA decode with e4m3 KV, one layer per step (quantising append, "
                               "batch decode)"}[name],
            "batch": B, "num_qo_heads": Hq, "num_kv_heads": Hkv, "head_dim": D, "page_size": P, "ctx": ctx_desc,
            "sum_ctx": int(ctx.sum()), "max_ctx": int(ctx.max()), "pool_pages_per_layer": pool_pages,
            "layer_planes_cycled": L, "kv_layout": "HND", "rope_theta": theta, "split_tokens": args.split_tokens,
            "seed": hex(args.seed), "plan": info}, **extra),
        "tokens_per_s": round(B / (ms_per_step * 1e-3), 1),
        "plan_ms_per_model_step": round(plan_ms, 4),
        "step_launch": graph_note,
        "step_calls": "append_decode_kv_cache + batch_decode_attention (3 launches)" if args.two_call
                      else "bz_decode_step (2 launches: decode kernel, then append + new-token term + split-K fold)"
                      if handler.step_form() == "one_call"
                      else "bz_decode_step (its choice for this plan: append, decode kernel, split-K combine)",
        "value_method": "graph replay (a layer loop without host work between the launches); the same steps launched "
                        "one by one from Python are eager_us_per_step" if not args.no_graph else "eager launches",
        "step_us_per_region": pct(region_us) if region_us is not None else None,
        "step_us_per_region_on_device": pct(device_us) if device_us is not None else None,
        # (the start-up transient after the idle gap in front of the regions, shown as it is)
        "step_us_first_regions": [round(float(x) * 1e3, 2) for x in region_us[:6]] if region_us is not None else None,
        "eager_us_per_step": round(eager_ms * 1e3, 3),
        "decode_call_us": pct(dec_ms),
        "decode_kernel_us": pct(kern_ms),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "frac_call": round(frac_call, 4), "frac_step": round(frac_step, 4),
                     "frac_step_device": round(alg_bytes / (float(device_us.mean()) * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)
                     if device_us is not None else None,
                     "traffic": traffic,
                     "traffic_source": "offline: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this workload "
                                       "(profiles/), not measured in this run",
                     "algorithmic_bytes_per_launch": int(alg_bytes),
                     "kernel": "decode kernel (bz::decode_mfma_kernel): `achieved` and `frac` are the algorithmic bytes "
                               "of the step over that kernel's own duration (HIP events recorded by the library on the "
                               "launch stream right around its launch); frac_call is the same bytes over the whole "
                               "attention call(s) of the step (decode_call_us: every launch needed for the result), "
                               "frac_step over ms_per_step (the host's clock around the timed regions), frac_step_device "
                               "over the same regions between two events on the stream (first kernel's start to last "
                               "kernel's end: without the host's launch latency at the head of a region)"},
    }
    if not args.no_cpu_baseline:
        import oracle  # the checker, used here only as the timed CPU baseline
        sb = B if name != "C5" else 16  # bounded sample: C5 in full would be minutes of CPU time
        odt = oracle.E4M3 if fp8 else (oracle.F16 if tdt == torch.float16 else oracle.BF16)
        qh = q.view(torch.int16).cpu().numpy().view(np.uint16)
        sp, sn, sh = wl.strides(BZ_LAYOUT_HND, Hkv, P, D)
        ks = k_scale.cpu().numpy() if fp8 else None
        vs = v_scale.cpu().numpy() if fp8 else None
        qdt = oracle.F16 if tdt == torch.float16 else oracle.BF16
        # the timed call once more on layer plane 0, then the checker over the very bits the device cached
        pt.set_layer(0, pool_pages)
        attention()
        out32 = torch.empty((B, Hq, D), dtype=torch.float32, device=dev)
        if not args.two_call:
            K.decode_step(handler, q, k_new, v_new, pt, out32, Hq, rope=rope, rope_theta=theta or 1e4, k_scale=k_scale,
                          v_scale=v_scale)
        else:
            K.batch_decode_attention(handler, q, pt, out32, Hq, rope_mode=BZ_ROPE_Q_ONLY if rope else BZ_ROPE_NONE,
                                     rope_theta=theta or 1e4, k_scale=k_scale, v_scale=v_scale)
        torch.cuda.synchronize()
        plane0 = pool[:plane]
        plane0 = plane0.cpu().numpy() if fp8 else plane0.view(torch.int16).cpu().numpy().view(np.uint16)
        kv = oracle.PagedKV(plane0, plane0[sp // 2:], indices[:int(indptr[sb])], indptr[:sb + 1], lpl[:sb], P, Hkv, D, sp,
                            sn, sh, odt)
        reps, t0 = 0, time.perf_counter()
        while reps == 0 or (time.perf_counter() - t0 < 10.0 and reps < 200):  # about 10 s of CPU work
            ref = oracle.batch_decode(qh[:sb], qdt, kv, Hq, rope_mode=oracle.ROPE_Q_ONLY if rope else oracle.ROPE_NONE,
                                      rope_theta=theta or 1e4, k_scale=ks, v_scale=vs, parallel=True)
            reps += 1
        cpu_s = (time.perf_counter() - t0) / reps
        res_json["max_abs_err_vs_cpu"] = float(np.abs(out[:sb].float().cpu().numpy() - ref).max())
        res_json["max_abs_err_vs_cpu_f32_out"] = float(np.abs(out32[:sb].cpu().numpy() - ref).max())
        res_json["checked"] = ("the output of the timed call (append with RoPE, then attention with q rotated inside), "
                               f"first {sb} sequences, against the CPU checker run on the pool as the call left it: "
                               "max_abs_err_vs_cpu for the 16-bit output the timed steps write, ..._f32_out for the same "
                               "call with an fp32 output")
        scale_up = float(ctx.sum()) / float(ctx[:sb].sum())
        res_json["cpu_baseline"] = {
            "value": round(cpu_s * scale_up * 1e6, 1), "unit": "us/step", "cores": oracle.num_threads(True),
            "kind": "port",
            "sample": f"batch decode (q rotated, no append) of the first {sb} of {B} sequences, mean of {reps} repetitions "
                      f"({cpu_s:.2f} s each), OpenMP over sequences, scaled by total/sample context tokens ({scale_up:.2f}x)",
            "host_cpus": os.cpu_count()}
    return res_json


def bench_prefill(args):
    import numpy as np
    import torch

    from blitz_scale_amd import kernel as K, workloads as wl
    from blitz_scale_amd._lib import BZ_LAYOUT_HND, BZ_PREFILL_BF16_HEAD_TAIL, BZ_ROPE_NONE, BZ_ROPE_Q_ONLY

    dev = "cuda"
    tdt = torch.float16 if args.prefill_dtype == "f16" else torch.bfloat16
    cfg = wl.CONFIGS["C4"]
    B, Hq, Hkv, D, P, theta = cfg["batch"], cfg["Hq"], cfg["Hkv"], cfg["D"], cfg["P"], cfg["rope_theta"]
    rng = np.random.default_rng(args.seed)
    lens = wl.ctx_lens_for(cfg, rng)
    if args.prefill_lens:
        lens = np.array([int(x.split("x")[-1]) for x in args.prefill_lens.split(",")
                         for _ in range(int(x.split("x")[0]) if "x" in x else 1)], dtype=lens.dtype)
        B = len(lens)
    if args.prefill_heads:
        Hq, Hkv = (int(x) for x in args.prefill_heads.split("/"))
    diagnostic = bool(args.prefill_lens or args.prefill_heads)
    indptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    N = int(indptr[-1])
    # page table with the reference's len+1 reservation, seeded page placement
    need = int(((lens + 1 + P - 1) // P).sum())
    pool_pages = int(np.ceil(need * cfg["oversub"]))
    indices, pindptr, lpl = wl.page_table_for(lens + 1, P, pool_pages, rng)
    stride_page, _, _ = wl.strides(BZ_LAYOUT_HND, Hkv, P, D)
    # The clock governor needs some tens of milliseconds of load before it settles (with 20 steps of 1.3 ms
    # the same kernel measures 12-15 % slower), hence a longer warm-up and run than the decode workloads.
    steps = args.steps or 300
    warmup = args.warmup if args.warmup is not None else 60
    g = torch.Generator(device=dev)
    g.manual_seed(args.seed)
    q = torch.randn((N, Hq, D), dtype=tdt, device=dev, generator=g)
    k = torch.randn((N, Hkv, D), dtype=tdt, device=dev, generator=g)
    v = torch.randn((N, Hkv, D), dtype=tdt, device=dev, generator=g)
    out = torch.empty_like(q)
    pool = torch.zeros(pool_pages * stride_page, dtype=tdt, device=dev)
    pt = K.PageTable(B, P, Hkv, D, pool, layout=BZ_LAYOUT_HND)
    pt.indices, pt.indptr, pt.last_page_len = indices, pindptr, lpl
    pt.upload()
    ip = torch.from_numpy(indptr).to(dev)
    float_ws = torch.empty(128 << 20, dtype=torch.uint8, device=dev)
    int_ws = torch.empty(8 << 20, dtype=torch.uint8, device=dev)
    handler = K.BatchPrefillRaggedHandler()
    if args.prefill_dtype == "bf16-head-tail":
        handler.set_bf16_mode(BZ_PREFILL_BF16_HEAD_TAIL)
    t0 = time.perf_counter()
    for _ in range(10):
        handler.plan(float_ws, float_ws.numel(), int_ws, int_ws.numel(), indptr, indptr, B, Hq, Hkv, D, P)
    torch.cuda.synchronize()
    plan_ms = (time.perf_counter() - t0) / 10 * 1e3

    def step(i, ev):
        # page store with K rotated on the way (into the pages and in place), then attention, which rotates q in
        # registers.  k is rotated again every step; rotations keep the N(0,1) statistics, so the work is
        # the same each time.
        if args.q_rope == "store":
            K.store_prefill_kv_cache(pt, k, v, ip, num_tokens=N, q=q, num_qo_heads=Hq, rope=True, rope_theta=theta)
        else:
            K.store_prefill_kv_cache(pt, k, v, ip, num_tokens=N, rope=2, rope_theta=theta)
        if ev is not None:  # torch events around the whole attention call, the library's own pair around its kernel
            ev[0].record()
            handler.set_timing_events(*kev.pair(i))
        K.batch_prefill_attention(handler, q, ip, k, v, ip, out, B, Hq, Hkv, D, causal=True, rope_theta=theta,
                                  rope_mode=BZ_ROPE_NONE if args.q_rope == "store" else BZ_ROPE_Q_ONLY)
        if ev is not None:
            ev[1].record()

    kev = HipEvents(steps)  # recorded by the library right around the attention kernel's launch
    ms_per_step, call_ms = timed(step, steps, warmup)
    handler.set_timing_events(None, None)
    att_ms = np.array([kev.elapsed_ms(i) for i in range(steps)])
    flops = float(sum(Hq * 4 * D * int(l) * (int(l) + 1) / 2 for l in lens))
    achieved = flops / (float(att_ms.mean()) * 1e-3) / 1e12
    res_json = {
        "metric": "ragged_causal_prefill_ms_per_step", "value": round(ms_per_step, 4), "unit": "ms/step",
        "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": round(ms_per_step, 6),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": args.prefill_dtype, "data": "synthetic",
        "config": {"workload": "C4: Llama-2-13B-shaped ragged causal prefill with RoPE + KV page store, one layer per step"
                               if not diagnostic else
                               f"C4's flow with prompt lengths {args.prefill_lens or 'as configured'} and {Hq}/{Hkv} heads "
                               "(diagnostic, not the configuration's)",
                   "batch": B, "num_qo_heads": Hq, "num_kv_heads": Hkv, "head_dim": D, "page_size": P,
                   "lens": "uniform[128,4096]" if not args.prefill_lens else args.prefill_lens, "tokens": N, "pool_pages": pool_pages, "rope_theta": theta,
                   "q_rotated_by": args.q_rope,
                   "seed": hex(args.seed)},
        "tokens_per_s": round(N / (ms_per_step * 1e-3), 1),
        "plan_ms_per_model_step": round(plan_ms, 4),
        "attention_kernel_us": pct(att_ms),
        "attention_call_us": pct(call_ms),
        "roofline": {"bound": "mfma", "achieved": round(achieved, 1), "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / MFMA_PEAK_TFLOPS, 4), "traffic": measured_traffic("C4", args),
                     "traffic_source": "offline: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this workload "
                                       "(profiles/), not measured in this run",
                     "algorithmic_flops_per_launch": flops,
                     "kernel": "ragged causal prefill attention kernel (bz::prefill_kernel): HIP events recorded by the library "
                               "on the launch stream right around its launch (attention_kernel_us); attention_call_us is "
                               "the whole call, with the kernel that writes the angle table of the q rotation in front"},
    }
    if not args.no_cpu_baseline:
        import oracle
        rows = np.sort(rng.choice(N, size=min(N, 6144), replace=False)).astype(np.int32)  # about 10 s of CPU work
        qh, kh, vh = (t.view(torch.int16).cpu().numpy().view(np.uint16) for t in (q, k, v))
        K.batch_prefill_attention(handler, q, ip, k, v, ip, out, B, Hq, Hkv, D, causal=True, rope_mode=BZ_ROPE_NONE)
        torch.cuda.synchronize()
        t0 = time.perf_counter()  # (checked without RoPE on either side: the same q and k bits, used as they are)
        ref = oracle.batch_prefill_ragged(qh, kh, vh, oracle.F16 if tdt == torch.float16 else oracle.BF16, indptr, Hq, Hkv, D,
                                          causal=True, rows=rows, parallel=True)
        cpu_s = time.perf_counter() - t0
        res_json["max_abs_err_vs_cpu"] = float(np.abs(out[torch.from_numpy(rows.astype(np.int64)).to(dev)].float().cpu().numpy() - ref).max())
        seen = sum(int(r - indptr[np.searchsorted(indptr, r, side="right") - 1]) + 1 for r in rows)
        total = sum(int(l) * (int(l) + 1) // 2 for l in lens)
        res_json["cpu_baseline"] = {
            "value": round(cpu_s * total / seen * 1e3, 1), "unit": "ms/step", "cores": oracle.num_threads(True),
            "kind": "port",
            "sample": f"{len(rows)} seeded rows x all heads ({seen} of {total} row-key pairs), attention only, OpenMP "
                      f"over rows, {cpu_s:.2f} s measured, scaled by pairs",
            "host_cpus": os.cpu_count()}
    return res_json


def bench_ends(args):
    """The row gathers and the greedy argmax either side of the layer loop (embedding, gather_last_token,
    batch_find_max) at Llama-3-8B sizes: each is one pass over its rows, reported in us and GB/s."""
    import numpy as np
    import torch

    import oracle
    from blitz_scale_amd import kernel as K

    vocab, hidden, ntok, batch = 128256, 4096, 8192, 128
    rng = np.random.default_rng(args.seed)
    g = torch.Generator(device="cuda")
    g.manual_seed(args.seed)
    w = torch.randn((vocab, hidden), dtype=torch.bfloat16, device="cuda", generator=g)
    ids = torch.from_numpy(rng.integers(0, vocab, size=ntok).astype(np.int32)).cuda()
    rows = torch.empty((ntok, hidden), dtype=torch.bfloat16, device="cuda")
    indptr = torch.from_numpy((np.arange(batch + 1) * (ntok // batch)).astype(np.int32)).cuda()
    last = torch.empty((batch, hidden), dtype=torch.bfloat16, device="cuda")
    logits = torch.randn((batch, vocab), dtype=torch.bfloat16, device="cuda", generator=g)
    arg = torch.empty(batch, dtype=torch.int32, device="cuda")
    steps = args.steps or 200
    warmup = args.warmup if args.warmup is not None else 20
    ops = {
        "embedding": (lambda: K.embedding(rows, ids, w, ntok, hidden), 2 * ntok * hidden * 2 + 4 * ntok),
        "gather_last_token": (lambda: K.gather_last_token(last, rows, indptr, ntok, batch, hidden),
                              2 * batch * hidden * 2 + 4 * (batch + 1)),
        "batch_find_max": (lambda: K.batch_find_max(arg, logits, batch, vocab), batch * vocab * 2 + 4 * batch),
    }
    out = {}
    total_ms = 0.0
    for name, (fn, nbytes) in ops.items():
        ms, ev = timed(lambda i, e: (e[0].record(), fn(), e[1].record()) if e is not None else fn(), steps, warmup)
        out[name] = {"us": pct(ev)["mean"], "algorithmic_bytes": nbytes,
                     "GB_per_s": round(nbytes / (float(ev.mean()) * 1e-3) / 1e9, 1)}
        total_ms += ms
    # The figures above are one eager call between two events: launch and event latency included, and the
    # operands of the repeated call come out of the last-level cache.  The kernels by themselves, from HBM:
    # ten calls on ten different inputs (330 MB of logits, 10 x 8192 different table rows) replayed from one
    # HIP graph, time per call.
    R = 10
    logits_r = [logits] + [torch.randn((batch, vocab), dtype=torch.bfloat16, device="cuda", generator=g) for _ in range(R - 1)]
    ids_r = [torch.from_numpy(rng.permutation(vocab)[:ntok].astype(np.int32)).cuda() for _ in range(R)]
    rows_r = [rows] + [torch.empty_like(rows) for _ in range(R - 1)]
    graph_ops = {
        "embedding": lambda j, s: K.embedding(rows_r[j], ids_r[j], w, ntok, hidden, stream=s),
        "gather_last_token": lambda j, s: K.gather_last_token(last, rows_r[j], indptr, ntok, batch, hidden, stream=s),
        "batch_find_max": lambda j, s: K.batch_find_max(arg, logits_r[j], batch, vocab, stream=s),
    }
    side = torch.cuda.Stream()
    for name, fn in graph_ops.items():
        graph = torch.cuda.CUDAGraph()
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            for j in range(R):
                fn(j, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        ms, _ = timed(lambda i, e: graph.replay(), max(steps // 4, 10), 3, torch_events=False)
        out[name]["us_in_graph_from_hbm"] = round(ms * 1e3 / R, 3)
        out[name]["GB_per_s_in_graph"] = round(out[name]["algorithmic_bytes"] / (ms * 1e-3 / R) / 1e9, 1)
    K.batch_find_max(arg, logits, batch, vocab)
    # parity on the spot (bit-exact)
    torch.cuda.synchronize()
    lg = logits.view(torch.int16).cpu().numpy().view(np.uint16)
    from blitz_scale_amd._lib import BZ_BF16
    ok = bool(np.array_equal(arg.cpu().numpy().view(np.uint32), oracle.batch_find_max(lg, BZ_BF16)))
    dom = out["batch_find_max"]
    return {"metric": "model_ends_us_per_step", "value": round(total_ms * 1e3, 3), "unit": "us/step", "n_gpus": 1,
            "steps": steps, "warmup": warmup, "ms_per_step": round(total_ms, 6), "higher_is_better": False,
            "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": {"workload": "ENDS: embedding of 8192 tokens, last-token gather and greedy argmax for 128 "
                                   "sequences, Llama-3-8B sizes (hidden 4096, vocabulary 128256)"},
            "ops": out, "argmax_bit_exact_vs_cpu": ok,
            "roofline": {"bound": "hbm", "achieved": dom["GB_per_s_in_graph"], "peak": 8000.0, "unit": "GB/s",
                         "frac": round(dom["GB_per_s_in_graph"] / 8000.0, 4), "traffic": None,
                         "kernel": "bz::batch_find_max_kernel (the largest of the three), time per call in a "
                                   "replayed graph of ten calls over ten different inputs"}}


def bench_migrate(args):
    """KV migration payload of a prefilled batch: pack every (page, layer) of 16 prompts of 2048 tokens,
    Llama-3-8B geometry (32 layers, 8 kv heads, D 128, P 16, bf16: 128 KiB per token), into one buffer
    and scatter it into other pages of a second pool.  Bytes: payload read + payload written, per pass."""
    import numpy as np
    import torch

    from blitz_scale_amd import kernel as K
    from blitz_scale_amd._lib import BZ_E4M3

    layers, Hkv, P, D, nreq, ntok = 32, 8, 16, 128, 16, 2048
    sp = 2 * Hkv * P * D
    n = nreq * ntok // P
    max_pages = 2 * n
    rng = np.random.default_rng(args.seed)
    g = torch.Generator(device="cuda")
    g.manual_seed(args.seed)
    src = torch.randn(layers * max_pages * sp, dtype=torch.bfloat16, device="cuda", generator=g)
    dst = torch.zeros_like(src)
    spt, dpt = K.PageTable(nreq, P, Hkv, D, src), K.PageTable(nreq, P, Hkv, D, dst)
    src_ids = torch.from_numpy(rng.permutation(max_pages)[:n].astype(np.int32)).cuda()
    dst_ids = torch.from_numpy(rng.permutation(max_pages)[:n].astype(np.int32)).cuda()
    payload = K.kv_wire_bytes(spt, n, layers)
    wire = torch.empty(payload, dtype=torch.uint8, device="cuda")
    ks = torch.full((layers, Hkv), 5.0 / 448, dtype=torch.float32, device="cuda")
    steps = args.steps or 20
    warmup = args.warmup if args.warmup is not None else 3
    ops = {
        "pack": (lambda: K.pack_kv_pages(spt, max_pages, src_ids, 0, layers, wire), 2 * payload),
        "unpack": (lambda: K.unpack_kv_pages(dpt, max_pages, dst_ids, 0, layers, wire), 2 * payload),
        "pack_e4m3_wire": (lambda: K.pack_kv_pages(spt, max_pages, src_ids, 0, layers, wire, wire_dtype=BZ_E4M3,
                                                   k_scale=ks, v_scale=ks), payload + payload // 2),
    }
    out = {}
    for name, (fn, nbytes) in ops.items():
        ms, ev = timed(lambda i, e: (e[0].record(), fn(), e[1].record()) if e is not None else fn(), steps, warmup)
        out[name] = {"us": pct(ev)["mean"], "algorithmic_bytes": nbytes,
                     "GB_per_s": round(nbytes / (float(ev.mean()) * 1e-3) / 1e9, 1)}
    # parity on the spot: the receiver's pages hold the sender's bits
    ops["pack"][0]()
    ops["unpack"][0]()
    torch.cuda.synchronize()
    s3 = src.view(torch.int16).view(layers, max_pages, sp)
    d3 = dst.view(torch.int16).view(layers, max_pages, sp)
    ok = bool(torch.equal(s3[:, src_ids.long()], d3[:, dst_ids.long()]))
    ms = (out["pack"]["us"] + out["unpack"]["us"]) * 1e-3
    dom = out["pack"]
    return {"metric": "kv_migration_pack_unpack_ms", "value": round(ms, 4), "unit": "ms/step", "n_gpus": 1,
            "steps": steps, "warmup": warmup, "ms_per_step": round(ms, 6), "higher_is_better": False,
            "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": {"workload": "MIGRATE: wire payload of 16 prompts x 2048 tokens, Llama-3-8B KV geometry "
                                   f"(32 layers, {n} pages, {payload / 2**30:.1f} GiB): pack on the sender + unpack "
                                   "on the receiver"},
            "ops": out, "round_trip_bit_exact": ok,
            "roofline": {"bound": "hbm", "achieved": dom["GB_per_s"], "peak": 8000.0, "unit": "GB/s",
                         "frac": round(dom["GB_per_s"] / 8000.0, 4), "traffic": None,
                         "kernel": "bz::wire_kernel (pack), payload read + payload written"}}


def bench_layers(args):
    """Small-batch decode through all 32 layers of a Llama-3-8B-shaped model (attention part of each layer:
    fused RoPE + KV append, paged decode), launched eagerly and replayed from one HIP graph.  At this
    size every kernel is shorter than a launch, so the step is bound by the launches, which is what the
    graph removes.  One plan and one page-table upload per step serve all layers, as in the reference
    (src/model/llama.h:363-375)."""
    import numpy as np
    import torch

    from blitz_scale_amd import kernel as K, workloads as wl
    from blitz_scale_amd._lib import BZ_LAYOUT_HND, BZ_ROPE_NONE

    layers, B, Hq, Hkv, D, P, ctx = 32, 8, 32, 8, 128, 16, 1024
    rng = np.random.default_rng(args.seed)
    lens = np.full(B, ctx, np.int64)
    max_pages = 2 * B * (ctx // P + 1)
    indices, indptr, lpl = wl.page_table_for(lens, P, max_pages, rng)
    stride_page, _, _ = wl.strides(BZ_LAYOUT_HND, Hkv, P, D)
    g = torch.Generator(device="cuda")
    g.manual_seed(args.seed)
    pool = torch.randn(layers * max_pages * stride_page, dtype=torch.bfloat16, device="cuda", generator=g)
    q = torch.randn((layers, B, Hq, D), dtype=torch.bfloat16, device="cuda", generator=g)
    k = torch.randn((layers, B, Hkv, D), dtype=torch.bfloat16, device="cuda", generator=g)
    v = torch.randn((layers, B, Hkv, D), dtype=torch.bfloat16, device="cuda", generator=g)
    q_raw = q.clone()
    out = torch.empty_like(q)
    pts = []
    for l in range(layers):
        pt = K.PageTable(B, P, Hkv, D, pool, layout=BZ_LAYOUT_HND)
        pt.set_layer(l, max_pages)
        pt.indices, pt.indptr, pt.last_page_len = indices, indptr, lpl
        pts.append(pt)
    pts[0].upload()
    for pt in pts[1:]:
        pt.indices_d, pt.indptr_d, pt.last_page_len_d = pts[0].indices_d, pts[0].indptr_d, pts[0].last_page_len_d
    float_ws = torch.empty(128 << 20, dtype=torch.uint8, device="cuda")
    int_ws = torch.empty(8 << 20, dtype=torch.uint8, device="cuda")
    handler = K.BlitzBatchDecodeHandler()
    handler.plan(float_ws, float_ws.numel(), int_ws, int_ws.numel(), indptr, lpl, B, Hq, Hkv, D, P,
                 split_tokens=args.split_tokens)

    def step_layers(stream=None):
        for l in range(layers):
            if args.two_call:  # the reference's two calls: append (rotates q and k in place), then attention
                K.append_decode_kv_cache(pts[l], k[l], v[l], q=q[l], num_qo_heads=Hq, rope=True, rope_theta=5e5,
                                         stream=stream)
                K.batch_decode_attention(handler, q[l], pts[l], out[l], Hq, rope_mode=BZ_ROPE_NONE, stream=stream)
            else:              # both as one call (two launches; q is rotated inside the kernels and left as it is)
                K.decode_step(handler, q[l], k[l], v[l], pts[l], out[l], Hq, rope=True, rope_theta=5e5, stream=stream)

    steps = args.steps or 50
    warmup = args.warmup if args.warmup is not None else 5
    eager_ms, _ = timed(lambda i, e: step_layers(), steps, warmup, torch_events=False)
    q.copy_(q_raw)
    torch.cuda.synchronize()
    step_layers()
    torch.cuda.synchronize()
    want = out.clone()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    q.copy_(q_raw)
    torch.cuda.synchronize()
    with torch.cuda.graph(graph, stream=side):
        step_layers(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    q.copy_(q_raw)
    out.zero_()
    graph.replay()
    torch.cuda.synchronize()
    same = bool(torch.equal(out.view(torch.int16), want.view(torch.int16)))
    graph_ms, _ = timed(lambda i, e: graph.replay(), steps, warmup, torch_events=False)

    # The same replay with the reference's per-step host work in front of it (page-table upload and
    # plan(), src/model/llama.h:363-375, src/blitz/stub.h:1288-1313) ...
    def host_then_replay(i, e):
        pts[0].upload()
        handler.plan(float_ws, float_ws.numel(), int_ws, int_ws.numel(), indptr, lpl, B, Hq, Hkv, D, P,
                     split_tokens=args.split_tokens)
        graph.replay()
    host_ms, _ = timed(host_then_replay, steps, warmup, torch_events=False)
    t0 = time.perf_counter()
    for _ in range(200):
        handler.plan(float_ws, float_ws.numel(), int_ws, int_ws.numel(), indptr, lpl, B, Hq, Hkv, D, P,
                     split_tokens=args.split_tokens)
    plan_us = (time.perf_counter() - t0) / 200 * 1e6
    torch.cuda.synchronize()
    # ... and with the table taken as running `horizon` steps ahead of the present (same table and plan:
    # the measured lengths are the state at the end of the horizon): one upload and one plan serve
    # `horizon` steps, a device counter says how far the present lags, and the replayed graph ends by
    # counting it down.  Nothing but graph.replay() happens on the host inside the horizon.
    horizon = 32
    ahead = torch.tensor([horizon - 1], dtype=torch.int32, device="cuda")
    for pt in pts:
        pt.steps_ahead_d = ahead

    def step_ahead(stream=None):
        step_layers(stream)
        K.steps_ahead_advance(ahead, stream=stream)

    torch.cuda.synchronize()
    graph2 = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph2, stream=side):
        step_ahead(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()

    def replay_ahead(i, e):
        if i % horizon == 0:  # the host's turn, once per horizon: grow the table, upload, plan, reset the counter
            pts[0].upload()
            for pt in pts:
                pt.indices_d, pt.indptr_d, pt.last_page_len_d = (pts[0].indices_d, pts[0].indptr_d,
                                                                 pts[0].last_page_len_d)
            handler.plan(float_ws, float_ws.numel(), int_ws, int_ws.numel(), indptr, lpl, B, Hq, Hkv, D, P,
                         split_tokens=args.split_tokens)
            ahead.fill_(horizon - 1)
        graph2.replay()
    ahead_ms, _ = timed(replay_ahead, max(steps, 2 * horizon), warmup, torch_events=False)
    ahead_only_ms, _ = timed(lambda i, e: graph2.replay(), steps, warmup, torch_events=False)
    kv_bytes = layers * B * ctx * 2 * Hkv * D * 2
    return {"metric": "small_batch_decode_32_layers_us", "value": round(graph_ms * 1e3, 2), "unit": "us/step",
            "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": round(graph_ms, 6),
            "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": {"workload": "LAYERS: attention part (fused RoPE + append, paged decode) of 32 Llama-3-8B "
                                   f"layers, batch {B}, context {ctx}, one plan per step; value = HIP-graph replay",
                       "calls_per_layer": "append + attention" if args.two_call else "decode_step"},
            "eager_us_per_step": round(eager_ms * 1e3, 2), "graph_us_per_step": round(graph_ms * 1e3, 2),
            "us_per_layer": {"eager": round(eager_ms * 1e3 / layers, 2), "graph": round(graph_ms * 1e3 / layers, 2)},
            "graph_replay_bit_exact_vs_eager": same,
            "with_host_work_us_per_step": {"upload_and_plan_every_step": round(host_ms * 1e3, 2),
                                           f"table_{horizon}_steps_ahead": round(ahead_ms * 1e3, 2),
                                           "replay_alone_with_counter": round(ahead_only_ms * 1e3, 2),
                                           "plan_call_host_us": round(plan_us, 2)},
            "roofline": {"bound": "hbm", "achieved": round(kv_bytes / (graph_ms * 1e-3) / 1e9, 1), "peak": 8000.0,
                         "unit": "GB/s", "frac": round(kv_bytes / (graph_ms * 1e-3) / 1e9 / 8000.0, 4), "traffic": None,
                         "kernel": "whole replayed step (launch-latency bound at this size, not a kernel figure)"}}


def bench_rawk(args):
    """A cache that holds K as the projection left it (the reference's convention, kRoPELlama inside every decode
    call, src/kernel/attention_decode.cu:35): 128 sequences of 1024 tokens, Llama-3-8B heads, bf16.  Three figures:
    the decode call that rotates every cached K row itself (BZ_ROPE_FULL), the one pass that converts the cache to
    the rotated-K convention (bz_rope_cached_k), and the decode call over the converted cache (BZ_ROPE_Q_ONLY)."""
    import numpy as np
    import torch

    import oracle
    from blitz_scale_amd import kernel as K, workloads as wl
    from blitz_scale_amd._lib import BZ_LAYOUT_HND, BZ_ROPE_FULL, BZ_ROPE_Q_ONLY

    B, Hq, Hkv, D, P, ctx_len, theta = 128, 32, 8, 128, 16, 1024, 5e5
    rng = np.random.default_rng(args.seed)
    ctx = np.full(B, ctx_len)
    pool_pages = B * ctx_len // P
    indices, indptr, lpl = wl.page_table_for(ctx, P, pool_pages, rng)
    stride_page, sn, sh = wl.strides(BZ_LAYOUT_HND, Hkv, P, D)
    g = torch.Generator(device="cuda")
    g.manual_seed(args.seed)
    L = 4  # planes cycled so that no call finds its K/V in a cache
    pool = torch.randn(L * pool_pages * stride_page, dtype=torch.bfloat16, device="cuda", generator=g)
    raw0 = pool[:pool_pages * stride_page].clone()
    q = torch.randn((B, Hq, D), dtype=torch.bfloat16, device="cuda", generator=g)
    out = torch.empty((B, Hq, D), dtype=torch.float32, device="cuda")
    pt = K.PageTable(B, P, Hkv, D, pool, layout=BZ_LAYOUT_HND)
    pt.indices, pt.indptr, pt.last_page_len = indices, indptr, lpl
    pt.upload()
    float_ws = torch.empty(128 << 20, dtype=torch.uint8, device="cuda")
    int_ws = torch.empty(8 << 20, dtype=torch.uint8, device="cuda")
    handler = K.BlitzBatchDecodeHandler()
    handler.plan(float_ws, float_ws.numel(), int_ws, int_ws.numel(), indptr, lpl, B, Hq, Hkv, D, P)
    steps = args.steps or 40
    warmup = args.warmup if args.warmup is not None else 8
    kv_bytes = float(B * ctx_len * Hkv * D * 2 * 2)

    def run(fn):
        def step(i, e):
            pt.set_layer(i % L, pool_pages)
            if e is not None:
                e[0].record()
            fn()
            if e is not None:
                e[1].record()
        _, ev = timed(step, steps, warmup)
        return ev

    full = run(lambda: K.batch_decode_attention(handler, q, pt, out, Hq, rope_mode=BZ_ROPE_FULL, rope_theta=theta))
    pt.set_layer(0, pool_pages)
    K.batch_decode_attention(handler, q, pt, out, Hq, rope_mode=BZ_ROPE_FULL, rope_theta=theta)
    torch.cuda.synchronize()
    out_full = out.clone()
    # (a rotation keeps the magnitude of a row, so the pass can be timed over and over on the same planes)
    conv = run(lambda: K.rope_cached_k(pt, rope_theta=theta))
    pool[:pool_pages * stride_page].copy_(raw0)
    pt.set_layer(0, pool_pages)
    K.rope_cached_k(pt, rope_theta=theta)  # plane 0: the raw cache, converted once (the other planes only feed the timing)
    q_only = run(lambda: K.batch_decode_attention(handler, q, pt, out, Hq, rope_mode=BZ_ROPE_Q_ONLY, rope_theta=theta))
    pt.set_layer(0, pool_pages)
    K.batch_decode_attention(handler, q, pt, out, Hq, rope_mode=BZ_ROPE_Q_ONLY, rope_theta=theta)
    torch.cuda.synchronize()
    res = {"metric": "raw_k_cache_decode_us_per_call", "value": pct(full)["mean"], "unit": "us/call", "n_gpus": 1, "steps": steps,
           "warmup": warmup, "ms_per_step": round(float(full.mean()), 6), "higher_is_better": False, "scaling": "weak",
           "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
           "config": {"workload": "RAWK: decode over a cache with K as projected (the reference's kRoPELlama convention), "
                                  "128 sequences x 1024 tokens, 32/8 heads, head_dim 128, page 16"},
           "decode_rope_full_us": pct(full), "convert_cache_once_us": pct(conv), "decode_q_only_after_conversion_us": pct(q_only),
           "GB_per_s": {"decode_rope_full": round(kv_bytes / float(full.mean()) / 1e6, 1),
                        "convert_cache_once (K read + written)": round(kv_bytes / float(conv.mean()) / 1e6, 1),
                        "decode_q_only_after_conversion": round(kv_bytes / float(q_only.mean()) / 1e6, 1)},
           "max_abs_diff_between_the_two_routes": float((out - out_full).abs().max()),
           "roofline": {"bound": "hbm", "achieved": round(kv_bytes / float(full.mean()) / 1e6, 1), "peak": HBM_PEAK_GBPS,
                        "unit": "GB/s", "frac": round(kv_bytes / float(full.mean()) / 1e6 / HBM_PEAK_GBPS, 4), "traffic": None,
                        "kernel": "bz_batch_decode with BZ_ROPE_FULL (general kernel, angles from a table); K and V bytes of "
                                  "the batch over the call's duration (torch events)"}}
    if not args.no_cpu_baseline:
        sb = 16
        plane0 = raw0.view(torch.int16).cpu().numpy().view(np.uint16)
        kv = oracle.PagedKV(plane0, plane0[stride_page // 2:], indices[:int(indptr[sb])], indptr[:sb + 1], lpl[:sb], P, Hkv, D,
                            stride_page, sn, sh, oracle.BF16)
        qh = q.view(torch.int16).cpu().numpy().view(np.uint16)
        t0 = time.perf_counter()
        ref = oracle.batch_decode(qh[:sb], oracle.BF16, kv, Hq, rope_mode=oracle.ROPE_FULL, rope_theta=theta, parallel=True)
        cpu_s = time.perf_counter() - t0
        res["max_abs_err_vs_cpu"] = {"decode_rope_full": float(np.abs(out_full[:sb].cpu().numpy() - ref).max()),
                                     "convert_then_q_only": float(np.abs(out[:sb].cpu().numpy() - ref).max())}
        res["cpu_baseline"] = {"value": round(cpu_s * B / sb * 1e6, 1), "unit": "us/call", "cores": oracle.num_threads(True),
                               "kind": "port", "sample": f"kRoPELlama decode of the first {sb} of {B} sequences, scaled by {B // sb}x",
                               "host_cpus": os.cpu_count()}
    return res


def bench_mfma_ceiling(args):
    """What the matrix pipes sustain on this GPU without any memory traffic (blitz_scale_amd/probes/mfma_ceiling.hip,
    a stand-alone program run here as a child process): the yardstick beside the data sheet's 2.5 PFLOP/s for the
    prefill kernel's figure."""
    import re
    import subprocess
    exe = os.path.join(ROOT, "blitz_scale_amd", "probes", "mfma_ceiling")
    if not os.path.exists(exe):
        sys.exit("bench.py: blitz_scale_amd/probes/mfma_ceiling is not built (python -c 'import __graft_entry__ as g; g.build()')")
    t0 = time.perf_counter()
    out = subprocess.run([exe], capture_output=True, text=True, timeout=600)
    if out.returncode != 0:
        sys.exit("bench.py: the probe failed:\n" + out.stdout + out.stderr)
    rows = {}
    for line in out.stdout.splitlines():
        m = re.match(r"(.*?)\s+([\d.]+) ms\s+([\d.]+) TFLOP/s\s+clock (\d+) MHz\s+pipe use (\d+) %", line)
        if m:  # the program runs every variant twice: the second pass is the settled one
            rows[m.group(1).strip()] = {"TFLOP_per_s": float(m.group(3)), "clock_MHz": int(m.group(4)),
                                        "pipe_use_at_that_clock_pct": int(m.group(5))}
    key = "+ LDS every instruction + exp, pack, dot2"
    return {"metric": "mfma_ceiling_tflops", "value": rows[key]["TFLOP_per_s"], "unit": "TFLOP/s", "n_gpus": 1, "steps": 1,
            "warmup": 1, "ms_per_step": round((time.perf_counter() - t0) * 1e3, 1), "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "f16", "data": "synthetic",
            "config": {"workload": "MFMA_CEILING: v_mfma_f32_32x32x16_f16 at full rate, 2 waves per SIMD on all 256 CUs, no "
                                   "memory traffic; variants add what attention needs beside each matrix instruction"},
            "variants": rows,
            "roofline": {"bound": "mfma", "achieved": rows[key]["TFLOP_per_s"], "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": round(rows[key]["TFLOP_per_s"] / MFMA_PEAK_TFLOPS, 4), "traffic": None,
                         "kernel": "probe loop with one LDS operand read, one exponential, half a pack and half a row-sum "
                                   "instruction per matrix instruction (`value`); the other variants are in `variants`"}}


def main():
    args = parse()
    if args.workload == "MFMA_CEILING":  # (a child process does the GPU work: nothing here touches the GPU before it)
        print(json.dumps(bench_mfma_ceiling(args)))
        return
    import torch
    from blitz_scale_amd import _lib
    _lib.load()  # fails loudly if the HIP library is not built
    torch.cuda.set_device(0)
    if args.calibrate_copy:
        src = torch.empty(1 << 29, dtype=torch.bfloat16, device="cuda").normal_()  # 1 GiB read + 1 GiB written per copy
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if args.workload == "ENDS":
        res = bench_ends(args)
    elif args.workload == "MIGRATE":
        res = bench_migrate(args)
    elif args.workload == "LAYERS":
        res = bench_layers(args)
    elif args.workload == "RAWK":
        res = bench_rawk(args)
    else:
        res = bench_prefill(args) if args.workload == "C4" else bench_decode(args, args.workload)
    print(json.dumps(res))


if __name__ == "__main__":
    main()
