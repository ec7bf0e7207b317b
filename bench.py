#!/usr/bin/env python3
"""Benchmark of the multi-LoRA batching operator on one MI355X.

Workload (the shape the headline metric is quoted on): decode BGMV -- 256 tokens, one per
request, x[256,4096] fp16, 64 resident adapters of rank 16, per-token adapter id ~ Zipf(0.6),
4096 -> 4096, y += scale * (x @ A_a.T) @ B_a.  One *step* is one decode step's worth of this op:
the op applied on `--layers` (32) different layers, each with its own pool slice, x and y, so the
operands of consecutive launches do not sit in cache.  The layer loop is captured in a HIP graph
(the op allocates nothing and only launches kernels on the caller's stream) and replayed.

Prints ONE JSON line: value = microseconds per LoRA layer-op; `roofline` = achieved algorithmic
HBM bytes/s of the dominant kernel against the 8 TB/s peak, measured with HIP events on the launch
stream; `cpu_baseline` = the reference's PyTorch per-segment path restated on CPU, timed on this
host's cores on the same workload.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published peak

# HBM bytes per launch of the dominant kernel measured with rocprofv3 --pmc (FETCH_SIZE, WRITE_SIZE),
# scaled by the same counters' reading for a plain copy of known size; None until measured.
MEASURED_TRAFFIC_BYTES = {"decode_kernel": 23_570_000, "expand_kernel": 13_050_000,
                          "shrink_kernel": 10_580_000}  # profiles/config2_decode_hbm_traffic_pmc.txt


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--layers", type=int, default=32)
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly from Python instead of replaying a HIP graph")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true", help="skip the layer, drop-in entry point and step legs")
    ap.add_argument("--no-step5", action="store_true", help="skip the 32-layer serving step of configuration 5")
    ap.add_argument("--bm-shrink", type=int, default=None)
    ap.add_argument("--bm-expand", type=int, default=None)
    ap.add_argument("--ksplit", type=int, default=None)
    ap.add_argument("--reduce-in-expand", type=int, default=None, help="1: expand sums the split-K chunks, 0: shrink does")
    ap.add_argument("--one-launch", type=int, default=None,
                    help="1: shrink and expand as work items of one grid, 0: two launches (default: the tile table's choice)")
    ap.add_argument("--pmc-copy-mib", type=int, default=0,
                    help="first run one plain device copy of this many MiB: a kernel of known traffic to scale "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings with")
    ap.add_argument("--only-config", type=int, default=0,
                    help="with --all-configs: report this benchmark configuration only (1, 3, 4, 5, or 2: the headline's "
                         "decode batch on all seven projections of a layer)")
    ap.add_argument("--only-target", default=None,
                    help="with --all-configs --only-config N: time this target only (q, k, v, o, gate, up, down) and "
                         "no multi-target group, so that a profile of the run holds one shape per kernel")
    ap.add_argument("--all-configs", metavar="FILE", default=None,
                    help="also measure every target of configs 1,3,4,5 and write a JSON report to FILE")
    return ap.parse_args()


def build_layers(torch, W, dev, L):
    """Layer 0 is the seeded benchmark workload; the other layers reuse its ids and pool index
    (the reference shares a_start/a_len/a_loc across layers and indexes key_buffer[layer]) with
    their own random weights, x and y."""
    w = W.config2()
    wd = w.to(dev)
    t = wd.targets[0]
    p = t.pool
    g = torch.Generator(device=dev).manual_seed(2002)
    kb, vb, xs, ys = [p.key_buffer], [p.value_buffer], [wd.x[4096]], [wd.y0["q"].clone()]
    for _ in range(1, L):
        kb.append((torch.randn(p.key_buffer.shape, generator=g, device=dev) * 0.02).to(w.dtype))
        vb.append((torch.randn(p.value_buffer.shape, generator=g, device=dev) * 0.02).to(w.dtype))
        xs.append(torch.randn(w.T, 4096, generator=g, device=dev).to(w.dtype))
        ys.append(torch.randn(w.T, 4096, generator=g, device=dev).to(w.dtype))
    return w, wd, kb, vb, xs, ys


def time_graph(torch, fn, reps, warm, use_graph):
    """Average milliseconds of one call of fn() (which enqueues work on the current stream),
    from HIP events recorded on that stream around `reps` back-to-back repetitions."""
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        for _ in range(2):
            fn()
        graph = None
        if use_graph:
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=s):
                fn()
        run = graph.replay if graph is not None else fn
        for _ in range(warm):
            run()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        e0.record()
        for _ in range(reps):
            run()
        e1.record()
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3 / reps
        ev_ms = e0.elapsed_time(e1) / reps
    torch.cuda.current_stream().wait_stream(s)
    return ev_ms, wall_ms


def cpu_baseline(torch, w, budget_s=15.0):
    """The reference's per-segment PyTorch path (valora/models/bmm/lora_bmm_infer.py:342-352)
    restated in oracle/, on this host's cores: decode tokens are length-1 segments after grouping
    consecutive equal ids."""
    from oracle import lora_oracle as O
    t = w.targets[0]
    p = t.pool
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    dense = [p.dense(a, t.slot) for a in range(p.n_adapters)]
    A_list, B_list = [d[0] for d in dense], [d[1] for d in dense]
    segs = O.segments_from_ids(w.ids.tolist())
    scal = [float(s) for s in p.a_scaling]
    x, y0 = w.x[t.h_in], w.y0[t.name]
    kind = "native " + str(w.dtype).replace("torch.", "")
    compute = None
    try:
        t0 = time.perf_counter()
        O.per_segment_mm(y0, x, A_list, B_list, segs, scal)
        first = time.perf_counter() - t0
        if first > 2.0:
            raise RuntimeError("16-bit CPU matmul too slow")
    except Exception:
        compute, kind = torch.float32, "fp32 compute on 16-bit-rounded inputs"
    for _ in range(3):
        O.per_segment_mm(y0, x, A_list, B_list, segs, scal, compute_dtype=compute)
    times = []
    t_start = time.perf_counter()
    while len(times) < 10 or (time.perf_counter() - t_start < budget_s and len(times) < 2000):
        t0 = time.perf_counter()
        O.per_segment_mm(y0, x, A_list, B_list, segs, scal, compute_dtype=compute)
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    return {"value": round(med * 1e6, 2), "unit": "us/layer", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"{len(times)} repetitions of the full config-2 op (256 tokens -> {len(segs)} segments), "
                      f"median; {kind}; min {times[0] * 1e6:.1f} us"}


COLD_BYTES = 1 << 30   # four times the 256 MB last-level cache of the MI355X


def pool_copies(p, n_max):
    """Copies of a pool's two weight buffers to rotate over, COLD_BYTES in all (at most `n_max` of each): the first is
    the pool's own."""
    per = (p.key_buffer.numel() + p.value_buffer.numel()) * p.key_buffer.element_size()
    n = max(1, min(n_max, -(-COLD_BYTES // per)))
    return ([p.key_buffer] + [p.key_buffer.clone() for _ in range(n - 1)],
            [p.value_buffer] + [p.value_buffer.clone() for _ in range(n - 1)])


def bench_all_configs(torch, W, LoraPlan, dev, path, use_graph, only=0, only_target=None):
    """Per-target timing of the other benchmark configurations and of the headline's decode batch on all seven
    projections of a layer (report only; the JSON line of the default run is config 2's q).  Each target's shrink+expand is replayed back to back on 4 copies of y
    so that the read-modify-write does not hit the same lines (`us`: x and the pool may sit in the
    last-level cache), and once more over 1 GiB of x / y copies and as much of pool copies (`us_cold`: what a
    forward pass sees, where every layer has its own adapter weights)."""
    report = {}
    for n in ((only,) if only else (1, 2, 3, 4, 5)):
        # 2: the headline's decode batch with LoRA on all seven projections of a layer (the headline itself is its q)
        w = W.decode_layer() if n == 2 else W.CONFIGS[n]()
        wd = w.to(dev)
        R = max(w.targets[0].pool.ranks)
        rows = {}
        total_us = 0.0
        for t in wd.targets:
            if only_target and t.name != only_target:
                continue
            p = t.pool
            plan = LoraPlan(wd.ids, p.a_start, p.a_len, R, hidden=t.h_in)
            ycopies = [wd.y0[t.name].clone() for _ in range(4)]
            x = wd.x[t.h_in]

            def fn():
                for yy in ycopies:
                    plan.apply(yy, x, p.key_buffer, p.value_buffer, p.a_start, p.a_len, p.a_loc, t.slot, p.a_scaling)

            def fs():
                for yy in ycopies:
                    plan.shrink(x, p.key_buffer, p.a_start, p.a_len, p.a_loc, t.slot)

            def fe():
                for yy in ycopies:
                    plan.expand(yy, p.value_buffer, p.a_start, p.a_len, p.a_loc, t.slot, p.a_scaling)

            ms, _ = time_graph(torch, fn, 30, 3, use_graph)
            ms_s, _ = time_graph(torch, fs, 30, 3, use_graph)
            ms_e, _ = time_graph(torch, fe, 30, 3, use_graph)
            us = ms * 1e3 / 4
            # the same op on operands no cache holds: enough copies of x and y to walk through COLD_BYTES
            n_cold = max(4, -(-COLD_BYTES // (x.numel() * 2 + ycopies[0].numel() * 2)))
            xc = [x.clone() for _ in range(n_cold)]
            yc = [wd.y0[t.name].clone() for _ in range(n_cold)]
            kc, vc = pool_copies(p, n_cold)

            def fc():
                for i, (xx, yy) in enumerate(zip(xc, yc)):
                    plan.apply(yy, xx, kc[i % len(kc)], vc[i % len(vc)], p.a_start, p.a_len, p.a_loc, t.slot, p.a_scaling)

            ms_c, _ = time_graph(torch, fc, 10, 2, use_graph)
            us_cold = ms_c * 1e3 / n_cold
            del xc, yc, kc, vc
            b, f = w.algorithmic_bytes(t.name), w.flops(t.name)
            rows[t.name] = {"us": round(us, 2), "us_cold": round(us_cold, 2),
                            "shrink_us": round(ms_s * 250, 2), "expand_us": round(ms_e * 250, 2),
                            "bytes": b, "flops": f, "gbps": round(b / us / 1e3, 1),
                            "hbm_frac": round(b / us / 1e3 / HBM_PEAK_GBPS, 4), "tflops": round(f / us / 1e6, 2),
                            "tile": [plan.bm_shrink, plan.ksplit, plan.bm_expand]}
            total_us += us
        # targets that read the same x, in one shrink + one expand launch
        groups, fused_total = {}, total_us
        for names in (("q", "k", "v"), ("gate", "up")):
            ts = [t for t in wd.targets if t.name in names]
            if len(ts) < 2 or only_target:
                continue
            p = ts[0].pool
            plan = LoraPlan(wd.ids, p.a_start, p.a_len, R, hidden=ts[0].h_in)
            ycopies = [[wd.y0[t.name].clone() for t in ts] for _ in range(4)]
            x, slots = wd.x[ts[0].h_in], [t.slot for t in ts]

            def fm():
                for ys in ycopies:
                    plan.apply_multi(ys, x, p.key_buffer, p.value_buffer, p.a_start, p.a_len, p.a_loc, slots,
                                     p.a_scaling)

            ms, _ = time_graph(torch, fm, 30, 3, use_graph)
            us = ms * 1e3 / 4
            n_cold = max(4, -(-COLD_BYTES // (x.numel() * 2 + sum(y.numel() for y in ycopies[0]) * 2)))
            xc = [x.clone() for _ in range(n_cold)]
            yc = [[wd.y0[t.name].clone() for t in ts] for _ in range(n_cold)]
            kc, vc = pool_copies(p, n_cold)

            def fmc():
                for i, (xx, ys) in enumerate(zip(xc, yc)):
                    plan.apply_multi(ys, xx, kc[i % len(kc)], vc[i % len(vc)], p.a_start, p.a_len, p.a_loc, slots,
                                     p.a_scaling)

            ms_c, _ = time_graph(torch, fmc, 10, 2, use_graph)
            us_cold = ms_c * 1e3 / n_cold
            del xc, yc, kc, vc
            separate = sum(rows[t.name]["us"] for t in ts)
            # x is read once for the whole group
            b = sum(w.algorithmic_bytes(t.name) for t in ts) - (len(ts) - 1) * w.T * ts[0].h_in * 2
            groups["+".join(t.name for t in ts)] = {"us": round(us, 2), "us_cold": round(us_cold, 2),
                                                    "separate_us": round(separate, 2),
                                                    "bytes": b, "gbps": round(b / us / 1e3, 1),
                                                    "hbm_frac": round(b / us / 1e3 / HBM_PEAK_GBPS, 4)}
            fused_total += us - separate
        report[f"config{n}"] = {"tokens": w.T, "dtype": str(w.dtype), "max_rank": R, "targets": rows,
                                "us_per_layer": round(total_us, 2), "multi_target": groups,
                                "us_per_layer_multi_target": round(fused_total, 2)}
        del wd
        torch.cuda.empty_cache()
    if not only:
        report["adapter_residency"] = bench_adapter_residency(torch, dev)
        report["config5_step"] = bench_config5_step(torch, W, dev, use_graph)
        report["decode_step"] = bench_config5_step(torch, W, dev, use_graph, decode_only=True)
        report["config4_prefill_step"] = bench_config4_prefill_step(torch, W, dev, use_graph)
    with open(path, "w") as f:
        json.dump(report, f, indent=1)


def bench_config5_step(torch, W, dev, use_graph, decode_only=False):
    """The serving step of benchmark configuration 5: 32 decoder layers of the 7B shape (hidden 4096, 32 heads,
    MLP 11008, random weights), 128 decode tokens with cached contexts of 256..2048 tokens plus 2 prefill
    requests of 512 tokens, 64 resident adapters (ranks 16/32/64, Zipf 0.8), LoRA on all 7 projections.  The base
    model is stock PyTorch (mm, scaled_dot_product_attention); reported: step time with LoRA, base-only step time
    and their difference.  The KV cache is shared by the layers (it only serves the timing of the base step).
    ``decode_only``: the same step for the decode batch of configuration 2 instead (256 tokens, one per request,
    64 adapters of rank 16, fp16, no prefill requests)."""
    import torch.nn.functional as F
    from valora_amd.layer import LayerPlans, LayerPools, LayerWeights, layer_forward
    H, MLP, heads, L = 4096, 11008, 32, 32
    d = H // heads
    w5 = W.decode_layer() if decode_only else W.CONFIGS[5]()
    dt = w5.dtype
    wd = w5.to(dev)
    T, n_dec = w5.T, (w5.T if decode_only else 128)
    pa, pu, pdn = wd.target("q").pool, wd.target("gate").pool, wd.target("down").pool
    idx = (pa.a_start, pa.a_len, pa.a_loc, pa.a_scaling)
    g = torch.Generator(device=dev).manual_seed(55)
    rnd = lambda *shape, s=1.0: (torch.randn(*shape, device=dev, generator=g) * s).to(dt)
    layers = []
    for _ in range(L):
        wts = LayerWeights(rnd(H, H, s=H ** -0.5), rnd(H, H, s=H ** -0.5), rnd(H, H, s=H ** -0.5), rnd(H, H, s=H ** -0.5),
                           rnd(H, MLP, s=H ** -0.5), rnd(H, MLP, s=H ** -0.5), rnd(MLP, H, s=MLP ** -0.5),
                           torch.ones(H, device=dev, dtype=dt), torch.ones(H, device=dev, dtype=dt))
        pools = LayerPools(tuple(rnd(*b.shape, s=0.02) for b in (pa.key_buffer, pa.value_buffer)),
                           tuple(rnd(*b.shape, s=0.02) for b in (pu.key_buffer, pu.value_buffer)),
                           tuple(rnd(*b.shape, s=0.02) for b in (pdn.key_buffer, pdn.value_buffer)), *idx)
        layers.append((wts, pools))
    plans = LayerPlans(wd.ids, pa.a_start, pa.a_len, max(pa.ranks), H, MLP)
    gl = torch.Generator().manual_seed(56)
    # (decode only: short contexts, so that stock PyTorch's masked attention does not bury the difference the
    # step is run for under its own run-to-run spread)
    kv_len = torch.randint(64, 257, (n_dec,), generator=gl) if decode_only else torch.randint(256, 2049, (n_dec,), generator=gl)
    Lmax = int(kv_len.max())
    kc, vc = rnd(n_dec, heads, Lmax, d), rnd(n_dec, heads, Lmax, d)
    mask = (torch.arange(Lmax)[None, :] < kv_len[:, None]).to(dev)[:, None, None, :]
    pre = [] if decode_only else [(n_dec + i * 512, n_dec + (i + 1) * 512) for i in range(2)]

    def attention(q, k, v):
        out = torch.empty_like(q)
        out[:n_dec] = F.scaled_dot_product_attention(q[:n_dec].view(n_dec, heads, 1, d), kc, vc,
                                                     attn_mask=mask).reshape(n_dec, H)
        for b, e in pre:
            qq, kk, vv = (t[b:e].view(512, heads, d).transpose(0, 1).unsqueeze(0) for t in (q, k, v))
            out[b:e] = F.scaled_dot_product_attention(qq, kk, vv, is_causal=True)[0].transpose(0, 1).reshape(512, H)
        return out

    pos = torch.cat([kv_len.float()] + [torch.arange(512).float() for _ in pre]).to(dev)
    freq = 1.0 / (10000 ** (torch.arange(0, d, 2, device=dev).float() / d))
    ang = torch.cat((pos[:, None] * freq[None], pos[:, None] * freq[None]), dim=-1)
    cos, sin = ang.cos().to(dt), ang.sin().to(dt)
    x0 = rnd(T, H)

    def step(lora):
        x = x0
        for wts, pools in layers:
            x = layer_forward(x, wts, pools if lora else None, plans if lora else None, attention, heads, cos, sin)
        return x

    out = {}
    reps = 20 if decode_only else 5
    # the figure of interest is the difference of two step times that are ten to fifteen times larger than it: both
    # are measured three times, alternating, and the medians are reported
    runs = {"base_only": [], "with_lora": []}
    modes = {}
    for _ in range(3):
        for name, lora in (("base_only", False), ("with_lora", True)):
            try:
                ms, _ = time_graph(torch, lambda: step(lora), reps, 2, use_graph)
                mode = "hip graph replay" if use_graph else "eager"
            except Exception as exc:   # a library call that cannot be captured: time it eagerly
                torch.cuda.synchronize()
                ms, _ = time_graph(torch, lambda: step(lora), reps, 2, False)
                mode = f"eager ({type(exc).__name__} during capture)"
            runs[name].append(ms)
            modes[name] = mode
    for name, v in runs.items():
        out[name] = {"ms_per_step": round(sorted(v)[1], 3), "launch": modes[name],
                     "runs_ms": [round(x, 3) for x in v]}
    out["lora_overhead_ms"] = round(out["with_lora"]["ms_per_step"] - out["base_only"]["ms_per_step"], 3)
    out["tokens"] = T
    out["lora_calls_per_layer"] = 4
    return out


def bench_config4_prefill_step(torch, W, dev, use_graph, n_layers=8):
    """LoRA inside a prefill forward pass of benchmark configuration 4 (16 requests of 256 image + 16..128 text
    tokens, 16 adapters of rank 64, LoRA on all 7 projections): `n_layers` decoder layers of the 7B shape with
    stock PyTorch `mm` and per-request causal attention around the LoRA calls.  Reported per layer: base only,
    with LoRA, and the difference -- what the ops cost when y has just been written by the base projection and
    is read again right after, as opposed to the back-to-back figures of the per-target report."""
    from valora_amd.layer import LayerPlans, LayerPools, LayerWeights, layer_forward, segment_attention
    H, MLP, heads, dt = 4096, 11008, 32, torch.bfloat16
    w4 = W.CONFIGS[4]()
    wd = w4.to(dev)
    pa, pu, pdn = wd.target("q").pool, wd.target("gate").pool, wd.target("down").pool
    idx = (pa.a_start, pa.a_len, pa.a_loc, pa.a_scaling)
    g = torch.Generator(device=dev).manual_seed(44)
    rnd = lambda *shape, s=1.0: (torch.randn(*shape, device=dev, generator=g) * s).to(dt)
    layers = []
    for _ in range(n_layers):
        wts = LayerWeights(rnd(H, H, s=H ** -0.5), rnd(H, H, s=H ** -0.5), rnd(H, H, s=H ** -0.5), rnd(H, H, s=H ** -0.5),
                           rnd(H, MLP, s=H ** -0.5), rnd(H, MLP, s=H ** -0.5), rnd(MLP, H, s=MLP ** -0.5),
                           torch.ones(H, device=dev, dtype=dt), torch.ones(H, device=dev, dtype=dt))
        pools = LayerPools(tuple(rnd(*b.shape, s=0.02) for b in (pa.key_buffer, pa.value_buffer)),
                           tuple(rnd(*b.shape, s=0.02) for b in (pu.key_buffer, pu.value_buffer)),
                           tuple(rnd(*b.shape, s=0.02) for b in (pdn.key_buffer, pdn.value_buffer)), *idx)
        layers.append((wts, pools))
    plans = LayerPlans(wd.ids, pa.a_start, pa.a_len, max(pa.ranks), H, MLP)
    attention = segment_attention([int(n) for n in w4.b_seq_len.tolist()], heads)
    x0 = rnd(w4.T, H)

    def step(lora):
        x = x0
        for wts, pools in layers:
            x = layer_forward(x, wts, pools if lora else None, plans if lora else None, attention, heads)
        return x

    us = {}
    for name, lora in (("base_only", False), ("with_lora", True)):
        us[name] = min(time_graph(torch, lambda: step(lora), 5, 2, use_graph)[0] for _ in range(2)) * 1e3 / n_layers
    return {"tokens": w4.T, "layers": n_layers, "us_per_layer_base_only": round(us["base_only"], 1),
            "us_per_layer_with_lora": round(us["with_lora"], 1),
            "lora_us_per_layer": round(us["with_lora"] - us["base_only"], 1), "lora_calls_per_layer": 4}


def bench_adapter_residency(torch, dev):
    """Loading an adapter into the paged pool and dropping adapters again: one rank-64 adapter of a
    32-layer, 4096-wide model is 2 x 32 x 256 rows of 8 KB (134 MB), moved by one row-scatter launch
    per buffer; the HBM figure counts every byte read once and written once."""
    from valora_amd import _lib
    from valora_amd.infer_adapter import InferAdapter, LoraAdapterWeights, MemoryAllocator
    net = dict(num_hidden_layers=32, hidden_size=4096, num_attention_heads=32)
    rows_total = 16384
    mm = MemoryAllocator(rows_total, 0, torch.float16, 32, 128, 32, dev)
    out = {}
    for r in (16, 64):
        n = 4 * r
        packed = torch.randn(32, 2, n, 4096, device=dev).to(torch.float16)
        loc = torch.randperm(rows_total, device=dev)[:n].contiguous()
        L, st_of = _lib.lib(), _lib.current_stream
        esz = 2

        def scatter_both():
            for which, buf in ((0, mm.key_buffer), (1, mm.value_buffer)):
                _lib.check(L.mlora_pool_scatter_rows(st_of(dev), _lib.ptr(buf), rows_total, rows_total * 4096 * esz,
                                                     _lib.c_void_p(packed.data_ptr() + which * n * 4096 * esz),
                                                     2 * n * 4096 * esz, _lib.ptr(loc), n, 4096 * esz, 32))

        ms, _ = time_graph(torch, scatter_both, 20, 3, False)
        moved = 2 * packed.numel() * esz
        out[f"load_rank{r}"] = {"us": round(ms * 1e3, 1), "bytes_read_plus_written": moved,
                                "gbps": round(moved / ms / 1e6, 1), "hbm_frac": round(moved / ms / 1e6 / HBM_PEAK_GBPS, 4),
                                "launches": 2, "reference_launches": 64}
    # allocator and re-index latency with 200 resident adapters
    ia = InferAdapter.init(mm)
    small = dict(num_hidden_layers=32, hidden_size=4096, num_attention_heads=32)
    ads = [LoraAdapterWeights(f"a{i}", 16, 32.0, small, torch.zeros(32, 2, 64, 4096, dtype=torch.float16))
           for i in range(200)]
    t0 = time.perf_counter()
    ia.load_adapters(ads)
    torch.cuda.synchronize()
    out["load_200_adapters_rank16_ms_wall"] = round((time.perf_counter() - t0) * 1e3, 2)
    t0 = time.perf_counter()
    ia.offload_adapters([f"a{i}" for i in range(0, 200, 2)])
    torch.cuda.synchronize()
    out["offload_100_of_200_ms_wall"] = round((time.perf_counter() - t0) * 1e3, 3)

    def alloc_free():
        idx = mm.alloc(256)
        mm.free(idx)

    ms, _ = time_graph(torch, alloc_free, 50, 3, False)
    out["alloc256_plus_free_us"] = round(ms * 1e3, 2)

    # merging one adapter into the q, k, v, o weights of a layer (4 x [4096, 4096]): every weight element
    # is read once and written once
    from valora_amd.merge import merge_adapter
    ia2 = InferAdapter.init(mm)
    for r in (16, 64):
        ad = LoraAdapterWeights.dummy(f"m{r}", r, 2.0 * r, net, pin=False)
        ia2.load_adapters([ad])
        idx = ia2.idx_map[f"m{r}"]
        wsets = [[torch.randn(4096, 4096, device=dev).to(torch.float16) for _ in range(4)] for _ in range(3)]
        state = {"i": 0}

        def merge_layer():
            ws = wsets[state["i"] % 3]
            state["i"] += 1
            merge_adapter(ws, mm.key_buffer[0], mm.value_buffer[0], ia2.a_start, ia2.a_len, ia2.a_loc, idx, 2.0, r)

        ms, _ = time_graph(torch, merge_layer, 30, 3, False)
        moved = 4 * 2 * 4096 * 4096 * 2
        out[f"merge_layer_rank{r}"] = {"us": round(ms * 1e3, 1), "bytes_read_plus_written": moved,
                                       "gbps": round(moved / ms / 1e6, 1),
                                       "hbm_frac": round(moved / ms / 1e6 / HBM_PEAK_GBPS, 4), "launches": 1}
    return out


def bench_byte_heavy_decode(torch, W, LoraPlan, dev, use_graph, reps):
    """Decode batches (one token per request, 4096 -> 4096, fp16, adapters drawn Zipf(0.7) over 128) whose adapters
    weigh a few hundred MB: the same kernels as the headline, where the op is long enough for its bytes to decide.
    Bytes are algorithmic: x + y read + y write + A and B of the adapters the batch really touches."""
    out = []
    H = 4096
    for T, A, r in ((256, 128, 64), (512, 128, 128), (1024, 128, 64), (1024, 128, 128)):
        g = torch.Generator().manual_seed(T + A + r)
        ids = W.zipf_ids(A, T, 0.7, g)
        pool = W.make_pool([r] * A, H, H, torch.float16, g, True, n_slots=1).to(dev)
        x = torch.randn(T, H, generator=g).half().to(dev)
        ys = [torch.zeros(T, H, dtype=torch.float16, device=dev) for _ in range(4)]
        plan = LoraPlan(ids.to(dev), pool.a_start, pool.a_len, r, n_slots=1, hidden=H)

        def run():
            for y in ys:
                plan.apply(y, x, pool.key_buffer, pool.value_buffer, pool.a_start, pool.a_len, pool.a_loc, 0, pool.a_scaling)

        ms, _ = time_graph(torch, run, max(10, reps // 4), 3, use_graph)
        us = ms * 1e3 / len(ys)
        touched = len(set(ids.tolist()))
        nbytes = 3 * T * H * 2 + 2 * touched * r * H * 2
        out.append({"tokens": T, "rank": r, "adapters_touched": touched, "us": round(us, 2), "bytes": nbytes,
                    "gbps": round(nbytes / us / 1e3, 1), "hbm_frac": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 3),
                    "tile": [plan.bm_shrink, plan.ksplit, plan.bm_expand], "one_launch": plan.one_launch})
        del pool, x, ys, plan
        torch.cuda.empty_cache()
    return out


def bench_single_adapter_vs_gemm(torch, W, LoraPlan, dev, use_graph, reps):
    """One adapter for the whole batch: the op is then two dense skinny matrix products, y += s * (x @ A^T) @ B, which
    the vendor's GEMM library can do as torch.mm + Tensor.addmm_ (operands laid out the way the library likes them).
    A yardstick from outside this code base for what the device gives on these shapes; 4096 -> 4096, fp16."""
    out = []
    H, n = 4096, 8
    for T, r in ((256, 16), (256, 64), (4096, 16), (4096, 64), (16384, 16), (16384, 64)):
        g = torch.Generator().manual_seed(T + r)
        pool = W.make_pool([r], H, H, torch.float16, g, False, n_slots=1, heads=1).to(dev)
        ids = torch.zeros(T, dtype=torch.long, device=dev)
        gd = torch.Generator(device=dev).manual_seed(T + r)
        xs = [torch.randn(T, H, generator=gd, device=dev).half() for _ in range(n)]
        ys = [torch.randn(T, H, generator=gd, device=dev).half() for _ in range(n)]
        vs = [torch.empty(T, r, dtype=torch.float16, device=dev) for _ in range(n)]
        a_t = (torch.randn(H, r, generator=gd, device=dev) * 0.02).half()
        b = (torch.randn(r, H, generator=gd, device=dev) * 0.02).half()
        plan = LoraPlan(ids, pool.a_start, pool.a_len, r, n_slots=1, hidden=H)

        def ours():
            for l in range(n):
                plan.apply(ys[l], xs[l], pool.key_buffer, pool.value_buffer, pool.a_start, pool.a_len, pool.a_loc, 0,
                           pool.a_scaling)

        def gemm():
            for l in range(n):
                torch.mm(xs[l], a_t, out=vs[l])
                ys[l].addmm_(vs[l], b, alpha=0.5)

        k = max(10, reps // 4)
        us_ours = time_graph(torch, ours, k, 3, use_graph)[0] * 1e3 / n
        us_gemm = time_graph(torch, gemm, k, 3, use_graph)[0] * 1e3 / n
        nbytes = (3 * T * H + 2 * r * H) * 2
        out.append({"tokens": T, "rank": r, "us": round(us_ours, 2), "torch_mm_addmm_us": round(us_gemm, 2),
                    "gbps": round(nbytes / us_ours / 1e3, 1), "tile": [plan.bm_shrink, plan.ksplit, plan.bm_expand],
                    "one_launch": plan.one_launch})
        del pool, xs, ys, vs, plan
        torch.cuda.empty_cache()
    return out


def bench_tile_edge(torch, W, LoraPlan, dev, kb, vb, xs, ys, use_graph, n_draws=200, n_layers=8):
    """The headline shape over `n_draws` seeded Zipf(0.6) draws of its per-token adapter ids (256 tokens, 64 rank-16
    adapters, same pools, x and y as the headline): the device holds the one-launch grid of 64 tiles of up to 16 tokens
    at once, and a draw has 55-66 of them.  Per draw: the one-launch op and, on the same operands, the two-launch op
    with the same split (bit-identical results); reported: median, p99 and max of the one-launch time and the worst
    ratio to the same draw's two launches."""
    pool_idx = None
    rows = []
    for seed in range(n_draws):
        g = torch.Generator().manual_seed(7000 + seed)
        ids = W.zipf_ids(64, 256, 0.6, g)
        cnt = torch.bincount(ids, minlength=64)
        n_tiles = int(((cnt + 15) // 16).sum())
        idd = ids.to(dev)
        if pool_idx is None:
            pool_idx = W.config2().to(dev).targets[0].pool
        p = pool_idx
        us = []
        for kw in (dict(one_launch=True, ksplit=4),
                   dict(one_launch=False, bm_shrink=16, bm_expand=16, ksplit=4, reduce_in_expand=True)):
            plan = LoraPlan(idd, p.a_start, p.a_len, 16, hidden=4096, **kw)

            def run():
                for l in range(n_layers):
                    plan.apply(ys[l], xs[l], kb[l], vb[l], p.a_start, p.a_len, p.a_loc, 0, p.a_scaling)

            us.append(time_graph(torch, run, 10, 2, use_graph)[0] * 1e3 / n_layers)
        rows.append((n_tiles, us[0], us[1]))
    one = sorted(r[1] for r in rows)
    by_tiles = {}
    for n, a, b in rows:
        by_tiles.setdefault(n, []).append((a, b))
    return {"draws": n_draws, "layers_per_timing": n_layers,
            "one_launch_us": {"median": round(one[len(one) // 2], 2), "p99": round(one[int(0.99 * (len(one) - 1))], 2),
                              "max": round(one[-1], 2)},
            "two_launch_us_median": round(sorted(r[2] for r in rows)[len(rows) // 2], 2),
            "worst_one_over_two_of_a_draw": round(max(a / b for _, a, b in rows), 3),
            "by_tile_count": {str(n): {"draws": len(v), "one_launch_us": round(sum(a for a, _ in v) / len(v), 2),
                                       "two_launch_us": round(sum(b for _, b in v) / len(v), 2)}
                              for n, v in sorted(by_tiles.items())}}


def bench_extras(torch, W, LoraPlan, dev, L, w, wd, kb, vb, xs, ys, use_graph, reps, no_step5):
    """Legs beside the headline, all on the config-2 decode shape with the same rotation over `L` layers'
    buffers: a whole attention block's LoRA work per layer, and the same shrink + expand pair reached through
    each of the reference's entry points (what an unchanged caller of the reference gets), replayed from a HIP
    graph and launched eagerly from Python."""
    from valora_amd import atmm_ops, kernels, lora_prefill
    p = wd.targets[0].pool
    idx = (p.a_start, p.a_len, p.a_loc)
    T, H, R = w.T, 4096, 16
    ids = wd.ids
    g = torch.Generator(device=dev).manual_seed(2003)
    rnd = lambda: torch.randn(T, H, generator=g, device=dev).to(w.dtype)
    out = {}

    # -- one layer's attention LoRA: q, k, v read the same x (one call), o reads the attention output
    plan = LoraPlan(ids, p.a_start, p.a_len, R, hidden=H)
    yk, yv, yo = [rnd() for _ in range(L)], [rnd() for _ in range(L)], [rnd() for _ in range(L)]

    def layer():
        for l in range(L):
            plan.apply_multi([ys[l], yk[l], yv[l]], xs[l], kb[l], vb[l], *idx, (0, 1, 2), p.a_scaling)
            plan.apply(yo[l], xs[(l + 1) % L], kb[l], vb[l], *idx, 3, p.a_scaling)

    ms, _ = time_graph(torch, layer, reps, 5, use_graph)
    out["layer_us"] = round(ms * 1e3 / L, 3)
    out["layer_us_is"] = "q+k+v in one mlora_lora_apply_multi call + o in one mlora_lora_apply call, per layer"
    del yk, yv, yo

    # -- the op between its producer and its consumer: y = x @ W (the base projection) -> the op on y -> a kernel
    #    that reads y, per layer with distinct weights; the difference to the same loop without the op is what the op
    #    costs where y is warm from the projection and wanted again right after
    gw = torch.Generator(device=dev).manual_seed(2004)
    Ws = [(torch.randn(H, H, generator=gw, device=dev) * 0.02).to(w.dtype) for _ in range(L)]
    zs = [torch.empty(T, H, dtype=w.dtype, device=dev) for _ in range(L)]

    def forward(lora):
        def run():
            for l in range(L):
                torch.mm(xs[l], Ws[l], out=ys[l])
                if lora:
                    plan.apply(ys[l], xs[l], kb[l], vb[l], *idx, 0, p.a_scaling)
                torch.mul(ys[l], 0.5, out=zs[l])
        return run

    ms_base, _ = time_graph(torch, forward(False), reps, 5, use_graph)
    ms_lora, _ = time_graph(torch, forward(True), reps, 5, use_graph)
    out["in_forward"] = {"base_us_per_layer": round(ms_base * 1e3 / L, 3), "with_lora_us_per_layer": round(ms_lora * 1e3 / L, 3),
                         "lora_us_per_layer": round((ms_lora - ms_base) * 1e3 / L, 3),
                         "is": "per layer: y = x @ W (torch.mm) -> the LoRA op on y -> an elementwise kernel that reads y; "
                               "the op's cost = difference to the same loop without it"}
    del Ws, zs

    # -- the reference's entry points: delta = shrink(x); y += expand(delta), two calls per layer
    delta = [torch.zeros(T, R, dtype=w.dtype, device=dev) for _ in range(L)]

    def bgmv_pair():
        for l in range(L):
            kernels.dispatch_bgmv(delta[l], xs[l], kb[l], *idx, ids, 0, p.a_scaling)
            kernels.dispatch_bgmv(ys[l], delta[l], vb[l], *idx, ids, 0, p.a_scaling)

    from valora_amd import segments
    oc, rc, li, st, n_runs = segments.count_consecutive_requests(p.a_len, ids)   # runs of equal ids, as the
    P = int(n_runs.item())                                                        # reference's caller builds them
    tmp = torch.empty(256, dtype=torch.uint8, device=dev)

    def sgmm_pair():
        for l in range(L):
            atmm_ops.dispatch_bgmv(delta[l], xs[l], kb[l], *idx, ids, 0, p.a_scaling, oc, rc, li, st, tmp, P,
                                   64, 32, 32, 32, 32, 32)
            atmm_ops.dispatch_bgmv(ys[l], delta[l], vb[l], *idx, ids, 0, p.a_scaling, oc, rc, li, st, tmp, P,
                                   32, 64, 32, 32, 32, 32)

    b_start = torch.arange(T, dtype=torch.int32, device=dev)
    b_len = torch.ones(T, dtype=torch.int32, device=dev)

    def prefill_pair():
        for l in range(L):
            lora_prefill.lora_get_qkvo_fwd_shrink(xs[l], kb[l], delta[l], p.a_loc, p.a_start, p.a_len, b_start, b_len,
                                                  ids, H, 0, R, 1)
            lora_prefill.lora_get_qkvo_fwd_expand(delta[l], vb[l], ys[l], p.a_scaling, p.a_loc, p.a_start, p.a_len,
                                                  b_start, b_len, ids, H, 0, R, 1)

    legs = {}
    for name, fn in (("valora._kernels.dispatch_bgmv", bgmv_pair), ("atmm_ops.dispatch_bgmv", sgmm_pair),
                     ("lora_prefill.lora_get_qkvo_fwd_*", prefill_pair)):
        ev_g, _ = time_graph(torch, fn, reps, 5, True)
        ev_e, wall_e = time_graph(torch, fn, max(10, reps // 4), 3, False)
        legs[name] = {"graph_us_per_layer": round(ev_g * 1e3 / L, 3), "eager_us_per_layer": round(ev_e * 1e3 / L, 3),
                      "eager_host_us_per_layer": round(wall_e * 1e3 / L, 3)}
    # the same pair when every call sorts the tokens and cuts the tiles itself (plan = NULL at the C ABI)
    from valora_amd import _plan_cache
    _plan_cache.set_enabled(False)
    try:
        ev_g, _ = time_graph(torch, bgmv_pair, max(10, reps // 4), 3, True)
        legs["valora._kernels.dispatch_bgmv, no plan reuse"] = {"graph_us_per_layer": round(ev_g * 1e3 / L, 3)}
    finally:
        _plan_cache.set_enabled(True)
    out["dropin_pair"] = legs
    out["dropin_pair_is"] = ("shrink + expand of the config-2 op through the reference's own entry points (two calls per "
                             "layer, torch binding -> one C-ABI call each with the cached plan of the batch); graph = HIP "
                             "graph replay, eager = launched from Python call by call (events / host wall clock)")
    try:
        out["tile_edge"] = bench_tile_edge(torch, W, LoraPlan, dev, kb, vb, xs, ys, use_graph)
    except Exception as exc:    # the headline does not depend on this leg
        out["tile_edge"] = {"error": f"{type(exc).__name__}: {exc}"}
    try:
        out["byte_heavy_decode"] = bench_byte_heavy_decode(torch, W, LoraPlan, dev, use_graph, reps)
    except Exception as exc:    # the headline does not depend on this leg
        out["byte_heavy_decode"] = {"error": f"{type(exc).__name__}: {exc}"}
    try:
        out["single_adapter_vs_gemm"] = bench_single_adapter_vs_gemm(torch, W, LoraPlan, dev, use_graph, reps)
    except Exception as exc:
        out["single_adapter_vs_gemm"] = {"error": f"{type(exc).__name__}: {exc}"}
    if not no_step5:
        try:
            s5 = bench_config5_step(torch, W, dev, use_graph)
            out["config5_step"] = s5
        except Exception as exc:    # the headline does not depend on this leg
            out["config5_step"] = {"error": f"{type(exc).__name__}: {exc}"}
        try:
            out["decode_step"] = bench_config5_step(torch, W, dev, use_graph, decode_only=True)
        except Exception as exc:
            out["decode_step"] = {"error": f"{type(exc).__name__}: {exc}"}
    return out


def main():
    args = parse()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported (nothing in this build uses a second GPU)",
              file=sys.stderr)
        sys.exit(2)
    import torch
    from valora_amd import workloads as W
    from valora_amd.plan import LoraPlan

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    if args.pmc_copy_mib > 0:
        src = torch.ones(args.pmc_copy_mib << 19, dtype=torch.float16, device=dev)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)          # reads and writes exactly pmc_copy_mib MiB
        torch.cuda.synchronize()
        del src, dst
    L = args.layers
    w, wd, kb, vb, xs, ys = build_layers(torch, W, dev, L)
    t = wd.targets[0]
    p = t.pool
    plan = LoraPlan(wd.ids, p.a_start, p.a_len, 16, hidden=4096, bm_shrink=args.bm_shrink,
                    bm_expand=args.bm_expand, ksplit=args.ksplit,
                    reduce_in_expand=None if args.reduce_in_expand is None else bool(args.reduce_in_expand),
                    one_launch=None if args.one_launch is None else bool(args.one_launch))
    idx = (p.a_start, p.a_len, p.a_loc)
    use_graph = not args.no_graph

    fused = plan.one_launch

    def layers_only():
        for l in range(L):
            plan.apply(ys[l], xs[l], kb[l], vb[l], *idx, 0, p.a_scaling)

    def step():
        # what a serving step does for this op: sort the batch's tokens by adapter and cut the tiles ONCE
        # (the reference rebuilds its segment tensors once per forward, model_rpc.py:381), then one op per layer
        plan.rebuild()
        layers_only()

    def shrink_only():
        for l in range(L):
            plan.shrink(xs[l], kb[l], *idx, 0)

    def expand_only():
        for l in range(L):
            plan.expand(ys[l], vb[l], *idx, 0, p.a_scaling)

    # ---- the timed region: W warm-up steps, then exactly K steps between two synchronisations
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        step()
        graph = None
        if use_graph:
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=s):
                step()
        run = graph.replay if graph is not None else step
        for _ in range(args.warmup):
            run()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            run()
        torch.cuda.synchronize()
        ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    torch.cuda.current_stream().wait_stream(s)
    us_per_layer = ms_per_step * 1e3 / L

    # ---- per-kernel durations (HIP events on the launch stream, same layer rotation)
    reps = max(10, min(args.steps, 200))
    sh_ms, _ = time_graph(torch, shrink_only, reps, 5, use_graph)
    ex_ms, _ = time_graph(torch, expand_only, reps, 5, use_graph)
    op_ms, _ = time_graph(torch, layers_only, reps, 5, use_graph)
    # one plan build: 32 builds back to back in one graph (what the build costs as a node of a step's graph: its
    # kernel), and a graph that holds nothing but one build (what a replay of a one-kernel graph costs: mostly the
    # graph launch itself, which varies from box to box and is not the build's)

    def plans_32():
        for _ in range(32):
            plan.rebuild()

    plan_ms = time_graph(torch, plans_32, reps, 5, use_graph)[0] / 32
    plan_alone_ms, _ = time_graph(torch, plan.rebuild, reps, 5, use_graph)
    sh_us, ex_us, op_us = sh_ms * 1e3 / L, ex_ms * 1e3 / L, op_ms * 1e3 / L

    s_el = 2
    used = sorted(set(w.ids.tolist()))
    r_sum = sum(w.targets[0].pool.ranks[a] for a in used)
    bytes_shrink = w.T * 4096 * s_el + r_sum * 4096 * s_el
    bytes_expand = r_sum * 4096 * s_el + 2 * w.T * 4096 * s_el
    bytes_op = w.algorithmic_bytes("q")
    assert bytes_op == bytes_shrink + bytes_expand
    if fused:
        dom = ("decode_kernel", bytes_op, op_us)
    else:
        dom = ("expand_kernel", bytes_expand, ex_us) if ex_us >= sh_us else ("shrink_kernel", bytes_shrink, sh_us)
    achieved = dom[1] / (dom[2] * 1e-6) / 1e9
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": MEASURED_TRAFFIC_BYTES.get(dom[0]),
                "kernel": dom[0], "algorithmic_bytes_per_launch": dom[1], "avg_launch_us": round(dom[2], 3),
                "shrink_kernel_us": round(sh_us, 3), "expand_kernel_us": round(ex_us, 3),
                "op_bytes": bytes_op, "op_us_events": round(op_us, 3),
                "op_achieved_gbps": round(bytes_op / (op_us * 1e-6) / 1e9, 1),
                "method": "HIP events on the launch stream around %d graph replays of %d launches (the op alone, "
                          "without the once-per-step plan build)" % (reps, L)}

    out = {
        "metric": "lora_op_us_per_layer", "value": round(us_per_layer, 3), "unit": "us/layer", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "config2 decode BGMV: 256 tokens (1/request), 64 adapters rank 16, Zipf(0.6) ids, "
                               "4096->4096, fp16, shrink+expand; one step = this op on %d layers" % L,
                   "step": "mlora_build_plan (token sort + tile cut, once per step) + the op on every layer, all "
                           "inside the timed region" + (", one hip graph" if use_graph else ""),
                   "layers_per_step": L, "tokens": w.T, "adapters_touched": len(used),
                   "launch": "hip graph replay" if use_graph else "eager python launches",
                   "kernels": "shrink and expand items of one grid, one launch" if fused else "shrink then expand, two launches",
                   "tile": {"bm_shrink": plan.bm_shrink, "ksplit": plan.ksplit, "bm_expand": plan.bm_expand}},
        "hbm_gbps": round(bytes_op / (us_per_layer * 1e-6) / 1e9, 1),
        "hbm_frac": round(bytes_op / (us_per_layer * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
        "roofline": roofline,
        "plan_us": round(plan_ms * 1e3, 3),
        "plan_us_is": "one mlora_build_plan as a node among others of a graph (32 builds back to back in one graph, per build)",
        "plan_us_one_kernel_graph": round(plan_alone_ms * 1e3, 3),
    }
    if not args.no_extras:
        out["extra"] = bench_extras(torch, W, LoraPlan, dev, L, w, wd, kb, vb, xs, ys, use_graph, reps, args.no_step5)
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(torch, w)
    if args.all_configs:
        bench_all_configs(torch, W, LoraPlan, dev, args.all_configs, use_graph, args.only_config, args.only_target)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
