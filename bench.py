#!/usr/bin/env python3
"""Benchmark of the MoE layer hot path on one MI355X.

Workload (the headline configuration): Mixtral-8x7B-shape layer, d_model 4096, 8 experts, top-2 with
renormalisation, expert d_ff 14336, bf16 weights resident in HBM (2.8 GB), bf16 activations
already on the device.  A step is one layer forward over one batch of T tokens through the
C ABI (`atenia_moe_hip_layer_forward_device`).  The default run times the prefill point
T=4096 (the headline tokens/s, MFMA-bound) and the decode points T=1 and T=16 (HBM-bound);
`--sweep 128,512` adds more batch sizes, `--config` picks another layer shape (tiny_f32 is the
reference's own CPU-runnable case on the GPU's f32 path).

Prints ONE JSON line.  `roofline` describes the dominant kernel of the headline batch, timed
live with HIP events on the launch stream; `decode.roofline` the same for T=1;
`cpu_baseline` is the CPU oracle (a C restatement of the reference's certified per-token
path, not the reference binary) timed on this box's host cores on a bounded token sample.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# Benchmark configurations.  The headline metric is quoted on mixtral_bf16; the others are
# reported with --config.
CONFIGS = {
    # Tiny f32 layer (f32 storage, f64 accumulation: the reference's certified arithmetic on the
    # GPU), T = 64: the configuration the reference's own CPU path is quoted on.
    "tiny_f32": dict(d=1024, E=8, k=2, f=2048, fs=0, gated=False, conv=0, wd="f32",
                     zipf=False, sweep=(64,)),
    "mixtral_bf16": dict(d=4096, E=8, k=2, f=14336, fs=0, gated=False, conv=0, wd="bf16",
                         zipf=False, sweep=(1, 16, 32, 64, 128, 512, 4096)),
    "mixtral_int8": dict(d=4096, E=8, k=2, f=14336, fs=0, gated=False, conv=0, wd="int8",
                         zipf=False, sweep=(1, 16, 32, 64, 128, 4096)),
    # per-group int8 (one scale per output row and 128 input elements, Q8_0-style)
    "mixtral_int8g": dict(d=4096, E=8, k=2, f=14336, fs=0, gated=False, conv=0, wd="int8g",
                          zipf=False, sweep=(1, 16, 32, 64, 128, 4096)),
    "qwen_bf16": dict(d=2048, E=60, k=4, f=1408, fs=5632, gated=True, conv=1, wd="bf16",
                      zipf=False, unit_logits=True, sweep=(1, 16, 64, 128, 256, 8192)),
    "deepseek_bf16": dict(d=2048, E=64, k=6, f=1408, fs=2816, gated=False, conv=1, wd="bf16",
                          zipf=True, sweep=(1, 16, 64, 128, 1024, 16384)),
    # Two shapes of the reference's model families (src/moe/family.rs) outside the benchmark list,
    # kept to see how the kernel plan's bounds carry over: Mixtral-8x22B, and a layer of 128
    # narrow experts with top-8 routing.
    "mixtral22b_bf16": dict(d=6144, E=8, k=2, f=16384, fs=0, gated=False, conv=0, wd="bf16",
                            zipf=False, sweep=(1, 64, 512, 4096)),
    "narrow128_bf16": dict(d=2048, E=128, k=8, f=768, fs=0, gated=False, conv=1, wd="bf16",
                           zipf=False, unit_logits=True, sweep=(1, 64, 512, 4096)),
    # DeepSeek-V3 router shape (256 experts in 8 groups, top-8 of the 4 best groups) in front of
    # narrow experts: times the sigmoid / group-limited routing path, not a checkpoint shape.
    "v3route_bf16": dict(d=7168, E=256, k=8, f=256, fs=256, gated=False, conv=1, wd="bf16",
                         zipf=False, sweep=(1, 256, 4096),
                         v3=dict(n_group=8, topk_group=4, scale=2.5, norm=True)),
}
D_MODEL, N_EXPERTS, TOP_K, D_FF = 4096, 8, 2, 14336
D_FF_SHARED = 0
W_BYTES = 2
GROUP = 0  # per-group int8: input elements per scale
GRAPH = False  # --graph: also time small batches replayed from HIP graphs
W_STD = 0.02
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E, GB/s
PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA, TFLOP/s
CONFIG_NAME = "mixtral_bf16"
ACT = 1  # element type of the device activations: capi.ACT_BF16, or capi.ACT_F32 for f32 layers
# Arithmetic type the expert kernels compute in, per storage type.
DTYPE = {"bf16": "bf16", "int8": "bf16 (int8 weights widened in registers, W8A16)",
         "int8g": "bf16 (int8 weights widened in registers, W8A16)", "f32": "f64"}


def measured_hbm_traffic():
    """HBM bytes per launch (read + written) of the expert kernels as rocprofv3 measured them:
    the `traffic <config> <tokens> <stage> <bytes>` lines that rocprof_summary.py writes into the
    counter summaries under profiles/ (FETCH_SIZE / WRITE_SIZE passes scaled by a plain device
    copy of known size).  {(config, tokens): {stage: (bytes, file, kernels_sha)}}; empty when no
    summary is there.  A summary carries the hash of the kernel sources it was taken with
    (`kernels_sha <hash>`): its figures are quoted only while that hash equals the one of the
    sources in this tree, otherwise `traffic` is null and `traffic_source` says why."""
    import glob
    out = {}
    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", "*hbm_counters*.txt"))):
        sha = None
        with open(path) as fh:
            for ln in fh:
                f = ln.split()
                if len(f) == 2 and f[0] == "kernels_sha":
                    sha = f[1]
                if len(f) == 5 and f[0] == "traffic":
                    out.setdefault((f[1], int(f[2])), {})[f[3]] = (float(f[4]), os.path.basename(path), sha)
    return out


MEASURED_HBM_TRAFFIC = measured_hbm_traffic()
try:
    from rocprof_summary import kernels_sha
    KERNELS_SHA = kernels_sha()
except Exception:  # the sources do not travel with every deployment of the library
    KERNELS_SHA = None


def traffic_of(config, tokens, stage):
    """(bytes or None, source description) for roofline.traffic."""
    hit = MEASURED_HBM_TRAFFIC.get((config, tokens), {}).get(stage)
    if hit is None:
        return None, None
    nbytes, path, sha = hit
    src = {"file": "profiles/" + path, "kernels_sha": sha, "this_build": KERNELS_SHA,
           "current": sha is not None and sha == KERNELS_SHA}
    return (nbytes if src["current"] else None), src


def make_weights(torch, np, seed, f32=False):
    """~N(0, 0.02) weights generated on the GPU.  bf16 / int8 configurations: truncated to bf16
    (the reference's storage convention, src/tensor/tensor.rs:306-308), returned as host uint16
    arrays.  f32 configuration: the f32 values themselves."""
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)

    def bf16_bits(shape):
        w = torch.randn(shape, generator=g, device="cuda", dtype=torch.float32) * W_STD
        if f32:
            return w.cpu().numpy()
        bits = (w.view(torch.int32) >> 16).to(torch.int16)
        return bits.cpu().numpy().view(np.uint16)

    gate = np.stack([bf16_bits((D_FF, D_MODEL)) for _ in range(N_EXPERTS)])
    up = np.stack([bf16_bits((D_FF, D_MODEL)) for _ in range(N_EXPERTS)])
    down = np.stack([bf16_bits((D_MODEL, D_FF)) for _ in range(N_EXPERTS)])
    router = bf16_bits((N_EXPERTS, D_MODEL))
    shared = None
    if D_FF_SHARED:
        shared = (bf16_bits((D_FF_SHARED, D_MODEL)), bf16_bits((D_FF_SHARED, D_MODEL)),
                  bf16_bits((D_MODEL, D_FF_SHARED)), upcast(np, bf16_bits((D_MODEL,))))
    return router, gate, up, down, shared


def upcast(np, bits):
    if bits.dtype == np.float32:
        return bits
    return (bits.astype(np.uint32) << 16).view(np.float32)


def measure(torch, np, capi, layer, T, steps, warmup, seed):
    """Times `steps` forwards of a T-token batch; returns a dict of figures."""
    n_buf = 8 if T <= 64 else 3
    g = torch.Generator(device="cuda")
    g.manual_seed(seed + T)
    xs = [torch.randn((T, D_MODEL), generator=g, device="cuda", dtype=torch.float32)
          for _ in range(n_buf)]
    if ACT == capi.ACT_BF16:
        xs = [x.to(torch.bfloat16) for x in xs]
    out = torch.empty((T, D_MODEL), device="cuda", dtype=torch.float32)
    stream = torch.cuda.current_stream().cuda_stream

    def step(i):
        layer.forward_device(xs[i % n_buf].data_ptr(), ACT, T, out.data_ptr(), stream)

    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        step(i)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps

    # The same steps replayed from HIP graphs (one per input buffer), as a serving loop would
    # issue them: no per-launch host work between the kernels of a step.
    graph_ms = None
    if GRAPH and T <= 64:
        side = torch.cuda.Stream()
        graphs = []
        with torch.cuda.stream(side):
            for i in range(n_buf):
                g_ = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g_, stream=side):
                    layer.forward_device(xs[i].data_ptr(), ACT, T, out.data_ptr(),
                                         torch.cuda.current_stream().cuda_stream)
                graphs.append(g_)
        torch.cuda.synchronize()
        for i in range(warmup):
            graphs[i % n_buf].replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(steps):
            graphs[i % n_buf].replay()
        torch.cuda.synchronize()
        graph_ms = (time.perf_counter() - t0) * 1e3 / steps

    # Per-stage durations: HIP events recorded by the library on the launch stream.
    layer.set_profiling(True)
    acc = np.zeros(capi.N_STAGES, dtype=np.float64)
    active = 0
    for i in range(steps):
        step(i)
        acc += layer.stage_ms()
        _, _, counts, _, _ = layer.last_routing(T)
        active += int((counts > 0).sum())
    layer.set_profiling(False)
    stage_ms = acc / steps
    launches = layer.stage_launches()
    rc, tok, ex = layer.status(stream)
    if rc != 0:
        raise RuntimeError(f"device status {rc} at token {tok}, expert {ex}")
    U = active / steps  # experts with at least one token (mean over steps)

    eb = W_BYTES  # bytes per stored weight
    # int8: one f32 scale per output row, or per output row and group of GROUP input elements
    sc_up = (4 * (-(-D_MODEL // GROUP) if GROUP else 1)) if W_BYTES == 1 else 0
    sc_down = (4 * (-(-D_FF // GROUP) if GROUP else 1)) if W_BYTES == 1 else 0
    sc_sdown = (4 * (-(-D_FF_SHARED // GROUP) if GROUP and D_FF_SHARED else 1)) if W_BYTES == 1 else 0
    fs = D_FF_SHARED
    # the shared expert (if any) runs as a second launch of the same kernels; both launches
    # of a stage are timed together, so their bytes / flops are added together too
    bytes_up = U * (2 * D_FF * D_MODEL * eb + 2 * D_FF * sc_up) + 2 * fs * D_MODEL * eb + 2 * fs * sc_up
    bytes_down = (U * (D_MODEL * D_FF * eb + D_MODEL * sc_down) + fs * D_MODEL * eb +
                  (D_MODEL * sc_sdown if fs else 0))
    bytes_fwd = (bytes_up + bytes_down + N_EXPERTS * D_MODEL * 4 +
                 T * D_MODEL * ((2 if ACT == capi.ACT_BF16 else 4) + 4))
    P = T * TOP_K
    flops_up = 4.0 * P * D_MODEL * D_FF + 4.0 * T * D_MODEL * fs
    flops_down = 2.0 * P * D_MODEL * D_FF + 2.0 * T * D_MODEL * fs
    flops_fwd = T * (2.0 * D_MODEL * N_EXPERTS + 6.0 * TOP_K * D_MODEL * D_FF + 6.0 * D_MODEL * fs)
    r = dict(
        tokens=T, ms_per_step=wall_ms, tokens_per_s=T / (wall_ms * 1e-3),
        graph_replay_ms_per_step=graph_ms,
        active_experts=U,
        stage_ms={n: float(v) for n, v in zip(capi.STAGES, stage_ms)},
        stage_launches={n: int(v) for n, v in zip(capi.STAGES, launches)},
        forward_gbs=bytes_fwd / (wall_ms * 1e-3) / 1e9,
        forward_tflops=flops_fwd / (wall_ms * 1e-3) / 1e12,
        forward_hbm_frac=bytes_fwd / (wall_ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
        forward_mfma_frac=flops_fwd / (wall_ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
        algorithmic_bytes=bytes_fwd, algorithmic_flops=flops_fwd,
    )
    up_ms, down_ms = stage_ms[2], stage_ms[3]
    dom, dom_ms, dom_bytes, dom_flops = (
        ("expert_gate_up", up_ms, bytes_up, flops_up) if up_ms >= down_ms
        else ("expert_down", down_ms, bytes_down, flops_down))
    traffic, traffic_src = traffic_of(CONFIG_NAME, T, dom)
    # HBM-bound while the weights outweigh the arithmetic: below ~300 rows per expert.
    hbm_bound = W_BYTES == 4 or ((dom_flops / (PEAK_BF16_TFLOPS * 1e12)) <
                                 (dom_bytes / (PEAK_HBM_GBS * 1e9)))
    if hbm_bound:
        ach = dom_bytes / (dom_ms * 1e-3) / 1e9
        r["roofline"] = dict(bound="hbm", kernel=dom, achieved=ach, peak=PEAK_HBM_GBS,
                             unit="GB/s", frac=ach / PEAK_HBM_GBS,
                             traffic=traffic, traffic_source=traffic_src,
                             kernel_ms=float(dom_ms), algorithmic_bytes=dom_bytes)
    else:
        ach = dom_flops / (dom_ms * 1e-3) / 1e12
        r["roofline"] = dict(bound="mfma", kernel=dom, achieved=ach, peak=PEAK_BF16_TFLOPS,
                             unit="TFLOP/s", frac=ach / PEAK_BF16_TFLOPS,
                             traffic=traffic, traffic_source=traffic_src,
                             kernel_ms=float(dom_ms), algorithmic_flops=dom_flops)
    return r, xs[0], out


def measure_block(torch, np, capi, layer, T, steps, warmup, seed):
    """The decoder layer's FFN block (RMSNorm * gamma -> layer -> residual add, f32 residual
    stream on the device) next to the bare layer forward on f32 rows of the same batch."""
    g = torch.Generator(device="cuda")
    g.manual_seed(seed + 7 * T)
    x1 = torch.randn((T, D_MODEL), generator=g, device="cuda", dtype=torch.float32)
    gamma = 1.0 + 0.1 * torch.randn((D_MODEL,), generator=g, device="cuda", dtype=torch.float32)
    out = torch.empty_like(x1)
    stream = torch.cuda.current_stream().cuda_stream

    def timed(fn):
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / steps

    fwd = timed(lambda: layer.forward_device(x1.data_ptr(), capi.ACT_F32, T, out.data_ptr(), stream))
    res = {"tokens": T, "forward_f32_rows_ms": fwd}
    for name, pol in (("graph_f32", capi.NORM_GRAPH_F32), ("f64", capi.NORM_F64)):
        ms = timed(lambda: layer.block_forward_device(x1.data_ptr(), T, gamma.data_ptr(), 1e-5, pol,
                                                      out.data_ptr(), stream))
        res[f"block_{name}_ms"] = ms
        res[f"block_{name}_over_forward_ms"] = ms - fwd
    rc, tok, ex = layer.status(stream)
    if rc != 0:
        raise RuntimeError(f"device status {rc} at token {tok}, expert {ex}")
    # the norm kernel reads x once from HBM (the second pass hits L2) and writes y once
    res["norm_algorithmic_bytes"] = 8.0 * T * D_MODEL
    return res


def measure_dequant(torch, capi, steps, warmup, seed):
    """The INT8 -> BF16 dequantisation launchers on one Mixtral expert projection ([K, N] =
    [4096, 14336] and its transpose), timed with events on the launch stream.  Algorithmic bytes
    per launch: K*N int8 read + 2*K*N bf16 written + the scales."""
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    stream = torch.cuda.current_stream().cuda_stream
    res = []
    for k, n in ((D_MODEL, D_FF), (D_FF, D_MODEL)):
        # six weight / output pairs in rotation (1 GB in all), so that no launch finds its
        # operands in the 256 MB Infinity Cache
        qs = [torch.randint(-127, 128, (k, n), generator=g, device="cuda", dtype=torch.int8)
              for _ in range(6)]
        outs = [torch.empty((k, n), device="cuda", dtype=torch.bfloat16) for _ in range(6)]
        for gs in (0, 128):
            ng = (k + gs - 1) // gs if gs else 1
            sc = torch.rand((ng, n), generator=g, device="cuda", dtype=torch.float32) * 1e-3 + 1e-4

            def fn(i):
                rc = capi.int8_to_bf16_launch_device(qs[i % 6].data_ptr(), sc.data_ptr(),
                                                     outs[i % 6].data_ptr(), k, n, group_size=gs,
                                                     stream=stream)
                if rc != 0:
                    raise RuntimeError(f"dequant launch failed: {rc}")
            for i in range(warmup):
                fn(i)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for i in range(steps):
                fn(i)
            e1.record()
            torch.cuda.synchronize()
            ms = e0.elapsed_time(e1) / steps
            nbytes = 3.0 * k * n + 4.0 * ng * n
            res.append({"k": k, "n": n, "group_size": gs, "us": ms * 1e3, "algorithmic_bytes": nbytes,
                        "gbs": nbytes / ms / 1e6, "hbm_frac": nbytes / ms / 1e6 / PEAK_HBM_GBS})
    return res


# Batch sizes the benchmark list names per configuration (decode and prefill points).
BENCHMARK_SWEEPS = {
    "tiny_f32": (64,),
    "mixtral_bf16": (1, 16, 128, 512, 4096),
    "mixtral_int8": (1, 16, 4096),
    "qwen_bf16": (1, 256, 8192),
    "deepseek_bf16": (1, 1024, 16384),
}
# Layer-output bar against the CPU path: max|a - ref| / max|ref|.
PARITY_BAR = {"f32": 1e-5, "bf16": 1e-2, "int8": 1e-2, "int8g": 1e-2}


def compact(config, r):
    """One entry of the `configs` list: what a table row needs."""
    hbm = r["roofline"]["bound"] == "hbm"
    return dict(config=config, tokens=r["tokens"], ms_per_step=r["ms_per_step"],
                tokens_per_s=r["tokens_per_s"], bound=r["roofline"]["bound"],
                forward_frac=r["forward_hbm_frac"] if hbm else r["forward_mfma_frac"],
                forward_hbm_frac=r["forward_hbm_frac"], forward_mfma_frac=r["forward_mfma_frac"],
                active_experts=r["active_experts"], stage_ms=r["stage_ms"],
                roofline=r["roofline"])


def build_config(torch, np, capi, name, seed, tmax):
    """Sets the module's shape globals to configuration `name`, generates its weights and builds
    its layer (experts resident in HBM).  Returns what the measurements and the CPU check need."""
    global D_MODEL, N_EXPERTS, TOP_K, D_FF, D_FF_SHARED, W_BYTES, CONFIG_NAME, GROUP, ACT
    cfg = CONFIGS[name]
    CONFIG_NAME = name
    D_MODEL, N_EXPERTS, TOP_K, D_FF, D_FF_SHARED = cfg["d"], cfg["E"], cfg["k"], cfg["f"], cfg["fs"]
    f32w = cfg["wd"] == "f32"
    W_BYTES = 4 if f32w else 1 if cfg["wd"] in ("int8", "int8g") else 2
    ACT = capi.ACT_F32 if f32w else capi.ACT_BF16
    GROUP = 128 if cfg["wd"] == "int8g" else 0
    router, gate, up, down, shared = make_weights(torch, np, seed, f32=f32w)
    router_f32 = upcast(np, router)
    if cfg["zipf"] or cfg.get("unit_logits"):  # router rows ~ N(0, 1/d): logits ~ N(0, 1)
        router_f32 = router_f32 * np.float32(1.0 / (W_STD * np.sqrt(D_MODEL)))
        router_f32 = upcast(np, capi.f32_to_bf16_trunc(router_f32))
    kw = dict(w_router=router_f32, top_k=TOP_K, convention=cfg["conv"], max_tokens_hint=tmax)
    if cfg["zipf"]:  # plus a log-Zipf(1.2) bias: skewed expert load
        rank = np.random.default_rng(seed).permutation(N_EXPERTS) + 1.0
        kw["router_bias"] = (-1.2 * np.log(rank)).astype(np.float32)
    if shared is not None and cfg["gated"]:
        kw["shared_gate"] = shared[3]
    # what the CPU path computes with: the stored values, upcast / dequantised to f32
    stored = dict(w_gate=upcast(np, gate), w_up=upcast(np, up), w_down=upcast(np, down))
    if shared is not None:
        stored.update(s_gate=upcast(np, shared[0]), s_up=upcast(np, shared[1]),
                      s_down=upcast(np, shared[2]))
    if cfg["wd"] in ("int8", "int8g"):
        # int8 of the bf16-valued weights (per output row, or per row and 128-element group),
        # 0.1 % of rows scaled x8 first
        rng = np.random.default_rng(seed + 1)
        per_group = cfg["wd"] == "int8g"
        if per_group:
            kw["group_size"] = 128

        def q8(bits, name):
            w = upcast(np, bits)
            rows = w.reshape(-1, w.shape[-1])
            rows[rng.choice(rows.shape[0], size=rows.shape[0] // 1000, replace=False)] *= 8.0
            q, sc = capi.quantize_per_group_i8(w, 128) if per_group else capi.quantize_per_row_i8(w)
            full = np.repeat(sc, 128, axis=-1)[..., :w.shape[-1]] if per_group else sc[..., None]
            stored[name] = q.astype(np.float32) * full
            return q, sc
        (gate, sg), (up, su), (down, sd) = q8(gate, "w_gate"), q8(up, "w_up"), q8(down, "w_down")
        kw.update(scale_gate=sg, scale_up=su, scale_down=sd)
        if shared is not None:
            (g_, a1), (u_, a2), (d_, a3) = (q8(shared[0], "s_gate"), q8(shared[1], "s_up"),
                                            q8(shared[2], "s_down"))
            shared = (g_, u_, d_, shared[3])
            kw.update(s_scale_gate=a1, s_scale_up=a2, s_scale_down=a3)
        wdt = capi.WEIGHT_INT8_PER_GROUP if per_group else capi.WEIGHT_INT8_W8A16
    else:
        wdt = capi.WEIGHT_F32 if f32w else capi.WEIGHT_BF16
    if shared is not None:
        kw.update(s_gate=shared[0], s_up=shared[1], s_down=shared[2])
    layer = capi.Layer(w_gate=gate, w_up=up, w_down=down, weight_dtype=wdt, **kw)
    e_bias = None
    if cfg.get("v3"):
        v3 = cfg["v3"]
        e_bias = (0.05 * np.random.default_rng(seed + 2).standard_normal(N_EXPERTS)).astype(np.float32)
        layer.set_v3_router(v3["n_group"], v3["topk_group"], v3["scale"], v3["norm"], e_bias)
    return dict(name=name, cfg=cfg, layer=layer, router_f32=router_f32, kw=kw, stored=stored,
                e_bias=e_bias)


def cpu_and_parity(torch, np, capi, ctx, x_head, out_head, tokens, cpu_tokens):
    """The CPU path (the oracle: checker and reported baseline, never part of what is timed on
    the GPU) on the first n tokens of the batch, and the parity report of the batch: routing of
    every token against the CPU path, the smallest routing margin of the batch (k-th minus
    (k+1)-th largest logit: how close the batch comes to a tie, the reference's fragility signal,
    tests/moe_cert2_qwen_decomposition_test.rs:79-86), and on the n sample tokens the layer-output
    bar max|a - ref| / max|ref| plus the reference's own metric block (src/moe/numerical.rs:58-88)."""
    from oracle import moe_oracle as ora
    cfg, layer, kw = ctx["cfg"], ctx["layer"], ctx["kw"]
    flops_tok = 2.0 * D_MODEL * N_EXPERTS + 6.0 * TOP_K * D_MODEL * D_FF + 6.0 * D_MODEL * D_FF_SHARED
    n = cpu_tokens if cpu_tokens > 0 else int(1024 * 704.7e6 / flops_tok)
    n = max(1, min(n, tokens))
    if cfg.get("v3") and cpu_tokens < 0:
        n = min(n, 512)  # that path runs token by token on one core
    # the batch recomputed once so that `out_head` matches `x_head`
    layer.forward_device(x_head.data_ptr(), ACT, tokens, out_head.data_ptr(),
                         torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    idx_gpu, *_ = layer.last_routing(tokens)
    xs = x_head[:n].to(torch.float32).cpu().numpy()
    got = out_head[:n].cpu().numpy()
    oL = ora.Layer(w_router=ctx["router_f32"], top_k=TOP_K, convention=cfg["conv"],
                   shared_gate=kw.get("shared_gate"), router_bias=kw.get("router_bias"),
                   **ctx["stored"])
    cores = ora.hw_threads()
    ora.set_threads(cores)
    if cfg.get("v3"):  # the DeepSeek-V3 router in front of the same experts (one thread)
        v3 = cfg["v3"]
        cores = 1
        run = lambda rows: oL.v3_forward(rows, ctx["e_bias"], v3["n_group"], v3["topk_group"],
                                         v3["scale"], v3["norm"])[:2]
    else:
        run = lambda rows: oL.execute(rows)[:2]
    run(xs[:1])  # warm the pages
    t0 = time.perf_counter()
    ref, o_idx = run(xs)
    dt = time.perf_counter() - t0
    cpu = dict(value=n / dt, unit="tokens/s", cores=cores, kind="port",
               sample=f"{n} tokens of the T={tokens} batch, certified policy "
                      "(f32 weights, f64 accumulation), rows parallel over the cores used")
    margin = None
    if cfg.get("v3"):  # routing checked on the sample the CPU path ran
        o_all, idx_gpu, n_routed = o_idx, idx_gpu[:n], n
    else:
        o_all, _, logits = oL.route_tokens(x_head.to(torch.float32).cpu().numpy(), want_logits=True)
        n_routed = int(tokens)
        if TOP_K < N_EXPERTS:
            srt = np.sort(logits.astype(np.float64), axis=1)[:, ::-1]
            gaps = srt[:, TOP_K - 1] - srt[:, TOP_K]
            margin = dict(min_routing_margin=float(gaps.min()), at_token=int(gaps.argmin()),
                          median_routing_margin=float(np.median(gaps)))
    bar = PARITY_BAR[cfg["wd"]]
    rel = float(np.abs(got - ref).max() / np.abs(ref).max())
    parity = dict(
        routing_mismatched_tokens=int((idx_gpu != o_all).any(axis=1).sum()),
        tokens_routed=n_routed,
        max_rel_err_vs_cpu_path=rel, bar=bar, within_bar=bool(rel <= bar),
        sample_tokens=n)
    if margin:
        parity.update(margin)
    # the reference's metric block (max_abs_diff, mean_abs_diff, rmse over the sample; its
    # argmax check is made per output row, as it is made per logits vector there)
    m = ora.numerical_metrics(got, ref)
    rows = [ora.numerical_metrics(got[i], ref[i])["argmax_match"] for i in range(n)]
    parity.update(max_abs_diff=m["max_abs_diff"], mean_abs_diff=m["mean_abs_diff"], rmse=m["rmse"],
                  argmax_match_rows=int(sum(rows)), argmax_rows=n)
    return cpu, parity


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=20)  # 20 x 2.4 ms: the clocks are up by then
    ap.add_argument("--config", default="mixtral_bf16", choices=sorted(CONFIGS),
                    help="layer shape (the headline metric is quoted on mixtral_bf16)")
    ap.add_argument("--tokens", type=int, default=0,
                    help="headline batch size T (default: the config's largest)")
    ap.add_argument("--decode-tokens", type=str, default="1,16",
                    help="decode batch sizes, comma separated (empty = skip); reported as "
                         "`decode` (the first) and `decode<T>` (the others)")
    ap.add_argument("--sweep", type=str, default="default",
                    help="extra batch sizes, comma separated (default: 128 and 512 tokens where the "
                         "configuration lists them; \"all\": the configuration's own list)")
    ap.add_argument("--all-configs", choices=("auto", "yes", "no"), default="auto",
                    help="after the headline block, time every configuration of the benchmark list "
                         "at its own batch sizes (`configs`); auto = with the default configuration "
                         "unless the CPU leg is switched off")
    ap.add_argument("--cpu-tokens", type=int, default=-1,
                    help="tokens of the CPU-baseline sample (0 = skip; default: about 12 s of "
                         "CPU work on 16 cores)")
    ap.add_argument("--host-steps", type=int, default=3,
                    help="timed calls of the host-buffer entry point on the headline batch (0 = skip)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 1 GiB device copy (reference point for HBM counters)")
    ap.add_argument("--graph", action="store_true",
                    help="also time batches of up to 64 tokens replayed from HIP graphs")
    ap.add_argument("--block", action="store_true",
                    help="also time the decoder-layer FFN block entry point (norm + layer + residual)")
    ap.add_argument("--dequant", action="store_true",
                    help="also time the INT8 -> BF16 dequantisation launchers")
    ap.add_argument("--seed", type=int, default=1234)
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py: this path runs on one GPU (all experts resident in one HBM, no "
              "collectives); --gpus must be 1", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    from ateniaengine_amd import capi

    if not capi.available():
        print("bench.py: no gfx950 device; the HIP path has no fallback", file=sys.stderr)
        sys.exit(3)
    torch.cuda.set_device(0)
    global GRAPH
    GRAPH = a.graph
    cfg = CONFIGS[a.config]
    if a.tokens <= 0:
        a.tokens = max(cfg["sweep"])
    decode_ts = [int(t) for t in a.decode_tokens.split(",") if t]
    decode_ts = [t for t in decode_ts if t > 0 and t != a.tokens and
                 (t in cfg["sweep"] or a.decode_tokens != "1,16")]
    if a.sweep == "all":
        a.sweep = ",".join(str(t) for t in cfg["sweep"] if t != a.tokens and t not in decode_ts)
    elif a.sweep == "default":  # the batch sizes of the configuration's own list between the two
        a.sweep = ",".join(str(t) for t in (128, 512)
                           if t in cfg["sweep"] and t != a.tokens and t not in decode_ts)
    sweep_ts = [int(t) for t in a.sweep.split(",") if t and int(t) > 0]  # "0" = none
    ctx = build_config(torch, np, capi, a.config, a.seed, max([a.tokens] + decode_ts + sweep_ts))
    layer = ctx["layer"]

    if a.calibrate_copy:
        src = torch.empty(1 << 28, device="cuda", dtype=torch.float32)  # 1 GiB
        src.fill_(1.0)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    head, x_head, out_head = measure(torch, np, capi, layer, a.tokens, a.steps, a.warmup, a.seed)
    decodes = {}
    for t in decode_ts:
        decodes[t], _, _ = measure(torch, np, capi, layer, t, max(a.steps, 50), max(a.warmup, 10),
                                   a.seed)
    sweep = []
    for t in sweep_ts:
        r, _, _ = measure(torch, np, capi, layer, t, a.steps if t >= 512 else max(a.steps, 50),
                          a.warmup, a.seed)
        sweep.append(r)

    block = None
    if a.block:
        block = [measure_block(torch, np, capi, layer, t, a.steps if t >= 512 else max(a.steps, 50),
                               a.warmup, a.seed)
                 for t in sorted({a.tokens} | set(decode_ts) | set(sweep_ts)) if t > 0]

    # The entry point a caller of the reference's op reaches: [T * d] f32 in host memory in and
    # out (src/amg/graph.rs:5572-5589 hands a Vec<f32> over).  PCIe-inclusive, never `value`.
    host = None
    if a.host_steps > 0:
        xh = x_head.to(torch.float32).cpu().numpy()
        oh = np.zeros_like(xh)  # the caller's output buffer, its pages touched once
        layer.forward(xh, out=oh)
        t0 = time.perf_counter()
        for _ in range(a.host_steps):
            layer.forward(xh, out=oh)
        host_ms = (time.perf_counter() - t0) * 1e3 / a.host_steps
        # the same entry point when the caller's buffers are page-locked (hipHostMalloc /
        # torch pin_memory): the copies then run as direct DMA
        xp = torch.empty((a.tokens, D_MODEL), dtype=torch.float32, pin_memory=True)
        op = torch.empty((a.tokens, D_MODEL), dtype=torch.float32, pin_memory=True)
        xp.copy_(torch.from_numpy(xh))
        call = lambda: capi._check(capi.lib().atenia_moe_hip_layer_forward(
            layer._h, xp.data_ptr(), a.tokens, op.data_ptr()))
        call()
        t0 = time.perf_counter()
        for _ in range(a.host_steps):
            call()
        pinned_ms = (time.perf_counter() - t0) * 1e3 / a.host_steps
        host = dict(tokens=a.tokens, forward_host_ms=host_ms, forward_host_pinned_ms=pinned_ms,
                    tokens_per_s=a.tokens / (host_ms * 1e-3),
                    host_bytes_moved=2.0 * a.tokens * D_MODEL * 4,
                    note="atenia_moe_hip_layer_forward, synchronous, [T*d] f32 in and out: "
                         "pageable caller buffers / page-locked caller buffers")
        del xp, op, xh, oh

    cpu = None
    parity = None
    if a.cpu_tokens != 0:
        cpu, parity = cpu_and_parity(torch, np, capi, ctx, x_head, out_head, a.tokens, a.cpu_tokens)

    f32w = cfg["wd"] == "f32"
    line = {
        "metric": "Mixtral-shape MoE layer tok/s; decode HBM GB/s and prefill MFMA TFLOPS",
        "value": head["tokens_per_s"], "unit": "tokens/s", "n_gpus": 1, "steps": a.steps,
        "warmup": a.warmup, "ms_per_step": head["ms_per_step"], "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": DTYPE[cfg["wd"]], "data": "synthetic",
        "config": {"workload": f"{a.config}: MoE layer, d_model={D_MODEL}, experts={N_EXPERTS}, "
                               f"top_k={TOP_K}, d_ff={D_FF}, shared d_ff={D_FF_SHARED}, "
                               f"{cfg['wd']} weights resident in HBM, "
                               f"{'f32' if f32w else 'bf16'} activations, "
                               f"T={a.tokens} tokens per step",
                   "tokens_per_step": a.tokens},
        "roofline": head["roofline"],
        "cpu_baseline": cpu,
        "prefill": head,
        "decode": decodes.get(decode_ts[0]) if decode_ts else None,
        "sweep": sweep,
        "parity": parity,
        "host_entry": host,
        "kernels_sha": KERNELS_SHA,
    }
    for t in decode_ts[1:]:
        line[f"decode{t}"] = decodes[t]
    if block is not None:
        line["block"] = block
    if a.dequant:
        line["dequant"] = measure_dequant(torch, capi, max(a.steps, 50), a.warmup, a.seed)

    # Every configuration of the benchmark list at its own batch sizes, one compact entry per
    # (configuration, T) (the reference's own bench walks its three families in one run,
    # tests/moe_perf_scale_bench.rs:70-75); the headline configuration's entries repeat the
    # figures above.  Weights are generated on the device as for the headline; the CPU path is
    # timed on the headline only, here it checks a small token sample per configuration.
    if a.all_configs == "auto":
        a.all_configs = "yes" if a.config == "mixtral_bf16" and a.cpu_tokens != 0 else "no"
    if a.all_configs == "yes":
        entries = [compact(a.config, r) for r in
                   sorted([head] + list(decodes.values()) + sweep, key=lambda r: r["tokens"])]
        parities = {a.config: parity}
        layer.close()
        del ctx, layer, x_head, out_head
        for name in BENCHMARK_SWEEPS:
            if name == a.config:
                continue
            ts = BENCHMARK_SWEEPS[name]
            ctx = build_config(torch, np, capi, name, a.seed, max(ts))
            xo = None
            for t in ts:
                r, x_t, out_t = measure(torch, np, capi, ctx["layer"], t,
                                        a.steps if t >= 512 else max(a.steps, 50), a.warmup, a.seed)
                entries.append(compact(name, r))
                xo = (x_t, out_t, t)
            _, parities[name] = cpu_and_parity(torch, np, capi, ctx, xo[0], xo[1], xo[2],
                                               min(xo[2], 64))
            if CONFIGS[name]["wd"] == "f32":
                # the reference's other expert arithmetic for f32 layers (NumericPolicy::Strict,
                # and what Fast falls back to: f32 accumulation, numeric_policy.rs:36-75)
                ctx["layer"].set_numeric_policy(capi.POLICY_STRICT)
                r, _, _ = measure(torch, np, capi, ctx["layer"], ts[-1], max(a.steps, 50), a.warmup, a.seed)
                e = compact(name, r)
                e["numeric_policy"] = "strict"
                entries.append(e)
                ctx["layer"].set_numeric_policy(capi.POLICY_CERTIFIED)
            ctx["layer"].close()
            del ctx, xo
        line["configs"] = entries
        line["configs_parity"] = parities
    print(json.dumps(line))


if __name__ == "__main__":
    main()
