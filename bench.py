#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload vanilla|all|...]

A "step" is one `forward` of the vanilla causal GQA attention module on the Llama3-8B shape
(batch 1, 32 query / 8 KV heads, seq 4096, head_dim 128, fp16): the configuration the headline
metric is quoted on.  Inputs are synthetic, generated from a seed, and resident in HBM before the
timed region.  Timing follows the reference's own method (vanilla_llama_benchmark.py:254-294): one
cold call, warm-ups on a side stream, `forward` captured into a graph, K replays -- bracketed here
by device synchronisation and a wall clock for `value`, and by events on the launch stream for the
kernel's own duration (`roofline`).

Prints ONE JSON line.  `value` = causal-halved attention flops (4*B*H*S^2*D/2) per second.  The same
line carries the RMSNorm [4096x4096] HBM rate (rotating buffers, so the 256 MB last-level cache
cannot serve the reads), the other variants' rates when --workload all, and the CPU oracle timed on
this machine's host cores on a bounded sample of the same workload.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="all",
                    help="all (the headline, RMSNorm, the four other prefill workloads and the decode-append timings: the "
                         "default), headline (vanilla attention + RMSNorm only), or one of vanilla rmsnorm prenorm qknorm "
                         "keyformer roco decode, or sweep (vanilla attention over sequence lengths and head shapes)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-decode", action="store_true", help="with --workload all: skip the decode-append timings")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="budget for the CPU baseline sample")
    ap.add_argument("--inputs", default="randn", choices=("randn", "zeros"),
                    help="zeros: run the headline attention on all-zero Q, K, V instead of the benchmark's N(0,1) data -- a "
                         "diagnostic for profiler runs (same instructions, no switching activity: the difference is the "
                         "board's clock under its power limit); the line's `data` says so and it is not the benchmark")
    ap.add_argument("--no-zero-leg", action="store_true",
                    help="skip the all-zero-input diagnostic launch of the headline kernel (profiler runs: every dispatch "
                         "of the kernel in the trace is then the benchmark's)")
    ap.add_argument("--calibrate", action="store_true",
                    help="also run the library's plain copy kernel on 256 MiB (3 launches) so that a rocprofv3 --pmc run "
                         "of this command holds a kernel of known HBM traffic to scale FETCH_SIZE / WRITE_SIZE by")
    return ap.parse_args()


CLOCK_WARMUP_S = 0.25      # untimed replays before any timed region: the board's clocks take tens of ms to settle
REPEATS = 5                # the timed region (exactly `steps` forwards) is run this many times; the median is reported


def _settle(replay, stream, seconds=CLOCK_WARMUP_S):
    """Untimed replays until `seconds` of device work have run (a cold board is about 10 % slower for the first
    30 ms of a burst than in steady state, and a single short timed region would measure mostly that)."""
    import torch
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        with torch.cuda.stream(stream):
            for _ in range(4):
                replay()
        stream.synchronize()


def graph_timed(module, tensors, steps, warmup, per_graph=20, with_samples=False):
    """The reference driver's sequence -- cold call, warm-ups on a side stream, `forward` captured into a
    graph, replays -- except that one graph holds up to `per_graph` consecutive forwards, so that the gaps
    between graph launches (about as long as 5% of one attention kernel) stay out of the kernel timing.
    A timed region is exactly `steps` forwards between device synchronisations; it is run REPEATS times after
    the clocks have settled and the median region is reported.  Returns (wall ms/step, event ms/step)
    [, the event ms/step of every region]."""
    import torch
    args = [tensors[p] for p in module.TENSOR_PARAMS]
    module.forward(*args)                       # cold call (allocates the module's workspaces)
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for _ in range(max(warmup, 1)):
            module.forward(*args)
    stream.synchronize()
    sizes = [per_graph] * (steps // per_graph) + ([steps % per_graph] if steps % per_graph else [])
    graphs = {}
    for n in set(sizes):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.stream(stream):
            with torch.cuda.graph(g, stream=stream):
                for _ in range(n):
                    module.forward(*args)
        graphs[n] = g
    stream.synchronize()
    _settle(graphs[sizes[0]].replay, stream)
    regions = []
    for _ in range(REPEATS):
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        with torch.cuda.stream(stream):
            start.record()
            for n in sizes:
                graphs[n].replay()
            end.record()
        torch.cuda.synchronize()
        regions.append(((time.perf_counter() - t0) * 1e3 / steps, start.elapsed_time(end) / steps))
    regions_by_ev = sorted(regions, key=lambda r: r[1])
    wall_ms, ev_ms = regions_by_ev[len(regions) // 2]
    if with_samples:
        return wall_ms, ev_ms, [r[1] for r in regions]
    return wall_ms, ev_ms


def rotating_timed(fn_for, n_buffers, steps, warmup):
    """One graph holding n_buffers launches, each on its own buffer set (so a launch never finds its data in
    the last-level cache), replayed until `steps` launches have run; REPEATS such regions after the clocks have
    settled, the median reported; returns (wall ms/launch, event ms/launch).
    Capturing takes the Python call overhead -- longer than a 13 us kernel -- out of the timed region."""
    import torch
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for i in range(max(warmup, n_buffers)):
            fn_for(i % n_buffers)
    stream.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            for i in range(n_buffers):
                fn_for(i)
    stream.synchronize()
    reps = max(1, (steps + n_buffers - 1) // n_buffers)
    _settle(graph.replay, stream, 0.1)
    n = reps * n_buffers
    regions = []
    for _ in range(REPEATS):
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        with torch.cuda.stream(stream):
            start.record()
            for _ in range(reps):
                graph.replay()
            end.record()
        torch.cuda.synchronize()
        regions.append(((time.perf_counter() - t0) * 1e3 / n, start.elapsed_time(end) / n))
    regions.sort(key=lambda r: r[1])
    return regions[len(regions) // 2]


def attn_inputs(cfg, seed=42):
    import torch
    from triton_amd.configs import randn_half
    g = torch.Generator().manual_seed(seed)
    B, Hq, Hkv, S, D = cfg["batch"], cfg["n_heads"], cfg["n_kv_heads"], cfg["seq"], cfg["head_dim"]
    q = randn_half((B, Hq, S, D), g); k = randn_half((B, Hkv, S, D), g); v = randn_half((B, Hkv, S, D), g)
    return q, k, v


def bench_vanilla(steps, warmup, inputs="randn", zero_leg=True):
    import torch
    from triton_amd import configs, modules
    cfg = configs.VANILLA
    q, k, v = attn_inputs(cfg)
    t = dict(Q=q.cuda(), K=k.cuda(), V=v.cuda(), O=torch.zeros_like(q).cuda())
    if inputs == "zeros":
        for name in "QKV":
            t[name].zero_()
    wall, ev, samples = graph_timed(modules.get("vanilla"), t, steps, warmup, with_samples=True)
    zero_ms = None
    if inputs == "randn" and zero_leg:
        # The same launch on all-zero inputs (same instructions and memory traffic, no switching activity in the
        # datapaths): what the kernel's cycles alone take when the board does not lower its clock.
        tz = {name: torch.zeros_like(x) for name, x in t.items()}
        _, zero_ms = graph_timed(modules.get("vanilla"), tz, min(steps, 100), warmup)
    flops = configs.attn_flops(cfg["batch"], cfg["n_heads"], cfg["seq"], cfg["seq"], cfg["head_dim"], True)
    from triton_amd import ops
    kernel = ops.attention_kernel_name(t["Q"], t["K"], t["V"], t["O"], cfg["head_dim"] ** -0.5, True)
    return dict(wall_ms=wall, kernel_ms=ev, flops=flops, tflops=flops / wall / 1e9, kernel_tflops=flops / ev / 1e9,
                tensors=(q, k, v), kernel=kernel, region_ms=samples, zero_inputs_kernel_ms=zero_ms)


def bench_sweep(steps, warmup):
    """Vanilla attention over sequence lengths and the two head shapes of the benchmark configurations (not part of the
    default run): TFLOP/s on N(0,1) inputs and on all-zero inputs per shape, same timing method as the headline."""
    import torch
    from triton_amd import configs, modules
    m = modules.get("vanilla")
    rows = []
    shapes = [("llama3 GQA 32/8 x 128", 1, 32, 8, 128, S, True) for S in (512, 1024, 2048, 4096, 8192, 16384, 32768)]
    shapes += [("llama3 GQA 32/8 x 128", 4, 32, 8, 128, 4096, True), ("llama3 GQA 32/8 x 128", 1, 32, 8, 128, 4096, False)]
    shapes += [("falcon MQA 71/1 x 64", 1, 71, 1, 64, S, True) for S in (1024, 2048, 4096, 8192, 16384)]
    for label, B, Hq, Hkv, D, S, causal in shapes:
        g = torch.Generator(device="cuda").manual_seed(42)
        t = dict(Q=torch.randn(B, Hq, S, D, device="cuda", generator=g).half(),
                 K=torch.randn(B, Hkv, S, D, device="cuda", generator=g).half(),
                 V=torch.randn(B, Hkv, S, D, device="cuda", generator=g).half())
        t["O"] = torch.zeros_like(t["Q"])
        mod = m if causal else modules.get("vanilla", causal=False)
        n = max(10, min(steps, int(2e13 / configs.attn_flops(B, Hq, S, S, D, causal))))
        flops = configs.attn_flops(B, Hq, S, S, D, causal)
        _, ev = graph_timed(mod, t, n, warmup, per_graph=min(20, n))
        for x in "QKV":
            t[x].zero_()
        _, evz = graph_timed(mod, t, n, warmup, per_graph=min(20, n))
        rows.append(dict(shape=label, batch=B, seq=S, causal=causal, us=round(ev * 1e3, 2), tflops=round(flops / ev / 1e9, 1),
                         frac=round(flops / ev / 1e9 / configs.MFMA_F16_PEAK_TFLOPS, 4),
                         zero_inputs_us=round(evz * 1e3, 2), zero_inputs_frac=round(flops / evz / 1e9 / configs.MFMA_F16_PEAK_TFLOPS, 4)))
        del t
        torch.cuda.empty_cache()
    return rows


def bench_rmsnorm(steps, warmup):
    import torch
    from triton_amd import configs, modules
    cfg = configs.RMSNORM
    R = 16                                            # 16 x (32 MiB in + 32 MiB out) = 1 GiB >> 256 MB cache
    gen = torch.Generator(device="cuda").manual_seed(42)
    xs = [torch.randn(cfg["rows"], cfg["cols"], device="cuda", generator=gen).half() for _ in range(R)]
    ys = [torch.empty_like(x) for x in xs]
    gamma = (1 + 0.02 * torch.randn(cfg["cols"], device="cuda", generator=gen)).half()
    m = modules.get("rms", eps=cfg["eps"])
    wall, ev = rotating_timed(lambda i: m.forward(xs[i], ys[i], gamma), R, max(steps, 64), warmup)
    hot_wall, hot_ev = rotating_timed(lambda i: m.forward(xs[0], ys[0], gamma), 4, max(steps, 64), warmup)
    # the same footprint through a plain copy kernel: what a 1:1 read/write stream reaches on this machine
    from triton_amd import ops
    _, copy_ev = rotating_timed(lambda i: ops.calibration_copy(xs[i], ys[i]), R, max(steps, 64), warmup)
    # ... and through a copy this build did not write: torch's Tensor.copy_ (device to device) on the same buffer pairs
    _, tcopy_ev = rotating_timed(lambda i: ys[i].copy_(xs[i]), R, max(steps, 64), warmup)
    nbytes = configs.rmsnorm_bytes(cfg["rows"], cfg["cols"])
    cbytes = 2 * cfg["rows"] * cfg["cols"] * 2
    return dict(kernel_us=ev * 1e3, gbps=nbytes / ev / 1e6, frac=nbytes / ev / 1e6 / configs.HBM_PEAK_GBPS,
                hot_cache_gbps=nbytes / hot_ev / 1e6, bytes=nbytes, rotating_buffers=R,
                copy_gbps=cbytes / copy_ev / 1e6, copy_us=copy_ev * 1e3,
                torch_copy_gbps=cbytes / tcopy_ev / 1e6, torch_copy_us=tcopy_ev * 1e3)


def bench_variant(name, steps, warmup):
    import torch
    from triton_amd import configs, modules
    randn_half = configs.randn_half
    g = torch.Generator().manual_seed(42)
    if name == "qknorm":
        cfg = configs.QKNORM
        q, k, v = attn_inputs(cfg)
        D = cfg["head_dim"]
        t = dict(Q=q.cuda(), K=k.cuda(), V=v.cuda(), O=torch.zeros_like(q).cuda(),
                 gamma_q=randn_half((D,), g, 1, 0.02).cuda(), gamma_k=randn_half((D,), g, 1, 0.02).cuda())
        m = modules.get("qknorm", eps=cfg["eps"])
        flops = configs.attn_flops(1, cfg["n_heads"], cfg["seq"], cfg["seq"], D, True)
    elif name == "prenorm":
        cfg = configs.PRENORM
        S, N, D = cfg["seq"], cfg["hidden"], cfg["head_dim"]
        nkv = cfg["n_kv_heads"] * D
        t = dict(X=randn_half((1, S, N), g).cuda(), gamma=randn_half((N,), g, 1, 0.02).cuda(),
                 WQ=randn_half((N, N), g, 0, 0.02).cuda(), WK=randn_half((N, nkv), g, 0, 0.02).cuda(),
                 WV=randn_half((N, nkv), g, 0, 0.02).cuda(), O=torch.zeros(1, S, N, dtype=torch.float16, device="cuda"))
        m = modules.get("prenorm", head_dim=D, eps=cfg["eps"])
        flops = configs.qkv_gemm_flops(S, N, N, nkv) + configs.attn_flops(1, cfg["n_heads"], S, S, D, True)
    elif name in ("keyformer", "roco"):
        cfg = configs.KEYFORMER if name == "keyformer" else configs.ROCO
        q, k, v = attn_inputs(cfg)
        B, Hq, S, D = 1, cfg["n_heads"], cfg["seq"], cfg["head_dim"]
        t = dict(Q=q.cuda(), K=k.cuda(), V=v.cuda(), O=torch.zeros_like(q).cuda())
        if name == "keyformer":
            gen = torch.Generator(device="cuda").manual_seed(cfg["noise_seed"])     # throughput only: device-side noise
            u = torch.rand(B, Hq, S, S, device="cuda", generator=gen).clamp_(1e-10, 1 - 1e-7)
            t["noise"] = -torch.log(-torch.log(u)); del u
            t["C_out"] = torch.zeros(B, Hq, S, device="cuda")
            m = modules.get("keyformer", tau=cfg["tau"])
        else:
            t["C_out1"] = torch.zeros(B, Hq, S, device="cuda"); t["C_out2"] = torch.zeros(B, Hq, S, device="cuda")
            m = modules.get("roco", stats="mean_std")       # the output form the RoCo configuration names
        flops = configs.attn_flops(1, Hq, S, S, D, True)
    else:
        raise SystemExit(f"unknown workload {name}")
    wall, ev = graph_timed(m, t, steps, warmup)
    out = dict(ms=ev, tflops=flops / ev / 1e9, frac_mfma=flops / ev / 1e9 / configs.MFMA_F16_PEAK_TFLOPS)
    if name == "keyformer":
        S, Hq = cfg["seq"], cfg["n_heads"]
        nbytes = Hq * S * (S + 1) // 2 * 4 + 83886080 + Hq * S * 4 * 4
        out.update(algorithmic_bytes=nbytes, gbps=nbytes / ev / 1e6, frac_hbm=nbytes / ev / 1e6 / configs.HBM_PEAK_GBPS)
    return out


def bench_decode(steps, warmup):
    """The reference's own problem form (M new tokens projected, appended to the caches, attended over P+M keys;
    convert_eval_rms.py:33-60).  Microseconds per forward for each variant at the Llama and Falcon widths, and the
    bytes that must move.  `<variant>_us`: forwards back to back, 20 per graph, i.e. the GPU's own time per forward;
    `<variant>_replay_us`: the way the reference's drivers time a candidate, one forward per graph replay, which for
    steps this short also measures how fast the host can launch graphs (10-30 us per replay, by the box)."""
    import torch
    from triton_amd import configs, modules
    out = {}
    for name, cfg in (("llama", configs.DECODE_LLAMA), ("falcon", configs.DECODE_FALCON)):
        M, N, D, H, P = cfg["M"], cfg["N"], cfg["D"], cfg["H"], cfg["P"]
        g = torch.Generator(device="cuda").manual_seed(42)
        rnd = lambda *shape: torch.randn(*shape, device="cuda", generator=g).clamp_(-1, 1).mul_(0.01).half()
        t = dict(X=rnd(M, N), WQ=rnd(N, N), WK=rnd(N, N), WV=rnd(N, N), K_cache=rnd(H, P + M, D), V_cache=rnd(H, P + M, D),
                 O2=torch.zeros(M, N, dtype=torch.float16, device="cuda"),
                 noise=torch.randn(H, M, P + M, device="cuda", generator=g).half())
        for c in ("C_out", "C_out1", "C_out2"):
            t[c] = torch.zeros(H, P + M, dtype=torch.float16, device="cuda")
        res = {"weights_and_cache_bytes": 3 * N * N * 2 + 2 * H * (P + M) * D * 2}
        for v in ("vanilla", "prenorm", "qknorm", "keyformer", "roco"):
            m = modules.get(v, "decode", head_dim=D)
            _, ev = graph_timed(m, t, steps, warmup, per_graph=20)
            res[v + "_us"] = round(ev * 1e3, 2)
            _, ev = graph_timed(m, t, steps, warmup, per_graph=1)
            res[v + "_replay_us"] = round(ev * 1e3, 2)
        out[name] = res
    # the reference's other two workloads at the first shape its drivers list (lora_benchmark.py:545, gmlp_benchmark.py:53-64)
    g = torch.Generator(device="cuda").manual_seed(42)
    rnd = lambda *shape: torch.randn(*shape, device="cuda", generator=g).clamp_(-1, 1).mul_(0.01).half()
    M, N, P, R = 16, 1024, 512, 64
    t = dict(X=rnd(M, N), W=rnd(N, P), A=rnd(N, R), B=rnd(R, P), O=torch.zeros(M, P, dtype=torch.float16, device="cuda"))
    for pg, key in ((20, "lora_M16_N1024_P512_R64_us"), (1, "lora_M16_N1024_P512_R64_replay_us")):
        _, ev = graph_timed(modules.get("lora", "linear"), t, steps, warmup, per_graph=pg)
        out[key] = round(ev * 1e3, 2)
    K = 1024
    t = dict(X=torch.randn(M, K, device="cuda", generator=g).half(), W1=torch.randn(K, N, device="cuda", generator=g).half(),
             W2=torch.randn(K, N, device="cuda", generator=g).half(), O=torch.zeros(M, N, dtype=torch.float16, device="cuda"))
    for pg, key in ((20, "gmlp_M16_K1024_N1024_us"), (1, "gmlp_M16_K1024_N1024_replay_us")):
        _, ev = graph_timed(modules.get("gmlp", "linear"), t, steps, warmup, per_graph=pg)
        out[key] = round(ev * 1e3, 2)
    return out


def mfma_ceiling():
    """TFLOP/s of the MFMA-only yardstick kernel with all-zero and with random fp16 operands."""
    import torch
    from triton_amd import ops
    out = {}
    sink = torch.empty(512 * 256, dtype=torch.float32, device="cuda")
    for name, ops_t in (("zero_operands", torch.zeros(32768, dtype=torch.float16, device="cuda")),
                        ("random_operands", torch.randn(32768, device="cuda").half())):
        for _ in range(2):
            ops.calibration_mfma(ops_t, sink, 4000, 512)
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        start.record()
        flops = 0.0
        for _ in range(5):
            flops += ops.calibration_mfma(ops_t, sink, 4000, 512)
        end.record()
        torch.cuda.synchronize()
        out[name] = flops / start.elapsed_time(end) / 1e9
    return out


def cpu_baseline(q, k, v, budget_s):
    """The CPU oracle (oracle/ref.py, eager PyTorch fp32 on the host cores) on a bounded sample of the
    headline workload: whole query heads at the full S=4096, head by head, until the time budget is
    spent.  Rate = causal-halved flops of the heads done / seconds."""
    import torch
    from oracle import ref
    from triton_amd import configs
    cores = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    cores = max(1, min(cores, int(os.environ.get("OMP_NUM_THREADS", cores))))
    torch.set_num_threads(cores)
    B, Hq, S, D = q.shape
    G = Hq // k.shape[1]
    scale = D ** -0.5
    ref.attention(q[:, :1, :512], k[:, :1, :512], v[:, :1, :512], scale, True)       # warm-up
    done, t0 = 0, time.perf_counter()
    while done == 0 or time.perf_counter() - t0 < budget_s:      # whole heads, cycling over the workload's heads
        h = done % Hq
        ref.attention(q[:, h:h + 1], k[:, h // G:h // G + 1], v[:, h // G:h // G + 1], scale, True)
        done += 1
    dt = time.perf_counter() - t0
    flops = configs.attn_flops(B, done, S, S, D, True)
    return dict(value=flops / dt / 1e12, unit="TFLOP/s", cores=cores, kind="port",
                sample=f"{done} query-head passes (heads of the same workload, S={S}, D={D}, full rows, fp32 eager "
                       f"PyTorch oracle) in {dt:.1f} s")


def main():
    a = parse()
    if a.gpus != 1:
        print(f"bench.py measures one GPU only (got --gpus {a.gpus}): this build's hot path is single-GPU; "
              "heads shard across GPUs without collectives, and no multi-GPU figure is produced.", file=sys.stderr)
        raise SystemExit(2)
    import torch
    from triton_amd import _lib, configs
    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a GPU: there is no CPU fallback for the kernels")
    _lib.check("trn_check_device", _lib.load().trn_check_device())

    if a.calibrate:
        from triton_amd import ops
        src = torch.ones(256 << 20, dtype=torch.uint8, device="cuda"); dst = torch.empty_like(src)
        for _ in range(3):
            ops.calibration_copy(src, dst)
        torch.cuda.synchronize()
        del src, dst
    wl = a.workload
    extra = {}
    van = bench_vanilla(a.steps, a.warmup, a.inputs, not a.no_zero_leg) if wl in ("headline", "all", "vanilla") else None
    if wl in ("headline", "all", "rmsnorm"):
        extra["rmsnorm"] = bench_rmsnorm(a.steps, a.warmup)
    def guarded(fn, *args):
        """The other workloads ride along with the headline in the default run: a failure in one of them is
        reported in its place and does not cost the line (asked for alone, it is raised)."""
        if wl != "all":
            return fn(*args)
        try:
            return fn(*args)
        except Exception as e:
            return {"error": f"{type(e).__name__}: {e}"}
    for name in ("prenorm", "qknorm", "keyformer", "roco"):
        if wl in ("all", name):
            extra[name] = guarded(bench_variant, name, max(a.steps // 4, 10), a.warmup)
            torch.cuda.empty_cache()
    if wl == "decode" or (wl == "all" and not a.no_decode):
        extra["decode_append_M16_P1024"] = guarded(bench_decode, 100, a.warmup)
    if wl == "sweep":
        extra["attention_sweep"] = bench_sweep(a.steps, a.warmup)
    if van is None:                       # a single non-headline workload was asked for
        print(json.dumps({"workload": wl, **extra}))
        return

    peak = configs.MFMA_F16_PEAK_TFLOPS
    # HBM bytes per launch of the dominant kernel, measured offline with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
    # (recipe and scaling in profiles/); null until that file exists.
    traffic = None
    traffic_of = None       # SHA-256 of the kernel source the counters were taken on
    tpath = os.path.join(ROOT, "profiles", "attn_fwd_llama3_s4096_hbm_traffic.txt")
    if os.path.exists(tpath):
        with open(tpath) as f:
            for ln in f:
                if ln.startswith("hbm_bytes_per_launch:"):
                    traffic = int(ln.split(":")[1])
                if ln.startswith("kernel_source_sha256:"):
                    traffic_of = ln.split(":")[1].strip()
    import hashlib
    with open(os.path.join(ROOT, "triton_amd", "csrc", "attn_fwd16.hip"), "rb") as f:
        src_now = hashlib.sha256(f.read()).hexdigest()
    # (the figure is a counter reading taken offline: say so when the kernel's source has changed since)
    traffic_current = traffic is not None and traffic_of == src_now
    line = {
        "metric": "attn TFLOP/s + % fp16 MFMA peak (Llama3-8B, S=4096); RMSNorm HBM GB/s",
        "value": round(van["tflops"], 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(van["wall_ms"], 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic" if a.inputs == "randn" else "all-zero inputs: a diagnostic run, not the benchmark",
        "config": {"workload": "vanilla causal GQA attention, batch 1, seq 4096, 32 q heads / 8 kv heads, head_dim 128",
                   "flops_per_step": van["flops"], "flop_convention": "4*B*H*S^2*D/2 (causal-halved)",
                   "timing": f"graph replay on a side stream, 20 forwards per graph; {CLOCK_WARMUP_S} s of untimed replays, "
                             f"then {REPEATS} regions of exactly --steps forwards each, the median region reported"},
        "pct_of_fp16_mfma_peak": round(100 * van["tflops"] / peak, 2),
        "roofline": {"bound": "mfma", "achieved": round(van["kernel_tflops"], 2), "peak": peak, "unit": "TFLOP/s",
                     "frac": round(van["kernel_tflops"] / peak, 4), "traffic": traffic,
                     "kernel": van["kernel"], "kernel_ms": round(van["kernel_ms"], 5),
                     "kernel_ms_per_region": [round(x, 5) for x in van["region_ms"]],
                     "traffic_source": "profiles/attn_fwd_llama3_s4096_hbm_traffic.txt (rocprofv3 --pmc FETCH_SIZE / "
                                       "WRITE_SIZE of this command, scaled by the library's copy kernel)",
                     "traffic_taken_on_this_kernel_source": traffic_current},
    }
    ceil = mfma_ceiling()
    line["roofline"]["mfma_only_kernel_tflops"] = {k: round(v, 1) for k, v in ceil.items()}
    line["roofline"]["frac_of_mfma_only_random_operands"] = round(van["kernel_tflops"] / ceil["random_operands"], 4)
    if van["zero_inputs_kernel_ms"] is not None:
        line["roofline"]["same_kernel_on_all_zero_inputs"] = {
            "kernel_ms": round(van["zero_inputs_kernel_ms"], 5),
            "frac": round(van["flops"] / van["zero_inputs_kernel_ms"] / 1e9 / peak, 4),
            "note": "diagnostic: same instructions and traffic without switching activity (the board holds its clock)"}
    if "rmsnorm" in extra:
        r = extra["rmsnorm"]
        line["rmsnorm"] = {"value": round(r["gbps"], 1), "unit": "GB/s", "frac_of_hbm_peak": round(r["frac"], 4),
                           "kernel_us": round(r["kernel_us"], 3), "bytes": r["bytes"],
                           "rotating_buffers": r["rotating_buffers"], "cache_hot_gbps": round(r["hot_cache_gbps"], 1),
                           "plain_copy_same_footprint_gbps": round(r["copy_gbps"], 1),
                           "plain_copy_same_footprint_us": round(r["copy_us"], 3),
                           "torch_copy_same_footprint_gbps": round(r["torch_copy_gbps"], 1),
                           "torch_copy_same_footprint_us": round(r["torch_copy_us"], 3),
                           "workload": "RMSNorm fp16 [4096 x 4096], gamma, eps 1e-5"}
    for name in ("prenorm", "qknorm", "keyformer", "roco"):
        if name in extra:
            line[name] = {k: (round(v, 4) if isinstance(v, float) else v) for k, v in extra[name].items()}
    if "decode_append_M16_P1024" in extra:
        line["decode_append_M16_P1024"] = extra["decode_append_M16_P1024"]
    if not a.no_cpu:
        line["cpu_baseline"] = cpu_baseline(*van["tensors"], a.cpu_seconds)
        line["cpu_baseline"]["value"] = round(line["cpu_baseline"]["value"], 4)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
