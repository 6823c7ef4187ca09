"""Counterpart of the reference's benchmark drivers for the hand-written modules.

The reference's `<variant>_<model>_benchmark.py` scripts read IR candidates, generate a module per candidate and time
its `forward` (vanilla_llama_benchmark.py:131-139 tensors, :243-294 timing, :515-547 result records).  With the code
generator bypassed there is one candidate per variant -- the hand-written module -- so this driver keeps everything
either side of it: the tensor configurations (a JSON list of {"M","N","D","H","P"} as in the reference's
`evaluation/<model>_configs.json`, or the built-in decode shapes), the tensor recipe (`randn.clamp(-1,1)*0.01`, outputs
zeroed), the timing sequence (cold call, 10 warm-ups on a side stream, capture, 100 graph replays, mean ms) and the
result records (`ir_id`, `ir_expression`, `execution_time_ms`, `tensor_config`, `error`), appended to `--output`
one configuration at a time like the reference's incremental save.

    python -m triton_amd.benchmark --variant vanilla --model llama --output vanilla_llama.json
    python -m triton_amd.benchmark --variant roco --configs my_shapes.json
    python -m triton_amd.benchmark --ir candidates.txt --start 0 --num 10      # recognise and time IR candidates

With `--ir` the candidates of an IR file (`id: expression` lines) are each mapped to the module that computes them
(triton_amd/ir.py) and timed under their own `ir_id`; one that is not an attention variant is recorded with its error.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
from typing import Dict, List, Optional

VARIANTS = ("vanilla", "prenorm", "qknorm", "keyformer", "roco")
LINEAR_VARIANTS = ("lora", "gmlp")       # the reference's lora_benchmark.py / gmlp_benchmark.py workloads
# the shapes those two drivers list (lora_benchmark.py:545-548; gmlp_benchmark.py has the same commented list with
# the LoRA keys, its class reads M, N, K: the first one is used with K = N)
LORA_CONFIGS = [{"M": 16, "N": 1024, "P": 512, "R": 64}, {"M": 32, "N": 1024, "P": 512, "R": 64},
                {"M": 16, "N": 2048, "P": 1024, "R": 128}, {"M": 8, "N": 512, "P": 256, "R": 32}]
GMLP_CONFIGS = [{"M": 16, "N": 1024, "K": 1024}, {"M": 32, "N": 1024, "K": 1024}, {"M": 16, "N": 2048, "K": 2048}]


def tensor_shapes(cfg: Dict[str, int]) -> Dict[str, tuple]:
    """Shapes of the tensors the reference drivers allocate for a configuration
    (vanilla_llama_benchmark.py:42-77, keyformer_llama_benchmark.py:74-79, roco_llama_benchmark.py:74-75;
    lora_benchmark.py:41-53 for {M,N,P,R}, gmlp_benchmark.py:53-64 for {M,N,K})."""
    if "R" in cfg:
        M, N, P, R = cfg["M"], cfg["N"], cfg["P"], cfg["R"]
        return {"X": (M, N), "W": (N, P), "A": (N, R), "B": (R, P), "O": (M, P)}
    if "K" in cfg:
        M, N, K = cfg["M"], cfg["N"], cfg["K"]
        return {"X": (M, K), "W1": (K, N), "W2": (K, N), "O": (M, N)}
    M, N, D, P = cfg["M"], cfg["N"], cfg["D"], cfg["P"]
    H = cfg.get("H", N // D)
    return {"X": (M, N), "WQ": (N, N), "WK": (N, N), "WV": (N, N), "K_cache": (H, P + M, D), "V_cache": (H, P + M, D),
            "O2": (M, N), "noise": (H, M, P + M), "C_out": (H, P + M), "C_out1": (H, P + M), "C_out2": (H, P + M)}


OUTPUTS = ("O2", "C_out", "C_out1", "C_out2", "O")


def make_tensors(cfg: Dict[str, int], names: List[str], device: str = "cuda"):
    """Inputs `randn.clamp(-1, 1) * 0.01`, outputs zero, all fp16 (vanilla_llama_benchmark.py:131-139)."""
    import torch
    shapes = tensor_shapes(cfg)
    out = {}
    for n in names:
        if n not in shapes:
            raise ValueError(f"Unknown tensor parameter: {n}")
        if n in OUTPUTS:
            out[n] = torch.zeros(shapes[n], dtype=torch.float16, device=device)
        elif "K" in cfg:       # the gated-MLP driver draws plain randn (gmlp_benchmark.py:96)
            out[n] = torch.randn(shapes[n], dtype=torch.float16, device=device)
        else:
            out[n] = torch.randn(shapes[n], dtype=torch.float16, device=device).clamp(-1, 1) * 0.01
    return out


def time_module(module, tensors, warmup_runs: int = 10, benchmark_runs: int = 100) -> float:
    """Mean milliseconds per `forward`, measured as the reference does (vanilla_llama_benchmark.py:243-294)."""
    import torch
    for n in OUTPUTS:
        if n in tensors:
            tensors[n].zero_()
    args = [tensors[p] for p in module.TENSOR_PARAMS]
    stream = torch.cuda.Stream()
    module.forward(*args)                       # first call (the reference's autotune call)
    torch.cuda.synchronize()
    with torch.cuda.stream(stream):
        for _ in range(warmup_runs):
            module.forward(*args)
    stream.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            module.forward(*args)
    stream.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    with torch.cuda.stream(stream):
        start.record()
        for _ in range(benchmark_runs):
            graph.replay()
        end.record()
    stream.synchronize()
    if "O2" in tensors and torch.isnan(tensors["O2"]).any().item():
        print(f"WARNING: NaN values detected in O2 tensor!")
    return start.elapsed_time(end) / benchmark_runs


def append_record(path: str, record: dict) -> None:
    """The reference's incremental save: read the list, append, write back (vanilla_llama_benchmark.py:515-547)."""
    try:
        with open(path) as f:
            data = json.load(f)
    except (OSError, ValueError):
        data = []
    data.append(record)
    os.makedirs(os.path.dirname(os.path.abspath(path)), exist_ok=True)
    with open(path, "w") as f:
        json.dump(data, f, indent=2)


def candidates_from_ir(path: str, start: int = 0, num: Optional[int] = 10) -> List[tuple]:
    """(ir_id, expression, variant or None, reason[, constructor arguments read off the IR]) for the candidates of an IR file with id >= start, at most `num`
    of them (the reference's --start / --num / --end, vanilla_llama_benchmark.py:749-753); each is recognised by its
    dataflow instead of being compiled."""
    from . import ir
    out = []
    for ir_id, expr in ir.read_ir_file(path):
        if ir_id < start or (num is not None and len(out) >= num):
            continue
        m = ir.recognise(expr)
        out.append((ir_id, expr, m.variant, m.reason, m.kwargs))
    return out


def run(variant: str, configs: List[Dict[str, int]], output: str, warmup_runs: int = 10, benchmark_runs: int = 100,
        candidates: Optional[List[tuple]] = None) -> List[dict]:
    import torch

    from . import modules
    if not torch.cuda.is_available():
        raise SystemExit("Error: no GPU available; the hand-written kernels have no CPU path")
    if candidates is None:              # no IR file: the one candidate is the hand-written module of `variant`
        form = "linear" if variant in LINEAR_VARIANTS else "decode-append"
        candidates = [(f"trinity_hip/{variant}", f"hand-written gfx950 module ({variant}, {form} form)", variant, "")]
    records = []
    for cfg in configs:
        for ir_id, expr, var, reason, *rest in candidates:
            consts = rest[0] if rest else {}
            rec = {"ir_id": ir_id, "ir_expression": expr, "execution_time_ms": float("inf"), "tensor_config": dict(cfg), "error": None}
            try:
                if var is None:         # the reference records a candidate it cannot compile and carries on (:206-210)
                    raise ValueError(f"unsupported IR: {reason}")
                module = modules.get(var, "linear", **consts) if var in LINEAR_VARIANTS else modules.get(var, "decode", head_dim=cfg["D"], **consts)
                tensors = make_tensors(cfg, module.TENSOR_PARAMS)
                rec["execution_time_ms"] = time_module(module, tensors, warmup_runs, benchmark_runs)
            except Exception as e:      # ... and one that fails at run time (:329-332)
                rec["error"] = str(e)
            records.append(rec)
            append_record(output, rec)
            print(f"  IR {rec['ir_id']}" + (f" [{var}]" if var else "") + f" {rec['tensor_config']}: "
                  + (f"{rec['execution_time_ms']:.4f} ms" if rec["error"] is None else f"error: {rec['error']}"))
        torch.cuda.empty_cache()
    return records


def print_report(records: List[dict], top_k: int) -> None:
    """Best candidates per tensor configuration (vanilla_llama_benchmark.py:574-602)."""
    seen = []
    for r in records:
        if r["tensor_config"] not in seen:
            seen.append(r["tensor_config"])
    for i, cfg in enumerate(seen):
        print(f"\nConfiguration {i + 1}:\n  Tensor Shape: M={cfg['M']}, N={cfg['N']}")
        valid = sorted((r for r in records if r["tensor_config"] == cfg and r["error"] is None),
                       key=lambda r: r["execution_time_ms"])[:top_k]
        if not valid:
            print("  No valid kernels found for this configuration")
        for j, r in enumerate(valid):
            print(f"    {j + 1}. IR {r['ir_id']}: {r['execution_time_ms']:.4f} ms")


def main(argv=None) -> int:
    from . import configs as shapes
    ap = argparse.ArgumentParser(description="Time the hand-written module of one variant the way the reference's drivers time a candidate")
    ap.add_argument("--variant", choices=VARIANTS + LINEAR_VARIANTS, default="vanilla")
    ap.add_argument("--model", choices=("llama", "falcon"), default="llama",
                    help="built-in decode shape (M=16, P=1024 at the model's widths) when --configs is not given")
    ap.add_argument("--configs", type=str, default=None, help="JSON file: a list of {M, N, D, H, P} tensor configurations")
    ap.add_argument("--output", type=str, default=None, help="result file (default ./<variant>_<model>.json)")
    ap.add_argument("--ir", type=str, default=None,
                    help="Path to the IR expressions file (`id: expression` lines): each candidate is recognised and timed")
    ap.add_argument("--start", type=int, default=0, help="Start from test case ID")
    ap.add_argument("--num", type=int, default=10, help="Number of expressions to benchmark")
    ap.add_argument("--end", action="store_true", help="Run from start ID to the last test case")
    ap.add_argument("--topk", type=int, default=5, help="Number of top kernels to report")
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--runs", type=int, default=100)
    a = ap.parse_args(argv)
    if a.configs:
        with open(a.configs) as f:
            cfgs = json.load(f)
        ok = lambda c: isinstance(c, dict) and ({"M", "N", "D", "P"} <= set(c) or {"M", "N", "P", "R"} <= set(c) or {"M", "N", "K"} <= set(c))
        if not isinstance(cfgs, list) or not all(ok(c) for c in cfgs):
            ap.error("--configs: expected a JSON list of objects with M, N, D, P (and optionally H), or M, N, P, R (LoRA), or M, N, K (gated MLP)")
    elif a.variant in LINEAR_VARIANTS:
        cfgs = [dict(c) for c in (LORA_CONFIGS if a.variant == "lora" else GMLP_CONFIGS)]
    else:
        cfgs = [dict(shapes.DECODE_LLAMA if a.model == "llama" else shapes.DECODE_FALCON)]
    cands = candidates_from_ir(a.ir, a.start, None if a.end else a.num) if a.ir else None
    out = a.output or f"./{a.variant}_{a.model}.json"
    with open(out, "w") as f:               # the reference starts a run from an empty list (:476)
        json.dump([], f)
    records = run(a.variant, cfgs, out, a.warmup, a.runs, cands)
    if cands is not None:
        print_report(records, a.topk)
    return 0


if __name__ == "__main__":
    sys.exit(main())
