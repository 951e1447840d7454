"""Benchmark of the decode hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload decode|decode_p12] [--no-cpu]
    python bench.py --workload gemv_bf16|gemv_p12|gemv_fp8|gemv_mxfp4|moe [--m M]      (the other configs, one kernel each)

A step is one decode step of a random-init Qwen3-4B-shaped dense stack (36 layers, hidden 2560, 32 query / 8 kv heads
of 128, SwiGLU 9728, vocab 151936; weights ~N(0, 0.02) in bf16, seeded N(0, 1) K/V for a 4096-token context), M = 1
token, replayed as one captured hipGraph with every operand already resident in HBM. It prints ONE JSON line:
`value` is the step's HBM stream in GB/s - the linear weights plus the K/V rows one step reads, divided by the step's
time - next to tokens/s and the fraction of the 8 TB/s HBM3E peak; `roofline` prices the dominant kernel (the bf16
streaming matvec at the qkv / gate_up / head shapes) from its own timed region, measured with device events on the
launch stream; `cpu_baseline` times the CPU oracle's AVX-512 / AVX2 matvec (a port of the reference's CPU path) on the
host's cores over a bounded sample of the same matrices.
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

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published
CTX = 4096
METRIC = "decode GEMV HBM GB/s (% of peak) + decode tok/s, Qwen3-4B-shape bf16 M=1"


def cpu_baseline(budget_s: float = 12.0) -> dict:
    """the oracle's bf16 matvec (the reference's CPU arithmetic, ported) over gate_up-shaped matrices drawn from a
    pool larger than 4x the last-level cache, every core, for about `budget_s` seconds"""
    import numpy as np

    import oracle

    R, C = 19456, 2560
    rng = np.random.default_rng(0x0B7B)
    pool = [rng.integers(0x3A00, 0x3D00, (R, C), dtype=np.uint16) for _ in range(12)]  # 1.2 GB of bf16 patterns
    x = rng.standard_normal((1, C)).astype(np.float32)
    cores = os.cpu_count() or 1
    oracle.gemv_bf16(pool[0], x, threads=0)
    t0 = time.perf_counter()
    calls = 0
    while time.perf_counter() - t0 < budget_s:
        oracle.gemv_bf16(pool[calls % len(pool)], x, threads=0)
        calls += 1
    dt = time.perf_counter() - t0
    per_call = R * C * 2 + C * 4 + R * 4
    gbs = calls * per_call / dt / 1e9
    # the same matvec on one thread (the reference's own criterion bench pins one: native/benches/gemv.rs:8-10)
    t1 = time.perf_counter()
    solo = 0
    while time.perf_counter() - t1 < budget_s / 4:
        oracle.gemv_bf16(pool[solo % len(pool)], x, threads=1)
        solo += 1
    d1 = time.perf_counter() - t1
    return {"value": round(gbs, 2), "unit": "GB/s", "cores": cores, "kind": "port", "isa": oracle.isa(),
            "one_thread_gbs": round(solo * per_call / d1 / 1e9, 2),
            "sample": f"{calls} bf16 matvecs [{R}x{C}] (the gate_up shape), 12 distinct matrices (1.2 GB) in rotation, "
                      f"f32 x and y, all {cores} host threads, {dt:.1f} s; then {solo} on one thread, {d1:.1f} s"}


def kernel_workload(args: argparse.Namespace) -> int:
    """The single-operator configs: one JSON line each, `value` the operator's HBM stream in GB/s. A step is one call
    over the next operand set of a pool larger than the last-level cache (256 MB), so nothing repeats from cache; the
    calls of one pass are replayed as a hipGraph and timed with device events.

      gemv_bf16   configs[0] (C1): W bf16 [9728, 2560], M rows of x
      gemv_p12    the same matrix packed to 12 bits a weight
      gemv_fp8    C5a: fp8.quantize(N(0, 0.02) [18432, 7168], (128, 128))
      gemv_mxfp4  C5b: the same source through the MXFP4 encoder
      moe         C4: router [128, 2048] + top-8 of 128 experts (gate_up [1536, 2048], down [2048, 768]), M tokens
    """
    import torch

    from btb_amd import fp8, mxfp4
    from btb_amd.moe import Experts, Router
    from btb_amd.native import Native
    from btb_amd.pack12 import P12Weight

    card = Native.card_kernels()
    dev, M = torch.device("cuda"), int(args.m)
    g = torch.Generator(device=dev).manual_seed(0x0B7B0500)
    bf = dict(dtype=torch.bfloat16, device=dev)

    def normal(*shape: int) -> torch.Tensor:
        return torch.randn(*shape, generator=g, device=dev, dtype=torch.float32) * 0.02

    name = args.workload
    if name == "moe":
        # two layers' stacks (3.6 GB) and sixteen sets of rows: every call routes to other experts, so a pass streams
        # 1.2 GB (one token) and more of distinct expert matrices - nothing comes back out of the 256 MB cache
        E, k, H, I, pool = 128, 8, 2048, 768, 16
        sets = [(Router(card, normal(E, H).to(torch.bfloat16), k), Experts(card, normal(E, 2 * I, H).to(torch.bfloat16),
                                                                           normal(E, H, I).to(torch.bfloat16)))
                for _ in range(2)]
        xs = [torch.randn(M, H, generator=g, device=dev).to(torch.bfloat16) for _ in range(pool)]
        distinct = []

        def call(i: int) -> None:
            router, experts = sets[i % 2]
            _, w, idx = router(xs[i])
            experts(xs[i], idx, w)

        for i in range(pool):  # the bytes a call streams: the router and every DISTINCT expert its picks name
            _, _, idx = sets[i % 2][0](xs[i])
            distinct.append(int(torch.unique(idx).numel()))
        per_expert = (2 * I * H + H * I) * 2
        nbytes = [E * H * 2 + d * per_expert for d in distinct]
        what = f"C4: top-{k} of {E} experts, gate_up [{2 * I}, {H}] + down [{H}, {I}] bf16, M={M} tokens"
        extra = {"distinct_experts": distinct}
        dtype = "bf16 weights and activations, f32 accumulate"
    else:
        R, C = (9728, 2560) if name in ("gemv_bf16", "gemv_p12") else (18432, 7168)
        # operands of a pass: over 1 GiB of stored weights, past four times the 256 MB last-level cache (the reference's
        # own rule for its timing pools: btb/machine.py:384-426)
        per = {"gemv_bf16": 2.0, "gemv_p12": 1.5, "gemv_fp8": 1.0, "gemv_mxfp4": 17 / 32}[name] * R * C
        pool = max(4, -(-1_100_000_000 // int(per)))
        mats = []
        for _ in range(pool):
            t = normal(R, C)
            if name == "gemv_bf16":
                mats.append(t.to(torch.bfloat16))
            elif name == "gemv_p12":
                mats.append(P12Weight.pack(t.to(torch.bfloat16), card))
            elif name == "gemv_fp8":
                q, sc = fp8.quantize(t, (128, 128))
                mats.append(fp8.F8Weight(q, sc, R, C))
            else:
                b, sc = mxfp4.quantize(t)
                mats.append(mxfp4.MxWeight(b.reshape(-1), sc.reshape(-1), R, C))
            del t
        x = torch.randn(M, C, generator=g, device=dev).to(torch.bfloat16)
        y = torch.empty(M, R, **bf)
        op = {"gemv_bf16": card.gemv, "gemv_p12": card.gemv_p12, "gemv_fp8": card.gemv_fp8, "gemv_mxfp4": card.gemv_mx4}[name]

        def call(i: int) -> None:
            op(mats[i], x, y)

        stored = [m.numel() * 2 if isinstance(m, torch.Tensor) else m.nbytes for m in mats]
        nbytes = [b + 2 * M * C + 2 * M * R for b in stored]
        what = f"{name} [{R}, {C}], M={M}"
        extra = {"weight_bytes": stored[0]}
        dtype = {"gemv_bf16": "bf16", "gemv_p12": "pack12 widened to bf16 in registers",
                 "gemv_fp8": "fp8 e4m3 x f32 block scale -> bf16 in registers",
                 "gemv_mxfp4": "mxfp4 -> bf16 in registers"}[name] + ", f32 accumulate"
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        for i in range(pool):
            call(i)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for i in range(pool):
            call(i)
    passes = max(1, (args.steps + pool - 1) // pool)
    for _ in range(max(1, args.warmup // pool)):
        graph.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(passes):
        graph.replay()
    e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) * 1e3 / (passes * pool)
    mean_bytes = sum(nbytes) / len(nbytes)
    gbs = mean_bytes / (us * 1e-6) / 1e9
    print(json.dumps({
        "metric": "decode matvec HBM GB/s (% of peak), one operator", "value": round(gbs, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": passes * pool, "warmup": args.warmup, "ms_per_step": round(us * 1e-3, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": dtype,
        "data": "synthetic: N(0, 0.02) weights, N(0, 1) x, seeded", "hbm_frac": round(gbs / HBM_PEAK_GBS, 4),
        "config": {"workload": what, "pool": pool, "algorithmic_bytes_per_step": int(mean_bytes), **extra},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None},
        "cpu_baseline": None,
    }))
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="decode",
                    choices=["decode", "decode_p12", "gemv_bf16", "gemv_p12", "gemv_fp8", "gemv_mxfp4", "moe"])
    ap.add_argument("--m", type=int, default=1, help="rows of x (tokens) for the single-operator workloads")
    ap.add_argument("--rows", type=int, default=1,
                    help="rows of a decode pass: 1 is the step the metric is quoted on, more a speculative verify pass")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU (no collectives, no sharding); use --gpus 1", file=sys.stderr)
        return 2
    if args.workload not in ("decode", "decode_p12"):
        return kernel_workload(args)
    if args.steps < 1 or args.warmup < 0 or args.steps + args.warmup > 480:
        print("bench.py: steps + warmup must stay within the cache's 480 spare rows", file=sys.stderr)
        return 2
    if not 1 <= args.rows <= 24:
        print("bench.py: a pass takes 1 to 24 rows here (the cache keeps 512 rows spare)", file=sys.stderr)
        return 2

    import torch

    from btb_amd.decode import QWEN3_4B, DecodeStep, random_stack
    from btb_amd.native import Native

    card = Native.card_kernels()  # raises where the HIP library or the GPU is missing: there is no fallback
    cfg = QWEN3_4B
    packed = args.workload == "decode_p12"
    weights = random_stack(card, cfg, packed=packed)
    cap = CTX + 512
    step = DecodeStep(card, cfg, weights, cap, T=args.rows)
    g = torch.Generator(device="cuda").manual_seed(0x0B7B0200)
    for i in range(cfg.layers):  # seeded K/V ~ N(0, 1) for the context
        step.kv[i, :, :, :CTX].copy_(torch.randn(2, cfg.kv_heads, CTX, cfg.head_dim, generator=g, device="cuda"))
    step.reset(CTX, 0)
    step.capture(warmup=2)
    step.reset(CTX, 0)

    stream = torch.cuda.current_stream()
    for _ in range(args.warmup):
        step.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record(stream)
    for _ in range(args.steps):
        step.replay()
    e1.record(stream)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms = e0.elapsed_time(e1) / args.steps
    n_keys = CTX + args.warmup + (args.steps + 1) / 2.0  # the average context over the timed steps
    wbytes, kvbytes = step.weight_bytes(), step.kv_bytes(int(n_keys))
    gbs = (wbytes + kvbytes) / (ms * 1e-3) / 1e9

    # -- the dominant kernel in a timed region of its own: the streaming matvec at the qkv, gate_up and head shapes
    #    (5.5 of the step's 8.0 GB of bf16 weights), over the model's own matrices, so nothing repeats from cache
    M = args.rows
    x = torch.randn(M, cfg.hidden, device="cuda").to(torch.bfloat16)
    outs = {n: torch.empty(M, r, dtype=torch.bfloat16, device="cuda")
            for n, r in (("qkv", cfg.qkv_rows), ("gu", 2 * cfg.intermediate), ("head", cfg.vocab))}

    def dominant() -> tuple[int, int]:
        launches = nbytes = 0
        for i in range(cfg.layers):
            for n in ("qkv", "gu"):
                lin = weights[f"layers.{i}.{n}"]
                lin.matvec(x, outs[n])
                launches += 1
                nbytes += lin.nbytes + M * (cfg.hidden * 2 + lin.shape[0] * 2)
        weights["head"].matvec(x, outs["head"])
        return launches + 1, nbytes + weights["head"].nbytes + M * (cfg.hidden * 2 + cfg.vocab * 2)

    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        launches, dom_bytes = dominant()
    torch.cuda.synchronize()
    gd = torch.cuda.CUDAGraph()
    with torch.cuda.graph(gd):
        dominant()
    gd.replay()
    torch.cuda.synchronize()
    reps = 10
    d0, d1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    d0.record(stream)
    for _ in range(reps):
        gd.replay()
    d1.record(stream)
    torch.cuda.synchronize()
    dom_us = d0.elapsed_time(d1) * 1e3 / (reps * launches)
    achieved = dom_bytes / launches / (dom_us * 1e-6) / 1e9
    traffic = None
    tpath = os.path.join(ROOT, "profiles", "traffic.json")
    if os.path.exists(tpath) and args.rows == 1:  # the counters were read for the one-row region
        with open(tpath) as f:
            entry = json.load(f).get(args.workload)
            traffic = None if entry is None else entry.get("bytes_per_launch")

    line = {
        "metric": METRIC,
        "value": round(gbs, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16 weights and activations, f32 accumulate" if not packed else
                 "pack12 weights widened to bf16 in registers, f32 accumulate",
        "data": "synthetic: random-init N(0, 0.02) weights, seeded N(0, 1) K/V",
        "tokens_per_s": round(1e3 / ms, 1),
        "hbm_frac": round(gbs / HBM_PEAK_GBS, 4),
        "config": {
            "workload": ("configs[1]: full decode step of a Qwen3-4B-shaped dense stack, M=1, ctx 4096, one hipGraph"
                         if not packed else
                         "configs[2]: the same stack with every linear in pack12, widened in registers")
                        + ("" if args.rows == 1 else f"; a verify pass of {args.rows} rows"),
            "rows": args.rows, "rows_per_s": round(args.rows * 1e3 / ms, 1),
            "layers": cfg.layers, "hidden": cfg.hidden, "q_heads": cfg.q_heads, "kv_heads": cfg.kv_heads,
            "head_dim": cfg.head_dim, "intermediate": cfg.intermediate, "vocab": cfg.vocab, "context": CTX,
            "weight_bytes_per_step": wbytes, "kv_bytes_per_step": kvbytes, "kernels_per_step": (4 + 6 * cfg.layers if args.rows == 1 else
                                 4 + 7 * cfg.layers if step.fused else 5 + 10 * cfg.layers),
            "host_wall_ms_per_step": round(wall * 1e3 / args.steps, 4),
        },
        "roofline": {
            "kernel": ("gemv_stream (streaming matvec, M=1)" if M == 1 else
                       f"the matvec at M={M} (gemv_stream to 4 rows, gemv_mfma_lds from 8)")
                      + " at the qkv / gate_up / head shapes",
            "bound": "hbm",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            "traffic": traffic,
            "launches": launches,
            "avg_launch_us": round(dom_us, 3),
            "bytes_per_launch": int(dom_bytes / launches),
        },
        "cpu_baseline": None if args.no_cpu else cpu_baseline(),
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
