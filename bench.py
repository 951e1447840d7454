"""Benchmark of the decode hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload decode|decode_p12] [--no-cpu]
    python bench.py --workload gemv_bf16|gemv_p12|gemv_fp8|gemv_mxfp4|moe|moe_mxfp4 [--m M]   (the other configs, one operator each)
    python bench.py --workload copy          (a plain 2^28-byte device copy: the scale of the FETCH_SIZE / WRITE_SIZE counters)
    python bench.py --workload ceiling       (the matvec's loads without the matvec: what the memory system gives such a kernel)

A step is one decode step of a random-init Qwen3-4B-shaped dense stack (36 layers, hidden 2560, 32 query / 8 kv heads
of 128, SwiGLU 9728, vocab 151936; weights ~N(0, 0.02) in bf16, seeded N(0, 1) K/V for a 4096-token context), M = 1
token, replayed as one captured hipGraph with every operand already resident in HBM. It prints ONE JSON line:
`value` is the step's HBM stream in GB/s - the linear weights plus the K/V rows one step reads, divided by the step's
time - next to tokens/s and the fraction of the 8 TB/s HBM3E peak.

`roofline` prices the kernels the step itself launches. Each class of launch - the qkv matvec with the residual add
and norm in its x load, the attention pair, the o matvec, the gate/up matvec with the add + norm and the SwiGLU fold,
the down matvec, the head matvec with the final norm - is timed in a graph region of its own over the model's own 36
matrices (so nothing repeats from cache), with device events on the launch stream; `roofline.kernels` lists them,
`roofline.kernel` / `achieved` / `frac` are those of the class that takes the most of the step's time, and
`roofline.all_matvecs` is the byte-weighted figure over every matvec class. `traffic` is not measured by this run: it
is the HBM bytes per launch of the dominant class from `rocprofv3 --pmc` runs of this same command, kept in
profiles/traffic.json (`traffic_source` names the summary).

`cpu_baseline` times the CPU oracle's AVX-512 / AVX2 matvec of the same stored form (a port of the reference's CPU
path, as `btb bench` times it per stored form: btb/machine.py:1000, 1018) on the host's cores over a bounded sample.
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
TRAFFIC = os.path.join(ROOT, "profiles", "traffic.json")


# ---------------------------------------------------------------------------------------------------------------
# the CPU leg: the oracle (a port of the reference's CPU kernels) on the host's cores, a bounded sample
# ---------------------------------------------------------------------------------------------------------------


def cpu_baseline(workload: str = "decode", m: int = 1, budget_s: float = 12.0) -> dict:
    """The oracle's matvec of the workload's stored form over matrices drawn in rotation from a pool (so the last-level
    cache does not hold them), every core, for about `budget_s` seconds, then a quarter of that on one thread.
    GB/s of the same algorithmic bytes the GPU figure counts."""
    import numpy as np

    import oracle
    from oracle import codecs

    rng = np.random.default_rng(0x0B7B)
    cores = os.cpu_count() or 1

    def bf16_bits(rows: int, cols: int) -> np.ndarray:
        return codecs.f32_to_bf16_bits((rng.standard_normal((rows, cols), dtype=np.float32) * np.float32(0.02)))

    if workload in ("decode", "gemv_bf16"):
        R, C = (19456, 2560) if workload == "decode" else (9728, 2560)
        pool = [rng.integers(0x3A00, 0x3D00, (R, C), dtype=np.uint16) for _ in range(12 if workload == "decode" else 24)]
        x = rng.standard_normal((m, C)).astype(np.float32)
        call = lambda i, t: oracle.gemv_bf16(pool[i % len(pool)], x, threads=t)
        per_call = R * C * 2 + m * (C + R) * 4
        what = f"bf16 matvecs [{R}x{C}]" + (" (the gate_up shape)" if workload == "decode" else "")
    elif workload in ("decode_p12", "gemv_p12"):
        R, C = (19456, 2560) if workload == "decode_p12" else (9728, 2560)
        lo, hi4, table, ei, ev = codecs.pack12_pack(bf16_bits(R, C))
        pool = [(lo.copy(), hi4.copy()) for _ in range(16 if workload == "decode_p12" else 32)]
        x = rng.standard_normal((m, C)).astype(np.float32)
        call = lambda i, t: oracle.gemv_p12(pool[i % len(pool)][0], pool[i % len(pool)][1], table, ei, ev, R, C, x, threads=t)
        per_call = lo.size + hi4.size + 16 + 5 * ei.size + m * (C + R) * 4
        what = f"pack12 matvecs [{R}x{C}] ({ei.size} escapes)"
    elif workload == "gemv_fp8":
        # random e4m3 bytes (no NaN patterns) and scales of the size quantising N(0, 0.02) gives: the kernel's speed
        # does not depend on the values, and encoding 132 M weights in numpy would take longer than the sample
        R, C = 18432, 7168
        q = rng.integers(0, 0x7F, (R, C), dtype=np.uint8) | (rng.integers(0, 2, (R, C), dtype=np.uint8) << 7)
        s = (rng.random((R // 128, C // 128), dtype=np.float32) + np.float32(0.5)) * np.float32(2e-4)
        pool = [q.copy() for _ in range(9)]
        x = rng.standard_normal((m, C)).astype(np.float32)
        call = lambda i, t: oracle.gemv_fp8(pool[i % len(pool)], s, x, threads=t)
        per_call = R * C + s.size * 4 + m * (C + R) * 4
        what = f"FP8 e4m3 matvecs [{R}x{C}], 128x128 scale blocks (random bytes)"
    elif workload == "gemv_mxfp4":
        R, C = 18432, 7168
        b = rng.integers(0, 256, (R, C // 32, 16), dtype=np.uint8)
        s = rng.integers(115, 123, (R, C // 32), dtype=np.uint8)
        pool = [b.copy() for _ in range(16)]
        x = rng.standard_normal((m, C)).astype(np.float32)
        call = lambda i, t: oracle.gemv_mxfp4(pool[i % len(pool)], s, R, C, x, threads=t)
        per_call = b.size + s.size + m * (C + R) * 4
        what = f"MXFP4 matvecs [{R}x{C}] (random bytes)"
    elif workload == "moe":
        from oracle import moe as omoe

        E, k, H, I = 128, 8, 2048, 768
        bits = lambda *shape: (rng.integers(0x3A00, 0x3D00, shape, dtype=np.uint16)
                               | (rng.integers(0, 2, shape, dtype=np.uint16) << 15))   # +-2^-11 .. 2^-5
        wr, gu, dn = bits(E, H), bits(E, 2 * I, H), bits(E, H, I)
        xs = [codecs.round_bf16(rng.standard_normal((m, H)).astype(np.float32)) for _ in range(16)]
        distinct = []

        def call(i, t):  # the oracle's layer runs its matvecs on every core (threads = 0 inside oracle/moe.py)
            _, _, _, picks = omoe.layer(wr, gu, dn, xs[i % len(xs)], k, dt="bf16")
            distinct.append(len(set(picks.reshape(-1).tolist())))

        per_call = None
        what = f"MoE layers: top-{k} of {E} experts, gate_up [{2 * I}x{H}] + down [{H}x{I}] bf16, {m} tokens"
    elif workload == "moe_mxfp4":
        from oracle import moe as omoe

        E, k, H, I = 128, 8, 2048, 768
        wr = (rng.integers(0x3A00, 0x3D00, (E, H), dtype=np.uint16) | (rng.integers(0, 2, (E, H), dtype=np.uint16) << 15))
        gb = rng.integers(0, 256, (E, 2 * I, H // 32, 16), dtype=np.uint8)
        gs = rng.integers(115, 123, (E, 2 * I, H // 32), dtype=np.uint8)
        db = rng.integers(0, 256, (E, H, I // 32, 16), dtype=np.uint8)
        ds = rng.integers(115, 123, (E, H, I // 32), dtype=np.uint8)
        xs = [codecs.round_bf16(rng.standard_normal((m, H)).astype(np.float32)) for _ in range(16)]
        distinct = []

        def call(i, t):
            x = xs[i % len(xs)]
            _, w, picks = omoe.router(wr, x, k, "bf16")
            omoe.experts_mx4(gb, gs, db, ds, x, picks, w, dt="bf16", oss=False)
            distinct.append(len(set(picks.reshape(-1).tolist())))

        per_call = None
        what = (f"MoE layers: top-{k} of {E} experts, gate_up [{2 * I}x{H}] + down [{H}x{I}] MXFP4 as stored (random "
                f"bytes), {m} tokens")
    else:
        raise ValueError(workload)

    call(0, 0)
    if workload in ("moe", "moe_mxfp4"):
        distinct.clear()
    t0 = time.perf_counter()
    calls = 0
    while time.perf_counter() - t0 < budget_s:
        call(calls, 0)
        calls += 1
    dt = time.perf_counter() - t0
    if workload in ("moe", "moe_mxfp4"):
        per_w = 2.0 if workload == "moe" else 17 / 32
        nbytes = sum(128 * 2048 * 2 + d * (2 * 768 * 2048 + 2048 * 768) * per_w for d in distinct)
        return {"value": round(nbytes / dt / 1e9, 2), "unit": "GB/s", "cores": cores, "kind": "port", "isa": oracle.isa(),
                "sample": f"{calls} {what} through the oracle's numpy + C layer, matvecs on all {cores} host threads, "
                          f"{dt:.1f} s; bytes = the router and every distinct picked expert"}
    gbs = calls * per_call / dt / 1e9
    t1 = time.perf_counter()
    solo = 0
    while time.perf_counter() - t1 < budget_s / 4:
        call(solo, 1)
        solo += 1
    d1 = time.perf_counter() - t1
    return {"value": round(gbs, 2), "unit": "GB/s", "cores": cores, "kind": "port", "isa": oracle.isa(),
            "one_thread_gbs": round(solo * per_call / d1 / 1e9, 2),
            "sample": f"{calls} {what}, {len(pool)} operand copies in rotation, f32 x and y (M={m}), all {cores} host "
                      f"threads, {dt:.1f} s; then {solo} on one thread, {d1:.1f} s"}


def traffic_entry(workload: str, key: str) -> dict | None:
    """HBM bytes per launch from the committed rocprofv3 --pmc summaries (a profile constant, not measured here)"""
    if not os.path.exists(TRAFFIC):
        return None
    with open(TRAFFIC) as f:
        return (json.load(f).get(workload) or {}).get(key)


# ---------------------------------------------------------------------------------------------------------------
# the single-operator configs
# ---------------------------------------------------------------------------------------------------------------


def apply_tuning(card, pairs: list[str]) -> dict[str, int]:
    """--tune KNOB=VALUE: the library's tuning knobs set before anything is timed; returned for the config record"""
    out: dict[str, int] = {}
    for item in pairs:
        key, _, value = item.partition("=")
        card.set_tuning(key.strip(), int(value))
        out[key.strip()] = int(value)
    return out


def copy_workload() -> int:
    """A device-to-device copy of 2^28 bytes, three times: under `rocprofv3 --pmc FETCH_SIZE` (or WRITE_SIZE) its
    dispatches read 2^28 bytes and write 2^28 bytes, which gives the unit the counter counts in on this GPU."""
    import torch

    n = 1 << 28
    a = torch.empty(n, dtype=torch.uint8, device="cuda")
    b = torch.randint(0, 255, (n,), dtype=torch.uint8, device="cuda")
    for _ in range(3):
        a.copy_(b)
    torch.cuda.synchronize()
    print(json.dumps({"workload": "copy", "bytes": n, "copies": 3}))
    return 0


def ceiling_workload(args: argparse.Namespace) -> dict:
    """What the memory system gives a kernel with the streaming matvec's load structure and nothing else to do
    (`btb_hip_stream_probe`): microseconds and TB/s at the sizes of the step's matrices, each over a pool of distinct
    copies past the 256 MB last-level cache, replayed as a hipGraph and timed like every other workload here."""
    import torch

    from btb_amd.decode import recording
    from btb_amd.native import Native

    card = Native.card_kernels()
    out = []
    for what, rows in (("o-sized [4096 x 2560]", 4096), ("qkv [6144 x 2560]", 6144), ("C1 / down-sized [9728 x 2560]", 9728),
                       ("gate/up [19456 x 2560]", 19456), ("head [151936 x 2560]", 151936)):
        nbytes = rows * 5120
        pool = max(3, -(-1_200_000_000 // nbytes))
        mats = [torch.empty(rows, 2560, dtype=torch.bfloat16, device="cuda").fill_(0.01 * (i + 1)) for i in range(pool)]
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):
            for m in mats:
                card.stream_probe(m)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with recording(graph):
            for m in mats:
                card.stream_probe(m)
        for _ in range(3):
            graph.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        reps = max(2, 2000 // pool // max(1, rows // 4096))
        e0.record(torch.cuda.current_stream())
        for _ in range(reps):
            graph.replay()
        e1.record(torch.cuda.current_stream())
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / (reps * pool)
        out.append({"matrix": what, "bytes": nbytes, "us": round(us, 2), "achieved": round(nbytes / us / 1e3, 1), "unit": "GB/s",
                    "frac_of_8TBs": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)})
        del graph, mats
        torch.cuda.empty_cache()
    return {"metric": "streaming ceiling: the matvec's loads without the matvec, HBM GB/s", "unit": "GB/s",
            "value": out[-2]["achieved"], "n_gpus": 1, "higher_is_better": True, "data": "constant-filled matrices",
            "config": {"workload": "btb_hip_stream_probe over bf16 [R, 2560] matrices, pools past the last-level cache"},
            "sizes": out}


def kernel_workload(args: argparse.Namespace) -> dict:
    """The single-operator configs: one JSON line each, `value` the operator's HBM stream in GB/s. A step is one call
    over the next operand set of a pool larger than the last-level cache (256 MB), so nothing repeats from cache; the
    calls of one pass are replayed as a hipGraph and timed with device events.

      gemv_bf16   configs[0] (C1): W bf16 [9728, 2560], M rows of x
      gemv_p12    the same matrix packed to 12 bits a weight
      gemv_fp8    C5a: fp8.quantize(N(0, 0.02) [18432, 7168], (128, 128))
      gemv_mxfp4  C5b: the same source through the MXFP4 encoder
      moe         C4: router [128, 2048] + top-8 of 128 experts (gate_up [1536, 2048], down [2048, 768]), M tokens
      moe_mxfp4   the same layer with its expert stacks stored as MXFP4
    """
    import torch

    from btb_amd import fp8, mxfp4
    from btb_amd.decode import recording
    from btb_amd.moe import Experts, Router
    from btb_amd.native import Native
    from btb_amd.pack12 import P12Weight

    card = Native.card_kernels()
    tuned = apply_tuning(card, args.tune)
    dev, M = torch.device("cuda"), int(args.m)
    g = torch.Generator(device=dev).manual_seed(0x0B7B0500)
    bf = dict(dtype=torch.bfloat16, device=dev)

    def normal(*shape: int) -> torch.Tensor:
        return torch.randn(*shape, generator=g, device=dev, dtype=torch.float32) * 0.02

    name = args.workload
    if name == "moe_mxfp4":
        # C4's layer with its experts stored as MXFP4 (what gpt-oss-style checkpoints ship): two layers' stacks and
        # sixteen sets of rows, as below
        from btb_amd.load import MxExperts
        from btb_amd.moe import MxExpertsLayer

        E, k, H, I, pool = 128, 8, 2048, 768, 16

        def mx_layer():
            gb, gs = mxfp4.quantize(normal(E * 2 * I, H))
            db, ds = mxfp4.quantize(normal(E * H, I))
            return MxExpertsLayer(card, MxExperts(gb.reshape(E, 2 * I, H // 32, 16), gs.reshape(E, 2 * I, H // 32),
                                                  db.reshape(E, H, I // 32, 16), ds.reshape(E, H, I // 32)), oss=False)

        sets = [(Router(card, normal(E, H).to(torch.bfloat16), k), mx_layer()) for _ in range(2)]
        xs = [torch.randn(M, H, generator=g, device=dev).to(torch.bfloat16) for _ in range(pool)]
        distinct = []

        def call(i: int) -> None:
            router, experts = sets[i % 2]
            _, w, idx = router(xs[i])
            experts(xs[i], idx, w)

        for i in range(pool):
            _, _, idx = sets[i % 2][0](xs[i])
            distinct.append(int(torch.unique(idx).numel()))
        per_expert = (2 * I * H + H * I) * 17 // 32
        nbytes = [E * H * 2 + d * per_expert for d in distinct]
        what = f"C4 with MXFP4 experts: top-{k} of {E}, gate_up [{2 * I}, {H}] + down [{H}, {I}] as stored, M={M} tokens"
        extra = {"distinct_experts": distinct}
        dtype = "mxfp4 expert weights widened to bf16 in registers, bf16 activations, f32 accumulate"
        kernel = "the routed layer over MXFP4 stacks: router matvec + routing, gate/up with the SwiGLU fold, down with the weighted sum"
    elif name == "moe":
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
        kernel = "the routed layer: router matvec + routing, gate/up with the SwiGLU fold, down with the weighted sum"
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
        kernel = ("gemv_stream (vector ALUs, v_dot2_f32_bf16)" if M <= 4 else
                  "gemv_mfma_lds (matrix cores, v_mfma_f32_16x16x32_bf16, weights staged through registers into LDS; "
                  "taken from 5 rows on)" if name == "gemv_bf16" else
                  "gemv_mfma_dl (matrix cores, v_mfma_f32_16x16x32_bf16, weights from memory straight into a ring in "
                  "LDS; taken from 5 rows on)")
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        for i in range(pool):
            call(i)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with recording(graph):
        for i in range(pool):
            call(i)
    passes = max(1, (args.steps + pool - 1) // pool)
    for _ in range(max(1, args.warmup // pool)):
        graph.replay()
    torch.cuda.synchronize()
    stream = torch.cuda.current_stream()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    for _ in range(passes):
        graph.replay()
    e1.record(stream)
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) * 1e3 / (passes * pool)
    mean_bytes = sum(nbytes) / len(nbytes)
    gbs = mean_bytes / (us * 1e-6) / 1e9
    tr = traffic_entry(name, f"m{M}")
    del graph
    return {
        "metric": "decode matvec HBM GB/s (% of peak), one operator", "value": round(gbs, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": passes * pool, "warmup": args.warmup, "ms_per_step": round(us * 1e-3, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": dtype,
        "data": "synthetic: N(0, 0.02) weights, N(0, 1) x, seeded", "hbm_frac": round(gbs / HBM_PEAK_GBS, 4),
        "config": {"workload": what, "pool": pool, "algorithmic_bytes_per_step": int(mean_bytes), **extra,
                   **({"tuning": tuned} if tuned else {})},
        "roofline": {"kernel": kernel, "bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "avg_launch_us": round(us, 3),
                     "bytes_per_launch": int(mean_bytes),
                     "traffic": None if tr is None else tr.get("bytes_per_launch"),
                     "traffic_source": None if tr is None else tr.get("source")},
        "cpu_baseline": None if args.no_cpu else cpu_baseline(name, M),
    }


# ---------------------------------------------------------------------------------------------------------------
# the decode step
# ---------------------------------------------------------------------------------------------------------------


def step_classes(step, card) -> list[dict]:
    """The classes of launch one step makes, each as a closure that issues that class over the model's 36 layers (the
    head: once) on the step's own buffers, with its launches and algorithmic bytes per pass. The calls are the ones
    `DecodeStep._body_fused` makes."""
    cfg, w = step.cfg, step.w
    Hq, Hk, D, H, I = cfg.q_heads, cfg.kv_heads, cfg.head_dim, cfg.hidden, cfg.intermediate
    L = cfg.layers
    lay = [f"layers.{i}." for i in range(L)]
    n_keys = int(step.n0[0]) + 1
    norm_in = 3 * H * 2  # residual row, block output row and norm weight read by an add + norm x load

    def qkv():
        for p in lay:
            card.gemv_norm(w[p + "qkv"].w, step.h, step.y, w[p + "ln1"], cfg.eps, step.h2, step.qkv)

    def attn():
        for i, p in enumerate(lay):
            card.attn_decode_qkv(step.qkv, w.get(p + "wq"), w.get(p + "wk"), cfg.eps, step.cos, step.sin, step.n0,
                                 step.kv[i, 0], step.kv[i, 1], step.att, Hq, Hk, D, step.scale, step.S, step.scratch)

    def o():
        for p in lay:
            w[p + "o"].matvec(step.att, step.y)

    def gu():
        for p in lay:
            card.gemv_norm(w[p + "gu"].w, step.h2, step.y, w[p + "ln2"], cfg.eps, step.h, step.m, glu=True)

    def down():
        for p in lay:
            w[p + "down"].matvec(step.m, step.y)

    def head():
        card.gemv_norm(w["head"].w, step.h, step.y, w["norm"], cfg.eps, None, step.logits)

    wb = lambda name: sum(w[p + name].nbytes for p in lay)
    kv = 2 * Hk * n_keys * D * 2
    return [
        {"name": "qkv matvec + residual add + RMSNorm (gemv_stream, X_ADDNORM)", "fn": qkv, "launches": L, "matvec": True,
         "bytes": wb("qkv") + L * (norm_in + H * 2 + cfg.qkv_rows * 2)},
        {"name": "decode attention: q/k norm + rope + cache write + attention over the spans, then the span merge "
                 "(attn_decode_qkv_kernel + attn_merge_kernel, two launches)", "fn": attn, "launches": L, "matvec": False,
         "kernels_per_launch": 2, "bytes": L * (kv + cfg.qkv_rows * 2 + Hq * D * 2)},
        {"name": "o matvec (gemv_stream)", "fn": o, "launches": L, "matvec": True,
         "bytes": wb("o") + L * (Hq * D * 2 + H * 2)},
        {"name": "gate/up matvec + residual add + RMSNorm + SwiGLU fold (gemv_stream, X_ADDNORM, E_GLU)", "fn": gu,
         "launches": L, "matvec": True, "bytes": wb("gu") + L * (norm_in + H * 2 + I * 2)},
        {"name": "down matvec (gemv_stream)", "fn": down, "launches": L, "matvec": True,
         "bytes": wb("down") + L * (I * 2 + H * 2)},
        {"name": "head matvec + final RMSNorm (gemv_stream, X_ADDNORM)", "fn": head, "launches": 1, "matvec": True,
         "bytes": w["head"].nbytes + norm_in + cfg.vocab * 2},
    ]


def time_region(torch, fn, launches: int, reps: int) -> float:
    """average microseconds per launch of `fn`'s launches, replayed as a hipGraph `reps` times between two device
    events recorded on the stream the graph runs on"""
    from btb_amd.decode import recording

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with recording(g):
        fn()
    g.replay()
    torch.cuda.synchronize()
    stream = torch.cuda.current_stream()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    for _ in range(reps):
        g.replay()
    e1.record(stream)
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / (reps * launches)


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="decode",
                    choices=["decode", "decode_p12", "gemv_bf16", "gemv_p12", "gemv_fp8", "gemv_mxfp4", "moe", "moe_mxfp4", "copy",
                             "ceiling"])
    ap.add_argument("--m", type=int, default=1, help="rows of x (tokens) for the single-operator workloads")
    ap.add_argument("--rows", type=int, default=1,
                    help="rows of a decode pass: 1 is the step the metric is quoted on, more a speculative verify pass")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-configs", action="store_true",
                    help="the default run: skip the other benchmark configurations it appends as `configs`")
    ap.add_argument("--tune", action="append", default=[], metavar="KNOB=VALUE",
                    help="set one of the library's tuning knobs before the run (repeatable); recorded in config")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU (no collectives, no sharding); use --gpus 1", file=sys.stderr)
        return 2
    if args.workload == "copy":
        return copy_workload()
    if args.workload == "ceiling":
        print(json.dumps(ceiling_workload(args)))
        return 0
    if args.workload not in ("decode", "decode_p12"):
        print(json.dumps(kernel_workload(args)))
        return 0
    if args.steps < 1 or args.warmup < 0 or args.steps + args.warmup > 480:
        print("bench.py: steps + warmup must stay within the cache's 480 spare rows", file=sys.stderr)
        return 2
    if not 1 <= args.rows <= 24:
        print("bench.py: a pass takes 1 to 24 rows here (the cache keeps 512 rows spare)", file=sys.stderr)
        return 2
    line = decode_workload(args)
    # the default run (the line the driver records) carries every other configuration of the benchmark beside the
    # headline: each one its own workload of this file, timed the same way, without its CPU leg
    if args.workload == "decode" and args.rows == 1 and not args.tune and not args.no_configs:
        line["configs"] = other_configs(args)
    print(json.dumps(line))
    return 0


def other_configs(args: argparse.Namespace) -> list[dict]:
    """configs[0] and [2]..[4] of the benchmark, one compact record each: the workload, microseconds a step (one
    operator call, or the whole packed decode step), achieved GB/s over its algorithmic bytes and the fraction of the
    8 TB/s peak. A workload that fails is recorded with its error instead of ending the run."""
    import gc

    import torch

    plan = [("gemv_bf16", 1), ("decode_p12", 1), ("moe", 1), ("moe", 4), ("moe", 8), ("moe_mxfp4", 1), ("moe_mxfp4", 4),
            ("moe_mxfp4", 8), ("gemv_fp8", 1), ("gemv_fp8", 8), ("gemv_fp8", 16), ("gemv_mxfp4", 1), ("gemv_mxfp4", 8),
            ("gemv_mxfp4", 16), ("gemv_p12", 1)]
    name_of = {"gemv_bf16": "configs[0]", "decode_p12": "configs[2]", "moe": "configs[3]", "moe_mxfp4": "configs[3], MXFP4 experts",
               "gemv_fp8": "configs[4a]", "gemv_mxfp4": "configs[4b]", "gemv_p12": "configs[0] in pack12"}
    out = []
    for workload, m in plan:
        sub = argparse.Namespace(**{**vars(args), "workload": workload, "m": m, "no_cpu": True, "tune": [],
                                    "steps": 100 if workload == "decode_p12" else 96, "warmup": 10 if workload == "decode_p12" else 32})
        try:
            d = decode_workload(sub) if workload == "decode_p12" else kernel_workload(sub)
            rec = {"config": name_of[workload], "workload": d["config"]["workload"], "us_per_step": round(d["ms_per_step"] * 1e3, 2),
                   "achieved": d["value"], "unit": "GB/s", "frac": d["hbm_frac"]}
            if workload == "decode_p12":
                rec["tokens_per_s"] = d["tokens_per_s"]
        except Exception as e:  # noqa: BLE001 - the headline line must still be printed
            rec = {"config": name_of[workload], "workload": f"{workload} M={m}", "error": f"{type(e).__name__}: {e}"[:200]}
        out.append(rec)
        gc.collect()
        torch.cuda.empty_cache()
    return out


def decode_workload(args: argparse.Namespace) -> dict:
    """the decode step (configs[1]; `decode_p12`: configs[2]) as one replayed hipGraph: the line's dict"""
    import torch

    from btb_amd.decode import QWEN3_4B, DecodeStep, random_stack
    from btb_amd.native import Native

    card = Native.card_kernels()  # raises where the HIP library or the GPU is missing: there is no fallback
    tuned = apply_tuning(card, args.tune)
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

    # -- the step's own launches, class by class, each in a timed graph region over the model's 36 layers
    roofline: dict = {"bound": "hbm", "peak": HBM_PEAK_GBS, "unit": "GB/s"}
    if args.rows == 1 and step.fused:
        step.reset(CTX, 0)
        torch.cuda.synchronize()
        kernels = []
        for c in step_classes(step, card):
            us = time_region(torch, c["fn"], c["launches"], reps=10)
            per = c["bytes"] / c["launches"]
            kernels.append({"name": c["name"], "launches_per_step": c["launches"] * c.get("kernels_per_launch", 1),
                            "avg_launch_us": round(us, 3), "bytes_per_launch": int(per),
                            "achieved": round(per / (us * 1e-6) / 1e9, 1),
                            "frac": round(per / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
                            "us_per_step": round(us * c["launches"], 1), "matvec": c["matvec"]})
        total_us = sum(k["us_per_step"] for k in kernels)
        for k in kernels:
            k["step_share"] = round(k["us_per_step"] / total_us, 4)
        dom = max(kernels, key=lambda k: k["us_per_step"])
        mv = [k for k in kernels if k["matvec"]]
        mv_bytes = sum(k["bytes_per_launch"] * k["launches_per_step"] for k in mv)
        mv_us = sum(k["us_per_step"] for k in mv)
        tr = traffic_entry(args.workload, "dominant")
        roofline.update({
            "kernel": dom["name"], "achieved": dom["achieved"], "frac": dom["frac"],
            "avg_launch_us": dom["avg_launch_us"], "bytes_per_launch": dom["bytes_per_launch"],
            "launches": dom["launches_per_step"], "step_share": dom["step_share"],
            "traffic": None if tr is None else tr.get("bytes_per_launch"),
            "traffic_source": None if tr is None else tr.get("source"),
            "all_matvecs": {"bytes_per_step": int(mv_bytes), "us_per_step": round(mv_us, 1),
                            "achieved": round(mv_bytes / (mv_us * 1e-6) / 1e9, 1),
                            "frac": round(mv_bytes / (mv_us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)},
            "regions_us_per_step": round(total_us, 1),
            "kernels": [{k2: v for k2, v in k.items() if k2 != "matvec"} for k in kernels],
        })
    else:
        # a verify pass: the whole pass is the region (its matvecs run as gemv_stream up to 4 rows and on the matrix
        # cores, gemv_mfma_lds, from 5 rows on)
        roofline.update({"kernel": f"the whole pass of {args.rows} rows (matvecs: gemv_stream to 4 rows, gemv_mfma_lds "
                                   f"from 5)", "achieved": round(gbs, 1), "frac": round(gbs / HBM_PEAK_GBS, 4),
                         "traffic": None, "traffic_source": None})

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
            "weight_bytes_per_step": wbytes, "kv_bytes_per_step": kvbytes,
            "kernels_per_step": (2 + 6 * cfg.layers if args.rows == 1 else
                                 3 + (7 - step.rows_attn_fused) * cfg.layers if step.fused else
                                 5 + (10 - step.rows_attn_fused - (step.glu_fold and not packed)) * cfg.layers),
            "host_wall_ms_per_step": round(wall * 1e3 / args.steps, 4),
            **({"tuning": tuned} if tuned else {}),
        },
        "roofline": roofline,
        "cpu_baseline": None if args.no_cpu else cpu_baseline(args.workload, 1),
    }
    del step
    return line


if __name__ == "__main__":
    raise SystemExit(main())
