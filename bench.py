#!/usr/bin/env python3
"""Benchmark of the weight-quantized linear path on one MI355X.

`python bench.py --gpus 1` prints ONE JSON line.  Its headline (`metric`, `value`, `roofline`, `cpu_baseline`) is the
configuration the metric is quoted on: QINT8 W8A8 `fc_add` at the Llama-7B MLP shapes -- up-projection 4096 -> 11008
and down-projection 11008 -> 4096 -- for M in {1, 8, 32, 64}; one "step" is one pass over those 8 fused linears.
`config.legs` carries the other legs of the metric, each with its own roofline (kernel named by the library's launch
plan, timed with events on the launch stream) and, where the oracle finishes a sample in seconds, its own CPU
baseline:
  cfg1  MXFP4 fc_plain, M = 16, 4096 x 4096, bias                              (HBM TB/s)
  cfg3  MXFP4 SwiGLU MLP block 4096 -> 11008 -> 4096, M in {1, 4, 16, 64}      (HBM TB/s)
  cfg4  MXFP4 linears of one 70B-shape decoder layer at M = 2048               (TFLOP/s; also the same layer in
        QINT8 and with the opt-in MXFP8 activations, labelled)
  cfg5  32-layer 7B-shape decoder, greedy decode, batch 1 and 16               (tokens/s)
Inputs are resident in HBM before every timed region; weights cycle through pools larger than the 256 MB Infinity
Cache so that every decode-shape launch streams its weight from HBM.  Every leg is timed for at least half a second
of wall time.  `--workload` runs one leg alone (the form the profiles under profiles/ were taken in).
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "tpp-pytorch-extension_amd"))

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E published peak
PEAKS_TFLOPS = {"bf16": 2500.0, "fp8": 5000.0, "int8": 5000.0, "fp4": 10100.0}
MIN_WALL_S = 0.5       # every leg is timed for at least this long
# BASELINE config 2 (the configuration the headline metric is quoted on); tests/ import these so that the shapes the
# parity tests run are the shapes timed here
CFG2_SHAPES = {"up": (11008, 4096), "down": (4096, 11008)}  # name -> (N, K)
CFG2_MS = [1, 8, 32, 64]
CFG3_MS = [1, 4, 16, 64]
CFG3_DIMS = (4096, 11008)        # hidden, intermediate
CFG4_DIMS = (2048, 8192, 28672)  # M, hidden, intermediate; q/k/v widths 8192 + 1024 + 1024


def algorithmic_bytes(fmt, M, N, K, qbs=256, bias=False, post_in=True):
    """weights + scales + X + bias + post-op input + Y (bf16 activations)."""
    if fmt == "qint8":
        w = N * K + 4 * N * (K // qbs)
    else:
        w = N * K // 2 + N * K // 32
    return w + 2 * M * K + (2 * N if bias else 0) + (2 * M * N if post_in else 0) + 2 * M * N


def make_inputs(torch, shapes, Ms, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    W = {name: (torch.randn((N, K), generator=g) * 0.02).to(torch.bfloat16) for name, (N, K) in shapes.items()}
    X = {(name, M): torch.randn((M, K), generator=g).to(torch.bfloat16)
         for name, (N, K) in shapes.items() for M in Ms}
    R = {(name, M): torch.randn((M, N), generator=g).to(torch.bfloat16)
         for name, (N, K) in shapes.items() for M in Ms}
    return W, X, R


def block_bf16(W):
    N, K = W.shape
    return W.view(N // 16, 16, K // 64, 32, 2).permute(0, 2, 3, 1, 4).contiguous()


def clone_weight(q):
    """A second copy of a quantized weight's native tiles (so that launches stream distinct bytes)."""
    c = q._clone_with(q.qdata, q.scales)
    c._native = tuple(t.clone() for t in q.native())
    return c


def time_blocks(torch, run_step, steps, warmup, min_wall=MIN_WALL_S):
    """`warmup` untimed steps, then blocks of EXACTLY `steps` steps, each bracketed by a synchronize on both sides,
    until the blocks add up to `min_wall` seconds: (mean ms per step over all blocks, number of blocks)."""
    for i in range(warmup):
        run_step(i)
    torch.cuda.synchronize()
    total, blocks, i = 0.0, 0, warmup
    while True:
        t0 = time.perf_counter()
        for _ in range(steps):
            run_step(i)
            i += 1
        torch.cuda.synchronize()
        total += time.perf_counter() - t0
        blocks += 1
        if total >= min_wall or blocks >= 20000:
            break
    return total * 1e3 / (steps * blocks), blocks


def events_us(torch, fire, launches_per_fire, min_wall=0.15, use_graph=True):
    """Mean duration (us) of one launch group: `fire(stream)` enqueues `launches_per_fire` of them on the stream it is
    given; timed between two events on that stream around graph replays (or eager calls) for >= min_wall seconds."""
    g = None
    if use_graph:
        try:
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                fire(torch.cuda.current_stream().cuda_stream)
        except Exception:
            g = None
    go = (lambda: g.replay()) if g is not None else (lambda: fire(torch.cuda.current_stream().cuda_stream))
    for _ in range(2):
        go()
    torch.cuda.synchronize()
    total_ms, n = 0.0, 0
    reps = 4
    while total_ms < min_wall * 1e3 and n < 100000:
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            go()
        e1.record()
        torch.cuda.synchronize()
        total_ms += e0.elapsed_time(e1)
        n += reps
        reps = min(reps * 2, 256)
    return total_ms * 1e3 / (n * launches_per_fire), n * launches_per_fire


def plan_lines(text):
    out = []
    for line in text.strip().splitlines():
        name, _, shape = line.partition(" grid=")
        out.append((name.replace("void ", ""), "grid=" + shape))
    return out


def kernel_plan(L, fmt, M, N, K, qbs, flags, ws_bytes):
    """Kernels one linear call enqueues, as the library itself reports them:
    [(profiler name, launch shape text), ...]; the last one is the GEMM."""
    buf = ctypes.create_string_buffer(4096)
    if fmt == "qint8":
        rc = L.tppx_plan_linear_qint8(M, N, K, qbs, 1, flags, ws_bytes, buf, len(buf))
    else:
        rc = L.tppx_plan_linear_mxfp4(M, N, K, flags, ws_bytes, buf, len(buf))
    return plan_lines(buf.value.decode()) if rc == 0 else []


def group_plan(L, fmt, Ns, M, K, dual, flags, ws_bytes, qbs=256):
    """The same for a fused group (q/k/v) or, dual = 1, the gate/up pair."""
    buf = ctypes.create_string_buffer(4096)
    arr = (ctypes.c_int64 * len(Ns))(*Ns)
    if fmt == "qint8":
        rc = L.tppx_plan_multi_linear_qint8(arr, len(Ns), M, K, qbs, 1, flags, ws_bytes, buf, len(buf))
    else:
        rc = L.tppx_plan_multi_linear_mxfp4(arr, len(Ns), M, K, dual, flags, ws_bytes, buf, len(buf))
    return plan_lines(buf.value.decode()) if rc == 0 else []


def oracle_mod():
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import oracle as O
    cores = len(os.sched_getaffinity(0))
    cores = min(cores, O.num_threads()) if O.num_threads() > 0 else cores
    O.set_num_threads(cores)
    return O, cores


def repeat_for(fn, seconds, max_n=400):
    fn()  # warm-up
    n, t0 = 0, time.perf_counter()
    while True:
        fn()
        n += 1
        dt = time.perf_counter() - t0
        if dt > seconds or n >= max_n:
            return n, dt


def t_bits(t):
    import numpy as np
    import torch
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


# ---------------------------------------------------------------------------------------------------------------
# config 2 (headline)
# ---------------------------------------------------------------------------------------------------------------
def run_decode(torch, _ops, args, per_channel=False):
    """per_channel: one scale per output channel (QINT8_BLOCK_SIZE = K for each weight: 4096 on the up-projection,
    11008 on the down-projection) instead of the reference default of 256-wide blocks."""
    dev = torch.device("cuda:0")
    fmt = args.fmt
    shapes = dict(CFG2_SHAPES)
    Ms = list(CFG2_MS)
    qbs = {name: (K if per_channel else 256) for name, (N, K) in shapes.items()}
    W, X, R = make_inputs(torch, shapes, Ms, 1236)

    def quant(t):
        if fmt != "qint8":
            return _ops.remap_and_quantize_mxfp4(t)
        old = _ops.QINT8_BLOCK_SIZE
        _ops.QINT8_BLOCK_SIZE = t.shape[1] * t.shape[2] * t.shape[4] if per_channel else 256
        try:
            return _ops.remap_and_quantize_qint8(t)
        finally:
            _ops.QINT8_BLOCK_SIZE = old

    # pool of weight sets: every (set, shape, M) gets its own copy so a step
    # touches len(Ms) * (45+45) MB = 360 MB of distinct weight bytes (QINT8)
    pool = []
    for s in range(max(1, args.pool)):
        ws = {}
        for name in shapes:
            base = quant(block_bf16(W[name]).to(dev))
            base.native()
            for M in Ms:
                ws[(name, M)] = clone_weight(base)
        pool.append(ws)
    Xd = {k: v.to(dev) for k, v in X.items()}
    Rd = {k: v.to(dev) for k, v in R.items()}
    empty = torch.empty(0, dtype=torch.bfloat16, device=dev)

    def step(ws):
        outs = []
        for M in Ms:
            for name in ("up", "down"):
                outs.append(torch.ops.tpp_llm.fc_add(Xd[(name, M)], ws[(name, M)], empty, Rd[(name, M)], 1.0))
        return outs

    bytes_per_step = sum(algorithmic_bytes(fmt, M, N, K, qbs[name]) for name, (N, K) in shapes.items() for M in Ms)
    flops_per_step = sum(2 * M * N * K for (N, K) in shapes.values() for M in Ms)

    graphs = None
    if not args.no_graph:
        try:
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for ws in pool:
                    step(ws)
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graphs = []
            for ws in pool:
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g):
                    keep = step(ws)
                graphs.append((g, keep))
        except Exception as e:  # graph capture unavailable: time eager launches
            print(f"bench.py: graph capture failed ({e!r}); timing eager launches", file=sys.stderr)
            graphs = None

    def run_step(i):
        if graphs is not None:
            graphs[i % len(graphs)][0].replay()
        else:
            step(pool[i % len(pool)])

    ms_per_step, blocks = time_blocks(torch, run_step, args.steps, args.warmup)
    value_tbs = bytes_per_step / (ms_per_step * 1e-3) / 1e12

    roof = roofline_decode(torch, fmt, pool, Xd, Rd, Ms, shapes, qbs, args)
    cpu = None if args.no_cpu else cpu_baseline_decode(fmt, W, X, R, Ms, shapes, qbs, bytes_per_step)
    return {
        "metric": "quant-GEMM HBM TB/s (decode)",
        "value": round(value_tbs, 4),
        "unit": "TB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8" if fmt == "qint8" else "bf16",
        "data": "synthetic",
        "config": {
            "workload": (("cfg2: QINT8 W8A8 (per-output-channel scales, QBS=K) fc_add" if per_channel else
                          "cfg2: QINT8 W8A8 (QBS=256) fc_add") if fmt == "qint8" else "MXFP4 fc_add")
            + ", Llama-7B MLP up 4096->11008 + down 11008->4096, M in {1,8,32,64}; one step = these 8 fused linears",
            "launch": "hipGraph replay of one step" if graphs is not None else "eager launches",
            "timed": f"{blocks} blocks of exactly {args.steps} steps, each between two synchronizes (>= {MIN_WALL_S} s in "
                     f"all); ms_per_step is their mean",
            "weight_pool_MB": round(len(pool) * len(Ms) * sum(algorithmic_bytes(fmt, 0, N, K, qbs[name], post_in=False)
                                                              for name, (N, K) in shapes.items()) / 1e6, 1),
            "bytes_per_step": bytes_per_step,
            "tflops": round(flops_per_step / (ms_per_step * 1e-3) / 1e12, 2),
        },
        "roofline": roof,
        "cpu_baseline": cpu,
    }


def roofline_decode(torch, fmt, pool, Xd, Rd, Ms, shapes, qbs_by_shape, args):
    """Each GEMM kernel of the step alone, between two events on the launch
    stream.  One graph per (shape, M) holds one launch per weight copy of that
    shape in the pool (> 256 MB, so every launch streams from HBM).  For QINT8
    kernels that do not quantize inside the GEMM the activation is quantized once
    beforehand and the timed launches reuse it (TPPX_FLAG_XQ_REUSE), so only the
    GEMM kernel runs.  achieved = algorithmic bytes of the call / mean kernel duration."""
    from tpp_pytorch_extension import _lib
    L = _lib.lib()
    dev = torch.device("cuda:0")
    ws = _lib.workspace(torch.empty(1, device=dev))
    stream = torch.cuda.current_stream().cuda_stream
    rows = []
    keep = []
    for M in Ms:
        for name, (N, K) in shapes.items():
            x, r = Xd[(name, M)], Rd[(name, M)]
            y = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
            copies = [w.native() for wset in pool for (nm, _m), w in wset.items() if nm == name]
            qb = qbs_by_shape[name]
            if fmt == "qint8":
                xq = torch.empty(((M + 63) // 64 * 64, K), dtype=torch.int8, device=dev)
                sa = torch.empty(((M + 63) // 64 * 64, K // qb), dtype=torch.float32, device=dev)
                keep += [xq, sa]

                def call(qn, sn, flags, st, qb=qb):
                    _lib.check(L.tppx_linear_qint8(x.data_ptr(), xq.data_ptr(), sa.data_ptr(), qn.data_ptr(),
                                                   sn.data_ptr(), None, r.data_ptr(), None, y.data_ptr(), M, N, K, qb,
                                                   3, 1.0, flags, ws.data_ptr(), ws.numel(), st))
                reuse = _lib.FLAG_XQ_REUSE
            else:
                def call(qn, sn, flags, st):
                    _lib.check(L.tppx_linear_mxfp4(x.data_ptr(), qn.data_ptr(), sn.data_ptr(), None, r.data_ptr(), None,
                                                   y.data_ptr(), M, N, K, 3, 1.0, flags, ws.data_ptr(), ws.numel(), st))
                reuse = 0
            keep += [y]
            plan_call = kernel_plan(L, fmt, M, N, K, qb, 0, ws.numel())       # what an op call enqueues
            plan = kernel_plan(L, fmt, M, N, K, qb, reuse, ws.numel())        # what is timed here
            call(copies[0][0], copies[0][1], 0, stream)  # quantizes the activation where the path keeps it
            torch.cuda.synchronize()

            def fire(st):
                for qn, sn in copies:
                    call(qn, sn, reuse, st)

            avg_us, n_launch = events_us(torch, fire, len(copies), use_graph=not args.no_graph)
            call_us = avg_us
            if len(plan_call) > len(plan):  # the whole call: activation quantizer + GEMM

                def fire_call(st):
                    for qn, sn in copies:
                        call(qn, sn, 0, st)

                call_us, _ = events_us(torch, fire_call, len(copies), use_graph=not args.no_graph)
            nbytes = algorithmic_bytes(fmt, M, N, K, qb)
            rows.append({
                "kernel": plan[-1][0] if plan else "?",
                "launch": plan[-1][1] if plan else "",
                "call": f"{name} M={M} N={N} K={K}",
                "kernels_per_call": len(plan_call),
                "avg_launch_us": round(avg_us, 3),
                "call_us": round(call_us, 3),
                "bytes_per_launch": nbytes,
                "achieved": round(nbytes / avg_us / 1e3, 1),
                "frac": round(nbytes / avg_us / 1e3 / HBM_PEAK_GBS, 4),
                "call_frac": round(nbytes / call_us / 1e3 / HBM_PEAK_GBS, 4),
                "launches_timed": n_launch,
            })
    # the dominant kernel = the one a step spends most time in (each runs once per step)
    dom = max(rows, key=lambda r: r["avg_launch_us"])
    traffic = measured_traffic(dom["kernel"], dom["call"])
    return {
        "bound": "hbm",
        "kernel": dom["kernel"],
        "call": dom["call"],
        "achieved": dom["achieved"],
        "peak": HBM_PEAK_GBS,
        "unit": "GB/s",
        "frac": dom["frac"],
        "traffic": traffic,
        "avg_launch_us": dom["avg_launch_us"],
        "bytes_per_launch": dom["bytes_per_launch"],
        "launches_timed": dom["launches_timed"],
        "timing": "events on the launch stream around graph replays of this kernel alone; frac = the call's algorithmic "
                  "bytes / the GEMM kernel's time, call_frac = the same bytes / (activation quantizer + GEMM)",
        "all_gemm_kernels": rows,
    }


def measured_traffic(kernel, call):
    """HBM bytes per launch of `kernel` from the committed counter summary
    (FETCH_SIZE + WRITE_SIZE, scaled by a copy kernel of known size); None when
    no summary covers this kernel and call."""
    path = os.path.join(ROOT, "profiles", "traffic_pmc.json")
    try:
        with open(path) as f:
            table = json.load(f)
    except (OSError, ValueError):
        return None
    for e in table.get("kernels", []):
        if e.get("kernel") == kernel and e.get("call") == call:
            return e.get("hbm_bytes_per_launch")
    return None


def cpu_baseline_decode(fmt, W, X, R, Ms, shapes, qbs, bytes_per_step, seconds=10.0):
    """The oracle's restatement of the reference CPU path on the host cores,
    one step's worth of linears on the same seeded inputs, repeated for about
    10 s."""
    O, cores = oracle_mod()
    qw = {}
    for name in shapes:
        Wf = W[name].float().numpy()
        qw[name] = O.remap_quantize_qint8(Wf, env_block=qbs[name])[:2] if fmt == "qint8" else O.remap_quantize_mxfp4(Wf)
    lin = O.linear_qint8 if fmt == "qint8" else O.linear_mxfp4
    xs = {k: t_bits(v) for k, v in X.items()}
    rs = {k: t_bits(v) for k, v in R.items()}

    def one_step():
        for M in Ms:
            for name in shapes:
                q, s = qw[name]
                lin(xs[(name, M)], q, s, None, O.POST_ADD_SCALE, rs[(name, M)], None, 1.0, O.MODE_FAITHFUL)

    n, dt = repeat_for(one_step, seconds)
    sec = dt / n
    return {
        "value": round(bytes_per_step / sec / 1e12, 5),
        "unit": "TB/s",
        "cores": cores,
        "kind": "port",
        "sample": f"{n} passes over the same 8-linear step (C/OpenMP restatement of the reference recipe, "
                  f"faithful bf16 re-rounding; not the libxsmm JIT), {round(sec * 1e3, 1)} ms per step",
    }


# ---------------------------------------------------------------------------------------------------------------
# config 2's shapes with QINT4 and ternary QINT2 weights (the other members of the reference's W8A8 class): decode
# steps stream the codes at their own width
# ---------------------------------------------------------------------------------------------------------------
def leg_low_bit(torch, _ops, args):
    from tpp_pytorch_extension import _lib
    L = _lib.lib()
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(1240)
    rows, total_bytes, total_us = [], 0.0, 0.0
    for kind, bits in (("qint4", 4), ("qint2", 2)):
        for name, (N, K) in CFG2_SHAPES.items():
            nc = 16  # 16 copies x 11..22 MB per shape: beyond the 256 MB Infinity Cache together with the other shape

            def mk():
                W = (torch.randn((N, K), generator=g, device=dev) * 0.02).to(torch.bfloat16)
                if kind == "qint4":
                    t = W.view(N // 16, 16, K // 256, 128, 2).permute(0, 2, 3, 1, 4).contiguous()
                    w = _ops.quantize_int4sym(t, 256, 2, True)
                else:
                    w = _ops.remap_and_quantize_qint2_intlv(block_bf16(W))
                w.native_packed()
                w._native = None  # the decode step needs the packed codes only
                return w

            ws = [mk() for _ in range(nc)]
            for M in (1, 8):
                x = torch.randn((M, K), generator=g, device=dev).to(torch.bfloat16)
                r = torch.randn((M, N), generator=g, device=dev).to(torch.bfloat16)

                def fire(_st):
                    return [_ops.fc_add(x, w, None, r, 1.0) for w in ws]

                fire(None)
                us, n = events_us(torch, fire, nc, use_graph=not args.no_graph)
                nbytes = N * K * bits // 8 + 4 * N * (K // 256) + 2 * M * K + 4 * M * N
                rows.append({"kernel": kind, "call": f"{name} M={M}", "kernels_per_call": 1, "avg_launch_us": round(us, 3),
                             "bytes_per_launch": nbytes, "achieved": round(nbytes / us / 1e3, 1),
                             "frac": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4), "launches_timed": n})
                total_bytes += nbytes
                total_us += us
            del ws
    dom = max(rows, key=lambda r: r["avg_launch_us"])
    buf = ctypes.create_string_buffer(1024)
    return {
        "leg": "cfg2-qint4-qint2", "metric": "quant-GEMM HBM TB/s (decode)", "value": round(total_bytes / total_us / 1e6, 4),
        "unit": "TB/s", "ms_per_step": round(total_us / 1e3, 5), "dtype": "int8",
        "workload": "cfg2 shapes, QINT4 and ternary QINT2 weights (codes streamed at 4 / 2 bits), fc_add, M in {1,8}",
        "roofline": {"bound": "hbm", "kernel": "skinny_qint8_fq_kernel<.., 4 | 2> (" + dom["kernel"] + ")", "call": dom["call"],
                     "achieved": dom["achieved"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": dom["frac"], "traffic": None,
                     "avg_launch_us": dom["avg_launch_us"], "bytes_per_launch": dom["bytes_per_launch"],
                     "all_gemm_kernels": rows},
        "cpu_baseline": None,
    }


# ---------------------------------------------------------------------------------------------------------------
# config 1: one MXFP4 fc_plain, M = 16, 4096 x 4096, bias
# ---------------------------------------------------------------------------------------------------------------
def leg_cfg1(torch, _ops, args):
    from tpp_pytorch_extension import _lib
    L = _lib.lib()
    dev = torch.device("cuda:0")
    M, N, K = 16, 4096, 4096
    g = torch.Generator(device="cpu").manual_seed(1235)
    W = (torch.randn((N, K), generator=g) * 0.02).to(torch.bfloat16)
    x = torch.randn((M, K), generator=g).to(torch.bfloat16)
    bias = (torch.randn((N,), generator=g) * 0.01).to(torch.bfloat16)
    base = _ops.remap_and_quantize_mxfp4(block_bf16(W).to(dev))
    copies = [clone_weight(base) for _ in range(32)]  # 32 x 8.9 MB = 285 MB of distinct weight bytes
    xd, bd = x.to(dev), bias.to(dev)

    def fire(_st):
        return [torch.ops.tpp_llm.fc_plain(xd, w, bd, -1, []) for w in copies]

    fire(None)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        keep = fire(None)
    ms, blocks = time_blocks(torch, lambda i: graph.replay(), 4, 2)
    us_call = ms * 1e3 / len(copies)
    nbytes = algorithmic_bytes("mxfp4", M, N, K, bias=True, post_in=False)
    ev_us, n_launch = events_us(torch, lambda st: graph.replay(), len(copies), use_graph=False)
    plan = kernel_plan(L, "mxfp4", M, N, K, 256, 0, _lib.WORKSPACE_BYTES)
    cpu = None
    if not args.no_cpu:
        O, cores = oracle_mod()
        q, sc = O.remap_quantize_mxfp4(W.float().numpy())
        xb, bb = t_bits(x), t_bits(bias)
        n, dt = repeat_for(lambda: O.linear_mxfp4(xb, q, sc, bb, O.POST_NONE, None, None, 1.0, O.MODE_FAITHFUL), 3.0)
        cpu = {"value": round(nbytes * n / dt / 1e12, 5), "unit": "TB/s", "cores": cores, "kind": "port",
               "sample": f"{n} passes of the same linear on the same inputs, {round(dt / n * 1e3, 2)} ms each"}
    del keep
    return {
        "leg": "cfg1", "metric": "quant-GEMM HBM TB/s (decode)", "value": round(nbytes / us_call / 1e6, 4), "unit": "TB/s",
        "us_per_call": round(us_call, 3), "dtype": "bf16",
        "workload": "cfg1: MXFP4 fc_plain, M=16, K=N=4096, bf16 bias; 32 weight copies in rotation (285 MB), one HIP "
                    "graph of 32 calls replayed",
        "roofline": {"bound": "hbm", "kernel": plan[-1][0] if plan else "?", "launch": plan[-1][1] if plan else "",
                     "achieved": round(nbytes / ev_us / 1e3, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(nbytes / ev_us / 1e3 / HBM_PEAK_GBS, 4), "traffic": None,
                     "avg_launch_us": round(ev_us, 3), "bytes_per_launch": nbytes, "launches_timed": n_launch},
        "cpu_baseline": cpu,
    }


# ---------------------------------------------------------------------------------------------------------------
# config 3: MXFP4 SwiGLU MLP block, M in {1, 4, 16, 64}
# ---------------------------------------------------------------------------------------------------------------
def cfg3_bytes(M, H=4096, I=11008):
    """weights + scales of the three projections, X, residual, out, and the intermediate written once + read once."""
    w = 3 * (H * I // 2 + H * I // 32)
    return w + 3 * (2 * M * H) + 2 * (2 * M * I)


def leg_cfg3(torch, _ops, args):
    from tpp_pytorch_extension import _lib
    L = _lib.lib()
    dev = torch.device("cuda:0")
    H, I = CFG3_DIMS
    Ms = list(CFG3_MS)
    g = torch.Generator(device="cpu").manual_seed(1237)
    Wg = (torch.randn((I, H), generator=g) * 0.02).to(torch.bfloat16)
    Wu = (torch.randn((I, H), generator=g) * 0.02).to(torch.bfloat16)
    Wd = (torch.randn((H, I), generator=g) * 0.02).to(torch.bfloat16)
    X = {M: torch.randn((M, H), generator=g).to(torch.bfloat16) for M in Ms}
    base = [_ops.remap_and_quantize_mxfp4(block_bf16(w).to(dev)) for w in (Wg, Wu, Wd)]
    pool = [{M: [clone_weight(b) for b in base] for M in Ms} for _ in range(2)]  # 2 x 4 x 72 MB = 575 MB
    Xd = {M: X[M].to(dev) for M in Ms}

    def step(ws):
        return [torch.ops.tpp_llm.swiglu_mlp(Xd[M], ws[M][0], ws[M][1], ws[M][2], Xd[M], 1.0) for M in Ms]

    for ws in pool:
        step(ws)
    torch.cuda.synchronize()
    graphs = []
    for ws in pool:
        gr = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gr):
            keep = step(ws)
        graphs.append((gr, keep))
    ms, blocks = time_blocks(torch, lambda i: graphs[i % 2][0].replay(), 20, 5)
    bytes_per_step = sum(cfg3_bytes(M) for M in Ms)

    # each launch alone: gate/up pair, down projection
    rows = []
    wsb = _lib.WORKSPACE_BYTES
    for M in Ms:
        xin = Xd[M]
        inter = _ops.swiglu_gate_up(xin, pool[0][M][0], pool[0][M][1])
        sets = [p[M] for p in pool] + [[clone_weight(b) for b in base] for _ in range(10)]  # 12 x 72 MB

        def fire_gu(_st):
            return [_ops.swiglu_gate_up(xin, w[0], w[1]) for w in sets]

        def fire_dn(_st):
            return [_ops.fc_add(inter, w[2], None, xin, 1.0) for w in sets]

        for nm, fire, nb, pl in (
                ("gate/up", fire_gu, 2 * (H * I // 2 + H * I // 32) + 2 * M * H + 2 * M * I,
                 group_plan(L, "mxfp4", [I, I], M, H, 1, 0, wsb)),
                ("down", fire_dn, (H * I // 2 + H * I // 32) + 2 * M * I + 2 * (2 * M * H),
                 kernel_plan(L, "mxfp4", M, H, I, 256, 0, wsb))):
            us, n = events_us(torch, fire, len(sets), use_graph=not args.no_graph)
            rows.append({"kernel": pl[-1][0] if pl else "?", "launch": pl[-1][1] if pl else "", "call": f"{nm} M={M}",
                         "kernels_per_call": len(pl), "avg_launch_us": round(us, 3), "bytes_per_launch": nb,
                         "achieved": round(nb / us / 1e3, 1), "frac": round(nb / us / 1e3 / HBM_PEAK_GBS, 4),
                         "launches_timed": n})
        del sets, inter
    dom = max(rows, key=lambda r: r["avg_launch_us"])
    cpu = None
    if not args.no_cpu:
        O, cores = oracle_mod()
        qs = [O.remap_quantize_mxfp4(w.float().numpy()) for w in (Wg, Wu, Wd)]
        xb = {M: t_bits(X[M]) for M in Ms}

        def one():
            for M in Ms:
                gate = O.linear_mxfp4(xb[M], qs[0][0], qs[0][1], None, O.POST_SILU, None, None, 1.0, O.MODE_FAITHFUL)
                it = O.linear_mxfp4(xb[M], qs[1][0], qs[1][1], None, O.POST_MUL, gate, None, 1.0, O.MODE_FAITHFUL)
                O.linear_mxfp4(it, qs[2][0], qs[2][1], None, O.POST_ADD_SCALE, xb[M], None, 1.0, O.MODE_FAITHFUL)

        n, dt = repeat_for(one, 6.0)
        cpu = {"value": round(bytes_per_step * n / dt / 1e12, 5), "unit": "TB/s", "cores": cores, "kind": "port",
               "sample": f"{n} passes over the same four MLP blocks, {round(dt / n * 1e3, 1)} ms per step"}
    per_m = {}
    for M in Ms:
        us = sum(r["avg_launch_us"] for r in rows if r["call"].endswith(f"M={M}"))
        per_m[str(M)] = {"us_per_block": round(us, 2), "TB/s": round(cfg3_bytes(M) / us / 1e6, 3)}
    return {
        "leg": "cfg3", "metric": "quant-GEMM HBM TB/s (decode)",
        "value": round(bytes_per_step / (ms * 1e-3) / 1e12, 4), "unit": "TB/s", "ms_per_step": round(ms, 5), "dtype": "bf16",
        "workload": "cfg3: MXFP4 SwiGLU MLP block (torch.ops.tpp_llm.swiglu_mlp = gate/up launch + down launch), hidden "
                    "4096, intermediate 11008, M in {1,4,16,64}; one step = the four blocks; two weight sets of 288 MB "
                    "alternate; HIP graph replay",
        "bytes_per_step": bytes_per_step, "per_M": per_m,
        "roofline": {"bound": "hbm", "kernel": dom["kernel"], "call": dom["call"], "achieved": dom["achieved"],
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": dom["frac"],
                     "traffic": measured_traffic(dom["kernel"], dom["call"]),
                     "avg_launch_us": dom["avg_launch_us"], "bytes_per_launch": dom["bytes_per_launch"],
                     "launches_timed": dom["launches_timed"], "all_gemm_kernels": rows},
        "cpu_baseline": cpu,
    }


# ---------------------------------------------------------------------------------------------------------------
# config 4: prefill GEMMs of one 70B-shape decoder layer at M = 2048
# ---------------------------------------------------------------------------------------------------------------
def leg_cfg4(torch, _ops, args, pfmt="mxfp4", fp8=False, cpu=True):
    """M = 2048 tokens through the linears of one decoder layer with hidden 8192 (fused qkv 8192 -> 8192+1024+1024,
    o 8192 -> 8192 + residual, then the MLP block gate/up 8192 -> 28672 with silu * mul and down 28672 -> 8192 +
    residual through the package's swiglu_mlp op, whose result is bit-identical to fc_silu, fc_mul, fc_add in
    sequence).  One step = those three op calls (seven GEMMs)."""
    from tpp_pytorch_extension import _lib
    L = _lib.lib()
    dev = torch.device("cuda:0")
    M, H, I = CFG4_DIMS
    g = torch.Generator(device=dev).manual_seed(1238)
    fp8 = bool(fp8) and pfmt == "mxfp4"
    old_fp8 = _ops.ACT_FP8
    _ops.ACT_FP8 = fp8
    try:
        quant = _ops.remap_and_quantize_mxfp4 if pfmt == "mxfp4" else _ops.remap_and_quantize_qint8

        def mk(N, K):
            W = (torch.randn((N, K), generator=g, device=dev) * 0.02).to(torch.bfloat16)
            q = quant(W.view(N // 16, 16, K // 64, 32, 2).permute(0, 2, 3, 1, 4).contiguous())
            q.native()
            return q

        wq, wk, wv, wo = mk(H, H), mk(1024, H), mk(1024, H), mk(H, H)
        wg, wu, wd = mk(I, H), mk(I, H), mk(H, I)
        x = torch.randn((M, H), generator=g, device=dev).to(torch.bfloat16)
        res = torch.randn((M, H), generator=g, device=dev).to(torch.bfloat16)
        inter = torch.randn((M, I), generator=g, device=dev).to(torch.bfloat16)
        empty = torch.empty(0, dtype=torch.bfloat16, device=dev)

        def step(_i=0):
            q, k, v = torch.ops.tpp_llm.qkv_gemm(x, [wq, wk, wv], [empty] * 3)
            h = torch.ops.tpp_llm.fc_add(q, wo, empty, res, 1.0)
            return torch.ops.tpp_llm.swiglu_mlp(h, wg, wu, wd, h, 1.0), k, v

        gemms = [("qkv", 10240, H), ("o", H, H), ("gate", I, H), ("up", I, H), ("down", H, I)]
        flops = sum(2.0 * M * N * K for _, N, K in gemms)
        ms, blocks = time_blocks(torch, step, 3, 2)

        peak = PEAKS_TFLOPS["fp8" if fp8 else "bf16"] if pfmt == "mxfp4" else PEAKS_TFLOPS["int8"]
        unit = "TFLOP/s" if pfmt == "mxfp4" else "TOP/s"
        flags = _lib.FLAG_ACT_FP8 if fp8 else 0
        wsb = lambda K: (33 * M * K) // 32 if fp8 else _lib.WORKSPACE_BYTES  # noqa: E731
        ops = [
            ("qkv M=2048 N=10240 K=8192", lambda st: torch.ops.tpp_llm.qkv_gemm(x, [wq, wk, wv], [empty] * 3),
             2.0 * M * 10240 * H, group_plan(L, pfmt, [H, 1024, 1024], M, H, 0, flags, wsb(H))),
            ("o M=2048 N=8192 K=8192", lambda st: torch.ops.tpp_llm.fc_add(x, wo, empty, res, 1.0),
             2.0 * M * H * H, kernel_plan(L, pfmt, M, H, H, 256, flags, wsb(H))),
            ("gate/up M=2048 N=2x28672 K=8192 " + ("(silu*mul in the epilogue)" if pfmt == "mxfp4" else "(fc_silu, then fc_mul)"), lambda st: _ops.swiglu_gate_up(x, wg, wu),
             4.0 * M * I * H, (group_plan(L, pfmt, [I, I], M, H, 1, flags, max(wsb(H), 2 * M * I + wsb(H)))
                               if pfmt == "mxfp4" else kernel_plan(L, pfmt, M, I, H, 256, flags, wsb(H)))),
            ("down M=2048 N=8192 K=28672", lambda st: torch.ops.tpp_llm.fc_add(inter, wd, empty, res, 1.0),
             2.0 * M * H * I, kernel_plan(L, pfmt, M, H, I, 256, flags, wsb(I))),
        ]
        wb = (lambda N, K: N * K // 2 + N * K // 32) if pfmt == "mxfp4" else (lambda N, K: N * K + 4 * N * (K // 256))
        # algorithmic bytes per call: weights + scales, activations in, outputs (and the residual) -- what an ideal
        # single pass would move; the kernels are MFMA-bound, the measured HBM traffic is reported beside it
        algo = [wb(10240, H) + 2 * M * H + 2 * M * 10240, wb(H, H) + 2 * M * H + 4 * M * H,
                2 * wb(I, H) + 2 * M * H + 2 * M * I, wb(H, I) + 2 * M * I + 4 * M * H]
        rows = []
        for (name, fn, fl, pl), nb in zip(ops, algo):
            us, n = events_us(torch, fn, 1, use_graph=False)
            gemm = [p for p in pl if "quant_act" not in p[0] and "silu_mul" not in p[0]]
            rows.append({"kernel": gemm[-1][0] if gemm else "?", "launch": gemm[-1][1] if gemm else "", "call": name,
                         "kernels_per_call": len(pl), "avg_launch_us": round(us, 1), "flops_per_launch": fl,
                         "bytes_per_launch": nb, "achieved": round(fl / us / 1e6, 1), "frac": round(fl / us / 1e6 / peak, 4),
                         "launches_timed": n})
        dom = max(rows, key=lambda r: r["avg_launch_us"] if r["call"].startswith("down") else 0)
        cpu_b = cpu_baseline_prefill(H, pfmt) if (cpu and not args.no_cpu and not fp8) else None
    finally:
        _ops.ACT_FP8 = old_fp8
    label = ("cfg4: MXFP4" + (" weights x MXFP8 activations (opt-in, NOT the reference's arithmetic)" if fp8 else
                              " (bf16 activations, the reference's arithmetic)")) if pfmt == "mxfp4" else \
        "cfg4's layer with QINT8 W8A8 (QBS=256; not a BASELINE configuration)"
    return {
        "leg": "cfg4" + ("" if pfmt == "mxfp4" and not fp8 else ("-act-fp8" if fp8 else "-qint8")),
        "metric": "quant-GEMM TFLOP/s (prefill)", "value": round(flops / (ms * 1e-3) / 1e12, 2), "unit": unit,
        "ms_per_step": round(ms, 4), "dtype": ("fp8" if fp8 else "bf16") if pfmt == "mxfp4" else "int8",
        "workload": label + " linears of one decoder layer (hidden 8192, intermediate 28672, kv 1024) at M = 2048: "
                            "qkv_gemm, fc_add(o), swiglu_mlp(gate, up, down); eager op calls",
        "flops_per_step": flops,
        "roofline": {"bound": "mfma", "kernel": dom["kernel"], "call": dom["call"] +
                     (" (activation quantiser included)" if (fp8 or pfmt == "qint8") else ""),
                     "achieved": dom["achieved"], "peak": peak, "unit": unit, "frac": dom["frac"],
                     "traffic": measured_traffic(dom["kernel"], dom["call"]),
                     "avg_launch_us": dom["avg_launch_us"], "flops_per_launch": dom["flops_per_launch"],
                     "bytes_per_launch": dom["bytes_per_launch"], "launches_timed": dom["launches_timed"],
                     "timing": "events on the launch stream around eager launches of this op alone",
                     "all_gemm_kernels": rows},
        "cpu_baseline": cpu_b,
    }


def leg_w4a8(torch, _ops, args):
    """The reference's USE_MXFP4_INT8 mode (W4A8: MXFP4 weights as integers x int8 activations over blocks of 32,
    src/csrc/fused_gemm.h:965-978) on the linears of config 4's layer at M = 2048, one fc_plain / fc_add call per
    weight (the mode has no fused q/k/v or gate/up launch).  Not a BASELINE configuration; run alone with
    --workload w4a8."""
    dev = torch.device("cuda:0")
    M, H, I = CFG4_DIMS
    g = torch.Generator(device=dev).manual_seed(1239)

    def mk(N, K):
        W = (torch.randn((N, K), generator=g, device=dev) * 0.02).to(torch.bfloat16)
        q = _ops.remap_and_quantize_mxfp4(W.view(N // 16, 16, K // 64, 32, 2).permute(0, 2, 3, 1, 4).contiguous(),
                                          int8_layout=True)
        q.native_w4a8_wide()
        return q

    shapes = [("qkv", 10240, H), ("o", H, H), ("gate", I, H), ("up", I, H), ("down", H, I)]
    ws = {name: mk(N, K) for name, N, K in shapes}
    xs = {H: torch.randn((M, H), generator=g, device=dev).to(torch.bfloat16),
          I: torch.randn((M, I), generator=g, device=dev).to(torch.bfloat16)}
    res = torch.randn((M, H), generator=g, device=dev).to(torch.bfloat16)
    empty = torch.empty(0, dtype=torch.bfloat16, device=dev)

    def call(name, K):
        if name in ("o", "down"):
            return torch.ops.tpp_llm.fc_add(xs[K], ws[name], empty, res, 1.0)
        return torch.ops.tpp_llm.fc_plain(xs[K], ws[name], empty, -1, [])

    def step(_i=0):
        return [call(name, K) for name, _, K in shapes]

    flops = sum(2.0 * M * N * K for _, N, K in shapes)
    ms, blocks = time_blocks(torch, step, 3, 2)
    peak = PEAKS_TFLOPS["bf16"]  # the block sums run on the bf16 MFMA
    rows = []
    for name, N, K in shapes:
        us, n = events_us(torch, lambda st, name=name, K=K: call(name, K), 1, use_graph=False)
        fl = 2.0 * M * N * K
        rows.append({"kernel": "tppx::linear_w4a8_wide_kernel", "call": f"{name} M={M} N={N} K={K} (row quantizer included)",
                     "kernels_per_call": 2, "avg_launch_us": round(us, 1), "flops_per_launch": fl,
                     "bytes_per_launch": 2 * N * K + 2 * M * K + 2 * M * N, "achieved": round(fl / us / 1e6, 1),
                     "frac": round(fl / us / 1e6 / peak, 4), "launches_timed": n})
    dom = max(rows, key=lambda r: r["avg_launch_us"])
    return {
        "leg": "w4a8", "metric": "quant-GEMM TFLOP/s (prefill)", "value": round(flops / (ms * 1e-3) / 1e12, 2),
        "unit": "TFLOP/s", "ms_per_step": round(ms, 4), "dtype": "int8 activations x 4-bit weights (exact block sums on the bf16 MFMA)",
        "workload": "config 4's layer under the reference's USE_MXFP4_INT8 mode (W4A8), M = 2048: one call per weight "
                    "(q/k/v as one 10240-channel weight, o, gate, up, down); eager op calls; not a BASELINE configuration",
        "flops_per_step": flops,
        "roofline": {"bound": "mfma", "kernel": dom["kernel"], "call": dom["call"], "achieved": dom["achieved"],
                     "peak": peak, "unit": "TFLOP/s", "frac": dom["frac"], "traffic": None,
                     "avg_launch_us": dom["avg_launch_us"], "flops_per_launch": dom["flops_per_launch"],
                     "bytes_per_launch": dom["bytes_per_launch"], "launches_timed": dom["launches_timed"],
                     "timing": "events on the launch stream around eager launches of this op alone",
                     "all_gemm_kernels": rows},
        "cpu_baseline": None,
    }


def cpu_baseline_prefill(H, pfmt="mxfp4", seconds=8.0):
    """The oracle's MXFP4 (or QINT8) linear on a bounded sample: 256 rows through a 2048 x 8192 slice of a
    projection, faithful mode."""
    import numpy as np
    O, cores = oracle_mod()
    rng = np.random.default_rng(7)
    Ms, N = 256, 2048
    W = (rng.standard_normal((N, H), dtype=np.float32) * 0.02).astype(np.float32)
    xf = rng.standard_normal((Ms, H), dtype=np.float32)
    xb = (xf.view(np.uint32) >> 16).astype(np.uint16)  # truncation is fine for a timing input
    if pfmt == "mxfp4":
        q, sc = O.remap_quantize_mxfp4(W)
        lin = O.linear_mxfp4
    else:
        q, sc, _ = O.remap_quantize_qint8(W)
        lin = O.linear_qint8
    n, dt = repeat_for(lambda: lin(xb, q, sc, None, O.POST_NONE, None, None, 1.0, O.MODE_FAITHFUL), seconds, 200)
    fl = 2.0 * Ms * N * H
    return {"value": round(fl * n / dt / 1e12, 4), "unit": "TFLOP/s" if pfmt == "mxfp4" else "TOP/s", "cores": cores,
            "kind": "port",
            "sample": f"{n} passes of a {Ms} x {N} x {H} {pfmt.upper()} linear (C/OpenMP restatement of the reference "
                      f"recipe, faithful mode; not the libxsmm JIT), {round(dt / n * 1e3, 1)} ms each"}


# ---------------------------------------------------------------------------------------------------------------
# config 5: 32-layer 7B-shape decoder, greedy decode
# ---------------------------------------------------------------------------------------------------------------
_MODEL = {}


def cfg5_model(torch):
    if "m" not in _MODEL:
        from tpp_pytorch_extension.llm import fused_llama_infer as F
        _MODEL["m"] = F.LlamaDecoder(hidden=4096, inter=11008, n_layers=32, n_heads=32, n_kv_heads=32, vocab=32000,
                                     max_positions=4096, weight_dtype="mxfp4", seed=1239)
    return _MODEL["m"]


def leg_cfg5(torch, args, B, cpu=True):
    """BASELINE config 5: 32-layer Llama-2-7B-shape decoder, all linears (and the lm_head) MXFP4, KV cache
    pre-filled with 2048 positions of N(0,1), greedy decode of 128 new tokens for B sequences from
    random token ids; the decode step is one replayed HIP graph."""
    dev = torch.device("cuda:0")
    ctx, new = 2048, 128
    model = cfg5_model(torch)
    tok = torch.randint(0, 32000, (B,), generator=torch.Generator().manual_seed(5), dtype=torch.int64).to(dev)
    out = model.greedy_decode(tok, model.new_cache(B, ctx, ctx + new + 32), 8)  # warm-up run
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    out = model.greedy_decode(tok, model.new_cache(B, ctx, ctx + new + 32), new)
    torch.cuda.synchronize()
    wall_with_capture = time.perf_counter() - t0
    # the replays alone (capture and warm-up step excluded), repeated until >= MIN_WALL_S
    total, runs = 0.0, 0
    while total < MIN_WALL_S and runs < 50:
        cache = model.new_cache(B, ctx, ctx + new + 32)
        total += model.time_decode_steps(tok, cache, new)
        runs += 1
        del cache
    steps_t = total / runs
    ms = steps_t * 1e3 / new
    lin_bytes = 32 * (3 * 4096 * 4096 + 4096 * 4096 + 3 * 11008 * 4096) * (0.5 + 1.0 / 32) + 32000 * 4096 * (0.5 + 1.0 / 32)
    kv_bytes = B * 32 * 2 * 32 * (ctx + new / 2) * 128 * 2
    achieved = (lin_bytes + kv_bytes) / (ms * 1e-3) / 1e9
    cpu_b = None
    if cpu and not args.no_cpu:
        cpu_b = cpu_baseline_tokens(B)
    return {
        "leg": f"cfg5-batch{B}", "metric": "7B-shape decode tokens/s", "value": round(B * new / steps_t, 1),
        "unit": "tokens/s", "ms_per_step": round(ms, 4), "dtype": "bf16",
        "workload": f"cfg5: 32-layer Llama-2-7B-shape decoder, MXFP4 linears and lm_head, bf16 RMSNorm / rotary / KV cache, "
                    f"context {ctx} of N(0,1), greedy decode of {new} tokens, batch {B}; one HIP graph per decode step, "
                    f"replayed; {runs} runs of {new} steps timed",
        "wall_s_one_run_including_capture": round(wall_with_capture, 4), "tokens_per_run": int(out.numel()),
        "roofline": {"bound": "hbm", "kernel": "whole decode step (one graph)",
                     "per_kernel": f"profiles/decoder_step_kernels_cfg5_batch{B}_stats.txt",
                     "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": measured_traffic("whole decode step", f"cfg5 batch {B}"),
                     "bytes_per_step": int(lin_bytes + kv_bytes)},
        "cpu_baseline": cpu_b,
    }


def cpu_baseline_tokens(B, seconds=6.0):
    """The oracle's composition of ONE decoder layer's decode step (the reference recipe: RMSNorm, q/k/v, rotary,
    attention over 2048 cached keys, o + residual, RMSNorm, gate/up, down + residual) on the host cores, times 32
    layers, plus the MXFP4 lm_head: a bounded sample of the 32-layer step."""
    import numpy as np
    O, cores = oracle_mod()
    rng = np.random.default_rng(11)
    hidden, inter, Nh, H, ctx = 4096, 11008, 32, 128, 2048

    def qw(N, K):
        return O.remap_quantize_mxfp4((rng.standard_normal((N, K), dtype=np.float32) * 0.02).astype(np.float32))

    def bf(a):
        return (np.ascontiguousarray(a, np.float32).view(np.uint32) >> 16).astype(np.uint16)

    Wq, Wk, Wv, Wo = qw(hidden, hidden), qw(hidden, hidden), qw(hidden, hidden), qw(hidden, hidden)
    Wg, Wu, Wd = qw(inter, hidden), qw(inter, hidden), qw(hidden, inter)
    Wl = qw(32000, hidden)
    kc = bf(rng.standard_normal((B, Nh, ctx + 1, H), dtype=np.float32))
    vc = bf(rng.standard_normal((B, Nh, ctx + 1, H), dtype=np.float32))
    x = bf(rng.standard_normal((B, hidden), dtype=np.float32))
    gam = np.ones(hidden, np.float32)
    inv = 1.0 / (10000.0 ** (np.arange(0, H, 2, dtype=np.float32) / H))
    fr = np.outer(np.arange(4096, dtype=np.float32), inv)
    emb = np.stack([np.cos(np.concatenate([fr, fr], -1)), np.sin(np.concatenate([fr, fr], -1))]).astype(np.float32)
    pos = np.full((B, 1), ctx, np.int64)

    def mm(a, w, post=O.POST_NONE, pin=None):
        return O.linear_mxfp4(a, w[0], w[1], None, post, pin, None, 1.0, O.MODE_FAITHFUL)

    def layer():
        h = O.rms_norm(x, gam, 1e-5)
        q, k, v = mm(h, Wq), mm(h, Wk), mm(h, Wv)
        q = O.rotary_llama(q.reshape(B, 1, -1), emb, pos, Nh, H).reshape(B, Nh, H)
        k = O.rotary_llama(k.reshape(B, 1, -1), emb, pos, Nh, H).reshape(B, Nh, H)
        kc[:, :, ctx] = k
        vc[:, :, ctx] = v.reshape(B, Nh, H)
        c = O.attn_decode(q, kc, vc).reshape(B, hidden)
        so = mm(c, Wo, O.POST_ADD_SCALE, x)
        h2 = O.rms_norm(so, gam, 1e-5)
        g = mm(h2, Wg, O.POST_SILU)
        return mm(mm(h2, Wu, O.POST_MUL, g), Wd, O.POST_ADD_SCALE, so)

    n, dt = repeat_for(layer, seconds, 200)
    t_layer = dt / n
    n2, dt2 = repeat_for(lambda: mm(x, Wl), 1.0, 50)
    t_step = 32 * t_layer + dt2 / n2
    return {"value": round(B / t_step, 3), "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": f"{n} passes of one decoder layer's decode step at batch {B} (oracle composition, "
                      f"{round(t_layer * 1e3, 1)} ms each) x 32 layers + the lm_head ({round(dt2 / n2 * 1e3, 1)} ms): "
                      f"{round(t_step * 1e3, 1)} ms per token step"}


def run_prompt(torch, args):
    """Prompt processing on the 7B-shape decoder of config 5: `--batch` sequences of `--prompt-len` (2048) random
    token ids through the 32 layers in one pass (MXFP4 linears on the large-M kernels, causal attention, keys
    appended to an empty cache), then the lm_head on the last position.  Not a BASELINE configuration; reported as
    prompt tokens/s."""
    from tpp_pytorch_extension.llm import fused_llama_infer as F
    dev = torch.device("cuda:0")
    B, S = args.batch, args.prompt_len
    model = cfg5_model(torch)
    prompt = torch.randint(0, 32000, (B, S), generator=torch.Generator().manual_seed(6), dtype=torch.int64).to(dev)
    steps, warmup = max(2, min(args.steps, 8)), max(1, min(args.warmup, 2))
    caches = [F.TppCache(S + 32) for _ in range(steps + warmup)]
    for c in caches[:warmup]:
        model.prefill(prompt, c)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for c in caches[warmup:]:
        model.prefill(prompt, c)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    lin_flops = 2.0 * B * S * 32 * (4 * 4096 * 4096 + 3 * 11008 * 4096) + 2.0 * B * 32000 * 4096
    attn_flops = 32 * 4.0 * B * 32 * 128 * (S * (S + 1) / 2)
    tf = (lin_flops + attn_flops) / (ms * 1e-3) / 1e12
    return {
        "metric": "7B-shape prompt tokens/s", "value": round(B * S / (ms * 1e-3), 1), "unit": "tokens/s", "n_gpus": 1,
        "steps": steps, "warmup": warmup, "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"32-layer Llama-2-7B-shape decoder, MXFP4 linears, prompt of {S} tokens x batch {B} in "
                               f"one pass onto an empty KV cache", "launch": "eager op calls", "batch": B},
        "roofline": {"bound": "mfma", "kernel": "whole prompt pass (GEMMs + causal attention + glue)",
                     "achieved": round(tf, 1), "peak": PEAKS_TFLOPS["bf16"], "unit": "TFLOP/s",
                     "frac": round(tf / PEAKS_TFLOPS["bf16"], 4), "traffic": None,
                     "flops_per_step": lin_flops + attn_flops},
        "cpu_baseline": None}


def short_kernel(name):
    return name.replace("tppx::", "").replace("_kernel", "").replace("skinny_", "sk_").replace(" ", "")


def compact_rows(rows):
    """[kernel, call, GEMM-kernel us, frac of peak, kernels per call, whole-call us] per GEMM of a leg."""
    out = []
    for r in rows:
        row = [short_kernel(r["kernel"]), r["call"].split(" N=")[0].split(" (")[0], round(r["avg_launch_us"], 2),
               round(r["frac"], 3)]
        if r["kernels_per_call"] > 1 and "call_us" in r:  # a quantizer launch in front: kernels per call, whole-call us
            row += [r["kernels_per_call"], round(r.get("call_us", r["avg_launch_us"]), 2)]
        out.append(row)
    return out


def compact_roofline(r, leg=False):
    if not r:
        return r
    keep = ("bound", "kernel", "call", "achieved", "peak", "unit", "frac", "traffic", "avg_launch_us") + \
        (() if leg else ("bytes_per_launch", "flops_per_launch", "bytes_per_step"))
    out = {k: r[k] for k in keep if k in r}
    out["kernel"] = short_kernel(out.get("kernel", ""))[:40]
    if "call" in out:
        out["call"] = out["call"].split(" (")[0]
    return out


def compact_cpu(c, leg=False):
    if not c:
        return c
    out = dict(c)
    out["sample"] = out.get("sample", "").split(" (")[0][:40 if leg else 110]
    if leg:  # same host, same threads and the same kind of baseline as the headline's
        out.pop("cores", None)
        out.pop("kind", None)
    return out


def compact_leg(leg):
    """What the one-line record keeps of a leg (the verbose form goes to stderr)."""
    if "roofline" not in leg:
        return leg
    # value, unit, ms_per_step, the dominant kernel, its duration and fraction are in the line's `summary` row of the leg
    roof = compact_roofline(leg["roofline"], True)
    for k in ("kernel", "avg_launch_us", "frac", "unit", "peak"):
        roof.pop(k, None)
    out = {"leg": leg["leg"], "dtype": leg["dtype"],
           "workload": leg["workload"].split(";")[0].split(" linears of")[0].split(", Llama")[0][:60], "roofline": roof,
           "cpu_baseline": compact_cpu(leg["cpu_baseline"], True)}
    rows = leg["roofline"].get("all_gemm_kernels")
    if rows:
        out["gemm_kernels"] = compact_rows(rows)
    return out


def summary_of(headline, legs):
    """One row per leg, the headline first: [leg, value, unit, ms_per_step, dominant kernel, its us, its fraction of
    the roofline, HBM traffic / algorithmic bytes (or None), CPU value].  The LAST key of the line."""
    rows = []
    for name, d in [("cfg2", headline)] + [(l.get("leg"), l) for l in legs]:
        r = d.get("roofline")
        if not r:
            rows.append([name, d.get("error") or d.get("skipped")])
            continue
        tr = r.get("traffic")
        ratio = round(tr / r["bytes_per_launch"], 3) if tr and r.get("bytes_per_launch") else None
        cpu = d.get("cpu_baseline") or {}
        rows.append([name, d["value"], d["unit"], d.get("ms_per_step", round(d.get("us_per_call", 0.0) / 1e3, 6)),
                     short_kernel(r.get("kernel", ""))[:32],
                     r.get("avg_launch_us"), r.get("frac"), ratio, cpu.get("value")])
    return rows


def leg_as_line(leg, args):
    """A leg run alone (--workload ...) printed in the shape of the headline line."""
    return {"metric": leg["metric"], "value": leg["value"], "unit": leg["unit"], "n_gpus": 1, "steps": args.steps,
            "warmup": args.warmup, "ms_per_step": leg.get("ms_per_step", leg.get("us_per_call", 0.0) / 1e3),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": leg["dtype"],
            "data": "synthetic", "config": {k: v for k, v in leg.items() if k not in ("roofline", "cpu_baseline", "metric",
                                                                                      "value", "unit", "dtype")},
            "roofline": leg["roofline"], "cpu_baseline": leg["cpu_baseline"]}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--fmt", default="qint8", choices=["qint8", "mxfp4"])
    ap.add_argument("--batch", type=int, default=1, help="sequences for --workload tokens (1 or 16 in the baseline)")
    ap.add_argument("--prompt-len", type=int, default=2048, help="tokens per sequence for --workload prompt")
    ap.add_argument("--workload", default="all", choices=["all", "decode", "cfg1", "cfg3", "prefill", "tokens", "prompt", "w4a8"],
                    help="all = the headline (config 2) plus every other leg of the metric under config.legs (default); "
                         "decode = the headline alone; cfg1 / cfg3 / prefill (config 4) / tokens (config 5) = that leg "
                         "alone; prompt = a 2048-token prompt through the 7B-shape decoder; w4a8 = config 4's layer under the "
                         "reference's USE_MXFP4_INT8 mode (never part of the default run)")
    ap.add_argument("--prefill-fmt", default="mxfp4", choices=["mxfp4", "qint8"],
                    help="weight format of --workload prefill (BASELINE config 4 is MXFP4; qint8 = the same layer W8A8)")
    ap.add_argument("--act-fp8", action="store_true",
                    help="--workload prefill, MXFP4: quantise activations to MXFP8 and use the block-scaled MFMA "
                         "(opt-in; not the reference's arithmetic, whose activations stay bf16)")
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying a HIP graph")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--pool", type=int, default=2, help="number of distinct weight sets cycled through")
    ap.add_argument("--pmc-calibrate", action="store_true",
                    help="also run three plain 256 MiB device copies, the known-size reference for scaling "
                         "FETCH_SIZE / WRITE_SIZE counter readings")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU; --gpus must be 1 (every box has one GPU and the "
              "path has no collectives)", file=sys.stderr)
        sys.exit(2)

    import torch
    import tpp_pytorch_extension  # noqa: F401
    from tpp_pytorch_extension import _ops

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    torch.cuda.set_device(torch.device("cuda:0"))

    if args.pmc_calibrate:
        src = torch.ones(64 * 1024 * 1024, dtype=torch.int32, device="cuda:0")  # 256 MiB read + 256 MiB written
        for _ in range(3):
            dst = src.clone()
        torch.cuda.synchronize()
        del src, dst
        torch.cuda.empty_cache()

    if args.workload == "cfg1":
        return print(json.dumps(leg_as_line(leg_cfg1(torch, _ops, args), args)))
    if args.workload == "cfg3":
        return print(json.dumps(leg_as_line(leg_cfg3(torch, _ops, args), args)))
    if args.workload == "prefill":
        return print(json.dumps(leg_as_line(leg_cfg4(torch, _ops, args, args.prefill_fmt, args.act_fp8), args)))
    if args.workload == "tokens":
        return print(json.dumps(leg_as_line(leg_cfg5(torch, args, args.batch), args)))
    if args.workload == "prompt":
        return print(json.dumps(run_prompt(torch, args)))
    if args.workload == "w4a8":
        return print(json.dumps(leg_as_line(leg_w4a8(torch, _ops, args), args)))

    t_start = time.perf_counter()
    out = run_decode(torch, _ops, args)
    if args.workload == "all":
        legs = []

        def per_channel_leg():
            d = run_decode(torch, _ops, args, per_channel=True)
            return {"leg": "cfg2-per-channel", "metric": d["metric"], "value": d["value"], "unit": d["unit"],
                    "ms_per_step": d["ms_per_step"], "dtype": d["dtype"], "workload": d["config"]["workload"],
                    "roofline": d["roofline"], "cpu_baseline": d["cpu_baseline"]}

        todo = [
            ("cfg2-per-channel", per_channel_leg),
            ("cfg2-qint4-qint2", lambda: leg_low_bit(torch, _ops, args)),
            ("cfg1", lambda: leg_cfg1(torch, _ops, args)),
            ("cfg3", lambda: leg_cfg3(torch, _ops, args)),
            ("cfg4", lambda: leg_cfg4(torch, _ops, args, "mxfp4", False)),
            ("cfg4-qint8", lambda: leg_cfg4(torch, _ops, args, "qint8", False)),
            ("cfg4-act-fp8", lambda: leg_cfg4(torch, _ops, args, "mxfp4", True)),
            ("cfg5-batch1", lambda: leg_cfg5(torch, args, 1)),
            ("cfg5-batch16", lambda: leg_cfg5(torch, args, 16)),
        ]
        for name, fn in todo:
            t0 = time.perf_counter()
            if t0 - t_start > 420.0:  # the whole run stays well inside ten minutes
                legs.append({"leg": name, "skipped": "time budget of the run used up"})
                continue
            try:
                leg = fn()
            except Exception as e:  # a leg that fails must not take the headline with it
                leg = {"leg": name, "error": repr(e)[:300]}
            leg["leg_wall_s"] = round(time.perf_counter() - t0, 1)
            legs.append(leg)
            torch.cuda.synchronize()
            torch.cuda.empty_cache()
        _MODEL.clear()
        # the verbose record (launch shapes, launch counts, full kernel names) goes to stderr, one line per leg; the
        # one line on stdout keeps every leg in a compact form and ends with a summary row per leg
        print("bench.py verbose: " + json.dumps({"leg": "cfg2", "roofline": out["roofline"], "config": out["config"]}),
              file=sys.stderr)
        for leg in legs:
            print("bench.py verbose: " + json.dumps(leg), file=sys.stderr)
        out["config"]["legs"] = [compact_leg(l) for l in legs]
        out["config"]["run_wall_s"] = round(time.perf_counter() - t_start, 1)
        out["config"]["gemm_kernels_columns"] = "kernel, call, kernel us, frac[, kernels per call, call us]"
        out["config"].pop("timed", None)
        out["config"]["gemm_kernels"] = compact_rows(out["roofline"].pop("all_gemm_kernels"))
        out["roofline"] = compact_roofline(out["roofline"])
        out["cpu_baseline"] = compact_cpu(out["cpu_baseline"])
        out["summary_columns"] = "leg, value, unit, ms_per_step, dominant kernel, its us, roofline frac, HBM traffic / algorithmic bytes, cpu value"
        out["summary"] = summary_of(out, legs)
    print(json.dumps(out, separators=(",", ":")))


if __name__ == "__main__":
    main()
