#!/usr/bin/env python3
"""Throughput of homura's elementwise / broadcast / reduction path on one MI355X.

A step is one pass of the hot path over one batch of BASELINE.json configs[1]: the bf16 broadcast
chain  ((x[8,2048,4096] + bias[4096]) * scale[8,2048,1]) + residual_f32[8,2048,4096]  through the
C++ host layer (type promotion, broadcasting, output allocation) and the C ABI, three kernel
launches. `value` is algorithmic bytes per step / time per step with every input resident in HBM.

The same JSON line carries
  roofline      the dominant kernel of the step (the bf16 + f32 -> f32 add), timed on its own with
                HIP events on the stream it is launched on;
  cpu_baseline  the CPU oracle (a port of homura's single-threaded CPU backend) timed on one host
                core on the same workload;
  ops           achieved GB/s and fraction of the 8 TB/s HBM peak for every op of every BASELINE
                config (--ops none to skip; cfg = index into BASELINE.json's configs); algorithmic bytes:
                every input read once and the output written once, broadcast operands at their own size.

usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--ops all|none]
"""
import argparse
import ctypes
import json
import math
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# HBM bytes per launch of the bf16 + f32 -> f32 add kernel at configs[1], from rocprofv3 --pmc FETCH_SIZE
# and --pmc WRITE_SIZE (two runs), each scaled by the reading of a plain copy of known size:
# (196 633.6 x 1.99962 = 393 193, + 262 144.0 x 1.0) KiB; profiles/map_rows_add_bf16_f32_configs1_chain.md.
ADD_KERNEL_TRAFFIC_BYTES = 671065088
TRAFFIC_SOURCE = ("profiles/map_rows_add_bf16_f32_configs1_chain.md: a constant from that profile's FETCH_SIZE / "
                  "WRITE_SIZE readings, not a reading of this run")
METRIC = "achieved HBM GB/s & % of MI355X peak per op; speedup vs host-CPU reference"


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--ops", choices=["all", "none"], default="all")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--calibrate", type=int, default=0, metavar="K",
                    help="first run K plain f32 copies of 67 108 864 elements (268 435 456 B read, the same written): "
                         "the known-size kernel that rocprofv3 FETCH_SIZE / WRITE_SIZE readings are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: this path has no cross-GPU step (every box has one GPU); got --gpus {args.gpus}",
              file=sys.stderr)
        sys.exit(2)

    import homura_amd
    from tests.support import DT, GPU, NP, from_f64, normal, tensor, uniform, words

    h = homura_amd.load_host()
    hip = ctypes.CDLL("libamdhip64.so")
    stream = ctypes.c_void_p(h.stream_handle(GPU))

    def event():
        e = ctypes.c_void_p()
        assert hip.hipEventCreate(ctypes.byref(e)) == 0
        return e

    def timed(fn, iters, warmup):
        """Average milliseconds per call of fn over `iters` calls, by HIP events on the kernels' stream."""
        for _ in range(warmup):
            fn()
        h.synchronize(GPU)
        a, b = event(), event()
        assert hip.hipEventRecord(a, stream) == 0
        for _ in range(iters):
            fn()
        assert hip.hipEventRecord(b, stream) == 0
        assert hip.hipEventSynchronize(b) == 0
        h.synchronize(GPU)
        ms = ctypes.c_float()
        assert hip.hipEventElapsedTime(ctypes.byref(ms), a, b) == 0
        hip.hipEventDestroy(a)
        hip.hipEventDestroy(b)
        return ms.value / iters

    # ---- configs[1]: the broadcast + promotion chain --------------------------------------------------
    B, S, H = 8, 2048, 4096
    N = B * S * H
    host_x = from_f64(normal(0x5EED0001, N), DT.BF16)
    host_bias = from_f64(normal(0x5EED0002, H, 0.0, 0.02), DT.BF16)
    host_scale = from_f64(uniform(0x5EED0003, B * S, 0.5, 1.5), DT.BF16)
    host_res = from_f64(normal(0x5EED0004, N), DT.F32)
    x = tensor(host_x, DT.BF16, [B, S, H], GPU)
    bias = tensor(host_bias, DT.BF16, [H], GPU)
    scale = tensor(host_scale, DT.BF16, [B, S, 1], GPU)
    residual = tensor(host_res, DT.F32, [B, S, H], GPU)

    def chain():
        return x.add(bias).mul(scale).add(residual)

    if args.calibrate:
        from homura_amd import capi

        ctx = capi.Context(0)
        src, dst = ctx.malloc(4 * N), ctx.malloc(4 * N)
        capi.check(capi.lib.hmr_memset(ctx.handle, src.ptr, 0x3C, 4 * N))
        flat = lambda buf: capi.make_desc(buf.ptr, capi.F32, [N], [1])
        d_dst, d_src = flat(dst), flat(src)
        for _ in range(args.calibrate):
            capi.check(capi.lib.hmr_copy(ctx.handle, ctypes.byref(d_dst), ctypes.byref(d_src)))
        ctx.synchronize()
        src.free()
        dst.free()
        ctx.close()

    # x + bias: 2N + 2N + the bias; t * scale: 2N + 2N + the scales; t + residual with the promotion fused: 2N + 4N + 4N.
    chain_bytes = (4 * N + 2 * H) + (4 * N + 2 * B * S) + 10 * N
    # Untimed: bring the GPU out of its idle clocks before anything is measured (a fresh process starts at
    # low clocks and the first few milliseconds of kernels run up to 15 % slow). The W warm-up steps follow.
    for _ in range(200):
        chain()
    h.synchronize(GPU)
    ms_step = timed(chain, args.steps, args.warmup)
    value = chain_bytes / (ms_step * 1e-3) / 1e9

    # The same three launches captured once into a HIP graph through the library's stream and replayed: what
    # the chain costs without the gaps between launches. Reported beside `value`, never as it: homura calls the
    # entry points one by one.
    graph_ms = None
    try:
        graph, executable = ctypes.c_void_p(), ctypes.c_void_p()
        assert hip.hipStreamBeginCapture(stream, 2) == 0  # hipStreamCaptureModeRelaxed
        try:
            g1 = x.add(bias)
            g2 = g1.mul(scale)
            g3 = g2.add(residual)
        finally:
            ended = hip.hipStreamEndCapture(stream, ctypes.byref(graph))
        assert ended == 0 and graph.value
        assert hip.hipGraphInstantiate(ctypes.byref(executable), graph, None, None, ctypes.c_size_t(0)) == 0
        graph_ms = timed(lambda: hip.hipGraphLaunch(executable, stream), args.steps, args.warmup)
        hip.hipGraphExecDestroy(executable)
        hip.hipGraphDestroy(graph)
        del g1, g2, g3
    except AssertionError:
        graph_ms = None

    # The dominant kernel: bf16 + f32 -> f32 (10 bytes per element).
    t2 = x.add(bias).mul(scale)
    ms_add = timed(lambda: t2.add(residual), max(args.steps, 20), 3)
    add_bytes = 10 * N
    achieved = add_bytes / (ms_add * 1e-3) / 1e9
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": ADD_KERNEL_TRAFFIC_BYTES,
                "traffic_source": TRAFFIC_SOURCE,
                "kernel": "map_rows_kernel<FloatBinary<ADD, f32, bf16, f32>> (bf16 + f32 -> f32)",
                "algorithmic_bytes_per_launch": add_bytes, "us_per_launch": round(ms_add * 1e3, 2)}

    # ---- every op of every config ------------------------------------------------------------------------
    ops = []
    if args.ops == "all":
        ops = per_op_table(h, timed, tensor, from_f64, normal, uniform, words, DT, GPU, NP, x, bias, scale, residual, t2)

    # Per config, the op furthest below the roofline among the rows whose inputs and results come from HBM (the
    # rows "for comparison" left out): carried inside `config`, which the driver's record keeps whole.
    per_config = {}
    for key in range(5):
        judged = [r for r in ops if r["cfg"] == key and r.get("mode") == "hbm" and "for comparison" not in r["op"]]
        if not judged:
            continue
        lowest = min(judged, key=lambda r: r["frac"])
        per_config[str(key)] = {"rows": len(judged), "lowest_frac": lowest["frac"], "op": lowest["op"].split(" [")[0],
                                "us": lowest["us"], "highest_frac": max(r["frac"] for r in judged)}
    cold = next((r for r in ops if r["cfg"] == 1 and r.get("mode") == "hbm" and "residual" in r["op"]), None)
    if cold is not None:
        roofline["frac_from_cold_hbm"] = cold["frac"]
        roofline["us_from_cold_hbm"] = cold["us"]

    # ---- CPU baseline: the oracle on one host core, same workload ------------------------------------------
    cpu = None
    if not args.no_cpu:
        from tests import oracle

        h.register_cpu_backend(oracle.backend_address())
        cx = tensor(host_x, DT.BF16, [B, S, H])
        cb = tensor(host_bias, DT.BF16, [H])
        cs = tensor(host_scale, DT.BF16, [B, S, 1])
        cr = tensor(host_res, DT.F32, [B, S, H])
        dt = None
        for _ in range(5):  # the first pass also pages the buffers in; the best of five is reported
            t0 = time.perf_counter()
            cx.add(cb).mul(cs).add(cr)
            took = time.perf_counter() - t0
            dt = took if dt is None else min(dt, took)
        # The CPU path follows the reference: the bf16 intermediate is cast to f32 by a separate copy.
        cpu = {"value": round(chain_bytes / dt / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
               "host_cores_available": os.cpu_count(),
               "sample": "the whole of configs[1] (67 108 864 elements per op), best of five passes, C++ port of "
                         "homura's single-threaded CPU backend, g++ -O2 -ffp-contract=off",
               "seconds": round(dt, 3), "gpu_speedup": round(value / (chain_bytes / dt / 1e9), 1)}

    line = {
        "metric": METRIC, "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "configs[1]: ((x_bf16[8,2048,4096] + bias_bf16[4096]) * scale_bf16[8,2048,1]) + "
                               "residual_f32[8,2048,4096] -> f32; 3 kernel launches per step",
                   "storage": "bf16 operands and intermediates, f32 residual and result; every op computes in f32",
                   "algorithmic_bytes_per_step": chain_bytes, "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4),
                   "graph_replay": None if graph_ms is None else {
                       "ms_per_step": round(graph_ms, 4), "gbs": round(chain_bytes / (graph_ms * 1e-3) / 1e9, 1),
                       "what": "the same three launches captured into one HIP graph and replayed (not `value`)"},
                   "seeds": "SplitMix64 0x5EED0001..4",
                   "per_config": per_config or None,
                   "per_config_what": "per BASELINE config, over its rows measured with inputs AND results rotating "
                                      "through HBM: the lowest fraction of the 8 TB/s peak, its op and time, and the "
                                      "highest fraction"},
        "roofline": roofline, "cpu_baseline": cpu, "ops": ops,
    }
    print(json.dumps(line))


def per_op_table(h, timed, tensor, from_f64, normal, uniform, words, DT, GPU, NP, x, bias, scale, residual, t2):
    """[{cfg, op, mode, bytes, us, gbs, frac}] for the ops of BASELINE.json configs[0..4] (cfg = index) and for the
    callers built next to the path (cfg null).

    mode "hbm": several sets of inputs AND as many result slots in rotation, sized so that the results in rotation
    and the inputs in rotation each exceed the 256 MB memory-side cache: every byte a call reads comes from HBM and
    every byte it writes goes there. These rows are each config's figures. mode "cache": the same buffers every
    call (the result block is the one the previous call wrote), shown beside them: what the same kernel reaches
    while the memory-side cache absorbs part of the traffic."""
    rows = []
    MALL = 256 << 20

    def clone(t):
        return h.full(t.shape, 0, t.dtype, GPU).copy_(t)

    def add(cfg, op, nbytes, fns, iters=50, mode=None):
        """fns: one callable, or several over disjoint buffers that are cycled."""
        fns = fns if isinstance(fns, list) else [fns]
        k = [0]

        def call():
            fns[k[0] % len(fns)]()
            k[0] += 1

        # The host work between two ops (generating the next inputs) lets the GPU fall back to idle clocks:
        # run the op untimed for about 30 ms first, then time `iters` launches, three times over, and keep the
        # fastest of the three averages (a row's launches share the GPU with nothing, so the slower ones measure the
        # clocks settling after the host work, not the op).
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < 0.03:
            for _ in range(10):
                call()
            h.synchronize(GPU)
        ms = min(timed(call, iters, 3) for _ in range(3))
        gbs = nbytes / (ms * 1e-3) / 1e9
        rows.append({"cfg": cfg, "op": op, "mode": mode, "bytes": nbytes, "us": round(ms * 1e3, 2), "gbs": round(gbs, 1),
                     "frac": round(gbs / HBM_PEAK_GBS, 4)})

    def hbm(cfg, op, nbytes, inputs, fn, in_bytes, out_bytes, iters=50, cache=False):
        """The op over copies of `inputs` (a tuple of tensors) in rotation, results kept in as many slots; as many
        sets as it takes for the inputs and the results in rotation to exceed the memory-side cache 1.25 times
        each (at least three)."""
        need = lambda b: -(-(MALL * 5 // 4) // b) if b >= (1 << 20) else 0
        sets = max(3, need(in_bytes), need(out_bytes))
        copies = [inputs] + [tuple(clone(t) for t in inputs) for _ in range(sets - 1)]
        kept = [None] * sets
        add(cfg, f"{op} [{sets} input sets and {sets} results in rotation]", nbytes,
            [lambda i=i: kept.__setitem__(i, fn(*copies[i])) for i in range(sets)], iters, "hbm")
        del kept
        if cache:
            add(cfg, f"{op} [same buffers]", nbytes, lambda: fn(*inputs), iters, "cache")

    def copy_row(cfg, op, nbytes, source, view_of):
        """One hmr_copy per call, from three sources into three destinations in rotation."""
        sources = [source, clone(source), clone(source)]
        targets = [h.full(view_of(t).shape, 0, t.dtype, GPU) for t in sources]
        add(cfg, f"{op} [3 sources and 3 destinations in rotation]", nbytes,
            [lambda i=i: targets[i].copy_(view_of(sources[i])) for i in range(3)], 50, "hbm")

    N = x.num_elements()
    # configs[0]: f32 add [4096, 4096].
    n1 = 4096 * 4096
    a0 = tensor(uniform(0x5EED0100, n1, -1.0, 1.0).astype(np.float32), DT.F32, [4096, 4096], GPU)
    b0 = tensor(uniform(0x5EED0101, n1, -1.0, 1.0).astype(np.float32), DT.F32, [4096, 4096], GPU)
    hbm(0, "add f32 [4096,4096]", 12 * n1, (a0, b0), lambda a, b: a.add(b), 8 * n1, 4 * n1, 40, cache=True)
    del a0, b0
    # configs[1]: the three steps.
    hbm(1, "x_bf16 + bias_bf16[4096] (inner broadcast)", 4 * N + 2 * 4096, (x,), lambda t: t.add(bias), 2 * N, 2 * N, cache=True)
    hbm(1, "t_bf16 * scale_bf16[8,2048,1] (row broadcast)", 4 * N + 2 * 8 * 2048, (x,), lambda t: t.mul(scale), 2 * N, 2 * N, cache=True)
    hbm(1, "t_bf16 + residual_f32 -> f32 (promotion fused)", 10 * N, (t2, residual), lambda t, r: t.add(r), 6 * N, 4 * N, 30, cache=True)
    # The plain copy of the same bytes under the same rotation: what a 134 MB -> 134 MB stream reaches on this part.
    copy_row(1, "hmr_copy bf16 [8,2048,4096] (for comparison: the same bytes as x + bias, no arithmetic)", 4 * N, x, lambda t: t)
    h.set_fused_promotion(False)
    add(1, "t_bf16 + residual_f32 -> f32 (reference style: cast kernel + add, 2 launches) [same buffers]", 18 * N,
        lambda: t2.add(residual), 30, "cache")
    h.set_fused_promotion(True)
    # configs[2]: reductions of f32 [16384, 4096] and of its bf16 copy.
    R, C = 16384, 4096
    xf = residual.reshape([R, C])
    for name, nbytes, fn in (
            ("sum dim=-1 f32", 4 * N + 4 * R, lambda t: t.sum_dim(-1, False)),
            ("mean dim=-1 f32", 4 * N + 4 * R, lambda t: t.mean_dim(-1, False)),
            ("amax dim=-1 f32 (max_dim: values + i64 indices)", 4 * N + 12 * R, lambda t: t.max_dim(-1, False)),
            ("var(unbiased) dim=-1 f32", 4 * N + 4 * R, lambda t: t.var_dim(-1, 1, False)),
            ("sum dim=0 f32", 4 * N + 4 * C, lambda t: t.sum_dim(0, False)),
            ("mean dim=0 f32", 4 * N + 4 * C, lambda t: t.mean_dim(0, False)),
            ("amax dim=0 f32 (max_dim: values + i64 indices)", 4 * N + 12 * C, lambda t: t.max_dim(0, False)),
            ("var(unbiased) dim=0 f32", 4 * N + 4 * C, lambda t: t.var_dim(0, 1, False)),
            ("sum over all elements f32", 4 * N + 4, lambda t: t.sum())):
        hbm(2, name, nbytes, (xf,), fn, 4 * N, 0, 40)
    xb = xf.to(DT.BF16)
    hbm(2, "sum dim=-1 bf16", 2 * N + 2 * R, (xb,), lambda t: t.sum_dim(-1, False), 2 * N, 0, 40)
    del xb
    # configs[3]: permuted bf16 unary; int64 tensors.
    p = tensor(from_f64(normal(0x5EED0400, N, 0.0, 2.0), DT.BF16), DT.BF16, [8, 2048, 32, 128], GPU)
    view = lambda t: t.permute([0, 2, 1, 3])
    hbm(3, "silu bf16 [8,2048,32,128].permute(0,2,1,3) -> contiguous", 4 * N, (p,), lambda t: view(t).silu(), 2 * N, 2 * N, cache=True)
    hbm(3, "gelu(erf) bf16, same view", 4 * N, (p,), lambda t: view(t).gelu(), 2 * N, 2 * N, cache=True)
    copy_row(3, "hmr_copy bf16 of the same view -> contiguous (for comparison: the same bytes, no lookup)", 4 * N, p, view)
    hbm(3, "silu bf16 on a contiguous tensor of the same size (for comparison)", 4 * N, (p,), lambda t: t.silu(), 2 * N, 2 * N)
    del p
    w1 = words(0x5EED0401, N)
    w2 = words(0x5EED0402, N)
    ia = tensor(((w1 % np.uint64(2001)).astype(np.int64) - 1000), DT.I64, [8, 2048, 4096], GPU)
    ib = tensor(((w2 % np.uint64(2001)).astype(np.int64) - 1000), DT.I64, [8, 2048, 4096], GPU)
    del w1, w2
    hbm(3, "bitwise_and i64", 24 * N, (ia, ib), lambda a, b: a.bitwise_and(b), 16 * N, 8 * N, 20)
    hbm(3, "greater i64 -> bool", 17 * N, (ia, ib), lambda a, b: a.greater(b), 16 * N, N, 20)
    mask = ia.greater(ib)
    hbm(3, "where(mask, a, b) i64", 25 * N, (mask, ia, ib), lambda m, a, b: h.where_(m, a, b), 17 * N, 8 * N, 20)
    del ia, ib, mask
    # configs[4] case 1: bf16 logits [4096, 32000].
    n5a = 4096 * 32000
    logits = tensor(from_f64(normal(0x5EED0500, n5a, 0.0, 3.0), DT.BF16), DT.BF16, [4096, 32000], GPU)
    hbm(4, "softmax bf16 [4096,32000]", 4 * n5a, (logits,), lambda t: t.softmax(-1), 2 * n5a, 2 * n5a, 30)
    hbm(4, "log_softmax bf16 [4096,32000]", 4 * n5a, (logits,), lambda t: t.log_softmax(-1), 2 * n5a, 2 * n5a, 30)
    del logits
    # configs[4] case 2: causal f32 scores [32, 2048, 2048].
    n5b = 32 * 2048 * 2048
    s = normal(0x5EED0501, n5b).astype(np.float32).reshape(32, 2048, 2048)
    s[:, np.triu_indices(2048, 1)[0], np.triu_indices(2048, 1)[1]] = -np.inf
    scores = tensor(s, DT.F32, [32, 2048, 2048], GPU)
    del s
    hbm(4, "softmax f32 [32,2048,2048] causal", 8 * n5b, (scores,), lambda t: t.softmax(-1), 4 * n5b, 4 * n5b, 20)
    hbm(4, "log_softmax f32 [32,2048,2048] causal", 8 * n5b, (scores,), lambda t: t.log_softmax(-1), 4 * n5b, 4 * n5b, 20)
    # The callers next to the path (cfg null: not a BASELINE config): the optimizers' single-rounding steps on
    # 67 108 864 parameters, a whole SGD / Adam update (bytes = the sum over its kernels), triangles of the causal
    # scores and flips.
    del scores
    for dt, name, size in ((DT.F32, "f32", 4), (DT.BF16, "bf16", 2)):
        prm = x.to(dt) if dt != DT.BF16 else x
        grd = residual.to(dt) if dt != DT.F32 else residual
        third = prm.mul(0.5).add(1.5)
        add(None, f"scaled_add {name} (p + alpha * g)", 3 * size * N, lambda: h.scaled_add(prm, grd, -0.01))
        add(None, f"lerp step {name}", 3 * size * N, lambda: h.lerp_step(prm, grd, 0.1))
        add(None, f"addcmul step {name}", 4 * size * N, lambda: h.addcmul_step(prm, grd, third, 0.001))
        add(None, f"addcdiv step {name}", 4 * size * N, lambda: h.addcdiv_step(prm, grd, third, -0.01))
        buf = grd.mul(0.5)
        add(None, f"sgd step {name}, momentum 0.9 (3 kernels: mul, 2 scaled_add)", 8 * size * N,
            lambda: h.sgd_step(prm, grd, buf, lr=0.01, momentum=0.9))
        state = h.adam_step(prm, grd, None, lr=1e-3)[1]
        add(None, f"adam step {name} (7 kernels: lerp, mul, addcmul, sqrt, div, add, addcdiv)", 19 * size * N,
            lambda: h.adam_step(prm, grd, state, lr=1e-3))
        del prm, grd, third, buf, state
    mat = residual.reshape([8192, 8192])
    v1, v2 = residual.narrow(0, 0, 1).narrow(1, 0, 2).reshape([8192]), residual.narrow(0, 1, 1).narrow(1, 0, 2).reshape([8192])
    add(None, "addr f32 [8192,8192] (beta 0.5, alpha -1.5: one kernel)", 8 * N + 8 * 8192, lambda: mat.addr(v1, v2, 0.5, -1.5))
    add(None, "addr f32 [8192,8192] without input (beta 0)", 4 * N + 8 * 8192, lambda: mat.addr(v1, v2, 0, -1.5))
    del mat, v1, v2
    xf = residual.reshape([16384, 4096])
    add(None, "exclusive_cumprod f32 [16384,4096] dim=0 (slabs through LDS, a sequential chain per column)", 8 * N,
        lambda: h.exclusive_cumprod(xf, 0, False), 5)
    add(None, "exclusive_cumprod f32 [16384,4096] dim=1 (slabs through LDS, a sequential chain per row)", 8 * N,
        lambda: h.exclusive_cumprod(xf, 1, True), 5)
    del xf
    # Softmax plans beyond rows that fit a workgroup's registers, and reductions over two dimensions (inputs and
    # results in rotation, as for the configs' rows).
    cols32 = residual.reshape([4096, 16384])
    hbm(None, "softmax(dim=0) f32 [4096,16384] (rows across memory: running maxima, two passes)", 8 * N, (cols32,),
        lambda t: t.softmax(0), 4 * N, 4 * N, 10)
    hbm(None, "log_softmax(dim=0) f32 [4096,16384]", 8 * N, (cols32,), lambda t: t.log_softmax(0), 4 * N, 4 * N, 10)
    del cols32
    cols16 = h.full([4, 8, 2048, 4096], 0, DT.BF16, GPU).copy_(x.reshape([1, 8, 2048, 4096]).expand([4, 8, 2048, 4096])).reshape([64, 1024, 4096])
    hbm(None, "softmax(dim=1) bf16 [64,1024,4096] (rows across memory, read once into registers)", 16 * N, (cols16,),
        lambda t: t.softmax(1), 8 * N, 8 * N, 5)
    del cols16
    long_rows = residual.narrow(0, 0, 4).reshape([8, 4194304])
    hbm(None, "softmax(dim=1) f32 [8,4194304] (rows cut across workgroups: two launches)", 4 * N, (long_rows,),
        lambda t: t.softmax(1), 2 * N, 2 * N, 20)
    del long_rows
    stats = residual.reshape([64, 256, 4096])
    hbm(None, "sum over (0,2) f32 [64,256,4096] (rows made of runs)", 4 * N, (stats,), lambda t: t.sum_dim([0, 2], False), 4 * N, 0, 30)
    hbm(None, "var(unbiased) over (0,2) f32 [64,256,4096]", 4 * N, (stats,), lambda t: t.var_dim([0, 2], 1, False), 4 * N, 0, 30)
    del stats
    turned = residual.reshape([16384, 4096])
    hbm(None, "sum of all elements of a transposed view f32 [16384,4096].T", 4 * N, (turned,), lambda t: t.transpose(0, 1).sum(), 4 * N, 0, 30)
    del turned
    y = x.reshape([16384, 4096]).softmax(-1)
    gy = t2.reshape([16384, 4096])
    add(None, "softmax backward bf16 [16384,4096] (7 kernels: 2 casts, mul, sum, sub, mul, cast)", 2 * N * (3 + 3 + 6 + 2 + 4 + 6 + 3),
        lambda: h.grad_softmax(gy, y, -1, False), 10)
    del y, gy
    # Indexing: an embedding lookup and its gradient (vocabulary 32 768 x 4096 bf16, 16 384 tokens), gather and
    # scatter_add along the rows of the f32 matrix. Bytes: rows moved + indices (+ the target's read and write).
    vocab, hidden, tokens = 32768, 4096, 16384
    table = x.reshape([16384, 4096]).narrow(0, 0, 1).expand([2, 16384, 4096]).reshape([vocab, hidden]).contiguous()
    ids = tensor((words(0x5EED0600, tokens) % np.uint64(vocab)).astype(np.int64), DT.I64, [tokens], GPU)
    add(None, "index_select bf16 [32768,4096] rows by 16384 ids (embedding lookup)", 4 * tokens * hidden + 8 * tokens,
        lambda: table.index_select(0, ids), 10)
    grads = x.reshape([16384, 4096])
    zeros = h.full([vocab, hidden], 0.0, DT.BF16, GPU)
    add(None, "index_add bf16 16384 rows into [32768,4096] (embedding gradient: copy, check, sort, ordered sums)",
        4 * vocab * hidden + 2 * tokens * hidden + 4 * tokens * hidden, lambda: zeros.index_add(0, ids, grads), 5)
    # Advanced indexing: the same rows through an index tensor (check, rows of tiles) and written back
    # (copy of the table, winners per row, the winners' rows).
    add(None, "x[ids] bf16 [32768,4096] by 16384 ids (advanced indexing: check, rows)",
        4 * tokens * hidden + 16 * tokens, lambda: table.index_tensors([ids]), 10)
    add(None, "index_put bf16 16384 rows into [32768,4096] (copy, check, positions, last write wins)",
        4 * vocab * hidden + 4 * tokens * hidden + 24 * tokens, lambda: table.index_put_tensors([ids], grads, False), 5)
    del table, grads, zeros
    mat = residual.reshape([16384, 4096])
    cols = tensor((words(0x5EED0601, 16384 * 512) % np.uint64(4096)).astype(np.int32), DT.I32, [16384, 512], GPU)
    add(None, "gather f32 [16384,4096] dim 1 by i32 [16384,512]", (4 + 4 + 4) * 16384 * 512, lambda: mat.gather(1, cols), 10)
    vals = mat.narrow(1, 0, 512)
    add(None, "scatter_add f32 [16384,512] into [16384,4096] dim 1 (copy, check, ordered sums line by line in LDS)",
        8 * N + (4 + 4 + 8) * 16384 * 512, lambda: mat.scatter_add(1, cols, vals), 3)
    # A boolean mask over the f32 matrix, 60 % true: the coordinates (count, scan, write; two i64 per true element),
    # then the selected elements (the mask is the only index: one i64 position per true element, one element per pick).
    keep = tensor((words(0x5EED0602, N) % np.uint64(5) < 3).astype(np.uint8), DT.Bool, [16384, 4096], GPU)
    kept = int((words(0x5EED0602, N) % np.uint64(5) < 3).sum())
    add(None, "mask coordinates bool [16384,4096], 60 % true (count, scan, coordinates)", 2 * N + 16 * kept,
        lambda: keep.mask_coordinates(), 5)
    add(None, "x[mask] f32 [16384,4096], 60 % true (count, scan, positions in the flattened mask, picks)", 2 * N + 24 * kept,
        lambda: mat.index_tensors([keep]), 3)
    seven = tensor(np.array([7.0], dtype=np.float32), DT.F32, [], GPU)
    add(None, "x[mask] = v f32 [16384,4096], one value (one select between the value and x)", 9 * N,
        lambda: mat.index_put_tensors([keep], seven, False), 5)
    del mat, cols, vals, keep, seven
    shape = [8, 2048, 4096]
    add(None, "rand f32 [8,2048,4096] (Philox on the device, write only)", 4 * N, lambda: h.rand(shape, DT.F32, GPU))
    add(None, "rand bf16 [8,2048,4096]", 2 * N, lambda: h.rand(shape, DT.BF16, GPU))
    add(None, "randn f32 [8,2048,4096] (Box-Muller, f64 polynomials)", 4 * N, lambda: h.randn(shape, DT.F32, GPU), 10)
    add(None, "randint [0, 1024) i64 [8,2048,4096] (no rejection)", 8 * N, lambda: h.randint(0, 1024, shape, DT.I64, GPU), 10)
    add(None, "randint [-5, 6) i64 [8,2048,4096] (rejection: count + write as if none, scan, rewrite only if any + a read-back)", 8 * N,
        lambda: h.randint(-5, 6, shape, DT.I64, GPU), 5)
    # General layouts: transposed and permuted views made contiguous or combined with a contiguous operand (a tile
    # of the two dimensions goes through LDS), and every other column (one element per lane).
    sqm = residual.reshape([8192, 8192])
    sqt = sqm.transpose(0, 1)
    add(None, "transpose f32 [8192,8192] -> contiguous (tiles through LDS, 16-byte accesses)", 8 * N, lambda: sqt.contiguous(), 10)
    add(None, "transposed + contiguous f32 [8192,8192] (tiles through LDS, 16-byte accesses)", 12 * N, lambda: sqt.add(sqm), 10)
    sqb = x.reshape([8192, 8192]).transpose(0, 1)
    add(None, "transpose bf16 [8192,8192] -> contiguous (tiles through LDS, 16-byte accesses)", 4 * N, lambda: sqb.contiguous(), 10)
    cube = residual.reshape([64, 1024, 1024]).permute([2, 0, 1])
    add(None, "permute(2,0,1) f32 [64,1024,1024] -> contiguous (tiles through LDS, 16-byte accesses)", 8 * N, lambda: cube.contiguous(), 10)
    halfcols = sqm.slice(1, 0, 8192, 2)
    add(None, "every other column f32 [8192,4096] -> contiguous (general kernel, four elements per lane in flight)", 4 * N,
        lambda: halfcols.contiguous(), 10)
    del sqm, sqt, sqb, cube, halfcols
    sq = residual.reshape([16, 2048, 2048])
    add(None, "triu(1) f32 [16,2048,2048] (reads the kept half)", 6 * N, lambda: sq.triu(1))
    add(None, "tril(0) f32 [16,2048,2048] (reads the kept half)", 6 * N, lambda: sq.tril(0))
    add(None, "flip f32 [8,2048,4096] dims [1] (rows reversed)", 8 * N, lambda: residual.flip([1]))
    add(None, "flip f32 [8,2048,4096] dims [2] (elements of a row reversed)", 8 * N, lambda: residual.flip([2]))
    return rows


if __name__ == "__main__":
    main()
