"""Benchmark of the SC-MXFP4 W4A8 hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--reps R]

One step = one pass of the dense W4A8 linear (activation-quantization prologue + fused-unpack INT8-MFMA GEMM + bf16
epilogue, through the C ABI entry scmx_linear_w4a8) over the four Qwen3-1.7B-shaped layers at M = 2048 tokens
(BASELINE config 1): qkv 4096x2048, o_proj 2048x2048, gate_up 12288x2048, down 2048x6144.  Inputs are seeded
synthetic tensors already resident in HBM; weight sets rotate so that consecutive steps do not reuse cached weights.
`value` is INT8 TOPS = 2*M*N*K summed over the layers / time.

Timing protocol (the reference's, kernels/bench.swift:111-119 and e2e/bench_fused.py:71-91): every figure is taken
after a warm-up of W steps and at least half a second of the same work, over R repetitions of K back-to-back steps,
each repetition bracketed by events on the launch stream; the MEDIAN repetition is reported, the fastest one beside
it.  The same run also reports the GEMM kernel alone (roofline), the step without its prologues, the decode GEMV's
achieved HBM GB/s (config 2), the grouped expert passes (configs 3 and 4) and a CPU baseline (the numpy oracle on the
host cores).  Prints ONE JSON line.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_INT8_TOPS = 5000.0        # MI355X dense INT8 MFMA, published
# HBM-side bytes per GEMM launch (mean over the four layer launches of one step), from rocprofv3 TCC counters of this
# workload: FETCH_SIZE x 2.0 + WRITE_SIZE x 1.0 KiB, both factors calibrated on a 256 MiB device copy.  Per layer
# (fetched + written MiB): qkv 24.5 + 16.1, gate_up 41.6 + 48.4, o_proj and down together 80.8 + 16.
GEMM_TRAFFIC_BYTES = int((24.5 + 16.1 + 41.6 + 48.4 + 80.8 + 16) * 2 ** 20 / 4)
PEAK_HBM_GBPS = 8000.0         # MI355X HBM3E, published
M_TOKENS = 2048
LAYERS = [("qkv", 4096, 2048), ("o_proj", 2048, 2048), ("gate_up", 12288, 2048), ("down", 2048, 6144)]
DECODE = LAYERS + [("lm_head", 151936, 2048)]


def packed_random(rng, n, k):
    """Random SC-MXFP4 codes: statistically the quantized N(0, 0.02) matrix's storage (all 16 codes and 4 shifts occur);
    throughput does not depend on the values."""
    codes = rng.integers(0, 2 ** 32, n * k // 8, dtype=np.uint64).astype(np.uint32)
    bc = rng.integers(0, 256, (n, k // 128), dtype=np.uint16).astype(np.uint8)
    ws = np.exp2(rng.integers(-12, -6, n)).astype(np.float32)
    return codes, bc, ws


def acts(rng, m, k):
    x = rng.standard_normal((m, k)).astype(np.float32)
    x[:, rng.choice(k, max(1, round(0.01 * k)), replace=False)] *= 20
    return x


WARM_SCALE = 1.0   # --warm-seconds / 0.5: profiler runs set it to 0 so that counter passes see few dispatches


def timed(torch, stream, fn, steps, reps=10, warmup=0, warm_s=0.5):
    """fn(i) enqueues one step.  Warm up (`warmup` steps, then until `warm_s` seconds have passed), then time `reps`
    repetitions of `steps` back-to-back steps, each between two events on `stream`.  Returns (median, min) ms per step."""
    i = 0
    for _ in range(warmup):
        fn(i)
        i += 1
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < warm_s * WARM_SCALE:
        for _ in range(max(1, min(steps, 16))):
            fn(i)
            i += 1
        torch.cuda.synchronize()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(reps + 1)]
    ev[0].record(stream)
    for r in range(reps):
        for _ in range(steps):
            fn(i)
            i += 1
        ev[r + 1].record(stream)
    torch.cuda.synchronize()
    per = sorted(ev[r].elapsed_time(ev[r + 1]) / steps for r in range(reps))
    return (per[reps // 2] if reps % 2 else 0.5 * (per[reps // 2 - 1] + per[reps // 2])), per[0]


def cpu_baseline(budget_s=12.0):
    """The oracle's path (numpy): per-token INT8 quantization, float64-BLAS integer GEMM, FP32 scaling, bf16 rounding,
    for the four layers at M = 2048 with pre-decoded INT8 weights; repeated until the time budget is used."""
    from oracle import bf16, linear
    rng = np.random.default_rng(1)
    work = []
    for _, n, k in LAYERS:
        wq = rng.integers(-96, 97, (n, k)).astype(np.int8)
        ws = np.exp2(rng.integers(-12, -6, n)).astype(np.float32)
        work.append((bf16.rnd(acts(rng, M_TOKENS, k)), wq, ws))
    ops = sum(2.0 * M_TOKENS * n * k for _, n, k in LAYERS)
    reps, t0 = 0, time.perf_counter()
    while True:
        for x, wq, ws in work:
            xq, xs = linear.act_quant(x)
            linear.epilogue(linear.int_gemm(xq, wq), xs, ws, 1)
        reps += 1
        el = time.perf_counter() - t0
        if el > budget_s or reps >= 50:
            break
    try:
        from threadpoolctl import threadpool_info
        threads = max([p.get("num_threads", 1) for p in threadpool_info()] + [1])
    except Exception:
        threads = os.cpu_count()
    return {"value": round(ops * reps / el / 1e12, 4), "unit": "TOPS", "cores": int(threads), "kind": "port",
            "sample": f"{reps} pass(es) of the 4 layers at M={M_TOKENS} (act quant + float64 BLAS integer GEMM + bf16 "
                      f"epilogue, INT8 weights pre-decoded), {el:.1f} s"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--reps", type=int, default=10, help="timed repetitions of --steps steps (median reported)")
    ap.add_argument("--warm-seconds", type=float, default=0.5,
                    help="time-based warm-up of the headline leg (the other legs scale with it); 0 under a profiler")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-decode", action="store_true", help="skip the decode GEMV leg")
    ap.add_argument("--no-moe", action="store_true", help="skip the grouped mixture-of-experts leg")
    ap.add_argument("--no-sweep", action="store_true", help="skip the M = 512 / 8192 prefill sweep")
    ap.add_argument("--no-quant", action="store_true", help="skip the device quantizer leg")
    ap.add_argument("--no-model", action="store_true", help="skip the whole-model prefill / decode leg")
    ap.add_argument("--profile-copy", action="store_true",
                    help="first run one plain 256 MiB device copy: the known-size kernel that calibrates FETCH_SIZE / "
                         "WRITE_SIZE when this command runs under rocprofv3 --pmc")
    a = ap.parse_args()
    if a.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this path runs on ONE GPU (no sharding, no collectives); --gpus must be 1", file=sys.stderr)
        sys.exit(2)

    global WARM_SCALE
    WARM_SCALE = max(0.0, a.warm_seconds) / 0.5
    import torch
    import mxfp4_int8_m5_amd as pkg
    lib = pkg._lib.load()
    fmt = pkg.sc_format.DEFAULT.c_struct()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    stream = torch.cuda.current_stream()
    sp = C.c_void_p(stream.cuda_stream)
    rng = np.random.default_rng(1)

    def up(arr):
        arr = np.ascontiguousarray(arr)
        if arr.dtype == np.uint32:
            arr = arr.view(np.int32)
        return torch.from_numpy(arr).to(dev)

    if a.profile_copy:
        src = torch.empty(256 * 2 ** 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ---- prefill: weight sets rotate (> 256 MB in total, beyond the last-level cache) --------------------------
    set_bytes = sum(n * k // 2 + n * k // 128 + 4 * n for _, n, k in LAYERS)
    n_sets = max(2, -(-300 * 2 ** 20 // set_bytes))
    sets = []
    for _ in range(n_sets):
        sets.append([tuple(up(t) for t in packed_random(rng, n, k)) for _, n, k in LAYERS])
    xs_in = {k: up(acts(rng, M_TOKENS, k)).to(torch.bfloat16) for k in sorted({k for _, _, k in LAYERS})}
    outs = [torch.empty((M_TOKENS, n), dtype=torch.bfloat16, device=dev) for _, n, _ in LAYERS]
    ws_bytes = max(lib.scmx_linear_w4a8_workspace(M_TOKENS, k) for _, _, k in LAYERS)
    workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)

    def check(rc):
        if rc != 0:
            raise RuntimeError(lib.scmx_last_error().decode())

    calls = []
    for s in sets:
        step = []
        for (name, n, k), (codes, bc, ws), out in zip(LAYERS, s, outs):
            step.append((C.byref(fmt), xs_in[k].data_ptr(), codes.data_ptr(), bc.data_ptr(), ws.data_ptr(), None,
                         out.data_ptr(), 1, M_TOKENS, n, k, workspace.data_ptr(), ws_bytes, sp))
        calls.append(step)

    def run_step(i):
        for args in calls[i % n_sets]:
            check(lib.scmx_linear_w4a8(*args))

    timeit = lambda fn, steps, **kw: timed(torch, stream, fn, steps, **kw)   # noqa: E731
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)   # for the short side legs
    ms_step, ms_step_min = timeit(run_step, a.steps, reps=a.reps, warmup=a.warmup)
    ops_step = sum(2.0 * M_TOKENS * n * k for _, n, k in LAYERS)
    tops = ops_step / (ms_step * 1e-3) / 1e12

    # the same step without its prologues (activations quantized beforehand), and the prologues alone: where the
    # difference between `value` and the GEMM kernel's rate goes
    # (in the layout the fused layer quantizes into for the shape: by rows, or in 32x32 blocks for the large tiles)
    def quantized(x, m, n, k):
        blocked = bool(lib.scmx_mm_w4a8_prefers_blocked(m, n, k))
        mp = (m + 31) // 32 * 32
        xq = torch.empty(mp * k, dtype=torch.int8, device=dev)
        xs = torch.empty(mp, dtype=torch.float32, device=dev)
        quant = lib.scmx_act_quant_blocked if blocked else lib.scmx_act_quant
        qargs = (x.data_ptr(), xq.data_ptr(), xs.data_ptr(), m, mp if blocked else m, k, sp)
        check(quant(*qargs))
        return xq, xs, (lib.scmx_mm_w4a8_blocked if blocked else lib.scmx_mm_w4a8), quant, qargs, blocked

    pre = [quantized(xs_in[k], M_TOKENS, n, k) for _, n, k in LAYERS]
    gcalls = [[(pre[li][2], (C.byref(fmt), pre[li][0].data_ptr(), pre[li][1].data_ptr(), codes.data_ptr(), bc.data_ptr(),
                             ws.data_ptr(), None, out.data_ptr(), 1, M_TOKENS, n, k, sp))
               for li, ((name, n, k), (codes, bc, ws), out) in enumerate(zip(LAYERS, st, outs))] for st in sets]

    def run_gemms(i):
        for mm, args in gcalls[i % n_sets]:
            check(mm(*args))

    def run_prologues(i):
        for _, _, _, quant, qargs, _ in pre:
            check(quant(*qargs))
    ms_gemms, _ = timeit(run_gemms, a.steps, reps=a.reps, warm_s=0.3)
    ms_pro, _ = timeit(run_prologues, a.steps, reps=a.reps, warm_s=0.2)
    step_parts = {"step_ms": round(ms_step, 4), "step_ms_min": round(ms_step_min, 4),
                  "gemms_only_ms": round(ms_gemms, 4), "gemms_only_tops": round(ops_step / ms_gemms / 1e9, 1),
                  "prologues_only_ms": round(ms_pro, 4),
                  "value_over_gemms_only": round(ms_gemms / ms_step, 3),
                  "activation_layout": {name: "blocked" if p[5] else "rows" for (name, _, _), p in zip(LAYERS, pre)},
                  "note": "4 layers per step; gemms_only = the four GEMM launches of the step back to back on pre-quantized "
                          "activations (scmx_mm_w4a8_blocked where the fused layer quantizes into 32x32 blocks, else "
                          "scmx_mm_w4a8); prologues_only = its four activation-quantization launches"}

    # ---- roofline of the dominant kernel (the fused-unpack GEMM alone, activations pre-quantized) -------------------
    per_shape = {}
    tot_ops = tot_ms = 0.0
    for li, (name, n, k) in enumerate(LAYERS):
        argl = [g[li] for g in gcalls]
        ms, ms_min = timeit(lambda i: check(argl[i % n_sets][0](*argl[i % n_sets][1])), max(20, a.steps), reps=a.reps, warm_s=0.5)
        ops = 2.0 * M_TOKENS * n * k
        per_shape[name] = {"us": round(ms * 1e3, 2), "us_min": round(ms_min * 1e3, 2), "tops": round(ops / ms / 1e9, 1),
                           "pct_peak": round(ops / ms / 1e9 / PEAK_INT8_TOPS * 100, 2)}
        if pre[li][5] and not a.no_sweep:   # the same GEMM on activations quantized by rows, for comparison
            rq = torch.empty(M_TOKENS * k, dtype=torch.int8, device=dev)
            check(lib.scmx_act_quant(xs_in[k].data_ptr(), rq.data_ptr(), pre[li][1].data_ptr(), M_TOKENS, M_TOKENS, k, sp))
            rargs = [(ar[0], rq.data_ptr()) + ar[2:] for _, ar in argl]
            ms_r, _ = timeit(lambda i: check(lib.scmx_mm_w4a8(*rargs[i % n_sets])), 20, reps=5, warm_s=0.2)
            per_shape[name]["us_row_layout"] = round(ms_r * 1e3, 2)
            del rq
        tot_ops += ops
        tot_ms += ms
    achieved = tot_ops / tot_ms / 1e9
    roofline = {"bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_INT8_TOPS, "unit": "TFLOP/s",
                "frac": round(achieved / PEAK_INT8_TOPS, 4), "traffic": GEMM_TRAFFIC_BYTES, "kernel": "scmx::gemm_kernel (mm_w4a8 / mm_w4a8_blocked, as the fused layer launches it)",
                "note": "INT8 ops 2MNK counted as (FL)OPs; sum over the 4 layer shapes / sum of their launch durations "
                        "(median repetition of back-to-back launches between events on the launch stream), "
                        "activations pre-quantized", "per_shape": per_shape}

    # ---- the ROCm library's INT8 GEMM on the same shapes: what tuned vendor code reaches here with resident INT8 ----
    # weights, INT32 output, no unpack and no epilogue (a reference point for the fraction of peak, not a baseline)
    library = {}
    if not a.no_sweep:
        try:
            for name, n, k in LAYERS:
                xa = torch.randint(-127, 128, (M_TOKENS, k), dtype=torch.int8, device=dev)
                wb = torch.randint(-127, 128, (n, k), dtype=torch.int8, device=dev).t()
                ms, _ = timeit(lambda i: torch._int_mm(xa, wb), 20, reps=5, warm_s=0.2)
                library[name] = {"us": round(ms * 1e3, 2), "tops": round(2.0 * M_TOKENS * n * k / ms / 1e9, 1)}
                del xa, wb
            library["what"] = "torch._int_mm at M = %d: INT8 x INT8 -> INT32, weights already INT8, no epilogue" % M_TOKENS
        except Exception as exc:   # the comparison is optional: a build of torch without this op must not stop the bench
            library = {"error": str(exc)[:200]}

    # ---- prefill sweep over M (config 1's other token counts): GEMM kernel alone, per shape ---------------------------
    sweep = {}
    if not a.no_sweep:
        for m in (512, 8192):
            for li, (name, n, k) in enumerate(LAYERS):
                x = up(acts(rng, m, k)).to(torch.bfloat16)
                out = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
                xq, xs, mm, _, _, _ = quantized(x, m, n, k)
                argl = []
                for s in sets:
                    codes, bc, ws = s[li]
                    argl.append((C.byref(fmt), xq.data_ptr(), xs.data_ptr(), codes.data_ptr(), bc.data_ptr(), ws.data_ptr(),
                                 None, out.data_ptr(), 1, m, n, k, sp))
                ms, _ = timeit(lambda i: check(mm(*argl[i % n_sets])), 20, reps=a.reps, warm_s=0.3)
                ops = 2.0 * m * n * k
                sweep[f"{name}_m{m}"] = {"us": round(ms * 1e3, 2), "tops": round(ops / ms / 1e9, 1),
                                         "pct_peak": round(ops / ms / 1e9 / PEAK_INT8_TOPS * 100, 2)}
                del x, xq, xs, out

    # ---- grouped mixture-of-experts prefill (config 3: 64 experts, top-8, hidden 2048, intermediate 1024, 4096 tokens) ---
    moe = {}
    if not a.no_moe:
        from mxfp4_int8_m5_amd import sc_kernels as SK, sc_moe as SM
        T, E, TOPK, D, Fi, TM = 4096, 64, 8, 2048, 1024, int(os.environ.get('SCMX_BENCH_TM', '256'))
        R = T * TOPK
        logits = rng.standard_normal((T, E)) + rng.standard_normal(E) * 1.5      # biased router: skewed expert loads
        logits_d = up(logits.astype(np.float32)).to(torch.bfloat16)              # router logits, resident
        x = up(acts(rng, T, D)).to(torch.bfloat16)

        def experts(n, k):
            parts = [packed_random(rng, n, k) for _ in range(E)]
            return (up(np.stack([q[0] for q in parts])), up(np.stack([q[1] for q in parts])),
                    up(np.stack([q[2] for q in parts])))
        gu, dn = experts(2 * Fi, D), experts(D, Fi)       # gate|up rows interleaved for the SwiGLU epilogue

        def moe_pass():
            xq, xs = SK.act_quant(x, T)
            inds, scores = SM.route(logits_d, TOPK, renorm=True)
            pos, tok, _, off, tstart, mt = SM.route_sort(inds, E, TM)
            h = SM.moe_mm(xq, R, gu[0], gu[1], gu[2], off, tstart, mt, 2 * Fi, 3, xscale=xs, tile=(TM, 64, 4), gather=tok)
            hq, hs = SK.act_quant(h, R)
            y = SM.moe_mm(hq, R, dn[0], dn[1], dn[2], off, tstart, mt, D, 1, xscale=hs, tile=(TM, 64, 4))
            return SM.moe_combine(y, pos, scores, x, None, 0.0, T, quant=False)[0]

        ms, ms_min3 = timeit(lambda i: moe_pass(), 10, reps=a.reps, warm_s=0.3)
        tiles = int(SM.route_sort(SM.route(logits_d, TOPK)[0], E, TM)[4][-1].item())
        ops = 2.0 * R * 3 * Fi * D
        moe = {"workload": "BASELINE configs[3]: act quant + router (softmax, top-8, renormalisation) + token sort + grouped gate_up GEMM (SwiGLU epilogue) + act "
                           "quant + grouped down GEMM + weighted combine", "tokens": T, "experts": E, "topk": TOPK,
               "row_tile": TM, "row_tiles": tiles, "padded_rows_pct": round((tiles * TM / R - 1) * 100, 1),
               "ms": round(ms, 4), "ms_min": round(ms_min3, 4), "tops": round(ops / ms / 1e9, 1),
               "pct_peak": round(ops / ms / 1e9 / PEAK_INT8_TOPS * 100, 2)}
        del gu, dn, x
        torch.cuda.empty_cache()

        # ---- config 4: 256 routed experts + 1 shared (top-8 + shared = 9 slots), hidden 2048, intermediate 512, the
        # 16-element-block power-of-two format; random code words (the kernels' time does not depend on the values)
        from mxfp4_int8_m5_amd import sc_decode as SD, sc_format as SF
        f16 = SF.Format(block=16)
        T4, E4, D4, F4, TM4 = 2048, 257, 2048, 512, int(os.environ.get('SCMX_BENCH_TM4', '64'))
        R4 = T4 * 9
        gen = torch.Generator(device=dev).manual_seed(4)

        def experts16(n, k):
            return (torch.randint(-2 ** 31, 2 ** 31 - 1, (E4, n * k // 8), dtype=torch.int32, device=dev, generator=gen),
                    torch.randint(0, 256, (E4, n, k // 64), dtype=torch.uint8, device=dev, generator=gen),
                    torch.full((E4, n), 2.0 ** -9, dtype=torch.float32, device=dev))
        gu4, dn4 = experts16(2 * F4, D4), experts16(D4, F4)
        lg = rng.standard_normal((T4, E4 - 1)) + rng.standard_normal(E4 - 1) * 1.5
        lg_d = up(lg.astype(np.float32)).to(torch.bfloat16)
        sg_d = up(rng.standard_normal(T4).astype(np.float32)).to(torch.bfloat16)    # the shared expert's gate logits
        inds4 = SM.route(lg_d, 8, renorm=True, shared_logit=sg_d)[0]                 # [T4, 9]: top-8 + the shared slot
        x4 = up(acts(rng, T4, D4)).to(torch.bfloat16)

        def pass4():
            xq, xs = SK.act_quant(x4, T4)
            inds9, _ = SM.route(lg_d, 8, renorm=True, shared_logit=sg_d)
            pos, tok, _, off, tstart, mt = SM.route_sort(inds9, E4, TM4)
            h = SM.moe_mm(xq, R4, gu4[0], gu4[1], gu4[2], off, tstart, mt, 2 * F4, 3, xscale=xs, tile=(TM4, 64, 4),
                          gather=tok, fmt=f16)
            hq, hs = SK.act_quant(h, R4)
            return SM.moe_mm(hq, R4, dn4[0], dn4[1], dn4[2], off, tstart, mt, D4, 1, xscale=hs, tile=(TM4, 64, 4), fmt=f16)

        ms4, ms4_min = timeit(lambda i: pass4(), 10, reps=a.reps, warm_s=0.3)
        # batch-1 decode: the 9-slot gate|up and down GEMVs of one token, replayed from a HIP graph
        xq1, xs1 = SK.act_quant(x4[:1].contiguous(), 1)
        TOK_PER_GRAPH = 20
        eidxs = [inds4[(97 * t) % T4, :8].contiguous() for t in range(TOK_PER_GRAPH)]   # every token its own routed experts

        def token4(eidx):
            a1 = SD.gemv(xq1, gu4[0], gu4[1], xs1, gu4[2], 2 * F4, 3, eidx=eidx, xstride=0, shared=E4 - 1, fmt=f16)
            return SD.gemv(a1, dn4[0], dn4[1], None, dn4[2], D4, 1, eidx=eidx, xstride=1, pro=1, shared=E4 - 1, fmt=f16)
        side = torch.cuda.Stream()
        side.wait_stream(stream)
        with torch.cuda.stream(side):
            token4(eidxs[0])
        stream.wait_stream(side)
        # 20 tokens' GEMV pairs per graph (the dense decode legs put as many calls in theirs): the figure is kernel time and
        # the gaps between dependent kernels, not the cost of launching a two-kernel graph
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for t in range(TOK_PER_GRAPH):
                token4(eidxs[t])
        for _ in range(3):
            graph.replay()
        torch.cuda.synchronize()
        e0.record(stream)
        for _ in range(10):
            graph.replay()
        e1.record(stream)
        torch.cuda.synchronize()
        us_tok = e0.elapsed_time(e1) / (10 * TOK_PER_GRAPH) * 1e3
        bytes_tok = 9 * 3 * F4 * D4 * (0.5 + 1.0 / 64)
        ops4 = 2.0 * R4 * 3 * F4 * D4
        # config 4's prefill streams every expert's weights once for ~72 rows each: 278 op/B, below the ~630 op/B ridge,
        # so its roof is HBM: packed expert weights + bf16 tokens in + bf16 rows out
        bytes4 = E4 * 3 * F4 * D4 * (0.5 + 1.0 / 64) + 2.0 * T4 * D4 + 2.0 * R4 * D4
        moe["config4"] = {"workload": "BASELINE configs[4]: 257 experts (256 routed + shared), 9 slots per token, 16-block "
                                      "format; prefill of 2048 tokens (act quant, router with the shared slot, sort, two grouped GEMMs, act quant) and "
                                      "the two 9-slot GEMVs of a decode token (20 tokens with their own routed experts per replayed graph)",
                          "prefill_ms": round(ms4, 4), "prefill_ms_min": round(ms4_min, 4),
                          "prefill_tops": round(ops4 / ms4 / 1e9, 1), "prefill_bound": "hbm",
                          "prefill_gbps": round(bytes4 / ms4 / 1e6, 1),
                          "prefill_pct_hbm": round(bytes4 / ms4 / 1e6 / PEAK_HBM_GBPS * 100, 1), "row_tile": TM4,
                          "decode_us_per_token": round(us_tok, 2), "decode_gbps": round(bytes_tok / us_tok / 1e3, 1)}
        del gu4, dn4, graph
        torch.cuda.empty_cache()

    # ---- decode GEMV: achieved HBM GB/s, weights rotating beyond the cache -----------------------------------------
    decode = {}
    if not a.no_decode:
        del sets, calls
        torch.cuda.empty_cache()
        fmt_mx = pkg._lib.CFormat()
        lib.scmx_mxfp4_format(C.byref(fmt_mx))

        def mxfp4_random(n, k):
            """A standard MXFP4 tensor read in place: random E2M1 nibbles, one E8M0 byte per 32-block (each row's bytes
            within 3 of its lowest), and the row scales 2^(lowest - 128) the kernels place the blocks with."""
            codes = rng.integers(0, 2 ** 32, n * k // 8, dtype=np.uint64).astype(np.uint32)
            e8 = (rng.integers(0, 4, (n, k // 32)) + rng.integers(100, 120, (n, 1))).astype(np.uint8)
            return codes, e8, np.exp2(e8.min(1).astype(np.float64) - 128).astype(np.float32)

        # "" = the reference's own storage (2-bit block codes, e2e/sc_format.py:4-15); "_mxfp4" = BASELINE config 2's
        # wording, nibbles + one E8M0 byte per 32-block, read in place
        for form, cfmt, bc_bytes, gen in (("", fmt, 1.0 / 128, lambda n, k: packed_random(rng, n, k)),
                                          ("_mxfp4", fmt_mx, 1.0 / 32, mxfp4_random)):
            for name, n, k in DECODE:
                bytes_call = n * k * (0.5 + bc_bytes) + 4 * n + 2 * k + 2 * n      # packed codes + block bytes + row
                copies = max(2, -(-320 * 2 ** 20 // int(bytes_call)))              # scales + bf16 in / out
                copies = min(copies, 160)
                wsets = [tuple(up(t) for t in gen(n, k)) for _ in range(copies)]
                for batch in (1, 4):
                    x = up(acts(rng, batch, k)).to(torch.bfloat16)
                    out = torch.empty((batch, n), dtype=torch.bfloat16, device=dev)
                    argl = [(C.byref(cfmt), x.data_ptr(), None, c.data_ptr(), b.data_ptr(), w.data_ptr(), None, out.data_ptr(),
                             1, 1, None, C.c_float(0.0), batch, n, k, None, 0, 0, -1, sp) for c, b, w in wsets]
                    reps_d = max(copies, 100)
                    ms_d, ms_d_min = timeit(lambda i: check(lib.scmx_gemv(*argl[i % copies])), reps_d, reps=a.reps, warmup=copies,
                                       warm_s=0.2)
                    us = ms_d * 1e3
                    # the same call on one weight set over and over: what the layer costs when its weights stay in the
                    # last-level cache (the protocol of e2e/bench_gemv_qwen35.py:16-18 reports both)
                    ms_r, _ = timeit(lambda i: check(lib.scmx_gemv(*argl[0])), reps_d, reps=max(3, a.reps // 2), warmup=5,
                                     warm_s=0.05)
                    # the same launches replayed from a HIP graph: kernel time without the host's per-call launch cost
                    ncap = min(copies, 40)
                    side = torch.cuda.Stream()
                    side.wait_stream(stream)
                    graph = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(graph, stream=side):
                        ssp = C.c_void_p(torch.cuda.current_stream().cuda_stream)
                        for i in range(ncap):
                            check(lib.scmx_gemv(*(argl[i][:-1] + (ssp,))))
                    stream.wait_stream(side)
                    ms_g, _ = timeit(lambda i: graph.replay(), max(2, 100 // ncap), reps=a.reps, warm_s=0.1)
                    us_g = ms_g * 1e3 / ncap
                    bts = n * k * (0.5 + bc_bytes) + 4 * n + batch * (2 * k + 2 * n)
                    decode[f"{name}_b{batch}{form}"] = {"us": round(us, 2), "us_min": round(ms_d_min * 1e3, 2),
                                                  "gbps": round(bts / us / 1e3, 1),
                                                  "pct_hbm": round(bts / us / 1e3 / PEAK_HBM_GBPS * 100, 1),
                                                  "us_resident": round(ms_r * 1e3, 2),
                                                  "us_graph": round(us_g, 2), "gbps_graph": round(bts / us_g / 1e3, 1),
                                                  "pct_hbm_graph": round(bts / us_g / 1e3 / PEAK_HBM_GBPS * 100, 1)}
                    del graph
                del wsets
                torch.cuda.empty_cache()

    # ---- offline quantizer on the device: float32 weights -> packed SC-MXFP4 -----------------------------------
    quant = {}
    if not a.no_quant:
        torch.cuda.empty_cache()
        n, k = 12288, 2048
        wf = torch.randn((n, k), device=dev) * 0.02
        qc = torch.empty(n * k // 8, dtype=torch.int32, device=dev)
        qb = torch.empty((n, k // 128), dtype=torch.uint8, device=dev)
        qw = torch.empty(n, dtype=torch.float32, device=dev)
        qargs = (wf.data_ptr(), 0, n, k, 32, qc.data_ptr(), qb.data_ptr(), qw.data_ptr(), sp)
        for _ in range(2):
            check(lib.scmx_quantize_sc(*qargs))
        torch.cuda.synchronize()
        e0.record(stream)
        for _ in range(10):
            check(lib.scmx_quantize_sc(*qargs))
        e1.record(stream)
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) / 10 * 1e3
        quant = {"workload": f"float32 {n}x{k} -> codes + block codes + row scales (exponent search over 3 candidates "
                             "in float64, bit-identical to the host quantizer)", "us": round(us, 1),
                 "gweights_per_s": round(n * k / us / 1e3, 2),
                 "gbps": round(n * k * (2 * 4 + 0.5 + 1.0 / 128) / us / 1e3, 1)}   # the row is read twice
        from mxfp4_int8_m5_amd import pack_format as PF
        fam_name = "e2m1/B16/M1..10"
        PF.pack_matrix(wf[:2048], fam_name)
        torch.cuda.synchronize()
        e0.record(stream)
        for _ in range(5):
            PF.pack_matrix(wf[:2048], fam_name)
        e1.record(stream)
        torch.cuda.synchronize()
        us_f = e0.elapsed_time(e1) / 5 * 1e3
        quant["family"] = {"workload": f"float32 2048x{k} -> format {fam_name} (8 row bases x 10 block multipliers tried "
                                       "per block, float32, bit-identical to the host quantizer)", "us": round(us_f, 1),
                           "gweights_per_s": round(2048 * k / us_f / 1e3, 2)}
        if not a.no_cpu:
            from oracle import layout as olayout
            wh = wf[:256].cpu().numpy().astype(np.float64)
            t0 = time.perf_counter()
            olayout.quantize(wh)
            quant["cpu_oracle_gweights_per_s"] = round(256 * k / (time.perf_counter() - t0) / 1e9, 4)
            from oracle import family as ofamily
            t0 = time.perf_counter()
            ofamily.quantize(wh[:64].astype(np.float32), ofamily.member(fam_name))
            quant["family"]["cpu_oracle_gweights_per_s"] = round(64 * k / (time.perf_counter() - t0) / 1e9, 5)
        del wf, qc, qb, qw

    # ---- whole model: Qwen3-1.7B architecture with random packed weights, prefill and batch-1 decode -----------------
    model = {}
    if not a.no_model:
        torch.cuda.empty_cache()
        from mxfp4_int8_m5_amd import fused_qwen3 as FQ
        args = FQ.Qwen3Args()                          # 28 layers, hidden 2048, intermediate 6144, 16 / 8 heads of 128
        g = torch.Generator(device=dev).manual_seed(0)
        D, Fi, hq, hk, d = (args.hidden_size, args.intermediate_size, args.num_attention_heads,
                            args.num_key_value_heads, args.head_dim)
        shapes = {"self_attn.q_proj": (hq * d, D), "self_attn.k_proj": (hk * d, D), "self_attn.v_proj": (hk * d, D),
                  "self_attn.o_proj": (D, hq * d), "mlp.gate_proj": (Fi, D), "mlp.up_proj": (Fi, D),
                  "mlp.down_proj": (D, Fi)}

        def rand_packed(n, k):                         # random codes; shifts 0..3; row scales near 2^-7 / sqrt(k / 2048)
            codes = torch.randint(-2 ** 31, 2 ** 31 - 1, (n * k // 8,), dtype=torch.int32, device=dev, generator=g)
            bc = torch.randint(0, 256, (n, k // 128), dtype=torch.uint8, device=dev, generator=g)
            return codes, bc, torch.full((n,), 2.0 ** -10 * (2048 / k) ** 0.5, device=dev)
        ones = lambda n: torch.ones(n, dtype=torch.bfloat16, device=dev)   # noqa: E731
        params = {"model.embed_tokens.weight": (torch.randn((args.vocab_size, D), device=dev, generator=g) * 0.05),
                  "model.norm.weight": ones(D)}
        packed = {}
        for i in range(args.num_hidden_layers):
            pre = f"model.layers.{i}."
            params.update({pre + "input_layernorm.weight": ones(D), pre + "post_attention_layernorm.weight": ones(D),
                           pre + "self_attn.q_norm.weight": ones(d), pre + "self_attn.k_norm.weight": ones(d)})
            for n, (o, k) in shapes.items():
                packed[f"layers.{i}.{n}"] = rand_packed(o, k)
        fm = FQ.FusedQwen3(args, params, packed)
        del params, packed
        ids = torch.randint(0, args.vocab_size, (M_TOKENS,), device=dev, generator=g)
        fm.hidden(ids)
        torch.cuda.synchronize()
        e0.record(stream)
        for _ in range(3):
            fm.hidden(ids)
        e1.record(stream)
        torch.cuda.synchronize()
        ms_p = e0.elapsed_time(e1) / 3
        model = {"workload": "Qwen3-1.7B architecture (28 blocks), random packed weights; prefill of 2048 tokens into "
                             "a fresh cache (hidden states), then batch-1 decode steps at context 131..163 (bf16 output head unless "
                             "named otherwise)",
                 "prefill_ms": round(ms_p, 2), "prefill_tokens_per_s": round(M_TOKENS / ms_p * 1e3, 0)}
        for name, kw in (("decode_eager", {}), ("decode_graph_per_half_block", {"graphs": True}),
                         ("decode_graph_per_step", {"graphs": "step"}),
                         ("decode_graph_per_step_all_prologues_fused", {"graphs": "step", "fuse_prologue": True}),
                         ("decode_graph_per_step_all_prologues_fused_packed_head",
                          {"graphs": "step", "fuse_prologue": True, "head": "packed"})):
            cache = fm.make_cache(512)
            fm.hidden(ids[:128], cache)
            dec = FQ.DecodeQwen3(fm, **kw)
            for j in range(3):
                dec.step(ids[128 + j:129 + j], cache)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for j in range(32):
                dec.step(ids[131 + j:132 + j], cache)
            torch.cuda.synchronize()
            model[name + "_tokens_per_s"] = round(32 / (time.perf_counter() - t0), 1)
        # the prefill attention kernel alone against the array library's op (2048 tokens, 16 / 8 heads of 128)
        import torch.nn.functional as TF
        from mxfp4_int8_m5_amd import sc_kernels as SK
        qa = torch.randn(M_TOKENS, hq, d, device=dev, generator=g).to(torch.bfloat16)
        ka = torch.randn(hk, M_TOKENS, d, device=dev, generator=g).to(torch.bfloat16)
        va = torch.randn(hk, M_TOKENS, d, device=dev, generator=g).to(torch.bfloat16)
        for label, fn in (("attn_prefill_us", lambda: SK.attn_prefill(qa.transpose(0, 1), ka, va, 0)),
                          ("torch_attention_us", lambda: TF.scaled_dot_product_attention(
                              qa.transpose(0, 1)[None], ka[None], va[None], is_causal=True, enable_gqa=True))):
            for _ in range(3):
                fn()
            torch.cuda.synchronize()
            e0.record(stream)
            for _ in range(20):
                fn()
            e1.record(stream)
            torch.cuda.synchronize()
            model[label] = round(e0.elapsed_time(e1) / 20 * 1e3, 1)
        del qa, ka, va
        # the same at a long context: 4000 cached tokens in a 4096-row cache (the decode attention then cuts the rows of a
        # head into ranges; without that one workgroup per head would read 2 MB of K and V per block)
        cache = fm.make_cache(4096)
        long_ids = torch.randint(0, args.vocab_size, (4064,), device=dev, generator=g)
        fm.hidden(long_ids[:2000], cache)
        fm.hidden(long_ids[2000:4000], cache)
        dec = FQ.DecodeQwen3(fm, graphs="step", fuse_prologue=True, head="packed")
        for j in range(3):
            dec.step(long_ids[4000 + j:4001 + j], cache)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for j in range(32):
            dec.step(long_ids[4003 + j:4004 + j], cache)
        torch.cuda.synchronize()
        model["decode_graph_per_step_all_prologues_fused_packed_head_context_4000_tokens_per_s"] = round(
            32 / (time.perf_counter() - t0), 1)
        del fm, dec, cache
        torch.cuda.empty_cache()

    result = {
        "metric": "INT8 TOPS, W4A8 prefill GEMM M=2048 (Qwen3-1.7B layer shapes), 1 GPU; decode GEMV GB/s alongside",
        "value": round(tops, 2), "unit": "TOPS", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(ms_step, 4), "ms_per_step_min": round(ms_step_min, 4), "repetitions": a.reps,
        "timing": "median of `repetitions` repetitions of `steps` back-to-back steps after `warmup` steps + 0.5 s of warm-up",
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8", "data": "synthetic",
        "config": {"workload": "BASELINE configs[1] at M=2048: SC-MXFP4 W4A8 linear (act-quant prologue + fused-unpack "
                               "INT8 MFMA GEMM + bf16 epilogue) over qkv 4096x2048, o_proj 2048x2048, gate_up 12288x2048, "
                               "down 2048x6144", "tokens": M_TOKENS, "weight_sets_rotated": n_sets},
        "pct_int8_peak": round(tops / PEAK_INT8_TOPS * 100, 2),
        "system": {"library": lib.scmx_version().decode(), "torch": torch.__version__, "rocm": torch.version.hip,
                   "device": torch.cuda.get_device_name(0),
                   "compute_units": torch.cuda.get_device_properties(0).multi_processor_count,
                   "host_cores": os.cpu_count()},
        "step_parts": step_parts,
        "roofline": roofline,
        "prefill_sweep": sweep,
        "library_int8_gemm": library,
        "moe": moe,
        "decode": decode,
        "quantize": quant,
        "model": model,
    }
    if not a.no_cpu:
        result["cpu_baseline"] = cpu_baseline()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
