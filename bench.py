#!/usr/bin/env python3
"""Benchmark of the MoE verify step (BASELINE config 2) on one MI355X.

A step = one MoE layer of a verify window: T = 16 rows, hidden 2048, 512 IQ3_S experts (gate|up 2048 -> 2 x 512, down
512 -> 2048), top-10, one shared expert, f32 router of 513 rows. Inputs are resident in HBM before the timed region.
Steps cycle through LAYERS distinct weight sets (about 11 GB) and fresh activations so that a step's ~190 MB working set
is cold with respect to the 256 MB Infinity Cache.

Prints ONE JSON line: whole-step throughput, the roofline of the dominant kernel (the routed gate|up mat-vec, timed on
its own with events on the launch stream) and the CPU baseline (the oracle on the host's cores, bounded sample).
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "tests"))

N, FF, NEXP, TOPK, T = 2048, 512, 512, 10, 16
HBM_PEAK = 8.0e12
# HBM bytes of one gate|up launch from the FETCH_SIZE / WRITE_SIZE counter runs (profiles/moe_gate_up_hbm_traffic.md),
# as a ratio to the launch's algorithmic bytes at the profiled routing (139.2 distinct experts): 136.8 MB / 127.1 MB
GATE_UP_TRAFFIC_RATIO = 1.076
IQ3S_BLOCK = 110
GU_BYTES = 2 * FF * (N // 256) * IQ3S_BLOCK      # 901,120 per expert
DN_BYTES = N * (FF // 256) * IQ3S_BLOCK          # 450,560 per expert
ROUTER_BYTES = (NEXP + 1) * N * 4                # 4,202,496
XIO_BYTES = 2 * T * N * 4                        # x in + out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--layers", type=int, default=16, help="distinct weight sets cycled through")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="budget of the CPU baseline leg (0: skip)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain device copy of 256 MiB, the known-size kernel that scales the FETCH_SIZE / WRITE_SIZE counters")
    ap.add_argument("--raw-layout", action="store_true", help="leave the weights as raw ggml blocks (skip the load-time re-laying)")
    ap.add_argument("--workload", choices=["verify", "prefill"], default="verify",
                    help="verify: BASELINE config 2 (the headline metric, the default); prefill: config 5, one MoE layer over prompt chunks of 512 rows")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1", file=sys.stderr)
        sys.exit(2)
    if args.workload == "prefill":
        return prefill_main(args)

    import numpy as np
    import torch
    import fnx_gpu
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = fnx_gpu.Dev()
    pkg, lib, t = dev.pkg, dev.lib, torch
    g = torch.Generator(device="cuda")
    g.manual_seed(1234)

    def rand_iq3s(nblocks):
        b = torch.randint(0, 256, (nblocks, IQ3S_BLOCK), dtype=torch.uint8, device="cuda", generator=g)
        d = (torch.rand(nblocks, device="cuda", generator=g) * 3e-4 + 1e-5).to(torch.float16)
        b[:, 0:2] = d.view(torch.uint8).reshape(nblocks, 2)
        return b.reshape(-1)

    layers = []
    for _ in range(args.layers):
        router = (torch.randn((NEXP + 1, N), device="cuda", generator=g) * 0.02).contiguous()
        gu = rand_iq3s(NEXP * 2 * FF * N // 256)
        down = rand_iq3s(NEXP * N * FF // 256)
        sh_gu = rand_iq3s(2 * FF * N // 256)
        sh_down = rand_iq3s(N * FF // 256)
        # the CPU leg reads raw ggml blocks: keep weight set 0's before the load-time re-laying (fnx_iq3s_repack, in place)
        raw = [a.cpu().numpy() for a in (gu, down, sh_gu, sh_down)] if not layers and args.cpu_seconds > 0 else None
        if not args.raw_layout:
            for w in (gu, down, sh_gu, sh_down):
                dev.ok(lib.fnx_iq3s_repack(w.data_ptr(), w.data_ptr(), w.numel() // IQ3S_BLOCK * 256, dev.st()))
        pk = not args.raw_layout
        L = pkg.MoeLayer(N, FF, NEXP, TOPK, router.data_ptr(), 0, pkg.dw(gu, N, 2 * FF, packed=pk), GU_BYTES, pkg.dw(down, FF, N, packed=pk),
                         DN_BYTES, pkg.dw(sh_gu, N, 2 * FF, packed=pk), pkg.dw(sh_down, FF, N, packed=pk))
        layers.append((L, router, gu, down, sh_gu, sh_down, raw))
    NX = 64
    xs = torch.randn((NX, T, N), device="cuda", generator=g)
    outs = torch.zeros((NX, T, N), device="cuda")
    P = T * TOPK
    ws_t = dict(xq=dev.zeros(T * (N // 32) * 36, t.uint8), logits=dev.zeros((T, NEXP + 1), t.float32), topi=dev.zeros((T, TOPK), t.int32),
                topw=dev.zeros((T, TOPK), t.float32), jobs_gu=dev.zeros((P + 1) * 136, t.uint8), jobs_dn=dev.zeros((P + 1) * 136, t.uint8),
                njobs=dev.zeros(2, t.int32), gu=dev.zeros((P + T, 2 * FF), t.float32), part=dev.zeros((P + T, N), t.float32))
    ws = pkg.MoeWs(*(ws_t[k].data_ptr() for k in ("xq", "logits", "topi", "topw", "jobs_gu", "jobs_dn", "njobs", "gu", "part")))
    st = dev.st()

    def step(i):
        L = layers[i % args.layers][0]
        x = xs[i % NX]
        dev.ok(lib.fnx_moe_verify_layer(C.byref(L), x.data_ptr(), T, outs[i % NX].data_ptr(), C.byref(ws), st))

    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").random_()
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)
        torch.cuda.synchronize()

    # ---- whole steps
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(args.warmup + i)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt / args.steps * 1e3

    # ---- distinct experts per step (for the algorithmic bytes), from the routing the steps produced
    njobs = []
    for i in range(min(args.steps, 64)):
        step(args.warmup + i)
        torch.cuda.synchronize()
        njobs.append(int(ws_t["njobs"][0].item()))
    u_mean = float(np.mean(njobs))
    step_bytes = u_mean * (GU_BYTES + DN_BYTES) + (GU_BYTES + DN_BYTES) + ROUTER_BYTES + XIO_BYTES

    # ---- the dominant kernel: the window's gate|up launch (routed experts + the shared expert), timed with events the
    # library records on the launch stream around each of the window's five launches (fnx_layer_profile)
    names = ["router+q8_1", "topk/jobs/plan", "gate|up", "down", "combine"]
    per_launch = np.zeros(5)
    reps = max(50, min(args.steps, 200))
    ms5 = np.zeros(5, dtype=np.float32)
    fused = not args.raw_layout
    if fused:
        dev.ok(lib.fnx_layer_profile(1))
        for i in range(reps + 10):
            step(args.warmup + i)
            dev.ok(lib.fnx_layer_profile_read(ms5.ctypes.data))
            if i >= 10:
                per_launch += ms5
        dev.ok(lib.fnx_layer_profile(0))
        per_launch /= reps
        k_ms = float(per_launch[2])
        kernel_name = "k_moe_gate_up_passes (unit64)"
        # algorithmic bytes of one launch: the distinct experts' and the shared expert's gate|up blocks, the window's
        # q8_1 rows, the f32 outputs
        k_bytes = (u_mean + 1) * GU_BYTES + T * (N // 32) * 36 + (P + T) * 2 * FF * 4
    else:
        evs = []
        for i in range(reps + 10):
            L, x = layers[i % args.layers][0], xs[i % NX]
            dev.ok(lib.fnx_quantize_q8_1(x.data_ptr(), ws.xq, N, T, st))
            dev.ok(lib.fnx_router_route(L.router, 0, x.data_ptr(), ws.logits, T, N, NEXP, TOPK, ws.topi, ws.topw, ws.jobs_gu, ws.jobs_dn, ws.njobs, st))
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            dev.ok(lib.fnx_moe_gate_up(C.byref(L.gu), L.gu_stride, ws.jobs_gu, ws.njobs, P, ws.xq, ws.gu, TOPK, st))
            e1.record()
            evs.append((e0, e1))
        torch.cuda.synchronize()
        k_ms = float(np.mean([a.elapsed_time(b) for a, b in evs[10:]]))
        kernel_name = "k_iq3s_jobs<64, narrow, raw> (routed gate|up)"
        k_bytes = u_mean * GU_BYTES + T * (N // 32) * 36 + P * 2 * FF * 4
    achieved = k_bytes / (k_ms * 1e-3)

    # ---- CPU baseline: the oracle on the host's cores, same workload (layer set 0), bounded sample
    cpu = None
    if args.cpu_seconds > 0:
        import oracle_lib
        oracle = oracle_lib.Oracle()
        threads = min(os.cpu_count() or 1, 16)
        L, router = layers[0][0], layers[0][1]
        h = [router.cpu().numpy()] + layers[0][6]
        xh = xs[0].cpu().numpy()
        r = oracle.moe_verify_layer(N, FF, NEXP, TOPK, *h, xh, threads=threads)   # warm-up, and a last parity check
        dev.ok(lib.fnx_moe_verify_layer(C.byref(L), xs[0].data_ptr(), T, outs[0].data_ptr(), C.byref(ws), st))
        torch.cuda.synchronize()
        err = float(np.linalg.norm(outs[0].cpu().numpy() - r["out"]) / np.linalg.norm(r["out"]))
        same = bool(np.array_equal(ws_t["topi"].cpu().numpy(), r["topi"]))
        c0 = time.perf_counter()
        n_cpu = 0
        while time.perf_counter() - c0 < args.cpu_seconds or n_cpu < 2:
            oracle.moe_verify_layer(N, FF, NEXP, TOPK, *h, xh, threads=threads)
            n_cpu += 1
        cdt = time.perf_counter() - c0
        cpu = {"value": n_cpu / cdt, "unit": "layer-steps/s", "cores": threads, "kind": "port",
               "sample": f"{n_cpu} layer-steps of the same workload (weight set 0, T=16) on the oracle (q8_1 x IQ3_S restated from the reference, not ggml's Q8_K kernel)",
               "parity_rel_l2": err, "routing_identical": same}

    line = {
        "metric": "MoE verify steps/sec at T=16 + IQ3_S expert GEMV achieved HBM GB/s (% peak)",
        "value": args.steps / dt,
        "unit": "layer-steps/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8 x IQ3_S (i32 dot, f32 accumulate)", "data": "synthetic",
        "config": {"workload": "config 2: one MoE verify layer, T=16, hidden 2048, 512 IQ3_S experts top-10, SwiGLU ff 512, shared expert, f32 router",
                   "weight_layout": "raw ggml blocks" if args.raw_layout else "unit64 (re-laid once at load, same bytes)", "weight_sets": args.layers, "distinct_experts_per_step": u_mean, "step_algorithmic_bytes": step_bytes,
                   "step_hbm_frac": step_bytes / (ms_per_step * 1e-3) / HBM_PEAK},
        "roofline": {"bound": "hbm", "kernel": kernel_name, "achieved": achieved / 1e9, "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK, "traffic": k_bytes * GATE_UP_TRAFFIC_RATIO if fused else None, "kernel_ms": k_ms, "algorithmic_bytes": k_bytes,
                     "window_launch_us": {n_: round(float(v) * 1e3, 2) for n_, v in zip(names, per_launch)}},
        "cpu_baseline": cpu,
    }
    print(json.dumps(line))


def prefill_main(args):
    """BASELINE config 5: one MoE layer over prompt chunks of 512 rows (5,120 routed pairs), expert popularity Zipf(1.1)
    imposed through a constant input feature and a bias column of the router. A step = one chunk."""
    import numpy as np
    import torch
    import fnx_gpu
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = fnx_gpu.Dev()
    pkg, lib, t = dev.pkg, dev.lib, torch
    g = torch.Generator(device="cuda")
    g.manual_seed(4321)
    CH, PF = 512, 64
    steps, warmup = min(args.steps, 76), min(args.warmup, 8)
    nsets = min(args.layers, 4)

    def rand_iq3s(nblocks):
        b = torch.randint(0, 256, (nblocks, IQ3S_BLOCK), dtype=torch.uint8, device="cuda", generator=g)
        d = (torch.rand(nblocks, device="cuda", generator=g) * 3e-4 + 1e-5).to(torch.float16)
        b[:, 0:2] = d.view(torch.uint8).reshape(nblocks, 2)
        return b.reshape(-1)

    pop = 1.0 / np.arange(1, NEXP + 1) ** 1.1
    layers = []
    for _ in range(nsets):
        router = torch.randn((NEXP + 1, N), device="cuda", generator=g) * 0.02
        bias = np.zeros(NEXP + 1, dtype=np.float32)
        bias[:NEXP] = np.log(pop / pop.sum())[np.random.default_rng(len(layers)).permutation(NEXP)]
        router[:, 0] = torch.from_numpy(bias).cuda()
        router = router.contiguous()
        ws_ = [rand_iq3s(NEXP * 2 * FF * N // 256), rand_iq3s(NEXP * N * FF // 256), rand_iq3s(2 * FF * N // 256), rand_iq3s(N * FF // 256)]
        raw = [a.cpu().numpy() for a in ws_] if not layers and args.cpu_seconds > 0 else None
        for w in ws_:
            dev.ok(lib.fnx_iq3s_repack(w.data_ptr(), w.data_ptr(), w.numel() // IQ3S_BLOCK * 256, dev.st()))
        gu, down, sh_gu, sh_down = ws_
        L = pkg.MoeLayer(N, FF, NEXP, TOPK, router.data_ptr(), 0, pkg.dw(gu, N, 2 * FF, packed=True), GU_BYTES, pkg.dw(down, FF, N, packed=True),
                         DN_BYTES, pkg.dw(sh_gu, N, 2 * FF, packed=True), pkg.dw(sh_down, FF, N, packed=True))
        layers.append((L, router, ws_, raw))
    NX = 8
    xs = torch.randn((NX, CH, N), device="cuda", generator=g)
    xs[:, :, 0] = 1.0   # the constant feature the router's bias column multiplies
    outs = torch.zeros((NX, CH, N), device="cuda")
    P = CH * TOPK
    J, S = P // PF + NEXP, (CH + PF - 1) // PF
    b = dict(logits=dev.zeros((CH, NEXP + 1), t.float32), topi=dev.zeros((CH, TOPK), t.int32), topw=dev.zeros((CH, TOPK), t.float32),
             cnt=dev.zeros(NEXP, t.int32), jbase=dev.zeros(NEXP, t.int32), jobs_gu=dev.zeros((J + S, 130), t.int32),
             jobs_dn=dev.zeros((J + S, 130), t.int32), njobs=dev.zeros(2, t.int32), xh=dev.zeros((CH, N), t.float16),
             gu=dev.zeros((P + CH, 2 * FF), t.float32), h16=dev.zeros((P + CH, FF), t.float16), part=dev.zeros((P + CH, N), t.float32))
    order = ("logits", "topi", "topw", "cnt", "jbase", "jobs_gu", "jobs_dn", "njobs", "xh", "gu", "h16", "part")
    ws = pkg.PfWs(*[b[k].data_ptr() for k in order])
    st = dev.st()

    def step(i):
        dev.ok(lib.fnx_moe_prefill_layer(C.byref(layers[i % nsets][0]), xs[i % NX].data_ptr(), CH, outs[i % NX].data_ptr(), C.byref(ws), st))

    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        step(warmup + i)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    # routing statistics of the chunks
    active, jobs = [], []
    for i in range(min(steps, 16)):
        step(warmup + i)
        torch.cuda.synchronize()
        active.append(int((b["cnt"] > 0).sum().item()))
        jobs.append(int(b["njobs"][0].item()))
    u_mean, j_mean = float(np.mean(active)), float(np.mean(jobs))
    # the two matrix-core launches on their own, with events on the launch stream (torch's current stream)
    reps = 20
    evs = []
    for i in range(reps + 3):
        L = layers[i % nsets][0]
        step(i)   # routes chunk i: the jobs and xh in the workspace are this chunk's
        e = [torch.cuda.Event(enable_timing=True) for _ in range(4)]
        e[0].record()
        dev.ok(lib.fnx_moe_gate_up_mma(C.byref(L.gu), L.gu_stride, ws.jobs_gu, ws.njobs, J, ws.xh, ws.gu, st))
        e[1].record()
        dev.ok(lib.fnx_swiglu_h16(ws.gu, FF, P + CH, ws.h16, st))
        e[2].record()
        dev.ok(lib.fnx_moe_down_mma(C.byref(L.down), L.down_stride, ws.jobs_dn, ws.njobs, J, ws.h16, ws.part, st))
        e[3].record()
        evs.append(e)
    torch.cuda.synchronize()
    gu_ms = float(np.mean([e[0].elapsed_time(e[1]) for e in evs[3:]]))
    sw_ms = float(np.mean([e[1].elapsed_time(e[2]) for e in evs[3:]]))
    dn_ms = float(np.mean([e[2].elapsed_time(e[3]) for e in evs[3:]]))
    gu_bytes = u_mean * GU_BYTES + CH * N * 2 + P * 2 * FF * 4
    dn_bytes = u_mean * DN_BYTES + P * FF * 2 + P * N * 4
    gu_flops, dn_flops = 2.0 * P * 2 * FF * N, 2.0 * P * N * FF
    step_bytes = (u_mean + 1) * (GU_BYTES + DN_BYTES) + ROUTER_BYTES + 2 * CH * N * 4
    step_flops = 2.0 * (P + CH) * 3 * FF * N + 2.0 * CH * (NEXP + 1) * N
    MFMA_F16 = 2.5e15
    cpu = None
    if args.cpu_seconds > 0:
        import oracle_lib
        oracle = oracle_lib.Oracle()
        threads = min(os.cpu_count() or 1, 16)
        CS = 64   # rows of the CPU sample
        h = [layers[0][1].cpu().numpy()] + layers[0][3]
        xc = xs[0, :CS].cpu().numpy()
        c0 = time.perf_counter()
        r = oracle.moe_prefill_layer(N, FF, NEXP, TOPK, *h, xc, threads=threads)
        cdt = time.perf_counter() - c0
        step(0)
        torch.cuda.synchronize()
        # the chunk's first CS rows are routed alone by the oracle: compare the rows' outputs (a row's result does not depend on its chunk)
        err = float(np.linalg.norm(outs[0, :CS].cpu().numpy() - r["out"]) / np.linalg.norm(r["out"]))
        cpu = {"value": CS / cdt, "unit": "tokens/s per layer", "cores": threads, "kind": "port",
               "sample": f"one pass of the oracle's prefill layer over the first {CS} rows of chunk 0 (f16 operands, f64 accumulation)",
               "parity_rel_l2": err}
    line = {
        "metric": "prefill MoE tokens/sec per layer (chunks of 512 rows) + grouped IQ3_S expert GEMM achieved GB/s and MFMA utilisation",
        "value": CH * steps / dt, "unit": "tokens/s per layer", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": dt / steps * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16 x f16 (IQ3_S dequantised once to f16), f32 accumulate", "data": "synthetic",
        "config": {"workload": "config 5: one MoE layer over prompt chunks of 512 rows, 5,120 routed pairs, 512 IQ3_S experts top-10 with Zipf(1.1) popularity, shared expert",
                   "weight_sets": nsets, "active_experts_per_chunk": u_mean, "jobs_per_chunk": j_mean, "step_algorithmic_bytes": step_bytes,
                   "step_flops": step_flops, "step_hbm_frac": step_bytes / (dt / steps) / HBM_PEAK, "step_mfma_frac": step_flops / (dt / steps) / MFMA_F16},
        "roofline": {"bound": "hbm", "kernel": "k_moe_mma_block (routed gate|up, unit64)", "achieved": gu_bytes / (gu_ms * 1e-3) / 1e9, "peak": HBM_PEAK / 1e9,
                     "unit": "GB/s", "frac": gu_bytes / (gu_ms * 1e-3) / HBM_PEAK, "traffic": None, "kernel_ms": gu_ms, "algorithmic_bytes": gu_bytes,
                     "mfma_tflops": gu_flops / (gu_ms * 1e-3) / 1e12, "mfma_frac": gu_flops / (gu_ms * 1e-3) / MFMA_F16,
                     "down": {"kernel_ms": dn_ms, "achieved": dn_bytes / (dn_ms * 1e-3) / 1e9, "mfma_tflops": dn_flops / (dn_ms * 1e-3) / 1e12},
                     "swiglu_ms": sw_ms},
        "cpu_baseline": cpu,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
