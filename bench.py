#!/usr/bin/env python3
"""Benchmark of the MoE verify step on one MI355X. "benchmark config N" below: the N-th entry of BASELINE.json's "configs"
(1: a lone IQ3_S mat-vec, 2: the MoE verify layer - the headline, 3: argmax + lookup + acceptance, 4: the reduced decoder's
verify step, 5: the prompt path's MoE layer).

A step = one MoE layer of a verify window: T = 16 rows, hidden 2048, 512 IQ3_S experts (gate|up 2048 -> 2 x 512, down
512 -> 2048), top-10, one shared expert, f32 router of 513 rows. Inputs are resident in HBM before the timed region.
Steps cycle through LAYERS distinct weight sets (about 11 GB) and fresh activations so that a step's ~190 MB working set
is cold with respect to the 256 MB Infinity Cache.

Prints ONE JSON line: whole-step throughput, the roofline of the dominant kernel (the window's one launch, timed
with events on the launch stream), what a read-only kernel reaches on the same GPU (roofline.stream_read_GBps), config 1
(config.gemv), and the CPU baseline (the oracle on the host's cores, bounded sample). The experts are IQ3_S blocks encoded
from N(0, 0.02) weights (--weights bytes: uniformly random blocks).
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
PKG_DIR = os.path.join(ROOT, "qwen3.8-flash-next-2x-p100_amd")


def harness():
    """the package's host-side harness over the C ABI (the package's directory name is not a Python identifier)"""
    import importlib
    import importlib.util
    name = "fnx_mi355x_pkg"
    if name not in sys.modules:
        spec = importlib.util.spec_from_file_location(name, os.path.join(PKG_DIR, "__init__.py"), submodule_search_locations=[PKG_DIR])
        mod = importlib.util.module_from_spec(spec)
        sys.modules[name] = mod
        spec.loader.exec_module(mod)
    return importlib.import_module(name + ".harness")


def oracle_side():
    """the CPU oracle's bindings (test infrastructure, under tests/): for the cpu_baseline legs only"""
    tests = os.path.join(ROOT, "tests")
    if tests not in sys.path:
        sys.path.insert(0, tests)
    import oracle_lib
    return oracle_lib


N, FF, NEXP, TOPK, T = 2048, 512, 512, 10, 16
HBM_PEAK = 8.0e12
# HBM bytes of one window launch of the default run (gaussian weights, 16 sets, unit64), measured by two rocprofv3 --pmc
# runs of this file (FETCH_SIZE, then WRITE_SIZE, each scaled by a 256 MiB copy: profiles/moe_window_hbm_traffic.md), and
# the distinct experts per step they were measured at. Not measured in the run: emitted only for that configuration.
WINDOW_TRAFFIC = {"bytes": 209.47e6, "algorithmic_bytes": 192.96e6, "distinct_experts_per_step": 138.45,
                   "source": "profiles/moe_window_hbm_traffic.md (rocprofv3 --pmc FETCH_SIZE, WRITE_SIZE of this file's default workload; scaled to "
                             "this run's algorithmic bytes; not measured in this run)"}
# the same for the prompt path's gate|up launch (profiles/prefill_chunk_counters.md: FETCH_SIZE x 2 + WRITE_SIZE)
PF_WINDOW_TRAFFIC = {"bytes": 132.0e6, "algorithmic_bytes": 98.6e6,
                      "source": "profiles/prefill_chunk_counters.md (rocprofv3 --pmc FETCH_SIZE, WRITE_SIZE of this file's prefill workload, k_moe_mma_wave16_gu; "
                                "scaled to this run's algorithmic bytes; not measured in this run)"}
IQ3S_BLOCK = 110
GU_BYTES = 2 * FF * (N // 256) * IQ3S_BLOCK      # 901,120 per expert
DN_BYTES = N * (FF // 256) * IQ3S_BLOCK          # 450,560 per expert
ROUTER_BYTES = (NEXP + 1) * N * 4                # 4,202,496
XIO_BYTES = 2 * T * N * 4                        # x in + out


def stream_calibration(dev, torch, np):
    """What this GPU gives a kernel that only reads (fnx_stream_read: the library's calibration kernels, no decode): plain
    and nontemporal 16-byte loads and the unit64 plane loads of the expert kernels over 1 GiB (the asymptote), and the
    plane loads over one launch of the size of the window's gate|up and down launches (launch ramp included). Events on
    the launch stream; every launch reads a region no launch of the last seven read."""
    lib, st = dev.lib, dev.st()
    UNIT = 880
    buf = torch.empty(1 << 30, dtype=torch.uint8, device="cuda").random_()
    sink = torch.zeros(4, dtype=torch.int32, device="cuda")

    def rate(variant, blocks, threads, nbytes):
        regions = max(1, min(8, (1 << 30) // nbytes))
        evs = []
        for i in range(13):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            dev.ok(lib.fnx_stream_read(buf.data_ptr() + (i % regions) * nbytes, nbytes, variant, blocks, threads, sink.data_ptr(), st))
            e1.record()
            evs.append((e0, e1))
        torch.cuda.synchronize()
        return nbytes / (float(np.mean([a.elapsed_time(b) for a, b in evs[3:]])) * 1e-3) / 1e9

    whole = (1 << 30) // (16 * UNIT) * (16 * UNIT)
    gate_up, down = 152064 * UNIT, 75776 * UNIT   # about 148.5 matrices of 901,120 and of 450,560 bytes
    return {"plain_16B_loads_1GiB": rate(1, 512, 512, whole), "nontemporal_16B_loads_1GiB": rate(5, 512, 512, whole),
            "unit64_plane_loads_1GiB": rate(6, 512, 512, whole),
            "unit64_plane_loads_one_launch_134MB": rate(9, 256, 1024, gate_up), "unit64_plane_loads_one_launch_67MB": rate(9, 256, 1024, down),
            # four units as one lane-interleaved record (six loads a lane of 16, 16, 16, 4, 4, 8 bytes), plain and nontemporal
            "quad_records_1GiB": rate(14, 512, 512, whole), "quad_records_nontemporal_1GiB": rate(15, 512, 512, whole),
            "quad_records_one_launch_134MB": rate(14, 256, 1024, gate_up), "quad_records_nontemporal_one_launch_134MB": rate(15, 256, 1024, gate_up),
            "quad_records_nontemporal_one_launch_67MB": rate(15, 256, 1024, down),
            "nontemporal_16B_loads_one_launch_134MB": rate(5, 256, 1024, gate_up)}


def gemv_measure(dev, torch, np, steps):
    """benchmark config 1: a 4096 x 2048 IQ3_S matrix (3,604,480 bytes) over T = 1 and T = 16 q8_1 rows: (a) one matrix a
    launch, cycling through 1,024 distinct matrices (3.7 GB) so that every launch reads its weights from HBM: a launch of
    3.6 MB is bound by the launch, not by HBM; (b) one fnx_mmvq launch of 1,024 jobs over the 1,024 matrices through the
    table of matrix pointers: the kernel's streaming rate."""
    fnx_gpu = harness()
    pkg, lib, st = dev.pkg, dev.lib, dev.st()
    g = torch.Generator(device="cuda")
    g.manual_seed(11)
    ROWS, COLS, NM = 4096, 2048, 1024
    mbytes = ROWS * COLS // 256 * IQ3S_BLOCK
    w = _rand_iq3s(torch, g, NM * ROWS * COLS // 256)
    dev.ok(lib.fnx_iq3s_repack(w.data_ptr(), w.data_ptr(), w.numel() // IQ3S_BLOCK * 256, st))
    ep = torch.tensor([w.data_ptr() + i * mbytes for i in torch.randperm(NM).tolist()], dtype=torch.int64, device="cuda")
    lone, many = {}, {}
    for T in (1, 16):
        x = torch.randn((T, COLS), device="cuda", generator=g)
        xq = torch.zeros(T * (COLS // 32) * 36, dtype=torch.uint8, device="cuda")
        dev.ok(lib.fnx_quantize_q8_1(x.data_ptr(), xq.data_ptr(), COLS, T, st))
        jobs = np.zeros(NM, dtype=fnx_gpu.JOB_DTYPE)
        jobs["w"] = np.arange(NM)
        jobs["n"] = T
        jobs["y"][:, :T] = np.arange(T)[None, :]
        jobs["out"][:, :T] = np.arange(NM)[:, None] * T + np.arange(T)[None, :]
        dj = dev.up(jobs.view(np.uint8).reshape(-1))
        out = torch.zeros((NM * T, ROWS), device="cuda")
        Ws = [pkg.dw(w.data_ptr() + i * mbytes, COLS, ROWS, packed=True) for i in range(NM)]
        n1 = max(steps, 512)
        for i in range(64):
            dev.ok(lib.fnx_mmvq(C.byref(Ws[i % NM]), 0, dj.data_ptr(), None, 1, xq.data_ptr(), out.data_ptr(), ROWS, st))
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for i in range(n1):
            dev.ok(lib.fnx_mmvq(C.byref(Ws[(64 + i) % NM]), 0, dj.data_ptr(), None, 1, xq.data_ptr(), out.data_ptr(), ROWS, st))
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) / n1 * 1e3
        nbytes = mbytes + T * (COLS // 32) * 36 + T * ROWS * 4
        lone[f"T{T}"] = {"us_per_launch": us, "algorithmic_bytes": nbytes, "GBps": nbytes / (us * 1e-6) / 1e9, "hbm_frac": nbytes / (us * 1e-6) / HBM_PEAK}
        Wall = pkg.dw(w.data_ptr(), COLS, ROWS, ep=ep.data_ptr(), packed=True)
        evs = []
        for i in range(8):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            dev.ok(lib.fnx_mmvq(C.byref(Wall), 0, dj.data_ptr(), None, NM, xq.data_ptr(), out.data_ptr(), ROWS, st))
            b.record()
            evs.append((a, b))
        torch.cuda.synchronize()
        us = float(np.mean([a.elapsed_time(b) for a, b in evs[2:]])) * 1e3
        nbytes = NM * (mbytes + T * ROWS * 4) + T * (COLS // 32) * 36
        many[f"T{T}"] = {"us_per_launch": us, "algorithmic_bytes": nbytes, "GBps": nbytes / (us * 1e-6) / 1e9, "hbm_frac": nbytes / (us * 1e-6) / HBM_PEAK}
    # (c) the same launch over copies in the prompt path's layout (tile16, fnx_iq3s_tile16): jobs of many rows decoded
    # straight into the matrix cores' operands (k_iq3s_jobs_mma16); the layout to keep for experts that see many rows a job
    many16 = {}
    one16 = lib.fnx_iq3s_tile16_bytes(ROWS, COLS, 1)
    w16 = torch.zeros(one16 * NM, dtype=torch.uint8, device="cuda")
    dev.ok(lib.fnx_iq3s_tile16(w.data_ptr(), w16.data_ptr(), ROWS, COLS, NM, st))
    ep16 = torch.tensor([w16.data_ptr() + i * one16 for i in torch.randperm(NM).tolist()], dtype=torch.int64, device="cuda")
    for T in (1, 16):
        x = torch.randn((T, COLS), device="cuda", generator=g)
        xq = torch.zeros(T * (COLS // 32) * 36, dtype=torch.uint8, device="cuda")
        dev.ok(lib.fnx_quantize_q8_1(x.data_ptr(), xq.data_ptr(), COLS, T, st))
        jobs = np.zeros(NM, dtype=fnx_gpu.JOB_DTYPE)
        jobs["w"] = np.arange(NM)
        jobs["n"] = T
        jobs["y"][:, :T] = np.arange(T)[None, :]
        jobs["out"][:, :T] = np.arange(NM)[:, None] * T + np.arange(T)[None, :]
        dj = dev.up(jobs.view(np.uint8).reshape(-1))
        out = torch.zeros((NM * T, ROWS), device="cuda")
        Wall = pkg.dw(w16.data_ptr(), COLS, ROWS, ep=ep16.data_ptr(), tile16=True)
        evs = []
        for i in range(8):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            dev.ok(lib.fnx_mmvq(C.byref(Wall), 0, dj.data_ptr(), None, NM, xq.data_ptr(), out.data_ptr(), ROWS, st))
            b.record()
            evs.append((a, b))
        torch.cuda.synchronize()
        us = float(np.mean([a.elapsed_time(b) for a, b in evs[2:]])) * 1e3
        nbytes = NM * (one16 + T * ROWS * 4) + T * (COLS // 32) * 36
        many16[f"T{T}"] = {"us_per_launch": us, "algorithmic_bytes": nbytes, "GBps": nbytes / (us * 1e-6) / 1e9, "hbm_frac": nbytes / (us * 1e-6) / HBM_PEAK}
    del w, w16, out
    torch.cuda.empty_cache()
    return {"lone_matrix_a_launch": lone, "launch_of_1024_matrices": many, "launch_of_1024_matrices_tile16": many16}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--layers", type=int, default=16, help="distinct weight sets cycled through")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="budget of the CPU baseline leg (0: skip)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain device copy of 256 MiB, the known-size kernel that scales the FETCH_SIZE / WRITE_SIZE counters")
    ap.add_argument("--weights", choices=["gaussian", "bytes"], default="gaussian",
                    help="gaussian: experts IQ3_S-encoded from N(0, 0.02) weights (benchmark config 2's recipe); bytes: uniformly random blocks")
    ap.add_argument("--shared-q8", action="store_true",
                    help="the shared expert as dense split Q8_0 (the reference's own form, three more launches a window) instead of IQ3_S")
    ap.add_argument("--no-extras", action="store_true", help="skip the legs beside the metric (verify: streaming calibration, config 1, the other weight kind; prefill: two chunks in flight)")
    ap.add_argument("--raw-layout", action="store_true", help="verify: leave the weights as raw ggml blocks (skip the load-time re-laying); prefill: unit64 only, no tile16 copies")
    ap.add_argument("--down-unit64", action="store_true", help="prefill: leave the down matrices in the unit64 layout (k_moe_mma) instead of tile16 (k_moe_mma_wave16)")
    ap.add_argument("--workload", choices=["verify", "prefill", "decoder", "head", "gemv"], default="verify",
                    help="verify: benchmark config 2 (the headline metric, the default); prefill: config 5, one MoE layer over prompt chunks of 512 "
                         "rows; decoder: config 4, a verify step of the reduced decoder plus the draft layer; head: config 3, argmax + prompt "
                         "lookup + acceptance; gemv: config 1, one IQ3_S matrix over T = 1 and 16 rows")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1", file=sys.stderr)
        sys.exit(2)
    other = {"prefill": prefill_main, "decoder": decoder_main, "head": head_main, "gemv": gemv_main}.get(args.workload)
    if other:
        print(json.dumps(other(args)))
        return

    import numpy as np
    import torch
    fnx_gpu = harness()
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

    # the experts of benchmark config 2: IQ3_S blocks encoded from N(0, 0.02) weights. BANK distinct matrices of each kind
    # are encoded (this build's encoder, on the GPU) and every expert of every weight set is a copy of one of them at an
    # address of its own, so the bytes a step reads are as cold and as many as with 512 different experts
    BANK = 32
    bank = None
    if args.weights == "gaussian":
        import importlib
        enc = importlib.import_module("fnx_mi355x_pkg.iq3s_encode")
        bank = (enc.encode_iq3s(torch.randn((BANK, 2 * FF * N), device="cuda", generator=g) * 0.02).view(BANK, GU_BYTES),
                enc.encode_iq3s(torch.randn((BANK, N * FF), device="cuda", generator=g) * 0.02).view(BANK, DN_BYTES))

    def weight_set(kind, i):
        if kind == "bytes":
            return [rand_iq3s(NEXP * 2 * FF * N // 256), rand_iq3s(NEXP * N * FF // 256), rand_iq3s(2 * FF * N // 256), rand_iq3s(N * FF // 256)]
        pick = torch.randint(0, BANK, (NEXP,), device="cuda", generator=g)
        return [bank[0][pick].reshape(-1), bank[1][pick].reshape(-1), bank[0][i % BANK].clone(), bank[1][i % BANK].clone()]

    def make_sets(kind, count, keep_raw):
        sets = []
        for i in range(count):
            router = (torch.randn((NEXP + 1, N), device="cuda", generator=g) * 0.02).contiguous()
            gu, down, sh_gu, sh_down = weight_set(kind, i)
            # the CPU leg reads raw ggml blocks: keep weight set 0's before the load-time re-laying (fnx_iq3s_repack, in place)
            raw = [a.cpu().numpy() for a in (gu, down, sh_gu, sh_down)] if not sets and keep_raw else None
            (gu, down, sh_gu, sh_down), dws = fnx_gpu.pack_moe_weights(dev, [gu, down, sh_gu, sh_down], N, FF, not args.raw_layout)
            L = pkg.MoeLayer(N, FF, NEXP, TOPK, router.data_ptr(), 0, dws[0], GU_BYTES, dws[1], DN_BYTES, dws[2], dws[3])
            if args.shared_q8:
                q8 = [torch.randint(-127, 128, (2 * FF, N), dtype=torch.int8, device="cuda", generator=g),
                      (torch.rand((2 * FF, N // 32), device="cuda", generator=g) * 3e-4 + 1e-5).to(torch.float16),
                      torch.randint(-127, 128, (N, FF), dtype=torch.int8, device="cuda", generator=g),
                      (torch.rand((N, FF // 32), device="cuda", generator=g) * 3e-4 + 1e-5).to(torch.float16)]
                L.sh_gu_q8 = pkg.Q8S(q8[0].data_ptr(), q8[1].data_ptr(), 2 * FF, N)
                L.sh_down_q8 = pkg.Q8S(q8[2].data_ptr(), q8[3].data_ptr(), N, FF)
                if raw is not None:
                    raw = raw[:2] + [None, None, ((q8[0].cpu().numpy(), q8[1].cpu().numpy().view(np.uint16)), (q8[2].cpu().numpy(), q8[3].cpu().numpy().view(np.uint16)))]
                sh_gu = q8   # keeps the tensors alive
            sets.append((L, router, gu, down, sh_gu, sh_down, raw))
        return sets

    layers = make_sets(args.weights, args.layers, args.cpu_seconds > 0)
    NX = 64
    xs = torch.randn((NX, T, N), device="cuda", generator=g)
    outs = torch.zeros((NX, T, N), device="cuda")
    P = T * TOPK
    ws_t = dict(xq=dev.zeros(T * (N // 32) * 36, t.uint8), logits=dev.zeros((T, NEXP + 1), t.float32), topi=dev.zeros((T, TOPK), t.int32),
                topw=dev.zeros((T, TOPK), t.float32), jobs_gu=dev.zeros((P + 1) * 136, t.uint8), jobs_dn=dev.zeros((P + 1) * 136, t.uint8),
                njobs=dev.zeros(2, t.int32), gu=dev.zeros((P + T, 2 * FF), t.float32), part=dev.zeros((P + T, N), t.float32),
                sync=dev.zeros(pkg.MOE_SYNC_WORDS, t.int32))
    ws = pkg.MoeWs(*(ws_t[k].data_ptr() for k in ("xq", "logits", "topi", "topw", "jobs_gu", "jobs_dn", "njobs", "gu", "part", "sync")))
    st = dev.st()

    def step(i, sets=None):
        L = (sets or layers)[i % args.layers][0]
        x = xs[i % NX]
        dev.ok(lib.fnx_moe_verify_layer(C.byref(L), x.data_ptr(), T, outs[i % NX].data_ptr(), C.byref(ws), st))

    PREROLL_MS = 50.0
    preroll = {"ms": 0.0, "steps": 0}

    def timed_steps(sets=None):
        """W warm-up steps, then untimed steps until PREROLL_MS have passed whatever W is (so that a short timed region is
        not measured on clocks that have just come up from idle), then exactly K timed steps between two synchronisations"""
        for i in range(args.warmup):
            step(i, sets)
        torch.cuda.synchronize()
        p0, n_pre = time.perf_counter(), 0
        while (time.perf_counter() - p0) * 1e3 < PREROLL_MS:
            for i in range(64):
                step(args.warmup + n_pre + i, sets)
            n_pre += 64
            torch.cuda.synchronize()
        preroll["ms"], preroll["steps"] = (time.perf_counter() - p0) * 1e3, n_pre
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)   # on the launch stream (torch's current one)
        t0 = time.perf_counter()
        e0.record()
        for i in range(args.steps):
            step(args.warmup + n_pre + i, sets)
        e1.record()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        preroll["event_ms"] = e0.elapsed_time(e1)
        return dt

    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").random_()
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)
        torch.cuda.synchronize()

    # ---- whole steps
    dt = timed_steps()
    ms_per_step = dt / args.steps * 1e3
    headline_preroll = dict(preroll)

    # ---- distinct experts per step (for the algorithmic bytes), from the routing the steps produced
    njobs = []
    for i in range(min(args.steps, 64)):
        step(args.warmup + i)
        torch.cuda.synchronize()
        njobs.append(int(ws_t["njobs"][0].item()))
    u_mean = float(np.mean(njobs))
    step_bytes = u_mean * (GU_BYTES + DN_BYTES) + (GU_BYTES + DN_BYTES) + ROUTER_BYTES + XIO_BYTES

    # ---- the dominant kernel: the window's one launch (router, top-k, gate|up, SwiGLU, down, combine), timed with events the
    # library records on the launch stream around it (fnx_layer_profile)
    names = ["before the window (a split-Q8_0 shared expert's dense launches)", "k_moe_window"]
    per_launch = np.zeros(2)
    reps = max(50, min(args.steps, 200))
    ms2 = np.zeros(2, dtype=np.float32)
    fused = not args.raw_layout
    if fused:
        dev.ok(lib.fnx_layer_profile(1))
        for i in range(reps + 10):
            step(args.warmup + i)
            dev.ok(lib.fnx_layer_profile_read(ms2.ctypes.data))
            if i >= 10:
                per_launch += ms2
        dev.ok(lib.fnx_layer_profile(0))
        per_launch /= reps
        # the kernel's average duration: events on the launch stream around the timed region's K launches, which follow one
        # another with nothing between them (per_launch: one launch at a time from an idle GPU, with an event either side)
        k_ms = headline_preroll["event_ms"] / args.steps if not args.shared_q8 else float(per_launch[1])
        kernel_name = "k_moe_window (unit64; the whole window is this one launch)"
        # algorithmic bytes of the launch: the step's (the distinct experts' and the shared expert's blocks, the router, x in, out)
        k_bytes = step_bytes
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

    # ---- beside the headline: what a read-only kernel reaches on this GPU, config 1, and the same steps over uniformly
    # random blocks (the codebook lookups' bank conflicts depend on the codes)
    stream = gemv = other_ms = None
    if not args.no_extras and fused:
        stream = stream_calibration(dev, torch, np)
        other = "bytes" if args.weights == "gaussian" else "gaussian"
        if other == "bytes" or bank is not None:
            alt = make_sets(other, args.layers, False)
            other_ms = timed_steps(alt) / args.steps * 1e3
            del alt
            torch.cuda.empty_cache()
        gemv = gemv_measure(dev, torch, np, 512)
    traffic = None
    if fused and not args.shared_q8 and WINDOW_TRAFFIC["bytes"] and abs(u_mean - WINDOW_TRAFFIC["distinct_experts_per_step"]) < 3:
        traffic = WINDOW_TRAFFIC["bytes"] * k_bytes / WINDOW_TRAFFIC["algorithmic_bytes"]

    # ---- CPU baseline: the oracle on the host's cores, same workload (layer set 0), bounded sample
    cpu = None
    if args.cpu_seconds > 0:
        oracle_lib = oracle_side()
        oracle = oracle_lib.Oracle()
        threads = min(os.cpu_count() or 1, 16)
        L, router = layers[0][0], layers[0][1]
        h = [router.cpu().numpy()] + layers[0][6][:4]
        okw = dict(threads=threads, sh_q8=layers[0][6][4]) if args.shared_q8 else dict(threads=threads)
        xh = xs[0].cpu().numpy()
        r = oracle.moe_verify_layer(N, FF, NEXP, TOPK, *h, xh, **okw)   # warm-up, and a last parity check
        dev.ok(lib.fnx_moe_verify_layer(C.byref(L), xs[0].data_ptr(), T, outs[0].data_ptr(), C.byref(ws), st))
        torch.cuda.synchronize()
        err = float(np.linalg.norm(outs[0].cpu().numpy() - r["out"]) / np.linalg.norm(r["out"]))
        same = bool(np.array_equal(ws_t["topi"].cpu().numpy(), r["topi"]))
        c0 = time.perf_counter()
        n_cpu = 0
        while time.perf_counter() - c0 < args.cpu_seconds or n_cpu < 2:
            oracle.moe_verify_layer(N, FF, NEXP, TOPK, *h, xh, **okw)
            n_cpu += 1
        cdt = time.perf_counter() - c0
        cpu = {"value": n_cpu / cdt, "unit": "layer-steps/s", "cores": threads, "kind": "port",
               "sample": f"{n_cpu} layer-steps of the same workload (weight set 0, T=16) on the oracle (q8_1 x IQ3_S restated from the reference, not ggml's Q8_K kernel)",
               "parity_rel_l2": err, "routing_identical": same}

    # ---- the other workloads in short (their own lines: --workload head / decoder / prefill): a few steps each, CPU legs off
    others = None
    if not args.no_extras and fused:
        import copy
        del layers, xs, outs
        torch.cuda.empty_cache()
        short = copy.copy(args)
        short.cpu_seconds, short.no_extras = 0.0, True
        short.steps, short.warmup = 200, 20
        hd = head_main(short)
        short.steps, short.warmup = 30, 5
        dc = decoder_main(short)
        torch.cuda.empty_cache()
        short.steps, short.warmup, short.layers = 76, 8, 4
        pf = prefill_main(short)
        others = {
            "head": {"workload": hd["config"]["workload"], "us_per_round": hd["ms_per_step"] * 1e3, "argmax_us": hd["config"]["argmax_us"],
                     "lookup_us": hd["config"]["lookup_us"], "accept_us": hd["config"]["accept_us"], "identical_to_oracle": hd["config"]["identical_to_oracle"]},
            "decoder": {"workload": dc["config"]["workload"], "ms_per_step": dc["ms_per_step"], "steps": dc["steps"], "step_hbm_frac": dc["config"]["step_hbm_frac"],
                        "attention_TBps": dc["config"]["attention_GBps"] / 1e3, "head_TBps": dc["config"]["head_GBps"] / 1e3,
                        "decode_round_ms_graph_replay": dc["config"]["decode_round"]["ms_graph_replay"]},
            "prefill": {"workload": pf["config"]["workload"], "chunk_us": pf["ms_per_step"] * 1e3, "steps": pf["steps"], "tokens_per_s": pf["value"],
                        "piecewise_bound_frac": pf["roofline"]["piecewise_bound"]["chunk_frac"], "gate_up_us": pf["roofline"]["kernel_ms"] * 1e3,
                        "gate_up_mfma_frac": pf["roofline"]["mfma_frac"], "gate_up_hbm_frac": pf["roofline"]["frac"],
                        "down_us": pf["roofline"]["down"]["kernel_ms"] * 1e3,
                        "gate_up_traffic_ratio": (pf["roofline"]["traffic"] / pf["roofline"]["algorithmic_bytes"]) if pf["roofline"]["traffic"] else None},
        }

    line = {
        "metric": "MoE verify steps/sec at T=16 + IQ3_S expert GEMV achieved HBM GB/s (% peak)",
        "value": args.steps / dt,
        "unit": "layer-steps/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "preroll_ms": headline_preroll["ms"], "preroll_steps": headline_preroll["steps"],
        "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8 x IQ3_S (i32 dot, f32 accumulate)",
        "data": ("synthetic: experts IQ3_S-encoded from N(0, 0.02) weights by this build's encoder (32 distinct matrices of each kind, copied to "
                 "512 experts x the weight sets at addresses of their own)" if args.weights == "gaussian" else
                 "synthetic: uniformly random IQ3_S blocks") + ", f32 router N(0, 0.02), activations N(0, 1)",
        "config": {"workload": "config 2: one MoE verify layer, T=16, hidden 2048, 512 IQ3_S experts top-10, SwiGLU ff 512, shared expert, f32 router",
                   "weights": args.weights, "shared_expert": "split Q8_0 (dense launches)" if args.shared_q8 else "IQ3_S (inside the window's launches)",
                   "weight_layout": "raw ggml blocks" if args.raw_layout else "unit64 (re-laid once at load, same bytes)", "weight_sets": args.layers, "distinct_experts_per_step": u_mean, "step_algorithmic_bytes": step_bytes,
                   "step_hbm_frac": step_bytes / (ms_per_step * 1e-3) / HBM_PEAK,
                   "ms_per_step_other_weights": None if other_ms is None else {("bytes" if args.weights == "gaussian" else "gaussian"): other_ms},
                   "gemv": gemv, "others": others},
        "roofline": {"bound": "hbm", "kernel": kernel_name, "achieved": achieved / 1e9, "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK, "traffic": traffic, "traffic_source": WINDOW_TRAFFIC["source"] if traffic else None,
                     "kernel_ms": k_ms, "algorithmic_bytes": k_bytes,
                     "window_launch_us": {n_: round(float(v) * 1e3, 2) for n_, v in zip(names, per_launch)},
                     "stream_read_GBps": stream,
                     "frac_of_stream_read_1GiB": None if not stream else achieved / 1e9 / stream["unit64_plane_loads_1GiB"]},
        "cpu_baseline": cpu,
    }
    print(json.dumps(line))


def _rand_iq3s(torch, g, nblocks):
    b = torch.randint(0, 256, (nblocks, IQ3S_BLOCK), dtype=torch.uint8, device="cuda", generator=g)
    d = (torch.rand(nblocks, device="cuda", generator=g) * 3e-4 + 1e-5).to(torch.float16)
    b[:, 0:2] = d.view(torch.uint8).reshape(nblocks, 2)
    return b.reshape(-1)


def gemv_main(args):
    """benchmark config 1 on its own (gemv_measure)"""
    import numpy as np
    import torch
    fnx_gpu = harness()
    dev = fnx_gpu.Dev()
    res = gemv_measure(dev, torch, np, args.steps)
    many, lone = res["launch_of_1024_matrices"], res["lone_matrix_a_launch"]
    line = {"metric": "IQ3_S GEMV achieved HBM GB/s (config 1: 4096 x 2048, T = 1 and 16)", "value": many["T16"]["GBps"], "unit": "GB/s", "n_gpus": 1,
            "steps": max(args.steps, 512), "warmup": 64, "ms_per_step": many["T16"]["us_per_launch"] / 1e3, "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "int8 x IQ3_S (i32 dot, f32 accumulate)", "data": "synthetic: uniformly random IQ3_S blocks",
            "config": {"workload": "config 1: IQ3_S 4096 x 2048 mat-vec over 1,024 distinct matrices, one launch for all (the value) and one launch each",
                       "gemv": res},
            "roofline": {"bound": "hbm", "kernel": "k_iq3s_jobs (unit64, 1,024 jobs of 16 rows)", "achieved": many["T16"]["GBps"], "peak": HBM_PEAK / 1e9,
                         "unit": "GB/s", "frac": many["T16"]["hbm_frac"], "traffic": None,
                         "note": "one matrix a launch (3.6 MB) is bound by the launch: " + f"{lone['T16']['us_per_launch']:.1f} us at T = 16"},
            "cpu_baseline": None}
    return line


def head_main(args):
    """benchmark config 3: argmax over 16 x 151,936 f32 logits (forced to the draft on 70% of the rows), prompt lookup
    over a 38,862-token context with 200 copied spans, greedy acceptance; device forms, one stream."""
    import numpy as np
    import torch
    fnx_gpu = harness()
    oracle_lib = oracle_side()
    dev = fnx_gpu.Dev()
    lib = dev.lib
    oracle = oracle_lib.Oracle()
    rng = np.random.default_rng(3)
    V, NCTX, R = 151936, 38862, 16
    ctx = rng.integers(0, V, NCTX).astype(np.int32)
    for _ in range(200):
        ln, src, dst = int(rng.integers(8, 65)), int(rng.integers(0, NCTX - 200)), int(rng.integers(200, NCTX - 64))
        ctx[dst:dst + ln] = ctx[src:src + ln]
    # the context ends inside a copied span, so the lookup finds a run
    ctx[-12:] = ctx[1000:1012]
    g = torch.Generator(device="cuda")
    g.manual_seed(5)
    NL = 8
    logits = [torch.randn((R, V), device="cuda", generator=g) for _ in range(NL)]
    d1 = int(ctx[1012])
    drafts, match = oracle.lookup_drafts(ctx, 15, d1)
    rows = np.concatenate([[int(ctx[-1])], drafts]).astype(np.int32)[:R]
    keep = rng.random(R) < 0.7
    for lg in logits:   # row j's argmax is the next row's token on 70% of the rows
        for j in range(len(rows) - 1):
            if keep[j]:
                lg[j, int(rows[j + 1])] = lg[j].max() + 1.0
    t = torch
    dctx, dd1 = dev.up(ctx), dev.up(np.array([d1], dtype=np.int32))
    dout, dn, dm = dev.zeros(15, t.int32), dev.zeros(1, t.int32), dev.zeros(1, t.int32)
    drows = dev.up(np.pad(rows, (0, R - len(rows))))
    bv, bi, keys, err, nacc = dev.zeros(R, t.float32), dev.zeros(R, t.int32), dev.zeros(32, t.int64), dev.zeros(1, t.int32), dev.zeros(1, t.int32)
    st = dev.st()

    def timed(fn, n):
        for i in range(20):
            fn(i)
        e0, e1 = t.cuda.Event(enable_timing=True), t.cuda.Event(enable_timing=True)
        t.cuda.synchronize()
        e0.record()
        for i in range(n):
            fn(i)
        e1.record()
        t.cuda.synchronize()
        return e0.elapsed_time(e1) / n * 1e3

    n = max(args.steps, 200)
    us_arg = timed(lambda i: dev.ok(lib.fnx_argmax(logits[i % NL].data_ptr(), V, R, 0, bv.data_ptr(), bi.data_ptr(), keys.data_ptr(), err.data_ptr(), st)), n)
    us_lk = timed(lambda i: dev.ok(lib.fnx_lookup_drafts_dev(dctx.data_ptr(), NCTX, 3, 15, dd1.data_ptr(), dout.data_ptr(), dn.data_ptr(), dm.data_ptr(), st)), n)
    us_acc = timed(lambda i: dev.ok(lib.fnx_accept_greedy_dev(drows.data_ptr(), bi.data_ptr(), len(rows), nacc.data_ptr(), st)), n)

    def all3(i):
        dev.ok(lib.fnx_argmax(logits[i % NL].data_ptr(), V, R, 0, bv.data_ptr(), bi.data_ptr(), keys.data_ptr(), err.data_ptr(), st))
        dev.ok(lib.fnx_accept_greedy_dev(drows.data_ptr(), bi.data_ptr(), len(rows), nacc.data_ptr(), st))
        dev.ok(lib.fnx_lookup_drafts_dev(dctx.data_ptr(), NCTX, 3, 15, dd1.data_ptr(), dout.data_ptr(), dn.data_ptr(), dm.data_ptr(), st))
    us_all = timed(all3, n)
    # the sampler's candidates over the same rows (the non-greedy half of acceptance): 64 a row, no penalty or bias lists
    tk_v, tk_i = dev.zeros((R, 64), t.float32), dev.zeros((R, 64), t.int32)
    us_top = timed(lambda i: dev.ok(lib.fnx_top_tokens(logits[i % NL].data_ptr(), V, R, 0, None, None, None, 0, None, None, None, None, None,
                                                       tk_v.data_ptr(), tk_i.data_ptr(), err.data_ptr(), st)), n)
    # parity on this exact input
    all3(0)
    t.cuda.synchronize()
    o = bi.cpu().numpy()
    _, want_i, _ = oracle.argmax(logits[0].cpu().numpy())
    same = bool(np.array_equal(o, want_i)) and int(nacc.item()) == oracle.accept_greedy(rows, o[:len(rows)]) and \
        list(dout.cpu().numpy()[:int(dn.item())]) == list(drafts) and int(dm.item()) == match
    c0 = time.perf_counter()
    reps = 0
    while args.cpu_seconds > 0 and (time.perf_counter() - c0 < min(args.cpu_seconds, 5.0) or reps < 2):
        oracle.argmax(logits[0].cpu().numpy()) if reps == 0 else None
        oracle.lookup_drafts(ctx, 15, d1)
        oracle.accept_greedy(rows, o[:len(rows)])
        reps += 1
    cpu_us = (time.perf_counter() - c0) / max(reps, 1) * 1e6
    arg_bytes = R * V * 4
    line = {"metric": "verify head: argmax + acceptance + prompt lookup per round (config 3)", "value": 1e6 / us_all, "unit": "rounds/s", "n_gpus": 1,
            "steps": n, "warmup": 20, "ms_per_step": us_all / 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32 compare / int32",
            "data": "synthetic",
            "config": {"workload": "config 3: logits 16 x 151,936 f32, context 38,862 int32 with 200 copied spans, key 3, up to 15 drafts",
                       "argmax_us": us_arg, "lookup_us": us_lk, "accept_us": us_acc, "top_tokens_us": us_top, "drafts": int(len(drafts)), "accepted": int(nacc.item()),
                       "identical_to_oracle": same},
            "roofline": {"bound": "hbm", "kernel": "k_argmax", "achieved": arg_bytes / (us_arg * 1e-6) / 1e9, "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                         "frac": arg_bytes / (us_arg * 1e-6) / HBM_PEAK, "traffic": None, "algorithmic_bytes": arg_bytes,
                         "note": "one launch whose rows' last blocks decode the keys: about 4 us of fixed cost and 3 us for the chain of atomics at its end; the scan itself is 1.2 us at peak"},
            "cpu_baseline": None if not reps else {"value": 1e6 / cpu_us, "unit": "rounds/s", "cores": 1, "kind": "port",
                                                   "sample": f"{reps} rounds of lookup + acceptance on the oracle (the argmax scan once)"}}
    return line


def decoder_main(args):
    """benchmark config 4: a verify step of the reduced decoder (4 layers of GQA attention, 16 q / 2 kv heads of 256, f16
    cache at 32,768 positions, and the config-2 MoE block) over 1 + 15 rows, the output head over 151,936 tokens, greedy
    acceptance, then the draft layer over the same rows. Random weights (the test-suite's model class at full size); a
    step's weights are cold (the ~3.7 GB a step reads exceed the 256 MB cache many times). The CPU leg runs the same step
    once on the oracle and compares the two."""
    import numpy as np
    import torch
    fnx_gpu = harness()
    dev = fnx_gpu.Dev()
    pkg, lib, t = dev.pkg, dev.lib, torch
    g = torch.Generator(device="cuda")
    g.manual_seed(44)
    NQ, NKV, HD, NL, V, CTX, R = 16, 2, 256, 4, 151936, 32768, 16
    oracle = None
    if args.cpu_seconds > 0:
        oracle_lib = oracle_side()
        oracle = oracle_lib.Oracle()
    model = fnx_gpu.SyntheticDecoder(seed=44, n=N, nq=NQ, nkv=NKV, nlayers=NL, vocab=V, max_ctx=CTX, nexp=NEXP, topk=TOPK, ff=FF, cheap_draws=True)
    dd = fnx_gpu.DecoderDev(dev, model)
    rng = np.random.default_rng(45)
    cells = [(rng.standard_normal((CTX - R, NKV, HD), dtype=np.float32).astype(np.float16),
              rng.standard_normal((CTX - R, NKV, HD), dtype=np.float32).astype(np.float16)) for _ in range(NL + 1)]
    dd.set_caches(cells)
    D, M, ws, arr = dd.D, dd.M, dd.ws, dd.layer_arr
    z = dev.zeros
    pos = torch.full((1,), CTX - R, dtype=torch.int32, device="cuda")
    toks = torch.randint(0, V, (8, R), dtype=torch.int32, device="cuda", generator=g)
    nacc = z(1, t.int32)
    st = dev.st()

    def step(i):
        tk = toks[i % 8]
        dev.ok(lib.fnx_decoder_verify(C.byref(D), tk.data_ptr(), R, pos.data_ptr(), C.byref(ws), st))
        dev.ok(lib.fnx_accept_greedy_dev(tk.data_ptr(), ws.best_i, R, nacc.data_ptr(), st))
        dev.ok(lib.fnx_mtp_draft(C.byref(D), C.byref(M), ws.hidden, tk.data_ptr(), R, pos.data_ptr(), C.byref(ws), st))

    steps, warmup = min(args.steps, 50), min(args.warmup, 5)
    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        step(warmup + i)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    # the attention on its own (the K/V scan of one layer): events on the launch stream
    evs = []
    L0 = arr[0]
    caches = [(arr[l].kc, arr[l].vc) for l in range(NL)] + [(M.layer.kc, M.layer.vc)]   # in turn: 335 MB, more than the Infinity Cache holds
    for i in range(23):
        e0, e1 = t.cuda.Event(enable_timing=True), t.cuda.Event(enable_timing=True)
        e0.record()
        kc_, vc_ = caches[i % len(caches)]
        dev.ok(lib.fnx_attn(ws.qg, kc_, vc_, ws.att, NQ, NKV, pos.data_ptr(), R, CTX, ws.attn_scratch, st))
        e1.record()
        evs.append((e0, e1))
    hv = []
    for i in range(13):
        e0, e1 = t.cuda.Event(enable_timing=True), t.cuda.Event(enable_timing=True)
        e0.record()
        dev.ok(lib.fnx_q8s_gemv(C.byref(D.head if i % 2 else M.head), ws.xq, ws.logits, V, R, st))
        e1.record()
        hv.append((e0, e1))
    torch.cuda.synchronize()
    attn_ms = float(np.mean([a.elapsed_time(c) for a, c in evs[3:]]))
    head_ms = float(np.mean([a.elapsed_time(c) for a, c in hv[3:]]))
    # whole decode rounds that the host only enqueues (fnx_decode_round: verify, acceptance, commit, draft layer, prompt
    # lookup and the next window, the state in device words): eagerly, and as replays of one captured round. With random
    # weights no draft is ever right: a window is the last token and one draft, and a round keeps one token.
    NR, P0 = 24, CTX - 4096
    rctx = torch.randint(0, V, (CTX + 64,), dtype=torch.int32, device="cuda", generator=g)
    rstate, rrows, rscratch = z(pkg.RS_WORDS, t.int32), z(16, t.int32), z(16, t.int32)
    RD = pkg.Round(rstate.data_ptr(), rrows.data_ptr(), rctx.data_ptr(), CTX + 64, None, 0, 1, 3, 15, rscratch.data_ptr())

    def reset_rounds():
        rstate.zero_()
        rstate[pkg.RS_NCTX], rstate[pkg.RS_POS], rstate[pkg.RS_ROWS] = P0 + 1, P0, 1
        rrows.zero_()
        rrows[0] = rctx[P0]

    # the same with an MTP chain of three drafts (random weights: the lookup never fires, so every round runs the chain)
    chain_src = z(N, t.float32)
    RD3 = pkg.Round(rstate.data_ptr(), rrows.data_ptr(), rctx.data_ptr(), CTX + 64, None, 0, 1, 3, 15, rscratch.data_ptr(), 3, chain_src.data_ptr())

    def a_round(rd=None):
        dev.ok(lib.fnx_decode_round(C.byref(D), C.byref(M), C.byref(rd if rd is not None else RD), C.byref(ws), dev.st()))

    def timed_rounds(run):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(NR):
            run()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / NR * 1e3

    reset_rounds()
    for _ in range(3):
        a_round()
    round_eager_ms = timed_rounds(a_round)
    kept_eager = int(rstate[pkg.RS_NCTX].item()) - (P0 + 1)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        a_round()
    reset_rounds()
    for _ in range(3):
        graph.replay()
    round_graph_ms = timed_rounds(graph.replay)
    kept_graph = int(rstate[pkg.RS_NCTX].item()) - (P0 + 1)
    assert int(rstate[pkg.RS_STOP].item()) == 0 and int(rstate[pkg.RS_ROUNDS].item()) == NR + 3 and kept_graph == kept_eager, "rounds went wrong"
    reset_rounds()
    for _ in range(3):
        a_round(RD3)
    round_chain_ms = timed_rounds(lambda: a_round(RD3))
    assert int(rstate[pkg.RS_STOP].item()) == 0 and int(rstate[pkg.RS_ROWS].item()) == 4, "the chain's rounds went wrong"
    # what the chain's launches cost a round that does not run it: a stopped session repeats its round, chain switched off
    rstate[pkg.RS_STOP] = 1
    stopped_ms = timed_rounds(a_round)
    stopped_chain_ms = timed_rounds(lambda: a_round(RD3))
    # ---- CPU baseline and parity: the same step (window, acceptance, draft layer) once on the oracle, on the host's cores
    cpu = None
    if oracle is not None:
        threads = min(os.cpu_count() or 1, 16)
        import tiny_decoder as td   # under tests/, on the path since oracle_side()
        sess = td.OracleSession(td.TinyDecoder.of(model, oracle), threads=threads)
        for (kc, vc), (k, v) in zip(sess.caches + [sess.mtp_cache], cells):
            kc[:CTX - R], vc[:CTX - R] = k.view(np.uint16), v.view(np.uint16)
        rows = [int(x) for x in toks[0].cpu().numpy()]
        c0 = time.perf_counter()
        a = sess.verify(rows, CTX - R, routing=True, taps=True)
        na = oracle.accept_greedy(np.asarray(rows, dtype=np.int32), a["best"])
        da = sess.draft(a["hidden"], rows, CTX - R)
        cdt = time.perf_counter() - c0
        dd.set_caches(cells)   # the timed rounds above wrote cells of their own
        got = dd.verify(rows, CTX - R)
        nb = dev.accept(np.asarray(rows, dtype=np.int32), got["best"])
        _, dev_topi = dd.verify_routing(rows, CTX - R)
        same_route = [all(set(dev_topi[l, r_].tolist()) == set(a["route_topi"][l, r_].tolist()) for l in range(NL)) for r_ in range(R)]
        rel = lambda x, y: float(np.linalg.norm(x.astype(np.float64) - y) / np.linalg.norm(y.astype(np.float64)))
        rows_h = [rel(got["hidden"][r_], a["hidden"][r_]) for r_ in range(R) if same_route[r_]]
        rows_l = [rel(got["logits"][r_], a["logits"][r_]) for r_ in range(R) if same_route[r_]]
        gd = dd.draft(a["hidden"], rows, CTX - R)
        # where the chain's rows can part from the oracle's: the q8_1 codes of each layer's output-projection input (the
        # attention's rows), the device's chain walked layer by layer (fnx_decoder_layer: the window's own launches)
        def differ(l, r):
            want_q = oracle.quantize_q8_1(a["taps"]["att"][l]).reshape(r["att_q8"].shape)
            return (int(np.count_nonzero(r["att_q8"][..., 4:] != want_q[..., 4:])) +
                    int(np.count_nonzero(r["att_q8"][..., :2].view(np.uint16) != want_q[..., :2].view(np.uint16))))

        code_steps, own_steps, layer_rel, x = [], [], [], a["taps"]["x_in"][0]
        for l in range(NL):
            r = dd.layer(x, l, CTX - R)
            code_steps.append(differ(l, r))
            x = r["x_mid"] + r["moe"]
            # the same layer on the oracle's own input rows: the steps that start in this layer, and the layer's rows against the oracle's
            r = dd.layer(a["taps"]["x_in"][l], l, CTX - R)
            own_steps.append(differ(l, r))
            layer_rel.append(rel(r["x_mid"] + r["moe"], a["taps"]["x_mid"][l] + a["taps"]["moe"][l]))
        cpu = {"value": 1.0 / cdt, "unit": "steps/s", "cores": threads, "kind": "port",
               "sample": "1 step of the same workload (window of 16 rows at position 32,752, acceptance, draft layer) on the oracle",
               "parity": {"rows_routed_as_the_oracle": int(sum(same_route)), "rows": R,
                          "picks_identical": int(np.count_nonzero(got["best"] == a["best"])), "accepted_cpu_gpu": [int(na), int(nb)],
                          "hidden_rel_l2": rel(got["hidden"][same_route], a["hidden"][same_route]),
                          "logits_rel_l2": rel(got["logits"][same_route], a["logits"][same_route]),
                          "hidden_rel_l2_rows_max": max(rows_h), "hidden_rel_l2_rows_median": float(np.median(rows_h)),
                          "logits_rel_l2_rows_max": max(rows_l), "logits_rel_l2_rows_median": float(np.median(rows_l)),
                          "draft_picks_identical": int(np.count_nonzero(gd["best"] == da["best"])),
                          "draft_hidden_rel_l2": rel(gd["hidden"], da["hidden"]),
                          "q8_1_codes_and_scales_that_differ_at_each_layers_output_projection_input": code_steps,
                          "codes_there_per_layer": int(R * NQ * HD),
                          "the_same_with_each_layer_fed_the_oracles_rows": own_steps,
                          "layer_output_rel_l2_with_each_layer_fed_the_oracles_rows": layer_rel,
                          "note": "float figures over the rows whose ten experts are the oracle's in every layer (a row that parts does so at a near-tie of "
                                  "two router logits: tests/test_gpu_full_shapes.py proves it per row). The MoE half is the oracle's bit for bit on equal "
                                  "inputs; the attention's rows differ in the last bits (MFMA sums, sin/cos), which now and then moves one q8_1 code of the "
                                  "output projection's input by one step (counted above, per layer): ~1e-3 of that row, carried on by the layers after it; "
                                  "rows without a step upstream are the oracle's bit for bit. A layer fed the oracle's own rows meets 1e-3 over the whole tensor and starts a handful of "
                                  "steps at most; the counts of the chain's later layers are those first steps' consequences (rows already 1e-3 apart flip codes by the percent)"}}
    kv_bytes = 2 * CTX * NKV * HD * 2
    head_bytes = V * N + V * (N // 32) * 2
    dense_bytes = (NQ * 2 * HD * N + 2 * NKV * HD * N + N * NQ * HD) * 34 // 32
    moe_bytes = 139.2 * (GU_BYTES + DN_BYTES) + (GU_BYTES + DN_BYTES) + ROUTER_BYTES
    step_bytes = (NL + 1) * (kv_bytes + dense_bytes + moe_bytes) + 2 * head_bytes + 2 * N * N * 34 // 32
    line = {"metric": "verify steps/sec of the reduced decoder + draft layer (config 4)", "value": steps / dt, "unit": "steps/s", "n_gpus": 1,
            "steps": steps, "warmup": warmup, "ms_per_step": dt / steps * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "int8 dot (IQ3_S, Q8_0) + f32 attention on an f16 cache", "data": "synthetic",
            "config": {"workload": "config 4: 4 layers (GQA 16q/2kv x 256 at 32,768 positions + MoE as config 2) + head 151,936 + acceptance + draft layer, 16 rows",
                       "step_algorithmic_bytes": step_bytes, "step_hbm_frac": step_bytes / (dt / steps) / HBM_PEAK,
                       "attention_ms_per_layer": attn_ms, "attention_GBps": kv_bytes / (attn_ms * 1e-3) / 1e9, "head_ms": head_ms,
                       "head_GBps": head_bytes / (head_ms * 1e-3) / 1e9,
                       "decode_round": {"what": "verify 16 rows (2 count) + accept + commit + draft layer + lookup + next window at position 28,672, no host wait",
                                        "rounds": NR, "ms_eager": round_eager_ms, "ms_graph_replay": round_graph_ms,
                                        "tokens_kept_per_round": kept_graph / (NR + 3),
                                        "ms_eager_with_chain_of_3": round_chain_ms,
                                        "ms_two_chain_steps_switched_off": stopped_chain_ms - stopped_ms}},
            "roofline": {"bound": "hbm", "kernel": "k_q8s_gemv (output head 151,936 x 2048)", "achieved": head_bytes / (head_ms * 1e-3) / 1e9,
                         "peak": HBM_PEAK / 1e9, "unit": "GB/s", "frac": head_bytes / (head_ms * 1e-3) / HBM_PEAK, "traffic": None, "kernel_ms": head_ms,
                         "algorithmic_bytes": head_bytes},
            "cpu_baseline": cpu}
    return line


def prefill_main(args):
    """benchmark config 5: one MoE layer over prompt chunks of 512 rows (5,120 routed pairs), expert popularity Zipf(1.1)
    imposed through a constant input feature and a bias column of the router. A step = one chunk."""
    import numpy as np
    import torch
    fnx_gpu = harness()
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
        gu64 = pkg.dw(gu, N, 2 * FF, packed=True)   # the unit64 copy's descriptor, kept for the two-launch leg
        L = pkg.MoeLayer(N, FF, NEXP, TOPK, router.data_ptr(), 0, gu64, GU_BYTES, pkg.dw(down, FF, N, packed=True),
                         DN_BYTES, pkg.dw(sh_gu, N, 2 * FF, packed=True), pkg.dw(sh_down, FF, N, packed=True))
        if not args.raw_layout:   # the gate|up matrices in the prompt path's own layout beside the unit64 copy
            gu16 = torch.zeros(lib.fnx_iq3s_tile16_bytes(2 * FF, N, NEXP), dtype=torch.uint8, device="cuda")
            sh16 = torch.zeros(lib.fnx_iq3s_tile16_bytes(2 * FF, N, 1), dtype=torch.uint8, device="cuda")
            dev.ok(lib.fnx_iq3s_tile16(gu.data_ptr(), gu16.data_ptr(), 2 * FF, N, NEXP, dev.st()))
            dev.ok(lib.fnx_iq3s_tile16(sh_gu.data_ptr(), sh16.data_ptr(), 2 * FF, N, 1, dev.st()))
            L.gu, L.gu_stride, L.sh_gu = pkg.dw(gu16, N, 2 * FF, tile16=True), lib.fnx_iq3s_tile16_bytes(2 * FF, N, 1), pkg.dw(sh16, N, 2 * FF, tile16=True)
            ws_ = ws_ + [gu16, sh16]
            if not args.down_unit64:   # and the down matrices
                dn16 = torch.zeros(lib.fnx_iq3s_tile16_bytes(N, FF, NEXP), dtype=torch.uint8, device="cuda")
                shd16 = torch.zeros(lib.fnx_iq3s_tile16_bytes(N, FF, 1), dtype=torch.uint8, device="cuda")
                dev.ok(lib.fnx_iq3s_tile16(down.data_ptr(), dn16.data_ptr(), N, FF, NEXP, dev.st()))
                dev.ok(lib.fnx_iq3s_tile16(sh_down.data_ptr(), shd16.data_ptr(), N, FF, 1, dev.st()))
                L.down, L.down_stride, L.sh_down = pkg.dw(dn16, FF, N, tile16=True), lib.fnx_iq3s_tile16_bytes(N, FF, 1), pkg.dw(shd16, FF, N, tile16=True)
                ws_ = ws_ + [dn16, shd16]
        layers.append((L, router, ws_, raw, gu64))
    NX = 8
    xs = torch.randn((NX, CH, N), device="cuda", generator=g)
    xs[:, :, 0] = 1.0   # the constant feature the router's bias column multiplies
    outs = torch.zeros((NX, CH, N), device="cuda")
    P = CH * TOPK
    J, S = P // PF + NEXP, (CH + PF - 1) // PF
    order = ("logits", "topi", "topw", "cnt", "jbase", "jobs_gu", "jobs_dn", "njobs", "xh", "gu", "h16", "part")

    def workspace():
        bufs = dict(logits=dev.zeros((CH, NEXP + 1), t.float32), topi=dev.zeros((CH, TOPK), t.int32), topw=dev.zeros((CH, TOPK), t.float32),
                    cnt=dev.zeros(NEXP, t.int32), jbase=dev.zeros(NEXP, t.int32), jobs_gu=dev.zeros((J + S, 130), t.int32),
                    jobs_dn=dev.zeros((J + S, 130), t.int32), njobs=dev.zeros(2, t.int32), xh=dev.zeros((CH, N), t.float16),
                    gu=dev.zeros((P + CH, 2 * FF), t.float32), h16=dev.zeros((P + CH, FF), t.float16), part=dev.zeros((P + CH, N), t.float32))
        return bufs, pkg.PfWs(*[bufs[k].data_ptr() for k in order])

    b, ws = workspace()
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
    # Two chunks in flight: the chunks of a prompt are independent within a layer, so a caller may give every other chunk
    # a stream and a workspace of its own; one chunk's small routing launches then run beside the other's big ones.
    # (Reported beside the metric, which stays one chunk after the other on one stream.)
    dt2 = None
    if not args.no_extras:
        b2, ws2 = workspace()
        streams = [torch.cuda.Stream(), torch.cuda.Stream()]
        both = [(ws, streams[0]), (ws2, streams[1])]

        def step2(i):
            w, s_ = both[i & 1]
            dev.ok(lib.fnx_moe_prefill_layer(C.byref(layers[i % nsets][0]), xs[i % NX].data_ptr(), CH, outs[i % NX].data_ptr(), C.byref(w), s_.cuda_stream))

        for i in range(4):
            step2(i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(steps):
            step2(4 + i)
        torch.cuda.synchronize()
        dt2 = time.perf_counter() - t0
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
    fused_h = not args.raw_layout   # tile16 gate|up matrices leave h = silu(gate) * up from the gate|up launch itself
    evs = []
    for i in range(reps + 3):
        L = layers[i % nsets][0]
        step(i)   # routes chunk i: the jobs and xh in the workspace are this chunk's
        e = [torch.cuda.Event(enable_timing=True) for _ in range(5)]
        e[0].record()
        # the products as a launch of their own (fnx_moe_gate_up_mma takes raw blocks and unit64: the unit64 copy), then SwiGLU
        dev.ok(lib.fnx_moe_gate_up_mma(C.byref(layers[i % nsets][4]), GU_BYTES, ws.jobs_gu, ws.njobs, J, ws.xh, ws.gu, st))
        e[1].record()
        dev.ok(lib.fnx_swiglu_h16(ws.gu, FF, P + CH, ws.h16, st))
        e[2].record()
        if fused_h:   # what the layer runs: h from one launch
            dev.ok(lib.fnx_moe_gate_up_h16_mma(C.byref(L.gu), L.gu_stride, ws.jobs_gu, ws.njobs, J, ws.xh, ws.h16, st))
        e[3].record()
        dev.ok(lib.fnx_moe_down_mma(C.byref(L.down), L.down_stride, ws.jobs_dn, ws.njobs, J, ws.h16, ws.part, st))
        e[4].record()
        evs.append(e)
    torch.cuda.synchronize()
    gu2_ms = float(np.mean([e[0].elapsed_time(e[1]) for e in evs[3:]]))
    sw_ms = float(np.mean([e[1].elapsed_time(e[2]) for e in evs[3:]]))
    gu_ms = float(np.mean([e[2].elapsed_time(e[3]) for e in evs[3:]])) if fused_h else gu2_ms
    dn_ms = float(np.mean([e[3].elapsed_time(e[4]) for e in evs[3:]]))
    # the reference's other prompt family (kernels.hpp:324-325, its moe_q8 mode): the same jobs over q8_1 activations on the int8
    # matrix cores - a stated option beside the metric's f16 family, whose results differ from it by the q8_1 rounding
    q8 = None
    if not args.raw_layout and not args.down_unit64 and not args.no_extras:
        xq = torch.zeros(CH * (N // 32) * 36, dtype=torch.uint8, device="cuda")
        evq = []
        for i in range(reps + 3):
            L = layers[i % nsets][0]
            step(i)
            e = [torch.cuda.Event(enable_timing=True) for _ in range(4)]
            e[0].record()
            dev.ok(lib.fnx_quantize_q8_1(xs[i % NX].data_ptr(), xq.data_ptr(), N, CH, st))
            e[1].record()
            dev.ok(lib.fnx_moe_gate_up_big(C.byref(L.gu), L.gu_stride, ws.jobs_gu, ws.njobs, J, xq.data_ptr(), ws.gu, st))
            e[2].record()
            dev.ok(lib.fnx_moe_down_big(C.byref(L.down), L.down_stride, ws.jobs_dn, ws.njobs, J, ws.gu, ws.part, st))
            e[3].record()
            evq.append(e)
        torch.cuda.synchronize()
        q8 = {"quantize_us": float(np.mean([e[0].elapsed_time(e[1]) for e in evq[3:]])) * 1e3,
              "gate_up_big_us": float(np.mean([e[1].elapsed_time(e[2]) for e in evq[3:]])) * 1e3,
              "down_big_us": float(np.mean([e[2].elapsed_time(e[3]) for e in evq[3:]])) * 1e3,
              "note": "routed jobs only, k_iq3s_jobs_mma16<1 | 2> over the tile16 copies; the f16 family's routed launches beside them: "
                      f"{gu_ms * 1e3:.1f} + {dn_ms * 1e3:.1f} us"}
    # the routed gate|up launch: the experts' matrices, x as f16, and h as f16 (the products themselves, f32, where h is a launch of its own)
    gu_bytes = u_mean * GU_BYTES + CH * N * 2 + (P * FF * 2 if fused_h else P * 2 * FF * 4)
    dn_bytes = u_mean * DN_BYTES + P * FF * 2 + P * N * 4
    gu_flops, dn_flops = 2.0 * P * 2 * FF * N, 2.0 * P * N * FF
    step_bytes = (u_mean + 1) * (GU_BYTES + DN_BYTES) + ROUTER_BYTES + 2 * CH * N * 4
    step_flops = 2.0 * (P + CH) * 3 * FF * N + 2.0 * CH * (NEXP + 1) * N
    MFMA_F16 = 2.5e15
    cpu = None
    if args.cpu_seconds > 0:
        oracle_lib = oracle_side()
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
    gu_kernel = ("k_moe_mma (routed gate|up over unit64, a wave a task of 32 rows x 32 tokens; h by fnx_swiglu_h16)" if args.raw_layout else
                 "k_moe_mma_wave16_gu (routed gate|up over tile16, leaves h = silu(gate) * up; a wave a pair of gate and up tiles, a job's up to 64 tokens a decode)")
    line = {
        "metric": "prefill MoE tokens/sec per layer (chunks of 512 rows) + grouped IQ3_S expert GEMM achieved GB/s and MFMA utilisation",
        "value": CH * steps / dt, "unit": "tokens/s per layer", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": dt / steps * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16 x f16 (IQ3_S dequantised once to f16), f32 accumulate", "data": "synthetic",
        "config": {"workload": "config 5: one MoE layer over prompt chunks of 512 rows, 5,120 routed pairs, 512 IQ3_S experts top-10 with Zipf(1.1) popularity, shared expert",
                   "weight_sets": nsets, "active_experts_per_chunk": u_mean, "jobs_per_chunk": j_mean, "step_algorithmic_bytes": step_bytes,
                   "step_flops": step_flops, "step_hbm_frac": step_bytes / (dt / steps) / HBM_PEAK, "step_mfma_frac": step_flops / (dt / steps) / MFMA_F16},
        "roofline": {"bound": "hbm", "kernel": gu_kernel, "achieved": gu_bytes / (gu_ms * 1e-3) / 1e9, "peak": HBM_PEAK / 1e9,
                     "unit": "GB/s", "frac": gu_bytes / (gu_ms * 1e-3) / HBM_PEAK,
                     "traffic": PF_WINDOW_TRAFFIC["bytes"] * gu_bytes / PF_WINDOW_TRAFFIC["algorithmic_bytes"] if nsets == 4 and not args.raw_layout else None,
                     "traffic_source": PF_WINDOW_TRAFFIC["source"] if nsets == 4 and not args.raw_layout else None, "kernel_ms": gu_ms, "algorithmic_bytes": gu_bytes,
                     "mfma_tflops": gu_flops / (gu_ms * 1e-3) / 1e12, "mfma_frac": gu_flops / (gu_ms * 1e-3) / MFMA_F16,
                     "down": {"kernel": "k_moe_mma (unit64)" if args.down_unit64 or args.raw_layout else "k_moe_mma_wave16 (tile16)", "kernel_ms": dn_ms, "achieved": dn_bytes / (dn_ms * 1e-3) / 1e9, "mfma_tflops": dn_flops / (dn_ms * 1e-3) / 1e12},
                     "two_launches": {"gate_up_ms": gu2_ms, "swiglu_ms": sw_ms, "note": "fnx_moe_gate_up_mma (k_moe_mma over the unit64 copy, f32 products written) and fnx_swiglu_h16"},
                     # the piecewise bound: a launch cannot be faster than its bytes at the HBM peak or its flops at the MFMA peak
                     "piecewise_bound": {"gate_up_us": max(gu_bytes / HBM_PEAK, gu_flops / MFMA_F16) * 1e6,
                                         "gate_up_frac": max(gu_bytes / HBM_PEAK, gu_flops / MFMA_F16) / (gu_ms * 1e-3),
                                         "chunk_us": max(step_bytes / HBM_PEAK, step_flops / MFMA_F16) * 1e6,
                                         "chunk_frac": max(step_bytes / HBM_PEAK, step_flops / MFMA_F16) / (dt / steps)}},
        "cpu_baseline": cpu,
        # not the metric: two streams with a workspace each, chunks dealt to them in turn
        "two_chunks_in_flight": {"ms_per_chunk": dt2 / steps * 1e3, "tokens_per_s": CH * steps / dt2} if dt2 else None,
        "q8_1_family": q8,
    }
    return line


if __name__ == "__main__":
    main()
