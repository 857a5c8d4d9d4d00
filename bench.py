#!/usr/bin/env python3
"""Benchmark of the AutogradExtension hot path on one MI355X.

A step is one conv2dBackwardData + conv2dBackwardFilterBias at the ResNet-50
stage-2 3x3 shape (input 56x56x64, batch 32, 64 filters, stride 1, pad 1); the
headline value is the pair's TFLOP/s over exactly --steps steps.  The
bandwidth-bound half of the metric (batchnormBackward at 56x56x256x32,
pool2dBackward max/avg 3x3 s2 p1 at 112x112x64x32) is timed the same way in
its own loops and reported in `ops`, with whole buffer sets (inputs AND outputs)
rotated over more than 512 MB so that no call finds its operands in the 256 MB
memory-side cache.  Every figure is the median of 5 timed repeats of --steps calls.

`--step resnet50|speech` instead runs whole training steps through the C++ host
layer (flashlight_amd/lib/flhip_step_bench) and prints their time with a breakdown
per operation class.

All inputs are resident in HBM before any timed region starts.  Timing uses HIP
events on the stream the kernels are launched on (torch's current stream, whose
handle is passed through the C ABI).
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK = {"hbm_GBps": 8000.0, "f32_TFLOPs": 157.3, "bf16_TFLOPs": 2500.0}
CONV_FLOP = 2 * 32 * 64 * 56 * 56 * 64 * 9          # one pass, 7.398752256e9
# HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs, scaled by
# the same counters on the library's copy kernel (see profiles/); None = not measured.
MEASURED_TRAFFIC = {"conv2d_bwd_data_f32": 61.7e6, "conv2d_bwd_filter_f32": 93.7e6,
                    "conv2d_bwd_data_bf16": 37.0e6, "conv2d_bwd_filter_bf16": 45.3e6}
# where those constants come from: they are typed in from that file, not read from a run of this script
TRAFFIC_SOURCE = "profiles/bench_conv3x3_bn_pool__hbm_traffic_sq_counters.md"


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=0, help="timed steps (default 100; 20 for --step)")
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--dtype", choices=["f32", "bf16", "f16"], default="f32",
                    help="storage type (f16: with --layers, --plans or --step)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--only", default="", help="comma list of ops to time (debugging/profiling)")
    ap.add_argument("--layers", choices=["resnet50", "speech"], default="",
                    help="instead of the bench line: time every conv layer of configs[4] (ResNet-50, batch 32) "
                         "or configs[3] (21x1 speech layers) in all three passes and print a table")
    ap.add_argument("--plans", choices=["resnet50", "speech"], default="",
                    help="instead of the bench line: time every kernel family (plan) of the two backward passes "
                         "on the layers of a network and list where the fastest is not the default rule's choice")
    ap.add_argument("--step", choices=["resnet50", "speech"], default="",
                    help="instead of the bench line: a whole training step of configs[4] (ResNet-50, 224x224x3) or "
                         "configs[3] (speech stack) through the host modules, with a per-operation-class breakdown")
    ap.add_argument("--batch", type=int, default=0, help="batch size for --step (default 64 / 16) and --layers (default 32 / 16)")
    ap.add_argument("--repeats", type=int, default=5, help="timed repeats of --steps calls; the median is reported")
    ap.add_argument("--rnn", action="store_true",
                    help="instead of the bench line: time rnn / rnnBackward (LSTM, GRU) at a few sizes")
    ap.add_argument("--linear", action="store_true",
                    help="instead of the bench line: time fl::linear's forward product and backward pass (dx, dW, db) "
                         "at the sizes of a speech model's layers, in --dtype")
    return ap.parse_args()


def main():
    a = parse()
    if a.steps <= 0:
        a.steps = 20 if a.step else 100
    if a.gpus != 1:
        sys.stderr.write("bench.py: this build runs on one GPU; --gpus %d is not supported "
                         "(no collectives or sharding are part of it)\n" % a.gpus)
        return 2
    if a.step:
        return step_bench(a)
    import torch
    if not torch.cuda.is_available():
        sys.stderr.write("bench.py: no GPU visible\n")
        return 1
    import flashlight_amd as fa
    fa.capi.lib()                      # fails loudly when the HIP library is missing
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    tdt = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}[a.dtype]
    if a.layers:
        return layer_sweep(a, fa, torch, tdt)
    if a.plans:
        return plan_sweep(a, fa, torch, tdt)
    if a.rnn:
        return rnn_sweep(a, fa, torch)
    if a.linear:
        return linear_sweep(a, fa, torch)
    if a.dtype == "f16":
        print("bench.py: --dtype f16 goes with --layers, --plans or --step (the bench line is quoted in f32, with bf16 beside it)",
              file=sys.stderr)
        return 1
    gen = torch.Generator(device=dev).manual_seed(0)

    def randn(*shape, scale=1.0, shift=0.0):
        return torch.randn(shape, device=dev, generator=gen) * scale + shift

    def timed(fn, steps, warmup, spread=None):
        """Seconds per call: `repeats` brackets of exactly `steps` calls each (HIP events on
        the launch stream), the median bracket reported; `spread` receives min and max."""
        for i in range(warmup):
            fn(i)
        torch.cuda.synchronize()
        runs = []
        for _ in range(max(a.repeats, 1)):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            t0 = time.perf_counter()
            e0.record()
            for i in range(steps):
                fn(i)
            e1.record()
            torch.cuda.synchronize()
            runs.append((e0.elapsed_time(e1) * 1e-3 / steps, (time.perf_counter() - t0) / steps))
        runs.sort()
        if spread is not None:
            spread["us_min"], spread["us_max"] = runs[0][0] * 1e6, runs[-1][0] * 1e6
        return runs[len(runs) // 2]

    only = set(x for x in a.only.split(",") if x)
    want = lambda name: not only or name in only
    ops = []

    # The timed loops call the C ABI directly on preallocated outputs and
    # workspaces (a few microseconds of host time per call), so the GPU never
    # waits for Python.
    import ctypes as C
    from flashlight_amd import capi
    L = capi.lib()
    S = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    P = lambda t: C.c_void_p(t.data_ptr())

    def checked(fn):
        """Runs fn once and raises on a non-zero status; returns fn."""
        capi.check(fn(0))
        return fn

    # ---- conv pair at cfg 2 --------------------------------------------------
    pair_info = {}

    def conv_block(dname, headline):
        """Times the conv ops of cfg 2 in storage type `dname`.  Every figure comes twice: with whole
        operand sets (x, dy, y, dx, dw, db) rotated over more than 512 MB per op, so that no call finds
        its operands in the 256 MB memory-side cache (`us`), and on one set (`us_cache_warm`)."""
        tag = capi.F32 if dname == "f32" else capi.BF16
        ttype = torch.float32 if dname == "f32" else torch.bfloat16
        esz = 4 if dname == "f32" else 2
        nsets = 11 * 4 // esz          # two tensors of 25.7 MB (fp32) per op and set: 565 MB per op
        w = randn(64, 64, 3, 3, scale=1.0 / 24.0).to(ttype)          # Kaiming normal, fan-in 576
        b = randn(64)
        xs = [randn(32, 64, 56, 56).to(ttype) for _ in range(nsets)]
        dys = [randn(32, 64, 56, 56).to(ttype) for _ in range(nsets)]
        ys = [torch.empty_like(xs[0]) for _ in range(nsets)]
        dxs = [torch.empty_like(xs[0]) for _ in range(nsets)]
        dws = [torch.empty((64, 64, 3, 3), device=dev) for _ in range(nsets)]
        dbs = [torch.empty(64, device=dev) for _ in range(nsets)]
        cd = capi.ConvDesc(32, 64, 56, 56, 64, 3, 3, 1, 1, 1, 1, 1, 1, 1, tag)
        nws = L.flhip_conv2d_workspace_bytes(C.byref(cd), capi.CONV_BWD_FILTER)
        nws_f = L.flhip_conv2d_workspace_bytes(C.byref(cd), capi.CONV_FWD)
        nws_d = L.flhip_conv2d_workspace_bytes(C.byref(cd), capi.CONV_BWD_DATA)
        ws = torch.empty(max(nws, 16), dtype=torch.uint8, device=dev)
        ws_f = torch.empty(max(nws_f, 16), dtype=torch.uint8, device=dev)
        ws_d = torch.empty(max(nws_d, 16), dtype=torch.uint8, device=dev)
        peak_mfma = PEAK["f32_TFLOPs"] if dname == "f32" else PEAK["bf16_TFLOPs"]
        cdp, wp, bp, wsp, wsfp, wsdp = C.byref(cd), P(w), P(b), P(ws), P(ws_f), P(ws_d)
        xp, dyp, yp, dxp = [P(t) for t in xs], [P(t) for t in dys], [P(t) for t in ys], [P(t) for t in dxs]
        dwp, dbp = [P(t) for t in dws], [P(t) for t in dbs]
        f_fwd = checked(lambda i: L.flhip_conv2d_fwd(cdp, xp[i % nsets], wp, bp, yp[i % nsets], wsfp, nws_f, S))
        f_bwd_data = checked(lambda i: L.flhip_conv2d_bwd_data(cdp, dyp[i % nsets], wp, dxp[i % nsets], wsdp, nws_d, S))
        f_bwd_filter = checked(lambda i: L.flhip_conv2d_bwd_filter(cdp, xp[i % nsets], dyp[i % nsets], dwp[i % nsets],
                                                                   dbp[i % nsets], wsp, nws, S))

        def conv_pair(i):
            f_bwd_data(i)
            f_bwd_filter(i)

        res = (None, None)
        tensor_bytes = xs[0].numel() * esz
        if want("conv_pair"):
            sp = {}
            res = timed(conv_pair, a.steps, a.warmup, sp)
            warm, _ = timed(lambda i: conv_pair(0), a.steps, a.warmup)
            ach = 2 * CONV_FLOP / res[0] / 1e12
            pair_info[dname] = {"us": res[0] * 1e6, "us_cache_warm": warm * 1e6, "achieved": ach, "peak": peak_mfma,
                                "frac": ach / peak_mfma, "achieved_cache_warm": 2 * CONV_FLOP / warm / 1e12,
                                "buffer_sets_rotated": nsets, "rotation_footprint_MB": nsets * 3 * tensor_bytes / 1e6, **sp}
        for name, fn, ntens in (("conv2d_fwd", f_fwd, 2), ("conv2d_bwd_data", f_bwd_data, 2),
                                ("conv2d_bwd_filter_bias", f_bwd_filter, 2)):
            if not want(name):
                continue
            sp = {}
            s, _ = timed(fn, a.steps, a.warmup, sp)
            warm, _ = timed(lambda i: fn(0), a.steps, a.warmup)
            ach = CONV_FLOP / s / 1e12
            ops.append({"op": name, "workload": "32x64x56x56, 64 filters 3x3 s1 p1", "dtype": dname,
                        "us": s * 1e6, "bound": "mfma", "achieved": ach, "peak": peak_mfma,
                        "unit": "TFLOP/s", "frac": ach / peak_mfma, "buffer_sets_rotated": nsets,
                        "rotation_footprint_MB": nsets * ntens * tensor_bytes / 1e6,
                        "us_cache_warm": warm * 1e6, "TFLOPs_cache_warm": CONV_FLOP / warm / 1e12, **sp})
        del xs, dys, ys, dxs
        return res if headline else (None, None)

    pair_s, pair_wall = conv_block(a.dtype, True)
    # the same ops in the other storage type (bf16 storage, fp32 accumulate, when the
    # headline runs in fp32): listed under "ops", not part of `value`
    other = "bf16" if a.dtype == "f32" else "f32"
    if not only or "other_dtype" in only:
        conv_block(other, False)

    # ---- bandwidth ops at cfg 3 (fp32) ----------------------------------------
    def bw_op(name, workload, nbytes, fn, nsets, footprint):
        if not want(name):
            return
        checked(fn)
        sp = {}
        s, _ = timed(fn, a.steps, a.warmup, sp)
        ach = nbytes / s / 1e9
        # the same call on one buffer set every time: operands may sit in the 256 MB
        # memory-side cache (reported beside the cold figure, never as `achieved`)
        warm, _ = timed(lambda i: fn(0), a.steps, a.warmup)
        ops.append({"op": name, "workload": workload, "dtype": "f32", "us": s * 1e6,
                    "bound": "hbm", "achieved": ach, "peak": PEAK["hbm_GBps"], "unit": "GB/s",
                    "frac": ach / PEAK["hbm_GBps"], "algorithmic_bytes": nbytes,
                    "buffer_sets_rotated": nsets, "rotation_footprint_MB": footprint / 1e6,
                    "us_cache_warm": warm * 1e6, "GBps_cache_warm": nbytes / warm / 1e9, **sp})

    if want("batchnorm_bwd") or want("batchnorm_fwd_train"):
        nsets = 3            # x, dy and the output of every set: 3 x 308 MB
        bx = [randn(32, 256, 56, 56, scale=2 ** 0.5, shift=0.5) for _ in range(nsets)]
        bdy = [randn(32, 256, 56, 56) for _ in range(nsets)]
        bout = [torch.empty_like(bx[0]) for _ in range(nsets)]
        gamma = randn(256, scale=0.1, shift=1.0)
        beta = torch.zeros(256, device=dev)
        rm, rv = torch.zeros(256, device=dev), torch.ones(256, device=dev)
        dg, dbt = torch.empty(256, device=dev), torch.empty(256, device=dev)
        T = bx[0].numel() * 4
        bd = capi.BnDesc(32, 256, 56 * 56, capi.F32)
        bnws = L.flhip_bn_workspace_bytes(C.byref(bd))
        bws = torch.empty(max(bnws, 16), dtype=torch.uint8, device=dev)
        sm = [torch.empty(256, device=dev) for _ in range(nsets)]
        si = [torch.empty(256, device=dev) for _ in range(nsets)]
        bdp, bwsp = C.byref(bd), P(bws)
        bxp, bdyp, boutp = [P(t) for t in bx], [P(t) for t in bdy], [P(t) for t in bout]
        smp, sip = [P(t) for t in sm], [P(t) for t in si]
        gp, btp, rmp, rvp, dgp, dbtp = P(gamma), P(beta), P(rm), P(rv), P(dg), P(dbt)
        f_bn_fwd = lambda i: L.flhip_bn_fwd_train(bdp, bxp[i % nsets], gp, btp, boutp[i % nsets],
                                                  smp[i % nsets], sip[i % nsets], rmp, rvp,
                                                  0.1, 1e-5, bwsp, bnws, S)
        for i in range(nsets):
            capi.check(f_bn_fwd(i))
        bw_op("batchnorm_fwd_train", "56x56x256x32, axes {2}", 2 * T, f_bn_fwd, nsets, nsets * 2 * T)
        bw_op("batchnorm_bwd", "56x56x256x32, axes {2}", 3 * T,
              lambda i: L.flhip_bn_bwd(bdp, bxp[i % nsets], bdyp[i % nsets], gp, smp[i % nsets],
                                       sip[i % nsets], boutp[i % nsets], dgp, dbtp, bwsp, bnws, S),
              nsets, nsets * 3 * T)
        del bx, bdy, bout

    if any(want(n) for n in ("pool2d_max_fwd", "pool2d_max_bwd", "pool2d_avg_fwd", "pool2d_avg_bwd")):
        nsets = 5            # x (or dx), y (or dy) and the argmax bytes of every set: 5 x 135 MB
        px_ = [torch.round(randn(32, 64, 112, 112) * 8) / 8 for _ in range(nsets)]
        pdy = [randn(32, 64, 56, 56) for _ in range(nsets)]
        pam = [torch.empty((32, 64, 56, 56), dtype=torch.uint8, device=dev) for _ in range(nsets)]
        pyo = [torch.empty((32, 64, 56, 56), device=dev) for _ in range(nsets)]
        pdx = [torch.empty((32, 64, 112, 112), device=dev) for _ in range(nsets)]
        pdm = capi.PoolDesc(32, 64, 112, 112, 3, 3, 2, 2, 1, 1, 0, capi.F32)
        pda = capi.PoolDesc(32, 64, 112, 112, 3, 3, 2, 2, 1, 1, 2, capi.F32)
        pdmp, pdap = C.byref(pdm), C.byref(pda)
        pyop, pdxp = [P(t) for t in pyo], [P(t) for t in pdx]
        pxp, pdyp, pamp = [P(t) for t in px_], [P(t) for t in pdy], [P(t) for t in pam]
        f_max_fwd = lambda i: L.flhip_pool2d_fwd(pdmp, pxp[i % nsets], pyop[i % nsets], pamp[i % nsets], S)
        for i in range(nsets):
            capi.check(f_max_fwd(i))
        nx, ny = px_[0].numel() * 4, pdy[0].numel() * 4
        wl = "112x112x64x32, 3x3 s2 p1"
        bw_op("pool2d_max_fwd", wl, nx + ny + ny // 4, f_max_fwd, nsets, nsets * (nx + ny + ny // 4))
        bw_op("pool2d_max_bwd", wl, nx + ny + ny // 4,
              lambda i: L.flhip_pool2d_bwd(pdmp, pdyp[i % nsets], pamp[i % nsets], pdxp[i % nsets], S),
              nsets, nsets * (nx + ny + ny // 4))
        bw_op("pool2d_avg_fwd", wl, nx + ny,
              lambda i: L.flhip_pool2d_fwd(pdap, pxp[i % nsets], pyop[i % nsets], None, S), nsets, nsets * (nx + ny))
        bw_op("pool2d_avg_bwd", wl, nx + ny,
              lambda i: L.flhip_pool2d_bwd(pdap, pdyp[i % nsets], None, pdxp[i % nsets], S), nsets,
              nsets * (nx + ny))
        del px_, pdy, pam, pyo, pdx

    if "copy" in only:
        # known-size kernel for calibrating hardware byte counters (never part of the default run)
        ca = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
        cb = torch.empty_like(ca)
        cap, cbp = P(ca), P(cb)
        bw_op("copy", "flhip_copy_bytes 256 MiB", 2 * (256 << 20),
              lambda i: L.flhip_copy_bytes(cap, cbp, 256 << 20, S), 1, 2 * (256 << 20))

    torch.cuda.synchronize()
    by = {}
    for o in ops:
        other_conv = o["op"].startswith("conv2d") and o["dtype"] != a.dtype
        by.setdefault(o["op"] + "_" + o["dtype"] if other_conv else o["op"], o)

    # ---- CPU baselines (rank 0, bounded sample) --------------------------------
    cpu_port = cpu_onednn = cpu_bw = None
    if not a.no_cpu and not only:
        cpu_port, cpu_onednn = cpu_legs()
        cpu_bw = cpu_bandwidth_legs()

    out = {
        "metric": "TFLOP/s conv2dBackwardData+Filter (ResNet-50 3x3) + GB/s BN/pool backward, 1 GPU",
        "value": (2 * CONV_FLOP / pair_s / 1e12) if pair_s else None,
        "unit": "TFLOP/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": pair_s * 1e3 if pair_s else None, "repeats": a.repeats,
        "wall_ms_per_step": pair_wall * 1e3 if pair_wall else None,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": a.dtype, "data": "synthetic",
        "config": {"workload": "configs[1]: conv2dBackwardData + conv2dBackwardFilterBias, input "
                               "56x56x64 batch 32, 64 filters 3x3 stride 1 pad 1, bias on"},
        "bn_bwd_GBps": by.get("batchnorm_bwd", {}).get("achieved"),
        "pool_max_bwd_GBps": by.get("pool2d_max_bwd", {}).get("achieved"),
        "pool_avg_bwd_GBps": by.get("pool2d_avg_bwd", {}).get("achieved"),
    }
    if a.dtype in pair_info:
        out["value_cache_warm"] = pair_info[a.dtype]["achieved_cache_warm"]
        out["ms_per_step_cache_warm"] = pair_info[a.dtype]["us_cache_warm"] * 1e-3
        out["pair"] = pair_info[a.dtype]
    if "conv2d_bwd_data" in by:
        o = by["conv2d_bwd_data"]
        out["roofline"] = {
            "kernel": ("slab_conv_kernel<float, true>" if a.dtype == "f32" else "strip16_conv_kernel") +
                      " (conv2dBackwardData, one launch per call)",
            "bound": "mfma", "achieved": o["achieved"], "peak": o["peak"], "unit": "TFLOP/s",
            "frac": o["frac"], "avg_launch_us": o["us"], "avg_launch_us_cache_warm": o["us_cache_warm"],
            "traffic": MEASURED_TRAFFIC.get("conv2d_bwd_data_" + a.dtype), "traffic_source": TRAFFIC_SOURCE}
    if "conv2d_bwd_filter_bias" in by:
        o = by["conv2d_bwd_filter_bias"]
        out["roofline_bwd_filter"] = {
            "kernel": "wgrad_slab_kernel<float> + wgrad_reduce_kernel (conv2dBackwardFilterBias, two launches per call)"
                      if a.dtype == "f32" else "wgrad_dma32_kernel<1> + wgrad_taps_reduce_kernel",
            "bound": "mfma", "achieved": o["achieved"], "peak": o["peak"], "unit": "TFLOP/s",
            "frac": o["frac"], "avg_call_us": o["us"], "avg_call_us_cache_warm": o["us_cache_warm"],
            "traffic": MEASURED_TRAFFIC.get("conv2d_bwd_filter_" + a.dtype), "traffic_source": TRAFFIC_SOURCE}
    if "bf16" in pair_info:
        # the 16-bit half of the target ("or bf16"): the same pair in bf16 storage against the bf16 matrix peak
        pi = pair_info["bf16"]
        out["roofline_bf16_pair"] = {
            "kernel": "strip16_conv_kernel + wgrad_dma32_kernel<1> + wgrad_taps_reduce_kernel (three launches per step)",
            "bound": "mfma", "achieved": pi["achieved"], "peak": pi["peak"], "unit": "TFLOP/s", "frac": pi["frac"],
            "us_per_step": pi["us"], "us_per_step_cache_warm": pi["us_cache_warm"],
            "traffic": (MEASURED_TRAFFIC["conv2d_bwd_data_bf16"] + MEASURED_TRAFFIC["conv2d_bwd_filter_bf16"]),
            "traffic_source": TRAFFIC_SOURCE}
    out["ops"] = ops
    # the reference's CPU path: the oneDNN primitives its extension requests (through PyTorch-CPU,
    # whose embedded oneDNN executes them); the C restatement used as the parity checker is listed
    # beside it
    out["cpu_baseline"] = cpu_onednn
    out["cpu_port"] = cpu_port
    out["cpu_onednn_bandwidth_ops"] = cpu_bw
    print(json.dumps(out))
    return 0


# (count in the network, N, C, H, W, K, KH, KW, sy, sx, py, px); ResNet-50 v1.5 as built by
# flashlight/pkg/vision/models/Resnet.cpp:210-230 (stride on the 3x3), batch 32
RESNET50_LAYERS = [(1, 32, 3, 224, 224, 64, 7, 7, 2, 2, 3, 3)] + [
    (cnt, 32, c, h, h, k, ks, ks, s, s, ks // 2, ks // 2) for (cnt, h, c, k, ks, s) in [
        (1, 56, 64, 64, 1, 1), (4, 56, 64, 256, 1, 1), (2, 56, 256, 64, 1, 1), (3, 56, 64, 64, 3, 1),
        (1, 56, 256, 128, 1, 1), (1, 56, 128, 128, 3, 2), (1, 56, 256, 512, 1, 2), (4, 28, 128, 512, 1, 1),
        (3, 28, 512, 128, 1, 1), (3, 28, 128, 128, 3, 1), (1, 28, 512, 256, 1, 1), (1, 28, 256, 256, 3, 2),
        (1, 28, 512, 1024, 1, 2), (6, 14, 256, 1024, 1, 1), (5, 14, 1024, 256, 1, 1), (5, 14, 256, 256, 3, 1),
        (1, 14, 1024, 512, 1, 1), (1, 14, 512, 512, 3, 2), (1, 14, 1024, 2048, 1, 2), (3, 7, 512, 2048, 1, 1),
        (2, 7, 2048, 512, 1, 1), (2, 7, 512, 512, 3, 1)]]
# configs[3]: [1500, 1, 80, 16] through three 21x1 SAME convolutions, the last with stride 2
SPEECH_LAYERS = [(1, 16, 80, 1, 1500, 250, 1, 21, 1, 1, 0, 10), (1, 16, 250, 1, 1500, 250, 1, 21, 1, 1, 0, 10),
                 (1, 16, 250, 1, 1500, 250, 1, 21, 1, 2, 0, 10)]


def rnn_sweep(a, fa, torch):
    """Wall-clock times of rnn / rnnBackward through the C ABI (a.steps calls after a.warmup);
    TFLOP/s counts the matrix products only (input and recurrent projections; twice that
    in the backward pass)."""
    ops = fa.ops
    def timed(fn):
        for _ in range(max(a.warmup, 1)):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(a.steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / a.steps * 1e3
    for mode, name, gates in ((ops.RNN_LSTM, "LSTM", 4), (ops.RNN_GRU, "GRU", 3)):
        for (I, H, L, bidir, T, B) in ((512, 512, 2, True, 200, 32), (1024, 1024, 1, False, 100, 64),
                                       (256, 256, 2, False, 50, 16)):
            n = ops.rnn_param_count(I, H, L, mode, bidir)
            x = torch.randn(T, B, I, device="cuda")
            w = torch.randn(n, device="cuda") / H ** 0.5
            y, hy, cy, res = ops.rnn(x, None, None, w, H, L, mode, bidir)
            dy = torch.randn_like(y)
            tf = timed(lambda: ops.rnn(x, None, None, w, H, L, mode, bidir))
            tb = timed(lambda: ops.rnn_backward(x, w, res, H, L, mode, bidir, dy))
            D = 2 if bidir else 1
            fl = sum(D * 2.0 * gates * H * ((I if l == 0 else D * H) + H) * T * B for l in range(L))
            print("%-4s input %d hidden %d layers %d dirs %d T %d batch %d: fwd %.2f ms (%.1f TFLOP/s)  "
                  "bwd %.2f ms (%.1f TFLOP/s)" % (name, I, H, L, D, T, B, tf, fl / tf / 1e9, tb, 2 * fl / tb / 1e9),
                  flush=True)
    return 0


def linear_sweep(a, fa, torch):
    """Times of fl::linear's forward product (weight x input + bias) and of its backward pass (input gradient,
    weight gradient, bias gradient) through the C ABI, by HIP events over a.steps calls after a.warmup; TFLOP/s
    counts the one product forward and the two backward."""
    ops = fa.ops
    tdt = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}[a.dtype]
    def timed(fn):
        for _ in range(max(a.warmup, 1)):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(a.steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / a.steps * 1e3
    for (fin, fout, frames) in ((2000, 2000, 4000), (1024, 1024, 12000), (1200, 1200, 3000), (80, 2000, 12000),
                                (2048, 1000, 256)):
        x = torch.randn(frames, fin, device="cuda").to(tdt)
        w = (torch.randn(fin, fout, device="cuda") / fin ** 0.5).to(tdt)
        b = torch.randn(fout, device="cuda")
        dy = torch.randn(frames, fout, device="cuda").to(tdt)
        tf = timed(lambda: ops.linear(x, w, b))
        tb = timed(lambda: ops.linear_backward(dy, x, w))
        fl = 2.0 * fin * fout * frames
        print("%s Linear %d -> %d over %d frames: forward %.1f us (%.0f TFLOP/s)  backward %.1f us (%.0f TFLOP/s)"
              % (a.dtype, fin, fout, frames, tf, fl / tf / 1e6, tb, 2 * fl / tb / 1e6), flush=True)
    return 0


def layer_sweep(a, fa, torch, tdt):
    """Per-layer times of the three conv passes through the C ABI (HIP events around
    a.steps launches after a.warmup); the first layer of a network has no backward-data
    in training (its input needs no gradient), so it is left out of the totals."""
    capi, L = fa.capi, fa.capi.lib()
    tag = capi.F32 if tdt == torch.float32 else capi.BF16 if tdt == torch.bfloat16 else capi.F16
    S = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    P = lambda t: C.c_void_p(t.data_ptr())

    def timed(fn):
        for _ in range(max(a.warmup, 1)):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(a.steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / a.steps * 1e3

    def chk(rc):
        if rc != 0:
            raise RuntimeError(L.flhip_last_error())

    layers = RESNET50_LAYERS if a.layers == "resnet50" else SPEECH_LAYERS
    tot, flops = [0.0, 0.0, 0.0], 0.0
    print("| n | input NxCxHxW | K | window | stride | GFLOP | fwd us (TFLOP/s) | bwd-data us | bwd-filter us |")
    print("|---|---|---|---|---|---|---|---|---|")
    for i, (cnt, N, Ci, H, W, K, kh, kw, sy, sx, py, px) in enumerate(layers):
        N = a.batch or N
        x = torch.randn(N, Ci, H, W, device="cuda").to(tdt)
        w = (torch.randn(K, Ci, kh, kw, device="cuda") / (Ci * kh * kw) ** 0.5).to(tdt)
        cd = capi.ConvDesc(N, Ci, H, W, K, kh, kw, sy, sx, py, px, 1, 1, 1, tag)
        oh, ow = C.c_int32(), C.c_int32()
        chk(L.flhip_conv2d_out_dims(C.byref(cd), C.byref(oh), C.byref(ow)))
        y = torch.empty(N, K, oh.value, ow.value, device="cuda", dtype=tdt)
        dy, dx = torch.randn_like(y), torch.empty_like(x)
        dw = torch.empty(K, Ci, kh, kw, device="cuda")
        nws = max(L.flhip_conv2d_workspace_bytes(C.byref(cd), p) for p in (capi.CONV_FWD, capi.CONV_BWD_DATA,
                                                                           capi.CONV_BWD_FILTER))
        ws = torch.empty(max(nws, 16), dtype=torch.uint8, device="cuda")
        gf = 2.0 * N * K * oh.value * ow.value * Ci * kh * kw / 1e9
        t = [timed(lambda: chk(L.flhip_conv2d_fwd(C.byref(cd), P(x), P(w), None, P(y), P(ws), nws, S))),
             timed(lambda: chk(L.flhip_conv2d_bwd_data(C.byref(cd), P(dy), P(w), P(dx), P(ws), nws, S))),
             timed(lambda: chk(L.flhip_conv2d_bwd_filter(C.byref(cd), P(x), P(dy), P(dw), None, P(ws), nws, S)))]
        first = i == 0
        for j in range(3):
            if not (first and j == 1):
                tot[j] += cnt * t[j]
                flops += cnt * gf
        print("| %d | %dx%dx%dx%d | %d | %dx%d | %d,%d | %.2f | %.1f (%.1f) | %.1f (%.1f) | %.1f (%.1f) |" % (
            cnt, N, Ci, H, W, K, kh, kw, sy, sx, gf, t[0], gf / t[0] * 1e3, t[1], gf / t[1] * 1e3, t[2],
            gf / t[2] * 1e3), flush=True)
    print("totals over the network (counts applied, first layer without bwd-data): fwd %.2f ms, bwd-data %.2f ms, "
          "bwd-filter %.2f ms, sum %.2f ms for %.1f GFLOP = %.1f TFLOP/s (%s)" % (
              tot[0] / 1e3, tot[1] / 1e3, tot[2] / 1e3, sum(tot) / 1e3, flops, flops / sum(tot) * 1e3, a.dtype))
    return 0


def plan_sweep(a, fa, torch, tdt):
    """Every plan of the two backward passes (flhip_conv2d_bwd_*_plan) on every layer of a network: the time of the
    default rule, of the fastest plan, and which plans the library declined.  This is the measurement that
    HipAutogradExtension::createBenchmarkOptions makes per layer at run time in benchmark mode."""
    capi, L = fa.capi, fa.capi.lib()
    tag = capi.F32 if tdt == torch.float32 else capi.BF16 if tdt == torch.bfloat16 else capi.F16
    S = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    P = lambda t: C.c_void_p(t.data_ptr())
    steps = a.steps if a.steps != 100 else 20

    def timed(fn):
        for _ in range(3):
            rc = fn()
            if rc == capi.DECLINED:
                return None
            capi.check(rc)
        torch.cuda.synchronize()
        best = 1e30
        for _ in range(3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(steps):
                fn()
            e1.record()
            torch.cuda.synchronize()
            best = min(best, e0.elapsed_time(e1) / steps * 1e3)
        return best

    layers = RESNET50_LAYERS if a.plans == "resnet50" else SPEECH_LAYERS
    print("| input NxCxHxW | K | window | stride | pass | default rule us | fastest plan | us | default / fastest |")
    print("|---|---|---|---|---|---|---|---|---|")
    gain = {"data": [0.0, 0.0], "filter": [0.0, 0.0]}
    for i, (cnt, N, Ci, H, W, K, kh, kw, sy, sx, py, px) in enumerate(layers):
        N = a.batch or N
        x = torch.randn(N, Ci, H, W, device="cuda").to(tdt)
        w = (torch.randn(K, Ci, kh, kw, device="cuda") / (Ci * kh * kw) ** 0.5).to(tdt)
        cd = capi.ConvDesc(N, Ci, H, W, K, kh, kw, sy, sx, py, px, 1, 1, 1, tag)
        oh, ow = C.c_int32(), C.c_int32()
        capi.check(L.flhip_conv2d_out_dims(C.byref(cd), C.byref(oh), C.byref(ow)))
        dy = torch.randn(N, K, oh.value, ow.value, device="cuda").to(tdt)
        dx = torch.empty_like(x)
        dw = torch.empty(K, Ci, kh, kw, device="cuda")
        for pname, pas in (("data", capi.CONV_BWD_DATA), ("filter", capi.CONV_BWD_FILTER)):
            if pname == "data" and i == 0 and a.plans == "resnet50":
                continue                      # the first layer's input needs no gradient
            nws = L.flhip_conv2d_workspace_bytes(C.byref(cd), pas)
            ws = torch.empty(max(nws, 16), dtype=torch.uint8, device="cuda")
            times = {}
            for plan in range(-1, L.flhip_conv2d_plan_count(pas)):
                if plan == 9:                             # the direct kernels are never competitive
                    continue
                if pas == capi.CONV_BWD_DATA:
                    t = timed(lambda: L.flhip_conv2d_bwd_data_plan(C.byref(cd), P(dy), P(w), P(dx), P(ws), nws, plan, S))
                else:
                    t = timed(lambda: L.flhip_conv2d_bwd_filter_plan(C.byref(cd), P(x), P(dy), P(dw), None, P(ws), nws, plan, S))
                if t is not None:
                    times[plan] = t
            best = min((p for p in times if p >= 0), key=lambda p: times[p])
            gain[pname][0] += cnt * times[-1]
            gain[pname][1] += cnt * times[best]
            mark = " **" if times[best] < 0.95 * times[-1] else ""
            print("| %dx%dx%dx%d | %d | %dx%d | %d,%d | bwd-%s | %.1f | %d: %s | %.1f | %.2f%s |" % (
                N, Ci, H, W, K, kh, kw, sy, sx, pname, times[-1], best, L.flhip_conv2d_plan_name(pas, best).decode(),
                times[best], times[-1] / times[best], mark), flush=True)
    for pname in ("data", "filter"):
        print("bwd-%s over the network (counts applied): default rule %.2f ms, fastest plan per layer %.2f ms (%s)" % (
            pname, gain[pname][0] / 1e3, gain[pname][1] / 1e3, a.dtype))
    return 0


def cpu_legs():
    """(1) the C restatement in oracle/ on a bounded sample of the conv pair;
    (2) the same oneDNN primitives the reference requests, reached through
    PyTorch-CPU, on the full batch.  Both on this host's cores."""
    import numpy as np
    import torch
    from oracle import flref
    threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or min(os.cpu_count() or 1, 16)
    rng = np.random.default_rng(0)
    nb = 32                                             # the full batch
    x = rng.standard_normal((nb, 64, 56, 56)).astype(np.float32)
    w = (rng.standard_normal((64, 64, 3, 3)) / 24).astype(np.float32)
    dy = rng.standard_normal((nb, 64, 56, 56)).astype(np.float32)
    d = flref.conv_desc(x.shape, w.shape, (1, 1), (1, 1))
    flref.conv2d_bwd_data(d, dy[:1], w)                 # warm-up (thread pool, page faults)
    reps, t0 = 0, time.perf_counter()
    while True:
        flref.conv2d_bwd_data(d, dy, w)
        flref.conv2d_bwd_filter(d, x, dy)
        reps += 1
        el = time.perf_counter() - t0
        if el > 12.0:
            break
    flop = 2 * CONV_FLOP * nb / 32 * reps
    port = {"value": flop / el / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sample": "%d repetitions of the pair on the full batch of %d, oracle/flref.c with "
                      "OpenMP, %.1f s" % (reps, nb, el)}

    torch.set_num_threads(threads)
    xt = torch.from_numpy(rng.standard_normal((32, 64, 56, 56)).astype(np.float32))
    wt = torch.from_numpy(w)
    dyt = torch.from_numpy(rng.standard_normal((32, 64, 56, 56)).astype(np.float32))
    conv_bw = torch.ops.aten.convolution_backward

    def pair():
        conv_bw(dyt, xt, wt, [64], [1, 1], [1, 1], [1, 1], False, [0, 0], 1, [True, False, False])
        conv_bw(dyt, xt, wt, [64], [1, 1], [1, 1], [1, 1], False, [0, 0], 1, [False, True, True])

    for _ in range(3):
        pair()
    reps, t0 = 0, time.perf_counter()
    while True:
        pair()
        reps += 1
        el = time.perf_counter() - t0
        if el > 8.0:
            break
    onednn = {"value": 2 * CONV_FLOP * reps / el / 1e12, "unit": "TFLOP/s", "cores": threads,
              "kind": "reference",
              "detail": "oneDNN %s through PyTorch-CPU aten::convolution_backward: the backward-data and "
                        "backward-weights(+bias) primitives the reference's oneDNN extension requests "
                        "(its own C++ cannot be built offline)" % _onednn_version(),
              "sample": "%d repetitions of the pair on the full batch of 32, %.1f s" % (reps, el)}
    return port, onednn


def cpu_bandwidth_legs():
    """The bandwidth-bound ops of cfg 3 on this host's cores through PyTorch-CPU with
    oneDNN tensors (`to_mkldnn`: the pooling / batch-normalisation primitives the
    reference's oneDNN extension requests); a few seconds each.  GB/s by the same
    algorithmic bytes as the GPU figures."""
    import torch
    import torch.nn.functional as F
    threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or min(os.cpu_count() or 1, 16)
    torch.set_num_threads(threads)
    g = torch.Generator().manual_seed(0)
    out = []

    def leg(name, nbytes, fn, budget=2.5):
        try:
            fn()
            reps, t0 = 0, time.perf_counter()
            while True:
                fn()
                reps += 1
                el = time.perf_counter() - t0
                if el > budget:
                    break
            out.append({"op": name, "ms": el / reps * 1e3, "GBps": nbytes * reps / el / 1e9,
                        "cores": threads, "sample": "%d repetitions, %.1f s" % (reps, el)})
        except Exception as e:      # a primitive PyTorch does not route to oneDNN on this host
            out.append({"op": name, "error": str(e)[:200]})

    T = 32 * 256 * 56 * 56 * 4
    x = (torch.randn(32, 256, 56, 56, generator=g) * 2 ** 0.5 + 0.5).to_mkldnn()
    dy = torch.randn(32, 256, 56, 56, generator=g).to_mkldnn()
    gamma = torch.randn(256, generator=g) * 0.1 + 1
    beta = torch.zeros(256)
    leg("batchnorm_fwd_train", 2 * T,
        lambda: torch.ops.aten.native_batch_norm(x, gamma, beta, None, None, True, 0.0, 1e-5))

    y_, sm_, sv_ = torch.ops.aten.native_batch_norm(x, gamma, beta, None, None, True, 0.0, 1e-5)
    leg("batchnorm_bwd", 3 * T,
        lambda: torch.ops.aten.native_batch_norm_backward(dy, x, gamma, None, None, sm_, sv_, True, 1e-5,
                                                          [True, True, True]))
    del y_

    def bn_fwd_bwd():
        xr = x.to_dense().requires_grad_(True)
        y = F.batch_norm(xr.to_mkldnn(), None, None, gamma, beta, True, 0.0, 1e-5)
        y.backward(dy)
    leg("batchnorm_fwd_train+bwd (autograd, includes layout conversions)", 5 * T, bn_fwd_bwd)
    del x, dy

    nx, ny = 32 * 64 * 112 * 112 * 4, 32 * 64 * 56 * 56 * 4
    px = (torch.round(torch.randn(32, 64, 112, 112, generator=g) * 8) / 8).to_mkldnn()
    leg("pool2d_max_fwd", nx + ny + ny // 4, lambda: torch.max_pool2d(px, 3, 2, 1))
    leg("pool2d_avg_fwd", nx + ny, lambda: F.avg_pool2d(px, 3, 2, 1, count_include_pad=False))
    pdy = torch.randn(32, 64, 56, 56, generator=g).to_mkldnn()
    leg("pool2d_avg_bwd", nx + ny,
        lambda: torch.ops.aten.avg_pool2d_backward(pdy, px, [3, 3], [2, 2], [1, 1], False, False, None))
    # max pooling's backward primitive needs the forward primitive's workspace, which PyTorch only keeps
    # inside autograd: its time alone is the difference of the two legs "fwd+bwd" and "fwd" below

    def pool_fwd_bwd(avg):
        xr = px.to_dense().requires_grad_(True)
        xm = xr.to_mkldnn()
        y = F.avg_pool2d(xm, 3, 2, 1, count_include_pad=False) if avg else torch.max_pool2d(xm, 3, 2, 1)
        y.backward(pdy)
    leg("pool2d_max_fwd+bwd (autograd, includes layout conversions)", 2 * (nx + ny + ny // 4),
        lambda: pool_fwd_bwd(False))
    leg("pool2d_avg_fwd+bwd (autograd, includes layout conversions)", 2 * (nx + ny),
        lambda: pool_fwd_bwd(True))
    return out


def step_bench(a):
    """Whole training steps through the C++ host layer: runs flashlight_amd/lib/flhip_step_bench
    (built by flashlight_amd.build) and prints its JSON line."""
    import subprocess
    exe = os.path.join(ROOT, "flashlight_amd", "lib", "flhip_step_bench")
    if not os.path.exists(exe):
        sys.stderr.write("bench.py: %s is missing; build it with `python -m flashlight_amd.build`\n" % exe)
        return 1
    batch = a.batch or (64 if a.step == "resnet50" else 16)
    r = subprocess.run([exe, a.step, str(batch), str(a.steps), str(min(a.warmup, 5)), a.dtype],
                       capture_output=True, text=True)
    sys.stderr.write(r.stderr)
    if r.returncode != 0:
        return r.returncode
    rec = json.loads(r.stdout.strip().splitlines()[-1])
    bd = rec["breakdown_ms"]
    conv = sum(v for k, v in bd.items() if k.startswith("conv_"))
    busy = sum(v for k, v in bd.items() if k not in ("span", "host_gaps"))
    rec["conv_share_of_device_time"] = conv / busy if busy else None
    rec["non_conv_share_of_device_time"] = 1 - conv / busy if busy else None
    print(json.dumps(rec))
    return 0


def _onednn_version():
    import re
    import torch
    m = re.search(r"MKL-DNN (v[0-9.]+)", torch.__config__.show())
    return m.group(1) if m else "?"


if __name__ == "__main__":
    sys.exit(main())
