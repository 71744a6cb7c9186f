#!/usr/bin/env python3
"""Benchmark of the PULP-NN int8 kernel path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-layers] [--no-cpu]

A step is one pass of the hot path over one batch of synthetic input: the
pointwise 1x1 convolution 28x28x128 -> 256 channels at batch 256 (scalar
multiplier requantisation + ReLU), the configuration the headline metric is
quoted on.  Inputs are resident in HBM before the timed region; successive steps
rotate through enough buffer sets (> 256 MB in total) that the Infinity Cache
cannot hold them.  A timed region is exactly K steps between two device
synchronisations.  K steps of a 17 us kernel are far too short to time once, and
the shader clock of this GPU settles only after some 10 ms of continuous work (a
burst of a few launches of the MFMA-bound convolution runs up to a third slower
than the same launches in a long run), so regions are repeated back to back, at
least 10 times and until 60 ms have been timed.  The median over the regions is
the reported value; the first region, minimum, 10th and 90th percentile go into
the record next to it ("timing").  The last line printed is the JSON record.

Besides the headline workload the record carries, under "layers", the other
single-layer configurations (3x3 conv at batch 256, depthwise 3x3 stride 1 and 2
at batch 256, the 64-bit batch-norm 3x3 conv at batch 64 with its max-pool and
linear layer) and the whole MobileNet chain, each with its own roofline object.

The process exits with status 1 (and "value": null) if any output differs from
the CPU oracle.
"""
import argparse
import json
import math
import os
import re
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_INT8_OPS = 5.0e15   # MI355X dense int8 MFMA, op/s
PEAK_HBM = 8.0e12        # MI355X HBM3E, B/s
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "bench_all_layers_hbm_traffic.txt")
TRACE_FILE = os.path.join(ROOT, "profiles", "bench_all_layers_kernel_trace.txt")
# The kernel each workload is expected to dispatch to.  The library does not report what it launched, so these
# names are checked against the committed kernel trace of this same benchmark (tests/test_bench_kernels.py, and
# `kernel_in_committed_trace` in every roofline object): a dispatch rule that changes without the profiles being
# regenerated shows up there.
KERNELS = {
    "cfg1_pointwise": "pw_stream_kernel<4, 2, 4, 1, true, 1, 16>",
    "cfg0_conv": "igemm_kernel<2, 4, 2, 3, 0, 2, 5>",
    "cfg2_dw_s1": "dw3x3_lin_kernel<1, 1, 0, true, true>",
    "cfg2_dw_s2": "dw3x3_stream_kernel<2, 1, 0>",
    "cfg4_conv": "igemm_patch_kernel<0, 0>",
    "cfg4_maxpool": "maxpool16_kernel<false, true>",
    "cfg4_linear": "linear_skinny_kernel<0>",
}


def traced_kernels():
    """Kernel names (up to the argument list) of the committed kernel-trace summary; empty if it is missing."""
    if not os.path.exists(TRACE_FILE):
        return set()
    names = set()
    for line in open(TRACE_FILE):
        m = re.match(r"^(?:void )?(\w+(?:<.*?>)?)\(", line)
        if m:
            names.add(m.group(1))
    return names


def profiled_traffic():
    """HBM bytes per launch from the committed rocprofv3 counter summary (FETCH_SIZE and WRITE_SIZE, scaled by
    what the same counters read for a plain copy): {(kernel name, grid size): bytes}.  Empty if the file is
    missing; a kernel that has changed its name since the profile was taken is simply not found."""
    out = {}
    if not os.path.exists(TRAFFIC_FILE):
        return out
    for line in open(TRAFFIC_FILE):
        m = re.match(r"^(\S.*?)\s+(\d+)\s+([\d.]+)\s+([\d.]+)\s+(\d+)(?:\s+(\d+)\s+([\d.]+))?\s*$", line)
        if m:
            out[(m.group(1).strip(), int(m.group(2)))] = int(m.group(5))
    return out


def traffic_for(table, kernel_prefix):
    hits = [v for (name, _), v in table.items() if name.startswith(kernel_prefix)]
    return hits[0] if len(hits) == 1 else None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-layers", action="store_true", help="skip the per-layer table")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--quick", action="store_true", help="time 6 ms per workload instead of 60 (for runs under a profiler)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (--gpus 1): every layer is independent per image, so "
                 "more GPUs would each take a slice of the batch with no exchange; no multi-GPU figure is produced")

    import numpy as np
    import torch

    from pulp_nn_amd import PulpNN, workloads

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    libs = {32: PulpNN(32), 64: PulpNN(64)}
    for L in libs.values():
        L.use_torch_stream()     # the library queues on torch's current stream, which the events below time
    traffic = profiled_traffic()
    traced = traced_kernels()
    failures = []

    def t(a):
        return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).cuda()

    probe_buf = torch.zeros((4096, 2), dtype=torch.int64, device="cuda")

    def time_launches(fn, steps, warmup, min_ms=None, min_repeats=10, max_repeats=4000, series=False):
        """fn(i) queues one step on torch's current stream (the library's stream).  Times regions of exactly
        `steps` steps, each between two synchronisations, one after the other; returns (median wall ms per step,
        median device ms per step from HIP events, timing summary).  Behind every region the library's clock probe
        is queued (20 us, outside the timed interval): the shader clock the region left the GPU at."""
        min_ms = (6.0 if args.quick else 60.0) if min_ms is None else min_ms
        for i in range(warmup):
            fn(i)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        walls, devs, timed, it = [], [], 0.0, warmup
        while len(walls) < min_repeats or (timed < min_ms and len(walls) < max_repeats):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            e0.record()
            for _ in range(steps):
                fn(it)
                it += 1
            e1.record()
            libs[32].clock_probe(probe_buf[len(walls)])
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            walls.append((t1 - t0) * 1e3 / steps)
            devs.append(e0.elapsed_time(e1) / steps)
            timed += e0.elapsed_time(e1)
        srt = sorted(devs)

        def pct(q):
            return srt[min(len(srt) - 1, int(q * len(srt)))]

        summary = {"regions": len(devs), "steps_per_region": steps, "timed_ms": round(timed, 1),
                   "device_us_per_step": {"first_region": round(devs[0] * 1e3, 2), "min": round(srt[0] * 1e3, 2),
                                          "p10": round(pct(0.10) * 1e3, 2), "median": round(statistics.median(devs) * 1e3, 2),
                                          "p90": round(pct(0.90) * 1e3, 2),
                                          "median_after_first_10ms": round(statistics.median(
                                              devs[min(len(devs) - 1, next((n for n in range(len(devs)) if sum(devs[:n + 1]) * steps >= 10.0),
                                                                            len(devs) - 1)):]) * 1e3, 2)}}
        pr = probe_buf[:len(devs)].cpu().numpy()
        mhz = [round(100.0 * float(c) / float(t)) if t else 0 for t, c in pr]
        summary["shader_mhz_behind_region"] = {"first_region": mhz[0], "min": min(mhz), "median": int(statistics.median(mhz)),
                                               "max": max(mhz)}
        if series:
            # the first regions one by one: [device us per step, shader MHz behind the region]
            summary["first_regions"] = [[round(d * 1e3, 2), m] for d, m in list(zip(devs, mhz))[:24]]
        return statistics.median(walls), statistics.median(devs), summary

    def rotating(nbytes):
        """How many buffer sets make the rotation exceed the 256 MB Infinity Cache twice over."""
        return max(2, int(math.ceil(600e6 / nbytes)))

    def roofline(bound, ops, nbytes, dev_ms, kernel):
        sec = dev_ms * 1e-3
        r = {"bound": bound, "kernel": kernel}
        if bound == "mfma":
            r.update(achieved=round(ops / sec / 1e12, 2), peak=PEAK_INT8_OPS / 1e12, unit="TOP/s (int8, 2 x MAC)",
                     frac=round(ops / sec / PEAK_INT8_OPS, 4))
        else:
            r.update(achieved=round(nbytes / sec / 1e9, 1), peak=PEAK_HBM / 1e9, unit="GB/s",
                     frac=round(nbytes / sec / PEAK_HBM, 4))
        r["algorithmic_bytes_per_launch"] = nbytes
        # (from the committed counter summary, looked up by the kernel this layer is expected to dispatch to; null if
        # that kernel has no line there)
        r["traffic"] = traffic_for(traffic, kernel.split("(")[0].strip())
        r["traffic_measured_in_this_run"] = False
        r["kernel_in_committed_trace"] = kernel.split("(")[0].strip() in traced
        return r

    # ---- headline: config 1 -------------------------------------------------
    c1 = workloads.config1(batch=256)
    L = libs[32]
    B, H, W, Ci = c1["x"].shape
    Co = c1["w"].shape[0]
    nset = rotating(c1["bytes"])
    x0 = t(c1["x"])
    xs = [x0] + [x0.clone() for _ in range(nset - 1)]
    outs = [torch.zeros((B, H, W, Co), dtype=torch.uint8, device="cuda") for _ in range(nset)]
    w, bias = t(c1["w"]), t(c1["bias"])
    L.set_batch(B)

    def step_c1(i):
        j = i % nset
        L.pulp_nn_pointwise_HoWo_parallel(xs[j], None, bias, outs[j], w, None, None, c1["out_mult"], c1["out_shift"],
                                          W, H, Ci, W, H, Co, 1, 1, 0, 0, 0, 0, 1, 1, c1["relu"], c1["bn"])

    wall_ms, dev_ms, timing = time_launches(step_c1, args.steps, args.warmup, series=True)

    # parity of what was just computed, on a sample of the batch (the oracle is the checker, outside the timed region)
    import oracle
    nchk = 4
    want = oracle.pointwise(c1["x"][:nchk], c1["w"], c1["bias"], None, None, c1["out_mult"], c1["out_shift"],
                            c1["relu"], c1["bn"], 32)
    parity = all(bool(np.array_equal(o[:nchk].cpu().numpy(), want)) for o in outs)
    if not parity:
        failures.append("configs[1] pointwise")

    gops = c1["ops"] / (wall_ms * 1e-3) / 1e9
    head_kernel = KERNELS["cfg1_pointwise"]
    rec = {
        "metric": "int8 GOPS and % int8 MFMA peak per conv layer at batch 256; bit-exact",
        "value": round(gops, 1),
        "unit": "GOPS",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8 x uint8 -> int32 (MFMA), integer requantisation to uint8",
        "data": "synthetic (seeded PCG64: activations U[0,255], weights U[-128,127])",
        "config": {"workload": "configs[1]: pointwise 1x1 conv 28x28x128 -> 256, batch 256, "
                               "out_mult/out_shift requantisation + ReLU (pulp_nn_pointwise_HoWo_parallel)",
                   "batch": B, "gemm_MxNxK": [B * H * W, Co, Ci], "buffer_sets_rotated": nset},
        "timed_regions": timing["regions"],
        "timing": timing,
        "images_per_s": round(B / (wall_ms * 1e-3), 1),
        "device_ms_per_step": round(dev_ms, 5),
        "parity": "bit-exact vs CPU oracle on %d images of every buffer set" % nchk if parity else "MISMATCH vs CPU oracle",
        "mfma_frac": round(c1["ops"] / (dev_ms * 1e-3) / PEAK_INT8_OPS, 4),
        "roofline": {
            "bound": "hbm",
            "kernel": head_kernel + " (weights-stationary pointwise, scalar-multiplier epilogue)",
            "achieved": round(c1["bytes"] / (dev_ms * 1e-3) / 1e9, 1),
            "peak": PEAK_HBM / 1e9,
            "unit": "GB/s",
            "frac": round(c1["bytes"] / (dev_ms * 1e-3) / PEAK_HBM, 4),
            "algorithmic_bytes_per_launch": c1["bytes"],
            # HBM bytes per launch read at run time from the committed counter summary (rocprofv3 --pmc FETCH_SIZE
            # x 2.0 + WRITE_SIZE x 1.0, the factors a plain copy of known size shows); null if the file has no
            # line for this kernel
            "traffic": traffic_for(traffic, head_kernel),
            "traffic_source": "profiles/bench_all_layers_hbm_traffic.txt",
            "traffic_measured_in_this_run": False,
            "kernel_in_committed_trace": head_kernel in traced,
        },
    }

    # ---- the other single-layer configurations ------------------------------
    layers = []

    def layer_record(name, ops, nbytes, wall, dev, tm, ok, bound, kernel, **extra):
        rec_ = {"layer": name, "ms": round(dev, 5), "wall_ms": round(wall, 5), "timing": tm["device_us_per_step"],
                "gops": round(ops / (dev * 1e-3) / 1e9, 1),
                "mfma_frac": round(ops / (dev * 1e-3) / PEAK_INT8_OPS, 4),
                "hbm_gbs": round(nbytes / (dev * 1e-3) / 1e9, 1),
                "hbm_frac": round(nbytes / (dev * 1e-3) / PEAK_HBM, 4),
                "roofline": roofline(bound, ops, nbytes, dev, kernel),
                "parity": "bit-exact" if ok else "MISMATCH"}
        rec_["shader_mhz_behind_region"] = tm["shader_mhz_behind_region"]
        if "first_regions" in tm:
            rec_["first_regions"] = tm["first_regions"]
        rec_.update(extra)
        layers.append(rec_)
        if not ok:
            failures.append(name)

    if not args.no_layers:
        steps, warm = max(10, args.steps // 4), max(3, args.warmup // 4)

        # config 0 at batch 256: 3x3 conv, 32-bit batch-norm
        c0 = workloads.config0(batch=256)
        L = libs[32]
        nset = rotating(c0["bytes"])
        x0 = t(c0["x"])
        xs0 = [x0] + [x0.clone() for _ in range(min(nset, 64) - 1)]
        outs0 = [torch.zeros((256, 16, 16, 64), dtype=torch.uint8, device="cuda") for _ in range(len(xs0))]
        w0, b0, k0, l0 = t(c0["w"]), t(c0["bias"]), t(c0["k"]), t(c0["lam"])
        L.set_batch(256)

        def step_c0(i):
            j = i % len(xs0)
            L.pulp_nn_conv_Ho_parallel(xs0[j], None, b0, outs0[j], w0, k0, l0, 0, c0["out_shift"], 16, 16, 32, 16, 16,
                                       64, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1)

        wall, dev, tm = time_launches(step_c0, steps, warm)
        want = oracle.conv(c0["x"][:8], c0["w"], c0["bias"], c0["k"], c0["lam"], 0, c0["out_shift"], c0["pads"],
                           c0["strides"], 1, 1, 32)
        layer_record(c0["name"] + "_b256", c0["ops"], c0["bytes"], wall, dev, tm,
                     np.array_equal(outs0[0][:8].cpu().numpy(), want), "mfma",
                     KERNELS["cfg0_conv"] + " (128 x 64 tiles, whole K in one pass)",
                     note="6.3 MB and 2.4 GOP per launch: bound by launch and memory latency, not by a pipe")
        del xs0, outs0

        # config 2: depthwise 3x3, stride 1 through pulp_nn_depthwise_3x3_s1, stride 2 through depthwise_generic
        for stride in (1, 2):
            c2 = workloads.config2(batch=256, stride=stride)
            ho = c2["out_hw"][0]
            xin = c2["x"] if stride == 2 else np.pad(c2["x"], ((0, 0), (0, 0), (1, 1), (0, 0)))
            nset = rotating(c2["bytes"])
            x0 = t(xin)
            xs2 = [x0] + [x0.clone() for _ in range(nset - 1)]
            outs2 = [torch.zeros((256, ho, ho, 128), dtype=torch.uint8, device="cuda") for _ in range(nset)]
            w2, b2, k2, l2 = t(c2["w"]), t(c2["bias"]), t(c2["k"]), t(c2["lam"])

            if stride == 1:
                def step_c2(i):
                    j = i % nset
                    L.pulp_nn_depthwise_3x3_s1(xs2[j], outs2[j], 58, 56, 128, 1, 1, w2, c2["out_shift"], 0, k2, l2,
                                               1, 1, None)
                want = oracle.depthwise_3x3_s1(xin[:2], c2["w"], c2["k"], c2["lam"], 0, c2["out_shift"], 1, 1, 1, 1, 32)
                kern = KERNELS["cfg2_dw_s1"]
            else:
                def step_c2(i):
                    j = i % nset
                    L.pulp_nn_depthwise_generic(xs2[j], None, b2, outs2[j], w2, None, k2, l2, 0, c2["out_shift"],
                                                56, 56, 128, 28, 28, 128, 3, 3, 1, 1, 1, 1, 2, 2, 1, 1)
                want = oracle.depthwise_generic(xin[:2], c2["w"], c2["bias"], c2["k"], c2["lam"], 0, c2["out_shift"],
                                                (1, 1, 1, 1), (2, 2), 1, 1, 32)
                kern = KERNELS["cfg2_dw_s2"]
            wall, dev, tm = time_launches(step_c2, steps, warm)
            layer_record(c2["name"] + "_b256", c2["ops"], c2["bytes"], wall, dev, tm,
                         np.array_equal(outs2[0][:2].cpu().numpy(), want), "hbm", kern)
            del xs2, outs2

        # config 4: 64-bit batch-norm 3x3 conv at batch 64 (the MFMA-bound layer)
        c4 = workloads.config4(batch=64, relu=1)
        L4 = libs[64]
        x4 = t(c4["x"])
        nset = 4
        xs4 = [x4] + [x4.clone() for _ in range(nset - 1)]
        outs4 = [torch.zeros((64, 63, 63, 256), dtype=torch.uint8, device="cuda") for _ in range(nset)]
        w4, b4, k4, l4 = t(c4["w"]), t(c4["bias"]), t(c4["k"]), t(c4["lam"])
        L4.set_batch(64)

        def step_c4(i):
            j = i % nset
            L4.pulp_nn_conv_Ho_parallel(xs4[j], None, b4, outs4[j], w4, k4, l4, 0, c4["out_shift"], 64, 64, 256, 63, 63,
                                        256, 3, 3, 1, 0, 1, 0, 1, 1, 1, 1)

        wall, dev, tm = time_launches(step_c4, max(5, steps // 4), 2, series=True)
        want = oracle.conv(c4["x"][:1], c4["w"], c4["bias"], c4["k"], c4["lam"], 0, c4["out_shift"], c4["pads"],
                           c4["strides"], 1, 1, 64, out_hw=(63, 63))
        layer_record(c4["name"] + "_b64", c4["ops"], c4["bytes"], wall, dev, tm,
                     np.array_equal(outs4[0][:1].cpu().numpy(), want), "mfma",
                     KERNELS["cfg4_conv"] + " (persistent workgroups on patches of 4 x 64 pixels x 256 channels, LDS-direct loads)",
                     note="random int8 operands: the matrix cores alone sustain 3.6-4.0 POP/s on this data (the clock "
                          "drops under the power limit: profiles/mfma_ceiling.txt); where this kernel's time goes, part "
                          "by part: profiles/conv_cfg4_phases_ablation.txt")
        # the rest of configuration 4: maxpool 2x2 s2 (63 -> 32) and the 1024 -> 4096 linear layer
        pooled = [torch.zeros((64, 32, 32, 256), dtype=torch.uint8, device="cuda") for _ in range(nset)]

        def step_mp(i):
            j = i % nset
            L4.pulp_nn_maxpool(outs4[j], pooled[j], 63, 63, 256, 32, 32, 2, 2, 0, 0, 0, 0, 2, 2)

        wall, dev, tm = time_launches(step_mp, steps, warm)
        want = oracle.maxpool(outs4[0][:2].cpu().numpy(), (2, 2), (2, 2), out_hw=(32, 32))
        mp_bytes = 64 * (63 * 63 * 256 + 32 * 32 * 256)
        layer_record("cfg4_maxpool2x2_s2_63x63x256_b64", 0, mp_bytes, wall, dev, tm,
                     np.array_equal(pooled[0][:2].cpu().numpy(), want), "hbm", KERNELS["cfg4_maxpool"])
        gen = torch.Generator(device="cuda")
        gen.manual_seed(20244)
        vec = torch.randint(0, 256, (64, 1024), dtype=torch.uint8, device="cuda", generator=gen)
        lw, lb, lk, ll = t(c4["lin_w"]), t(c4["lin_bias"]), t(c4["lin_k"]), t(c4["lin_lam"])
        lout = torch.zeros((64, 4096), dtype=torch.uint8, device="cuda")

        def step_lin(i):
            L4.pulp_nn_linear(vec, lb, lout, lw, lk, ll, 0, c4["lin_shift"], 1024, 4096, 1, 1)

        wall, dev, tm = time_launches(step_lin, steps, warm)
        want = oracle.linear(vec.cpu().numpy(), c4["lin_w"], c4["lin_bias"], c4["lin_k"], c4["lin_lam"], 0,
                             c4["lin_shift"], 1, 1, 64)
        layer_record("cfg4_linear_1024_4096_b64", 2 * 64 * 1024 * 4096, 64 * (1024 + 4096) + 4096 * 1024 + 4096 * 17,
                     wall, dev, tm, np.array_equal(lout.cpu().numpy(), want), "hbm", KERNELS["cfg4_linear"],
                     note="4.5 MB per launch: bound by launch and memory latency")
        del xs4, outs4, pooled

        # configuration 3: the whole MobileNetV1-0.5 chain at batch 256, the layout change in front of every
        # depthwise layer fused into it (pulp_nn_hip_depthwise_hwc)
        from pulp_nn_amd import mobilenet
        net = mobilenet.build(256)
        runner = mobilenet.Runner(libs[32], net)
        x3 = t(net["x"])

        def step_net(i):
            runner.run(x3)

        wall, dev, tm = time_launches(step_net, max(5, steps // 4), 2)
        libs[32].sync()
        import hashlib
        dig = json.load(open(os.path.join(ROOT, "tests", "golden", "config_digests.json")))["cfg3_b256_logits"]["sha256"]
        ok = hashlib.sha256(runner.logits.cpu().numpy().tobytes()).hexdigest() == dig
        if not ok:
            failures.append("cfg3 chain")
        layers.append({"layer": "cfg3_mobilenet_v1_0.5_128x128_b256 (whole chain)", "ms": round(dev, 5),
                       "wall_ms": round(wall, 5), "timing": tm["device_us_per_step"],
                       "shader_mhz_behind_region": tm["shader_mhz_behind_region"], "gops": round(net["ops"] / (dev * 1e-3) / 1e9, 1),
                       "launches": runner.launches if hasattr(runner, "launches") else None,
                       "images_per_s": round(256 / (wall * 1e-3), 1),
                       "mfma_frac": round(net["ops"] / (dev * 1e-3) / PEAK_INT8_OPS, 4),
                       "parity": "bit-exact (logits digest)" if ok else "MISMATCH"})
        # one block of that chain on its own: 3x3 depthwise + pointwise on 8 x 8 x 256 planes, as one launch
        # (pulp_nn_hip_dw_pw_hwc) and as the two launches the reference's call sequence makes
        Lb = libs[32]
        Lb.set_batch(256)
        rb = np.random.Generator(np.random.PCG64(77))
        Cb, Wb = 256, 8
        xb = rb.integers(0, 256, (256, Wb, Wb, Cb), dtype=np.uint8)
        dww = rb.integers(-128, 128, (Cb, 3, 3), dtype=np.int8)
        pww = rb.integers(-128, 128, (Cb, Cb), dtype=np.int8)
        kb1, lb1 = rb.integers(2 ** 12, 2 ** 14, Cb).astype(np.int32), rb.integers(-2 ** 16, 2 ** 16, Cb).astype(np.int32)
        kb2, lb2 = rb.integers(2 ** 8, 2 ** 10, Cb).astype(np.int32), rb.integers(-2 ** 16, 2 ** 16, Cb).astype(np.int32)
        sh1, sh2 = 16, 20
        xbd, dwwd, pwwd = t(xb), t(dww), t(pww)
        kb1d, lb1d, kb2d, lb2d = t(kb1), t(lb1), t(kb2), t(lb2)
        mid = torch.zeros((256, Wb, Wb, Cb), dtype=torch.uint8, device="cuda")
        ob1, ob2 = torch.zeros_like(mid), torch.zeros_like(mid)

        def step_block_fused(i):
            Lb.dw_pw_hwc(xbd, ob1, Wb, Wb, Cb, Wb, Wb, Cb, 1, dwwd, None, kb1d, lb1d, 0, sh1, 1, 1,
                         pwwd, None, kb2d, lb2d, 0, sh2, 1, 1)

        def step_block_two(i):
            Lb.depthwise_hwc(xbd, None, mid, dwwd, kb1d, lb1d, 0, sh1, Wb, Wb, Cb, Wb, Wb, 1, 1, 1)
            Lb.pulp_nn_pointwise_HoWo_parallel(mid, None, None, ob2, pwwd, kb2d, lb2d, 0, sh2, Wb, Wb, Cb, Wb, Wb, Cb,
                                               1, 1, 0, 0, 0, 0, 1, 1, 1, 1)

        _, dev_f, _ = time_launches(step_block_fused, steps, 5)
        _, dev_t, _ = time_launches(step_block_two, steps, 5)
        Lb.sync()
        nchk = 8
        want_mid = oracle.depthwise_generic(np.ascontiguousarray(xb[:nchk].transpose(0, 3, 1, 2)), dww, None, kb1, lb1, 0, sh1,
                                            (1, 1, 1, 1), (1, 1), 1, 1)
        want_b = oracle.pointwise(want_mid, pww, None, kb2, lb2, 0, sh2, 1, 1)
        ok = np.array_equal(ob1[:nchk].cpu().numpy(), want_b) and np.array_equal(ob2.cpu().numpy(), ob1.cpu().numpy())
        if not ok:
            failures.append("cfg3 block")
        blk_bytes = 2 * 256 * Wb * Wb * Cb + Cb * 9 + Cb * Cb + 4 * Cb * 4
        layers.append({"layer": "cfg3_block_dw3x3_pw_8x8x256_b256", "ms": round(dev_f, 5), "ms_two_launches": round(dev_t, 5),
                       "hbm_gbs": round(blk_bytes / (dev_f * 1e-3) / 1e9, 1), "hbm_frac": round(blk_bytes / (dev_f * 1e-3) / PEAK_HBM, 4),
                       "parity": "bit-exact (8 images vs the oracle's two-layer chain; all images vs the two launches)" if ok else "MISMATCH",
                       "note": "8.4 MB per launch: bound by launch and memory latency"})
        rec["layers"] = layers

    # ---- CPU baseline: the oracle on this machine's host cores --------------------
    if not args.no_cpu:
        threads = oracle.default_threads()
        n_img = 64
        xs_cpu = c1["x"][:n_img]
        oracle.pointwise(xs_cpu[:threads], c1["w"], c1["bias"], None, None, c1["out_mult"], c1["out_shift"], 1, 0, 32,
                         nthreads=threads)
        reps, t0 = 0, time.perf_counter()
        while True:
            oracle.pointwise(xs_cpu, c1["w"], c1["bias"], None, None, c1["out_mult"], c1["out_shift"], 1, 0, 32,
                             nthreads=threads)
            reps += 1
            el = time.perf_counter() - t0
            if el > 12.0:
                break
        cpu_gops = (c1["ops"] / 256 * n_img * reps) / el / 1e9
        rec["cpu_baseline"] = {
            "value": round(cpu_gops, 2), "unit": "GOPS", "cores": threads, "kind": "port",
            "sample": "%d x %d images of the same workload (scalar C restatement of the reference, -O3 "
                      "-march=native, one image row per OpenMP task), %.1f s" % (reps, n_img, el),
            "images_per_s": round(n_img * reps / el, 1)}

        # configs[0] as BASELINE.json states it: batch 1, one thread (the reference runs one image on one cluster)
        def cpu_timed(fn, budget_s):
            fn()
            reps, t0 = 0, time.perf_counter()
            while True:
                fn()
                reps += 1
                el = time.perf_counter() - t0
                if el > budget_s:
                    return el / reps, reps

        c0 = workloads.config0(batch=1)
        sec, reps = cpu_timed(lambda: oracle.conv(c0["x"], c0["w"], c0["bias"], c0["k"], c0["lam"], 0, c0["out_shift"],
                                                  c0["pads"], c0["strides"], 1, 1, 32, nthreads=1), 2.0)
        rec["cpu_baseline_cfg0_b1"] = {
            "value": round(c0["ops"] / sec / 1e9, 2), "unit": "GOPS", "cores": 1, "kind": "port",
            "ms_per_image": round(sec * 1e3, 4), "images_per_s": round(1.0 / sec, 1),
            "sample": "configs[0] (3x3 conv 16x16x32 -> 64, 32-bit batch-norm + ReLU), batch 1, one thread, %d runs" % reps}
        if not args.no_layers:
            # the other layers on the host cores, a few images each (reported baselines, not targets)
            cpu_layers = {}
            c2 = workloads.config2(batch=2 * threads, stride=1)
            xin = np.pad(c2["x"], ((0, 0), (0, 0), (1, 1), (0, 0)))
            sec, reps = cpu_timed(lambda: oracle.depthwise_3x3_s1(xin, c2["w"], c2["k"], c2["lam"], 0, c2["out_shift"], 1, 1,
                                                                 1, 1, 32, nthreads=threads), 3.0)
            cpu_layers["cfg2_depthwise3x3_s1"] = {"gops": round(c2["ops"] / sec / 1e9, 2), "images_per_s": round(2 * threads / sec, 1)}
            c2 = workloads.config2(batch=2 * threads, stride=2)
            sec, reps = cpu_timed(lambda: oracle.depthwise_generic(c2["x"], c2["w"], c2["bias"], c2["k"], c2["lam"], 0,
                                                                  c2["out_shift"], (1, 1, 1, 1), (2, 2), 1, 1, 32,
                                                                  nthreads=threads), 3.0)
            cpu_layers["cfg2_depthwise3x3_s2"] = {"gops": round(c2["ops"] / sec / 1e9, 2), "images_per_s": round(2 * threads / sec, 1)}
            c4 = workloads.config4(batch=1, relu=1)
            sec, reps = cpu_timed(lambda: oracle.conv(c4["x"], c4["w"], c4["bias"], c4["k"], c4["lam"], 0, c4["out_shift"],
                                                      c4["pads"], c4["strides"], 1, 1, 64, out_hw=(63, 63), nthreads=threads), 5.0)
            cpu_layers["cfg4_conv3x3_bn64"] = {"gops": round(c4["ops"] / sec / 1e9, 2), "images_per_s": round(1.0 / sec, 2)}
            rec["cpu_baseline_layers"] = {"cores": threads, "kind": "port", "layers": cpu_layers,
                                          "sample": "2 x cores images per depthwise call, one image per convolution call, "
                                                    "3-5 s each"}

    if failures:
        rec["value"] = None
        rec["parity_failures"] = failures
    print(json.dumps(rec))
    if failures:
        sys.exit(1)


if __name__ == "__main__":
    main()
