#!/usr/bin/env python3
"""Benchmark of the dense feed-forward hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg4|cfg5|cfg3|cfg2|cfg1]

A "step" is one pass of the path over one batch of synthetic input that is already resident in
HBM when the timed region starts: forward + backward + update (training workloads), forward
(cfg5), one epoch of sequential rows (cfg1/cfg2, exact mode).  One JSON line is printed.

Default workload cfg4 = BASELINE.json configs[3], the configuration its metric and target are
quoted on: MLP 4096-4096-4096-4096-4096-1024, ReLU, softmax cross-entropy, batch 8192, bf16
weights/activations, fp32 accumulation, fp32 master weights, SGD with momentum.

The default run adds, outside the timed region and under "detail" (--no-extras leaves them out):
  sustained    200 further steps, the configuration's own schedule length
  loss_check   the same warm-up + timed steps from the same start in fp32 on the GPU: the bf16 loss
               has to be the fp32 loss within 2e-2
  infer        the metric's other half: cfg5 (e4m3 inference, batch 16384) timed the same way, with
               its own roofline entry
  vendor_gemm  the vendor library's plain bf16 GEMM on the step's two product shapes: what the chip
               sustains on them, beside the published peak
  other_configs  BASELINE.json's other configurations at their default step counts, value and ms per
               step each: cfg3 (fp32 training), cfg1 and cfg2 (exact mode, one network), and cfg1 with
               1024 and 4096 networks side by side in one launch
"""
import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "glades-ml_amd"))

PEAKS = {"bf16": 2500.0, "fp8": 5000.0, "f32": 157.3}  # dense MFMA, TFLOP/s
HBM_PEAK = 8000.0  # GB/s

# Memory bytes per launch of a workload's dominant kernel, from two `rocprofv3 --pmc` runs of this
# script (FETCH_SIZE, then WRITE_SIZE, KiB per dispatch averaged over the kernel's launches), each
# scaled by what the same counter reads for the 1 GiB copy of `--workload copy`
# (FETCH_SIZE x 2.000, WRITE_SIZE x 1.000); profiles/gemm_lowprec_pmc.md has the runs.  The
# counters sit between L2 and the fabric, so lines re-fetched from the memory-side cache count again.
# A workload / kernel pair that was not measured reports null.
TRAFFIC_PROFILE = "profiles/gemm_lowprec_pmc.md"


def measured_traffic(workload, kernel):
    """(bytes per launch, source) from the `traffic` lines of the committed counter summary, or (None, None):
    `traffic <workload> <kernel> fetch_kib F write_kib W fetch_scale a write_scale b commit <hash>`."""
    try:
        for line in open(os.path.join(ROOT, TRAFFIC_PROFILE)):
            t = line.split()
            if len(t) >= 13 and t[0] == "traffic" and t[1] == workload and t[2] == kernel:
                kv = dict(zip(t[3::2], t[4::2]))
                byts = (float(kv["fetch_kib"]) * float(kv["fetch_scale"]) + float(kv["write_kib"]) * float(kv["write_scale"])) * 1024
                return int(byts), f"{TRAFFIC_PROFILE}, rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of commit {kv['commit']} (not measured in this run)"
    except (OSError, KeyError, ValueError):
        pass
    return None, None


WORKLOADS = {
    "cfg4": dict(desc="bf16 train MLP 4096-4096-4096-4096-4096-1024 ReLU softmax-CE, batch 8192, SGD momentum 0.9, fp32 master",
                 sizes=[4096, 4096, 4096, 4096, 4096, 1024], batch=8192, rows=262144, dtype="bf16", kind="train"),
    "cfg5": dict(desc="e4m3 inference MLP 8192-8192-8192-8192-1024 ReLU, batch 16384, fp32 scale per weight output channel, activations re-quantised per token between layers",
                 sizes=[8192, 8192, 8192, 8192, 1024], batch=16384, rows=16384, dtype="fp8", kind="infer"),
    "cfg3": dict(desc="fp32 train MLP 784-1024-1024-10 ReLU softmax-CE, batch 512, SGD lr .05 momentum .9 L2 1e-4",
                 sizes=[784, 1024, 1024, 10], batch=512, rows=60000, dtype="f32", kind="train"),
    "cfg2": dict(desc="exact mode MLP 32-64-64-1 tanh/tanh/linear MSE, 10000 rows, mb 256, lr .01 momentum .9",
                 sizes=[32, 64, 64, 1], batch=256, rows=10000, dtype="f32", kind="exact"),
    "cfg1": dict(desc="exact mode MLP 4-16-3 sigmoid BCE, 150 rows, mb 150, lr .01 momentum .9",
                 sizes=[4, 16, 3], batch=150, rows=150, dtype="f32", kind="exact"),
    # the two narrow configurations in canonical (batched) mode; cfg1 here is BASELINE.json's configs[0] as written
    "cfg1_canonical": dict(desc="canonical mode MLP 4-16-3 sigmoid / softmax cross-entropy, 150 rows, full batch, lr .1 momentum .9, Xavier-uniform",
                           sizes=[4, 16, 3], batch=150, rows=150, dtype="f32", kind="narrow"),
    "cfg2_canonical": dict(desc="canonical mode MLP 32-64-64-1 tanh/tanh/linear MSE, 10000 rows, mb 256, lr .01 momentum .9",
                           sizes=[32, 64, 64, 1], batch=256, rows=10000, dtype="f32", kind="narrow"),
}


def train_flops_per_sample(sizes):
    w = [sizes[l] * sizes[l + 1] for l in range(len(sizes) - 1)]
    return 6 * sum(w) - 2 * w[0]  # forward + weight gradient everywhere, back-prop except layer 0


def infer_flops_per_sample(sizes):
    return 2 * sum(sizes[l] * sizes[l + 1] for l in range(len(sizes) - 1))


def he_weights(sizes, seed):
    rng = np.random.default_rng(seed)
    return [(rng.standard_normal((sizes[l + 1], sizes[l]), dtype=np.float32) * np.float32(np.sqrt(2.0 / sizes[l])))
            for l in range(len(sizes) - 1)]


def hip_timed(net, fn, steps):
    """Wall time of `steps` calls bracketed by device synchronisation on both sides."""
    import torch
    net.sync()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for s in range(steps):
        fn(s)
    net.sync()
    torch.cuda.synchronize()
    return time.perf_counter() - t0


def kernel_profile(net, fn, steps):
    """Per-kernel HIP-event timing (events recorded on the stream the kernels run on)."""
    net.profile(True)
    net.profile_reset()
    for s in range(steps):
        fn(s)
    net.sync()
    tab = net.profile_table()
    net.profile(False)
    return tab


def run_canonical(w, args):
    import torch
    import pyglades as pg
    sizes, B, N = w["sizes"], w["batch"], w["rows"]
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev)
    g.manual_seed(1234)
    dt = {"bf16": pg.BF16, "f32": pg.F32, "fp8": pg.FP8_INFER}[w["dtype"]]
    nl = len(sizes) - 1
    acts = [pg.RELU] * (nl - 1) + ([pg.SOFTMAX] if w["kind"] == "train" else [pg.RELU])
    if w["name"] == "cfg3":
        hyper = dict(lr=0.05, mom=0.9, wd2=1e-4)
    else:
        hyper = dict(lr=0.01, mom=0.9, wd2=0.0)
    spec = pg.make_spec(sizes, acts, cost=pg.CLASSIFICATION, mode=pg.MODE_CANONICAL, dtype=dt, batch=B, **hyper)
    net = pg.Net(spec)
    Ws = he_weights(sizes, 42)
    for l in range(nl):
        net.set_params(l, Ws[l])
    # synthetic table, generated on the device (torch is only the allocator / generator here)
    if w["name"] == "cfg3":
        X = torch.rand((N, sizes[0]), device=dev, generator=g, dtype=torch.float32)
    else:
        X = torch.randn((N, sizes[0]), device=dev, generator=g, dtype=torch.float32)
    Y = None
    if w["kind"] == "train":
        T = torch.randn((sizes[0], sizes[-1]), device=dev, generator=g, dtype=torch.float32)
        Y = torch.zeros((N, sizes[-1]), device=dev, dtype=torch.float32)
        for r in range(0, N, 32768):
            lab = (X[r:r + 32768] @ T).argmax(1)
            Y[r:r + 32768].scatter_(1, lab[:, None], 1.0)
        del T
    torch.cuda.synchronize()
    net.set_dataset_device(X.data_ptr(), Y.data_ptr() if Y is not None else 0, N)
    nb = N // B
    if w["kind"] == "train":
        fn = lambda s: net.train_step((s % nb) * B, B, want_metrics=False)  # noqa: E731
        flops = train_flops_per_sample(sizes)
    else:
        net.quantize_fp8(want=False)
        net.set_fp8_activation_scaling(pg.FP8_ACT_PER_TOKEN if getattr(args, "fp8_act", "block32") == "per_token" else pg.FP8_ACT_BLOCK32)
        fn = lambda s: net.forward_resident((s % nb) * B, B)  # noqa: E731
        flops = infer_flops_per_sample(sizes)
    for s in range(args.warmup):
        fn(s)
    el = hip_timed(net, fn, args.steps)
    loss = net.last_metrics().loss if w["kind"] == "train" else None
    prof = kernel_profile(net, fn, min(args.steps, 5))
    more = {}
    if w["kind"] == "train" and getattr(args, "extras", False):
        # the configuration's own schedule length, untouched by the short timed region's boost clocks
        n_sus = 200
        el_sus = hip_timed(net, fn, n_sus)
        more["sustained"] = dict(steps=n_sus, ms_per_step=round(el_sus / n_sus * 1e3, 4), value=round(n_sus * B / el_sus, 1),
                                 step_frac_of_peak=round(flops * B / (el_sus / n_sus) / 1e12 / PEAKS[w["dtype"]], 4))
    net.close()
    if w["kind"] == "train" and w["dtype"] == "bf16" and getattr(args, "extras", False):
        # the same warm-up + timed steps from the same start in fp32 (the path that is pinned to the CPU
        # restatement): the low-precision run's last loss has to be the fp32 run's within 2e-2
        ref = pg.Net(pg.make_spec(sizes, acts, cost=pg.CLASSIFICATION, mode=pg.MODE_CANONICAL, dtype=pg.F32, batch=B, **hyper))
        for l in range(nl):
            ref.set_params(l, Ws[l])
        ref.set_dataset_device(X.data_ptr(), Y.data_ptr(), N)
        for s_ in range(args.warmup):
            ref.train_step((s_ % nb) * B, B, want_metrics=False)
        for s_ in range(args.steps):
            ref.train_step((s_ % nb) * B, B, want_metrics=False)
        ref_loss = ref.last_metrics().loss
        ref.close()
        rel = abs(loss - ref_loss) / abs(ref_loss)
        more["loss_check"] = dict(bf16=loss, fp32=ref_loss, rel=round(rel, 6), tolerance=2e-2, ok=bool(rel <= 2e-2))
    # dominant kernel + its algorithmic FLOPs per launch
    gemm_names = {
        "bf16": {"gemm_bf16_forward": "fwd_hidden", "gemm_bf16_forward_out": "fwd_out", "gemm_bf16_dgrad": "dgrad",
                 "gemm_bf16_wgrad_sgd": "wgrad_t256", "gemm_bf16_wgrad_sgd_t128": "wgrad_t128"},
        "fp8": {"gemm_fp8_forward": "fwd_hidden", "gemm_fp8_forward_out": "fwd_out"},
        "f32": {"gemm_f32_forward": "fwd_all", "gemm_f32_dgrad": "dgrad", "gemm_f32_wgrad_sgd": "wgrad"},
    }[w["dtype"]]
    wl = [sizes[l] * sizes[l + 1] for l in range(nl)]
    # the bf16 weight gradient of a layer runs on 128 x 128 tiles where 256 x 256 ones would leave CUs idle
    # (the library's rule); the two are separate kernels in the profile
    small = [(sizes[l + 1] // 256) * (sizes[l] // 256) < 256 for l in range(nl)]
    per_step = {"fwd_hidden": 2 * B * sum(wl[:-1]), "fwd_out": 2 * B * wl[-1], "fwd_all": 2 * B * sum(wl),
                "dgrad": 2 * B * sum(wl[1:]), "wgrad": 2 * B * sum(wl),
                "wgrad_t256": 2 * B * sum(w_ for w_, sm in zip(wl, small) if not sm),
                "wgrad_t128": 2 * B * sum(w_ for w_, sm in zip(wl, small) if sm)}
    psteps = min(args.steps, 5)
    kern = {}
    for name, (ms, cnt) in prof.items():
        kern[name] = dict(total_ms=ms, launches=cnt, avg_ms=ms / max(cnt, 1))
    dom = max((n for n in kern if n in gemm_names), key=lambda n: kern[n]["total_ms"])
    fl_launch = per_step[gemm_names[dom]] * psteps / kern[dom]["launches"]
    ach = fl_launch / (kern[dom]["avg_ms"] * 1e-3) / 1e12
    peak = PEAKS[w["dtype"]]
    traffic, traffic_source = measured_traffic(w["name"], dom)
    roof = dict(bound="mfma", kernel=dom, achieved=round(ach, 2), peak=peak, unit="TFLOP/s", frac=round(ach / peak, 4),
                traffic=traffic, traffic_source=traffic_source, flop_per_launch=fl_launch,
                avg_launch_ms=round(kern[dom]["avg_ms"], 4))
    total_ms = sum(k["total_ms"] for k in kern.values())
    breakdown = {n: round(k["total_ms"] / psteps, 4) for n, k in sorted(kern.items(), key=lambda kv: -kv[1]["total_ms"])}
    value = args.steps * B / el
    step_tflops = flops * B / (el / args.steps) / 1e12
    extra = dict(step_tflops=round(step_tflops, 2), step_frac_of_peak=round(step_tflops / peak, 4),
                 kernel_ms_per_step=breakdown, kernel_ms_sum=round(total_ms / psteps, 4), final_loss=loss, **more)
    return value, el, roof, extra


def vendor_gemm_rates(sizes, B, iters=30):
    """The vendor library's plain bf16 GEMM (torch.matmul -> hipBLASLt: one output, no epilogue) on the
    three product shapes of a hidden layer's training step: what this chip sustains on them under its
    power limit, beside the published peak."""
    import torch
    dev = torch.device("cuda:0")
    n = sizes[1]
    shapes = {"forward / back-propagation (batch x n x n)": (B, n, n), "weight gradient (n x n x batch)": (n, n, B)}
    out = {}
    for name, (M, N, K) in shapes.items():
        a = torch.randn((M, K), device=dev, dtype=torch.bfloat16)
        b = torch.randn((N, K), device=dev, dtype=torch.bfloat16)
        for _ in range(5):
            torch.matmul(a, b.t())
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(iters):
            torch.matmul(a, b.t())
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / iters
        tf = 2.0 * M * N * K / dt / 1e12
        out[name] = dict(ms=round(dt * 1e3, 4), tflops=round(tf, 1), frac_of_peak=round(tf / PEAKS["bf16"], 4))
    return out


def run_exact(w, args):
    import pyglades as pg
    sizes, N, mb = w["sizes"], w["rows"], w["batch"]
    rng = np.random.default_rng(1234)
    if w["name"] == "cfg2":
        t = np.arange(N + 32, dtype=np.float64)
        f, ph = rng.random(3) * 0.05 + 0.01, rng.random(3) * 6.28
        sig = sum(np.sin(2 * np.pi * f[k] * t + ph[k]) for k in range(3)) + rng.standard_normal(N + 32) * 0.05
        sig = (sig - sig.min()) / (sig.max() - sig.min())
        X = np.stack([sig[i:i + 32] for i in range(N)]).astype(np.float32)
        Y = sig[32:32 + N, None].astype(np.float32)
        acts, params, cost = [pg.TANH, pg.TANH, pg.LINEAR], [0, 0, 1.0], pg.REGRESSION
    else:
        c = rng.random((3, 4)) * 8
        lab = np.repeat(np.arange(3), 50)
        X = (c[lab] + rng.standard_normal((150, 4)) * 0.5).astype(np.float32)
        X = ((X - X.min(0)) / (X.max(0) - X.min(0)) * 0.98 + 0.01).astype(np.float32)
        Y = np.where(np.eye(3)[lab] > 0, 0.99, 0.01).astype(np.float32)
        acts, params, cost = [pg.SIGMOID, pg.SIGMOID], [0, 0], pg.CLASSIFICATION
    nl = len(sizes) - 1
    spec = pg.make_spec(sizes, acts, lr=0.01, mom=0.9, act_params=params, batch=mb, cost=cost, mode=pg.MODE_EXACT)
    K = max(1, args.subnets)   # networks trained side by side (the subnets of a MetaNetwork), one workgroup each
    nets = []
    for _ in range(K):
        net = pg.Net(spec)
        for l in range(nl):
            lim = np.sqrt(6.0 / (sizes[l] + sizes[l + 1]))
            net.set_params(l, rng.uniform(-lim, lim, (sizes[l + 1], sizes[l])).astype(np.float32), 0.0)
        net.set_dataset(X, Y)
        nets.append(net)
    net = nets[0]

    def epochs(n):
        if K == 1:
            return net.run_epochs_exact(n)[0]
        return pg.run_epochs_exact_multi(nets, n)[0]

    for _ in range(args.warmup):
        epochs(1)
    net.sync()
    t0 = time.perf_counter()
    ms = epochs(args.steps)   # one launch, `steps` epochs
    net.sync()
    el = time.perf_counter() - t0
    kname = "exact_epochs" if K == 1 else "exact_epochs_multi"
    prof = kernel_profile(net, lambda s: epochs(1), 3)
    for n in nets:
        n.close()
    value = K * args.steps * N / el
    k = prof[kname]
    bytes_per_sample = 4 * (sizes[0] + sizes[-1])
    ach = K * bytes_per_sample * N / (k[0] / k[1] * 1e-3) / 1e9
    roof = dict(bound="hbm", kernel=kname, achieved=round(ach, 4), peak=HBM_PEAK, unit="GB/s",
                frac=round(ach / HBM_PEAK, 8), traffic=None, avg_launch_ms=round(k[0] / k[1], 4),
                note="latency-bound: one persistent workgroup per network, rows strictly sequential")
    extra = dict(final_loss=ms[-1][0], final_accuracy=ms[-1][1], flop_per_sample=train_flops_per_sample(sizes), subnets=K)
    return value, el, roof, extra


def narrow_tables(w, pg_or_po):
    """Synthetic tables, activations and weights of the two narrow configurations."""
    m = pg_or_po
    sizes, N = w["sizes"], w["rows"]
    rng = np.random.default_rng(1234)
    if w["name"].startswith("cfg2"):
        t = np.arange(N + 32, dtype=np.float64)
        f, ph = rng.random(3) * 0.05 + 0.01, rng.random(3) * 6.28
        sig = sum(np.sin(2 * np.pi * f[k] * t + ph[k]) for k in range(3)) + rng.standard_normal(N + 32) * 0.05
        X = np.stack([sig[i:i + 32] for i in range(N)]).astype(np.float32)
        Y = sig[32:32 + N, None].astype(np.float32)
        acts, params, cost, hyper = [m.TANH, m.TANH, m.LINEAR], [0, 0, 1.0], m.REGRESSION, dict(lr=0.01, mom=0.9)
    else:
        c = rng.random((3, 4)) * 8
        lab = np.repeat(np.arange(3), 50)
        X = (c[lab] + rng.standard_normal((150, 4)) * 0.5).astype(np.float32)
        Y = np.eye(3, dtype=np.float32)[lab]
        acts, params, cost, hyper = [m.SIGMOID, m.SOFTMAX], [0, 0], m.CLASSIFICATION, dict(lr=0.1, mom=0.9)
    nl = len(sizes) - 1
    Ws = [rng.uniform(-1, 1, (sizes[l + 1], sizes[l])).astype(np.float32) * np.float32(np.sqrt(6.0 / (sizes[l] + sizes[l + 1]))) for l in range(nl)]
    return X, Y, acts, params, cost, hyper, Ws


def run_narrow(w, args):
    """Canonical mode on a narrow network: `steps` epochs through ghip_net_run_epochs_canonical, with the
    library's own choice of kernels (value) and with each of the two paths forced (detail)."""
    import pyglades as pg
    sizes, N, B = w["sizes"], w["rows"], w["batch"]
    X, Y, acts, params, cost, hyper, Ws = narrow_tables(w, pg)
    nl = len(sizes) - 1
    res = {}
    for path, code in (("auto", pg.CANON_PATH_AUTO), ("one_workgroup", pg.CANON_PATH_ONE_WORKGROUP), ("launches", pg.CANON_PATH_LAUNCHES)):
        net = pg.Net(pg.make_spec(sizes, acts, act_params=params, cost=cost, mode=pg.MODE_CANONICAL, dtype=pg.F32, batch=B, **hyper))
        for l in range(nl):
            net.set_params(l, Ws[l])
        net.set_canonical_path(code)
        net.set_dataset(X, Y)
        for _ in range(max(1, args.warmup)):
            net.run_epochs_canonical(B, 1)
        net.sync()
        t0 = time.perf_counter()
        ms = net.run_epochs_canonical(B, args.steps)
        net.sync()
        el = time.perf_counter() - t0
        prof = kernel_profile(net, lambda s_: net.run_epochs_canonical(B, args.steps), 1)
        net.close()
        res[path] = dict(el=el, loss=ms[-1][0], prof=prof)
    el = res["auto"]["el"]
    value = args.steps * N / el
    prof = res["auto"]["prof"]
    dom = max(prof, key=lambda k: prof[k][0])
    kernel_ms = sum(v[0] for v in prof.values())
    bytes_per_sample = 4 * (sizes[0] + sizes[-1])
    ach = args.steps * N * bytes_per_sample / (kernel_ms * 1e-3) / 1e9
    roof = dict(bound="hbm", kernel=dom, achieved=round(ach, 4), peak=HBM_PEAK, unit="GB/s", frac=round(ach / HBM_PEAK, 8), traffic=None,
                avg_launch_ms=round(prof[dom][0] / prof[dom][1], 4),
                note="latency- and issue-bound: table traffic is 4 (inputs + outputs) bytes per row against a few thousand multiply-adds")
    extra = dict(final_loss=res["auto"]["loss"], flop_per_sample=train_flops_per_sample(sizes),
                 paths={k: dict(ms_per_epoch=round(v["el"] / args.steps * 1e3, 4), value=round(args.steps * N / v["el"], 1),
                                launches_per_call=int(sum(c for _, c in v["prof"].values()))) for k, v in res.items()})
    return value, el, roof, extra


def cpu_baseline(w, budget_s=20.0):
    """The CPU restatement (oracle/, kind "port") timed on this host's cores on a bounded sample.  `cores` = the
    threads used, `nproc` = the cores this process may run on; exact mode runs on one thread as the reference does,
    canonical mode on one thread AND on all cores (value = all cores, `one_thread` beside it)."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import pyoracle as po
    sizes = w["sizes"]
    nl = len(sizes) - 1
    nproc = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    cores = min(16, nproc)
    rng = np.random.default_rng(7)
    if w["kind"] == "exact":
        acts = [po.TANH, po.TANH, po.LINEAR] if w["name"] == "cfg2" else [po.SIGMOID, po.SIGMOID]
        params = [0, 0, 1.0] if w["name"] == "cfg2" else [0, 0]
        cost = po.REGRESSION if w["name"] == "cfg2" else po.CLASSIFICATION
        net = po.ExactNet(po.make_spec(sizes, acts, lr=0.01, mom=0.9, act_params=params, batch=w["batch"], cost=cost))
        for l in range(nl):
            net.set_weights(l, (rng.standard_normal((sizes[l + 1], sizes[l])) * 0.1).astype(np.float32))
        N = w["rows"]
        X = rng.random((N, sizes[0])).astype(np.float32)
        Y = (rng.random((N, sizes[-1])) * 0.98 + 0.01).astype(np.float32)
        ep, t0 = 0, time.perf_counter()
        with np.errstate(all="ignore"):
            while time.perf_counter() - t0 < min(budget_s, 5.0):
                net.epoch(X, Y, want_preds=False)
                ep += 1
        el = time.perf_counter() - t0
        return dict(value=round(ep * N / el, 1), unit="samples/s", cores=1, nproc=nproc, kind="port",
                    sample=f"{ep} epochs of {N} rows, exact mode, 1 thread (the reference is single-threaded)")
    if w["kind"] == "narrow":
        X, Y, acts, params, cost, hyper, Ws = narrow_tables(w, po)
        N, B = w["rows"], w["batch"]
        out = {}
        for threads in (1, cores):
            po.lib().go_set_threads(threads)
            net = po.CanonNet(po.make_spec(sizes, acts, act_params=params, cost=cost, **hyper))
            for l in range(nl):
                net.set_params(l, Ws[l])
            ep, t0 = 0, time.perf_counter()
            while time.perf_counter() - t0 < min(budget_s, 3.0):
                for r0 in range(0, N, B):
                    net.step(X[r0:r0 + B], Y[r0:r0 + B])
                ep += 1
            out[threads] = (ep * N / (time.perf_counter() - t0), ep)
        best = max(out, key=lambda k: out[k][0])
        return dict(value=round(out[best][0], 1), unit="samples/s", cores=best, nproc=nproc, kind="port",
                    one_thread=round(out[1][0], 1), all_cores=round(out[cores][0], 1),
                    sample=f"{out[best][1]} epochs of {N} rows in batches of {B}, canonical mode, fp32; 1 thread and {cores} OpenMP threads timed, the faster reported")
    acts = [po.RELU] * (nl - 1) + ([po.SOFTMAX] if w["kind"] == "train" else [po.RELU])
    rows = {"cfg4": 256, "cfg5": 256, "cfg3": 512}.get(w["name"], 256)
    X = rng.standard_normal((rows, sizes[0]), dtype=np.float32)
    Y = np.eye(sizes[-1], dtype=np.float32)[rng.integers(0, sizes[-1], rows)]
    Ws = [(rng.standard_normal((sizes[l + 1], sizes[l]), dtype=np.float32) * np.float32(np.sqrt(2.0 / sizes[l]))) for l in range(nl)]
    rates = {}
    for threads, share in ((cores, 0.8), (1, 0.2)):
        po.lib().go_set_threads(threads)
        net = po.CanonNet(po.make_spec(sizes, acts, lr=0.01, mom=0.9, cost=po.CLASSIFICATION))
        for l in range(nl):
            net.set_params(l, Ws[l])
        reps, t0 = 0, time.perf_counter()
        while True:
            if w["kind"] == "train":
                net.step(X, Y)
            else:
                net.forward(X)
            reps += 1
            if time.perf_counter() - t0 > budget_s * share / 2 or reps >= 50:
                break
        rates[threads] = (reps * rows / (time.perf_counter() - t0), reps)
        del net
    what = "fwd+bwd+update steps" if w["kind"] == "train" else "fp32 forwards"
    return dict(value=round(rates[cores][0], 1), unit="samples/s", cores=cores, nproc=nproc, kind="port", one_thread=round(rates[1][0], 1),
                sample=f"{rates[cores][1]} {what} of {rows} rows (1/{w['batch'] // rows} of a batch), fp32, {cores} OpenMP threads ({rates[1][1]} on 1 thread for one_thread)")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None)
    ap.add_argument("--warmup", type=int, default=None)
    ap.add_argument("--workload", default="cfg4", choices=sorted(WORKLOADS) + ["copy"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true",
                    help="cfg4: skip the untimed extras (fp32 loss check, 200-step sustained rate, cfg5 inference leg, vendor GEMM rates, the other configurations)")
    ap.add_argument("--fp8-act", default="block32", choices=["block32", "per_token"],
                    help="cfg5: activations re-quantised with an E8M0 scale per token and 32 units in the products' epilogues (default), or with one fp32 scale per token by a kernel of its own")
    ap.add_argument("--subnets", type=int, default=1,
                    help="exact workloads: this many networks (MetaNetwork subnets) side by side in one launch; value is their sum")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1", file=sys.stderr)
        sys.exit(2)
    if args.workload == "copy":
        # calibration target for the FETCH_SIZE / WRITE_SIZE counters: a plain device-to-device copy
        # of a known size (1 GiB read + 1 GiB written per launch)
        import torch
        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda:0").normal_()
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps or 10):
            dst.copy_(src)
        torch.cuda.synchronize()
        el = time.perf_counter() - t0
        print(json.dumps({"workload": "copy", "bytes_read_per_launch": src.numel() * 4, "bytes_written_per_launch": src.numel() * 4,
                          "launches": args.steps or 10, "GBps": 2 * src.numel() * 4 * (args.steps or 10) / el / 1e9}))
        return
    w = dict(WORKLOADS[args.workload], name=args.workload)
    if args.steps is None:
        args.steps = {"cfg4": 40, "cfg5": 40, "cfg3": 200, "cfg2": 5, "cfg1": 200, "cfg1_canonical": 500, "cfg2_canonical": 10}[args.workload]
    if args.warmup is None:
        args.warmup = {"cfg4": 5, "cfg5": 5, "cfg3": 20, "cfg2": 1, "cfg1": 5, "cfg1_canonical": 1, "cfg2_canonical": 1}[args.workload]
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    args.extras = args.workload == "cfg4" and not args.no_extras
    if w["kind"] == "exact":
        value, el, roof, extra = run_exact(w, args)
        unit_rows = w["rows"]
    elif w["kind"] == "narrow":
        value, el, roof, extra = run_narrow(w, args)
        unit_rows = w["rows"]
    else:
        value, el, roof, extra = run_canonical(w, args)
        unit_rows = w["batch"]
    if args.extras:
        # the metric's other half, inference samples/s, on its own configuration (cfg5), in the same run; a leg
        # that fails reports why and leaves the headline line intact
        try:
            w5 = dict(WORKLOADS["cfg5"], name="cfg5")
            a5 = argparse.Namespace(steps=40, warmup=5, extras=False)
            v5, el5, roof5, extra5 = run_canonical(w5, a5)
            extra["infer"] = dict(metric="infer samples/sec", value=round(v5, 1), unit="samples/s", steps=a5.steps, warmup=a5.warmup,
                                  ms_per_step=round(el5 / a5.steps * 1e3, 4), dtype="fp8", workload="cfg5: " + w5["desc"],
                                  activation_scaling="per token, an E8M0 scale per 32 units, written by the producing product's epilogue",
                                  flop_per_sample=infer_flops_per_sample(w5["sizes"]), roofline=roof5,
                                  step_frac_of_peak=extra5["step_frac_of_peak"], kernel_ms_per_step=extra5["kernel_ms_per_step"])
            if not args.no_cpu_baseline:
                extra["infer"]["cpu_baseline"] = cpu_baseline(w5, budget_s=8.0)
            # the same pass with one fp32 scale per token, re-quantised by a kernel of its own
            a5.fp8_act = "per_token"
            v5t, el5t, roof5t, extra5t = run_canonical(w5, a5)
            extra["infer"]["per_token_fp32_scale"] = dict(value=round(v5t, 1), ms_per_step=round(el5t / a5.steps * 1e3, 4),
                                                          step_frac_of_peak=extra5t["step_frac_of_peak"], kernel_ms_per_step=extra5t["kernel_ms_per_step"])
        except Exception as e:  # noqa: BLE001
            extra["infer"] = dict(error=repr(e))
        try:
            extra["vendor_gemm"] = vendor_gemm_rates(w["sizes"], w["batch"])
        except Exception as e:  # noqa: BLE001
            extra["vendor_gemm"] = dict(error=repr(e))
        others = {}
        for name, subnets in (("cfg3", 1), ("cfg1", 1), ("cfg2", 1), ("cfg1", 1024), ("cfg1", 4096), ("cfg1_canonical", 1), ("cfg2_canonical", 1)):
            key = name if subnets == 1 else f"{name}_x{subnets}"
            try:
                wo = dict(WORKLOADS[name], name=name)
                ao = argparse.Namespace(steps={"cfg3": 200, "cfg2": 5, "cfg1": 200, "cfg1_canonical": 500, "cfg2_canonical": 10}[name],
                                        warmup={"cfg3": 20, "cfg2": 1, "cfg1": 5, "cfg1_canonical": 1, "cfg2_canonical": 1}[name],
                                        extras=False, subnets=subnets)
                run = {"exact": run_exact, "narrow": run_narrow}.get(wo["kind"], run_canonical)
                vo, elo, roofo, extrao = run(wo, ao)
                others[key] = dict(value=round(vo, 1), unit="samples/s", steps=ao.steps, ms_per_step=round(elo / ao.steps * 1e3, 4),
                                   dtype=wo["dtype"], workload=f"{name}: {wo['desc']}" + (f", {subnets} subnets side by side" if subnets > 1 else ""),
                                   kernel=roofo["kernel"], kernel_avg_launch_ms=roofo["avg_launch_ms"],
                                   roofline={k: roofo[k] for k in ("bound", "kernel", "achieved", "peak", "unit", "frac", "traffic") if k in roofo})
                if "step_frac_of_peak" in extrao:
                    others[key]["step_frac_of_peak"] = extrao["step_frac_of_peak"]
                if "paths" in extrao:
                    others[key]["paths"] = extrao["paths"]
                if not args.no_cpu_baseline and subnets == 1:
                    others[key]["cpu_baseline"] = cpu_baseline(wo, budget_s=6.0)
            except Exception as e:  # noqa: BLE001
                others[key] = dict(error=repr(e))
        extra["other_configs"] = others
    out = {
        "metric": "train samples/sec (fwd+bwd+update)" if w["kind"] != "infer" else "infer samples/sec",
        "value": round(value, 1), "unit": "samples/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(el / args.steps * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": w["dtype"], "data": "synthetic",
        "config": {"workload": f"{args.workload}: {w['desc']}" + (f", {args.subnets} subnets side by side" if w["kind"] == "exact" and args.subnets > 1 else ""),
                   "rows_per_step": unit_rows,
                   "flop_per_sample": train_flops_per_sample(w["sizes"]) if w["kind"] != "infer" else infer_flops_per_sample(w["sizes"])},
        "roofline": roof,
    }
    if w["kind"] == "infer":
        out["config"]["activation_scaling"] = ("one fp32 scale per token, a re-quantisation kernel between layers" if args.fp8_act == "per_token" else
                                               "per token, an E8M0 scale per 32 units, written by the producing product's epilogue")
    out["detail"] = extra
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(w)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
