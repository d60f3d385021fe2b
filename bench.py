#!/usr/bin/env python3
"""Benchmark of the conv / max-pool hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-extra] [--per-layer]

A step is one pass of the conv hot path over one synthetic batch that is already
resident in HBM: forward, backward-data and backward-weight (+ bias gradient) of
a single conv layer, N=32, 64->64 channels, 56x56, 3x3, stride 1, pad 1, fp32.
Prints ONE JSON line.  `value` is the conv fwd+bwd rate in TFLOP/s over exactly K
steps timed with events on the library's own stream.

`roofline` describes the dominant kernel (the implicit-GEMM MFMA kernel that runs
forward and backward-data): algorithmic FLOPs of one launch divided by the mean
duration of that launch, taken from event pairs the library records directly
around the kernel in a second pass over the same K steps.

`cpu_baseline` times the NumPy restatement of the reference algorithm (the
parity oracle) on the host cores of this machine, on the same workload; its
`other_workloads` hold the same for the max-pool, README-net, ResNet-18 training
and ResNet-18 inference configurations, each beside the GPU figure in `extra`.

`--per-layer` times every distinct ResNet-18 convolution (N=32) pass by pass and
prints one JSON line with a row per (layer, pass).

The ResNet-18 workloads of `extra` are a caller of the package, not part of it: the model
(and the NumPy forward used as their CPU leg) is tests/resnet18.py, so the test tree has
to be present beside this file; `--no-extra` runs without it.

Everything goes through libxsmi355.so; there is no fallback path.
"""
import argparse
import json
import os
import re
import statistics
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(1, os.path.join(ROOT, "tests"))      # the ResNet-18 workload (tests/resnet18.py) is a caller of the package

FP32_MFMA_PEAK_TFLOPS = 157.3
HBM_PEAK_GBPS = 8000.0

# the benchmark conv configuration: N, C, H, W, K, R, S, stride, pad
CONV = dict(N=32, C=64, H=56, W=56, K=64, R=3, S=3, stride=(1, 1), pad=1)
# the benchmark max-pool configuration
POOL = dict(N=32, C=64, H=112, W=112, k=3, stride=(2, 2), pad=1)

# The 11 distinct convolutions of ResNet-18 at N=32, 224x224 input: name, count, Cin, Cout, H_in, k, stride, pad
RESNET18_CONVS = [
    ("stem 3->64 7x7/2 224", 1, 3, 64, 224, 7, 2, 3),
    ("layer1 64->64 3x3 56", 4, 64, 64, 56, 3, 1, 1),
    ("layer2.0a 64->128 3x3/2 56", 1, 64, 128, 56, 3, 2, 1),
    ("layer2.0s 64->128 1x1/2 56", 1, 64, 128, 56, 1, 2, 0),
    ("layer2 128->128 3x3 28", 3, 128, 128, 28, 3, 1, 1),
    ("layer3.0a 128->256 3x3/2 28", 1, 128, 256, 28, 3, 2, 1),
    ("layer3.0s 128->256 1x1/2 28", 1, 128, 256, 28, 1, 2, 0),
    ("layer3 256->256 3x3 14", 3, 256, 256, 14, 3, 1, 1),
    ("layer4.0a 256->512 3x3/2 14", 1, 256, 512, 14, 3, 2, 1),
    ("layer4.0s 256->512 1x1/2 14", 1, 256, 512, 14, 1, 2, 0),
    ("layer4 512->512 3x3 7", 3, 512, 512, 7, 3, 1, 1),
]


def tap_sk_traffic_bytes():
    """HBM bytes per launch of the headline kernel on the CONV workload: measured with hardware counters (FETCH_SIZE and
    WRITE_SIZE runs of `bench.py --traffic-run`, each scaled by what the same counter reads for the plain copy kernel)
    and kept with the measurement, in the line of profiles/conv_pool_hbm_traffic_pmc.md that starts with
    `roofline.traffic`.  None when that file is not there."""
    path = os.path.join(ROOT, "profiles", "conv_pool_hbm_traffic_pmc.md")
    try:
        with open(path) as f:
            for line in f:
                m = re.match(r"\s*`?roofline\.traffic`?\s*[:=]\s*([0-9.]+(?:e[0-9]+)?)\s*bytes", line)
                if m:
                    return float(m.group(1))
    except OSError:
        pass
    return None


def conv_flops(c):
    oh = (c["H"] + 2 * c["pad"] - c["R"]) // c["stride"][0] + 1
    ow = (c["W"] + 2 * c["pad"] - c["S"]) // c["stride"][1] + 1
    return 2.0 * c["N"] * oh * ow * c["K"] * c["C"] * c["R"] * c["S"]


def make_conv_inputs(c):
    x = np.random.default_rng(1).standard_normal((c["N"], c["C"], c["H"], c["W"]), dtype=np.float32)
    fan_in = c["C"] * c["R"] * c["S"]
    w = (np.random.default_rng(2).standard_normal((c["K"], c["C"], c["R"], c["S"])) * np.sqrt(2.0 / fan_in)).astype(np.float32)
    b = np.zeros((c["K"],), dtype=np.float32)
    dy = np.random.default_rng(3).standard_normal((c["N"], c["K"], c["H"], c["W"]), dtype=np.float32)
    return x, w, b, dy


PREHEAT_S = 0.6


def preheat(be, launch, seconds=PREHEAT_S, batch=20):
    """Untimed launches until `seconds` of wall time have passed.  The GPU's shader clock takes tens of
    milliseconds of continuous load to climb from its idle state to its sustained value (measured with the
    kernels' own cycle counters: 1.9 GHz in the first few milliseconds, 2.35 GHz after ~0.1 s), so every timed
    section is preceded by this ramp; it is not part of any reported time."""
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(batch):
            launch()
        be.synchronize()


def batch_ms(be, launch, n):
    """Average duration of n back-to-back launches, from two events on the library's stream."""
    e0, e1 = be.Event(), be.Event()
    be.synchronize()
    e0.record()
    for _ in range(n):
        launch()
    e1.record()
    ms = e0.elapsed_ms(e1)
    be.synchronize()
    return ms / n


def bench_conv(be, steps, warmup):
    K = be.kernels
    c = CONV
    x, w, b, dy = make_conv_inputs(c)
    dx_, dw_, db_, ddy = be.to_device(x), be.to_device(w), be.to_device(b), be.to_device(dy)
    y = be.empty((c["N"], c["K"], c["H"], c["W"]))
    gx = be.empty(x.shape); gw = be.empty(w.shape); gb = be.empty(b.shape)

    def step():
        K.conv2d_fwd(dx_, dw_, db_, c["stride"], c["pad"], out=y)
        K.conv2d_bwd_data(ddy, dw_, x.shape, c["stride"], c["pad"], dx=gx)
        K.conv2d_bwd_weight(ddy, dx_, w.shape, c["stride"], c["pad"], dw=gw, db=gb)

    preheat(be, step)
    for _ in range(warmup):
        step()
    be.synchronize()
    e0, e1 = be.Event(), be.Event()
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        step()
    e1.record()
    ms = e0.elapsed_ms(e1)
    be.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3

    # second pass: each op launched K times back to back between one pair of events on the library's
    # stream, so the average launch duration carries no per-launch event overhead.  "fwd"/"bwd_data"/
    # "bwd_weight" are whole ops (filter layout kernel or split reduction included); "*_kernel" repeat the
    # forward / backward-data launch with XSMI_CONV_WS_PACKED, i.e. the tap-major MFMA kernel alone.
    per = {
        "fwd": batch_ms(be, lambda: K.conv2d_fwd(dx_, dw_, db_, c["stride"], c["pad"], out=y), steps),
        "bwd_data": batch_ms(be, lambda: K.conv2d_bwd_data(ddy, dw_, x.shape, c["stride"], c["pad"], dx=gx), steps),
        "bwd_weight": batch_ms(be, lambda: K.conv2d_bwd_weight(ddy, dx_, w.shape, c["stride"], c["pad"], dw=gw, db=gb), steps),
    }
    K.conv2d_fwd(dx_, dw_, db_, c["stride"], c["pad"], out=y)
    per["fwd_kernel"] = batch_ms(be, lambda: K.conv2d_fwd(dx_, dw_, db_, c["stride"], c["pad"], out=y, packed=True), steps)
    K.conv2d_bwd_data(ddy, dw_, x.shape, c["stride"], c["pad"], dx=gx)
    per["bwd_data_kernel"] = batch_ms(be, lambda: K.conv2d_bwd_data(ddy, dw_, x.shape, c["stride"], c["pad"], dx=gx, packed=True), steps)
    return ms / steps, wall_ms / steps, per


def make_pool_inputs(p):
    rng = np.random.default_rng(4)
    x = rng.standard_normal((p["N"], p["C"], p["H"], p["W"]), dtype=np.float32)
    flat = x.reshape(-1, p["W"])
    pick = rng.choice(flat.size, size=flat.size // 20, replace=False)      # 5 % ties with the right-hand neighbour
    r, col = np.divmod(pick, p["W"])
    flat[r, col] = flat[r, (col + 1) % p["W"]]
    oh = (p["H"] + 2 * p["pad"] - p["k"]) // p["stride"][0] + 1
    ow = (p["W"] + 2 * p["pad"] - p["k"]) // p["stride"][1] + 1
    dy = np.random.default_rng(5).standard_normal((p["N"], p["C"], oh, ow), dtype=np.float32)
    return x, dy


POOL_SETS = 10       # disjoint buffer sets the memory-bound kernels rotate over


def bench_pool(be, steps, warmup):
    """Max-pool forward / backward and the plain copy kernel, HBM-true: consecutive launches work on POOL_SETS
    disjoint buffer sets (10 x 135 MB per direction and kernel; even the 32 MB a backward launch reads come to 320 MB over a round, beyond the 256 MB of last-level cache), so no
    launch finds its operands cached by the previous one.  The "warm" figures repeat one set and are cache-assisted;
    they are reported for comparison only."""
    K = be.kernels
    p = POOL
    x, dy = make_pool_inputs(p)
    sets = []
    for _ in range(POOL_SETS):
        sets.append(dict(x=be.to_device(x), dy=be.to_device(dy), y=be.empty(dy.shape), idx=be.empty(dy.shape, np.uint8),
                         gx=be.empty(x.shape)))
    nel = x.size + dy.size + dy.size // 4
    copies = [(be.empty((nel,)), be.empty((nel,))) for _ in range(POOL_SETS)]
    for c_src, _ in copies:
        c_src.fill_zero()
    state = {"i": 0}

    def nxt():
        state["i"] = (state["i"] + 1) % POOL_SETS
        return state["i"]

    def fwd(b):
        K.maxpool2d_fwd(b["x"], p["k"], p["stride"], p["pad"], out=b["y"], idx=b["idx"])

    def bwd(b):
        K.maxpool2d_bwd(b["dy"], b["idx"], x.shape, p["k"], p["stride"], p["pad"], dx=b["gx"])

    for b in sets:
        fwd(b); bwd(b)
    for c_src, c_dst in copies:                          # every buffer has been written once before anything is timed
        K.copy_kernel(c_dst, c_src)
    preheat(be, lambda: (fwd(sets[nxt()]), bwd(sets[nxt()]), K.copy_kernel(*copies[nxt()][::-1])))
    n = max(steps, 4 * POOL_SETS)
    n -= n % POOL_SETS
    fm = batch_ms(be, lambda: fwd(sets[nxt()]), n)
    bm = batch_ms(be, lambda: bwd(sets[nxt()]), n)
    cm = batch_ms(be, lambda: K.copy_kernel(*copies[nxt()][::-1]), n)
    fm_w = batch_ms(be, lambda: fwd(sets[0]), n)
    bm_w = batch_ms(be, lambda: bwd(sets[0]), n)
    cm_w = batch_ms(be, lambda: K.copy_kernel(copies[0][1], copies[0][0]), n)
    bytes_alg = x.nbytes + dy.nbytes + dy.size          # x + y + 1-byte index  (fwd);  dy + idx + dx  (bwd)
    gbps = lambda ms: bytes_alg / ms / 1e6
    return {
        "maxpool_workload": "N=32 C=64 112x112, 3x3 stride 2 pad 1, fp32, 5%% ties; launches rotate over %d disjoint buffer "
                            "sets (%.0f MB in total per kernel)" % (POOL_SETS, POOL_SETS * bytes_alg / 1e6),
        "maxpool_algorithmic_MB": bytes_alg / 1e6,
        "maxpool_fwd_ms": fm, "maxpool_fwd_GBps": gbps(fm), "maxpool_fwd_frac_hbm": gbps(fm) / HBM_PEAK_GBPS,
        "maxpool_bwd_ms": bm, "maxpool_bwd_GBps": gbps(bm), "maxpool_bwd_frac_hbm": gbps(bm) / HBM_PEAK_GBPS,
        "copy_kernel_GBps": 2 * 4 * nel / cm / 1e6, "copy_kernel_MB_each_way": 4 * nel / 1e6,
        "same_buffers_cache_assisted": {"maxpool_fwd_GBps": gbps(fm_w), "maxpool_bwd_GBps": gbps(bm_w),
                                        "copy_kernel_GBps": 2 * 4 * nel / cm_w / 1e6},
    }


def bench_per_layer(be, reps):
    """Every distinct ResNet-18 convolution at N=32, pass by pass (forward incl. bias, backward-data,
    backward-weight incl. bias gradient): whole ops as the training step issues them (filter layout kernels and split
    reductions included), `reps` launches back to back between two events after a clock ramp.

    Each (layer, pass) is preceded by one fill launch of 1024 * (index + 1) floats, so that a kernel trace of this mode
    can be cut into its rows: that launch shows up as `ew_kernel<FillF>` with a grid of 256 * (index + 1) threads.  The
    second timing of a forward or backward-data row (`ms_layout_ahead`: the filter's layout made ahead of the pass, as
    a training step has it) follows a fill of 1024 * (index + 129) floats."""
    K = be.kernels
    rows = []
    marker = be.empty((1024 * (3 * len(RESNET18_CONVS) + 129),))
    rng = np.random.default_rng(11)
    for name, count, c, k, h, r, st, pad in RESNET18_CONVS:
        oh = (h + 2 * pad - r) // st + 1
        x = be.to_device(rng.standard_normal((32, c, h, h), dtype=np.float32))
        w = be.to_device((rng.standard_normal((k, c, r, r)) * np.sqrt(2.0 / (c * r * r))).astype(np.float32))
        b = be.to_device(np.zeros((k,), np.float32))
        dy = be.to_device(rng.standard_normal((32, k, oh, oh), dtype=np.float32))
        y = be.empty(dy.shape); gx = be.empty(x.shape); gw = be.empty(w.shape); gb = be.empty((k,))
        flops = 2.0 * 32 * oh * oh * k * c * r * r
        passes = {
            "fwd": lambda: K.conv2d_fwd(x, w, b, (st, st), pad, out=y),
            "bwd_data": lambda: K.conv2d_bwd_data(dy, w, x.shape, (st, st), pad, dx=gx),
            "bwd_weight": lambda: K.conv2d_bwd_weight(dy, x, w.shape, (st, st), pad, dw=gw, db=gb),
        }
        # the same passes as a training step runs them: the filter's layout was made ahead (on the second stream,
        # after the optimizer's update), so the pass itself is the convolution kernel alone
        ahead = {
            "fwd": lambda: K.conv2d_fwd(x, w, b, (st, st), pad, out=y, keep_layout=True),
            "bwd_data": lambda: K.conv2d_bwd_data(dy, w, x.shape, (st, st), pad, dx=gx, keep_layout=True),
        }
        for pname, fn in passes.items():
            if pname == "bwd_data" and c == 3:
                continue                                  # the network input needs no gradient
            be.lib.call("xsmi_fill", marker.cptr, 0.0, 1024 * (len(rows) + 1))
            preheat(be, fn, seconds=0.25)
            ms = batch_ms(be, fn, reps)
            tf = flops / (ms * 1e-3) / 1e12
            row = {"layer": name, "count": count, "pass": pname, "ms": ms, "gflop": flops / 1e9, "tflops": tf,
                   "frac_fp32_mfma_peak": tf / FP32_MFMA_PEAK_TFLOPS}
            if pname in ahead:
                be.lib.call("xsmi_fill", marker.cptr, 0.0, 1024 * (len(rows) + 129))
                preheat(be, ahead[pname], seconds=0.1)
                row["ms_layout_ahead"] = batch_ms(be, ahead[pname], reps)
            rows.append(row)
        del x, w, b, dy, y, gx, gw, gb
    total_ms = sum(r_["ms"] * r_["count"] for r_ in rows)
    ahead_ms = sum(r_.get("ms_layout_ahead", r_["ms"]) * r_["count"] for r_ in rows)
    total_gflop = sum(r_["gflop"] * r_["count"] for r_ in rows)
    return {"per_layer": rows, "conv_ms_per_training_step": total_ms, "conv_gflop_per_training_step": total_gflop,
            "conv_tflops_whole_network": total_gflop / total_ms, "reps": reps,
            "conv_ms_per_training_step_layouts_ahead": ahead_ms,
            "frac_fp32_mfma_peak_whole_network": total_gflop / total_ms / FP32_MFMA_PEAK_TFLOPS}


README_N = 256


def make_readme_inputs():
    """README functional net: x 256x1x28x28 ~N(0,1), Conv2D(8, 2x2) He-normal + ReLU, MaxPool 2x2, Dense 1352->10
    ~N(0, 0.1), uniform labels."""
    rng = np.random.default_rng(0)
    x = rng.standard_normal((README_N, 1, 28, 28), dtype=np.float32)
    wc = (rng.standard_normal((8, 1, 2, 2)) * np.sqrt(2.0 / 4)).astype(np.float32)
    wd = (rng.standard_normal((1352, 10)) * 0.1).astype(np.float32)
    labels = rng.integers(0, 10, size=(README_N,))
    return x, wc, wd, labels


def bench_readme_net(be, steps, warmup):
    """README net, one fwd+bwd+SGD step through the layer API on device-resident tensors (launch-bound: 11.9 MFLOP)."""
    import xshinnosuke_amd as xs
    from xshinnosuke_amd.layers import Conv2D, MaxPooling2D, Flatten, Dense
    from xshinnosuke_amd.nn.models import Sequential
    from xshinnosuke_amd.optim import SGD
    x, wc, wd, labels = make_readme_inputs()
    xs.GLOBAL.INPUTS = None
    xs.GLOBAL.USE_CUDA = True
    try:
        net = Sequential(Conv2D(8, 2, activation='relu'), MaxPooling2D(2), Flatten(), Dense(10))
        xt, yt = xs.tensor(x).to('cuda'), xs.tensor(labels).to('cuda')
        with xs.no_grad():
            net(xt)
        xs.GLOBAL.INPUTS = None
        conv, dense = net._graph[0], net._graph[3]
        conv.parameters()[0].eval = be.to_device(wc)
        dense.parameters()[0].eval = be.to_device(wd)
        params = [q for l in (conv, dense) for q in l.parameters() if q is not None]
        opt = SGD(params, lr=0.01)
        crit = xs.nn.CrossEntropyLoss()

        def step():
            opt.zero_grad()
            loss = crit(net(xt), yt)
            loss.backward()
            opt.step()
            return loss

        for _ in range(warmup + 5):
            step()
        be.synchronize()
        e0, e1 = be.Event(), be.Event()
        t0 = time.perf_counter()
        e0.record()
        for _ in range(steps):
            loss = step()
        e1.record()
        ms = e0.elapsed_ms(e1)
        be.synchronize()
        wall = (time.perf_counter() - t0) * 1e3
        out = {"readme_net_ms_per_step": ms / steps, "readme_net_wall_ms_per_step": wall / steps,
               "readme_net_images_per_sec": README_N * steps / (ms * 1e-3), "readme_net_last_loss": loss.item(),
               "readme_net_workload": "N=256x1x28x28, Conv2D(8, 2x2, relu) + MaxPool 2x2 + Flatten + Dense(10), cross-entropy, "
                                      "SGD lr 0.01; fwd+bwd+step through the layer API, device-resident"}
        # this step is bound by the host issuing its launches: recorded once and replayed it is bound by the device
        graph = be.StepGraph()
        with graph.capture():
            loss = step()
        for _ in range(warmup + 5):
            graph.replay()
        be.synchronize()
        e0.record()
        for _ in range(steps):
            graph.replay()
        e1.record()
        ms = e0.elapsed_ms(e1)
        be.synchronize()
        out.update({"readme_net_graph_ms_per_step": ms / steps, "readme_net_graph_images_per_sec": README_N * steps / (ms * 1e-3),
                    "readme_net_graph_last_loss": loss.item()})
        graph.close()
        return out
    finally:
        xs.GLOBAL.USE_CUDA = False
        xs.GLOBAL.INPUTS = None


def bench_resnet18(be, steps, warmup):
    """ResNet-18 (BasicBlock [2,2,2,2], 7x7/2 stem, 3x3/2 max-pool, global avg pool, FC 1000) fwd+bwd+SGD through the
    layer API on device-resident tensors: N=32x3x224x224 fp32, He-normal weights, random labels."""
    import xshinnosuke_amd as xs
    from resnet18 import ResNet18
    from xshinnosuke_amd.optim import SGD
    np.random.seed(6)
    x = xs.tensor(np.random.default_rng(6).standard_normal((32, 3, 224, 224), dtype=np.float32)).to('cuda')
    y = xs.tensor(np.random.default_rng(7).integers(0, 1000, size=(32,))).to('cuda')
    net = ResNet18(classes=1000, pool=7).to('cuda')
    crit = xs.nn.CrossEntropyLoss()
    with xs.no_grad():
        net(x)                               # creates the parameters
    xs.GLOBAL.INPUTS = None
    opt = SGD(net.parameters(), lr=0.01)

    def step():
        opt.zero_grad()
        loss = crit(net(x), y)
        loss.backward()
        opt.step()
        return loss

    preheat(be, step, batch=5)
    for _ in range(warmup):
        step()
    be.synchronize()
    t0 = time.perf_counter()
    e0, e1 = be.Event(), be.Event()
    e0.record()
    for _ in range(steps):
        loss = step()
    enqueue = (time.perf_counter() - t0) * 1e3       # the host has issued every launch; the device is still running
    e1.record()
    ms = e0.elapsed_ms(e1)
    be.synchronize()
    wall = (time.perf_counter() - t0) * 1e3
    out = {"resnet18_train_images_per_sec": 32 * steps / (ms * 1e-3), "resnet18_ms_per_step": ms / steps,
           # device memory beside tensors: shared and per-filter workspaces plus the library's own scratch
           "resnet18_workspace_MB": be.workspace_bytes() / 1e6,
           "resnet18_wall_ms_per_step": wall / steps, "resnet18_host_enqueue_ms_per_step": enqueue / steps,
           "resnet18_last_loss": loss.item(),
           "resnet18_workload": "N=32x3x224x224 fp32, fwd+bwd+SGD, batch-statistics BN, device-resident, layer API"}
    # the same step recorded once as a step graph and replayed: one call per step instead of ~230
    graph = be.StepGraph()
    with graph.capture():
        loss = step()
    for _ in range(warmup):
        graph.replay()
    be.synchronize()
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        graph.replay()
    enqueue = (time.perf_counter() - t0) * 1e3
    e1.record()
    ms = e0.elapsed_ms(e1)
    be.synchronize()
    out.update({"resnet18_graph_images_per_sec": 32 * steps / (ms * 1e-3), "resnet18_graph_ms_per_step": ms / steps,
                "resnet18_graph_host_enqueue_ms_per_step": enqueue / steps, "resnet18_graph_last_loss": loss.item()})
    graph.close()
    xs.GLOBAL.USE_CUDA = False
    return out


def bench_resnet18_infer(be, steps, warmup, with_oracle=True):
    """ResNet-18 N=256 forward only, moving-statistics BN, convolutions allowed to use bf16 MFMA operands; the fp32
    forward of the same weights and input runs beside it.  With `with_oracle` the NumPy/oracle forward of the first
    and the last image (the images of a batch are independent under moving statistics) is timed on the host and
    gives the logits' relative L2 distance for both precisions."""
    import xshinnosuke_amd as xs
    from resnet18 import ResNet18
    xs.GLOBAL.INPUTS = None
    out = {}
    ref = None
    if with_oracle:
        sec, ref, net, X, pick = cpu_resnet18_inference(2)
        out["resnet18_infer_cpu_oracle"] = {"sec_for_images": sec, "images": len(pick), "images_per_sec": len(pick) / sec,
                                            "cores": _blas_threads(), "sample": "oracle forward of images 0 and 255 of the batch"}
    else:
        np.random.seed(7)
        X = np.random.default_rng(7).standard_normal((256, 3, 224, 224), dtype=np.float32)
        net = ResNet18(classes=1000, pool=7).to('cuda')
    x = xs.tensor(X).to('cuda')
    xs.GLOBAL.TRAINING = False
    try:
        with xs.no_grad():
            logits = {}
            for mode in ("fp32", "bf16"):
                with xs.conv_precision(mode):
                    preheat(be, lambda: net(x), batch=2)
                    for _ in range(warmup):
                        y = net(x)
                    be.synchronize()
                    e0, e1 = be.Event(), be.Event()
                    e0.record()
                    for _ in range(steps):
                        y = net(x)
                    e1.record()
                    ms = e0.elapsed_ms(e1)
                    be.synchronize()
                    logits[mode] = y.numpy().astype(np.float64)
                    out["resnet18_infer_%s_images_per_sec" % mode] = 256 * steps / (ms * 1e-3)
                    out["resnet18_infer_%s_ms_per_batch" % mode] = ms / steps
    finally:
        xs.GLOBAL.TRAINING = True
        xs.GLOBAL.USE_CUDA = False
        xs.GLOBAL.INPUTS = None
    d = logits["bf16"] - logits["fp32"]
    out["resnet18_infer_bf16_logits_rel_l2_vs_fp32_kernels"] = float(np.linalg.norm(d) / np.linalg.norm(logits["fp32"]))
    if ref is not None:
        r64 = ref.astype(np.float64)
        for mode in ("fp32", "bf16"):
            out["resnet18_infer_%s_logits_rel_l2_vs_oracle" % mode] = float(
                np.linalg.norm(logits[mode][pick] - r64) / np.linalg.norm(r64))
    out["resnet18_infer_workload"] = ("N=256x3x224x224, forward only, moving-statistics BN (fresh: mean 0, var 1), "
                                      "batch norm folded into the convolutions; fp32 = float32 NCHW tensors and fp32 MFMA; bf16 = "
                                      "bf16 MFMA operands with fp32 accumulation, activations between the stem and the "
                                      "average pool kept as channels-last bf16 tensors (conv, add+ReLU, max-pool read and write "
                                      "them directly)")
    return out


def traffic_run(be, reps=3):
    """A short fixed sequence for hardware-counter runs (one counter set per profiler run): the conv workload's three
    kernels, the max-pool pair, and the plain copy kernel of known size that calibrates the byte counters."""
    K = be.kernels
    c, p = CONV, POOL
    x, w, b, dy = make_conv_inputs(c)
    dx_, dw_, db_, ddy = be.to_device(x), be.to_device(w), be.to_device(b), be.to_device(dy)
    y = be.empty(dy.shape); gx = be.empty(x.shape); gw = be.empty(w.shape); gb = be.empty(b.shape)
    px = be.to_device(np.random.default_rng(4).standard_normal((p["N"], p["C"], p["H"], p["W"]), dtype=np.float32))
    pdy = be.to_device(np.random.default_rng(5).standard_normal((p["N"], p["C"], p["H"] // 2, p["W"] // 2), dtype=np.float32))
    py = be.empty(pdy.shape); pidx = be.empty(pdy.shape, np.uint8); pgx = be.empty(px.shape)
    src = be.empty((px.size + pdy.size + pdy.size // 4,)); dst = be.empty(src.shape)
    def conv_step():
        K.conv2d_fwd(dx_, dw_, db_, c["stride"], c["pad"], out=y)
        K.conv2d_bwd_data(ddy, dw_, x.shape, c["stride"], c["pad"], dx=gx)
        K.conv2d_bwd_weight(ddy, dx_, w.shape, c["stride"], c["pad"], dw=gw, db=gb)
    # the bf16 forward at the inference size of config 5 (N=256, 128->128, 28x28, 3x3): 128 x 128 tiles
    ix = be.to_device(np.random.default_rng(8).standard_normal((256, 128, 28, 28), dtype=np.float32))
    iw = be.to_device(np.random.default_rng(9).standard_normal((128, 128, 3, 3), dtype=np.float32) * np.float32(0.03))
    iy = be.empty((256, 128, 28, 28))
    # the first layer of ResNet-18 at N=32 (3 -> 64, 7x7, stride 2)
    sx = be.to_device(np.random.default_rng(10).standard_normal((32, 3, 224, 224), dtype=np.float32))
    sw = be.to_device(np.random.default_rng(11).standard_normal((64, 3, 7, 7), dtype=np.float32) * np.float32(0.1))
    sy = be.empty((32, 64, 112, 112))
    preheat(be, conv_step, seconds=0.3)          # counters of the last dispatches are read at the sustained clock
    for _ in range(reps):
        K.conv2d_fwd(ix, iw, None, (1, 1), 1, out=iy, bf16=True)
        K.conv2d_fwd(sx, sw, None, (2, 2), 3, out=sy)
        conv_step()
        K.conv2d_fwd(dx_, dw_, db_, c["stride"], c["pad"], out=y, bf16=True)
        K.maxpool2d_fwd(px, p["k"], p["stride"], p["pad"], out=py, idx=pidx)
        K.maxpool2d_bwd(pdy, pidx, px.shape, p["k"], p["stride"], p["pad"], dx=pgx)
        K.copy_kernel(dst, src)
        be.synchronize()
    return {"traffic_run": reps, "copy_kernel_bytes_each_way": src.nbytes}


def _blas_threads():
    try:
        from threadpoolctl import threadpool_info
        return int(max([p.get("num_threads", 1) for p in threadpool_info()] or [1]))
    except Exception:
        return int(os.cpu_count() or 1)


def _median_after_warmup(fn, timed=3):
    times = []
    for _ in range(timed + 1):                 # the first run is the warm-up
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    return statistics.median(times[1:]), times[1:]


def cpu_conv_step(c):
    import oracle
    x, w, b, dy = make_conv_inputs(c)

    def step():
        y, col = oracle.conv2d_fwd(x, w, b.reshape(1, -1), c["stride"], c["pad"])
        oracle.conv2d_bwd(dy, x.shape, w, col, c["stride"], c["pad"],
                          np.zeros_like(x), np.zeros_like(w), np.zeros((1, c["K"]), dtype=np.float32))
    return _median_after_warmup(step)


def cpu_pool_step():
    import oracle
    p = POOL
    x, dy = make_pool_inputs(p)

    def step():
        y, am = oracle.max_pool2d_fwd(x, p["k"], p["stride"], p["pad"])
        oracle.max_pool2d_bwd(dy, am, x.shape, p["k"], p["stride"], p["pad"], np.zeros_like(x))
    return _median_after_warmup(step)


def cpu_readme_step():
    """README net fwd+bwd+SGD: conv / ReLU / max-pool through the oracle, dense + cross-entropy in NumPy float64."""
    import oracle
    x, wc, wd, labels = make_readme_inputs()
    bc = np.zeros((8,), np.float32); bd = np.zeros((1, 10))
    wd64 = wd.astype(np.float64)
    rows = np.arange(len(labels))

    def step():
        y1, col = oracle.conv2d_fwd(x, wc, bc, (1, 1), 0)
        a1 = oracle.relu_fwd(y1)
        p1, am = oracle.max_pool2d_fwd(a1, 2, None, 0)
        flat = p1.reshape(p1.shape[0], -1).astype(np.float64)
        z = flat @ wd64 + bd
        z -= z.max(axis=1, keepdims=True)
        sm = np.exp(z); sm /= sm.sum(axis=1, keepdims=True)
        g = sm; g[rows, labels] -= 1; g /= len(labels)
        dwd = flat.T @ g; dbd = g.sum(axis=0, keepdims=True)
        dflat = (g @ wd64.T).astype(np.float32)
        da1 = oracle.max_pool2d_bwd(dflat.reshape(p1.shape), am, a1.shape, 2, (2, 2), 0, np.zeros_like(a1))
        dy1 = oracle.relu_bwd(da1, y1)
        _, dwc, dbc = oracle.conv2d_bwd(dy1, x.shape, wc, col, (1, 1), 0, None, np.zeros_like(wc), np.zeros_like(bc))
        return wc - 0.01 * dwc, bc - 0.01 * dbc, wd64 - 0.01 * dwd, bd - 0.01 * dbd
    return _median_after_warmup(step)


def cpu_resnet18_hot_path():
    """The conv / max-pool share of one ResNet-18 N=32 training step on the CPU path: forward + backward of each of the
    11 distinct convolutions (oracle, float64 im2col + GEMM + col2im) timed once after a warm-up on the first one and
    weighted by how often the layer occurs, plus the 3x3/2 max-pool forward + backward.  Batch norm, ReLU, residual
    adds, the dense tail and the optimizer are not in this sample."""
    import oracle
    rng = np.random.default_rng(12)
    total, per = 0.0, {}
    first = True
    for name, count, c, k, h, r, st, pad in RESNET18_CONVS:
        oh = (h + 2 * pad - r) // st + 1
        x = rng.standard_normal((32, c, h, h), dtype=np.float32)
        w = (rng.standard_normal((k, c, r, r)) * np.sqrt(2.0 / (c * r * r))).astype(np.float32)
        b = np.zeros((1, k), np.float32)
        dy = rng.standard_normal((32, k, oh, oh), dtype=np.float32)

        def step():
            y, col = oracle.conv2d_fwd(x, w, b, (st, st), pad)
            oracle.conv2d_bwd(dy, x.shape, w, col, (st, st), pad, None if c == 3 else np.zeros_like(x),
                              np.zeros_like(w), np.zeros((1, k), np.float32))
        if first:
            step()
            first = False
        t0 = time.perf_counter()
        step()
        per[name] = time.perf_counter() - t0
        total += count * per[name]
        del x, w, dy
    px, pdy = make_pool_inputs(POOL)
    t0 = time.perf_counter()
    y, am = oracle.max_pool2d_fwd(px, 3, (2, 2), 1)
    oracle.max_pool2d_bwd(pdy, am, px.shape, 3, (2, 2), 1, np.zeros_like(px))
    per["max-pool 3x3/2 112"] = time.perf_counter() - t0
    total += per["max-pool 3x3/2 112"]
    return total, per


def cpu_resnet18_inference(images=2):
    """Oracle forward of ResNet-18 (moving-statistics batch norm) on `images` images of the N=256 inference input;
    returns (seconds, logits, the network) so that the GPU logits of the same images can be compared."""
    import xshinnosuke_amd as xs
    from resnet18 import ResNet18, oracle_forward
    np.random.seed(7)
    X = np.random.default_rng(7).standard_normal((256, 3, 224, 224), dtype=np.float32)
    pick = [0, 255][:images]
    xs.GLOBAL.INPUTS = None
    net = ResNet18(classes=1000, pool=7).to('cuda')
    with xs.no_grad():
        net(xs.tensor(X[:1]).to('cuda'))
    xs.GLOBAL.INPUTS = None
    t0 = time.perf_counter()
    ref = oracle_forward(net, X[pick])
    sec = time.perf_counter() - t0
    return sec, ref, net, X, pick


def cpu_baseline(extra):
    """Oracle (NumPy restatement of the reference algorithm) on the host cores.  The headline entry is the conv
    workload (median of 3 steps after a warm-up); `other_workloads` hold the other configurations, each with the GPU
    figure measured earlier in this run beside it."""
    threads = _blas_threads()
    c = CONV
    sec, all_sec = cpu_conv_step(c)
    out = {
        "value": 3 * conv_flops(c) / sec / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
        "sample": "full workload (N=32 conv fwd+bwd), 1 warm-up + 3 timed steps (median), NumPy %s float64 "
                  "im2col+GEMM+col2im; os.cpu_count=%s" % (np.__version__, os.cpu_count()),
        "sec_per_step": sec, "sec_all": all_sec,
    }
    others = {}
    psec, _ = cpu_pool_step()
    bytes_alg = 2 * (POOL["N"] * POOL["C"] * (POOL["H"] * POOL["W"] + (POOL["H"] // 2) * (POOL["W"] // 2) * 1.25) * 4)
    others["maxpool_fwd_bwd"] = {"sec_per_step": psec, "GBps_algorithmic": bytes_alg / psec / 1e9, "cores": threads,
                                 "sample": "full workload (fwd + bwd), 1 warm-up + 3 timed (median)",
                                 "gpu_ms_fwd_plus_bwd": (extra or {}).get("maxpool_fwd_ms", float("nan")) +
                                                        (extra or {}).get("maxpool_bwd_ms", float("nan"))}
    rsec, _ = cpu_readme_step()
    others["readme_net_step"] = {"sec_per_step": rsec, "images_per_sec": README_N / rsec, "cores": threads,
                                 "sample": "full workload (N=256 fwd+bwd+SGD), 1 warm-up + 3 timed (median)",
                                 "gpu_ms_per_step": (extra or {}).get("readme_net_ms_per_step")}
    hsec, per = cpu_resnet18_hot_path()
    others["resnet18_train_hot_path"] = {
        "sec_per_step": hsec, "images_per_sec": 32 / hsec, "cores": threads, "per_layer_sec": per,
        "sample": "conv + max-pool fwd+bwd of one N=32 step: each distinct conv geometry timed once (after one warm-up), "
                  "weighted by its count; batch norm / ReLU / add / dense / optimizer not included",
        "gpu_ms_per_whole_step": (extra or {}).get("resnet18_ms_per_step")}
    out["other_workloads"] = others
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the host-side NumPy baseline")
    ap.add_argument("--traffic-run", action="store_true",
                    help="run a short fixed kernel sequence (conv, max-pool, calibration copy) for counter collection and exit")
    ap.add_argument("--no-extra", action="store_true", help="skip the max-pool / copy / README-net / ResNet-18 measurements")
    ap.add_argument("--per-layer", action="store_true",
                    help="time every distinct ResNet-18 convolution (N=32) pass by pass, print one JSON line and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (got --gpus %d); the conv/pool path is data-parallel "
                 "over the batch and no multi-GPU figure is produced" % args.gpus)

    from xshinnosuke_amd import backend as be
    be.init(0)
    info = be.device_info()
    if args.traffic_run:
        print(json.dumps(traffic_run(be)))
        return
    if args.per_layer:
        print(json.dumps(bench_per_layer(be, max(10, args.steps // 10))))
        return

    ms_step, wall_ms_step, per = bench_conv(be, args.steps, args.warmup)
    flops_pass = conv_flops(CONV)
    value = 3 * flops_pass / (ms_step * 1e-3) / 1e12
    igemm_ms = 0.5 * (per["fwd_kernel"] + per["bwd_data_kernel"])      # the same kernel, one launch each per step
    achieved = flops_pass / (igemm_ms * 1e-3) / 1e12
    out = {
        "metric": "conv fwd+bwd TFLOP/s", "value": value, "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "single conv layer fwd+bwd (dX, dW, db): N=32, Cin=Cout=64, 56x56, 3x3, stride 1, pad 1, "
                               "fp32 NCHW, x~N(0,1), He-normal weights, dY~N(0,1); inputs resident in HBM",
                   "gflop_per_step": 3 * flops_pass / 1e9},
        "frac_fp32_mfma_peak": value / FP32_MFMA_PEAK_TFLOPS,
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": FP32_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": achieved / FP32_MFMA_PEAK_TFLOPS, "traffic": tap_sk_traffic_bytes(),
                     "kernel": "tap_sk_f32_kernel<3>", "flop_per_launch": flops_pass, "avg_launch_ms": igemm_ms},
        "ops_ms": {"conv_fwd": per["fwd"], "conv_bwd_data": per["bwd_data"], "conv_bwd_weight": per["bwd_weight"]},
        "kernels_ms": {"tap_sk_fwd": per["fwd_kernel"], "tap_sk_bwd_data": per["bwd_data_kernel"]},
        "ops_tflops": {k: flops_pass / (per[k] * 1e-3) / 1e12 for k in ("fwd", "bwd_data", "bwd_weight")},
        "wall_ms_per_step": wall_ms_step,
        "preheat_s": PREHEAT_S,
        "device": {"name": info["name"], "arch": info["arch"], "cus": info["cu_count"], "clock_mhz": info["clock_khz"] / 1000.0},
    }
    if not args.no_extra:
        out["extra"] = bench_pool(be, max(args.steps, 20), args.warmup)
        be.release_cached_memory()
        out["extra"].update(bench_readme_net(be, max(20, args.steps), args.warmup))
        out["extra"].update(bench_resnet18(be, max(5, args.steps // 5), 3))
        be.release_cached_memory()
        out["extra"].update(bench_resnet18_infer(be, 3, 1, with_oracle=not args.no_cpu))
        be.release_cached_memory()
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(out.get("extra"))
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))


if __name__ == "__main__":
    main()
