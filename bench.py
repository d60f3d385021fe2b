#!/usr/bin/env python3
"""Benchmark of the conv / max-pool hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-extra]

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
parity oracle) on the host cores of this machine, on the same workload.

Everything goes through libxsmi355.so; there is no fallback path.
"""
import argparse
import json
import os
import statistics
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(1, os.path.join(ROOT, "tests"))      # the ResNet-18 workload (tests/resnet18.py) is a caller of the package

FP32_MFMA_PEAK_TFLOPS = 157.3
HBM_PEAK_GBPS = 8000.0

# BASELINE conv config: N, C, H, W, K, R, S, stride, pad
CONV = dict(N=32, C=64, H=56, W=56, K=64, R=3, S=3, stride=(1, 1), pad=1)
# BASELINE max-pool config
POOL = dict(N=32, C=64, H=112, W=112, k=3, stride=(2, 2), pad=1)


# HBM bytes per launch of tap_igemm_f32_kernel on the CONV workload, from two hardware-counter runs
# (FETCH_SIZE 13 480.7 KiB scaled by 1.9996, the factor that makes the plain copy kernel's known read size come
# out right, plus WRITE_SIZE 25 088.0 KiB at factor 1.0): 27.60 MB read + 25.69 MB written.
TAP_IGEMM_TRAFFIC_BYTES = 53.46e6


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


def bench_pool(be, steps, warmup):
    K = be.kernels
    p = POOL
    rng = np.random.default_rng(4)
    x = rng.standard_normal((p["N"], p["C"], p["H"], p["W"]), dtype=np.float32)
    flat = x.reshape(-1, p["W"])
    pick = rng.choice(flat.size, size=flat.size // 20, replace=False)
    r, col = np.divmod(pick, p["W"])
    flat[r, col] = flat[r, (col + 1) % p["W"]]
    oh = (p["H"] + 2 * p["pad"] - p["k"]) // p["stride"][0] + 1
    ow = (p["W"] + 2 * p["pad"] - p["k"]) // p["stride"][1] + 1
    dy = np.random.default_rng(5).standard_normal((p["N"], p["C"], oh, ow), dtype=np.float32)
    dx_, ddy = be.to_device(x), be.to_device(dy)
    y = be.empty(dy.shape); idx = be.empty(dy.shape, np.uint8); gx = be.empty(x.shape)
    def pair():
        K.maxpool2d_fwd(dx_, p["k"], p["stride"], p["pad"], out=y, idx=idx)
        K.maxpool2d_bwd(ddy, idx, x.shape, p["k"], p["stride"], p["pad"], dx=gx)
    preheat(be, pair)
    for _ in range(warmup):
        pair()
    be.synchronize()
    fm = batch_ms(be, lambda: K.maxpool2d_fwd(dx_, p["k"], p["stride"], p["pad"], out=y, idx=idx), steps)
    bm = batch_ms(be, lambda: K.maxpool2d_bwd(ddy, idx, x.shape, p["k"], p["stride"], p["pad"], dx=gx), steps)
    # plain copy of the same number of bytes, for the achievable-bandwidth reference
    src = be.empty((x.size + dy.size + dy.size // 4,)); dst = be.empty(src.shape)
    for _ in range(warmup):
        K.copy_kernel(dst, src)
    cm = batch_ms(be, lambda: K.copy_kernel(dst, src), steps)
    bytes_alg = x.nbytes + dy.nbytes + dy.size          # x + y + 1-byte index  (fwd);  dy + idx + dx  (bwd)
    return {
        "maxpool_workload": "N=32 C=64 112x112, 3x3 stride 2 pad 1, fp32, 5% ties",
        "maxpool_algorithmic_MB": bytes_alg / 1e6,
        "maxpool_fwd_ms": fm, "maxpool_fwd_GBps": bytes_alg / fm / 1e6, "maxpool_fwd_frac_hbm": bytes_alg / fm / 1e6 / HBM_PEAK_GBPS,
        "maxpool_bwd_ms": bm, "maxpool_bwd_GBps": bytes_alg / bm / 1e6, "maxpool_bwd_frac_hbm": bytes_alg / bm / 1e6 / HBM_PEAK_GBPS,
        "copy_kernel_GBps": 2 * src.nbytes / cm / 1e6, "copy_kernel_MB_each_way": src.nbytes / 1e6,
    }


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
    e1.record()
    ms = e0.elapsed_ms(e1)
    be.synchronize()
    wall = (time.perf_counter() - t0) * 1e3
    xs.GLOBAL.USE_CUDA = False
    return {"resnet18_train_images_per_sec": 32 * steps / (ms * 1e-3), "resnet18_ms_per_step": ms / steps,
            "resnet18_wall_ms_per_step": wall / steps, "resnet18_last_loss": loss.item(),
            "resnet18_workload": "N=32x3x224x224 fp32, fwd+bwd+SGD, batch-statistics BN, device-resident, layer API"}


def bench_resnet18_infer(be, steps, warmup):
    """ResNet-18 N=256 forward only, moving-statistics BN, convolutions allowed to use bf16 MFMA operands; the fp32
    forward of the same weights and input runs beside it and gives the logits' relative L2 distance."""
    import xshinnosuke_amd as xs
    from resnet18 import ResNet18
    xs.GLOBAL.INPUTS = None
    X = np.random.default_rng(7).standard_normal((256, 3, 224, 224), dtype=np.float32)
    x = xs.tensor(X).to('cuda')
    net = ResNet18(classes=1000, pool=7).to('cuda')
    out = {}
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
    out["resnet18_infer_bf16_logits_rel_l2_vs_fp32"] = float(np.linalg.norm(d) / np.linalg.norm(logits["fp32"]))
    out["resnet18_infer_workload"] = ("N=256x3x224x224, forward only, moving-statistics BN (fresh: mean 0, var 1), "
                                      "fp32 tensors in HBM, batch norm folded into the convolutions; bf16 = each conv rewrites "
                                      "its input as a channels-last bf16 copy and multiplies bf16 operands with fp32 accumulation")
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
    preheat(be, conv_step, seconds=0.3)          # counters of the last dispatches are read at the sustained clock
    for _ in range(reps):
        K.conv2d_fwd(ix, iw, None, (1, 1), 1, out=iy, bf16=True)
        conv_step()
        K.conv2d_fwd(dx_, dw_, db_, c["stride"], c["pad"], out=y, bf16=True)
        K.maxpool2d_fwd(px, p["k"], p["stride"], p["pad"], out=py, idx=pidx)
        K.maxpool2d_bwd(pdy, pidx, px.shape, p["k"], p["stride"], p["pad"], dx=pgx)
        K.copy_kernel(dst, src)
        be.synchronize()
    return {"traffic_run": reps, "copy_kernel_bytes_each_way": src.nbytes}


def cpu_baseline():
    """Oracle (NumPy restatement of the reference algorithm) on the host cores, same workload."""
    import oracle
    try:
        from threadpoolctl import threadpool_info
        threads = max([p.get("num_threads", 1) for p in threadpool_info()] or [1])
    except Exception:
        threads = os.cpu_count() or 1
    c = CONV
    x, w, b, dy = make_conv_inputs(c)
    times = []
    for i in range(3):                       # 1 warm-up + 2 timed
        t0 = time.perf_counter()
        y, col = oracle.conv2d_fwd(x, w, b.reshape(1, -1), c["stride"], c["pad"])
        oracle.conv2d_bwd(dy, x.shape, w, col, c["stride"], c["pad"],
                          np.zeros_like(x), np.zeros_like(w), np.zeros((1, c["K"]), dtype=np.float32))
        times.append(time.perf_counter() - t0)
        del y, col
    sec = statistics.mean(times[1:])
    return {
        "value": 3 * conv_flops(c) / sec / 1e12, "unit": "TFLOP/s", "cores": int(threads), "kind": "port",
        "sample": "full workload (N=32 conv fwd+bwd), 1 warm-up + 2 timed steps, NumPy %s float64 im2col+GEMM+col2im; "
                  "os.cpu_count=%s" % (np.__version__, os.cpu_count()),
        "sec_per_step": sec,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the host-side NumPy baseline")
    ap.add_argument("--traffic-run", action="store_true",
                    help="run a short fixed kernel sequence (conv, max-pool, calibration copy) for counter collection and exit")
    ap.add_argument("--no-extra", action="store_true", help="skip the max-pool / copy measurements")
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
                     "frac": achieved / FP32_MFMA_PEAK_TFLOPS, "traffic": TAP_IGEMM_TRAFFIC_BYTES,
                     "kernel": "tap_igemm_f32_kernel", "flop_per_launch": flops_pass, "avg_launch_ms": igemm_ms},
        "ops_ms": {"conv_fwd": per["fwd"], "conv_bwd_data": per["bwd_data"], "conv_bwd_weight": per["bwd_weight"]},
        "kernels_ms": {"tap_igemm_fwd": per["fwd_kernel"], "tap_igemm_bwd_data": per["bwd_data_kernel"]},
        "ops_tflops": {k: flops_pass / (per[k] * 1e-3) / 1e12 for k in ("fwd", "bwd_data", "bwd_weight")},
        "wall_ms_per_step": wall_ms_step,
        "preheat_s": PREHEAT_S,
        "device": {"name": info["name"], "arch": info["arch"], "cus": info["cu_count"], "clock_mhz": info["clock_khz"] / 1000.0},
    }
    if not args.no_extra:
        out["extra"] = bench_pool(be, max(args.steps, 20), args.warmup)
        out["extra"].update(bench_resnet18(be, max(5, args.steps // 5), 3))
        be.release_cached_memory()
        out["extra"].update(bench_resnet18_infer(be, 3, 1))
        be.release_cached_memory()
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline()
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))


if __name__ == "__main__":
    main()
