#!/usr/bin/env python3
"""Forward-path benchmark.  One step = one forward pass of the workload over one synthetic batch that is
already resident in HBM.  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload all|resnet50|alexnet|vgg16|lstm|conv1|...]

Default (`all`): the headline -- ResNet-50 (the reference's own topology), fp32, batch 64, the configuration the
metric is quoted on -- timed over K steps, and in the same line, under "configs", the other four benchmarked
configurations (AlexNet conv1 + pool b32, AlexNet b128, VGG-16 b32, 2-layer LSTM T64 b64) and, under "memops", the
memory-bound kernels one by one.  Besides the throughput a network's record carries
  roofline:     the convolution layers' algorithmic FLOP / their HIP-event time, against the fp32 MFMA peak
  cpu_baseline: the reference's CPU algorithm (oracle port, OpenBLAS, all host cores) on a bounded sample.
`--workload NAME` runs that one workload alone (what the profiles under profiles/ are taken with).
"""
import argparse
import json
import os
import re
import sys
import tempfile
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from nebula_amd.zoo import synthetic_weights as make_weights      # noqa: E402

PEAK_FP32_MFMA_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0

# HBM traffic of the convolution layers is a counter measurement (rocprofv3 --pmc FETCH_SIZE, then WRITE_SIZE, over
# `bench.py --workload NAME`, each scaled by what the same counter reads for `--workload copy`), kept with the
# profile summary it comes from.  The summary names the launches it was taken with; the figure is reported only
# when this run's launches are the same.
TRAFFIC_PROFILES = {("resnet50", 64): os.path.join(ROOT, "profiles", "conv_igemm_resnet50_b64.md")}


def measured_traffic(workload_name, batch, conv_tiles):
    """(bytes per convolution layer, note) from the profile summary of this workload, or (None, why not)."""
    path = TRAFFIC_PROFILES.get((workload_name, batch))
    if not path or not os.path.exists(path):
        return None, "no counter profile of this workload"
    text = open(path).read()
    tiles = re.search(r"^conv_tiles: (.*)$", text, re.M)
    traffic = re.search(r"^traffic_bytes_per_layer: ([0-9.eE+]+)$", text, re.M)
    if not tiles or not traffic:
        return None, "the profile summary holds no traffic figure"
    if tiles.group(1).strip() != conv_tiles.strip():
        return None, "the counter profile was taken with other launches than this run's"
    return float(traffic.group(1)), "FETCH_SIZE + WRITE_SIZE of " + os.path.relpath(path, ROOT)


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def workload(name, batch):
    from nebula_amd import zoo
    table = {
        "resnet50": (lambda b: zoo.resnet50_cfg(b, fuse_shortcut=True, in_place=True), 64, "normal", "he",
                     "ResNet-50 (Nebula topology) fp32 forward, batch %d, 3x224x224 N(0,1)"),
        "alexnet": (zoo.alexnet_cfg, 128, "uniform", "he", "AlexNet fp32 forward, batch %d, 3x227x227 U[0,1)"),
        "vgg16": (zoo.vgg16_cfg, 32, "normal", "he", "VGG-16 fp32 forward, batch %d, 3x224x224 N(0,1)"),
        "conv1": (zoo.conv1_pool_cfg, 32, "uniform", "he", "AlexNet conv1+ReLU+maxpool fp32, batch %d"),
        "lstm": (lambda b: zoo.lstm_cfg(b, last_step_only=True), 64, "normal", "lstm",
                 "2-layer LSTM 1024/1024 T=64 + 10000-way projection and softmax on the last step, batch %d"),
        "rnn": (zoo.rnn_cfg, 32, "normal", "he",
                "rnn_large: 5 normalised RNN layers of 1024, T=40, 8713-way projection and softmax on every step, batch %d"),
        "dbn": (zoo.dbn_cfg, 32, "uniform", "he", "dbn_large: 4 RBM layers + 62-way classifier on 3x128x128 U[0,1), batch %d"),
        "mlp": (zoo.mlp_cfg, 32, "uniform", "he", "mlp_large: 5 relu layers + 62-way classifier on 3x128x128 U[0,1), batch %d"),
    }
    fn, default_batch, xdist, wdist, text = table[name]
    b = batch or default_batch
    return fn(b), b, xdist, wdist, text % b


def cpu_baseline(cfg_fn, specs_weights, xdist, sample_batch, is_lstm, rng):
    """The reference's CPU algorithm (per-image im2col + sgemm, separate bias/BN/activation passes) through
    the oracle port with OpenBLAS on all host cores, on a bounded sample of the same workload."""
    from oracle import binding as ob
    cores = int(os.environ.get("OMP_NUM_THREADS", "0")) or os.cpu_count() or 1
    cores = min(cores, len(os.sched_getaffinity(0)))
    blas = ob.use_openblas(threads=cores)
    if not blas:
        ob.use_custom_gemm()
        ob.set_threads(cores)
    net = ob.OracleNet(cfg_fn(sample_batch))
    net.load_weights(specs_weights)
    if is_lstm:
        T = net.net["time_steps"]
        x = rng.standard_normal((T, sample_batch, net.net["input_size"])).astype(np.float32)
    else:
        shape = (sample_batch, net.net["channels"], net.net["height"], net.net["width"])
        x = (rng.random(shape) if xdist == "uniform" else rng.standard_normal(shape)).astype(np.float32)
    # Feed-forward networks: one untimed forward (workspace first touch, BLAS threads start), then the mean of
    # three.  Recurrent networks keep their state between calls as the reference does, so they are timed on the
    # one forward pass of a fresh object.
    timed = 1 if is_lstm else 3
    if not is_lstm:
        net.forward(x)
    t0 = time.perf_counter()
    for _ in range(timed):
        outs = net.forward(x)
    dt = (time.perf_counter() - t0) / timed
    ob.use_custom_gemm()
    ob.set_threads(1)
    return sample_batch / dt, cores, dt, timed, ("OpenBLAS (scipy bundle)" if blas else "reference-style threaded GEMM"), x, outs


def copy_calibration(args):
    """K launches of the library's copy kernel over 256 MiB: reads 256 MiB and writes 256 MiB per launch."""
    from nebula_amd import hip
    ctx = hip.Ctx(0)
    n = 64 << 20
    src, dst = ctx.array(np.ones(n, np.float32)), ctx.empty((n,))
    for _ in range(args.warmup):
        ctx.copy(dst, src)
    ctx.sync()
    ctx.timer_start()
    for _ in range(args.steps):
        ctx.copy(dst, src)
    ms = ctx.timer_stop() / args.steps
    print(json.dumps({"metric": "copy kernel GB/s (read+write)", "value": round(2 * 4 * n / ms / 1e6, 1), "unit": "GB/s",
                      "bytes_read_per_launch": 4 * n, "bytes_written_per_launch": 4 * n, "steps": args.steps,
                      "ms_per_launch": round(ms, 4)}), flush=True)
    ctx.close()


def single_conv(args):
    """One convolution layer (bias + ReLU epilogue) at batch --batch (default 64) through nbl_conv2d_fwd."""
    from nebula_amd import hip
    C_, H, W, F, k, st, pad = (int(v) for v in args.conv_shape.split(","))
    B = args.batch or 64
    ctx = hip.Ctx(0)
    rng = np.random.default_rng(0)
    w = (rng.standard_normal((F, C_, k, k)) * np.sqrt(2.0 / (C_ * k * k))).astype(np.float32)
    plan = ctx.conv_pack(w, np.zeros(F, np.float32), None, H=H, W=W, stride=st, pad=pad, act="relu")
    plan.set_variant(args.conv_variant)
    plan.set_split(args.conv_split)
    x = ctx.array(rng.standard_normal((B, C_, H, W)).astype(np.float32))
    y = ctx.empty((B, F, plan.OH, plan.OW))
    if args.conv_residual:              # the layer as ResNet runs it: the following shortcut fused into the epilogue
        conn = ctx.array(rng.standard_normal((B, F, plan.OH, plan.OW)).astype(np.float32))
        run = lambda: plan.with_shortcut(x, conn, "relu", out=y)
    else:
        run = lambda: plan(x, out=y)
    for _ in range(args.warmup):
        run()
    ctx.sync()
    ctx.timer_start()
    for _ in range(args.steps):
        run()
    ms = ctx.timer_stop() / args.steps
    variant, parts = plan.last_launch()
    flop = plan.flop_per_image * B
    print(json.dumps({"metric": "conv layer TFLOP/s", "value": round(flop / ms / 1e9, 2), "unit": "TFLOP/s", "shape": args.conv_shape,
                      "batch": B, "gemm": {"M": F, "N": B * plan.OH * plan.OW, "K": C_ * k * k}, "tile_variant": variant,
                      "k_slices": parts, "ms_per_launch": round(ms, 4), "steps": args.steps}), flush=True)
    ctx.close()


def conv_work_grid(args):
    """The 64x64 tile of conv_igemm_kernel against how a launch is cut: output tiles per resident-block slot (6 slots per
    CU) and k-tiles per tile.  256 filters on 16x16 maps (16 tiles per image, so the batch sets the tile count); a 3x3 layer
    (tap-major gather) and a 1x1 layer (vector gather) at three depths each; tile shape pinned, no k-split."""
    from nebula_amd import hip
    ctx = hip.Ctx(0)
    rng = np.random.default_rng(0)
    F, HW, slots = 256, 16, 6 * 256
    batches = [48, 96, 98, 192, 196, 384, 768]
    rows = []
    for k, pad, chans in ((3, 1, (16, 64, 128)), (1, 0, (128, 256, 512))):
        for C_ in chans:
            w = (rng.standard_normal((F, C_, k, k)) * np.sqrt(2.0 / (C_ * k * k))).astype(np.float32)
            plan = ctx.conv_pack(w, np.zeros(F, np.float32), None, H=HW, W=HW, stride=1, pad=pad, act="relu")
            plan.set_variant(4)
            plan.set_split(0)
            rec = {"layer": "%dx%d, %d channels" % (k, k, C_), "k_tiles_per_tile": C_ * k * k // 16, "tflops": {}}
            for B in batches:
                x = ctx.array(np.tile(rng.standard_normal((8, C_, HW, HW)).astype(np.float32), (B // 8 + 1, 1, 1, 1))[:B])
                y = ctx.empty((B, F, HW, HW))
                # the device takes some 50 ms of work to reach its sustained clock after an idle moment (the upload above)
                ctx.timer_start()
                for _ in range(3):
                    plan(x, out=y)
                est = max(ctx.timer_stop() / 3, 1e-3)
                for _ in range(int(60.0 / est) + 1):
                    plan(x, out=y)
                ctx.sync()
                reps = int(40.0 / est) + 1
                ctx.timer_start()
                for _ in range(reps):
                    plan(x, out=y)
                ms = ctx.timer_stop() / reps
                assert plan.last_launch() == (4, 1)
                rec["tflops"]["%.2f" % (16.0 * B / slots)] = round(plan.flop_per_image * B / ms / 1e9, 1)
                x.free(); y.free()
            log(rec)
            rows.append(rec)
    ctx.close()
    print(json.dumps({"metric": "conv_igemm_kernel 64x64 tile, TFLOP/s by tiles per resident-block slot and k-tiles per tile",
                      "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s", "tiles_per_slot": ["%.2f" % (16.0 * B / slots) for B in batches],
                      "rows": rows}), flush=True)


def image_input(args):
    """Device-side image preprocessing (nbl_image_to_input): 64 byte images of 375x500x3 -> 3x224x224 float planes."""
    from nebula_amd import hip
    ctx = hip.Ctx(0)
    B = args.batch or 64
    rng = np.random.default_rng(1)
    imgs = ctx.array(rng.integers(0, 256, (B, 375, 500, 3), dtype=np.uint8), dtype=np.uint8)
    for _ in range(args.warmup):
        out = ctx.image_to_input(imgs, 224, 224)
        out.free()
    out = ctx.empty((B, 3, 224, 224))
    ctx.sync()
    ctx.timer_start()
    for _ in range(args.steps):
        ctx.check(hip.lib().nbl_image_to_input(ctx.h, imgs.ptr, B, 375, 500, 3, out.ptr, 224, 224))
    ms = ctx.timer_stop() / args.steps
    # every output pixel reads 4 source pixels of 3 bytes and writes 3 floats; compulsory traffic is the two tensors
    print(json.dumps({"metric": "image preprocessing images/s", "value": round(B / ms * 1e3, 1), "unit": "images/s",
                      "ms_per_launch": round(ms, 4), "bytes_in": int(imgs.nbytes), "bytes_out": int(out.nbytes),
                      "GBps": round((imgs.nbytes + out.nbytes) / ms / 1e6, 1), "steps": args.steps}), flush=True)
    ctx.close()


def memory_bound_kernels(args, emit=True):
    """The bandwidth-bound kernels at the sizes the benchmarked networks (AlexNet, VGG-16, ResNet-50, the LSTM) give them, each timed on its own through the C ABI
    (HIP events on the library's stream, back-to-back launches).  For every kernel: algorithmic bytes per launch (the
    tensors it must read and write once), microseconds per launch and the fraction of the 8 TB/s HBM peak.  The copy
    kernel is the yardstick: what a plain read-once / write-once stream reaches on this machine."""
    from nebula_amd import hip
    ctx = hip.Ctx(0)
    l = hip.lib()
    rng = np.random.default_rng(3)
    out = []

    def timed(name, nbytes, launch, note=""):
        if args.only and args.only not in name:
            return
        for _ in range(args.warmup):
            launch()
        ctx.sync()
        t_ramp = time.perf_counter()         # sustained clock: keep the device busy for 20 ms before timing
        while (time.perf_counter() - t_ramp) * 1e3 < min(args.ramp_ms, 20.0):
            for _ in range(20):
                launch()
            ctx.sync()
        ctx.timer_start()
        for _ in range(args.steps):
            launch()
        us = ctx.timer_stop() * 1e3 / args.steps
        gbs = nbytes / us / 1e3
        rec = {"kernel": name, "bytes": int(nbytes), "us": round(us, 2), "GBps": round(gbs, 1), "frac_of_8TBps": round(gbs / PEAK_HBM_GBS, 3)}
        if note:
            rec["note"] = note
        out.append(rec)
        log(rec)

    def rand(shape):
        # device-resident random data without a 200 MB host array per tensor: one 16 MB block repeated
        n = int(np.prod(shape))
        block = rng.standard_normal(min(n, 1 << 22)).astype(np.float32)
        a = ctx.empty(shape)
        reps = -(-n // block.size)
        host = np.tile(block, reps)[:n]
        a.upload(host)
        return a

    # yardstick
    n = 64 << 20
    src, dst = rand((n,)), ctx.empty((n,))
    timed("copy (nbl_copy_d2d) 256 MiB", 2 * 4 * n, lambda: ctx.copy(dst, src))
    src.free(); dst.free()

    # max-pool 3x3 / 2 on ResNet-50's stem output at batch 64, as inference runs it (no argmax table) and as the
    # reference's forward does (table written)
    B, C_, H = 64, 64, 112
    x = rand((B, C_, H, H)); y = ctx.empty((B, C_, 56, 56)); idx = ctx.empty((B, C_, 56, 56), dtype=np.uint32)
    io = 4 * (x.size + y.size)
    timed("maxpool 3x3/2 64x64x112x112 (no argmax table)", io,
          lambda: ctx.check(l.nbl_pool_fwd(ctx.h, x.ptr, y.ptr, None, B, C_, H, H, 3, 2, 0, hip.POOL_MAX)))
    timed("maxpool 3x3/2 64x64x112x112 (+ argmax table)", io + 4 * y.size,
          lambda: ctx.check(l.nbl_pool_fwd(ctx.h, x.ptr, y.ptr, idx.ptr, B, C_, H, H, 3, 2, 0, hip.POOL_MAX)))
    x.free(); y.free(); idx.free()
    # VGG-16's first max-pool 2x2 / 2 at batch 32
    x = rand((32, 64, 224, 224)); y = ctx.empty((32, 64, 112, 112))
    timed("maxpool 2x2/2 32x64x224x224 (no argmax table)", 4 * (x.size + y.size),
          lambda: ctx.check(l.nbl_pool_fwd(ctx.h, x.ptr, y.ptr, None, 32, 64, 224, 224, 2, 2, 0, hip.POOL_MAX)))
    x.free(); y.free()
    # AlexNet's first max-pool 3x3 / 2 at batch 128: rows of 55 floats (not whole 16-byte pieces)
    x = rand((128, 96, 55, 55)); y = ctx.empty((128, 96, 27, 27))
    timed("maxpool 3x3/2 128x96x55x55 (no argmax table)", 4 * (x.size + y.size),
          lambda: ctx.check(l.nbl_pool_fwd(ctx.h, x.ptr, y.ptr, None, 128, 96, 55, 55, 3, 2, 0, hip.POOL_MAX)))
    x.free(); y.free()
    # ResNet-50's closing 7x7 average pool
    x = rand((64, 2048, 7, 7)); y = ctx.empty((64, 2048))
    timed("avgpool 7x7 64x2048x7x7", 4 * (x.size + y.size),
          lambda: ctx.check(l.nbl_pool_fwd(ctx.h, x.ptr, y.ptr, None, 64, 2048, 7, 7, 7, 7, 0, hip.POOL_AVG)))
    x.free(); y.free()

    # shortcuts as stand-alone layers (fuse_shortcut=0): same shape, and a stage entry (stride 2, fewer channels)
    prev = rand((64, 256, 56, 56)); conn = rand((64, 256, 56, 56)); y = ctx.empty((64, 256, 56, 56))
    timed("shortcut same shape 64x256x56x56 + relu", 12 * y.size,
          lambda: ctx.check(l.nbl_shortcut_fwd(ctx.h, prev.ptr, conn.ptr, y.ptr, 64, 256, 56, 56, 256, 56, 56, hip.ACT["relu"])))
    # in-place activation, bias and batchnorm primitives on the same tensor
    timed("activation relu in place, 51.4 M elements", 8 * y.size,
          lambda: ctx.check(l.nbl_activation_fwd(ctx.h, y.ptr, y.size, hip.ACT["relu"])))
    timed("activation leaky in place, 51.4 M elements", 8 * y.size,
          lambda: ctx.check(l.nbl_activation_fwd(ctx.h, y.ptr, y.size, hip.ACT["leaky"])))
    bias = rand((256,)); var = ctx.array(rng.uniform(0.5, 1.5, 256).astype(np.float32))
    timed("forward_bias 64x256x56x56", 8 * y.size,
          lambda: ctx.check(l.nbl_forward_bias(ctx.h, y.ptr, bias.ptr, 256, 56 * 56, 64)))
    timed("batchnorm_inference 64x256x56x56", 8 * y.size,
          lambda: ctx.check(l.nbl_batchnorm_inference(ctx.h, y.ptr, bias.ptr, var.ptr, bias.ptr, 256, 56 * 56, 64)))
    prev.free(); y.free()
    prev = rand((64, 512, 28, 28)); y = ctx.empty((64, 512, 28, 28))
    timed("shortcut stage entry 64x256x56x56 -> 64x512x28x28 + relu", 8 * y.size + 4 * (64 * 256 * 28 * 28),
          lambda: ctx.check(l.nbl_shortcut_fwd(ctx.h, prev.ptr, conn.ptr, y.ptr, 64, 256, 56, 56, 512, 28, 28, hip.ACT["relu"])),
          note="residual counted as the 28x28 samples it adds; it touches every other 32-byte piece of two rows out of four")
    prev.free(); conn.free(); y.free()

    # softmax: the recurrent driver's 4096 x 10000 (all time steps), and 64 x 1000 / 128 x 1000 (image nets)
    for rows, n_ in ((4096, 10000), (64, 10000), (64, 1000), (128, 1000)):
        x = rand((rows, n_)); y = ctx.empty((rows, n_))
        timed("softmax %d x %d" % (rows, n_), 8 * rows * n_,
              lambda: ctx.check(l.nbl_softmax_fwd(ctx.h, x.ptr, y.ptr, rows, n_)))
        x.free(); y.free()

    # weight-streaming connected layers (the whole layer: product, split-K reduction, bias, relu)
    for name, B_, I, O in (("VGG-16 fc6", 32, 25088, 4096), ("AlexNet fc6", 128, 9216, 4096), ("VGG-16 fc7", 32, 4096, 4096),
                           ("LSTM projection (last step)", 64, 1024, 10000)):
        label = "connected %s  %d x %d -> %d" % (name, B_, I, O)
        if args.only and args.only not in label:
            continue
        w = (rng.standard_normal((O, 8)).astype(np.float32) * 0.01).repeat(I // 8, axis=1)
        plan = ctx.fc_pack(w, np.zeros(O, np.float32), None, "relu")
        del w
        x = rand((B_, I)); y = ctx.empty((B_, O))
        timed(label, 4 * (I * O + B_ * I + B_ * O), lambda: plan(x, out=y))
        # a product with more FLOP per byte than the machine balance (157.3 TFLOP/s over 8 TB/s) is bound by the matrix pipe
        out[-1]["flop_per_byte"] = round(2.0 * B_ * I * O / out[-1]["bytes"], 1)
        out[-1]["matrix_bound"] = out[-1]["flop_per_byte"] > PEAK_FP32_MFMA_TFLOPS * 1e12 / (PEAK_HBM_GBS * 1e9)
        x.free(); y.free()
    ctx.close()
    # a kernel that moves less than 64 MB lasts a few microseconds: its figure is launch time, not bandwidth
    for r in out:
        r["launch_bound"] = r["bytes"] < (64 << 20)
    if not emit:
        return out
    rated = [r["frac_of_8TBps"] for r in (out if args.only else out[1:]) if not r["launch_bound"] and not r.get("matrix_bound")]
    worst = min(rated) if rated else None
    print(json.dumps({"metric": "memory-bound kernels, fraction of the 8 TB/s HBM peak (lowest of the kernels that move 64 MB or more and are not matrix-bound)", "value": worst,
                      "unit": "fraction", "steps": args.steps, "warmup": args.warmup, "peak_GBps": PEAK_HBM_GBS, "kernels": out}), flush=True)


def recurrent_driver(args):
    """The recurrent driver's test step (models/networks/recurrent.cc): one-hot words of a 10000-word vocabulary,
    T = 64 steps x `batch` sequences, 2 x LSTM 1024, projection + softmax on every row, perplexity update
    (--recurrent-net rnn: rnn_large's shape instead, 5 normalised RNN layers of 1024, T = 40, 8713 words, batch 32).
    Timed twice: one-hot rows as token indices (gather), and as the dense [T*B x V] matrix the reference builds."""
    from nebula_amd import zoo
    from nebula_amd.net import Network
    rng = np.random.default_rng(5)
    if args.recurrent_net == "rnn":
        B = args.batch or 32
        T, V, H = 40, 8713, 1024
        cfg = zoo.rnn_cfg(batch=B, time_steps=T, input_size=V, hidden=H, layers=5)
        net = Network(cfg)
        net.load_weight_blob(make_weights(net.weight_layout(), rng, "he"))
    else:
        B = args.batch or 64
        T, V, H = 64, 10000, 1024
        cfg = zoo.lstm_cfg(batch=B, time_steps=T, input_size=V, hidden=H, layers=2, classes=V)
        net = Network(cfg)
        net.load_weight_blob(make_weights(net.weight_layout(), rng, "lstm"))
    net.softmax_copy(False)              # the probabilities stay on the device; the perplexity sum is computed there
    tokens = rng.integers(0, V, (T, B)).astype(np.uint32)
    labels = np.roll(tokens.ravel(), -1).reshape(T, B)
    out = {}
    for mode in ("tokens", "dense one-hot"):
        if mode == "tokens":
            net.set_input_tokens(tokens)
        else:
            x = np.zeros((T * B, V), np.float32)
            x[np.arange(T * B), tokens.ravel()] = 1.0
            net.set_input(x)
        for _ in range(args.warmup):
            net.forward()
            ppl = net.accumulate_perplexity(labels)
        net.sync()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            net.forward()
            ppl = net.accumulate_perplexity(labels)
        net.sync()
        ms = (time.perf_counter() - t0) * 1e3 / args.steps
        layer_ms = np.array(net.forward_timed())
        out[mode] = {"ms_per_step": round(ms, 3), "sequences_per_s": round(B / ms * 1e3, 1), "words_per_s": round(T * B / ms * 1e3),
                     "layer_ms": [round(float(v), 3) for v in layer_ms], "perplexity_figure": round(float(ppl), 2)}
        log(mode, out[mode])
    net.close()
    print(json.dumps({"metric": "recurrent driver step (%s) sequences/s" % ("rnn_large shape" if args.recurrent_net == "rnn" else "PTB shape"),
                      "value": out["tokens"]["sequences_per_s"],
                      "unit": "sequences/s", "batch": B, "time_steps": T, "vocabulary": V, "steps": args.steps,
                      "tokens": out["tokens"], "dense_one_hot": out["dense one-hot"]}), flush=True)


CPU_SAMPLES = {"resnet50": 8, "alexnet": 16, "vgg16": 2, "conv1": 32, "lstm": 4, "rnn": 4, "dbn": 32, "mlp": 32}


def run_network(name, args, steps, warmup, cpu_sample):
    """Times one network workload and returns its record (the keys of the bench line)."""
    from nebula_amd import hip
    from nebula_amd.net import Network

    cfg, batch, xdist, wdist, text = workload(name, args.batch)
    is_lstm = name in ("lstm", "rnn")        # recurrent: units are sequences, rows are time steps x sequences
    rng = np.random.default_rng(20240611)
    if args.launches == "search":
        hip.lib().nbl_launch_table_clear()          # every convolution problem is measured on the first pass
    elif args.launches == "model":
        hip.lib().nbl_launch_table_clear()
        hip.lib().nbl_launch_table_set_search(0)    # the built-in cost model decides
    net = Network(cfg)
    blob = make_weights(net.weight_layout(), rng, wdist)
    log("workload:", text, "| weights: %.1f MB" % (blob.nbytes / 1e6))
    with tempfile.NamedTemporaryFile("wb", suffix=".wgh", delete=False) as f:
        f.write(blob.tobytes())
        wpath = f.name
    net.load_weights(wpath)
    os.unlink(wpath)
    n_in = net.batch_size * net.input_size
    x = (rng.random(n_in, dtype=np.float32) if xdist == "uniform" else rng.standard_normal(n_in).astype(np.float32))
    net.set_input(x)                     # resident in HBM before the timed region
    del x
    kinds = [net.layer_info(i)["kind"] for i in range(net.num_layers)]
    conv_layers = [i for i, k in enumerate(kinds) if k == "convolutional_layer"]
    if args.pin_launches:
        pinned = json.load(open(args.pin_launches))
        assert [p["layer"] for p in pinned] == conv_layers, "--pin-launches: the file lists other layers than this workload has"
        for p in pinned:
            net.conv_pin_launch(p["layer"], p["variant"], p["k_slices"] if p["k_slices"] > 1 else 0)
    use_graph = args.graph == 1
    if use_graph:
        net.set_graph(True)              # pass 1 eager, pass 2 recorded, replays from pass 3 (all inside the warm-up)
        warmup = max(warmup, 3)

    t_first = time.perf_counter()
    net.forward()
    net.sync()
    first_ms = (time.perf_counter() - t_first) * 1e3
    for _ in range(max(warmup - 1, 0)):
        net.forward()
    net.sync()
    # Clock ramp: after an idle moment the device takes some 100 ms of work to reach its sustained clock, and W passes
    # of a small workload are over long before that (AlexNet's first layer alone at batch 32: 74 us per launch in the
    # first milliseconds, 65 us sustained).  Untimed passes go on until --ramp-ms of work have gone by.
    ramp_passes = 0
    t_ramp = time.perf_counter()
    while (time.perf_counter() - t_ramp) * 1e3 < args.ramp_ms:
        for _ in range(8):
            net.forward()
        net.sync()
        ramp_passes += 8
    # timed region: K forward passes, synchronised on both sides; HIP events on the library's own stream
    net.timer_start()
    t0 = time.perf_counter()
    for _ in range(steps):
        net.forward()
    ev_ms = net.timer_stop()
    net.sync()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / steps
    # what was timed must be a forward pass: finite outputs, and probability rows that sum to one
    final = net.output(net.num_layers - 1 if kinds[-1] != "cost_layer" else net.num_layers - 2)
    assert np.isfinite(final).all(), "bench.py: the timed network produced non-finite outputs"
    if "softmax_layer" in kinds:
        sm = max(i for i, k in enumerate(kinds) if k == "softmax_layer")
        rows_out = batch if name == "lstm" else net.batch_size
        probs = net.output(sm).reshape(net.batch_size, -1)[:rows_out]
        assert np.abs(probs.sum(1) - 1.0).max() < 1e-3, "bench.py: softmax rows of the timed network do not sum to 1"
    # tile shape and k slices each convolution launch of the timed passes used, and where the choice came from
    variant_names = [hip.lib().nbl_conv2d_variant_name(v).decode() for v in range(hip.lib().nbl_conv2d_num_variants() + 1)]
    launches = []
    for i in conv_layers:
        v, g = net.conv_last_launch(i)
        launches.append({"layer": i, "variant": v, "tile": variant_names[v] if 0 <= v < len(variant_names) else str(v), "k_slices": g,
                         "source": net.conv_launch_source(i)})
    if args.dump_launches:
        with open(args.dump_launches, "w") as f:
            json.dump(launches, f)
    sources = sorted({p["source"] for p in launches})
    conv_tiles = " ".join("%d:%s%s" % (p["layer"], p["tile"], "/%d" % p["k_slices"] if p["k_slices"] > 1 else "") for p in launches)
    value = batch / (wall / steps)        # images (or sequences) per second
    log("timed %d steps: wall %.3f ms/step, events %.3f ms/step, first pass %.1f ms" % (steps, ms_per_step, ev_ms / steps, first_ms))

    # HIP events around every layer, in passes of their own over the same network: the layers' shares of a step
    layer_ms = np.zeros(net.num_layers)
    reps = max(3, min(10, steps))
    for _ in range(reps):
        layer_ms += np.array(net.forward_timed())
    layer_ms /= reps
    flops = np.array([net.layer_flop(i) for i in range(net.num_layers)]) * net.batch_size
    by_kind = {}
    for k, ms in zip(kinds, layer_ms):
        by_kind[k] = by_kind.get(k, 0.0) + ms
    log("per-layer-kind ms:", {k: round(v, 3) for k, v in by_kind.items()})
    fused = "fuse_shortcut=1" in cfg
    extra = {}
    if is_lstm:
        # per row: 2*(I+H)*4H (lstm), 2*(I+2*O)*O (rnn)
        rec = [i for i, k in enumerate(kinds) if k in ("lstm_layer", "rnn_layer")]
        dom_ms = float(layer_ms[rec].sum())
        steps_per_layer = net.time_step
        achieved = float(flops[rec].sum()) / (dom_ms * 1e-3) / 1e12 if dom_ms > 0 else 0.0
        roofline = {"bound": "mfma", "kernel": "%s_step_kernel" % name,
                    "covers": "the %d recurrent layers as layers: one input product over all %d time steps (gemm_nt_stream_kernel) and "
                              "%d dependent step kernels each; HIP events around each layer in passes of their own" % (len(rec), steps_per_layer, steps_per_layer),
                    "achieved": round(achieved, 3), "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s",
                    "frac": round(achieved / PEAK_FP32_MFMA_TFLOPS, 4), "traffic": None,
                    "layers_per_step": len(rec), "avg_layer_ms": round(dom_ms / max(len(rec), 1), 4)}
    elif name in ("dbn", "mlp"):
        # weight streaming: every layer reads its [O][I] matrix once per step
        fc = [i for i, k in enumerate(kinds) if k in ("connected_layer", "rbm_layer")]
        dom_ms = float(layer_ms[fc].sum())
        fc_bytes = sum(4.0 * (net.layer_info(i)["input_size"] * net.layer_info(i)["output_size"]
                              + net.batch_size * (net.layer_info(i)["input_size"] + net.layer_info(i)["output_size"])) for i in fc)
        gbps = fc_bytes / (dom_ms * 1e-3) / 1e9 if dom_ms > 0 else 0.0
        roofline = {"bound": "hbm", "kernel": "gemm_nt_stream_kernel",
                    "covers": "the %d connected layers as layers (product, split-K reduction, bias, activation); HIP events around each layer in passes of their own" % len(fc),
                    "achieved": round(gbps, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(gbps / PEAK_HBM_GBS, 4), "traffic": None,
                    "layers_per_step": len(fc), "avg_layer_ms": round(dom_ms / max(len(fc), 1), 4),
                    "algorithmic_bytes_per_layer": round(fc_bytes / max(len(fc), 1)),
                    "tflops": round(float(flops[fc].sum()) / (dom_ms * 1e-3) / 1e12, 2) if dom_ms > 0 else 0.0}
    else:
        conv = conv_layers
        dom_ms = float(layer_ms[conv].sum())
        achieved = float(flops[conv].sum()) / (dom_ms * 1e-3) / 1e12 if dom_ms > 0 else 0.0
        # the strip kernel takes the layers with very few input channels (index one past the tile shapes)
        n_strip = sum(1 for p in launches if p["tile"] == "strip")
        n_finish = sum(1 for p in launches if p["k_slices"] > 1)
        strip_ms = float(sum(layer_ms[p["layer"]] for p in launches if p["tile"] == "strip"))
        # algorithmic bytes of the same launches: input + weights + output (+ the residual a fused shortcut reads)
        algo_bytes = 0.0
        for i in conv:
            info = net.layer_info(i)
            weights = net.layer_flop(i) / (2.0 * info["output_height"] * info["output_width"])
            residual = info["output_size"] if i + 1 < len(kinds) and kinds[i + 1] == "shortcut_layer" and fused else 0
            algo_bytes += 4.0 * (net.batch_size * (info["input_size"] + info["output_size"] + residual) + weights)
        traffic, traffic_note = measured_traffic(name, batch, conv_tiles)
        roofline = {"bound": "mfma", "kernel": "conv_strip_kernel" if strip_ms > 0.5 * dom_ms else "conv_igemm_kernel",
                    "covers": "all %d convolution layers as layers: %d conv_igemm_kernel and %d conv_strip_kernel launches plus the %d "
                              "conv_split_finish_kernel launches behind k-split ones; HIP events around each layer in passes of their own "
                              "(%d passes, the events' own gaps included)" % (len(conv), len(conv) - n_strip, n_strip, n_finish, reps),
                    "achieved": round(achieved, 3), "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s",
                    "frac": round(achieved / PEAK_FP32_MFMA_TFLOPS, 4),
                    "traffic": traffic, "traffic_source": traffic_note,
                    "layers_per_step": len(conv), "avg_layer_ms": round(dom_ms / max(len(conv), 1), 4),
                    "algorithmic_bytes_per_layer": round(algo_bytes / len(conv)),
                    "algorithmic_flop_per_layer": round(float(flops[conv].sum()) / len(conv))}
        # the memory-bound layers of the same step, against the HBM peak: bytes each must read and write once
        mem = {}
        for i, k in enumerate(kinds):
            info = net.layer_info(i)
            if k in ("maxpool_layer", "avgpool_layer"):
                mem.setdefault("pooling", [0.0, 0.0])
                mem["pooling"][0] += 4.0 * net.batch_size * (info["input_size"] + info["output_size"]); mem["pooling"][1] += layer_ms[i]
            elif k in ("connected_layer", "rbm_layer"):
                b = 4.0 * (info["input_size"] * info["output_size"] + net.batch_size * (info["input_size"] + info["output_size"]))
                if 2.0 * net.batch_size * info["input_size"] * info["output_size"] / b <= PEAK_FP32_MFMA_TFLOPS * 1e3 / PEAK_HBM_GBS:
                    mem.setdefault("connected", [0.0, 0.0])
                    mem["connected"][0] += b; mem["connected"][1] += layer_ms[i]
            elif k == "shortcut_layer" and not fused:
                mem.setdefault("shortcut", [0.0, 0.0])
                mem["shortcut"][0] += 12.0 * net.batch_size * info["output_size"]; mem["shortcut"][1] += layer_ms[i]
        extra["memory_bound_layers"] = {k: {"bytes": round(b), "ms": round(ms, 4), "GBps": round(b / ms / 1e6, 1) if ms > 0 else 0.0,
                                            "frac_of_8TBps": round(b / ms / 1e6 / PEAK_HBM_GBS, 3) if ms > 0 else 0.0}
                                        for k, (b, ms) in mem.items()}
        if name == "conv1":
            extra["conv_ms"] = round(float(layer_ms[0]), 4)
            extra["pool_ms"] = round(float(layer_ms[1]), 4)

    result = {
        "metric": "ResNet-50 fp32 fwd images/s (bs64, 1 GPU); conv GEMM % of fp32 MFMA peak" if name == "resnet50"
                  else "%s fp32 fwd %s/s (1 GPU)" % (name, "sequences" if is_lstm else "images"),
        "value": round(value, 2), "unit": "sequences/s" if is_lstm else "images/s",
        "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": text, "batch": batch, "weights": "random-init (seeded), inference batchnorm folded",
                   "launch": "hip graph replay" if use_graph and net.graph_active else "eager",
                   "first_pass_ms": round(first_ms, 1), "clock_ramp": "%d untimed passes (%d ms) after the %d warm-up passes" % (ramp_passes, args.ramp_ms, warmup)},
        "roofline": roofline,
    }
    if conv_layers:
        result["config"]["conv_launches"] = ("pinned from " + os.path.basename(args.pin_launches) if args.pin_launches
                                             else sources[0] if len(sources) == 1 else "+".join(sources))
        result["config"]["conv_tiles"] = conv_tiles
    result.update(extra)

    if cpu_sample != 0:
        sample = cpu_sample if cpu_sample > 0 else CPU_SAMPLES[name]
        cfg_fn = (lambda b: workload(name, b)[0])
        ips, cores, dt, timed, blas, xs, outs = cpu_baseline(cfg_fn, blob, xdist, sample, is_lstm, np.random.default_rng(7))
        result["cpu_baseline"] = {"value": round(ips, 3), "unit": result["unit"], "cores": cores, "kind": "port",
                                  "sample": "%d %s of the same workload, %s (%.1f s per forward), %s" % (
                                      sample, "sequences" if is_lstm else "images",
                                      "1 timed forward of a fresh network" if timed == 1 else "1 warm-up + mean of %d timed forwards" % timed,
                                      dt, blas)}
        log("cpu baseline: %.2f %s on %d cores (%s)" % (ips, result["unit"], cores, blas))
    net.close()
    return result


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="all", choices=["all", "resnet50", "alexnet", "vgg16", "lstm", "conv1", "rnn", "dbn", "mlp", "copy", "conv", "convgrid", "images", "ptb", "memops"],
                    help="all (default): the ResNet-50 headline plus the other benchmarked configurations and the memory-bound kernels "
                         "in one line; a network name: that network alone; copy: a plain 256 MiB device-to-device copy kernel, the "
                         "known-size load that HBM traffic counters are calibrated against; conv: one convolution layer "
                         "(--conv-shape) through the C ABI, for counter passes over a single kernel")
    ap.add_argument("--conv-shape", default="512,28,28,256,1,1,0", help="C,H,W,F,k,stride,pad of --workload conv")
    ap.add_argument("--conv-variant", type=int, default=-1, help="tile shape index of --workload conv (-1: launch table or search)")
    ap.add_argument("--conv-split", type=int, default=-1, help="k-split mode of --workload conv (-1 launch table or search, 0 off, 1 model)")
    ap.add_argument("--conv-residual", type=int, default=0, help="1: --workload conv adds a same-shape residual and relu in the epilogue (fused shortcut)")
    ap.add_argument("--batch", type=int, default=0)
    ap.add_argument("--only", default="", help="--workload memops: time only the kernels whose label contains this text (counter passes over one kernel)")
    ap.add_argument("--cpu-sample", type=int, default=-1, help="images in the CPU baseline sample (0 = skip)")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--recurrent-net", default="lstm", choices=["lstm", "rnn"], help="network of --workload ptb")
    ap.add_argument("--launches", default="table", choices=["table", "search", "model"],
                    help="where convolution launches take their tile shape and k-split from: the shipped launch table (problems it does "
                         "not list are measured on first use), a fresh search of every problem, or the built-in cost model alone")
    ap.add_argument("--ramp-ms", type=float, default=100.0, help="untimed passes run for this long after the warm-up passes, so that the timed "
                    "passes see the device's sustained clock (0: none)")
    ap.add_argument("--dump-launches", default="", help="write the tile shape and k-split every convolution layer ran with (JSON) to this file")
    ap.add_argument("--pin-launches", default="", help="run every convolution layer with the tile shape and k-split listed in this file "
                    "(as written by --dump-launches): repeats another run's launches exactly, e.g. under counter collection")
    ap.add_argument("--graph", type=int, default=0, help="1: forward passes are replays of a recorded HIP graph, 0 (default): eager "
                    "launches (the passes are GPU-bound on this machine: both take the same time)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (every layer is batch-parallel with no exchange; "
                 "more GPUs would each take batch/N images). Re-run with --gpus 1.")

    if args.workload == "copy":
        return copy_calibration(args)
    if args.workload == "conv":
        return single_conv(args)
    if args.workload == "convgrid":
        return conv_work_grid(args)
    if args.workload == "images":
        return image_input(args)
    if args.workload == "ptb":
        return recurrent_driver(args)
    if args.workload == "memops":
        return memory_bound_kernels(args)

    cpu = 0 if args.no_cpu else args.cpu_sample
    if args.workload != "all":
        print(json.dumps(run_network(args.workload, args, args.steps, args.warmup, cpu)), flush=True)
        return
    if args.batch:
        sys.exit("bench.py: --batch goes with a single --workload")
    result = run_network("resnet50", args, args.steps, args.warmup, cpu)
    configs = []
    for name in ("conv1", "alexnet", "vgg16", "lstm"):
        r = run_network(name, args, args.steps, args.warmup, cpu)
        rec = {"workload": r["config"]["workload"], "name": name, "batch": r["config"]["batch"], "ms_per_step": r["ms_per_step"],
               "value": r["value"], "unit": r["unit"], "steps": r["steps"], "warmup": r["warmup"], "roofline": r["roofline"],
               "first_pass_ms": r["config"]["first_pass_ms"]}
        for k in ("conv_launches", "conv_tiles"):
            if k in r["config"]:
                rec[k] = r["config"][k]
        for k in ("memory_bound_layers", "conv_ms", "pool_ms", "cpu_baseline"):
            if k in r:
                rec[k] = r[k]
        configs.append(rec)
    result["configs"] = configs
    mem_args = argparse.Namespace(**vars(args))
    mem_args.steps, mem_args.warmup = min(args.steps, 50), min(max(args.warmup, 3), 10)
    result["memops"] = [{k: r[k] for k in ("kernel", "bytes", "us", "GBps", "frac_of_8TBps", "launch_bound") if k in r} | ({"matrix_bound": True} if r.get("matrix_bound") else {})
                        for r in memory_bound_kernels(mem_args, emit=False)]
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
