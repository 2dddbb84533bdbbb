#!/usr/bin/env python3
"""Benchmark of the CNN backward pass on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--serial] [--headline-only] [--config NAME]

Defaults: 20 warm-up and 100 timed passes (a shorter region ends while the clocks are still ramping).

Workload: VGG-11-style network, fp32, batch 256, 3x32x32 N(0,1) inputs, 10 uniform classes, eight
3x3/pad-1 convolutions (64,128,256,256,512,512,512,512) each with non-affine batch norm and ReLU,
max-pool 2 after convolutions 1,2,4,6,8, FC 512->10, softmax cross entropy; He-normal weights.
A step is one cnnBackward call through the C boundary (copy of the loss errors into the delta
buffer included), device-complete on return; the forward pass runs once, untimed, to produce z.
Inputs, weights and z are resident in HBM before the timed region starts.

Prints ONE JSON line: backward images/sec, plus
  roofline      the dominant kernel (largest summed time): algorithmic FLOPs / its average launch
                duration, measured with HIP events on the library's stream in a second pass of the
                same K steps (the first, timed pass runs without per-launch events), against the
                157.3 TFLOP/s fp32-MFMA peak;
  kernels       the same accounting for every kernel class of the backward pass;
  bandwidth_kernels  pool+activation and batch-norm backward run alone at the two largest layers'
                shapes, against the 8 TB/s HBM peak;
  cpu_baseline  the gradient path the reference checks itself against (torch autograd of the same network,
                float32, batch 256) on the host cores: median of 10 passes after 3 warm-ups, backward only
                (`value`) and forward + backward; `c_port` beside it is the C restatement of the reference's
                algorithm (float32, OpenMP) on a smaller batch.
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

PEAK_MFMA_F32_TFLOPS = 157.3
PEAK_MFMA_F64_TFLOPS = 78.6
PEAK_HBM_GBS = 8000.0

KC = dict(conv_dw=0, conv_dx=1, conv_fwd=2, fc_gemm=3, splitk_reduce=4, bn_bwd=5, bn_fwd=6, pool_bwd=7, pool_fwd=8,
          act_bwd=9, act_fwd=10, bias_grad=11, softmax=12, permute=13, blas1=14, pool_act_bwd=15, kfac_factor=16,
          spd_inverse=17)
MFMA_CLASSES = ("conv_dw", "conv_dx", "conv_fwd", "fc_gemm", "kfac_factor", "spd_inverse")
TILES = {0: "", 1: "64x64", 2: "64x128", 3: "128x64", 4: "128x128", 5: "96x128", 6: "dense2x2", 7: "cell4x4", 8: "cell8x8", 9: "skinny"}


def measured_traffic(kernel):
    """HBM bytes per launch of `kernel` as measured with hardware counters (FETCH_SIZE, WRITE_SIZE) in separate
    profiler runs of this program; the figures and the commands behind them are kept as text under profiles/.
    Returns (bytes, file name, commit of the tree the counters were taken at) or (None, None, None)."""
    import glob
    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", "*hbm_traffic.txt"))):
        found, tree = None, None
        for line in open(path):
            f = line.split()
            if len(f) == 3 and f[0] == "traffic_bytes_per_launch" and f[1] == kernel:
                found = int(f[2])
            if len(f) == 2 and f[0] == "tree":
                tree = f[1]
        if found is not None:
            return found, os.path.relpath(path, ROOT), tree
    return None, None, None


def tree_commit():
    import subprocess
    try:
        rev = subprocess.run(["git", "-C", ROOT, "rev-parse", "--short", "HEAD"], stdout=subprocess.PIPE,
                             stderr=subprocess.DEVNULL, text=True, timeout=10).stdout.strip()
    except (OSError, subprocess.SubprocessError):
        rev = ""
    if rev:
        return rev
    try:  # a copy of the tree without its history: the commit the build step noted
        with open(os.path.join(ROOT, "fitre_amd", "BUILD_TREE")) as f:
            return f.read().strip() or None
    except OSError:
        return None


def live_fraction(layer):
    """Share of the (output cell, window tap) pairs of a convolution layer whose tap lies inside the image: what is left of
    the window-count work 2*M*K*Cout when the products with the zero padding are not counted."""
    def live(size, out, k, stride, pad):
        return sum(1 for o in range(out) for t in range(k) if 0 <= o * stride - pad + t < size)
    k = layer.kSize
    return (live(layer.height, layer.outHeight, k, layer.stride, layer.padding) *
            live(layer.width, layer.outWidth, k, layer.stride, layer.padding)) / float(k * k * layer.outHeight * layer.outWidth)


def conv_live_fractions(model, batch):
    """Algorithmic work 2*M*K*Cout of every convolution layer's gradient launches -> the live_fraction of the layers with
    that work (two layers can share it: VGG-11's 256 -> 256 on 8x8 maps and 512 -> 512 on 4x4 maps)."""
    table = {}
    for c in range(model.cLayers):
        l = model.convLayer[c]
        work = 2.0 * batch * l.outHeight * l.outWidth * l.inChannels * l.kSize ** 2 * l.outChannels
        table.setdefault(round(work), []).append(live_fraction(l))
    return table


# kernel variants that leave out the products with the padding, and the live fraction of the maps they run on
SKIPS_PADDING = {"/dense2x2": 16 / 36.0, "/cell4x4": 100 / 144.0, "/cell8x8": 484 / 576.0}


def launch_live_fraction(kernel, work, conv_live):
    """(live fraction of the layer a launch belongs to, whether its kernel leaves the padding's products out).  Layers
    of equal work: a variant kernel names its map size; the other kernels run the layers the variants do not take, the
    larger maps."""
    for suffix, frac in SKIPS_PADDING.items():
        if kernel.endswith(suffix):
            return frac, True
    return max(conv_live.get(round(work), [1.0])), False


def kernel_table(rows, steps, launches=None, conv_live=None, fc_batch=None):
    """Per kernel class (and tile variant): launches per step, average launch duration, achieved rate against the
    bound of its class (fp32 MFMA for the contraction kernels, HBM for the others); with `launches`, also the
    four largest shapes of each kernel on their own (`largest`: work in FLOP resp. bytes).
    Convolution gradients (conv_live given): the library counts the window-count work 2*M*K*Cout per launch; `frac` is
    by the multiply-adds the kernel EXECUTES (the cell and dense variants leave out the products with the padding, the
    nine-tap kernels do not), `frac_ninetap` by the window count (can exceed 1 for those variants), `frac_useful` by the
    work without any product with the padding.  Fully connected products at a batch of at most 128 (fc_batch) move
    more bytes of weights than they can multiply: they are scored against HBM, bytes = the weight matrix once."""
    kernels = {}
    big = largest_launches(launches) if launches else {}
    executed, useful = {}, {}
    if launches and conv_live:
        for kernel, cls, work, ms in launches:
            if cls not in ("conv_dw", "conv_dx"):
                continue
            live, skips = launch_live_fraction(kernel, work, conv_live)
            executed[kernel] = executed.get(kernel, 0.0) + work * (live if skips else 1.0)
            useful[kernel] = useful.get(kernel, 0.0) + work * live
    for r in rows:
        avg_us = 1e3 * r["ms"] / r["launches"]
        mfma = r["cls"] in MFMA_CLASSES
        if r["cls"] == "fc_gemm" and fc_batch is not None and fc_batch <= 128:
            nbytes = 2.0 * r["work"] / fc_batch              # work = 2 * batch * in * out FLOP -> 4 * in * out bytes
            rate = nbytes / (r["ms"] * 1e-3) / 1e9 if r["ms"] > 0 else 0.0
            kernels[r["kernel"]] = dict(bound="hbm", launches_per_step=r["launches"] / steps, avg_us=round(avg_us, 2),
                                        ms_per_step=round(r["ms"] / steps, 4), achieved=round(rate, 1), unit="GB/s",
                                        frac=round(rate / PEAK_HBM_GBS, 4),
                                        frac_mfma=round(r["work"] / (r["ms"] * 1e-3) / 1e12 / PEAK_MFMA_F32_TFLOPS, 4) if r["ms"] > 0 else 0.0,
                                        note="batch %d: bytes = the layer's weight matrix once (read for the input gradient, "
                                             "written for the weight gradient)" % fc_batch)
            if r["kernel"] in big:   # per-launch work is in FLOP; the same conversion to bytes
                kernels[r["kernel"]]["largest"] = [dict(e, work=2.0 * e["work"] / fc_batch,
                                                        achieved=round(2.0 * e["work"] / fc_batch / (e["avg_us"] * 1e-6) / 1e9, 1),
                                                        frac=round(2.0 * e["work"] / fc_batch / (e["avg_us"] * 1e-6) / 1e9 / PEAK_HBM_GBS, 4))
                                                   for e in big[r["kernel"]]]
            continue
        rate = r["work"] / (r["ms"] * 1e-3) / (1e12 if mfma else 1e9) if r["ms"] > 0 else 0.0
        peak = PEAK_MFMA_F32_TFLOPS if mfma else PEAK_HBM_GBS
        kernels[r["kernel"]] = dict(bound="mfma" if mfma else "hbm", launches_per_step=r["launches"] / steps,
                                    avg_us=round(avg_us, 2), ms_per_step=round(r["ms"] / steps, 4),
                                    achieved=round(rate, 2 if mfma else 1), unit="TFLOP/s" if mfma else "GB/s",
                                    frac=round(rate / peak, 4))
        if r["kernel"] in executed and r["work"] > 0:
            k = kernels[r["kernel"]]
            k["frac_ninetap"] = k["frac"]
            k["work_ninetap_gflop_per_step"] = round(r["work"] / steps / 1e9, 3)
            k["work_executed_gflop_per_step"] = round(executed[r["kernel"]] / steps / 1e9, 3)
            k["achieved"] = round(rate * executed[r["kernel"]] / r["work"], 2)
            k["frac"] = round(k["achieved"] / peak, 4)
            k["frac_useful"] = round(rate * useful[r["kernel"]] / r["work"] / peak, 4)
        if r["kernel"] in big:
            kernels[r["kernel"]]["largest"] = big[r["kernel"]]
        if r["kernel"].endswith("/dense2x2"):
            kernels[r["kernel"]]["note"] = ("3x3 windows on 2x2 maps as dense products: of the nine-tap 2*M*K*Cout the kernel "
                                            "executes 16/36 (the rest multiplies padding)")
        if r["kernel"].endswith("/cell8x8"):
            kernels[r["kernel"]]["note"] = ("weight gradient of 3x3 windows on 8x8 maps, a reduction pair being one cell of two "
                                            "images: of the nine-tap 2*M*K*Cout the kernel executes 484/576 (the rest "
                                            "multiplies padding)")
        if r["kernel"].endswith("/cell4x4"):
            kernels[r["kernel"]]["note"] = ("3x3 windows on 4x4 maps, an MFMA block being one cell of 32 images: of the "
                                            "nine-tap 2*M*K*Cout the kernel executes 100/144 (the rest multiplies padding)")
    return kernels


def read_launches(L):
    """Every accounted launch of the last accounting period: (kernel name, class, work, ms)."""
    n = C.c_long()
    L.check(L.hip.fitre_hip_profile_launch_count(C.byref(n)))
    names = {v: k for k, v in KC.items()}
    out = []
    cls, tile, ms, work = C.c_int(), C.c_int(), C.c_double(), C.c_double()
    for i in range(n.value):
        L.check(L.hip.fitre_hip_profile_read_launch(i, C.byref(cls), C.byref(tile), C.byref(ms), C.byref(work)))
        name = names[cls.value]
        out.append((name + ("/" + TILES[tile.value] if tile.value else ""), name, work.value, ms.value))
    return out


def largest_launches(launches, keep=4):
    """Per kernel, the `keep` shapes that carry the most algorithmic work (launches of equal work are one shape:
    the same layer in every step), each with its own average duration and fraction of its bound — class averages
    are dominated by the many launches that last a few microseconds."""
    shapes = {}
    for kernel, cls, work, ms in launches:
        e = shapes.setdefault((kernel, cls, work), [0, 0.0])
        e[0] += 1
        e[1] += ms
    out = {}
    for (kernel, cls, work), (n, ms) in shapes.items():
        mfma = cls in MFMA_CLASSES
        t = ms * 1e-3 / n
        rate = work / t / (1e12 if mfma else 1e9) if t > 0 else 0.0
        out.setdefault(kernel, []).append(dict(work=work, launches=n, avg_us=round(t * 1e6, 2), achieved=round(rate, 2 if mfma else 1),
                                               frac=round(rate / (PEAK_MFMA_F32_TFLOPS if mfma else PEAK_HBM_GBS), 4)))
    return {k: sorted(v, key=lambda e: -e["work"])[:keep] for k, v in out.items()}


def read_profile(L):
    rows = []
    for name, cls in KC.items():
        for tile in range(len(TILES)):
            n, ms, work = C.c_long(), C.c_double(), C.c_double()
            L.check(L.hip.fitre_hip_profile_read_tile(cls, tile, C.byref(n), C.byref(ms), C.byref(work)))
            if n.value:
                rows.append(dict(kernel=name + ("/" + TILES[tile] if tile else ""), cls=name, launches=n.value,
                                 ms=ms.value, work=work.value))
    return rows


def gpu_leg(args):
    from fitre_amd import lib as L
    from fitre_amd.harness import Device, GpuModel, at, batch_inputs, build_vgg11, he_weights

    batch = 256
    dev = Device(0)
    if args.serial:
        L.check(L.hip.fitre_hip_lanes_enable(0))
    name = C.create_string_buffer(128)
    cus = C.c_int()
    L.check(L.hip.fitre_hip_device_info(C.byref(cus), None, None, None, None, name, 128))
    model = build_vgg11(batch, bn=True)
    rng = np.random.default_rng(0xF17E0003)
    w = he_weights(model, rng).astype(np.float32)
    x, y = batch_inputs(model, batch, rng)
    gm = GpuModel(dev, model, w, x.astype(np.float32), y, batch)
    conv_live = conv_live_fractions(model, batch)
    loss = gm.forward()  # untimed: produces z, probs and the loss errors
    # one plain copy of known size (64 Mi floats: 256 MiB read, 256 MiB written), outside the timed
    # region: the kernel that hardware traffic counters of the same run are scaled by
    cal_n = 1 << 26
    cal_src, cal_dst = dev.zeros(cal_n), dev.zeros(cal_n)
    L.check(L.hip.fitre_hip_copy(cal_n, cal_src, cal_dst))
    dev.sync()
    dev.free(cal_src)
    dev.free(cal_dst)

    def run(steps):
        for _ in range(steps):
            gm.backward()  # copies errors -> delta, calls cnnBackward; device-complete on return

    run(args.warmup)
    dev.sync()
    ev0, ev1 = C.c_void_p(), C.c_void_p()
    L.check(L.hip.fitre_hip_event_create(C.byref(ev0)))
    L.check(L.hip.fitre_hip_event_create(C.byref(ev1)))
    dev.sync()
    L.check(L.hip.fitre_hip_event_record(ev0))
    t0 = time.perf_counter()
    run(args.steps)
    dev.sync()
    t1 = time.perf_counter()
    L.check(L.hip.fitre_hip_event_record(ev1))
    ms_events = C.c_float()
    L.check(L.hip.fitre_hip_event_elapsed_ms(ev0, ev1, C.byref(ms_events)))
    wall = t1 - t0

    # second pass of the same steps with per-launch events
    L.check(L.hip.fitre_hip_profile_enable(1))
    run(args.steps)
    dev.sync()
    L.check(L.hip.fitre_hip_profile_enable(0))
    rows = read_profile(L)
    launches = read_launches(L)
    # the forward pass that produces z (not part of the metric), for orientation
    gm.forward()
    dev.sync()
    t0f = time.perf_counter()
    for _ in range(10):
        gm.forward()
    dev.sync()
    forward_ms = 1e3 * (time.perf_counter() - t0f) / 10
    gm.backward()  # dx of the last forward pass, for the legs below
    grad = gm.get("grad")
    finite = bool(np.isfinite(grad).all() and np.isfinite(loss))
    kfac, bandwidth, others = None, None, None
    if not args.headline_only:
        kfac = kfac_leg(L, dev, gm, model, batch, min(10, max(2, args.steps // 4)))
        kfac["hessian_vector_ms"] = hv_leg(L, dev, gm, model, batch, min(10, max(2, args.steps // 4)))
        kfac["trust_region_step_ms"] = kfac_step_leg(L, dev, gm, model, batch, 3)
    gm.release()
    if not args.headline_only:
        bandwidth = bandwidth_leg(L, dev, batch)
        others = other_configs_leg(L, dev)
    dev.close()

    kernels = kernel_table(rows, args.steps, launches, conv_live, batch)
    dom = max(rows, key=lambda r: r["ms"])
    dk = kernels[dom["kernel"]]
    roofline = dict(kernel=dom["kernel"], bound=dk["bound"], achieved=dk["achieved"],
                    peak=PEAK_MFMA_F32_TFLOPS if dk["bound"] == "mfma" else PEAK_HBM_GBS, unit=dk["unit"],
                    frac=dk["frac"], traffic=None, avg_launch_us=dk["avg_us"],
                    launches_per_step=dk["launches_per_step"])
    for key in ("frac_ninetap", "frac_useful", "work_executed_gflop_per_step", "work_ninetap_gflop_per_step"):
        if key in dk:
            roofline[key] = dk[key]
    traffic, source, taken_at = measured_traffic(dom["kernel"])
    roofline["traffic"] = traffic
    # (a plain string: nested objects inside `roofline` do not survive every reader of this line)
    roofline["traffic_source"] = ("%s: FETCH_SIZE / WRITE_SIZE of separate rocprofv3 --pmc runs of this program, scaled by the "
                                  "calibration copy; counters taken at commit %s, this tree is %s; not re-measured in this run"
                                  % (source, taken_at, tree_commit()))
    conv_rows = [r for r in rows if r["cls"] in ("conv_dw", "conv_dx")]
    conv_ms, conv_work = sum(r["ms"] for r in conv_rows), sum(r["work"] for r in conv_rows)
    conv_executed = sum(kernels[r["kernel"]].get("work_executed_gflop_per_step", r["work"] / args.steps / 1e9) for r in conv_rows)
    conv = dict(ms_per_step=round(conv_ms / args.steps, 4), gflop_per_step_ninetap=round(conv_work / args.steps / 1e9, 2),
                gflop_per_step_executed=round(conv_executed, 2), unit="TFLOP/s")
    conv["achieved"] = round(conv_executed * 1e9 / (conv_ms / args.steps * 1e-3) / 1e12, 2) if conv_ms else 0.0
    conv["frac"] = round(conv["achieved"] / PEAK_MFMA_F32_TFLOPS, 4)
    conv["frac_ninetap"] = round(conv_work / (conv_ms * 1e-3) / 1e12 / PEAK_MFMA_F32_TFLOPS, 4) if conv_ms else 0.0
    conv["note"] = ("frac: multiply-adds the kernels execute; frac_ninetap: the window count 2*M*K*Cout of every layer, which "
                    "includes products with the zero padding that the cell and dense kernels leave out")
    return dict(wall=wall, ms_events=ms_events.value, batch=batch, loss=loss, finite=finite,
                device=name.value.decode(), compute_units=cus.value, roofline=roofline, kernels=kernels,
                conv_backward_gemms=conv, kfac_factors=kfac, bandwidth_kernels=bandwidth, forward_ms=round(forward_ms, 4),
                other_configs=others)


OTHER_CONFIGS = ("lenet_b128", "lenet_bn_b1024", "alexnet_224_b64")


def other_configs_leg(L, dev, steps=10, only=None):
    """Backward images/sec of the other benchmark networks (the same step: copy of the loss errors + one
    cnnBackward): LeNet-style b128, the same with batch norm b1024, AlexNet-style 3x224x224 b64 with 1000 classes.
    Each with the per-launch accounting of a second pass of the same steps: every kernel class against its
    bound, and `roofline` = the class with the largest summed time."""
    from fitre_amd.harness import GpuModel, batch_inputs, build_alexnet, build_lenet, he_weights
    out = {}
    for name, build, batch in (("lenet_b128", lambda: build_lenet(128), 128),
                               ("lenet_bn_b1024", lambda: build_lenet(1024, bn=True), 1024),
                               ("alexnet_224_b64", lambda: build_alexnet(64), 64)):
        if only and name != only:
            continue
        model = build()
        rng = np.random.default_rng(0xF17E0005 + batch)
        w = he_weights(model, rng).astype(np.float32)
        x, y = batch_inputs(model, batch, rng)
        gm = GpuModel(dev, model, w, x.astype(np.float32), y, batch)
        gm.forward()
        for _ in range(3):
            gm.backward()
        dev.sync()
        t0 = time.perf_counter()
        for _ in range(steps):
            gm.backward()
        dev.sync()
        dt = time.perf_counter() - t0
        L.check(L.hip.fitre_hip_profile_enable(1))
        for _ in range(steps):
            gm.backward()
        dev.sync()
        L.check(L.hip.fitre_hip_profile_enable(0))
        rows = read_profile(L)
        kernels = kernel_table(rows, steps, read_launches(L), conv_live_fractions(model, batch), batch)
        dom = max(rows, key=lambda r: r["ms"])
        dk = kernels[dom["kernel"]]
        out[name] = dict(images_per_s=round(batch * steps / dt, 1), ms_per_step=round(1e3 * dt / steps, 4),
                         finite=bool(np.isfinite(gm.get("grad")).all()),
                         launches_per_step=sum(r["launches"] for r in rows) / steps,
                         kernel_ms_per_step=round(sum(r["ms"] for r in rows) / steps, 4),
                         roofline=dict(kernel=dom["kernel"], bound=dk["bound"], achieved=dk["achieved"],
                                       peak=PEAK_MFMA_F32_TFLOPS if dk["bound"] == "mfma" else PEAK_HBM_GBS,
                                       unit=dk["unit"], frac=dk["frac"], avg_launch_us=dk["avg_us"],
                                       launches_per_step=dk["launches_per_step"]),
                         kernels=kernels)
        gm.release()
    return out


def bandwidth_leg(L, dev, batch, reps=20):
    """The bandwidth-bound backward step of a layer (max-pool 2 + ReLU + batch norm, the entry point
    cnnBackward calls) run alone at the shapes of the two largest layers, 64 x 32x32 and 128 x 16x16 maps
    per image: algorithmic bytes / kernel time against the 8 TB/s HBM peak, per-launch events as in
    `kernels`, with a plain copy of the same tensor beside it.  Inside the backward pass the per-class
    averages of `kernels` are dominated by the small layers' launches; the tensors here are the ones
    that carry the bytes.  The same buffers are used by every repeat, so part of the traffic is served
    by the memory-side cache, as it is in the pass itself (a layer's delta is read right after it is
    written)."""
    hip = L.hip
    rng = np.random.default_rng(0xF17E0004)
    relu, max_pool = 13, 0  # CNN_ACT_RELU, MAX_POOL
    out = {}
    for name, channels, hw in (("layer0_64x32x32", 64, 32), ("layer1_128x16x16", 128, 16)):
        per = batch * hw * hw
        n = channels * per
        zhat = dev.upload(rng.standard_normal(n).astype(np.float32))
        var = dev.upload(np.ones(channels, np.float32))
        dpool, dact, dbn, bias = dev.zeros(n), dev.zeros(n), dev.zeros(n), dev.zeros(channels)
        delta = dev.upload(rng.standard_normal(n // 4).astype(np.float32))
        nb = hip.fitre_hip_batch_norm_workspace(channels, per)
        ws = dev.alloc(nb)

        def step():
            L.check(hip.fitre_hip_pool_act_bn_backward(max_pool, relu, delta, 1, 0, zhat, None, var, channels, batch, hw, hw, 2, 2, 0,
                                                       hw // 2, hw // 2, 1e-5, dpool, dact, dbn, bias, ws, nb))
            L.check(hip.fitre_hip_copy(n, zhat, dbn))

        step()
        dev.sync()
        L.check(hip.fitre_hip_profile_enable(1))
        for _ in range(reps):
            step()
        dev.sync()
        L.check(hip.fitre_hip_profile_enable(0))
        rows = {r["cls"]: r for r in read_profile(L)}
        # pool_act_bwd: delta (pooled) and zhat read, two gradients written; bn_bwd: gradient and zhat read,
        # result written; blas1: the copy, read + write
        want = dict(pool_act_bwd=4.0 * (n / 4 + 3 * n), bn_bwd=12.0 * n + 8.0 * channels, blas1=8.0 * n)
        entry = {}
        for cls, nbytes in want.items():
            r = rows[cls]
            t = r["ms"] * 1e-3 / r["launches"]
            entry["copy" if cls == "blas1" else cls] = dict(us=round(t * 1e6, 2), achieved=round(nbytes / t / 1e9, 1), unit="GB/s",
                                                            frac=round(nbytes / t / 1e9 / PEAK_HBM_GBS, 4))
        out[name] = entry
        for p in (zhat, var, dpool, dact, dbn, bias, delta, ws):
            dev.free(p)
    # What a plain copy reaches when nothing it touches is in a cache: 1 GiB read and 1 GiB written per pass, four
    # times the memory-side cache.  The tensors of a backward pass are in that state (z comes from the forward pass,
    # several hundred megabytes earlier); the layer-sized repeats above run partly out of the cache.
    big = 1 << 28
    src, dst = dev.zeros(big), dev.zeros(big)
    L.check(hip.fitre_hip_copy(big, src, dst))
    dev.sync()
    L.check(hip.fitre_hip_profile_enable(1))
    for _ in range(5):
        L.check(hip.fitre_hip_copy(big, src, dst))
    dev.sync()
    L.check(hip.fitre_hip_profile_enable(0))
    r = {r["cls"]: r for r in read_profile(L)}["blas1"]
    t = r["ms"] * 1e-3 / r["launches"]
    out["copy_1GiB_uncached"] = dict(us=round(t * 1e6, 2), achieved=round(8.0 * big / t / 1e9, 1), unit="GB/s",
                                     frac=round(8.0 * big / t / 1e9 / PEAK_HBM_GBS, 4))
    dev.free(src)
    dev.free(dst)
    return out


def kfac_leg(L, dev, gm, model, batch, passes):
    """Kronecker factors of every layer from the z / dx the backward pass left behind (not part of the
    images/sec metric): computeOmegaZFactors + computeLambdaDeltaFactors, `passes` times."""
    from fitre_amd.structs import KFAC_CURVATURE_INFO

    info = KFAC_CURVATURE_INFO()
    L.cnn.computeKFACStorageIndices(C.byref(model), C.byref(info))
    last = model.cLayers + model.lLayers
    omega = dev.zeros(info.OmegaZOffsets[last])
    lam = dev.zeros(info.LambdaGOffsets[last])
    ws = dev.alloc(4 * L.cnn.kfacFactorsMemRequired(C.byref(model), batch))

    def run():
        L.cnn.computeOmegaZFactors(C.byref(info), C.byref(model), C.byref(gm.data), batch, None, gm.z, omega,
                                   model.zOffsets, model.zztOffsets, ws)
        L.cnn.computeLambdaDeltaFactors(C.byref(info), C.byref(model), batch, gm.dx, None, lam, model.zOffsets,
                                        model.zztOffsets, ws)

    run()
    dev.sync()
    t0 = time.perf_counter()
    for _ in range(passes):
        run()
    dev.sync()
    wall_ms = 1e3 * (time.perf_counter() - t0) / passes
    L.check(L.hip.fitre_hip_profile_enable(1))  # resets the tables
    for _ in range(passes):
        run()
    dev.sync()
    L.check(L.hip.fitre_hip_profile_enable(0))
    rows = [r for r in read_profile(L) if r["cls"] == "kfac_factor"]
    ms, work = sum(r["ms"] for r in rows), sum(r["work"] for r in rows)
    rate = work / (ms * 1e-3) / 1e12 if ms else 0.0
    out = dict(ms_per_pass=round(wall_ms, 4), kernel_ms_per_pass=round(ms / passes, 4),
               gflop_per_pass=round(work / passes / 1e9, 2), achieved=round(rate, 2), unit="TFLOP/s",
               frac=round(rate / PEAK_MFMA_F32_TFLOPS, 4),
               note="upper-triangle flops n(n+1)*positions; all %d layers, both sides" % last)

    # factors + damped inverses of every layer, then the natural gradient of the gradient in HBM
    oinv, linv = omega, lam  # the factor storage is free again: the full passes build factors in scratch
    ngrad = dev.zeros(model.pSize)
    info.regLambda, info.dampGamma = 1e-3, 0.0  # the damping of the KFAC configuration
    info.OmegaZInv, info.LambdaGInv = oinv.value, linv.value
    info.gradient, info.nGradient = gm.grad.value, ngrad.value
    need = max(L.cnn.kfacInverseMemRequired(C.byref(model), batch), L.cnn.kfacNaturalGradientMemRequired(C.byref(model)))
    ws2 = dev.alloc(4 * need + 512)

    def inverses():
        L.cnn.computeOmegaZ(C.byref(info), C.byref(model), C.byref(gm.data), batch, None, gm.z, oinv, model.zOffsets,
                            model.zztOffsets, ws2, None, None, None, None)
        L.cnn.computeLambdaDelta(C.byref(info), C.byref(model), batch, gm.dx, None, linv, model.zOffsets, model.zztOffsets,
                                 ws2, None, None, None, None)

    inverses()
    dev.sync()
    t0 = time.perf_counter()
    for _ in range(3):
        inverses()
    dev.sync()
    out["factors_and_inverses_ms"] = round(1e3 * (time.perf_counter() - t0) / 3, 3)
    # the same pass once more with launch accounting: its float64 products and leaf factorisations
    L.check(L.hip.fitre_hip_profile_enable(1))
    inverses()
    dev.sync()
    L.check(L.hip.fitre_hip_profile_enable(0))
    rows64 = [r for r in read_profile(L) if r["cls"] in ("kfac_factor", "spd_inverse")]
    ms64, work64 = sum(r["ms"] for r in rows64), sum(r["work"] for r in rows64)
    out["factors_and_inverses"] = dict(
        arithmetic="f64 (v_mfma_f64_16x16x4f64): factors accumulated, factorised and inverted in double; inverses stored as float "
                   "pairs; input-side factors with few positions behind them kept in low-rank form",
        launches=int(sum(r["launches"] for r in rows64)), kernel_ms=round(ms64, 3), gflop=round(work64 / 1e9, 1),
        achieved=round(work64 / (out["factors_and_inverses_ms"] * 1e-3) / 1e12, 2), unit="TFLOP/s", bound="mfma_f64",
        peak=PEAK_MFMA_F64_TFLOPS, frac=round(work64 / (out["factors_and_inverses_ms"] * 1e-3) / 1e12 / PEAK_MFMA_F64_TFLOPS, 4),
        note="work as accounted per launch (2MNK per product, MNK for a symmetric result, 2n^3/3 per 64-order leaf; zero blocks of "
             "triangular operands are skipped but counted); achieved = that work / the pass's wall time over four streams; "
             "kernel_ms sums the launches of all streams")
    L.cnn.computeNaturalGradient(C.byref(model), C.byref(info), ws2, None)
    dev.sync()
    t0 = time.perf_counter()
    for _ in range(passes):
        L.cnn.computeNaturalGradient(C.byref(model), C.byref(info), ws2, None)
    dev.sync()
    out["natural_gradient_ms"] = round(1e3 * (time.perf_counter() - t0) / passes, 4)
    out["natural_gradient_finite"] = bool(np.isfinite(dev.download(ngrad, model.pSize)).all())
    out["damping"] = 1e-3
    for q in (omega, lam, ws, ws2, ngrad):
        dev.free(q)
    return out


def hv_leg(L, dev, gm, model, batch, passes):
    """cnnHv (R-operator forward and backward passes) along a random direction, on the z / dx in HBM."""
    v = dev.upload(np.random.default_rng(5).standard_normal(model.pSize).astype(np.float32))
    hv = dev.zeros(model.pSize)
    ws = dev.alloc(4 * L.cnn.cnnHvMemRequired(C.byref(model)) + 512)

    def run():
        L.cnn.cnnHv(C.byref(model), C.byref(gm.data), gm.z, gm.probs, gm.errors, gm.dx, v, hv, 0, batch, ws, None, 0.0)

    run()
    dev.sync()
    t0 = time.perf_counter()
    for _ in range(passes):
        run()
    dev.sync()
    ms = 1e3 * (time.perf_counter() - t0) / passes
    for q in (v, hv, ws):
        dev.free(q)
    return round(ms, 4)


def kfac_step_leg(L, dev, gm, model, batch, repeats):
    """The pieces above as ONE timed sequence, the way a KFAC trust-region step strings them together: full
    backward, the factors and damped inverses of both sides (one pass), the natural gradient, one Hessian-vector product."""
    from fitre_amd.structs import KFAC_CURVATURE_INFO

    info = KFAC_CURVATURE_INFO()
    L.cnn.computeKFACStorageIndices(C.byref(model), C.byref(info))
    last = model.cLayers + model.lLayers
    oinv, linv = dev.zeros(info.OmegaZOffsets[last]), dev.zeros(info.LambdaGOffsets[last])
    ngrad, hv = dev.zeros(model.pSize), dev.zeros(model.pSize)
    info.regLambda, info.dampGamma = 1e-3, 0.0
    info.OmegaZInv, info.LambdaGInv = oinv.value, linv.value
    info.gradient, info.nGradient = gm.grad.value, ngrad.value
    need = max(L.cnn.kfacInverseMemRequired(C.byref(model), batch), L.cnn.kfacNaturalGradientMemRequired(C.byref(model)),
               L.cnn.cnnHvMemRequired(C.byref(model)))
    ws = dev.alloc(4 * need + 512)

    def step():
        gm.backward()
        L.cnn.computeOmegaZAndLambdaDelta(C.byref(info), C.byref(model), C.byref(gm.data), batch, None, gm.z, gm.dx, None,
                                          model.zOffsets, model.zztOffsets, ws)
        L.cnn.computeNaturalGradient(C.byref(model), C.byref(info), ws, None)
        L.cnn.cnnHv(C.byref(model), C.byref(gm.data), gm.z, gm.probs, gm.errors, gm.dx, ngrad, hv, 0, batch, ws, None, 0.0)

    step()
    dev.sync()
    t0 = time.perf_counter()
    for _ in range(repeats):
        step()
    dev.sync()
    ms = 1e3 * (time.perf_counter() - t0) / repeats
    for q in (oinv, linv, ngrad, hv, ws):
        dev.free(q)
    return round(ms, 3)


def cpu_model_name():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def c_port_leg(batch=64, repeats=5):
    """float32 build of the oracle (the reference's algorithm restated in C, OpenMP over the host
    cores): one forward, then `repeats` backward passes on the same network at a smaller batch."""
    from fitre_amd.harness import batch_inputs, build_vgg11, he_weights
    from oracle.oracle import Oracle

    o = Oracle(double=False)
    model = build_vgg11(batch, bn=True)
    rng = np.random.default_rng(1)
    w = he_weights(model, rng).astype(np.float32)
    x, y = batch_inputs(model, batch, rng)
    _, z, _, errors = o.forward(model, w, x, y, 10, batch)
    o.backward(model, w, x, z, errors, batch)  # warm-up
    t0 = time.perf_counter()
    for _ in range(repeats):
        o.backward(model, w, x, z, errors, batch)
    dt = time.perf_counter() - t0
    cores = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    return dict(value=round(batch * repeats / dt, 2), unit="images/s (backward only)", cores=cores,
                sample="VGG-11 backward, float32, batch %d x %d passes, C restatement of the reference's algorithm with OpenMP"
                       % (batch, repeats))


def cpu_leg(batch=256, warmup=3, repeats=10):
    """The CPU gradient path the reference checks itself against (pytorch/gradtest: torch autograd through conv2d /
    batch_norm / relu / max_pool2d / linear / cross_entropy), as the oracle's torch model, float32, on the host
    cores, at the benchmark's own network and batch: `warmup` untimed passes, `repeats` timed, medians.  `value` is
    the backward-only rate (the GPU metric is backward-only); forward + backward is given beside it."""
    import torch
    from oracle import torchref
    from fitre_amd.harness import batch_inputs, build_vgg11, he_weights

    model = build_vgg11(batch, bn=True)
    rng = np.random.default_rng(0xF17E0003)
    w = he_weights(model, rng)
    x, y = batch_inputs(model, batch, rng)
    both, back = torchref.time_gradient(model, w, x, y, batch, dtype=torch.float32, warmup=warmup, repeats=repeats)
    return dict(value=round(batch / back, 2), unit="images/s", cores=os.cpu_count(), threads=torch.get_num_threads(),
                kind="port", cpu=cpu_model_name(),
                forward_backward_images_per_s=round(batch / both, 2),
                backward_ms=round(1e3 * back, 2), forward_backward_ms=round(1e3 * both, 2),
                sample="torch %s autograd, float32, VGG-11 + batch norm, batch %d, 3x32x32: median of %d passes after %d "
                       "warm-ups; value = backward only (loss.backward() with the forward pass done), "
                       "forward_backward_images_per_s = both" % (torch.__version__, batch, repeats, warmup))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--serial", action="store_true",
                    help="run every kernel on one stream (for kernel tracers: durations do not overlap)")
    ap.add_argument("--headline-only", action="store_true",
                    help="only the headline workload (no factor / inverse / Hessian-vector / bandwidth / other-network legs): "
                         "under a kernel tracer every launch then belongs to the VGG-11 batch-256 passes")
    ap.add_argument("--config", choices=OTHER_CONFIGS, default=None,
                    help="run ONLY this other benchmark network (its forward pass once, 3 + steps + steps backward passes) and "
                         "print its entry of other_configs: under a kernel tracer every launch then belongs to it")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (the reference path is single-device and every "
                 "box here has one GPU); --gpus %d is not supported" % args.gpus)

    if args.config:
        from fitre_amd import lib as L
        from fitre_amd.harness import Device
        dev = Device(0)
        if args.serial:
            L.check(L.hip.fitre_hip_lanes_enable(0))
        print(json.dumps({args.config: other_configs_leg(L, dev, steps=args.steps, only=args.config)[args.config]}))
        dev.close()
        return
    g = gpu_leg(args)
    seconds = g["ms_events"] * 1e-3
    value = g["batch"] * args.steps / seconds
    line = {
        "metric": "backward images/sec, VGG-11 fp32 b=256 on 1 MI355X",
        "value": round(value, 1),
        "unit": "images/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(1e3 * seconds / args.steps, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "VGG-11-style CNN backward (cnnBackward), fp32, batch 256, 3x32x32, BN+ReLU, 10 classes",
                   "batch": g["batch"], "device": g["device"], "compute_units": g["compute_units"]},
        "roofline": g["roofline"],
        "conv_backward_gemms": g["conv_backward_gemms"],
        "kfac_factors": g["kfac_factors"],
        "bandwidth_kernels": g["bandwidth_kernels"],
        "forward_ms_per_pass": g["forward_ms"],
        "other_configs": g["other_configs"],
        "kernels": g["kernels"],
        "wall_ms_per_step": round(1e3 * g["wall"] / args.steps, 4),
        "loss": round(g["loss"], 6),
        "finite": g["finite"],
    }
    if not args.no_cpu:
        try:
            line["cpu_baseline"] = cpu_leg()
            line["cpu_baseline"]["c_port"] = c_port_leg()
        except ImportError as exc:  # no torch on the box: the C restatement alone
            line["cpu_baseline"] = dict(c_port_leg(), kind="port", note="torch not importable: %s" % exc)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
