#!/usr/bin/env python3
"""Benchmark of the convolution training hot path on one MI355X.

Workload (benchmark configuration 2): AlexNet conv2 shape, ungrouped -- batch 256, input 96x27x27
N(0,1), 256 filters 5x5, stride 1, pad 2, weights N(0,0.01), bias 0.1, output gradient N(0,1).
One step = ConvolutionBridge forward + backward (lower, forward GEMM with remap+bias epilogue,
out-grad remap, data-gradient GEMM, lift + bias gradient, weight-gradient GEMM) on tensors that
are already resident in HBM.  Prints ONE JSON line.

    python bench.py --gpus 1 --steps 20 --warmup 5

`value` is the images/sec of that layer.  The same line carries, outside `value`, the other half of
the headline metric -- `iterations`: ms per LeNet (batch 64) and per AlexNet-shaped CaffeNet (batch 256)
training iteration, each with a whole-iteration roofline, its per-layer times and a CPU baseline of the
same chain -- and `configs`: the stage lines of the LeNet conv1 and AlexNet conv1 layers
(`--headline-only` leaves both out).  `--workload <name>` prints any one of them as a line of its own.
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

CONFIGS = {
    # name: (b, d, n, k, s, p, o)
    "lenet_conv1": (64, 1, 28, 5, 1, 0, 20),
    "alexnet_conv2": (256, 96, 27, 5, 1, 2, 256),
    "alexnet_conv1": (256, 3, 227, 11, 4, 0, 96),
    # geometries beyond the reference's benchmark files, for the direct paths that cover them: a VGG-sized 3 x 3
    # layer (images in column bands), a 7 x 7 stride-1 layer, a 1 x 1 layer (products on the tensors as they lie)
    "vgg_conv1_2": (32, 64, 224, 3, 1, 1, 64),
    "conv7x7_56": (32, 64, 56, 7, 1, 3, 64),
    "pointwise_28": (64, 256, 28, 1, 1, 0, 256),
    # 3 x 3 on 14 x 14 maps and 5 x 5 on 28 x 28 maps: output sizes the weight gradient has compile-time instances for
    "conv3x3_14": (256, 256, 14, 3, 1, 1, 256),
    "conv5x5_28": (128, 96, 28, 5, 1, 2, 256),
}
SEEDS = {"alexnet_conv1": 1234, "alexnet_conv2": 1235, "lenet_conv1": 1236, "vgg_conv1_2": 1237, "conv7x7_56": 1238,
         "pointwise_28": 1239, "conv3x3_14": 1240, "conv5x5_28": 1241}
PEAK_FP32_MFMA_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0
# HBM bytes per launch (fetched + written) come from the committed counter summaries under profiles/
# (rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE runs of this file, one counter per run, each scaled by what
# the same counter reads for a 1 GiB device copy): the tables are parsed, not copied.  Not measured by
# this run: the record names the summary the figure comes from.  A row is looked up by the kernel
# instance the library reports it launched, so a change of tile choice leaves `traffic` null instead of
# attaching an old figure to another kernel.
TRAFFIC_SOURCE = {("alexnet_conv2", "direct"): "profiles/conv2_fwd_bwd_hbm_traffic_and_mfma.md",
                  ("alexnet_conv2", "lowering"): "profiles/conv2_lowering_path_hbm_traffic_and_mfma.md",
                  ("alexnet_conv1", "direct"): "profiles/conv1_fwd_bwd_trace_traffic_mfma.md",
                  ("lenet_conv1", "direct"): "profiles/lenet_conv1_layer_trace_traffic.md",
                  ("vgg_conv1_2", "direct"): "profiles/wide_3x3_layer_trace_traffic_mfma.md",
                  ("conv7x7_56", "direct"): "profiles/conv7x7_stride1_layer_trace_traffic_mfma.md",
                  ("pointwise_28", "direct"): "profiles/pointwise_layer_trace_traffic_mfma.md",
                  ("conv3x3_14", "direct"): "profiles/conv3x3_on_14x14_layer_trace_traffic_mfma.md",
                  ("conv5x5_28", "direct"): "profiles/conv5x5_on_28x28_layer_trace_traffic_mfma.md",
                  ("caffenet", "direct"): "profiles/caffenet_iteration_kernel_trace.md",
                  ("lenet", "direct"): "profiles/lenet_iteration_kernel_trace.md"}
# which launches of a kernel a stage means, where a summary lists one kernel's launches by role
STAGE_ROLE = {"GEMM": "forward", "GEMM Data": "data-gradient", "GEMM Wghts": "weight-gradient"}


def _squash(name):
    return "".join(name.split())


def parse_traffic_table(path):
    """{(kernel instance without blanks, role or ""): fetched + written bytes per dispatch} from the markdown
    tables of a counter summary (columns `kernel`, `fetched MB`, `written MB`)."""
    out = {}
    try:
        lines = open(os.path.join(ROOT, path)).read().splitlines()
    except OSError:
        return out
    cols = None
    for line in lines:
        if not line.startswith("|"):
            cols = None
            continue
        cells = [c.strip() for c in line.strip().strip("|").split("|")]
        if cols is None:
            cols = cells if "kernel" in cells and "fetched MB" in cells and "written MB" in cells else None
            continue
        if set(cells[0]) <= set("-: "):
            continue
        name = cells[0].strip("`")
        role = ""
        if name.endswith(")") and " (" in name:
            name, role = name[:name.rindex(" (")], name[name.rindex(" (") + 2:-1].split()[0]
        try:
            nbytes = (float(cells[cols.index("fetched MB")]) + float(cells[cols.index("written MB")])) * 1e6
        except ValueError:
            continue
        out[(_squash(name), role)] = nbytes
    return out


def traffic_of(workload, path_kind, stage, kernel):
    """(bytes, source file) for the kernel instance that ran, or (None, None) when the committed summary of this
    workload has no row for it."""
    source = TRAFFIC_SOURCE.get((workload, path_kind))
    if not source or not kernel:
        return None, None
    table = parse_traffic_table(source)
    name = _squash(kernel.split(" ")[0])
    for key in ((name, STAGE_ROLE.get(stage, "")), (name, "")):
        if key in table:
            return table[key], source
    return None, None


def synth(cfg, seed, torch):
    """Seeded synthetic tensors of the benchmark configurations, generated on the host and uploaded."""
    import numpy as np
    b, d, n, k, s, p, o = CONFIGS[cfg]
    m = (n + 2 * p - k) // s + 1
    rng = np.random.default_rng(seed)
    if cfg == "alexnet_conv1":
        x = rng.uniform(0, 255, (b, d, n, n)).astype(np.float32)
        x -= np.array([104, 117, 123], np.float32)[None, :, None, None]
        bias = np.zeros(o, np.float32)
    elif cfg == "lenet_conv1":
        x = rng.uniform(0, 1, (b, d, n, n)).astype(np.float32)
        bias = np.zeros(o, np.float32)
    else:
        x = rng.standard_normal((b, d, n, n), dtype=np.float32)
        bias = np.full(o, 0.1, np.float32)
    w = (rng.standard_normal((o, d, k, k), dtype=np.float32) * np.float32(0.01))
    og = rng.standard_normal((b, o, m, m), dtype=np.float32)
    return x, w, bias, og


def host_cores():
    """Host cores this process may use (the box's share, not what the machine has)."""
    cores = os.cpu_count() or 1
    try:
        cores = min(cores, len(os.sched_getaffinity(0)))
    except Exception:
        pass
    if os.environ.get("OMP_NUM_THREADS", "").isdigit():
        cores = min(cores, int(os.environ["OMP_NUM_THREADS"]))
    return max(cores, 1)


def cct_partitions(cores, batch):
    """DeepNet::get_hw_concurrency (src/DeepNet.h:716-725): the largest power of two not above the hardware
    threads, capped by the batch (src/DeepNet.h:1102-1105)."""
    return min(2 ** int(math.floor(math.log2(max(cores, 1)))), batch)


def cpu_baseline(cfg, seed):
    """The CPU oracle (a port of CcT's CPUDriver path, GEMMs through OpenBLAS when found) timed on
    this host with CcT's own threading policy: P = min(2^floor(log2 cores), b) batch partitions,
    one BLAS thread each (src/DeepNet.h:716-725, 1102-1105)."""
    from concurrent.futures import ThreadPoolExecutor
    import numpy as np
    from oracle import cct_oracle as O
    b, d, n, k, s, p, o = CONFIGS[cfg]
    cores = host_cores()
    P = cct_partitions(cores, b)
    blas = O.bind_openblas(1)
    x, w, bias, og = synth(cfg, seed, None)
    bounds = [(i * b // P, (i + 1) * b // P) for i in range(P)]

    def part(lohi):
        lo, hi = lohi
        _, low = O.conv_forward(x[lo:hi], w, bias, k, s, p)
        O.conv_backward((hi - lo, d, n, n), w, og[lo:hi], low, k, s, p)

    def run():
        t0 = time.perf_counter()
        with ThreadPoolExecutor(P) as ex:
            list(ex.map(part, bounds))
        return time.perf_counter() - t0

    warm = run()
    reps = max(1, min(3, int(20.0 / max(warm, 1e-3))))
    times = sorted(run() for _ in range(reps))
    med = times[len(times) // 2]
    O.unbind_openblas()
    result = {
        "value": b / med, "unit": "images/sec", "cores": P, "kind": "port",
        "sample": "full %s workload (b=%d), 1 warm-up + %d timed passes, median; %d batch partitions x 1 BLAS "
                  "thread; sgemm=%s" % (cfg, b, reps, P, "OpenBLAS (scipy bundle)" if blas else "plain loops"),
    }
    # the other way to spend the same cores: one partition, all of them inside the BLAS calls
    if O.bind_openblas(cores):
        def whole():
            t0 = time.perf_counter()
            part((0, b))
            return time.perf_counter() - t0
        whole()
        t2 = sorted(whole() for _ in range(reps))[reps // 2]
        O.unbind_openblas()
        result["one_partition_all_blas_threads"] = {"value": b / t2, "unit": "images/sec", "cores": cores}
    return result


def net_workload(workload):
    """Seeded synthetic tensors of benchmark configurations 4 (lenet) and 5 (caffenet): images, labels,
    layer list, solver and one (weights, bias) pair per weight layer and channel group, generated on
    the host.  Fillers follow the reference's prototxts: gaussian weights (std 0.01; 0.005 for
    fc6/fc7) and bias 0.1 for CaffeNet, xavier-sized gaussian weights and zero bias for LeNet."""
    import numpy as np
    from caffecontroll_amd import nets
    rng = np.random.default_rng(1234 + (4 if workload == "lenet" else 5))
    if workload == "lenet":
        B, D, S, classes = 64, 1, 28, 10
        layers = nets.lenet_layers()
        x = rng.uniform(0, 1, (B, D, S, S)).astype(np.float32)
        solver = dict(base_lr=0.01, momentum=0.9, weight_decay=0.0005, lr_policy="inv", gamma=0.0001, power=0.75)
    else:
        B, D, S, classes = 256, 3, 227, 1000
        layers = nets.caffenet_layers(groups=True)
        x = rng.uniform(0, 255, (B, D, S, S)).astype(np.float32)
        x -= np.array([104, 117, 123], np.float32)[None, :, None, None]
        solver = dict(base_lr=0.01, momentum=0.9, weight_decay=0.0005, lr_policy="step", gamma=0.1, stepsize=100000)
    labels = rng.integers(0, classes, B).astype(np.float32)
    params = {}
    d, n, n_fc = D, S, 0
    for li, L in enumerate(layers):
        if L.type == nets.CONV:
            g = max(L.group, 1)
            shapes = [(L.num_output // g, d // g, L.kernel_size, L.kernel_size)] * g
            n = (n + 2 * L.pad - L.kernel_size) // L.stride + 1
            d = L.num_output
        elif L.type == nets.FC:
            shapes = [(L.num_output, d * n * n)]
            d, n = L.num_output, 1
        elif L.type == nets.MAXPOOL:
            n = (n - L.kernel_size) // L.stride + 1
            continue
        else:
            continue
        std = 0.01
        if L.type == nets.FC and workload == "caffenet":
            n_fc += 1
            std = 0.005 if n_fc <= 2 else 0.01
        for gi, shp in enumerate(shapes):
            if workload == "lenet":
                std = float(np.sqrt(1.0 / np.prod(shp[1:])))  # xavier-sized
            w = rng.standard_normal(shp, dtype=np.float32) * np.float32(std)
            bias = np.full(shp[0], 0.1 if workload == "caffenet" else 0.0, np.float32)
            params[(li, gi)] = (w, bias)
    return dict(B=B, D=D, S=S, classes=classes, layers=layers, x=x, labels=labels, solver=solver, params=params)


# Loss per image of the FIRST forward pass of the workloads above (before any update), as the CPU
# oracle computes it on the same tensors; tests/test_gpu_nets.py holds the device to the oracle on
# exactly these tensors, and every bench run checks its own first loss against the figure.
FIRST_LOSS_PER_IMAGE = {"caffenet": 6.914681, "lenet": 2.291778}


def net_flop(wl):
    """Algorithmic FLOP of one training iteration: 2 * outputs * contraction per GEMM-shaped product, three
    products per weight layer (forward, data gradient, weight gradient), two for the first weight layer, which
    computes no data gradient (src/DeepNet.h:1108-1110).  Returns (total, {layer index: FLOP per product})."""
    from caffecontroll_amd import nets
    d, n, first, total, per_layer = wl["D"], wl["S"], True, 0.0, {}
    for li, L in enumerate(wl["layers"]):
        if L.type == nets.CONV:
            m = (n + 2 * L.pad - L.kernel_size) // L.stride + 1
            f = 2.0 * L.num_output * wl["B"] * m * m * L.kernel_size ** 2 * (d // max(L.group, 1))
            d, n = L.num_output, m
        elif L.type == nets.FC:
            f = 2.0 * L.num_output * wl["B"] * d * n * n
            d, n = L.num_output, 1
        elif L.type == nets.MAXPOOL:
            n = (n - L.kernel_size) // L.stride + 1
            continue
        else:
            continue
        per_layer[li] = f
        total += f * (2 if first else 3)
        first = False
    return total, per_layer


LAYER_TYPE_NAMES = {1: "conv", 2: "fc", 3: "relu", 4: "maxpool", 5: "lrn", 6: "dropout", 7: "softmax_loss", 8: "concat"}


def net_cpu_baseline(workload):
    """One training iteration of the same chain on the CPU oracle with CcT's threading policy (src/DeepNet.h:716-725,
    1102-1105, 1165-1167, 1397): convolution, pooling, LRN, ReLU and dropout cut into P = min(2^floor(log2 cores),
    batch) batch partitions with one BLAS thread each, inner-product layers as one partition on P/2 BLAS threads."""
    import numpy as np
    from oracle import cct_oracle as O
    from oracle.oracle_net import OracleNet
    from caffecontroll_amd import nets
    wl = net_workload(workload)
    B, layers = wl["B"], wl["layers"]
    cores = host_cores()
    P = cct_partitions(cores, B)
    blas = O.bind_openblas(1)
    sv = wl["solver"]
    ref = OracleNet(O, layers, B, wl["D"], wl["S"],
                    dict(base_lr=sv["base_lr"], momentum=sv["momentum"], weight_decay=sv["weight_decay"]),
                    partitions=P, fc_blas_threads=max(P // 2, 1) if blas else 0)
    for key, (w, bias) in wl["params"].items():
        ref.params[key]["w"][...] = w.reshape(ref.params[key]["w"].shape)
        ref.params[key]["b"][...] = bias
    rng = np.random.default_rng(5)
    d, n = wl["D"], wl["S"]
    for li, (dd, nn) in enumerate(ref.shapes):
        if layers[li].type == nets.DROPOUT:
            ref.masks[li] = rng.integers(0, 2 ** 32, B * dd * nn * nn, dtype=np.uint64).astype(np.uint32)

    def run():
        t0 = time.perf_counter()
        ref.forward(wl["x"], wl["labels"])
        ref.backward()
        return time.perf_counter() - t0

    warm = run()   # also pays the first touch of the lowered matrices
    reps = max(1, min(10 if workload == "lenet" else 2, int(15.0 / max(warm, 1e-3))))
    times = sorted(run() for _ in range(reps))
    med = times[len(times) // 2]
    if blas:
        O.unbind_openblas()
    return {"value": med * 1e3, "unit": "ms", "images_per_sec": B / med, "cores": P, "kind": "port",
            "sample": "one full %s training iteration (batch %d): 1 warm-up + %d timed, median; %d batch partitions x 1 "
                      "BLAS thread for convolution / pooling / LRN / ReLU / dropout, inner-product layers on %d BLAS "
                      "threads; sgemm=%s" % (workload, B, reps, P, max(P // 2, 1),
                                             "OpenBLAS (scipy bundle)" if blas else "plain loops")}


def net_iteration(args, torch, np, workload=None, steps=None, warmup=None, with_cpu=True):
    """benchmark configurations 4 and 5: one step = forward + backward + SGD update of every layer,
    synthetic images and labels already on the device."""
    from caffecontroll_amd import HIPDriver, nets
    workload = workload or args.workload
    steps = steps or args.steps
    warmup = args.warmup if warmup is None else warmup
    drv = HIPDriver(0)
    drv.set_stream(torch.cuda.current_stream().cuda_stream)
    wl = net_workload(workload)
    B, D, S, classes, layers, x, labels = (wl[k] for k in ("B", "D", "S", "classes", "layers", "x", "labels"))
    rng = np.random.default_rng(99)
    net = nets.Net(B, D, S, layers, nets.solver_param(**wl["solver"]))
    for (li, gi), (w, bias) in wl["params"].items():
        wp, wn = net.tensor(li, nets.MODEL, gi)
        bp, bn = net.tensor(li, nets.BIAS, gi)
        assert wn == w.size and bn == bias.size
        drv.memcpy(wp, w.ctypes.data, w.nbytes, 0)
        drv.memcpy(bp, bias.ctypes.data, bias.nbytes, 0)
    drv.memcpy(net.input_ptr(), x.ctypes.data, x.nbytes, 0)
    drv.memcpy(net.labels_ptr(), labels.ctypes.data, labels.nbytes, 0)
    # the first forward pass (dropout off, so that nothing random enters) must reproduce the oracle's loss
    net.set_train(False)
    net.forward()
    first_loss = net.loss() / B
    net.set_train(True)
    want = FIRST_LOSS_PER_IMAGE[workload]
    if not abs(first_loss - want) <= 1e-3 * want:
        raise SystemExit("bench.py: first-pass loss per image %.5f differs from the oracle's %.5f" % (first_loss, want))

    pipeline = None
    if args.input_pipeline and workload == args.workload:
        # Raw 256x256 byte images in host memory stand in for the LMDB records; every step the
        # loader copies one batch into pinned staging, uploads it on its copy stream while the
        # previous iteration computes, and the transform kernel (mean, random crop, mirror, scale)
        # writes the network's input.
        from caffecontroll_amd import corpus
        H = 256 if workload == "caffenet" else S
        crop = S if H != S else 0
        mean = rng.uniform(100, 125, (D, H, H)).astype(np.float32) if workload == "caffenet" else None
        scale = 1.0 if workload == "caffenet" else 0.00390625
        cp = corpus.Corpus.create(B, D, H, H, crop_size=crop, scale=scale, mirror=crop > 0, phase=0, mean=mean, seed=1)
        pool = [(rng.integers(0, 256, (B, D, H, H), dtype=np.uint8), rng.integers(0, classes, B).astype(np.float32))
                for _ in range(2)]
        fed = [0]

        def feed():
            px, lb, _ = cp.stage()
            src = pool[fed[0] % len(pool)]
            for i in range(B):          # one copy per record, as the per-image workers do
                px[i] = src[0][i]
            lb[...] = src[1]
            cp.submit()
            fed[0] += 1

        feed()
        # the transform kernel alone: bytes read (raw + mean) and written (float batch) per launch
        raw_dev = torch.from_numpy(pool[0][0]).cuda()
        par_dev = torch.zeros((B, 3), dtype=torch.int32, device="cuda")
        mean_dev = torch.from_numpy(mean).cuda() if mean is not None else None
        out_dev = torch.empty((B, D, S, S), device="cuda")
        tm = drv.timer()
        for rep in range(3):
            if rep == 1:
                tm.start()
            for _ in range(10 if rep else 2):
                corpus.transform_batch(out_dev, raw_dev, mean_dev, par_dev, B, D, H, H, crop, scale)
        tm.stop()
        t_ms = tm.elapsed_ms() / 20
        t_bytes = B * D * S * S * (1 + 4 + (4 if mean is not None else 0))
        pipeline = {"raw_bytes_per_batch": int(B * D * H * H), "float_bytes_per_batch": int(B * D * S * S * 4),
                    "transform_kernel_ms": round(t_ms, 4), "transform_kernel_GBps": round(t_bytes / t_ms / 1e6, 1)}
        del raw_dev, out_dev

    def step():
        if pipeline is not None:
            cp.consume(net.input_ptr(), net.labels_ptr())
        net.forward()
        net.backward()
        if pipeline is not None:
            feed()

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    loss = net.loss() / B
    ms = elapsed * 1e3 / steps

    # A few more iterations with per-layer events on the library's stream (outside the timed region): where
    # the iteration's time goes, and the product kernel the iteration waits for longest.
    total_flop, layer_flop = net_flop(wl)
    prof_steps = 5 if workload == "caffenet" else 20
    net.set_profiling(True)
    layer_ms = [[0.0, 0.0] for _ in layers]
    stage_ms, stage_kernel, update_ms = {}, {}, 0.0
    for it in range(prof_steps + 1):
        net.forward()
        net.backward()
        if it == 0:
            continue   # the first profiled pass creates the events
        for li in range(len(layers)):
            f, b_ = net.layer_ms(li)
            layer_ms[li][0] += f
            layer_ms[li][1] += b_
            if layers[li].type == nets.CONV:
                for bi, ent in enumerate(net.conv_stages(li)):
                    for name, (t, kern) in ent.items():
                        stage_ms[(li, bi, name)] = stage_ms.get((li, bi, name), 0.0) + t
                        stage_kernel[(li, bi, name)] = kern
        update_ms += net.update_ms()
    net.set_profiling(False)
    per_layer = []
    for li, L in enumerate(layers):
        f, b_ = layer_ms[li][0] / prof_steps, layer_ms[li][1] / prof_steps
        if f <= 0 and b_ <= 0:
            continue   # in-place layers folded into their neighbours' stores
        ent = {"layer": li, "type": LAYER_TYPE_NAMES.get(L.type, str(L.type)), "forward_ms": round(f, 4),
               "backward_ms": round(b_, 4)}
        if li in layer_flop:
            ent["flop_per_product"] = layer_flop[li]
        per_layer.append(ent)
    products = []
    for (li, bi, name), t in stage_ms.items():
        if name not in STAGE_ROLE:
            continue
        t /= prof_steps
        flop = layer_flop[li] / max(len([k for k in stage_ms if k[0] == li and k[2] == name]), 1)
        products.append({"layer": li, "stage": name, "kernel": stage_kernel[(li, bi, name)], "ms": round(t, 4),
                         "tflops": round(flop / t / 1e9, 2), "frac": round(flop / t / 1e9 / PEAK_FP32_MFMA_TFLOPS, 4),
                         "flop_per_launch": flop})
    products.sort(key=lambda e: -e["ms"])
    dom = products[0] if products else None
    traffic, source = traffic_of(workload, "direct", dom["stage"], dom["kernel"]) if dom else (None, None)
    achieved = total_flop / ms / 1e9
    result = {
        "metric": "ms per %s train iteration (1 GPU)" % ("LeNet" if workload == "lenet" else "AlexNet-shaped"),
        "value": round(ms, 4), "unit": "ms", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic", "images_per_sec": round(B * 1e3 / ms, 1),
        "config": {"workload": "%s: fwd+bwd+SGD, batch %d, %dx%dx%d inputs, %d classes%s" % (
            workload, B, D, S, S, classes, ", conv2/4/5 in 2 groups" if workload == "caffenet" else "")},
        "first_loss_per_image": round(float(first_loss), 5), "oracle_first_loss_per_image": want,
        "final_loss_per_image": round(float(loss), 5),
        # whole iteration against the fp32 matrix peak: every FLOP of the iteration's GEMM-shaped products over the
        # wall time of the iteration (element-wise layers, SGD and launch gaps count as lost time); `dominant` is the
        # product kernel with the longest average launch, priced on its own algorithmic FLOP
        "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / PEAK_FP32_MFMA_TFLOPS, 4), "flop_per_iteration": total_flop,
                     "traffic": traffic, "traffic_source": source,
                     "dominant": dom, "scope": "whole iteration"},
        "layers": per_layer, "sgd_update_ms": round(update_ms / prof_steps, 4),
        "conv_products": products,
        **({"input_pipeline": pipeline} if pipeline is not None else {}),
    }
    net.close()
    del net
    if with_cpu and not args.no_cpu_baseline:
        result["cpu_baseline"] = net_cpu_baseline(workload)
    return result


def host_layers(args, cfg, torch, np, steps=10, warmup=3):
    """The same layer with its input and output layers in (page-locked) HOST memory, the placement
    ParallelizedBridge handles with share_pointer_with_prev/next_bridge = false
    (src/bridges/ParallelizedBridge_impl.hxx:595-621, 686-705): every forward uploads the input and downloads the
    output, every backward uploads the output gradient and downloads the input gradient.  Measured both ways:
    the batch in pieces with copies and kernels overlapped, and the reference's blocking copy - pass - copy
    sequence.  PCIe-inclusive, so never `value`."""
    from caffecontroll_amd import HIPDriver
    from caffecontroll_amd.bridges import ConvolutionLayer, solver_param
    b, d, n, k, s, p, o = CONFIGS[cfg]
    m = (n + 2 * p - k) // s + 1
    drv = HIPDriver(0)
    drv.set_stream(torch.cuda.current_stream().cuda_stream)
    x, w, bias, og = synth(cfg, SEEDS[cfg], torch)
    pin = lambda a: torch.from_numpy(a).pin_memory()
    h_in, h_ig = pin(x), torch.empty((b, d, n, n)).pin_memory()
    h_out, h_og = torch.empty((b, o, m, m)).pin_memory(), pin(og)
    moved = 4.0 * 2 * (b * d * n * n + b * o * m * m)
    out = {"bytes_over_the_link_per_step": moved, "host_memory": "page-locked"}
    for mode in ("overlapped", "blocking"):
        # ParallelizedBridge::backward (copies, gradients, SGD update); a zero learning rate keeps the weights put
        layer = ConvolutionLayer(b, d, n, k, s, p, o, h_in.numpy(), h_ig.numpy(), h_out.numpy(), h_og.numpy(),
                                 share_prev=False, share_next=False, solver=solver_param(base_lr=0.0))
        drv.memcpy(layer.model_ptr(), w.ctypes.data, w.nbytes, 0)
        drv.memcpy(layer.bias_ptr(), bias.ctypes.data, bias.nbytes, 0)
        layer.set_staging(mode == "overlapped")
        for _ in range(warmup):
            layer.forward()
            layer.backward(with_update=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            layer.forward()
            layer.backward(with_update=True)
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / steps
        out[mode] = {"ms_per_step": round(ms, 4), "images_per_sec": round(b * 1e3 / ms, 1),
                     "link_GBps": round(moved / ms / 1e6, 1), "in_pieces": layer.staging_overlapped()}
        layer.close()
    return out


def conv_layer(args, cfg, torch, np, steps, warmup, with_lowering=True, with_cpu=True):
    """One of the single-layer configurations: `steps` timed passes of ConvolutionBridge forward + backward on tensors
    resident in HBM; returns the record (headline fields, per-stage times, rooflines, CPU baseline)."""
    from caffecontroll_amd import HIPDriver
    from caffecontroll_amd.bridges import ConvolutionLayer
    b, d, n, k, s, p, o = CONFIGS[cfg]
    m = (n + 2 * p - k) // s + 1
    seed = SEEDS[cfg]
    drv = HIPDriver(0)
    drv.set_stream(torch.cuda.current_stream().cuda_stream)

    x, w, bias, og = synth(cfg, seed, torch)
    in_data = torch.from_numpy(x).cuda()
    in_grad = torch.empty_like(in_data)
    out_data = torch.empty((b, o, m, m), device="cuda")
    out_grad = torch.from_numpy(og).cuda()
    need_dgrad = not args.no_data_grad
    # algorithmic work per launch
    lower_bytes = 4.0 * (b * d * n * n + b * m * m * k * k * d)
    gemm_flop = 2.0 * o * (b * m * m) * (k * k * d)

    def run_path(level, steps, warmup):
        """`steps` timed passes of forward + backward at one path level (None = the bridge's default);
        returns (level in effect, wall seconds, per-stage records with the kernel instance that ran)."""
        layer = ConvolutionLayer(b, d, n, k, s, p, o, in_data, in_grad, out_data, out_grad)
        drv.memcpy(layer.model_ptr(), w.ctypes.data, w.nbytes, 0)
        drv.memcpy(layer.bias_ptr(), bias.ctypes.data, bias.nbytes, 0)
        layer.set_options(fused=level, profile=True, needs_backward_grad=need_dgrad)
        path = layer.path()
        for _ in range(warmup):
            layer.forward()
            layer.backward(with_update=False)
        torch.cuda.synchronize()
        stage_sum = {}
        t0 = time.perf_counter()
        for _ in range(steps):
            layer.forward()
            layer.backward(with_update=False)
            # reading the stage events waits for the step's last kernel (one host sync per step,
            # as a training loop that reads its loss does)
            for name, ms in layer.stage_ms().items():
                stage_sum[name] = stage_sum.get(name, 0.0) + ms
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        kernels = layer.stage_kernels()
        layer.close()
        per_stage = {}
        for name, total in stage_sum.items():
            if total <= 0:
                continue
            ms = total / steps
            ent = {"ms": round(ms, 4), "kernel": kernels.get(name, "")}
            if name in ("GEMM", "GEMM Data", "GEMM Wghts"):
                ent["tflops"] = round(gemm_flop / ms / 1e9, 2)
                ent["frac_fp32_mfma_peak"] = round(gemm_flop / ms / 1e9 / PEAK_FP32_MFMA_TFLOPS, 4)
            elif name in ("Lower Cube", "Inverse Lwr"):
                nbytes = lower_bytes
                if name == "Inverse Lwr" and path == 1:
                    # the same launch also reads the output gradient once for the bias gradient
                    nbytes += 4.0 * b * o * m * m
                    ent["includes"] = "bias-gradient reduction in the same launch"
                ent["algorithmic_bytes"] = nbytes
                ent["gbs"] = round(nbytes / ms / 1e6, 1)
                ent["frac_hbm_peak"] = round(nbytes / ms / 1e6 / PEAK_HBM_GBS, 4)
            per_stage[name] = ent
        return path, elapsed, per_stage

    path, elapsed, per_stage = run_path(0 if args.unfused else (None if args.path < 0 else args.path), steps, warmup)
    ms_per_step = elapsed * 1e3 / steps

    def mfma_roofline(stages):
        # dominant kernel = the product kernel with the longest average launch
        dom = max((g for g in ("GEMM", "GEMM Data", "GEMM Wghts") if g in stages), key=lambda g: stages[g]["ms"])
        ent = stages[dom]
        traffic, source = traffic_of(cfg, "direct" if path >= 2 and stages is per_stage else "lowering", dom, ent["kernel"])
        return {"bound": "mfma", "achieved": ent["tflops"], "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s",
                "frac": ent["frac_fp32_mfma_peak"], "traffic": traffic, "traffic_source": source,
                "kernel": ent["kernel"], "stage": dom, "flop_per_launch": gemm_flop, "avg_launch_ms": ent["ms"]}

    def hbm_roofline(stages):
        # the HBM-bound kernels of the lowering path: the one further from the peak
        names = [g for g in ("Lower Cube", "Inverse Lwr") if g in stages]
        if not names:
            return None
        worst = min(names, key=lambda g: stages[g]["frac_hbm_peak"])
        ent = stages[worst]
        traffic, source = traffic_of(cfg, "lowering", worst, ent["kernel"])
        return {"bound": "hbm", "achieved": ent["gbs"], "peak": PEAK_HBM_GBS, "unit": "GB/s",
                "frac": ent["frac_hbm_peak"], "traffic": traffic, "traffic_source": source, "kernel": ent["kernel"],
                "stage": worst, "bytes_per_launch": ent["algorithmic_bytes"], "avg_launch_ms": ent["ms"]}

    result = {
        "metric": "images/sec conv fwd+bwd (1 GPU)", "value": round(b * steps / elapsed, 1),
        "unit": "images/sec", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "%s: conv fwd+bwd b=%d d=%d n=%d k=%d s=%d p=%d o=%d%s%s" % (
            cfg, b, d, n, k, s, p, o, "" if need_dgrad else " (no data gradient)",
            " (path level %d)" % path)},
        "roofline": mfma_roofline(per_stage), "stages": per_stage,
    }
    if hbm_roofline(per_stage):
        result["roofline_hbm"] = hbm_roofline(per_stage)
    elif with_lowering:
        # The same layer once more through the reference's stage sequence (lower, GEMM, remap, GEMM,
        # lift, GEMM; path level 1), outside `value`: per-stage times of the lowering path and the
        # HBM-bound lowering / lifting kernels against the 8 TB/s roofline.
        _, low_elapsed, low_stages = run_path(1, max(3, min(steps, 10)), 2)
        result["stages_lowering_path"] = low_stages
        result["lowering_path_ms_per_step"] = round(low_elapsed * 1e3 / max(3, min(steps, 10)), 4)
        result["roofline_hbm"] = hbm_roofline(low_stages)
        result["roofline_mfma_lowering_path"] = mfma_roofline(low_stages)
    if with_cpu:
        result["cpu_baseline"] = cpu_baseline(cfg, seed)
    return result


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="alexnet_conv2", choices=sorted(CONFIGS) + ["lenet", "caffenet"],
                    help="a single conv layer (default: AlexNet conv2, the headline config) or a whole training "
                         "iteration of LeNet (b=64) / CaffeNet (b=256, grouped conv2/4/5)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--headline-only", action="store_true",
                    help="alexnet_conv2 only: leave out the `iterations` (LeNet, CaffeNet) and `configs` (LeNet conv1, "
                         "AlexNet conv1) records that the default line carries beside the headline")
    ap.add_argument("--host-layers", action="store_true",
                    help="single conv layers: also time the layer with its input and output layers in page-locked host "
                         "memory (copies overlapped with the kernels, and the blocking sequence beside it)")
    ap.add_argument("--input-pipeline", action="store_true",
                    help="lenet/caffenet: feed every iteration through the input pipeline (raw bytes in host memory "
                         "-> pinned staging -> asynchronous upload -> transform kernel)")
    ap.add_argument("--unfused", action="store_true", help="staged forward (GEMM, remap, bias) and separate bias gradient")
    ap.add_argument("--path", type=int, default=-1, choices=[-1, 0, 1, 2, 3],
                    help="conv path level: 0 separate passes, 1 fused epilogues, 2 direct data gradient, 3 all "
                         "direct kernels (no lowered matrix); -1 = the bridge's default")
    ap.add_argument("--no-lowering-path", action="store_true",
                    help="skip the extra passes at path level 1 that report the lowering / lifting stages")
    ap.add_argument("--no-data-grad", action="store_true", help="first-layer mode: skip data-gradient GEMM and lift")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run 5 device-to-device copies of 1 GiB (a plain copy kernel of known size, used "
                         "to scale rocprofv3's FETCH_SIZE / WRITE_SIZE counters) and exit")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU (batch sharding over several GPUs is a design note, "
              "not built); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from caffecontroll_amd import HIPDriver, load
    from caffecontroll_amd.bridges import ConvolutionLayer

    load()
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    if args.copy_calibration:
        drv = HIPDriver(0)
        nbytes = 1 << 30
        src = torch.ones(nbytes // 4, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(5):
            drv.memcpy(dst, src, nbytes, 2)
        drv.device_sync()
        print(json.dumps({"copy_calibration_bytes_read": nbytes, "copy_calibration_bytes_written": nbytes,
                          "copies": 5}))
        return
    if args.workload in ("lenet", "caffenet"):
        print(json.dumps(net_iteration(args, torch, np)))
        return
    result = conv_layer(args, args.workload, torch, np, args.steps, args.warmup,
                        with_lowering=not args.no_lowering_path, with_cpu=not args.no_cpu_baseline)
    extras = args.workload == "alexnet_conv2" and not args.headline_only and args.path < 0 and not args.unfused \
        and not args.no_data_grad
    if args.host_layers or extras:
        result["host_resident_layers"] = host_layers(args, args.workload, torch, np)
    if extras:
        # the other half of the headline metric and the remaining single-layer configurations, outside `value`
        result["configs"] = {
            cfg: conv_layer(args, cfg, torch, np, 50 if cfg == "lenet_conv1" else args.steps, args.warmup,
                            with_lowering=not args.no_lowering_path, with_cpu=not args.no_cpu_baseline)
            for cfg in ("lenet_conv1", "alexnet_conv1")}
        result["iterations"] = {
            "lenet": net_iteration(args, torch, np, workload="lenet", steps=200, warmup=20),
            "caffenet": net_iteration(args, torch, np, workload="caffenet", steps=max(args.steps, 10), warmup=5)}
    print(json.dumps(result))


if __name__ == "__main__":
    main()
