#!/usr/bin/env python3
"""Benchmark of the bandwidth-bound low-memory operators at ResNet-50 batch-184
shapes (fp32) on one MI355X.

A "step" is one pass of the hot path over one synthetic batch:
  1. BatchNorm backward from the in-place OUTPUT on [184,256,56,56]
  2. ReLU backward from the 1-bit mask on [184,256,56,56]
  3. max-pool 3x3/s2/p1 backward from 4-bit indices, [184,64,56,56] -> [184,64,112,112]
All inputs are resident in HBM before the timed region.  `value` is the
algorithmic bytes of one step (each operand read once, each result written
once) divided by the measured time per step.  Each operator is also timed on
its own with events recorded on the launch stream; the BatchNorm backward
(the dominant one) is reported in `roofline`, the others in `kernels`.

The same operators are timed on the host's cores through the stock PyTorch
CPU path on a slice of the batch (`cpu_baseline`).

Prints one JSON line.
"""
import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth, GB/s
# HBM bytes per launch come from hardware counters, which cannot be read inside this program:
# two `rocprofv3 --pmc` runs of `bench.py --only lm_ops` (FETCH_SIZE, then WRITE_SIZE), turned
# into this file by `bench.py --traffic-summary FETCH_DIR WRITE_DIR` (counter values scaled by
# what the same counter reads for the plain copy of known size that `--only lm_ops` makes first)
TRAFFIC_FILE = ROOT / "profiles" / "lm_ops_bs184_hbm_traffic.json"
# kernel (substring of its name in the counter output) behind each operator of the step
TRAFFIC_KERNELS = {"bn_bwd_from_output": "bn_resident_kernel<4, 1,", "relu_bwd_mask": "relu_bwd_mask_vec",
                   "maxpool_bwd_idx": "maxpool_bwd_k3s2p1",
                   "linear_triad_2r1w (torch add, same tensors)": "vectorized_elementwise_kernel"}


def load_traffic():
    """{operator: HBM bytes per launch} from the committed counter summary, {} if absent."""
    try:
        return {k: int(v) for k, v in json.loads(TRAFFIC_FILE.read_text())["bytes_per_launch"].items()}
    except (OSError, ValueError, KeyError):
        return {}


def traffic_summary(fetch_dir, write_dir):
    """Write TRAFFIC_FILE from the counter_collection.csv files of the two counter runs."""
    import csv
    copy_bytes = E * 4   # the yardstick copy reads and writes one tensor of E floats

    def per_kernel(folder, counter):
        acc = {}
        for f in Path(folder).rglob("*counter_collection.csv"):
            with open(f, newline="") as fh:
                for r in csv.DictReader(fh):
                    if r["Counter_Name"] == counter:
                        acc.setdefault(r["Kernel_Name"], []).append(float(r["Counter_Value"]))
        return acc

    def pick(acc, needle, largest=False):
        hits = [(k, v) for k, v in acc.items() if needle in k]
        if not hits:
            return None
        if largest:   # torch launches small element-wise kernels too: the triad is the big one
            hits = [max(hits, key=lambda kv: max(kv[1]))]
            return max(hits[0][1])
        vals = [x for _, v in hits for x in v]
        return sum(vals) / len(vals)
    fetch, write = per_kernel(fetch_dir, "FETCH_SIZE"), per_kernel(write_dir, "WRITE_SIZE")
    yard_f, yard_w = pick(fetch, "copyBuffer"), pick(write, "copyBuffer")
    if not yard_f or not yard_w:
        raise SystemExit("no copy kernel in the counter output: run `bench.py --only lm_ops`")
    scale_f, scale_w = copy_bytes / (yard_f * 1024.0), copy_bytes / (yard_w * 1024.0)
    out = {}
    for op, needle in TRAFFIC_KERNELS.items():
        big = "triad" in op
        f, w = pick(fetch, needle, big), pick(write, needle, big)
        if f is not None and w is not None:
            out[op] = int(round(f * 1024.0 * scale_f + w * 1024.0 * scale_w))
    doc = {"what": "HBM bytes per launch = FETCH_SIZE and WRITE_SIZE (KiB per dispatch) of two rocprofv3 "
                   "--pmc runs of `python3 bench.py --only lm_ops --steps 3 --warmup 1`, each scaled by "
                   "what the same counter reads for a plain copy of %d bytes" % copy_bytes,
           "scale": {"FETCH_SIZE": round(scale_f, 4), "WRITE_SIZE": round(scale_w, 4)},
           "bytes_per_launch": out}
    TRAFFIC_FILE.write_text(json.dumps(doc, indent=1) + "\n")
    print(json.dumps(doc))

N, C, H, W = 184, 256, 56, 56          # BN / ReLU tensor
PN, PC, PH_IN, PW_IN = 184, 64, 112, 112  # max-pool input
E = N * C * H * W
BYTES_BN = 3 * E * 4                    # read dy, read y, write dx
BYTES_RELU = 2 * E * 4 + E // 8         # read dy, read mask, write dx
BYTES_POOL = E * 4 + (E // 4) * 4 + (E // 4) // 2  # write dx, read dy, read packed idx
BYTES_STEP = BYTES_BN + BYTES_RELU + BYTES_POOL


def gpu_bench(steps, warmup, calibrate=False):
    import torch

    import monet_amd.lm_ops as lm_ops
    from monet_amd.lm_ops import bn as bn_ops
    from monet_amd.lm_ops import pool as pool_ops
    from monet_amd.lm_ops import relu as relu_ops

    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    # Every operator gets SETS independent input sets and takes them in turn, so that no operand is
    # read again before more than a gigabyte of other traffic has passed: inside a training step an
    # operator's inputs come from memory, while a loop over ONE set keeps the smaller ones (the
    # pooled gradient and its indices, 166 MB) in the 256 MB memory-side cache and flatters the
    # kernel (max-pool backward: 0.122 ms in such a loop, 0.188 ms inside the ResNet-50 step).
    SETS = 3
    gamma = torch.rand(C, device=dev) + 0.5
    beta = torch.randn(C, device=dev) * 0.1
    bn_sets, relu_sets, pool_sets = [], [], []
    for _ in range(SETS):
        # --- BN-from-output inputs: y = BN_train(x), dy ~ N(0,1)
        x = torch.randn(N, C, H, W, device=dev)
        y, save_mean, save_invstd = bn_ops.bn_forward_train(x, gamma, beta, None, None, 0.1, 1e-5)
        bn_sets.append((torch.randn(N, C, H, W, device=dev), y, save_invstd))
        # --- ReLU mask of an N(0,1) tensor; the backward runs in place on its own gradient
        _, mask = relu_ops.relu_forward_with_mask(x, want_output=False)
        relu_sets.append((torch.randn(N, C, H, W, device=dev), mask))
        del x
        # --- max-pool indices of an N(0,1) tensor
        px = torch.randn(PN, PC, PH_IN, PW_IN, device=dev)
        _, idx4, geo = pool_ops.max_pool2d_with_packed_indices(px, 3, 2, 1, 1, False)
        pool_sets.append((torch.randn(PN, PC, PH_IN // 2, PW_IN // 2, device=dev), idx4, geo))
        in_shape = list(px.shape)
        del px
    dy, y, save_invstd = bn_sets[0]
    torch.cuda.synchronize()

    def op_bn(k=0):
        d, yy, inv = bn_sets[k % SETS]
        return bn_ops.bn_backward_from_output(d, yy, gamma, beta, inv)

    def op_relu(k=0):
        g, m = relu_sets[k % SETS]
        return relu_ops.relu_backward_from_mask(g, m)

    def op_pool(k=0):
        d, i4, geo = pool_sets[k % SETS]
        return pool_ops.max_pool2d_backward_from_packed_indices(d, i4, geo, in_shape)

    if calibrate:
        # one plain copy of E floats (E*4 bytes read, E*4 written): the yardstick the HBM
        # traffic counters of the other kernels are scaled by; and a 2-read-1-write pass over
        # the same three tensors in plain address order (the BatchNorm backward visits the
        # same bytes channel by channel)
        scratch = torch.empty_like(dy)
        scratch.copy_(dy)
        torch.add(dy, y, out=scratch)
        del scratch
    ops = [("bn_bwd_from_output", op_bn, BYTES_BN), ("relu_bwd_mask", op_relu, BYTES_RELU),
           ("maxpool_bwd_idx", op_pool, BYTES_POOL)]
    traffic = load_traffic()
    for k in range(warmup):
        for _, fn, _ in ops:
            fn(k)
    torch.cuda.synchronize()
    ev = {name: [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
                 for _ in range(steps)] for name, _, _ in ops}
    t0 = time.perf_counter()
    for k in range(steps):
        for name, fn, _ in ops:
            a, b = ev[name][k]
            a.record()
            fn(k)
            b.record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / steps
    kernels = {}
    for name, fn, nbytes in ops:
        ms = sum(a.elapsed_time(b) for a, b in ev[name]) / steps
        gbs = nbytes / (ms * 1e-3) / 1e9
        kernels[name] = {"ms": round(ms, 4), "bytes": nbytes, "GB/s": round(gbs, 1),
                         "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": traffic.get(name)}
        # the same operator over ONE input set, back to back (operands that fit the memory-side
        # cache stay there): reported beside the number above, never used for `value`
        for _ in range(3):
            fn(0)
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(steps):
            fn(0)
        b.record()
        torch.cuda.synchronize()
        kernels[name]["ms_same_operands_back_to_back"] = round(a.elapsed_time(b) / steps, 4)
    # ceiling for a 2-read-1-write pass over tensors of this size in plain address order
    tri_out = torch.empty_like(dy)
    for _ in range(warmup):
        torch.add(dy, y, out=tri_out)
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    a.record()
    for _ in range(steps):
        torch.add(dy, y, out=tri_out)
    b.record()
    torch.cuda.synchronize()
    ms = a.elapsed_time(b) / steps
    kernels["linear_triad_2r1w"] = {"ms": round(ms, 4), "bytes": BYTES_BN,
                                    "GB/s": round(BYTES_BN / (ms * 1e-3) / 1e9, 1),
                                    "frac": round(BYTES_BN / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                                    "in_step": False, "what": "torch.add over the same three tensors"}
    del tri_out
    # the forward kernels of the same operators, timed on their own (not part of the step), each
    # over three input tensors in turn
    del bn_sets[1:], relu_sets[1:], pool_sets[1:]
    xs = [torch.randn(N, C, H, W, device=dev) for _ in range(SETS)]
    pxs = [torch.randn(PN, PC, PH_IN, PW_IN, device=dev) for _ in range(SETS)]
    fwd = [("relu_fwd_mask", lambda k: relu_ops.relu_forward_with_mask(xs[k % SETS]), 2 * E * 4 + E // 8),
           ("bn_fwd_train", lambda k: bn_ops.bn_forward_train(xs[k % SETS], gamma, beta, None, None, 0.1, 1e-5),
            2 * E * 4),
           ("maxpool_fwd_idx", lambda k: pool_ops.max_pool2d_with_packed_indices(pxs[k % SETS], 3, 2, 1, 1, False),
            BYTES_POOL)]
    for name, fn, nbytes in fwd:
        for k in range(warmup):
            fn(k)
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        a.record()
        for k in range(steps):
            fn(k)
        b.record()
        torch.cuda.synchronize()
        ms = a.elapsed_time(b) / steps
        gbs = nbytes / (ms * 1e-3) / 1e9
        kernels[name] = {"ms": round(ms, 4), "bytes": nbytes, "GB/s": round(gbs, 1),
                         "frac": round(gbs / HBM_PEAK_GBS, 4), "in_step": False}
    return ms_per_step, kernels


def cpu_baseline(sample_n=23, reps=5):
    """Stock PyTorch CPU operators on `sample_n` of the 184 images, all host threads."""
    import torch

    from oracle import cpu_path

    threads = torch.get_num_threads()
    torch.manual_seed(0)
    x = torch.randn(sample_n, C, H, W)
    gamma = torch.rand(C) + 0.5
    beta = torch.randn(C) * 0.1
    y, mean, invstd = cpu_path.bn_forward(x, gamma, beta)
    dy = torch.randn_like(x)
    px = torch.randn(sample_n, PC, PH_IN, PW_IN)
    py, pidx = cpu_path.maxpool_forward(px, 3, 2, 1)
    pdy = torch.randn_like(py)

    def step():
        cpu_path.bn_backward(dy, x, gamma, mean, invstd)
        cpu_path.relu_backward(dy, y)
        cpu_path.maxpool_backward(pdy, px, 3, 2, 1, pidx)

    step()  # warm-up
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        step()
        times.append(time.perf_counter() - t0)
    med = sorted(times)[len(times) // 2]
    nbytes = BYTES_STEP * sample_n / N

    def median_ms(fn, n=3):
        fn()
        ts = []
        for _ in range(n):
            t0 = time.perf_counter()
            fn()
            ts.append(time.perf_counter() - t0)
        return sorted(ts)[len(ts) // 2] * 1e3
    # the layer3 convolution of the convolution benchmark, three directions, same slice of the batch
    g = CONV_SHAPE
    cx = torch.randn(sample_n, g["C"], g["H"], g["W"])
    cw = torch.randn(g["K"], g["C"], g["R"], g["S"]) * (2.0 / (g["K"] * 9)) ** 0.5
    cdy = torch.randn(sample_n, g["K"], g["H"], g["W"])
    cflops = 2.0 * cdy.numel() * g["C"] * 9
    conv_legs = {}
    for i, name in enumerate(("fwd", "bwd_data", "bwd_weight")):
        if i == 0:
            ms = median_ms(lambda: cpu_path.conv_forward(cx, cw, g["stride"], g["pad"]))
        else:
            mask = [i == 1, i == 2, False]
            ms = median_ms(lambda: cpu_path.conv_backward(cdy, cx, cw, g["stride"], g["pad"], mask))
        conv_legs[name] = {"ms": round(ms, 3), "TFLOP/s": round(cflops / ms / 1e9, 3)}
    # the stem block (7x7/2 convolution, BatchNorm, ReLU, 3x3/2 max-pool; batch 8 of 3x224x224),
    # forward + backward through stock autograd: 2 warm-up + median of 5
    stem, sx = cpu_path.stem_block(8)
    cpu_path.stem_step(stem, sx)
    stem_ms = median_ms(lambda: cpu_path.stem_step(stem, sx), 5)
    return {"value": round(nbytes / med / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"{sample_n} of {N} images of the same three operators through stock PyTorch "
                      f"CPU ops (torch {torch.__version__}), 1 warm-up + median of {reps}",
            "conv_layer3": {"sample": f"{sample_n} of {N} images, fp32, torch CPU convolution "
                                      f"(mkldnn {torch.backends.mkldnn.is_available()}), 1 warm-up + median of 3",
                            **conv_legs},
            "stem_block": {"sample": "batch 8, forward + backward, 2 warm-up + median of 5",
                           "ms": round(stem_ms, 2), "images_per_s": round(8 / stem_ms * 1e3, 1)}}


MFMA_F32_PEAK_TFLOPS = 157.3   # MI355X published dense fp32 matrix rate
MFMA_BF16_PEAK_TFLOPS = 2500.0  # ... and dense bf16
CONV_SHAPE = dict(N=184, C=256, K=256, R=3, S=3, H=14, W=14, stride=1, pad=1)  # ResNet-50 layer3
# Matrix-core work each entry of the convolution benchmark really issues, from hardware counters
# (they cannot be read inside this program): one `rocprofv3 --pmc SQ_INSTS_VALU_MFMA_MOPS_F32
# SQ_INSTS_VALU_MFMA_MOPS_BF16 SQ_VALU_MFMA_BUSY_CYCLES GRBM_GUI_ACTIVE` run of
# `bench.py --only conv --steps 3 --warmup 1`, turned into this file by
# `bench.py --mfma-summary PMC_DIR BENCH_STDOUT`.
MFMA_FILE = ROOT / "profiles" / "conv_bs184_mfma_flops.json"
MARKER = "spin_kernel"   # torch.cuda._sleep: separates the entries in the counter output


def load_mfma():
    """{entry path: {"flop": issued per call, "mfma": "f32" | "bf16", "busy": ...}}, {} if absent."""
    try:
        return json.loads(MFMA_FILE.read_text())["entries"]
    except (OSError, ValueError, KeyError):
        return {}


def mfma_summary(pmc_dir, bench_stdout):
    """Write MFMA_FILE.  The benchmark launches one marker kernel before every entry and prints
    the entries in order (`order`), with the calls each made; the dispatches between two markers
    are one entry's.  flop = MFMA_MOPS * 512 (one counter unit is 512 floating-point operations
    on this chip; the direct kernels come out at exactly their algorithmic count)."""
    import csv
    line = [l for l in Path(bench_stdout).read_text().splitlines() if l.startswith("{")][-1]
    conv = json.loads(line)["conv"]
    order, calls = conv["order"], conv["calls_per_entry"]
    rows = {}
    for f in Path(pmc_dir).rglob("*counter_collection.csv"):
        with open(f, newline="") as fh:
            for r in csv.DictReader(fh):
                d = rows.setdefault(int(r["Dispatch_Id"]), {"name": r["Kernel_Name"]})
                d[r["Counter_Name"]] = d.get(r["Counter_Name"], 0.0) + float(r["Counter_Value"])
    segments, cur = [], None
    for did in sorted(rows):
        if MARKER in rows[did]["name"]:
            cur = []
            segments.append(cur)
        elif cur is not None:
            cur.append(rows[did])
    if len(segments) != len(order):
        raise SystemExit("%d marked segments for %d entries" % (len(segments), len(order)))
    entries = {}
    for name, seg in zip(order, segments):
        if name.endswith("/probe"):
            continue
        f32 = sum(d.get("SQ_INSTS_VALU_MFMA_MOPS_F32", 0.0) for d in seg) * 512.0 / calls
        b16 = sum(d.get("SQ_INSTS_VALU_MFMA_MOPS_BF16", 0.0) for d in seg) * 512.0 / calls
        busy = sum(d.get("SQ_VALU_MFMA_BUSY_CYCLES", 0.0) for d in seg)
        act = sum(d.get("GRBM_GUI_ACTIVE", 0.0) for d in seg if d.get("SQ_VALU_MFMA_BUSY_CYCLES", 0.0) > 0)
        kernels = sorted({d["name"].split("(")[0][:100] for d in seg if
                          d.get("SQ_VALU_MFMA_BUSY_CYCLES", 0.0) > 0})
        entries[name] = {"flop": f32 + b16, "mfma": "bf16" if b16 > f32 else "f32",
                         # busy cycles of the 1024 SIMDs over the cycles of the kernels that use them
                         "busy": round(busy / (1024.0 * act / 8.0), 3) if act else None,
                         "kernels": kernels}
    doc = {"what": "matrix-core floating-point operations per call of every entry of `python3 bench.py "
                   "--only conv --steps 3 --warmup 1`, from rocprofv3 --pmc SQ_INSTS_VALU_MFMA_MOPS_F32 "
                   "SQ_INSTS_VALU_MFMA_MOPS_BF16 SQ_VALU_MFMA_BUSY_CYCLES GRBM_GUI_ACTIVE (flop = MOPS * "
                   "512; busy = MFMA busy cycles / (1024 SIMDs * GRBM_GUI_ACTIVE / 8 XCDs) over the "
                   "kernels of the entry that use the matrix cores)",
           "entries": entries}
    MFMA_FILE.write_text(json.dumps(doc, indent=1) + "\n")
    print(json.dumps(doc))


def conv_bench(steps, warmup):
    """Forward / backward-data / backward-weight of the ResNet-50 layer3 3x3 convolution at
    batch 184, every kernel variant the solver can select, fp32 and bf16; two 1x1 shapes of the
    same network (where the three-slice variant applies) and one large-plane UNet shape.
    `TFLOP/s_effective` counts the direct convolution's 2*N*K*P*Q*C*R*S per call whatever the
    kernel does; `frac_mfma` is the matrix-core work the kernels really issue (hardware counters,
    MFMA_FILE) per second against the peak of the matrix instruction they use - Winograd issues
    2.24x fewer operations than the direct form, the three-slice variant six times as many in
    bf16 - so it never exceeds 1."""
    import torch

    from monet_amd.lm_ops import conv as cv
    from monet_amd import _lib
    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    issued = load_mfma()
    order = []

    def timed(path, fn, flops):
        torch.cuda._sleep(1)       # the marker kernel
        order.append(path)
        for _ in range(warmup):
            fn()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        a.record()
        for _ in range(steps):
            fn()
        b.record()
        torch.cuda.synchronize()
        ms = a.elapsed_time(b) / steps
        out = {"ms": round(ms, 4), "TFLOP/s_effective": round(flops / ms / 1e9, 1)}
        cnt = issued.get(path)
        if cnt:
            peak = MFMA_BF16_PEAK_TFLOPS if cnt["mfma"] == "bf16" else MFMA_F32_PEAK_TFLOPS
            out.update({"mfma": cnt["mfma"], "issued_flop_per_call": cnt["flop"],
                        "frac_mfma": round(cnt["flop"] / ms / 1e9 / peak, 4)})
        else:
            out["frac_mfma"] = None
        return out

    def runs(path, fn, n):
        """Variants of one direction that take this shape: {variant: callable}.  The trial calls
        get a marker and an entry of their own ("/probe"), which the counter summary drops."""
        torch.cuda._sleep(1)
        order.append(path + "/probe")
        ok = {}
        for v in range(n):
            try:
                fn(v)
                ok[v] = (lambda v=v: fn(v))
            except _lib.MonetHipError as e:
                if e.status != _lib.MN_EUNSUPPORTED:
                    raise
        return ok

    def directions(prefix, g, x, w, dy, which=("fwd", "bwd_data", "bwd_weight")):
        out = {}
        flops = 2.0 * dy.numel() * w.shape[1] * w.shape[2] * w.shape[3]
        table = {
            "fwd": (cv.n_fwd_algos(x.dtype), lambda v: cv.conv_forward(
                x, w, None, g["pad"], g["stride"], 1, 1, v)),
            "bwd_data": (cv.n_bwd_ip_algos(x.dtype), lambda v: cv.conv_backward_input(
                list(x.shape), dy, w, g["pad"], g["stride"], 1, 1, v)),
            "bwd_weight": (cv.n_bwd_wt_algos(x.dtype), lambda v: cv.conv_backward_weight(
                list(w.shape), dy, x, g["pad"], g["stride"], 1, 1, v)),
        }
        for d in which:
            n, fn = table[d]
            for v, call in runs(prefix + d, fn, n).items():
                key = "%s_v%d" % (d, v)
                out[key] = timed(prefix + key, call, flops)
        out["flops_per_call"] = flops
        return out

    def problem(g):
        torch.cuda._sleep(1)            # the set-up work is nobody's entry
        order.append("setup/probe")
        x = torch.randn(g["N"], g["C"], g["H"], g["W"], device=dev)
        w = torch.randn(g["K"], g["C"], g["R"], g["S"], device=dev) * (2.0 / (g["K"] * g["R"] * g["S"])) ** 0.5
        y = cv.conv_forward(x, w, None, g["pad"], g["stride"], 1, 1, 0)
        return x, w, torch.randn_like(y)

    c = CONV_SHAPE
    x, w, dy = problem(c)
    res = {"shape": c, "dtype": "f32", "peak_TFLOP/s": MFMA_F32_PEAK_TFLOPS}
    res.update(directions("", c, x, w, dy))
    # the same problem on bf16 channels-last tensors (bf16 matrix cores, fp32 accumulation)
    cl = lambda t: t.to(torch.bfloat16).contiguous(memory_format=torch.channels_last)
    res["bf16"] = {"layout": "channels-last", "peak_TFLOP/s": MFMA_BF16_PEAK_TFLOPS}
    res["bf16"].update(directions("bf16/", c, cl(x), cl(w), cl(dy)))
    del x, w, dy
    # 1x1 convolutions of the same network, fp32: variant 4 splits every operand into three bf16
    # slices and accumulates the six significant products on the bf16 matrix cores
    for name, g in (("pointwise_1024_256_14x14", dict(N=184, C=1024, K=256, R=1, S=1, H=14, W=14, stride=1, pad=0)),
                    ("pointwise_64_256_56x56", dict(N=184, C=64, K=256, R=1, S=1, H=56, W=56, stride=1, pad=0))):
        x, w, dy = problem(g)
        res[name] = {"shape": g}
        res[name].update(directions(name + "/", g, x, w, dy, ("fwd", "bwd_data")))
        del x, w, dy
    # one large-plane shape (UNet batch 11, 128 -> 128 channels at 208 x 304), forward and
    # backward-weight: where the one-kernel Winograd variants are the fastest
    u = dict(N=11, C=128, K=128, R=3, S=3, H=208, W=304, stride=1, pad=1)
    x, w, dy = problem(u)
    res["unet_128ch_208x304"] = {"shape": u}
    res["unet_128ch_208x304"].update(directions("unet_128ch_208x304/", u, x, w, dy, ("fwd", "bwd_weight")))
    del x, w, dy
    # the stem (3 -> 64 channels, 7x7, stride 2): variant 1 of forward and backward-weight are
    # kernels of their own
    st = dict(N=184, C=3, K=64, R=7, S=7, H=224, W=224, stride=2, pad=3)
    x, w, dy = problem(st)
    res["stem_3_64_224x224"] = {"shape": st}
    res["stem_3_64_224x224"].update(directions("stem_3_64_224x224/", st, x, w, dy, ("fwd", "bwd_weight")))
    res["order"] = order
    res["calls_per_entry"] = steps + warmup
    return res


E2E_MODE = "inplace_conv_multiway_newnode"
E2E_BS = 184
UNET_BS = 11


def _release():
    """Drop what earlier runs left behind (wrappers and optimizers hold reference cycles)."""
    import gc

    import torch
    gc.collect()
    torch.cuda.empty_cache()


def _train_ms(model, x, loss_fn, iters, warmup, foreign=0):
    """ms per SGD step (forward, loss, backward, momentum update) and peak MB of the job
    (`foreign` = bytes other parts of this program still hold on the device)."""
    import torch
    opt = torch.optim.SGD(model.parameters(), lr=0.01, momentum=0.9)

    def step():
        opt.zero_grad(set_to_none=True)
        loss_fn(model(x)).backward()
        opt.step()
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    t0 = torch.cuda.Event(enable_timing=True)
    t1 = torch.cuda.Event(enable_timing=True)
    t0.record()
    for _ in range(iters):
        step()
    t1.record()
    torch.cuda.synchronize()
    return t0.elapsed_time(t1) / iters, (torch.cuda.max_memory_allocated() - foreign) / 2**20


def _schedules(name, bs, make_model, input_shape, x, loss_fn, modes, iters, warmup, res):
    """Times `make_model()` under every committed schedule of `modes` (unconstrained, 10 GB,
    6 GB), then with stock PyTorch autograd.  Overhead is against the unconstrained schedule
    of the same operator set; peak_MB is the allocator's peak over the timed steps, with
    weights, batch, gradients and optimizer state."""
    import torch

    from monet_amd.monet_wrapper import MONeTWrapper
    dev = x.device
    _release()
    # what the device holds that is not this job's batch (and labels): nothing, normally
    foreign = max(0, torch.cuda.memory_allocated() - x.numel() * x.element_size() - (64 << 20))
    for suffix, mode in modes:
        base = None
        for budget in (100, 10, 6):
            sol = ROOT / "data" / ("solution_%s_%d_%s_%.2f.pkl" % (name, bs, mode, budget))
            if not sol.exists():
                continue
            model = MONeTWrapper(make_model(), str(sol), input_shape).to(dev)
            model.train()
            ms, mb = _train_ms(model, x, loss_fn, iters, warmup, foreign)
            key = ("unconstrained" if budget == 100 else "budget_%dGB" % budget) + suffix
            print("[bench] %s %s: %.2f ms/step, peak %.0f MiB" % (name, key, ms, mb),
                  file=sys.stderr, flush=True)
            res[key] = {"images_per_s": round(bs / ms * 1e3, 1), "ms_per_step": round(ms, 2),
                        "peak_MB": round(mb, 1)}
            if budget == 100:
                base = ms
            else:
                res[key]["within_budget"] = bool(mb <= budget * 1024)
                if base:
                    res[key]["overhead_vs_unconstrained"] = round(ms / base - 1.0, 4)
            del model
            _release()
    model = make_model().to(dev).train()
    ms, mb = _train_ms(model, x, loss_fn, iters, warmup, foreign)
    res["stock_pytorch"] = {"images_per_s": round(bs / ms * 1e3, 1), "ms_per_step": round(ms, 2),
                            "peak_MB": round(mb, 1)}
    del model
    _release()
    return res


def end_to_end(iters=20, warmup=100):
    """ResNet-50 (torchvision topology, random init), batch 184, fp32 SGD steps with cross
    entropy over 1000 classes: under the solved 10 GB and 6 GB schedules, under the
    unconstrained schedule (same kernels, nothing recomputed) and with stock PyTorch autograd;
    three operator sets (the reference's; BatchNorm+ReLU and add+ReLU pairs fused; also
    BatchNorm+add+ReLU at the end of a residual block).  Timing protocol of the reference
    (monet/schedule.py:430-443): 100 warm-up steps, then 20 timed steps between two events."""
    import torch

    from monet_amd.models import resnet50
    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    x = torch.randn(E2E_BS, 3, 224, 224, device=dev)
    target = torch.randint(0, 1000, (E2E_BS,), device=dev)
    res = {"model": "resnet50", "batch": E2E_BS, "dtype": "f32", "unit": "images/s",
           "step": "forward + cross entropy + backward + SGD momentum update",
           "timed_steps": iters, "warmup_steps": warmup}
    modes = (("", E2E_MODE), ("_fused", "fused_" + E2E_MODE), ("_fused2", "fused2_" + E2E_MODE))
    return _schedules("resnet50", E2E_BS, resnet50, (3, 224, 224), x,
                      lambda out: torch.nn.functional.cross_entropy(out, target), modes, iters,
                      warmup, res)


def end_to_end_unet(iters=20, warmup=100):
    """The reference's UNet (models/unet) with 2 output classes, batch 11, 3 x 416 x 608, fp32
    SGD steps with softmax cross entropy over per-pixel labels, same runs as for ResNet-50."""
    import torch

    from monet_amd.models import build_model
    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    _, shape, _ = build_model("unet")
    x = torch.randn((UNET_BS,) + tuple(shape), device=dev)
    target = torch.randint(0, 2, (UNET_BS, shape[1], shape[2]), device=dev)
    res = {"model": "unet (2 classes)", "batch": UNET_BS, "input": list(shape), "dtype": "f32",
           "unit": "images/s",
           "step": "forward + per-pixel softmax cross entropy + backward + SGD momentum update",
           "timed_steps": iters, "warmup_steps": warmup}
    modes = (("", E2E_MODE), ("_fused", "fused_" + E2E_MODE))
    return _schedules("unet", UNET_BS, lambda: build_model("unet")[0], tuple(shape), x,
                      lambda out: torch.nn.functional.cross_entropy(out, target), modes, iters,
                      warmup, res)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-end-to-end", action="store_true")
    ap.add_argument("--only", choices=["conv", "lm_ops", "resnet50", "unet"], default=None,
                    help="run one section alone (for profiling under rocprofv3)")
    ap.add_argument("--traffic-summary", nargs=2, metavar=("FETCH_DIR", "WRITE_DIR"), default=None,
                    help="no GPU work: turn the output folders of the two counter runs of "
                         "`--only lm_ops` into profiles/lm_ops_bs184_hbm_traffic.json")
    ap.add_argument("--mfma-summary", nargs=2, metavar=("PMC_DIR", "BENCH_STDOUT"), default=None,
                    help="no GPU work: turn the output folder of the counter run of `--only conv` and "
                         "what that run printed into profiles/conv_bs184_mfma_flops.json")
    args = ap.parse_args()
    if args.traffic_summary:
        traffic_summary(*args.traffic_summary)
        return
    if args.mfma_summary:
        mfma_summary(*args.mfma_summary)
        return
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)",
              file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    if args.only == "conv":
        print(json.dumps({"conv": conv_bench(args.steps, args.warmup)}))
        return
    if args.only == "resnet50":
        print(json.dumps({"end_to_end": end_to_end()}))
        return
    if args.only == "unet":
        print(json.dumps({"end_to_end_unet": end_to_end_unet()}))
        return
    ms_per_step, kernels = gpu_bench(args.steps, args.warmup, calibrate=args.only == "lm_ops")
    if args.only == "lm_ops":
        print(json.dumps({"ms_per_step": ms_per_step, "kernels": kernels}))
        return
    value = BYTES_STEP / (ms_per_step * 1e-3) / 1e9
    bn = kernels["bn_bwd_from_output"]
    out = {
        "metric": "lm_ops HBM GB/s (algorithmic bytes / time; BN-from-output bwd + ReLU-mask bwd "
                  "+ maxpool-index bwd at ResNet-50 bs184 shapes)",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "isolated bandwidth-bound lm_ops at ResNet-50 bs184 shapes, fp32: "
                               "BN bwd from output [184,256,56,56]; ReLU 1-bit-mask bwd "
                               "[184,256,56,56]; maxpool3x3s2 bwd [184,64,56,56]->[184,64,112,112]",
                   "bytes_per_step": BYTES_STEP},
        "roofline": {"bound": "hbm", "kernel": "bn_bwd_from_output (bn_prepare_kernel + bn_resident_kernel launches)",
                     "achieved": bn["GB/s"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": bn["frac"], "traffic": bn["traffic"]},
        "kernels": kernels,
    }
    out["conv"] = conv_bench(args.steps, args.warmup)
    if not args.no_end_to_end:
        out["end_to_end"] = e2e = end_to_end()
        out["end_to_end_unet"] = end_to_end_unet()
        # the reference's own headline (ResNet-50, batch 184, 10 GB budget, its operator set):
        # throughput of whole training steps and the overhead against the unconstrained schedule
        head = e2e.get("budget_10GB")
        if head:
            out["config"]["resnet50_bs184_10GB"] = {
                "images_per_s": head["images_per_s"], "ms_per_step": head["ms_per_step"],
                "overhead_vs_unconstrained": head.get("overhead_vs_unconstrained"),
                "peak_MB": head["peak_MB"], "within_budget": head.get("within_budget"),
                "stock_pytorch_images_per_s": e2e["stock_pytorch"]["images_per_s"],
                "warmup_steps": e2e["warmup_steps"], "timed_steps": e2e["timed_steps"]}
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
